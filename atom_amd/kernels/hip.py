"""The engine's kernel library: hand-written HIP for gfx950 behind a C interface,
called through ctypes on PyTorch's current stream.

Every method checks on the host that the operands have the shapes, types and
device the kernel and its grid assume, and raises before anything is launched.
There is no fallback: without a GPU or without the built library, construction fails.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch

from . import build as _build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
_STATUS = {
    1: "unsupported element type",
    2: "operand shapes do not fit the kernel",
    3: "unsupported configuration",
    4: "kernel launch failed",
    5: "a size exceeds what the kernel can hold",
}


class KernelError(RuntimeError):
    pass


@dataclass(frozen=True)
class ChipFigures:
    """What was measured on a GPU and decides between two ways of running the same product.  The ways differ in
    speed and, by rounding, in the last bits of their sums; both are tested against the same reference."""

    stream_bytes_per_us: float     # weights the whole chip streams in a few-rows product, bytes per microsecond
    cu_bytes_per_us: float         # what a single CU draws at most
    split_bytes_per_us: float      # the same product with K cut between blocks (more blocks, shorter)
    add_norm_us: float             # the add-norm kernel that a product cut along K needs beside it
    library_tile: int              # rows and columns of the BLAS library's large tiles
    library_slice_k: int           # the least K a slice of a library product keeps ...
    library_slice_k_many: int      # ... and once there are more than library_many_tiles tiles
    library_many_tiles: int
    decode_parts_root: float       # parts of a decode row x sqrt(requests x KV heads) at which attention + merge take least


# by the architecture name the device reports (before its ':' suffixes)
CHIPS = {
    # MI355X, 8 rows: a CU draws 28 GB/s at most (22 when all 256 share the chip's 5.6 TB/s); a kernel costs 3.4 us
    # beside its bytes and the add-norm kernel 5 us.  With tiles of 16 columns: 32B down (320 blocks, 2 on 64 of
    # the CUs): 60.0 us folded against 47.2 + 5.2 the split way; 32B o: 22.5 against 19.2 + 5.2; 4B down (160
    # blocks): 14.6 against 11.2 + 4.7; 8B down (256 blocks): 20.3 against 18.3 + 4.7.  With tiles of 12 columns
    # (427 and 214 blocks): 32B down 52.0 folded, 32B o 20.2, 4B down 13.5.
    "gfx950": ChipFigures(stream_bytes_per_us=5.6e6, cu_bytes_per_us=28e3, split_bytes_per_us=5.5e6, add_norm_us=5.0,
                          library_tile=256, library_slice_k=2048, library_slice_k_many=4096, library_many_tiles=64,
                          # decode attention from the QKV product plus the merge, 2 / 4 / 8 requests of 8 KV heads at
                          # 1,030 to 8,200 keys: least time at 40-64 / 28-48 / 20-28 parts (a part's chain of
                          # dependent steps shortens with more parts, the merge and the waves' set-up grow); a step
                          # of 8 requests at 2,100 keys: 3.853 / 3.816 / 3.790 / 3.837 ms with 32 / 28 / 24 / 20 parts
                          decode_parts_root=192.0),
}


@dataclass
class AttentionMeta:
    """What attention needs to know about a step's batch, on the device, for one
    group of layers that share block tables.

    token_seq[t]      index of the request (row of block_tables) token t belongs to, -1 for padding
    positions[t]      absolute position of token t in its request
    block_tables      [num_seqs, max_blocks] page ids of each request, in order of position
    cu_seqlens_q      [num_seqs + 1] first token of each request in the flat token axis
    context_lens      [num_seqs] keys of each request once this step's tokens are written
    The three ``max_``/``num_`` numbers are host copies used to pick a kernel and its grid.
    """

    token_seq: torch.Tensor
    positions: torch.Tensor
    block_tables: torch.Tensor
    cu_seqlens_q: torch.Tensor
    context_lens: torch.Tensor
    num_seqs: int
    num_tokens: int
    max_q_len: int
    max_context_len: int
    page_size: int
    # requests 0 .. num_prefill-1 bring more than one token (prompt portions), the rest one each;
    # prefill_tiles [num_tiles, 2] lists (request, first row) of every tile of rows_per_tile rows
    num_prefill: int = 0
    prefill_tiles: torch.Tensor | None = None
    rows_per_tile: int = 16
    # the same for other tile heights: rows -> [num_tiles, 2]
    tiles_by_rows: dict | None = None


class DeferredSum:
    """A matrix product that is still a sum of slices: ``partial`` float32 [splits, rows, width], plus an
    optional bias over the width.  The skinny product leaves its result like this when it cuts K; the
    kernel that reads it next (norm, rotation, SiLU-mul) adds the slices in slice order while it reads.
    ``dtype`` is the type the product has once it is a tensor (``HipKernels.materialize``)."""

    def __init__(self, partial: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype):
        self.partial = partial
        self.bias = bias
        self.dtype = dtype

    @property
    def shape(self):
        return self.partial.shape[1:]

    @property
    def device(self):
        return self.partial.device

    @property
    def splits(self) -> int:
        return self.partial.shape[0]

    @property
    def stride(self) -> int:
        return self.partial.shape[1] * self.partial.shape[2]


class PendingNorm:
    """An RMS norm that has not been applied yet: float32 rows ``r`` [*, width]; ``xg`` = bfloat16(r * weight),
    the same rows times the norm's weight; ``ss`` [*, parts], partial sums of squares of the rows of ``r`` (all
    three left by the product that wrote ``r``); eps; and optionally which rows are meant (``rows``, int32).  The
    few-rows product takes ``xg`` as its input and multiplies its float32 sums by the rows' 1 / rms
    (``HipKernels.linear`` / ``linear_silu``); ``HipKernels.materialize`` runs the norm kernel on ``r``."""

    def __init__(self, r, xg, ss, weight, eps: float, rows, dtype: torch.dtype):
        self.r, self.xg, self.ss, self.weight, self.eps, self.rows, self.dtype = r, xg, ss, weight, float(eps), rows, dtype

    @property
    def shape(self):
        return torch.Size((self.rows.numel() if self.rows is not None else self.r.shape[0], self.r.shape[1]))

    @property
    def device(self):
        return self.r.device


class PendingProduct:
    """``x @ weight.T (+ bias)`` of few rows that has not been launched: what follows decides its epilogue (a norm
    with the residual stream adds the sum in place; anything else takes the plain product)."""

    def __init__(self, x, weight, bias, dtype: torch.dtype):
        self.x, self.weight, self.bias, self.dtype = x, weight, bias, dtype
        self.split = False   # set by a norm that wants the product as a sum of K slices (see pending_norm)

    @property
    def shape(self):
        return torch.Size((self.x.shape[0], self.weight.shape[0]))

    @property
    def device(self):
        return self.weight.device


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


class HipKernels:
    """Loads (building first if need be) the kernel library and binds its entry points."""

    name = "hip"

    def __init__(self, device: str | torch.device = "cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError(
                "atom_amd runs on an AMD GPU only: torch.cuda.is_available() is False and there is no CPU path")
        self.device = torch.device(device)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        path = _build.build()
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"could not load the kernel library {path}: {e}") from e
        self.path = path
        for fn in ("atom_embedding", "atom_feed_tokens", "atom_rmsnorm", "atom_silu_mul", "atom_qk_norm_rope_kv_write",
                   "atom_gemm_skinny", "atom_gemm_skinny_splits", "atom_gemm_skinny_supports", "atom_splitk_reduce",
                   "atom_paged_attention_generic", "atom_gemm_f32", "atom_sample", "atom_exponential_noise",
                   "atom_attention_mfma_supports", "atom_attention_decode", "atom_attention_prefill",
                   "atom_attention_prefill_tile_rows", "atom_attention_decode_fused",
                   "atom_attention_decode_fused_supports", "atom_gemm_rows", "atom_gemm_rows_parts",
                   "atom_gemm_rows_supports", "atom_gemm_tile", "atom_gemm_tile_splits", "atom_gemm_tile_supports",
                   "atom_layernorm", "atom_embedding_scaled", "atom_sum_concat", "atom_gated_act", "atom_latent_prepare",
                   "atom_heads_gemm", "atom_latent_attention", "atom_conv_silu_state", "atom_delta_rule",
                   "atom_delta_out", "atom_router_choose", "atom_experts_gate_up", "atom_experts_down",
                   "atom_latent_attention_mfma", "atom_latent_mfma_supports", "atom_latent_mfma_tokens_per_tile",
                   "atom_experts_grouped", "atom_experts_grouped_tiles", "atom_experts_grouped_supports",
                   "atom_heads_gemm_mfma", "atom_heads_gemm_mfma_supports", "atom_rmsnorm_post", "atom_rmsnorm_rows",
                   "atom_cast_rows", "atom_token_gate", "atom_embedding_bigram", "atom_rglru_scan",
                   "atom_keys_as_values_write", "atom_sigmoid_gate", "atom_bias_rows", "atom_linear_scan", "atom_token_shift",
                   "atom_step_decay", "atom_group_norm_gate", "atom_qkv_plain_write", "atom_narrow_heads",
                   "atom_mean_of_norms", "atom_embedding_positions", "atom_unary_act", "atom_stream_add", "atom_scale_rows",
                   "atom_stream_norm", "atom_sum_norm", "atom_shift_rows", "atom_qkv_rot_write",
                   "atom_attention_together", "atom_attention_together_tiles", "atom_attention_together_tiles_supports",
                   "atom_together_sum_parts"):
            getattr(self.lib, fn).restype = ctypes.c_int
        self.allow_library_gemm = True
        # bfloat16 products of few rows run this library's own weight-streaming kernels: up to 64 rows, and
        # up to 128 for the narrow products that atom_gemm_skinny_supports names; the BLAS library takes the rest.
        self.use_skinny_gemm = True
        self.skinny_max_rows = 128
        # up to 8 bfloat16 rows: the product with the norm before it and the residual sum after it folded in
        self.use_rows_gemm = True
        self.split_library_products = True
        # 65 to 256 bfloat16 rows, products no wider than 8,192 columns: the kernel whose grid of tiles and K slices
        # is cut to the chip's CUs (the BLAS library's large tiles leave most of the chip idle there)
        self.use_tile_gemm = True
        self.tile_rows = (65, 256)
        self.tile_max_width = 8192
        self.narrow_row_tiles = True   # tiles of 12 or 8 columns in the few-rows product where they spread better
        self.rows_waves = 0     # 4 or 8 forces the waves a block of that kernel (0: its own choice)
        self.use_mfma_attention = True
        self.use_tiled_prefill = True
        # Its blocks have eight waves whose halves take the key tiles in turn (D <= 128): True, False, or None for the
        # choice by the size of the launch (see _prefill_in_halves)
        self.prefill_key_halves = None
        self.prefill_low_blocks = None   # True / False forces 16 / 32 tokens a wave in the blocks of eight waves
        self.use_fused_decode = True    # decode-only steps of few rows: norm, rotation and cache write inside attention
        self.use_together_tiles = True  # attention with the heads together on the matrix cores, for prompt portions
        self.use_mfma_latent = True     # attention over latent pages on the matrix cores (bfloat16, sizes it is built for)
        # routed experts: from this many (token, choice) pairs on, the pairs are sorted by expert and run as grouped
        # products on the matrix cores; below, every pair reads its expert's rows itself
        self.grouped_experts_from = 64
        self.heads_mfma_from = 1       # rows from which the per-head products run on the matrix cores
        self.heads_split_from = 9      # ... and from which the exact ones do, on a float32 input's three pieces
        self._ws: dict[str, torch.Tensor] = {}
        self._extensions: dict = {}
        self._zeroed: dict[str, torch.Tensor] = {}   # workspaces that every kernel leaves all zero
        props = torch.cuda.get_device_properties(self.device)
        self.num_cus = props.multi_processor_count
        arch = str(getattr(props, "gcnArchName", "")).split(":")[0]
        # the figures of the part these kernels are written for stand in for an unknown one: only speed depends on them
        self.chip = CHIPS.get(arch, CHIPS["gfx950"])

    def workspace(self, name: str, numel: int, dtype=torch.float32) -> torch.Tensor:
        """A scratch tensor that only grows; one per name.  While a HIP graph is being captured the
        tensor comes from the graph's own pool instead, so that the graph never holds memory
        that a later, larger request would free."""
        if torch.cuda.is_current_stream_capturing():
            return torch.empty(max(numel, 1), dtype=dtype, device=self.device)
        t = self._ws.get(name)
        if t is None or t.numel() < numel or t.dtype != dtype:
            t = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._ws[name] = t
        return t

    # the span names of the operations in a profiler trace, the reference's where it has one
    # (atom/model_ops/attention_mha.py:199, 483, 729: "rope_cache", "paged_attention_*", "prefill_attention")
    _SPANS = {"embedding": "embedding", "rmsnorm": "rmsnorm", "silu_mul": "silu_mul",
              "qk_norm_rope_kv_write": "rope_cache", "paged_attention": "paged_attention",
              "linear": "linear", "linear_silu": "linear_silu", "sample": "sample"}

    def mark_trace(self) -> None:
        """Wraps every operation of this object in a ``torch.profiler.record_function`` span, so that a
        profiler trace shows which kernels belong to which operation (the reference's ``--mark-trace``,
        atom/utils/decorators.py:232-257, in its record_function form).  Off by default: a span costs
        host time in every call."""
        for method, span in self._SPANS.items():
            inner = getattr(self, method)
            if getattr(inner, "_marked", False):
                continue

            def marked(*args, _inner=inner, _span=span, **kwargs):
                with torch.profiler.record_function(_span):
                    return _inner(*args, **kwargs)
            marked._marked = True
            setattr(self, method, marked)

    def attention_tile_rows(self, dtype, head_dim: int, page_size: int, group: int, max_q_len: int) -> tuple[int, int]:
        """The heights of the tiles of query rows that ``paged_attention`` wants listed for a step whose
        longest prompt portion has ``max_q_len`` tokens: (of the kernel whose waves load their own keys, of
        the kernel whose waves share key tiles); 0 where a kernel is not used (float32 steps list nothing)."""
        if (dtype != torch.bfloat16 or not self.use_mfma_attention
                or not self.lib.atom_attention_mfma_supports(head_dim, page_size, group)):
            return 0, 0
        tall = 0
        if max_q_len >= 32 and self.use_tiled_prefill:
            tall = int(self.lib.atom_attention_prefill_tile_rows(head_dim, page_size, group))
        return (32 if max_q_len > 16 else 16), tall

    def decode_parts(self, seqs: int, hkv: int, max_context: int) -> int:
        """Over how many waves a decode row's keys are split: enough waves to fill the chip,
        at least 64 keys each."""
        rows = max(1, seqs * hkv)
        want = -(-8 * self.num_cus // rows)
        if want > 8:   # more parts than one block merges itself: the merge kernel's time counts too
            want = min(want, max(9, round(self.chip.decode_parts_root / math.sqrt(rows))))
        return max(1, min(want, 64, -(-max_context // 64)))

    # ------------------------------------------------------------------ helpers

    def load_extension(self, sources: list[str], lib_name: str) -> ctypes.CDLL:
        """For a part that brings HIP kernels of its own: compiles ``sources`` with this library's flags (once;
        ``kernels.build.build_sources``) and loads the result.  The part declares its entry points' types on the
        returned library and calls them with ``pointer(tensor)`` and ``stream()``; ``check`` is the operand test
        every method here uses."""
        key = (tuple(sources), lib_name)
        if key not in self._extensions:
            try:
                self._extensions[key] = ctypes.CDLL(_build.build_sources(list(sources), lib_name))
            except OSError as e:
                raise KernelError(f"could not load the kernels of {lib_name}: {e}") from e
        return self._extensions[key]

    def stream(self):
        """The handle of PyTorch's current stream on this device, as kernels' C entry points take it."""
        return self._stream()

    @staticmethod
    def pointer(t: torch.Tensor | None):
        return _ptr(t)

    def check(self, name: str, t: torch.Tensor, dtype=None, shape=None):
        return self._check(name, t, dtype, shape)

    def _stream(self):
        # the current stream's handle, the short way: these few calls are made hundreds of times a step
        return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(self._device_index))

    def _check(self, name: str, t: torch.Tensor, dtype=None, shape=None):
        """Every operand of every call goes through here (a step makes over a thousand such calls):
        the passing case costs a few attribute reads, the failing one says what is wrong."""
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
        if not t.is_cuda:
            raise KernelError(f"{name}: must live on the GPU, is on {t.device}")
        if not t.is_contiguous():
            raise KernelError(f"{name}: must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
        if dtype is not None:
            have = t.dtype
            if have is not dtype and (not isinstance(dtype, (tuple, list)) or have not in dtype):
                raise KernelError(f"{name}: element type {have} not in {dtype}")
        if shape is not None:
            have = t.shape
            ok = len(shape) == len(have)
            if ok:
                for want, got in zip(shape, have):
                    if want is not None and want != got:
                        ok = False
                        break
            if not ok:
                raise KernelError(f"{name}: shape {tuple(have)} does not match {tuple(shape)}")
        return t

    def _done(self, what: str, status: int):
        if status != 0:
            raise KernelError(f"{what}: {_STATUS.get(status, f'status {status}')}")

    @staticmethod
    def _code(t: torch.Tensor) -> int:
        try:
            return _DTYPE_CODE[t.dtype]
        except KeyError:
            raise KernelError(f"element type {t.dtype} is not supported (float32 and bfloat16 are)") from None

    def _sum_args(self, x):
        """The four trailing arguments that say whether an input is a tensor or a sum of slices."""
        if isinstance(x, DeferredSum):
            self._check("slices", x.partial, torch.float32)
            if x.bias is not None:
                self._check("bias of the slices", x.bias, torch.float32, (x.shape[1],))
            return _ptr(x.partial), x.splits, ctypes.c_long(x.stride), _ptr(x.bias)
        return None, 0, ctypes.c_long(0), None

    def materialize(self, x):
        """A tensor from what may still be a sum of slices, a product not launched yet or a norm not applied yet."""
        if isinstance(x, PendingProduct):
            return self._rows_product(x.x, x.weight, x.bias, x.dtype)
        if isinstance(x, PendingNorm):
            out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
            # the float32 rows as a sum of one slice: the norm kernel reads float32 and writes the step's type
            return self.rmsnorm(DeferredSum(x.r.unsqueeze(0), None, x.dtype), x.weight, x.eps, out, rows=x.rows)
        if hasattr(x, "terms"):
            # a sum of scaled terms that a mixer handed on, added up in float32
            out = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
            return self.sum_norm(out, 0.0, x.terms, x.scales, None, 0.0)
        if not isinstance(x, DeferredSum):
            return x
        rows, width = x.shape
        y = torch.empty((rows, width), dtype=x.dtype, device=x.device)
        self._done("splitk_reduce", self.lib.atom_splitk_reduce(
            _ptr(x.partial), _ptr(x.bias), _ptr(y), rows, width, x.splits, int(x.dtype == torch.float32),
            self._stream()))
        return y

    # ---- the few-rows product with the norm before it and the residual sum after it folded in

    def _rows_takes(self, x, weight) -> bool:
        m, k = x.shape
        return bool(self.use_rows_gemm and 1 <= m <= 8 and weight.dtype == torch.bfloat16
                    and (isinstance(x, PendingNorm) or x.dtype == torch.bfloat16)
                    and self.lib.atom_gemm_rows_supports(m, weight.shape[0], k))

    def rows_cols(self, n: int) -> int:
        """Output columns a block of the few-rows product owns for a width of ``n``: 16, or 12 or 8 where that
        takes at least a fifth off the columns of the busiest CU (2,560 columns are 160 tiles of 16 for 256 CUs,
        but 214 of 12; 5,120 and 6,144 are 1.25 and 1.5 tiles of 16 a CU, and 1.67 and 2 of 12).  A block streams
        its columns' rows of w at what one CU draws, so the busiest CU's columns are the product's time wherever
        the chip as a whole is not the limit."""
        if not self.narrow_row_tiles:
            return 16
        def busiest(cols: int) -> int:   # columns of the CU with the most blocks
            tiles = -(-n // cols)
            return -(-tiles // self.num_cus) * cols

        best = 16
        for cols in (12, 8):
            if busiest(cols) * 5 <= busiest(16) * 4 and busiest(cols) < busiest(best):
                best = cols
        return best

    def _rows_residual_pays(self, n: int, k: int) -> bool:
        """Whether the few-rows product with the residual sum folded in beats the product with K cut between
        blocks followed by the add-norm kernel.  The folded one owns ``rows_cols(n)`` columns and all of K per block, so
        its blocks are all the parallelism there is, and it takes as long as its busiest CU needs for its
        blocks' rows of w.  The figures are the chip's (``CHIPS``)."""
        chip = self.chip
        cols = self.rows_cols(n)
        tiles = -(-n // cols)
        folded = max(n * 2 * k / chip.stream_bytes_per_us,                                  # the chip's pace,
                     -(-tiles // self.num_cus) * cols * 2 * k / chip.cu_bytes_per_us)       # the busiest CU's
        split = n * k * 2 / chip.split_bytes_per_us + chip.add_norm_us
        return folded <= split

    def _rows_launch(self, x, weight, bias, mode: int, y=None, res=None, ss_out=None, xg_out=None, g_next=None,
                     out_f32: bool = False, act: int = 0):
        m, k = x.shape
        n = weight.shape[0] // 2 if mode == 1 else weight.shape[0]
        self._check("linear weight", weight, torch.bfloat16, (weight.shape[0], k))
        if bias is not None:
            self._check("linear bias", bias, torch.float32, (weight.shape[0],))
        if isinstance(x, PendingNorm):
            self._check("norm input", x.xg, torch.bfloat16, (None, k))
            self._check("sums of squares", x.ss, torch.float32, (x.xg.shape[0], None))
            if x.rows is not None:
                self._check("norm row choice", x.rows, torch.int32, (m,))
            head = (_ptr(x.xg), _ptr(x.rows), _ptr(x.ss), x.ss.shape[1], ctypes.c_float(x.eps))
        else:
            self._check("linear input", x, torch.bfloat16, (m, k))
            head = (_ptr(x), None, None, 0, ctypes.c_float(0.0))
        self._done("gemm_rows", self.lib.atom_gemm_rows(
            *head, _ptr(weight), _ptr(bias), _ptr(y), _ptr(res), _ptr(ss_out), _ptr(xg_out), _ptr(g_next), m, n, k,
            mode, int(out_f32), 16 if mode == 1 else self.rows_cols(n), int(self.rows_waves), act, 1, ctypes.c_long(0),
            ctypes.c_long(0), ctypes.c_long(0), self._stream()))

    def _rows_product(self, x, weight, bias, out_dtype):
        y = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=weight.device)
        self._rows_launch(x, weight, bias, 0, y=y, out_f32=out_dtype == torch.float32)
        return y

    def pending_norm(self, x, residual, weight, eps: float, rows=None):
        """``residual += x`` where x is a product that has not been launched (it is launched now, the sum formed
        in place where the product leaves the matrix cores), and the norm of the sum left pending for the product
        that follows.  None if ``x`` is anything else: the caller then takes ``rmsnorm``."""
        if not isinstance(x, PendingProduct) or residual is None:
            return None
        m, n = x.shape
        if not self._rows_residual_pays(n, x.weight.shape[1]) and not isinstance(x.x, PendingNorm):
            x.split = True    # rmsnorm() launches it with K cut between blocks and adds the slices itself
            return None
        self._check("residual", residual, torch.float32, (m, n))
        self._check("norm weight", weight, torch.float32, (n,))
        inner = x.x
        if isinstance(inner, PendingNorm) and inner.r.data_ptr() == residual.data_ptr():
            inner = self.materialize(inner)   # the product may not read the rows it adds to
        ss = torch.empty((m, self.lib.atom_gemm_rows_parts(n, self.rows_cols(n))), dtype=torch.float32,
                         device=residual.device)
        xg = torch.empty((m, n), dtype=torch.bfloat16, device=residual.device)
        self._rows_launch(inner, x.weight, x.bias, 2, res=residual, ss_out=ss, xg_out=xg, g_next=weight)
        return PendingNorm(residual, xg, ss, weight, eps, rows, x.dtype)

    # ------------------------------------------------------------------ kernels

    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        vocab, hidden = table.shape
        tokens = ids.numel()
        self._check("embedding table", table, (torch.float32, torch.bfloat16))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("embedding out", out, (torch.float32, torch.bfloat16), (tokens, hidden))
        self._done("embedding", self.lib.atom_embedding(
            _ptr(table), self._code(table), _ptr(ids), _ptr(out), self._code(out), tokens, hidden, vocab,
            self._stream()))
        return out

    def feed_tokens(self, ids: torch.Tensor, source: torch.Tensor, sampled: torch.Tensor) -> torch.Tensor:
        """``ids[t] = sampled[source[t]]`` where ``source[t] >= 0`` (all int32, in place): token ids that the
        last step's sampler left on the device."""
        n = ids.numel()
        self._check("token ids", ids, torch.int32, (n,))
        self._check("token sources", source, torch.int32, (n,))
        self._check("sampled ids", sampled, torch.int32, (None,))
        self._done("feed_tokens", self.lib.atom_feed_tokens(
            _ptr(ids), _ptr(source), _ptr(sampled), n, sampled.numel(), self._stream()))
        return ids

    def rmsnorm(self, x, weight, eps: float, out, residual=None, mode: str = "plain", rows=None):
        """mode 'plain': out = norm(x); 'init': residual = x, out = norm(x);
        'add': residual += x, out = norm(residual).  With ``rows`` only those source
        rows are normed (into out[0..len(rows))) and the residual is not written."""
        if isinstance(x, PendingProduct) and x.split:
            x = self.linear(x.x, x.weight, x.bias, x.dtype, defer=True, few_rows=False)
        if isinstance(x, (PendingProduct, PendingNorm)):
            x = self.materialize(x)
        width = x.shape[-1]
        code = {"plain": 0, "init": 1, "add": 2}[mode]
        deferred = isinstance(x, DeferredSum)
        if not deferred:
            self._check("norm input", x, (torch.float32, torch.bfloat16), (None, width))
        self._check("norm weight", weight, torch.float32, (width,))
        n_out = rows.numel() if rows is not None else x.shape[0]
        self._check("norm out", out, x.dtype, (n_out, width))
        if code:
            if residual is None:
                raise KernelError("norm: this mode needs the residual stream")
            self._check("residual", residual, torch.float32, tuple(x.shape))
        if rows is not None:
            self._check("norm rows", rows, torch.int32, (n_out,))
        self._done("rmsnorm", self.lib.atom_rmsnorm(
            None if deferred else _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), self._code(out),
            n_out, width, ctypes.c_float(eps), code, *self._sum_args(x), self._stream()))
        return out

    def silu_mul(self, x, out):
        rows, two = x.shape
        if two % 2:
            raise KernelError("silu_mul: the input width must be even (gate | up)")
        deferred = isinstance(x, DeferredSum)
        if not deferred:
            self._check("silu_mul input", x, (torch.float32, torch.bfloat16))
        self._check("silu_mul out", out, x.dtype, (rows, two // 2))
        self._done("silu_mul", self.lib.atom_silu_mul(None if deferred else _ptr(x), _ptr(out), self._code(out), rows,
                                                      two // 2, *self._sum_args(x), self._stream()))
        return out

    def qk_norm_rope_kv_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, cos, sin, positions,
                              slots, num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int,
                              page_size: int, eps: float, write_kv: bool = True):
        if isinstance(qkv, PendingProduct):
            # the float32 product as a sum of one slice: the kernel reads it with the precision it reads slices
            full = self._rows_product(qkv.x, qkv.weight, qkv.bias, torch.float32)
            qkv = DeferredSum(full.unsqueeze(0), None, qkv.dtype)
        tokens = qkv.shape[0]
        dt = qkv.dtype
        deferred = isinstance(qkv, DeferredSum)
        if deferred:
            if tuple(qkv.shape) != (tokens, (num_heads + 2 * num_kv_heads) * head_dim):
                raise KernelError(f"qkv: shape {tuple(qkv.shape)} does not fit the heads")
        else:
            self._check("qkv", qkv, (torch.float32, torch.bfloat16),
                        (tokens, (num_heads + 2 * num_kv_heads) * head_dim))
        self._check("q out", q_out, dt, (tokens, num_heads, head_dim))
        if write_kv:
            self._check("key pages", k_cache, dt, (None, num_kv_heads, page_size, head_dim))
            self._check("value pages", v_cache, dt, (k_cache.shape[0], num_kv_heads, head_dim, page_size))
            self._check("slot mapping", slots, torch.int32, (tokens,))
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                self._check(name, w, torch.float32, (head_dim,))
        if rotary_dim:
            self._check("cos table", cos, torch.float32, (None, rotary_dim // 2))
            self._check("sin table", sin, torch.float32, tuple(cos.shape))
            self._check("positions", positions, torch.int32, (tokens,))
        self._done("qk_norm_rope_kv_write", self.lib.atom_qk_norm_rope_kv_write(
            None if deferred else _ptr(qkv), _ptr(q_out), _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None,
            _ptr(q_weight), _ptr(k_weight), _ptr(cos) if rotary_dim else None, _ptr(sin) if rotary_dim else None,
            _ptr(positions) if rotary_dim else None, _ptr(slots) if write_kv else None, self._code(q_out), tokens,
            num_heads, num_kv_heads, head_dim, rotary_dim, page_size, ctypes.c_float(eps), int(bool(write_kv)),
            *self._sum_args(qkv), self._stream()))
        return q_out

    def _attention_mfma(self, q, k_cache, v_cache, out, meta, scale, window, parts=None, softcap=None, chunk=None,
                        sink=None):
        tokens, hq, d = q.shape
        _, hkv, page_size, _ = k_cache.shape
        self._check("cu_seqlens_q", meta.cu_seqlens_q, torch.int32, (meta.num_seqs + 1,))
        self._check("context_lens", meta.context_lens, torch.int32, (meta.num_seqs,))
        bt = meta.block_tables
        if bt.shape[0] != meta.num_seqs:
            raise KernelError("attention: one block table row per request is needed")
        if meta.num_prefill:
            tiles, rows, tiled = meta.prefill_tiles, meta.rows_per_tile, 0
            if meta.max_q_len >= 32 and meta.tiles_by_rows and self.use_tiled_prefill:
                # long portions: the kernel whose waves share key tiles through LDS
                want = self.lib.atom_attention_prefill_tile_rows(d, page_size, hq // hkv)
                if want and want in meta.tiles_by_rows:
                    tiles, rows = meta.tiles_by_rows[want], want
                    blocks = tiles.shape[0] * hq * 32 // (4 * want)
                    tiled = 2 if self._prefill_in_halves(blocks, meta) else 1
                    if tiled == 2 and self._prefill_low_blocks(blocks, d, meta):
                        tiled = 3
            self._check("prefill tiles", tiles, torch.int32, (None, 2))
            if not tiled and rows not in (16, 32):
                raise KernelError("attention: tiles hold 16 or 32 rows")
            self._done("attention_prefill", self.lib.atom_attention_prefill(
                _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q), _ptr(meta.context_lens),
                _ptr(bt), bt.shape[1], _ptr(tiles), tiles.shape[0], rows, tiled, hq, hkv, d, page_size,
                ctypes.c_float(scale), int(window or 0), int(chunk or 0), ctypes.c_float(softcap or 0.0), _ptr(sink),
                self._stream()))
        seqs = meta.num_seqs - meta.num_prefill
        if seqs:
            if parts is None:
                visible = min(meta.max_context_len, window) if window else meta.max_context_len
                if chunk:
                    visible = min(visible, chunk)
                parts = self.decode_parts(seqs, hkv, visible)
            ws_o = ws_ml = None
            if parts > 1:
                ws_o = self.workspace("attn_o", seqs * hq * parts * d)
                ws_ml = self.workspace("attn_ml", seqs * hq * parts * 2)
            self._done("attention_decode", self.lib.atom_attention_decode(
                _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q), _ptr(meta.context_lens),
                _ptr(bt), bt.shape[1], meta.num_prefill, seqs, hq, hkv, d, page_size, ctypes.c_float(scale),
                int(window or 0), int(chunk or 0), ctypes.c_float(softcap or 0.0), parts, _ptr(ws_o), _ptr(ws_ml),
                _ptr(sink), self._stream()))
        return out

    def _prefill_in_halves(self, blocks: int, meta) -> bool:
        """Whether the prefill kernel with shared key tiles runs blocks of eight waves (one a CU, the key tiles taken
        in turn by the block's halves) rather than of four (two a CU, each on its own).  Measured on an MI355X with
        32 / 8 heads of 128: two blocks of four waves keep each other's SIMDs busy as long as both run, so they win
        when a CU has a queue of them (8,192 fresh tokens: 640 against 690 us) or when all blocks are about as long
        (2,048 tokens behind 8,192 cached: 355 against 390 us); a block of eight waves does not depend on a
        neighbour, and wins when there is none (a portion of 512 tokens behind 3,072 cached, 128 blocks: 74 against
        99 us) or when the long blocks of a fresh prompt outlive their short neighbours (2,048 tokens: 64 against
        72 us)."""
        if self.prefill_key_halves is not None:
            return bool(self.prefill_key_halves)
        if blocks <= self.num_cus:
            return True
        return blocks <= 2 * self.num_cus and 2 * meta.max_context_len < 3 * meta.max_q_len

    def _prefill_low_blocks(self, blocks: int, head_dim: int, meta) -> bool:
        """Whether the blocks of eight waves take 16 query tokens a wave instead of 32 (twice the blocks, each with
        half the products per key tile it stages): when the launch would otherwise leave half of the CUs without a
        block (512 tokens behind 3,072 cached: 65 against 78 us), and for fresh prompts of up to a block a CU, whose
        blocks are mostly short (549 / 768 / 1,024 tokens: 16 / 20 / 29 against 21 / 24 / 30 us; behind 2,048 cached
        tokens the same launches take 82-90 against 62-68 us, so those keep 32 tokens a wave)."""
        if self.prefill_low_blocks is not None:
            return bool(self.prefill_low_blocks) and head_dim <= 128
        if head_dim > 128:
            return False
        return 2 * blocks <= self.num_cus or (blocks <= self.num_cus and 2 * meta.max_context_len < 3 * meta.max_q_len)

    def fused_decode_attention(self, qkv, k_cache, v_cache, out, meta: AttentionMeta, scale: float, window, q_weight,
                               k_weight, cos, sin, slots, num_heads: int, num_kv_heads: int, head_dim: int,
                               rotary_dim: int, eps: float, write_kv: bool = True, parts: int | None = None):
        """For a step in which every request brings one token: per-head norm of q and k, rotation, the write of the
        new keys and values and attention over the pages in one kernel (and the merge of the key ranges), starting
        from the QKV product, which has to be one that has not been launched yet (a few-rows ``PendingProduct``; it is
        launched here with float32 output).  Returns ``out``, or None when this case is not taken: the caller then
        runs ``qk_norm_rope_kv_write`` and ``paged_attention``."""
        page_size = meta.page_size
        if (not self.use_fused_decode or not isinstance(qkv, PendingProduct) or meta.num_prefill or out.dtype != torch.bfloat16
                or rotary_dim != head_dim or cos is None
                or not self.lib.atom_attention_decode_fused_supports(head_dim, page_size, num_heads // num_kv_heads)):
            return None
        tokens = qkv.shape[0]
        if meta.num_seqs != tokens or tuple(qkv.shape) != (tokens, (num_heads + 2 * num_kv_heads) * head_dim):
            return None
        self._check("key pages", k_cache, torch.bfloat16, (None, num_kv_heads, page_size, head_dim))
        self._check("value pages", v_cache, torch.bfloat16, (k_cache.shape[0], num_kv_heads, head_dim, page_size))
        self._check("attention out", out, torch.bfloat16, (tokens, num_heads, head_dim))
        self._check("cu_seqlens_q", meta.cu_seqlens_q, torch.int32, (tokens + 1,))
        self._check("context_lens", meta.context_lens, torch.int32, (tokens,))
        self._check("block tables", meta.block_tables, torch.int32, (tokens, None))
        self._check("cos table", cos, torch.float32, (None, head_dim // 2))
        self._check("sin table", sin, torch.float32, tuple(cos.shape))
        if meta.max_context_len > cos.shape[0]:
            raise KernelError("attention: a position lies beyond the rotation tables")
        if meta.max_context_len > meta.block_tables.shape[1] * page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                self._check(name, w, torch.float32, (head_dim,))
        if write_kv:
            self._check("slot mapping", slots, torch.int32, (tokens,))
        full = self._rows_product(qkv.x, qkv.weight, qkv.bias, torch.float32)
        if parts is None:
            visible = min(meta.max_context_len, window) if window else meta.max_context_len
            parts = self.decode_parts(tokens, num_kv_heads, visible)
        ws_o = ws_ml = None
        if parts > 1:
            ws_o = self.workspace("attn_o", tokens * num_heads * parts * head_dim)
            ws_ml = self.workspace("attn_ml", tokens * num_heads * parts * 2)
        bt = meta.block_tables
        self._done("attention_decode_fused", self.lib.atom_attention_decode_fused(
            _ptr(full), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin), _ptr(slots) if write_kv else None,
            ctypes.c_float(eps), int(bool(write_kv)), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.cu_seqlens_q),
            _ptr(meta.context_lens), _ptr(bt), bt.shape[1], 0, tokens, num_heads, num_kv_heads, head_dim, page_size,
            ctypes.c_float(scale), int(window or 0), parts, _ptr(ws_o), _ptr(ws_ml), self._stream()))
        return out

    def paged_attention(self, q, k_cache, v_cache, out, meta: AttentionMeta, scale: float,
                        window: int | None = None, parts: int | None = None, softcap: float | None = None,
                        chunk: int | None = None, sink=None):
        """Attention of the step's queries over the pages.  ``window``: only the latest that many keys;
        ``chunk``: only the keys of the query's own run of that many positions, counted from position 0;
        ``softcap``: a score s becomes ``softcap * tanh(s / softcap)``; ``sink`` (float32 [Hq]): ``exp(sink[h])``
        joins head h's denominator with no key and no value (the matrix-core kernels only: ask
        ``takes_sink`` first)."""
        tokens, hq, d = q.shape
        _, hkv, page_size, _ = k_cache.shape
        dt = q.dtype
        if hq % hkv:
            raise KernelError(f"attention: {hq} query heads are not a multiple of {hkv} key/value heads")
        self._check("q", q, (torch.float32, torch.bfloat16))
        self._check("key pages", k_cache, dt, (None, hkv, page_size, d))
        self._check("value pages", v_cache, dt, (k_cache.shape[0], hkv, d, page_size))
        self._check("attention out", out, dt, (tokens, hq, d))
        self._check("token_seq", meta.token_seq, torch.int32, (tokens,))
        self._check("positions", meta.positions, torch.int32, (tokens,))
        self._check("block tables", meta.block_tables, torch.int32, (None, None))
        if meta.page_size != page_size:
            raise KernelError("attention: the batch's page size differs from the cache's")
        if meta.max_context_len > meta.block_tables.shape[1] * page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        group = hq // hkv
        if softcap and not scale > 0:
            raise KernelError("attention: a cap on the scores needs a positive scale")
        if sink is not None:
            self._check("sink", sink, torch.float32, (hq,))
        if (dt == torch.bfloat16 and self.use_mfma_attention
                and self.lib.atom_attention_mfma_supports(d, page_size, group)):
            return self._attention_mfma(q, k_cache, v_cache, out, meta, scale, window, parts, softcap, chunk, sink)
        if sink is not None:
            raise KernelError("attention: the general kernel has no sink; ask takes_sink before")
        self._done("paged_attention", self.lib.atom_paged_attention_generic(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(meta.token_seq), _ptr(meta.positions),
            _ptr(meta.block_tables), meta.block_tables.shape[1], self._code(q), tokens, hq, hkv, d, page_size,
            ctypes.c_float(scale), int(window or 0), int(chunk or 0), ctypes.c_float(softcap or 0.0), self._stream()))
        return out

    def takes_sink(self, dtype, head_dim: int, value_dim: int, page_size: int, group: int) -> bool:
        """Whether ``paged_attention`` takes a ``sink`` for these sizes: the matrix-core kernels, whose keys and
        values have one head size."""
        return bool(dtype == torch.bfloat16 and self.use_mfma_attention and head_dim == value_dim
                    and self.lib.atom_attention_mfma_supports(head_dim, page_size, group))

    def _library_slices(self, m: int, n: int, k: int) -> int:
        """Into how many slices of K a product that goes to the BLAS library is cut when its reader can add
        slices.  Measured on an MI355X with the o and down products of the 4B, 8B and 32B shapes at 544 to 4,096
        rows, the add-norm that reads the slices included: the library's kernels leave much of the chip idle
        while a product has fewer tiles of 256 x 256 than the chip has CUs, and the most slices that keep
        tiles x slices within the CUs win (8B down: 96 -> 58 us at 544 rows, 140 -> 108 at 1,024, 210 -> 197 at
        2,048; 32B down 373 -> 247 at 1,024), as long as a slice keeps 2,048 of K, and 4,096 once there are more
        than 64 tiles.  Products that widen (whose reader here is the rotation kernel, which wants a tensor for
        many rows) are left whole."""
        if not self.split_library_products or n > k:
            return 1
        chip = self.chip
        tiles = -(-m // chip.library_tile) * -(-n // chip.library_tile)
        for slices in (4, 2):
            per = k // slices
            if (k % (slices * 8) == 0 and tiles * slices <= self.num_cus and per >= chip.library_slice_k
                    and (tiles <= chip.library_many_tiles or per >= chip.library_slice_k_many)):
                return slices
        return 1

    def _tile(self, x, weight) -> bool:
        m, k = x.shape
        n = weight.shape[0]
        return bool(self.use_tile_gemm and self.tile_rows[0] <= m <= self.tile_rows[1] and n <= self.tile_max_width
                    and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                    and self.lib.atom_gemm_tile_supports(m, n, k))

    def _skinny(self, x, weight) -> bool:
        m, k = x.shape
        return bool(self.use_skinny_gemm and m <= self.skinny_max_rows and x.dtype == torch.bfloat16
                    and weight.dtype == torch.bfloat16 and self.lib.atom_gemm_skinny_supports(m, weight.shape[0], k))

    def linear(self, x, weight, bias=None, out_dtype=None, defer: bool = False, few_rows: bool = True):
        """``x @ weight.T (+ bias)``.  bfloat16 operands with at most 64 rows (narrow products: 128) run this
        library's own weight-streaming kernels, 65 to 256 rows of products up to 8,192 columns wide its kernel of
        tiles and K slices cut to the chip; the rest goes to the BLAS library, as the reference's engine
        does for its matrix products; anything with a float32 operand runs this library's float32
        kernel (plain FMA, no reduced-precision mode).  With ``defer`` the result may come back as a
        ``DeferredSum`` for a kernel that adds the slices while it reads them."""
        if isinstance(x, (DeferredSum, PendingProduct)):
            x = self.materialize(x)
        m, k = x.shape
        n = weight.shape[0]
        if m and few_rows and self._rows_takes(x, weight):
            if defer:
                return PendingProduct(x, weight, bias, out_dtype or x.dtype)
            return self._rows_product(x, weight, bias, out_dtype or x.dtype)
        x = self.materialize(x)
        self._check("linear input", x, (torch.float32, torch.bfloat16))
        self._check("linear weight", weight, (torch.float32, torch.bfloat16), (n, k))
        out_dtype = out_dtype or x.dtype
        if bias is not None:
            self._check("linear bias", bias, torch.float32, (n,))
        if self._tile(x, weight):
            splits = self.lib.atom_gemm_tile_splits(m, n, k, self.num_cus)
            if splits == 1:
                y = torch.empty((m, n), dtype=out_dtype, device=x.device)
                self._done("gemm_tile", self.lib.atom_gemm_tile(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(y), None, m, n, k, 1, int(out_dtype == torch.float32),
                    self._stream()))
                return y
            partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            self._done("gemm_tile", self.lib.atom_gemm_tile(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, n, k, splits, 0, self._stream()))
            result = DeferredSum(partial, bias, out_dtype)
            # a product that widens is read next by the rotation kernel, which wants a tensor for this many rows
            return result if defer and n <= k else self.materialize(result)
        if m and self._skinny(x, weight):
            splits = self.lib.atom_gemm_skinny_splits(m, n, k, 0)
            if splits == 1:
                y = torch.empty((m, n), dtype=out_dtype, device=x.device)
                self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(y), None, m, n, k, int(out_dtype == torch.float32), 0,
                    self._stream()))
                return y
            partial = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, n, k, 0, 0, self._stream()))
            result = DeferredSum(partial, bias, out_dtype)
            return result if defer else self.materialize(result)
        if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and self.allow_library_gemm:
            slices = self._library_slices(m, n, k) if defer else 1
            if slices > 1:
                # a product with too few tiles to fill the chip: K in slices as one batched product with float32
                # output, left as a sum that the norm behind it adds while it reads
                part = k // slices
                partial = torch.bmm(x.view(m, slices, part).transpose(0, 1),
                                    weight.view(n, slices, part).permute(1, 2, 0), out_dtype=torch.float32)
                return DeferredSum(partial, bias, out_dtype)
            if bias is None and out_dtype == torch.bfloat16:
                return torch.nn.functional.linear(x, weight)
            # float32 out, or a bias: the library writes its float32 sums as they are, so that logits have the
            # same precision whatever the number of rows, and a bias is added before anything is rounded
            y = torch.mm(x, weight.t(), out_dtype=torch.float32)
            if bias is not None:
                self._done("bias_rows", self.lib.atom_bias_rows(_ptr(y), _ptr(bias), m, n, self._stream()))
            return y if out_dtype == torch.float32 else y.to(out_dtype)
        y = torch.empty((m, n), dtype=out_dtype, device=x.device)
        self._done("gemm_f32", self.lib.atom_gemm_f32(
            _ptr(x), self._code(x), _ptr(weight), self._code(weight), _ptr(bias), _ptr(y), self._code(y), m, n, k,
            self._stream()))
        return y

    _ROWS_ACT = {"silu": 1, "relu": 2, "gelu_tanh": 3, "relu_squared": 4, "tanh": 5}

    def linear_act(self, x, weight, bias, activation: str, out_dtype=None):
        """``act(x @ weight.T + bias)`` in ``x``'s type (or ``out_dtype``): one kernel where the few-rows product takes it (a pending
        norm of ``x`` folded in as well), else the product and the activation entry by entry."""
        if activation not in self._ROWS_ACT:
            raise KernelError(f"linear_act: unknown activation {activation!r}; known: {sorted(self._ROWS_ACT)}")
        if isinstance(x, (DeferredSum, PendingProduct)):
            x = self.materialize(x)
        m = x.shape[0]
        if m and self._rows_takes(x, weight):
            y = torch.empty((m, weight.shape[0]), dtype=out_dtype or x.dtype, device=weight.device)
            self._rows_launch(x, weight, bias, 0, y=y, act=self._ROWS_ACT[activation], out_f32=y.dtype == torch.float32)
            return y
        up = self.linear(x, weight, bias, out_dtype=out_dtype)
        out = torch.empty(tuple(up.shape), dtype=up.dtype, device=up.device)
        return self.unary_act(up, out, activation)

    def linear_side_by_side(self, xs, weights, out_dtype=None):
        """``ys[b] = xs[b] @ weights[b].T`` for ``xs`` [B, rows, k] and ``weights`` [B, n, k]: one launch where the
        few-rows product takes the sizes, else a product each."""
        B, m, k = xs.shape
        n = weights.shape[1]
        out_dtype = out_dtype or xs.dtype
        if weights.shape[0] != B or weights.shape[2] != k:
            raise KernelError("linear_side_by_side: as many weights as inputs, of the inputs' inner size")
        if m and B > 1 and xs.is_contiguous() and weights.is_contiguous() and self._rows_takes(xs[0], weights[0]):
            self._check("linear input", xs, torch.bfloat16)
            self._check("linear weight", weights, torch.bfloat16)
            ys = torch.empty((B, m, n), dtype=out_dtype, device=xs.device)
            self._done("gemm_rows", self.lib.atom_gemm_rows(
                _ptr(xs), None, None, 0, ctypes.c_float(0.0), _ptr(weights), None, _ptr(ys), None, None, None, None, m, n, k,
                0, int(out_dtype == torch.float32), self.rows_cols(n), int(self.rows_waves), 0, B, ctypes.c_long(m * k),
                ctypes.c_long(n * k), ctypes.c_long(m * n), self._stream()))
            return [ys[b] for b in range(B)]
        return [self.linear(xs[b], weights[b], None, out_dtype=out_dtype) for b in range(B)]

    def linear_silu(self, x, weight, bias=None):
        """``silu(x @ Wg.T + bg) * (x @ Wu.T + bu)`` for ``weight`` = gate rows then up rows: one kernel
        where the skinny product does not cut K, else the product and SiLU-mul over its slices."""
        m, k = x.shape
        two = weight.shape[0]
        if two % 2:
            raise KernelError("linear_silu: the weight must hold as many gate rows as up rows")
        inter = two // 2
        if m and self._rows_takes(x, weight):
            act = torch.empty((m, inter), dtype=x.dtype, device=weight.device)
            self._rows_launch(x, weight, bias, 1, y=act)
            return act
        x = self.materialize(x)
        if m and self._skinny(x, weight):
            self._check("linear input", x, torch.bfloat16)
            self._check("linear weight", weight, torch.bfloat16, (two, k))
            if bias is not None:
                self._check("linear bias", bias, torch.float32, (two,))
            act = torch.empty((m, inter), dtype=x.dtype, device=x.device)
            splits = self.lib.atom_gemm_skinny_splits(m, inter, k, 1)
            if splits == 1:
                self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(act), None, m, inter, k, 0, 1, self._stream()))
                return act
            partial = torch.empty((splits, m, two), dtype=torch.float32, device=x.device)
            self._done("gemm_skinny", self.lib.atom_gemm_skinny(
                _ptr(x), _ptr(weight), None, None, _ptr(partial), m, inter, k, 0, 1, self._stream()))
            return self.silu_mul(DeferredSum(partial, bias, x.dtype), act)
        gate_up = self.linear(x, weight, bias)
        act = torch.empty((m, inter), dtype=x.dtype, device=x.device)
        return self.silu_mul(gate_up, act)

    # ------------------------------------------------------------------ layer norm and the float32 stream

    _NORM_MODES = {"plain": 0, "init": 1, "add": 2, "post": 3}

    def layernorm(self, x, weight, bias, eps: float, out, residual=None, mode: str = "plain", rows=None,
                  next_weight=None, next_bias=None):
        """Layer norm with weight and bias in float32.  mode 'plain': out = LN(x); 'init': residual = x,
        out = LN(x); 'add': residual += x, out = LN(residual); 'post': residual += LN(x) and then
        out = LN(residual; next_weight, next_bias) (``out`` None: the sum alone).  With ``rows`` ('plain' and
        'add') only those source rows are normed and the residual is not written.  ``x`` and ``out`` may have
        different element types."""
        x = self.materialize(x)
        width = x.shape[-1]
        code = self._NORM_MODES[mode]
        self._check("norm input", x, (torch.float32, torch.bfloat16), (None, width))
        self._check("norm weight", weight, torch.float32, (width,))
        self._check("norm bias", bias, torch.float32, (width,))
        n_out = rows.numel() if rows is not None else x.shape[0]
        if out is not None:
            self._check("norm out", out, (torch.float32, torch.bfloat16), (n_out, width))
        elif code != 3:
            raise KernelError("norm: only the 'post' mode may leave out its output")
        if code:
            if residual is None:
                raise KernelError("norm: this mode needs the residual stream")
            self._check("residual", residual, torch.float32, tuple(x.shape))
        if rows is not None:
            if code in (1, 3):
                raise KernelError("norm: this mode takes all rows")
            self._check("norm rows", rows, torch.int32, (n_out,))
        if code == 3 and out is not None:
            self._check("next norm weight", next_weight, torch.float32, (width,))
            self._check("next norm bias", next_bias, torch.float32, (width,))
        self._done("layernorm", self.lib.atom_layernorm(
            _ptr(x), self._code(x), _ptr(residual), _ptr(weight), _ptr(bias), _ptr(next_weight), _ptr(next_bias),
            _ptr(out), self._code(out) if out is not None else 0, _ptr(rows), n_out, width, ctypes.c_float(eps), code,
            self._stream()))
        return out

    def embedding_scaled(self, table, ids, out, scale: float):
        """``out = table[ids] * scale`` in float32."""
        vocab, hidden = table.shape
        tokens = ids.numel()
        self._check("embedding table", table, (torch.float32, torch.bfloat16))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("embedding out", out, torch.float32, (tokens, hidden))
        self._done("embedding_scaled", self.lib.atom_embedding_scaled(
            _ptr(table), self._code(table), _ptr(ids), _ptr(out), tokens, hidden, vocab, ctypes.c_float(scale),
            self._stream()))
        return out

    def sum_concat(self, hidden, residual, first, out):
        """``out[t] = [residual[t] + hidden[t] ; first[t]]`` (``residual`` None: hidden alone)."""
        hidden = self.materialize(hidden)
        tokens, width = hidden.shape
        self._check("hidden", hidden, (torch.float32, torch.bfloat16))
        if residual is not None:
            self._check("residual", residual, torch.float32, (tokens, width))
        self._check("first rows", first, torch.float32, (tokens, width))
        self._check("joined rows", out, (torch.float32, torch.bfloat16), (tokens, 2 * width))
        self._done("sum_concat", self.lib.atom_sum_concat(
            _ptr(hidden), self._code(hidden), _ptr(residual), _ptr(first), _ptr(out), self._code(out), tokens, width,
            self._stream()))
        return out

    _ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}

    def gated_act(self, x, out, activation: str):
        """``out = act(gate) * up`` for ``x`` = gate | up."""
        x = self.materialize(x)
        rows, two = x.shape
        if two % 2:
            raise KernelError("gated_act: the input width must be even (gate | up)")
        if activation not in self._ACTIVATIONS:
            raise KernelError(f"gated_act: unknown activation {activation!r}; known: {sorted(self._ACTIVATIONS)}")
        self._check("gated_act input", x, (torch.float32, torch.bfloat16))
        self._check("gated_act out", out, x.dtype, (rows, two // 2))
        self._done("gated_act", self.lib.atom_gated_act(_ptr(x), _ptr(out), self._code(out), rows, two // 2,
                                                        self._ACTIVATIONS[activation], self._stream()))
        return out

    def linear_f32(self, x, weight, bias=None):
        """``x @ weight.T (+ bias)`` summed in float32 whatever the operands' types, float32 out: for the few
        products that have to be 32-bit sums (a router's logits).  bfloat16 operands take the engine's ordinary
        products with float32 output; anything with a float32 operand runs plain float32 multiply-adds."""
        x = self.materialize(x)
        m, k = x.shape
        n = weight.shape[0]
        self._check("linear input", x, (torch.float32, torch.bfloat16))
        self._check("linear weight", weight, (torch.float32, torch.bfloat16), (n, k))
        if bias is not None:
            self._check("linear bias", bias, torch.float32, (n,))
        if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and k % 8 == 0:
            # products of two bfloat16 numbers are exact in float32, and the matrix cores add them in float32
            return self.linear(x, weight, bias, out_dtype=torch.float32)
        y = torch.empty((m, n), dtype=torch.float32, device=x.device)
        self._done("gemm_f32", self.lib.atom_gemm_f32(_ptr(x), self._code(x), _ptr(weight), self._code(weight), _ptr(bias),
                                                      _ptr(y), F32, m, n, k, self._stream()))
        return y

    # ------------------------------------------------------------------ attention over a cache of latents

    def latent_prepare(self, proj, q_off: int, kv_off: int, heads: int, dim: int, rot: int, rank: int, rot_dims: int,
                       norm_weight, eps: float, freq, mult: float, positions, slots, pages, q_abs, q_scale: float):
        """From the float32 product ``proj`` [tokens, *] (queries of ``heads`` x (dim + rot) at ``q_off``, the
        down-projection of rank + rot at ``kv_off``): the RMS-normed latent and the rotated shared key part go to
        row ``slots[t]`` of ``pages`` (None: no write), the queries' rotated parts, times ``q_scale``, to
        ``q_abs[t, h, rank:]``."""
        tokens, ld = proj.shape
        width = rank + rot
        self._check("projections", proj, torch.float32)
        self._check("latent norm weight", norm_weight, torch.float32, (rank,))
        self._check("positions", positions, torch.int32, (tokens,))
        self._check("absorbed queries", q_abs, (torch.float32, torch.bfloat16), (tokens, heads, width))
        if rot_dims:
            self._check("rotation frequencies", freq, torch.float64, (rot_dims // 2,))
        if slots is not None:
            self._check("slot mapping", slots, torch.int32, (tokens,))
            self._check("latent pages", pages, q_abs.dtype, (None, None, width))
        self._done("latent_prepare", self.lib.atom_latent_prepare(
            _ptr(proj), ld, q_off, kv_off, heads, dim, rot, rank, rot_dims, _ptr(norm_weight), ctypes.c_float(eps),
            _ptr(freq) if rot_dims else None, ctypes.c_float(mult), _ptr(positions), _ptr(slots),
            _ptr(pages) if slots is not None else None, _ptr(q_abs), self._code(q_abs), tokens, ctypes.c_float(q_scale),
            self._stream()))
        return q_abs

    def heads_gemm(self, x, x_offset: int, ldx: int, hsx: int, weight, y, y_offset: int, ldy: int, hsy: int, heads: int,
                   m: int, n: int, k: int, alpha: float = 1.0, gate=None, gate_offset: int = 0, ldg: int = 0,
                   exact: bool = False):
        """One small product per head: ``y[t, h, :n] = alpha * x[t, h, :k] @ weight[h].T`` (times
        ``sigmoid(gate[t, h])`` when given), with ``x`` and ``y`` addressed as flat arrays: element (t, h, i) of x
        sits at ``x_offset + t * ldx + h * hsx + i``.  ``weight`` is [heads, n, k].  ``exact``: a float32 input is
        multiplied as it is, not rounded for the matrix cores: float32 multiply-adds for few rows or float32
        weights, and for many rows with bfloat16 weights the matrix cores on the input's three bfloat16 pieces,
        whose products with a bfloat16 weight are exact."""
        self._check("per-head input", x, (torch.float32, torch.bfloat16))
        self._check("per-head weight", weight, (torch.float32, torch.bfloat16), (heads, n, k))
        self._check("per-head out", y, (torch.float32, torch.bfloat16))
        if m:
            if x_offset + (m - 1) * ldx + (heads - 1) * hsx + k > x.numel():
                raise KernelError("heads_gemm: the input is smaller than its strides say")
            if y_offset + (m - 1) * ldy + (heads - 1) * hsy + n > y.numel():
                raise KernelError("heads_gemm: the output is smaller than its strides say")
        gp = None
        if gate is not None:
            self._check("per-head gate", gate, torch.float32)
            if m and gate_offset + (m - 1) * ldg + heads > gate.numel():
                raise KernelError("heads_gemm: the gate is smaller than its strides say")
            gp = ctypes.c_void_p(gate.data_ptr() + 4 * gate_offset)
        xp = ctypes.c_void_p(x.data_ptr() + x.element_size() * x_offset)
        yp = ctypes.c_void_p(y.data_ptr() + y.element_size() * y_offset)
        split = bool(exact and x.dtype == torch.float32)
        if (weight.dtype == torch.bfloat16 and m >= (self.heads_split_from if split else self.heads_mfma_from)
                and self.lib.atom_heads_gemm_mfma_supports(
                self._code(x), BF16, ctypes.c_long(x_offset), ctypes.c_long(ldx), ctypes.c_long(hsx), k)):
            # many rows: the same product on the matrix cores (a float32 input is rounded to bfloat16 on the way in)
            self._done("heads_gemm_mfma", self.lib.atom_heads_gemm_mfma(
                xp, self._code(x), ctypes.c_long(ldx), ctypes.c_long(hsx), _ptr(weight), yp, self._code(y),
                ctypes.c_long(ldy), ctypes.c_long(hsy), gp, ctypes.c_long(ldg), heads, m, n, k, ctypes.c_float(alpha),
                int(split), self._stream()))
            return y
        self._done("heads_gemm", self.lib.atom_heads_gemm(
            xp, self._code(x), ctypes.c_long(ldx), ctypes.c_long(hsx), _ptr(weight), self._code(weight), yp,
            self._code(y), ctypes.c_long(ldy), ctypes.c_long(hsy), gp, ctypes.c_long(ldg), heads, m, n, k,
            ctypes.c_float(alpha), self._stream()))
        return y

    def latent_parts(self, meta: AttentionMeta, heads: int, window: int | None) -> int:
        """Over how many blocks a row's keys are split in the matrix-core kernel: one for steps with prompt
        portions (their tiles fill the chip); for single tokens enough blocks to fill it twice, 128 keys each at
        least."""
        if meta.max_q_len > 1:
            return 1
        blocks = max(1, meta.num_seqs * -(-heads // 64))
        visible = min(meta.max_context_len, window) if window else meta.max_context_len
        return max(1, min(-(-2 * self.num_cus // blocks), -(-visible // 128), 64))

    def latent_attention(self, q_abs, pages, out, meta: AttentionMeta, rank: int, sink=None, window: int | None = None,
                         parts: int | None = None):
        """Attention of ``q_abs`` [tokens, heads, rank + rot] over pages [num_pages, page_size, rank + rot] whose
        rows are shared by all heads; the weighted sums of the rows' first ``rank`` entries land in ``out``
        [tokens, heads, rank].  ``sink`` [heads] joins every softmax's denominator.  bfloat16 with sizes the
        matrix-core kernel is built for runs there (``parts``: blocks a row's keys are split over), anything else
        the general kernel."""
        tokens, heads, width = q_abs.shape
        dt = q_abs.dtype
        self._check("absorbed queries", q_abs, (torch.float32, torch.bfloat16))
        self._check("latent pages", pages, dt, (None, meta.page_size, width))
        self._check("attention out", out, dt, (tokens, heads, rank))
        self._check("token_seq", meta.token_seq, torch.int32, (tokens,))
        self._check("positions", meta.positions, torch.int32, (tokens,))
        self._check("block tables", meta.block_tables, torch.int32, (None, None))
        if sink is not None:
            self._check("sink", sink, torch.float32, (heads,))
        if meta.max_context_len > meta.block_tables.shape[1] * meta.page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        if dt == torch.bfloat16 and self.use_mfma_latent and self.lib.atom_latent_mfma_supports(rank, width):
            self._check("cu_seqlens_q", meta.cu_seqlens_q, torch.int32, (meta.num_seqs + 1,))
            self._check("context_lens", meta.context_lens, torch.int32, (meta.num_seqs,))
            if meta.block_tables.shape[0] != meta.num_seqs:
                raise KernelError("attention: one block table row per request is needed")
            if parts is None:
                parts = self.latent_parts(meta, heads, window)
            ws_o = ws_ml = None
            if parts > 1:
                ws_o = self.workspace("latent_o", tokens * heads * parts * rank)
                ws_ml = self.workspace("latent_ml", tokens * heads * parts * 2)
            self._done("latent_attention_mfma", self.lib.atom_latent_attention_mfma(
                _ptr(q_abs), _ptr(pages), _ptr(out), _ptr(ws_o), _ptr(ws_ml), _ptr(meta.cu_seqlens_q),
                _ptr(meta.context_lens), _ptr(meta.block_tables), meta.block_tables.shape[1], _ptr(sink), meta.num_seqs,
                tokens, heads, rank, width, meta.page_size, int(window or 0), parts, self._stream()))
            return out
        self._done("latent_attention", self.lib.atom_latent_attention(
            _ptr(q_abs), _ptr(pages), _ptr(out), _ptr(meta.token_seq), _ptr(meta.positions), _ptr(meta.block_tables),
            meta.block_tables.shape[1], _ptr(sink), self._code(q_abs), tokens, heads, rank, width - rank,
            meta.page_size, int(window or 0), self._stream()))
        return out

    # ------------------------------------------------------------------ the gated delta rule

    def conv_silu_state(self, x, channels: int, taps_weight, state, cu_seqlens_q, slot_of_seq, out,
                        max_q_len: int | None = None, bias=None, activation: str = "silu", x_offset: int = 0):
        """Short causal convolution per channel over each request's tokens (plus ``bias`` per channel when given),
        then SiLU (``activation`` "none": nothing).  ``x`` float32 [tokens, >=
        channels] (the first ``channels`` columns are convolved); ``taps_weight`` [channels, taps], last column the
        current token's; ``state`` float32 [slots, >= (taps - 1) * channels]: a request's last taps - 1 inputs, read
        and written back.  Requests with slot -1 are padding.  ``max_q_len``: the most tokens a request brings (an
        upper bound sizes the grid; default: all tokens)."""
        tokens, ldx = x.shape
        taps = taps_weight.shape[1]
        seqs = slot_of_seq.numel()
        self._check("convolution input", x, torch.float32)
        self._check("taps", taps_weight, (torch.float32, torch.bfloat16), (channels, taps))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("convolution out", out, torch.float32, (tokens, channels))
        if bias is not None:
            self._check("convolution bias", bias, torch.float32, (channels,))
        if activation not in ("silu", "none"):
            raise KernelError(f"conv_silu_state: unknown activation {activation!r}")
        if x_offset < 0 or ldx < x_offset + channels or state.shape[1] < (taps - 1) * channels:
            raise KernelError("conv_silu_state: the input or the state is narrower than the channels need")
        self._done("conv_silu_state", self.lib.atom_conv_silu_state(
            ctypes.c_void_p(x.data_ptr() + 4 * x_offset), ldx, _ptr(taps_weight), self._code(taps_weight), taps, channels, _ptr(state),
            ctypes.c_long(state.shape[1]), _ptr(cu_seqlens_q), _ptr(slot_of_seq), seqs,
            tokens if max_q_len is None else min(tokens, max_q_len), _ptr(out), _ptr(bias),
            0 if activation == "silu" else 1, self._stream()))
        return out

    def delta_rule(self, qkv, gates, a_off: int, b_off: int, a_log, dt_bias, state, state_off: int, cu_seqlens_q,
                   slot_of_seq, out, heads: int, kv_heads: int, dim: int, vdim: int, decay=None,
                   per_channel: bool = False):
        """The gated delta recurrence over each request's tokens.  ``qkv`` float32 [tokens, 2 kv_heads dim + heads
        vdim] (q | k | v after convolution and SiLU); ``gates`` float32 [tokens, *] with the raw beta inputs at
        ``b_off`` and, unless ``decay`` (float32 [tokens, *]) holds them, the raw decay inputs at ``a_off``: one
        per head, or with ``per_channel`` one per head and key channel (``dt_bias`` likewise); the heads' matrices
        [heads, dim, vdim] start at ``state_off`` of a slot's row of ``state``.  ``out`` float32 [tokens, heads,
        vdim].  ``qkv`` and the decay inputs are used up: q and k are made unit vectors and the raw decay inputs
        become the decays, in place, for all tokens side by side before the recurrence walks them."""
        tokens, channels = qkv.shape
        seqs = slot_of_seq.numel()
        decay = gates if decay is None else decay
        wide = heads * (dim if per_channel else 1)
        self._check("delta decay inputs", decay, torch.float32, (tokens, None))
        if a_off < 0 or a_off + wide > decay.shape[1]:
            raise KernelError("delta_rule: the decay inputs do not fit their tensor")
        self._check("delta q|k|v", qkv, torch.float32, (tokens, 2 * kv_heads * dim + heads * vdim))
        self._check("delta gates", gates, torch.float32, (tokens, None))
        self._check("A_log", a_log, torch.float32, (heads,))
        self._check("dt_bias", dt_bias, torch.float32, (wide,))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("delta out", out, torch.float32, (tokens, heads, vdim))
        self._done("delta_rule", self.lib.atom_delta_rule(
            _ptr(qkv), tokens, channels, _ptr(gates), gates.shape[1], _ptr(decay), decay.shape[1], a_off, b_off,
            int(bool(per_channel)), _ptr(a_log), _ptr(dt_bias), _ptr(state),
            ctypes.c_long(state.shape[1]), ctypes.c_long(state_off), _ptr(cu_seqlens_q), _ptr(slot_of_seq), seqs,
            _ptr(out), heads, kv_heads, dim, vdim, self._stream()))
        return out

    def delta_out(self, o, gates, gate_off: int, weight, eps: float, out, activation: str = "silu"):
        """``out[t, h] = o[t, h] / rms(o[t, h]) * weight * silu(gate[t, h])`` (``activation`` "sigmoid": times the
        gate's sigmoid) with the gate's rows at ``gate_off`` of ``gates`` (float32)."""
        if activation not in ("silu", "sigmoid"):
            raise KernelError(f"delta_out: unknown activation {activation!r}")
        tokens, heads, vdim = o.shape
        self._check("read-out", o, torch.float32)
        self._check("gates", gates, torch.float32, (tokens, None))
        self._check("read-out norm weight", weight, torch.float32, (vdim,))
        self._check("gated read-out", out, (torch.float32, torch.bfloat16), (tokens, heads * vdim))
        self._done("delta_out", self.lib.atom_delta_out(
            _ptr(o), _ptr(gates), gates.shape[1], gate_off, _ptr(weight), ctypes.c_float(eps), _ptr(out),
            self._code(out), tokens, heads, vdim, 0 if activation == "silu" else 1, self._stream()))
        return out

    # ------------------------------------------------------------------ linear recurrences with a matrix state

    @staticmethod
    def _at(t: torch.Tensor, offset: int):
        return ctypes.c_void_p(t.data_ptr() + t.element_size() * offset)

    SCAN_RUN = 64     # tokens of a run of the linear recurrences (a multiple of 16)

    def linear_scan(self, r, r_off: int, r_heads: int, k, k_off: int, k_heads: int, v, v_off: int, w, w_off: int,
                    state, state_off: int, cu_seqlens_q, slot_of_seq, out, heads: int, dim: int, vdim: int,
                    per_channel: bool = True, w_bias=None, v_scale=None, bonus=None, skip=None,
                    max_q_len: int | None = None, step_bias=None, a_log=None):
        """A linear recurrence with a state of ``dim`` x ``vdim`` per head over each request's tokens:
        ``S <- diag(w) S + k v^T`` with the read-out ``o = (S_before + diag(bonus) k v^T)^T r`` where ``bonus``
        [heads, dim] is given, else ``o = S_after^T r``.  All inputs float32 [tokens, *], read from a column offset:
        ``r`` and ``k`` hold ``r_heads`` / ``k_heads`` heads of ``dim`` entries (head h reads head
        ``h // (heads / r_heads)``), ``v`` ``heads`` x ``vdim``, ``w`` the decays, ``heads`` x ``dim`` with
        ``per_channel`` and else one per head; with ``w_bias`` [heads, dim] the decay is ``exp(-exp(w + w_bias))``.
        With ``a_log`` [heads] and ``step_bias`` [heads] (one decay per head) ``w`` holds raw step sizes:
        ``step = softplus(w + step_bias)`` multiplies v on its way into the state and the decay is
        ``exp(-exp(a_log) step)``.  ``v_scale`` [tokens, heads] multiplies v on its way into the state; ``skip`` [heads] adds ``skip * v`` (v as
        given) to the read-out.  The heads' matrices [heads, dim, vdim] start at ``state_off`` of a slot's row of
        ``state``; requests with slot -1 are padding.  ``out`` float32 [tokens, heads * vdim].  ``max_q_len``: the most tokens a
        request brings (an upper bound; default: all tokens); beyond ``SCAN_RUN`` tokens requests are cut into runs of
        that length that are worked side by side, through scratch memory of a state per run."""
        tokens = out.shape[0]
        seqs = slot_of_seq.numel()
        if heads % r_heads or heads % k_heads:
            raise KernelError("linear_scan: the heads are not a multiple of the r or k heads")
        for name, t, off, wide in (("r", r, r_off, r_heads * dim), ("k", k, k_off, k_heads * dim),
                                   ("v", v, v_off, heads * vdim), ("w", w, w_off, heads * (dim if per_channel else 1))):
            self._check(f"scan {name}", t, torch.float32, (tokens, None))
            if off < 0 or off + wide > t.shape[1]:
                raise KernelError(f"linear_scan: {name} does not fit its tensor")
        self._check("scan out", out, torch.float32, (tokens, heads * vdim))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        if w_bias is not None:
            self._check("decay bias", w_bias, torch.float32, (heads * dim,))
        if v_scale is not None:
            self._check("step sizes", v_scale, torch.float32, (tokens, heads))
        mode, bias = (1, w_bias) if w_bias is not None else (0, None)
        if a_log is not None:
            if per_channel or w_bias is not None or v_scale is not None or bonus is not None or step_bias is None:
                raise KernelError("linear_scan: raw step sizes go with one decay per head, a step bias and nothing else")
            self._check("A_log", a_log, torch.float32, (heads,))
            self._check("step bias", step_bias, torch.float32, (heads,))
            mode, bias = 2, step_bias
        if bonus is not None:
            self._check("bonus", bonus, torch.float32, (heads, dim))
        if skip is not None:
            self._check("skip", skip, torch.float32, (heads,))
        L = ctypes.c_long
        longest = tokens if max_q_len is None else min(tokens, max_q_len)
        run_len, places, run_state, run_decay = 0, 0, None, None
        if longest > self.SCAN_RUN:
            run_len = self.SCAN_RUN
            places = -(-tokens // run_len) + seqs
            run_state = torch.empty((places, heads, dim, vdim), dtype=torch.float32, device=out.device)
            run_decay = torch.empty((places, heads, dim), dtype=torch.float32, device=out.device)
        self._done("linear_scan", self.lib.atom_linear_scan(
            self._at(r, r_off), L(r.shape[1]), heads // r_heads, self._at(k, k_off), L(k.shape[1]), heads // k_heads,
            self._at(v, v_off), L(v.shape[1]), self._at(w, w_off), L(w.shape[1]), int(bool(per_channel)), _ptr(bias),
            mode, _ptr(a_log), _ptr(v_scale), L(heads), _ptr(bonus), _ptr(skip), _ptr(out),
            L(heads * vdim), _ptr(state), L(state.shape[1]), L(state_off), _ptr(cu_seqlens_q), _ptr(slot_of_seq), seqs,
            heads, dim, vdim, tokens, run_len, _ptr(run_state), _ptr(run_decay), L(places), self._stream()))
        return out

    def token_shift(self, x, mu, mixes, state, state_off: int, cu_seqlens_q, slot_of_seq, token_seq):
        """``mixes[s, t] = x[t] + (x[t - 1] - x[t]) * mu[s]``; the row before a request's first token of the step is
        what its state slot holds at ``state_off`` (float32, zeros for a fresh request), and the request's last row
        of the step is left there."""
        tokens, width = x.shape
        n = mu.shape[0]
        seqs = slot_of_seq.numel()
        self._check("shift input", x, (torch.float32, torch.bfloat16))
        self._check("shift weights", mu, torch.float32, (n, width))
        self._check("shifted mixes", mixes, x.dtype, (n, tokens, width))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("token_seq", token_seq, torch.int32, (tokens,))
        self._done("token_shift", self.lib.atom_token_shift(
            _ptr(x), self._code(x), _ptr(mu), n, _ptr(mixes), _ptr(state), ctypes.c_long(state.shape[1]),
            ctypes.c_long(state_off), _ptr(cu_seqlens_q), _ptr(slot_of_seq), _ptr(token_seq), tokens, width,
            self._stream()))
        return mixes

    def step_decay(self, raw, raw_off: int, dt_bias, a_log, dt, decay):
        """``dt = softplus(raw + dt_bias)``, ``decay = exp(-exp(a_log) dt)`` per (token, head); ``raw`` float32
        [tokens, *] read from column ``raw_off``."""
        tokens, heads = dt.shape
        self._check("raw step sizes", raw, torch.float32, (tokens, None))
        if raw_off < 0 or raw_off + heads > raw.shape[1]:
            raise KernelError("step_decay: the raw step sizes do not fit their tensor")
        self._check("dt_bias", dt_bias, torch.float32, (heads,))
        self._check("A_log", a_log, torch.float32, (heads,))
        self._check("step sizes", dt, torch.float32, (tokens, heads))
        self._check("decays", decay, torch.float32, (tokens, heads))
        self._done("step_decay", self.lib.atom_step_decay(
            self._at(raw, raw_off), ctypes.c_long(raw.shape[1]), _ptr(dt_bias), _ptr(a_log), _ptr(dt), _ptr(decay),
            tokens, heads, self._stream()))
        return dt, decay

    def group_norm_gate(self, y, groups: int, weight, eps: float, out, gate=None, gate_off: int = 0,
                        gate_first: bool = False):
        """RMS norm of each of ``groups`` equal parts of a row of ``y`` (float32), times ``weight`` (one per entry;
        None: ones), with a SiLU gate from column ``gate_off`` of ``gate`` (float32) that multiplies the row before
        the norm (``gate_first``) or after it."""
        tokens, width = y.shape
        if width % groups:
            raise KernelError(f"group_norm_gate: {width} entries do not split into {groups} equal parts")
        self._check("rows to norm", y, torch.float32)
        if weight is not None:
            self._check("norm weight", weight, torch.float32, (width,))
        self._check("normed rows", out, (torch.float32, torch.bfloat16), (tokens, width))
        gp, ldg = None, 0
        if gate is not None:
            self._check("gate", gate, torch.float32, (tokens, None))
            if gate_off < 0 or gate_off + width > gate.shape[1]:
                raise KernelError("group_norm_gate: the gate does not fit its tensor")
            gp, ldg = self._at(gate, gate_off), gate.shape[1]
        self._done("group_norm_gate", self.lib.atom_group_norm_gate(
            _ptr(y), ctypes.c_long(width), gp, ctypes.c_long(ldg), _ptr(weight), _ptr(out), self._code(out), tokens,
            groups, width // groups, ctypes.c_float(eps), int(bool(gate_first)), self._stream()))
        return out

    # ------------------------------------------------------------------ attention without rotation

    def qkv_plain_write(self, proj, q_out, k_cache, v_cache, positions, slots, num_heads: int, num_kv_heads: int,
                        head_dim: int, value_dim: int, page_size: int, unit_norm: bool, eps: float,
                        temperature: tuple | None = None, write_kv: bool = True):
        """From the float32 product ``proj`` [tokens, q | k | v]: q (with ``unit_norm`` divided by each head's root
        mean square, as k is; times the token's temperature ``1 + coef ln(floor((p + 1) / every) + 1)`` for
        ``temperature`` = (coef, every)) to ``q_out`` [tokens, heads, padded], k and v to the pages, whose head
        size ``padded`` >= max(head_dim, value_dim) is ``q_out``'s; what lies beyond a head's own entries is zero."""
        tokens = proj.shape[0]
        dp = q_out.shape[2]
        dt = q_out.dtype
        self._check("q|k|v", proj, torch.float32, (tokens, None))
        if proj.shape[1] < (num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim:
            raise KernelError("qkv_plain_write: the product is narrower than its heads")
        self._check("q out", q_out, (torch.float32, torch.bfloat16), (tokens, num_heads, dp))
        if dp < head_dim or dp < value_dim:
            raise KernelError("qkv_plain_write: the padded head size is smaller than a head")
        if write_kv:
            self._check("key pages", k_cache, dt, (None, num_kv_heads, page_size, dp))
            self._check("value pages", v_cache, dt, (k_cache.shape[0], num_kv_heads, dp, page_size))
            self._check("slot mapping", slots, torch.int32, (tokens,))
        coef, every = (float(temperature[0]), int(temperature[1])) if temperature else (0.0, 1)
        if coef != 0.0:
            if every <= 0:
                raise KernelError("qkv_plain_write: the temperature's step must be positive")
            self._check("positions", positions, torch.int32, (tokens,))
        self._done("qkv_plain_write", self.lib.atom_qkv_plain_write(
            _ptr(proj), ctypes.c_long(proj.shape[1]), _ptr(q_out), _ptr(k_cache) if write_kv else None,
            _ptr(v_cache) if write_kv else None, self._code(q_out), _ptr(positions) if coef != 0.0 else None,
            _ptr(slots) if write_kv else None, tokens, num_heads, num_kv_heads, head_dim, value_dim, dp, page_size,
            int(bool(unit_norm)), ctypes.c_float(eps), ctypes.c_float(coef), every, self._stream()))
        return q_out

    def narrow_heads(self, x, value_dim: int):
        """The first ``value_dim`` entries of every head of ``x`` [tokens, heads, padded], as [tokens, heads *
        value_dim]."""
        tokens, heads, dp = x.shape
        self._check("padded heads", x, (torch.float32, torch.bfloat16))
        if value_dim == dp:
            return x.view(tokens, heads * dp)
        out = torch.empty((tokens, heads * value_dim), dtype=x.dtype, device=x.device)
        self._done("narrow_heads", self.lib.atom_narrow_heads(_ptr(x), _ptr(out), self._code(x),
                                                              ctypes.c_long(tokens * heads), dp, value_dim, self._stream()))
        return out

    def mean_of_norms(self, xs, weights, eps: float, out):
        """``out = mean_b(xs[b] / rms(xs[b]) * weights[b])`` over up to four inputs of ``out``'s shape and type."""
        n = len(xs)
        if not 1 <= n <= 4 or len(weights) != n:
            raise KernelError("mean_of_norms: one to four inputs, a weight each")
        tokens, width = out.shape
        self._check("mean of norms", out, (torch.float32, torch.bfloat16))
        xs = [self.materialize(x) for x in xs]
        for x, w in zip(xs, weights):
            self._check("normed input", x, out.dtype, (tokens, width))
            self._check("norm weight", w, torch.float32, (width,))
        xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
        wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
        self._done("mean_of_norms", self.lib.atom_mean_of_norms(xp, wp, n, _ptr(out), self._code(out), tokens, width,
                                                                ctypes.c_float(eps), self._stream()))
        return out

    def embedding_positions(self, table, rows, ids, positions, out):
        """``out = table[ids] + rows[positions]`` in float32."""
        vocab, hidden = table.shape
        tokens = ids.numel()
        self._check("embedding table", table, (torch.float32, torch.bfloat16))
        self._check("position rows", rows, table.dtype, (None, hidden))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("positions", positions, torch.int32, (tokens,))
        self._check("embedding out", out, torch.float32, (tokens, hidden))
        self._done("embedding_positions", self.lib.atom_embedding_positions(
            _ptr(table), _ptr(rows), self._code(table), _ptr(ids), _ptr(positions), _ptr(out), tokens, hidden, vocab,
            rows.shape[0], self._stream()))
        return out

    def scale_rows(self, x, scale: float):
        """``x *= scale`` in place for a float32 ``x``."""
        self._check("rows to scale", x, torch.float32)
        self._done("scale_rows", self.lib.atom_scale_rows(_ptr(x), ctypes.c_long(x.numel()), ctypes.c_float(scale),
                                                          self._stream()))
        return x

    _UNARY = {"silu": 0, "relu": 1, "gelu_tanh": 2, "relu_squared": 3, "tanh": 4}

    def unary_act(self, x, out, activation: str):
        """``out = act(x)`` entry by entry."""
        x = self.materialize(x)
        if activation not in self._UNARY:
            raise KernelError(f"unary_act: unknown activation {activation!r}; known: {sorted(self._UNARY)}")
        self._check("activation input", x, (torch.float32, torch.bfloat16))
        self._check("activation out", out, x.dtype, tuple(x.shape))
        self._done("unary_act", self.lib.atom_unary_act(_ptr(x), _ptr(out), self._code(x), ctypes.c_long(x.numel()),
                                                        self._UNARY[activation], self._stream()))
        return out

    # ------------------------------------------------------------------ a float32 stream with normed summands

    def rmsnorm_post(self, x, weight, eps: float, stream, out=None):
        """``stream += x / rms(x) * weight`` in float32 (``stream`` float32, in place); ``out``, when given,
        receives the stream's new rows in its own type."""
        x = self.materialize(x)
        rows, width = x.shape
        self._check("norm input", x, (torch.float32, torch.bfloat16), (rows, width))
        self._check("norm weight", weight, torch.float32, (width,))
        self._check("stream", stream, torch.float32, (rows, width))
        if out is not None:
            self._check("stream copy", out, (torch.float32, torch.bfloat16), (rows, width))
        self._done("rmsnorm_post", self.lib.atom_rmsnorm_post(
            _ptr(x), self._code(x), _ptr(weight), ctypes.c_float(eps), _ptr(stream), _ptr(out),
            self._code(out) if out is not None else 0, rows, width, self._stream()))
        return out

    def rmsnorm_rows(self, x, weight, eps: float, rows, out):
        """``out[r] = norm(x[rows[r]]) * weight`` for float32 ``x``, written in ``out``'s type (``rows`` None: every
        row in turn)."""
        n, width = x.shape
        self._check("norm input", x, torch.float32, (n, width))
        self._check("norm weight", weight, torch.float32, (width,))
        if rows is not None:
            self._check("norm rows", rows, torch.int32, (None,))
        n_out = rows.numel() if rows is not None else n
        self._check("norm out", out, (torch.float32, torch.bfloat16), (n_out, width))
        self._done("rmsnorm_rows", self.lib.atom_rmsnorm_rows(
            _ptr(x), _ptr(weight), ctypes.c_float(eps), _ptr(rows), n, _ptr(out), self._code(out), n_out, width,
            self._stream()))
        return out

    def stream_norm(self, stream, x, weight, eps: float, out, init: bool = False):
        """``stream += x`` (``init``: ``stream = x``) for float32 rows, and ``out = norm(stream) * weight`` in
        ``out``'s type, one kernel."""
        n, width = stream.shape
        self._check("stream", stream, torch.float32, (n, width))
        self._check("summand", x, torch.float32, (n, width))
        self._check("norm weight", weight, torch.float32, (width,))
        self._check("norm out", out, (torch.float32, torch.bfloat16), (n, width))
        self._done("stream_norm", self.lib.atom_stream_norm(
            _ptr(stream), _ptr(x), _ptr(weight), ctypes.c_float(eps), _ptr(out), self._code(out), n, width,
            int(bool(init)), self._stream()))
        return out

    def stream_add(self, stream, x, init: bool = False):
        """``stream += x`` (``init``: ``stream = x``) for a float32 ``stream`` and an ``x`` of any type."""
        x = self.materialize(x)
        self._check("stream", stream, torch.float32)
        self._check("summand", x, (torch.float32, torch.bfloat16), tuple(stream.shape))
        self._done("stream_add", self.lib.atom_stream_add(_ptr(stream), _ptr(x), self._code(x),
                                                          ctypes.c_long(stream.numel()), int(bool(init)), self._stream()))
        return stream

    def cast_rows(self, x, dtype):
        """Float32 rows in another type."""
        self._check("rows", x, torch.float32)
        out = torch.empty(tuple(x.shape), dtype=dtype, device=x.device)
        self._done("cast_rows", self.lib.atom_cast_rows(_ptr(x), _ptr(out), self._code(out), ctypes.c_long(x.numel()),
                                                        self._stream()))
        return out

    def token_gate(self, raw, table, col_off: int, ids, out):
        """``out[t, j] = gelu_tanh(raw[t, j]) * table[ids[t], col_off + j]``."""
        tokens, dim = raw.shape
        self._check("gate input", raw, torch.float32, (tokens, dim))
        self._check("token table", table, (torch.float32, torch.bfloat16), (None, None))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("gated rows", out, (torch.float32, torch.bfloat16), (tokens, dim))
        if col_off < 0 or col_off + dim > table.shape[1]:
            raise KernelError("token_gate: the columns asked for are not in the table")
        self._done("token_gate", self.lib.atom_token_gate(
            _ptr(raw), _ptr(table), self._code(table), table.shape[1], col_off, _ptr(ids), table.shape[0], _ptr(out),
            self._code(out), tokens, dim, self._stream()))
        return out

    def embedding_bigram(self, table, pairs, ids, state, cu_seqlens_q, slot_of_seq, token_seq, out, buckets: int,
                         mul_prev: int, mul_cur: int):
        """``out[t] = table[id] + pairs[(previous id * mul_prev + id * mul_cur) mod buckets]`` in float32, row
        ``buckets`` of ``pairs`` for a request's first token.  ``state`` int32 [slots, 1] holds a request's last
        token + 1 between steps (0: none yet) and is moved on."""
        vocab, hidden = table.shape
        tokens, seqs = ids.numel(), slot_of_seq.numel()
        self._check("embedding table", table, (torch.float32, torch.bfloat16))
        self._check("pair table", pairs, table.dtype, (buckets + 1, hidden))
        self._check("token ids", ids, torch.int32, (tokens,))
        self._check("previous tokens", state, torch.int32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("token_seq", token_seq, torch.int32, (tokens,))
        self._check("embedding out", out, torch.float32, (tokens, hidden))
        self._done("embedding_bigram", self.lib.atom_embedding_bigram(
            _ptr(table), _ptr(pairs), self._code(table), _ptr(ids), _ptr(state), ctypes.c_long(state.shape[1]),
            _ptr(cu_seqlens_q), _ptr(slot_of_seq), _ptr(token_seq), _ptr(out), tokens, hidden, vocab, buckets,
            ctypes.c_long(mul_prev), ctypes.c_long(mul_cur), self._stream()))
        return out

    # ------------------------------------------------------------------ the real-gated linear recurrence

    #: tokens of a run of the gated recurrence's scan (the kernel's own constant)
    RGLRU_RUN = 64

    def rglru_scan(self, u, gates, ra_bias, ri_bias, lam, proj, y_off: int, state, state_off: int, cu_seqlens_q,
                   slot_of_seq, out, decay_scale: float, max_q_len: int | None = None):
        """``S <- a S + sqrt(1 - a^2) (i u)``, ``out = S * gelu_tanh(y)`` over each request's tokens, with
        ``r = sigmoid(gates[0] + ra_bias)``, ``i = sigmoid(gates[1] + ri_bias)``, ``a = exp(-decay_scale r
        softplus(lam))``.  ``u`` float32 [tokens, channels]; ``gates`` float32 [2, tokens, channels]; ``y`` the
        ``channels`` columns of ``proj`` (float32) from ``y_off``; S at ``state_off`` of a slot's row of ``state``.
        ``max_q_len``: the most tokens a request brings (an upper bound; default: all tokens); beyond a run's
        length, runs of a request are scanned side by side."""
        tokens, channels = u.shape
        seqs = slot_of_seq.numel()
        self._check("recurrence input", u, torch.float32, (tokens, channels))
        self._check("recurrence gates", gates, torch.float32, (2, tokens, channels))
        self._check("recurrence gate bias", ra_bias, torch.float32)
        self._check("input gate bias", ri_bias, torch.float32)
        if ra_bias.numel() != channels or ri_bias.numel() != channels:
            raise KernelError("rglru_scan: the gates' biases need one entry per channel")
        self._check("decay parameter", lam, torch.float32, (channels,))
        self._check("branches", proj, torch.float32, (tokens, None))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("recurrence out", out, (torch.float32, torch.bfloat16), (tokens, channels))
        gi = ctypes.c_void_p(gates.data_ptr() + 4 * tokens * channels)
        longest = tokens if max_q_len is None else min(tokens, max_q_len)
        ws, ws_floats = None, 0
        if longest > self.RGLRU_RUN:
            ws_floats = seqs * channels * (1 + 2 * -(-longest // self.RGLRU_RUN))
            ws = self.workspace("rglru_runs", ws_floats)
        self._done("rglru_scan", self.lib.atom_rglru_scan(
            _ptr(u), _ptr(gates), gi, _ptr(ra_bias), _ptr(ri_bias), _ptr(lam), _ptr(proj), proj.shape[1], y_off,
            _ptr(state), ctypes.c_long(state.shape[1]), ctypes.c_long(state_off), _ptr(cu_seqlens_q), _ptr(slot_of_seq),
            seqs, _ptr(out), self._code(out), channels, ctypes.c_float(decay_scale), longest, _ptr(ws),
            ctypes.c_long(ws_floats), self._stream()))
        return out

    # ------------------------------------------------------------------ attention whose values are its keys

    def keys_as_values_write(self, proj, q_out, k_cache, v_cache, q_weight, k_weight, freq, rot_dims: int, positions,
                             slots, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, eps: float,
                             write_kv: bool = True):
        """From the float32 product ``proj`` [tokens, >= (heads + kv_heads) dim] (q | k | ...): q and k RMS-normed
        over their whole rows (weights [heads dim] and [kv_heads dim]; None: no norm), pairs (2i, 2i + 1) of the
        first ``rot_dims`` entries of each head turned by ``position * freq[i]``; q to ``q_out``, the normed and
        rotated k to the key pages, k as projected to the value pages."""
        tokens, ld = proj.shape
        self._check("projections", proj, torch.float32)
        if ld < (num_heads + num_kv_heads) * head_dim:
            raise KernelError("keys_as_values_write: the product is narrower than q and k")
        self._check("q out", q_out, (torch.float32, torch.bfloat16), (tokens, num_heads, head_dim))
        dt = q_out.dtype
        if q_weight is not None:
            self._check("q norm weight", q_weight, torch.float32, (num_heads * head_dim,))
        if k_weight is not None:
            self._check("k norm weight", k_weight, torch.float32, (num_kv_heads * head_dim,))
        if rot_dims:
            self._check("rotation frequencies", freq, torch.float64, (rot_dims // 2,))
            self._check("positions", positions, torch.int32, (tokens,))
        if write_kv:
            self._check("key pages", k_cache, dt, (None, num_kv_heads, page_size, head_dim))
            self._check("value pages", v_cache, dt, (k_cache.shape[0], num_kv_heads, head_dim, page_size))
            self._check("slot mapping", slots, torch.int32, (tokens,))
        self._done("keys_as_values_write", self.lib.atom_keys_as_values_write(
            _ptr(proj), ld, _ptr(q_out), _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None,
            self._code(q_out), _ptr(q_weight), _ptr(k_weight), _ptr(freq) if rot_dims else None, rot_dims,
            _ptr(positions) if rot_dims else None, _ptr(slots) if write_kv else None, tokens, num_heads, num_kv_heads,
            head_dim, page_size, ctypes.c_float(eps), self._stream()))
        return q_out

    def sigmoid_gate(self, x, gates, gate_off: int, out):
        """``out = x * sigmoid(gates[:, gate_off : gate_off + width])`` (``gates`` float32)."""
        rows, width = x.shape
        self._check("gated input", x, (torch.float32, torch.bfloat16), (rows, width))
        self._check("gates", gates, torch.float32, (rows, None))
        self._check("gated out", out, x.dtype, (rows, width))
        if gate_off < 0 or gate_off + width > gates.shape[1]:
            raise KernelError("sigmoid_gate: the gate's columns are not in their tensor")
        self._done("sigmoid_gate", self.lib.atom_sigmoid_gate(
            _ptr(x), self._code(x), _ptr(gates), gates.shape[1], gate_off, _ptr(out), rows, width, self._stream()))
        return out

    # ------------------------------------------------------------------ routed experts

    # ------------------------------------------------------------------ a stream normed after every sum; heads together

    def sum_norm(self, stream, alpha: float, summands, scales, weight, eps: float, out=None):
        """``stream <- rms_norm(alpha * stream + sum_i scales[i] * summands[i]) * weight`` in float32, in place
        (``weight`` None: the sum alone; ``alpha`` 0: the stream's old rows are not read); up to four summands of
        float32 or bfloat16.  ``out``, when given, receives the new rows in its own type.  Returns ``stream``."""
        rows, width = stream.shape
        self._check("stream", stream, torch.float32, (rows, width))
        summands = [self.materialize(y) for y in summands]
        if len(summands) > 4 or len(summands) != len(scales):
            raise KernelError("sum_norm: up to four summands, a scale each")
        for y in summands:
            self._check("summand", y, (torch.float32, torch.bfloat16), (rows, width))
        if weight is not None:
            self._check("norm weight", weight, torch.float32, (width,))
        if out is not None:
            self._check("stream copy", out, (torch.float32, torch.bfloat16), (rows, width))
        terms = []
        for i in range(4):
            if i < len(summands):
                terms += [_ptr(summands[i]), self._code(summands[i]), ctypes.c_float(scales[i])]
            else:
                terms += [None, 0, ctypes.c_float(0.0)]
        self._done("sum_norm", self.lib.atom_sum_norm(
            _ptr(stream), ctypes.c_float(alpha), *terms, len(summands), _ptr(weight), ctypes.c_float(eps), _ptr(out),
            self._code(out) if out is not None else 0, rows, width, self._stream()))
        return stream

    def shift_rows(self, x, mu, out, state, state_off: int, cu_seqlens_q, slot_of_seq, token_seq):
        """``out[t] = x[t] + (x[t - 1] - x[t]) * mu``; the row before a request's first token of the step is what its
        state slot holds at ``state_off`` (float32, zeros for a fresh request), and the request's last row of the
        step is left there.  ``x`` and ``out`` float32 or bfloat16, independently."""
        tokens, width = x.shape
        seqs = slot_of_seq.numel()
        self._check("shift input", x, (torch.float32, torch.bfloat16))
        self._check("shift weight", mu, torch.float32, (width,))
        self._check("shifted rows", out, (torch.float32, torch.bfloat16), (tokens, width))
        self._check("state", state, torch.float32, (None, None))
        self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
        self._check("slot_of_seq", slot_of_seq, torch.int32, (seqs,))
        self._check("token_seq", token_seq, torch.int32, (tokens,))
        self._done("shift_rows", self.lib.atom_shift_rows(
            _ptr(x), self._code(x), _ptr(mu), _ptr(out), self._code(out), _ptr(state), ctypes.c_long(state.shape[1]),
            ctypes.c_long(state_off), _ptr(cu_seqlens_q), _ptr(slot_of_seq), _ptr(token_seq), tokens, width,
            self._stream()))
        return out

    def qkv_rot_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, freq, rot_dims: int, positions, slots,
                      num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, page_size: int, eps: float,
                      v_source=None, v_blend=None, v_keep=None):
        """From the float32 rows ``q | k | v`` of every token: RMS norm of every q and k head with a weight per
        entry (None: no norm), rotation of the pairs (i, i + rot_dims / 2) of every head by ``position * freq[i]``
        (``freq`` float64), ``v_keep`` (float32 [tokens, G * DV]) receives the values as they are, and with
        ``v_source`` (float32, the same shape) the values become ``(1 - l) v + l v_source``, ``l = v_blend`` (one
        float32 number on the device).  q goes to ``q_out`` [tokens, H, D], k to the key pages [pages, G, page, D],
        v to the value pages [pages, G, DV, page] at ``slots`` (-1: no write)."""
        tokens, ld = qkv.shape
        H, G, D, DV = num_heads, num_kv_heads, head_dim, value_dim
        self._check("q | k | v", qkv, torch.float32)
        dt = q_out.dtype
        self._check("q", q_out, (torch.float32, torch.bfloat16), (tokens, H, D))
        self._check("key pages", k_cache, dt, (None, G, page_size, D))
        self._check("value pages", v_cache, dt, (k_cache.shape[0], G, DV, page_size))
        self._check("slot mapping", slots, torch.int32, (tokens,))
        for name, w in (("q norm weight", q_weight), ("k norm weight", k_weight)):
            if w is not None:
                self._check(name, w, torch.float32, (D,))
        if rot_dims:
            self._check("rotation frequencies", freq, torch.float64, (rot_dims // 2,))
            self._check("positions", positions, torch.int32, (tokens,))
        for name, t in (("source values", v_source), ("kept values", v_keep)):
            if t is not None:
                self._check(name, t, torch.float32, (tokens, G * DV))
        if v_source is not None:
            self._check("blend", v_blend, torch.float32, ())
        self._done("qkv_rot_write", self.lib.atom_qkv_rot_write(
            _ptr(qkv), ld, _ptr(q_out), _ptr(k_cache), _ptr(v_cache), self._code(q_out), _ptr(q_weight), _ptr(k_weight),
            _ptr(freq) if rot_dims else None, int(rot_dims), _ptr(positions) if rot_dims else None, _ptr(slots), tokens,
            H, G, D, DV, page_size, ctypes.c_float(eps), _ptr(v_source), _ptr(v_blend) if v_source is not None else None,
            _ptr(v_keep), self._stream()))
        return q_out

    def attention_together(self, q, k_cache, v_cache, out, token_seq, positions, block_tables, scale: float,
                           head_scale=None, sink=None, talk=None, window: int | None = None,
                           max_context_len: int | None = None, cu_seqlens_q=None, max_q_len: int | None = None,
                           parts: int | None = None):
        """Softmax attention of the step's queries over the pages with a token's heads worked through together:
        ``head_scale`` (float32 [H]) multiplies the scaled scores of a head, ``sink`` (float32 [H]) joins the
        softmax's denominator as ``exp(sink[h])`` without a value, ``talk`` (float32 [H, H]) mixes the heads'
        finished weights, ``w_h <- sum_g talk[h, g] w_g``, before head h applies them to the values of its own
        key/value head.  Value heads [pages, G, DV, page] may differ in size from key heads [pages, G, page, D].

        A step with prompt portions (``max_q_len`` > 1, ``cu_seqlens_q`` given) runs on the matrix cores where the
        sizes allow (bfloat16; tiles of 16 tokens of a request); otherwise a block a (token, set of heads), with the
        keys of few tokens cut over ``parts`` blocks (None: chosen so that the launch fills the chip)."""
        tokens, H, D = q.shape
        _, G, page_size, _ = k_cache.shape
        DV = v_cache.shape[2]
        dt = q.dtype
        self._check("q", q, (torch.float32, torch.bfloat16))
        self._check("key pages", k_cache, dt, (None, G, page_size, D))
        self._check("value pages", v_cache, dt, (k_cache.shape[0], G, DV, page_size))
        self._check("attention out", out, dt, (tokens, H, DV))
        self._check("token_seq", token_seq, torch.int32, (tokens,))
        self._check("positions", positions, torch.int32, (tokens,))
        self._check("block tables", block_tables, torch.int32, (None, None))
        if max_context_len is not None and max_context_len > block_tables.shape[1] * page_size:
            raise KernelError("attention: a context is longer than its block table can name")
        for name, w in (("head scale", head_scale), ("sink", sink)):
            if w is not None:
                self._check(name, w, torch.float32, (H,))
        if talk is not None:
            self._check("head mixing", talk, torch.float32, (H, H))
        if (self.use_together_tiles and dt == torch.bfloat16 and cu_seqlens_q is not None and (max_q_len or 0) > 1
                and self.lib.atom_attention_together_tiles_supports(H, G, D, DV, page_size, int(talk is not None))):
            seqs = cu_seqlens_q.numel() - 1
            self._check("cu_seqlens_q", cu_seqlens_q, torch.int32, (seqs + 1,))
            if block_tables.shape[0] != seqs:
                raise KernelError("attention: one block table row per request is needed")
            if parts is None:
                # up to eight blocks a CU (their waves hide each other's waits for memory), every part with at least four chunks of 16 keys
                blocks = (tokens // 16 + seqs + 1) * (1 if talk is not None else G)
                reach = block_tables.shape[1] * page_size if max_context_len is None else max_context_len
                parts = max(1, min(8, 8 * self.num_cus // blocks, reach // 64))
            ws_ml = ws_o = None
            if parts > 1:
                ws_ml = self.workspace("together_ml", tokens * H * parts * 2)
                ws_o = self.workspace("together_o", tokens * parts * H * DV)
            self._done("attention_together_tiles", self.lib.atom_attention_together_tiles(
                _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(cu_seqlens_q), _ptr(positions), _ptr(block_tables),
                block_tables.shape[1], tokens, seqs, H, G, D, DV, page_size, ctypes.c_float(scale), _ptr(head_scale),
                _ptr(sink), _ptr(talk), int(window or 0), int(parts), _ptr(ws_ml), _ptr(ws_o), self._stream()))
            if parts > 1:
                self._done("together_sum_parts", self.lib.atom_together_sum_parts(
                    _ptr(ws_o), _ptr(out), self._code(out), int(parts), tokens, H * DV, self._stream()))
            return out
        sets = tokens * (1 if talk is not None else G)
        if parts is None:
            reach = block_tables.shape[1] * page_size if max_context_len is None else max_context_len
            if window:
                reach = min(reach, window + 63)
            # two blocks a CU where the keys allow, every part with at least two chunks of 64 keys
            parts = max(1, min(-(-2 * self.num_cus // max(sets, 1)), reach // 128)) if sets < self.num_cus else 1
        ws_ml = ws_o = ws_s = None
        stride = block_tables.shape[1] * page_size
        if parts > 1:
            ws_ml = self.workspace("together_ml", tokens * H * parts * 2)
            ws_o = self.workspace("together_o", tokens * parts * H * DV)
            if tokens * H * stride <= 1 << 24:
                # the second launch reads the first one's scores instead of the keys again (up to 64 MB of them)
                ws_s = self.workspace("together_s", tokens * H * stride)
        self._done("attention_together", self.lib.atom_attention_together(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), self._code(q), _ptr(token_seq), _ptr(positions),
            _ptr(block_tables), block_tables.shape[1], tokens, H, G, D, DV, page_size, ctypes.c_float(scale),
            _ptr(head_scale), _ptr(sink), _ptr(talk), int(window or 0), int(parts), _ptr(ws_ml), _ptr(ws_o), _ptr(ws_s),
            ctypes.c_long(stride), self._stream()))
        return out

    def router_choose(self, logits, correction, top: int, renormalize: bool = False):
        """(ids int32 [tokens, top], weights float32 [tokens, top]) from float32 router logits: scores are
        sigmoids; the choice adds ``correction`` to them, the weights do not."""
        tokens, experts = logits.shape
        self._check("router logits", logits, torch.float32)
        if correction is not None:
            self._check("router correction", correction, torch.float32, (experts,))
        ids = torch.empty((tokens, top), dtype=torch.int32, device=logits.device)
        weights = torch.empty((tokens, top), dtype=torch.float32, device=logits.device)
        self._done("router_choose", self.lib.atom_router_choose(
            _ptr(logits), _ptr(correction), _ptr(ids), _ptr(weights), tokens, experts, top, int(bool(renormalize)),
            self._stream()))
        return ids, weights

    def experts_forward(self, x, gate_up, down, ids, weights, activation: str = "silu"):
        """``sum_k weights[t, k] * down[e] (act(gate[e] x) * (up[e] x))`` with e = ids[t, k].  ``gate_up``
        [experts, 2 ff, width] (gate rows, then up rows), ``down`` [experts, width, ff]."""
        x = self.materialize(x)
        tokens, width = x.shape
        experts, two_ff, _ = gate_up.shape
        ff = two_ff // 2
        top = ids.shape[1]
        self._check("experts input", x, (torch.float32, torch.bfloat16))
        self._check("expert gate|up", gate_up, (torch.float32, torch.bfloat16), (experts, 2 * ff, width))
        self._check("expert down", down, gate_up.dtype, (experts, width, ff))
        self._check("expert ids", ids, torch.int32, (tokens, top))
        self._check("expert weights", weights, torch.float32, (tokens, top))
        if activation not in self._ACTIVATIONS:
            raise KernelError(f"experts: unknown activation {activation!r}")
        if (x.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 and tokens * top >= self.grouped_experts_from
                and self.lib.atom_experts_grouped_supports(ff, width, experts)):
            tiles = self.lib.atom_experts_grouped_tiles(tokens * top, experts)
            ints = self.workspace("experts_ints", tiles * 65 + tokens * top, torch.int32)
            act = self.workspace("experts_act", tiles * 64 * ff, torch.bfloat16)
            rows = self.workspace("experts_rows", tiles * 64 * width)
            y = torch.empty((tokens, width), dtype=x.dtype, device=x.device)
            self._done("experts_grouped", self.lib.atom_experts_grouped(
                _ptr(x), _ptr(gate_up), _ptr(down), _ptr(ids), _ptr(weights), _ptr(ints),
                ctypes.c_void_p(ints.data_ptr() + 4 * tiles), ctypes.c_void_p(ints.data_ptr() + 4 * tiles * 65), _ptr(act),
                _ptr(rows), _ptr(y), tokens, top, experts, ff, width, self._ACTIVATIONS[activation], self._stream()))
            return y
        act = torch.empty((tokens * top, ff), dtype=x.dtype, device=x.device)
        self._done("experts_gate_up", self.lib.atom_experts_gate_up(
            _ptr(x), _ptr(gate_up), self._code(gate_up), _ptr(ids), _ptr(act), self._code(x), tokens, top, ff, width,
            self._ACTIVATIONS[activation], self._stream()))
        y = torch.empty((tokens, width), dtype=x.dtype, device=x.device)
        self._done("experts_down", self.lib.atom_experts_down(
            _ptr(act), _ptr(down), self._code(down), _ptr(ids), _ptr(weights), _ptr(y), self._code(x), tokens, top, ff,
            width, self._stream()))
        return y

    def sample(self, logits, temperatures, out, top_ks=None, top_ps=None, noise=None, seeds=None, counters=None,
               eps: float = 1e-10):
        rows, vocab = logits.shape
        self._check("logits", logits, torch.float32)
        self._check("sampled ids", out, torch.int32, (rows,))
        if temperatures is not None:
            self._check("temperatures", temperatures, torch.float32, (rows,))
        if top_ks is not None:
            self._check("top_ks", top_ks, torch.int32, (rows,))
        if top_ps is not None:
            self._check("top_ps", top_ps, torch.float32, (rows,))
        stride = 0
        if noise is not None:
            self._check("noise", noise, torch.float32, (None, vocab))
            if noise.shape[0] not in (1, rows):
                raise KernelError("noise must have one row or one per logits row")
            stride = vocab if noise.shape[0] == rows and rows > 1 else 0
        else:
            if temperatures is not None and (seeds is None or counters is None):
                raise KernelError("sampling without given noise needs seeds and counters")
        if seeds is not None:
            self._check("seeds", seeds, torch.int64, (rows,))
            self._check("counters", counters, torch.int64, (rows,))
        # every row's maximum (and, without filters, its race) is spread over 64 blocks: chunk maxima, chunk winners
        ws_vals = self.workspace("sample_vals", rows * 128)
        ws_idx = self.workspace("sample_idx", rows * 128, torch.int32)
        ws_filter = None
        if temperatures is not None and (top_ks is not None or top_ps is not None) and vocab >= 16384:
            # histograms of the threshold search: zero when made, and left zero by every call
            need = rows * (4096 * 12 + 32)
            ws_filter = self._zeroed.get("sample_filter")
            if ws_filter is None or ws_filter.numel() < need:
                if torch.cuda.is_current_stream_capturing():
                    # making it would record a fill node into the graph; the caller samples these rows once
                    # outside a capture first, which leaves the workspace in place
                    raise KernelError("sample: the top-k / top-p workspace has to exist before a graph is captured "
                                      f"({rows} rows need {need} bytes)")
                ws_filter = torch.zeros(need, dtype=torch.uint8, device=self.device)
                self._zeroed["sample_filter"] = ws_filter
        self._done("sample", self.lib.atom_sample(
            _ptr(logits), _ptr(temperatures), _ptr(top_ks), _ptr(top_ps), _ptr(noise), ctypes.c_long(stride),
            _ptr(seeds), _ptr(counters), _ptr(out), rows, vocab, ctypes.c_float(eps), _ptr(ws_vals), _ptr(ws_idx),
            _ptr(ws_filter), self._stream()))
        return out

    def exponential_noise(self, seeds, counters, vocab: int):
        rows = seeds.numel()
        self._check("seeds", seeds, torch.int64, (rows,))
        self._check("counters", counters, torch.int64, (rows,))
        out = torch.empty((rows, vocab), dtype=torch.float32, device=seeds.device)
        self._done("exponential_noise", self.lib.atom_exponential_noise(
            _ptr(out), _ptr(seeds), _ptr(counters), rows, vocab, self._stream()))
        return out
