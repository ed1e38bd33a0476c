"""Savidra on the GPU: every new kernel alone against the plain implementation's function of the same mechanism
(float32 and bfloat16 where the kernel has both), attention with a key made to stand out far away, at page borders
and behind a sink, heads that take each other's weights, then the engine on tiny models: whole prompts,
token-by-token tails, portions down to two tokens, mixed batches with pages and slots used again, decode steps
replayed from graphs, long decoding, greedy generation through ``LLMEngine``, ``bin/trace_run`` and the command
line."""

import pytest
import torch

import plain_savidra as ps
import replay
import savidra_tiny as st
from helpers import gpu_ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    scale = max(1e-6, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= TOL[dtype] * scale, f"{what}: {err:.3e} > {TOL[dtype] * scale:.3e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def f32(t):
    return t.to(torch.float32).to(DEV).contiguous()


def _batch(lens, slots):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    seq_of = [s for s, n in enumerate(lens) for _ in range(n)]
    return cu, i32(cu), i32(slots), i32(seq_of)


# ------------------------------------------------------------------ the stream's kernels


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("width,terms", [(40, 1), (176, 2), (1000, 2), (4096, 1), (52, 4)])
def test_norm_of_a_sum_becomes_the_stream(out_dtype, width, terms):
    ops = gpu_ops()
    rows, alpha, eps = 7, 1.5, 1e-5
    stream = rnd((rows, width), 1)
    ys = [rnd((rows, width), 10 + k).to(torch.bfloat16 if k % 2 else torch.float32) for k in range(terms)]
    scales = [0.7, 1.3, -0.4, 2.0][:terms]
    w = 0.2 * rnd((width,), 3)
    total = alpha * stream.double() + sum(s * y.double() for s, y in zip(scales, ys))
    want = ps.one_plus_norm(total, w.double(), eps)
    got = f32(stream)
    copy = torch.empty((rows, width), dtype=out_dtype, device=DEV)
    ops.sum_norm(got, alpha, [y.to(DEV) for y in ys], scales, f32(1 + w), eps, copy)
    close(got, want, torch.float32, "stream")
    close(copy, want, out_dtype, "copy")
    # no weight: the sum alone; alpha 0: whatever the stream held is not read
    junk = torch.full((rows, width), float("nan"), device=DEV)
    ops.sum_norm(junk, 0.0, [y.to(DEV) for y in ys], scales, None, 0.0)
    close(junk, sum(s * y.double() for s, y in zip(scales, ys)), torch.float32, "sum alone")


@pytest.mark.parametrize("x_dtype", DTYPES)
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("width,off", [(50, 3), (208, 0), (2048, 8)])
def test_blend_with_the_previous_token_across_steps(x_dtype, out_dtype, width, off):
    """Two steps over three requests in slots 2, 0 and 3 (one sits the second step out, a new one starts in a slot
    whose row was cleared): the row before a request's first token of a step is what the slot holds."""
    ops = gpu_ops()
    mu = torch.sigmoid(rnd((width,), 5))
    state = torch.zeros((4, off + width + 5), device=DEV)
    rows = {r: rnd((n, width), 20 + k).to(x_dtype) for k, (r, n) in enumerate([("a", 9), ("b", 4), ("c", 6)])}
    kept = {r: torch.zeros(width, dtype=torch.float64) for r in rows}
    for lens, who, slots in (([5, 1, 3], ["a", "b", "c"], [2, 0, 3]), ([4, 3], ["a", "b"], [2, 0])):
        cu, d_cu, d_slots, d_seq = _batch(lens, slots)
        x, want = [], []
        for r, n in zip(who, lens):
            part, rows[r] = rows[r][:n], rows[r][n:]
            h, kept[r] = ps.token_shift(part.double(), mu.double(), kept[r])
            x.append(part)
            want.append(h)
        out = torch.empty((sum(lens), width), dtype=out_dtype, device=DEV)
        ops.shift_rows(torch.cat(x).to(DEV).contiguous(), f32(mu), out, state, off, d_cu, d_slots, d_seq)
        close(out, torch.cat(want), out_dtype, f"step of {lens}")
    assert torch.equal(state[1], torch.zeros_like(state[1])) and float(state[:, :off].abs().max() if off else 0) == 0


# ------------------------------------------------------------------ q, k and v on their way to the pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,DV,rot,page,normed,blend", [(4, 2, 10, 6, 6, 4, True, None), (2, 1, 12, 20, 12, 16, True, "blend"),
                                                           (3, 3, 7, 7, 0, 8, False, "keep"), (6, 3, 128, 64, 32, 16, True, "blend"),
                                                           (1, 1, 14, 3, 2, 16, True, "keep")])
def test_norm_rotation_blend_and_page_write(dtype, H, G, D, DV, rot, page, normed, blend):
    ops = gpu_ops()
    T, pages, eps = 11, 6, 1e-5
    ld = (H + G) * D + G * DV + 3
    qkv = rnd((T, ld), 1)
    qw, kw = (1 + 0.2 * rnd((D,), 2), 1 + 0.2 * rnd((D,), 3)) if normed else (None, None)
    positions = [0, 1, 2, 37, 38, 1000, 5, 6, 7, 8, 123456]
    slots = [5, 0, -1, 23, 7, 8, 9, 10, 11, 12, 13][:T]
    slots = [s if s < pages * page else s % (pages * page) for s in slots]
    freq = torch.tensor([77.0 ** (-2.0 * i / max(rot, 1)) / 3.0 for i in range(rot // 2)], dtype=torch.float64)
    q, k, v = torch.split(qkv.double()[:, :ld - 3], [H * D, G * D, G * DV], dim=-1)
    q, k = q.reshape(T, H, D), k.reshape(T, G, D)
    if normed:
        q, k = ps.plain_norm(q, qw.double(), eps), ps.plain_norm(k, kw.double(), eps)
    at = torch.tensor(positions)
    q, k = ps.rotate_half(q, at, rot, 77.0, 3.0), ps.rotate_half(k, at, rot, 77.0, 3.0)
    source = rnd((T, G * DV), 9) if blend == "blend" else None
    lam = torch.tensor(0.3)
    keep = torch.empty((T, G * DV), device=DEV) if blend == "keep" else None
    v_want = (1 - 0.3) * v + 0.3 * source.double() if source is not None else v
    q_out = torch.empty((T, H, D), dtype=dtype, device=DEV)
    k_cache = torch.zeros((pages, G, page, D), dtype=dtype, device=DEV)
    v_cache = torch.zeros((pages, G, DV, page), dtype=dtype, device=DEV)
    ops.qkv_rot_write(f32(qkv), q_out, k_cache, v_cache, f32(qw) if normed else None, f32(kw) if normed else None,
                      freq.to(DEV), rot, i32(positions), i32(slots), H, G, D, DV, page, eps,
                      v_source=f32(source) if source is not None else None, v_blend=lam.to(DEV) if source is not None else None,
                      v_keep=keep)
    close(q_out, q, dtype, "q")
    if keep is not None:
        close(keep, v, torch.float32, "kept values")
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        p, o = divmod(slot, page)
        close(k_cache[p, :, o, :], k[t], dtype, f"key of token {t}")
        close(v_cache[p, :, :, o], v_want[t].view(G, DV), dtype, f"value of token {t}")
    written = {divmod(s, page) for s in slots if s >= 0}
    for p in range(pages):
        for o in range(page):
            if (p, o) not in written:
                assert float(k_cache[p, :, o].abs().max()) == 0 and float(v_cache[p, :, :, o].abs().max()) == 0


# ------------------------------------------------------------------ attention with the heads together


def _paged(keys, values, page, dtype, order_seed):
    """Keys [n, G, D] and values [n, G, DV] of one request laid into pages in a shuffled order."""
    n, G, D = keys.shape
    DV = values.shape[2]
    blocks = -(-n // page)
    perm = torch.randperm(blocks + 3, generator=torch.Generator().manual_seed(order_seed))[:blocks].tolist()
    k_cache = torch.zeros((blocks + 3, G, page, D), dtype=dtype)
    v_cache = torch.zeros((blocks + 3, G, DV, page), dtype=dtype)
    for j in range(n):
        k_cache[perm[j // page], :, j % page] = keys[j].to(dtype)
        v_cache[perm[j // page], :, :, j % page] = values[j].to(dtype)
    return k_cache.to(DEV), v_cache.to(DEV), perm


def _attend(ops, q, keys, values, positions, page, dtype, scale, temp=None, sink=None, talk=None, seed=0, how="blocks",
            window=None):
    """``how``: "blocks" (a block a token and set of heads), "parts" (a token's keys cut over three blocks), "tiles"
    (the rows as a prompt portion of one request: the matrix cores where the sizes allow)."""
    T, H, D = q.shape
    k_cache, v_cache, perm = _paged(keys, values, page, dtype, seed)
    out = torch.empty((T, H, values.shape[2]), dtype=dtype, device=DEV)
    dev = lambda t: f32(t) if t is not None else None  # noqa: E731
    more = {"blocks": dict(parts=1), "parts": dict(parts=3), "tiles": dict(cu_seqlens_q=i32([0, T]), max_q_len=T, parts=1),
            "tile parts": dict(cu_seqlens_q=i32([0, T]), max_q_len=T, parts=3)}[how]
    ops.attention_together(q.to(dtype).to(DEV), k_cache, v_cache, out, i32([0] * T), i32(positions), i32([perm]), scale,
                           head_scale=dev(temp), sink=dev(sink), talk=dev(talk), max_context_len=keys.shape[0],
                           window=window, **more)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("how", ["blocks", "parts", "tiles", "tile parts"])
@pytest.mark.parametrize("H,G,D,DV,page,n,sink,talk,temp", [
    (4, 2, 10, 6, 4, 70, True, False, False), (6, 3, 6, 4, 16, 131, False, True, True), (2, 1, 12, 20, 8, 64, True, True, True),
    (8, 2, 128, 32, 16, 300, True, False, False), (6, 2, 48, 16, 16, 257, False, True, True), (1, 1, 14, 3, 16, 65, False, True, False),
    (16, 4, 64, 64, 16, 200, False, True, True), (3, 3, 7, 7, 4, 5, False, False, False), (8, 2, 128, 128, 16, 300, False, True, True),
    (8, 8, 64, 128, 8, 100, True, True, False), (12, 3, 64, 32, 4, 90, True, False, True), (32, 2, 128, 64, 16, 150, True, False, False)])
def test_attention_against_plain(dtype, how, H, G, D, DV, page, n, sink, talk, temp):
    ops = gpu_ops()
    q, keys, values = rnd((n, H, D), 1).to(dtype), rnd((n, G, D), 2).to(dtype), rnd((n, G, DV), 3).to(dtype)
    sk = 1.5 * rnd((H,), 4) if sink else None
    tk = torch.eye(H) + 0.3 * rnd((H, H), 5) if talk else None
    tp = 1 + 0.3 * rnd((H,), 6) if temp else None
    rows = sorted({0, 1, 2, page - 1, page, n // 2, 63, 64, 65, n - 2, n - 1} & set(range(n)))
    if how.startswith("tile"):       # more than a tile of rows, the last tile not full
        rows = sorted(set(rows) | set(range(max(0, n - 40), n, 2)))
    at = torch.tensor(rows)
    w = ps.softmax_weights(q[rows].double(), keys.double(), at, torch.arange(n), 0.3,
                           sink=sk.double() if sink else None, temp=tp.double() if temp else None)
    if talk:
        w = torch.einsum("hg,gij->hij", tk.double(), w)
    want = ps.apply_weights(w, values.double(), H).view(len(rows), H, DV)
    got = _attend(ops, q[rows], keys, values, rows, page, dtype, 0.3, tp, sk, tk, seed=n, how=how)
    close(got, want, dtype, "attention")


@pytest.mark.parametrize("parts", [1, 2, 7])
@pytest.mark.parametrize("talk", [False, True])
def test_tiles_of_several_requests(talk, parts):
    """Portions of three requests and a single token in one launch, each behind a different number of cached tokens:
    every block finds its request and tile from its index alone."""
    ops = gpu_ops()
    H, G, D, DV, page, dtype = 4, 2, 64, 32, 16, torch.bfloat16
    lens, cached = [37, 1, 16, 50], [5, 80, 0, 100]
    tk = torch.eye(H) + 0.3 * rnd((H, H), 5) if talk else None
    blocks = [-(-(c + n) // page) for n, c in zip(lens, cached)]
    k_cache = torch.zeros((sum(blocks) + 1, G, page, D), dtype=dtype)
    v_cache = torch.zeros((sum(blocks) + 1, G, DV, page), dtype=dtype)
    tables = torch.zeros((4, max(blocks)), dtype=torch.int32)
    qs, wants, positions, seq_of, at = [], [], [], [], 1
    for r, (n, c) in enumerate(zip(lens, cached)):
        keys, values = rnd((c + n, G, D), 10 + r).to(dtype), rnd((c + n, G, DV), 20 + r).to(dtype)
        tables[r, :blocks[r]] = torch.arange(at, at + blocks[r])
        for j in range(c + n):
            k_cache[at + j // page, :, j % page] = keys[j]
            v_cache[at + j // page, :, :, j % page] = values[j]
        at += blocks[r]
        q = rnd((n, H, D), 30 + r).to(dtype)
        pos = torch.arange(c, c + n)
        w = ps.softmax_weights(q.double(), keys.double(), pos, torch.arange(c + n), 0.2)
        if talk:
            w = torch.einsum("hg,gij->hij", tk.double(), w)
        wants.append(ps.apply_weights(w, values.double(), H).view(n, H, DV))
        qs.append(q)
        positions += pos.tolist()
        seq_of += [r] * n
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    out = torch.empty((sum(lens), H, DV), dtype=dtype, device=DEV)
    ops.attention_together(torch.cat(qs).to(DEV), k_cache.to(DEV), v_cache.to(DEV), out, i32(seq_of), i32(positions),
                           tables.to(DEV), 0.2, talk=f32(tk) if talk else None, max_context_len=150, cu_seqlens_q=i32(cu),
                           max_q_len=max(lens), parts=parts)
    close(out, torch.cat(wants), dtype, "tiles of several requests")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 1, 15, 16, 63, 64, 127, 128, 700])
def test_a_far_key_is_found_and_a_later_one_is_not(dtype, far):
    """Among 900 keys one is made to answer the query of the last token; its value shows in the output.  The same key
    placed one position after the query is not seen."""
    ops = gpu_ops()
    n, H, G, D, DV, page = 900, 2, 1, 16, 8, 16
    keys, values = 0.1 * rnd((n, G, D), 1), rnd((n, G, DV), 2)
    q = 0.1 * rnd((1, H, D), 3)
    q[0, :, 0], keys[far, 0, 0] = 6.0, 6.0
    values[far, 0] = 50.0
    for how in ("blocks", "parts"):
        got = _attend(ops, q, keys, values, [n - 1], page, dtype, 1.0, how=how)
        assert float(got.float().min()) > 45.0, how
    got = _attend(ops, q, keys, values, [far - 1], page, dtype, 1.0) if far else None
    assert got is None or float(got.float().abs().max()) < 10.0
    # a sink as large as the key's score takes half of the weight and brings no value
    got = _attend(ops, q, keys, values, [n - 1], page, dtype, 1.0, sink=torch.tensor([36.0, -40.0]))
    assert 20.0 < float(got[0, 0].float().mean()) < 30.0 and float(got[0, 1].float().min()) > 45.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("how", ["blocks", "parts", "tiles", "tile parts"])
@pytest.mark.parametrize("window", [1, 9, 16, 64, 65, 200])
def test_a_window_holds_the_token_itself_and_the_ones_before(dtype, how, window):
    """The design has no window; the kernels offer one to others.  A key made to stand out is seen by the query
    ``window - 1`` positions after it and not by the next, with and without mixed heads, and everything matches the
    plain weights."""
    ops = gpu_ops()
    n, H, G, D, DV, page = 300, 4, 2, 64, 32, 16
    q, keys, values = 0.3 * rnd((n, H, D), 1), 0.3 * rnd((n, G, D), 2), rnd((n, G, DV), 3)
    at_key = 120
    q[:, :, 0], keys[at_key, :, 0] = 5.0, 8.0
    values[at_key] = 40.0
    q, keys, values = q.to(dtype), keys.to(dtype), values.to(dtype)
    tk = torch.eye(H) + 0.2 * rnd((H, H), 5)
    rows = sorted({at_key, at_key + window - 1, at_key + window, 0, 63, 64, n - 1} & set(range(n)))
    at = torch.tensor(rows)
    for talk in (None, tk):
        w = ps.softmax_weights(q[rows].double(), keys.double(), at, torch.arange(n), 0.5, window=window)
        if talk is not None:
            w = torch.einsum("hg,gij->hij", talk.double(), w)
        want = ps.apply_weights(w, values.double(), H).view(len(rows), H, DV)
        got = _attend(ops, q[rows], keys, values, rows, page, dtype, 0.5, talk=talk, seed=window, how=how, window=window)
        close(got, want, dtype, f"window {window}")
        if talk is None and at_key + window < n:
            inside, outside = rows.index(at_key + window - 1), rows.index(at_key + window)
            assert float(got[inside].float().mean()) > 30.0 and float(got[outside].float().abs().mean()) < 10.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_that_take_each_others_weights(dtype):
    """Head 0 looks at key 3, head 1 at key 40 (another page); swapped by the mixing, each reads the other's key
    from its own value head."""
    ops = gpu_ops()
    n, D, DV, page = 90, 8, 4, 16
    keys, values = torch.zeros(n, 2, D), rnd((n, 2, DV), 1)
    q = torch.zeros(1, 2, D)
    q[0, 0, 0] = q[0, 1, 1] = 9.0
    keys[3, 0, 0] = keys[40, 1, 1] = 9.0
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    got = _attend(ops, q, keys, values, [n - 1], page, dtype, 1.0, talk=swap).float().cpu()
    close(got[0, 0], values[40, 0].to(dtype), dtype, "head 0")
    close(got[0, 1], values[3, 1].to(dtype), dtype, "head 1")


# ------------------------------------------------------------------ a sink in the one-walk kernels


@pytest.mark.parametrize("H,G,D,page", [(4, 2, 64, 16), (8, 2, 128, 16), (2, 2, 64, 8), (16, 1, 128, 16), (6, 6, 32, 4)])
@pytest.mark.parametrize("cached,fresh", [(0, 70), (37, 200), (300, 33), (700, 1), (5, 1), (64, 2)])
def test_sink_in_the_paged_kernels(H, G, D, page, cached, fresh):
    """A prompt portion behind cached tokens, or a single token whose keys are cut over several parts: the sink is
    where a row's running maximum and sum start, and counts once."""
    from atom_amd.kernels.hip import AttentionMeta

    ops = gpu_ops()
    dtype, n = torch.bfloat16, cached + fresh
    if not ops.takes_sink(dtype, D, D, page, H // G):
        pytest.skip("the matrix-core kernels do not take these sizes")
    q, keys, values = rnd((n, H, D), 1).to(dtype), rnd((n, G, D), 2).to(dtype), rnd((n, G, D), 3).to(dtype)
    sink = 2.0 * rnd((H,), 4) + 1.0
    k_cache, v_cache, perm = _paged(keys, values, page, dtype, n)
    rows = list(range(cached, n))
    at = torch.tensor(rows)
    w = ps.softmax_weights(q[rows].double(), keys.double(), at, torch.arange(n), 0.25, sink=sink.double())
    want = ps.apply_weights(w, values.double(), H).view(fresh, H, D)
    for parts in ([None] if fresh > 1 else [None, 1, 3, 8]):
        meta = AttentionMeta(token_seq=i32([0] * fresh), positions=i32(rows), block_tables=i32([perm]),
                             cu_seqlens_q=i32([0, fresh]), context_lens=i32([n]), num_seqs=1, num_tokens=fresh,
                             max_q_len=fresh, max_context_len=n, page_size=page, num_prefill=1 if fresh > 1 else 0)
        if fresh > 1:
            short, tall = ops.attention_tile_rows(dtype, D, page, H // G, fresh)
            if short:
                meta.rows_per_tile = short
                meta.prefill_tiles = i32([[0, r] for r in range(0, fresh, short)])
            if tall:
                meta.tiles_by_rows = {tall: i32([[0, r] for r in range(0, fresh, tall)])}
        out = torch.empty((fresh, H, D), dtype=dtype, device=DEV)
        ops.paged_attention(q[rows].to(DEV).contiguous(), k_cache, v_cache, out, meta, 0.25, parts=parts, sink=f32(sink))
        close(out, want, dtype, f"parts {parts}")
        plain = torch.empty_like(out)
        ops.paged_attention(q[rows].to(DEV).contiguous(), k_cache, v_cache, plain, meta, 0.25, parts=parts)
        assert float((plain.float() - out.float()).abs().max()) > 1e-3, "the sink changes nothing"


# ------------------------------------------------------------------ the engine

LENGTHS = {"A": [1, 7, 33, 150, 64, 300], "B": [2, 19, 45, 260, 128], "C": [3, 40, 17, 270, 96, 161], "D": [1, 9, 70, 200],
           "E": [1, 2, 50, 130]}
F32_TOL = dict(max=1e-4, mean=2e-5)
BF16_TOL = dict(max=6e-2, mean=1.2e-2)


def _requests(which, seed=0):
    return {f"r{k}": st.ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


def _check(steps, results, requests, which, dtype, what):
    rows = replay.collect(steps, results)
    over, judged = [], 0
    for rid, tokens in requests.items():
        want = st.oracle(which, tokens)
        scale = float(want.abs().max())
        assert len(rows[rid]) == len(tokens)
        for pos, got in sorted(rows[rid].items()):
            assert torch.isfinite(got).all(), f"{what} request {rid} position {pos}: not finite"
            diff = (got.double() - want[pos]).abs()
            worst, mean = float(diff.max()) / scale, float(diff.mean()) / scale
            judged += 1
            if dtype == "float32":
                assert worst <= F32_TOL["max"] and mean <= F32_TOL["mean"], \
                    f"{what} request {rid} position {pos}: max {worst:.3e} mean {mean:.3e} of the largest logit"
            elif worst > BF16_TOL["max"] or mean > BF16_TOL["mean"]:
                over.append((rid, pos, worst, mean))
    assert len(over) <= 0.02 * judged, f"{what}: {len(over)} of {judged} over: {over[:5]}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut, dtype):
    requests = _requests(which)
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 16) // 16)
    core = st.core(which, dtype, gpu_ops(), DEV, num_pages=pages, page_size=16, graph_sizes=[1, 2, 4] if cut != "whole" else None)
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, which, dtype, f"{which}/{cut}/{dtype}")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)
    if cut == "tail":
        assert core.graphs is not None and core.graphs.replays >= 32, "single tokens replay captured graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pages_slots_used_again_and_long_decoding(dtype):
    """Pages of 4 tokens, two state slots for five requests, and 150 tokens decoded one by one, every one compared."""
    requests = {"long": st.ids("A", 330, 1), "b": st.ids("A", 23, 2), "c": st.ids("A", 50, 3), "d": st.ids("A", 9, 4),
                "e": st.ids("A", 31, 5)}
    steps = replay.mixed(requests, seed=6, max_live=2, decode_tail=150)
    pages = -(-replay.peak_tokens(steps, 4) // 4)
    core = st.core("A", dtype, gpu_ops(), DEV, num_pages=pages, page_size=4, max_num_seqs=2, graph_sizes=[1, 2])
    results = replay.run_in_process(core, steps)
    _check(steps, results, requests, "A", dtype, f"A/page4/{dtype}")


def test_logits_do_not_depend_on_the_batch_or_the_cut():
    """float32: a request's logits alone, cut in portions, and beside others differ by rounding of sums only."""
    requests = _requests("C")
    runs = []
    for cut in ("whole", "portions", "mixed"):
        steps = getattr(replay, cut)(requests)
        core = st.core("C", "float32", gpu_ops(), DEV, num_pages=80, page_size=16)
        runs.append(replay.collect(steps, replay.run_in_process(core, steps)))
    for rid in requests:
        for pos in runs[0][rid]:
            for other in runs[1:]:
                assert float((runs[0][rid][pos] - other[rid][pos]).abs().max()) <= 2e-5 * float(runs[0][rid][pos].abs().max())


def test_stream_after_every_layer():
    """float32: the stream after each layer against the plain implementation's, so that a fault shows at the layer
    that makes it."""
    from atom_amd.engine.core import StepEntry

    tokens = st.ids("B", 45, 8)
    trail = []
    ps.PlainSavidra(st.CONFIGS["B"], st.tensors("B")).forward(tokens, trail)
    core = st.core("B", "float32", gpu_ops(), DEV, num_pages=8, page_size=16)
    got = []
    blocks = core.model.blocks
    originals = [b.forward for b in blocks]

    def watch(inner):
        def forward(ctx, hidden, residual, cache):
            out = inner(ctx, hidden, residual, cache)
            got.append(out[0].clone().cpu())
            return out
        return forward

    for b, inner in zip(blocks, originals):
        b.forward = watch(inner)
    try:
        core.step([StepEntry("a", tokens, [len(tokens) - 1])])
    finally:
        for b, inner in zip(blocks, originals):
            b.forward = inner
    assert len(got) == len(trail)
    for layer, (mine, want) in enumerate(zip(got, trail)):
        close(mine, want, torch.float32, f"after layer {layer}")


@pytest.mark.parametrize("which,dtype", [("A", "fp32"), ("B", "fp32"), ("C", "fp32"), ("C", "bf16")])
def test_greedy_generation_through_the_engine(which, dtype):
    from atom_amd import LLMEngine, SamplingParams

    llm = LLMEngine(st.folder(which), dtype=dtype, ops=gpu_ops(), kv_cache_block_size=16, num_kvcache_blocks=64,
                    max_num_seqs=4, max_num_batched_tokens=64, max_model_len=384)
    prompts = [st.ids(which, n, 70 + n) for n in (1, 9, 40, 130, 65)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt)
        assert len(out["token_ids"]) == 10
        for token in out["token_ids"]:
            logits = st.oracle(which, tokens)[-1]
            best = int(logits.argmax())
            slack = 0.0 if dtype == "fp32" else 0.06 * float(logits.abs().max())
            assert token == best or float(logits[best] - logits[token]) <= slack
            tokens.append(token)
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_program(dtype, tmp_path):
    requests = {k: v for k, v in list(_requests("B").items())[:4]}
    steps = replay.mixed(requests, seed=2, max_live=3)
    results = replay.run_program(st.folder("B"), dtype, steps, str(tmp_path / "out"), replay.peak_tokens(steps, 64),
                                 st.CONFIGS["B"]["vocab"])
    _check(steps, results, requests, "B", dtype, f"program/{dtype}")


def test_command_line():
    """``python -m atom_amd.examples.simple_inference`` on a Savidra folder: the registry picks the design from
    config.json; greedy completions are the plain implementation's."""
    import random
    import re
    import subprocess
    import sys

    cmd = [sys.executable, "-m", "atom_amd.examples.simple_inference", "--model", st.folder("A"), "--temperature", "0",
           "--max-tokens", "6", "--block_size", "16", "--num-kvcache-blocks", "32", "--max-num-seqs", "4", "--dtype", "fp32",
           "--max-model-len", "256", "--seed", "3"]
    res = subprocess.run(cmd, cwd=replay.ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert res.stdout.count("Completion:") == 3 and res.stdout.count("finish_reason=max_tokens") == 3
    rng = random.Random(3)
    prompts = [[rng.randrange(st.CONFIGS["A"]["vocab"]) for _ in range(n)] for n in (5, 17, 33)]
    shown = [eval(m) for m in re.findall(r"Completion: (\[.*?\])", res.stdout)]
    for prompt, out in zip(prompts, shown):
        tokens = list(prompt)
        for token in out:
            assert token == int(st.oracle("A", tokens)[-1].argmax())
            tokens.append(token)
