// Linear recurrences with a matrix state per head, and what stands around them.
//
// The state S of a head has K rows (key channels) and V columns (value channels), float32, and lives in the
// request's state slot.  Per token, with a key k, a read vector r, a value v and a decay w (one per key channel, or
// one per head):
//
//   read_before (a bonus u per key channel for the current token):
//       o = (S + diag(u) k v^T)^T r;   S <- diag(w) S + k v^T
//   read_after:
//       S <- diag(w) S + k v^T;        o = S^T r
//
// v may first be multiplied by a step size per (token, head), and o may receive skip[h] * (the unscaled v).  The
// columns of S never meet, so a column lives in registers, spread over LPC adjacent lanes of 16 rows each.  A wave
// owns 64 / LPC columns of one head; the waves of a block (up to four) own neighbouring columns and share what they
// stage in LDS for 16 (8 where a lane holds four columns) tokens at a time: r, k and the decays (formed on the way: as given, or exp(-exp(x + bias))),
// the block's columns of v and the step sizes.
//
// Requests that bring no more than a run's length of tokens are walked by one block per (request, head, columns):
// the state comes from the slot and goes back there.  Longer requests are cut into runs that are worked side by
// side, which the recurrence allows because a run acts on the state as S -> diag(a) S + B:
//   1. every run but a request's last forms B (its tokens applied to a zero state) and a (the product of its decays);
//   2. per request the state before each run is folded from the slot's state through the runs ahead of it;
//   3. every run walks its tokens again from that state and writes the outputs; the last run leaves the state in
//      the slot.
// Run j of request s (tokens from t0) has the scratch place t0 / R + s + j, which no other run has.  A token's
// result depends on its own request only; cutting a request differently changes the order of roundings, no more.
//
// Around it: token_shift (a token's input mixed with the previous token's, the previous token kept per request),
// step_decay (softplus step sizes and the decays exp(-exp(A_log) dt) of a state-space layer), group_norm_gate (RMS
// norm in equal parts of a row, a weight per entry, a SiLU gate before or after the norm).
#include "common.h"

constexpr int kScanRows = 16;    // rows of S a lane holds
constexpr int kScanStage = 16;   // tokens staged at a time
constexpr int kScanWaves = 4;    // the most waves of a block

struct ScanArgs {
  const float* r; long ldr; int r_div;       // head h reads r-head h / r_div, K entries each
  const float* k; long ldk; int k_div;
  const float* v; long ldv;                  // [T, H * V] at v
  const float* w; long ldw; int w_per_channel;   // [T, H * K] or [T, H]
  const float* w_bias; int w_mode;           // 0: w is the decay; 1: decay = exp(-exp(w + w_bias[h * K + i]));
                                             // 2 (one decay per head): step = softplus(w + w_bias[h]) multiplies v,
  const float* a_log;                        //    decay = exp(-exp(a_log[h]) step)
  const float* v_scale; long ldvs;           // [T, H] or null
  const float* bonus;                        // [H, K]: read_before; null: read_after
  const float* skip;                         // [H] or null
  float* out; long ldo;                      // [T, H * V]
  float* state; long slot_stride; long state_off;
  const int* cu_seqlens; const int* slot_of_seq;
  int num_seqs, H, K, V, lpc, waves;
  int run_len;                               // R, a multiple of kScanStage; 0: a request is one run whatever its length
  float* run_state;                          // [places, H, K, V]: B of a run after pass 1, the state before it after pass 2
  float* run_decay;                          // [places, H, K]: the product of a run's decays
};

// Which request and which of its runs the block with index b works on: the last s with cu[s] / R + s <= b.
__device__ __forceinline__ bool scan_place(const ScanArgs& a, int b, int& seq, int& run, int& runs) {
  if (a.run_len == 0) {
    seq = b; run = 0; runs = 1;
    return true;
  }
  int lo = 0, hi = a.num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (a.cu_seqlens[mid] / a.run_len + mid <= b) lo = mid; else hi = mid - 1;
  }
  seq = lo;
  const int t0 = a.cu_seqlens[seq], len = a.cu_seqlens[seq + 1] - t0;
  runs = max(1, (len + a.run_len - 1) / a.run_len);
  run = b - (t0 / a.run_len + seq);
  return run >= 0 && run < runs;
}

// The sum of v over the LPC adjacent lanes that share a column, in each of them, by data-parallel permutes within a
// row of 16 lanes (no trip through LDS): neighbours, pairs, then the mirrored half-row and row.
template <int CTRL>
__device__ __forceinline__ float scan_dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

template <int LPC>
__device__ __forceinline__ float scan_group_sum(float v) {
  if constexpr (LPC >= 2) v = scan_dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  if constexpr (LPC >= 4) v = scan_dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  if constexpr (LPC >= 8) v = scan_dpp_add<0x141>(v);   // row_half_mirror
  if constexpr (LPC >= 16) v = scan_dpp_add<0x140>(v);  // row_mirror
  return v;
}

// PASS 0: a run with outputs (the whole request, or pass 3 of a long one); PASS 1: B and a of a run, no outputs.
// LPC lanes share a column's rows; a lane holds its 16 rows of CPL adjacent columns, so that a staged r, k or w
// entry read from LDS serves CPL columns.
// PERHEAD: one decay per head, staged once per token instead of once per row.
template <int PASS, int LPC, int CPL, bool BEFORE, bool PERHEAD>
// (four waves a SIMD, 128 registers; the walk with a bonus and four columns a lane needs more and takes two)
__global__ void __launch_bounds__(64 * kScanWaves)
__attribute__((amdgpu_waves_per_eu(PASS == 0 && BEFORE && CPL > 1 ? 2 : 4)))
linear_scan_kernel(ScanArgs a) {
  constexpr int kStage = CPL > 1 ? kScanStage / 2 : kScanStage;   // wide lanes: half the LDS, so that more blocks fit
  extern __shared__ float staged[];          // [kStage][NW * KP + VW + 2, padded]: r, k, (w), the block's v columns, step, decay
  const int h = blockIdx.y;
  constexpr int cols = kWave / LPC;          // lanes groups of a wave, CPL columns each
  constexpr int KP = LPC * kScanRows;
  const int VW = a.waves * cols * CPL;       // columns of v the block owns
  constexpr int NW = PERHEAD ? 2 : 3;        // rows of K entries staged per token
  const int per_token = NW * KP + ((VW + 5) & ~3);   // a token's rows stay 16-byte aligned
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int col0 = blockIdx.z * VW;
  const int vcol = (wave * cols + lane / LPC) * CPL;   // the lane's first column among the block's
  const int col = col0 + vcol;
  const int part = lane % LPC;               // which 16 rows of the columns
  const int row0 = part * kScanRows;
  const int K = a.K, V = a.V;
  int seq, run, runs;
  if (!scan_place(a, blockIdx.x, seq, run, runs)) return;
  if (PASS == 1 && run == runs - 1) return;  // nothing follows a request's last run
  const int s0 = a.cu_seqlens[seq], s1 = a.cu_seqlens[seq + 1];
  const int t0 = a.run_len == 0 ? s0 : s0 + run * a.run_len;
  const int t1 = a.run_len == 0 ? s1 : min(s1, t0 + a.run_len);
  const int slot = a.slot_of_seq[seq];
  if (slot < 0) {                            // a padding row: nothing to carry, its output is never read
    if (PASS == 0)
      for (int t = t0; t < t1; ++t)
        for (int c = 0; c < CPL; ++c)
          if (col + c < V && part == 0) a.out[(size_t)t * a.ldo + (size_t)h * V + col + c] = 0.f;
    return;
  }
  const size_t place = a.run_len == 0 ? 0 : (size_t)(s0 / a.run_len + seq + run);
  float* S_slot = a.state + (size_t)slot * a.slot_stride + a.state_off + (size_t)h * K * V;
  float* S_run = a.run_state != nullptr ? a.run_state + (place * a.H + h) * (size_t)K * V : nullptr;
  float S[CPL][kScanRows];
  if (PASS == 1) {
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
      for (int i = 0; i < kScanRows; ++i) S[c][i] = 0.f;
  } else {
    const float* from = runs > 1 ? S_run : S_slot;
#pragma unroll
    for (int i = 0; i < kScanRows; ++i)
#pragma unroll
      for (int c = 0; c < CPL; ++c)
        S[c][i] = (col + c < V && row0 + i < K) ? from[(size_t)(row0 + i) * V + col + c] : 0.f;
  }
  float u[kScanRows];                        // PASS 0: the bonus; PASS 1: the product of the run's decays
  constexpr bool before = BEFORE;
#pragma unroll
  for (int i = 0; i < kScanRows; ++i)
    u[i] = PASS == 1 ? 1.f : ((before && row0 + i < K) ? a.bonus[(size_t)h * K + row0 + i] : 0.f);
  const float skip = a.skip != nullptr ? a.skip[h] : 0.f;
  const int rh = h / a.r_div, kh = h / a.k_div;

  // One decay per head, first pass: B = sum_t (prod_{s > t} w_s) k_t (dt_t v_t)^T is formed from the run's last token
  // to its first with the product of the decays behind a token as a factor on its v: one multiply-add a (row, column).
  constexpr bool kBackward = PASS == 1 && PERHEAD;
  float behind = 1.f;                        // kBackward: the product of the decays of the tokens already walked
  const int stages = (t1 - t0 + kStage - 1) / kStage;
  for (int st = 0; st < stages; ++st) {
    const int base = t0 + (kBackward ? stages - 1 - st : st) * kStage;
    const int n = min(kStage, t1 - base);
    __syncthreads();
    // four entries a thread at a time, every load of the four asked for before the first is used
    for (int e0 = tid; e0 < n * KP; e0 += 4 * blockDim.x) {
      float rv[4], kv[4], wv[4], wb[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int e = e0 + x * blockDim.x;
        const int j = e / KP, i = e - j * KP;
        const size_t t = (size_t)(base + j);
        rv[x] = 0.f, kv[x] = 0.f, wv[x] = 1.f, wb[x] = 0.f;
        if (e < n * KP && i < K) {
          if (PASS == 0) rv[x] = a.r[t * a.ldr + (size_t)rh * K + i];
          kv[x] = a.k[t * a.ldk + (size_t)kh * K + i];
          if (!PERHEAD) {
            wv[x] = a.w_per_channel ? a.w[t * a.ldw + (size_t)h * K + i] : a.w[t * a.ldw + h];
            if (a.w_mode == 1) wb[x] = a.w_bias[(size_t)h * K + i];
          }
        }
      }
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int e = e0 + x * blockDim.x;
        if (e < n * KP) {
          const int j = e / KP, i = e - j * KP;
          float* dst = staged + (size_t)j * per_token;
          dst[i] = rv[x];
          dst[KP + i] = kv[x];
          if (!PERHEAD) dst[2 * KP + i] = (a.w_mode == 1 && i < K) ? expf(-expf(wv[x] + wb[x])) : wv[x];
        }
      }
    }
    for (int e = tid; e < n * (VW + 2); e += blockDim.x) {
      const int j = e / (VW + 2), c = e - j * (VW + 2);
      const size_t t = (size_t)(base + j);
      float x;
      if (c >= VW) {                           // the token's step size, then (one decay per head) its decay
        float step = a.v_scale != nullptr ? a.v_scale[t * a.ldvs + h] : 1.f;
        float decay = 1.f;
        if (PERHEAD) {
          decay = a.w[t * a.ldw + h];
          if (a.w_mode == 2) {
            const float z = decay + a.w_bias[h];
            step = z > 20.f ? z : log1pf(expf(z));
            decay = expf(-expf(a.a_log[h]) * step);
          }
        }
        x = c == VW ? step : decay;
      } else {
        x = col0 + c < V ? a.v[t * a.ldv + (size_t)h * V + col0 + c] : 0.f;
      }
      staged[(size_t)j * per_token + NW * KP + c] = x;
    }
    __syncthreads();
    for (int jj = 0; jj < n; ++jj) {
      const int j = kBackward ? n - 1 - jj : jj;
      const float* src = staged + (size_t)j * per_token;
      const float4* r4 = reinterpret_cast<const float4*>(src + row0);
      const float4* k4 = reinterpret_cast<const float4*>(src + KP + row0);
      const float4* w4 = reinterpret_cast<const float4*>(src + (NW - 1) * KP + row0);   // PERHEAD: not read
      const float step = src[NW * KP + VW];
      const float head_decay = src[NW * KP + VW + 1];
      float v_raw[CPL], v[CPL], acc[CPL];
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        v_raw[c] = src[NW * KP + vcol + c];
        v[c] = v_raw[c] * step;
        acc[c] = 0.f;
      }
      if (kBackward) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) v[c] *= behind;
        behind *= head_decay;
#pragma unroll
        for (int q = 0; q < kScanRows / 4; ++q) {
          const float4 kq = k4[q];
          const float kk[4] = {kq.x, kq.y, kq.z, kq.w};
#pragma unroll
          for (int x = 0; x < 4; ++x)
#pragma unroll
            for (int c = 0; c < CPL; ++c) S[c][4 * q + x] = fmaf(kk[x], v[c], S[c][4 * q + x]);
        }
        continue;
      }
#pragma unroll
      for (int q = 0; q < kScanRows / 4; ++q) {
        const float4 kq = k4[q];
        const float4 wq = PERHEAD ? float4{head_decay, head_decay, head_decay, head_decay} : w4[q];
        const float kk[4] = {kq.x, kq.y, kq.z, kq.w}, ww[4] = {wq.x, wq.y, wq.z, wq.w};
        if (PASS == 1) {
#pragma unroll
          for (int x = 0; x < 4; ++x) {
#pragma unroll
            for (int c = 0; c < CPL; ++c) S[c][4 * q + x] = ww[x] * S[c][4 * q + x] + kk[x] * v[c];
            u[4 * q + x] *= ww[x];
          }
        } else {
          const float4 rq = r4[q];
          const float rr[4] = {rq.x, rq.y, rq.z, rq.w};
          if (before) {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              const float ru = rr[x] * u[4 * q + x];
#pragma unroll
              for (int c = 0; c < CPL; ++c) {
                const float kv = kk[x] * v[c];
                acc[c] += rr[x] * S[c][4 * q + x] + ru * kv;
                S[c][4 * q + x] = ww[x] * S[c][4 * q + x] + kv;
              }
            }
          } else {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
#pragma unroll
              for (int c = 0; c < CPL; ++c) {
                S[c][4 * q + x] = ww[x] * S[c][4 * q + x] + kk[x] * v[c];
                acc[c] += rr[x] * S[c][4 * q + x];
              }
            }
          }
        }
      }
      if (PASS == 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
          const float sum = scan_group_sum<LPC>(acc[c]);
          if (col + c < V && part == 0) a.out[(size_t)(base + j) * a.ldo + (size_t)h * V + col + c] = sum + skip * v_raw[c];
        }
      }
    }
  }
  if (PASS == 1) {
    if (kBackward) {
#pragma unroll
      for (int i = 0; i < kScanRows; ++i) u[i] = behind;   // every row of the head decays alike
    }
#pragma unroll
    for (int i = 0; i < kScanRows; ++i)
#pragma unroll
      for (int c = 0; c < CPL; ++c)
        if (col + c < V && row0 + i < K) S_run[(size_t)(row0 + i) * V + col + c] = S[c][i];
    if (col == 0) {
      float* decay = a.run_decay + (place * a.H + h) * (size_t)K;
#pragma unroll
      for (int i = 0; i < kScanRows; ++i)
        if (row0 + i < K) decay[row0 + i] = u[i];
    }
  } else if (run == runs - 1) {
#pragma unroll
    for (int i = 0; i < kScanRows; ++i)
#pragma unroll
      for (int c = 0; c < CPL; ++c)
        if (col + c < V && row0 + i < K) S_slot[(size_t)(row0 + i) * V + col + c] = S[c][i];
  }
}

// Pass 2: per request of several runs and per entry of S, the state before every run: the slot's state before the
// first, then S <- a_j S + B_j from run to run; it takes B's place.
__global__ void __launch_bounds__(256) linear_scan_fold_kernel(ScanArgs a) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int K = a.K, V = a.V;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= K * V) return;
  const int slot = a.slot_of_seq[seq];
  const int t0 = a.cu_seqlens[seq], len = a.cu_seqlens[seq + 1] - t0;
  const int runs = (len + a.run_len - 1) / a.run_len;
  if (slot < 0 || runs <= 1) return;
  const int row = e / V;
  const size_t first = (size_t)(t0 / a.run_len + seq);
  const size_t stride = (size_t)a.H * K * V, dstride = (size_t)a.H * K;
  float* B = a.run_state + (first * a.H + h) * (size_t)K * V + e;
  const float* decay = a.run_decay + (first * a.H + h) * (size_t)K + row;
  float S = a.state[(size_t)slot * a.slot_stride + a.state_off + (size_t)h * K * V + e];
  constexpr int kAhead = 8;
  for (int j0 = 0; j0 < runs; j0 += kAhead) {
    float b[kAhead], d[kAhead];
#pragma unroll
    for (int c = 0; c < kAhead; ++c) {
      const bool has = j0 + c < runs - 1;
      b[c] = has ? B[(size_t)(j0 + c) * stride] : 0.f;
      d[c] = has ? decay[(size_t)(j0 + c) * dstride] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < kAhead; ++c) {
      if (j0 + c < runs) {
        B[(size_t)(j0 + c) * stride] = S;
        S = d[c] * S + b[c];
      }
    }
  }
}

ATOM_EXPORT int atom_linear_scan(const float* r, long ldr, int r_div, const float* k, long ldk, int k_div, const float* v,
                                 long ldv, const float* w, long ldw, int w_per_channel, const float* w_bias, int w_mode,
                                 const float* a_log, const float* v_scale, long ldvs, const float* bonus, const float* skip, float* out,
                                 long ldo, float* state, long slot_stride, long state_off, const int* cu_seqlens,
                                 const int* slot_of_seq, int num_seqs, int H, int K, int V, int tokens, int run_len,
                                 float* run_state, float* run_decay, long places, hipStream_t stream) {
  if (H <= 0 || K <= 0 || V <= 0 || num_seqs < 0 || r_div <= 0 || k_div <= 0 || tokens < 0) return ATOM_BAD_SHAPE;
  if (r == nullptr || k == nullptr || v == nullptr || w == nullptr || out == nullptr || state == nullptr) return ATOM_BAD_SHAPE;
  if (cu_seqlens == nullptr || slot_of_seq == nullptr) return ATOM_BAD_SHAPE;
  if (w_mode < 0 || w_mode > 2) return ATOM_UNSUPPORTED;
  if (w_mode == 1 && (w_bias == nullptr || !w_per_channel)) return ATOM_BAD_SHAPE;
  if (w_mode == 2 && (w_bias == nullptr || a_log == nullptr || w_per_channel)) return ATOM_BAD_SHAPE;
  if (w_mode == 2 && (bonus != nullptr || v_scale != nullptr)) return ATOM_UNSUPPORTED;
  if (state_off < 0 || slot_stride < state_off + (long)H * K * V) return ATOM_BAD_SHAPE;
  if (K > 16 * kScanRows) return ATOM_TOO_LARGE;
  if (run_len < 0 || run_len % kScanStage) return ATOM_BAD_SHAPE;
  const long need = run_len > 0 ? (long)(tokens + run_len - 1) / run_len + num_seqs : 0;
  if (run_len > 0 && (run_state == nullptr || run_decay == nullptr || places < need)) return ATOM_BAD_SHAPE;
  if (num_seqs == 0) return ATOM_OK;
  int lpc = 1;
  while (lpc * kScanRows < K) lpc <<= 1;
  const int cols = kWave / lpc;
  // long requests in runs: four columns a lane, so that a staged row serves four columns, where that still leaves
  // waves enough to fill the chip; otherwise one column a lane, which gives the most waves
  const bool wide = run_len > 0 && V >= 4 * cols && need * H * ((V + 4 * cols - 1) / (4 * cols)) >= 2048;
  const int cpl = wide ? 4 : 1;
  const int waves = min(kScanWaves, (V + cols * cpl - 1) / (cols * cpl));
  const int vw = waves * cols * cpl;
  const long blocks_x = run_len > 0 ? need : num_seqs;
  if (blocks_x > 0x7fffffff || H > 65535 || (V + vw - 1) / vw > 65535 || ((long)K * V + 255) / 256 > 65535) return ATOM_TOO_LARGE;
  ScanArgs a{r, ldr, r_div, k, ldk, k_div, v, ldv, w, ldw, w_per_channel, w_bias, w_mode, a_log, v_scale, ldvs, bonus, skip,
             out, ldo, state, slot_stride, state_off, cu_seqlens, slot_of_seq, num_seqs, H, K, V, lpc, waves, run_len,
             run_len > 0 ? run_state : nullptr, run_len > 0 ? run_decay : nullptr};
  const bool perhead = !w_per_channel && bonus == nullptr;   // one staged decay a token instead of one a row
  const size_t smem = (size_t)(cpl > 1 ? kScanStage / 2 : kScanStage) *
                      ((perhead ? 2 : 3) * lpc * kScanRows + ((vw + 5) & ~3)) * sizeof(float);
  const dim3 grid((unsigned)blocks_x, H, (V + vw - 1) / vw), block(kWave * waves);
#define ATOM_SCAN_LAUNCH(PASS, LPC, CPL)                                                                     \
  if (perhead)                                                                                               \
    hipLaunchKernelGGL((linear_scan_kernel<PASS, LPC, CPL, false, true>), grid, block, smem, stream, a);     \
  else if (PASS == 0 && bonus != nullptr)                                                                    \
    hipLaunchKernelGGL((linear_scan_kernel<PASS, LPC, CPL, true, false>), grid, block, smem, stream, a);     \
  else                                                                                                       \
    hipLaunchKernelGGL((linear_scan_kernel<PASS, LPC, CPL, false, false>), grid, block, smem, stream, a)
#define ATOM_SCAN_BY_LPC(PASS, CPL)                       \
  switch (lpc) {                                          \
    case 1: ATOM_SCAN_LAUNCH(PASS, 1, CPL); break;        \
    case 2: ATOM_SCAN_LAUNCH(PASS, 2, CPL); break;        \
    case 4: ATOM_SCAN_LAUNCH(PASS, 4, CPL); break;        \
    case 8: ATOM_SCAN_LAUNCH(PASS, 8, CPL); break;        \
    default: ATOM_SCAN_LAUNCH(PASS, 16, CPL); break;      \
  }
  if (run_len > 0) {
    if (cpl == 4) { ATOM_SCAN_BY_LPC(1, 4) } else { ATOM_SCAN_BY_LPC(1, 1) }
    hipLaunchKernelGGL(linear_scan_fold_kernel, dim3(num_seqs, H, (unsigned)(((long)K * V + 255) / 256)), dim3(256), 0, stream, a);
  }
  if (cpl == 4) { ATOM_SCAN_BY_LPC(0, 4) } else { ATOM_SCAN_BY_LPC(0, 1) }
#undef ATOM_SCAN_BY_LPC
#undef ATOM_SCAN_LAUNCH
  return launch_status();
}

// ------------------------------------------------------------------ a token's input mixed with the previous token's

// mixes[s, t, :] = x[t] + (x[t - 1] - x[t]) * mu[s] for s < n; x[t - 1] of a request's first token of the step is
// the row its state slot holds (zeros for a fresh request), and the step's last row of the request is left there.
// The block of a request's first token reads the slot before it writes it, column by column.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ x, const float* __restrict__ mu, int n, T* __restrict__ mixes,
                   float* __restrict__ state, long slot_stride, long state_off, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ slot_of_seq, const int* __restrict__ token_seq, int tokens, int width) {
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const T* row = x + (size_t)t * width;
  const bool padding = seq < 0;
  const int first = padding ? t : cu_seqlens[seq];
  const int slot = padding ? -1 : slot_of_seq[seq];
  const bool heads = t == first;             // the request's first token of this step
  const int last = padding ? t : cu_seqlens[seq + 1] - 1;
  float* kept = slot >= 0 ? state + (size_t)slot * slot_stride + state_off : nullptr;
  #pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float cur = to_f32(row[i]);
    float prev;
    if (heads) {
      prev = kept != nullptr ? kept[i] : 0.f;
      if (kept != nullptr) kept[i] = to_f32(x[(size_t)last * width + i]);
    } else {
      prev = to_f32(x[(size_t)(t - 1) * width + i]);
    }
    const float d = prev - cur;
    for (int s = 0; s < n; ++s)
      mixes[((size_t)s * tokens + t) * width + i] = from_f32<T>(cur + d * mu[(size_t)s * width + i]);
  }
}

// The same with 16 bytes a thread and every load of a thread asked for before the first is used: widths that are a
// multiple of 16 / sizeof(T), up to 8 mixes, rows and state rows 16-byte aligned.
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_vec_kernel(const T* __restrict__ x, const float* __restrict__ mu, int n, T* __restrict__ mixes,
                       float* __restrict__ state, long slot_stride, long state_off, const int* __restrict__ cu_seqlens,
                       const int* __restrict__ slot_of_seq, const int* __restrict__ token_seq, int tokens, int width) {
  constexpr int N = 16 / sizeof(T);
  union Pack { uint4 raw; T e[N]; };
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const bool padding = seq < 0;
  const int first = padding ? t : cu_seqlens[seq];
  const int slot = padding ? -1 : slot_of_seq[seq];
  const bool heads = t == first;
  const int last = padding ? t : cu_seqlens[seq + 1] - 1;
  float* kept = slot >= 0 ? state + (size_t)slot * slot_stride + state_off : nullptr;
  for (int c = threadIdx.x; c < width / N; c += blockDim.x) {
    const int i0 = c * N;
    Pack cur, before, tail;
    cur.raw = *reinterpret_cast<const uint4*>(x + (size_t)t * width + i0);
    float prev[N];
    if (heads) {
      tail.raw = *reinterpret_cast<const uint4*>(x + (size_t)last * width + i0);
#pragma unroll
      for (int q = 0; q < N / 4; ++q) {
        float4 k4 = kept != nullptr ? *reinterpret_cast<const float4*>(kept + i0 + 4 * q) : float4{0.f, 0.f, 0.f, 0.f};
        prev[4 * q] = k4.x, prev[4 * q + 1] = k4.y, prev[4 * q + 2] = k4.z, prev[4 * q + 3] = k4.w;
      }
    } else {
      before.raw = *reinterpret_cast<const uint4*>(x + (size_t)(t - 1) * width + i0);
#pragma unroll
      for (int i = 0; i < N; ++i) prev[i] = to_f32(before.e[i]);
    }
    float4 m[8][N / 4];
#pragma unroll
    for (int sx = 0; sx < 8; ++sx)
      if (sx < n) {
#pragma unroll
        for (int q = 0; q < N / 4; ++q) m[sx][q] = *reinterpret_cast<const float4*>(mu + (size_t)sx * width + i0 + 4 * q);
      }
    if (heads && kept != nullptr) {
#pragma unroll
      for (int q = 0; q < N / 4; ++q)
        *reinterpret_cast<float4*>(kept + i0 + 4 * q) = float4{to_f32(tail.e[4 * q]), to_f32(tail.e[4 * q + 1]),
                                                                to_f32(tail.e[4 * q + 2]), to_f32(tail.e[4 * q + 3])};
    }
#pragma unroll
    for (int sx = 0; sx < 8; ++sx)
      if (sx < n) {
        Pack res;
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
          const float w4[4] = {m[sx][q].x, m[sx][q].y, m[sx][q].z, m[sx][q].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float cv = to_f32(cur.e[4 * q + i]);
            res.e[4 * q + i] = from_f32<T>(cv + (prev[4 * q + i] - cv) * w4[i]);
          }
        }
        *reinterpret_cast<uint4*>(mixes + ((size_t)sx * tokens + t) * width + i0) = res.raw;
      }
  }
}

ATOM_EXPORT int atom_token_shift(const void* x, int dtype, const float* mu, int n, void* mixes, float* state,
                                 long slot_stride, long state_off, const int* cu_seqlens, const int* slot_of_seq,
                                 const int* token_seq, int tokens, int width, hipStream_t stream) {
  if (tokens < 0 || width <= 0 || n <= 0 || state_off < 0 || slot_stride < state_off + width) return ATOM_BAD_SHAPE;
  if (x == nullptr || mu == nullptr || mixes == nullptr || state == nullptr) return ATOM_BAD_SHAPE;
  if (cu_seqlens == nullptr || slot_of_seq == nullptr || token_seq == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  const int per = dtype == ATOM_F32 ? 4 : 8;
  const bool vec = n <= 8 && width % per == 0 && ((uintptr_t)x | (uintptr_t)mixes | (uintptr_t)mu | (uintptr_t)state) % 16 == 0 &&
                   slot_stride % 4 == 0 && state_off % 4 == 0;
  if (vec) {
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((token_shift_vec_kernel<T>), dim3(tokens), dim3(256), 0, stream,
                                                   (const T*)x, mu, n, (T*)mixes, state, slot_stride, state_off, cu_seqlens,
                                                   slot_of_seq, token_seq, tokens, width));
    return launch_status();
  }
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((token_shift_kernel<T>), dim3(tokens), dim3(256), 0, stream, (const T*)x, mu,
                                                 n, (T*)mixes, state, slot_stride, state_off, cu_seqlens, slot_of_seq,
                                                 token_seq, tokens, width));
  return launch_status();
}

// ------------------------------------------------------------------ step sizes and decays of a state-space layer

// dt[t, h] = softplus(raw[t, h] + dt_bias[h]) (no clamp), decay[t, h] = exp(-exp(A_log[h]) dt[t, h]).
__global__ void step_decay_kernel(const float* __restrict__ raw, long ld, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, float* __restrict__ dt, float* __restrict__ decay,
                                  int heads, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / heads;
  const int h = (int)(idx - t * heads);
  const float z = raw[t * ld + h] + dt_bias[h];
  const float step = z > 20.f ? z : log1pf(expf(z));
  dt[idx] = step;
  decay[idx] = expf(-expf(a_log[h]) * step);
}

ATOM_EXPORT int atom_step_decay(const float* raw, long ld, const float* dt_bias, const float* a_log, float* dt,
                                float* decay, int tokens, int heads, hipStream_t stream) {
  if (tokens < 0 || heads <= 0 || ld < heads) return ATOM_BAD_SHAPE;
  if (raw == nullptr || dt_bias == nullptr || a_log == nullptr || dt == nullptr || decay == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)tokens * heads;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  hipLaunchKernelGGL(step_decay_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, raw, ld, dt_bias, a_log, dt, decay,
                     heads, total);
  return launch_status();
}

// ------------------------------------------------------------------ RMS norm in equal parts of a row, with a gate

// out[t, g, :] = y / rms(y) * weight * silu(gate)      (gate_first 0: the gate multiplies the normed row)
// out[t, g, :] = z / rms(z) * weight, z = y * silu(gate) (gate_first 1: the gate comes before the norm)
// for each of `groups` equal parts of a row of y (float32); gate: float32 [T, ldg], the row's gate values from
// column 0 (null: no gate); weight: float32 [groups * gw] (null: ones).  A part no wider than 256 is summed by one wave (a row's parts spread
// over the waves of up to 64 blocks), a wider one by the whole block of its token.
__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

template <typename T>
__global__ void __launch_bounds__(256)
group_norm_gate_kernel(const float* __restrict__ y, long ldy, const float* __restrict__ gate, long ldg,
                       const float* __restrict__ weight, T* __restrict__ out, int groups, int gw, float eps,
                       int gate_first) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const float* yr = y + t * ldy;
  const float* gr = gate != nullptr ? gate + t * ldg : nullptr;
  T* dst = out + t * (size_t)groups * gw;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, waves = blockDim.x / kWave;
  if (gw <= 256) {
    for (int g = blockIdx.y * waves + wave; g < groups; g += gridDim.y * waves) {
      const int base = g * gw;
      float vals[4];
      float ss = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = lane + r * kWave;
        float v = 0.f;
        if (i < gw) {
          v = yr[base + i];
          if (gate_first && gr != nullptr) v *= silu_f(gr[base + i]);
        }
        vals[r] = v;
        ss += v * v;
      }
      const float inv = 1.f / sqrtf(wave_sum(ss) / (float)gw + eps);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = lane + r * kWave;
        if (i < gw) {
          float v = vals[r] * inv;
          if (weight != nullptr) v *= weight[base + i];
          if (!gate_first && gr != nullptr) v *= silu_f(gr[base + i]);
          dst[base + i] = from_f32<T>(v);
        }
      }
    }
    return;
  }
  for (int g = 0; g < groups; ++g) {
    const int base = g * gw;
    float ss = 0.f;
    #pragma unroll 4
    for (int i = threadIdx.x; i < gw; i += blockDim.x) {
      float v = yr[base + i];
      if (gate_first && gr != nullptr) v *= silu_f(gr[base + i]);
      ss += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)gw + eps);
    #pragma unroll 4
    for (int i = threadIdx.x; i < gw; i += blockDim.x) {
      float v = yr[base + i];
      const float s = gr != nullptr ? silu_f(gr[base + i]) : 1.f;
      if (gate_first) v *= s;
      v *= inv;
      if (weight != nullptr) v *= weight[base + i];
      if (!gate_first) v *= s;
      dst[base + i] = from_f32<T>(v);
    }
  }
}

// Parts wider than 256 entries whose rows are 16-byte aligned: a part's entries (up to 8,192) stay in registers, four
// consecutive ones a load, every load asked for before the first is used; memory is read once.
template <typename T>
__global__ void __launch_bounds__(256)
group_norm_gate_vec_kernel(const float* __restrict__ y, long ldy, const float* __restrict__ gate, long ldg,
                           const float* __restrict__ weight, T* __restrict__ out, int groups, int gw, float eps,
                           int gate_first) {
  constexpr int PER = 8;
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const float* yr = y + t * ldy;
  const float* gr = gate != nullptr ? gate + t * ldg : nullptr;
  T* dst = out + t * (size_t)groups * gw;
  for (int g = 0; g < groups; ++g) {
    const int base = g * gw;
    float4 v[PER], sg[PER], w[PER];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = (threadIdx.x + r * 256) * 4;
      v[r] = sg[r] = float4{0.f, 0.f, 0.f, 0.f};
      w[r] = float4{1.f, 1.f, 1.f, 1.f};
      if (i < gw) {
        v[r] = *reinterpret_cast<const float4*>(yr + base + i);
        if (gr != nullptr) sg[r] = *reinterpret_cast<const float4*>(gr + base + i);
        if (weight != nullptr) w[r] = *reinterpret_cast<const float4*>(weight + base + i);
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      if (gr != nullptr) sg[r] = float4{silu_f(sg[r].x), silu_f(sg[r].y), silu_f(sg[r].z), silu_f(sg[r].w)};
      else sg[r] = float4{1.f, 1.f, 1.f, 1.f};
      if (gate_first) v[r] = float4{v[r].x * sg[r].x, v[r].y * sg[r].y, v[r].z * sg[r].z, v[r].w * sg[r].w};
      ss += v[r].x * v[r].x + v[r].y * v[r].y + v[r].z * v[r].z + v[r].w * v[r].w;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)gw + eps);
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = (threadIdx.x + r * 256) * 4;
      if (i < gw) {
        float o[4] = {v[r].x * inv * w[r].x, v[r].y * inv * w[r].y, v[r].z * inv * w[r].z, v[r].w * inv * w[r].w};
        if (!gate_first) o[0] *= sg[r].x, o[1] *= sg[r].y, o[2] *= sg[r].z, o[3] *= sg[r].w;
#pragma unroll
        for (int x = 0; x < 4; ++x) dst[base + i + x] = from_f32<T>(o[x]);
      }
    }
  }
}

ATOM_EXPORT int atom_group_norm_gate(const float* y, long ldy, const float* gate, long ldg, const float* weight, void* out,
                                     int out_dtype, int tokens, int groups, int gw, float eps, int gate_first,
                                     hipStream_t stream) {
  if (tokens < 0 || groups <= 0 || gw <= 0 || ldy < (long)groups * gw) return ATOM_BAD_SHAPE;
  if (gate != nullptr && ldg < (long)groups * gw) return ATOM_BAD_SHAPE;
  if (y == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  const bool vec = gw > 256 && gw <= 8192 && gw % 4 == 0 && ldy % 4 == 0 && (gate == nullptr || ldg % 4 == 0) &&
                   ((uintptr_t)y | (uintptr_t)gate | (uintptr_t)weight) % 16 == 0;
  if (vec) {
    ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((group_norm_gate_vec_kernel<T>), dim3(tokens), dim3(256), 0, stream, y,
                                                       ldy, gate, ldg, weight, (T*)out, groups, gw, eps, gate_first));
    return launch_status();
  }
  // narrow parts: a wave a part, the parts of a row spread over blocks
  const unsigned across = gw <= 256 ? (unsigned)min(64, (groups + 3) / 4) : 1u;
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((group_norm_gate_kernel<T>), dim3(tokens, across), dim3(256), 0, stream, y,
                                                     ldy, gate, ldg, weight, (T*)out, groups, gw, eps, gate_first));
  return launch_status();
}
