// Attention with a token's heads worked through together (see attention_together.hip for what is computed), on the
// matrix cores: bfloat16, key heads of 64 or 128 entries, value heads of 32, 64 or 128, up to 16 heads a block,
// pages of a multiple of four tokens.  For steps that bring prompt portions.
//
// A block of four waves owns a tile of up to 16 consecutive query tokens of one request and a set of heads: all of
// them when the heads' weights are mixed, else the query heads of one key/value head.  The heads are dealt out to the
// waves.  Both products are formed transposed, so a lane always holds values of one query token (lane % 16):
//
//     S^T[key][query] = K[key][:] . Q[query][:]        A = K rows from the key pages, B = Q (kept in registers)
//     O^T[d][query]   = V^T[d][key] . W[query][key]    A = V^T rows (value pages hold keys contiguously), B = W
//
// The first product leaves lane (query, g = lane / 16) with the scores of keys 4g .. 4g + 3 of a chunk of 16, which
// is the B operand of the second.  The keys are walked twice: once for every (query, head)'s maximum and sum, which
// are per-lane numbers, then for the finished weights.  Mixing the heads is entrywise in this layout: the waves
// exchange their heads' weights of a chunk through LDS (two buffers in turn, one barrier a chunk) and every wave
// forms sum_g talk[h, g] w_g for its own heads.  Chunks are counted from position 0.  A chunk's key rows are asked for
// one chunk ahead of their use and its value rows before its scores are formed, so a wave waits for memory less.
//
// Where the tiles alone would leave the chip idle, a tile's chunks are cut over `parts` blocks (three launches, as in
// attention_together.hip: maxima and sums, shares of the weighted sum, their sum in the order of the parts).
//
// A block finds its request and tile from the block index alone: tile j of request s has the place
// cu[s] / 16 + s + j, which is unique, so the launch needs no list of tiles from the host.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float tg_f32x4;
typedef __attribute__((ext_vector_type(4))) short tg_s16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 tg_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 tg_bf16x4;

constexpr int kTileWaves = 4;
constexpr int kTileRows = 16;

struct TogetherTileArgs {
  const bf16_t* q; const bf16_t* k_cache; const bf16_t* v_cache; bf16_t* out;
  const int* cu_q; const int* positions; const int* block_tables;
  int max_blocks, num_seqs, H, G, page_size, window;
  float scale_log2;
  const float* head_scale; const float* sink; const float* talk;
  int parts;          // > 1: a tile's chunks are cut over this many blocks (grid z), in three launches
  float* ws_ml;       // [tokens, H, parts, 2]: a part's maximum (exp2 domain) and sum
  float* ws_o;        // [tokens, parts, H, DV]: a part's share of the weighted sum
};

// PASS 0: both walks over all of the tile's chunks.  PASS 1: the maximum and sum of this part's chunks.  PASS 2: the
// parts' maxima and sums merged in the order of the parts, then this part's share of the weighted sum.
template <int D, int NDV, int HPW, int PASS>
__global__ void __launch_bounds__(kTileWaves * kWave)
together_tile_kernel(TogetherTileArgs a) {
  constexpr int DV = 16 * NDV;
  constexpr float kLog2e = 1.4426950408889634f;
  __shared__ tg_f32x4 pbuf[2][HPW * kTileWaves][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n = lane & 15, g4 = lane >> 4;
  // the request and the tile of this block: the last s with cu[s] / 16 + s <= b
  const int b = blockIdx.x;
  int lo = 0, hi = a.num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (a.cu_q[mid] / kTileRows + mid <= b) lo = mid; else hi = mid - 1;
  }
  const int seq = lo;
  const int t_begin = a.cu_q[seq], t_end = a.cu_q[seq + 1];
  const int tile = b - (t_begin / kTileRows + seq);
  if (tile < 0 || tile * kTileRows >= t_end - t_begin) return;   // the whole block leaves together
  const int t0 = t_begin + tile * kTileRows;
  const int rows = t_end - t0 < kTileRows ? t_end - t0 : kTileRows;
  const bool row_ok = n < rows;
  const int pos = row_ok ? a.positions[t0 + n] : -1;
  const int pos_lo = a.positions[t0], pos_hi = a.positions[t0 + rows - 1];
  const int first_row = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const int first_blk = (a.window > 0 && pos_lo - a.window + 1 > 0) ? pos_lo - a.window + 1 : 0;
  const int* table = a.block_tables + (size_t)seq * a.max_blocks;
  const bool mixes = a.talk != nullptr;
  const int HB = mixes ? a.H : a.H / a.G;
  const int h0 = mixes ? 0 : blockIdx.y * HB;
  const int group = a.H / a.G;
  const int ps = a.page_size;

  // A wave whose share of the heads is not full works a stand-in head (the block's first, with a query of zeros) and
  // stores nothing for it: the loops below then have no branch around their loads.
  tg_bf16x8 qf[HPW][D / 32];
  float top[HPW], den[HPW], hs[HPW];
  bool own[HPW];
  int head[HPW];
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int hh = wave + kTileWaves * u;
    own[u] = hh < HB;
    const int h = head[u] = h0 + (own[u] ? hh : 0);
    const bf16_t* qr = a.q + ((size_t)(t0 + (row_ok ? n : 0)) * a.H + h) * D + 8 * g4;
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
      tg_bf16x8 v = *reinterpret_cast<const tg_bf16x8*>(qr + 32 * j);
      if (!row_ok || !own[u]) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.f;
      }
      qf[u][j] = v;
    }
    top[u] = -INFINITY;
    den[u] = 0.f;
    hs[u] = a.scale_log2 * (a.head_scale != nullptr ? a.head_scale[h] : 1.f);
  }

  // The 16 key rows from base as this lane's part of the A operand of the first product (head u's key/value head).
  struct KeyRows { tg_bf16x8 f[D / 32]; };
  auto load_keys = [&](int u, int base) -> KeyRows {
    const int h = head[u];
    int key = base + n;                       // the key row this lane brings
    if (key > pos_hi) key = pos_hi;           // beyond the tile's last key: any valid row, masked in the scores
    const int page = table[key / ps], off = key - key / ps * ps;
    const bf16_t* kr = a.k_cache + (((size_t)page * a.G + h / group) * ps + off) * (size_t)D + 8 * g4;
    KeyRows k;
#pragma unroll
    for (int j = 0; j < D / 32; ++j) k.f[j] = *reinterpret_cast<const tg_bf16x8*>(kr + 32 * j);
    return k;
  };
  // scores of head u against those keys, in the exp2 domain, -inf where the lane's query does not see the key
  auto scores = [&](int u, const KeyRows& k, int base) -> tg_f32x4 {
    tg_f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < D / 32; ++j) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k.f[j], qf[u][j], s, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = base + 4 * g4 + i;
      s[i] = (key >= first_row && key <= pos) ? s[i] * hs[u] : -INFINITY;
    }
    return s;
  };
  // The values of the four keys from base + 4 g4, rows n + 16 t of head u's value head: the A operand of the second
  // product.  One page holds the four.
  struct ValueRows { tg_bf16x4 f[NDV]; };
  auto load_values = [&](int u, int base) -> ValueRows {
    int key0 = base + 4 * g4;
    if (key0 > pos_hi) key0 = pos_hi & ~3;      // unseen by every query: any valid place, the weights are zero
    const int page = table[key0 / ps], off = key0 - key0 / ps * ps;
    const int kvh = head[u] / group;
    const bf16_t* vr = a.v_cache + (((size_t)page * a.G + kvh) * DV + n) * (size_t)ps + off;
    ValueRows v;
#pragma unroll
    for (int t = 0; t < NDV; ++t) v.f[t] = *reinterpret_cast<const tg_bf16x4*>(vr + (size_t)16 * t * ps);
    return v;
  };

  int start = first_blk / kTileRows * kTileRows;
  int stop = pos_hi + 1;                       // chunks from start up to, not including, stop
  if (PASS != 0) {
    const int chunks = (pos_hi - start) / kTileRows + 1;
    const int each = (chunks + a.parts - 1) / a.parts;
    const int c0 = blockIdx.z * each, c1 = c0 + each < chunks ? c0 + each : chunks;
    stop = start + c1 * kTileRows;
    start += c0 * kTileRows;                   // start >= stop: this part has no chunk
  }
  KeyRows ahead[HPW];
  if (PASS != 2) {
  // every (query, head)'s maximum and sum; the next chunk's key rows are asked for before this chunk's are used
#pragma unroll
  for (int u = 0; u < HPW; ++u) ahead[u] = load_keys(u, start);
  for (int base = start; base < stop; base += kTileRows) {
    KeyRows now[HPW];
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      now[u] = ahead[u];
      ahead[u] = load_keys(u, base + kTileRows);    // past the last chunk: the tile's last key again, not used
    }
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const tg_f32x4 s = scores(u, now[u], base);
      const float cm = rows_max(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
      const float m_new = fmaxf(top[u], cm);
      // no branch around the exchange between lanes: a query that has seen no key yet keeps a sum of zero
      const float m_at = m_new == -INFINITY ? 0.f : m_new;
      const float part = exp2f(s[0] - m_at) + exp2f(s[1] - m_at) + exp2f(s[2] - m_at) + exp2f(s[3] - m_at);
      den[u] = den[u] * exp2f(top[u] - m_at) + rows_sum(part);
      top[u] = m_new;
    }
  }
  }
  if (PASS == 1) {
    if (row_ok && g4 == 0) {
#pragma unroll
      for (int u = 0; u < HPW; ++u) {
        if (!own[u]) continue;
        float* ml = a.ws_ml + (((size_t)(t0 + n) * a.H + h0 + wave + kTileWaves * u) * a.parts + blockIdx.z) * 2;
        ml[0] = top[u], ml[1] = den[u];
      }
    }
    return;
  }
  if (PASS == 2 && row_ok) {
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      if (!own[u]) continue;
      const float* ml = a.ws_ml + ((size_t)(t0 + n) * a.H + h0 + wave + kTileWaves * u) * a.parts * 2;
      float m = -INFINITY, l = 0.f;
      for (int p = 0; p < a.parts; ++p) m = fmaxf(m, ml[2 * p]);
      for (int p = 0; p < a.parts; ++p)
        if (ml[2 * p] != -INFINITY) l += ml[2 * p + 1] * exp2f(ml[2 * p] - m);
      top[u] = m, den[u] = l;
    }
  }
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    float m = top[u], l = den[u];
    if (a.sink != nullptr && row_ok) {
      const float sk = a.sink[head[u]] * kLog2e;
      const float m_new = fmaxf(m, sk);
      l = l * exp2f(m - m_new) + exp2f(sk - m_new);
      m = m_new;
    }
    den[u] = l > 0.f ? 1.f / l : 0.f;
    top[u] = m == -INFINITY ? 0.f : m;
  }

  // the weights, their mixing, the weighted sum of the values
  tg_f32x4 acc[HPW][NDV];
#pragma unroll
  for (int u = 0; u < HPW; ++u)
#pragma unroll
    for (int t = 0; t < NDV; ++t) acc[u][t] = tg_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < HPW; ++u) ahead[u] = load_keys(u, start);
  int turn = 0;
  for (int base = start; base < stop; base += kTileRows, turn ^= 1) {
    KeyRows now[HPW];
    ValueRows vals[HPW];
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      now[u] = ahead[u];
      vals[u] = load_values(u, base);          // in flight while the scores are formed
      ahead[u] = load_keys(u, base + kTileRows);
    }
    tg_f32x4 w[HPW];
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      const tg_f32x4 s = scores(u, now[u], base);
#pragma unroll
      for (int i = 0; i < 4; ++i) w[u][i] = exp2f(s[i] - top[u]) * den[u];   // exp2(-inf) = 0 where unseen
      if (mixes) pbuf[turn][wave + kTileWaves * u][lane] = w[u];
    }
    if (mixes) {
      __syncthreads();
#pragma unroll
      for (int u = 0; u < HPW; ++u) {
        const float* row = a.talk + (size_t)head[u] * a.H;
        tg_f32x4 m = {0.f, 0.f, 0.f, 0.f};
        for (int g = 0; g < a.H; ++g) {
          const float c = row[g];
          const tg_f32x4 p = pbuf[turn][g][lane];
          m[0] += c * p[0], m[1] += c * p[1], m[2] += c * p[2], m[3] += c * p[3];
        }
        w[u] = m;
      }
    }
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      tg_bf16x4 pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) pb[i] = (__bf16)w[u][i];
#pragma unroll
      for (int t = 0; t < NDV; ++t)
        acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(tg_s16x4, vals[u].f[t]),
                                                              __builtin_bit_cast(tg_s16x4, pb), acc[u][t], 0, 0, 0);
    }
  }
  if (!row_ok) return;
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    if (!own[u]) continue;
    const int h = h0 + wave + kTileWaves * u;
    if (PASS == 2) {
      float* dst = a.ws_o + (((size_t)(t0 + n) * a.parts + blockIdx.z) * a.H + h) * DV + 4 * g4;
#pragma unroll
      for (int t = 0; t < NDV; ++t) *reinterpret_cast<tg_f32x4*>(dst + 16 * t) = acc[u][t];
      continue;
    }
    bf16_t* dst = a.out + ((size_t)(t0 + n) * a.H + h) * DV + 4 * g4;
#pragma unroll
    for (int t = 0; t < NDV; ++t) {
      tg_bf16x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (__bf16)acc[u][t][i];
      *reinterpret_cast<tg_bf16x4*>(dst + 16 * t) = o;
    }
  }
}

static bool together_tile_takes(int H, int G, int D, int DV, int page_size, bool mixes) {
  const int HB = mixes ? H : H / G;
  return (D == 64 || D == 128) && (DV == 32 || DV == 64 || DV == 128) && HB >= 1 && HB <= 16 && page_size % 4 == 0;
}

ATOM_EXPORT int atom_attention_together_tiles_supports(int H, int G, int D, int DV, int page_size, int mixes) {
  return (H > 0 && G > 0 && H % G == 0 && together_tile_takes(H, G, D, DV, page_size, mixes != 0)) ? 1 : 0;
}

template <int D, int NDV, int HPW>
static void together_tile_passes(const TogetherTileArgs& a, dim3 grid, hipStream_t stream) {
  const dim3 block(kTileWaves * kWave);
  if (a.parts == 1) {
    hipLaunchKernelGGL((together_tile_kernel<D, NDV, HPW, 0>), grid, block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((together_tile_kernel<D, NDV, HPW, 1>), grid, block, 0, stream, a);
    hipLaunchKernelGGL((together_tile_kernel<D, NDV, HPW, 2>), grid, block, 0, stream, a);
  }
}

template <int D, int NDV>
static int together_tile_launch(const TogetherTileArgs& a, dim3 grid, int HB, hipStream_t stream) {
  if (HB <= 4) together_tile_passes<D, NDV, 1>(a, grid, stream);
  else if (HB <= 8) together_tile_passes<D, NDV, 2>(a, grid, stream);
  else together_tile_passes<D, NDV, 4>(a, grid, stream);
  return launch_status();
}

ATOM_EXPORT int atom_attention_together_tiles(const void* q, const void* k_cache, const void* v_cache, void* out,
                                              const int* cu_q, const int* positions, const int* block_tables,
                                              int max_blocks, int tokens, int num_seqs, int H, int G, int D, int DV,
                                              int page_size, float scale, const float* head_scale, const float* sink,
                                              const float* talk, int window, int parts, float* ws_ml, float* ws_o,
                                              hipStream_t stream) {
  if (tokens < 0 || num_seqs <= 0 || H <= 0 || G <= 0 || H % G || max_blocks <= 0 || window < 0) return ATOM_BAD_SHAPE;
  if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (cu_q == nullptr || positions == nullptr || block_tables == nullptr) return ATOM_BAD_SHAPE;
  const bool mixes = talk != nullptr;
  if (!together_tile_takes(H, G, D, DV, page_size, mixes)) return ATOM_UNSUPPORTED;
  if (parts < 1 || parts > 65535 || (parts > 1 && (ws_ml == nullptr || ws_o == nullptr))) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  const int HB = mixes ? H : H / G;
  TogetherTileArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, cu_q, positions,
                     block_tables, max_blocks, num_seqs, H, G, page_size, window, scale * 1.4426950408889634f,
                     head_scale, sink, talk, parts, ws_ml, ws_o};
  const dim3 grid(tokens / kTileRows + num_seqs + 1, mixes ? 1 : G, parts);
#define ATOM_TILE(DD, NN) return together_tile_launch<DD, NN>(a, grid, HB, stream)
  if (D == 64) {
    if (DV == 32) ATOM_TILE(64, 2);
    if (DV == 64) ATOM_TILE(64, 4);
    ATOM_TILE(64, 8);
  }
  if (DV == 32) ATOM_TILE(128, 2);
  if (DV == 64) ATOM_TILE(128, 4);
  ATOM_TILE(128, 8);
#undef ATOM_TILE
}
