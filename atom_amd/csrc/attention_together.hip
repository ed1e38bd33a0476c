// Paged softmax attention with the heads of a token worked through together: any head sizes (value heads may differ
// from key heads), float32 or bfloat16, every query token of a mixed batch.
//
//   score_h(j) = (q_h . k_g(j)) * scale * head_scale[h]          (head_scale null: 1)
//   w_h(j)     = exp(score_h(j) - m_h) / (sum_j' exp(score_h(j') - m_h) + exp(sink[h] - m_h))     (sink null: no such summand)
//   w'_h(j)    = sum_g talk[h, g] w_g(j)                          (talk null: w' = w)
//   out_h      = sum_j w'_h(j) v_{kv head of h}(j)
//
// A block owns one token and a set of heads: all of them when the heads' weights are mixed, else the query heads of
// one key/value head.  Mixing needs the finished weights of all heads at a key, so the keys are walked twice: first
// for every head's maximum and sum, then again for the weights themselves, their mixing and the weighted sum of the
// values.  Keys are taken 64 at a time in chunks counted from position 0, so a token's result depends on its own
// keys only: not on the batch, not on how a prompt was cut, not on which pages hold the keys.
//
// Few tokens with long contexts (decode steps) are cut over `parts` blocks a (token, head set): every part takes a run
// of whole chunks.  One launch leaves each part's maximum and sum, a second merges them (a few numbers), forms the
// weights of its own keys and leaves its share of the weighted sum, which a third adds up in the order of the parts.
//
// Pages: keys [pages, G, page, D]; values [pages, G, DV, page].
#include "common.h"

constexpr int kTogetherThreads = 256;
constexpr int kTogetherChunk = 64;     // keys a pass; a wave's width, so a head's chunk is reduced by one wave
constexpr int kTogetherAcc = 32;       // (head, value entry) pairs a thread may own

struct TogetherArgs {
  const int* token_seq; const int* positions; const int* block_tables; int max_blocks;
  int H, G, D, DV, page_size, window;
  float scale;
  const float* head_scale; const float* sink; const float* talk;
  int parts;          // > 1: the keys of a token are cut over this many blocks
  float* ws_ml;       // [tokens, H, parts, 2]: a part's maximum and sum
  float* ws_o;        // [tokens, parts, H, DV]: a part's share of the weighted sum
  float* ws_s;        // [tokens, H, s_stride] or null: the scores of the first launch, kept for the second
  long s_stride;      // at least the longest context
};

// The chunks [c0, c1) of a token's visible keys that part `part` takes, counted from the chunk that holds `first`.
__device__ __forceinline__ void together_part(int start, int pos, int parts, int part, int& base0, int& base1) {
  const int chunks = (pos - start) / kTogetherChunk + 1;
  const int each = (chunks + parts - 1) / parts;
  const int c0 = part * each, c1 = c0 + each < chunks ? c0 + each : chunks;
  base0 = start + c0 * kTogetherChunk;
  base1 = start + c1 * kTogetherChunk;     // exclusive; base0 >= base1: the part is empty
}

// q . k over D entries; 16 bytes of the key row a load where `wide` says the rows allow it
__device__ __forceinline__ float together_dot(const float* __restrict__ qr, const float* __restrict__ kr, int D, bool wide) {
  float d = 0.f;
  if (wide) {
    for (int i = 0; i < D; i += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(kr + i);
      d += qr[i] * k4.x + qr[i + 1] * k4.y + qr[i + 2] * k4.z + qr[i + 3] * k4.w;
    }
  } else {
    for (int i = 0; i < D; ++i) d += qr[i] * kr[i];
  }
  return d;
}

__device__ __forceinline__ float together_dot(const float* __restrict__ qr, const bf16_t* __restrict__ kr, int D, bool wide) {
  float d = 0.f;
  if (wide) {
    union Pack { uint4 raw; bf16_t e[8]; };
    for (int i = 0; i < D; i += 8) {
      Pack p;
      p.raw = *reinterpret_cast<const uint4*>(kr + i);
#pragma unroll
      for (int e = 0; e < 8; ++e) d += qr[i + e] * to_f32(p.e[e]);
    }
  } else {
    for (int i = 0; i < D; ++i) d += qr[i] * to_f32(kr[i]);
  }
  return d;
}

// scores of the block's heads against the keys lo .. hi of a chunk that starts at base, into s[hb][kTogetherChunk]
// (-inf outside lo .. hi)
template <typename T>
__device__ __forceinline__ void together_scores(const TogetherArgs& a, const T* __restrict__ k_cache, const int* table,
                                                const float* qs, float* s, int h0, int HB, int base, int lo, int hi) {
  const int group = a.H / a.G;
  for (int item = threadIdx.x; item < HB * kTogetherChunk; item += kTogetherThreads) {
    const int hh = item / kTogetherChunk, j = item - hh * kTogetherChunk;
    const int key = base + j;
    float v = -INFINITY;
    if (key >= lo && key <= hi) {
      const int h = h0 + hh;
      const int page = table[key / a.page_size], off = key % a.page_size;
      const T* kr = k_cache + (((size_t)page * a.G + h / group) * a.page_size + off) * (size_t)a.D;
      const float d = together_dot(qs + (size_t)hh * a.D, kr, a.D, a.D % (16 / (int)sizeof(T)) == 0);
      v = d * a.scale * (a.head_scale != nullptr ? a.head_scale[h] : 1.f);
    }
    s[item] = v;
  }
}

// sum over the keys lo .. hi of wr[key] * v(key) for one (value head, entry) whose row starts row_off elements into a
// page: the value pages hold a page's keys contiguously, 16 bytes of them a load where the run allows it.  pages[]
// holds the page of every page-sized run of the chunk, counted from the run that holds `base` (so that no look-up
// in the block table stands between a thread and its loads).
template <typename T>
__device__ __forceinline__ float together_values(const T* __restrict__ v_cache, size_t page_stride, size_t row_off,
                                                 const int* pages, const float* wr, int base, int lo, int hi,
                                                 int page_size, float sum) {
  const int run0 = base / page_size;
  for (int key = lo; key <= hi;) {
    const int page = pages[key / page_size - run0], off = key % page_size;
    int run = page_size - off;
    if (run > hi - key + 1) run = hi - key + 1;
    const T* vr = v_cache + (size_t)page * page_stride + row_off + off;
    int u = 0;
    if (sizeof(T) == 2 && page_size % 8 == 0) {
      union Pack { uint4 raw; bf16_t e[8]; };
      for (; u + 8 <= run && (off + u) % 8 == 0; u += 8) {
        Pack p;
        p.raw = *reinterpret_cast<const uint4*>(vr + u);
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += wr[key + u + e] * to_f32(p.e[e]);
      }
    }
    for (; u < run; ++u) sum += wr[key + u] * to_f32(vr[u]);
    key += run;
  }
  return sum;
}

template <typename T>
__global__ void __launch_bounds__(kTogetherThreads)
attention_together_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                          T* __restrict__ out, TogetherArgs a) {
  extern __shared__ float lds[];
  const int t = blockIdx.x;
  const int HB = a.talk != nullptr ? a.H : a.H / a.G;   // heads of this block
  const int h0 = a.talk != nullptr ? 0 : blockIdx.y * HB;
  float* qs = lds;                                  // HB * D
  float* s = qs + (size_t)HB * a.D;                 // HB * chunk: scores, then weights
  float* mixed = s + (size_t)HB * kTogetherChunk;   // HB * chunk: mixed weights (talk only)
  float* top = mixed + (a.talk != nullptr ? (size_t)HB * kTogetherChunk : 0);   // HB: running maximum
  float* den = top + HB;                            // HB: running sum, later its inverse
  int* pg = reinterpret_cast<int*>(den + HB);       // chunk: the pages of the chunk's runs of keys
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  constexpr int waves = kTogetherThreads / kWave;
  const int seq = a.token_seq[t];
  const int items = HB * a.DV;
  if (seq < 0) {   // padding row
    for (int e = tid; e < items; e += kTogetherThreads) out[((size_t)t * a.H + h0) * a.DV + e] = from_f32<T>(0.f);
    return;
  }
  const int pos = a.positions[t];
  const int* table = a.block_tables + (size_t)seq * a.max_blocks;
  for (int e = tid; e < HB * a.D; e += kTogetherThreads) qs[e] = to_f32(q[((size_t)t * a.H + h0) * a.D + e]);
  for (int e = tid; e < HB; e += kTogetherThreads) top[e] = -INFINITY, den[e] = 0.f;
  __syncthreads();
  const int first = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const int start = first / kTogetherChunk * kTogetherChunk;

  // every head's maximum and sum
  for (int base = start; base <= pos; base += kTogetherChunk) {
    const int lo = base > first ? base : first;
    const int hi = base + kTogetherChunk - 1 < pos ? base + kTogetherChunk - 1 : pos;
    together_scores(a, k_cache, table, qs, s, h0, HB, base, lo, hi);
    __syncthreads();
    for (int hh = wave; hh < HB; hh += waves) {     // a head is always the same wave's
      const float v = s[hh * kTogetherChunk + lane];
      const float m_old = top[hh];
      const float m_new = fmaxf(m_old, wave_max(v));   // finite: a chunk holds at least one visible key
      const float sum = wave_sum(expf(v - m_new));
      if (lane == 0) {
        den[hh] = den[hh] * (m_old == -INFINITY ? 0.f : expf(m_old - m_new)) + sum;
        top[hh] = m_new;
      }
    }
    __syncthreads();
  }
  for (int hh = tid; hh < HB; hh += kTogetherThreads) {
    float m = top[hh], l = den[hh];
    if (a.sink != nullptr) {
      const float sk = a.sink[h0 + hh];
      const float m_new = fmaxf(m, sk);
      l = l * expf(m - m_new) + expf(sk - m_new);
      m = m_new;
    }
    top[hh] = m;
    den[hh] = 1.f / l;
  }
  __syncthreads();

  // the weights, their mixing, the weighted sum of the values
  float acc[kTogetherAcc];
#pragma unroll
  for (int r = 0; r < kTogetherAcc; ++r) acc[r] = 0.f;
  const int group = a.H / a.G;
  for (int base = start; base <= pos; base += kTogetherChunk) {
    const int lo = base > first ? base : first;
    const int hi = base + kTogetherChunk - 1 < pos ? base + kTogetherChunk - 1 : pos;
    together_scores(a, k_cache, table, qs, s, h0, HB, base, lo, hi);
    for (int r = tid; r <= hi / a.page_size - base / a.page_size; r += kTogetherThreads) pg[r] = table[base / a.page_size + r];
    // a thread turns the scores it wrote itself into weights
    for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
      const int hh = item / kTogetherChunk;
      s[item] = expf(s[item] - top[hh]) * den[hh];    // exp(-inf) = 0 outside lo .. hi
    }
    __syncthreads();
    const float* w = s;
    if (a.talk != nullptr) {
      for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
        const int hh = item / kTogetherChunk, j = item - hh * kTogetherChunk;
        const float* row = a.talk + (size_t)hh * a.H;
        float m = 0.f;
        for (int g = 0; g < a.H; ++g) m += row[g] * s[g * kTogetherChunk + j];
        mixed[item] = m;
      }
      __syncthreads();
      w = mixed;
    }
#pragma unroll
    for (int r = 0; r < kTogetherAcc; ++r) {
      const int e = tid + r * kTogetherThreads;
      if (e < items) {
        const int hh = e / a.DV, i = e - hh * a.DV;
        const int kvh = (h0 + hh) / group;
        const float* wr = w + hh * kTogetherChunk - base;   // wr[key]
        acc[r] = together_values(v_cache, (size_t)a.G * a.DV * a.page_size, ((size_t)kvh * a.DV + i) * a.page_size, pg, wr,
                                 base, lo, hi, a.page_size, acc[r]);
      }
    }
    __syncthreads();   // s and mixed are rewritten by the next chunk
  }
#pragma unroll
  for (int r = 0; r < kTogetherAcc; ++r) {
    const int e = tid + r * kTogetherThreads;
    if (e < items) out[((size_t)t * a.H + h0) * a.DV + e] = from_f32<T>(acc[r]);
  }
}

// PASS 1: the maximum and sum of every head over this part's keys.  PASS 2: the parts' maxima and sums merged, then
// this part's weights, their mixing and its share of the weighted sum.
template <typename T, int PASS>
__global__ void __launch_bounds__(kTogetherThreads)
attention_together_part_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                               TogetherArgs a) {
  extern __shared__ float lds[];
  const int t = blockIdx.x, part = blockIdx.z;
  const int HB = a.talk != nullptr ? a.H : a.H / a.G;
  const int h0 = a.talk != nullptr ? 0 : blockIdx.y * HB;
  float* qs = lds;
  float* s = qs + (size_t)HB * a.D;
  float* mixed = s + (size_t)HB * kTogetherChunk;
  float* top = mixed + (a.talk != nullptr ? (size_t)HB * kTogetherChunk : 0);
  float* den = top + HB;
  int* pg = reinterpret_cast<int*>(den + HB);
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  constexpr int waves = kTogetherThreads / kWave;
  const int seq = a.token_seq[t];
  const int items = HB * a.DV;
  if (seq < 0) {   // padding row: no maximum, no sum, no share
    if (PASS == 1) {
      for (int hh = tid; hh < HB; hh += kTogetherThreads) {
        float* ml = a.ws_ml + (((size_t)t * a.H + h0 + hh) * a.parts + part) * 2;
        ml[0] = -INFINITY, ml[1] = 0.f;
      }
    } else {
      for (int e = tid; e < items; e += kTogetherThreads) a.ws_o[(((size_t)t * a.parts + part) * a.H + h0) * a.DV + e] = 0.f;
    }
    return;
  }
  const int pos = a.positions[t];
  const int* table = a.block_tables + (size_t)seq * a.max_blocks;
  for (int e = tid; e < HB * a.D; e += kTogetherThreads) qs[e] = to_f32(q[((size_t)t * a.H + h0) * a.D + e]);
  const int first = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
  const int start = first / kTogetherChunk * kTogetherChunk;
  int base0, base1;
  together_part(start, pos, a.parts, part, base0, base1);
  if (PASS == 1) {
    for (int e = tid; e < HB; e += kTogetherThreads) top[e] = -INFINITY, den[e] = 0.f;
    __syncthreads();
    for (int base = base0; base < base1; base += kTogetherChunk) {
      const int lo = base > first ? base : first;
      const int hi = base + kTogetherChunk - 1 < pos ? base + kTogetherChunk - 1 : pos;
      together_scores(a, k_cache, table, qs, s, h0, HB, base, lo, hi);
      if (a.ws_s != nullptr) {   // a thread keeps the scores it formed itself
        for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
          const int hh = item / kTogetherChunk, key = base + item - hh * kTogetherChunk;
          if (key >= lo && key <= hi) a.ws_s[((size_t)t * a.H + h0 + hh) * a.s_stride + key] = s[item];
        }
      }
      __syncthreads();
      for (int hh = wave; hh < HB; hh += waves) {
        const float v = s[hh * kTogetherChunk + lane];
        const float m_old = top[hh];
        const float m_new = fmaxf(m_old, wave_max(v));
        const float sum = wave_sum(expf(v - m_new));
        if (lane == 0) {
          den[hh] = den[hh] * (m_old == -INFINITY ? 0.f : expf(m_old - m_new)) + sum;
          top[hh] = m_new;
        }
      }
      __syncthreads();
    }
    for (int hh = tid; hh < HB; hh += kTogetherThreads) {
      float* ml = a.ws_ml + (((size_t)t * a.H + h0 + hh) * a.parts + part) * 2;
      ml[0] = top[hh], ml[1] = den[hh];
    }
    return;
  }
  // the parts' maxima and sums: a wave a head, a lane a part, so that the loads go out together
  for (int hh = wave; hh < HB; hh += waves) {
    const float* ml = a.ws_ml + ((size_t)t * a.H + h0 + hh) * a.parts * 2;
    float m = -INFINITY;
    for (int p = lane; p < a.parts; p += kWave) m = fmaxf(m, ml[2 * p]);
    m = wave_max(m);
    if (a.sink != nullptr) m = fmaxf(m, a.sink[h0 + hh]);
    float l = 0.f;
    for (int p = lane; p < a.parts; p += kWave) {
      const float mp = ml[2 * p];
      if (mp != -INFINITY) l += ml[2 * p + 1] * expf(mp - m);
    }
    l = wave_sum(l);
    if (a.sink != nullptr) l += expf(a.sink[h0 + hh] - m);
    if (lane == 0) top[hh] = m, den[hh] = 1.f / l;
  }
  __syncthreads();
  float acc[kTogetherAcc];
#pragma unroll
  for (int r = 0; r < kTogetherAcc; ++r) acc[r] = 0.f;
  const int group = a.H / a.G;
  for (int base = base0; base < base1; base += kTogetherChunk) {
    const int lo = base > first ? base : first;
    const int hi = base + kTogetherChunk - 1 < pos ? base + kTogetherChunk - 1 : pos;
    if (a.ws_s != nullptr) {
      for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
        const int hh = item / kTogetherChunk, key = base + item - hh * kTogetherChunk;
        s[item] = (key >= lo && key <= hi) ? a.ws_s[((size_t)t * a.H + h0 + hh) * a.s_stride + key] : -INFINITY;
      }
    } else {
      together_scores(a, k_cache, table, qs, s, h0, HB, base, lo, hi);
    }
    for (int r = tid; r <= hi / a.page_size - base / a.page_size; r += kTogetherThreads) pg[r] = table[base / a.page_size + r];
    for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
      const int hh = item / kTogetherChunk;
      s[item] = expf(s[item] - top[hh]) * den[hh];
    }
    __syncthreads();
    const float* w = s;
    if (a.talk != nullptr) {
      for (int item = tid; item < HB * kTogetherChunk; item += kTogetherThreads) {
        const int hh = item / kTogetherChunk, j = item - hh * kTogetherChunk;
        const float* row = a.talk + (size_t)hh * a.H;
        float m = 0.f;
        for (int g = 0; g < a.H; ++g) m += row[g] * s[g * kTogetherChunk + j];
        mixed[item] = m;
      }
      __syncthreads();
      w = mixed;
    }
#pragma unroll
    for (int r = 0; r < kTogetherAcc; ++r) {
      const int e = tid + r * kTogetherThreads;
      if (e < items) {
        const int hh = e / a.DV, i = e - hh * a.DV;
        const int kvh = (h0 + hh) / group;
        const float* wr = w + hh * kTogetherChunk - base;
        acc[r] = together_values(v_cache, (size_t)a.G * a.DV * a.page_size, ((size_t)kvh * a.DV + i) * a.page_size, pg, wr,
                                 base, lo, hi, a.page_size, acc[r]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < kTogetherAcc; ++r) {
    const int e = tid + r * kTogetherThreads;
    if (e < items) a.ws_o[(((size_t)t * a.parts + part) * a.H + h0) * a.DV + e] = acc[r];
  }
}

template <typename T>
__global__ void together_sum_parts_kernel(const float* __restrict__ ws_o, T* __restrict__ out, int parts, int row, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / row;
  const size_t e = idx - t * row;
  // the loads of four parts are asked for together; the shares are still added in the order of the parts
  const float* src = ws_o + t * parts * row + e;
  float sum = 0.f;
  int p = 0;
  for (; p + 4 <= parts; p += 4) {
    const float a = src[(size_t)p * row], b = src[(size_t)(p + 1) * row], c = src[(size_t)(p + 2) * row], d = src[(size_t)(p + 3) * row];
    sum = (((sum + a) + b) + c) + d;
  }
  for (; p < parts; ++p) sum += src[(size_t)p * row];
  out[idx] = from_f32<T>(sum);
}

ATOM_EXPORT int atom_together_sum_parts(const float* ws_o, void* out, int dtype, int parts, int tokens, int row,
                                        hipStream_t stream) {
  if (ws_o == nullptr || out == nullptr || parts < 1 || tokens < 0 || row <= 0) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)tokens * row;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((together_sum_parts_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                 ws_o, (T*)out, parts, row, total));
  return launch_status();
}

static size_t together_lds(int H, int G, int D, bool talk) {
  const int HB = talk ? H : H / G;
  return ((size_t)HB * D + (size_t)HB * kTogetherChunk * (talk ? 2 : 1) + 2 * (size_t)HB + kTogetherChunk) * sizeof(float);
}

ATOM_EXPORT int atom_attention_together(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                                        const int* token_seq, const int* positions, const int* block_tables,
                                        int max_blocks, int tokens, int H, int G, int D, int DV, int page_size,
                                        float scale, const float* head_scale, const float* sink, const float* talk,
                                        int window, int parts, float* ws_ml, float* ws_o, float* ws_s, long s_stride,
                                        hipStream_t stream) {
  if (tokens < 0 || H <= 0 || G <= 0 || D <= 0 || DV <= 0 || page_size <= 0 || max_blocks <= 0) return ATOM_BAD_SHAPE;
  if (H % G || window < 0) return ATOM_BAD_SHAPE;
  if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (token_seq == nullptr || positions == nullptr || block_tables == nullptr) return ATOM_BAD_SHAPE;
  const bool mixes = talk != nullptr;
  const int HB = mixes ? H : H / G;
  if ((size_t)HB * DV > (size_t)kTogetherAcc * kTogetherThreads) return ATOM_TOO_LARGE;
  const size_t smem = together_lds(H, G, D, mixes);
  if (smem > 64 * 1024) return ATOM_TOO_LARGE;
  if (tokens == 0) return ATOM_OK;
  if (parts < 1 || parts > 65535 || (parts > 1 && (ws_ml == nullptr || ws_o == nullptr))) return ATOM_BAD_SHAPE;
  TogetherArgs a{token_seq, positions, block_tables, max_blocks, H, G, D, DV, page_size, window, scale, head_scale, sink,
                 talk, parts, ws_ml, ws_o, parts > 1 ? ws_s : nullptr, s_stride};
  if (a.ws_s != nullptr && s_stride < (long)max_blocks * page_size) return ATOM_BAD_SHAPE;
  dim3 grid(tokens, mixes ? 1 : G, parts), block(kTogetherThreads);
  if (parts == 1) {
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((attention_together_kernel<T>), grid, block, smem, stream, (const T*)q,
                                                   (const T*)k_cache, (const T*)v_cache, (T*)out, a));
    return launch_status();
  }
  const size_t total = (size_t)tokens * H * DV;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((attention_together_part_kernel<T, 1>), grid, block, smem, stream, (const T*)q, (const T*)k_cache,
                       (const T*)v_cache, a);
    hipLaunchKernelGGL((attention_together_part_kernel<T, 2>), grid, block, smem, stream, (const T*)q, (const T*)k_cache,
                       (const T*)v_cache, a);
    hipLaunchKernelGGL((together_sum_parts_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, ws_o, (T*)out, parts,
                       H * DV, total);
  });
  return launch_status();
}
