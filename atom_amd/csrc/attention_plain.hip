// Attention without rotation whose values have a size of their own: from the float32 product [q | k | v] of a
// token (H query heads and G key heads of D entries, G value heads of DV entries),
//
//   with unit_norm, every q and k head is divided by its root mean square (eps under the root, no weight);
//   q is multiplied by the token's temperature 1 + coef * ln(floor((p + 1) / every) + 1) (coef 0: none);
//   q goes to q_out [T, H, DP]; k to the key pages [pages, G, page, DP]; v to the value pages [pages, G, DP, page].
//
// DP >= max(D, DV) is the head size of the pages and of the attention kernels that read them: entries beyond D of
// q are written as zeros, entries beyond D of the key pages and beyond DV of the value pages are never written and
// stay the zeros they were allocated as, so scores and weighted sums are those of the unpadded heads.
// A block per token, a wave per head in turn.
//
// mean_of_norms: out = (1 / n) sum_b x_b / rms(x_b) * w_b over n inputs of one width, the way side-by-side mixers
// are brought together.  embedding_positions: table[id] + rows[position] as float32.  unary_act: an activation
// applied entry by entry.  stream_add: a summand of any type into the float32 stream.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
qkv_plain_write_kernel(const float* __restrict__ proj, long ld, T* __restrict__ q_out, T* __restrict__ k_cache,
                       T* __restrict__ v_cache, const int* __restrict__ positions, const int* __restrict__ slots, int H,
                       int G, int D, int DV, int DP, int page_size, int unit_norm, float eps, float coef, int every) {
  const size_t t = blockIdx.x;
  const float* row = proj + t * ld;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, waves = blockDim.x / kWave;
  float temp = 1.f;
  if (coef != 0.f) temp = 1.f + coef * logf((float)((positions[t] + 1) / every) + 1.f);
  const int slot = slots != nullptr ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  for (int head = wave; head < H + G; head += waves) {
    const bool is_k = head >= H;
    const float* src = row + (size_t)head * D;
    float inv = 1.f;
    if (unit_norm) {
      float ss = 0.f;
      for (int i = lane; i < D; i += kWave) ss += src[i] * src[i];
      inv = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
    }
    if (!is_k) {
      T* dst = q_out + (t * H + head) * (size_t)DP;
      for (int i = lane; i < DP; i += kWave) dst[i] = from_f32<T>(i < D ? src[i] * inv * temp : 0.f);
    } else if (slot >= 0) {
      T* dst = k_cache + (((size_t)page * G + (head - H)) * page_size + off) * (size_t)DP;
      for (int i = lane; i < D; i += kWave) dst[i] = from_f32<T>(src[i] * inv);
    }
  }
  if (slot >= 0) {
    const float* vr = row + (size_t)(H + G) * D;
    #pragma unroll 4
    for (int e = threadIdx.x; e < G * DV; e += blockDim.x) {
      const int g = e / DV, i = e - g * DV;
      v_cache[(((size_t)page * G + g) * DP + i) * (size_t)page_size + off] = from_f32<T>(vr[e]);
    }
  }
}

ATOM_EXPORT int atom_qkv_plain_write(const float* proj, long ld, void* q_out, void* k_cache, void* v_cache, int dtype,
                                     const int* positions, const int* slots, int tokens, int H, int G, int D, int DV,
                                     int DP, int page_size, int unit_norm, float eps, float coef, int every,
                                     hipStream_t stream) {
  if (tokens < 0 || H <= 0 || G <= 0 || D <= 0 || DV <= 0 || DP < D || DP < DV || page_size <= 0) return ATOM_BAD_SHAPE;
  if (ld < (long)(H + G) * D + (long)G * DV) return ATOM_BAD_SHAPE;
  if (proj == nullptr || q_out == nullptr) return ATOM_BAD_SHAPE;
  if (slots != nullptr && (k_cache == nullptr || v_cache == nullptr)) return ATOM_BAD_SHAPE;
  if (coef != 0.f && (positions == nullptr || every <= 0)) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((qkv_plain_write_kernel<T>), dim3(tokens), dim3(256), 0, stream, proj, ld,
                                                 (T*)q_out, (T*)k_cache, (T*)v_cache, positions, slots, H, G, D, DV, DP,
                                                 page_size, unit_norm, eps, coef, every));
  return launch_status();
}

// The first dv of every head's dp entries, head after head: attention's output without its padding.
template <typename T>
__global__ void narrow_heads_kernel(const T* __restrict__ x, T* __restrict__ out, int dp, int dv, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t head = idx / dv;
  out[idx] = x[head * dp + (idx - head * dv)];
}

ATOM_EXPORT int atom_narrow_heads(const void* x, void* out, int dtype, long heads, int dp, int dv, hipStream_t stream) {
  if (heads < 0 || dv <= 0 || dp < dv || x == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)heads * dv;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((narrow_heads_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                 (const T*)x, (T*)out, dp, dv, total));
  return launch_status();
}

// ------------------------------------------------------------------ the mean of RMS-normed rows

struct NormedInputs {
  const void* x[4];
  const float* w[4];
};

template <typename T>
__global__ void __launch_bounds__(256)
mean_of_norms_kernel(NormedInputs in, int n, T* __restrict__ out, int width, float eps) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  float inv[4];
  for (int b = 0; b < n; ++b) {
    const T* row = (const T*)in.x[b] + t * width;
    float ss = 0.f;
    #pragma unroll 4
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float v = to_f32(row[i]);
      ss += v * v;
    }
    inv[b] = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  }
  const float share = 1.f / (float)n;
  #pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float sum = 0.f;
    for (int b = 0; b < n; ++b) sum += to_f32(((const T*)in.x[b])[t * width + i]) * inv[b] * in.w[b][i];
    out[t * width + i] = from_f32<T>(sum * share);
  }
}

// Rows of up to 512 groups of 16 bytes: every input's row stays in registers, all loads asked for before the first is
// used, one barrier pair for all the sums of squares.
template <typename T>
__global__ void __launch_bounds__(256)
mean_of_norms_vec_kernel(NormedInputs in, int n, T* __restrict__ out, int width, float eps) {
  constexpr int N = 16 / sizeof(T);
  union Pack { uint4 raw; T e[N]; };
  __shared__ float scratch[4][4];
  const size_t t = blockIdx.x;
  const int chunks = width / N;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  Pack x[4][2];
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int c = threadIdx.x + r * 256;
      x[b][r].raw = uint4{0u, 0u, 0u, 0u};
      if (b < n && c < chunks) x[b][r].raw = reinterpret_cast<const uint4*>((const T*)in.x[b] + t * width)[c];
    }
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int i = 0; i < N; ++i) ss += to_f32(x[b][r].e[i]) * to_f32(x[b][r].e[i]);
    ss = wave_sum(ss);
    if (lane == 0) scratch[b][wave] = ss;
  }
  __syncthreads();
  float inv[4];
#pragma unroll
  for (int b = 0; b < 4; ++b)
    inv[b] = 1.f / sqrtf((scratch[b][0] + scratch[b][1] + scratch[b][2] + scratch[b][3]) / (float)width + eps);
  const float share = 1.f / (float)n;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = threadIdx.x + r * 256;
    if (c < chunks) {
      float sum[N];
#pragma unroll
      for (int i = 0; i < N; ++i) sum[i] = 0.f;
#pragma unroll
      for (int b = 0; b < 4; ++b)
        if (b < n) {
#pragma unroll
          for (int q = 0; q < N / 4; ++q) {
            const float4 w4 = *reinterpret_cast<const float4*>(in.w[b] + (size_t)c * N + 4 * q);
            sum[4 * q] += to_f32(x[b][r].e[4 * q]) * inv[b] * w4.x;
            sum[4 * q + 1] += to_f32(x[b][r].e[4 * q + 1]) * inv[b] * w4.y;
            sum[4 * q + 2] += to_f32(x[b][r].e[4 * q + 2]) * inv[b] * w4.z;
            sum[4 * q + 3] += to_f32(x[b][r].e[4 * q + 3]) * inv[b] * w4.w;
          }
        }
      Pack res;
#pragma unroll
      for (int i = 0; i < N; ++i) res.e[i] = from_f32<T>(sum[i] * share);
      reinterpret_cast<uint4*>(out + t * width)[c] = res.raw;
    }
  }
}

ATOM_EXPORT int atom_mean_of_norms(const void* const* xs, const float* const* ws, int n, void* out, int dtype, int tokens,
                                   int width, float eps, hipStream_t stream) {
  if (n < 1 || n > 4 || tokens < 0 || width <= 0 || xs == nullptr || ws == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  NormedInputs in{};
  for (int b = 0; b < n; ++b) {
    if (xs[b] == nullptr || ws[b] == nullptr) return ATOM_BAD_SHAPE;
    in.x[b] = xs[b];
    in.w[b] = ws[b];
  }
  if (tokens == 0) return ATOM_OK;
  const int per = dtype == ATOM_F32 ? 4 : 8;
  bool vec = width % per == 0 && width / per <= 512 && (uintptr_t)out % 16 == 0;
  for (int b = 0; b < n; ++b) vec = vec && ((uintptr_t)xs[b] | (uintptr_t)ws[b]) % 16 == 0;
  if (vec) {
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((mean_of_norms_vec_kernel<T>), dim3(tokens), dim3(256), 0, stream, in, n,
                                                   (T*)out, width, eps));
    return launch_status();
  }
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((mean_of_norms_kernel<T>), dim3(tokens), dim3(256), 0, stream, in, n,
                                                 (T*)out, width, eps));
  return launch_status();
}

// ------------------------------------------------------------------ token rows plus learned position rows

template <typename T>
__global__ void __launch_bounds__(256)
embedding_positions_kernel(const T* __restrict__ table, const T* __restrict__ rows, const int* __restrict__ ids,
                           const int* __restrict__ positions, float* __restrict__ out, int width, int vocab,
                           int max_positions) {
  const size_t t = blockIdx.x;
  int id = ids[t], p = positions[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  p = p < 0 ? 0 : (p >= max_positions ? max_positions - 1 : p);
  const T* a = table + (size_t)id * width;
  const T* b = rows + (size_t)p * width;
  #pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[t * width + i] = to_f32(a[i]) + to_f32(b[i]);
}

ATOM_EXPORT int atom_embedding_positions(const void* table, const void* rows, int dtype, const int* ids,
                                         const int* positions, float* out, int tokens, int width, int vocab,
                                         int max_positions, hipStream_t stream) {
  if (tokens < 0 || width <= 0 || vocab <= 0 || max_positions <= 0) return ATOM_BAD_SHAPE;
  if (table == nullptr || rows == nullptr || ids == nullptr || positions == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((embedding_positions_kernel<T>), dim3(tokens), dim3(256), 0, stream,
                                                 (const T*)table, (const T*)rows, ids, positions, out, width, vocab,
                                                 max_positions));
  return launch_status();
}

// ------------------------------------------------------------------ an activation entry by entry

// act 0: SiLU, 1: ReLU, 2: tanh-GELU, 3: the square of ReLU, 4: tanh
__device__ __forceinline__ float unary_act_of(float z, int act) {
  if (act == 0) return z / (1.f + expf(-z));
  if (act == 1) return fmaxf(z, 0.f);
  if (act == 2) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (act == 3) {
    const float p = fmaxf(z, 0.f);
    return p * p;
  }
  return tanhf(z);
}

template <typename T>
__global__ void unary_act_kernel(const T* __restrict__ x, T* __restrict__ out, int act, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = from_f32<T>(unary_act_of(to_f32(x[idx]), act));
}

// 16 bytes a thread: `groups` groups of 16 / sizeof(T) entries, both pointers 16-byte aligned
template <typename T>
__global__ void unary_act_vec_kernel(const T* __restrict__ x, T* __restrict__ out, int act, size_t groups) {
  constexpr int N = 16 / sizeof(T);
  const size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= groups) return;
  union Pack { uint4 raw; T e[N]; } in, res;
  in.raw = reinterpret_cast<const uint4*>(x)[g];
#pragma unroll
  for (int i = 0; i < N; ++i) res.e[i] = from_f32<T>(unary_act_of(to_f32(in.e[i]), act));
  reinterpret_cast<uint4*>(out)[g] = res.raw;
}

ATOM_EXPORT int atom_unary_act(const void* x, void* out, int dtype, long total, int act, hipStream_t stream) {
  if (total < 0 || act < 0 || act > 4 || x == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (total == 0) return ATOM_OK;
  const int per = dtype == ATOM_F32 ? 4 : 8;
  const bool vec = total % per == 0 && ((uintptr_t)x | (uintptr_t)out) % 16 == 0;
  const size_t work = vec ? (size_t)total / per : (size_t)total;
  const size_t blocks = (work + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  if (vec) {
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((unary_act_vec_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                   (const T*)x, (T*)out, act, work));
  } else {
    ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((unary_act_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                   (const T*)x, (T*)out, act, (size_t)total));
  }
  return launch_status();
}

// ------------------------------------------------------------------ a summand into the float32 stream

template <typename T>
__global__ void stream_add_kernel(float* __restrict__ stream, const T* __restrict__ x, size_t total, int init) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const float v = to_f32(x[idx]);
  stream[idx] = init ? v : stream[idx] + v;
}

ATOM_EXPORT int atom_stream_add(float* stream_rows, const void* x, int dtype, long total, int init, hipStream_t stream) {
  if (total < 0 || stream_rows == nullptr || x == nullptr) return ATOM_BAD_SHAPE;
  if (total == 0) return ATOM_OK;
  const size_t blocks = ((size_t)total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((stream_add_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                                                 stream_rows, (const T*)x, (size_t)total, init));
  return launch_status();
}

__global__ void scale_rows_kernel(float* __restrict__ x, size_t total, float scale) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < total) x[idx] *= scale;
}

ATOM_EXPORT int atom_scale_rows(float* x, long total, float scale, hipStream_t stream) {
  if (total < 0 || x == nullptr) return ATOM_BAD_SHAPE;
  if (total == 0) return ATOM_OK;
  const size_t blocks = ((size_t)total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  hipLaunchKernelGGL(scale_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, (size_t)total, scale);
  return launch_status();
}
