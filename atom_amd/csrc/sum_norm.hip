// Kernels around a float32 residual stream that is normed after every sum, and the step between a packed q | k | v
// product and attention over pages whose value heads have a size of their own.
//
//   sum_norm        stream <- rms_norm(alpha * stream + sum_i scale_i * y_i) * w   (w null: the sum alone; alpha 0:
//                   the stream is not read), up to four summands of float32 or bfloat16, all in float32; the new
//                   rows optionally also in another type for the products that read them next
//   shift_rows      out[t] = x[t] + (x[t - 1] - x[t]) * mu; the row before a request's first token of the step is what
//                   its state slot holds (float32), and the request's last row of the step is left there
//   qkv_rot_write   per token: RMS norm of every q and k head with a weight per entry (no weight: no norm), rotation
//                   of the pairs (i, i + rot_dims / 2) of every head by position * freq[i] (float64 angle, reduced,
//                   float32 sine and cosine), values optionally kept as they are (float32) and optionally blended
//                   with another layer's, v <- (1 - l) v + l v_source; q goes to q_out [T, H, D], k to the key pages
//                   [pages, G, page, D], v to the value pages [pages, G, DV, page]
#include "common.h"

struct SumTerms {
  const void* y[4];
  int dtype[4];
  float scale[4];
  int n;
};

__device__ __forceinline__ float term_at(const void* y, int dtype, size_t at) {
  return dtype == ATOM_F32 ? static_cast<const float*>(y)[at] : to_f32(static_cast<const bf16_t*>(y)[at]);
}

template <typename T>
__global__ void __launch_bounds__(256)
sum_norm_kernel(float* __restrict__ stream, float alpha, SumTerms terms, const float* __restrict__ weight, float eps,
                T* __restrict__ out, int width) {
  extern __shared__ float row[];
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  float ss = 0.f;
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = alpha != 0.f ? alpha * stream[base + i] : 0.f;
    // the terms by constant index, so that the argument's arrays stay in scalar registers
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (k < terms.n) v += terms.scale[k] * term_at(terms.y[k], terms.dtype[k], base + i);
    row[i] = v;
    ss += v * v;
  }
  float inv = 1.f;
  if (weight != nullptr) inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {   // a thread reads back what it wrote itself
    const float v = weight != nullptr ? row[i] * inv * weight[i] : row[i];
    stream[base + i] = v;
    if (out != nullptr) out[base + i] = from_f32<T>(v);
  }
}

ATOM_EXPORT int atom_sum_norm(float* stream, float alpha, const void* y0, int d0, float s0, const void* y1, int d1,
                              float s1, const void* y2, int d2, float s2, const void* y3, int d3, float s3, int n,
                              const float* weight, float eps, void* out, int out_dtype, int rows, int width,
                              hipStream_t stream_id) {
  if (rows < 0 || width <= 0 || n < 0 || n > 4 || stream == nullptr) return ATOM_BAD_SHAPE;
  if (width > 15360) return ATOM_TOO_LARGE;
  SumTerms terms{{y0, y1, y2, y3}, {d0, d1, d2, d3}, {s0, s1, s2, s3}, n};
  for (int i = 0; i < n; ++i) {
    if (terms.y[i] == nullptr) return ATOM_BAD_SHAPE;
    if (terms.dtype[i] != ATOM_F32 && terms.dtype[i] != ATOM_BF16) return ATOM_BAD_DTYPE;
  }
  if (rows == 0) return ATOM_OK;
  const size_t smem = (size_t)width * sizeof(float);
  if (out == nullptr) out_dtype = ATOM_F32;
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((sum_norm_kernel<T>), dim3(rows), dim3(256), smem, stream_id, stream,
                                                     alpha, terms, weight, eps, (T*)out, width));
  return launch_status();
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
shift_rows_kernel(const TI* __restrict__ x, const float* __restrict__ mu, TO* __restrict__ out, float* __restrict__ state,
                  long slot_stride, long state_off, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_of_seq,
                  const int* __restrict__ token_seq, int width) {
  const int t = blockIdx.x;
  const int seq = token_seq[t];
  const bool padding = seq < 0;
  const int first = padding ? t : cu_seqlens[seq];
  const int slot = padding ? -1 : slot_of_seq[seq];
  const bool heads = t == first;             // the request's first token of this step
  const int last = padding ? t : cu_seqlens[seq + 1] - 1;
  float* kept = slot >= 0 ? state + (size_t)slot * slot_stride + state_off : nullptr;
  const TI* row = x + (size_t)t * width;
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float cur = to_f32(row[i]);
    float prev;
    if (heads) {
      // only this block touches the slot's row in this launch: it reads the old row and leaves the step's last
      prev = kept != nullptr ? kept[i] : 0.f;
      if (kept != nullptr) kept[i] = to_f32(x[(size_t)last * width + i]);
    } else {
      prev = to_f32(x[(size_t)(t - 1) * width + i]);
    }
    out[(size_t)t * width + i] = from_f32<TO>(cur + (prev - cur) * mu[i]);
  }
}

ATOM_EXPORT int atom_shift_rows(const void* x, int x_dtype, const float* mu, void* out, int out_dtype, float* state,
                                long slot_stride, long state_off, const int* cu_seqlens, const int* slot_of_seq,
                                const int* token_seq, int tokens, int width, hipStream_t stream) {
  if (tokens < 0 || width <= 0 || state_off < 0 || slot_stride < state_off + width) return ATOM_BAD_SHAPE;
  if (x == nullptr || mu == nullptr || out == nullptr || state == nullptr) return ATOM_BAD_SHAPE;
  if (cu_seqlens == nullptr || slot_of_seq == nullptr || token_seq == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
#define ATOM_SHIFT(TI, TO)                                                                                          \
  hipLaunchKernelGGL((shift_rows_kernel<TI, TO>), dim3(tokens), dim3(256), 0, stream, (const TI*)x, mu, (TO*)out,   \
                     state, slot_stride, state_off, cu_seqlens, slot_of_seq, token_seq, width)
  if (x_dtype == ATOM_F32 && out_dtype == ATOM_F32) ATOM_SHIFT(float, float);
  else if (x_dtype == ATOM_F32 && out_dtype == ATOM_BF16) ATOM_SHIFT(float, bf16_t);
  else if (x_dtype == ATOM_BF16 && out_dtype == ATOM_BF16) ATOM_SHIFT(bf16_t, bf16_t);
  else if (x_dtype == ATOM_BF16 && out_dtype == ATOM_F32) ATOM_SHIFT(bf16_t, float);
  else return ATOM_BAD_DTYPE;
#undef ATOM_SHIFT
  return launch_status();
}

__device__ __forceinline__ void half_turn_angle(int position, double freq, float* c, float* s) {
  double a = (double)position * freq;
  const double two_pi = 6.283185307179586476925286766559;
  a -= two_pi * floor(a / two_pi);
  sincosf((float)a, s, c);
}

template <typename T>
__global__ void __launch_bounds__(256)
qkv_rot_write_kernel(const float* __restrict__ qkv, int ld, T* __restrict__ q_out, T* __restrict__ k_cache,
                     T* __restrict__ v_cache, const float* __restrict__ qw, const float* __restrict__ kw,
                     const double* __restrict__ freq, int rot_dims, const int* __restrict__ positions,
                     const int* __restrict__ slots, int H, int G, int D, int DV, int page_size, float eps,
                     const float* __restrict__ v_source, const float* __restrict__ v_blend, float* __restrict__ v_keep) {
  extern __shared__ float lds[];
  const int half = rot_dims / 2;
  float* turn = lds;                 // cosines of the token's angles, then their sines
  float* inv = lds + 2 * half;       // 1 / rms of every q head, then of every k head
  const int t = blockIdx.x;
  const int Q = H * D, K = G * D, V = G * DV;
  const float* qr = qkv + (size_t)t * ld;
  const float* kr = qr + Q;
  const float* vr = kr + K;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave, waves = blockDim.x / kWave;
  for (int head = wave; head < H + G; head += waves) {
    const bool is_k = head >= H;
    const float* w = is_k ? kw : qw;
    float r = 1.f;
    if (w != nullptr) {
      const float* row = is_k ? kr + (size_t)(head - H) * D : qr + (size_t)head * D;
      float ss = 0.f;
      for (int i = lane; i < D; i += kWave) ss += row[i] * row[i];
      r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
    }
    if (lane == 0) inv[head] = r;
  }
  const int pos = rot_dims > 0 ? positions[t] : 0;
  for (int i = threadIdx.x; i < half; i += blockDim.x) half_turn_angle(pos, freq[i], &turn[i], &turn[half + i]);
  __syncthreads();
  const int slot = slots != nullptr ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
#pragma unroll 4
  for (int e = threadIdx.x; e < Q + K; e += blockDim.x) {
    const bool is_k = e >= Q;
    const int j = is_k ? e - Q : e;
    const float* row = is_k ? kr : qr;
    const float* w = is_k ? kw : qw;
    const int head = j / D, i = j - head * D;
    const float r = inv[is_k ? H + head : head];
    float v = row[j] * (w != nullptr ? r * w[i] : 1.f);
    if (i < rot_dims) {
      const bool upper = i >= half;
      const int pi = upper ? i - half : i + half;          // the other entry of the pair
      const float p = row[j - i + pi] * (w != nullptr ? r * w[pi] : 1.f);
      const int a = upper ? i - half : i;
      const float c = turn[a], s = turn[half + a];
      v = upper ? v * c + p * s : v * c - p * s;
    }
    if (!is_k) {
      q_out[(size_t)t * Q + j] = from_f32<T>(v);
    } else if (slot >= 0) {
      k_cache[(((size_t)page * G + head) * page_size + off) * D + i] = from_f32<T>(v);
    }
  }
  const float lam = (v_source != nullptr && v_blend != nullptr) ? v_blend[0] : 0.f;
#pragma unroll 4
  for (int j = threadIdx.x; j < V; j += blockDim.x) {
    float v = vr[j];
    if (v_keep != nullptr) v_keep[(size_t)t * V + j] = v;
    if (v_source != nullptr) v = (1.f - lam) * v + lam * v_source[(size_t)t * V + j];
    if (slot >= 0) {
      const int head = j / DV, i = j - head * DV;
      v_cache[(((size_t)page * G + head) * DV + i) * page_size + off] = from_f32<T>(v);
    }
  }
}

ATOM_EXPORT int atom_qkv_rot_write(const float* qkv, int ld, void* q_out, void* k_cache, void* v_cache, int dtype,
                                   const float* qw, const float* kw, const double* freq, int rot_dims,
                                   const int* positions, const int* slots, int tokens, int H, int G, int D, int DV,
                                   int page_size, float eps, const float* v_source, const float* v_blend, float* v_keep,
                                   hipStream_t stream) {
  if (tokens < 0 || H <= 0 || G <= 0 || D <= 0 || DV <= 0 || page_size <= 0 || ld < (H + G) * D + G * DV) return ATOM_BAD_SHAPE;
  if (rot_dims < 0 || rot_dims > D || (rot_dims & 1)) return ATOM_BAD_SHAPE;
  if (rot_dims > 0 && (freq == nullptr || positions == nullptr)) return ATOM_BAD_SHAPE;
  if (qkv == nullptr || q_out == nullptr) return ATOM_BAD_SHAPE;
  if (slots != nullptr && (k_cache == nullptr || v_cache == nullptr)) return ATOM_BAD_SHAPE;
  if (v_source != nullptr && v_blend == nullptr) return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  const size_t smem = (size_t)(rot_dims + H + G) * sizeof(float);
  if (smem > 48 * 1024) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((qkv_rot_write_kernel<T>), dim3(tokens), dim3(256), smem, stream, qkv, ld,
                                                 (T*)q_out, (T*)k_cache, (T*)v_cache, qw, kw, freq, rot_dims, positions,
                                                 slots, H, G, D, DV, page_size, eps, v_source, v_blend, v_keep));
  return launch_status();
}
