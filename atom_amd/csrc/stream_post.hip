// Kernels around a float32 residual stream whose summands are normed on their way in, and the two token lookups
// that feed it.
//
//   rmsnorm_post      stream += x / rms(x) * w (float32, nothing rounded on the way), and optionally a copy of the
//                     stream's new rows in the step's type for the products that read them next
//   rmsnorm_rows      norm of chosen float32 rows, written in another type
//   cast_rows         float32 rows in another type
//   bias_rows         y[r, :] += bias for float32 rows
//   token_gate        gelu_tanh(a[t, j]) * table[id[t], col_off + j]
//   embedding_bigram  table[id] + pairs[(previous id * mul_prev + id * mul_cur) mod buckets], float32; a request's
//                     first token takes row `buckets`; the previous token of a request's next token is kept per
//                     state slot (last id + 1; 0: none yet)
#include "common.h"

__device__ __forceinline__ float gelu_tanh_f(float z) {
  const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.f + tanhf(inner));
}

template <typename TX, typename TO>
__global__ void __launch_bounds__(256)
rmsnorm_post_kernel(const TX* __restrict__ x, const float* __restrict__ weight, float eps, float* __restrict__ stream,
                    TO* __restrict__ out, int width) {
  extern __shared__ float smem[];
  float* vals = smem;
  float* scratch = smem + width;
  const size_t row = blockIdx.x;
  const TX* xr = x + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_f32(xr[i]);
    vals[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  float* sr = stream + row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float s = sr[i] + vals[i] * inv * weight[i];
    sr[i] = s;
    if (out != nullptr) out[row * width + i] = from_f32<TO>(s);
  }
}

// The same for widths that are a multiple of 4 and at most 4 * 256 * VPT: a thread keeps VPT groups of 4 consecutive
// elements in registers, every load of a row is issued before the sum of squares is formed (16-byte accesses of the
// stream and the weight, 8- or 16-byte ones of x), and nothing goes through LDS but the reduction.
template <typename T>
struct Quad;
template <>
struct Quad<float> {
  float4 v;
  __device__ __forceinline__ void get(float* f) const { f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w; }
  __device__ __forceinline__ void set(const float* f) { v = make_float4(f[0], f[1], f[2], f[3]); }
};
template <>
struct alignas(8) Quad<bf16_t> {
  bf16_t v[4];
  __device__ __forceinline__ void get(float* f) const {
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = static_cast<float>(v[e]);
  }
  __device__ __forceinline__ void set(const float* f) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = static_cast<bf16_t>(f[e]);
  }
};

template <typename TX, typename TO, int VPT>
__global__ void __launch_bounds__(256)
rmsnorm_post_vec_kernel(const TX* __restrict__ x, const float* __restrict__ weight, float eps, float* __restrict__ stream,
                        TO* __restrict__ out, int width) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const TX* xr = x + row * width;
  float* sr = stream + row * width;
  Quad<TX> xq[VPT];
  float4 sq[VPT], wq[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * 256) * 4;
    if (i < width) {
      xq[j] = *reinterpret_cast<const Quad<TX>*>(xr + i);
      sq[j] = *reinterpret_cast<const float4*>(sr + i);
      wq[j] = *reinterpret_cast<const float4*>(weight + i);
    }
  }
  float vals[VPT][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * 256) * 4;
    if (i < width) {
      xq[j].get(vals[j]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += vals[j][e] * vals[j][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int i = (threadIdx.x + j * 256) * 4;
    if (i < width) {
      float s4[4] = {sq[j].x, sq[j].y, sq[j].z, sq[j].w};
      const float w4[4] = {wq[j].x, wq[j].y, wq[j].z, wq[j].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) s4[e] += vals[j][e] * inv * w4[e];
      *reinterpret_cast<float4*>(sr + i) = make_float4(s4[0], s4[1], s4[2], s4[3]);
      if (out != nullptr) {
        Quad<TO> o;
        o.set(s4);
        *reinterpret_cast<Quad<TO>*>(out + row * width + i) = o;
      }
    }
  }
}

ATOM_EXPORT int atom_rmsnorm_post(const void* x, int x_dtype, const float* weight, float eps, float* stream, void* out,
                                  int out_dtype, int rows, int width, hipStream_t stream_handle) {
  if (rows < 0 || width <= 0 || x == nullptr || weight == nullptr || stream == nullptr) return ATOM_BAD_SHAPE;
  if (width > 32768) return ATOM_TOO_LARGE;
  if (rows == 0) return ATOM_OK;
  const size_t smem = (size_t)(width + 16) * sizeof(float);
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)stream % 16 == 0) && ((uintptr_t)weight % 16 == 0) &&
                       (out == nullptr || (uintptr_t)out % 16 == 0);
  const int vpt = (width % 4 == 0 && aligned) ? (width + 1023) / 1024 : 0;   // groups of 4 a thread; 0: the general kernel
#define LAUNCH(TX, TO)                                                                                               \
  do {                                                                                                               \
    if (vpt == 1)                                                                                                    \
      hipLaunchKernelGGL((rmsnorm_post_vec_kernel<TX, TO, 1>), dim3(rows), dim3(256), 0, stream_handle, (const TX*)x, \
                         weight, eps, stream, (TO*)out, width);                                                      \
    else if (vpt == 2)                                                                                               \
      hipLaunchKernelGGL((rmsnorm_post_vec_kernel<TX, TO, 2>), dim3(rows), dim3(256), 0, stream_handle, (const TX*)x, \
                         weight, eps, stream, (TO*)out, width);                                                      \
    else if (vpt >= 3 && vpt <= 4)                                                                                   \
      hipLaunchKernelGGL((rmsnorm_post_vec_kernel<TX, TO, 4>), dim3(rows), dim3(256), 0, stream_handle, (const TX*)x, \
                         weight, eps, stream, (TO*)out, width);                                                      \
    else if (vpt >= 5 && vpt <= 8)                                                                                   \
      hipLaunchKernelGGL((rmsnorm_post_vec_kernel<TX, TO, 8>), dim3(rows), dim3(256), 0, stream_handle, (const TX*)x, \
                         weight, eps, stream, (TO*)out, width);                                                      \
    else                                                                                                             \
      hipLaunchKernelGGL((rmsnorm_post_kernel<TX, TO>), dim3(rows), dim3(256), smem, stream_handle, (const TX*)x,    \
                         weight, eps, stream, (TO*)out, width);                                                      \
  } while (0)
  const bool out_bf16 = out != nullptr && out_dtype == ATOM_BF16;
  if (out != nullptr && out_dtype != ATOM_BF16 && out_dtype != ATOM_F32) return ATOM_BAD_DTYPE;
  if (x_dtype == ATOM_F32) {
    if (out_bf16) LAUNCH(float, bf16_t); else LAUNCH(float, float);
  } else if (x_dtype == ATOM_BF16) {
    if (out_bf16) LAUNCH(bf16_t, bf16_t); else LAUNCH(bf16_t, float);
  } else {
    return ATOM_BAD_DTYPE;
  }
#undef LAUNCH
  return launch_status();
}

template <typename TO>
__global__ void __launch_bounds__(256)
rmsnorm_rows_kernel(const float* __restrict__ x, const float* __restrict__ weight, float eps,
                    const int* __restrict__ rows, int num_src, TO* __restrict__ out, int width) {
  extern __shared__ float smem[];
  float* vals = smem;
  float* scratch = smem + width;
  const int src = rows ? rows[blockIdx.x] : (int)blockIdx.x;
  TO* dst = out + (size_t)blockIdx.x * width;
  if (src < 0 || src >= num_src) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_f32<TO>(0.f);
    return;
  }
  const float* xr = x + (size_t)src * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = xr[i];
    vals[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_f32<TO>(vals[i] * inv * weight[i]);
}

ATOM_EXPORT int atom_rmsnorm_rows(const float* x, const float* weight, float eps, const int* rows, int num_src, void* out,
                                  int out_dtype, int num_rows, int width, hipStream_t stream) {
  if (num_rows < 0 || num_src < 0 || width <= 0 || x == nullptr || weight == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (width > 32768) return ATOM_TOO_LARGE;
  if (num_rows == 0) return ATOM_OK;
  const size_t smem = (size_t)(width + 16) * sizeof(float);
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((rmsnorm_rows_kernel<T>), dim3(num_rows), dim3(256), smem, stream,
                                                     x, weight, eps, rows, num_src, (T*)out, width));
  return launch_status();
}

// stream[r] = (init ? 0 : stream[r]) + x[r] for float32 rows, and out[r] = norm(stream[r]) * weight in out's type: a
// float32 summand (an embedding's output) starts the stream or joins it, and the stream is normed for the sublayer
// that reads it next.  A block a row, the row's sum kept in LDS between the two walks.
template <typename TO>
__global__ void __launch_bounds__(256)
stream_norm_kernel(float* __restrict__ stream, const float* __restrict__ x, const float* __restrict__ weight, float eps,
                   TO* __restrict__ out, int width, int init) {
  extern __shared__ float smem[];
  float* vals = smem;
  float* scratch = smem + width;
  const size_t r = blockIdx.x;
  float* sr = stream + r * width;
  const float* xr = x + r * width;
  float ss = 0.f;
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = init ? xr[i] : sr[i] + xr[i];
    sr[i] = v;
    vals[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[r * width + i] = from_f32<TO>(vals[i] * inv * weight[i]);
}

ATOM_EXPORT int atom_stream_norm(float* stream_rows, const float* x, const float* weight, float eps, void* out, int out_dtype,
                                 int num_rows, int width, int init, hipStream_t stream) {
  if (num_rows < 0 || width <= 0 || stream_rows == nullptr || x == nullptr || weight == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (width > 32768) return ATOM_TOO_LARGE;
  if (num_rows == 0) return ATOM_OK;
  const size_t smem = (size_t)(width + 16) * sizeof(float);
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((stream_norm_kernel<T>), dim3(num_rows), dim3(256), smem, stream,
                                                     stream_rows, x, weight, eps, (T*)out, width, init));
  return launch_status();
}

template <typename TO>
__global__ void cast_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<TO>(x[i]);
}

ATOM_EXPORT int atom_cast_rows(const float* x, void* out, int out_dtype, long n, hipStream_t stream) {
  if (n < 0 || x == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  if (n == 0) return ATOM_OK;
  const size_t blocks = ((size_t)n + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  ATOM_DISPATCH_DTYPE(out_dtype, hipLaunchKernelGGL((cast_rows_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream, x,
                                                     (T*)out, (size_t)n));
  return launch_status();
}

// y[r, :] += bias for float32 rows (the bias of a library product whose output stays float32); 16-byte accesses
// where the width allows them.
__global__ void bias_rows_kernel(float* __restrict__ y, const float* __restrict__ bias, int width, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < total) y[idx] += bias[idx % width];
}

__global__ void bias_rows_vec_kernel(float4* __restrict__ y, const float4* __restrict__ bias, int quads, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float4 v = y[idx];
  const float4 b = bias[idx % quads];
  v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
  y[idx] = v;
}

ATOM_EXPORT int atom_bias_rows(float* y, const float* bias, int rows, int width, hipStream_t stream) {
  if (rows < 0 || width <= 0 || y == nullptr || bias == nullptr) return ATOM_BAD_SHAPE;
  size_t total = (size_t)rows * width;
  if (total == 0) return ATOM_OK;
  const bool vec = width % 4 == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)bias % 16 == 0;
  if (vec) total /= 4;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
  if (vec)
    hipLaunchKernelGGL(bias_rows_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (float4*)y, (const float4*)bias,
                       width / 4, total);
  else
    hipLaunchKernelGGL(bias_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, y, bias, width, total);
  return launch_status();
}

template <typename TT, typename TO>
__global__ void token_gate_kernel(const float* __restrict__ raw, const TT* __restrict__ table, int ld_table, int col_off,
                                  const int* __restrict__ ids, int vocab, TO* __restrict__ out, int dim, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / dim;
  const int j = (int)(idx - t * dim);
  const int id = ids[t];
  const float e = (id >= 0 && id < vocab) ? to_f32(table[(size_t)id * ld_table + col_off + j]) : 0.f;
  out[idx] = from_f32<TO>(gelu_tanh_f(raw[idx]) * e);
}

ATOM_EXPORT int atom_token_gate(const float* raw, const void* table, int table_dtype, int ld_table, int col_off,
                                const int* ids, int vocab, void* out, int out_dtype, int tokens, int dim,
                                hipStream_t stream) {
  if (tokens < 0 || dim <= 0 || col_off < 0 || col_off + dim > ld_table || vocab <= 0) return ATOM_BAD_SHAPE;
  if (raw == nullptr || table == nullptr || ids == nullptr || out == nullptr) return ATOM_BAD_SHAPE;
  const size_t total = (size_t)tokens * dim;
  if (total == 0) return ATOM_OK;
  const size_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffu) return ATOM_TOO_LARGE;
#define LAUNCH(TT, TO)                                                                                              \
  hipLaunchKernelGGL((token_gate_kernel<TT, TO>), dim3((unsigned)blocks), dim3(256), 0, stream, raw, (const TT*)table, \
                     ld_table, col_off, ids, vocab, (TO*)out, dim, total)
  if (table_dtype == ATOM_F32 && out_dtype == ATOM_F32) LAUNCH(float, float);
  else if (table_dtype == ATOM_F32 && out_dtype == ATOM_BF16) LAUNCH(float, bf16_t);
  else if (table_dtype == ATOM_BF16 && out_dtype == ATOM_F32) LAUNCH(bf16_t, float);
  else if (table_dtype == ATOM_BF16 && out_dtype == ATOM_BF16) LAUNCH(bf16_t, bf16_t);
  else return ATOM_BAD_DTYPE;
#undef LAUNCH
  return launch_status();
}

// A block per token.  The block of a request's first token of the step alone touches the request's state: it reads
// the previous token from it and, once every thread has, writes the step's last token there.
template <typename T>
__global__ void __launch_bounds__(256)
embedding_bigram_kernel(const T* __restrict__ table, const T* __restrict__ pairs, const int* __restrict__ ids,
                        int* __restrict__ state, long state_stride, const int* __restrict__ cu_seqlens,
                        const int* __restrict__ slot_of_seq, const int* __restrict__ token_seq,
                        float* __restrict__ out, int hidden, int vocab, int buckets, long mul_prev, long mul_cur) {
  const int t = blockIdx.x;
  float* dst = out + (size_t)t * hidden;
  const int seq = token_seq[t];
  const int id = ids[t];
  const int slot = seq >= 0 ? slot_of_seq[seq] : -1;
  if (seq < 0 || slot < 0 || id < 0 || id >= vocab) {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = 0.f;
    return;
  }
  const int begin = cu_seqlens[seq];
  int prev;
  if (t == begin) {
    prev = state[(size_t)slot * state_stride] - 1;
    __syncthreads();
    if (threadIdx.x == 0) state[(size_t)slot * state_stride] = ids[cu_seqlens[seq + 1] - 1] + 1;
  } else {
    prev = ids[t - 1];
  }
  long row = buckets;
  if (prev >= 0) {
    row = ((long)prev * mul_prev + (long)id * mul_cur) % buckets;
    if (row < 0) row += buckets;
  }
  const T* a = table + (size_t)id * hidden;
  const T* b = pairs + (size_t)row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32(a[i]) + to_f32(b[i]);
}

ATOM_EXPORT int atom_embedding_bigram(const void* table, const void* pairs, int dtype, const int* ids, int* state,
                                      long state_stride, const int* cu_seqlens, const int* slot_of_seq,
                                      const int* token_seq, float* out, int tokens, int hidden, int vocab, int buckets,
                                      long mul_prev, long mul_cur, hipStream_t stream) {
  if (tokens < 0 || hidden <= 0 || vocab <= 0 || buckets <= 0 || state_stride < 1) return ATOM_BAD_SHAPE;
  if (table == nullptr || pairs == nullptr || ids == nullptr || state == nullptr || cu_seqlens == nullptr ||
      slot_of_seq == nullptr || token_seq == nullptr || out == nullptr)
    return ATOM_BAD_SHAPE;
  if (tokens == 0) return ATOM_OK;
  ATOM_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((embedding_bigram_kernel<T>), dim3(tokens), dim3(256), 0, stream,
                                                 (const T*)table, (const T*)pairs, ids, state, state_stride, cu_seqlens,
                                                 slot_of_seq, token_seq, out, hidden, vocab, buckets, mul_prev, mul_cur));
  return launch_status();
}
