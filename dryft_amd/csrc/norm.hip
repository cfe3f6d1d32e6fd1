// RMSNorm and residual-add + RMSNorm over rows of any width.
//
//   res_new = T(res + sum_p delta[p])          (the sum in float, rounded once)
//   y       = T( T(res_new * rsqrt(mean(res_new^2) + eps)) * w )
//
// Statistics are float; the normalised value is rounded to the activation
// dtype before the weight multiply, as the reference does
// (engine/dryft_qwen3/model.py:28-32, kernels/rmsnorm.py:21-39). With T = float
// every rounding is the identity. `delta` may be given as several float
// partial sums (the split-K outputs of a matrix product), which are added here
// instead of in a pass of their own.
#include "common.h"

template <typename T, typename D>
__global__ void add_rmsnorm_kernel(const T* __restrict__ res, const D* __restrict__ delta, int n_partials,
                                   int64_t partial_stride, const void* __restrict__ w, int w_f32,
                                   T* __restrict__ res_out, T* __restrict__ y, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* r_in = res + row * width;
  T* r_out = res_out + row * width;
  T* y_row = y + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = load_as_float(r_in + i);
    if (n_partials > 0) {
      float d = 0.f;
      for (int p = 0; p < n_partials; ++p) d += load_as_float(delta + p * partial_stride + row * width + i);
      v = rounded_as<T>(v + d);
      store_from_float(r_out + i, v);
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
  const T* r_back = n_partials > 0 ? r_out : r_in;   // each thread re-reads what it wrote itself
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = load_as_float(r_back + i);
    const float n = rounded_as<T>(v * inv);
    store_from_float(y_row + i, n * load_vector(w, i, w_f32));
  }
}

// The same for rows whose width is a multiple of 8 and at most 8 * 8 * blockDim: a thread owns runs of 8
// contiguous values, reads them with 16-byte loads issued together, and keeps them in registers between the
// two passes. This is the kernel that decoding steps use: few rows, so latency rather than bandwidth counts: the
// weights are asked for together with the row, so that nothing has to come from memory after the reduction.
#define NORM_VEC_RUNS 8   // runs of 8 values a thread may hold

template <typename T, typename D, int RUNS>
__global__ __launch_bounds__(512) void add_rmsnorm_vec_kernel(const T* __restrict__ res, const D* __restrict__ delta,
                                                              int n_partials, int64_t partial_stride,
                                                              const void* __restrict__ w, int w_f32,
                                                              T* __restrict__ res_out, T* __restrict__ y, int width,
                                                              float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int64_t base = row * width;
  float v[RUNS][8], wv[RUNS][8];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int i = (r * blockDim.x + threadIdx.x) * 8;
    if (i < width) {
      load8_as_float(res + base + i, v[r]);
      if (w_f32) load8_as_float((const float*)w + i, wv[r]);
      else load8_as_float((const bf16_t*)w + i, wv[r]);
      if (n_partials > 0) {
        float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        int p = 0;
        for (; p + 4 <= n_partials; p += 4) {             // four loads in flight; added in the order 0, 1, ...
          float t[4][8];
#pragma unroll
          for (int u = 0; u < 4; ++u) load8_as_float(delta + (p + u) * partial_stride + base + i, t[u]);
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < 8; ++j) d[j] += t[u][j];
        }
        for (; p < n_partials; ++p) {
          float t[8];
          load8_as_float(delta + p * partial_stride + base + i, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) d[j] += t[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[r][j] = rounded_as<T>(v[r][j] + d[j]);
        store8_from_float(res_out + base + i, v[r]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[r][j] * v[r][j];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
#pragma unroll
  for (int r = 0; r < RUNS; ++r) {
    const int i = (r * blockDim.x + threadIdx.x) * 8;
    if (i < width) {
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = rounded_as<T>(v[r][j] * inv) * wv[r][j];
      store8_from_float(y + base + i, o);
    }
  }
}

template <typename T, typename D>
static void launch_norm_vec(const void* res, const void* delta, int n_partials, int64_t partial_stride, const void* w,
                            int w_f32, void* res_out, void* y, int n_rows, int width, float eps, hipStream_t stream) {
  const int runs_total = width / 8;
  int threads = 64;
  // few rows: latency counts, one run a thread; many rows: throughput counts, fuller threads in fewer waves
  const int per_thread = n_rows >= 256 ? 2 : 1;
  while (threads < 512 && per_thread * threads < runs_total) threads *= 2;
  const int runs = (runs_total + threads - 1) / threads;
  dim3 grid(n_rows), block(threads);
#define NV(R)                                                                                                        \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, D, R>), grid, block, 0, stream, (const T*)res, (const D*)delta,      \
                     n_partials, partial_stride, w, w_f32, (T*)res_out, (T*)y, width, eps)
  if (runs <= 1) NV(1);
  else if (runs <= 2) NV(2);
  else if (runs <= 4) NV(4);
  else NV(8);
#undef NV
}

// delta_kind: 0 = none (plain norm), 1 = same dtype as the activations, 2 = float partial sums
DRYFT_API int dryft_add_rmsnorm(const void* res, const void* delta, int delta_kind, int n_partials,
                                int64_t partial_stride, const void* w, int w_f32, void* res_out, void* y,
                                int n_rows, int width, float eps, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  const int threads = width >= 2048 ? 512 : 256;
  dim3 grid(n_rows), block(threads);
  if (delta_kind == 0) n_partials = 0;
  const bool aligned = (((uintptr_t)res | (uintptr_t)delta | (uintptr_t)res_out | (uintptr_t)y | (uintptr_t)w) & 15) == 0 &&
                       (partial_stride % 4) == 0;
  if (width % 8 == 0 && width <= 8 * NORM_VEC_RUNS * 512 && aligned) {
    if (is_f32)
      launch_norm_vec<float, float>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    else if (delta_kind == 2)
      launch_norm_vec<bf16_t, float>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    else
      launch_norm_vec<bf16_t, bf16_t>(res, delta, n_partials, partial_stride, w, w_f32, res_out, y, n_rows, width, eps, stream);
    return DRYFT_LAUNCH_CHECK();
  }
  if (is_f32) {
    hipLaunchKernelGGL((add_rmsnorm_kernel<float, float>), grid, block, 0, stream, (const float*)res,
                       (const float*)delta, n_partials, partial_stride, w, w_f32, (float*)res_out, (float*)y, width,
                       eps);
  } else if (delta_kind == 2) {
    hipLaunchKernelGGL((add_rmsnorm_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)res,
                       (const float*)delta, n_partials, partial_stride, w, w_f32, (bf16_t*)res_out, (bf16_t*)y,
                       width, eps);
  } else {
    hipLaunchKernelGGL((add_rmsnorm_kernel<bf16_t, bf16_t>), grid, block, 0, stream, (const bf16_t*)res,
                       (const bf16_t*)delta, n_partials, partial_stride, w, w_f32, (bf16_t*)res_out, (bf16_t*)y,
                       width, eps);
  }
  return DRYFT_LAUNCH_CHECK();
}

// res_out = T(res + delta): the last residual sum of a stack that is not followed by a norm.
template <typename T>
__global__ void add_rows_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) store_from_float(out + i, load_as_float(a + i) + load_as_float(b + i));
}

DRYFT_API int dryft_add_rows(const void* a, const void* b, void* out, int64_t n, int is_f32, hipStream_t stream) {
  if (n <= 0) return 0;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (is_f32)
    hipLaunchKernelGGL(add_rows_kernel<float>, grid, block, 0, stream, (const float*)a, (const float*)b, (float*)out, n);
  else
    hipLaunchKernelGGL(add_rows_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)a, (const bf16_t*)b,
                       (bf16_t*)out, n);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The norms of a float32 residual stream, for layers that norm a branch's output before it is added
// and norm the stream again for the next branch. One launch does, per row,
//
//   d      = sum_p delta[p]                                     (the branch's output; T, or float partial sums)
//   x_new  = x + d * rsqrt(mean(d^2) + eps) * wb + extra + vec   (each term optional; without wb, d is added as it is)
//   y      = T( x_new * rsqrt(mean(x_new^2) + eps) * w )         (optional)
//
// with x given as float32, in the activation dtype (the embedding's output, which starts a stream) or
// not at all, `extra` a row tensor in the activation dtype and `vec` one vector for every row. All of it
// is float arithmetic; only y is rounded, once. The row is held in LDS between the passes (dynamic
// shared memory of `width` floats), and a thread touches the same elements in every pass.
// `form` chooses other norms: bit 0, the branch's norm takes the mean off first (a layer norm without bias:
// (d - mean) * rsqrt(mean((d - mean)^2) + eps) * wb); bit 1, the same for y; bit 2, y is x_new itself, only rounded
// (a sublayer that reads the stream as it is).
template <typename T, typename D>
__global__ __launch_bounds__(256) void stream_norm_kernel(const void* __restrict__ x_in, int x_kind,
                                                          const D* __restrict__ delta, int n_partials,
                                                          int64_t partial_stride, const void* __restrict__ wb,
                                                          int wb_f32, const T* __restrict__ extra,
                                                          const void* __restrict__ vec, int vec_f32,
                                                          const void* __restrict__ w, int w_f32,
                                                          float* __restrict__ x_out, T* __restrict__ y, int width,
                                                          float eps, int form) {
  extern __shared__ __attribute__((aligned(16))) float held[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  float inv_d = 1.f, mean_d = 0.f;
  if (n_partials > 0) {
    float ss = 0.f, sd = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      float d = 0.f;
      for (int p = 0; p < n_partials; ++p) d += load_as_float(delta + p * partial_stride + base + i);
      held[i] = d;
      ss += d * d;
      sd += d;
    }
    if (wb != nullptr) {
      if (form & 1) {
        mean_d = block_sum(sd, scratch) / (float)width;
        ss = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) { const float t = held[i] - mean_d; ss += t * t; }
      }
      inv_d = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
    }
  }
  float ss = 0.f, sv = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = 0.f;
    if (x_kind == 2) v = ((const float*)x_in)[base + i];
    else if (x_kind == 1) v = load_as_float((const T*)x_in + base + i);
    if (n_partials > 0) v += wb != nullptr ? (held[i] - mean_d) * inv_d * load_vector(wb, i, wb_f32) : held[i];
    if (extra != nullptr) v += load_as_float(extra + base + i);
    if (vec != nullptr) v += load_vector(vec, i, vec_f32);
    held[i] = v;
    if (x_out != nullptr) x_out[base + i] = v;
    ss += v * v;
    sv += v;
  }
  if (y == nullptr) return;
  if (form & 4) {
    for (int i = threadIdx.x; i < width; i += blockDim.x) store_from_float(y + base + i, held[i]);
    return;
  }
  float mean = 0.f;
  if (form & 2) {
    mean = block_sum(sv, scratch) / (float)width;
    ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) { const float t = held[i] - mean; ss += t * t; }
  }
  const float inv = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    store_from_float(y + base + i, (held[i] - mean) * inv * load_vector(w, i, w_f32));
}

// The same for rows whose width is a multiple of 8 with 16-byte aligned operands: a thread owns runs of 8
// contiguous values, moves them with 16-byte loads and stores, and asks for four partial sums at a time, so that a
// row of a decoding step (latency, not bandwidth) costs a few trips to memory instead of one per value and part.
template <typename T, typename D>
__global__ __launch_bounds__(256) void stream_norm_vec_kernel(const void* __restrict__ x_in, int x_kind,
                                                              const D* __restrict__ delta, int n_partials,
                                                              int64_t partial_stride, const void* __restrict__ wb,
                                                              int wb_f32, const T* __restrict__ extra,
                                                              const void* __restrict__ vec, int vec_f32,
                                                              const void* __restrict__ w, int w_f32,
                                                              float* __restrict__ x_out, T* __restrict__ y, int width,
                                                              float eps, int form) {
  extern __shared__ __attribute__((aligned(16))) float held[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  float inv_d = 1.f, mean_d = 0.f;
  if (n_partials > 0) {
    float ss = 0.f, sd = 0.f;
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
      float d[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      int p = 0;
      for (; p + 4 <= n_partials; p += 4) {               // four loads in flight; added in the order 0, 1, ...
        float t[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) load8_as_float(delta + (p + u) * partial_stride + base + i, t[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int j = 0; j < 8; ++j) d[j] += t[u][j];
      }
      for (; p < n_partials; ++p) {
        float t[8];
        load8_as_float(delta + p * partial_stride + base + i, t);
#pragma unroll
        for (int j = 0; j < 8; ++j) d[j] += t[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) { ss += d[j] * d[j]; sd += d[j]; }
      store8_from_float(held + i, d);
    }
    if (wb != nullptr) {
      if (form & 1) {
        mean_d = block_sum(sd, scratch) / (float)width;
        ss = 0.f;
        for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
          float d[8];
          load8_as_float(held + i, d);
#pragma unroll
          for (int j = 0; j < 8; ++j) ss += (d[j] - mean_d) * (d[j] - mean_d);
        }
      }
      inv_d = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
    }
  }
  float ss = 0.f, sv = 0.f;
  for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, t[8];
    if (x_kind == 2) load8_as_float((const float*)x_in + base + i, v);
    else if (x_kind == 1) load8_as_float((const T*)x_in + base + i, v);
    if (n_partials > 0) {
      load8_as_float(held + i, t);
      if (wb != nullptr) {
        float wv[8];
        if (wb_f32) load8_as_float((const float*)wb + i, wv); else load8_as_float((const bf16_t*)wb + i, wv);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += (t[j] - mean_d) * inv_d * wv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] += t[j];
      }
    }
    if (extra != nullptr) {
      load8_as_float(extra + base + i, t);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += t[j];
    }
    if (vec != nullptr) {
      if (vec_f32) load8_as_float((const float*)vec + i, t); else load8_as_float((const bf16_t*)vec + i, t);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += t[j];
    }
    store8_from_float(held + i, v);
    if (x_out != nullptr) store8_from_float(x_out + base + i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) { ss += v[j] * v[j]; sv += v[j]; }
  }
  if (y == nullptr) return;
  if (form & 4) {
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
      float v[8];
      load8_as_float(held + i, v);
      store8_from_float(y + base + i, v);
    }
    return;
  }
  float mean = 0.f;
  if (form & 2) {
    mean = block_sum(sv, scratch) / (float)width;
    ss = 0.f;
    for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
      float v[8];
      load8_as_float(held + i, v);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (v[j] - mean) * (v[j] - mean);
    }
  }
  const float inv = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x * 8; i < width; i += blockDim.x * 8) {
    float v[8], wv[8];
    load8_as_float(held + i, v);
    if (w_f32) load8_as_float((const float*)w + i, wv); else load8_as_float((const bf16_t*)w + i, wv);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (v[j] - mean) * inv * wv[j];
    store8_from_float(y + base + i, v);
  }
}

#define STREAM_NORM_MAX_WIDTH 16384   // 64 KiB of LDS a row

// x_kind: 0 = no stream yet, 1 = the stream in the activation dtype, 2 = float32.
// delta_kind: 0 = none, 1 = activation dtype, 2 = float partial sums.
DRYFT_API int dryft_stream_norm(const void* x_in, int x_kind, const void* delta, int delta_kind, int n_partials,
                                int64_t partial_stride, const void* wb, int wb_f32, const void* extra,
                                const void* vec, int vec_f32, const void* w, int w_f32, float* x_out, void* y,
                                int n_rows, int width, float eps, int is_f32, int form, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || width > STREAM_NORM_MAX_WIDTH || (y != nullptr && w == nullptr && !(form & 4))) return -1;
  if (delta_kind == 0) n_partials = 0;
  dim3 grid(n_rows), block(256);
  const size_t lds = (size_t)width * sizeof(float);
#define SN(TT, DD)                                                                                                   \
  hipLaunchKernelGGL((stream_norm_kernel<TT, DD>), grid, block, lds, stream, x_in, x_kind, (const DD*)delta,        \
                     n_partials, partial_stride, wb, wb_f32, (const TT*)extra, vec, vec_f32, w, w_f32, x_out,       \
                     (TT*)y, width, eps, form)
#define SNV(TT, DD)                                                                                                  \
  hipLaunchKernelGGL((stream_norm_vec_kernel<TT, DD>), grid, block, lds, stream, x_in, x_kind, (const DD*)delta,    \
                     n_partials, partial_stride, wb, wb_f32, (const TT*)extra, vec, vec_f32, w, w_f32, x_out,       \
                     (TT*)y, width, eps, form)
  const bool aligned = (((uintptr_t)x_in | (uintptr_t)delta | (uintptr_t)wb | (uintptr_t)extra | (uintptr_t)vec |
                         (uintptr_t)w | (uintptr_t)x_out | (uintptr_t)y) & 15) == 0 && partial_stride % 4 == 0;
  if (width % 8 == 0 && aligned) {
    if (is_f32) SNV(float, float);
    else if (delta_kind == 2) SNV(bf16_t, float);
    else SNV(bf16_t, bf16_t);
    return DRYFT_LAUNCH_CHECK();
  }
#undef SNV
  if (is_f32) SN(float, float);
  else if (delta_kind == 2) SN(bf16_t, float);
  else SN(bf16_t, bf16_t);
#undef SN
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The mean of two branches that are each normed first: per row
//
//   a = sum_p A[p] (+ bias_a),  b = sum_p B[p] (+ bias_b)        (a branch's output: T, or float partial sums)
//   out = ( a * rsqrt(mean(a^2) + eps) * wa  +  b * rsqrt(mean(b^2) + eps) * wb ) / 2
//
// in float, stored as float32 (the consumer norms it once more before it enters the stream). Both rows wait in LDS
// (dynamic shared memory of 2 * width floats).
template <typename DA, typename DB>
__global__ __launch_bounds__(256) void rms_pair_mean_kernel(const DA* __restrict__ a, int a_parts, int64_t a_stride,
                                                            const float* __restrict__ a_bias, const float* __restrict__ wa,
                                                            const DB* __restrict__ b, int b_parts, int64_t b_stride,
                                                            const float* __restrict__ b_bias, const float* __restrict__ wb,
                                                            float* __restrict__ out, int width, float eps) {
  extern __shared__ __attribute__((aligned(16))) float held[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * width;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float x = a_bias ? a_bias[i] : 0.f, y = b_bias ? b_bias[i] : 0.f;
    for (int p = 0; p < a_parts; ++p) x += load_as_float(a + p * a_stride + base + i);
    for (int p = 0; p < b_parts; ++p) y += load_as_float(b + p * b_stride + base + i);
    held[i] = x;
    held[width + i] = y;
    sa += x * x;
    sb += y * y;
  }
  const float inv_a = rsqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float inv_b = rsqrtf(block_sum(sb, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    out[base + i] = 0.5f * (held[i] * inv_a * wa[i] + held[width + i] * inv_b * wb[i]);
}

// a_kind / b_kind: 1 = activation dtype [rows, width], 2 = float partial sums [parts, rows, width].
DRYFT_API int dryft_rms_pair_mean(const void* a, int a_kind, int a_parts, int64_t a_stride, const float* a_bias,
                                  const float* wa, const void* b, int b_kind, int b_parts, int64_t b_stride,
                                  const float* b_bias, const float* wb, float* out, int n_rows, int width, float eps,
                                  int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || 2 * width > STREAM_NORM_MAX_WIDTH || a_parts < 1 || b_parts < 1) return -1;
  dim3 grid(n_rows), block(256);
  const size_t lds = (size_t)2 * width * sizeof(float);
  const bool fa = is_f32 || a_kind == 2, fb = is_f32 || b_kind == 2;
#define PM(DA, DB)                                                                                                    \
  hipLaunchKernelGGL((rms_pair_mean_kernel<DA, DB>), grid, block, lds, stream, (const DA*)a, a_parts, a_stride, a_bias, \
                     wa, (const DB*)b, b_parts, b_stride, b_bias, wb, out, width, eps)
  if (fa && fb) PM(float, float);
  else if (fa) PM(float, bf16_t);
  else if (fb) PM(bf16_t, float);
  else PM(bf16_t, bf16_t);
#undef PM
  return DRYFT_LAUNCH_CHECK();
}
