// SwiGLU's elementwise half: y = T( T(silu(g)) * u ) with g = gu[:, :I], u = gu[:, I:],
// silu(g) = g / (1 + exp(-g)) evaluated in float
// (reference: engine/dryft_qwen3/model.py:44-46, kernels/silu_mul.py:23-32).
#include "common.h"

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ y, int inter, int64_t gu_stride) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float g = load_as_float(gu + row * gu_stride + i);
  const float u = load_as_float(gu + row * gu_stride + inter + i);
  const float s = rounded_as<T>(g / (1.f + expf(-g)));
  store_from_float(y + row * inter + i, s * u);
}

// Eight values per thread with 16-byte loads and stores, for widths and strides that are multiples of 8.
typedef __attribute__((ext_vector_type(4))) uint32_t au4;

__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ y,
                                                           int inter, int64_t gu_stride) {
  const int64_t row = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= inter) return;
  const au4 g4 = *(const au4*)(gu + row * gu_stride + i);
  const au4 u4 = *(const au4*)(gu + row * gu_stride + inter + i);
  au4 o4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float g0 = __uint_as_float(g4[j] << 16), g1 = __uint_as_float(g4[j] & 0xffff0000u);
    const float u0 = __uint_as_float(u4[j] << 16), u1 = __uint_as_float(u4[j] & 0xffff0000u);
    const float s0 = rounded_as<bf16_t>(g0 / (1.f + expf(-g0))), s1 = rounded_as<bf16_t>(g1 / (1.f + expf(-g1)));
    o4[j] = (uint32_t)float_to_bf16(s0 * u0).bits | ((uint32_t)float_to_bf16(s1 * u1).bits << 16);
  }
  *(au4*)(y + row * inter + i) = o4;
}

DRYFT_API int dryft_silu_mul(const void* gu, void* y, int n_rows, int inter, int64_t gu_stride, int is_f32,
                             hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!is_f32 && inter % 8 == 0 && gu_stride % 8 == 0 && (((uintptr_t)gu | (uintptr_t)y) & 15) == 0) {
    dim3 vgrid(n_rows, (inter / 8 + 255) / 256);
    hipLaunchKernelGGL(silu_mul_vec_kernel, vgrid, dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter, gu_stride);
    return DRYFT_LAUNCH_CHECK();
  }
  dim3 grid(n_rows, (inter + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)y, inter, gu_stride);
  else
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter,
                       gu_stride);
  return DRYFT_LAUNCH_CHECK();
}

// A gated linear unit with clamped halves: g = min(gu[:, :I], limit), u = clamp(gu[:, I:], -limit, limit),
// y = T( g * sigmoid(alpha * g) * (u + 1) ), evaluated in float and rounded once.
template <typename T>
__global__ void glu_clamped_kernel(const T* __restrict__ gu, T* __restrict__ y, int inter, int64_t gu_stride,
                                   float limit, float alpha) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const float g = fminf(load_as_float(gu + row * gu_stride + i), limit);
  const float u = fminf(fmaxf(load_as_float(gu + row * gu_stride + inter + i), -limit), limit);
  store_from_float(y + row * inter + i, g / (1.f + expf(-alpha * g)) * (u + 1.f));
}

// Eight values per thread with 16-byte loads and stores, for widths and strides that are multiples of 8.
__global__ __launch_bounds__(256) void glu_clamped_vec_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ y,
                                                              int inter, int64_t gu_stride, float limit, float alpha) {
  const int64_t row = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= inter) return;
  float g[8], u[8], o[8];
  load8_as_float(gu + row * gu_stride + i, g);
  load8_as_float(gu + row * gu_stride + inter + i, u);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float gj = fminf(g[j], limit), uj = fminf(fmaxf(u[j], -limit), limit);
    o[j] = gj / (1.f + expf(-alpha * gj)) * (uj + 1.f);
  }
  store8_from_float(y + row * inter + i, o);
}

DRYFT_API int dryft_glu_clamped(const void* gu, void* y, int n_rows, int inter, int64_t gu_stride, float limit,
                                float alpha, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (!is_f32 && inter % 8 == 0 && gu_stride % 8 == 0 && (((uintptr_t)gu | (uintptr_t)y) & 15) == 0) {
    dim3 vgrid(n_rows, (inter / 8 + 255) / 256);
    hipLaunchKernelGGL(glu_clamped_vec_kernel, vgrid, dim3(256), 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter,
                       gu_stride, limit, alpha);
    return DRYFT_LAUNCH_CHECK();
  }
  dim3 grid(n_rows, (inter + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(glu_clamped_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)y, inter,
                       gu_stride, limit, alpha);
  else
    hipLaunchKernelGGL(glu_clamped_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)y, inter,
                       gu_stride, limit, alpha);
  return DRYFT_LAUNCH_CHECK();
}

// An output gate: y = T( a * sigmoid(g) ), a and g rows of `width` values with strides of their own (either
// may be a run of columns of a wider tensor).
template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ a, int64_t a_stride, const T* __restrict__ g,
                                    int64_t g_stride, T* __restrict__ y, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  const float gate = 1.f / (1.f + expf(-load_as_float(g + row * g_stride + i)));
  store_from_float(y + row * width + i, load_as_float(a + row * a_stride + i) * gate);
}

DRYFT_API int dryft_sigmoid_gate(const void* a, int64_t a_stride, const void* g, int64_t g_stride, void* y,
                                 int n_rows, int width, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  dim3 grid(n_rows, (width + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, block, 0, stream, (const float*)a, a_stride,
                       (const float*)g, g_stride, (float*)y, width);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)a, a_stride,
                       (const bf16_t*)g, g_stride, (bf16_t*)y, width);
  return DRYFT_LAUNCH_CHECK();
}

// The square of relu: y = T( max(x, 0)^2 ), rows of `width` values; x may be a run of columns of a wider tensor.
template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ y, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  const float r = fmaxf(load_as_float(x + row * x_stride + i), 0.f);
  store_from_float(y + row * width + i, r * r);
}

DRYFT_API int dryft_relu_squared(const void* x, int64_t x_stride, void* y, int n_rows, int width, int is_f32,
                                 hipStream_t stream) {
  if (n_rows <= 0) return 0;
  dim3 grid(n_rows, (width + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(relu_squared_kernel<float>, grid, block, 0, stream, (const float*)x, x_stride, (float*)y, width);
  else
    hipLaunchKernelGGL(relu_squared_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, x_stride, (bf16_t*)y, width);
  return DRYFT_LAUNCH_CHECK();
}

// A gate on what a token id brings: y[r, i] = T( gelu_tanh(g[r, i]) * table[token[r], col + i] ), with
// gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); the table's row is as wide as the caller says.
template <typename T>
__global__ void token_gate_kernel(const T* __restrict__ g, int64_t g_stride, const int* __restrict__ tokens,
                                  const T* __restrict__ table, int64_t table_stride, int col, int vocab,
                                  T* __restrict__ y, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  const int tok = min(max(tokens[row], 0), vocab - 1);
  const float z = load_as_float(g + row * g_stride + i);
  const float act = 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  store_from_float(y + row * width + i, act * load_as_float(table + (int64_t)tok * table_stride + col + i));
}

DRYFT_API int dryft_token_gate(const void* g, int64_t g_stride, const int* tokens, const void* table,
                               int64_t table_stride, int col, int vocab, void* y, int n_rows, int width, int is_f32,
                               hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (vocab <= 0 || col < 0 || col + width > table_stride) return -1;
  dim3 grid(n_rows, (width + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(token_gate_kernel<float>, grid, block, 0, stream, (const float*)g, g_stride, tokens,
                       (const float*)table, table_stride, col, vocab, (float*)y, width);
  else
    hipLaunchKernelGGL(token_gate_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)g, g_stride, tokens,
                       (const bf16_t*)table, table_stride, col, vocab, (bf16_t*)y, width);
  return DRYFT_LAUNCH_CHECK();
}

// A blend of two runs of columns, in place: a[r, i] = T( (1 - lam) a[r, i] + lam b[r, i] ), lam one float on the
// device. Float arithmetic, rounded once.
template <typename T>
__global__ void blend_columns_kernel(T* __restrict__ a, int64_t a_stride, const T* __restrict__ b, int64_t b_stride,
                                     const float* __restrict__ lam, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  const float l = *lam;
  T* p = a + row * a_stride + i;
  store_from_float(p, (1.f - l) * load_as_float(p) + l * load_as_float(b + row * b_stride + i));
}

DRYFT_API int dryft_blend_columns(void* a, int64_t a_stride, const void* b, int64_t b_stride, const float* lam,
                                  int n_rows, int width, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  dim3 grid(n_rows, (width + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(blend_columns_kernel<float>, grid, block, 0, stream, (float*)a, a_stride, (const float*)b,
                       b_stride, lam, width);
  else
    hipLaunchKernelGGL(blend_columns_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)a, a_stride, (const bf16_t*)b,
                       b_stride, lam, width);
  return DRYFT_LAUNCH_CHECK();
}
