// A state-space mixer with one scalar decay per head and token (the Mamba-2 recurrence), and its read-out.
//
//   dt_t = softplus(dt_raw_t + dt_bias_h)         a_t = exp(-exp(A_log_h) * dt_t)
//   S_t  = a_t S_(t-1) + dt_t B_t x_t^T           (S is N x P per head; B and C belong to the head's group)
//   y_t  = S_t^T C_t + D_h x_t
//
// The state is float32 in the state store and everything above is float arithmetic; x, B and C arrive in the
// activation dtype (the output of the short convolution). A workgroup owns one (sequence, head, run of up to PT
// value columns) and walks the sequence's rows of the step in order from the state the step before left: a prompt,
// a portion of one and a single token are the same code. Thread (p, r) holds rows r, r + R, ... of column p of S in
// registers (R = 256 / PT); the sums over N meet in LDS, once a token.
#include "common.h"

#define SSM_THREADS 256
#define SSM_MAX_STATE 256
#define SSM_BATCH 8              // tokens whose operands are brought into LDS together

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int PT>
__global__ __launch_bounds__(SSM_THREADS) void ssm_scan_kernel(
    const T* __restrict__ xbc, int64_t xbc_stride, int x_col, int b_col, int c_col, const float* __restrict__ dt_raw,
    int64_t dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ y, int H, int P, int N, int G, int write_state) {
  constexpr int R = SSM_THREADS / PT, NS = SSM_MAX_STATE / R;
  __shared__ float sB[SSM_BATCH][SSM_MAX_STATE], sC[SSM_BATCH][SSM_MAX_STATE], sx[SSM_BATCH][PT];
  __shared__ float sdt[SSM_BATCH], sa[SSM_BATCH];
  __shared__ float red[2][R][PT];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * PT;
  const int slot = seq_slot[seq], rows = q_len[seq];
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq];
  const int group = head / (H / G);
  const int p = threadIdx.x % PT, r = threadIdx.x / PT;
  const bool live = p0 + p < P;
  const int cnt = (N - r + R - 1) / R;                // rows of S this thread holds: r, r + R, ...
  float* mine = state + (((int64_t)slot * H + head) * N) * P + p0 + p;
  float S[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) S[i] = (live && i < cnt) ? mine[(int64_t)(r + i * R) * P] : 0.f;
  const float rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
  for (int t0 = 0; t0 < rows; t0 += SSM_BATCH) {
    const int nb = min(SSM_BATCH, rows - t0);
    __syncthreads();
    for (int i = threadIdx.x; i < nb * N; i += SSM_THREADS) {
      const int tt = i / N, n = i % N;
      const T* src = xbc + (first + t0 + tt) * xbc_stride;
      sB[tt][n] = load_as_float(src + b_col + group * N + n);
      sC[tt][n] = load_as_float(src + c_col + group * N + n);
    }
    for (int i = threadIdx.x; i < nb * PT; i += SSM_THREADS) {
      const int tt = i / PT, pp = i % PT;
      sx[tt][pp] = p0 + pp < P ? load_as_float(xbc + (first + t0 + tt) * xbc_stride + x_col + head * P + p0 + pp) : 0.f;
    }
    if (threadIdx.x < nb) {
      const float dt = softplus_f(dt_raw[(first + t0 + threadIdx.x) * dt_stride + head] + bias);
      sdt[threadIdx.x] = dt;
      sa[threadIdx.x] = expf(-rate * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float a = sa[tt], dtx = sdt[tt] * sx[tt][p];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        if (i < cnt) {
          const int n = r + i * R;
          S[i] = a * S[i] + dtx * sB[tt][n];
          acc += S[i] * sC[tt][n];
        }
      }
      const int par = tt & 1;
      red[par][r][p] = acc;
      __syncthreads();
      if (r == 0 && live) {
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < R; ++k) sum += red[par][k][p];
        y[(first + t0 + tt) * (int64_t)(H * P) + head * P + p0 + p] = sum + skip * sx[tt][p];
      }
    }
  }
  if (write_state && live) {
#pragma unroll
    for (int i = 0; i < NS; ++i)
      if (i < cnt) mine[(int64_t)(r + i * R) * P] = S[i];
  }
}

// ---------------------------------------------------------------------------------------------------
// Read-out: v = y * silu(z), then each of `parts` equal runs of v divided by its own root mean square, times the
// weight: out = v / sqrt(mean_part(v^2) + eps) * w. One workgroup per (row, part); float arithmetic, rounded once.
// A row whose sequence sits out gives zeros.
template <typename T>
__global__ __launch_bounds__(256) void gate_part_norm_kernel(const float* __restrict__ y, const T* __restrict__ z,
                                                             int64_t z_stride, int z_col, const float* __restrict__ w,
                                                             const int* __restrict__ row_slot, T* __restrict__ out,
                                                             int inner, int parts, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int part = blockIdx.y, len = inner / parts, c0 = part * len;
  if (row_slot[row] < 0) {
    for (int i = threadIdx.x; i < len; i += blockDim.x) store_from_float(out + row * inner + c0 + i, 0.f);
    return;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < len; i += blockDim.x) {
    const float g = load_as_float(z + row * z_stride + z_col + c0 + i);
    const float v = y[row * inner + c0 + i] * (g / (1.f + expf(-g)));
    ss += v * v;
  }
  const float inv = rsqrtf(block_sum(ss, scratch) / (float)len + eps);
  for (int i = threadIdx.x; i < len; i += blockDim.x) {
    const float g = load_as_float(z + row * z_stride + z_col + c0 + i);
    const float v = y[row * inner + c0 + i] * (g / (1.f + expf(-g)));
    store_from_float(out + row * inner + c0 + i, v * inv * w[c0 + i]);
  }
}

DRYFT_API int dryft_ssm_max_state() { return SSM_MAX_STATE; }

DRYFT_API int dryft_ssm_scan(const void* xbc, int64_t xbc_stride, int x_col, int b_col, int c_col, const float* dt_raw,
                             int64_t dt_stride, const float* dt_bias, const float* a_log, const float* d_skip,
                             const int* seq_slot, const int* cu_rows, const int* q_len, float* state, float* y, int n_seqs,
                             int H, int P, int N, int G, int write_state, int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || P <= 0 || N <= 0 || N > SSM_MAX_STATE || G <= 0 || H % G) return -1;
#define SSM_LAUNCH(TT, PTV)                                                                                          \
  hipLaunchKernelGGL((ssm_scan_kernel<TT, PTV>), dim3(n_seqs, H, (P + PTV - 1) / PTV), dim3(SSM_THREADS), 0, stream, \
                     (const TT*)xbc, xbc_stride, x_col, b_col, c_col, dt_raw, dt_stride, dt_bias, a_log, d_skip,     \
                     seq_slot, cu_rows, q_len, state, y, H, P, N, G, write_state)
  if (is_f32) {
    if (P > 32) SSM_LAUNCH(float, 64); else if (P > 16) SSM_LAUNCH(float, 32); else SSM_LAUNCH(float, 16);
  } else {
    if (P > 32) SSM_LAUNCH(bf16_t, 64); else if (P > 16) SSM_LAUNCH(bf16_t, 32); else SSM_LAUNCH(bf16_t, 16);
  }
#undef SSM_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_gate_part_norm(const float* y, const void* z, int64_t z_stride, int z_col, const float* w,
                                   const int* row_slot, void* out, int n_rows, int inner, int parts, float eps,
                                   int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (inner <= 0 || parts <= 0 || inner % parts) return -1;
  dim3 grid(n_rows, parts), block(256);
  if (is_f32)
    hipLaunchKernelGGL(gate_part_norm_kernel<float>, grid, block, 0, stream, y, (const float*)z, z_stride, z_col, w,
                       row_slot, (float*)out, inner, parts, eps);
  else
    hipLaunchKernelGGL(gate_part_norm_kernel<bf16_t>, grid, block, 0, stream, y, (const bf16_t*)z, z_stride, z_col, w,
                       row_slot, (bf16_t*)out, inner, parts, eps);
  return DRYFT_LAUNCH_CHECK();
}
