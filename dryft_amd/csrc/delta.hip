// The gated delta rule: a matrix state per head that decays, is corrected towards the token's value along the
// token's key, and is read with the token's query, in this order:
//
//   g_t = exp(-exp(A_log_h) * softplus(a_raw_t + dt_bias_h))      beta_t = sigmoid(b_raw_t)
//   S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t        (S is D x P per head)
//
// q and k (one per group of heads) arrive in the activation dtype from the short convolution and are made unit
// vectors here, x / sqrt(sum(x^2) + 1e-6), q also times D^-1/2. The state is float32 in the state store and all of
// the above is float arithmetic. A workgroup owns one (sequence, head, run of up to PT value columns) and walks the
// sequence's rows of the step in order from the state the step before left. Thread (p, r) holds rows r, r + R, ... of
// column p of S in registers (R = 256 / PT); the two sums over D of a token meet in LDS.
#include "common.h"

#define DELTA_THREADS 256
#define DELTA_MAX_DIM 256
#define DELTA_BATCH 8            // tokens whose operands are brought into LDS together

__device__ __forceinline__ float softplus_d(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int PT>
__global__ __launch_bounds__(DELTA_THREADS) void delta_steps_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* __restrict__ gates,
    int64_t gate_stride, int a_col, int b_col, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ out, int H, int G, int D, int P, float q_scale, float unit_eps,
    int write_state) {
  constexpr int R = DELTA_THREADS / PT, NS = DELTA_MAX_DIM / R, WAVES = DELTA_THREADS / WAVE;
  __shared__ float sq[DELTA_BATCH][DELTA_MAX_DIM], sk[DELTA_BATCH][DELTA_MAX_DIM], sv[DELTA_BATCH][PT];
  __shared__ float sg[DELTA_BATCH], sbeta[DELTA_BATCH];
  __shared__ float red_k[R][PT], red_o[2][R][PT];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * PT;
  const int slot = seq_slot[seq], rows = q_len[seq];
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq];
  const int group = head / (H / G);
  const int p = threadIdx.x % PT, r = threadIdx.x / PT;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const bool live = p0 + p < P;
  const int cnt = (D - r + R - 1) / R;
  float* mine = state + (((int64_t)slot * H + head) * D) * P + p0 + p;
  float S[NS];
#pragma unroll
  for (int i = 0; i < NS; ++i) S[i] = (live && i < cnt) ? mine[(int64_t)(r + i * R) * P] : 0.f;
  const float rate = expf(a_log[head]), bias = dt_bias[head];
  for (int t0 = 0; t0 < rows; t0 += DELTA_BATCH) {
    const int nb = min(DELTA_BATCH, rows - t0);
    __syncthreads();
    // a wave takes a token's q, then its k: load, sum of squares, unit length
    for (int job = wave; job < 2 * nb; job += WAVES) {
      const int tt = job >> 1, is_k = job & 1;
      const T* src = qkv + (first + t0 + tt) * qkv_stride + (is_k ? k_col : q_col) + group * D;
      float x[DELTA_MAX_DIM / WAVE], ss = 0.f;
#pragma unroll
      for (int i = 0; i < DELTA_MAX_DIM / WAVE; ++i) {
        const int d = lane + i * WAVE;
        x[i] = d < D ? load_as_float(src + d) : 0.f;
        ss += x[i] * x[i];
      }
      const float inv = rsqrtf(wave_sum(ss) + unit_eps) * (is_k ? 1.f : q_scale);
      float* dst = is_k ? sk[tt] : sq[tt];
#pragma unroll
      for (int i = 0; i < DELTA_MAX_DIM / WAVE; ++i) {
        const int d = lane + i * WAVE;
        if (d < D) dst[d] = x[i] * inv;
      }
    }
    for (int i = threadIdx.x; i < nb * PT; i += DELTA_THREADS) {
      const int tt = i / PT, pp = i % PT;
      sv[tt][pp] = p0 + pp < P ? load_as_float(qkv + (first + t0 + tt) * qkv_stride + v_col + head * P + p0 + pp) : 0.f;
    }
    if (threadIdx.x < nb) {
      const float* gr = gates + (first + t0 + threadIdx.x) * gate_stride;
      sg[threadIdx.x] = expf(-rate * softplus_d(gr[a_col + head] + bias));
      sbeta[threadIdx.x] = 1.f / (1.f + expf(-gr[b_col + head]));
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float g = sg[tt];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        if (i < cnt) {
          S[i] *= g;
          acc += S[i] * sk[tt][r + i * R];
        }
      }
      red_k[r][p] = acc;
      __syncthreads();
      float ks = 0.f;
#pragma unroll
      for (int k = 0; k < R; ++k) ks += red_k[k][p];
      const float u = sbeta[tt] * (sv[tt][p] - ks);
      acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        if (i < cnt) {
          const int d = r + i * R;
          S[i] += sk[tt][d] * u;
          acc += S[i] * sq[tt][d];
        }
      }
      const int par = tt & 1;
      red_o[par][r][p] = acc;
      __syncthreads();
      if (r == 0 && live) {
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < R; ++k) sum += red_o[par][k][p];
        out[(first + t0 + tt) * (int64_t)(H * P) + head * P + p0 + p] = sum;
      }
    }
  }
  if (write_state && live) {
#pragma unroll
    for (int i = 0; i < NS; ++i)
      if (i < cnt) mine[(int64_t)(r + i * R) * P] = S[i];
  }
}

DRYFT_API int dryft_delta_max_dim() { return DELTA_MAX_DIM; }

DRYFT_API int dryft_delta_steps(const void* qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* gates,
                                int64_t gate_stride, int a_col, int b_col, const float* dt_bias, const float* a_log,
                                const int* seq_slot, const int* cu_rows, const int* q_len, float* state, float* out,
                                int n_seqs, int H, int G, int D, int P, float q_scale, float unit_eps, int write_state,
                                int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > DELTA_MAX_DIM || P <= 0) return -1;
#define DELTA_LAUNCH(TT, PTV)                                                                                          \
  hipLaunchKernelGGL((delta_steps_kernel<TT, PTV>), dim3(n_seqs, H, (P + PTV - 1) / PTV), dim3(DELTA_THREADS), 0,     \
                     stream, (const TT*)qkv, qkv_stride, q_col, k_col, v_col, gates, gate_stride, a_col, b_col, dt_bias, \
                     a_log, seq_slot, cu_rows, q_len, state, out, H, G, D, P, q_scale, unit_eps, write_state)
  if (is_f32) {
    if (P > 32) DELTA_LAUNCH(float, 64); else if (P > 16) DELTA_LAUNCH(float, 32); else DELTA_LAUNCH(float, 16);
  } else {
    if (P > 32) DELTA_LAUNCH(bf16_t, 64); else if (P > 16) DELTA_LAUNCH(bf16_t, 32); else DELTA_LAUNCH(bf16_t, 16);
  }
#undef DELTA_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}
