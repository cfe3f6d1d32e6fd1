// The gated delta rule: a matrix state per head that decays, is corrected towards the token's value along the
// token's key, and is read with the token's query, in this order:
//
//   g_t = exp(-exp(A_log_h) * softplus(a_raw_t + dt_bias_h))      beta_t = sigmoid(b_raw_t)
//   S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t        (S is D x P per head)
//
// q and k (one per group of heads) arrive in the activation dtype from the short convolution and are made unit
// vectors here, x / sqrt(sum(x^2) + eps), q also times a factor. The state is float32 in the state store and all of
// the above is float arithmetic.
//
// One wave owns one (sequence, head, run of value columns) and walks the sequence's rows of the step in order from
// the state the step before left: a prompt, a portion of one and a single token are the same code. The walk is a
// chain of dependent steps, so what counts is how short one step is: a column of S lives in the registers of LPC
// neighbouring-by-stride lanes (D / LPC rows each, at most 64), so that both sums over D of a token are sums inside
// a thread plus one or two lane exchanges, with no barrier and no trip through LDS. The token's k and q are the same
// for every column: they wait in LDS, read as 16-byte broadcasts. Operands come in batches of eight tokens: while
// the wave walks one batch, the next one's loads are in flight; the unit lengths (a sum over D per token) are taken
// by four lanes a vector as the batch goes to LDS.
#include "common.h"

#define DELTA_MAX_DIM 256
#define DELTA_BATCH 8            // tokens whose operands are brought into LDS together
#define DELTA_ROWS 64            // rows of a column a lane holds at most

__device__ __forceinline__ float softplus_d(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int LPC>
__global__ __launch_bounds__(WAVE) void delta_steps_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* __restrict__ gates,
    int64_t gate_stride, int a_col, int b_col, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ out, int H, int G, int D, int P, float q_scale, float unit_eps,
    int write_state) {
  constexpr int CW = WAVE / LPC;                       // columns a wave owns
  constexpr int ROWS = DELTA_MAX_DIM / LPC < DELTA_ROWS ? DELTA_MAX_DIM / LPC : DELTA_ROWS;   // rows of a column a lane holds at most
  constexpr int R4 = ROWS / 4;
  constexpr int PER = DELTA_MAX_DIM / 4;               // values of a q or k vector one of its four lanes takes at most
  // a vector in LDS: LPC runs of `rdp` floats (the rows of one lane), padded to a multiple of 4 with zeros
  __shared__ __attribute__((aligned(16))) float sk[DELTA_BATCH][DELTA_MAX_DIM + 4 * LPC];
  __shared__ __attribute__((aligned(16))) float sq[DELTA_BATCH][DELTA_MAX_DIM + 4 * LPC];
  __shared__ float sv[DELTA_BATCH][CW], sg[DELTA_BATCH], sbeta[DELTA_BATCH];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * CW;
  const int slot = seq_slot[seq], rows = q_len[seq];
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq];
  const int group = head / (H / G);
  const int lane = threadIdx.x, col = lane % CW, sub = lane / CW;
  const bool live = p0 + col < P;
  const int rd = (D + LPC - 1) / LPC, rd4 = (rd + 3) / 4, rdp = 4 * rd4;     // rows a lane holds, in fours, padded
  float* mine = state + (((int64_t)slot * H + head) * D) * P + p0 + col;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int d = sub * rd + i;
    S[i] = (live && i < rd && d < D) ? mine[(int64_t)d * P] : 0.f;
  }
  const float rate = expf(a_log[head]), bias = dt_bias[head];
  // the batch's loads: lane l takes part (l % 4) of vector (l / 4): token (l / 8), q or k ((l / 4) % 2)
  const int vec = lane / 4, part = lane % 4, v_tok = vec >> 1, v_is_k = vec & 1;
  const int per = (D + 3) / 4;                          // values of a vector a lane takes
  float x[PER], vv[DELTA_BATCH * CW / WAVE], gate_a = 0.f, gate_b = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(DELTA_BATCH, rows - t0);
    if (v_tok < nb) {
      const T* src = qkv + (first + t0 + v_tok) * qkv_stride + (v_is_k ? k_col : q_col) + group * D + part * per;
#pragma unroll
      for (int i = 0; i < PER; ++i) x[i] = (i < per && part * per + i < D) ? load_as_float(src + i) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < DELTA_BATCH * CW / WAVE; ++j) {
      const int idx = lane + j * WAVE, tt = idx / CW, pp = idx % CW;
      vv[j] = (tt < nb && p0 + pp < P) ? load_as_float(qkv + (first + t0 + tt) * qkv_stride + v_col + head * P + p0 + pp) : 0.f;
    }
    if (lane < nb) {
      const float* gr = gates + (first + t0 + lane) * gate_stride;
      gate_a = gr[a_col + head];
      gate_b = gr[b_col + head];
    }
  };
  auto stage = [&](int t0) {
    const int nb = min(DELTA_BATCH, rows - t0);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) ss += x[i] * x[i];
    ss += __shfl_xor(ss, 1, WAVE);
    ss += __shfl_xor(ss, 2, WAVE);
    if (v_tok < nb) {
      const float inv = rsqrtf(ss + unit_eps) * (v_is_k ? 1.f : q_scale);
      float* dst = v_is_k ? sk[v_tok] : sq[v_tok];
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int d = part * per + i;
        if (i < per && d < D) dst[(d / rd) * rdp + d % rd] = x[i] * inv;
      }
    }
#pragma unroll
    for (int j = 0; j < DELTA_BATCH * CW / WAVE; ++j) {
      const int idx = lane + j * WAVE;
      sv[idx / CW][idx % CW] = vv[j];
    }
    if (lane < nb) {
      sg[lane] = expf(-rate * softplus_d(gate_a + bias));
      sbeta[lane] = 1.f / (1.f + expf(-gate_b));
    }
  };
  // the padding of every run stays zero for good
  for (int i = lane; i < DELTA_BATCH * (DELTA_MAX_DIM + 4 * LPC); i += WAVE) { (&sk[0][0])[i] = 0.f; (&sq[0][0])[i] = 0.f; }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  __builtin_amdgcn_wave_barrier();
  fetch(0);
  for (int t0 = 0; t0 < rows; t0 += DELTA_BATCH) {
    const int nb = min(DELTA_BATCH, rows - t0);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");      // the walk over the batch before is done with LDS
    __builtin_amdgcn_wave_barrier();
    stage(t0);
    if (t0 + DELTA_BATCH < rows) fetch(t0 + DELTA_BATCH);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    __builtin_amdgcn_wave_barrier();
    for (int tt = 0; tt < nb; ++tt) {
      const float g = sg[tt], beta = sbeta[tt], v = sv[tt][col];
      const vf4* kp = (const vf4*)(sk[tt] + sub * rdp);
      const vf4* qp = (const vf4*)(sq[tt] + sub * rdp);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R4; ++i) {
        if (i < rd4) {
          const vf4 kk = kp[i];
          acc += S[4 * i] * kk[0] + S[4 * i + 1] * kk[1] + S[4 * i + 2] * kk[2] + S[4 * i + 3] * kk[3];
        }
      }
#pragma unroll
      for (int o = CW; o < WAVE; o <<= 1) acc += __shfl_xor(acc, o, WAVE);
      const float u = beta * (v - g * acc);
      float res = 0.f;
#pragma unroll
      for (int i = 0; i < R4; ++i) {
        if (i < rd4) {
          const vf4 kk = kp[i], qq = qp[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            S[4 * i + j] = g * S[4 * i + j] + kk[j] * u;
            res += S[4 * i + j] * qq[j];
          }
        }
      }
#pragma unroll
      for (int o = CW; o < WAVE; o <<= 1) res += __shfl_xor(res, o, WAVE);
      if (sub == 0 && live) out[(first + t0 + tt) * (int64_t)(H * P) + head * P + p0 + col] = res;
    }
  }
  if (write_state && live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = sub * rd + i;
      if (i < rd && d < D) mine[(int64_t)d * P] = S[i];
    }
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
#define DELTA_LAUNCH(TT, L)                                                                                           \
  hipLaunchKernelGGL((delta_steps_kernel<TT, L>), dim3(n_seqs, H, (P + WAVE / L - 1) / (WAVE / L)), dim3(WAVE), 0,   \
                     stream, (const TT*)qkv, qkv_stride, q_col, k_col, v_col, gates, gate_stride, a_col, b_col, dt_bias, \
                     a_log, seq_slot, cu_rows, q_len, state, out, H, G, D, P, q_scale, unit_eps, write_state)
  // lanes a column: as few as hold its rows (64 each), and no more columns a wave than the head has
  int lpc = D > 128 ? 4 : (D > 64 ? 2 : 1);
  while (lpc < 4 && WAVE / lpc > P && WAVE / (2 * lpc) >= 8) lpc *= 2;
  if (is_f32) {
    if (lpc == 4) DELTA_LAUNCH(float, 4); else if (lpc == 2) DELTA_LAUNCH(float, 2); else DELTA_LAUNCH(float, 1);
  } else {
    if (lpc == 4) DELTA_LAUNCH(bf16_t, 4); else if (lpc == 2) DELTA_LAUNCH(bf16_t, 2); else DELTA_LAUNCH(bf16_t, 1);
  }
#undef DELTA_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}
