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
// chain of dependent steps, so what counts is how short one step is. A column of S lives in the registers of LPC
// neighbouring lanes (D / LPC rows each, at most 64): both sums over D of a token are sums inside a thread plus
// LPC's worth of lane exchanges inside a row of lanes, with no barrier and no trip through LDS. The host takes
// as many lanes a column as still leave every lane eight rows and the chip a wave per SIMD. The token's k and q
// are the same for every column: they wait in LDS, one run per lane of a column (runs a bank apart), read 16
// bytes at a time. Operands come in batches of eight tokens: while the wave walks one batch, the next one's loads
// are in flight; the unit lengths (a sum over D per token) are taken by four lanes a vector as the batch goes to LDS.
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
    int write_state, int vec8) {
  constexpr int CW = WAVE / LPC;                       // columns a wave owns
  constexpr int ROWS = DELTA_MAX_DIM / LPC < DELTA_ROWS ? DELTA_MAX_DIM / LPC : DELTA_ROWS;
  constexpr int R4 = ROWS / 4;
  constexpr int PER = DELTA_MAX_DIM / 4;               // values of a q or k vector one of its four lanes takes at most
  constexpr int VN = (DELTA_BATCH * CW + WAVE - 1) / WAVE;
  // a vector in LDS: LPC runs (the rows of one lane each), a run padded with zeros to a multiple of 4 floats and
  // followed by 4 more so that neighbouring runs start in different banks
  __shared__ __attribute__((aligned(16))) float sk[DELTA_BATCH][DELTA_MAX_DIM + 8 * LPC];
  __shared__ __attribute__((aligned(16))) float sq[DELTA_BATCH][DELTA_MAX_DIM + 8 * LPC];
  __shared__ float sv[DELTA_BATCH][CW], sg[DELTA_BATCH], sbeta[DELTA_BATCH];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * CW;
  const int slot = seq_slot[seq], rows = q_len[seq];
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq];
  const int group = head / (H / G);
  const int lane = threadIdx.x, sub = lane % LPC, col = lane / LPC;
  const bool live = p0 + col < P;
  const int rd = (D + LPC - 1) / LPC, rd4 = (rd + 3) / 4, run = 4 * rd4 + 4;    // rows a lane holds, in fours, a run in LDS
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
  const int per = vec8 ? D / 4 : (D + 3) / 4;           // values of a vector a lane takes
  const int run0 = (part * per) / rd, off0 = (part * per) % rd;   // where its first value goes
  float x[PER], vv[VN], gate_a = 0.f, gate_b = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(DELTA_BATCH, rows - t0);
    if (v_tok < nb) {
      const T* src = qkv + (first + t0 + v_tok) * qkv_stride + (v_is_k ? k_col : q_col) + group * D + part * per;
      if (vec8) {
#pragma unroll
        for (int i = 0; i < PER / 8; ++i) {
          float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if (8 * i < per) load8_as_float(src + 8 * i, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) x[8 * i + j] = t[j];
        }
      } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) x[i] = (i < per && part * per + i < D) ? load_as_float(src + i) : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
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
    ss = lanes_sum<4>(ss);
    if (v_tok < nb) {
      const float inv = rsqrtf(ss + unit_eps) * (v_is_k ? 1.f : q_scale);
      float* dst = v_is_k ? sk[v_tok] : sq[v_tok];
      int r = run0, o = off0;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        if (i < per && part * per + i < D) dst[r * run + o] = x[i] * inv;
        if (++o == rd) { o = 0; ++r; }
      }
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int idx = lane + j * WAVE;
      if (idx < DELTA_BATCH * CW) sv[idx / CW][idx % CW] = vv[j];
    }
    if (lane < nb) {
      sg[lane] = expf(-rate * softplus_d(gate_a + bias));
      sbeta[lane] = 1.f / (1.f + expf(-gate_b));
    }
  };
  if (4 * rd4 != rd || rd * LPC != D) {                // what pads the runs stays zero for good
    for (int i = lane; i < DELTA_BATCH * (DELTA_MAX_DIM + 8 * LPC); i += WAVE) { (&sk[0][0])[i] = 0.f; (&sq[0][0])[i] = 0.f; }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  fetch(0);
  for (int t0 = 0; t0 < rows; t0 += DELTA_BATCH) {
    const int nb = min(DELTA_BATCH, rows - t0);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");      // one wave: order only, the loads in flight stay in flight
    __builtin_amdgcn_wave_barrier();
    stage(t0);
    if (t0 + DELTA_BATCH < rows) fetch(t0 + DELTA_BATCH);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int tt = 0; tt < nb; ++tt) {
      const float g = sg[tt], beta = sbeta[tt], v = sv[tt][col];
      const vf4* kp = (const vf4*)(sk[tt] + sub * run);
      const vf4* qp = (const vf4*)(sq[tt] + sub * run);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R4; ++i) {
        if (i < rd4) {
          const vf4 kk = kp[i];
          acc += S[4 * i] * kk[0] + S[4 * i + 1] * kk[1] + S[4 * i + 2] * kk[2] + S[4 * i + 3] * kk[3];
        }
      }
      acc = lanes_sum<LPC>(acc);
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
      res = lanes_sum<LPC>(res);
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

// Lanes a column: as few as hold its rows (64 each), then more while every lane keeps eight rows or more and the
// launch stays within a wave per SIMD of the chip.
static int lanes_per_column(int rows_of_state, int n_seqs, int heads, int columns) {
  int lpc = rows_of_state > 128 ? 4 : (rows_of_state > 64 ? 2 : 1);
  while (lpc < 16) {
    const int next = 2 * lpc, cw = WAVE / next;
    if ((rows_of_state + next - 1) / next < 8) break;
    if ((int64_t)n_seqs * heads * ((columns + cw - 1) / cw) > 1024 && cw < columns) break;
    lpc = next;
  }
  return lpc;
}

DRYFT_API int dryft_delta_steps(const void* qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* gates,
                                int64_t gate_stride, int a_col, int b_col, const float* dt_bias, const float* a_log,
                                const int* seq_slot, const int* cu_rows, const int* q_len, float* state, float* out,
                                int n_seqs, int H, int G, int D, int P, float q_scale, float unit_eps, int write_state,
                                int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > DELTA_MAX_DIM || P <= 0) return -1;
  // 16-byte loads of q and k: a lane's quarter of a vector in whole pieces of 8 values, at aligned addresses
  const int vec8 = (D % 32 == 0 && q_col % 8 == 0 && k_col % 8 == 0 && qkv_stride % 8 == 0 && ((uintptr_t)qkv & 15) == 0) ? 1 : 0;
#define DELTA_LAUNCH(TT, L)                                                                                           \
  hipLaunchKernelGGL((delta_steps_kernel<TT, L>), dim3(n_seqs, H, (P + WAVE / L - 1) / (WAVE / L)), dim3(WAVE), 0,   \
                     stream, (const TT*)qkv, qkv_stride, q_col, k_col, v_col, gates, gate_stride, a_col, b_col, dt_bias, \
                     a_log, seq_slot, cu_rows, q_len, state, out, H, G, D, P, q_scale, unit_eps, write_state, vec8)
#define DELTA_PICK(TT)                                                                                                \
  switch (lpc) {                                                                                                      \
    case 16: DELTA_LAUNCH(TT, 16); break;                                                                             \
    case 8: DELTA_LAUNCH(TT, 8); break;                                                                               \
    case 4: DELTA_LAUNCH(TT, 4); break;                                                                               \
    case 2: DELTA_LAUNCH(TT, 2); break;                                                                               \
    default: DELTA_LAUNCH(TT, 1);                                                                                     \
  }
  const int lpc = lanes_per_column(D, n_seqs, H, P);
  if (is_f32) { DELTA_PICK(float) } else { DELTA_PICK(bf16_t) }
#undef DELTA_PICK
#undef DELTA_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}
