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

//
// Long prompts are cut into segments of `seg_rows` rows that run side by side (MODE 1, then the carry kernel, then
// MODE 2; MODE 0 walks a whole sequence). A token maps every column of the state alike, c -> g (I - beta k k^T) c +
// beta k v_c, so a segment's effect is S_out = A S_in + L with A (D x D) the product of its tokens' maps and L the
// state it reaches from zero. MODE 1 computes both for every segment but a sequence's last, without read-outs: L
// by the walk from zero, and A by the same walk, with values of zero, over the D columns of the unit matrix (the
// waves of the grid behind those of the value columns). The carry kernel walks a sequence's segments and leaves each
// the state that enters it; MODE 2 starts every segment from that state and writes its read-outs, and a sequence's
// last segment writes the state back. Segment x of the step belongs to the sequence s with seg_cu[s] <= x <
// seg_cu[s + 1] (prefix sums over the sequences; one that sits out has none).
template <typename T, int LPC, int MODE, int MAXN>
__global__ __launch_bounds__(WAVE) void delta_steps_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* __restrict__ gates,
    int64_t gate_stride, int a_col, int b_col, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ out, int H, int G, int D, int P, float q_scale, float unit_eps,
    int write_state, int vec8, const int* __restrict__ seg_cu, int n_seqs, int seg_rows, float* __restrict__ seg_state,
    float* __restrict__ seg_trans) {
  constexpr int CW = WAVE / LPC;                       // columns a wave owns
  constexpr int ROWS = MAXN / LPC < DELTA_ROWS ? MAXN / LPC : DELTA_ROWS;
  constexpr int R4 = ROWS / 4;
  constexpr int PER = MAXN / 4;                // values of a q or k vector one of its four lanes takes at most
  constexpr int VN = (DELTA_BATCH * CW + WAVE - 1) / WAVE;
  // a vector in LDS: LPC runs (the rows of one lane each), a run padded with zeros to a multiple of 4 floats and
  // followed by 4 more so that neighbouring runs start in different banks
  __shared__ __attribute__((aligned(16))) float sk[DELTA_BATCH][MAXN + 8 * LPC];
  __shared__ __attribute__((aligned(16))) float sq[DELTA_BATCH][MAXN + 8 * LPC];
  __shared__ float sv[DELTA_BATCH][CW], sg[DELTA_BATCH], sbeta[DELTA_BATCH];
  const int head = blockIdx.y, z_values = (P + CW - 1) / CW;
  const bool unit = MODE == 1 && (int)blockIdx.z >= z_values;      // this wave walks columns of the unit matrix
  const int p0 = (unit ? blockIdx.z - z_values : blockIdx.z) * CW;
  int seq = blockIdx.x, seg = 0, n_segs = 1;
  if (MODE != 0) {
    if ((int)blockIdx.x >= seg_cu[n_seqs]) return;
    seq = 0;
    while (seg_cu[seq + 1] <= (int)blockIdx.x) ++seq;
    seg = blockIdx.x - seg_cu[seq];
    n_segs = seg_cu[seq + 1] - seg_cu[seq];
    if (MODE == 1 && seg == n_segs - 1) return;                   // nobody needs the last segment's summary
  }
  const int slot = seq_slot[seq];
  const int rows = MODE == 0 ? q_len[seq] : min(seg_rows, q_len[seq] - seg * seg_rows);
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq] + (MODE == 0 ? 0 : seg * seg_rows);
  const int group = head / (H / G);
  const int lane = threadIdx.x, sub = lane % LPC, col = lane / LPC;
  const int width = unit ? D : P;                                  // columns of what this wave walks
  const bool live = p0 + col < width;
  const int rd = (D + LPC - 1) / LPC, rd4 = (rd + 3) / 4, run = 4 * rd4 + 4;    // rows a lane holds, in fours, a run in LDS
  float* mine = state + (((int64_t)slot * H + head) * D) * P + p0 + col;
  float* seg_mine = MODE == 0 ? nullptr
                    : unit    ? seg_trans + (((int64_t)blockIdx.x * H + head) * D + p0 + col) * D
                              : seg_state + (((int64_t)blockIdx.x * H + head) * D) * P + p0 + col;
  const float* from = MODE == 2 ? seg_mine : mine;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int d = sub * rd + i;
    if (MODE == 1) S[i] = (unit && live && i < rd && d == p0 + col) ? 1.f : 0.f;
    else S[i] = (live && i < rd && d < D) ? from[(int64_t)d * P] : 0.f;
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
      vv[j] = (!unit && tt < nb && p0 + pp < P) ? load_as_float(qkv + (first + t0 + tt) * qkv_stride + v_col + head * P + p0 + pp) : 0.f;
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
    for (int i = lane; i < DELTA_BATCH * (MAXN + 8 * LPC); i += WAVE) { (&sk[0][0])[i] = 0.f; (&sq[0][0])[i] = 0.f; }
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
      if (MODE == 1) {
#pragma unroll
        for (int i = 0; i < R4; ++i) {
          if (i < rd4) {
            const vf4 kk = kp[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) S[4 * i + j] = g * S[4 * i + j] + kk[j] * u;
          }
        }
        continue;
      }
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
  if (MODE == 2 && seg != n_segs - 1) return;                     // the last segment leaves the sequence's state
  float* to = MODE == 1 ? seg_mine : mine;
  if ((MODE == 1 || write_state) && live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int d = sub * rd + i;
      if (i < rd && d < D) to[unit ? d : (int64_t)d * P] = S[i];     // a column of A lies in one piece
    }
  }
}

// The state that enters each segment of a sequence: S_in[0] is the sequence's own state, S_in[s + 1] =
// A[s] S_in[s] + L[s]. One workgroup per (sequence, head, 4 columns), a thread a row of the state: the columns'
// current values wait in LDS, every thread reads them all (broadcasts) against its row of A (`seg_trans` holds A
// column by column, so that the threads of a wave read neighbouring words). The walk over a sequence's segments is a
// chain of dependent steps whose loads of A are what it waits for: few columns a workgroup (many workgroups) and many
// loads in flight a thread measured best. `seg_state` holds L when the kernel starts and S_in when it ends.
#define DELTA_CARRY_COLS 4
__global__ __launch_bounds__(DELTA_MAX_DIM) void delta_carry_kernel(
    const int* __restrict__ seq_slot, const int* __restrict__ seg_cu, const float* __restrict__ state,
    float* __restrict__ seg_state, const float* __restrict__ seg_trans, int H, int D, int P) {
  __shared__ __attribute__((aligned(16))) float held[2][DELTA_MAX_DIM][DELTA_CARRY_COLS];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * DELTA_CARRY_COLS, d = threadIdx.x;
  const int x0 = seg_cu[seq], n_segs = seg_cu[seq + 1] - x0, slot = seq_slot[seq];
  if (slot < 0 || n_segs <= 0) return;
  const bool row = d < D;
  if (row) {
    const float* src = state + (((int64_t)slot * H + head) * D + d) * P + p0;
#pragma unroll
    for (int c = 0; c < DELTA_CARRY_COLS; ++c) held[0][d][c] = p0 + c < P ? src[c] : 0.f;
  }
  __syncthreads();
  int cur = 0;
  for (int s = 0; s < n_segs; ++s) {
    const bool last = s + 1 == n_segs;
    if (row) {
      float* at = seg_state + ((((int64_t)(x0 + s)) * H + head) * D + d) * P + p0;
      float acc[DELTA_CARRY_COLS];
#pragma unroll
      for (int c = 0; c < DELTA_CARRY_COLS; ++c) {
        acc[c] = (!last && p0 + c < P) ? at[c] : 0.f;
        if (p0 + c < P) at[c] = held[cur][d][c];
      }
      if (!last) {
        const float* a_row = seg_trans + (((int64_t)(x0 + s)) * H + head) * D * D + d;
#pragma unroll 32
        for (int e = 0; e < D; ++e) {
          const float a = a_row[(int64_t)e * D];
#pragma unroll
          for (int c = 0; c < DELTA_CARRY_COLS; ++c) acc[c] += a * held[cur][e][c];
        }
#pragma unroll
        for (int c = 0; c < DELTA_CARRY_COLS; ++c) held[cur ^ 1][d][c] = acc[c];
      }
    }
    __syncthreads();
    cur ^= 1;
  }
}

DRYFT_API int dryft_delta_max_dim() { return DELTA_MAX_DIM; }

// Lanes a column: as few as hold its rows (64 each), then more while every lane keeps eight rows or more and the
// launch stays within `most` waves.
static int lanes_per_column(int rows_of_state, int walks, int heads, int columns, int most) {
  int lpc = rows_of_state > 128 ? 4 : (rows_of_state > 64 ? 2 : 1);
  while (lpc < 16) {
    const int next = 2 * lpc, cw = WAVE / next;
    if ((rows_of_state + next - 1) / next < 8) break;
    if ((int64_t)walks * heads * ((columns + cw - 1) / cw) > most && cw < columns) break;
    lpc = next;
  }
  return lpc;
}

DRYFT_API int dryft_delta_steps(const void* qkv, int64_t qkv_stride, int q_col, int k_col, int v_col, const float* gates,
                                int64_t gate_stride, int a_col, int b_col, const float* dt_bias, const float* a_log,
                                const int* seq_slot, const int* cu_rows, const int* q_len, float* state, float* out,
                                int n_seqs, int H, int G, int D, int P, float q_scale, float unit_eps, int write_state,
                                const int* seg_cu, int max_segs, int seg_rows, float* seg_state, float* seg_trans,
                                int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > DELTA_MAX_DIM || P <= 0) return -1;
  const bool cut = seg_cu != nullptr;
  if (cut && (max_segs <= 0 || seg_rows <= 0 || seg_state == nullptr || seg_trans == nullptr || !write_state)) return -1;
  const int walks = cut ? max_segs : n_seqs;
  // 16-byte loads of q and k: a lane's quarter of a vector in whole pieces of 8 values, at aligned addresses
  const int vec8 = (D % 32 == 0 && q_col % 8 == 0 && k_col % 8 == 0 && qkv_stride % 8 == 0 && ((uintptr_t)qkv & 15) == 0) ? 1 : 0;
  // MODE 1 walks the D columns of the unit matrix behind the P value columns. The kernel is built for states of up
  // to 64, 128 and 256 rows (X), so that a lane's registers and the loops over them fit the state at hand.
#define DELTA_LAUNCH(TT, L, M, X)                                                                                     \
  hipLaunchKernelGGL((delta_steps_kernel<TT, L, M, X>),                                                               \
                     dim3(walks, H, (P + WAVE / L - 1) / (WAVE / L) + (M == 1 ? (D + WAVE / L - 1) / (WAVE / L) : 0)), \
                     dim3(WAVE), 0, stream, (const TT*)qkv, qkv_stride, q_col, k_col, v_col, gates, gate_stride, a_col, \
                     b_col, dt_bias, a_log, seq_slot, cu_rows, q_len, state, out, H, G, D, P, q_scale, unit_eps,      \
                     write_state, vec8, seg_cu, n_seqs, seg_rows, seg_state, seg_trans)
#define DELTA_CASE(TT, M, X, L) if (maxn == X && lpc == L) { DELTA_LAUNCH(TT, L, M, X); } else
#define DELTA_PICK(TT, M)                                                                                             \
  DELTA_CASE(TT, M, 64, 1) DELTA_CASE(TT, M, 64, 2) DELTA_CASE(TT, M, 64, 4) DELTA_CASE(TT, M, 64, 8)                 \
  DELTA_CASE(TT, M, 128, 2) DELTA_CASE(TT, M, 128, 4) DELTA_CASE(TT, M, 128, 8) DELTA_CASE(TT, M, 128, 16)            \
  DELTA_CASE(TT, M, 256, 4) DELTA_CASE(TT, M, 256, 8) DELTA_CASE(TT, M, 256, 16) { return -1; }
  // a whole walk keeps to a wave a SIMD; segments, whose waves hold less, to two. The summaries walk P + D columns.
#define DELTA_RUN(M)                                                                                                  \
  {                                                                                                                   \
    const int lpc = lanes_per_column(D, walks, H, M == 1 ? P + D : P, M == 0 ? 1024 : 2048);                          \
    if (is_f32) { DELTA_PICK(float, M) } else { DELTA_PICK(bf16_t, M) }                                               \
  }
  const int maxn = D > 128 ? 256 : (D > 64 ? 128 : 64);
  if (!cut) {
    DELTA_RUN(0)
  } else {
    DELTA_RUN(1)
    hipLaunchKernelGGL(delta_carry_kernel, dim3(n_seqs, H, (P + DELTA_CARRY_COLS - 1) / DELTA_CARRY_COLS),
                       dim3((D + WAVE - 1) / WAVE * WAVE), 0, stream, seq_slot, seg_cu, state, seg_state, seg_trans, H, D, P);
    DELTA_RUN(2)
  }
#undef DELTA_RUN
#undef DELTA_PICK
#undef DELTA_CASE
#undef DELTA_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}
