// A state-space mixer with one scalar decay per head and token (the Mamba-2 recurrence), and its read-out.
//
//   dt_t = softplus(dt_raw_t + dt_bias_h)         a_t = exp(-exp(A_log_h) * dt_t)
//   S_t  = a_t S_(t-1) + dt_t B_t x_t^T           (S is N x P per head; B and C belong to the head's group)
//   y_t  = S_t^T C_t + D_h x_t
//
// The state is float32 in the state store and everything above is float arithmetic; x, B and C arrive in the
// activation dtype (the output of the short convolution). One wave owns one (sequence, head, run of value columns)
// and walks the sequence's rows of the step in order from the state the step before left: a prompt, a portion of
// one and a single token are the same code. The walk is a chain of dependent steps: a column of S lives in the
// registers of LPC neighbouring lanes (N / LPC rows each, at most 64), so that a token's sum over N is a sum inside
// a thread plus LPC's worth of lane exchanges inside a row of lanes, with no barrier. The host takes as many lanes
// a column as still leave every lane eight rows and the chip a wave per SIMD. B and C of a token are the same for
// every column: they wait in LDS, one run per lane of a column (runs a bank apart), read 16 bytes at a time.
// Operands come in batches of eight tokens; the next batch's loads are in flight while the wave walks this one.
#include "common.h"

#define SSM_MAX_STATE 256
#define SSM_BATCH 8              // tokens whose operands are brought into LDS together
#define SSM_ROWS 64              // rows of a column a lane holds at most

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

//
// Long prompts are cut into segments of `seg_rows` rows that run side by side (MODE 1, then the carry kernel, then
// MODE 2; MODE 0 walks a whole sequence). The recurrence is linear in the state and its decay one number per head
// and token, so a segment's effect is S_out = p S_in + L with p the product of the segment's decays and L the state
// it reaches from zero. MODE 1 computes L and p of every segment but a sequence's last (no read-outs); the carry
// kernel walks a sequence's segments and leaves each the state that enters it; MODE 2 starts every segment from that
// state and writes its read-outs, and a sequence's last segment writes the state back. Segment x of the step belongs
// to the sequence s with seg_cu[s] <= x < seg_cu[s + 1] (prefix sums over the sequences; one that sits out has none).
template <typename T, int LPC, int MODE, int MAXN>
__global__ __launch_bounds__(WAVE) void ssm_scan_kernel(
    const T* __restrict__ xbc, int64_t xbc_stride, int x_col, int b_col, int c_col, const float* __restrict__ dt_raw,
    int64_t dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ y, int H, int P, int N, int G, int write_state, int vec8,
    const int* __restrict__ seg_cu, int n_seqs, int seg_rows, float* __restrict__ seg_state,
    float* __restrict__ seg_decay) {
  constexpr int CW = WAVE / LPC;                       // columns a wave owns
  constexpr int ROWS = MAXN / LPC < SSM_ROWS ? MAXN / LPC : SSM_ROWS;
  constexpr int R4 = ROWS / 4;
  constexpr int PER = MAXN / 4;                // values of a B or C vector one of its four lanes takes at most
  constexpr int VN = (SSM_BATCH * CW + WAVE - 1) / WAVE;
  // a vector in LDS: LPC runs (the rows of one lane each), a run padded with zeros to a multiple of 4 floats and
  // followed by 4 more so that neighbouring runs start in different banks
  __shared__ __attribute__((aligned(16))) float sB[SSM_BATCH][MAXN + 8 * LPC];
  __shared__ __attribute__((aligned(16))) float sC[SSM_BATCH][MAXN + 8 * LPC];
  __shared__ float sx[SSM_BATCH][CW], sdt[SSM_BATCH], sa[SSM_BATCH];
  const int head = blockIdx.y, p0 = blockIdx.z * CW;
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
  const bool live = p0 + col < P;
  const int rd = (N + LPC - 1) / LPC, rd4 = (rd + 3) / 4, run = 4 * rd4 + 4;
  float* mine = state + (((int64_t)slot * H + head) * N) * P + p0 + col;
  float* seg_mine = MODE == 0 ? nullptr : seg_state + (((int64_t)blockIdx.x * H + head) * N) * P + p0 + col;
  const float* from = MODE == 2 ? seg_mine : mine;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int n = sub * rd + i;
    S[i] = (MODE != 1 && live && i < rd && n < N) ? from[(int64_t)n * P] : 0.f;
  }
  float decays = 1.f;
  const float rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
  // the batch's loads: lane l takes part (l % 4) of vector (l / 4): token (l / 8), B or C ((l / 4) % 2)
  const int vec = lane / 4, part = lane % 4, v_tok = vec >> 1, v_is_c = vec & 1;
  const int per = vec8 ? N / 4 : (N + 3) / 4;
  const int run0 = (part * per) / rd, off0 = (part * per) % rd;   // where its first value goes
  float bc[PER], xv[VN], dtr = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(SSM_BATCH, rows - t0);
    if (v_tok < nb) {
      const T* src = xbc + (first + t0 + v_tok) * xbc_stride + (v_is_c ? c_col : b_col) + group * N + part * per;
      if (vec8) {
#pragma unroll
        for (int i = 0; i < PER / 8; ++i) {
          float t[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if (8 * i < per) load8_as_float(src + 8 * i, t);
#pragma unroll
          for (int j = 0; j < 8; ++j) bc[8 * i + j] = t[j];
        }
      } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) bc[i] = (i < per && part * per + i < N) ? load_as_float(src + i) : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int idx = lane + j * WAVE, tt = idx / CW, pp = idx % CW;
      xv[j] = (tt < nb && p0 + pp < P) ? load_as_float(xbc + (first + t0 + tt) * xbc_stride + x_col + head * P + p0 + pp) : 0.f;
    }
    if (lane < nb) dtr = dt_raw[(first + t0 + lane) * dt_stride + head];
  };
  auto stage = [&](int t0) {
    const int nb = min(SSM_BATCH, rows - t0);
    if (v_tok < nb) {
      float* dst = v_is_c ? sC[v_tok] : sB[v_tok];
      int r = run0, o = off0;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        if (i < per && part * per + i < N) dst[r * run + o] = bc[i];
        if (++o == rd) { o = 0; ++r; }
      }
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int idx = lane + j * WAVE;
      if (idx < SSM_BATCH * CW) sx[idx / CW][idx % CW] = xv[j];
    }
    if (lane < nb) {
      const float dt = softplus_f(dtr + bias);
      sdt[lane] = dt;
      sa[lane] = expf(-rate * dt);
    }
  };
  if (4 * rd4 != rd || rd * LPC != N) {                // what pads the runs stays zero for good
    for (int i = lane; i < SSM_BATCH * (MAXN + 8 * LPC); i += WAVE) { (&sB[0][0])[i] = 0.f; (&sC[0][0])[i] = 0.f; }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  fetch(0);
  for (int t0 = 0; t0 < rows; t0 += SSM_BATCH) {
    const int nb = min(SSM_BATCH, rows - t0);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");      // one wave: order only, the loads in flight stay in flight
    __builtin_amdgcn_wave_barrier();
    stage(t0);
    if (t0 + SSM_BATCH < rows) fetch(t0 + SSM_BATCH);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int tt = 0; tt < nb; ++tt) {
      const float a = sa[tt], x = sx[tt][col], dtx = sdt[tt] * x;
      const vf4* bp = (const vf4*)(sB[tt] + sub * run);
      if (MODE == 1) {
        decays *= a;
#pragma unroll
        for (int i = 0; i < R4; ++i) {
          if (i < rd4) {
            const vf4 bb = bp[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) S[4 * i + j] = a * S[4 * i + j] + dtx * bb[j];
          }
        }
        continue;
      }
      const vf4* cp = (const vf4*)(sC[tt] + sub * run);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R4; ++i) {
        if (i < rd4) {
          const vf4 bb = bp[i], cc = cp[i];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            S[4 * i + j] = a * S[4 * i + j] + dtx * bb[j];
            acc += S[4 * i + j] * cc[j];
          }
        }
      }
      acc = lanes_sum<LPC>(acc);
      if (sub == 0 && live) y[(first + t0 + tt) * (int64_t)(H * P) + head * P + p0 + col] = acc + skip * x;
    }
  }
  if (MODE == 1 && blockIdx.z == 0 && lane == 0) seg_decay[(int64_t)blockIdx.x * H + head] = decays;
  if (MODE == 2 && seg != n_segs - 1) return;                     // the last segment leaves the sequence's state
  float* to = MODE == 1 ? seg_mine : mine;
  if ((MODE == 1 || write_state) && live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int n = sub * rd + i;
      if (i < rd && n < N) to[(int64_t)n * P] = S[i];
    }
  }
}

// The state that enters each segment of a sequence: S_in[0] is the sequence's own state, S_in[s + 1] =
// p[s] S_in[s] + L[s]. A thread an entry of the state; `seg_state` holds L when the kernel starts and S_in when it ends.
__global__ __launch_bounds__(256) void ssm_carry_kernel(const int* __restrict__ seq_slot, const int* __restrict__ seg_cu,
                                                        const float* __restrict__ state, float* __restrict__ seg_state,
                                                        const float* __restrict__ seg_decay, int H, int entries) {
  const int seq = blockIdx.x, head = blockIdx.y, e = blockIdx.z * 256 + threadIdx.x;
  const int x0 = seg_cu[seq], n_segs = seg_cu[seq + 1] - x0, slot = seq_slot[seq];
  if (slot < 0 || e >= entries) return;
  float held = state[((int64_t)slot * H + head) * entries + e];
  for (int s = 0; s < n_segs; ++s) {
    float* at = seg_state + ((int64_t)(x0 + s) * H + head) * entries + e;
    const float local = s + 1 < n_segs ? *at : 0.f;
    *at = held;
    if (s + 1 < n_segs) held = seg_decay[(int64_t)(x0 + s) * H + head] * held + local;
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

DRYFT_API int dryft_ssm_scan(const void* xbc, int64_t xbc_stride, int x_col, int b_col, int c_col, const float* dt_raw,
                             int64_t dt_stride, const float* dt_bias, const float* a_log, const float* d_skip,
                             const int* seq_slot, const int* cu_rows, const int* q_len, float* state, float* y, int n_seqs,
                             int H, int P, int N, int G, int write_state, const int* seg_cu, int max_segs, int seg_rows,
                             float* seg_state, float* seg_decay, int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (H <= 0 || P <= 0 || N <= 0 || N > SSM_MAX_STATE || G <= 0 || H % G) return -1;
  const bool cut = seg_cu != nullptr;
  if (cut && (max_segs <= 0 || seg_rows <= 0 || seg_state == nullptr || seg_decay == nullptr || !write_state)) return -1;
  const int walks = cut ? max_segs : n_seqs;
  // 16-byte loads of B and C: a lane's quarter of a vector in whole pieces of 8 values, at aligned addresses
  const int vec8 = (N % 32 == 0 && b_col % 8 == 0 && c_col % 8 == 0 && xbc_stride % 8 == 0 && ((uintptr_t)xbc & 15) == 0) ? 1 : 0;
  // The kernel is built for states of up to 64, 128 and 256 rows (X), so that a lane's registers and the loops over
  // them fit the state at hand.
#define SSM_LAUNCH(TT, L, M, X)                                                                                       \
  hipLaunchKernelGGL((ssm_scan_kernel<TT, L, M, X>), dim3(walks, H, (P + WAVE / L - 1) / (WAVE / L)), dim3(WAVE), 0, stream, \
                     (const TT*)xbc, xbc_stride, x_col, b_col, c_col, dt_raw, dt_stride, dt_bias, a_log, d_skip,      \
                     seq_slot, cu_rows, q_len, state, y, H, P, N, G, write_state, vec8, seg_cu, n_seqs, seg_rows,     \
                     seg_state, seg_decay)
#define SSM_CASE(TT, M, X, L) if (maxn == X && lpc == L) { SSM_LAUNCH(TT, L, M, X); } else
#define SSM_PICK(TT, M)                                                                                               \
  SSM_CASE(TT, M, 64, 1) SSM_CASE(TT, M, 64, 2) SSM_CASE(TT, M, 64, 4) SSM_CASE(TT, M, 64, 8)                         \
  SSM_CASE(TT, M, 128, 2) SSM_CASE(TT, M, 128, 4) SSM_CASE(TT, M, 128, 8) SSM_CASE(TT, M, 128, 16)                    \
  SSM_CASE(TT, M, 256, 4) SSM_CASE(TT, M, 256, 8) SSM_CASE(TT, M, 256, 16) { return -1; }
#define SSM_RUN(M) if (is_f32) { SSM_PICK(float, M) } else { SSM_PICK(bf16_t, M) }
  // a whole walk keeps to a wave a SIMD; segments, whose waves hold less, to two
  const int maxn = N > 128 ? 256 : (N > 64 ? 128 : 64);
  const int lpc = lanes_per_column(N, walks, H, P, cut ? 2048 : 1024);
  if (!cut) {
    SSM_RUN(0)
  } else {
    SSM_RUN(1)
    hipLaunchKernelGGL(ssm_carry_kernel, dim3(n_seqs, H, (N * P + 255) / 256), dim3(256), 0, stream, seq_slot, seg_cu,
                       state, seg_state, seg_decay, H, N * P);
    SSM_RUN(2)
  }
#undef SSM_RUN
#undef SSM_PICK
#undef SSM_CASE
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
