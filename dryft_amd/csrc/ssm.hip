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
// registers of LPC lanes (N / LPC rows each, at most 64), so that a token's sum over N is a sum inside a thread plus
// one or two lane exchanges, with no barrier. B and C of a token are the same for every column: they wait in LDS,
// read as 16-byte broadcasts. Operands come in batches of eight tokens; the next batch's loads are in flight while
// the wave walks the current one.
#include "common.h"

#define SSM_MAX_STATE 256
#define SSM_BATCH 8              // tokens whose operands are brought into LDS together
#define SSM_ROWS 64              // rows of a column a lane holds at most

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, int LPC>
__global__ __launch_bounds__(WAVE) void ssm_scan_kernel(
    const T* __restrict__ xbc, int64_t xbc_stride, int x_col, int b_col, int c_col, const float* __restrict__ dt_raw,
    int64_t dt_stride, const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
    const int* __restrict__ seq_slot, const int* __restrict__ cu_rows, const int* __restrict__ q_len,
    float* __restrict__ state, float* __restrict__ y, int H, int P, int N, int G, int write_state) {
  constexpr int CW = WAVE / LPC;                       // columns a wave owns
  constexpr int ROWS = SSM_MAX_STATE / LPC < SSM_ROWS ? SSM_MAX_STATE / LPC : SSM_ROWS;   // rows of a column a lane holds at most
  constexpr int R4 = ROWS / 4;
  constexpr int PER = SSM_MAX_STATE / 4;               // values of a B or C vector one of its four lanes takes at most
  // a vector in LDS: LPC runs of `rdp` floats (the rows of one lane), padded to a multiple of 4 with zeros
  __shared__ __attribute__((aligned(16))) float sB[SSM_BATCH][SSM_MAX_STATE + 4 * LPC];
  __shared__ __attribute__((aligned(16))) float sC[SSM_BATCH][SSM_MAX_STATE + 4 * LPC];
  __shared__ float sx[SSM_BATCH][CW], sdt[SSM_BATCH], sa[SSM_BATCH];
  const int seq = blockIdx.x, head = blockIdx.y, p0 = blockIdx.z * CW;
  const int slot = seq_slot[seq], rows = q_len[seq];
  if (slot < 0 || rows <= 0) return;
  const int64_t first = cu_rows[seq];
  const int group = head / (H / G);
  const int lane = threadIdx.x, col = lane % CW, sub = lane / CW;
  const bool live = p0 + col < P;
  const int rd = (N + LPC - 1) / LPC, rd4 = (rd + 3) / 4, rdp = 4 * rd4;
  float* mine = state + (((int64_t)slot * H + head) * N) * P + p0 + col;
  float S[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int n = sub * rd + i;
    S[i] = (live && i < rd && n < N) ? mine[(int64_t)n * P] : 0.f;
  }
  const float rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
  // the batch's loads: lane l takes part (l % 4) of vector (l / 4): token (l / 8), B or C ((l / 4) % 2)
  const int vec = lane / 4, part = lane % 4, v_tok = vec >> 1, v_is_c = vec & 1;
  const int per = (N + 3) / 4;
  float bc[PER], xv[SSM_BATCH * CW / WAVE], dtr = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(SSM_BATCH, rows - t0);
    if (v_tok < nb) {
      const T* src = xbc + (first + t0 + v_tok) * xbc_stride + (v_is_c ? c_col : b_col) + group * N + part * per;
#pragma unroll
      for (int i = 0; i < PER; ++i) bc[i] = (i < per && part * per + i < N) ? load_as_float(src + i) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < SSM_BATCH * CW / WAVE; ++j) {
      const int idx = lane + j * WAVE, tt = idx / CW, pp = idx % CW;
      xv[j] = (tt < nb && p0 + pp < P) ? load_as_float(xbc + (first + t0 + tt) * xbc_stride + x_col + head * P + p0 + pp) : 0.f;
    }
    if (lane < nb) dtr = dt_raw[(first + t0 + lane) * dt_stride + head];
  };
  auto stage = [&](int t0) {
    const int nb = min(SSM_BATCH, rows - t0);
    if (v_tok < nb) {
      float* dst = v_is_c ? sC[v_tok] : sB[v_tok];
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int n = part * per + i;
        if (i < per && n < N) dst[(n / rd) * rdp + n % rd] = bc[i];
      }
    }
#pragma unroll
    for (int j = 0; j < SSM_BATCH * CW / WAVE; ++j) {
      const int idx = lane + j * WAVE;
      sx[idx / CW][idx % CW] = xv[j];
    }
    if (lane < nb) {
      const float dt = softplus_f(dtr + bias);
      sdt[lane] = dt;
      sa[lane] = expf(-rate * dt);
    }
  };
  // the padding of every run stays zero for good
  for (int i = lane; i < SSM_BATCH * (SSM_MAX_STATE + 4 * LPC); i += WAVE) { (&sB[0][0])[i] = 0.f; (&sC[0][0])[i] = 0.f; }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  __builtin_amdgcn_wave_barrier();
  fetch(0);
  for (int t0 = 0; t0 < rows; t0 += SSM_BATCH) {
    const int nb = min(SSM_BATCH, rows - t0);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");      // the walk over the batch before is done with LDS
    __builtin_amdgcn_wave_barrier();
    stage(t0);
    if (t0 + SSM_BATCH < rows) fetch(t0 + SSM_BATCH);
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    __builtin_amdgcn_wave_barrier();
    for (int tt = 0; tt < nb; ++tt) {
      const float a = sa[tt], x = sx[tt][col], dtx = sdt[tt] * x;
      const vf4* bp = (const vf4*)(sB[tt] + sub * rdp);
      const vf4* cp = (const vf4*)(sC[tt] + sub * rdp);
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
#pragma unroll
      for (int o = CW; o < WAVE; o <<= 1) acc += __shfl_xor(acc, o, WAVE);
      if (sub == 0 && live) y[(first + t0 + tt) * (int64_t)(H * P) + head * P + p0 + col] = acc + skip * x;
    }
  }
  if (write_state && live) {
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int n = sub * rd + i;
      if (i < rd && n < N) mine[(int64_t)n * P] = S[i];
    }
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
#define SSM_LAUNCH(TT, L)                                                                                             \
  hipLaunchKernelGGL((ssm_scan_kernel<TT, L>), dim3(n_seqs, H, (P + WAVE / L - 1) / (WAVE / L)), dim3(WAVE), 0, stream, \
                     (const TT*)xbc, xbc_stride, x_col, b_col, c_col, dt_raw, dt_stride, dt_bias, a_log, d_skip,      \
                     seq_slot, cu_rows, q_len, state, y, H, P, N, G, write_state)
  // lanes a column: as few as hold its rows (64 each), and no more columns a wave than the head has
  int lpc = N > 128 ? 4 : (N > 64 ? 2 : 1);
  while (lpc < 4 && WAVE / lpc > P && WAVE / (2 * lpc) >= 8) lpc *= 2;
  if (is_f32) {
    if (lpc == 4) SSM_LAUNCH(float, 4); else if (lpc == 2) SSM_LAUNCH(float, 2); else SSM_LAUNCH(float, 1);
  } else {
    if (lpc == 4) SSM_LAUNCH(bf16_t, 4); else if (lpc == 2) SSM_LAUNCH(bf16_t, 2); else SSM_LAUNCH(bf16_t, 1);
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
