// A matrix state per head with a token-dependent decay (RWKV-style time mixing): the token shift, the decay, the
// recurrence token by token, and the read-out's norm and gate. Everything here is float arithmetic; T is the
// dtype of the projections around it.
#include "common.h"

#define WKV_MAX_DIM 256
#define WKV_BLENDS 5

// ---------------------------------------------------------------------------------------------------
// Token shift. With h' the row before (of the same sequence; the state `previous[slot]` for a sequence's first row
// of the step, which is zeros when the sequence starts), blend b is h + (h' - h) * mu[b], rounded once.
// out is [5, rows, width]. One workgroup a row.
template <typename T>
__global__ __launch_bounds__(256) void wkv_blend_kernel(const T* __restrict__ h, const float* __restrict__ previous,
                                                        const float* __restrict__ mu, const int* __restrict__ row_slot,
                                                        const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                                                        const int* __restrict__ seq_start, T* __restrict__ out, int rows,
                                                        int width) {
  const int64_t row = blockIdx.x;
  const int slot = row_slot[row];
  const bool first = slot < 0 || row_pos[row] == seq_start[row_seq[row]];
  const int64_t plane = (int64_t)rows * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float x = load_as_float(h + row * width + c);
    float p = 0.f;
    if (!first) p = load_as_float(h + (row - 1) * width + c);
    else if (slot >= 0) p = previous[(int64_t)slot * width + c];
    const float d = p - x;
#pragma unroll
    for (int b = 0; b < WKV_BLENDS; ++b) store_from_float(out + b * plane + row * width + c, x + d * mu[b * width + c]);
  }
}

DRYFT_API int dryft_wkv_blend(const void* h, const float* previous, const float* mu, const int* row_slot,
                              const int* row_seq, const int* row_pos, const int* seq_start, void* out, int rows,
                              int width, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (is_f32)
    hipLaunchKernelGGL(wkv_blend_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)h, previous, mu, row_slot,
                       row_seq, row_pos, seq_start, (float*)out, rows, width);
  else
    hipLaunchKernelGGL(wkv_blend_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)h, previous, mu,
                       row_slot, row_seq, row_pos, seq_start, (bf16_t*)out, rows, width);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The decay: w = exp(-exp(W_up tanh(low) + bias)), with `low` [rows, rank] the float accumulators of
// the first projection. R rows a workgroup share each weight row they read; a thread owns outputs n, n + 256, ...
template <typename W, int R>
__global__ __launch_bounds__(256) void wkv_decay_kernel(const float* __restrict__ low, const W* __restrict__ up,
                                                        const float* __restrict__ bias, float* __restrict__ decay,
                                                        int rows, int n_out, int rank) {
  extern __shared__ float t_low[];           // [R][rank]
  const int64_t row0 = (int64_t)blockIdx.x * R;
  for (int i = threadIdx.x; i < R * rank; i += blockDim.x) {
    const int64_t row = row0 + i / rank;
    t_low[i] = row < rows ? tanhf(low[row * rank + i % rank]) : 0.f;
  }
  __syncthreads();
  for (int n = blockIdx.y * blockDim.x + threadIdx.x; n < n_out; n += gridDim.y * blockDim.x) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    const W* w = up + (int64_t)n * rank;
    int j = 0;
    if (rank % 8 == 0 && ((uintptr_t)up & 15) == 0) {          // a row in 16-byte pieces
      for (; j < rank; j += 8) {
        float w8[8];
        load8_as_float(w + j, w8);
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r] += w8[e] * t_low[r * rank + j + e];
      }
    }
    for (; j < rank; ++j) {
      const float wj = load_as_float(w + j);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += wj * t_low[r * rank + j];
    }
    const float b = bias[n];
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (row0 + r < rows) decay[(row0 + r) * n_out + n] = expf(-expf(acc[r] + b));
  }
}

DRYFT_API int dryft_wkv_decay(const float* low, const void* up, const float* bias, float* decay, int rows, int n_out,
                              int rank, int up_is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (rank <= 0 || rank > 2048) return -1;
  if (rows >= 64) {
    const size_t lds = (size_t)8 * rank * sizeof(float);
    dim3 grid((rows + 7) / 8, 1);
    if (up_is_f32)
      hipLaunchKernelGGL((wkv_decay_kernel<float, 8>), grid, dim3(256), lds, stream, low, (const float*)up, bias, decay,
                         rows, n_out, rank);
    else
      hipLaunchKernelGGL((wkv_decay_kernel<bf16_t, 8>), grid, dim3(256), lds, stream, low, (const bf16_t*)up, bias, decay,
                         rows, n_out, rank);
  } else {
    const size_t lds = (size_t)rank * sizeof(float);
    dim3 grid(rows, (n_out + 255) / 256);          // few rows: a workgroup per 256 outputs, so that the chip has work
    if (up_is_f32)
      hipLaunchKernelGGL((wkv_decay_kernel<float, 1>), grid, dim3(256), lds, stream, low, (const float*)up, bias,
                         decay, rows, n_out, rank);
    else
      hipLaunchKernelGGL((wkv_decay_kernel<bf16_t, 1>), grid, dim3(256), lds, stream, low, (const bf16_t*)up, bias,
                         decay, rows, n_out, rank);
  }
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The recurrence, token by token. A workgroup of four waves takes 64 value columns of one (sequence, head), a wave 16
// of them. A lane keeps a tile of the state S [dim, dim] in registers: A = DK / 16 neighbouring key channels by four
// neighbouring columns (lane = 4 rg + cg: rows A rg .., columns 4 cg ..), so that per token it reads A values each of
// r, k and w and four of v from LDS for 4 A state entries (a lane that kept a whole column would read three values
// per entry, and LDS, not arithmetic, would bound the kernel). Per token
//
//   o_j = sum_i r_i S_ij + v_j sum_i r_i u_i k_i ;   S_ij <- w_i S_ij + k_i v_j
//
// A lane's four partial sums over its rows are added up over the wave's 16 row groups in five exchanges (halving
// what is exchanged twice, then plain sums), after which lane (rg = 0..3 by columns, cg) holds one column's sum.
// Sixteen tokens at a time go through LDS (r, k, w, v and the bonus sums, one number per token), and the next
// sixteen are on their way while these are computed. Wave 0 of head 0 also keeps the sequence's last input row as
// the next step's h' (`previous`), after every row of the step has been blended by the launch before.
#define WKV_GROUP 16

//
// Long prompts are cut into segments of `seg_rows` rows that run side by side (MODE 1, then the carry kernel, then
// MODE 2; MODE 0 walks a whole sequence). The recurrence is linear in the state, so a segment's effect on it is
// S_out = diag(P) S_in + L with P the product of the segment's decays per key channel and L the state it reaches from
// zero. MODE 1 computes L and P of every segment but a sequence's last (no outputs); the carry kernel walks a
// sequence's segments and leaves each the state that enters it; MODE 2 starts every segment from that state and
// writes its outputs, and a sequence's last segment writes the state back. Segment x of the step belongs to the
// sequence s with seg_cu[s] <= x < seg_cu[s + 1] (prefix sums over the sequences; one that sits out has none).
template <typename T, int DK, int MODE>
__global__ __launch_bounds__(256) void wkv_steps_kernel(const T* __restrict__ r, const T* __restrict__ k,
                                                        const T* __restrict__ v, const float* __restrict__ w,
                                                        const float* __restrict__ bonus, const int* __restrict__ seq_slot,
                                                        const int* __restrict__ cu_rows, const int* __restrict__ q_len,
                                                        float* __restrict__ state, float* __restrict__ o_raw,
                                                        const T* __restrict__ h, float* __restrict__ previous, int hidden,
                                                        int n_heads, int dim, int write_state,
                                                        const int* __restrict__ seg_cu, int n_seqs, int seg_rows,
                                                        float* __restrict__ seg_state, float* __restrict__ seg_decay) {
  constexpr int A = DK / 16;                      // key channels a lane keeps
  constexpr int NL = WKV_GROUP * DK / 256;        // elements of each of r, k, w that a thread brings in per group
  constexpr int NV = WKV_GROUP * 64 / 256;        // and of v
  __shared__ __attribute__((aligned(16))) float sh_r[WKV_GROUP][DK], sh_k[WKV_GROUP][DK], sh_w[WKV_GROUP][DK];
  __shared__ __attribute__((aligned(16))) float sh_v[WKV_GROUP][64], sh_u[DK], sh_b[WKV_GROUP];
  int seq = blockIdx.x, seg = 0, n_segs = 1;
  if (MODE != 0) {
    if ((int)blockIdx.x >= seg_cu[n_seqs]) return;
    seq = 0;
    while (seg_cu[seq + 1] <= (int)blockIdx.x) ++seq;
    seg = blockIdx.x - seg_cu[seq];
    n_segs = seg_cu[seq + 1] - seg_cu[seq];
    if (MODE == 1 && seg == n_segs - 1) return;                   // nobody needs the last segment's summary
  }
  const int head = blockIdx.y;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, rg = lane / 4, cg = lane % 4;
  const int col0 = blockIdx.z * 64;                               // the workgroup's first column
  const int slot = seq_slot[seq];
  const int row0 = cu_rows[seq] + seg * seg_rows;
  const int n = MODE == 0 ? q_len[seq] : min(seg_rows, q_len[seq] - seg * seg_rows);
  const int inner = n_heads * dim;
  if (slot < 0) {                      // a sequence that sits out: its rows of the output hold zeros
    for (int e = threadIdx.x; e < n * 64; e += 256)
      if (col0 + e % 64 < dim) o_raw[(int64_t)(row0 + e / 64) * inner + head * dim + col0 + e % 64] = 0.f;
    return;
  }
  if (n <= 0) return;
  const int my_col = col0 + 16 * wave + 4 * cg;                  // first of the lane's four columns
  float S[A][4], P[A];
  float* s_tile = state + (((int64_t)slot * n_heads + head) * dim + A * rg) * dim + my_col;
  float* seg_tile = MODE == 0 ? nullptr : seg_state + (((int64_t)blockIdx.x * n_heads + head) * dim + A * rg) * dim + my_col;
  const float* s_from = MODE == 2 ? seg_tile : s_tile;
#pragma unroll
  for (int e = 0; e < A; ++e) {
    P[e] = 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      S[e][j] = (MODE != 1 && A * rg + e < dim && my_col + j < dim) ? s_from[(int64_t)e * dim + j] : 0.f;
  }
  for (int i = threadIdx.x; i < DK; i += 256) sh_u[i] = i < dim ? bonus[head * dim + i] : 0.f;
  float nr[NL], nk[NL], nw[NL], nv[NV];
  auto fetch = [&](int t0) {
    const int g = min(WKV_GROUP, n - t0);
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int e = threadIdx.x + 256 * j, t = e / DK, i = e % DK;
      const bool in = t < g && i < dim;
      const int64_t at = (int64_t)(row0 + t0 + (in ? t : 0)) * inner + head * dim + (in ? i : 0);
      nr[j] = in ? load_as_float(r + at) : 0.f;
      nk[j] = in ? load_as_float(k + at) : 0.f;
      nw[j] = in ? w[at] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = threadIdx.x + 256 * j, t = e / 64, c = e % 64;
      const bool in = t < g && col0 + c < dim;
      nv[j] = in ? load_as_float(v + (int64_t)(row0 + t0 + t) * inner + head * dim + col0 + c) : 0.f;
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += WKV_GROUP) {
    const int g = min(WKV_GROUP, n - t0);
    __syncthreads();                   // the group before has been read
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int e = threadIdx.x + 256 * j;
      sh_r[e / DK][e % DK] = nr[j];
      sh_k[e / DK][e % DK] = nk[j];
      sh_w[e / DK][e % DK] = nw[j];
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = threadIdx.x + 256 * j;
      sh_v[e / 64][e % 64] = nv[j];
    }
    if (t0 + WKV_GROUP < n) fetch(t0 + WKV_GROUP);
    __syncthreads();
    for (int t = wave; MODE != 1 && t < g; t += 4) {             // the bonus sums, one number per token
      float b = 0.f;
      for (int i = lane; i < DK; i += WAVE) b += sh_r[t][i] * sh_u[i] * sh_k[t][i];
      b = wave_sum(b);
      if (lane == 0) sh_b[t] = b;
    }
    __syncthreads();
    // A token's partial sums need only LDS reads and multiply-adds; its exchanges between lanes are a chain of five
    // that waits on each step. So a full group first runs the multiply-adds of all its tokens and then the exchanges
    // of all of them, which do not depend on one another and overlap.
    auto token = [&](int t, float (&o)[4]) {
      float rr[A], kk[A], ww[A];
      if constexpr (A % 4 == 0) {
#pragma unroll
        for (int e = 0; e < A; e += 4) {
          const vf4 r4 = *(const vf4*)&sh_r[t][A * rg + e], k4 = *(const vf4*)&sh_k[t][A * rg + e];
          const vf4 w4 = *(const vf4*)&sh_w[t][A * rg + e];
#pragma unroll
          for (int x = 0; x < 4; ++x) { rr[e + x] = r4[x]; kk[e + x] = k4[x]; ww[e + x] = w4[x]; }
        }
      } else {
#pragma unroll
        for (int e = 0; e < A; ++e) { rr[e] = sh_r[t][A * rg + e]; kk[e] = sh_k[t][A * rg + e]; ww[e] = sh_w[t][A * rg + e]; }
      }
      const vf4 v4 = *(const vf4*)&sh_v[t][16 * wave + 4 * cg];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = 0.f;
#pragma unroll
      for (int e = 0; e < A; ++e)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (MODE != 1) o[j] += rr[e] * S[e][j];
          S[e][j] = ww[e] * S[e][j] + kk[e] * v4[j];
        }
      if (MODE == 1) {
#pragma unroll
        for (int e = 0; e < A; ++e) P[e] *= ww[e];
      }
    };
    const bool hi5 = lane & 32, hi4 = lane & 16;
    const int which = (hi5 ? 2 : 0) + (hi4 ? 1 : 0);             // the column of its four that a lane ends up holding
    auto reduce_store = [&](int t, const float (&o)[4]) {
      // over the 16 row groups (lane bits 2..5): send two and keep two, send one and keep one, then plain sums
      const float s0 = hi5 ? o[0] : o[2], s1 = hi5 ? o[1] : o[3];
      const float k0 = (hi5 ? o[2] : o[0]) + __shfl_xor(s0, 32, WAVE);
      const float k1 = (hi5 ? o[3] : o[1]) + __shfl_xor(s1, 32, WAVE);
      float sum = (hi4 ? k1 : k0) + __shfl_xor(hi4 ? k0 : k1, 16, WAVE);
      sum += __shfl_xor(sum, 8, WAVE);
      sum += __shfl_xor(sum, 4, WAVE);
      if ((lane & 12) == 0 && my_col + which < dim)
        o_raw[(int64_t)(row0 + t0 + t) * inner + head * dim + my_col + which] =
            sum + sh_v[t][16 * wave + 4 * cg + which] * sh_b[t];
    };
    if (MODE == 1) {
      for (int t = 0; t < g; ++t) {
        float o[4];
        token(t, o);
      }
    } else if (g == WKV_GROUP) {
      float op[WKV_GROUP][4];
#pragma unroll
      for (int t = 0; t < WKV_GROUP; ++t) token(t, op[t]);
#pragma unroll
      for (int t = 0; t < WKV_GROUP; ++t) reduce_store(t, op[t]);
    } else {
      for (int t = 0; t < g; ++t) {
        float o[4];
        token(t, o);
        reduce_store(t, o);
      }
    }
  }
  if (MODE == 1) {                     // the segment's summary: the state it reaches from zero, its decays' product
#pragma unroll
    for (int e = 0; e < A; ++e) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (A * rg + e < dim && my_col + j < dim) seg_tile[(int64_t)e * dim + j] = S[e][j];
      if (blockIdx.z == 0 && wave == 0 && cg == 0 && A * rg + e < dim)
        seg_decay[((int64_t)blockIdx.x * n_heads + head) * dim + A * rg + e] = P[e];
    }
    return;
  }
  if (MODE == 2 && seg != n_segs - 1) return;                     // the last segment leaves the sequence's state
  if (!write_state) return;
#pragma unroll
  for (int e = 0; e < A; ++e)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (A * rg + e < dim && my_col + j < dim) s_tile[(int64_t)e * dim + j] = S[e][j];
  if (head == 0 && blockIdx.z == 0 && wave == 0) {
    const T* last = h + (int64_t)(row0 + n - 1) * hidden;
    for (int cc = lane; cc < hidden; cc += WAVE) previous[(int64_t)slot * hidden + cc] = load_as_float(last + cc);
  }
}

// The state that enters each segment of a sequence: S_in[0] is the sequence's own state, S_in[s + 1] =
// diag(P[s]) S_in[s] + L[s]. One workgroup per (sequence, head, key channel), a thread a column; `seg_state` holds L
// on the way in and S_in on the way out.
__global__ __launch_bounds__(256) void wkv_carry_kernel(const int* __restrict__ seq_slot, const int* __restrict__ seg_cu,
                                                        const float* __restrict__ state, float* __restrict__ seg_state,
                                                        const float* __restrict__ seg_decay, int n_heads, int dim) {
  const int seq = blockIdx.x, head = blockIdx.y, slot = seq_slot[seq];
  const int x0 = seg_cu[seq], n_segs = seg_cu[seq + 1] - x0;
  if (slot < 0 || n_segs <= 0) return;
  for (int e = blockIdx.z * dim + threadIdx.x; e < (blockIdx.z + 1) * dim; e += blockDim.x) {
    float run = state[((int64_t)slot * n_heads + head) * dim * dim + e];
    for (int s = 0; s < n_segs; ++s) {
      float* at = seg_state + ((int64_t)(x0 + s) * n_heads + head) * dim * dim + e;
      const float local = *at;
      *at = run;
      if (s + 1 < n_segs) run = seg_decay[((int64_t)(x0 + s) * n_heads + head) * dim + e / dim] * run + local;
    }
  }
}

template <typename T, int MODE>
static int launch_wkv_steps(hipStream_t stream, const void* r, const void* k, const void* v, const float* w,
                            const float* bonus, const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs,
                            float* state, float* o_raw, const void* h, float* previous, int hidden, int n_heads, int dim,
                            int write_state, const int* seg_cu, int max_segs, int seg_rows, float* seg_state,
                            float* seg_decay) {
  dim3 grid(MODE == 0 ? n_seqs : max_segs, n_heads, (dim + 63) / 64), block(256);
#define WKV_CASE(DK)                                                                                               \
  hipLaunchKernelGGL((wkv_steps_kernel<T, DK, MODE>), grid, block, 0, stream, (const T*)r, (const T*)k, (const T*)v, \
                     w, bonus, seq_slot, cu_rows, q_len, state, o_raw, (const T*)h, previous, hidden, n_heads, dim,  \
                     write_state, seg_cu, n_seqs, seg_rows, seg_state, seg_decay)
  if (dim <= 16) WKV_CASE(16);
  else if (dim <= 32) WKV_CASE(32);
  else if (dim <= 64) WKV_CASE(64);
  else if (dim <= 128) WKV_CASE(128);
  else WKV_CASE(256);
#undef WKV_CASE
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_wkv_max_dim() { return WKV_MAX_DIM; }

DRYFT_API int dryft_wkv_steps(const void* r, const void* k, const void* v, const float* decay, const float* bonus,
                              const int* seq_slot, const int* cu_rows, const int* q_len, int n_seqs, float* state,
                              float* o_raw, const void* h, float* previous, int hidden, int n_heads, int dim,
                              int write_state, const int* seg_cu, int max_segs, int seg_rows, float* seg_state,
                              float* seg_decay, int is_f32, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (dim <= 0 || dim > WKV_MAX_DIM || n_heads <= 0 || n_heads > 65535) return -1;
#define WKV_RUN(T, MODE)                                                                                           \
  launch_wkv_steps<T, MODE>(stream, r, k, v, decay, bonus, seq_slot, cu_rows, q_len, n_seqs, state, o_raw, h, previous, \
                            hidden, n_heads, dim, write_state, seg_cu, max_segs, seg_rows, seg_state, seg_decay)
  if (seg_cu == nullptr) return is_f32 ? WKV_RUN(float, 0) : WKV_RUN(bf16_t, 0);
  if (max_segs <= 0) return 0;
  if (seg_rows <= 0 || seg_rows % WKV_GROUP || seg_state == nullptr || seg_decay == nullptr) return -1;
  int rc = is_f32 ? WKV_RUN(float, 1) : WKV_RUN(bf16_t, 1);
  if (rc) return rc;
  hipLaunchKernelGGL(wkv_carry_kernel, dim3(n_seqs, n_heads, dim), dim3(dim <= 64 ? 64 : 256), 0, stream, seq_slot, seg_cu, state, seg_state,
                     seg_decay, n_heads, dim);
  rc = DRYFT_LAUNCH_CHECK();
  if (rc) return rc;
  return is_f32 ? WKV_RUN(float, 2) : WKV_RUN(bf16_t, 2);
#undef WKV_RUN
}

// ---------------------------------------------------------------------------------------------------
// Read-out: out = o / sqrt(mean_head(o^2) + eps) * weight * silu(gate), one wave per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void wkv_out_kernel(const float* __restrict__ o_raw, const T* __restrict__ gate,
                                                      const float* __restrict__ weight, T* __restrict__ out, int rows,
                                                      int n_heads, int dim, float eps, int64_t gate_stride) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t job = (int64_t)blockIdx.x * 4 + wave;
  if (job >= (int64_t)rows * n_heads) return;
  const int head = job % n_heads;
  const int64_t at = job * dim;
  gate += (job / n_heads) * gate_stride + (int64_t)head * dim - at;      // the gate's rows may be a run of columns
  float ss = 0.f;
  for (int i = lane; i < dim; i += WAVE) { const float o = o_raw[at + i]; ss += o * o; }
  ss = wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)dim + eps);
  for (int i = lane; i < dim; i += WAVE) {
    const float g = load_as_float(gate + at + i);
    store_from_float(out + at + i, o_raw[at + i] * rinv * weight[head * dim + i] * (g / (1.f + expf(-g))));
  }
}

DRYFT_API int dryft_wkv_out(const float* o_raw, const void* gate, const float* weight, void* out, int rows, int n_heads,
                            int dim, float eps, int64_t gate_stride, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  const int64_t jobs = (int64_t)rows * n_heads;
  dim3 grid((unsigned)((jobs + 3) / 4)), block(256);
  if (is_f32)
    hipLaunchKernelGGL(wkv_out_kernel<float>, grid, block, 0, stream, o_raw, (const float*)gate, weight, (float*)out, rows,
                       n_heads, dim, eps, gate_stride);
  else
    hipLaunchKernelGGL(wkv_out_kernel<bf16_t>, grid, block, 0, stream, o_raw, (const bf16_t*)gate, weight, (bf16_t*)out,
                       rows, n_heads, dim, eps, gate_stride);
  return DRYFT_LAUNCH_CHECK();
}
