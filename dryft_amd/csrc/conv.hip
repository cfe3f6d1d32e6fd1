// A short causal convolution over time on every channel of a projection, with the sequence's last inputs kept as
// state so that a prompt, a portion of one and a single token are the same code.
//
//   y[t, c] = act( sum_j w[c, j] * u[t - taps + 1 + j, c] + b[c] ),      u = projection (+ its own bias)
//
// with zeros before a sequence's start. The inputs of the `taps - 1` positions before this step's rows come from
// `tail [slots, taps - 1, C]` (float32, zero for a sequence that starts); a second kernel moves the tail on once
// every row has read it. All arithmetic is float; y is rounded once.
#include "common.h"

#define CONV_MAX_TAPS 16

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const T* __restrict__ u, int64_t u_stride, int col,
                                                          const float* __restrict__ in_bias,
                                                          const float* __restrict__ w, const float* __restrict__ out_bias,
                                                          int taps, int act, const int* __restrict__ row_slot,
                                                          const int* __restrict__ row_seq,
                                                          const int* __restrict__ row_pos,
                                                          const int* __restrict__ seq_start,
                                                          const float* __restrict__ tail, T* __restrict__ out, int C) {
  const int64_t row = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = row_slot[row];
  if (slot < 0) {
    store_from_float(out + row * C + c, 0.f);
    return;
  }
  const int pos = row_pos[row], start = seq_start[row_seq[row]];
  const float ib = in_bias ? in_bias[c] : 0.f;
  float acc = out_bias ? out_bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j, p = pos - d;
    float v = 0.f;
    if (p >= start) v = load_as_float(u + (row - d) * u_stride + col + c) + ib;
    else if (p >= 0 && tail != nullptr) v = tail[((int64_t)slot * (taps - 1) + (p - start + taps - 1)) * C + c];
    acc += w[(int64_t)c * taps + j] * v;
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  store_from_float(out + row * C + c, acc);
}

// The same for eight neighbouring channels a thread, read and written 16 bytes at a time, with the weights tap by tap
// (`w_t [taps, C]`): for inputs, outputs and tails whose rows start at multiples of 8 channels.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(const T* __restrict__ u, int64_t u_stride, int col,
                                                              const float* __restrict__ in_bias,
                                                              const float* __restrict__ w_t,
                                                              const float* __restrict__ out_bias, int taps, int act,
                                                              const int* __restrict__ row_slot,
                                                              const int* __restrict__ row_seq,
                                                              const int* __restrict__ row_pos,
                                                              const int* __restrict__ seq_start,
                                                              const float* __restrict__ tail, T* __restrict__ out, int C) {
  const int64_t row = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= C) return;
  const int slot = row_slot[row];
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (slot < 0) {
    store8_from_float(out + row * C + c, acc);
    return;
  }
  const int pos = row_pos[row], start = seq_start[row_seq[row]];
  float ib[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (in_bias) load8_as_float(in_bias + c, ib);
  if (out_bias) load8_as_float(out_bias + c, acc);
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j, p = pos - d;
    float v[8], wj[8];
    if (p >= start) {
      load8_as_float(u + (row - d) * u_stride + col + c, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] += ib[i];
    } else if (p >= 0 && tail != nullptr) {
      load8_as_float(tail + ((int64_t)slot * (taps - 1) + (p - start + taps - 1)) * C + c, v);
    } else {
      continue;
    }
    load8_as_float(w_t + (int64_t)j * C + c, wj);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += wj[i] * v[i];
  }
  if (act == 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = acc[i] / (1.f + expf(-acc[i]));
  }
  store8_from_float(out + row * C + c, acc);
}

// The tail after the step: the last taps - 1 inputs of each sequence, from this step's rows and, where the step
// brought fewer, from the tail before. A thread owns one (sequence, channel) and reads everything before it writes.
template <typename T>
__global__ __launch_bounds__(256) void conv_tail_kernel(const T* __restrict__ u, int64_t u_stride, int col,
                                                        const float* __restrict__ in_bias, int taps,
                                                        const int* __restrict__ seq_slot,
                                                        const int* __restrict__ cu_rows, const int* __restrict__ q_len,
                                                        float* __restrict__ tail, int C) {
  const int seq = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int slot = seq_slot[seq], q = q_len[seq];
  if (c >= C || slot < 0 || q <= 0) return;
  const int keep = taps - 1;
  const int64_t first = cu_rows[seq];
  const float ib = in_bias ? in_bias[c] : 0.f;
  float* mine = tail + (int64_t)slot * keep * C + c;
  float v[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) {
    if (j < keep) {
      const int r = q - keep + j;             // the step's row that lands in place j, if it has one
      v[j] = r >= 0 ? load_as_float(u + (first + r) * u_stride + col + c) + ib : mine[(int64_t)(j + q) * C];
    }
  }
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
    if (j < keep) mine[(int64_t)j * C] = v[j];
}

DRYFT_API int dryft_conv_max_taps() { return CONV_MAX_TAPS; }

DRYFT_API int dryft_causal_conv(const void* u, int64_t u_stride, int col, const float* in_bias, const float* w,
                                const float* w_t, const float* out_bias, int taps, int act, const int* row_slot,
                                const int* row_seq, const int* row_pos, const int* seq_start, const float* tail, void* out,
                                int n_rows, int C, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (taps < 1 || taps > CONV_MAX_TAPS || C <= 0 || (taps > 1 && tail == nullptr)) return -1;
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  // steps of few rows keep the kernel of a channel a thread: eight times the threads for the same few loads each
  if (n_rows >= 32 && w_t != nullptr && C % 8 == 0 && col % 8 == 0 && u_stride % 8 == 0 && aligned(u) && aligned(out) && aligned(w_t) &&
      aligned(tail) && aligned(in_bias) && aligned(out_bias)) {
    dim3 grid(n_rows, (C / 8 + 255) / 256), block(256);
    if (is_f32)
      hipLaunchKernelGGL(causal_conv_vec_kernel<float>, grid, block, 0, stream, (const float*)u, u_stride, col, in_bias,
                         w_t, out_bias, taps, act, row_slot, row_seq, row_pos, seq_start, tail, (float*)out, C);
    else
      hipLaunchKernelGGL(causal_conv_vec_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)u, u_stride, col, in_bias,
                         w_t, out_bias, taps, act, row_slot, row_seq, row_pos, seq_start, tail, (bf16_t*)out, C);
    return DRYFT_LAUNCH_CHECK();
  }
  dim3 grid(n_rows, (C + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(causal_conv_kernel<float>, grid, block, 0, stream, (const float*)u, u_stride, col, in_bias, w,
                       out_bias, taps, act, row_slot, row_seq, row_pos, seq_start, tail, (float*)out, C);
  else
    hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)u, u_stride, col, in_bias, w,
                       out_bias, taps, act, row_slot, row_seq, row_pos, seq_start, tail, (bf16_t*)out, C);
  return DRYFT_LAUNCH_CHECK();
}

DRYFT_API int dryft_conv_tail(const void* u, int64_t u_stride, int col, const float* in_bias, int taps,
                              const int* seq_slot, const int* cu_rows, const int* q_len, float* tail, int n_seqs, int C,
                              int is_f32, hipStream_t stream) {
  if (n_seqs <= 0 || taps <= 1) return 0;
  if (taps > CONV_MAX_TAPS || C <= 0 || tail == nullptr) return -1;
  dim3 grid(n_seqs, (C + 255) / 256), block(256);
  if (is_f32)
    hipLaunchKernelGGL(conv_tail_kernel<float>, grid, block, 0, stream, (const float*)u, u_stride, col, in_bias, taps,
                       seq_slot, cu_rows, q_len, tail, C);
  else
    hipLaunchKernelGGL(conv_tail_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)u, u_stride, col, in_bias, taps,
                       seq_slot, cu_rows, q_len, tail, C);
  return DRYFT_LAUNCH_CHECK();
}
