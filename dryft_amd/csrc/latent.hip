// Pieces around attention whose queries, keys and values come through low-rank latents: the norms of the two
// latents, the rotation with the append to the paged cache, and the gate per head.
#include "common.h"

// ---------------------------------------------------------------------------------------------------
// RMS norms over two runs of columns of one projection: out_a = rms(src[:, col : col + n_a]) * w_a and out_b the
// same for the n_b columns after them (n_b may be 0). Float statistics, plain weights. A workgroup a row.
template <typename T>
__global__ __launch_bounds__(256) void rms_segments_kernel(const T* __restrict__ src, int64_t stride, int col,
                                                           const float* __restrict__ w_a, T* __restrict__ out_a, int n_a,
                                                           const float* __restrict__ w_b, T* __restrict__ out_b, int n_b,
                                                           float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* x = src + row * stride + col;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < n_a; i += blockDim.x) { const float v = load_as_float(x + i); sa += v * v; }
  for (int i = threadIdx.x; i < n_b; i += blockDim.x) { const float v = load_as_float(x + n_a + i); sb += v * v; }
  sa = block_sum(sa, scratch);
  sb = block_sum(sb, scratch);
  const float ra = 1.f / sqrtf(sa / (float)n_a + eps), rb = n_b ? 1.f / sqrtf(sb / (float)n_b + eps) : 0.f;
  for (int i = threadIdx.x; i < n_a; i += blockDim.x)
    store_from_float(out_a + row * n_a + i, load_as_float(x + i) * ra * w_a[i]);
  for (int i = threadIdx.x; i < n_b; i += blockDim.x)
    store_from_float(out_b + row * n_b + i, load_as_float(x + n_a + i) * rb * w_b[i]);
}

DRYFT_API int dryft_rms_segments(const void* src, int64_t stride, int col, const float* w_a, void* out_a, int n_a,
                                 const float* w_b, void* out_b, int n_b, float eps, int rows, int is_f32,
                                 hipStream_t stream) {
  if (rows <= 0) return 0;
  if (n_a <= 0 || n_b < 0) return -1;
  if (is_f32)
    hipLaunchKernelGGL(rms_segments_kernel<float>, dim3(rows), dim3(256), 0, stream, (const float*)src, stride, col, w_a,
                       (float*)out_a, n_a, w_b, (float*)out_b, n_b, eps);
  else
    hipLaunchKernelGGL(rms_segments_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, (const bf16_t*)src, stride, col,
                       w_a, (bf16_t*)out_a, n_a, w_b, (bf16_t*)out_b, n_b, eps);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// Rotation and append. A query head is [plain | rotated part] of q_raw; a key head is that head's plain part from
// `kv` and the one rotated key part that all heads share, at column krot_col of `down`; a value head comes from
// `kv` after the keys. Of a rotated part's first `rot` features, feature i turns with feature i + rot/2:
//
//   o[i] = x[i] c - x[i + rot/2] s,   o[i + rot/2] = x[i + rot/2] c + x[i] s,   c, s = cos, sin of pos * f_i
//
// in float with float32 tables [positions, rot/2], rounded once; the rest passes. With `pairs` feature 2i turns
// with feature 2i + 1 instead (the same tables, angle i for pair i). Keys go to pages [64][key_dim],
// values transposed to pages [page_dv][64] in the kernels' column order (rows from value_dim on are never
// written and stay zero). One wave per (row, head) of q, k and v.
template <typename T>
__global__ __launch_bounds__(256) void latent_rope_kv_kernel(
    const T* __restrict__ q_raw, const T* __restrict__ kv, const T* __restrict__ down, int64_t down_stride, int krot_col,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, const int* __restrict__ row_slot,
    const int* __restrict__ row_pos, T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int* __restrict__ page_table, int max_pages, int write_kv, int n_heads, int plain, int rot_dim, int v_dim,
    int page_dv, int pairs) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t row = blockIdx.x;
  const int job = blockIdx.y * 4 + wave;
  if (job >= 3 * n_heads) return;
  const int kind = job / n_heads, head = job % n_heads, key_dim = plain + rot_dim;
  const int slot = row_slot[row], pos = row_pos[row];
  if (kind == 0 && slot < 0) {
    for (int i = lane; i < key_dim; i += WAVE) store_from_float(q_out + (row * n_heads + head) * key_dim + i, 0.f);
    return;
  }
  if (kind != 0 && (slot < 0 || !write_kv)) return;
  int page = 0, in_page = 0;
  if (kind != 0) {
    page = page_of(page_table, max_pages, slot, pos);
    in_page = pos % PAGE_TOKENS;
    if (page < 0) return;          // no page: the host reserves one before the step; never write through a bad index
  }
  if (kind == 2) {
    const T* src = kv + row * (int64_t)(n_heads * (plain + v_dim)) + (int64_t)n_heads * plain + (int64_t)head * v_dim;
    T* dst = v_pages + ((int64_t)page * n_heads + head) * page_dv * PAGE_TOKENS + value_column(in_page);
    for (int i = lane; i < v_dim; i += WAVE) dst[(int64_t)i * PAGE_TOKENS] = src[i];
    return;
  }
  T* dst = kind == 0 ? q_out + (row * n_heads + head) * key_dim
                     : k_pages + (((int64_t)page * n_heads + head) * PAGE_TOKENS + in_page) * key_dim;
  const T* src_plain = kind == 0 ? q_raw + (row * n_heads + head) * key_dim
                                 : kv + row * (int64_t)(n_heads * (plain + v_dim)) + (int64_t)head * plain;
  const T* src_rot = kind == 0 ? src_plain + plain : down + row * down_stride + krot_col;
  for (int i = lane; i < plain; i += WAVE) dst[i] = src_plain[i];
  const int half = rot / 2;
  for (int i = lane; i < half; i += WAVE) {
    const float c = cos_t[(int64_t)pos * half + i], s = sin_t[(int64_t)pos * half + i];
    const int ia = pairs ? 2 * i : i, ib = pairs ? 2 * i + 1 : half + i;
    const float a = load_as_float(src_rot + ia), b = load_as_float(src_rot + ib);
    store_from_float(dst + plain + ia, a * c - b * s);
    store_from_float(dst + plain + ib, b * c + a * s);
  }
  for (int i = rot + lane; i < rot_dim; i += WAVE) dst[plain + i] = src_rot[i];
}

DRYFT_API int dryft_latent_rope_kv(const void* q_raw, const void* kv, const void* down, int64_t down_stride, int krot_col,
                                   const float* cos_t, const float* sin_t, int rot, const int* row_slot,
                                   const int* row_pos, void* q_out, void* k_pages, void* v_pages, const int* page_table,
                                   int max_pages, int write_kv, int n_rows, int n_heads, int plain, int rot_dim, int v_dim,
                                   int page_dv, int pairs, int is_f32, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (rot < 0 || rot % 2 || rot > rot_dim || n_heads <= 0 || v_dim > page_dv) return -1;
  dim3 grid(n_rows, (3 * n_heads + 3) / 4), block(256);
  if (is_f32)
    hipLaunchKernelGGL(latent_rope_kv_kernel<float>, grid, block, 0, stream, (const float*)q_raw, (const float*)kv,
                       (const float*)down, down_stride, krot_col, cos_t, sin_t, rot, row_slot, row_pos, (float*)q_out,
                       (float*)k_pages, (float*)v_pages, page_table, max_pages, write_kv, n_heads, plain, rot_dim, v_dim,
                       page_dv, pairs);
  else
    hipLaunchKernelGGL(latent_rope_kv_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q_raw, (const bf16_t*)kv,
                       (const bf16_t*)down, down_stride, krot_col, cos_t, sin_t, rot, row_slot, row_pos, (bf16_t*)q_out,
                       (bf16_t*)k_pages, (bf16_t*)v_pages, page_table, max_pages, write_kv, n_heads, plain, rot_dim,
                       v_dim, page_dv, pairs);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// out[row, head, :v_dim] = attn[row, head, :v_dim] * sigmoid(gate[row, head]); the heads of `attn` may be wider
// than v_dim (in_dim), `out` is packed. The gate's logits are columns g_col.. of `down`: one per head, or with
// `per_element` one per output (head by head, v_dim each).
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(const T* __restrict__ attn, const T* __restrict__ down,
                                                        int64_t down_stride, int g_col, T* __restrict__ out,
                                                        int64_t total, int n_heads, int in_dim, int v_dim,
                                                        int per_element) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int j = idx % v_dim;
  const int64_t rh = idx / v_dim, row = rh / n_heads;
  const int head = rh % n_heads;
  const float g = load_as_float(down + row * down_stride + g_col + (per_element ? head * v_dim + j : head));
  store_from_float(out + idx, load_as_float(attn + rh * in_dim + j) / (1.f + expf(-g)));
}

DRYFT_API int dryft_head_gate(const void* attn, const void* down, int64_t down_stride, int g_col, void* out, int rows,
                              int n_heads, int in_dim, int v_dim, int per_element, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (v_dim > in_dim) return -1;
  const int64_t total = (int64_t)rows * n_heads * v_dim;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (is_f32)
    hipLaunchKernelGGL(head_gate_kernel<float>, grid, block, 0, stream, (const float*)attn, (const float*)down,
                       down_stride, g_col, (float*)out, total, n_heads, in_dim, v_dim, per_element);
  else
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)attn, (const bf16_t*)down,
                       down_stride, g_col, (bf16_t*)out, total, n_heads, in_dim, v_dim, per_element);
  return DRYFT_LAUNCH_CHECK();
}
