// Routed experts on the device: the router's choice, the sort of (row, expert) pairs by expert, the grouped
// products over each expert's rows, and the weighted sum per row. No step of it needs the host, so a step that
// holds it can be captured.
#include "common.h"

#define MOE_MAX_EXPERTS 512
#define MOE_PER_LANE (MOE_MAX_EXPERTS / WAVE)
#define MOE_TILE 64            // pairs of one expert that a workgroup of the products takes

struct Best {
  float v;
  int i;
};

// The larger value; of equal values the lower index.
__device__ __forceinline__ Best wave_best(Best b) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const float v = __shfl_xor(b.v, o, WAVE);
    const int i = __shfl_xor(b.i, o, WAVE);
    if (v > b.v || (v == b.v && i < b.i)) { b.v = v; b.i = i; }
  }
  return b;
}

// ---------------------------------------------------------------------------------------------------
// Router. s = sigmoid(z); choice = s + correction. Experts form `groups` equal groups of neighbours; a group's
// score is the sum of its two largest choice scores (of its only one, if it has one); experts outside the `keep`
// best groups drop out. The `top` largest choice scores that remain are chosen, highest first, and weigh
// s / (sum of the chosen s + 1e-20) * scale. One wave a row; lane l holds experts l, l + 64, ...
// Other forms: `softmax` takes s = softmax(z) over all experts instead of the sigmoid; no correction (null): the
// choice scores are s itself; `group_best`: a group scores as its single largest choice score; without `renorm`
// the weights are s * scale as they are.
template <int PER>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int64_t stride,
                                                        const float* __restrict__ correction, int n_experts, int groups,
                                                        int keep, int top, float scale, int* __restrict__ chosen,
                                                        float* __restrict__ weights, int rows, int softmax,
                                                        int group_best, int renorm) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const float NEG = -__builtin_inff();
  float s[PER], c[PER];
  float z_max = NEG, z_sum = 0.f;
  if (softmax) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + WAVE * j;
      if (e < n_experts) z_max = fmaxf(z_max, logits[row * stride + e]);
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) z_max = fmaxf(z_max, __shfl_xor(z_max, o, WAVE));
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + WAVE * j;
      s[j] = e < n_experts ? expf(logits[row * stride + e] - z_max) : 0.f;
      z_sum += s[j];
    }
    z_sum = wave_sum(z_sum);
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + WAVE * j;
    if (!softmax) s[j] = 0.f;
    c[j] = NEG;
    if (e < n_experts) {
      s[j] = softmax ? s[j] / z_sum : 1.f / (1.f + expf(-logits[row * stride + e]));
      c[j] = s[j] + (correction != nullptr ? correction[e] : 0.f);
    }
  }
  if (keep < groups) {
    const int size = n_experts / groups;
    float score = NEG;               // lane g holds group g's score
    for (int g = 0; g < groups; ++g) {
      Best a{NEG, 0x7fffffff};
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const int e = lane + WAVE * j;
        if (e < n_experts && e / size == g && (c[j] > a.v || (c[j] == a.v && e < a.i))) { a.v = c[j]; a.i = e; }
      }
      a = wave_best(a);
      float sum = a.v;
      if (size >= 2 && !group_best) {
        Best b{NEG, 0x7fffffff};
#pragma unroll
        for (int j = 0; j < PER; ++j) {
          const int e = lane + WAVE * j;
          if (e < n_experts && e / size == g && e != a.i && (c[j] > b.v || (c[j] == b.v && e < b.i))) { b.v = c[j]; b.i = e; }
        }
        b = wave_best(b);
        sum += b.v;
      }
      if (lane == g) score = sum;
    }
    uint64_t kept = 0;
    for (int i = 0; i < keep; ++i) {
      Best a{(lane < groups && !((kept >> lane) & 1)) ? score : NEG, lane < groups ? lane : 0x7fffffff};
      if (lane < groups && ((kept >> lane) & 1)) a.i = 0x7fffffff;
      a = wave_best(a);
      if (a.i < groups) kept |= 1ull << a.i;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + WAVE * j;
      if (e < n_experts && !((kept >> (e / size)) & 1)) c[j] = NEG;
    }
  }
  float total = 0.f;
  for (int i = 0; i < top; ++i) {
    Best a{NEG, 0x7fffffff};
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = lane + WAVE * j;
      if (e < n_experts && (c[j] > a.v || (c[j] == a.v && e < a.i))) { a.v = c[j]; a.i = e; }
    }
    a = wave_best(a);
    float sv = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (lane + WAVE * j == a.i) { sv = s[j]; c[j] = NEG; }
    sv = wave_sum(sv);
    total += sv;
    if (lane == 0) {
      chosen[row * top + i] = a.i;
      weights[row * top + i] = sv;       // divided below
    }
  }
  if (lane == 0)       // the same lane wrote them
    for (int i = 0; i < top; ++i)
      weights[row * top + i] = renorm ? weights[row * top + i] / (total + 1e-20f) * scale : weights[row * top + i] * scale;
}

DRYFT_API int dryft_moe_max_experts() { return MOE_MAX_EXPERTS; }
DRYFT_API int dryft_moe_tile() { return MOE_TILE; }

DRYFT_API int dryft_moe_route(const float* logits, int64_t stride, const float* correction, int n_experts, int groups,
                              int keep, int top, float scale, int* chosen, float* weights, int rows, int softmax,
                              int group_best, int renorm, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (n_experts < 1 || n_experts > MOE_MAX_EXPERTS || top < 1 || top > n_experts || groups < 1 || groups > WAVE ||
      n_experts % groups || keep < 1 || keep > groups || keep * (n_experts / groups) < top)
    return -1;
#define MOE_ROUTE(PER)                                                                                              \
  hipLaunchKernelGGL(moe_route_kernel<PER>, dim3((rows + 3) / 4), dim3(256), 0, stream, logits, stride, correction,   \
                     n_experts, groups, keep, top, scale, chosen, weights, rows, softmax, group_best, renorm)
  if (n_experts <= WAVE) MOE_ROUTE(1);
  else if (n_experts <= 2 * WAVE) MOE_ROUTE(2);
  else MOE_ROUTE(MOE_PER_LANE);
#undef MOE_ROUTE
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// The plan of a step: pairs (row, k) sorted by expert (`sorted_pair`: place -> pair, `place_of`: pair -> place),
// every expert's run of places cut into tiles of MOE_TILE. One workgroup. Which place a pair gets within its
// expert's run depends on the order in which threads arrive; no result depends on it, since every pair's
// outputs are computed from its own row alone, in a fixed order.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ chosen, int n_pairs, int n_experts,
                                                        int* __restrict__ sorted_pair, int* __restrict__ place_of,
                                                        int* __restrict__ tile_expert, int* __restrict__ tile_start,
                                                        int* __restrict__ tile_rows, int* __restrict__ n_tiles,
                                                        int max_tiles) {
  __shared__ int counts[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) atomicAdd(&counts[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < n_experts; ++e) {
      cursor[e] = at;
      for (int s = 0; s < counts[e] && nt < max_tiles; s += MOE_TILE) {
        tile_expert[nt] = e;
        tile_start[nt] = at + s;
        tile_rows[nt] = min(MOE_TILE, counts[e] - s);
        ++nt;
      }
      at += counts[e];
    }
    *n_tiles = nt;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
    const int place = atomicAdd(&cursor[chosen[p]], 1);
    sorted_pair[place] = p;
    place_of[p] = place;
  }
}

DRYFT_API int dryft_moe_plan(const int* chosen, int n_pairs, int n_experts, int* sorted_pair, int* place_of,
                             int* tile_expert, int* tile_start, int* tile_rows, int* n_tiles, int max_tiles,
                             hipStream_t stream) {
  if (n_pairs <= 0) return 0;
  if (n_experts < 1 || n_experts > MOE_MAX_EXPERTS) return -1;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, chosen, n_pairs, n_experts, sorted_pair, place_of,
                     tile_expert, tile_start, tile_rows, n_tiles, max_tiles);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// A router that is a table: row r's experts are the `top` entries of the table's row of its token id, each with
// weight 1 / top.
__global__ __launch_bounds__(256) void moe_table_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table,
                                                              int* __restrict__ chosen, float* __restrict__ weights,
                                                              int n_pairs, int top, int vocab, int n_experts) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_pairs) return;
  const int tok = min(max(tokens[i / top], 0), vocab - 1);
  chosen[i] = min(max(table[(int64_t)tok * top + i % top], 0), n_experts - 1);
  weights[i] = 1.f / (float)top;
}

DRYFT_API int dryft_moe_table_route(const int* tokens, const int* table, int* chosen, float* weights, int rows, int top,
                                    int vocab, int n_experts, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (top <= 0 || vocab <= 0 || n_experts <= 0) return -1;
  const int n = rows * top;
  hipLaunchKernelGGL(moe_table_route_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, tokens, table, chosen, weights,
                     n, top, vocab, n_experts);
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// Grouped product, plain multiply-adds: for every tile of an expert's places, out[place] = W_e a[place]. A
// workgroup takes one tile (up to 64 places) and 64 outputs; K goes through LDS 32 at a time; a thread owns four
// places and four outputs. With `top` > 0 the operand rows are gathered: place -> pair -> row pair / top of `a`;
// otherwise `a` is already in place order. GLU: W_e holds gate rows then up rows; the clamped gated unit
// g * sigmoid(alpha g) * (u + offset), g = min(gate, limit), u = clamp(up, -limit, limit) (offset 0, alpha 1 and an
// infinite limit make it silu(gate) * up), is applied to the float
// accumulators and `n_out` counts its outputs. Without a gate, `act` = 1 stores the square of relu of the product
// (as it would have been stored in the activation dtype) instead of the product.
#define MOE_TN 64
#define MOE_TK 32

template <typename T, typename O, bool GLU>
__global__ __launch_bounds__(256) void moe_product_kernel(const T* __restrict__ a, int64_t a_stride,
                                                          const T* __restrict__ w, const int* __restrict__ sorted_pair,
                                                          const int* __restrict__ tile_expert,
                                                          const int* __restrict__ tile_start,
                                                          const int* __restrict__ tile_rows,
                                                          const int* __restrict__ n_tiles, O* __restrict__ out, int top,
                                                          int n_out, int k_dim, float limit, float alpha, float offset, int act) {
  __shared__ float sa[MOE_TILE][MOE_TK + 1];
  __shared__ float sw[(GLU ? 2 : 1) * MOE_TN][MOE_TK + 1];
  __shared__ int src_row[MOE_TILE];
  const int tile = blockIdx.x;
  if (tile >= *n_tiles) return;
  const int expert = tile_expert[tile], start = tile_start[tile], count = tile_rows[tile];
  const int n0 = blockIdx.y * MOE_TN;
  const int w_rows = GLU ? 2 * n_out : n_out;
  const T* we = w + (int64_t)expert * w_rows * k_dim;
  if (threadIdx.x < MOE_TILE)
    src_row[threadIdx.x] = threadIdx.x < count ? (top > 0 ? sorted_pair[start + threadIdx.x] / top : start + threadIdx.x) : -1;
  const int ty = threadIdx.x / 16, tx = threadIdx.x % 16;      // places ty + 16 i; outputs tx + 16 j
  constexpr int PM = MOE_TILE / 16;
  float acc[PM][4], acc_up[PM][4];
#pragma unroll
  for (int i = 0; i < PM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = acc_up[i][j] = 0.f;
  for (int k0 = 0; k0 < k_dim; k0 += MOE_TK) {
    __syncthreads();
    for (int e = threadIdx.x; e < MOE_TILE * MOE_TK; e += 256) {
      const int r = e / MOE_TK, kk = e % MOE_TK;
      const int row = src_row[r];
      sa[r][kk] = (row >= 0 && k0 + kk < k_dim) ? load_as_float(a + (int64_t)row * a_stride + k0 + kk) : 0.f;
    }
    for (int e = threadIdx.x; e < (GLU ? 2 : 1) * MOE_TN * MOE_TK; e += 256) {
      const int r = e / MOE_TK, kk = e % MOE_TK;
      const int n = n0 + r % MOE_TN;
      const int64_t w_row = (GLU && r >= MOE_TN) ? (int64_t)n_out + n : n;
      sw[r][kk] = (n < n_out && k0 + kk < k_dim) ? load_as_float(we + w_row * k_dim + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < MOE_TK; ++kk) {
      float av[PM];
#pragma unroll
      for (int i = 0; i < PM; ++i) av[i] = sa[ty + 16 * i][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = sw[tx + 16 * j][kk];
        const float u = GLU ? sw[MOE_TN + tx + 16 * j][kk] : 0.f;
#pragma unroll
        for (int i = 0; i < PM; ++i) {
          acc[i][j] += av[i] * b;
          if (GLU) acc_up[i][j] += av[i] * u;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < PM; ++i) {
    const int r = ty + 16 * i;
    if (r >= count) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= n_out) continue;
      float v = acc[i][j];
      if (GLU) {
        // the unit reads what the products would have stored in the activation dtype
        const float g = fminf(rounded_as<T>(v), limit);
        const float u = fminf(fmaxf(rounded_as<T>(acc_up[i][j]), -limit), limit);
        v = g / (1.f + expf(-alpha * g)) * (u + offset);
      } else if (act == 1) {
        const float r = fmaxf(rounded_as<T>(v), 0.f);
        v = r * r;
      }
      store_from_float(out + (int64_t)(start + r) * n_out + n, v);
    }
  }
}

// The same on the matrix cores (bfloat16, K a multiple of 8, rows at 16-byte addresses). A wave owns 16 outputs (for
// the gated unit 16 gate rows and the 16 up rows that go with them) and all 64 places of the tile: the weights are the
// first operand of v_mfma_f32_16x16x32_bf16, the operand rows the second, so accumulator entry i of lane (c, g) is
// output 4 g + i of place c. K goes in blocks of 64: lane (c, g) takes values 16 g .. 16 g + 15 of a block, 32
// contiguous bytes of its row, for both operands alike (a sum over K does not mind the order), the first eight for
// one instruction and the second eight for the next; four lanes then cover a whole 128-byte line of a row. Weights
// go straight from memory into that layout and every weight is read by one wave of the workgroup; the 64 operand
// rows, which all four waves need, go through LDS (gathered once per workgroup, two buffers, the next block of K on
// its way while this one is multiplied; rows 144 bytes apart so that 16 rows' 16-byte pieces fall into different
// banks).
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define MOE_X_STRIDE 72      // bf16 elements between two operand rows in LDS: 64 values and 16 bytes

template <typename O, bool GLU>
__global__ __launch_bounds__(256) void moe_product_mfma_kernel(const bf16_t* __restrict__ a, int64_t a_stride,
                                                               const bf16_t* __restrict__ w,
                                                               const int* __restrict__ sorted_pair,
                                                               const int* __restrict__ tile_expert,
                                                               const int* __restrict__ tile_start,
                                                               const int* __restrict__ tile_rows,
                                                               const int* __restrict__ n_tiles, O* __restrict__ out,
                                                               int top, int n_out, int k_dim, float limit, float alpha, float offset, int act) {
  constexpr int MT = MOE_TILE / 16;
  __shared__ __attribute__((aligned(16))) bf16_t sx[2][MOE_TILE * MOE_X_STRIDE];
  const int tile = blockIdx.x;
  if (tile >= *n_tiles) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.y * 4 + wave) * 16;
  const bool works = n0 < n_out;                              // a wave without outputs still helps to bring rows in
  const int expert = tile_expert[tile], start = tile_start[tile], count = tile_rows[tile];
  const int w_rows = GLU ? 2 * n_out : n_out;
  const bf16_t* we = w + (int64_t)expert * w_rows * k_dim;
  const int n_mine = min(n0 + c, n_out - 1);                  // rows beyond the last are read from it and never stored
  const bf16_t* w_gate = we + (int64_t)n_mine * k_dim + 16 * g;
  const bf16_t* w_up = we + ((int64_t)n_out + n_mine) * k_dim + 16 * g;
  // staging: thread (row = tid / 4, piece = tid % 4) brings 32 bytes of its row per block of K
  const int s_row = threadIdx.x / 4, s_piece = threadIdx.x % 4;
  const int s_place = start + min(s_row, count - 1);          // places beyond the tile's: its last one, never stored
  const bf16_t* s_src = a + (int64_t)(top > 0 ? sorted_pair[s_place] / top : s_place) * a_stride + 16 * s_piece;
  const int s_at = s_row * MOE_X_STRIDE + 16 * s_piece;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 p0, p1;
  auto fetch = [&](int k0) {
    p0 = k0 + 16 * s_piece < k_dim ? *(const bf16x8*)(s_src + k0) : zero;          // K is a multiple of 8
    p1 = k0 + 16 * s_piece + 8 < k_dim ? *(const bf16x8*)(s_src + k0 + 8) : zero;
  };
  f32x4 acc[MT], acc_up[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = acc_up[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  int buf = 0;
  for (int k0 = 0; k0 < k_dim; k0 += 64, buf ^= 1) {
    *(bf16x8*)(sx[buf] + s_at) = p0;
    *(bf16x8*)(sx[buf] + s_at + 8) = p1;
    if (k0 + 64 < k_dim) fetch(k0 + 64);
    bf16x8 wg0 = zero, wg1 = zero, wu0 = zero, wu1 = zero;
    if (works) {
      const bool in0 = k0 + 16 * g < k_dim, in1 = k0 + 16 * g + 8 < k_dim;
      if (in0) wg0 = *(const bf16x8*)(w_gate + k0);
      if (in1) wg1 = *(const bf16x8*)(w_gate + k0 + 8);
      if (GLU && in0) wu0 = *(const bf16x8*)(w_up + k0);
      if (GLU && in1) wu1 = *(const bf16x8*)(w_up + k0 + 8);
    }
    __syncthreads();               // this buffer is whole; the other one was last read before the barrier before
    if (works) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (16 * mt >= count) break;                            // a tile of few places (decoding) skips the empty rows
        const bf16_t* xr = sx[buf] + (16 * mt + c) * MOE_X_STRIDE + 16 * g;
        const bf16x8 x0 = *(const bf16x8*)xr, x1 = *(const bf16x8*)(xr + 8);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wg0, x0, acc[mt], 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wg1, x1, acc[mt], 0, 0, 0);
        if (GLU) {
          acc_up[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wu0, x0, acc_up[mt], 0, 0, 0);
          acc_up[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wu1, x1, acc_up[mt], 0, 0, 0);
        }
      }
    }
  }
  if (!works) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + c;
    if (m >= count) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n >= n_out) continue;
      float v = acc[mt][i];
      if (GLU) {
        const float gv = fminf(rounded_as<bf16_t>(v), limit);
        const float uv = fminf(fmaxf(rounded_as<bf16_t>(acc_up[mt][i]), -limit), limit);
        v = gv / (1.f + expf(-alpha * gv)) * (uv + offset);
      } else if (act == 1) {
        const float r = fmaxf(rounded_as<bf16_t>(v), 0.f);
        v = r * r;
      }
      store_from_float(out + (int64_t)(start + m) * n_out + n, v);
    }
  }
}

// For steps of few rows (decoding), where a tile holds at most 16 places: no LDS and no barrier. A wave walks K for
// its 16 outputs with the operand rows straight from memory (they are few and stay in the vector cache) and four
// blocks of K in flight, so that the weights, which are all the step reads, stream. Tiles of more places are walked
// 16 places at a time.
template <typename O, bool GLU>
__global__ __launch_bounds__(256) void moe_product_few_kernel(const bf16_t* __restrict__ a, int64_t a_stride,
                                                              const bf16_t* __restrict__ w,
                                                              const int* __restrict__ sorted_pair,
                                                              const int* __restrict__ tile_expert,
                                                              const int* __restrict__ tile_start,
                                                              const int* __restrict__ tile_rows,
                                                              const int* __restrict__ n_tiles, O* __restrict__ out,
                                                              int top, int n_out, int k_dim, float limit, float alpha, float offset, int act) {
  const int tile = blockIdx.x;
  if (tile >= *n_tiles) return;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, c = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.y * 4 + wave) * 16;
  if (n0 >= n_out) return;
  const int expert = tile_expert[tile], start = tile_start[tile], count = tile_rows[tile];
  const int w_rows = GLU ? 2 * n_out : n_out;
  const bf16_t* we = w + (int64_t)expert * w_rows * k_dim;
  const int n_mine = min(n0 + c, n_out - 1);
  const bf16_t* w_gate = we + (int64_t)n_mine * k_dim + 16 * g;
  const bf16_t* w_up = we + ((int64_t)n_out + n_mine) * k_dim + 16 * g;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int m0 = 0; m0 < count; m0 += 16) {
    const int place = start + min(m0 + c, count - 1);
    const bf16_t* x = a + (int64_t)(top > 0 ? sorted_pair[place] / top : place) * a_stride + 16 * g;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc_up = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < k_dim; k0 += 256) {
      bf16x8 wg[8], wu[8], xv[8];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + 64 * u;
        const bool in0 = k + 16 * g < k_dim, in1 = k + 16 * g + 8 < k_dim;     // K is a multiple of 8
        wg[2 * u] = in0 ? *(const bf16x8*)(w_gate + k) : zero;
        wg[2 * u + 1] = in1 ? *(const bf16x8*)(w_gate + k + 8) : zero;
        wu[2 * u] = (GLU && in0) ? *(const bf16x8*)(w_up + k) : zero;
        wu[2 * u + 1] = (GLU && in1) ? *(const bf16x8*)(w_up + k + 8) : zero;
        xv[2 * u] = in0 ? *(const bf16x8*)(x + k) : zero;
        xv[2 * u + 1] = in1 ? *(const bf16x8*)(x + k + 8) : zero;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wg[u], xv[u], acc, 0, 0, 0);
        if (GLU) acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wu[u], xv[u], acc_up, 0, 0, 0);
      }
    }
    const int m = m0 + c;
    if (m >= count) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 4 * g + i;
      if (n >= n_out) continue;
      float v = acc[i];
      if (GLU) {
        const float gv = fminf(rounded_as<bf16_t>(v), limit);
        const float uv = fminf(fmaxf(rounded_as<bf16_t>(acc_up[i]), -limit), limit);
        v = gv / (1.f + expf(-alpha * gv)) * (uv + offset);
      } else if (act == 1) {
        const float r = fmaxf(rounded_as<bf16_t>(v), 0.f);
        v = r * r;
      }
      store_from_float(out + (int64_t)(start + m) * n_out + n, v);
    }
  }
}

DRYFT_API int dryft_moe_product(const void* a, int64_t a_stride, const void* w, const int* sorted_pair,
                                const int* tile_expert, const int* tile_start, const int* tile_rows, const int* n_tiles,
                                int max_tiles, void* out, int out_is_f32, int top, int n_out, int k_dim, int glu,
                                float limit, float alpha, float offset, int act, int most_places, int is_f32, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (n_out <= 0 || k_dim <= 0 || (glu && out_is_f32 && !is_f32)) return -1;
  dim3 grid(max_tiles, (n_out + MOE_TN - 1) / MOE_TN), block(256);
  if (!is_f32 && k_dim % 8 == 0 && a_stride % 8 == 0 && (((uintptr_t)a | (uintptr_t)w) & 15) == 0) {
    if (most_places <= 16) {           // no expert can get more places than that: the kernel without LDS and barriers
#define MOE_FEW(O, G)                                                                                             \
  hipLaunchKernelGGL((moe_product_few_kernel<O, G>), grid, block, 0, stream, (const bf16_t*)a, a_stride,           \
                     (const bf16_t*)w, sorted_pair, tile_expert, tile_start, tile_rows, n_tiles, (O*)out, top, n_out, \
                     k_dim, limit, alpha, offset, act)
      if (glu) MOE_FEW(bf16_t, true);
      else if (out_is_f32) MOE_FEW(float, false);
      else MOE_FEW(bf16_t, false);
#undef MOE_FEW
      return DRYFT_LAUNCH_CHECK();
    }
#define MOE_MFMA(O, G)                                                                                            \
  hipLaunchKernelGGL((moe_product_mfma_kernel<O, G>), grid, block, 0, stream, (const bf16_t*)a, a_stride,          \
                     (const bf16_t*)w, sorted_pair, tile_expert, tile_start, tile_rows, n_tiles, (O*)out, top, n_out, \
                     k_dim, limit, alpha, offset, act)
    if (glu) MOE_MFMA(bf16_t, true);
    else if (out_is_f32) MOE_MFMA(float, false);
    else MOE_MFMA(bf16_t, false);
#undef MOE_MFMA
    return DRYFT_LAUNCH_CHECK();
  }
#define MOE_LAUNCH(T, O, G)                                                                                       \
  hipLaunchKernelGGL((moe_product_kernel<T, O, G>), grid, block, 0, stream, (const T*)a, a_stride, (const T*)w,   \
                     sorted_pair, tile_expert, tile_start, tile_rows, n_tiles, (O*)out, top, n_out, k_dim, limit, alpha, offset, act)
  if (is_f32) {
    if (glu) MOE_LAUNCH(float, float, true); else MOE_LAUNCH(float, float, false);
  } else if (glu) {
    MOE_LAUNCH(bf16_t, bf16_t, true);
  } else if (out_is_f32) {
    MOE_LAUNCH(bf16_t, float, false);
  } else {
    MOE_LAUNCH(bf16_t, bf16_t, false);
  }
#undef MOE_LAUNCH
  return DRYFT_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------------
// out[row] = sum_k weights[row, k] * y[place_of[row * top + k]]  (k in order)  + sigmoid(z_shared[row]) * shared[row]
// (without logits the shared expert is added as it is)
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place_of,
                                                          const float* __restrict__ weights, const T* __restrict__ shared,
                                                          const float* __restrict__ logits, int64_t logit_stride,
                                                          int shared_col, T* __restrict__ out, int top, int width) {
  const int64_t row = blockIdx.x;
  const float gate = shared ? (logits ? 1.f / (1.f + expf(-logits[row * logit_stride + shared_col])) : 1.f) : 0.f;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc += weights[row * top + k] * y[(int64_t)place_of[row * top + k] * width + c];
    if (shared) acc += gate * load_as_float(shared + row * width + c);
    store_from_float(out + row * width + c, acc);
  }
}

DRYFT_API int dryft_moe_combine(const float* y, const int* place_of, const float* weights, const void* shared,
                                const float* logits, int64_t logit_stride, int shared_col, void* out, int rows, int top,
                                int width, int is_f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  const dim3 grid(rows, rows <= 64 ? (width + 255) / 256 : 1);       // few rows: a workgroup per 256 columns
  if (is_f32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, y, place_of, weights,
                       (const float*)shared, logits, logit_stride, shared_col, (float*)out, top, width);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, dim3(256), 0, stream, y, place_of, weights,
                       (const bf16_t*)shared, logits, logit_stride, shared_col, (bf16_t*)out, top, width);
  return DRYFT_LAUNCH_CHECK();
}
