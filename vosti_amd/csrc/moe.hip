// A mixture of small feed-forward experts, each token through its `top` best of E: the router, the plan that sorts
// (token, choice) pairs by expert into tiles of 16 rows, the two projections as grouped products on the matrix unit,
// and the weighted sum of a token's experts.
//
//   z = W_router h (32-bit sums of the elements' exact products);  s = softmax(z) over all experts;  the `top` largest
//   s (the lower index wins a tie);  weight_k = s_k / (sum of the chosen s + weight_eps);
//   out = sum over the chosen k, in the order they were chosen, of weight_k * W_down[e_k] act(W_up[e_k] h),
//   act(u) = max(u, 0)^2.
//
// A row of a grouped product depends on its own inputs only (its sums run over the reduction axis in ascending slabs
// of 64 bytes), so a token's result does not depend on which other tokens share its tile or where the plan put it.
#include <algorithm>

#include "common.h"
#include "mma.h"
#include "vec.h"

#define MOE_TILE 16          // rows of a tile: pairs of one expert
#define MOE_ROUTE_TOKENS 8   // tokens a router workgroup shares an expert's weights among

// Router: idx [T, top] int32, wts [T, top] floats.  A workgroup of four waves takes MOE_ROUTE_TOKENS tokens; wave w
// computes the logits of experts w, w + 4, ... for all of them (lane l owns columns l, l + 64, ... in ascending order,
// then a butterfly), then waves take tokens and choose.
__global__ __launch_bounds__(256) void moe_route_kernel(int32_t* __restrict__ idx, float* __restrict__ wts, const elem_t* __restrict__ h,
                                                        const elem_t* __restrict__ router, int T, int W, int E, int top, float weight_eps) {
  extern __shared__ float logits[];      // [MOE_ROUTE_TOKENS][E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t0 = blockIdx.x * MOE_ROUTE_TOKENS;
  for (int e = wave; e < E; e += 4) {
    float acc[MOE_ROUTE_TOKENS];
#pragma unroll
    for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) acc[i] = 0.f;
    const elem_t* wr = router + (int64_t)e * W;
    for (int c = lane; c < W; c += 64) {
      const float wv = to_f32(wr[c]);
#pragma unroll
      for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) {
        const int t = min(t0 + i, T - 1);
        acc[i] = __builtin_fmaf(to_f32(h[(int64_t)t * W + c]), wv, acc[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < MOE_ROUTE_TOKENS; ++i) {
      const float v = wave_sum_xor(acc[i]);
      if (lane == 0) logits[i * E + e] = v;
    }
  }
  __syncthreads();
  for (int i = wave; i < MOE_ROUTE_TOKENS; i += 4) {
    const int t = t0 + i;
    if (t >= T) continue;
    float* z = logits + i * E;
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max_xor(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(z[e] - mx);
      z[e] = p;
      sum = sum + p;
    }
    sum = wave_sum_xor(sum);
    // The largest score `top` times; a chosen one is marked with -1 (scores are positive or zero).
    float chosen_sum = 0.f;
    float my_w = 0.f;
    int my_e = 0;
    for (int k = 0; k < top; ++k) {
      float best = -2.f;
      int best_e = 0x7fffffff;
      for (int e = lane; e < E; e += 64) {
        const float v = z[e];
        if (v > best) { best = v; best_e = e; }
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off, VK_WAVE);
        const int oe = __shfl_xor(best_e, off, VK_WAVE);
        if (ov > best || (ov == best && oe < best_e)) { best = ov; best_e = oe; }
      }
      const float score = best / sum;
      chosen_sum = chosen_sum + score;
      if (lane == k % 64 && k < 64) { my_w = score; my_e = best_e; }
      if (k >= 64 && lane == 0) { idx[(int64_t)t * top + k] = best_e; wts[(int64_t)t * top + k] = score; }
      if (lane == 0) z[best_e] = -1.f;
      __builtin_amdgcn_wave_barrier();
    }
    const float denom = chosen_sum + weight_eps;
    if (lane < top) {
      idx[(int64_t)t * top + lane] = my_e;
      wts[(int64_t)t * top + lane] = my_w / denom;
    }
    for (int k = 64 + lane; k < top; k += 64) wts[(int64_t)t * top + k] = wts[(int64_t)t * top + k] / denom;
  }
}

// The plan, by one workgroup.  counts the pairs of every expert, gives expert e the rows [start_e, start_e + 16 *
// ceil(count_e / 16)) and every pair a row among its expert's (in no fixed order: a row's result does not depend on
// its place).  row_pair [max_rows]: the pair (token * top + choice) of a row, or -1; pair_row [pairs]; tile_expert
// [max_tiles]: the expert of a tile, or -1 beyond the last.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t* __restrict__ idx, int32_t* __restrict__ row_pair,
                                                        int32_t* __restrict__ pair_row, int32_t* __restrict__ tile_expert, int pairs, int E,
                                                        int max_tiles) {
  extern __shared__ int32_t plan[];      // [E] counts, then [E] cursors
  int32_t* count = plan;
  int32_t* cursor = plan + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int r = threadIdx.x; r < max_tiles * MOE_TILE; r += blockDim.x) row_pair[r] = -1;
  for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&count[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int tile = 0;
    for (int e = 0; e < E; ++e) {
      const int n = (count[e] + MOE_TILE - 1) / MOE_TILE;
      cursor[e] = tile * MOE_TILE;
      for (int j = 0; j < n; ++j) tile_expert[tile + j] = e;
      tile += n;
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int row = atomicAdd(&cursor[idx[i]], 1);
    row_pair[row] = i;
    pair_row[i] = row;
  }
}

// One tile of 16 rows times 64 output features a wave, four waves a workgroup: out[row, f] = sum over k of
// x[row, k] * w[expert][f, k].  GATHER: the rows' inputs are the tokens' (row -> pair / top) and the output is
// act(.) as elements; else the inputs are the rows themselves and the output is 32-bit.
template <bool GATHER>
__global__ __launch_bounds__(256) void moe_gemm_kernel(void* __restrict__ out, int64_t ldo, const elem_t* __restrict__ x, int64_t ldx,
                                                       const elem_t* __restrict__ w, int64_t expert_stride, const int32_t* __restrict__ row_pair,
                                                       const int32_t* __restrict__ tile_expert, int top, int N, int K) {
  const int tile = blockIdx.x;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int f0 = (blockIdx.y * 4 + wave) * 64;
  if (f0 >= N) return;
  const int r16 = lane & 15, kq = lane >> 4;
  // Second operand: the tile's rows.
  const int row = tile * MOE_TILE + r16;
  const int pair = row_pair[row];
  const elem_t* xr = x + (GATHER ? (int64_t)(pair < 0 ? 0 : pair / top) : (int64_t)row) * ldx;
  const bool x_ok = pair >= 0;
  const elem_t* we = w + (int64_t)e * expert_stride;
  f32x4 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += VK_SLAB) {
    const int k = k0 + kq * VK_VEC;
    const bool k_ok = k < K;
    const frag_t xf = load_frag(xr + k, x_ok && k_ok);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int f = f0 + j * 16 + r16;
      const frag_t wf = load_frag(we + (int64_t)(f < N ? f : 0) * K + k, f < N && k_ok);
      acc[j] = mma_slab(wf, xf, acc[j]);
    }
  }
  // Lane l holds features 4 * (l / 16) + i of the feature tile for row l % 16.
  if (!x_ok) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = f0 + j * 16 + kq * 4 + i;
      if (f >= N) continue;
      const float v = acc[j][i];
      if (GATHER) {
        const float rl = fmaxf(v, 0.f);
        static_cast<elem_t*>(out)[(int64_t)row * ldo + f] = from_f32<elem_t>(rl * rl);
      } else {
        static_cast<float*>(out)[(int64_t)row * ldo + f] = v;
      }
    }
  }
}

// Zero columns [N, ldo) of the rows that hold a pair: the second product's reduction axis is padded.
__global__ __launch_bounds__(256) void moe_pad_kernel(elem_t* __restrict__ act, int64_t ldo, int N, const int32_t* __restrict__ row_pair) {
  const int row = blockIdx.x;
  if (row_pair[row] < 0) return;
  for (int c = N + threadIdx.x; c < ldo; c += 256) act[(int64_t)row * ldo + c] = from_f32<elem_t>(0.f);
}

// out[t, c] = sum over k < top, ascending, of wts[t, k] * y[pair_row[t * top + k], c], from zero.
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y, const float* __restrict__ wts,
                                                          const int32_t* __restrict__ pair_row, int W, int top) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < W; c += gridDim.y * 256) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) acc = acc + wts[(int64_t)t * top + k] * y[(int64_t)pair_row[(int64_t)t * top + k] * W + c];
    out[(int64_t)t * W + c] = acc;
  }
}

extern "C" {

// Rows that the plan may need for T tokens: every pair, and up to 15 rows of padding an expert that got any.
int vk_moe_max_tiles(int T, int top, int E) {
  const int64_t pairs = (int64_t)T * top;
  const int64_t busy = std::min<int64_t>(E, pairs);
  return (int)((pairs + busy * (MOE_TILE - 1)) / MOE_TILE);
}

int vk_moe_route(int32_t* idx, float* wts, const elem_t* h, const elem_t* router, int T, int W, int E, int top, float weight_eps,
                 hipStream_t st) {
  VK_REQUIRE(T >= 0 && W > 0 && E > 0 && top > 0 && top <= E && E <= 4096, "router: bad sizes T=%d W=%d E=%d top=%d (at most 4096 experts)", T, W, E, top);
  if (T == 0) return 0;
  moe_route_kernel<<<(T + MOE_ROUTE_TOKENS - 1) / MOE_ROUTE_TOKENS, 256, (size_t)MOE_ROUTE_TOKENS * E * sizeof(float), st>>>(idx, wts, h, router, T,
                                                                                                                          W, E, top, weight_eps);
  return vk_check_launch("router");
}

int vk_moe_plan(const int32_t* idx, int32_t* row_pair, int32_t* pair_row, int32_t* tile_expert, int T, int top, int E, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && E <= 4096, "expert plan: bad sizes T=%d top=%d E=%d", T, top, E);
  if (T == 0) return 0;
  moe_plan_kernel<<<1, 1024, (size_t)2 * E * sizeof(int32_t), st>>>(idx, row_pair, pair_row, tile_expert, T * top, E, vk_moe_max_tiles(T, top, E));
  return vk_check_launch("expert plan");
}

// act [max_rows, ldo] elements = relu(x[token of row] . w_up[expert of row])^2; w_up [E, N, K]; columns N..ldo zero.
int vk_moe_up(elem_t* act, int64_t ldo, const elem_t* x, int64_t ldx, const elem_t* w_up, const int32_t* row_pair, const int32_t* tile_expert,
              int T, int top, int E, int N, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && ldx % VK_VEC == 0 && ldx >= K && ldo >= N,
             "experts (up): bad sizes N=%d K=%d (K in whole 16-byte vectors)", N, K);
  VK_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w_up % 16) == 0, "experts (up): operands must be 16-byte aligned");
  if (T == 0) return 0;
  const int tiles = vk_moe_max_tiles(T, top, E);
  moe_gemm_kernel<true><<<dim3(tiles, (N + 255) / 256), 256, 0, st>>>(act, ldo, x, ldx, w_up, (int64_t)N * K, row_pair, tile_expert, top, N, K);
  if (vk_check_launch("experts (up)")) return 1;
  if (ldo > N) {
    moe_pad_kernel<<<tiles * MOE_TILE, 256, 0, st>>>(act, ldo, N, row_pair);
    return vk_check_launch("experts (padding)");
  }
  return 0;
}

// y [max_rows, N] floats = act[row] . w_down[expert of row]; w_down [E, N, K]; act rows of length lda >= K.
int vk_moe_down(float* y, const elem_t* act, int64_t lda, const elem_t* w_down, const int32_t* row_pair, const int32_t* tile_expert, int T,
                int top, int E, int N, int K, hipStream_t st) {
  VK_REQUIRE(T >= 0 && top > 0 && E > 0 && N > 0 && K > 0 && K % VK_VEC == 0 && lda % VK_VEC == 0 && lda >= K,
             "experts (down): bad sizes N=%d K=%d (K in whole 16-byte vectors)", N, K);
  VK_REQUIRE(((uintptr_t)act % 16) == 0 && ((uintptr_t)w_down % 16) == 0, "experts (down): operands must be 16-byte aligned");
  if (T == 0) return 0;
  const int tiles = vk_moe_max_tiles(T, top, E);
  moe_gemm_kernel<false><<<dim3(tiles, (N + 255) / 256), 256, 0, st>>>(y, N, act, lda, w_down, (int64_t)N * K, row_pair, tile_expert, top, N, K);
  return vk_check_launch("experts (down)");
}

int vk_moe_combine(float* out, const float* y, const float* wts, const int32_t* pair_row, int T, int W, int top, hipStream_t st) {
  VK_REQUIRE(T >= 0 && W > 0 && top > 0, "experts (sum): bad sizes T=%d W=%d top=%d", T, W, top);
  if (T == 0) return 0;
  const int by = std::min((W + 255) / 256, 64);
  moe_combine_kernel<<<dim3(T, by), 256, 0, st>>>(out, y, wts, pair_row, W, top);
  return vk_check_launch("experts (sum)");
}

}  // extern "C"
