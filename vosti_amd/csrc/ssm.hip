// A state-space recurrence with one decay per head, and the gated norm of its read-out.
//
// Per head h (its inputs B and C are those of group h / (H / G)), with the state S [N, P] and for every token in order:
//   dt = softplus(dt_raw + dt_bias[h]);  S <- exp(-exp(A_log[h]) * dt) * S + dt * B x^T;  y = S^T C + D[h] * x
// where x [P] is the head's input, B and C [N] the token's input and output vectors.  Everything here is 32-bit; the
// projection that feeds dt arrives as elements, x, B and C as the 32-bit output of the short convolution.
//
// A sequence's tokens are walked in order by one workgroup per (sequence, head, block of value columns).  A column's
// state is spread over R neighbouring lanes, each holding DR consecutive state rows in registers; a token's read-out is
// the sum over a lane's rows in ascending order and then a butterfly over the R lanes (group_sum), whatever the step's cut: the
// state that a step leaves in memory (per head [P][N], 32-bit) is what the next step starts from, bit for bit.  The
// inputs of a chunk of tokens go through LDS: the next chunk's are read from global memory into registers before this
// chunk is walked and written to the other LDS buffer after it (one barrier a chunk).
#include <algorithm>

#include "common.h"
#include "vec.h"

#define SSM_THREADS 256
#define SSM_CHUNK 16

struct SsmArgs {
  float* y;               // [T, H * P]
  const float* xbc;       // [T, ldx]: x (H heads of P) from column 0, B (G groups of N) from b_col, C from c_col
  int64_t ldx;
  int b_col, c_col;
  const elem_t* dt;       // dt_raw of head h at dt[t * lddt + h]
  int64_t lddt;
  const void* dt_bias;    // [H]
  const void* A_log;      // [H]
  const void* D;          // [H]
  int w_is_f32;
  float* state;           // per slot, from its start: H states [P][N]
  int64_t state_stride;
  const int32_t* cu_q;
  const int32_t* positions;
  const int32_t* slots;
  int H, G, N, P;
};

__device__ __forceinline__ float ssm_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// R lanes share a value column, each with DR consecutive state rows; a workgroup has 256 / R columns.  In LDS the
// state rows are padded with zeros to R * DR, so that no lane has to ask whether a row exists.  CH: tokens a chunk (16,
// or 1 for a step of single tokens, whose workgroups then need little LDS and all run at once; the arithmetic of a token
// is the same).
template <int R, int DR, int ROUNDS, int CH>
__global__ __launch_bounds__(SSM_THREADS) void ssm_scan_kernel(SsmArgs a) {
  extern __shared__ float lds[];
  constexpr int COLS = SSM_THREADS / R, NP = R * DR;
  // A token's row in LDS: B [NP], C [NP], the workgroup's x columns [COLS], dt, the decay, and two to a whole vector.
  constexpr int L1 = 2 * NP + COLS + 1, RS = 2 * NP + COLS + 4;
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int N = a.N, P = a.P, g = h / (a.H / a.G);
  const int col = tid / R, r = tid % R;
  const int p = blockIdx.z * COLS + col;
  const bool col_ok = p < P;
  const int first = a.cu_q[s], n_tok = a.cu_q[s + 1] - first;
  if (n_tok <= 0) return;
  const bool fresh = a.positions[first] == 0;

  float S[DR];
  float* st = a.state + (int64_t)a.slots[s] * a.state_stride + ((int64_t)h * P + (col_ok ? p : 0)) * N;
#pragma unroll
  for (int j = 0; j < DR; ++j) {
    const int n = r * DR + j;
    S[j] = (!fresh && col_ok && n < N) ? st[n] : 0.f;
  }
  const float bias = load_weight(a.dt_bias, a.w_is_f32, h);
  const float rate = expf(load_weight(a.A_log, a.w_is_f32, h));
  const float Dh = load_weight(a.D, a.w_is_f32, h);

  float reg[ROUNDS][CH];
  float dt_reg = 0.f;
  auto fetch = [&](int c) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int e = tid + rd * SSM_THREADS;
      // Where this thread's element of a token's row comes from: -1 nowhere (padding), else an offset from the row's start.
      int64_t src = -1;
      if (e < NP) { if (e < N) src = a.b_col + g * N + e; }
      else if (e < 2 * NP) { if (e - NP < N) src = a.c_col + g * N + (e - NP); }
      else if (e < 2 * NP + COLS) { if ((int)(blockIdx.z * COLS) + (e - 2 * NP) < P) src = h * P + blockIdx.z * COLS + (e - 2 * NP); }
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int t = c * CH + i;
        float v = 0.f;
        if (t < n_tok && src >= 0) v = a.xbc[(int64_t)(first + t) * a.ldx + src];
        reg[rd][i] = v;
      }
    }
    // The step sizes: thread i has token i's, so that their softplus and exponentials run side by side.
    dt_reg = 0.f;
    if (tid < CH && c * CH + tid < n_tok) dt_reg = to_f32(a.dt[(int64_t)(first + c * CH + tid) * a.lddt + h]);
  };
  auto stage = [&](float* dst) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd) {
      const int e = tid + rd * SSM_THREADS;
      if (e >= L1 - 1) continue;
#pragma unroll
      for (int i = 0; i < CH; ++i) dst[i * RS + e] = reg[rd][i];
    }
    if (tid < CH) {
      const float dtv = ssm_softplus(dt_reg + bias);
      dst[tid * RS + L1 - 1] = dtv;
      dst[tid * RS + L1] = expf(-rate * dtv);
    }
  };

  const int chunks = (n_tok + CH - 1) / CH;
  fetch(0);
  stage(lds);
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    if (c + 1 < chunks) fetch(c + 1);
    const float* cur = lds + (c & 1) * (CH * RS);
    const int m = min(CH, n_tok - c * CH);
    float* yout = a.y + (int64_t)(first + c * CH) * ((int64_t)a.H * P) + (int64_t)h * P + p;
    // Four tokens at a time: the states move on token by token, the four read-outs' sums over the lanes run side by side.
    for (int i0 = 0; i0 < m; i0 += 4) {
      float acc[4], xv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc[u] = 0.f;
        xv[u] = 0.f;
        if (i0 + u < m) {
          const float* row = cur + (i0 + u) * RS;
          xv[u] = row[2 * NP + col];
          const float dtv = row[L1 - 1], dA = row[L1];
          const float dx = dtv * xv[u];
          const float* Bp = row + r * DR;
          const float* Cp = row + NP + r * DR;
          if constexpr (DR % 4 == 0) {
#pragma unroll
            for (int q = 0; q < DR / 4; ++q) {
              const f32x4 b4 = *reinterpret_cast<const f32x4*>(Bp + 4 * q), c4 = *reinterpret_cast<const f32x4*>(Cp + 4 * q);
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                S[4 * q + j] = __builtin_fmaf(dA, S[4 * q + j], dx * b4[j]);
                acc[u] = __builtin_fmaf(S[4 * q + j], c4[j], acc[u]);
              }
            }
          } else {
#pragma unroll
            for (int j = 0; j < DR; ++j) {
              S[j] = __builtin_fmaf(dA, S[j], dx * Bp[j]);
              acc[u] = __builtin_fmaf(S[j], Cp[j], acc[u]);
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] = group_sum<R>(acc[u]);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (r == 0 && col_ok && i0 + u < m) yout[(int64_t)(i0 + u) * ((int64_t)a.H * P)] = acc[u] + Dh * xv[u];
    }
    if (c + 1 < chunks) stage(lds + ((c + 1) & 1) * (CH * RS));
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int j = 0; j < DR; ++j) {
      const int n = r * DR + j;
      if (n < N) st[n] = S[j];
    }
  }
}

// out[t, c] = (y[t, c] * silu(z[t, c])) / sqrt(mean over c's part of the squares + eps) * w[c], as elements, for rows
// of `inner` values in `parts` equal parts; the columns from inner to ldo are set to zero (a projection with a padded
// reduction axis reads them).  One workgroup per (token, part); thread t owns the part's elements t, t + 256, ...
__global__ __launch_bounds__(256) void ssm_gate_norm_kernel(elem_t* __restrict__ out, int64_t ldo, const float* __restrict__ y,
                                                            const elem_t* __restrict__ z, int64_t ldz, const void* __restrict__ w,
                                                            int w_is_f32, int inner, int parts, float eps) {
  __shared__ float red[4];
  const int t = blockIdx.x, part = blockIdx.y, size = inner / parts, c0 = part * size;
  float sum = 0.f;
  for (int c = threadIdx.x; c < size; c += 256) {
    const float zv = to_f32(z[(int64_t)t * ldz + c0 + c]);
    const float gv = y[(int64_t)t * inner + c0 + c] * (zv / (1.f + expf(-zv)));
    sum = sum + gv * gv;
  }
  sum = wave_sum_xor(sum);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
  __syncthreads();
  float total = red[0];
  total = total + red[1];
  total = total + red[2];
  total = total + red[3];
  const float rr = rsqrtf(total / (float)size + eps);
  for (int c = threadIdx.x; c < size; c += 256) {
    const float zv = to_f32(z[(int64_t)t * ldz + c0 + c]);
    const float gv = y[(int64_t)t * inner + c0 + c] * (zv / (1.f + expf(-zv)));
    out[(int64_t)t * ldo + c0 + c] = from_f32<elem_t>((gv * rr) * load_weight(w, w_is_f32, c0 + c));
  }
  if (part == 0)
    for (int c = inner + threadIdx.x; c < ldo; c += 256) out[(int64_t)t * ldo + c] = from_f32<elem_t>(0.f);
}

extern "C" {

// y [T, H, P] floats.  xbc: float rows of length ldx with x (H heads of P) from column 0, B (G groups of N) from b_col
// and C from c_col; dt: elements, the step size's pre-activation of head h at dt[t * lddt + h]; dt_bias, A_log, D: [H]
// (all floats or all elements).  state: per slot, the H states at its start, each [P][N].  T: the rows of y (every one of
// the S sequences brings at least one).
int vk_ssm_scan(float* y, const float* xbc, int64_t ldx, int b_col, int c_col, const elem_t* dt, int64_t lddt, const void* dt_bias,
                const void* A_log, const void* D, int w_is_f32, float* state, int64_t state_stride, const int32_t* cu_q,
                const int32_t* positions, const int32_t* slots, int S, int T, int H, int G, int N, int P, hipStream_t st) {
  VK_REQUIRE(S >= 0 && H > 0 && G > 0 && H % G == 0 && N > 0 && N <= 256 && P > 0, "state-space scan: bad sizes H=%d G=%d N=%d P=%d (N at most 256)",
             H, G, N, P);
  VK_REQUIRE(b_col >= H * P && c_col >= 0 && ldx >= (int64_t)std::max(b_col, c_col) + (int64_t)G * N && lddt >= H,
             "state-space scan: the rows do not hold the inputs");
  VK_REQUIRE(state_stride >= (int64_t)H * P * N, "state-space scan: the state does not hold the heads");
  VK_REQUIRE(H <= 65535, "state-space scan: too many heads");
  if (S == 0) return 0;
  const bool single_tokens = T == S;       // every sequence brings one token
  SsmArgs a;
  a.y = y; a.xbc = xbc; a.ldx = ldx; a.b_col = b_col; a.c_col = c_col; a.dt = dt; a.lddt = lddt; a.dt_bias = dt_bias; a.A_log = A_log; a.D = D;
  a.w_is_f32 = w_is_f32; a.state = state; a.state_stride = state_stride; a.cu_q = cu_q; a.positions = positions; a.slots = slots;
  a.H = H; a.G = G; a.N = N; a.P = P;
  // Lanes a column and rows a lane: 16 lanes from 128 state rows on (more workgroups, shorter sums a token), else 8.
#define SSM_SCAN(R, DR, ROUNDS)                                                                                                  \
  do {                                                                                                                           \
    constexpr int cols = SSM_THREADS / (R);                                                                                      \
    static_assert((2 * (R) * (DR) + cols + SSM_THREADS - 1) / SSM_THREADS <= (ROUNDS), "a round more is needed");                \
    VK_REQUIRE((P + cols - 1) / cols <= 65535, "state-space scan: too many columns");                                            \
    const dim3 grid(S, H, (P + cols - 1) / cols);                                                                                \
    if (single_tokens) {                                                                                                         \
      ssm_scan_kernel<R, DR, ROUNDS, 1><<<grid, SSM_THREADS, (size_t)2 * (2 * (R) * (DR) + cols + 4) * sizeof(float), st>>>(a);   \
    } else {                                                                                                                     \
      const size_t smem = (size_t)2 * SSM_CHUNK * (2 * (R) * (DR) + cols + 4) * sizeof(float);                                    \
      static bool raised = false;                                                                                                \
      if (!raised && smem > 48 * 1024) {                                                                                         \
        (void)hipFuncSetAttribute((const void*)ssm_scan_kernel<R, DR, ROUNDS, SSM_CHUNK>, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024); \
        raised = true;                                                                                                           \
      }                                                                                                                          \
      ssm_scan_kernel<R, DR, ROUNDS, SSM_CHUNK><<<grid, SSM_THREADS, smem, st>>>(a);                                             \
    }                                                                                                                            \
  } while (0)
  if (N <= 8) SSM_SCAN(8, 1, 1);
  else if (N <= 16) SSM_SCAN(8, 2, 1);
  else if (N <= 32) SSM_SCAN(8, 4, 1);
  else if (N <= 64) SSM_SCAN(8, 8, 1);
  else if (N < 128) SSM_SCAN(8, 16, 2);
  else if (N == 128) SSM_SCAN(16, 8, 2);
  else SSM_SCAN(16, 16, 3);
#undef SSM_SCAN
  return vk_check_launch("state-space scan");
}

// out [T, ldo] elements from y [T, inner] floats and the gate z (elements, row stride ldz); w [inner].
int vk_ssm_gate_norm(elem_t* out, int64_t ldo, const float* y, const elem_t* z, int64_t ldz, const void* w, int w_is_f32, int T, int inner,
                     int parts, float eps, hipStream_t st) {
  VK_REQUIRE(T >= 0 && inner > 0 && parts > 0 && inner % parts == 0 && parts <= 65535 && ldo >= inner && ldz >= inner && eps >= 0.f,
             "gated norm: bad sizes T=%d inner=%d parts=%d", T, inner, parts);
  if (T == 0) return 0;
  ssm_gate_norm_kernel<<<dim3(T, parts), 256, 0, st>>>(out, ldo, y, z, ldz, w, w_is_f32, inner, parts, eps);
  return vk_check_launch("gated norm");
}

}  // extern "C"
