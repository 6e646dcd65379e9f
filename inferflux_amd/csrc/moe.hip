// Mixture of experts: the router and the experts' products for rows that each choose their own experts.
//
//   ifx_moe_route     z = W_r h in float (formed here for steps of few rows, else given: a product of many rows belongs
//                     to the product kernels), score s = sigmoid(z) (or softmax over the experts), choice of `top` experts
//                     among those of the best `keep` of `groups` equal groups of neighbouring experts (a group's
//                     score: the sum of its `group_top` largest scores); the weights are the chosen scores as they
//                     are or divided by their sum.  With `choice_bias` [E] the choice (of groups and of experts) goes by
//                     s + choice_bias while the weights stay the scores s themselves.  Writes ids [T][top] (int32) and weights [T][top] (float), in
//                     descending order of score, the lower index first among equals.
//   ifx_moe_gate_up   a[t][j][:] = act(Wg[e] h_t, Wu[e] h_t) for e = ids[t][j]          (Wg, Wu [E][ff][K]; act: common.h)
//   ifx_moe_down      out[t][:] = sum_j weights[t][j] * Wd[e_j] a[t][j][:]              (Wd [E][N][ff])
//                     An id from `n_real` upwards names an identity expert, which has no weights: its output is the
//                     row h_t itself (ifx_moe_gate_up leaves such items alone, ifx_moe_down adds weights[t][j] * h_t).
//
// The two product kernels read the expert of every (row, choice) from device memory, so their grid depends on the
// step's layout alone.  One wave forms one output element at a time (lanes across k, the fixed-order sum of
// common.h), so a row's result does not depend on what shares its batch.  They are the path of the 32-bit mode and of
// steps of few rows; bfloat16 steps of many rows take the grouped matrix-core product (grouped_gemm.hip).
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_EXPERTS 1024
#define MAX_TOP 32

// eight consecutive elements as floats: one 16-byte load of bfloat16, two of float
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
  const bf16x8 t = *(const bf16x8*)p;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (float)t[i];
}
__device__ __forceinline__ void load8(const float* p, float* v) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// R dot products of x [K] with the rows w[r] [K] at once, lanes across k in 16-byte pieces (K a multiple of 8), every
// row's loads in flight together; each lane's partial sums, still to be added over the wave
template <int R, typename T>
__device__ __forceinline__ void dots8(const T* __restrict__ x, const T* const* w, int K, int lane, float* sum) {
#pragma unroll
  for (int r = 0; r < R; ++r) sum[r] = 0.f;
  // two pieces of every row a trip: 2 (R + 1) loads of 16 bytes in flight per lane
  for (int c = lane * 8; c < K; c += 2 * WAVE * 8) {
    const int c2 = c + WAVE * 8;
    const bool more = c2 < K;
    float xv[2][8], wv[2][R][8];
    load8(x + c, xv[0]);
#pragma unroll
    for (int r = 0; r < R; ++r) load8(w[r] + c, wv[0][r]);
    if (more) {
      load8(x + c2, xv[1]);
#pragma unroll
      for (int r = 0; r < R; ++r) load8(w[r] + c2, wv[1][r]);
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int i = 0; i < 8; ++i) sum[r] = fmaf(xv[0][i], wv[0][r][i], sum[r]);
    if (more)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < 8; ++i) sum[r] = fmaf(xv[1][i], wv[1][r][i], sum[r]);
  }
}

struct RouteArgs {
  const void* h; const void* w; const float* z; int* ids; float* weights;
  int T, K, E, top, groups, keep, group_top, softmax, renorm;
  float scale;
  const float* bias;     // [E] added to the logits, or null
  const float* choice_bias;   // [E] added to the scores for the choice alone, or null
};

template <typename T>
__global__ __launch_bounds__(1024) void moe_route_kernel(RouteArgs a) {
  __shared__ float s[MAX_EXPERTS];       // scores
  __shared__ float c[MAX_EXPERTS];       // what the choice goes by: the scores, plus the choice's bias
  __shared__ float gs[MAX_EXPERTS + MAX_TOP];      // group scores, and behind them the chosen scores in order
  __shared__ int shut[MAX_EXPERTS];      // 1: a group that is shut out
  __shared__ float red[16];
  const size_t t = blockIdx.x;
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, nw = blockDim.x / WAVE;
  const T* h = (const T*)a.h + t * a.K;
  const T* w = (const T*)a.w;
  if (a.z) {                     // the logits are somebody else's product (steps of many rows)
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) s[e] = a.z[t * a.E + e];
  } else if (a.K % 8 == 0) {
    for (int e0 = wid * 4; e0 < a.E; e0 += nw * 4) {          // four experts to a wave at a time
      const T* rows[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) rows[r] = w + (size_t)min(e0 + r, a.E - 1) * a.K;
      float z[4];
      dots8<4>(h, rows, a.K, lane, z);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = wave_sum(z[r]);
        if (lane == 0 && e0 + r < a.E) s[e0 + r] = v;
      }
    }
  } else {
    for (int e = wid; e < a.E; e += nw) {
      float z = 0.f;
      for (int k = lane; k < a.K; k += WAVE) z = fmaf(to_f(h[k]), to_f(w[(size_t)e * a.K + k]), z);
      z = wave_sum(z);
      if (lane == 0) s[e] = z;
    }
  }
  __syncthreads();
  if (a.bias) {
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) s[e] += a.bias[e];
    __syncthreads();
  }
  if (a.softmax) {
    float m = -INFINITY;
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) m = fmaxf(m, s[e]);
    m = block_max(m, red);
    float l = 0.f;
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) l += expf(s[e] - m);
    l = block_sum(l, red);
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) s[e] = expf(s[e] - m) / l;
  } else {
    for (int e = threadIdx.x; e < a.E; e += blockDim.x) s[e] = 1.0f / (1.0f + expf(-s[e]));
  }
  __syncthreads();
  for (int e = threadIdx.x; e < a.E; e += blockDim.x) c[e] = a.choice_bias ? s[e] + a.choice_bias[e] : s[e];
  __syncthreads();
  // Every thread ranks what it owns among its like (more of them score higher, or as high at a lower index): a group
  // among the groups, then an expert among the experts of the groups that are kept.  The rank is the place in the output.
  const int per = a.E / a.groups;
  for (int g = threadIdx.x; g < a.groups; g += blockDim.x) {
    float sum = 0.f;
    if (a.keep < a.groups) {           // the sum of the group's group_top highest scores
      int taken[8];
      for (int r = 0; r < a.group_top && r < per; ++r) {
        int best = -1;
        for (int e = g * per; e < (g + 1) * per; ++e) {
          bool used = false;
          for (int q = 0; q < r; ++q) used |= taken[q] == e;
          if (!used && (best < 0 || c[e] > c[best])) best = e;
        }
        taken[r] = best;
        sum += c[best];
      }
    }
    gs[g] = sum;
  }
  __syncthreads();
  for (int g = threadIdx.x; g < a.groups; g += blockDim.x) {
    int rank = 0;
    if (a.keep < a.groups)
      for (int o = 0; o < a.groups; ++o) rank += (gs[o] > gs[g] || (gs[o] == gs[g] && o < g)) ? 1 : 0;
    shut[g] = rank >= a.keep ? 1 : 0;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < a.E; e += blockDim.x) {
    if (shut[e / per]) continue;
    int rank = 0;
    for (int o = 0; o < a.E; ++o) rank += (!shut[o / per] && (c[o] > c[e] || (c[o] == c[e] && o < e))) ? 1 : 0;
    if (rank < a.top) {
      a.ids[t * a.top + rank] = e;
      gs[a.groups + rank] = s[e];        // (gs has room behind the groups: E >= groups + top is not needed, MAX_EXPERTS + ... see below)
    }
  }
  __syncthreads();
  if (threadIdx.x < a.top) {
    float total = 0.f;
    for (int r = 0; r < a.top; ++r) total += gs[a.groups + r];
    const float v = gs[a.groups + threadIdx.x];
    a.weights[t * a.top + threadIdx.x] = (a.renorm ? v / total : v) * a.scale;
  }
}

extern "C" int ifx_moe_route(const void* h, const void* w, int dtype, const float* z, int* ids, float* weights, int T, int K, int E,
                             int top, int groups, int keep, int group_top, int softmax, int renorm, float scale, const float* bias, const float* choice_bias, void* stream) {
  IFX_REQUIRE(z || (h && w), "moe_route: neither logits nor the rows and the router's weight");
  IFX_REQUIRE(T >= 0 && K > 0 && E > 0 && E <= MAX_EXPERTS, "moe_route: %d experts (at most %d), K=%d", E, MAX_EXPERTS, K);
  IFX_REQUIRE(groups > 0 && E % groups == 0 && keep > 0 && keep <= groups, "moe_route: %d experts in %d groups of which %d are kept", E, groups, keep);
  IFX_REQUIRE(group_top > 0 && group_top <= 8, "moe_route: a group's score sums its %d largest (1-8)", group_top);
  IFX_REQUIRE(top > 0 && top <= MAX_TOP && top <= keep * (E / groups), "moe_route: top %d of %d x %d experts", top, keep, E / groups);
  if (T == 0) return 0;
  RouteArgs a{h, w, z, ids, weights, T, K, E, top, groups, keep, group_top, softmax, renorm, scale, bias, choice_bias};
  // a wave takes four experts at a time: as many waves as that takes, up to 16 (the scores are a chain of trips to memory otherwise)
  const int threads = z ? WAVE * (E <= 64 ? 1 : 4) : WAVE * (E <= 16 ? 4 : (E <= 32 ? 8 : 16));
  hipStream_t s = (hipStream_t)stream;
  if (z || dtype == DT_F32) hipLaunchKernelGGL(moe_route_kernel<float>, dim3(T), dim3(threads), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(T), dim3(threads), 0, s, a);
  else IFX_FAIL("moe_route: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
#define ROWS_PER_WAVE 4
#define WAVES 4

template <typename T>
__global__ __launch_bounds__(WAVE * WAVES) void moe_gate_up_kernel(const T* __restrict__ h, const T* __restrict__ wg,
                                                                   const T* __restrict__ wu, const int* __restrict__ ids,
                                                                   T* __restrict__ act, int K, int ff, int top, int paired,
                                                                   int n_real, int act_kind, float limit) {
  const size_t item = blockIdx.x;                 // (row, choice)
  const size_t t = item / top;
  const int e = ids[item];
  if (e >= n_real) return;                        // an identity expert: nothing to form (the whole workgroup leaves)
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const T* x = h + t * K;
  const int i0 = (blockIdx.y * WAVES + wid) * ROWS_PER_WAVE;
  if (i0 >= ff) return;
  // paired: one tensor [E][2 ff][K] whose rows alternate 16 of Wg with the same 16 of Wu (what the grouped product reads)
  auto gate_row = [&](int i) { return paired ? wg + ((size_t)e * 2 * ff + (i / 16) * 32 + i % 16) * K : wg + ((size_t)e * ff + i) * K; };
  auto up_row = [&](int i) { return paired ? gate_row(i) + (size_t)16 * K : wu + ((size_t)e * ff + i) * K; };
  float sum[2 * ROWS_PER_WAVE];
  if (K % 8 == 0) {
    const T* rows[2 * ROWS_PER_WAVE];
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
      const int i = min(i0 + r, ff - 1);
      rows[2 * r] = gate_row(i);
      rows[2 * r + 1] = up_row(i);
    }
    dots8<2 * ROWS_PER_WAVE>(x, rows, K, lane, sum);
  } else {
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
      const int i = min(i0 + r, ff - 1);
      const T* g = gate_row(i);
      const T* u = up_row(i);
      float sg = 0.f, su = 0.f;
      for (int k = lane; k < K; k += WAVE) {
        const float xv = to_f(x[k]);
        sg = fmaf(xv, to_f(g[k]), sg);
        su = fmaf(xv, to_f(u[k]), su);
      }
      sum[2 * r] = sg; sum[2 * r + 1] = su;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) {
    const float sg = wave_sum(sum[2 * r]), su = wave_sum(sum[2 * r + 1]);
    if (lane == 0 && i0 + r < ff) act[item * ff + i0 + r] = from_f<T>(gated_act(sg, su, act_kind, limit));
  }
}

template <typename T>
__global__ __launch_bounds__(WAVE * WAVES) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ wd,
                                                                const int* __restrict__ ids, const float* __restrict__ weights,
                                                                T* __restrict__ out, int N, int ff, int top, int n_real,
                                                                const T* __restrict__ h) {
  const size_t t = blockIdx.x;
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int n0 = (blockIdx.y * WAVES + wid) * ROWS_PER_WAVE;
  if (n0 >= N) return;
  float y[ROWS_PER_WAVE];
#pragma unroll
  for (int r = 0; r < ROWS_PER_WAVE; ++r) y[r] = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[t * top + j];
    if (e >= n_real) {          // an identity expert: the row itself (N is the row's width)
#pragma unroll
      for (int r = 0; r < ROWS_PER_WAVE; ++r) y[r] = fmaf(weights[t * top + j], to_f(h[t * N + min(n0 + r, N - 1)]), y[r]);
      continue;
    }
    const T* a = act + (t * top + j) * ff;
    float sum[ROWS_PER_WAVE];
    if (ff % 8 == 0) {
      const T* rows[ROWS_PER_WAVE];
#pragma unroll
      for (int r = 0; r < ROWS_PER_WAVE; ++r) rows[r] = wd + ((size_t)e * N + min(n0 + r, N - 1)) * ff;
      dots8<ROWS_PER_WAVE>(a, rows, ff, lane, sum);
    } else {
      for (int r = 0; r < ROWS_PER_WAVE; ++r) {
        const T* w = wd + ((size_t)e * N + min(n0 + r, N - 1)) * ff;
        float s = 0.f;
        for (int k = lane; k < ff; k += WAVE) s = fmaf(to_f(a[k]), to_f(w[k]), s);
        sum[r] = s;
      }
    }
    const float wj = weights[t * top + j];
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) y[r] = fmaf(wj, wave_sum(sum[r]), y[r]);
  }
  if (lane == 0)
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r)
      if (n0 + r < N) out[t * N + n0 + r] = from_f<T>(y[r]);
}

extern "C" int ifx_moe_gate_up(const void* h, const void* wg, const void* wu, const int* ids, void* act, int dtype, int T, int K,
                               int ff, int top, int paired, int n_real, int act_kind, float limit, void* stream) {
  IFX_REQUIRE(T >= 0 && K > 0 && ff > 0 && top > 0, "moe_gate_up: bad sizes T=%d K=%d ff=%d top=%d", T, K, ff, top);
  IFX_REQUIRE(!paired || ff % 16 == 0, "moe_gate_up: paired weights need ff=%d to be a multiple of 16", ff);
  if (T == 0) return 0;
  const dim3 grid((unsigned)T * top, (ff + WAVES * ROWS_PER_WAVE - 1) / (WAVES * ROWS_PER_WAVE));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    hipLaunchKernelGGL(moe_gate_up_kernel<float>, grid, dim3(WAVE * WAVES), 0, s, (const float*)h, (const float*)wg, (const float*)wu, ids, (float*)act, K, ff, top, paired, n_real, act_kind, limit);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(moe_gate_up_kernel<bf16_t>, grid, dim3(WAVE * WAVES), 0, s, (const bf16_t*)h, (const bf16_t*)wg, (const bf16_t*)wu, ids, (bf16_t*)act, K, ff, top, paired, n_real, act_kind, limit);
  else IFX_FAIL("moe_gate_up: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

extern "C" int ifx_moe_down(const void* act, const void* wd, const int* ids, const float* weights, void* out, int dtype, int T,
                            int N, int ff, int top, int n_real, const void* h, void* stream) {
  IFX_REQUIRE(T >= 0 && N > 0 && ff > 0 && top > 0, "moe_down: bad sizes T=%d N=%d ff=%d top=%d", T, N, ff, top);
  IFX_REQUIRE(h != nullptr, "moe_down: the rows themselves are needed (identity experts read them)");
  if (T == 0) return 0;
  const dim3 grid(T, (N + WAVES * ROWS_PER_WAVE - 1) / (WAVES * ROWS_PER_WAVE));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    hipLaunchKernelGGL(moe_down_kernel<float>, grid, dim3(WAVE * WAVES), 0, s, (const float*)act, (const float*)wd, ids, weights, (float*)out, N, ff, top, n_real, (const float*)h);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, dim3(WAVE * WAVES), 0, s, (const bf16_t*)act, (const bf16_t*)wd, ids, weights, (bf16_t*)out, N, ff, top, n_real, (const bf16_t*)h);
  else IFX_FAIL("moe_down: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
