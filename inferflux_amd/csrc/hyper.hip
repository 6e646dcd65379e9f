// Hyper-connections: instead of one residual stream a row carries S of them, [T, S, H] float.
//
// A sub-block q reads u = sum_s in_q[s] x_s, and after it the streams become, all at once from the old ones,
//   x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y          (mix indexed [from, to])
// One kernel does the update for the sub-block that has just run and the reading for the one that follows:
//   1. (if y) the new streams from the old ones and y; (if the source is one stream) S copies of it;
//   2. (if in) u = sum_t in[t] x_t of the new streams, and out = u / sqrt(mean(u^2) + eps) * w in the activation type;
//      without a norm weight out = u in float (the sum of the streams with in = 1).
// One workgroup per row; the row's u waits in LDS for its root mean square.  Everything is float; y comes in the
// activation type or as float partial sums that are added in slice order.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_STREAMS 8

struct HcArgs {
  const float* src;      // [T, S, H], or [T, H] with broadcast
  int broadcast;
  float* dst;            // [T, S, H] (may be src); null: nothing is written
  const void* y;         // [T, H] or null
  int y_dtype, n_slices;
  size_t slice_stride;
  float y_scale;
  const float* mix;      // [S, S]
  const float* outw;     // [S]
  const float* inw;      // [S] or null
  const void* norm_w;    // [H] or null
  int norm_dtype;
  float eps;
  void* out;             // [T, H]
  int out_dtype;
  int S, H;
};

template <int S_MAX>
__global__ __launch_bounds__(256) void hc_kernel(HcArgs a) {
  extern __shared__ float u_row[];       // [H]
  __shared__ float red[16];
  __shared__ float w_mix[MAX_STREAMS * MAX_STREAMS], w_out[MAX_STREAMS], w_in[MAX_STREAMS];
  const int S = a.S, H = a.H;
  const size_t t = blockIdx.x;
  if (threadIdx.x < S * S && a.y) w_mix[threadIdx.x] = a.mix[threadIdx.x];
  if (threadIdx.x < S) {
    w_out[threadIdx.x] = a.y ? a.outw[threadIdx.x] : 0.f;
    w_in[threadIdx.x] = a.inw ? a.inw[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const float* src = a.src + (a.broadcast ? t * H : t * S * H);
  float* dst = a.dst ? a.dst + t * S * H : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += 256) {
    float x[S_MAX];
#pragma unroll
    for (int s = 0; s < S_MAX; ++s) x[s] = s < S ? src[a.broadcast ? c : (size_t)s * H + c] : 0.f;
    if (a.y) {
      float y;
      if (a.n_slices > 1) {
        const float* part = (const float*)a.y + t * H + c;
        y = part[0];
        for (int k = 1; k < a.n_slices; ++k) y += part[(size_t)k * a.slice_stride];
      } else {
        y = load_dyn(a.y, a.y_dtype, t * H + c);
      }
      y *= a.y_scale;
      float n[S_MAX];
#pragma unroll
      for (int to = 0; to < S_MAX; ++to) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < S_MAX; ++s)
          if (s < S && to < S) v = fmaf(w_mix[s * S + to], x[s], v);
        n[to] = fmaf(w_out[to < S ? to : 0], y, v);
      }
#pragma unroll
      for (int s = 0; s < S_MAX; ++s) x[s] = n[s];
    }
    if (dst && (a.y || a.broadcast)) {
#pragma unroll
      for (int s = 0; s < S_MAX; ++s)
        if (s < S) dst[(size_t)s * H + c] = x[s];
    }
    if (a.inw) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < S_MAX; ++s)
        if (s < S) u = fmaf(w_in[s], x[s], u);
      u_row[c] = u;
      ss = fmaf(u, u, ss);
    }
  }
  if (!a.inw) return;
  if (!a.norm_w) {
    for (int c = threadIdx.x; c < H; c += 256) ((float*)a.out)[t * H + c] = u_row[c];     // (a thread reads what it wrote)
    return;
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)H + a.eps);
  for (int c = threadIdx.x; c < H; c += 256) {
    const float v = u_row[c] * inv * load_dyn(a.norm_w, a.norm_dtype, c);
    if (a.out_dtype == DT_F32) ((float*)a.out)[t * H + c] = v;
    else ((bf16_t*)a.out)[t * H + c] = (bf16_t)v;
  }
}

extern "C" int ifx_hyper_step(const float* src, int broadcast, float* dst, const void* y, int y_dtype, int n_slices,
                              long long slice_stride, float y_scale, const float* mix, const float* outw, const float* inw,
                              const void* norm_w, int norm_dtype, float eps, void* out, int out_dtype, int T, int S, int H,
                              void* stream) {
  IFX_REQUIRE(T >= 0 && S > 0 && S <= MAX_STREAMS && H > 0, "hyper_step: T=%d, %d streams (at most %d), H=%d", T, S, MAX_STREAMS, H);
  IFX_REQUIRE(H <= 16000, "hyper_step: a row of %d does not fit in LDS", H);
  IFX_REQUIRE(src && (!y || (mix && outw && dst)), "hyper_step: an update needs the mixing matrix, the output weights and somewhere to write");
  IFX_REQUIRE(!broadcast || dst || !y, "hyper_step: copies of one stream need somewhere to go");
  IFX_REQUIRE(!inw || out, "hyper_step: a reading needs an output");
  IFX_REQUIRE(n_slices >= 1 && (n_slices == 1 || (slice_stride > 0 && y)), "hyper_step: %d slices", n_slices);
  if (T == 0) return 0;
  HcArgs a{src, broadcast, dst, y, y_dtype, n_slices, (size_t)slice_stride, y_scale, mix, outw, inw, norm_w, norm_dtype, eps, out, out_dtype, S, H};
  const size_t lds = (size_t)H * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  if (S <= 1) hipLaunchKernelGGL(hc_kernel<1>, dim3(T), dim3(256), lds, s, a);
  else if (S <= 2) hipLaunchKernelGGL(hc_kernel<2>, dim3(T), dim3(256), lds, s, a);
  else if (S <= 4) hipLaunchKernelGGL(hc_kernel<4>, dim3(T), dim3(256), lds, s, a);
  else hipLaunchKernelGGL(hc_kernel<8>, dim3(T), dim3(256), lds, s, a);
  IFX_LAUNCH_CHECK();
}
