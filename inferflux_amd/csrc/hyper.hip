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

// The same for rows whose width is a multiple of 4: a thread takes 4 neighbouring columns a trip, in 16-byte pieces (8-byte ones
// for y in bfloat16), and asks for everything a trip reads before it uses any of it: steps of few rows are a chain of
// trips to memory otherwise.  (A stream's element is read and written by the same thread, so updating in place is safe.)
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 hc_bf16x4;

template <int S_MAX>
__global__ __launch_bounds__(512) void hc_vec_kernel(HcArgs a) {
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
  const bool y_bf16 = a.y && a.n_slices == 1 && a.y_dtype == DT_BF16;
  const int stride = blockDim.x * 4;
  float ss = 0.f;
  for (int c = threadIdx.x * 4; c < H; c += stride) {
    float4 x[S_MAX];
    if (a.broadcast) {
      const float4 v = *(const float4*)(src + c);
#pragma unroll
      for (int s = 0; s < S_MAX; ++s) x[s] = v;
    } else {
#pragma unroll
      for (int s = 0; s < S_MAX; ++s) x[s] = s < S ? *(const float4*)(src + (size_t)s * H + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (a.y) {
      float4 y;
      if (y_bf16) {
        const hc_bf16x4 v = *(const hc_bf16x4*)((const bf16_t*)a.y + t * H + c);
        y = make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
      } else {                            // float, or float partial sums added in slice order
        const float* part = (const float*)a.y + t * H + c;
        y = *(const float4*)part;
        for (int k = 1; k < a.n_slices; ++k) {
          const float4 v = *(const float4*)(part + (size_t)k * a.slice_stride);
          y.x += v.x; y.y += v.y; y.z += v.z; y.w += v.w;
        }
      }
      y.x *= a.y_scale; y.y *= a.y_scale; y.z *= a.y_scale; y.w *= a.y_scale;
      float4 n[S_MAX];
#pragma unroll
      for (int to = 0; to < S_MAX; ++to) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int s = 0; s < S_MAX; ++s)
          if (s < S && to < S) {
            const float m = w_mix[s * S + to];
            v.x = fmaf(m, x[s].x, v.x); v.y = fmaf(m, x[s].y, v.y); v.z = fmaf(m, x[s].z, v.z); v.w = fmaf(m, x[s].w, v.w);
          }
        const float o = w_out[to < S ? to : 0];
        n[to] = make_float4(fmaf(o, y.x, v.x), fmaf(o, y.y, v.y), fmaf(o, y.z, v.z), fmaf(o, y.w, v.w));
      }
#pragma unroll
      for (int s = 0; s < S_MAX; ++s) x[s] = n[s];
    }
    if (dst && (a.y || a.broadcast)) {
#pragma unroll
      for (int s = 0; s < S_MAX; ++s)
        if (s < S) *(float4*)(dst + (size_t)s * H + c) = x[s];
    }
    if (a.inw) {
      float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int s = 0; s < S_MAX; ++s)
        if (s < S) {
          const float w = w_in[s];
          u.x = fmaf(w, x[s].x, u.x); u.y = fmaf(w, x[s].y, u.y); u.z = fmaf(w, x[s].z, u.z); u.w = fmaf(w, x[s].w, u.w);
        }
      *(float4*)(u_row + c) = u;
      ss = fmaf(u.x, u.x, ss); ss = fmaf(u.y, u.y, ss); ss = fmaf(u.z, u.z, ss); ss = fmaf(u.w, u.w, ss);
    }
  }
  if (!a.inw) return;
  if (!a.norm_w) {
    for (int c = threadIdx.x * 4; c < H; c += stride) *(float4*)((float*)a.out + t * H + c) = *(const float4*)(u_row + c);     // (a thread reads what it wrote)
    return;
  }
  const float inv = rsqrtf(block_sum(ss, red) / (float)H + a.eps);
  for (int c = threadIdx.x * 4; c < H; c += stride) {
    const float4 u = *(const float4*)(u_row + c);
    float v[4] = {u.x * inv, u.y * inv, u.z * inv, u.w * inv};
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= load_dyn(a.norm_w, a.norm_dtype, c + e);
    if (a.out_dtype == DT_F32) {
      *(float4*)((float*)a.out + t * H + c) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
      hc_bf16x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (__bf16)v[e];
      *(hc_bf16x4*)((bf16_t*)a.out + t * H + c) = o;
    }
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
  const auto aligned = [](const void* p) { return ((size_t)p & 15) == 0; };
  const bool y_halves = n_slices == 1 && y_dtype == DT_BF16;
  const bool vec = H % 4 == 0 && aligned(src) && aligned(dst) && aligned(out) && (n_slices == 1 || slice_stride % 4 == 0) &&
                   (y_halves ? ((size_t)y & 7) == 0 : aligned(y));
  if (vec) {
    // (a thread per 4 columns up to 512 threads: a step of few rows has one trip to memory instead of several in a row)
    const int threads = min(512, ((H / 4 + WAVE - 1) / WAVE) * WAVE);
    if (S <= 1) hipLaunchKernelGGL(hc_vec_kernel<1>, dim3(T), dim3(threads), lds, s, a);
    else if (S <= 2) hipLaunchKernelGGL(hc_vec_kernel<2>, dim3(T), dim3(threads), lds, s, a);
    else if (S <= 4) hipLaunchKernelGGL(hc_vec_kernel<4>, dim3(T), dim3(threads), lds, s, a);
    else hipLaunchKernelGGL(hc_vec_kernel<8>, dim3(T), dim3(threads), lds, s, a);
    IFX_LAUNCH_CHECK();
  }
  if (S <= 1) hipLaunchKernelGGL(hc_kernel<1>, dim3(T), dim3(256), lds, s, a);
  else if (S <= 2) hipLaunchKernelGGL(hc_kernel<2>, dim3(T), dim3(256), lds, s, a);
  else if (S <= 4) hipLaunchKernelGGL(hc_kernel<4>, dim3(T), dim3(256), lds, s, a);
  else hipLaunchKernelGGL(hc_kernel<8>, dim3(T), dim3(256), lds, s, a);
  IFX_LAUNCH_CHECK();
}
