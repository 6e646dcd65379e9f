// Small kernels over a step's rows that sit between products:
//   activation     out = act(x), act the tanh form of gelu or silu (a feed-forward without a gate); x may be a product's
//                  float partial sums
//   sigmoid_gate   out[t, c] = x[t, c] * sigmoid(g[t, c]), g columns of a wider projected row (or float partial sums of it)
//   gated_add      out[t, c] = sum_slices base[.][t, c] + sigmoid(h[t] . w) * extra[t, c]: a branch that every row takes,
//                  weighted by one number per row, added to the sum of the other branches
//   scale_softcap  x <- cap * tanh(x * scale / cap) in place on float rows (cap 0: x <- x * scale)
//   stream_add     x[t, c] <- x[t, c] + rows[t, c] + vec[c] in place on the float stream: what a pass of a looped span of
//                  layers feeds into the stream before its first layer (either operand may be absent)
//   diff_expand    q [T][H][2 d] -> [T][2 H][2 d]: head 2 h holds [q1 | 0] and head 2 h + 1 holds [0 | q2], so that attention
//                  kernels for heads of 2 d elements score each half against its half of the keys' rows [k1 | k2]
//   diff_combine   out[t, h, :] = o / sqrt(mean(o^2) + eps) * out_scale with o = a[t, 2 h, :] - lambda a[t, 2 h + 1, :]: the two
//                  maps of differential attention joined, a wave per (row, head)
// All arithmetic is float.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(const T* __restrict__ x, T* __restrict__ out, size_t n, int act) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = to_f(x[i]);
  out[i] = from_f<T>(act == ACT_GELU_TANH ? act_gelu_tanh(v) : act_silu(v));
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 row_bf16x8;

__global__ __launch_bounds__(256) void activation_bf16x8_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out, size_t n8, int act) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const row_bf16x8 v = ((const row_bf16x8*)x)[i];
  row_bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float f = (float)v[e];
    o[e] = (__bf16)(act == ACT_GELU_TANH ? act_gelu_tanh(f) : act_silu(f));
  }
  ((row_bf16x8*)out)[i] = o;
}

extern "C" int ifx_activation(const void* x, void* out, int dtype, long long n, int act, void* stream) {
  IFX_REQUIRE(n >= 0 && (act == ACT_SILU || act == ACT_GELU_TANH), "activation: n=%lld act=%d", n, act);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_BF16 && n % 8 == 0)
    hipLaunchKernelGGL(activation_bf16x8_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s, (const bf16_t*)x, (bf16_t*)out, (size_t)(n / 8), act);
  else if (dtype == DT_BF16)
    hipLaunchKernelGGL(activation_kernel<bf16_t>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const bf16_t*)x, (bf16_t*)out, (size_t)n, act);
  else if (dtype == DT_F32)
    hipLaunchKernelGGL(activation_kernel<float>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const float*)x, (float*)out, (size_t)n, act);
  else IFX_FAIL("activation: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

// act of a product left as float partial sums [n_slices][n] (added in slice order), written in the activation type
template <typename T>
__global__ __launch_bounds__(256) void activation_slices_kernel(const float* __restrict__ parts, int n_slices, size_t stride,
                                                                T* __restrict__ out, size_t n4, int act) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  float4 v = ((const float4*)parts)[i];
  for (int k = 1; k < n_slices; ++k) {
    const float4 w = *(const float4*)(parts + (size_t)k * stride + i * 4);
    v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
  }
  const float f[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) out[i * 4 + e] = from_f<T>(act == ACT_GELU_TANH ? act_gelu_tanh(f[e]) : act_silu(f[e]));
}

extern "C" int ifx_activation_slices(const float* parts, int n_slices, long long stride, void* out, int out_dtype, long long n,
                                     int act, void* stream) {
  IFX_REQUIRE(n >= 0 && n % 4 == 0 && stride % 4 == 0 && n_slices >= 1 && (act == ACT_SILU || act == ACT_GELU_TANH),
              "activation_slices: n=%lld stride=%lld slices=%d act=%d", n, stride, n_slices, act);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)((n / 4 + 255) / 256);
  if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(activation_slices_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, parts, n_slices, (size_t)stride, (bf16_t*)out, (size_t)(n / 4), act);
  else if (out_dtype == DT_F32)
    hipLaunchKernelGGL(activation_slices_kernel<float>, dim3(blocks), dim3(256), 0, s, parts, n_slices, (size_t)stride, (float*)out, (size_t)(n / 4), act);
  else IFX_FAIL("activation_slices: unknown dtype %d", out_dtype);
  IFX_LAUNCH_CHECK();
}

// x [T, C] of type T; g: columns g_col .. g_col + C - 1 of rows ld apart, of type T, or (n_slices > 1) float partial sums
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(const T* __restrict__ x, const void* __restrict__ g, int ld, int g_col,
                                                           int n_slices, size_t slice_stride, T* __restrict__ out, int C, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / C;
  const int c = (int)(i % C);
  float gv;
  if (n_slices > 1) {
    const float* p = (const float*)g + t * ld + g_col + c;
    gv = p[0];
    for (int k = 1; k < n_slices; ++k) gv += p[(size_t)k * slice_stride];
  } else {
    gv = to_f(((const T*)g)[t * ld + g_col + c]);
  }
  out[i] = from_f<T>(to_f(x[i]) / (1.0f + expf(-gv)));
}

extern "C" int ifx_sigmoid_gate(const void* x, const void* g, int ld, int g_col, int n_slices, long long slice_stride, void* out,
                                int dtype, int T, int C, void* stream) {
  IFX_REQUIRE(T >= 0 && C > 0 && ld >= g_col + C && g_col >= 0 && n_slices >= 1, "sigmoid_gate: T=%d C=%d ld=%d g_col=%d", T, C, ld, g_col);
  if (T == 0) return 0;
  const size_t n = (size_t)T * C;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)x, g, ld, g_col, n_slices, (size_t)slice_stride, (bf16_t*)out, C, n);
  else if (dtype == DT_F32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, s, (const float*)x, g, ld, g_col, n_slices, (size_t)slice_stride, (float*)out, C, n);
  else IFX_FAIL("sigmoid_gate: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

// One workgroup per row: the row's gate sigmoid(h . w) in float (1 where w is null), then out = sum of the base slices + gate * extra.
template <typename T>
__global__ __launch_bounds__(256) void gated_add_kernel(const void* __restrict__ base, int base_f32, int n_slices, size_t slice_stride,
                                                        const void* __restrict__ extra, int extra_f32, int extra_slices, size_t extra_stride,
                                                        const T* __restrict__ h, const T* __restrict__ w, int K, T* __restrict__ out, int N) {
  __shared__ float red[16];
  const size_t t = blockIdx.x;
  float gate = 1.0f;                 // (without a gate's weight the branch is added as it is)
  if (w) {
    float z = 0.f;
    for (int k = threadIdx.x; k < K; k += 256) z = fmaf(to_f(h[t * K + k]), to_f(w[k]), z);
    gate = 1.0f / (1.0f + expf(-block_sum(z, red)));
  }
  for (int c = threadIdx.x; c < N; c += 256) {
    float b;
    if (base_f32) {
      const float* p = (const float*)base + t * N + c;
      b = p[0];
      for (int k = 1; k < n_slices; ++k) b += p[(size_t)k * slice_stride];
    } else {
      b = to_f(((const T*)base)[t * N + c]);
    }
    float e;
    if (extra_f32) {
      const float* p = (const float*)extra + t * N + c;
      e = p[0];
      for (int k = 1; k < extra_slices; ++k) e += p[(size_t)k * extra_stride];
    } else {
      e = to_f(((const T*)extra)[t * N + c]);
    }
    out[t * N + c] = from_f<T>(fmaf(gate, e, b));
  }
}

extern "C" int ifx_gated_add(const void* base, int base_f32, int n_slices, long long slice_stride, const void* extra, int extra_f32,
                             int extra_slices, long long extra_stride, const void* h, const void* w, int K, void* out, int dtype,
                             int T, int N, void* stream) {
  IFX_REQUIRE(T >= 0 && N > 0 && K > 0 && n_slices >= 1 && extra_slices >= 1, "gated_add: T=%d N=%d K=%d", T, N, K);
  IFX_REQUIRE((n_slices == 1 || base_f32) && (extra_slices == 1 || extra_f32), "gated_add: partial sums are float");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(gated_add_kernel<bf16_t>, dim3(T), dim3(256), 0, s, base, base_f32, n_slices, (size_t)slice_stride, extra, extra_f32,
                       extra_slices, (size_t)extra_stride, (const bf16_t*)h, (const bf16_t*)w, K, (bf16_t*)out, N);
  else if (dtype == DT_F32)
    hipLaunchKernelGGL(gated_add_kernel<float>, dim3(T), dim3(256), 0, s, base, 1, n_slices, (size_t)slice_stride, extra, 1,
                       extra_slices, (size_t)extra_stride, (const float*)h, (const float*)w, K, (float*)out, N);
  else IFX_FAIL("gated_add: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

__global__ __launch_bounds__(256) void scale_softcap_kernel(float* __restrict__ x, size_t n, float scale, float cap) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = x[i] * scale;
  x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

extern "C" int ifx_scale_softcap(float* x, long long n, float scale, float cap, void* stream) {
  IFX_REQUIRE(n >= 0 && cap >= 0.f, "scale_softcap: n=%lld cap=%g", n, (double)cap);
  if (n == 0) return 0;
  hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, (size_t)n, scale, cap);
  IFX_LAUNCH_CHECK();
}

// x [T][H] float, rows [T][H] float or null, vec [H] of any type or null
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ x, const float* __restrict__ rows, const void* __restrict__ vec,
                                                         int vec_dtype, int H, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (rows) v += rows[i];
  if (vec) v += load_dyn(vec, vec_dtype, i % H);
  x[i] = v;
}

extern "C" int ifx_stream_add(float* x, const float* rows, const void* vec, int vec_dtype, int T, int H, void* stream) {
  IFX_REQUIRE(T >= 0 && H > 0, "stream_add: bad sizes T=%d H=%d", T, H);
  if (T == 0 || (!rows && !vec)) return 0;
  const size_t n = (size_t)T * H;
  hipLaunchKernelGGL(stream_add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, rows, vec, vec_dtype, H, n);
  IFX_LAUNCH_CHECK();
}

template <typename T>
__global__ __launch_bounds__(256) void diff_expand_kernel(const T* __restrict__ q, T* __restrict__ out, int d, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;        // an element of out
  if (i >= n) return;
  const int e = (int)(i % (2 * d));
  const size_t head2 = i / (2 * d);                               // (row, head, map)
  const int map = (int)(head2 & 1);
  out[i] = (e >= d) == (map == 1) ? q[(head2 >> 1) * 2 * d + e] : from_f<T>(0.f);
}

extern "C" int ifx_diff_expand(const void* q, void* out, int dtype, long long rows_heads, int d, void* stream) {
  IFX_REQUIRE(rows_heads >= 0 && d > 0, "diff_expand: bad sizes");
  const size_t n = (size_t)rows_heads * 4 * d;
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == DT_BF16) hipLaunchKernelGGL(diff_expand_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)q, (bf16_t*)out, d, n);
  else if (dtype == DT_F32) hipLaunchKernelGGL(diff_expand_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)q, (float*)out, d, n);
  else IFX_FAIL("diff_expand: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const T* __restrict__ a, T* __restrict__ out, size_t items, int dv, float lambda,
                                                           float out_scale, float eps) {
  const size_t item = (size_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;       // (row, head)
  const int lane = threadIdx.x % WAVE;
  if (item >= items) return;
  const T* a1 = a + item * 2 * dv;
  const T* a2 = a1 + dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += WAVE) {
    const float o = to_f(a1[c]) - lambda * to_f(a2[c]);
    ss = fmaf(o, o, ss);
  }
  const float f = out_scale / sqrtf(wave_sum(ss) / (float)dv + eps);
  for (int c = lane; c < dv; c += WAVE) out[item * dv + c] = from_f<T>((to_f(a1[c]) - lambda * to_f(a2[c])) * f);
}

extern "C" int ifx_diff_combine(const void* a, void* out, int dtype, long long rows_heads, int dv, float lambda, float out_scale, float eps,
                                void* stream) {
  IFX_REQUIRE(rows_heads >= 0 && dv > 0, "diff_combine: bad sizes");
  if (rows_heads == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const unsigned blocks = (unsigned)((rows_heads + 256 / WAVE - 1) / (256 / WAVE));
  if (dtype == DT_BF16)
    hipLaunchKernelGGL(diff_combine_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)a, (bf16_t*)out, (size_t)rows_heads, dv, lambda, out_scale, eps);
  else if (dtype == DT_F32)
    hipLaunchKernelGGL(diff_combine_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)a, (float*)out, (size_t)rows_heads, dv, lambda, out_scale, eps);
  else IFX_FAIL("diff_combine: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
