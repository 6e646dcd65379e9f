// The gated delta rule: a recurrence per head whose state is a matrix S [d, dv] that is decayed by one number per token
// and corrected towards the token's value along the token's key.
//
// For a request's tokens t = 0, 1, ... and value head h (which reads query/key head h / (heads / kv_heads)):
//
//   q = unit(q_in) * d^(-1/2),  k = unit(k_in),  unit(x) = x / sqrt(sum(x^2) + 1e-6)
//   beta = sigmoid(b_in),  g = exp(-exp(A_log[h]) * softplus(a_in + dt_bias[h]))
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q          (the read-out sees the token's own write)
//   out = o / sqrt(mean(o^2) + eps) * w_norm * silu(gate_in)              (the norm over the head's dv values)
//
// q_in, k_in, v come from ``u`` [T, ldu] (the convolution's output: q heads, then k heads, then v heads), gate_in, b_in,
// a_in from ``rows`` [T, ldr] at the given columns; all of them in the activation type.  Unit norms, beta, the decay and
// its logarithms, S, every sum, the norm and the gate are float whatever that type is.
//
// A request's S lives in its state slot, float32, at ``state_offset`` floats into the slot's row, laid out
// [head][value column][d_pad] with d_pad = CH * KS >= d.  A workgroup is one head of one request; thread (column j, run
// s) holds CH consecutive key channels of column j in registers, the KS threads of a column are neighbouring lanes and
// add their parts of S^T k and S^T q by butterfly shuffles (a fixed order).  Tokens are taken STAGE at a time: all
// threads load the stage's q, k, v into LDS, a wave per (token, vector) forms the unit norms, a thread per token beta
// and the decay; everybody walks the stage's tokens; a wave per token norms and gates o.  The order of a token's
// operations does not depend on how the request was cut into steps, so results are bit-equal across cuttings.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define STAGE 8
#define MAX_DPAD 256
#define MAX_DV 512

struct DeltaArgs {
  const void* u;          // [T, ldu]: q (G d) | k (G d) | v (H dv)
  int ldu;
  const void* rows;       // [T, ldr]: the gate's columns from col_g, beta's from col_b, the decay's from col_a
  int ldr, col_g, col_b, col_a;
  const float* A_log;     // [H]
  const float* dt_bias;   // [H]
  const void* norm_w;     // [dv]
  int norm_dtype;
  float eps;
  float* state;           // [slots, state_stride]
  size_t state_stride, state_offset;
  const int* q_start; const int* q_len; const int* slots;     // [R]
  void* out;              // [T, H dv]
  int H, G, d, dv, KS;
};

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <typename T, int CH>
__global__ __launch_bounds__(1024) void delta_kernel(DeltaArgs a) {
  __shared__ float q_s[STAGE][MAX_DPAD], k_s[STAGE][MAX_DPAD];
  __shared__ float v_s[STAGE][MAX_DV], o_s[STAGE][MAX_DV];
  __shared__ float beta_s[STAGE], g_s[STAGE];
  const int h = blockIdx.x, r = blockIdx.y;
  const int n = a.q_len[r];
  if (n <= 0) return;
  const int t0 = a.q_start[r];
  const int d = a.d, dv = a.dv, KS = a.KS, dpad = CH * KS;
  const int g = h / (a.H / a.G);
  const int tid = threadIdx.x, nthr = blockDim.x;
  const int wid = tid / WAVE, lane = tid % WAVE, nw = (nthr + WAVE - 1) / WAVE;
  const int j = tid / KS, s = tid % KS;              // this thread's column of S and its run of channels
  const bool owner = j < dv;
  float* Sp = a.state + (size_t)a.slots[r] * a.state_stride + a.state_offset + ((size_t)h * dv + (owner ? j : 0)) * dpad + s * CH;
  float S[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) S[i] = owner ? Sp[i] : 0.f;
  const T* u = (const T*)a.u;
  const T* rows = (const T*)a.rows;
  const float decay_rate = expf(a.A_log[h]), dt_b = a.dt_bias[h], q_mult = 1.0f / sqrtf((float)d);

  for (int base = 0; base < n; base += STAGE) {
    const int cnt = min(STAGE, n - base);
    __syncthreads();            // the last stage's output pass is done with o_s, its walk with q_s, k_s, v_s
    for (int x = tid; x < cnt * dpad; x += nthr) {
      const int tt = x / dpad, c = x % dpad;
      const size_t row = (size_t)(t0 + base + tt) * a.ldu;
      q_s[tt][c] = c < d ? to_f(u[row + (size_t)g * d + c]) : 0.f;
      k_s[tt][c] = c < d ? to_f(u[row + (size_t)(a.G + g) * d + c]) : 0.f;
    }
    for (int x = tid; x < cnt * dv; x += nthr) {
      const int tt = x / dv, c = x % dv;
      v_s[tt][c] = to_f(u[(size_t)(t0 + base + tt) * a.ldu + (size_t)2 * a.G * d + (size_t)h * dv + c]);
    }
    if (tid < cnt) {
      const size_t row = (size_t)(t0 + base + tid) * a.ldr;
      beta_s[tid] = 1.0f / (1.0f + expf(-to_f(rows[row + a.col_b + h])));
      g_s[tid] = expf(-decay_rate * softplus_f(to_f(rows[row + a.col_a + h]) + dt_b));
    }
    __syncthreads();
    // unit norms: a wave per (token, q or k); the lanes' squares added by the wave's butterfly
    for (int x = wid; x < 2 * cnt; x += nw) {
      float* vec = (x & 1) ? k_s[x >> 1] : q_s[x >> 1];
      float ss = 0.f;
      for (int c = lane; c < d; c += WAVE) ss = fmaf(vec[c], vec[c], ss);
      const float f = ((x & 1) ? 1.0f : q_mult) / sqrtf(wave_sum(ss) + 1e-6f);
      for (int c = lane; c < d; c += WAVE) vec[c] *= f;
    }
    __syncthreads();
    if (owner) {
      for (int tt = 0; tt < cnt; ++tt) {
        const float gd = g_s[tt], bt = beta_s[tt];
        const float* kk = k_s[tt] + s * CH;
        const float* qq = q_s[tt] + s * CH;
        float pred = 0.f;
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          S[i] *= gd;
          pred = fmaf(S[i], kk[i], pred);
        }
        for (int o = 1; o < KS; o <<= 1) pred += __shfl_xor(pred, o, WAVE);
        const float upd = bt * (v_s[tt][j] - pred);
        float out = 0.f;
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          S[i] = fmaf(kk[i], upd, S[i]);
          out = fmaf(S[i], qq[i], out);
        }
        for (int o = 1; o < KS; o <<= 1) out += __shfl_xor(out, o, WAVE);
        if (s == 0) o_s[tt][j] = out;
      }
    }
    __syncthreads();
    // the head's norm and gate: a wave per token
    for (int tt = wid; tt < cnt; tt += nw) {
      float ss = 0.f;
      for (int c = lane; c < dv; c += WAVE) ss = fmaf(o_s[tt][c], o_s[tt][c], ss);
      const float f = 1.0f / sqrtf(wave_sum(ss) / (float)dv + a.eps);
      const size_t row = (size_t)(t0 + base + tt);
      for (int c = lane; c < dv; c += WAVE) {
        const float gt = to_f(rows[row * a.ldr + a.col_g + (size_t)h * dv + c]);
        ((T*)a.out)[(row * a.H + h) * dv + c] = from_f<T>(o_s[tt][c] * f * load_dyn(a.norm_w, a.norm_dtype, c) * act_silu(gt));
      }
    }
  }
  if (owner) {
#pragma unroll
    for (int i = 0; i < CH; ++i) Sp[i] = S[i];
  }
}

extern "C" int ifx_delta_rule(const void* u, int ldu, const void* rows, int ldr, int col_g, int col_b, int col_a, int dtype,
                              const float* A_log, const float* dt_bias, const void* norm_w, int norm_dtype, float eps, float* state,
                              long long state_stride, long long state_offset, const int* q_start, const int* q_len, const int* slots,
                              void* out, int R, int H, int G, int d, int dv, int ch, int ks, void* stream) {
  IFX_REQUIRE(R >= 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0, "delta_rule: bad sizes R=%d H=%d G=%d d=%d dv=%d", R, H, G, d, dv);
  IFX_REQUIRE(ks > 0 && ks <= WAVE && (ks & (ks - 1)) == 0, "delta_rule: %d threads to a column (a power of two up to %d)", ks, WAVE);
  IFX_REQUIRE(ch * ks >= d && ch * ks <= MAX_DPAD, "delta_rule: %d x %d channels for heads of %d (at most %d)", ch, ks, d, MAX_DPAD);
  IFX_REQUIRE(dv <= MAX_DV && (long long)dv * ks <= 1024, "delta_rule: %d columns x %d threads do not fit a workgroup", dv, ks);
  IFX_REQUIRE(ldu >= 2 * G * d + H * dv && col_g >= 0 && col_b >= 0 && col_a >= 0, "delta_rule: rows too narrow");
  IFX_REQUIRE(state_stride >= state_offset + (long long)H * dv * ch * ks, "delta_rule: a state row of %lld floats is too short", state_stride);
  IFX_REQUIRE(R <= 65535, "delta_rule: too many requests for one launch");
  if (R == 0) return 0;
  DeltaArgs a{u, ldu, rows, ldr, col_g, col_b, col_a, A_log, dt_bias, norm_w, norm_dtype, eps, state, (size_t)state_stride,
              (size_t)state_offset, q_start, q_len, slots, out, H, G, d, dv, ks};
  const int threads = (dv * ks + WAVE - 1) / WAVE * WAVE;
  const dim3 grid(H, R);
  hipStream_t s = (hipStream_t)stream;
#define LAUNCH(TY, C) hipLaunchKernelGGL((delta_kernel<TY, C>), grid, dim3(threads), 0, s, a)
#define BY_CH(TY)                                             \
  do {                                                        \
    if (ch == 8) LAUNCH(TY, 8);                               \
    else if (ch == 16) LAUNCH(TY, 16);                        \
    else if (ch == 32) LAUNCH(TY, 32);                        \
    else if (ch == 64) LAUNCH(TY, 64);                        \
    else IFX_FAIL("delta_rule: %d channels a thread (8, 16, 32 or 64)", ch); \
  } while (0)
  if (dtype == DT_F32) BY_CH(float);
  else if (dtype == DT_BF16) BY_CH(bf16_t);
  else IFX_FAIL("delta_rule: unknown dtype %d", dtype);
#undef BY_CH
#undef LAUNCH
  IFX_LAUNCH_CHECK();
}
