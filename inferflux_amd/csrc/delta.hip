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
// [head][value column][d_pad] with d_pad = CH * KS >= d.  The columns of S never meet (column j is only ever read and
// written with v_j, u_j and o_j), so a head's columns are dealt to several workgroups of ``cols`` columns each, which
// spreads one request over many compute units.  In a workgroup thread (column j, run s) holds CH consecutive key channels
// of column j in registers; the KS threads of a column are neighbouring lanes and add their parts of S^T k and S^T q by
// butterfly shuffles (a fixed order).  Tokens are taken STAGE at a time: all threads load the stage's q, k and their
// columns of v into LDS (the next stage's are asked for before the walk and land in registers meanwhile), a few lanes per
// (token, vector) form the unit norms, a thread per token beta and the decay; everybody walks the stage's tokens and
// leaves o in LDS, from where it goes to ``o_raw`` [T, H dv] (float).  A second kernel, a wave per (token, head), norms and
// gates o.  The order of a token's operations does not depend on how the request was cut into steps, so results are
// bit-equal across cuttings.
#include "common.h"

IFX_DEFINE_LAST_ERROR()


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
  float* o_raw;           // [T, H dv]: the read-outs before their norm and gate
  int T, H, G, d, dv, KS, cols;
};

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

#define STAGE 16
#define MAX_DPAD 256
#define MAX_COLS 128
#define MAX_PRE 16          // q and k elements of a stage a thread fetches at most (STAGE * d_pad / threads)
#define MAX_PRE_V 8         // ... and v elements (STAGE * columns / threads)
//          // 16-byte-free prefetch: values a thread holds for the next stage (see below)

// The sum over the KS (a power of two) neighbouring lanes that share a column, in every one of them: neighbours within a
// row of 16 lanes swap through the lanes' own data paths (pairs, quads, mirrored halves of 8, mirrored rows of 16: a few
// cycles each, where a trip through the LDS crossbar costs a token's whole arithmetic); wider groups go on by shuffles.
// The order of the additions is fixed by the lane numbers.
#define DPP_OF(v, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), (ctrl), 0xF, 0xF, true))
// f[k] is 1 where the group has more than 2^k lanes and 0 where not: a step the group does not need adds nothing, and the
// walk has no branches for the steps within a row of 16 lanes.
struct LaneSteps { float f[4]; int lanes; };
__device__ __forceinline__ LaneSteps lane_steps(int KS) {
  return LaneSteps{{KS >= 2 ? 1.f : 0.f, KS >= 4 ? 1.f : 0.f, KS >= 8 ? 1.f : 0.f, KS >= 16 ? 1.f : 0.f}, KS};
}
__device__ __forceinline__ float column_sum(float v, const LaneSteps& st) {
  v = fmaf(st.f[0], DPP_OF(v, 0xB1), v);        // quad_perm [1, 0, 3, 2]
  v = fmaf(st.f[1], DPP_OF(v, 0x4E), v);        // quad_perm [2, 3, 0, 1]
  v = fmaf(st.f[2], DPP_OF(v, 0x141), v);       // row_half_mirror
  v = fmaf(st.f[3], DPP_OF(v, 0x140), v);       // row_mirror
  if (st.lanes >= 32) v += __shfl_xor(v, 16, WAVE);
  if (st.lanes >= 64) v += __shfl_xor(v, 32, WAVE);
  return v;
}

// A workgroup's meeting point for what it wrote to LDS: waits for the wave's own LDS operations and for the others, but
// not for loads from memory that are still on their way into registers (the next stage's), as __syncthreads() would.
#define LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

template <typename T, int CH>
__global__ __launch_bounds__(256) void delta_kernel(DeltaArgs a) {
  // LDS as the head's sizes need it (so that several workgroups share a compute unit): q and k of a stage [STAGE][dpad]
  // each, then its v and o [STAGE][cols] each
  extern __shared__ __attribute__((aligned(16))) float lds[];
  __shared__ float beta_s[STAGE + 1], g_s[STAGE + 1];      // (one more: the walk reads a token ahead, also behind the last)
  const int n_cb = (a.dv + a.cols - 1) / a.cols;
  const int h = blockIdx.x / n_cb, j0 = (blockIdx.x % n_cb) * a.cols, r = blockIdx.y;
  const int n = a.q_len[r];
  if (n <= 0) return;
  const int t0 = a.q_start[r];
  const int d = a.d, dv = a.dv, KS = a.KS, dpad = CH * KS;
  const int cols = min(a.cols, dv - j0);
  float* q_s = lds;
  float* k_s = lds + STAGE * dpad;
  float* v_s = lds + 2 * STAGE * dpad;
  float* o_s = v_s + STAGE * a.cols;
  const int g = h / (a.H / a.G);
  const int tid = threadIdx.x, nthr = blockDim.x;
  const int wid = tid / WAVE, lane = tid % WAVE, nw = (nthr + WAVE - 1) / WAVE;
  const int jl = tid / KS, s = tid % KS;             // this thread's column (within the workgroup's) and its run of channels
  const bool owner = jl < cols;
  float* Sp = a.state + (size_t)a.slots[r] * a.state_stride + a.state_offset + ((size_t)h * dv + j0 + (owner ? jl : 0)) * dpad + s * CH;
  float S[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) S[i] = owner ? Sp[i] : 0.f;
  const T* u = (const T*)a.u;
  const T* rows = (const T*)a.rows;
  const float decay_rate = expf(a.A_log[h]), dt_b = a.dt_bias[h], q_mult = 1.0f / sqrtf((float)d);
  const LaneSteps col_steps = lane_steps(KS);
  const int NL = nthr >= 256 ? 8 : (nthr >= 128 ? 4 : 2);      // lanes to a (token, vector) pair of a stage's 2 STAGE unit norms
  // What a thread fetches of a stage: elements x = tid, tid + nthr, ... of the stage's (token, channel) pairs of q and of k
  // and of its (token, column) pairs of v.  STAGE * dpad and STAGE * cols are at most MAX_PRE * nthr.
  // (dpad is a power of two; the places of a thread's v elements are the same in every stage and found once)
  const int per_qk = (STAGE * dpad + nthr - 1) / nthr, per_v = (STAGE * cols + nthr - 1) / nthr;
  const int dshift = __ffs(dpad) - 1;
  // a thread's v elements of a stage are x = tid, tid + nthr, ...: (token, column) = (x / cols, x % cols), stepped from the
  // first by (nthr / cols, nthr % cols) with a carry, so that one division a thread is all there is
  const int v_tt0 = tid / cols, v_c0 = tid - v_tt0 * cols, v_dq = nthr / cols, v_dr = nthr - v_dq * cols;
  float pq[MAX_PRE], pk[MAX_PRE], pv[MAX_PRE_V], pb = 0.f, pg = 0.f;
  auto fetch = [&](int base) {
    const int cnt = min(STAGE, n - base);
#pragma unroll
    for (int e = 0; e < MAX_PRE; ++e) {
      if (e >= per_qk) break;
      const int x = tid + e * nthr, tt = x >> dshift, c = x & (dpad - 1);
      const bool in = tt < cnt && c < d;
      const size_t row = (size_t)(t0 + base + (in ? tt : 0)) * a.ldu;
      pq[e] = in ? to_f(u[row + (size_t)g * d + c]) : 0.f;
      pk[e] = in ? to_f(u[row + (size_t)(a.G + g) * d + c]) : 0.f;
    }
    int tt = v_tt0, c = v_c0;
#pragma unroll
    for (int e = 0; e < MAX_PRE_V; ++e) {
      if (e >= per_v) break;
      const bool in = tt < cnt;
      pv[e] = in ? to_f(u[(size_t)(t0 + base + tt) * a.ldu + (size_t)2 * a.G * d + (size_t)h * dv + j0 + c]) : 0.f;
      tt += v_dq; c += v_dr;
      if (c >= cols) { c -= cols; ++tt; }
    }
    if (tid < cnt) {
      const size_t row = (size_t)(t0 + base + tid) * a.ldr;
      pb = to_f(rows[row + a.col_b + h]);
      pg = to_f(rows[row + a.col_a + h]);
    }
  };
  fetch(0);
  for (int base = 0; base < n; base += STAGE) {
    const int cnt = min(STAGE, n - base);
    LDS_BARRIER();              // the last stage's walk is done with q_s, k_s, v_s, its write-out with o_s
#pragma unroll
    for (int e = 0; e < MAX_PRE; ++e) {
      if (e >= per_qk) break;
      const int x = tid + e * nthr;
      if (x < STAGE * dpad) { q_s[x] = pq[e]; k_s[x] = pk[e]; }
    }
    {
      int tt = v_tt0, c = v_c0;
#pragma unroll
      for (int e = 0; e < MAX_PRE_V; ++e) {
        if (e >= per_v) break;
        if (tt < STAGE) v_s[tt * a.cols + c] = pv[e];
        tt += v_dq; c += v_dr;
        if (c >= cols) { c -= cols; ++tt; }
      }
    }
    if (tid < cnt) {
      beta_s[tid] = 1.0f / (1.0f + expf(-pb));
      g_s[tid] = expf(-decay_rate * softplus_f(pg + dt_b));
    }
    LDS_BARRIER();
    if (base + STAGE < n) fetch(base + STAGE);          // the next stage's loads are on their way during the norms and the walk
    // unit norms: NL neighbouring lanes per (token, q or k), all pairs at once; the lanes' squares added by column_sum
    {
      const LaneSteps norm_steps = lane_steps(NL);
      const int pair = tid / NL, l = tid % NL;
      float* vec = ((pair & 1) ? k_s : q_s) + min(pair >> 1, STAGE - 1) * dpad;
      const bool mine = pair < 2 * cnt;
      float ss = 0.f;
      if (mine)
        for (int c = l; c < d; c += NL) ss = fmaf(vec[c], vec[c], ss);
      ss = column_sum(ss, norm_steps);
      if (mine) {
        const float f = ((pair & 1) ? 1.0f : q_mult) / sqrtf(ss + 1e-6f);
        for (int c = l; c < d; c += NL) vec[c] *= f;
      }
    }
    LDS_BARRIER();
    if (owner) {
      // a token's k, q, v, decay and beta are read from LDS while the token before it is worked on; the sums over a
      // thread's channels run in four chains that are added at the end (a fixed order)
      const float* kp = k_s + s * CH;          // this thread's channels of the stage's first token; a token further: + dpad
      const float* qp = q_s + s * CH;
      const float* vp = v_s + jl;
      float kn[CH], qn[CH], vn = vp[0], gn = g_s[0], bn = beta_s[0];
#pragma unroll
      for (int i = 0; i < CH; ++i) { kn[i] = kp[i]; qn[i] = qp[i]; }
#pragma unroll 2
      for (int tt = 0; tt < cnt; ++tt) {
        float kk[CH], qq[CH];
        const float gd = gn, bt = bn, vt = vn;
#pragma unroll
        for (int i = 0; i < CH; ++i) { kk[i] = kn[i]; qq[i] = qn[i]; }
        // the token after this one, also behind the stage's last, where what is read lies inside the workgroup's LDS all the
        // same (the row behind q's last is k's first, behind k's last v's first, behind v's last o's first) and is never used
        kp += dpad; qp += dpad; vp += a.cols;
        vn = vp[0]; gn = g_s[tt + 1]; bn = beta_s[tt + 1];
#pragma unroll
        for (int i = 0; i < CH; ++i) { kn[i] = kp[i]; qn[i] = qp[i]; }
        float p4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          S[i] *= gd;
          p4[i & 3] = fmaf(S[i], kk[i], p4[i & 3]);
        }
        const float pred = column_sum((p4[0] + p4[1]) + (p4[2] + p4[3]), col_steps);
        const float upd = bt * (vt - pred);
        float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          S[i] = fmaf(kk[i], upd, S[i]);
          o4[i & 3] = fmaf(S[i], qq[i], o4[i & 3]);
        }
        const float out = column_sum((o4[0] + o4[1]) + (o4[2] + o4[3]), col_steps);
        if (s == 0) o_s[tt * a.cols + jl] = out;
      }
    }
    LDS_BARRIER();
    for (int x = tid; x < cnt * cols; x += nthr)
      a.o_raw[((size_t)(t0 + base + x / cols) * a.H + h) * dv + j0 + x % cols] = o_s[(x / cols) * a.cols + x % cols];
  }
  if (owner) {
#pragma unroll
    for (int i = 0; i < CH; ++i) Sp[i] = S[i];
  }
}

// out[t, h, :] = o_raw[t, h, :] / sqrt(mean(o_raw[t, h, :]^2) + eps) * w * silu(gate[t, h, :]): a wave per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void delta_finish_kernel(DeltaArgs a) {
  const size_t item = (size_t)blockIdx.x * (256 / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  if (item >= (size_t)a.T * a.H) return;
  const size_t t = item / a.H;
  const int h = (int)(item % a.H), dv = a.dv;
  const float* o = a.o_raw + item * dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += WAVE) ss = fmaf(o[c], o[c], ss);
  const float f = 1.0f / sqrtf(wave_sum(ss) / (float)dv + a.eps);
  const T* rows = (const T*)a.rows;
  for (int c = lane; c < dv; c += WAVE) {
    const float gt = to_f(rows[t * a.ldr + a.col_g + (size_t)h * dv + c]);
    ((T*)a.out)[item * dv + c] = from_f<T>(o[c] * f * load_dyn(a.norm_w, a.norm_dtype, c) * act_silu(gt));
  }
}

extern "C" int ifx_delta_rule(const void* u, int ldu, const void* rows, int ldr, int col_g, int col_b, int col_a, int dtype,
                              const float* A_log, const float* dt_bias, const void* norm_w, int norm_dtype, float eps, float* state,
                              long long state_stride, long long state_offset, const int* q_start, const int* q_len, const int* slots,
                              void* out, float* o_raw, int T, int R, int H, int G, int d, int dv, int ch, int ks, int cols, void* stream) {
  IFX_REQUIRE(R >= 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0, "delta_rule: bad sizes R=%d H=%d G=%d d=%d dv=%d", R, H, G, d, dv);
  IFX_REQUIRE(ks > 0 && ks <= WAVE && (ks & (ks - 1)) == 0, "delta_rule: %d threads to a column (a power of two up to %d)", ks, WAVE);
  IFX_REQUIRE(ch * ks >= d && ch * ks <= MAX_DPAD, "delta_rule: %d x %d channels for heads of %d (at most %d)", ch, ks, d, MAX_DPAD);
  IFX_REQUIRE(cols > 0 && cols <= MAX_COLS && cols * ks <= 256, "delta_rule: %d columns x %d threads do not fit a workgroup of 256", cols, ks);
  IFX_REQUIRE(STAGE * ch * ks <= MAX_PRE * 64 * ((cols * ks + 63) / 64) && STAGE * cols <= MAX_PRE_V * 64 * ((cols * ks + 63) / 64),
              "delta_rule: a stage of %d x %d channels and %d columns is more than its %d threads fetch", STAGE, ch * ks, cols, cols * ks);
  IFX_REQUIRE(T >= 0 && o_raw, "delta_rule: the read-outs need a place");
  IFX_REQUIRE(ldu >= 2 * G * d + H * dv && col_g >= 0 && col_b >= 0 && col_a >= 0, "delta_rule: rows too narrow");
  IFX_REQUIRE(state_stride >= state_offset + (long long)H * dv * ch * ks, "delta_rule: a state row of %lld floats is too short", state_stride);
  IFX_REQUIRE(R <= 65535, "delta_rule: too many requests for one launch");
  if (R == 0) return 0;
  DeltaArgs a{u, ldu, rows, ldr, col_g, col_b, col_a, A_log, dt_bias, norm_w, norm_dtype, eps, state, (size_t)state_stride,
              (size_t)state_offset, q_start, q_len, slots, out, o_raw, T, H, G, d, dv, ks, cols};
  const int threads = (cols * ks + WAVE - 1) / WAVE * WAVE;
  const dim3 grid(H * ((dv + cols - 1) / cols), R);
  hipStream_t s = (hipStream_t)stream;
  const size_t lds_bytes = ((size_t)2 * STAGE * (ch * ks + cols) + ch * ks) * sizeof(float);      // (+ a row: the walk reads a token ahead)
#define LAUNCH(TY, C) hipLaunchKernelGGL((delta_kernel<TY, C>), grid, dim3(threads), lds_bytes, s, a)
#define BY_CH(TY)                                             \
  do {                                                        \
    if (ch == 4) LAUNCH(TY, 4);                               \
    else if (ch == 8) LAUNCH(TY, 8);                          \
    else if (ch == 16) LAUNCH(TY, 16);                        \
    else if (ch == 32) LAUNCH(TY, 32);                        \
    else if (ch == 64) LAUNCH(TY, 64);                        \
    else IFX_FAIL("delta_rule: %d channels a thread (4, 8, 16, 32 or 64)", ch); \
  } while (0)
  if (dtype == DT_F32) BY_CH(float);
  else if (dtype == DT_BF16) BY_CH(bf16_t);
  else IFX_FAIL("delta_rule: unknown dtype %d", dtype);
#undef BY_CH
#undef LAUNCH
  if (T > 0) {
    const unsigned blocks = (unsigned)(((size_t)T * H + 256 / WAVE - 1) / (256 / WAVE));
    if (dtype == DT_F32) hipLaunchKernelGGL(delta_finish_kernel<float>, dim3(blocks), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(delta_finish_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, a);
  }
  IFX_LAUNCH_CHECK();
}
