// Gated linear attention: a recurrence per head whose state is a matrix and whose decay is a vector per token.
//
// For a request's tokens t = 0, 1, ..., per head, with keys and queries of d channels and values of dv:
//   alpha_t[i] = sigmoid(z_t[i] + b[i]) ^ (1 / tau) = exp(-softplus(-(z_t[i] + b[i])) / tau)
//   S_t[i, j]  = alpha_t[i] S_(t-1)[i, j] + k_t[i] v_t[j],        S_(-1) = 0
//   o_t[j]     = sum_i S_t[i, j] q_t[i] * q_scale
//   y_t[j]     = o_t[j] / sqrt(mean_j o_t[j]^2 + eps) * w[j] * silu(g_t[j])
//
// Rows are a step's flattened rows (requests end to end, a request's rows in position order).  q, k, v and g are columns
// of one projected row (the activation type, ld apart); z is float (the decay's second product, without its bias).
// Decays, their logarithms, S, o, the norm and the gate are float whatever the activation type.
//
// A request's S lives in its state slot, one float32 row per slot laid out [head][j][PARTS * DP]: a column j of S as
// PARTS runs of DP channels (channels at or beyond d are zero and stay zero).  A thread owns one run of one column (of two
// neighbouring columns where DP <= 32): DP (2 DP) numbers of S in registers; the PARTS threads of a column are neighbours in a wave and add their parts of o_t[j] by shuffles in a fixed
// order.  A workgroup is one head of one request (or of one chunk): dv * PARTS threads.  Tokens are taken STAGE at a time:
// the threads put q, k and alpha of the stage's tokens into LDS, a (token, channel) each (and form alpha on the way), everybody walks the
// stage's tokens, o goes to LDS, and a wave per token norms and gates it.
//
// MODE 0: a request's rows in one walk, from its slot and back into it.
// Long portions are cut into chunks that run side by side (the recurrence is linear in S):
// MODE 1: a chunk from S = 0; records its final S and the sum of its log alpha per channel.
// gla_combine: walks a request's chunks: chunk c's record becomes the state chunk c starts from,
//              S <- exp(sum log alpha) S + S_c; the request's new state goes into its slot.
// MODE 2: a chunk from the state it starts from; writes y.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define STAGE 8

struct GlaArgs {
  const void* rows;        // [T, ld] of the activation type
  int ld, q_col, k_col, v_col, g_col;
  const float* z;          // [T, H * d]
  const float* z_bias;     // [H * d] or null
  float inv_tau, q_scale, eps;
  const void* norm_w;      // [dv]
  int norm_dtype;
  float* state;            // [slots, state_stride]; S at state_offset of a row
  size_t state_stride, state_offset;
  const int* q_start;      // [R]
  const int* q_len;        // [R]
  const int* slots;        // [R]
  void* out;               // [T, H * dv] of the activation type
  int H, d, dv, parts;
  // chunks (MODE 1, 2)
  const int* chunk_req;    // [n_chunks]
  const int* chunk_t0;     // [n_chunks] first row
  const int* chunk_len;    // [n_chunks]
  float* chunk_state;      // [n_chunks, H * dv * parts * DP]
  float* chunk_loga;       // [n_chunks, H * d]
};

__device__ __forceinline__ float log_sigmoid(float x) {      // -softplus(-x), without overflow
  return x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
}

// (a thread's registers hold DP numbers of S: the more of them, the fewer threads a workgroup may have)
#define GLA_MAX_THREADS(DP) ((DP) <= 32 ? 1024 : ((DP) <= 64 ? 512 : 256))

template <typename T, int DP, int MODE, int COLS>
__global__ __launch_bounds__(GLA_MAX_THREADS(DP)) void gla_kernel(GlaArgs a) {
  extern __shared__ float lds[];
  const int d = a.d, dv = a.dv, parts = a.parts, H = a.H;
  float* lq = lds;                       // [STAGE][d]
  float* lk = lq + STAGE * d;            // [STAGE][d]
  float* la = lk + STAGE * d;            // [STAGE][d]
  float* lo = la + STAGE * d;            // [STAGE][dv]
  float* lg = lo + STAGE * dv;           // [STAGE][d]: the decays' logarithms (MODE 1 sums them per channel)
  const int unit = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  int t0, n;
  size_t s_at;                            // where this head's S lies
  float* sbase;
  if (MODE == 0) {
    t0 = a.q_start[unit]; n = a.q_len[unit];
    sbase = a.state + (size_t)a.slots[unit] * a.state_stride + a.state_offset;
  } else {
    t0 = a.chunk_t0[unit]; n = a.chunk_len[unit];
    sbase = a.chunk_state + (size_t)unit * H * dv * parts * DP;
  }
  if (n <= 0) return;
  s_at = (size_t)head * dv * parts * DP;
  // a thread owns COLS neighbouring columns j0 .. j0 + COLS - 1 of S for its run of DP channels: what it reads of a token's
  // q, k and decays from LDS serves COLS columns
  const int j0 = (tid / parts) * COLS, p = tid % parts;
  float S[COLS][DP];
  float* sp = sbase + s_at + ((size_t)j0 * parts + p) * DP;          // (column j0 + c lies c * parts * DP further)
#pragma unroll
  for (int c = 0; c < COLS; ++c) {
    if (MODE != 1 && j0 + c < dv) {
#pragma unroll
      for (int i = 0; i < DP; i += 4) {
        const float4 v = *(const float4*)(sp + (size_t)c * parts * DP + i);
        S[c][i] = v.x; S[c][i + 1] = v.y; S[c][i + 2] = v.z; S[c][i + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < DP; ++i) S[c][i] = 0.f;
    }
  }
  const T* rows = (const T*)a.rows;
  const int wid = tid / WAVE, lane = tid % WAVE, nw = (blockDim.x + WAVE - 1) / WAVE;
  float loga_sum = 0.f;
  for (int s0 = 0; s0 < n; s0 += STAGE) {
    const int ns = min(STAGE, n - s0);
    // the stage's q, k and decays: one (token, channel) a thread and trip, neighbouring threads on neighbouring channels
    for (int it = tid; it < ns * d; it += blockDim.x) {
      const int tt = it / d, ch = it - tt * d;
      const size_t t = (size_t)(t0 + s0 + tt);
      const float zq = a.z[t * (size_t)(H * d) + head * d + ch] + (a.z_bias ? a.z_bias[head * d + ch] : 0.f);
      const float kq = to_f(rows[t * a.ld + a.k_col + head * d + ch]);
      const float qq = MODE == 1 ? 0.f : to_f(rows[t * a.ld + a.q_col + head * d + ch]);
      const float la_t = log_sigmoid(zq) * a.inv_tau;
      if (MODE == 1) lg[it] = la_t;
      la[it] = expf(la_t);
      lk[it] = kq;
      lq[it] = qq * a.q_scale;
    }
    float vv[COLS][STAGE];
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
      for (int tt = 0; tt < STAGE; ++tt)
        vv[c][tt] = (j0 + c < dv && tt < ns) ? to_f(rows[(size_t)(t0 + s0 + tt) * a.ld + a.v_col + head * dv + j0 + c]) : 0.f;
    __syncthreads();
    if (MODE == 1 && tid < d)
      for (int tt = 0; tt < ns; ++tt) loga_sum += lg[tt * d + tid];
    for (int tt = 0; tt < ns; ++tt) {
      const float* aa = la + tt * d + p * DP;
      const float* kk = lk + tt * d + p * DP;
      const float* qv = lq + tt * d + p * DP;
      float acc[COLS];
#pragma unroll
      for (int c = 0; c < COLS; ++c) acc[c] = 0.f;
#pragma unroll
      for (int i = 0; i < DP; ++i) {
        if (p * DP + i < d) {              // (uniform over the lanes that share p; DP divides into d for the usual sizes)
          const float al = aa[i], kv = kk[i], qq = MODE != 1 ? qv[i] : 0.f;
#pragma unroll
          for (int c = 0; c < COLS; ++c) {
            S[c][i] = fmaf(al, S[c][i], kv * vv[c][tt]);
            if (MODE != 1) acc[c] = fmaf(S[c][i], qq, acc[c]);
          }
        }
      }
      if (MODE != 1) {
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
          float r = acc[c];
          for (int o = 1; o < parts; o <<= 1) r += __shfl_xor(r, o, WAVE);
          if (j0 + c < dv && p == 0) lo[tt * dv + j0 + c] = r;
        }
      }
    }
    __syncthreads();
    if (MODE != 1) {
      // a wave per token: the head's norm over dv, its weight, the gate
      for (int tt = wid; tt < ns; tt += nw) {
        const size_t t = (size_t)(t0 + s0 + tt);
        float ss = 0.f;
        for (int c = lane; c < dv; c += WAVE) ss = fmaf(lo[tt * dv + c], lo[tt * dv + c], ss);
        const float inv = rsqrtf(wave_sum(ss) / (float)dv + a.eps);
        for (int c = lane; c < dv; c += WAVE) {
          const float g = to_f(rows[t * a.ld + a.g_col + head * dv + c]);
          ((T*)a.out)[t * (size_t)(H * dv) + head * dv + c] =
              from_f<T>(lo[tt * dv + c] * inv * load_dyn(a.norm_w, a.norm_dtype, c) * act_silu(g));
        }
      }
    }
    __syncthreads();                       // (the next stage's loads overwrite what this stage read)
  }
  if (MODE != 2) {
#pragma unroll
    for (int c = 0; c < COLS; ++c)
      if (j0 + c < dv) {
#pragma unroll
        for (int i = 0; i < DP; i += 4)
          *(float4*)(sp + (size_t)c * parts * DP + i) = make_float4(S[c][i], S[c][i + 1], S[c][i + 2], S[c][i + 3]);
      }
  }
  if (MODE == 1 && tid < d) a.chunk_loga[(size_t)unit * H * d + head * d + tid] = loga_sum;
}

// One thread per number of a request's S: walks the request's chunks in order.  chunk_state[c] holds what chunk c
// reaches from zero and receives the state chunk c starts from.
struct CombineArgs {
  float* state; size_t state_stride, state_offset;
  const int* slots; const int* req_chunk0;       // [R + 1]: a request's chunks are req_chunk0[r] .. req_chunk0[r + 1] - 1
  float* chunk_state; const float* chunk_loga;
  int H, d, dv, parts, dp;
};

__global__ __launch_bounds__(256) void gla_combine_kernel(CombineArgs a) {
  const size_t per = (size_t)a.H * a.dv * a.parts * a.dp;
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= per) return;
  const int r = blockIdx.y;
  const int c0 = a.req_chunk0[r], c1 = a.req_chunk0[r + 1];
  if (c1 <= c0) return;
  const int run = a.parts * a.dp;
  const int i = (int)(e % run), head = (int)(e / run / a.dv);
  float* slot = a.state + (size_t)a.slots[r] * a.state_stride + a.state_offset + e;
  if (i >= a.d) return;                   // (padding: zero for ever)
  float S = *slot;
  for (int c = c0; c < c1; ++c) {
    float* cs = a.chunk_state + (size_t)c * per + e;
    const float mine = *cs;
    *cs = S;
    S = fmaf(expf(a.chunk_loga[(size_t)c * a.H * a.d + head * a.d + i]), S, mine);
  }
  *slot = S;
}

template <typename T, int DP, int MODE, int COLS>
static void launch_gla_mode(const GlaArgs& a, int units, int threads, size_t lds, hipStream_t s) {
  hipLaunchKernelGGL((gla_kernel<T, DP, MODE, COLS>), dim3(units, a.H), dim3(threads), lds, s, a);
}

// A launch of MODE with ``cols`` columns of S a thread (1, 2 or 4; what DP allows is checked by the caller).
template <typename T, int DP, int MODE>
static void launch_gla_cols(const GlaArgs& a, int units, int cols, int threads, size_t lds, hipStream_t s) {
  if constexpr (DP <= 16) { if (cols == 4) return launch_gla_mode<T, DP, MODE, 4>(a, units, threads, lds, s); }
  if constexpr (DP <= 32) { if (cols == 2) return launch_gla_mode<T, DP, MODE, 2>(a, units, threads, lds, s); }
  launch_gla_mode<T, DP, MODE, 1>(a, units, threads, lds, s);
}

template <typename T, int DP>
static int launch_gla(const GlaArgs& a, int R, int n_chunks, const int* req_chunk0, hipStream_t s) {
  // A thread holds 1, 2 or 4 columns of S as its registers allow (4 for runs of 16 channels, 2 for 32): what it reads of a
  // token's q, k and decays from LDS then serves several columns.  Two where possible (steps of single tokens, which are bound
  // by reading and writing S: 23 against 33 us for 64 requests of 16 heads x 64 x 128; chunks side by side: 86 + 64 against
  // 95 + 67 us for 2,048 rows), more only where a head's columns would not fit a workgroup otherwise.  The first d threads also
  // load, so a head of few values still gets a thread per key channel.
  constexpr int MAX_COLS = DP <= 16 ? 4 : (DP <= 32 ? 2 : 1);
  const auto threads_for = [&](int cols) { return ((max((a.dv + cols - 1) / cols * a.parts, a.d) + WAVE - 1) / WAVE) * WAVE; };
  int cols_chunk = min(2, MAX_COLS);
  while (cols_chunk < MAX_COLS && threads_for(cols_chunk) > GLA_MAX_THREADS(DP)) cols_chunk *= 2;
  const int cols_walk = cols_chunk;
  IFX_REQUIRE(threads_for(cols_chunk) <= GLA_MAX_THREADS(DP), "gla_scan: %d threads a head with %d channels each (at most %d)",
              threads_for(cols_chunk), DP, GLA_MAX_THREADS(DP));
  const size_t lds = (size_t)STAGE * (4 * a.d + a.dv) * sizeof(float);
  if (n_chunks == 0) {
    launch_gla_cols<T, DP, 0>(a, R, cols_walk, threads_for(cols_walk), lds, s);
    IFX_LAUNCH_CHECK();
  }
  launch_gla_cols<T, DP, 1>(a, n_chunks, cols_chunk, threads_for(cols_chunk), lds, s);
  CombineArgs c{a.state, a.state_stride, a.state_offset, a.slots, req_chunk0, a.chunk_state, a.chunk_loga, a.H, a.d, a.dv, a.parts, DP};
  const size_t per = (size_t)a.H * a.dv * a.parts * DP;
  hipLaunchKernelGGL(gla_combine_kernel, dim3((unsigned)((per + 255) / 256), R), dim3(256), 0, s, c);
  launch_gla_cols<T, DP, 2>(a, n_chunks, cols_chunk, threads_for(cols_chunk), lds, s);
  IFX_LAUNCH_CHECK();
}

// dp: channels a thread holds (16, 32, 64 or 128); parts: a power of two with parts * dp >= d; a head's columns, 1-4 a thread,
// times parts must fit a workgroup.
extern "C" int ifx_gla_scan(const void* rows, int dtype, int ld, int q_col, int k_col, int v_col, int g_col, const float* z,
                            const float* z_bias, float inv_tau, float q_scale, float eps, const void* norm_w, int norm_dtype,
                            float* state, long long state_stride, long long state_offset, const int* q_start, const int* q_len,
                            const int* slots, void* out, int T, int R, int H, int d, int dv, int dp, int parts,
                            int n_chunks, const int* chunk_req, const int* chunk_t0, const int* chunk_len,
                            const int* req_chunk0, float* chunk_state, float* chunk_loga, void* stream) {
  IFX_REQUIRE(T >= 0 && R >= 0 && H > 0 && d > 0 && dv > 0, "gla_scan: bad sizes T=%d R=%d H=%d d=%d dv=%d", T, R, H, d, dv);
  IFX_REQUIRE(parts > 0 && (parts & (parts - 1)) == 0 && parts <= WAVE && parts * dp >= d, "gla_scan: %d parts of %d channels for d=%d", parts, dp, d);
  IFX_REQUIRE(d <= 1024, "gla_scan: a head of %d key channels does not fit a workgroup", d);
  IFX_REQUIRE((state_offset % 4) == 0 && (state_stride % 4) == 0, "gla_scan: the state must lie at a multiple of 16 bytes");
  IFX_REQUIRE(state_stride >= state_offset + (long long)H * dv * parts * dp, "gla_scan: a state row of %lld floats is too short", state_stride);
  IFX_REQUIRE(n_chunks == 0 || (chunk_req && chunk_t0 && chunk_len && req_chunk0 && chunk_state && chunk_loga), "gla_scan: chunks without their lists");
  IFX_REQUIRE((size_t)STAGE * (4 * d + dv) * sizeof(float) <= 64 * 1024, "gla_scan: d=%d, dv=%d need more LDS than a workgroup has", d, dv);
  if (T == 0 || R == 0) return 0;
  GlaArgs a{rows, ld, q_col, k_col, v_col, g_col, z, z_bias, inv_tau, q_scale, eps, norm_w, norm_dtype, state,
            (size_t)state_stride, (size_t)state_offset, q_start, q_len, slots, out, H, d, dv, parts,
            chunk_req, chunk_t0, chunk_len, chunk_state, chunk_loga};
  hipStream_t s = (hipStream_t)stream;
#define GLA_CASE(TY, DPV) if (dp == DPV) return launch_gla<TY, DPV>(a, R, n_chunks, req_chunk0, s);
  if (dtype == DT_F32) { GLA_CASE(float, 16) GLA_CASE(float, 32) GLA_CASE(float, 64) GLA_CASE(float, 128) }
  else if (dtype == DT_BF16) { GLA_CASE(bf16_t, 16) GLA_CASE(bf16_t, 32) GLA_CASE(bf16_t, 64) GLA_CASE(bf16_t, 128) }
  else IFX_FAIL("gla_scan: unknown dtype %d", dtype);
#undef GLA_CASE
  IFX_FAIL("gla_scan: %d channels a thread (16, 32, 64 or 128)", dp);
}
