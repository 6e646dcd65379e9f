// Attention of many query heads over ONE shared kv head whose keys (K_DIM) and values (V_DIM) are wider than a wave of
// attn_mfma.hip can hold in registers, or of unequal width: what attention through a latent gives (keys = latent +
// rotated part, values = latent), at any size.  bf16 in, float accumulate, on the 16x16x32 matrix instruction.
//
// One wave per (row, group of 16 heads, split of the key range), for prompts' rows and decoded tokens alike.  The 16
// heads are the columns of the matrix tile, so a key or value is fetched once for all of them.  Their queries wait in
// LDS (16 x K_DIM bf16, read as the second operand of the score product step by step), which leaves the registers to
// the output: V_DIM / 16 tiles of four floats per lane.  Scores, softmax and the layout of both products are
// attn_mfma.hip's row kernel's (S^T[key, head] = K Q^T; O^T[dim, head] += V^T P^T), as is the form of the splits' partial
// results; a launch of its own merges them (a wave per (row, head), a lane a run of four elements), and a row in one
// split writes its output itself.
//
// Compile with -DK_DIM=<multiple of 8> -DV_DIM=<multiple of 16>.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#if !defined(K_DIM) || !defined(V_DIM)
#error "compile with -DK_DIM=<keys' width> -DV_DIM=<values' width>"
#endif
static_assert(K_DIM % 8 == 0 && K_DIM >= 8 && K_DIM <= 1024, "K_DIM must be a multiple of 8 up to 1024");
static_assert(V_DIM % 16 == 0 && V_DIM >= 16 && V_DIM <= 512, "V_DIM must be a multiple of 16 up to 512");
#define HEAD_DIM V_DIM
#include "attn_shared.h"      // D = V_DIM from here on: the width of outputs and partial results

constexpr int DK = K_DIM;
constexpr int KSK = (DK + 31) / 32;     // 32-wide steps of the score product
constexpr int QP = DK + 8;              // elements per query row in LDS (the padding spreads the 16 rows over the banks)

extern "C" int ifx_attn_wide_dims() { return DK * 1024 + D; }

__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_wide_rows_kernel(RowArgs a) {
  extern __shared__ __attribute__((aligned(16))) bf16_t qs[];      // [16][QP]
  const int split = blockIdx.x, hg = blockIdx.y, ri = blockIdx.z;
  const int lane = threadIdx.x, col = lane & 15, g4 = lane >> 4;
  const int row = a.rows ? a.rows[ri] : ri;
  const int P = a.P;
  const int pos = a.positions[row];
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int ka = max(lo, split * a.chunk), kb = min(pos + 1, (split + 1) * a.chunk);  // keys [ka, kb)
  const int* table = a.block_table + (size_t)a.row_req[row] * a.max_blocks;
  const int head = hg * 16 + col;
  const bool head_ok = head < a.nH;
  float* po = a.part_o + (((size_t)ri * a.nH + head) * a.max_splits + split) * D;
  float* pml = a.part_ml + (((size_t)ri * a.nH + head) * a.max_splits + split) * 2;
  if (ka >= kb) {  // nothing of this split is visible: the merge skips it
    if (head_ok && g4 == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
    return;
  }
  for (int piece = lane; piece < 16 * (DK / 8); piece += WAVE) {
    const int c = piece / (DK / 8), e = 8 * (piece % (DK / 8)), h = hg * 16 + c;
    *(bf16x8*)&qs[c * QP + e] = h < a.nH ? *(const bf16x8*)(a.q + ((size_t)row * a.nH + h) * DK + e) : zero8();
  }
  __syncthreads();          // (one wave: the queries are in LDS for all its lanes)
  floatx4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  for (int j0 = (ka / 32) * 32; j0 < kb; j0 += 32) {
    floatx4 s[2];
    bool live[2];
    const bf16_t* vp[2];
    float mb = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int k0 = j0 + 16 * t;      // 16 keys k0..k0+15, all in one page
      bool lv = k0 < kb && k0 + 16 > ka;
      const int page = lv ? table[k0 / P] : -1;
      lv = lv && page >= 0;
      live[t] = lv;
      const int off = k0 % P;
      const bf16_t* kp = a.k_cache + (((size_t)(lv ? page : 0)) * P + off + col) * DK + 8 * g4;
      vp[t] = a.v_cache + ((size_t)(lv ? page : 0) * D + col) * P + off + 4 * g4;
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (lv) {
        // all of the tile's key pieces are asked for before the first product (a chain of trips to memory otherwise)
        bf16x8 kop[KSK];
#pragma unroll
        for (int ks = 0; ks < KSK; ++ks) kop[ks] = 32 * ks + 8 * g4 < DK ? *(const bf16x8*)(kp + 32 * ks) : zero8();
#pragma unroll
        for (int ks = 0; ks < KSK; ++ks) {
          const int c = 32 * ks + 8 * g4;
          const bf16x8 qop = c < DK ? *(const bf16x8*)&qs[col * QP + c] : zero8();
          s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[ks], qop, s[t], 0, 0, 0);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = k0 + 4 * g4 + r;
        const bool vis = lv && key >= ka && key < kb;
        s[t][r] = vis ? s[t][r] * a.scale_log2e : -INFINITY;
        mb = fmaxf(mb, s[t][r]);
      }
      // one tile's key pieces at a time: both tiles' together cost 72 registers more and the second wave of a SIMD its place
      __builtin_amdgcn_sched_barrier(0);
    }
    const float m_new = fmaxf(m, col_max(mb));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    float psum = 0.f;
    bf16x4 pb[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = fast_exp2(s[t][r] - m_safe);
        psum += p;
        pb[t][r] = (__bf16)p;
      }
    l = l * alpha + psum;
    m = m_new;
    const bf16x8 pop = join4(pb[0], pb[1]);
    constexpr int VB = DT < 8 ? DT : 8;       // value tiles whose pieces are asked for together
#pragma unroll
    for (int d0 = 0; d0 < DT; d0 += VB) {
      bf16x4 v0[VB], v1[VB];
#pragma unroll
      for (int i = 0; i < VB; ++i) {
        const int dt = d0 + i;
        v0[i] = (live[0] && dt < DT) ? *(const bf16x4*)(vp[0] + (size_t)16 * dt * P) : zero4();
        v1[i] = (live[1] && dt < DT) ? *(const bf16x4*)(vp[1] + (size_t)16 * dt * P) : zero4();
      }
#pragma unroll
      for (int i = 0; i < VB; ++i) {
        const int dt = d0 + i;
        if (dt < DT) {
#pragma unroll
          for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(join4(v0[i], v1[i]), pop, o[dt], 0, 0, 0);
        }
      }
    }
  }
  l = col_sum(l);
  if (!head_ok) return;
  if (a.max_splits == 1) {      // the row's only split: the output itself, no partial result and no merge
    const float inv = finish_factor(m, l, 0, 0.f, nullptr, (size_t)row * a.nH + head, a.sinks, a.nH);      // (a sink score per head joins the sum here)
    bf16_t* orow = a.out + ((size_t)row * a.nH + head) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      bf16x4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = (__bf16)(o[dt][r] * inv);
      *(bf16x4*)(orow + 16 * dt + 4 * g4) = y;
    }
    return;
  }
  if (g4 == 0) { pml[0] = m; pml[1] = l; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) *(floatx4*)(po + 16 * dt + 4 * g4) = o[dt];
}

// out[row, head] = sum_s 2^(m_s - M) O_s / sum_s 2^(m_s - M) l_s over the row's splits in ascending order, M = max m_s.
// One wave per (row, head); a lane owns runs of four output elements.
__global__ __launch_bounds__(WAVE) void attn_wide_merge_kernel(RowArgs a) {
  constexpr int C4 = (D + 255) / 256;
  const int ri = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int row = a.rows ? a.rows[ri] : ri;
  const float* po = a.part_o + ((size_t)ri * a.nH + head) * a.max_splits * D;
  const float* pml = a.part_ml + ((size_t)ri * a.nH + head) * a.max_splits * 2;
  float M = -INFINITY;
  for (int s = lane; s < a.max_splits; s += WAVE) M = fmaxf(M, pml[2 * s]);
  M = wave_max(M);
  floatx4 acc[C4];
#pragma unroll
  for (int c = 0; c < C4; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
  float L = 0.f;
  for (int s = 0; s < a.max_splits; ++s) {
    const float ms = pml[2 * s];
    if (ms == -INFINITY) continue;          // uniform over the wave: a split without a visible key
    const float w = fast_exp2(ms - M);
    L += w * pml[2 * s + 1];
#pragma unroll
    for (int c = 0; c < C4; ++c) {
      const int e = 4 * lane + 256 * c;
      if (e < D) {
        const floatx4 v = *(const floatx4*)(po + (size_t)s * D + e);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[c][r] += w * v[r];
      }
    }
  }
  const float inv = finish_factor(M, L, 0, 0.f, nullptr, (size_t)row * a.nH + head, a.sinks, a.nH);
  bf16_t* orow = a.out + ((size_t)row * a.nH + head) * D;
#pragma unroll
  for (int c = 0; c < C4; ++c) {
    const int e = 4 * lane + 256 * c;
    if (e < D) {
      bf16x4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) y[r] = (__bf16)(acc[c][r] * inv);
      *(bf16x4*)(orow + e) = y;
    }
  }
}

// out [T, nH * V_DIM] for the rows named by ``rows`` (or rows 0..n_rows-1): split s of a row covers key positions
// [s * chunk, (s + 1) * chunk) (chunk a multiple of 32; max_splits * chunk must reach past every row's position), partial
// results in part_o [n_rows, nH, max_splits, V_DIM] and part_ml [n_rows, nH, max_splits, 2], merged by a second launch.
extern "C" int ifx_attn_wide(const void* q, const void* k_cache, const void* v_cache, void* out, const int* rows,
                             const int* row_req, const int* positions, const int* block_table, int max_blocks, int n_rows,
                             int nH, int d, int dv, int page_size, int window, int chunk, int max_splits, float scale,
                             float* part_o, float* part_ml, const float* sinks, void* stream) {
  IFX_REQUIRE(d == DK && dv == D, "attn_wide: built for keys of %d and values of %d, called with %d and %d", DK, D, d, dv);
  IFX_REQUIRE(n_rows >= 0 && n_rows <= 65535 && nH > 0 && (nH + 15) / 16 <= 65535, "attn_wide: %d rows, %d heads", n_rows, nH);
  IFX_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attn_wide: page_size %d must be a multiple of 16", page_size);
  IFX_REQUIRE(chunk > 0 && chunk % 32 == 0 && max_splits > 0 && max_splits <= 65535, "attn_wide: bad chunk %d / splits %d", chunk, max_splits);
  IFX_REQUIRE(part_o && part_ml, "attn_wide: needs scratch for the splits' partial results");
  if (n_rows == 0) return 0;
  RowArgs a{(const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, rows, row_req, positions, block_table,
            part_o, part_ml, (bf16_t*)out, max_blocks, n_rows, nH, 1, page_size, window, chunk, max_splits,
            scale * 1.4426950408889634f, 0, 0, 0};
  a.sinks = sinks;          // [nH] or null: a score per head in the softmax's denominator
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(attn_wide_rows_kernel, dim3(max_splits, (nH + 15) / 16, n_rows), dim3(WAVE), (size_t)16 * QP * sizeof(bf16_t), s, a);
  if (max_splits > 1) hipLaunchKernelGGL(attn_wide_merge_kernel, dim3(n_rows, nH), dim3(WAVE), 0, s, a);
  IFX_LAUNCH_CHECK();
}
