// Plain attention over the paged cache: any head size up to 640, float or bf16 storage, float
// math.  One wave per (query row, query head): each lane scores one key of a 64-key tile, the
// wave takes the tile's maximum and sum, then every lane accumulates its output elements over
// the tile's keys in ascending order.  Tiles are aligned to absolute key positions (multiples of
// 64), so the sequence of operations for a (position, head) is the same however the request was
// cut into steps: results are bit-equal across cuttings.  This is the attention of the 32-bit
// path and the reference beside the matrix-core kernels.
//
// Formula (runtime/backends/cuda/kernels/flash_attention.cu:71-72 GQA map, 86 causal limit, 144
// scale after the dot product, 152-173 online softmax): head h reads kv head h / (nH / nKV);
// the query at position p sees keys j with max(0, p - window + 1) <= j <= p; s_j = (q . k_j) *
// scale; o = sum_j softmax(s)_j v_j.
//
// Three further parameters, each off when zero: ``keep_first``, the first positions of a request that a windowed
// query still sees beside its window (j <= p and (p - j < window or j < keep_first)), at their true positions;
// ``has_sink``, a key without value whose score is ``sink_score`` and which only takes part in the softmax's
// denominator (with score 0: p_j = exp(s_j) / (1 + sum exp(s_j))); ``gate`` [T, nH], a factor on each head's output.
//
// ``sinks`` [nH] (or null) gives every head a sink score of its own.  ``chunk`` > 0 cuts the sequence into blocks of that
// many positions counted from its start, and a query sees only the keys of its own block (j <= p and j / chunk ==
// p / chunk; together with a window, both limits hold).
//
// Differential attention (``maps`` = 2): a head's query and a kv head's key are two vectors of d elements each, laid out
// one after the other; each pair gives a softmax map of its own over the same values, and the head's output is
// o = a_1 - lambda a_2, divided by its root mean square over the dv elements (norm_eps inside the root), times out_scale.
//
// Cache layouts: K [page][kv head][offset][maps d], V [page][kv head][dv][offset].  Values may have another width
// than keys (dv != d): the output row of a head then has dv elements.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_D 640
#define DC (MAX_D / WAVE)
#define WAVES_PER_BLOCK 4

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

struct AttnArgs {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  void* out;
  const int* row_req;
  const int* positions;
  const int* block_table;
  int max_blocks;
  int T, nH, nKV, d, dv, page_size, window;
  float scale;
  int keep_first;
  int has_sink;
  float sink_score;
  const float* gate;
  const float* sinks;
  int chunk;
  float lambda, out_scale, norm_eps;
};

template <typename T, int MAPS>
__global__ __launch_bounds__(WAVE * WAVES_PER_BLOCK) void attn_plain_kernel(AttnArgs a) {
  __shared__ float q_s[WAVES_PER_BLOCK][MAX_D];
  const int wid = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const long long item = (long long)blockIdx.x * WAVES_PER_BLOCK + wid;
  // All lanes of a wave share `item`, so the whole wave leaves together; no block-wide
  // barrier follows.
  if (item >= (long long)a.T * a.nH) return;
  const int row = (int)(item / a.nH), head = (int)(item % a.nH);
  const int d = a.d, dv = a.dv, P = a.page_size;
  const int kvh = head / (a.nH / a.nKV);
  const int pos = a.positions[row];
  const int* table = a.block_table + (size_t)a.row_req[row] * a.max_blocks;
  int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  if (a.chunk > 0) lo = max(lo, pos - pos % a.chunk);
  const int keep = lo > 0 ? min(a.keep_first, lo) : 0;      // keys [0, keep) and [lo, pos] are seen

  const int kd = MAPS * d;      // elements of a query's and a key's row
  const T* qrow = (const T*)a.q + ((size_t)row * a.nH + head) * kd;
  for (int e = lane; e < kd; e += WAVE) q_s[wid][e] = to_f(qrow[e]);
  // q_s[wid] is written and read by this wave only.
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0);

  // (the sink is a key of score sink_score whose value is zero: it starts the running maximum and sum)
  const bool sunk = a.has_sink || a.sinks;
  const float sink_score = a.sinks ? a.sinks[head] : a.sink_score;
  float m[MAPS], l[MAPS], acc[MAPS][DC];
#pragma unroll
  for (int w = 0; w < MAPS; ++w) {
    m[w] = sunk ? sink_score : -INFINITY;
    l[w] = sunk ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[w][c] = 0.f;
  }

  const T* Kc = (const T*)a.k_cache;
  const T* Vc = (const T*)a.v_cache;
  for (int t0 = keep > 0 ? 0 : (lo / WAVE) * WAVE; t0 <= pos; t0 += WAVE) {
    if (t0 >= keep && t0 + WAVE <= lo) {     // between the kept first keys and the window: on to the window's first tile
      t0 = (lo / WAVE) * WAVE - WAVE;
      continue;
    }
    const int j = t0 + lane;
    const bool valid = (j >= lo || j < keep) && j <= pos;
    int page = 0, off = 0;
    float s[MAPS], p[MAPS];
#pragma unroll
    for (int w = 0; w < MAPS; ++w) s[w] = -INFINITY;
    if (valid) {
      page = table[j / P];
      off = j % P;
#pragma unroll
      for (int w = 0; w < MAPS; ++w) {
        const T* kr = Kc + (((size_t)page * a.nKV + kvh) * P + off) * kd + w * d;
        const float* qv = q_s[wid] + w * d;
        float dot = 0.f;
        if (d % 8 == 0) {        // the key's row in 16-byte pieces; the same additions in the same order
          for (int e = 0; e < d; e += 8) {
            float kv[8];
            load8(kr + e, kv);
#pragma unroll
            for (int i = 0; i < 8; ++i) dot = fmaf(qv[e + i], kv[i], dot);
          }
        } else {
          for (int e = 0; e < d; ++e) dot = fmaf(qv[e], to_f(kr[e]), dot);
        }
        s[w] = dot * a.scale;
      }
    }
#pragma unroll
    for (int w = 0; w < MAPS; ++w) {
      const float m_new = fmaxf(m[w], wave_max(s[w]));  // finite: the tile holds a visible key
      p[w] = valid ? expf(s[w] - m_new) : 0.f;
      const float alpha = expf(m[w] - m_new);  // 0 on the first tile (m = -inf)
      l[w] = l[w] * alpha + wave_sum(p[w]);
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[w][c] *= alpha;
      m[w] = m_new;
    }
    if (P % 8 == 0) {
      // Eight keys at a time: they lie in one page, where a value element's eight entries are 16 consecutive bytes.
      // Keys outside the range have weight 0 and their entries (stale or zero, never written with anything that is
      // not finite) add nothing; an element's sum still runs over the keys in ascending order.
      for (int g = 0; g < WAVE; g += 8) {
        const int j0 = t0 + g;
        if (j0 > pos || (j0 + 7 < lo && j0 >= keep)) continue;  // uniform over the wave
        float pj[MAPS][8];
#pragma unroll
        for (int w = 0; w < MAPS; ++w)
#pragma unroll
          for (int i = 0; i < 8; ++i) pj[w][i] = __shfl(p[w], g + i, WAVE);
        const T* vb = Vc + ((size_t)table[j0 / P] * a.nKV + kvh) * dv * P + j0 % P;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          const int e = lane + c * WAVE;
          if (e < dv) {
            float vv[8];
            load8(vb + (size_t)e * P, vv);
#pragma unroll
            for (int w = 0; w < MAPS; ++w)
#pragma unroll
              for (int i = 0; i < 8; ++i) acc[w][c] = fmaf(pj[w][i], vv[i], acc[w][c]);
          }
        }
      }
    } else
    for (int jj = 0; jj < WAVE; ++jj) {
      float pj[MAPS];
      bool none = true;
#pragma unroll
      for (int w = 0; w < MAPS; ++w) {
        pj[w] = __shfl(p[w], jj, WAVE);
        none = none && pj[w] == 0.f;
      }
      const int pg = __shfl(page, jj, WAVE), of = __shfl(off, jj, WAVE);
      if (none) continue;  // uniform over the wave; keys outside the range are never read
      const T* vb = Vc + ((size_t)pg * a.nKV + kvh) * dv * P + of;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const int e = lane + c * WAVE;
        if (e < dv) {
          const float vv = to_f(vb[(size_t)e * P]);
#pragma unroll
          for (int w = 0; w < MAPS; ++w) acc[w][c] = fmaf(pj[w], vv, acc[w][c]);
        }
      }
    }
  }
  T* orow = (T*)a.out + ((size_t)row * a.nH + head) * dv;
  const float inv = (l[0] > 0.f ? 1.f / l[0] : 0.f) * (a.gate ? a.gate[(size_t)row * a.nH + head] : 1.f);
  if (MAPS == 1) {
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const int e = lane + c * WAVE;
      if (e < dv) orow[e] = from_f<T>(acc[0][c] * inv);
    }
    return;
  }
  // the second map subtracted, the head's root mean square over dv, the constant factor
  const float inv2 = (l[MAPS - 1] > 0.f ? 1.f / l[MAPS - 1] : 0.f) * a.lambda;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e = lane + c * WAVE;
    acc[0][c] = e < dv ? acc[0][c] * inv - acc[MAPS - 1][c] * inv2 : 0.f;
    ss = fmaf(acc[0][c], acc[0][c], ss);
  }
  const float f = a.out_scale / sqrtf(wave_sum(ss) / (float)dv + a.norm_eps);
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e = lane + c * WAVE;
    if (e < dv) orow[e] = from_f<T>(acc[0][c] * f);
  }
}

extern "C" int ifx_attn_plain(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                              const int* row_req, const int* positions, const int* block_table,
                              int max_blocks, int T, int nH, int nKV, int d, int dv, int page_size, int window,
                              float scale, int keep_first, int has_sink, float sink_score, const float* gate, const float* sinks,
                              int chunk, int maps, float lambda, float out_scale, float norm_eps, void* stream) {
  IFX_REQUIRE(keep_first >= 0, "attn_plain: keep_first %d", keep_first);
  IFX_REQUIRE(T >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_plain: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(maps == 1 || maps == 2, "attn_plain: %d maps (1 or 2)", maps);
  IFX_REQUIRE(chunk >= 0, "attn_plain: chunk %d", chunk);
  IFX_REQUIRE(d > 0 && maps * d <= MAX_D, "attn_plain: head_dim %d x %d outside 1..%d", maps, d, MAX_D);
  IFX_REQUIRE(dv > 0 && dv <= MAX_D, "attn_plain: value head_dim %d outside 1..%d", dv, MAX_D);
  IFX_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attn_plain: bad page_size/max_blocks/window");
  if (T == 0) return 0;
  AttnArgs a{q, k_cache, v_cache, out, row_req, positions, block_table, max_blocks, T, nH, nKV, d, dv, page_size, window, scale, keep_first, has_sink, sink_score, gate, sinks, chunk, lambda, out_scale, norm_eps};
  const long long items = (long long)T * nH;
  const unsigned blocks = (unsigned)((items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32 && maps == 1) hipLaunchKernelGGL((attn_plain_kernel<float, 1>), dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else if (dtype == DT_BF16 && maps == 1) hipLaunchKernelGGL((attn_plain_kernel<bf16_t, 1>), dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else if (dtype == DT_F32) hipLaunchKernelGGL((attn_plain_kernel<float, 2>), dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL((attn_plain_kernel<bf16_t, 2>), dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else IFX_FAIL("attn_plain: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
