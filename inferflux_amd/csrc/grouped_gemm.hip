// Products of many rows with one of several weights each, on the matrix cores (bfloat16 in, float sums): the experts of
// a mixture, where every (row, choice) takes the weight of the expert it chose, and the per-head products of attention
// through a latent, where every head has a weight of its own.
//
//   ifx_moe_sort       the (row, choice) items of a step ordered by expert, cut into tiles of TM items of one expert
//                      each; everything stays on the device (the grid of the products is sized by the most tiles
//                      there can be, and a workgroup without a tile leaves at once)
//   ifx_moe_gate_up_grouped   act[item] = silu(Wg[e] x) * (Wu[e] x), from weights whose rows alternate 16 of Wg with
//                      16 of Wu, so that a wave holds a gate tile and its up tile and the activation is its epilogue
//   ifx_moe_down_grouped      parts[choice][row] = weight[item] * Wd[e] act[item] in float: the choices of a row are
//                      the "slices" of a sum that the kernel which adds the result to the stream takes in order, so a
//                      row's result does not depend on where its items lay in the order
//                      An expert from `n_real` upwards is an identity expert without weights: the first product leaves its
//                      tiles alone and the second writes weight[item] * x[row] (`identity`, the rows as the first product
//                      read them; N is then the rows' width).  The first product's activation is `act` of common.h.
//   ifx_headwise_grouped      out[t][h][:N] = W[h] x[t][h], tiles of TM rows of one head
//
// One kernel does all three products.  A workgroup of four waves takes TM = 64 or 128 items and TN = 128 weight rows;
// steps of 64 k-values of both are staged in LDS (16-byte pieces, rows padded by 16 bytes against bank conflicts, the
// next step's pieces on their way into registers meanwhile).  The waves stand two by two: each multiplies 32 x MT items
// with two tiles of 32 weight rows on the 32x32x16 matrix instruction, C[weight row][item], so a lane ends up with
// runs of four consecutive output columns of one item.  Sums run over k in ascending order whatever the tile, so an
// item's result does not depend on what shares its tile.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define TM_MAX 128     // items to a tile: 64 or 128 (the caller's choice, the same for the list and the products)
#define TN 128
#define TK 64
#define LDP (TK + 8)
#define MAX_EXPERTS 1024


// ---------------------------------------------------------------------------------------
// ids [n_items] -> sorted [n_items] (items of expert 0, then of expert 1, ...), tiles (expert, first place in sorted,
// count) and their number.  One workgroup.  The order of an expert's items among themselves is not fixed; no result
// depends on it.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int n_items, int E, int TM, int* __restrict__ sorted,
                                                        int* __restrict__ tile_expert, int* __restrict__ tile_start,
                                                        int* __restrict__ tile_count, int* __restrict__ n_tiles) {
  __shared__ int cnt[MAX_EXPERTS];
  __shared__ int offs[MAX_EXPERTS];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += blockDim.x) atomicAdd(&cnt[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, n = 0;
    for (int e = 0; e < E; ++e) {
      offs[e] = at;
      for (int s = 0; s < cnt[e]; s += TM) {
        tile_expert[n] = e;
        tile_start[n] = at + s;
        tile_count[n] = min(TM, cnt[e] - s);
        ++n;
      }
      at += cnt[e];
    }
    *n_tiles = n;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_items; i += blockDim.x) {
    const int e = ids[i];
    sorted[offs[e] + atomicAdd(&cnt[e], 1)] = i;
  }
}

extern "C" int ifx_moe_sort(const int* ids, int n_items, int E, int tile_items, int* sorted, int* tile_expert, int* tile_start,
                            int* tile_count, int* n_tiles, void* stream) {
  IFX_REQUIRE(n_items >= 0 && E > 0 && E <= MAX_EXPERTS, "moe_sort: %d items, %d experts (at most %d)", n_items, E, MAX_EXPERTS);
  IFX_REQUIRE(tile_items == 64 || tile_items == 128, "moe_sort: tiles of %d items (64 or 128)", tile_items);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ids, n_items, E, tile_items, sorted, tile_expert,
                     tile_start, tile_count, n_tiles);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
enum { MODE_GATE_UP = 0, MODE_DOWN = 1, MODE_HEADS = 2 };

struct GroupedArgs {
  const bf16_t* x;          // item i of group g reads K values from x + (i / x_div) * x_row + g * x_group
  const bf16_t* w;          // [groups][NW][K]
  void* out;
  const int* sorted; const int* tile_expert; const int* tile_start; const int* tile_count; const int* n_tiles;   // (not MODE_HEADS)
  const float* weights;     // MODE_DOWN: [n_items]
  int K, NW, x_div, x_row, x_group;
  int T, top;               // MODE_DOWN: parts [top][T][NW]; MODE_HEADS: T rows, tiles_per_group = ceil(T / TM)
  int out_head, n_groups;   // MODE_HEADS: out [T][n_groups][out_head]
  int n_real;               // experts with weights; tiles of later ones are identity experts' (not MODE_HEADS)
  const bf16_t* identity;   // MODE_DOWN: [T][NW], what an identity expert hands back
  int act; float limit;     // MODE_GATE_UP: the activation
};

// MT: tiles of 32 items per wave (1: the workgroup takes 64 items, 2: 128)
template <int MODE, int MT>
__global__ __launch_bounds__(256) void grouped_kernel(GroupedArgs a) {
  constexpr int BM = 64 * MT;
  __shared__ __attribute__((aligned(16))) bf16_t ws[TN][LDP];
  __shared__ __attribute__((aligned(16))) bf16_t xs[BM][LDP];
  __shared__ int items[BM];
  const int tid = threadIdx.x;
  int group, start, count;
  if (MODE == MODE_HEADS) {
    const int per = (a.T + BM - 1) / BM;
    group = blockIdx.x / per;
    start = (blockIdx.x % per) * BM;
    count = min(BM, a.T - start);
  } else {
    const int tile = blockIdx.x;           // (the list was cut into tiles of BM items)
    if (tile >= *a.n_tiles) return;
    group = a.tile_expert[tile];
    start = a.tile_start[tile];
    count = min(a.tile_count[tile], BM);
  }
  const int n0 = blockIdx.y * TN;
  if (MODE != MODE_HEADS && group >= a.n_real) {        // an identity expert's tile (the whole workgroup)
    if (MODE == MODE_DOWN)
      for (int x = tid; x < count * TN; x += 256) {
        const int m = a.sorted[start + x / TN], n = n0 + x % TN;
        if (n < a.NW)
          ((float*)a.out)[((size_t)(m % a.top) * a.T + m / a.top) * a.NW + n] = a.weights[m] * (float)a.identity[(size_t)(m / a.top) * a.NW + n];
      }
    return;
  }
  for (int i = tid; i < BM; i += 256) items[i] = i < count ? (MODE == MODE_HEADS ? start + i : a.sorted[start + i]) : -1;
  __syncthreads();
  const int wave = tid / WAVE, lane = tid % WAVE, l32 = lane & 31, hi = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;          // this wave's items: 32 MT wm ..., its weight rows: 64 wn ...
  floatx16 acc[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;
  const bf16_t* wbase = a.w + (size_t)group * a.NW * a.K;
  const bf16_t* xbase = a.x + (size_t)group * a.x_group;
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (__bf16)0.f;
  // A step's pieces are asked for one step ahead: while the matrix cores work on step s from LDS, the loads of step
  // s + 1 are on their way into registers.  Pieces of 8 k-values: 8 to a row; TN rows of W and BM rows of x.
  constexpr int WP = TN * 8 / 256, XP = BM * 8 / 256;
  bf16x8 wv[WP], xv[XP];
  const bf16_t* wp[WP];
  const bf16_t* xp[XP];
  const int kc = 8 * (tid % 8);
#pragma unroll
  for (int p = 0; p < WP; ++p) {
    const int wrow = n0 + (tid + 256 * p) / 8;
    wp[p] = wrow < a.NW ? wbase + (size_t)wrow * a.K + kc : nullptr;
  }
#pragma unroll
  for (int p = 0; p < XP; ++p) {
    const int it = items[(tid + 256 * p) / 8];
    xp[p] = it >= 0 ? xbase + (size_t)(it / a.x_div) * a.x_row + kc : nullptr;
  }
  auto fetch = [&](int k0) {
    const bool in = k0 + kc < a.K;
#pragma unroll
    for (int p = 0; p < WP; ++p) wv[p] = (wp[p] && in) ? *(const bf16x8*)(wp[p] + k0) : zero;
#pragma unroll
    for (int p = 0; p < XP; ++p) xv[p] = (xp[p] && in) ? *(const bf16x8*)(xp[p] + k0) : zero;
  };
  fetch(0);
  for (int k0 = 0; k0 < a.K; k0 += TK) {
    __syncthreads();          // everyone is done with the last step's tiles
#pragma unroll
    for (int p = 0; p < WP; ++p) *(bf16x8*)&ws[(tid + 256 * p) / 8][kc] = wv[p];
#pragma unroll
    for (int p = 0; p < XP; ++p) *(bf16x8*)&xs[(tid + 256 * p) / 8][kc] = xv[p];
    __syncthreads();
    if (k0 + TK < a.K) fetch(k0 + TK);
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) {
      bf16x8 aop[2], bop[MT];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) aop[nt] = *(const bf16x8*)&ws[64 * wn + 32 * nt + l32][16 * ks + 8 * hi];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) bop[mt] = *(const bf16x8*)&xs[32 * MT * wm + 32 * mt + l32][16 * ks + 8 * hi];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aop[nt], bop[mt], acc[mt][nt], 0, 0, 0);
    }
  }
  // acc[mt][nt][i]: weight row n0 + 64 wn + 32 nt + 8 (i / 4) + 4 hi + i % 4 of item 32 MT wm + 32 mt + l32
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = items[32 * MT * wm + 32 * mt + l32];
    if (m < 0) continue;
    if (MODE == MODE_GATE_UP) {
      // a tile of 32 weight rows is 16 of Wg and the same 16 of Wu: acc[i] (i < 8) is the gate of what acc[i + 8] is the up of
      const int ff = a.NW / 2;
      bf16_t* act = (bf16_t*)a.out + (size_t)m * ff;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const int f = (n0 + 64 * wn + 32 * nt) / 2 + 8 * q + 4 * hi;
          if (f >= ff) continue;
          bf16x4 y;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = acc[mt][nt][4 * q + r], u = acc[mt][nt][8 + 4 * q + r];
            y[r] = (__bf16)gated_act(g, u, a.act, a.limit);
          }
          *(bf16x4*)(act + f) = y;
        }
    } else {
      const float wgt = MODE == MODE_DOWN ? a.weights[m] : 1.f;
      float* of = MODE == MODE_DOWN ? (float*)a.out + ((size_t)(m % a.top) * a.T + m / a.top) * a.NW : nullptr;
      bf16_t* ob = MODE == MODE_HEADS ? (bf16_t*)a.out + ((size_t)m * a.n_groups + group) * a.out_head : nullptr;
      const bool whole4 = a.NW % 4 == 0 && (MODE == MODE_DOWN || a.out_head % 4 == 0);      // runs of four columns, stored at once
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + 64 * wn + 32 * nt + 8 * q + 4 * hi;
          if (n >= a.NW) continue;
          if (whole4) {
            if (MODE == MODE_DOWN) {
              *(floatx4*)(of + n) = floatx4{wgt * acc[mt][nt][4 * q], wgt * acc[mt][nt][4 * q + 1], wgt * acc[mt][nt][4 * q + 2],
                                            wgt * acc[mt][nt][4 * q + 3]};
            } else {
              bf16x4 y;
#pragma unroll
              for (int r = 0; r < 4; ++r) y[r] = (__bf16)acc[mt][nt][4 * q + r];
              *(bf16x4*)(ob + n) = y;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (n + r >= a.NW) continue;
              if (MODE == MODE_DOWN) of[n + r] = wgt * acc[mt][nt][4 * q + r];
              else ob[n + r] = (bf16_t)acc[mt][nt][4 * q + r];
            }
          }
        }
    }
  }
}

static int check_common(int K, int x_row, int x_group) {
  return K > 0 && K % 8 == 0 && x_row % 8 == 0 && x_group % 8 == 0;
}

// act [n_items][ff] (bfloat16) from x [T][K] and the paired weights w [E][2 ff][K]; item i is row i / top.
extern "C" int ifx_moe_gate_up_grouped(const void* x, const void* w, void* act, const int* sorted, const int* tile_expert,
                                       const int* tile_start, const int* tile_count, const int* n_tiles, int max_tiles, int tile_items,
                                       int K, int ff, int top, int n_real, int act_kind, float limit, void* stream) {
  IFX_REQUIRE(check_common(K, K, 0) && ff > 0 && ff % 16 == 0 && top > 0, "moe_gate_up_grouped: K=%d must be a multiple of 8, ff=%d of 16", K, ff);
  if (max_tiles <= 0) return 0;
  GroupedArgs a{(const bf16_t*)x, (const bf16_t*)w, act, sorted, tile_expert, tile_start, tile_count, n_tiles, nullptr,
                K, 2 * ff, top, K, 0, 0, top, 0, 0, n_real, nullptr, act_kind, limit};
  const dim3 grid(max_tiles, (2 * ff + TN - 1) / TN);
  if (tile_items == 128) hipLaunchKernelGGL((grouped_kernel<MODE_GATE_UP, 2>), grid, dim3(256), 0, (hipStream_t)stream, a);
  else if (tile_items == 64) hipLaunchKernelGGL((grouped_kernel<MODE_GATE_UP, 1>), grid, dim3(256), 0, (hipStream_t)stream, a);
  else IFX_FAIL("moe_gate_up_grouped: tiles of %d items (64 or 128)", tile_items);
  IFX_LAUNCH_CHECK();
}

// parts [top][T][N] (float) = weights[item] * (Wd[e] act[item]), w [E][N][ff]
extern "C" int ifx_moe_down_grouped(const void* act, const void* w, float* parts, const float* weights, const int* sorted,
                                    const int* tile_expert, const int* tile_start, const int* tile_count, const int* n_tiles,
                                    int max_tiles, int tile_items, int T, int N, int ff, int top, int n_real, const void* identity,
                                    void* stream) {
  IFX_REQUIRE(check_common(ff, ff, 0) && N > 0 && top > 0 && T >= 0, "moe_down_grouped: ff=%d must be a multiple of 8", ff);
  if (max_tiles <= 0 || T == 0) return 0;
  GroupedArgs a{(const bf16_t*)act, (const bf16_t*)w, parts, sorted, tile_expert, tile_start, tile_count, n_tiles, weights,
                ff, N, 1, ff, 0, T, top, 0, 0, n_real, (const bf16_t*)identity, 0, 0.f};
  const dim3 grid(max_tiles, (N + TN - 1) / TN);
  if (tile_items == 128) hipLaunchKernelGGL((grouped_kernel<MODE_DOWN, 2>), grid, dim3(256), 0, (hipStream_t)stream, a);
  else if (tile_items == 64) hipLaunchKernelGGL((grouped_kernel<MODE_DOWN, 1>), grid, dim3(256), 0, (hipStream_t)stream, a);
  else IFX_FAIL("moe_down_grouped: tiles of %d items (64 or 128)", tile_items);
  IFX_LAUNCH_CHECK();
}

// out [T][H][out_head] (bfloat16): the first N elements of every head, W [H][N][K], head h of row t reads x + t * x_row + h * x_head
extern "C" int ifx_headwise_grouped(const void* x, const void* w, void* out, int T, int H, int K, int N, int x_row, int x_head,
                                    int out_head, void* stream) {
  IFX_REQUIRE(check_common(K, x_row, x_head) && N > 0 && H > 0 && out_head >= N, "headwise_grouped: K=%d, the rows of x (%d) and its heads (%d) must be multiples of 8", K, x_row, x_head);
  if (T <= 0) return 0;
  GroupedArgs a{(const bf16_t*)x, (const bf16_t*)w, out, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                K, N, 1, x_row, x_head, T, 1, out_head, H, H, nullptr, 0, 0.f};
  if (T > 64) hipLaunchKernelGGL((grouped_kernel<MODE_HEADS, 2>), dim3(((T + 127) / 128) * H, (N + TN - 1) / TN), dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL((grouped_kernel<MODE_HEADS, 1>), dim3(((T + 63) / 64) * H, (N + TN - 1) / TN), dim3(256), 0, (hipStream_t)stream, a);
  IFX_LAUNCH_CHECK();
}
