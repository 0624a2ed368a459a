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
//   ifx_headwise_grouped      out[t][h][:N] = W[h] x[t][h], tiles of TM rows of one head
//
// One kernel does all three products.  A workgroup of four waves takes TM = 64 items and TN = 64 weight rows; steps of
// 64 k-values of both are staged in LDS (16-byte pieces, rows padded by 16 bytes against bank conflicts), each wave
// multiplies its 16 items with the four tiles of 16 weight rows: C[weight row][item], so a lane ends up with four
// consecutive output columns of one item.  Sums run over k in ascending order whatever the tile, so an item's result
// does not depend on what shares its tile.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define TM 64
#define TN 64
#define TK 64
#define LDP (TK + 8)
#define MAX_EXPERTS 1024

extern "C" int ifx_grouped_tile_items() { return TM; }

// ---------------------------------------------------------------------------------------
// ids [n_items] -> sorted [n_items] (items of expert 0, then of expert 1, ...), tiles (expert, first place in sorted,
// count) and their number.  One workgroup.  The order of an expert's items among themselves is not fixed; no result
// depends on it.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int n_items, int E, int* __restrict__ sorted,
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

extern "C" int ifx_moe_sort(const int* ids, int n_items, int E, int* sorted, int* tile_expert, int* tile_start, int* tile_count,
                            int* n_tiles, void* stream) {
  IFX_REQUIRE(n_items >= 0 && E > 0 && E <= MAX_EXPERTS, "moe_sort: %d items, %d experts (at most %d)", n_items, E, MAX_EXPERTS);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, ids, n_items, E, sorted, tile_expert, tile_start,
                     tile_count, n_tiles);
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
};

template <int MODE>
__global__ __launch_bounds__(256) void grouped_kernel(GroupedArgs a) {
  __shared__ __attribute__((aligned(16))) bf16_t ws[TN][LDP];
  __shared__ __attribute__((aligned(16))) bf16_t xs[TM][LDP];
  __shared__ int items[TM];
  const int tid = threadIdx.x;
  int group, start, count;
  if (MODE == MODE_HEADS) {
    const int per = (a.T + TM - 1) / TM;
    group = blockIdx.x / per;
    start = (blockIdx.x % per) * TM;
    count = min(TM, a.T - start);
  } else {
    if ((int)blockIdx.x >= *a.n_tiles) return;
    group = a.tile_expert[blockIdx.x];
    start = a.tile_start[blockIdx.x];
    count = a.tile_count[blockIdx.x];
  }
  const int n0 = blockIdx.y * TN;
  if (tid < TM) items[tid] = tid < count ? (MODE == MODE_HEADS ? start + tid : a.sorted[start + tid]) : -1;
  __syncthreads();
  const int wave = tid / WAVE, lane = tid % WAVE, col = lane & 15, g4 = lane >> 4;
  floatx4 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) acc[nt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16_t* wbase = a.w + (size_t)group * a.NW * a.K;
  const bf16_t* xbase = a.x + (size_t)group * a.x_group;
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (__bf16)0.f;
  // A step's pieces are asked for one step ahead: while the matrix cores work on step s from LDS, the loads of step
  // s + 1 are on their way into registers.
  bf16x8 wv[2], xv[2];
  const bf16_t* wp[2];
  const bf16_t* xp[2];
  int kc[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int piece = tid + 256 * p, r = piece / 8;
    kc[p] = 8 * (piece % 8);
    const int wrow = n0 + r, it = items[r];
    wp[p] = wrow < a.NW ? wbase + (size_t)wrow * a.K + kc[p] : nullptr;
    xp[p] = it >= 0 ? xbase + (size_t)(it / a.x_div) * a.x_row + kc[p] : nullptr;
  }
  auto fetch = [&](int k0) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const bool in = k0 + kc[p] < a.K;
      wv[p] = (wp[p] && in) ? *(const bf16x8*)(wp[p] + k0) : zero;
      xv[p] = (xp[p] && in) ? *(const bf16x8*)(xp[p] + k0) : zero;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < a.K; k0 += TK) {
    __syncthreads();          // everyone is done with the last step's tiles
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int piece = tid + 256 * p, r = piece / 8;
      *(bf16x8*)&ws[r][kc[p]] = wv[p];
      *(bf16x8*)&xs[r][kc[p]] = xv[p];
    }
    __syncthreads();
    if (k0 + TK < a.K) fetch(k0 + TK);
#pragma unroll
    for (int ks = 0; ks < TK / 32; ++ks) {
      const bf16x8 bop = *(const bf16x8*)&xs[16 * wave + col][32 * ks + 8 * g4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const bf16x8 aop = *(const bf16x8*)&ws[16 * nt + col][32 * ks + 8 * g4];
        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aop, bop, acc[nt], 0, 0, 0);
      }
    }
  }
  const int m = items[16 * wave + col];
  if (m < 0) return;
  if (MODE == MODE_GATE_UP) {
    // weight rows n0 .. n0 + 63 are 16 of Wg, the same 16 of Wu, the next 16 of Wg, of Wu: columns n0 / 2 .. + 31 of act
    const int ff = a.NW / 2;
    bf16_t* act = (bf16_t*)a.out + (size_t)m * ff;
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      const int f = n0 / 2 + 16 * pr + 4 * g4;
      if (f >= ff) continue;
      bf16x4 y;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = acc[2 * pr][r], u = acc[2 * pr + 1][r];
        y[r] = (__bf16)(g / (1.0f + expf(-g)) * u);
      }
      *(bf16x4*)(act + f) = y;
    }
  } else if (MODE == MODE_DOWN) {
    const float wgt = a.weights[m];
    float* o = (float*)a.out + ((size_t)(m % a.top) * a.T + m / a.top) * a.NW;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + 16 * nt + 4 * g4 + r;
        if (n < a.NW) o[n] = wgt * acc[nt][r];
      }
  } else {
    bf16_t* o = (bf16_t*)a.out + ((size_t)m * a.n_groups + group) * a.out_head;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + 16 * nt + 4 * g4 + r;
        if (n < a.NW) o[n] = (bf16_t)acc[nt][r];
      }
  }
}

static int check_common(int K, int x_row, int x_group) {
  return K > 0 && K % 8 == 0 && x_row % 8 == 0 && x_group % 8 == 0;
}

// act [n_items][ff] (bfloat16) from x [T][K] and the paired weights w [E][2 ff][K]; item i is row i / top.
extern "C" int ifx_moe_gate_up_grouped(const void* x, const void* w, void* act, const int* sorted, const int* tile_expert,
                                       const int* tile_start, const int* tile_count, const int* n_tiles, int max_tiles, int K,
                                       int ff, int top, void* stream) {
  IFX_REQUIRE(check_common(K, K, 0) && ff > 0 && ff % 16 == 0 && top > 0, "moe_gate_up_grouped: K=%d must be a multiple of 8, ff=%d of 16", K, ff);
  if (max_tiles <= 0) return 0;
  GroupedArgs a{(const bf16_t*)x, (const bf16_t*)w, act, sorted, tile_expert, tile_start, tile_count, n_tiles, nullptr,
                K, 2 * ff, top, K, 0, 0, top, 0, 0};
  hipLaunchKernelGGL(grouped_kernel<MODE_GATE_UP>, dim3(max_tiles, (2 * ff + TN - 1) / TN), dim3(256), 0, (hipStream_t)stream, a);
  IFX_LAUNCH_CHECK();
}

// parts [top][T][N] (float) = weights[item] * (Wd[e] act[item]), w [E][N][ff]
extern "C" int ifx_moe_down_grouped(const void* act, const void* w, float* parts, const float* weights, const int* sorted,
                                    const int* tile_expert, const int* tile_start, const int* tile_count, const int* n_tiles,
                                    int max_tiles, int T, int N, int ff, int top, void* stream) {
  IFX_REQUIRE(check_common(ff, ff, 0) && N > 0 && top > 0 && T >= 0, "moe_down_grouped: ff=%d must be a multiple of 8", ff);
  if (max_tiles <= 0 || T == 0) return 0;
  GroupedArgs a{(const bf16_t*)act, (const bf16_t*)w, parts, sorted, tile_expert, tile_start, tile_count, n_tiles, weights,
                ff, N, 1, ff, 0, T, top, 0, 0};
  hipLaunchKernelGGL(grouped_kernel<MODE_DOWN>, dim3(max_tiles, (N + TN - 1) / TN), dim3(256), 0, (hipStream_t)stream, a);
  IFX_LAUNCH_CHECK();
}

// out [T][H][out_head] (bfloat16): the first N elements of every head, W [H][N][K], head h of row t reads x + t * x_row + h * x_head
extern "C" int ifx_headwise_grouped(const void* x, const void* w, void* out, int T, int H, int K, int N, int x_row, int x_head,
                                    int out_head, void* stream) {
  IFX_REQUIRE(check_common(K, x_row, x_head) && N > 0 && H > 0 && out_head >= N, "headwise_grouped: K=%d, the rows of x (%d) and its heads (%d) must be multiples of 8", K, x_row, x_head);
  if (T <= 0) return 0;
  GroupedArgs a{(const bf16_t*)x, (const bf16_t*)w, out, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                K, N, 1, x_row, x_head, T, 1, out_head, H};
  hipLaunchKernelGGL(grouped_kernel<MODE_HEADS>, dim3(((T + TM - 1) / TM) * H, (N + TN - 1) / TN), dim3(256), 0, (hipStream_t)stream, a);
  IFX_LAUNCH_CHECK();
}
