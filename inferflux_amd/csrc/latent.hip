// Helper kernels of attention through a latent: what lies between the mixer's matrix products and the paged
// attention kernels.
//
// The mixer projects its input down to a query latent, a key/value latent c (kv_rank wide) and one rotated key part
// k_r (rot_dim wide) that every head shares.  Per head the unrotated key is W_uk c and the value W_uv c, so the score
//   (q_n . W_uk c + q_r . k_r) * scale = ([W_uk^T q_n | q_r] . [c | k_r]) * scale
// and the head's output W_uv (sum_j a_j c_j): attention runs over one shared "kv head" whose key is [c | k_r]
// and whose value is c, with queries of kv_rank + rot_dim elements, and only c and k_r are cached.
//
//   ifx_latent_finish   after the down projections: RMS norm of the query latent (handed on), RMS norm of c and
//                       rotation of k_r, both written into the paged cache (K rows [c | k_r], V columns c; or V
//                       columns [c | k_r] too, for attention kernels that want values as wide as keys: the sums
//                       over k_r that they then return behind a head's kv_rank outputs are not used by anyone)
//   ifx_headwise        out[t, h, :] = W[h] x[t, h, :] for every head (W [H][N][K]), the products by W_uk^T and
//                       W_uv; optionally a tail of each head's input is rotated and appended to the head's output
//                       (the rotated query part)
//
// All sums in float in ascending k, one output element per thread: a row's result does not depend on the batch.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

template <typename TY>
__device__ __forceinline__ float sliced(const TY* __restrict__ y, int i, int n_slices, size_t stride) {
  float v = to_f(y[i]);
  for (int s = 1; s < n_slices; ++s) v += to_f(y[(size_t)s * stride + i]);
  return v;
}

// y [T][q_rank + kv_rank + rot_dim] (n_slices partial sums, slice_stride elements apart)
template <typename TY, typename T>
__global__ __launch_bounds__(256) void latent_finish_kernel(const TY* __restrict__ y, int n_slices, size_t slice_stride,
                                                            const void* __restrict__ wq, const void* __restrict__ wkv, int w_dtype,
                                                            const float* __restrict__ cs, const float* __restrict__ sn, int rot_dims,
                                                            const int* __restrict__ slots, T* __restrict__ cq,
                                                            T* __restrict__ k_cache, T* __restrict__ v_cache, int q_rank,
                                                            int kv_rank, int rot_dim, int page_size, float eps, int v_rows) {
  __shared__ float red[16];
  const size_t t = blockIdx.x;
  const int width = q_rank + kv_rank + rot_dim;
  const TY* yr = y + t * width;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
      const float v = sliced(yr, i, n_slices, slice_stride);
      ss = fmaf(v, v, ss);
    }
    const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      cq[t * q_rank + i] = from_f<T>(sliced(yr, i, n_slices, slice_stride) * r * load_dyn(wq, w_dtype, i));
  }
  if (!slots) return;
  const int slot = slots[t], page = slot / page_size, off = slot % page_size;
  const int d = kv_rank + rot_dim;
  T* krow = k_cache + (size_t)slot * d;                       // K [page][1][offset][d]
  T* vcol = v_cache + (size_t)page * v_rows * page_size + off;    // V [page][1][v_rows][offset], v_rows = kv_rank or d
  const TY* yc = yr + q_rank;
  float ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = sliced(yc, i, n_slices, slice_stride);
    ss = fmaf(v, v, ss);
  }
  const float r = 1.0f / sqrtf(block_sum(ss, red) / (float)kv_rank + eps);
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const T c = from_f<T>(sliced(yc, i, n_slices, slice_stride) * r * load_dyn(wkv, w_dtype, i));
    krow[i] = c;
    vcol[(size_t)i * page_size] = c;
  }
  const TY* yk = yc + kv_rank;
  const int half = rot_dims / 2;
  for (int i = threadIdx.x; i < rot_dim; i += blockDim.x) {
    float v = sliced(yk, i, n_slices, slice_stride);
    if (i < rot_dims) {
      const int p = i < half ? i : i - half;
      const float c = cs[t * half + p], s = sn[t * half + p];
      const float other = sliced(yk, i < half ? i + half : i - half, n_slices, slice_stride);
      v = i < half ? v * c - other * s : v * c + other * s;
    }
    krow[kv_rank + i] = from_f<T>(v);
    if (v_rows > kv_rank) vcol[(size_t)(kv_rank + i) * page_size] = from_f<T>(v);   // values as wide as keys: see the entry point
  }
}

extern "C" int ifx_latent_finish(const void* y, int y_dtype, int n_slices, long long slice_stride, const void* wq, const void* wkv,
                                 int w_dtype, const float* cs, const float* sn, int rot_dims, const int* slots, void* cq,
                                 void* k_cache, void* v_cache, int dtype, int T, int q_rank, int kv_rank, int rot_dim,
                                 int page_size, float eps, int v_rows, void* stream) {
  IFX_REQUIRE(T >= 0 && q_rank >= 0 && kv_rank > 0 && rot_dim >= 0, "latent_finish: bad sizes T=%d q_rank=%d kv_rank=%d rot_dim=%d", T, q_rank, kv_rank, rot_dim);
  IFX_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_dim, "latent_finish: %d of %d dimensions rotate", rot_dims, rot_dim);
  IFX_REQUIRE(rot_dims == 0 || (cs && sn), "latent_finish: a rotation needs its table");
  IFX_REQUIRE(!slots || (k_cache && v_cache && page_size > 0), "latent_finish: slots but no cache");
  IFX_REQUIRE(v_rows == kv_rank || v_rows == kv_rank + rot_dim, "latent_finish: values of %d rows (the latent's %d, or %d with the key part)", v_rows, kv_rank, kv_rank + rot_dim);
  IFX_REQUIRE(n_slices >= 1 && (n_slices == 1 || y_dtype == DT_F32), "latent_finish: partial sums are float32");
  IFX_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "latent_finish: unknown weight dtype %d", w_dtype);
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
#define LF_LAUNCH(TY, TT) \
  hipLaunchKernelGGL((latent_finish_kernel<TY, TT>), dim3(T), dim3(256), 0, s, (const TY*)y, n_slices, (size_t)slice_stride, wq, wkv, \
                     w_dtype, cs, sn, rot_dims, slots, (TT*)cq, (TT*)k_cache, (TT*)v_cache, q_rank, kv_rank, rot_dim, page_size, eps, v_rows)
  if (y_dtype == DT_F32 && dtype == DT_F32) LF_LAUNCH(float, float);
  else if (y_dtype == DT_F32 && dtype == DT_BF16) LF_LAUNCH(float, bf16_t);
  else if (y_dtype == DT_BF16 && dtype == DT_BF16) LF_LAUNCH(bf16_t, bf16_t);
  else IFX_FAIL("latent_finish: unsupported types y=%d out=%d", y_dtype, dtype);
#undef LF_LAUNCH
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// out[t][h][n] = sum_k W[h][n][k] * x[t][h * x_head + k]   (n < N), and for a tail of `tail` elements that follow
// the K inputs of each head, out[t][h][N + e] = the tail turned by the step's rotation table (its first rot_dims
// elements in split-half pairs, the rest as they are).  x rows are x_row apart, out rows H * (N + tail) wide.
struct HeadwiseArgs {
  const void* x; const void* w; void* out;
  const float* cs; const float* sn;
  int T, H, K, N, x_row, x_head, tail, rot_dims;
  int tile0;      // the launch's first tile (the tail's, when only the tails are wanted)
};

#define HW_TM 16
#define HW_TN 64
#define HW_TK 32

template <typename T>
__global__ __launch_bounds__(256) void headwise_kernel(HeadwiseArgs a) {
  __shared__ float xs[HW_TM][HW_TK];
  __shared__ float ws[HW_TN][HW_TK + 1];
  const int n_tiles = (a.N + HW_TN - 1) / HW_TN;
  const int h = blockIdx.y, t0 = blockIdx.x * HW_TM, tile = blockIdx.z + a.tile0;
  const int out_head = a.N + a.tail;
  const T* x = (const T*)a.x;
  T* out = (T*)a.out;
  if (tile == n_tiles) {      // the tail: rotate and copy
    const int half = a.rot_dims / 2;
    for (int idx = threadIdx.x; idx < HW_TM * a.tail; idx += blockDim.x) {
      const int t = t0 + idx / a.tail, e = idx % a.tail;
      if (t >= a.T) continue;
      const T* xt = x + (size_t)t * a.x_row + (size_t)h * a.x_head + a.K;
      float v = to_f(xt[e]);
      if (e < a.rot_dims) {
        const int p = e < half ? e : e - half;
        const float c = a.cs[(size_t)t * half + p], s = a.sn[(size_t)t * half + p];
        const float other = to_f(xt[e < half ? e + half : e - half]);
        v = e < half ? v * c - other * s : v * c + other * s;
      }
      out[((size_t)t * a.H + h) * out_head + a.N + e] = from_f<T>(v);
    }
    return;
  }
  const int n0 = tile * HW_TN;
  const int tx = threadIdx.x % HW_TN, ty = threadIdx.x / HW_TN;     // output column, group of four rows
  const T* w = (const T*)a.w + (size_t)h * a.N * a.K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < a.K; k0 += HW_TK) {
    for (int idx = threadIdx.x; idx < HW_TM * HW_TK; idx += blockDim.x) {
      const int m = idx / HW_TK, kk = idx % HW_TK, t = t0 + m, k = k0 + kk;
      xs[m][kk] = (t < a.T && k < a.K) ? to_f(x[(size_t)t * a.x_row + (size_t)h * a.x_head + k]) : 0.f;
    }
    for (int idx = threadIdx.x; idx < HW_TN * HW_TK; idx += blockDim.x) {
      const int n = idx / HW_TK, kk = idx % HW_TK, k = k0 + kk;
      ws[n][kk] = (n0 + n < a.N && k < a.K) ? to_f(w[(size_t)(n0 + n) * a.K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HW_TK; ++kk) {
      const float wv = ws[tx][kk];
#pragma unroll
      for (int m = 0; m < 4; ++m) acc[m] = fmaf(xs[ty * 4 + m][kk], wv, acc[m]);
    }
    __syncthreads();
  }
  if (n0 + tx < a.N)
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int t = t0 + ty * 4 + m;
      if (t < a.T) out[((size_t)t * a.H + h) * out_head + n0 + tx] = from_f<T>(acc[m]);
    }
}

// The same for steps of few rows: a thread owns one output element of one (row, head) and reads its weight row in
// 16-byte pieces, all asked for at once (a wave's rows are one contiguous run of memory); no LDS, no barrier.  The sum
// runs over k in the tiled kernel's order, so both give the same bits.
__device__ __forceinline__ void hw_load8(const bf16_t* p, float* v) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
  const bf16x8 t = *(const bf16x8*)p;
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (float)t[i];
}
__device__ __forceinline__ void hw_load8(const float* p, float* v) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

template <typename T>
__global__ __launch_bounds__(256) void headwise_rows_kernel(HeadwiseArgs a) {
  const int t = blockIdx.x, h = blockIdx.y, n = blockIdx.z * 256 + threadIdx.x;
  const int out_head = a.N + a.tail;
  const T* xt = (const T*)a.x + (size_t)t * a.x_row + (size_t)h * a.x_head;
  T* out = (T*)a.out + ((size_t)t * a.H + h) * out_head;
  if (n < a.N) {
    const T* w = (const T*)a.w + ((size_t)h * a.N + n) * a.K;
    float acc = 0.f;
#pragma unroll 4
    for (int k = 0; k < a.K; k += 8) {
      float xv[8], wv[8];
      hw_load8(xt + k, xv);
      hw_load8(w + k, wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc = fmaf(xv[i], wv[i], acc);
    }
    out[n] = from_f<T>(acc);
  } else if (n < out_head) {
    const int e = n - a.N, half = a.rot_dims / 2;
    float v = to_f(xt[a.K + e]);
    if (e < a.rot_dims) {
      const int p = e < half ? e : e - half;
      const float c = a.cs[(size_t)t * half + p], s = a.sn[(size_t)t * half + p];
      const float other = to_f(xt[a.K + (e < half ? e + half : e - half)]);
      v = e < half ? v * c - other * s : v * c + other * s;
    }
    out[n] = from_f<T>(v);
  }
}

#define HW_ROWS_MAX_T 16

extern "C" int ifx_headwise(const void* x, const void* w, void* out, int dtype, int T, int H, int K, int N, int x_row, int x_head,
                            int tail, const float* cs, const float* sn, int rot_dims, int tail_only, void* stream) {
  IFX_REQUIRE(T >= 0 && H > 0 && K > 0 && N > 0 && tail >= 0, "headwise: bad sizes T=%d H=%d K=%d N=%d tail=%d", T, H, K, N, tail);
  IFX_REQUIRE(x_head >= K + tail && x_row >= (H - 1) * x_head + K + tail, "headwise: the heads do not fit the rows of x");
  IFX_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= tail, "headwise: %d of a tail of %d rotate", rot_dims, tail);
  IFX_REQUIRE(rot_dims == 0 || (cs && sn), "headwise: a rotation needs its table");
  IFX_REQUIRE(H <= 65535, "headwise: %d heads", H);
  if (T == 0) return 0;
  HeadwiseArgs a{x, w, out, cs, sn, T, H, K, N, x_row, x_head, tail, rot_dims, 0};
  // tail_only: the products are somebody else's (the grouped matrix-core kernel's); only the tails are turned and copied
  IFX_REQUIRE(!tail_only || tail > 0, "headwise: tail_only without a tail");
  a.tile0 = tail_only ? (N + HW_TN - 1) / HW_TN : 0;
  hipStream_t s = (hipStream_t)stream;
  if (!tail_only && T <= HW_ROWS_MAX_T && K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0) {
    const dim3 grid(T, H, (N + tail + 255) / 256);
    if (dtype == DT_F32) hipLaunchKernelGGL(headwise_rows_kernel<float>, grid, dim3(256), 0, s, a);
    else if (dtype == DT_BF16) hipLaunchKernelGGL(headwise_rows_kernel<bf16_t>, grid, dim3(256), 0, s, a);
    else IFX_FAIL("headwise: unknown dtype %d", dtype);
    IFX_LAUNCH_CHECK();
  }
  const dim3 grid((T + HW_TM - 1) / HW_TM, H, tail_only ? 1 : (N + HW_TN - 1) / HW_TN + (tail > 0 ? 1 : 0));
  if (dtype == DT_F32) hipLaunchKernelGGL(headwise_kernel<float>, grid, dim3(256), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(headwise_kernel<bf16_t>, grid, dim3(256), 0, s, a);
  else IFX_FAIL("headwise: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
