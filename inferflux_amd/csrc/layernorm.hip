// Layer norm with a weight and no bias, over rows of up to MAX_H columns, all math in float:
//   y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w
// Two uses.  ifx_layernorm normalises rows of a tensor (the float32 stream before the head, optionally only the
// rows a list names, optionally with a delta added first).  ifx_add_layernorm is the arrangement in which the norm
// sits on a sub-block's output: stream[t] += LN(delta[t]) * w, and beside it the new stream rounded to the
// activation type, which is what the next sub-block reads.
//
// A workgroup takes a row, holds it in LDS as floats (read once from memory, partial sums of a sliced product added
// in slice order on the way), forms the mean and then the mean of the squared deviations from it, both by the
// fixed-order sums of common.h: a row's result never depends on the other rows of the launch.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_H 16000      // (the row and the sums fit 64 KB of LDS)

template <typename TX>
__device__ __forceinline__ float sliced(const TX* __restrict__ x, int i, int n_slices, size_t stride) {
  float v = to_f(x[i]);
  for (int s = 1; s < n_slices; ++s) v += to_f(x[(size_t)s * stride + i]);
  return v;
}

// the row's mean and 1 / sqrt(variance + eps) from the floats in `row`
__device__ __forceinline__ void moments(const float* row, int H, float eps, float* red, float& mean, float& rstd) {
  float s = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) s += row[i];
  mean = block_sum(s, red) / (float)H;
  float v = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float d = row[i] - mean;
    v = fmaf(d, d, v);
  }
  rstd = 1.0f / sqrtf(block_sum(v, red) / (float)H + eps);
}

template <typename TX, typename TD, typename TO>
__global__ __launch_bounds__(256) void layernorm_kernel(TX* __restrict__ x, const TD* __restrict__ delta, int n_slices,
                                                        size_t slice_stride, const void* __restrict__ weight, int w_dtype,
                                                        TO* __restrict__ out, const int* __restrict__ rows, int H, float eps,
                                                        int write_back) {
  extern __shared__ float row[];
  __shared__ float red[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  TX* xr = x + src * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_f(xr[i]);
    if (delta) {
      v += sliced(delta + src * H, i, n_slices, slice_stride);
      if (write_back) xr[i] = from_f<TX>(v);
    }
    row[i] = v;
  }
  __syncthreads();
  float mean, rstd;
  moments(row, H, eps, red, mean, rstd);
  TO* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = from_f<TO>((row[i] - mean) * rstd * load_dyn(weight, w_dtype, i));
}

template <typename TD, typename TC>
__global__ __launch_bounds__(256) void add_layernorm_kernel(float* __restrict__ stream, const TD* __restrict__ delta, int n_slices,
                                                            size_t slice_stride, const void* __restrict__ weight, int w_dtype,
                                                            TC* __restrict__ cast_out, int H, float eps) {
  extern __shared__ float row[];
  __shared__ float red[16];
  constexpr int NV = 8;          // rows of up to 256 NV columns: the stream and the weight are asked for before the sums
  const size_t t = blockIdx.x;
  float* s = stream + t * H;
  const bool ahead = H <= 256 * NV;
  float sv[NV], wv[NV];
  if (ahead) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = threadIdx.x + 256 * v;
      sv[v] = i < H ? s[i] : 0.f;
      wv[v] = i < H ? load_dyn(weight, w_dtype, i) : 0.f;
    }
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) row[i] = sliced(delta + t * H, i, n_slices, slice_stride);
  __syncthreads();
  float mean, rstd;
  moments(row, H, eps, red, mean, rstd);
  if (ahead) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int i = threadIdx.x + 256 * v;
      if (i < H) {
        const float x = sv[v] + (row[i] - mean) * rstd * wv[v];
        s[i] = x;
        if (cast_out) cast_out[t * H + i] = from_f<TC>(x);
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = s[i] + (row[i] - mean) * rstd * load_dyn(weight, w_dtype, i);
    s[i] = v;
    if (cast_out) cast_out[t * H + i] = from_f<TC>(v);
  }
}

template <typename TO>
__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f<TO>(x[i]);
}

// out = the float32 rows of x rounded to bfloat16 (what a sub-block that reads the stream itself is given first)
extern "C" int ifx_cast_rows(const float* x, void* out, int out_dtype, long long n, void* stream) {
  IFX_REQUIRE(n >= 0 && out_dtype == DT_BF16, "cast_rows: to bfloat16 only (dtype %d)", out_dtype);
  if (n == 0) return 0;
  hipLaunchKernelGGL(cast_rows_kernel<bf16_t>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, (bf16_t*)out, (size_t)n);
  IFX_LAUNCH_CHECK();
}

// out[r, :] = LN(x[src] (+ delta[src])) * weight, src = rows ? rows[r] : r.  x is float32 or bfloat16; with a delta
// and no row list the sum is written back to x.
extern "C" int ifx_layernorm(void* x, int x_dtype, const void* delta, int delta_dtype, int n_slices, long long slice_stride,
                             const void* weight, int w_dtype, void* out, int out_dtype, const int* rows, int n, int H,
                             float eps, void* stream) {
  IFX_REQUIRE(n >= 0 && H > 0 && H <= MAX_H, "layernorm: %d rows of %d columns (at most %d)", n, H, MAX_H);
  IFX_REQUIRE(n_slices >= 1, "layernorm: %d slices", n_slices);
  IFX_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "layernorm: unknown weight dtype %d", w_dtype);
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int wb = (delta && !rows) ? 1 : 0;
  const size_t lds = (size_t)H * sizeof(float);
#define LN_LAUNCH(TX, TD, TO) \
  hipLaunchKernelGGL((layernorm_kernel<TX, TD, TO>), dim3(n), dim3(256), lds, s, (TX*)x, (const TD*)delta, n_slices, \
                     (size_t)slice_stride, weight, w_dtype, (TO*)out, rows, H, eps, wb)
  const int dd = delta ? delta_dtype : DT_F32;
  if (x_dtype == DT_F32 && dd == DT_F32 && out_dtype == DT_F32) LN_LAUNCH(float, float, float);
  else if (x_dtype == DT_F32 && dd == DT_F32 && out_dtype == DT_BF16) LN_LAUNCH(float, float, bf16_t);
  else if (x_dtype == DT_F32 && dd == DT_BF16 && out_dtype == DT_BF16) LN_LAUNCH(float, bf16_t, bf16_t);
  else if (x_dtype == DT_BF16 && dd == DT_BF16 && out_dtype == DT_BF16) LN_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (x_dtype == DT_BF16 && dd == DT_F32 && out_dtype == DT_BF16) LN_LAUNCH(bf16_t, float, bf16_t);
  else IFX_FAIL("layernorm: unsupported types x=%d delta=%d out=%d", x_dtype, delta_dtype, out_dtype);
#undef LN_LAUNCH
  IFX_LAUNCH_CHECK();
}

// stream[t, :] += LN(delta[t, :]) * weight for every row; cast_out (or null) receives the new stream in cast_dtype.
extern "C" int ifx_add_layernorm(float* stream_rows, const void* delta, int delta_dtype, int n_slices, long long slice_stride,
                                 const void* weight, int w_dtype, void* cast_out, int cast_dtype, int T, int H, float eps,
                                 void* stream) {
  IFX_REQUIRE(T >= 0 && H > 0 && H <= MAX_H, "add_layernorm: %d rows of %d columns (at most %d)", T, H, MAX_H);
  IFX_REQUIRE(n_slices >= 1 && delta, "add_layernorm: needs a delta in at least one slice");
  IFX_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "add_layernorm: unknown weight dtype %d", w_dtype);
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = (size_t)H * sizeof(float);
#define ALN_LAUNCH(TD, TC) \
  hipLaunchKernelGGL((add_layernorm_kernel<TD, TC>), dim3(T), dim3(256), lds, s, stream_rows, (const TD*)delta, n_slices, \
                     (size_t)slice_stride, weight, w_dtype, (TC*)cast_out, H, eps)
  const int cd = cast_out ? cast_dtype : DT_BF16;
  if (delta_dtype == DT_F32 && cd == DT_BF16) ALN_LAUNCH(float, bf16_t);
  else if (delta_dtype == DT_F32 && cd == DT_F32) ALN_LAUNCH(float, float);
  else if (delta_dtype == DT_BF16 && cd == DT_BF16) ALN_LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == DT_BF16 && cd == DT_F32) ALN_LAUNCH(bf16_t, float);
  else IFX_FAIL("add_layernorm: unsupported types delta=%d cast=%d", delta_dtype, cast_dtype);
#undef ALN_LAUNCH
  IFX_LAUNCH_CHECK();
}
