// A selective state-space mixer's kernels: the short causal convolution with its activation, and the scan.
//
// Both work on a step's flattened rows (requests end to end, a request's rows in position order) and carry
// what a request needs from step to step in its state slot, one float32 row per slot:
//   [C * (taps - 1)]  the convolution's last taps - 1 inputs, [channel][oldest ... newest]
//   [C * N]           the recurrence's state S, [channel][state]
// A request that starts finds its slot zeroed, which is "zeros before the start" for the convolution and S = 0.
//
//   convolution   u[t, c] = silu(b[c] + sum_j w[c, j] x[t - (taps - 1) + j, c]), the last column of w the current
//                 token's; inputs before the step come from the slot, inputs before the request are zero.
//   scan          dt = softplus(dt_raw[t, c] + dt_bias[c]);  S[c, n] <- exp(dt A[c, n]) S[c, n] + dt u[t, c] B[t, n];
//                 y[t, c] = sum_n S[c, n] C[t, n] + D[c] u[t, c];  out[t, c] = y * silu(z[t, c]).
//
// Step sizes, decays, exponentials, the state and the sums are float whatever the activation type; u, B, C and z
// come in the activation type.  A token's result depends on the tokens of its request before it and on nothing
// else of the step: the order of the additions for (token, channel) is the same however the request was cut.
#include "common.h"

IFX_DEFINE_LAST_ERROR()

#define MAX_TAPS 16

struct ConvArgs {
  const void* x;         // [T, ld] of the activation type; the convolution's channels are columns 0 .. C-1
  int ld;
  const void* w;         // [C, taps]
  const void* b;         // [C] or null
  int w_dtype;
  float* state;          // [slots, state_stride]; the convolution's part starts at column 0
  size_t state_stride;
  const int* row_req;    // [T]
  const int* q_start;    // [R]
  const int* q_len;      // [R]
  const int* slots;      // [R]
  void* out;             // [T, C] of the activation type
  int T, R, C, taps;
};

template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(ConvArgs a) {
  const int c = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
  if (c >= a.C) return;
  const int r = a.row_req[t], t0 = a.q_start[r], i = t - t0, taps = a.taps;
  const float* st = a.state + (size_t)a.slots[r] * a.state_stride + (size_t)c * (taps - 1);
  const T* x = (const T*)a.x;
  float acc = a.b ? load_dyn(a.b, a.w_dtype, c) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = i - (taps - 1) + j;          // the input's place among the request's rows of this step
    const float xv = src >= 0 ? to_f(x[(size_t)(t0 + src) * a.ld + c]) : st[src + taps - 1];
    acc = fmaf(load_dyn(a.w, a.w_dtype, (size_t)c * taps + j), xv, acc);
  }
  ((T*)a.out)[(size_t)t * a.C + c] = from_f<T>(act_silu(acc));
}

// The same for bfloat16 rows with channels in eights and TAPS taps (known at compile time, so that every index below is):
// a thread takes eight neighbouring channels of one token, every tap's inputs as one 16-byte piece, the eight channels'
// weights as TAPS such pieces.  The sums are formed in the same order.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 conv_bf16x8;

// A workgroup is CONV_WG_ROWS consecutive rows by 256 / CONV_WG_ROWS threads of eight channels: a row that is an input of
// TAPS outputs is fetched from memory by one of them and found in the compute unit's cache by the others.
constexpr int CONV_WG_ROWS = 8;

template <int TAPS>
__global__ __launch_bounds__(256) void conv_silu_vec_kernel(ConvArgs a) {
  constexpr int WG_COLS = 256 / CONV_WG_ROWS;
  const int c = 8 * (blockIdx.x * WG_COLS + threadIdx.x % WG_COLS), t = blockIdx.y * CONV_WG_ROWS + threadIdx.x / WG_COLS;
  if (c >= a.C || t >= a.T) return;
  // Whether every input is a row of this step is known from two entries of row_req (a request's rows are contiguous), and
  // the TAPS rows before and at t exist whichever request they belong to: all of the thread's loads go out together.
  const int r = a.row_req[t], r_back = a.row_req[max(t - (TAPS - 1), 0)];
  const bf16_t* x = (const bf16_t*)a.x;
  conv_bf16x8 wv[TAPS], xv[TAPS];       // weights [8 channels][TAPS] as one run; inputs of tap j for the eight channels
#pragma unroll
  for (int j = 0; j < TAPS; ++j) wv[j] = *(const conv_bf16x8*)((const bf16_t*)a.w + (size_t)c * TAPS + 8 * j);
#pragma unroll
  for (int j = 0; j < TAPS; ++j) xv[j] = *(const conv_bf16x8*)(x + (size_t)max(t - (TAPS - 1) + j, 0) * a.ld + c);
  float acc[8];
  if (a.b) {
    const conv_bf16x8 b8 = *(const conv_bf16x8*)((const bf16_t*)a.b + c);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = (float)b8[e];
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  }
  if (t >= TAPS - 1 && r_back == r) {       // every input is a row of this step: the usual case
#pragma unroll
    for (int j = 0; j < TAPS; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf((float)wv[(e * TAPS + j) / 8][(e * TAPS + j) % 8], (float)xv[j][e], acc[e]);
  } else {
    const int t0 = a.q_start[r], i = t - t0;
    const float* st = a.state + (size_t)a.slots[r] * a.state_stride + (size_t)c * (TAPS - 1);
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int src = i - (TAPS - 1) + j;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float in = src >= 0 ? (float)x[(size_t)(t0 + src) * a.ld + c + e] : st[(size_t)e * (TAPS - 1) + src + TAPS - 1];
        acc[e] = fmaf((float)wv[(e * TAPS + j) / 8][(e * TAPS + j) % 8], in, acc[e]);
      }
    }
  }
  conv_bf16x8 y;
#pragma unroll
  for (int e = 0; e < 8; ++e) y[e] = (__bf16)act_silu(acc[e]);
  *(conv_bf16x8*)((bf16_t*)a.out + (size_t)t * a.C + c) = y;
}

// After the convolution has read the slots: every request's last taps - 1 inputs, from this step's rows and, where
// the step brought fewer, from what the slot held.  One thread owns a (request, channel): it reads before it writes.
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(ConvArgs a) {
  const int c = blockIdx.x * 256 + threadIdx.x, r = blockIdx.y;
  if (c >= a.C) return;
  const int n = a.q_len[r], t0 = a.q_start[r], keep = a.taps - 1;
  float* st = a.state + (size_t)a.slots[r] * a.state_stride + (size_t)c * keep;
  const T* x = (const T*)a.x;
  float v[MAX_TAPS - 1];
#pragma unroll
  for (int k = 0; k < MAX_TAPS - 1; ++k) {
    if (k >= keep) break;
    const int src = n - keep + k;
    v[k] = src >= 0 ? to_f(x[(size_t)(t0 + src) * a.ld + c]) : st[k + n];
  }
#pragma unroll
  for (int k = 0; k < MAX_TAPS - 1; ++k) {
    if (k >= keep) break;
    st[k] = v[k];
  }
}

extern "C" int ifx_causal_conv(const void* x, int dtype, int ld, const void* w, const void* b, int w_dtype, float* state,
                               long long state_stride, const int* row_req, const int* q_start, const int* q_len,
                               const int* slots, void* out, int T, int R, int C, int taps, void* stream) {
  IFX_REQUIRE(T >= 0 && R >= 0 && C > 0 && ld >= C, "causal_conv: bad sizes T=%d R=%d C=%d ld=%d", T, R, C, ld);
  IFX_REQUIRE(taps >= 1 && taps <= MAX_TAPS, "causal_conv: %d taps outside 1..%d", taps, MAX_TAPS);
  IFX_REQUIRE(state_stride >= (long long)C * (taps - 1), "causal_conv: a state row of %lld floats for %d x %d inputs", state_stride, C, taps - 1);
  IFX_REQUIRE(T <= 65535 && R <= 65535, "causal_conv: too many rows for one launch");
  if (T == 0 || R == 0) return 0;
  ConvArgs a{x, ld, w, b, w_dtype, state, (size_t)state_stride, row_req, q_start, q_len, slots, out, T, R, C, taps};
  hipStream_t s = (hipStream_t)stream;
  const unsigned cb = (unsigned)((C + 255) / 256);
  if (dtype == DT_F32) {
    hipLaunchKernelGGL(conv_silu_kernel<float>, dim3(cb, T), dim3(256), 0, s, a);
    if (taps > 1) hipLaunchKernelGGL(conv_state_kernel<float>, dim3(cb, R), dim3(256), 0, s, a);
  } else if (dtype == DT_BF16) {
    // (many rows only: a thread of eight channels leaves a step of few rows too few threads to fill the chip)
    const bool vec = C % 8 == 0 && ld % 8 == 0 && w_dtype == DT_BF16 && (long long)T * C >= (1 << 20);
    const dim3 vgrid((unsigned)((C / 8 + 256 / CONV_WG_ROWS - 1) / (256 / CONV_WG_ROWS)), (unsigned)((T + CONV_WG_ROWS - 1) / CONV_WG_ROWS));
    if (vec && taps == 4) hipLaunchKernelGGL(conv_silu_vec_kernel<4>, vgrid, dim3(256), 0, s, a);
    else if (vec && taps == 3) hipLaunchKernelGGL(conv_silu_vec_kernel<3>, vgrid, dim3(256), 0, s, a);
    else if (vec && taps == 2) hipLaunchKernelGGL(conv_silu_vec_kernel<2>, vgrid, dim3(256), 0, s, a);
    else
      hipLaunchKernelGGL(conv_silu_kernel<bf16_t>, dim3(cb, T), dim3(256), 0, s, a);
    if (taps > 1) hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(cb, R), dim3(256), 0, s, a);
  } else IFX_FAIL("causal_conv: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
struct ScanArgs {
  const void* u;         // [T, C] the convolution's output
  const float* dt_raw;   // [T, C] float: the step-size projection before bias and softplus
  const void* dt_bias;   // [C]
  const float* A;        // [C, N] float, negative
  const void* bc;        // [T, ld_bc]: B in columns 0 .. N-1, C in columns N .. 2N-1
  int ld_bc;
  const void* D;         // [C]
  int w_dtype;           // of dt_bias and D
  const void* z;         // [T, ld_z] the gate's input, first column at z
  int ld_z;
  float* state;          // [slots, state_stride]; S starts at column state_offset
  size_t state_stride, state_offset;
  const int* q_start;
  const int* q_len;
  const int* slots;
  void* out;             // [T, C]
  int R, C, N;
};

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// exp of a decay's exponent (<= 0).  With bfloat16 activations the hardware's 2^x (about two units in the last place of a
// float; a token's y is rounded to 8 bits of mantissa afterwards); in 32-bit the library's.
template <typename T> __device__ __forceinline__ float decay(float x) { return sizeof(T) == 2 ? __expf(x) : expf(x); }

// LANES lanes share a channel, each with NPT of its states (state n belongs to lane n / NPT); a token's sum over the
// states is added across them in a fixed order.  TOK tokens' inputs are asked for together, so that the recurrence,
// which is a chain from token to token, waits for memory once per TOK tokens.
//
// MODE 0: a workgroup row (blockIdx.y) is a request; its rows of the step are walked in order from the state in its
// slot, which receives the new state.  This is the whole scan for steps of few rows per request, and the only one in
// 32-bit, where a token's arithmetic must not depend on how its request was cut into steps.
// MODES 1-3 cut long portions into chunks that run side by side (the recurrence is linear in S: the state after a
// chunk is decay * (state before) + (state after the chunk from zero), decay = exp(A * sum of the chunk's dt)):
//   1  a workgroup row is a chunk: from S = 0 over the chunk's rows; writes the final S and the sum of dt, no output
//   2  a workgroup row is a request: walks its chunks, turns each chunk's entry into the state the chunk starts from,
//      and leaves the request's new state in its slot
//   3  a workgroup row is a chunk: from the state of pass 2 over the chunk's rows; writes the output
constexpr int LANES = 4, TOK = 4;

struct ChunkArgs {
  const int* chunk_req;    // [n_chunks] the request (place in the step) of each chunk
  const int* chunk_t0;     // [n_chunks] its first row of the step
  const int* chunk_len;    // [n_chunks]
  const int* req_chunk0;   // [R + 1] a request's chunks are req_chunk0[r] .. req_chunk0[r + 1] - 1
  float* chunk_state;      // [n_chunks, C, N]
  float* chunk_dt;         // [n_chunks, C]
};

template <typename T, int NPT, int MODE>
__global__ __launch_bounds__(256) void scan_kernel(ScanArgs a, ChunkArgs ch) {
  extern __shared__ __attribute__((aligned(16))) unsigned char scan_lds[];       // modes 1 and 3: the chunk's B and C rows
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int c_raw = idx / LANES, lg = idx % LANES;
  const bool active = c_raw < a.C;      // (the lanes of a channel are active together; in modes 1 and 3 nobody leaves before the barrier)
  if ((MODE == 0 || MODE == 2) && !active) return;
  const int c = active ? c_raw : a.C - 1;
  const int N = a.N, n0 = lg * NPT;
  float An[NPT];
#pragma unroll
  for (int k = 0; k < NPT; ++k) An[k] = n0 + k < N ? a.A[(size_t)c * N + n0 + k] : 0.f;
  if (MODE == 2) {
    const int r = blockIdx.y;
    float* S_mem = a.state + (size_t)a.slots[r] * a.state_stride + a.state_offset + (size_t)c * N + n0;
    float S[NPT];
#pragma unroll
    for (int k = 0; k < NPT; ++k) S[k] = n0 + k < N ? S_mem[k] : 0.f;
    for (int q = ch.req_chunk0[r]; q < ch.req_chunk0[r + 1]; ++q) {
      float* cs = ch.chunk_state + ((size_t)q * a.C + c) * N + n0;
      const float sum_dt = ch.chunk_dt[(size_t)q * a.C + c];
#pragma unroll
      for (int k = 0; k < NPT; ++k)
        if (n0 + k < N) {
          const float local = cs[k];
          cs[k] = S[k];
          S[k] = fmaf(expf(sum_dt * An[k]), S[k], local);
        }
    }
#pragma unroll
    for (int k = 0; k < NPT; ++k)
      if (n0 + k < N) S_mem[k] = S[k];
    return;
  }
  const int item = blockIdx.y;
  const int r = MODE == 0 ? item : ch.chunk_req[item];
  const int t0 = MODE == 0 ? a.q_start[r] : ch.chunk_t0[item], n_tok = MODE == 0 ? a.q_len[r] : ch.chunk_len[item];
  float* S_mem = MODE == 0 ? a.state + (size_t)a.slots[r] * a.state_stride + a.state_offset + (size_t)c * N + n0
                           : ch.chunk_state + ((size_t)item * a.C + c) * N + n0;
  float S[NPT];
#pragma unroll
  for (int k = 0; k < NPT; ++k) S[k] = (MODE != 1 && n0 + k < N) ? S_mem[k] : 0.f;
  const float dtb = load_dyn(a.dt_bias, a.w_dtype, c), Dc = load_dyn(a.D, a.w_dtype, c);
  const T* u = (const T*)a.u;
  const T* bc = (const T*)a.bc;
  const T* z = (const T*)a.z;
  float sum_dt = 0.f;
  // Modes 1 and 3: a chunk's B and C are the same for every channel; the workgroup copies them into LDS once (rows of
  // 2 N, the chunk's first row first) and the walk below reads them there instead of from memory.
  constexpr bool STAGED = MODE == 1 || MODE == 3;
  T* bc_s = (T*)scan_lds;
  if (STAGED) {
    const int per_row = 2 * N, total = n_tok * per_row;
    for (int i = threadIdx.x; i < total; i += 256) bc_s[i] = bc[(size_t)(t0 + i / per_row) * a.ld_bc + i % per_row];
    __syncthreads();
    if (!active) return;
  }
  const T* bc_rows = STAGED ? bc_s : bc + (size_t)t0 * a.ld_bc;        // row i of the walk starts at bc_rows + i * bc_ld
  const int bc_ld = STAGED ? 2 * N : a.ld_bc;
  // B and C of a token in 8-byte pieces where the sizes allow it (bfloat16, states in fours)
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 scan_bf16x4;
  const bool pieces = sizeof(T) == 2 && NPT % 4 == 0 && N % 4 == 0 && bc_ld % 4 == 0;
  const int lane0 = (threadIdx.x % WAVE) & ~(LANES - 1);      // the first of the channel's lanes
  for (int i0 = 0; i0 < n_tok; i0 += TOK) {
    float Bv[TOK][NPT], Cv[TOK][NPT];
    // Of the TOK tokens' inputs that all lanes of a channel need alike (u, the step size, the gate's input) each lane
    // fetches one token's and forms its step size; the others get them by shuffles (TOK == LANES).
    static_assert(TOK == LANES, "a channel's lanes take one token each");
    const size_t t_my = (size_t)t0 + min(i0 + lg, n_tok - 1);
    const float u_my = to_f(u[t_my * a.C + c]);
    const float dt_my = softplus_f(a.dt_raw[t_my * a.C + c] + dtb);
    const float z_my = MODE == 1 ? 0.f : to_f(z[t_my * a.ld_z + c]);
#pragma unroll
    for (int q = 0; q < TOK; ++q) {
      const bool live = i0 + q < n_tok;
      const T* row = bc_rows + (size_t)(i0 + (live ? q : 0)) * bc_ld;
      if (pieces) {
#pragma unroll
        for (int k = 0; k < NPT; k += 4) {
          const int n = min(n0 + k, N - 4);
          const scan_bf16x4 b4 = *(const scan_bf16x4*)((const bf16_t*)row + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) Bv[q][k + e] = (float)b4[e];
          if (MODE != 1) {
            const scan_bf16x4 c4 = *(const scan_bf16x4*)((const bf16_t*)row + N + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) Cv[q][k + e] = (float)c4[e];
          }
        }
      } else {
#pragma unroll
        for (int k = 0; k < NPT; ++k) {
          const int n = min(n0 + k, N - 1);
          Bv[q][k] = to_f(row[n]);
          Cv[q][k] = MODE == 1 ? 0.f : to_f(row[N + n]);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < TOK; ++q) {
      const float uq = __shfl(u_my, lane0 + q, WAVE), dt = __shfl(dt_my, lane0 + q, WAVE), zq = __shfl(z_my, lane0 + q, WAVE);
      if (i0 + q >= n_tok) break;
      const float dtu = dt * uq;
      sum_dt += dt;
      float y = 0.f;
#pragma unroll
      for (int k = 0; k < NPT; ++k) {
        if (n0 + k < N) {
          S[k] = fmaf(decay<T>(dt * An[k]), S[k], dtu * Bv[q][k]);
          if (MODE != 1) y = fmaf(S[k], Cv[q][k], y);
        }
      }
      if (MODE != 1) {
        y += __shfl_xor(y, 1, WAVE);      // the channel's four lanes are neighbours
        y += __shfl_xor(y, 2, WAVE);
        if (lg == 0) {
          y = fmaf(Dc, uq, y);
          ((T*)a.out)[((size_t)t0 + i0 + q) * a.C + c] = from_f<T>(y * act_silu(zq));
        }
      }
    }
  }
  if (MODE == 3) return;
#pragma unroll
  for (int k = 0; k < NPT; ++k)
    if (n0 + k < N) S_mem[k] = S[k];
  if (MODE == 1 && lg == 0) ch.chunk_dt[(size_t)item * a.C + c] = sum_dt;
}

template <typename T>
static int launch_scan(const ScanArgs& a, const ChunkArgs& ch, int n_chunks, int max_chunk, hipStream_t s) {
  const size_t lds = (size_t)max_chunk * 2 * a.N * sizeof(T);      // a chunk's B and C rows
  IFX_REQUIRE(n_chunks <= 0 || (max_chunk > 0 && lds <= 64 * 1024), "selective_scan: chunks of %d rows x %d states need %zu bytes of LDS",
              max_chunk, a.N, lds);
  const int npt = (a.N + LANES - 1) / LANES;
  const unsigned gx = (unsigned)(((size_t)a.C * LANES + 255) / 256);
  const dim3 grid(gx, a.R), grid_chunks(gx, n_chunks > 0 ? n_chunks : 1);
#define GO(NPT_)                                                                                  \
  do {                                                                                            \
    if (n_chunks <= 0) hipLaunchKernelGGL((scan_kernel<T, NPT_, 0>), grid, dim3(256), 0, s, a, ch); \
    else {                                                                                        \
      hipLaunchKernelGGL((scan_kernel<T, NPT_, 1>), grid_chunks, dim3(256), lds, s, a, ch);         \
      hipLaunchKernelGGL((scan_kernel<T, NPT_, 2>), grid, dim3(256), 0, s, a, ch);                \
      hipLaunchKernelGGL((scan_kernel<T, NPT_, 3>), grid_chunks, dim3(256), lds, s, a, ch);         \
    }                                                                                             \
  } while (0)
  if (npt <= 1) GO(1);
  else if (npt <= 2) GO(2);
  else if (npt <= 4) GO(4);
  else if (npt <= 6) GO(6);
  else if (npt <= 8) GO(8);
  else if (npt <= 12) GO(12);
  else if (npt <= 16) GO(16);
  else if (npt <= 32) GO(32);
  else IFX_FAIL("selective_scan: %d states per channel (at most %d)", a.N, 32 * LANES);
#undef GO
  IFX_LAUNCH_CHECK();
}

extern "C" int ifx_selective_scan(const void* u, int dtype, const float* dt_raw, const void* dt_bias, const float* A,
                                  const void* bc, int ld_bc, const void* D, int w_dtype, const void* z, int ld_z,
                                  float* state, long long state_stride, long long state_offset, const int* q_start,
                                  const int* q_len, const int* slots, void* out, int T, int R, int C, int N,
                                  int n_chunks, int max_chunk, const int* chunk_req, const int* chunk_t0, const int* chunk_len,
                                  const int* req_chunk0, float* chunk_state, float* chunk_dt, void* stream) {
  IFX_REQUIRE(n_chunks >= 0 && n_chunks <= 65535, "selective_scan: %d chunks", n_chunks);
  IFX_REQUIRE(n_chunks == 0 || (chunk_req && chunk_t0 && chunk_len && req_chunk0 && chunk_state && chunk_dt),
              "selective_scan: chunks need their lists and scratch");
  IFX_REQUIRE(T >= 0 && R >= 0 && C > 0 && N > 0, "selective_scan: bad sizes T=%d R=%d C=%d N=%d", T, R, C, N);
  IFX_REQUIRE(ld_bc >= 2 * N && ld_z >= C, "selective_scan: rows of %d for B and C of %d, of %d for a gate of %d", ld_bc, N, ld_z, C);
  IFX_REQUIRE(state_stride >= state_offset + (long long)C * N, "selective_scan: a state row of %lld floats for %lld + %d x %d", state_stride, state_offset, C, N);
  IFX_REQUIRE(R <= 65535, "selective_scan: too many requests for one launch");
  if (T == 0 || R == 0) return 0;
  ScanArgs a{u, dt_raw, dt_bias, A, bc, ld_bc, D, w_dtype, z, ld_z, state, (size_t)state_stride, (size_t)state_offset,
             q_start, q_len, slots, out, R, C, N};
  const ChunkArgs ch{chunk_req, chunk_t0, chunk_len, req_chunk0, chunk_state, chunk_dt};
  if (dtype == DT_F32) return launch_scan<float>(a, ch, n_chunks, max_chunk, (hipStream_t)stream);
  if (dtype == DT_BF16) return launch_scan<bf16_t>(a, ch, n_chunks, max_chunk, (hipStream_t)stream);
  IFX_FAIL("selective_scan: unknown dtype %d", dtype);
}
