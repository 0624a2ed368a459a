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
// Cache layouts: K [page][kv head][offset][d], V [page][kv head][dv][offset].  Values may have another width
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
};

template <typename T>
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
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int keep = lo > 0 ? min(a.keep_first, lo) : 0;      // keys [0, keep) and [lo, pos] are seen

  const T* qrow = (const T*)a.q + ((size_t)row * a.nH + head) * d;
  for (int e = lane; e < d; e += WAVE) q_s[wid][e] = to_f(qrow[e]);
  // q_s[wid] is written and read by this wave only.
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0);

  // (the sink is a key of score sink_score whose value is zero: it starts the running maximum and sum)
  float m = a.has_sink ? a.sink_score : -INFINITY, l = a.has_sink ? 1.f : 0.f;
  float acc[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) acc[c] = 0.f;

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
    float s = -INFINITY;
    if (valid) {
      page = table[j / P];
      off = j % P;
      const T* kr = Kc + (((size_t)page * a.nKV + kvh) * P + off) * d;
      float dot = 0.f;
      if (d % 8 == 0) {        // the key's row in 16-byte pieces; the same additions in the same order
        for (int e = 0; e < d; e += 8) {
          float kv[8];
          load8(kr + e, kv);
#pragma unroll
          for (int i = 0; i < 8; ++i) dot = fmaf(q_s[wid][e + i], kv[i], dot);
        }
      } else {
        for (int e = 0; e < d; ++e) dot = fmaf(q_s[wid][e], to_f(kr[e]), dot);
      }
      s = dot * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the tile holds a visible key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[c] *= alpha;
    if (P % 8 == 0) {
      // Eight keys at a time: they lie in one page, where a value element's eight entries are 16 consecutive bytes.
      // Keys outside the range have weight 0 and their entries (stale or zero, never written with anything that is
      // not finite) add nothing; an element's sum still runs over the keys in ascending order.
      for (int g = 0; g < WAVE; g += 8) {
        const int j0 = t0 + g;
        if (j0 > pos || (j0 + 7 < lo && j0 >= keep)) continue;  // uniform over the wave
        float pj[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) pj[i] = __shfl(p, g + i, WAVE);
        const T* vb = Vc + ((size_t)table[j0 / P] * a.nKV + kvh) * dv * P + j0 % P;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          const int e = lane + c * WAVE;
          if (e < dv) {
            float vv[8];
            load8(vb + (size_t)e * P, vv);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[c] = fmaf(pj[i], vv[i], acc[c]);
          }
        }
      }
    } else
    for (int jj = 0; jj < WAVE; ++jj) {
      const float pj = __shfl(p, jj, WAVE);
      const int pg = __shfl(page, jj, WAVE), of = __shfl(off, jj, WAVE);
      if (pj == 0.f) continue;  // uniform over the wave; keys outside the range are never read
      const T* vb = Vc + ((size_t)pg * a.nKV + kvh) * dv * P + of;
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const int e = lane + c * WAVE;
        if (e < dv) acc[c] = fmaf(pj, to_f(vb[(size_t)e * P]), acc[c]);
      }
    }
    m = m_new;
  }
  T* orow = (T*)a.out + ((size_t)row * a.nH + head) * dv;
  const float inv = (l > 0.f ? 1.f / l : 0.f) * (a.gate ? a.gate[(size_t)row * a.nH + head] : 1.f);
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e = lane + c * WAVE;
    if (e < dv) orow[e] = from_f<T>(acc[c] * inv);
  }
}

extern "C" int ifx_attn_plain(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                              const int* row_req, const int* positions, const int* block_table,
                              int max_blocks, int T, int nH, int nKV, int d, int dv, int page_size, int window,
                              float scale, int keep_first, int has_sink, float sink_score, const float* gate, void* stream) {
  IFX_REQUIRE(keep_first >= 0, "attn_plain: keep_first %d", keep_first);
  IFX_REQUIRE(T >= 0 && nH > 0 && nKV > 0 && nH % nKV == 0, "attn_plain: bad head counts nH=%d nKV=%d", nH, nKV);
  IFX_REQUIRE(d > 0 && d <= MAX_D, "attn_plain: head_dim %d outside 1..%d", d, MAX_D);
  IFX_REQUIRE(dv > 0 && dv <= MAX_D, "attn_plain: value head_dim %d outside 1..%d", dv, MAX_D);
  IFX_REQUIRE(page_size > 0 && max_blocks > 0 && window >= 0, "attn_plain: bad page_size/max_blocks/window");
  if (T == 0) return 0;
  AttnArgs a{q, k_cache, v_cache, out, row_req, positions, block_table, max_blocks, T, nH, nKV, d, dv, page_size, window, scale, keep_first, has_sink, sink_score, gate};
  const long long items = (long long)T * nH;
  const unsigned blocks = (unsigned)((items + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32) hipLaunchKernelGGL(attn_plain_kernel<float>, dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else if (dtype == DT_BF16) hipLaunchKernelGGL(attn_plain_kernel<bf16_t>, dim3(blocks), dim3(WAVE * WAVES_PER_BLOCK), 0, s, a);
  else IFX_FAIL("attn_plain: unknown dtype %d", dtype);
  IFX_LAUNCH_CHECK();
}
