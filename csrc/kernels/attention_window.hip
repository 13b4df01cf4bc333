// Windowed attention with kept first tokens over a plain-layout paged cache
// (k [nb, G, bs, dk], v [nb, G, bs, dv]; dk != dv allowed, any sizes), for the hybrid
// decoders.  Query i sees key j when j <= i and (i - j < window or j < keep_first);
// window <= 0 means plain causal attention.
//
//   rope_kv_store     rotates q and k on the first `rot` dims of a head (pair i, i + rot/2;
//                     cos / sin from an fp32 table), writes q, and k / v into the cache
//   window_attention  one wave per (token, query head): the token's visible keys are the
//                     kept first tokens plus the window, walked 64 keys at a time (one key
//                     per lane for the scores, one value column per lane for P.V) with an
//                     online softmax.  Prefill chunks and decode rows of a step take the
//                     same path, so a position's result does not depend on how the prompt
//                     was cut.  Scores, softmax weights and the weighted sum are fp32.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void rope_kv_store_kernel(
    const T* __restrict__ qkv, int64_t qkv_stride, const int64_t* __restrict__ positions,
    const float* __restrict__ table, int rot, int table_rows, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int64_t* __restrict__ slots, int H,
    int G, int dk, int dv, int bs, int num_blocks) {
  const int64_t t = blockIdx.x;
  const T* row = qkv + t * qkv_stride;
  int64_t pos = positions[t];
  if (pos < 0) pos = 0;
  if (pos >= table_rows) pos = table_rows - 1;        // host checks max_pos; never read past
  const float* cs = table != nullptr ? table + pos * rot : nullptr;
  const int half = rot >> 1;
  const int64_t slot = slots[t];
  const bool store = slot >= 0 && slot < (int64_t)num_blocks * bs;
  const int64_t blk = store ? slot / bs : 0, off = store ? slot % bs : 0;
  // q heads then k heads: (H + G) * dk elements, rotated pairwise on the first `rot` dims
  const int nqk = (H + G) * dk;
  for (int e = threadIdx.x; e < nqk; e += 256) {
    const int head = e / dk, i = e - head * dk;
    float v = to_f(row[e]);
    if (i < rot) {
      const int p = i < half ? i : i - half;
      const float c = cs[p], sn = cs[half + p];
      const float a = to_f(row[head * dk + p]), b = to_f(row[head * dk + half + p]);
      float oa, ob;
      neox_rot(a, b, c, sn, oa, ob);
      v = i < half ? oa : ob;
    }
    if (head < H) {
      q_out[(t * H + head) * dk + i] = from_f<T>(v);
    } else if (store) {
      k_cache[((blk * G + (head - H)) * bs + off) * dk + i] = from_f<T>(v);
    }
  }
  if (store) {
    const T* vrow = row + nqk;
    for (int e = threadIdx.x; e < G * dv; e += 256) {
      const int g = e / dv, i = e - g * dv;
      v_cache[((blk * G + g) * bs + off) * dv + i] = vrow[e];
    }
  }
}

constexpr int MAX_DV_PER_LANE = 8;     // dv <= 512

// grid (T, H), one wave.  LDS: q row [dk] fp32, p [64], value-row offsets [64].
template <typename T>
__global__ __launch_bounds__(64) void window_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ pbt, const int* __restrict__ ctx_lens, const int* __restrict__ dbt,
    int bt_stride, int P, int Tp, int H, int G, int dk, int dv, int bs, int num_blocks,
    float scale, int window, int keep_first, const float* __restrict__ gate) {
  extern __shared__ float lds[];
  float* qs = lds;                  // [dk]
  float* pw = lds + dk;             // [64]
  int* voff = (int*)(pw + 64);      // [64] (block * G + g) * bs + row
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  T* orow = out + ((int64_t)t * H + h) * dv;
  int pos;
  const int* bt;
  if (t < Tp) {
    int lo = 0, hi = P - 1;          // the sequence whose rows [qsl[i], qsl[i+1]) hold t
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
    }
    pos = seq_lens[lo] - (qsl[lo + 1] - qsl[lo]) + (t - qsl[lo]);
    bt = pbt + (int64_t)lo * bt_stride;
  } else {
    const int dd = t - Tp;
    pos = ctx_lens[dd] - 1;
    bt = dbt + (int64_t)dd * bt_stride;
  }
  if (pos < 0 || pos >= bt_stride * bs) {      // a padding row (or nothing to attend)
    for (int c = lane; c < dv; c += 64) orow[c] = from_f<T>(0.f);
    return;
  }
  const T* qrow = q + ((int64_t)t * H + h) * dk;
  for (int c = lane; c < dk; c += 64) qs[c] = to_f(qrow[c]);
  __syncthreads();
  const int lo_w = window > 0 ? max(0, pos - window + 1) : 0;
  const int ns = min(keep_first, lo_w);           // kept first tokens outside the window
  const int total = ns + (pos - lo_w + 1);
  float m = -INFINITY, l = 0.f;
  float acc[MAX_DV_PER_LANE];
#pragma unroll
  for (int u = 0; u < MAX_DV_PER_LANE; ++u) acc[u] = 0.f;
  for (int base = 0; base < total; base += 64) {
    const int idx = base + lane;
    const bool ok = idx < total;
    float s = -INFINITY;
    int ro = 0;
    if (ok) {
      const int j = idx < ns ? idx : lo_w + (idx - ns);
      int b = bt[j / bs];
      if (b < 0 || b >= num_blocks) b = 0;       // never index outside the pool
      ro = (b * G + g) * bs + (j % bs);
      const T* kr = k_cache + (int64_t)ro * dk;
      float d = 0.f;
      for (int c = 0; c < dk; ++c) d += qs[c] * to_f(kr[c]);
      s = d * scale;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float alpha = expf(m - mn);             // m = -inf at first: exp(-inf) = 0
    const float p = ok ? expf(s - mn) : 0.f;
    l = l * alpha + wave_sum(p);
    m = mn;
    __syncthreads();                              // the previous chunk's pw / voff were read
    pw[lane] = p;
    voff[lane] = ro;
    __syncthreads();
    const int cnt = min(64, total - base);
#pragma unroll
    for (int u = 0; u < MAX_DV_PER_LANE; ++u) {
      const int c = lane + 64 * u;
      if (c < dv) {
        float a = acc[u] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a += pw[jj] * to_f(v_cache[(int64_t)voff[jj] * dv + c]);
        acc[u] = a;
      }
    }
  }
  const float gt = gate != nullptr ? gate[(int64_t)t * H + h] : 1.f;
  const float inv = gt / l;
#pragma unroll
  for (int u = 0; u < MAX_DV_PER_LANE; ++u) {
    const int c = lane + 64 * u;
    if (c < dv) orow[c] = from_f<T>(acc[u] * inv);
  }
}

}  // namespace

#define KGC_DISPATCH_T(dtype, ...)                          \
  do {                                                      \
    if ((dtype) == DT_BF16) { typedef bf16 T; __VA_ARGS__; } \
    else if ((dtype) == DT_F16) { typedef f16 T; __VA_ARGS__; } \
    else { typedef float T; __VA_ARGS__; }                  \
  } while (0)

void launch_rope_kv_store(int dtype, const void* qkv, int64_t qkv_stride,
                          const int64_t* positions, const float* table, int rot, int table_rows,
                          void* q_out, void* k_cache, void* v_cache, const int64_t* slots, int T_,
                          int H, int G, int dk, int dv, int bs, int num_blocks, hipStream_t s) {
  if (T_ <= 0) return;
  KGC_DISPATCH_T(dtype, rope_kv_store_kernel<T><<<T_, 256, 0, s>>>(
      (const T*)qkv, qkv_stride, positions, table, rot, table_rows, (T*)q_out, (T*)k_cache,
      (T*)v_cache, slots, H, G, dk, dv, bs, num_blocks));
}

int window_attention_max_dv() { return 64 * MAX_DV_PER_LANE; }

void launch_window_attention(int dtype, void* out, const void* q, const void* k_cache,
                             const void* v_cache, const int* qsl, const int* seq_lens,
                             const int* pbt, const int* ctx_lens, const int* dbt, int bt_stride,
                             int P, int Tp, int T_, int H, int G, int dk, int dv, int bs,
                             int num_blocks, float scale, int window, int keep_first,
                             const float* gate, hipStream_t s) {
  if (T_ <= 0) return;
  const size_t lds = (size_t)(dk + 128) * sizeof(float);
  KGC_DISPATCH_T(dtype, window_attention_kernel<T><<<dim3(T_, H), 64, lds, s>>>(
      (T*)out, (const T*)q, (const T*)k_cache, (const T*)v_cache, qsl, seq_lens, pbt, ctx_lens,
      dbt, bt_stride, P, Tp, H, G, dk, dv, bs, num_blocks, scale, window, keep_first, gate));
}

}  // namespace kgc
