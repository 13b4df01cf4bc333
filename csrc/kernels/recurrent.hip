// mLSTM matrix-memory scan over per-sequence state slots (hybrid decoders).
//
// Per (step sequence, head) the state is S [d, dv], n [d] and the running log-scale m,
// all fp32 in HBM between steps.  With log gates i_t, f_t:
//     m' = max(f + m, i);  S' = e^(f + m - m') S + e^(i - m') k v^T;  n' likewise with k
//     o_t = S'^T q / (max(|n'.q|, e^(-m')) + 1e-6),   q scaled by d^-1/2
// A sequence chunk that starts at position 0 starts from zero state; any other chunk reads
// the slot the previous step left.  Prefill chunks and decode rows are the same scan (a
// decode row is a chunk of one token).
//
// grid (step sequences, heads, ceil(dv / 64)), 256 threads.  A workgroup owns 64 value
// columns of one head's S: lane = column, wave w holds a contiguous quarter of the rows in
// registers for the whole chunk, so S is read and written once per step.  Every wave keeps
// the whole n (lane l: n[l], n[l + 64], ...) and computes the denominator itself.  Tokens
// go in blocks of 8: their q | k, value columns and gates are staged in LDS (the next
// block's loads are issued before the current block is computed and parked in registers),
// each wave walks the block without a barrier, leaving its row partials of the numerators
// in LDS, and the four partials of each token are summed after the block's barrier.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

constexpr int NT = 256;
constexpr int NW = NT / 64;

constexpr int TB = 8;      // tokens per block

// RMAX: rows of S per thread (d <= 4 * RMAX, RMAX a multiple of 4); NU: n entries per lane
template <typename T, int RMAX>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(
    float* __restrict__ out, const T* __restrict__ qkvg, int64_t stride,
    const float* __restrict__ gates, float* __restrict__ S, float* __restrict__ nst,
    float* __restrict__ mst, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ ctx_lens, const int* __restrict__ slots, int P, int Tp, int H,
    int d, int dv, int num_slots) {
  constexpr int NU = (4 * RMAX + 63) / 64;
  constexpr int NQK = (TB * 2 * 4 * RMAX + NT - 1) / NT;   // staged q | k values per thread
  constexpr int NV = TB * 64 / NT;                          // staged v values per thread
  extern __shared__ float lds[];
  const int dp = 4 * RMAX;                // padded row count: q | k rows are [2 * dp] in LDS
  float* qk = lds;                        // [TB][2 * dp]: q (scaled) | k, zero beyond d
  float* vv = qk + TB * 2 * dp;           // [TB][64]
  float* gg = vv + TB * 64;               // [TB][2]: log input gate, log forget gate
  float* dens = gg + TB * 2;              // [TB]
  float* part = dens + TB;                // [TB][NW][64]
  const int s = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = blockIdx.z * 64 + lane;
  const bool colok = col < dv;
  int start, len, pos0;
  if (s < P) {
    start = qsl[s];
    len = qsl[s + 1] - start;
    pos0 = seq_lens[s] - len;
  } else {
    start = Tp + (s - P);
    len = 1;
    pos0 = ctx_lens[s - P] - 1;
  }
  const int slot = slots[s];
  if (slot < 0 || slot >= num_slots || pos0 < 0 || len <= 0) {   // padding: defined zeros
    if (wave == 0 && colok)
      for (int t = 0; t < len; ++t) out[((int64_t)(start + t) * H + h) * dv + col] = 0.f;
    return;
  }
  float* Ss = S + ((int64_t)slot * H + h) * d * dv;
  float* ns = nst + ((int64_t)slot * H + h) * d;
  float* ms = mst + (int64_t)slot * H + h;
  float Sr[RMAX], nr[NU];
  float m = 0.f;
  const bool fresh = pos0 == 0;
  const int rbase = wave * RMAX;          // this wave's rows: rbase .. rbase + RMAX - 1
#pragma unroll
  for (int i = 0; i < RMAX; ++i) {
    const int r = rbase + i;
    Sr[i] = (!fresh && r < d && colok) ? Ss[(int64_t)r * dv + col] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int r = lane + 64 * u;
    nr[u] = (!fresh && r < d) ? ns[r] : 0.f;
  }
  if (!fresh) m = *ms;
  const float qscale = 1.f / sqrtf((float)d);
  const int koff = H * d, voff = 2 * H * d;
  float pqk[NQK], pv[NV], pg = 0.f;

  // global -> registers for the block of tokens starting at t0 (zeros beyond the chunk / d)
  auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < NQK; ++j) {
      const int e = threadIdx.x + NT * j;
      const int tb = e / (2 * dp), c = e - tb * 2 * dp;
      float val = 0.f;
      if (tb < TB && t0 + tb < len) {
        const T* row = qkvg + (int64_t)(start + t0 + tb) * stride;
        if (c < dp) { if (c < d) val = to_f(row[h * d + c]) * qscale; }
        else if (c - dp < d) val = to_f(row[koff + h * d + (c - dp)]);
      }
      pqk[j] = val;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int e = threadIdx.x + NT * j, tb = e >> 6, c = blockIdx.z * 64 + (e & 63);
      pv[j] = (t0 + tb < len && c < dv)
                  ? to_f(qkvg[(int64_t)(start + t0 + tb) * stride + voff + h * dv + c]) : 0.f;
    }
    if (threadIdx.x < 2 * TB) {
      const int tb = threadIdx.x >> 1, which = threadIdx.x & 1;
      pg = t0 + tb < len ? gates[(int64_t)(start + t0 + tb) * 2 * H + which * H + h] : 0.f;
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int j = 0; j < NQK; ++j) {
      const int e = threadIdx.x + NT * j;
      if (e < TB * 2 * dp) qk[e] = pqk[j];
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) vv[threadIdx.x + NT * j] = pv[j];
    if (threadIdx.x < 2 * TB) gg[threadIdx.x] = pg;
  };

  fetch(0);
  park();
  __syncthreads();
  for (int t0 = 0; t0 < len; t0 += TB) {
    const int nb = min(TB, len - t0);
    if (t0 + TB < len) fetch(t0 + TB);           // in flight while this block is computed
    for (int tb = 0; tb < nb; ++tb) {
      const float* cq = qk + tb * 2 * dp;
      const float* ck = cq + dp;
      const float ig = gg[2 * tb], fg = gg[2 * tb + 1];
      const float mn = fmaxf(fg + m, ig);
      const float fa = expf(fg + m - mn), ia = expf(ig - mn);
      m = mn;
      float nq = 0.f;
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        const int r = lane + 64 * u;            // r < dp always; rows beyond d hold zeros
        nr[u] = fa * nr[u] + ia * ck[r];
        nq += nr[u] * cq[r];
      }
      nq = wave_sum(nq);
      if (wave == 0 && lane == 0) dens[tb] = fmaxf(fabsf(nq), expf(-mn)) + 1e-6f;
      const float iv = ia * vv[tb * 64 + lane];
      float n0 = 0.f, n1 = 0.f, n2 = 0.f, n3 = 0.f;       // independent chains
#pragma unroll
      for (int i = 0; i < RMAX; i += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(ck + rbase + i);
        const float4 q4 = *reinterpret_cast<const float4*>(cq + rbase + i);
        Sr[i] = fa * Sr[i] + k4.x * iv;
        Sr[i + 1] = fa * Sr[i + 1] + k4.y * iv;
        Sr[i + 2] = fa * Sr[i + 2] + k4.z * iv;
        Sr[i + 3] = fa * Sr[i + 3] + k4.w * iv;
        n0 += Sr[i] * q4.x;
        n1 += Sr[i + 1] * q4.y;
        n2 += Sr[i + 2] * q4.z;
        n3 += Sr[i + 3] * q4.w;
      }
      const float num = (n0 + n1) + (n2 + n3);
      part[(tb * NW + wave) * 64 + lane] = num;
    }
    __syncthreads();                              // partials complete; qk / vv / gg consumed
    for (int tb = wave; tb < nb; tb += NW) {
      if (colok) {
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) tot += part[(tb * NW + w) * 64 + lane];
        out[((int64_t)(start + t0 + tb) * H + h) * dv + col] = tot / dens[tb];
      }
    }
    if (t0 + TB < len) park();
    __syncthreads();                              // next block staged; partials consumed
  }
  // the step's final state back to the slot
#pragma unroll
  for (int i = 0; i < RMAX; ++i) {
    const int r = rbase + i;
    if (r < d && colok) Ss[(int64_t)r * dv + col] = Sr[i];
  }
  if (blockIdx.z == 0 && wave == 0) {
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int r = lane + 64 * u;
      if (r < d) ns[r] = nr[u];
    }
    if (lane == 0) *ms = m;
  }
}

static size_t scan_lds(int rmax) {
  return sizeof(float) * (size_t)(TB * 2 * 4 * rmax + TB * 64 + TB * 2 + TB + TB * NW * 64);
}

template <typename T>
void scan_dispatch(float* out, const T* qkvg, int64_t stride, const float* gates, float* S,
                   float* nst, float* mst, const int* qsl, const int* seq_lens,
                   const int* ctx_lens, const int* slots, int P, int D, int Tp, int H, int d,
                   int dv, int num_slots, hipStream_t s) {
  const dim3 grid(P + D, H, (dv + 63) / 64);
#define KGC_SCAN(R)                                                                          \
  mlstm_scan_kernel<T, R><<<grid, NT, scan_lds(R), s>>>(out, qkvg, stride, gates, S, nst, mst, \
                                                        qsl, seq_lens, ctx_lens, slots, P, Tp, \
                                                        H, d, dv, num_slots)
  if (d <= 64) KGC_SCAN(16);
  else if (d <= 128) KGC_SCAN(32);
  else if (d <= 256) KGC_SCAN(64);
  else KGC_SCAN(128);
#undef KGC_SCAN
}

}  // namespace

int mlstm_scan_max_dim() { return 512; }

void launch_mlstm_scan(int dtype, float* out, const void* qkvg, int64_t stride,
                       const float* gates, float* S, float* nst, float* mst, const int* qsl,
                       const int* seq_lens, const int* ctx_lens, const int* slots, int P, int D,
                       int Tp, int H, int d, int dv, int num_slots, hipStream_t s) {
  if (P + D <= 0) return;
  if (dtype == DT_BF16)
    scan_dispatch<bf16>(out, (const bf16*)qkvg, stride, gates, S, nst, mst, qsl, seq_lens,
                        ctx_lens, slots, P, D, Tp, H, d, dv, num_slots, s);
  else if (dtype == DT_F16)
    scan_dispatch<f16>(out, (const f16*)qkvg, stride, gates, S, nst, mst, qsl, seq_lens,
                       ctx_lens, slots, P, D, Tp, H, d, dv, num_slots, s);
  else
    scan_dispatch<float>(out, (const float*)qkvg, stride, gates, S, nst, mst, qsl, seq_lens,
                         ctx_lens, slots, P, D, Tp, H, d, dv, num_slots, s);
}

// ---- token shift and minGRU over per-sequence state vectors -----------------------------
namespace {

// The step sequence that holds row t: prefill chunk i (rows [qsl[i], qsl[i + 1])) or decode
// row t - Tp.  first / last: the chunk's first and last row; pos0: position of the first.
struct SeqOfRow { int idx, first, last, pos0; };

__device__ __forceinline__ SeqOfRow seq_of_row(int t, const int* qsl, const int* seq_lens,
                                               const int* ctx_lens, int P, int Tp) {
  SeqOfRow r;
  if (t < Tp) {
    int lo = 0, hi = P - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
    }
    r.idx = lo;
    r.first = qsl[lo];
    r.last = qsl[lo + 1] - 1;
    r.pos0 = seq_lens[lo] - (qsl[lo + 1] - qsl[lo]);
  } else {
    r.idx = P + (t - Tp);
    r.first = r.last = t;
    r.pos0 = ctx_lens[t - Tp] - 1;
  }
  return r;
}

// One workgroup per row: out = h + (prev - h) * mu.  The workgroup of a chunk's first row
// is the only one that touches the sequence's state: it reads the previous step's last row
// from it and then stores this chunk's last row, so no other workgroup races with it.
template <typename O>
__global__ __launch_bounds__(NT) void token_shift_kernel(
    O* __restrict__ out, const float* __restrict__ h, const float* __restrict__ mu,
    float* __restrict__ state, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ ctx_lens, const int* __restrict__ slots, int P, int Tp, int W,
    int num_slots) {
  const int t = blockIdx.x;
  const SeqOfRow sq = seq_of_row(t, qsl, seq_lens, ctx_lens, P, Tp);
  const int slot = slots[sq.idx];
  O* o = out + (int64_t)t * W;
  if (slot < 0 || slot >= num_slots) {                 // a padding row
    for (int c = threadIdx.x; c < W; c += NT) o[c] = from_f<O>(0.f);
    return;
  }
  const float* hr = h + (int64_t)t * W;
  if (t != sq.first) {
    const float* pr = hr - W;
    for (int c = threadIdx.x; c < W; c += NT) {
      const float cur = hr[c];
      o[c] = from_f<O>(cur + (pr[c] - cur) * mu[c]);
    }
    return;
  }
  float* st = state + (int64_t)slot * W;
  const float* lr = h + (int64_t)sq.last * W;
  const bool fresh = sq.pos0 <= 0;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float cur = hr[c];
    const float prev = fresh ? 0.f : st[c];
    o[c] = from_f<O>(cur + (prev - cur) * mu[c]);
    st[c] = lr[c];
  }
}

__device__ __forceinline__ float sigmoidf_(float v) { return 1.f / (1.f + expf(-v)); }

// grid (step sequences, ceil(width / 64)), one wave: lane = channel, tokens in order, the
// loads of MG_UNROLL tokens in flight ahead of the dependent S chain.
constexpr int MG_UNROLL = 8;

template <typename T>
__global__ __launch_bounds__(64) void mingru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ zxg, int64_t stride,
    const float* __restrict__ bias, float* __restrict__ state, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ ctx_lens,
    const int* __restrict__ slots, int P, int Tp, int width, int num_slots, int s0) {
  const int s = blockIdx.x + s0, c = blockIdx.y * 64 + threadIdx.x;
  if (c >= width) return;
  int start, len, pos0;
  if (s < P) {
    start = qsl[s];
    len = qsl[s + 1] - start;
    pos0 = seq_lens[s] - len;
  } else {
    start = Tp + (s - P);
    len = 1;
    pos0 = ctx_lens[s - P] - 1;
  }
  const int slot = slots[s];
  if (slot < 0 || slot >= num_slots) {                 // a padding row
    for (int t = start; t < start + len; ++t) out[(int64_t)t * width + c] = from_f<T>(0.f);
    return;
  }
  float* st = state + (int64_t)slot * width + c;
  float S = pos0 <= 0 ? 0.f : *st;
  const float bz = bias[c], bx = bias[width + c];
  for (int t0 = 0; t0 < len; t0 += MG_UNROLL) {
    float zv[MG_UNROLL], uv[MG_UNROLL], gv[MG_UNROLL];
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      const int t = start + min(t0 + u, len - 1);
      const T* row = zxg + (int64_t)t * stride;
      zv[u] = to_f(row[c]);
      uv[u] = to_f(row[width + c]);
      gv[u] = to_f(row[2 * width + c]);
    }
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      if (t0 + u < len) {
        const float z = sigmoidf_(zv[u] + bz);
        const float x = uv[u] + bx;
        const float cand = x >= 0.f ? x + 0.5f : sigmoidf_(x);
        S = (1.f - z) * S + z * cand;
        const float g = gv[u];
        out[(int64_t)(start + t0 + u) * width + c] = from_f<T>(S * (g * sigmoidf_(g)));
      }
    }
  }
  *st = S;
}

// Long prefill chunks of few sequences: the chunk is cut into blocks of MG_BLOCK tokens that
// run in parallel.  S_t = a_t S_(t-1) + b_t composes: a block maps its incoming state S to
// A S + B with A = prod a_t and B its own scan from zero.
//   reduce  every block's (A, B) per channel                       -> ws[block][0 / 1]
//   carry   per sequence, in block order: ws[block][0] = incoming S; S = A S + B
//   apply   every block again, in token order from its incoming S: the outputs, and the
//           last block stores the sequence's state
// A block's incoming state differs from the token-by-token value by rounding only.
constexpr int MG_BLOCK = 64;

struct BlockOfSeq { int seq, lb, nb; };

// block b of the step -> its sequence, its index in it, the sequence's block count
__device__ __forceinline__ BlockOfSeq block_of_seq(int b, const int* qsl, int P) {
  BlockOfSeq r{-1, 0, 0};
  int acc = 0;
  for (int i = 0; i < P; ++i) {
    const int nb = (qsl[i + 1] - qsl[i] + MG_BLOCK - 1) / MG_BLOCK;
    if (b < acc + nb) {
      r.seq = i;
      r.lb = b - acc;
      r.nb = nb;
      return r;
    }
    acc += nb;
  }
  return r;
}

template <typename T>
__global__ __launch_bounds__(64) void mingru_block_reduce_kernel(
    float* __restrict__ ws, const T* __restrict__ zxg, int64_t stride,
    const float* __restrict__ bias, const int* __restrict__ qsl, int P, int width) {
  const int c = blockIdx.y * 64 + threadIdx.x;
  const BlockOfSeq bq = block_of_seq(blockIdx.x, qsl, P);
  if (c >= width || bq.seq < 0) return;
  const int start = qsl[bq.seq] + bq.lb * MG_BLOCK;
  const int len = min(MG_BLOCK, qsl[bq.seq + 1] - start);
  const float bz = bias[c], bx = bias[width + c];
  float A = 1.f, B = 0.f;
  for (int t0 = 0; t0 < len; t0 += MG_UNROLL) {
    float zv[MG_UNROLL], uv[MG_UNROLL];
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      const T* row = zxg + (int64_t)(start + min(t0 + u, len - 1)) * stride;
      zv[u] = to_f(row[c]);
      uv[u] = to_f(row[width + c]);
    }
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      if (t0 + u < len) {
        const float z = sigmoidf_(zv[u] + bz);
        const float x = uv[u] + bx;
        const float cand = x >= 0.f ? x + 0.5f : sigmoidf_(x);
        A *= 1.f - z;
        B = (1.f - z) * B + z * cand;
      }
    }
  }
  ws[((int64_t)blockIdx.x * 2 + 0) * width + c] = A;
  ws[((int64_t)blockIdx.x * 2 + 1) * width + c] = B;
}

__global__ __launch_bounds__(64) void mingru_block_carry_kernel(
    float* __restrict__ ws, const float* __restrict__ state, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int width, int num_slots) {
  const int s = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
  if (c >= width) return;
  int base = 0;
  for (int i = 0; i < s; ++i) base += (qsl[i + 1] - qsl[i] + MG_BLOCK - 1) / MG_BLOCK;
  const int len = qsl[s + 1] - qsl[s];
  const int nb = (len + MG_BLOCK - 1) / MG_BLOCK;
  const int slot = slots[s];
  const bool fresh = seq_lens[s] - len <= 0 || slot < 0 || slot >= num_slots;
  float S = fresh ? 0.f : state[(int64_t)slot * width + c];
  for (int b = base; b < base + nb; ++b) {
    float* w0 = ws + ((int64_t)b * 2 + 0) * width + c;
    const float A = *w0, B = w0[width];
    *w0 = S;
    S = A * S + B;
  }
}

template <typename T>
__global__ __launch_bounds__(64) void mingru_block_apply_kernel(
    T* __restrict__ out, const float* __restrict__ ws, const T* __restrict__ zxg, int64_t stride,
    const float* __restrict__ bias, float* __restrict__ state, const int* __restrict__ qsl,
    const int* __restrict__ slots, int P, int width, int num_slots) {
  const int c = blockIdx.y * 64 + threadIdx.x;
  const BlockOfSeq bq = block_of_seq(blockIdx.x, qsl, P);
  if (c >= width || bq.seq < 0) return;
  const int start = qsl[bq.seq] + bq.lb * MG_BLOCK;
  const int len = min(MG_BLOCK, qsl[bq.seq + 1] - start);
  const int slot = slots[bq.seq];
  if (slot < 0 || slot >= num_slots) {                 // a padding sequence
    for (int t = start; t < start + len; ++t) out[(int64_t)t * width + c] = from_f<T>(0.f);
    return;
  }
  const float bz = bias[c], bx = bias[width + c];
  float S = ws[((int64_t)blockIdx.x * 2) * width + c];
  for (int t0 = 0; t0 < len; t0 += MG_UNROLL) {
    float zv[MG_UNROLL], uv[MG_UNROLL], gv[MG_UNROLL];
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      const T* row = zxg + (int64_t)(start + min(t0 + u, len - 1)) * stride;
      zv[u] = to_f(row[c]);
      uv[u] = to_f(row[width + c]);
      gv[u] = to_f(row[2 * width + c]);
    }
#pragma unroll
    for (int u = 0; u < MG_UNROLL; ++u) {
      if (t0 + u < len) {
        const float z = sigmoidf_(zv[u] + bz);
        const float x = uv[u] + bx;
        const float cand = x >= 0.f ? x + 0.5f : sigmoidf_(x);
        S = (1.f - z) * S + z * cand;
        const float g = gv[u];
        out[(int64_t)(start + t0 + u) * width + c] = from_f<T>(S * (g * sigmoidf_(g)));
      }
    }
  }
  if (bq.lb == bq.nb - 1) state[(int64_t)slot * width + c] = S;
}

}  // namespace

int mingru_scan_blocks(int P, int Tp, int width) {
  // blocks pay off when the sequences alone leave most CUs idle and the chunks are long
  const bool on = P > 0 && Tp / P >= 8 * MG_BLOCK && (int64_t)P * ((width + 63) / 64) < 1024;
  return on ? Tp / MG_BLOCK + P : 0;
}

void launch_token_shift(int out_dtype, void* out, const float* h, const float* mu, float* state,
                        const int* qsl, const int* seq_lens, const int* ctx_lens,
                        const int* slots, int P, int Tp, int T_, int W, int num_slots,
                        hipStream_t s) {
  if (T_ <= 0) return;
  if (out_dtype == DT_BF16)
    token_shift_kernel<bf16><<<T_, NT, 0, s>>>((bf16*)out, h, mu, state, qsl, seq_lens, ctx_lens,
                                               slots, P, Tp, W, num_slots);
  else if (out_dtype == DT_F16)
    token_shift_kernel<f16><<<T_, NT, 0, s>>>((f16*)out, h, mu, state, qsl, seq_lens, ctx_lens,
                                              slots, P, Tp, W, num_slots);
  else
    token_shift_kernel<float><<<T_, NT, 0, s>>>((float*)out, h, mu, state, qsl, seq_lens,
                                                ctx_lens, slots, P, Tp, W, num_slots);
}

void launch_mingru_scan(int dtype, void* out, const void* zxg, int64_t stride, const float* bias,
                        float* state, const int* qsl, const int* seq_lens, const int* ctx_lens,
                        const int* slots, int P, int D, int Tp, int width, int num_slots,
                        float* ws, int ws_blocks, hipStream_t s) {
  if (P + D <= 0) return;
  const int cg = (width + 63) / 64;
  int s0 = 0, ns = P + D;
#define KGC_MG(T)                                                                               \
  do {                                                                                          \
    if (ws != nullptr && ws_blocks > 0) {                                                       \
      const dim3 gb(ws_blocks, cg);                                                             \
      mingru_block_reduce_kernel<T><<<gb, 64, 0, s>>>(ws, (const T*)zxg, stride, bias, qsl, P,  \
                                                      width);                                   \
      mingru_block_carry_kernel<<<dim3(P, cg), 64, 0, s>>>(ws, state, qsl, seq_lens, slots,     \
                                                           width, num_slots);                   \
      mingru_block_apply_kernel<T><<<gb, 64, 0, s>>>((T*)out, ws, (const T*)zxg, stride, bias,  \
                                                     state, qsl, slots, P, width, num_slots);   \
      s0 = P;                                                                                   \
      ns = D;                                                                                   \
    }                                                                                           \
    if (ns > 0)                                                                                 \
      mingru_scan_kernel<T><<<dim3(ns, cg), 64, 0, s>>>((T*)out, (const T*)zxg, stride, bias,   \
                                                        state, qsl, seq_lens, ctx_lens, slots,  \
                                                        P, Tp, width, num_slots, s0);           \
  } while (0)
  if (dtype == DT_BF16) KGC_MG(bf16);
  else if (dtype == DT_F16) KGC_MG(f16);
  else KGC_MG(float);
#undef KGC_MG
}

}  // namespace kgc
