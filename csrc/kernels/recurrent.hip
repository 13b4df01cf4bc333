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

}  // namespace kgc
