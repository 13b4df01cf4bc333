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
// columns of one head's S: lane = column, wave w holds rows w, w + 4, ... in registers for
// the whole chunk, so S is read and written once per step.  Every wave keeps the whole n
// (lane l: n[l], n[l + 64], ...) and computes the denominator itself; the numerator's four
// row partials meet in LDS.  q / k of token t + 1 are fetched into registers while token t
// is computed and parked in a second LDS buffer before the token's single barrier.
#include "common.h"
#include "launch.h"

namespace kgc {

namespace {

constexpr int NT = 256;
constexpr int NW = NT / 64;

// RMAX: rows of S per thread (d <= 4 * RMAX); NU: n entries per lane (d <= 64 * NU)
template <typename T, int RMAX>
__global__ __launch_bounds__(NT) void mlstm_scan_kernel(
    float* __restrict__ out, const T* __restrict__ qkvg, int64_t stride,
    const float* __restrict__ gates, float* __restrict__ S, float* __restrict__ nst,
    float* __restrict__ mst, const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int* __restrict__ ctx_lens, const int* __restrict__ slots, int P, int Tp, int H,
    int d, int dv, int num_slots) {
  constexpr int NU = (4 * RMAX + 63) / 64;
  extern __shared__ float lds[];
  float* qk = lds;                       // [2][2 * d]: q | k of a token, double-buffered
  float* part = lds + 4 * d;             // [2][NW][64]
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
#pragma unroll
  for (int i = 0; i < RMAX; ++i) {
    const int r = wave + NW * i;
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
  // prologue: token 0's q | k into LDS buffer 0
  {
    const T* row = qkvg + (int64_t)start * stride;
    for (int e = threadIdx.x; e < 2 * d; e += NT)
      qk[e] = e < d ? to_f(row[h * d + e]) * qscale : to_f(row[koff + h * d + (e - d)]);
  }
  __syncthreads();
  for (int t = 0; t < len; ++t) {
    const int64_t tok = start + t;
    const T* row = qkvg + tok * stride;
    const float* cur = qk + (t & 1) * 2 * d;
    float* nxt = qk + ((t + 1) & 1) * 2 * d;
    // fetch the next token's q | k (held in registers across this token's math)
    float pre[(2 * 4 * RMAX + NT - 1) / NT];
    if (t + 1 < len) {
      const T* nrow = row + stride;
#pragma unroll
      for (int j = 0; j < (2 * 4 * RMAX + NT - 1) / NT; ++j) {
        const int e = threadIdx.x + NT * j;
        pre[j] = e < 2 * d ? (e < d ? to_f(nrow[h * d + e]) * qscale
                                    : to_f(nrow[koff + h * d + (e - d)])) : 0.f;
      }
    }
    const float ig = gates[tok * 2 * H + h], fg = gates[tok * 2 * H + H + h];
    const float v = colok ? to_f(row[voff + h * dv + col]) : 0.f;
    const float mn = fmaxf(fg + m, ig);
    const float fa = expf(fg + m - mn), ia = expf(ig - mn);
    m = mn;
    // normaliser and denominator (every wave, whole n)
    float nq = 0.f;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int r = lane + 64 * u;
      if (r < d) {
        nr[u] = fa * nr[u] + ia * cur[d + r];
        nq += nr[u] * cur[r];
      }
    }
    nq = wave_sum(nq);
    const float den = fmaxf(fabsf(nq), expf(-mn)) + 1e-6f;
    // memory update and this wave's rows of the numerator
    const float iv = ia * v;
    float num = 0.f;
#pragma unroll
    for (int i = 0; i < RMAX; ++i) {
      const int r = wave + NW * i;
      if (r < d) {
        Sr[i] = fa * Sr[i] + cur[d + r] * iv;
        num += Sr[i] * cur[r];
      }
    }
    float* pp = part + (t & 1) * NW * 64;
    pp[wave * 64 + lane] = num;
    if (t + 1 < len) {
#pragma unroll
      for (int j = 0; j < (2 * 4 * RMAX + NT - 1) / NT; ++j) {
        const int e = threadIdx.x + NT * j;
        if (e < 2 * d) nxt[e] = pre[j];
      }
    }
    __syncthreads();
    if (wave == 0 && colok) {
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) tot += pp[w * 64 + lane];
      out[(tok * H + h) * dv + col] = tot / den;
    }
  }
  // the step's final state back to the slot
#pragma unroll
  for (int i = 0; i < RMAX; ++i) {
    const int r = wave + NW * i;
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

template <typename T>
void scan_dispatch(float* out, const T* qkvg, int64_t stride, const float* gates, float* S,
                   float* nst, float* mst, const int* qsl, const int* seq_lens,
                   const int* ctx_lens, const int* slots, int P, int D, int Tp, int H, int d,
                   int dv, int num_slots, hipStream_t s) {
  const dim3 grid(P + D, H, (dv + 63) / 64);
  const size_t lds = (size_t)(4 * d + 2 * NW * 64) * sizeof(float);
#define KGC_SCAN(R)                                                                          \
  mlstm_scan_kernel<T, R><<<grid, NT, lds, s>>>(out, qkvg, stride, gates, S, nst, mst, qsl, \
                                                seq_lens, ctx_lens, slots, P, Tp, H, d, dv, \
                                                num_slots)
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
