// K7 SiLU-and-mul: out[t, i] = silu(x[t, i]) * x[t, I + i] over the fused gate_up
// projection output.  16-byte vector loads/stores (8 halves per lane), one vector
// per thread on a 2-D grid (memory-bound; no index division).
#include "common.h"
#include "launch.h"

namespace kgc {

// grid (ceil(I/8/256), rows): one 16-byte vector per thread, no index division
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out,
                                                       const T* __restrict__ x, int I) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c * 8 >= I) return;
  const int64_t r = blockIdx.y;
  const T* xr = x + r * 2 * I;
  Pack8<T> g, u, o;
  g.u = *reinterpret_cast<const u32x4*>(xr + c * 8);
  u.u = *reinterpret_cast<const u32x4*>(xr + I + c * 8);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float gf = to_f(g.h[j]);
    o.h[j] = from_f<T>(gf / (1.f + __expf(-gf)) * to_f(u.h[j]));
  }
  *reinterpret_cast<u32x4*>(out + r * I + c * 8) = o.u;
}

// any element type and any I (fp32 activations, intermediate sizes that are no multiple of 8)
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_any_kernel(T* __restrict__ out,
                                                           const T* __restrict__ x, int I) {
  const int64_t r = blockIdx.y;
  const T* xr = x + r * 2 * I;
  for (int c = blockIdx.x * 256 + threadIdx.x; c < I; c += gridDim.x * 256) {
    const float gf = to_f(xr[c]);
    out[r * I + c] = from_f<T>(gf / (1.f + expf(-gf)) * to_f(xr[I + c]));
  }
}

void launch_silu_mul(int dtype, void* out, const void* x, int64_t rows, int I, hipStream_t s) {
  if (dtype == DT_F32 || (I & 7)) {
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
      const int64_t n = std::min<int64_t>(rows - r0, 65535);
      const dim3 grid(std::min((I + 255) / 256, 64), (unsigned)n);
      if (dtype == DT_F32)
        silu_mul_any_kernel<float><<<grid, 256, 0, s>>>((float*)out + r0 * I,
                                                        (const float*)x + r0 * 2 * I, I);
      else if (dtype == DT_BF16)
        silu_mul_any_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out + r0 * I,
                                                       (const bf16*)x + r0 * 2 * I, I);
      else
        silu_mul_any_kernel<f16><<<grid, 256, 0, s>>>((f16*)out + r0 * I,
                                                      (const f16*)x + r0 * 2 * I, I);
    }
    return;
  }
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {   // gridDim.y <= 65535
    const int64_t n = std::min<int64_t>(rows - r0, 65535);
    const dim3 grid(((I >> 3) + 255) / 256, (unsigned)n);
    if (dtype == DT_BF16)
      silu_mul_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out + r0 * I, (const bf16*)x + r0 * 2 * I, I);
    else
      silu_mul_kernel<f16><<<grid, 256, 0, s>>>((f16*)out + r0 * I, (const f16*)x + r0 * 2 * I, I);
  }
}

}  // namespace kgc
