// Optional prologue of the fused MoE layer: RMSNorm of the token rows,
//   xn[t, k] = (x[t, k] * scale_t) * gamma[k],  scale_t = float(1 / sqrt(mean_k x[t,k]^2 + eps)),
// into the launcher's workspace, where the router and the gate/up projection then read
// their tokens. The reference's layer has no such step (its caller, vLLM's decoder layer,
// normalises before it calls the block; test/singleGPU/python/flashMoeOp.py:23-38 receives
// hidden states that are already normalised); it is here so that a caller can hand over
// the un-normalised residual stream and get `x + moe(rmsnorm(x))` back from one call.
//
// Arithmetic, chosen so that CPU and GPU agree bit for bit: the sum of squares in double
// (for bf16 rows it is exact whatever the order: 16-bit squares, 2^11 of them, exponents
// within 2^26 of each other in any sane activation row), 1 / sqrt in double, one rounding
// to float, then two float multiplications in the order written above, and for bf16
// layers one rounding to bf16 (nearest even).
#include "moe_device.h"

namespace fmoe {

template <typename DT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const void* x_, const void* gamma_, void* xn_, int T, int H,
                                                      double eps) {
  typedef typename DT::elem elem;
  constexpr int EPV = DT::EPV;
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);  // one wave per token
  if (t >= T) return;
  const elem* x = reinterpret_cast<const elem*>(x_) + static_cast<size_t>(t) * H;
  const elem* gamma = reinterpret_cast<const elem*>(gamma_);
  elem* xn = reinterpret_cast<elem*>(xn_) + static_cast<size_t>(t) * H;
  const int nvec = H / EPV;
  double ss = 0.0;
  for (int v = lane; v < nvec; v += 64) {
    float f[EPV];
    unpack<DT>(ld16(x + v * EPV), f);
#pragma unroll
    for (int i = 0; i < EPV; ++i) ss = fma(static_cast<double>(f[i]), static_cast<double>(f[i]), ss);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  const float scale = static_cast<float>(1.0 / sqrt(ss / static_cast<double>(H) + eps));
  for (int v = lane; v < nvec; v += 64) {
    float f[EPV], g[EPV];
    unpack<DT>(ld16(x + v * EPV), f);
    unpack<DT>(ld16(gamma + v * EPV), g);
#pragma unroll
    for (int i = 0; i < EPV; ++i) f[i] = __fmul_rn(__fmul_rn(f[i], scale), g[i]);
    if constexpr (EPV == 8) {
      st16(xn + v * EPV, u32x4{f2bf(f[0]) | (f2bf(f[1]) << 16), f2bf(f[2]) | (f2bf(f[3]) << 16),
                               f2bf(f[4]) | (f2bf(f[5]) << 16), f2bf(f[6]) | (f2bf(f[7]) << 16)});
    } else {
      st16(xn + v * EPV, u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                               __float_as_uint(f[3])});
    }
  }
}

hipError_t launch_rmsnorm(const void* x, const void* gamma, void* xn, int dtype, int T, int H, double eps,
                          hipStream_t stream) {
  const dim3 grid((T + 3) / 4), block(256);
  if (dtype == DT_BF16) {
    hipLaunchKernelGGL(rmsnorm_kernel<BF16>, grid, block, 0, stream, x, gamma, xn, T, H, eps);
  } else {
    hipLaunchKernelGGL(rmsnorm_kernel<F32>, grid, block, 0, stream, x, gamma, xn, T, H, eps);
  }
  return hipGetLastError();
}

}  // namespace fmoe
