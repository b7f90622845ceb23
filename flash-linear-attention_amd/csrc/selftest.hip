// Diagnostics: a tiny GEMM through the same MFMA fragment helpers the kernels
// use, so that operand/accumulator lane ownership can be verified on a device
// against a library matmul.
#include "fla_common.h"
#include "mfma_tiles.h"

namespace {

constexpr int LD = 32 + 8;

// One wave per 32x32 (modes 0, 2) or 16x16 (mode 1) output tile; the wave
// stages a [rows x 32] slab of A and of B in LDS per contraction step.
template <int MODE>
__global__ __launch_bounds__(64) void selftest_kernel(const bf16* __restrict__ A, const bf16* __restrict__ B,
                                                      float* __restrict__ C, int M, int N, int Kd) {
  constexpr int TS = (MODE == 1) ? 16 : 32;
  __shared__ __attribute__((aligned(16))) bf16 sA[32 * LD];
  __shared__ __attribute__((aligned(16))) bf16 sB[32 * LD];
  int lane = threadIdx.x;
  int m0 = blockIdx.x * TS, n0 = blockIdx.y * TS;
  f32x16 acc32 = zero16();
  f32x4 acc16 = zero4();
  for (int k0 = 0; k0 < Kd; k0 += 32) {
    for (int i = lane; i < TS * 32; i += 64) {
      int r = i / 32, c = i % 32;
      sA[r * LD + c] = A[(int64_t)(m0 + r) * Kd + k0 + c];
      sB[r * LD + c] = B[(int64_t)(n0 + r) * Kd + k0 + c];
    }
    __syncthreads();
    if (MODE == 0) {
      for (int s = 0; s < 32; s += 16)
        acc32 = Elem<bf16>::mfma32(lds_frag32<bf16>(sA, LD, 0, s, lane), lds_frag32<bf16>(sB, LD, 0, s, lane), acc32);
    } else if (MODE == 2) {
      for (int s = 0; s < 32; s += 16)
        acc32 = Elem<bf16>::mfma32(lds_frag32_perm<bf16>(sA, LD, 0, s, lane), lds_frag32_perm<bf16>(sB, LD, 0, s, lane),
                                   acc32);
    } else {
      acc16 = Elem<bf16>::mfma16(lds_frag16<bf16>(sA, LD, 0, 0, lane), lds_frag16<bf16>(sB, LD, 0, 0, lane), acc16);
    }
    __syncthreads();
  }
  if (MODE == 1) {
    for (int r = 0; r < 4; ++r) C[(int64_t)(m0 + 4 * (lane >> 4) + r) * N + n0 + (lane & 15)] = acc16[r];
  } else {
    for (int r = 0; r < 16; ++r) C[(int64_t)(m0 + c32_row(r, lane)) * N + n0 + (lane & 31)] = acc32[r];
  }
}

}  // namespace

extern "C" int fla_selftest_mfma(const void* A, const void* B, float* C, int64_t M, int64_t N, int64_t Kd, int mode,
                                 fla_stream_t stream) {
  FLA_REQUIRE(A && B && C, FLA_E_INVALID);
  FLA_REQUIRE(M > 0 && N > 0 && Kd > 0 && M % 32 == 0 && N % 32 == 0 && Kd % 32 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(M <= 4096 && N <= 4096, FLA_E_UNSUPPORTED);
  hipStream_t st = (hipStream_t)stream;
  const bf16* a = (const bf16*)A;
  const bf16* b = (const bf16*)B;
  if (mode == 0) {
    hipLaunchKernelGGL(selftest_kernel<0>, dim3(M / 32, N / 32), dim3(64), 0, st, a, b, C, (int)M, (int)N, (int)Kd);
  } else if (mode == 1) {
    hipLaunchKernelGGL(selftest_kernel<1>, dim3(M / 16, N / 16), dim3(64), 0, st, a, b, C, (int)M, (int)N, (int)Kd);
  } else if (mode == 2) {
    hipLaunchKernelGGL(selftest_kernel<2>, dim3(M / 32, N / 32), dim3(64), 0, st, a, b, C, (int)M, (int)N, (int)Kd);
  } else {
    return FLA_E_INVALID;
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}
