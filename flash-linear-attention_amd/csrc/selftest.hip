// Diagnostics: a tiny GEMM through the same MFMA fragment helpers the kernels
// use, so that operand/accumulator lane ownership can be verified on a device
// against a library matmul; and a probe of the rate at which a CU is fed when
// it streams rows the way the chunk scans do.
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

// One workgroup per CU (the LDS array sees to that) reads every row of one (sequence, head) of NT tensors
// [B, T, H, 128] (16-bit elements: 256-byte row pieces at a pitch of 256 H bytes), 64 rows at a time, each register
// refilled as soon as it is consumed - the access pattern of the staging waves of the chunk scans without their
// arithmetic.  `share` workgroups read the same (sequence, head), as the value slabs of a head do.  The XOR of all
// the words a workgroup read goes to sink[workgroup], which makes the result checkable.
template <int NT>
__global__ __launch_bounds__(256) void stream_tiles_kernel(const char* __restrict__ x, int64_t tensor_bytes,
                                                           uint32_t* __restrict__ sink, int T, int H, int share) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr int NP = 4 * NT;   // 16-byte pieces per thread and 64-row chunk
  __shared__ char pad[96 * 1024];
  pad[threadIdx.x * 64] = (char)T;
  const int tid = threadIdx.x;
  const int pair = blockIdx.x / share;
  const int b = pair / H, hh = pair % H;
  const uint32_t pitch = (uint32_t)H * 256u;
  uint32_t off[NP];
  const char* base[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid + 256 * i;   // piece index: tensor, row, 16-byte column
    off[i] = (uint32_t)((e % 1024) / 16) * pitch + (uint32_t)(e % 16) * 16u;
    base[i] = x + (int64_t)(e / 1024) * tensor_bytes + ((int64_t)b * T * H + hh) * 256;
  }
  const int nchunks = T / 64;
  const int64_t cstride = (int64_t)64 * pitch;
  u4 R[NP];
  u4 acc = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < NP; ++i) R[i] = *(const u4*)(base[i] + off[i]);
  for (int c = 1; c < nchunks; ++c) {
    const int64_t co = (int64_t)c * cstride;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      acc ^= R[i];
      R[i] = *(const u4*)(base[i] + co + off[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < NP; ++i) acc ^= R[i];
  uint32_t w = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  // wave, then workgroup
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) w ^= (uint32_t)__shfl_xor((int)w, m);
  uint32_t* red = (uint32_t*)(pad + 64 * 1024);
  __syncthreads();
  if ((tid & 63) == 0) red[tid >> 6] = w;
  __syncthreads();
  if (tid == 0) sink[blockIdx.x] = red[0] ^ red[1] ^ red[2] ^ red[3];
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

extern "C" int fla_selftest_stream_tiles(const void* x, int64_t tensor_bytes, int n_tensors, uint32_t* sink, int64_t B,
                                         int64_t T, int64_t H, int share, fla_stream_t stream) {
  FLA_REQUIRE(x && sink, FLA_E_INVALID);
  FLA_REQUIRE(B > 0 && H > 0 && T >= 64 && T % 64 == 0 && share >= 1 && n_tensors >= 1 && n_tensors <= 4,
              FLA_E_UNSUPPORTED);
  FLA_REQUIRE(tensor_bytes >= B * T * H * 256 && tensor_bytes % 16 == 0 && (uintptr_t)x % 16 == 0, FLA_E_INVALID);
  FLA_REQUIRE(B * H * share <= 65536 && H * 256 * 64 < (1LL << 31) / 64, FLA_E_UNSUPPORTED);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)(B * H * share));
  const char* xc = (const char*)x;
  switch (n_tensors) {
    case 1: hipLaunchKernelGGL(stream_tiles_kernel<1>, grid, dim3(256), 0, st, xc, tensor_bytes, sink, (int)T, (int)H, share); break;
    case 2: hipLaunchKernelGGL(stream_tiles_kernel<2>, grid, dim3(256), 0, st, xc, tensor_bytes, sink, (int)T, (int)H, share); break;
    case 3: hipLaunchKernelGGL(stream_tiles_kernel<3>, grid, dim3(256), 0, st, xc, tensor_bytes, sink, (int)T, (int)H, share); break;
    default: hipLaunchKernelGGL(stream_tiles_kernel<4>, grid, dim3(256), 0, st, xc, tensor_bytes, sink, (int)T, (int)H, share); break;
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}
