// chunk_local_cumsum: inclusive prefix (or suffix) sums of log-gates along
// time, restarting at every chunk boundary of every sequence.  fp32 output.
//
// HBM-streaming kernel: one lane owns VEC adjacent channels of one chunk and
// walks the chunk's rows with all loads issued up front; a wave therefore
// reads 64*VEC contiguous elements per row.  The reference forms the same
// sums with a [BT,BT] triangular-mask matmul (fla/ops/utils/cumsum.py:97-109);
// a running sum in registers needs no matrix unit and no LDS.
#include <mutex>

#include "fla_common.h"

namespace {

template <typename GT, int VEC>
struct VecLoad;

template <typename GT>
struct VecLoad<GT, 1> {
  static FLA_DEVICE void load(const GT* p, float* out) { out[0] = (float)p[0]; }
};
template <>
struct VecLoad<float, 4> {
  static FLA_DEVICE void load(const float* p, float* out) {
    f32x4 v = *(const f32x4*)p;
    out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
  }
};
template <>
struct VecLoad<bf16, 4> {
  static FLA_DEVICE void load(const bf16* p, float* out) {
    bf16x4 v = *(const bf16x4*)p;
    for (int i = 0; i < 4; ++i) out[i] = (float)v[i];
  }
};
template <>
struct VecLoad<f16, 4> {
  static FLA_DEVICE void load(const f16* p, float* out) {
    f16x4 v = *(const f16x4*)p;
    for (int i = 0; i < 4; ++i) out[i] = (float)v[i];
  }
};

// grid: (NT, ceil(H*S/VEC / 256), B) ; for fixed-length batches NT = ceil(T/BT).
// ROWS = rows handled per unrolled batch (BT is walked in batches of ROWS).
template <typename GT, int VEC, int ROWS>
__global__ __launch_bounds__(256) void cumsum_kernel(const GT* __restrict__ g, float* __restrict__ out,
                                                     int64_t T, int64_t HS, int BT, int reverse,
                                                     const int64_t* __restrict__ offsets,
                                                     const int64_t* __restrict__ indices, int inverse) {
  int64_t col = ((int64_t)blockIdx.y * 256 + threadIdx.x) * VEC;
  if (col >= HS) return;
  int64_t bos, len, ic;
  if (offsets) {
    int64_t n = indices[2 * (int64_t)blockIdx.x];
    ic = indices[2 * (int64_t)blockIdx.x + 1];
    bos = offsets[n];
    len = offsets[n + 1] - bos;
  } else {
    bos = (int64_t)blockIdx.z * T;
    len = T;
    ic = blockIdx.x;
  }
  int64_t t0 = ic * BT;
  int L = (int)((len - t0) < BT ? (len - t0) : BT);
  if (L <= 0) return;
  const GT* src = g + (bos + t0) * HS + col;
  float* dst = out + (bos + t0) * HS + col;
  // inverse: the input holds the sums and the output is the differences of consecutive rows (the
  // first row of the walk keeps its value); `run` then carries the previous row instead of the sum
  float run[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) run[i] = 0.f;
  for (int r0 = 0; r0 < L; r0 += ROWS) {
    float x[ROWS][VEC];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      int row = r0 + r;
      int rr = reverse ? (L - 1 - row) : row;
      if (row < L) {
        VecLoad<GT, VEC>::load(src + (int64_t)rr * HS, x[r]);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) x[r][i] = 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      int row = r0 + r;
      int rr = reverse ? (L - 1 - row) : row;
      float o[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        if (inverse) {
          o[i] = x[r][i] - run[i];
          run[i] = x[r][i];
        } else {
          run[i] += x[r][i];
          o[i] = run[i];
        }
      }
      if (row < L) {
        if (VEC == 4) {
          f32x4 o4 = {o[0], o[VEC > 1 ? 1 : 0], o[VEC > 2 ? 2 : 0], o[VEC > 3 ? 3 : 0]};
          *(f32x4*)(dst + (int64_t)rr * HS) = o4;
        } else {
          dst[(int64_t)rr * HS] = o[0];
        }
      }
    }
  }
}

template <typename GT>
int launch_cumsum(const void* g, float* out, int64_t B, int64_t T, int64_t H, int64_t S, int BT, int reverse,
                  const int64_t* offsets, const int64_t* indices, int64_t NT, hipStream_t stream, int inverse = 0) {
  int64_t HS = H * S;
  bool vec4 = (HS % 4 == 0) && (((uintptr_t)g) % (4 * sizeof(GT)) == 0) && (((uintptr_t)out) % 16 == 0);
  int64_t nt = offsets ? NT : fla_cdiv(T, BT);
  int64_t nb = offsets ? 1 : B;
  if (nt == 0 || nb == 0 || HS == 0) return FLA_OK;
  FLA_REQUIRE(nt <= 0x7fffffffLL && nb <= 65535 && fla_cdiv(HS, 256) <= 65535, FLA_E_UNSUPPORTED);
  if (vec4) {
    dim3 grid((unsigned)nt, (unsigned)fla_cdiv(HS / 4, 256), (unsigned)nb);
    hipLaunchKernelGGL((cumsum_kernel<GT, 4, 16>), grid, dim3(256), 0, stream, (const GT*)g, out, T, HS, BT, reverse,
                       offsets, indices, inverse);
  } else {
    dim3 grid((unsigned)nt, (unsigned)fla_cdiv(HS, 256), (unsigned)nb);
    hipLaunchKernelGGL((cumsum_kernel<GT, 1, 16>), grid, dim3(256), 0, stream, (const GT*)g, out, T, HS, BT, reverse,
                       offsets, indices, inverse);
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

// Second pass of the whole-sequence cumulative sum: out = local + (sum of the totals of the
// chunks before (reverse: after) this one in the same sequence).  `local` holds the chunk-local
// sums of the first pass, so a chunk's total is its last (reverse: first) row.
template <typename OT, int VEC>
__global__ __launch_bounds__(256) void cumsum_carry_kernel(const float* __restrict__ local, OT* __restrict__ out,
                                                           int64_t T, int64_t HS, int BT, int reverse,
                                                           const int64_t* __restrict__ offsets,
                                                           const int64_t* __restrict__ indices) {
  int64_t col = ((int64_t)blockIdx.y * 256 + threadIdx.x) * VEC;
  if (col >= HS) return;
  int64_t bos, len, ic;
  if (offsets) {
    int64_t n = indices[2 * (int64_t)blockIdx.x];
    ic = indices[2 * (int64_t)blockIdx.x + 1];
    bos = offsets[n];
    len = offsets[n + 1] - bos;
  } else {
    bos = (int64_t)blockIdx.z * T;
    len = T;
    ic = blockIdx.x;
  }
  const int64_t t0 = ic * BT;
  const int L = (int)((len - t0) < BT ? (len - t0) : BT);
  if (L <= 0) return;
  const int64_t nchunks = (len + BT - 1) / BT;
  float carry[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) carry[i] = 0.f;
  const int64_t c_lo = reverse ? ic + 1 : 0, c_hi = reverse ? nchunks : ic;
  for (int64_t c = c_lo; c < c_hi; ++c) {
    int64_t row = c * BT;
    if (!reverse) {
      int64_t rem = len - row;
      row += (rem < BT ? rem : BT) - 1;
    }
    float x[VEC];
    VecLoad<float, VEC>::load(local + (bos + row) * HS + col, x);
#pragma unroll
    for (int i = 0; i < VEC; ++i) carry[i] += x[i];
  }
  for (int r = 0; r < L; ++r) {
    float x[VEC];
    VecLoad<float, VEC>::load(local + (bos + t0 + r) * HS + col, x);
#pragma unroll
    for (int i = 0; i < VEC; ++i) out[(bos + t0 + r) * HS + col + i] = (OT)(x[i] + carry[i]);
  }
}

template <typename OT>
int launch_carry(const float* local, void* out, int64_t B, int64_t T, int64_t H, int64_t S, int BT, int reverse,
                 const int64_t* offsets, const int64_t* indices, int64_t NT, hipStream_t stream) {
  int64_t HS = H * S;
  bool vec4 = (HS % 4 == 0) && (((uintptr_t)local) % 16 == 0);
  int64_t nt = offsets ? NT : fla_cdiv(T, BT);
  int64_t nb = offsets ? 1 : B;
  if (nt == 0 || nb == 0 || HS == 0) return FLA_OK;
  FLA_REQUIRE(nt <= 0x7fffffffLL && nb <= 65535 && fla_cdiv(HS, 256) <= 65535, FLA_E_UNSUPPORTED);
  if (vec4) {
    dim3 grid((unsigned)nt, (unsigned)fla_cdiv(HS / 4, 256), (unsigned)nb);
    hipLaunchKernelGGL((cumsum_carry_kernel<OT, 4>), grid, dim3(256), 0, stream, local, (OT*)out, T, HS, BT, reverse,
                       offsets, indices);
  } else {
    dim3 grid((unsigned)nt, (unsigned)fla_cdiv(HS, 256), (unsigned)nb);
    hipLaunchKernelGGL((cumsum_carry_kernel<OT, 1>), grid, dim3(256), 0, stream, local, (OT*)out, T, HS, BT, reverse,
                       offsets, indices);
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

extern "C" int fla_chunk_local_cumsum(const void* g, float* out, int g_dtype, int64_t B, int64_t T, int64_t H,
                                      int64_t S, int64_t chunk_size, int reverse, const int64_t* offsets,
                                      const int64_t* indices, int64_t NT, fla_stream_t stream) {
  FLA_REQUIRE(g && out, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H >= 0 && S >= 1 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(chunk_size > 0 && (chunk_size & (chunk_size - 1)) == 0, FLA_E_INVALID);
  FLA_REQUIRE(chunk_size <= (1 << 20), FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(indices != nullptr && B == 1, FLA_E_INVALID);
  hipStream_t st = (hipStream_t)stream;
  switch (g_dtype) {
    case FLA_F32: return launch_cumsum<float>(g, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    case FLA_BF16: return launch_cumsum<bf16>(g, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    case FLA_F16: return launch_cumsum<f16>(g, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    default: return FLA_E_UNSUPPORTED;
  }
}

extern "C" int fla_chunk_local_cumsum_inverse(const float* g_cumsum, float* out, int64_t B, int64_t T, int64_t H,
                                              int64_t S, int64_t chunk_size, int reverse, const int64_t* offsets,
                                              const int64_t* indices, int64_t NT, fla_stream_t stream) {
  FLA_REQUIRE(g_cumsum && out, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H >= 0 && S >= 1 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(chunk_size > 0 && (chunk_size & (chunk_size - 1)) == 0, FLA_E_INVALID);
  FLA_REQUIRE(chunk_size <= (1 << 20), FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(indices != nullptr && B == 1, FLA_E_INVALID);
  return launch_cumsum<float>(g_cumsum, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT,
                              (hipStream_t)stream, 1);
}

extern "C" int fla_chunk_global_cumsum(const void* s, float* ws_local, void* out, int s_dtype, int out_dtype, int64_t B,
                                       int64_t T, int64_t H, int64_t S, int64_t chunk_size, int reverse,
                                       const int64_t* offsets, const int64_t* indices, int64_t NT,
                                       fla_stream_t stream) {
  FLA_REQUIRE(s && ws_local && out, FLA_E_INVALID);
  int rc = fla_chunk_local_cumsum(s, ws_local, s_dtype, B, T, H, S, chunk_size, reverse, offsets, indices, NT, stream);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case FLA_F32: return launch_carry<float>(ws_local, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    case FLA_BF16: return launch_carry<bf16>(ws_local, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    case FLA_F16: return launch_carry<f16>(ws_local, out, B, T, H, S, (int)chunk_size, reverse, offsets, indices, NT, st);
    default: return FLA_E_UNSUPPORTED;
  }
}

// ---------------------------------------------------------------------------
// fla_chunk_global_cumsum for callers that cannot allocate (code under HIP graph capture, serving
// loops, harnesses that forbid hipMalloc): the chunk-local sums of the first pass live in a
// file-scope device array instead of a caller workspace.  Each GPU holds its own copy of the array
// at its own address, so the address is looked up once per device (hipGetSymbolAddress with that
// device current) and only that pointer is handed to the kernels; the array's name itself is a
// host-side stand-in and never a kernel argument.  Every element the second pass reads has been
// written by the first pass of the same call, so nothing needs clearing between calls.  All calls
// on one GPU share the array: calls that overlap on one GPU (different streams) race.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float scratch[FLA_STATIC_SCRATCH_FLOATS];

namespace {
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];   // per device; written once under g_scratch_mu
std::mutex g_scratch_mu;

int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return FLA_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    float* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return FLA_E_INVALID;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return FLA_OK;
}
}  // namespace

extern "C" int fla_chunk_global_cumsum_static(const void* s, void* out, int s_dtype, int out_dtype, int64_t B, int64_t T,
                                              int64_t H, int64_t S, int64_t chunk_size, int reverse,
                                              const int64_t* offsets, const int64_t* indices, int64_t NT,
                                              fla_stream_t stream) {
  FLA_REQUIRE(s && out, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H >= 0 && S >= 1, FLA_E_INVALID);
  // sizes first: an input that does not fit is refused before anything touches the device
  const int64_t cap = FLA_STATIC_SCRATCH_FLOATS;
  if (B > 0 && T > 0 && H > 0) {
    FLA_REQUIRE(B <= cap && T <= cap / B && H <= cap / (B * T) && S <= cap / (B * T * H), FLA_E_SCRATCH);
  }
  float* ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc) return rc;
  return fla_chunk_global_cumsum(s, ws, out, s_dtype, out_dtype, B, T, H, S, chunk_size, reverse, offsets, indices, NT,
                                 stream);
}
