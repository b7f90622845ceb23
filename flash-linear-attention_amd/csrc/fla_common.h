// Shared device/host helpers for the gfx950 (CDNA4, wave64) kernels.
//
// Conventions used by every kernel in this directory
//   * tensors are seq-first: q,k [B,T,H,K], v,o [B,T,H,V], per-head scalars [B,T,H];
//     a packed variable-length batch is [1,T_total,H,*] plus int64 offsets[N+1].
//   * recurrent state is fp32 [N,H,K,V].
//   * entry points return 0, a positive hipError_t, or a negative FLA_E_* code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fla_hip.h"

typedef __bf16 bf16;
typedef _Float16 f16;
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define FLA_DEVICE __device__ __forceinline__

#define FLA_CHECK_LAUNCH()                         \
  do {                                             \
    hipError_t e__ = hipGetLastError();            \
    if (e__ != hipSuccess) return (int)e__;        \
  } while (0)

#define FLA_REQUIRE(cond, code) \
  do {                          \
    if (!(cond)) return (code); \
  } while (0)

static inline int64_t fla_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------
// element type traits: 16-bit storage types with their 4/8-wide vectors and
// the matching gfx950 MFMA instructions (fp32 accumulate).
// ---------------------------------------------------------------------------
template <typename T>
struct Elem;

template <>
struct Elem<bf16> {
  typedef bf16x4 v4;
  typedef bf16x8 v8;
  static FLA_DEVICE f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static FLA_DEVICE f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // c + sum of the eight products, on the packed dot-product instruction (no unpacked temporaries)
  static FLA_DEVICE float dot8(v8 a, v8 b, float c) {
    typedef bf16 v2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c = __builtin_amdgcn_fdot2_f32_bf16(v2{a[2 * i], a[2 * i + 1]}, v2{b[2 * i], b[2 * i + 1]}, c, false);
    return c;
  }
};

template <>
struct Elem<f16> {
  typedef f16x4 v4;
  typedef f16x8 v8;
  static FLA_DEVICE f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static FLA_DEVICE f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static FLA_DEVICE float dot8(v8 a, v8 b, float c) {
    typedef f16 v2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c = __builtin_amdgcn_fdot2(v2{a[2 * i], a[2 * i + 1]}, v2{b[2 * i], b[2 * i + 1]}, c, false);
    return c;
  }
};

// MFMA operand/accumulator ownership on wave64 (l = lane id):
//   32x32x16: A lane l holds A[row = l%32][k = 8*(l/32) .. +7]
//             B lane l holds B[k = 8*(l/32) .. +7][col = l%32]
//             C reg r of lane l is C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32]
//   16x16x32: A lane l holds A[row = l%16][k = 8*(l/16) .. +7]
//             B lane l holds B[k = 8*(l/16) .. +7][col = l%16]
//             C reg r of lane l is C[row = 4*(l/16) + r][col = l%16]
// The contraction index may be permuted freely as long as A and B agree.
FLA_DEVICE int c32_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <typename T>
FLA_DEVICE float to_f32(T x) { return (float)x; }

template <typename T>
FLA_DEVICE T from_f32(float x) { return (T)x; }

// exp(x) for x <= 0, 0 otherwise: decay factors must never amplify
// (fla/ops/utils/exp.py:9-10).
FLA_DEVICE float safe_exp(float x) { return x <= 0.f ? __expf(x) : 0.f; }

// DPP row operations (a DPP row is 16 consecutive lanes); lanes without a source read 0.
template <int CTRL>
FLA_DEVICE float dpp_f32(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
// inclusive prefix / suffix sums across the 16 lanes of a DPP row (VALU only, no LDS traffic)
FLA_DEVICE float row_prefix16(float x) {
  x += dpp_f32<0x111>(x);  // row_shr:1
  x += dpp_f32<0x112>(x);  // row_shr:2
  x += dpp_f32<0x114>(x);  // row_shr:4
  x += dpp_f32<0x118>(x);  // row_shr:8
  return x;
}
FLA_DEVICE float row_suffix16(float x) {
  x += dpp_f32<0x101>(x);  // row_shl:1
  x += dpp_f32<0x102>(x);  // row_shl:2
  x += dpp_f32<0x104>(x);  // row_shl:4
  x += dpp_f32<0x108>(x);  // row_shl:8
  return x;
}

// Sum over an aligned group of N (8 or 16) consecutive lanes, result in every lane of the group: two
// exchanges inside the quads, then the mirror images of the half row and the row (VALU only).
template <int N>
FLA_DEVICE float group_allsum(float x) {
  static_assert(N == 8 || N == 16, "lanes per group");
  x += dpp_f32<0xB1>(x);    // quad_perm [1,0,3,2]
  x += dpp_f32<0x4E>(x);    // quad_perm [2,3,0,1]
  x += dpp_f32<0x141>(x);   // row_half_mirror
  if (N == 16) x += dpp_f32<0x140>(x);   // row_mirror
  return x;
}

// Sum over the 32 lanes of a half wave (lanes 0-31 or 32-63); the result is valid in the second DPP row of the half
// (lanes 16-31 and 48-63): group sums of 16, then row_bcast:15 hands the first row's total to the second.
FLA_DEVICE float half_wave_sum_hi(float x) {
  x = group_allsum<16>(x);
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x142, 0xA, 0xF, true));   // row_bcast:15 into rows 1, 3
  return x;
}
// Sum over the 64 lanes of a wave, valid in the last DPP row (lanes 48-63): as above, then row_bcast:31 hands the
// first half's total to the last row.
FLA_DEVICE float wave_sum_lane63(float x) {
  x = half_wave_sum_hi(x);
  x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x143, 0xC, 0xF, true));   // row_bcast:31 into rows 2, 3
  return x;
}

// A row of 8 * N elements is held by N adjacent lanes, 8 elements each: x / sqrt(sum x^2 + eps) of this lane's
// piece, rounded to T (fla/modules/l2norm.py:18-40: eps inside the square root).
template <typename T, int N>
FLA_DEVICE typename Elem<T>::v8 l2norm_piece(typename Elem<T>::v8 x, float eps) {
  float f[8], ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    f[i] = (float)x[i];
    ss = fmaf(f[i], f[i], ss);
  }
  const float rstd = __builtin_amdgcn_rsqf(group_allsum<N>(ss) + eps);
  typename Elem<T>::v8 y;
#pragma unroll
  for (int i = 0; i < 8; ++i) y[i] = (T)(f[i] * rstd);
  return y;
}

// 1 / sqrt(sum x^2 + eps) of the row this lane's 8-element piece belongs to (N adjacent lanes hold the row): the
// squares on the packed dot-product instruction, the sum over the lanes as in group_allsum.
template <typename T, int N>
FLA_DEVICE float l2norm_rstd(typename Elem<T>::v8 x, float eps) {
  return __builtin_amdgcn_rsqf(group_allsum<N>(Elem<T>::dot8(x, x, 0.f)) + eps);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() carries a fence over
// global memory as well: a wave with global stores in flight then drains its whole vector
// memory queue (loads included) at every barrier, which exposes the full memory latency of
// register prefetches once per chunk.  Use only where the waves exchange data through LDS.
FLA_DEVICE void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

struct SeqSpan {
  int64_t bos;  // first token row of the sequence in the packed [B*T] row space
  int64_t len;  // number of tokens
};

// Rows are addressed in the flattened [B*T] space; for a packed batch B == 1.
FLA_DEVICE SeqSpan seq_span(const int64_t* offsets, int n, int64_t T) {
  SeqSpan s;
  if (offsets) {
    s.bos = offsets[n];
    s.len = offsets[n + 1] - s.bos;
  } else {
    s.bos = (int64_t)n * T;
    s.len = T;
  }
  return s;
}
