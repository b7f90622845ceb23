// LDS -> MFMA operand fragment loaders.  Tiles are stored with the contraction
// index contiguous ("row-major over k") and a row pitch `ld` that is a
// multiple of 8 elements, so every fragment is one 16-byte LDS read.
#pragma once
#include "fla_common.h"

// 32x32x16 operand: 32 rows starting at row0, contraction slice [k0, k0+16).
template <typename T>
FLA_DEVICE typename Elem<T>::v8 lds_frag32(const T* tile, int ld, int row0, int k0, int lane) {
  return *(const typename Elem<T>::v8*)(tile + (row0 + (lane & 31)) * ld + k0 + 8 * (lane >> 5));
}

// Time-contiguous 16-bit tiles ([row][t], pitch 144 bytes) that are written by lanes owning four
// adjacent rows each see a lane stride of 64 bytes modulo 256, i.e. a quarter of the banks.
// XOR-ing row bits 4-5 into the index of the 16-byte slot along t spreads such writes over all
// banks; a fragment read stays conflict-free.  Writer and reader both map t through swz16.
FLA_DEVICE int swz16(int row, int t) { return t ^ (((row >> 4) & 3) << 3); }

template <typename T>
FLA_DEVICE typename Elem<T>::v8 lds_frag32_swz(const T* tile, int ld, int row0, int k0, int lane) {
  const int row = row0 + (lane & 31);
  return *(const typename Elem<T>::v8*)(tile + row * ld + swz16(row, k0 + 8 * (lane >> 5)));
}

// Same slice with the contraction index permuted inside the 16-slice: slot
// (g = lane/32, e) holds k0 + 8*(e/4) + 4*g + e%4.  This is the order in which
// a 32x32 accumulator's registers enumerate rows, so an accumulator converted
// to 16-bit can be fed back as the other operand without a shuffle.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 lds_frag32_perm(const T* tile, int ld, int row0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  const T* p = tile + (row0 + (lane & 31)) * ld + k0 + 4 * (lane >> 5);
  v4 lo = *(const v4*)p;
  v4 hi = *(const v4*)(p + 8);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// 16x16x32 operand: 16 rows starting at row0, contraction slice [k0, k0+32).
template <typename T>
FLA_DEVICE typename Elem<T>::v8 lds_frag16(const T* tile, int ld, int row0, int k0, int lane) {
  return *(const typename Elem<T>::v8*)(tile + (row0 + (lane & 15)) * ld + k0 + 8 * (lane >> 4));
}

// 16x16x32 operand with the contraction index permuted inside the 32-slice: slot
// (g = lane/16, e) holds k0 + 16*(e/4) + 4*g + e%4.  This is the order in which two
// stacked 16x16 accumulators (rows k0.. and k0+16..) enumerate their rows, so a pair
// of accumulators converted to 16-bit is the other operand without a shuffle.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 lds_frag16_perm(const T* tile, int ld, int row0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  const T* p = tile + (row0 + (lane & 15)) * ld + k0 + 4 * (lane >> 4);
  v4 lo = *(const v4*)p;
  v4 hi = *(const v4*)(p + 16);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

FLA_DEVICE f32x4 zero4();

// One 16x16 fp32 tile C = sign * A B with A [16 x nk] and B [nk x 16] in LDS
// (fp32, nk a multiple of 4), on the fp32 matrix instruction 16x16x4:
//   A lane l holds A[l%16][l/16], B lane l holds B[l/16][l%16],
//   C reg r of lane l is C[4*(l/16) + r][l%16].
FLA_DEVICE void lds_mm16_f32(const float* A, int lda, const float* B, int ldb, float* C, int ldc, int nk, float sign,
                             int lane) {
  const int r = lane & 15, q = lane >> 4;
  f32x4 acc = zero4();
  for (int k0 = 0; k0 < nk; k0 += 4)
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A[r * lda + k0 + q], B[(k0 + q) * ldb + r], acc, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) C[(4 * q + i) * ldc + r] = sign * acc[i];
}

FLA_DEVICE f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}
FLA_DEVICE f32x4 zero4() {
  f32x4 z = {0.f, 0.f, 0.f, 0.f};
  return z;
}

// Operands whose contraction index is the tile's ROW (tile[kk][m], pitch ld) come out of LDS through the
// transposing load ds_read_b64_tr_b16: it hands lane j of a 16-lane group element j of each of the four rows whose
// 8-byte pieces the group's lanes 4i .. 4i+3 address.
// 32x32x16 operand: 32 operand rows m0 .. m0+31 (contiguous in LDS), contraction slice [k0, k0+16) (tile rows).
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag32_tr(const T* tile, int ld, int m0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef short s4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s4 lds_s4;
  const int s = lane & 15, g = lane >> 4;
  const T* p0 = tile + (k0 + 8 * (g >> 1) + (s >> 2)) * ld + m0 + 16 * (g & 1) + 4 * (s & 3);
  s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)p0);
  s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p0 + 4 * ld));
  return __builtin_shufflevector(__builtin_bit_cast(v4, lo), __builtin_bit_cast(v4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
}

// 16x16x32 operand: 16 operand rows k0 .. k0+15, contraction slice [t0, t0+32) in accumulator-row order (slot
// (g = lane/16, e) holds t0 + 16*(e/4) + 4*g + e%4, as frag16_t of chunk_common.h delivers it from a transposed copy).
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag16_tr(const T* tile, int ld, int k0, int t0, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef short s4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s4 lds_s4;
  const int j = lane & 15, g = lane >> 4;
  const T* p0 = tile + (t0 + 4 * g + (j >> 2)) * ld + k0 + 4 * (j & 3);
  s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)p0);
  s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(p0 + 16 * ld));
  return __builtin_shufflevector(__builtin_bit_cast(v4, lo), __builtin_bit_cast(v4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
}
