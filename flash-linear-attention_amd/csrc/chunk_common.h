// Helpers shared by the chunk kernels: chunk geometry, vector loads with
// conversion to fp32, the XCD-aware workgroup renumbering.
#pragma once
#include <mutex>
#include <unordered_map>
#include "fla_common.h"
#include "mfma_tiles.h"

namespace {

constexpr int BT = 64;        // chunk length
constexpr int LDT = BT + 8;   // row pitch of time-contiguous 16-bit LDS tiles
constexpr int LDM = BT + 4;   // row pitch of fp32 64-column LDS tiles

// A word of zeros in device memory: where the gate loads of an operator without gates point, so
// that the loaded value needs no select (a select right behind a load makes the wave wait for it).
__device__ float kZeroWord = 0.f;  // never written; not const, so that it lives in the global address space like the tensors

template <typename X>
struct Load;
template <>
struct Load<float> {
  static FLA_DEVICE void x4(const float* p, float* o) {
    f32x4 v = *(const f32x4*)p;
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
  }
};
template <>
struct Load<bf16> {
  static FLA_DEVICE void x4(const bf16* p, float* o) {
    bf16x4 v = *(const bf16x4*)p;
    for (int i = 0; i < 4; ++i) o[i] = (float)v[i];
  }
};
template <>
struct Load<f16> {
  static FLA_DEVICE void x4(const f16* p, float* o) {
    f16x4 v = *(const f16x4*)p;
    for (int i = 0; i < 4; ++i) o[i] = (float)v[i];
  }
};

// Workgroups of one launch are dealt round-robin to the 8 XCDs by linear id.
// Renumber so that consecutive logical ids share an XCD (and its L2).
FLA_DEVICE int64_t xcd_remap(int64_t id, int64_t total) {
  if (total % 8 != 0) return id;
  return (id % 8) * (total / 8) + id / 8;
}

// Work items of the serial scan kernels: one per (sequence, head, value-column slab).
// Workgroups are dispatched in blockIdx order and dealt round-robin to the 8 XCDs; the slabs
// of one (sequence, head) are placed on the same XCD (they read the same q/k/gate rows, which
// then hit in that XCD's L2), and (sequence, head) items are taken in dispatch order, so that
// with `seq_order` (sequence ids, longest first) the longest sequences start first.  A launch that fits
// the chip in one wave of workgroups (at most one per CU, all start together) instead gives each XCD a
// contiguous run of items, i.e. whole sequences where the batch allows: an XCD then walks an eighth of the
// pages instead of all of them (189 against 191 us on 8 sequences x 16 heads x 4096 tokens).
constexpr int64_t kNumCUs = 256;
struct ScanItem {
  int slab;       // value-column slab
  int64_t item;   // (position in seq_order) * H + head
};
FLA_DEVICE ScanItem scan_item(int nslab) {
  const int64_t p = blockIdx.x, tot = gridDim.x;
  ScanItem s;
  if (tot % (8 * nslab) == 0) {
    s.slab = (int)((p / 8) % nslab);
    if (tot <= kNumCUs) s.item = (p % 8) * (tot / (8 * nslab)) + p / (8 * nslab);
    else s.item = (p / (8 * nslab)) * 8 + p % 8;
  } else {
    s.slab = (int)(p % nslab);
    s.item = p / nslab;
  }
  return s;
}

struct ChunkLoc {
  int64_t row0;   // first token row of the chunk in the flattened [B*T] space
  int L;          // valid rows
  int64_t cglob;  // global chunk index (addresses per-chunk states)
};

// Chunk-parallel kernels run on a grid (chunks, H[, slices]); (batch, chunk) for equal lengths,
// rows of `indices` otherwise.  Workgroups are dispatched x-fastest, so the linear id is split
// head-fastest: workgroups that run together take different heads of the same chunks, whose rows
// are adjacent in memory, and the traffic spreads evenly over the memory channels (a
// chunk-fastest order makes concurrent workgroups hit the same address bits 8-11).
FLA_DEVICE ChunkLoc locate_chunk_at(int64_t lin, const int64_t* offsets, const int64_t* indices, int64_t T, int ntfix,
                                    int H, int* head) {
  const int64_t cidx = lin / H;
  *head = (int)(lin % H);
  ChunkLoc c;
  int64_t bos, len, ic;
  if (offsets) {
    int64_t n = indices[2 * cidx];
    ic = indices[2 * cidx + 1];
    bos = offsets[n];
    len = offsets[n + 1] - bos;
  } else {
    bos = (cidx / ntfix) * T;
    ic = cidx % ntfix;
    len = T;
  }
  c.row0 = bos + ic * BT;
  int64_t rem = len - ic * BT;
  c.L = (int)(rem < BT ? rem : BT);
  c.cglob = cidx;
  return c;
}
// The same for kernels that walk many items per workgroup: the item number fits 32 bits (launchers check it),
// and a 32-bit division is a dozen instructions where the 64-bit one is several hundred.
FLA_DEVICE ChunkLoc locate_chunk_at32(uint32_t lin, const int64_t* offsets, const int64_t* indices, int64_t T, int ntfix,
                                      int H, int* head) {
  const uint32_t cidx = lin / (uint32_t)H;
  *head = (int)(lin - cidx * (uint32_t)H);
  ChunkLoc c;
  int64_t bos, len;
  uint32_t ic;
  if (offsets) {
    const int64_t n = indices[2 * (int64_t)cidx];
    ic = (uint32_t)indices[2 * (int64_t)cidx + 1];
    bos = offsets[n];
    len = offsets[n + 1] - bos;
  } else {
    const uint32_t b = cidx / (uint32_t)ntfix;
    ic = cidx - b * (uint32_t)ntfix;
    bos = (int64_t)b * T;
    len = T;
  }
  c.row0 = bos + (int64_t)ic * BT;
  const int64_t rem = len - (int64_t)ic * BT;
  c.L = (int)(rem < BT ? rem : BT);
  c.cglob = cidx;
  return c;
}
FLA_DEVICE ChunkLoc locate_chunk(const int64_t* offsets, const int64_t* indices, int64_t T, int ntfix, int H,
                                 int* head) {
  return locate_chunk_at((int64_t)blockIdx.y * gridDim.x + blockIdx.x, offsets, indices, T, ntfix, H, head);
}

inline int chunk_grid(const int64_t* offsets, const int64_t* indices, int64_t B, int64_t T, int64_t H, int64_t NT,
                      dim3* grid, int* ntfix) {
  if (offsets) FLA_REQUIRE(indices != nullptr && B == 1, FLA_E_INVALID);
  int64_t nf = (T + BT - 1) / BT;
  int64_t nblk = offsets ? NT : B * nf;
  FLA_REQUIRE(nblk <= 0x7fffffffLL && H <= 65535, FLA_E_UNSUPPORTED);
  *grid = dim3((unsigned)nblk, (unsigned)H);
  *ntfix = (int)nf;
  return FLA_OK;
}

// Workgroups of `kernel` (256 threads, no dynamic LDS) that the chip holds at once: the grid of a kernel whose
// workgroups walk many items each.  Asked of the runtime once per kernel address; the small table is shared by
// every instantiation and guarded by a mutex (entry points may be called from several host threads).
inline int64_t resident_workgroups_of(const void* kernel) {
  static std::mutex mu;
  static std::unordered_map<const void*, int> per_cu;
  std::lock_guard<std::mutex> lock(mu);
  auto it = per_cu.find(kernel);
  if (it == per_cu.end()) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, 0) != hipSuccess || n < 1) n = 1;
    it = per_cu.emplace(kernel, n).first;
  }
  return (int64_t)it->second * kNumCUs;
}
template <typename Kern>
inline int64_t resident_workgroups(Kern kernel) {
  return resident_workgroups_of((const void*)kernel);
}

// dst = src (or zeros when src is NULL), n floats: what the state gradient of a batch without any
// chunk is (d initial_state = d final_state).  A kernel rather than a memset / memcpy call, so that
// the launch can sit in a captured graph like the rest.
__global__ void copy_or_zero_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = src ? src[i] : 0.f;
}
inline int copy_or_zero(const float* src, float* dst, int64_t n, hipStream_t st) {
  if (!dst || n <= 0) return FLA_OK;
  const int64_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(copy_or_zero_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, st, src, dst, n);
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

// ---------------------------------------------------------------------------
// Operand fragments of the 16x16x32 MFMA for the one-pass forward kernels, whose accumulators go
// straight back into MFMA operands.
// ---------------------------------------------------------------------------
// Measured on gfx950 (one wave per SIMD): LDS reads peak at
// 256 B/clk per CU, writes near 80 B/clk.  For the access shape of an MFMA operand
// fragment (16 consecutive rows x 4 column groups per wave) the full read rate is reached
// by 8-byte reads whose groups are 8 bytes apart and whose row pitch is 16 bytes past a
// multiple of 256 (or 144 bytes); the same bytes fetched as one 16-byte read, or as a
// paired two-address read, run at half that rate.  A fragment is therefore two separate
// 8-byte reads (volatile, so that they are not fused into a paired read): accumulator rows
// {4g..4g+3} and {16+4g..16+4g+3} of a 32-slice, the order in which stacked 16x16
// accumulators fed straight back as the other operand enumerate their rows.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag16(const T* tile, int ld, int row0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef __attribute__((address_space(3))) const volatile v4 lds_v4;
  const T* p = tile + (row0 + (lane & 15)) * ld + k0 + 4 * (lane >> 4);
  v4 lo = *(lds_v4*)p;
  v4 hi = *(lds_v4*)(p + 16);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Time-contiguous tiles ([row][t], pitch LDT = 144 bytes) are written by lanes that own
// four adjacent rows each, i.e. with a row stride of four between neighbouring lanes
// (64 bytes modulo 256: unswizzled, such writes run 5x slower); XOR-ing row bits 4-5
// into the 16-byte slot index spreads them over all banks.  A fragment read covers the 16
// rows of one 16-row tile and sees a lane-uniform term.
FLA_DEVICE int swz_t(int row, int t) { return t ^ ((row >> 1) & 24); }

template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag16_t(const T* tile, int row0, int t0, int lane) {
  typedef typename Elem<T>::v4 v4;
  const int row = row0 + (lane & 15), t = t0 + 4 * (lane >> 4);
  typedef __attribute__((address_space(3))) const volatile v4 lds_v4;
  const T* p = tile + row * LDT;
  v4 lo = *(lds_v4*)(p + swz_t(row, t));
  v4 hi = *(lds_v4*)(p + swz_t(row, t + 16));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// A lower-triangular 64x64 tile stored as its ten 16x16 blocks on and below the diagonal, block (i, j) at
// index i (i + 1) / 2 + j, each block row-major.
constexpr int kTriElems = 10 * 256;

// A operand (16 rows x 32 contraction indices in accumulator-row order) of row tile tt, column pair s,
// from a packed triangular tile: block (tt, 2s) gives the first four indices of each group, block
// (tt, 2s + 1) the second four; above the diagonal that block is not stored and reads as zero.  A
// block is 512 contiguous bytes and the 64 lanes read each of its 8-byte pieces once.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag_tri(const T* tile, int tt, int s, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef __attribute__((address_space(3))) const volatile v4 lds_v4;
  const T* p = tile + (tt * (tt + 1) / 2 + 2 * s) * 256 + (lane & 15) * 16 + 4 * (lane >> 4);
  v4 lo = *(lds_v4*)p;
  v4 hi = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
  if (2 * s + 1 <= tt) hi = *(lds_v4*)(p + 256);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Largest exponent handed to exp() where a decay is inverted (e^{-G}); keeps the operand finite in
// 16-bit storage.  bf16 has fp32's exponent range; fp16 ends at 65504 (e^{11}), so fp16 chunks leave the
// single-reference arithmetic much earlier (e^{8} |k| stays representable for |k| up to 20).
template <typename T>
struct InvDecayLimit {
  static constexpr float value = 80.f;
};
template <>
struct InvDecayLimit<f16> {
  static constexpr float value = 8.f;
};

}  // namespace
