// Chunked gated delta rule forward for gfx950 (chunk size 64, 16-bit q/k/v,
// fp32 state).  gamma below is the chunk-local prefix sum of the scalar
// per-head log-gate g (fp32, produced by fla_chunk_local_cumsum).
//
//   gdr_fwd_wy_kernel   one workgroup per (chunk, head):
//                         M  = strict_lower(diag(beta) K K^T)            (MFMA)
//                         Aw = (I + M)^-1                                (fp32, blocked)
//                         Au = Aw * Gamma,  Gamma_ij = e^{gamma_i - gamma_j}
//                         w  = Aw (beta K),  u = Au (beta V)             (MFMA)
//                       The reference inverts I + M and I + M*Gamma separately
//                       (fla/ops/gated_delta_rule/wy_fast.py:150-208); since
//                       M*Gamma = D M D^-1 with D = diag(e^gamma), the second
//                       inverse is D Aw D^-1 = Aw * Gamma elementwise, so one
//                       inversion serves both.
//   gdr_fwd_h_kernel    serial scan per (sequence, head, 32 value columns):
//                         store h_c;  v_new = u - (w e^gamma) h_c;
//                         h <- e^{gamma_last} h_c + (k e^{gamma_last-gamma})^T v_new
//                       (fla/ops/common/chunk_delta_h.py:71-119).
//   chunk_fwd_o_kernel  one workgroup per (chunk, head):
//                         o = s (e^gamma * (q h_c) + tril(q k^T * Gamma) v_new)
//                       (fla/ops/common/chunk_o.py:68-101).  The scalar gate is
//                       applied to the fp32 scores / accumulators, so every
//                       exponent is <= 0 whatever the gate magnitude.
#include <type_traits>

#include "chunk_common.h"

namespace {

struct WyParams {
  const void* k;
  const void* v;
  const float* beta;
  const float* gam;
  void* w;
  void* u;
  void* Aw;
  void* Au;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  const void* Aw_in;   // both given: w = Aw_in (beta k), u = Au_in (beta v) on these matrices, nothing is inverted
  const void* Au_in;
};

// out^T tile = X^T-tile A^T for a lower-triangular 16-bit A [64 x 64] in LDS and
// X^T [columns][t] in LDS.  The transposed product leaves each lane with four
// consecutive output columns of one row (8-byte LDS writes in wy_store).
template <typename T, int N>
FLA_DEVICE void wy_apply(const T* sA, const T* sXT, f32x16* acc, int wave, int lane) {
  typedef typename Elem<T>::v8 v8;
  constexpr int TN = N / 64;
  const int rw = wave >> 1, cw = wave & 1;
  const int jsteps = (rw + 1) * 2;  // A is lower triangular
#pragma unroll
  for (int t = 0; t < TN; ++t) acc[t] = zero16();
  for (int js = 0; js < jsteps; ++js) {
    v8 a = lds_frag32<T>(sA, LDT, rw * 32, js * 16, lane);
#pragma unroll
    for (int t = 0; t < TN; ++t)
      acc[t] = Elem<T>::mfma32(lds_frag32<T>(sXT, LDT, (cw * TN + t) * 32, js * 16, lane), a, acc[t]);
  }
}

// accumulators of wy_apply -> row-major 16-bit tile [64][N + 8] in LDS
template <typename T, int N>
FLA_DEVICE void wy_acc_to_lds(T* sOut, const f32x16* acc, int wave, int lane) {
  typedef typename Elem<T>::v4 v4;
  constexpr int TN = N / 64;
  const int rw = wave >> 1, cw = wave & 1;
  T* op = sOut + (rw * 32 + (lane & 31)) * (N + 8) + 4 * (lane >> 5);
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      v4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (T)acc[t][4 * r4 + e];
      *(v4*)(op + (cw * TN + t) * 32 + 8 * r4) = o;
    }
}

// LDS tile [64][N + 8] -> global rows of pitch row_pitch, 16 bytes per lane, whole rows per wave
template <typename T, int N>
FLA_DEVICE void wy_store(const T* sOut, T* out, int64_t row_pitch, int L, int tid) {
  typedef typename Elem<T>::v8 v8;
  constexpr int CPR = N / 8, RPI = 256 / CPR;  // 16-byte columns per row, rows per pass
  const int c8 = (tid % CPR) * 8, r = tid / CPR;
#pragma unroll
  for (int i = r; i < BT; i += RPI)
    if (i < L) *(v8*)(out + (int64_t)i * row_pitch + c8) = *(const v8*)(sOut + i * (N + 8) + c8);
}

// rows [r0, r0+R) x four columns held in registers -> beta-scaled transposed 16-bit tile [column][t]
template <typename T, int R>
FLA_DEVICE void wy_stage_t(T* dstT, const typename Elem<T>::v4* reg, const float* sBeta, int r0, int c4) {
  typedef T tv __attribute__((ext_vector_type(R)));
  float b[R];
#pragma unroll
  for (int i = 0; i < R; i += 4) *(f32x4*)&b[i] = *(const f32x4*)&sBeta[r0 + i];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    tv o;
#pragma unroll
    for (int i = 0; i < R; ++i) o[i] = (T)((float)reg[i][j] * b[i]);
    *(tv*)&dstT[(c4 + j) * LDT + r0] = o;
  }
}

// One step of the forward substitution of wy_invert: x[c] += nm[J] * (x[c] of lane J of this DPP row), c <= J.
template <int J>
FLA_DEVICE void wy_subst_step(float (&x)[16], const float (&nm)[16]) {
#pragma unroll
  for (int c = 0; c <= J; ++c) x[c] = fmaf(nm[J], dpp_f32<0x150 + J>(x[c]), x[c]);   // row_newbcast:J
  if constexpr (J < 14) wy_subst_step<J + 1>(x, nm);
}

// X = (I + M)^-1 for a strictly lower triangular fp32 M [64][LDM] in LDS, into sX [64][LDM]
// (lower triangle valid; the upper right quadrant is used as scratch and holds garbage afterwards).
// 16x16 diagonal blocks by forward substitution, then block merges X_ba = -X_bb (M_ba X_aa) on the
// fp32 matrix instruction.  Called by all 256 threads after a barrier behind the writes of M; ends
// with a barrier, after which X is complete.  The barriers order LDS traffic only.
FLA_DEVICE void wy_invert(const float* sM, float* sX, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  float* sT = sX + 32;  // rows 0..31, columns 32..63 of X
  // the 16x16 blocks (0,1) and (2,3) of X are read by the 32x32 merges but never written
  for (int e = tid; e < 512; e += 256) {
    int blk = e >> 8, i = (e >> 4) & 15, j = e & 15;
    sX[(32 * blk + i) * LDM + 32 * blk + 16 + j] = 0.f;
  }
  // 16x16 diagonal blocks by forward substitution, all four at once on the first wave: DPP row b is block b,
  // a lane holds row i of its block of M (zero on and above the diagonal) and of X.  Step j subtracts
  // M[i][j] X[j][:] from every row; X[j][:] reaches the 16 lanes of the block through row_newbcast:j, so the
  // 120 dependent updates are register-to-register (the order of the products in every entry's sum is j
  // ascending, as a row-by-row substitution forms them).
  if (tid < 64) {
    const int b = tid >> 4, i = tid & 15;
    const float* Mr = sM + (16 * b + i) * LDM + 16 * b;
    float nm[16], x[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 m = *(const f32x4*)&Mr[4 * q];
#pragma unroll
      for (int e = 0; e < 4; ++e) nm[4 * q + e] = -m[e];
    }
#pragma unroll
    for (int c = 0; c < 16; ++c) x[c] = (c == i) ? 1.f : 0.f;
    wy_subst_step<0>(x, nm);
    float* Xr = sX + (16 * b + i) * LDM + 16 * b;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 o = {x[4 * q], x[4 * q + 1], x[4 * q + 2], x[4 * q + 3]};
      *(f32x4*)&Xr[4 * q] = o;
    }
  }
  lds_barrier();
  // ---- 32x32 diagonal blocks: X_ba = -X_bb (M_ba X_aa) for the block pairs (1,0) and (3,2)
  {
    const int a0 = 32 * (wave & 1), b0 = a0 + 16;  // waves 0 and 1 take one pair each
    if (wave < 2) lds_mm16_f32(sM + b0 * LDM + a0, LDM, sX + a0 * LDM + a0, LDM, sT + 16 * wave, LDM, 16, 1.f, lane);
    lds_barrier();
    if (wave < 2) lds_mm16_f32(sX + b0 * LDM + b0, LDM, sT + 16 * wave, LDM, sX + b0 * LDM + a0, LDM, 16, -1.f, lane);
  }
  lds_barrier();
  // ---- 64x64: X_BA = -X_BB (M_BA X_AA), one 16x16 output tile per wave
  {
    const int i0 = 16 * (wave >> 1), j0 = 16 * (wave & 1);
    lds_mm16_f32(sM + (32 + i0) * LDM, LDM, sX + j0, LDM, sT + i0 * LDM + j0, LDM, 32, 1.f, lane);
    lds_barrier();
    lds_mm16_f32(sX + (32 + i0) * LDM + 32, LDM, sT + j0, LDM, sX + (32 + i0) * LDM + j0, LDM, 32, -1.f, lane);
  }
  lds_barrier();

}

// The inversion keeps M and X = (I + M)^-1 in fp32.  Two LDS regions are
// reused over the kernel's life so that four workgroups fit a CU:
//   region A: k row-major -> M (fp32) -> Aw | Au (16-bit)
//   region B: [q row-major -> score tile] -> X (fp32; its always-zero upper
//             right quadrant doubles as the scratch tile of the block merges)
//             -> (beta k)^T -> (beta v)^T
// k and v stay in registers from the initial load until their transposed,
// beta-scaled tiles are written.
template <typename T, int K, int V>
__global__ __launch_bounds__(256, K <= 128 ? 4 : 2) void gdr_fwd_wy_kernel(WyParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int CG = K / 4, RG = 256 / CG, RPT = BT / RG;
  constexpr int CGV = V / 4, RGV = 256 / CGV, RPTV = BT / RGV;
  constexpr int KV = K > V ? K : V;
  constexpr int RA_BYTES = (BT * LDK * 2 > 2 * BT * LDT * 2) ? BT * LDK * 2 : 2 * BT * LDT * 2;
  constexpr int RB_BYTES0 = (KV * LDT * 2 > BT * LDM * 4) ? KV * LDT * 2 : BT * LDM * 4;
  constexpr int RB_BYTES = RB_BYTES0 > BT * LDK * 2 ? RB_BYTES0 : BT * LDK * 2;
  static_assert(RA_BYTES >= BT * LDM * 4 && RA_BYTES >= BT * LDK * 2, "region A holds M and the w tile");
  static_assert(RB_BYTES >= BT * (V + 8) * 2, "region B holds the u tile");
  __shared__ __attribute__((aligned(16))) char sRA[RA_BYTES];
  __shared__ __attribute__((aligned(16))) char sRB[RB_BYTES];
  __shared__ __attribute__((aligned(16))) float sBeta[BT];
  __shared__ float sGam[BT];
  T* sK = (T*)sRA;
  float* sM = (float*)sRA;
  T* sAw = (T*)sRA;
  T* sAu = sAw + BT * LDT;
  float* sX = (float*)sRB;
  T* sXbT = (T*)sRB;    // (beta k)^T, later (beta v)^T

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // workgroups that run together take different heads of the same chunks: their rows are
  // adjacent in memory, so the traffic spreads over all memory channels
  const int H = p.H;
  int hh;
  ChunkLoc cl = locate_chunk(p.offsets, p.indices, p.T, p.NTfix, H, &hh);
  const int L = cl.L;
  const int64_t row0 = cl.row0;

  // ---- loads
  const int rg = tid / CG, c4 = (tid % CG) * 4;
  const int rgv = tid / CGV, cv4 = (tid % CGV) * 4;
  v4 kreg[RPT], vreg[RPTV];
  {
    const T* kp = (const T*)p.k + (row0 * H + hh) * (int64_t)K + c4;
    const T* vp = (const T*)p.v + (row0 * H + hh) * (int64_t)V + cv4;
    const v4 z = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      int row = rg * RPT + i;
      kreg[i] = row < L ? *(const v4*)(kp + (int64_t)row * H * K) : z;
    }
#pragma unroll
    for (int i = 0; i < RPTV; ++i) {
      int row = rgv * RPTV + i;
      vreg[i] = (row < L && p.u) ? *(const v4*)(vp + (int64_t)row * H * V) : z;
    }
  }
  if (tid < BT) {
    bool ok = tid < L;
    sBeta[tid] = ok ? p.beta[(row0 + tid) * H + hh] : 0.f;
    sGam[tid] = p.gam ? p.gam[(row0 + (ok ? tid : L - 1)) * H + hh] : 0.f;
  }
  if (p.Aw_in) {
    // the two matrices as the caller kept them ([rows, H, 64], lower triangular): masked copies to LDS
    const int i = tid >> 2, j0 = (tid & 3) * 16;
    v8 aw[2], au[2];
#pragma unroll
    for (int h8 = 0; h8 < 2; ++h8) {
      const int64_t off = ((row0 + (i < L ? i : L - 1)) * H + hh) * (int64_t)BT + j0 + 8 * h8;
      aw[h8] = *(const v8*)((const T*)p.Aw_in + off);
      au[h8] = *(const v8*)((const T*)p.Au_in + off);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (i >= L || j0 + 8 * h8 + e > i) aw[h8][e] = au[h8][e] = (T)0.f;
    }
    *(v8*)&sAw[i * LDT + j0] = aw[0];
    *(v8*)&sAw[i * LDT + j0 + 8] = aw[1];
    *(v8*)&sAu[i * LDT + j0] = au[0];
    *(v8*)&sAu[i * LDT + j0 + 8] = au[1];
  } else {
#pragma unroll
  for (int i = 0; i < RPT; ++i) *(v4*)&sK[(rg * RPT + i) * LDK + c4] = kreg[i];
  __syncthreads();

  // ---- S = k k^T on the lower-triangular 32x32 quadrants; M = beta_i S_ij (j < i)
  {
    const int qi = wave >> 1, qj = wave & 1;
    f32x16 s = zero16();
    if (qj <= qi) {
#pragma unroll
      for (int ks = 0; ks < K; ks += 16)
        s = Elem<T>::mfma32(lds_frag32<T>(sK, LDK, qi * 32, ks, lane), lds_frag32<T>(sK, LDK, qj * 32, ks, lane), s);
    }
    __syncthreads();  // k row-major fully consumed: its storage becomes M
    if (qj <= qi) {
      const int j = qj * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int i = qi * 32 + c32_row(r, lane);
        sM[i * LDM + j] = (j < i) ? sBeta[i] * s[r] : 0.f;
      }
    }
  }
  __syncthreads();

  wy_invert(sM, sX, tid);

  // ---- Aw, Au in 16-bit (LDS for the products, optionally global for the backward pass)
  {
    const int i = tid >> 2, j0 = (tid & 3) * 16;
    const float gi = sGam[i];
    v8 aw[2], au[2];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      f32x4 xv = *(const f32x4*)&sX[i * LDM + j0 + 4 * q];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int jj = 4 * q + e, j = j0 + jj;
        float x = (j <= i) ? xv[e] : 0.f;  // the upper right quadrant held merge scratch
        float gamma = (j <= i) ? __expf(gi - sGam[j]) : 0.f;
        aw[jj >> 3][jj & 7] = (T)x;
        au[jj >> 3][jj & 7] = (T)(x * gamma);
      }
    }
    *(v8*)&sAw[i * LDT + j0] = aw[0];
    *(v8*)&sAw[i * LDT + j0 + 8] = aw[1];
    *(v8*)&sAu[i * LDT + j0] = au[0];
    *(v8*)&sAu[i * LDT + j0 + 8] = au[1];
    if (i < L) {
      int64_t off = ((row0 + i) * H + hh) * (int64_t)BT + j0;
      if (p.Aw) {
        *(v8*)((T*)p.Aw + off) = aw[0];
        *(v8*)((T*)p.Aw + off + 8) = aw[1];
      }
      if (p.Au) {
        *(v8*)((T*)p.Au + off) = au[0];
        *(v8*)((T*)p.Au + off + 8) = au[1];
      }
    }
  }
  }
  __syncthreads();  // X fully consumed: its storage becomes (beta k)^T
  f32x16 accw[K / 64], accu[V / 64];
  wy_stage_t<T, RPT>(sXbT, kreg, sBeta, rg * RPT, c4);
  __syncthreads();
  wy_apply<T, K>(sAw, sXbT, accw, wave, lane);
  __syncthreads();  // (beta k)^T fully consumed: its storage becomes (beta v)^T
  if (p.u) {        // u is optional: a forward that forms v_new from the triangular tiles needs w alone
    wy_stage_t<T, RPTV>(sXbT, vreg, sBeta, rgv * RPTV, cv4);
    __syncthreads();
    wy_apply<T, V>(sAu, sXbT, accu, wave, lane);
    __syncthreads();  // both operand regions are free: they carry the output tiles to whole-row stores
  }
  T* sWo = (T*)sRA;
  T* sUo = (T*)sRB;
  wy_acc_to_lds<T, K>(sWo, accw, wave, lane);
  if (p.u) wy_acc_to_lds<T, V>(sUo, accu, wave, lane);
  __syncthreads();
  wy_store<T, K>(sWo, (T*)p.w + (row0 * H + hh) * (int64_t)K, (int64_t)H * K, L, tid);
  if (p.u) wy_store<T, V>(sUo, (T*)p.u + (row0 * H + hh) * (int64_t)V, (int64_t)H * V, L, tid);
}

// ---------------------------------------------------------------------------
// Chunk-parallel preparation for the one-pass forward (fla_chunk_gated_delta_rule_fwd_scan): per
// (chunk, head) the lower-triangular 64x64 matrix the scan applies to value-column slabs,
//   Tu  = (Aw * Gamma) diag(beta)        Tu_ij  = Aw_ij e^{gamma_i - gamma_j} beta_j   (j <= i)
// With it  v_new = u - e^{gamma} (w h) = Tu (v - e^{gamma} (k h))  (u = Tu v and
// e^{gamma} w = Tu diag(e^{gamma}) k, since Aw Gamma-scaling is D Aw D^-1 and diagonal matrices
// commute), so neither w nor u is formed and the scan reads k, q, v and these 5 KB instead of
// k, q, w, u and a 8 KB score tile (the gated scores q k^T are formed inside the scan, which holds q and k
// anyway; this launch reads k alone).  Only the ten 16x16 blocks on and below the diagonal are stored,
// block (tt, jb) at index tt (tt + 1) / 2 + jb, each block row-major: at [chunk, head, 10, 16, 16].
// Rows past the end of a short chunk come out as zeros (beta is zero there).
struct PrepParams {
  const void* k;
  const float* beta;
  const float* g;      // raw log-gates [rows, H] (g_is_cumsum == 0) or their chunk-local prefix sums, or NULL
  int g_is_cumsum;
  float* gam_out;      // [rows, H]: the chunk-local prefix sums (written when g is raw), or NULL
  void* AT;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  void* w;             // KEEP: w = Aw (beta k) [rows, H, K] and Aw [rows, H, 64], what the backward reads
  void* Aw;
  float l2_eps;        // L2N: k is un-normalised; the launch works with k / sqrt(sum k^2 + l2_eps) ...
  float* rk_out;       //      ... and leaves the factors 1 / sqrt(sum k^2 + l2_eps), fp32 [rows, H], for the scan
};

// resident workgroups per CU (register budget): four, or three for the variant that also writes w and Aw
constexpr int kPrepResident = 4, kPrepResidentKeep = 3;
FLA_DEVICE int tri_block(int tt, int jb) { return tt * (tt + 1) / 2 + jb; }

// A workgroup walks several (chunk, head) items (grid-stride) and loads the k rows, beta and the gate
// of its next item into registers once the matrix products of the current one have released their
// accumulators: the loads land while the inversion runs (measured: worth about 4 %; the launch is a chain
// of short dependent phases - removing the inversion, the stores or the loads each saves 15-20 % - rather
// than bound by one resource).
// KEEP: the forward of a pass that will be differentiated also leaves w = Aw (beta k) and Aw in memory (the WY
// launch of the reference's decomposition, without a second inversion and a second pass over k).
// L2N: k arrives un-normalised (what l2_norm(k) in front of the operator would normalise,
// fla/layers/gated_deltanet.py:235).  The rows are not rewritten: k^ = r k with r = 1 / sqrt(sum k^2 + eps) per row, so
// k^ k^T = diag(r) (k k^T) diag(r) and the factors go onto the rows and columns of the product; r comes from the
// pieces the lanes hold anyway (a row of K elements sits in K / 8 adjacent lanes) and is left in memory for the scan.
template <typename T, int K, bool KEEP, bool L2N = false>
__global__ __launch_bounds__(256, KEEP ? kPrepResidentKeep : kPrepResident) void gdr_fwd_prep_kernel(PrepParams p, int64_t total) {
  static_assert(!(KEEP && L2N), "a forward that keeps w and Aw takes normalised keys");
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int CG = K / 4, RG = 256 / CG, RPT = BT / RG;
  constexpr int R_BYTES = BT * LDK * 2 > BT * LDM * 4 ? BT * LDK * 2 : BT * LDM * 4;
  __shared__ __attribute__((aligned(16))) char sRA[R_BYTES];   // k row-major -> M (fp32) -> packed Tu tile
  __shared__ __attribute__((aligned(16))) char sRB[R_BYTES];   // X (fp32) -> KEEP: k row-major again
  __shared__ __attribute__((aligned(16))) float sBeta[BT];
  __shared__ __attribute__((aligned(16))) float sGam[BT];
  __shared__ __attribute__((aligned(16))) float sRk[L2N ? BT : 4];   // L2N: 1 / |k_t| (zero past the end of the chunk)
  T* sK = (T*)sRA;
  float* sM = (float*)sRA;
  T* sK2 = (T*)sRB;
  T* sTu = (T*)sRA;
  T* sAb = (T*)sRA + kTriElems;   // KEEP: Aw diag(beta), row-major [64][LDT], behind the packed tile
  static_assert((kTriElems + BT * LDT) * 2 <= R_BYTES, "region A holds the packed tile and Aw diag(beta)");
  float* sX = (float*)sRB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = p.H;
  // 16-byte pieces: a lane owns 8 adjacent columns of NPL rows
  constexpr int C8 = K / 8, RPP = 256 / C8, NPL = BT / RPP;
  const int r0 = tid / C8, c8 = (tid % C8) * 8;
  const uint32_t pitch = (uint32_t)H * K * 2;   // bytes between rows of one head
  uint32_t off[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) off[i] = (uint32_t)(r0 + RPP * i) * pitch + c8 * 2;
  const v8 z = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};

  struct Item {
    int L, hh;
    int64_t row0, cglob;
    v8 k[NPL];
    float beta, g;   // wave 0: this lane's row
  };
  // Items are numbered head-fastest: item = chunk * H + head.  The walk keeps (chunk, head) and advances
  // them by the grid size without a division; the chunk's place in its sequence comes from 32-bit
  // arithmetic on wave-uniform values (scalar loads for a packed batch).
  const uint32_t step_c = gridDim.x / (uint32_t)H, step_h = gridDim.x % (uint32_t)H;
  uint32_t it_chunk = blockIdx.x / (uint32_t)H, it_head = blockIdx.x % (uint32_t)H;
  auto fetch = [&](Item& it) __attribute__((always_inline)) {
    const uint32_t cidx = __builtin_amdgcn_readfirstlane(it_chunk);
    const int hh = (int)__builtin_amdgcn_readfirstlane(it_head);
    ChunkLoc cl;
    {
      int64_t bos, len;
      uint32_t ic;
      if (p.offsets) {
        const int64_t n = p.indices[2 * (int64_t)cidx];
        ic = (uint32_t)p.indices[2 * (int64_t)cidx + 1];
        bos = p.offsets[n];
        len = p.offsets[n + 1] - bos;
      } else {
        const uint32_t b = cidx / (uint32_t)p.NTfix;
        ic = cidx - b * (uint32_t)p.NTfix;
        bos = (int64_t)b * p.T;
        len = p.T;
      }
      cl.row0 = bos + (int64_t)ic * BT;
      const int64_t rem = len - (int64_t)ic * BT;
      cl.L = (int)(rem < BT ? rem : BT);
      cl.cglob = cidx;
    }
    it.L = cl.L;
    it.hh = hh;
    it.row0 = cl.row0;
    it.cglob = cl.cglob;
    const char* kp = (const char*)p.k + (cl.row0 * H + hh) * (int64_t)K * 2;
    const uint32_t lim = (uint32_t)(cl.L - 1) * pitch + c8 * 2;   // rows past the end: re-read the last one
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const uint32_t o = off[i] < lim ? off[i] : lim;
      it.k[i] = *(const v8*)(kp + o);
    }
    if (wave == 0) {
      const int64_t gi = (cl.row0 + (lane < cl.L ? lane : cl.L - 1)) * H + hh;
      it.beta = p.beta[gi];
      it.g = p.g ? p.g[gi] : 0.f;
    }
  };

  auto advance = [&]() {
    it_chunk += step_c;
    it_head += step_h;
    if (it_head >= (uint32_t)H) {
      it_head -= (uint32_t)H;
      ++it_chunk;
    }
  };
  Item cur;
  int64_t lin = blockIdx.x;
  if (lin >= total) return;
  fetch(cur);
  for (;;) {
    const int L = cur.L;
    const int hh = cur.hh;
    const int64_t row0 = cur.row0, cglob = cur.cglob;
    // ---- k row-major (rows past the end of the chunk zero), beta, gamma
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int row = r0 + RPP * i;
      const v8 kr = cur.k[i];
      if constexpr (L2N) {
        const float rk = l2norm_rstd<T, K / 8>(kr, p.l2_eps);
        if (c8 == 0) {
          sRk[row] = row < L ? rk : 0.f;
          if (row < L) p.rk_out[(row0 + row) * H + hh] = rk;
        }
      }
      *(v8*)&sK[row * LDK + c8] = row < L ? kr : z;
    }
    if (wave == 0) {
      const bool ok = lane < L;
      sBeta[lane] = ok ? cur.beta : 0.f;
      float gam = cur.g;   // a cumulative gate: rows past the end carry the last valid row's
      if (p.g && !p.g_is_cumsum) {
        // inclusive prefix sum over the 64 rows: DPP row scans plus the totals of the earlier rows of 16;
        // rows past the end add zero, so they carry the last valid row's sum
        float x = row_prefix16(ok ? cur.g : 0.f);
        const float t0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 15));
        const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 31));
        const float t2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 47));
        const int r = lane >> 4;
        gam = x + (r >= 1 ? t0 : 0.f) + (r >= 2 ? t1 : 0.f) + (r >= 3 ? t2 : 0.f);
        if (p.gam_out && ok) p.gam_out[(row0 + lane) * H + hh] = gam;
      }
      sGam[lane] = gam;
    }
    lds_barrier();   // LDS-only barriers throughout: a full one would wait for the loads issued further down
    const int64_t next = lin + gridDim.x;
    const bool more = next < total;   // workgroup-uniform

    // ---- S = k k^T on the lower-triangular 32x32 quadrants
    const int qi = wave >> 1, qj = wave & 1;
    f32x16 s = zero16();
    if (qj <= qi) {
#pragma unroll
      for (int ks = 0; ks < K; ks += 16) {
        s = Elem<T>::mfma32(lds_frag32<T>(sK, LDK, qi * 32, ks, lane), lds_frag32<T>(sK, LDK, qj * 32, ks, lane), s);
      }
    }
    lds_barrier();  // k row-major fully consumed: its storage becomes M
    if (qj <= qi) {
      // s: lane <-> column j, registers <-> four consecutive rows i per quad
      const int j = qj * 32 + (lane & 31);
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int ib = qi * 32 + 8 * r4 + 4 * (lane >> 5);
        f32x4 b = *(const f32x4*)&sBeta[ib];
        if constexpr (L2N) {
          const f32x4 ri = *(const f32x4*)&sRk[ib];
          const float rj = sRk[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) b[e] *= ri[e] * rj;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) sM[(ib + e) * LDM + j] = (j < ib + e) ? b[e] * s[4 * r4 + e] : 0.f;
      }
    }
    lds_barrier();  // M complete; region B becomes X
    // the next item's rows start their way to the registers now: the matrix products above no longer
    // hold their accumulators, and the inversion below needs few registers and no memory
    v8 kkeep[KEEP ? NPL : 1];
    if constexpr (KEEP) {
#pragma unroll
      for (int i = 0; i < NPL; ++i) kkeep[i] = cur.k[i];
    }
    if (more) {
      advance();
      fetch(cur);
    }

    wy_invert(sM, sX, tid);

    // ---- Tu = (X * Gamma) diag(beta): the ten 16x16 blocks of the lower triangle are dealt to the waves; a lane
    // holds four adjacent columns of one row, and a block leaves for memory as 512 contiguous bytes straight
    // from the registers (the packed tile is never staged)
    {
      const int wv = __builtin_amdgcn_readfirstlane(wave);
      const int r = lane >> 2, c4 = 4 * (lane & 3);
      T* at = (T*)p.AT + (cglob * H + hh) * (int64_t)kTriElems;
#pragma unroll
      for (int pass = 0; pass < 3; ++pass) {
        const int idx = wv + 4 * pass;          // tri_block(tt, jb)
        if (idx < 10) {
          const int tt = idx >= 6 ? 3 : idx >= 3 ? 2 : idx >= 1 ? 1 : 0;
          const int jb = idx - tt * (tt + 1) / 2;
          const int i = 16 * tt + r, j0 = 16 * jb + c4;
          const f32x4 xv = *(const f32x4*)&sX[i * LDM + j0];
          const f32x4 gj = *(const f32x4*)&sGam[j0];
          const f32x4 bj = *(const f32x4*)&sBeta[j0];
          const float gi = sGam[i];
          // X is zero above the diagonal of a diagonal block; the exponent there is set to zero so that the product stays zero
          const f32x4 x = xv;
          v4 tu;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float d = gi - gj[e];
            tu[e] = (T)(x[e] * __expf(tt != jb || c4 + e <= r ? d : 0.f) * bj[e]);
          }
          *(v4*)(at + idx * 256 + 4 * lane) = tu;
          if constexpr (KEEP) {
            // Aw row piece to memory; Aw diag(beta) as a row-major 16-bit tile in region A (M is dead)
            v4 aw, ab;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              aw[e] = (T)x[e];
              ab[e] = (T)(x[e] * bj[e]);
            }
            *(v4*)&sAb[i * LDT + j0] = ab;
            if (i < L) *(v4*)((T*)p.Aw + ((row0 + i) * H + hh) * (int64_t)BT + j0) = aw;
          }
        }
      }
      if constexpr (KEEP) {
        // the blocks above the diagonal of Aw and of Aw diag(beta) are zero
        const v4 z4 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
          const int u = wv + 4 * pass;          // the six blocks (tt, jb), jb > tt
          if (u < 6) {
            const int tt = u >= 5 ? 2 : u >= 3 ? 1 : 0;
            const int jb = u - (tt == 0 ? 0 : tt == 1 ? 3 : 5) + tt + 1;
            const int i = 16 * tt + r, j0 = 16 * jb + c4;
            *(v4*)&sAb[i * LDT + j0] = z4;
            if (i < L) *(v4*)((T*)p.Aw + ((row0 + i) * H + hh) * (int64_t)BT + j0) = z4;
          }
        }
      }
    }
    if constexpr (KEEP) {
      lds_barrier();   // X fully consumed
      // its storage takes k row-major again (rows past the end of the chunk zero)
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int row = r0 + RPP * i;
        *(v8*)&sK2[row * LDK + c8] = row < L ? kkeep[i] : z;
      }
    }
    if constexpr (KEEP) {
      lds_barrier();   // k row-major complete
      // w^T = k^T (Aw diag(beta))^T: a lane ends up with one time row and four consecutive key channels per quad
      const int rw = wave & 1, cb = wave >> 1;   // rows 32 rw .., key channels (K / 2) cb ..
      constexpr int TN = K / 64;
      f32x16 acc[TN];
#pragma unroll
      for (int t = 0; t < TN; ++t) acc[t] = zero16();
      const int jsteps = (rw + 1) * 2;           // Aw is lower triangular
      for (int js = 0; js < jsteps; ++js) {
        const v8 a = lds_frag32<T>(sAb, LDT, rw * 32, js * 16, lane);
#pragma unroll
        for (int t = 0; t < TN; ++t)
          acc[t] = Elem<T>::mfma32(frag32_tr<T>(sK2, LDK, (cb * TN + t) * 32, js * 16, lane), a, acc[t]);
      }
      const int i = rw * 32 + (lane & 31);
      if (i < L) {
        T* wp = (T*)p.w + ((row0 + i) * H + hh) * (int64_t)K + 4 * (lane >> 5);
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            v4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (T)acc[t][4 * r4 + e];
            *(v4*)(wp + (cb * TN + t) * 32 + 8 * r4) = o;
          }
      }
    }
    if (!more) break;
    lin = next;
    lds_barrier();  // the packed tiles are on their way: the tiles of the next item may be written
  }
}

// ---------------------------------------------------------------------------
struct DHParams {
  const void* k;
  const void* w;
  const void* u;
  const float* gam;
  const float* h0;
  void* h;
  void* v_new;
  float* ht;
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  int64_t T;
  int H, V, N;
  void* h2;  // with the transposed fragment layout: a second copy in FLA_H_FRAGMENT order, or NULL
};

// One workgroup: all K rows x 32 value columns of one (sequence, head) state.
// Wave w keeps the 32x32 state tiles kt = w, w+4, ... in MFMA accumulators.
// HL: 0 row-major [K,V] in T, 1 fragment order in T, 2 row-major fp32.
// VN: v_new is written (its store is unconditional, so the choice is made at compile time).
template <typename T, int K, int HL, bool VN>
__global__ __launch_bounds__(256) void gdr_fwd_h_kernel(DHParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  typedef T t2 __attribute__((ext_vector_type(2)));
  constexpr int BV = 32;
  constexpr int LDK = K + 8;
  constexpr int CG = K / 4, RG = 256 / CG, RPT = BT / RG;
  constexpr int KT32 = K / 32;
  constexpr int NKT = (KT32 + 3) / 4;  // state tiles per wave
  __shared__ __attribute__((aligned(16))) T sW[BT * LDK];    // w e^gamma, row-major
  __shared__ __attribute__((aligned(16))) T sKt[K * LDT];    // (k e^{gamma_last-gamma})^T, swz16
  __shared__ __attribute__((aligned(16))) T sUt[BV * LDT];   // u^T
  __shared__ __attribute__((aligned(16))) T sHt[BV * LDK];   // h^T in 16-bit
  __shared__ __attribute__((aligned(16))) T sVnT[BV * LDT];  // v_new^T

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = p.H, V = p.V;
  const int nvt = V / BV;
  int64_t id = xcd_remap(blockIdx.x, gridDim.x);
  const int vt = (int)(id % nvt);
  const int nh = (int)(id / nvt);
  const int n = nh / H, hh = nh % H;
  const int vbase = vt * BV;
  SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);

  // HL == 3 additionally keeps every tile transposed (rows v, cols k): the global copy is
  // then written in FLA_H_FRAGMENT_T order for the backward kernels, which contract over v.
  constexpr bool TR = (HL == 3);
  f32x16 acc[NKT];
  f32x16 acct[TR ? NKT : 1];
#pragma unroll
  for (int a = 0; a < NKT; ++a) {
    acc[a] = zero16();
    if (TR) acct[a] = zero16();
    int kt = wave + 4 * a;
    if (p.h0 && kt < KT32) {
      const float* h0p = p.h0 + (int64_t)nh * K * V;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[a][r] = h0p[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)];
        if (TR) acct[a][r] = h0p[(int64_t)(kt * 32 + (lane & 31)) * V + vbase + c32_row(r, lane)];
      }
    }
  }

  // Prefetch registers.  Two independent sets, each refilled right after the staging step that
  // consumed it, one full iteration before its next use, so that no register copy and no wait
  // sits between issuing a load and the end of the iteration:
  //   WU: w as (RPT rows x 4 cols), u as (4 rows x 2 cols), gamma per row  -> sW, sUt
  //   KR: k as (RPT rows x 4 cols), gamma of the chunk's last row          -> sKt
  const int rg = tid / CG, c4 = (tid % CG) * 4;
  const int urg = tid >> 4, uc2 = (tid & 15) * 2;
  struct WURegs {
    v4 w[RPT];
    float gam[RPT];
    t2 u[4];
  };
  struct KRegs {
    v4 k[RPT];
    float glast;
  };
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };
  // Addressing: a wave-uniform 64-bit base per chunk plus 32-bit per-lane byte offsets that are
  // computed once.  Every load is unconditional: rows past the end of a short (last) chunk are
  // redirected to its last row (one unsigned minimum) and masked where they are used.
  const uint32_t pitchK = (uint32_t)H * K * sizeof(T), pitchV = (uint32_t)H * V * sizeof(T), pitchG = (uint32_t)H * 4;
  uint32_t offk[RPT], offg[RPT], offu[4];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    offk[i] = (uint32_t)(rg * RPT + i) * pitchK + c4 * sizeof(T);
    offg[i] = p.gam ? (uint32_t)(rg * RPT + i) * pitchG : 0u;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) offu[i] = (uint32_t)(urg * 4 + i) * pitchV + uc2 * sizeof(T);
  const char* gw = (const char*)p.w + (sp.bos * H + hh) * (int64_t)K * sizeof(T);
  const char* gk = (const char*)p.k + (sp.bos * H + hh) * (int64_t)K * sizeof(T);
  const char* gu = (const char*)p.u + ((sp.bos * H + hh) * (int64_t)V + vbase) * sizeof(T);
  const char* gg = p.gam ? (const char*)(p.gam + sp.bos * H + hh) : (const char*)&kZeroWord;
  const int64_t stepG = p.gam ? (int64_t)BT * pitchG : 0;
  auto load_wu = [&](int64_t c, WURegs& R) {
    const uint32_t last = (uint32_t)(chunk_len(c) - 1);
    const uint32_t limk = last * pitchK + c4 * sizeof(T), limu = last * pitchV + uc2 * sizeof(T);
    const uint32_t limg = p.gam ? last * pitchG : 0u;
    const char* wb = gw + c * (int64_t)BT * pitchK;
    const char* ub = gu + c * (int64_t)BT * pitchV;
    const char* gb = gg + c * stepG;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      R.w[i] = *(const v4*)(wb + (offk[i] < limk ? offk[i] : limk));
      R.gam[i] = *(const float*)(gb + (offg[i] < limg ? offg[i] : limg));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) R.u[i] = *(const t2*)(ub + (offu[i] < limu ? offu[i] : limu));
  };
  auto load_k = [&](int64_t c, KRegs& R) {
    const uint32_t last = (uint32_t)(chunk_len(c) - 1);
    const uint32_t limk = last * pitchK + c4 * sizeof(T);
    const char* kb = gk + c * (int64_t)BT * pitchK;
#pragma unroll
    for (int i = 0; i < RPT; ++i) R.k[i] = *(const v4*)(kb + (offk[i] < limk ? offk[i] : limk));
    R.glast = *(const float*)(gg + c * stepG + (p.gam ? last * pitchG : 0u));
  };
  // state-independent operand tiles of one chunk; the gates of its rows stay in registers for
  // the key tile of the same chunk, which is staged half an iteration later
  float grow[RPT];
  auto stage_wu = [&](const WURegs& R) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      int row = rg * RPT + i;
      grow[i] = R.gam[i];
      float eg = __expf(R.gam[i]);
      v4 wv;
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = (T)((float)R.w[i][j] * eg);
      *(v4*)&sW[row * LDK + c4] = wv;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      v4 uv = v4{R.u[0][j], R.u[1][j], R.u[2][j], R.u[3][j]};
      *(v4*)&sUt[(uc2 + j) * LDT + urg * 4] = uv;
    }
  };
  // a lane owns RPT consecutive time rows of 4 key columns: one vector write per column
  auto stage_k = [&](const KRegs& R, int L) {
    // (in pieces of at most one 16-byte slot, the unit the swizzle permutes)
    constexpr int PW = RPT < 8 ? RPT : 8;
    typedef T rvec __attribute__((ext_vector_type(PW)));
    float e[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) e[i] = (rg * RPT + i) < L ? __expf(R.glast - grow[i]) : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int i0 = 0; i0 < RPT; i0 += PW) {
        rvec x;
#pragma unroll
        for (int i = 0; i < PW; ++i) x[i] = (T)((float)R.k[i0 + i][j] * e[i0 + i]);
        *(rvec*)&sKt[(c4 + j) * LDT + swz16(c4 + j, rg * RPT + i0)] = x;
      }
    }
  };
  // state entering chunk c: 16-bit transpose in LDS for the MFMA, global copy for the output kernel
  auto publish_h = [&](int64_t c) {
#pragma unroll
    for (int a = 0; a < NKT; ++a) {
      int kt = wave + 4 * a;
      if (kt < KT32) {
        v8 lo, hi;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          lo[r] = (T)acc[a][r];
          hi[r] = (T)acc[a][r + 8];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v4 x;
#pragma unroll
          for (int b = 0; b < 4; ++b) x[b] = (q < 2) ? lo[4 * q + b] : hi[4 * (q - 2) + b];
          *(v4*)&sHt[(lane & 31) * LDK + kt * 32 + 8 * q + 4 * (lane >> 5)] = x;
        }
        if (p.h) {
          int64_t blk = ((chunk0 + c) * H + hh) * (int64_t)K * V;
          if (HL == 1) {
            T* hp = (T*)p.h + blk + (((int64_t)kt * (V / 32) + vt) * 64 + lane) * 16;
            *(v8*)hp = lo;
            *(v8*)(hp + 8) = hi;
          } else if (HL == 3) {
            T* hp = (T*)p.h + blk + (((int64_t)vt * (K / 32) + kt) * 64 + lane) * 16;
            v8 tl, th;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
              tl[r] = (T)acct[a][r];
              th[r] = (T)acct[a][r + 8];
            }
            *(v8*)hp = tl;
            *(v8*)(hp + 8) = th;
            if (p.h2) {
              T* hq = (T*)p.h2 + blk + (((int64_t)kt * (V / 32) + vt) * 64 + lane) * 16;
              *(v8*)hq = lo;
              *(v8*)(hq + 8) = hi;
            }
          } else if (HL == 0) {
            T* hp = (T*)p.h + blk;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              hp[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] = (T)acc[a][r];
          } else {
            float* hp = (float*)p.h + blk;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              hp[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] = acc[a][r];
          }
        }
      }
    }
  };

  // Two barriers per chunk and single-buffered tiles:
  //   phase A (after barrier 1): v_new from sW, sUt, sHt;  stage sKt of the same chunk
  //   phase B (after barrier 2): state update from sKt, sVnT;  v_new leaves as 16-byte row pieces;
  //                              stage sW, sUt, sHt of the next chunk
  WURegs WU;
  KRegs KR;
  const int st = tid >> 2, sp8 = (tid & 3) * 8;  // v_new store: time row, first of 8 value columns
  auto step = [&](int64_t c, auto more) {
    const int L = chunk_len(c);
    lds_barrier();  // (1)
    // ---- v_new = u - (w e^gamma) h : wave w owns rows 16w..16w+15, two 16-column tiles
    {
      f32x4 d[2] = {zero4(), zero4()};
#pragma unroll
      for (int ks = 0; ks < K; ks += 32) {
        v8 a = lds_frag16<T>(sW, LDK, wave * 16, ks, lane);
#pragma unroll
        for (int j = 0; j < 2; ++j) d[j] = Elem<T>::mfma16(a, lds_frag16<T>(sHt, LDK, j * 16, ks, lane), d[j]);
      }
      const int tr = wave * 16 + 4 * (lane >> 4);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        int vc = j * 16 + (lane & 15);
        v4 uu = *(const v4*)&sUt[vc * LDT + tr];
        v4 vn;
#pragma unroll
        for (int r = 0; r < 4; ++r) vn[r] = (T)((float)uu[r] - d[j][r]);
        *(v4*)&sVnT[vc * LDT + tr] = vn;
      }
    }
    stage_k(KR, L);
    const float dec = __expf(KR.glast);
    if constexpr (decltype(more)::value) load_k(c + 1, KR);
    lds_barrier();  // (2)
    // ---- h <- e^{gamma_last} h + (k e^{gamma_last-gamma})^T v_new
#pragma unroll
    for (int a = 0; a < NKT; ++a) {
      int kt = wave + 4 * a;
      if (kt < KT32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] *= dec;
        if (TR) {
#pragma unroll
          for (int r = 0; r < 16; ++r) acct[a][r] *= dec;
        }
#pragma unroll
        for (int s = 0; s < BT; s += 16) {
          v8 fk = lds_frag32_swz<T>(sKt, LDT, kt * 32, s, lane);
          v8 fv = lds_frag32<T>(sVnT, LDT, 0, s, lane);
          acc[a] = Elem<T>::mfma32(fk, fv, acc[a]);
          if (TR) acct[a] = Elem<T>::mfma32(fv, fk, acct[a]);
        }
      }
    }
    if constexpr (VN) {
      // rows past the end of a short chunk repeat its last row (same address, same data), so the
      // store is unconditional and the waits for the loads in flight stay exact
      const int sr = st < L ? st : L - 1;
      v8 x;
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = sVnT[(sp8 + j) * LDT + sr];
      *(v8*)((T*)p.v_new + ((sp.bos + c * BT + sr) * H + hh) * (int64_t)V + vbase + sp8) = x;
    }
    if constexpr (decltype(more)::value) {
      stage_wu(WU);
      publish_h(c + 1);
      load_wu(c + 2 < nchunks ? c + 2 : nchunks - 1, WU);
      // keeps the loads here, at the end of the iteration: without it they are merged with the
      // prologue's copy at the top of the loop and start half an iteration later
      asm volatile("" ::: "memory");
    }
  };
  if (nchunks > 0) {
    load_wu(0, WU);
    stage_wu(WU);
    publish_h(0);
    load_wu(nchunks > 1 ? 1 : 0, WU);
    load_k(0, KR);
    for (int64_t c = 0; c + 1 < nchunks; ++c) step(c, std::true_type{});
    step(nchunks - 1, std::false_type{});
  }
  if (p.ht) {
    float* htp = p.ht + (int64_t)nh * K * V;
#pragma unroll
    for (int a = 0; a < NKT; ++a) {
      int kt = wave + 4 * a;
      if (kt < KT32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) htp[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] = acc[a][r];
      }
    }
  }
}

// ---------------------------------------------------------------------------
struct DOParams {
  const void* q;
  const void* k;
  const void* v;
  const float* gam;
  const void* h;
  void* o;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  float scale;
};

template <typename T, int K, int V>
__global__ __launch_bounds__(256) void chunk_fwd_o_kernel(DOParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int C8 = K / 8;                 // 16-byte pieces per row
  constexpr int NP = BT * C8 / 256;          // pieces per thread
  constexpr int CGV = V / 4, RGV = 256 / CGV, RPTV = BT / RGV;
  constexpr int KT32 = K / 32, TV = V / 64;
  __shared__ __attribute__((aligned(16))) T sQK[2 * BT * LDK];  // q | k (later P); at the end the output tile
  __shared__ __attribute__((aligned(16))) T sVt[V * LDT];
  __shared__ float sGam[BT];
  T* sQ = sQK;
  T* sK = sQK + BT * LDK;
  T* sP = sK;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // workgroups that run together take different heads of the same chunks: their rows are
  // adjacent in memory, so the traffic spreads over all memory channels
  const int H = p.H;
  int hh;
  ChunkLoc cl = locate_chunk(p.offsets, p.indices, p.T, p.NTfix, H, &hh);
  const int L = cl.L;
  const int64_t row0 = cl.row0;

  v8 qreg[NP], kreg[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    if (row < L) {
      int64_t off = ((row0 + row) * H + hh) * (int64_t)K + c8;
      qreg[i] = *(const v8*)((const T*)p.q + off);
      kreg[i] = *(const v8*)((const T*)p.k + off);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) qreg[i][j] = kreg[i][j] = (T)0.f;
    }
  }
  const int rgv = tid / CGV, cv4 = (tid % CGV) * 4;
  v4 vreg[RPTV];
#pragma unroll
  for (int i = 0; i < RPTV; ++i) {
    int row = rgv * RPTV + i;
    if (row < L) vreg[i] = *(const v4*)((const T*)p.v + ((row0 + row) * H + hh) * (int64_t)V + cv4);
    else vreg[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
  }
  if (tid < BT) sGam[tid] = p.gam ? p.gam[(row0 + (tid < L ? tid : L - 1)) * H + hh] : 0.f;
  const int rw = wave >> 1, cw = wave & 1;
  v8 hf[KT32][TV][2];
  {
    const T* hp = (const T*)p.h + (cl.cglob * H + hh) * (int64_t)K * V;
#pragma unroll
    for (int kt = 0; kt < KT32; ++kt)
#pragma unroll
      for (int tv = 0; tv < TV; ++tv) {
        const T* f = hp + (((int64_t)kt * (V / 32) + (cw * TV + tv)) * 64 + lane) * 16;
        hf[kt][tv][0] = *(const v8*)f;
        hf[kt][tv][1] = *(const v8*)(f + 8);
      }
  }
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    *(v8*)&sQ[row * LDK + c8] = qreg[i];
    *(v8*)&sK[row * LDK + c8] = kreg[i];
  }
  {
    // a lane owns RPTV consecutive time rows of 4 value columns: one vector write per column
    typedef T rvec __attribute__((ext_vector_type(RPTV)));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      rvec x;
#pragma unroll
      for (int i = 0; i < RPTV; ++i) x[i] = vreg[i][j];
      *(rvec*)&sVt[(cv4 + j) * LDT + rgv * RPTV] = x;
    }
  }
  __syncthreads();

  // Every product is formed transposed (operands swapped): a lane then holds one time row and four
  // consecutive columns per register quad, so the score tile and the output tile are written to
  // LDS with 8-byte vectors and the output leaves as whole rows.
  const int qi = wave >> 1, qj = wave & 1;
  f32x16 s = zero16();   // s[4a+b] = (q k^T)[i][j0+b], i = 32 qi + lane%32, j0 = 32 qj + 8a + 4 (lane/32)
  if (qj <= qi) {
#pragma unroll
    for (int ks = 0; ks < K; ks += 16)
      s = Elem<T>::mfma32(lds_frag32<T>(sK, LDK, qj * 32, ks, lane), lds_frag32<T>(sQ, LDK, qi * 32, ks, lane), s);
  }
  __syncthreads();  // all reads of sK done before P overwrites it
  {
    const int i = qi * 32 + (lane & 31);
    const float gi = sGam[i];
#pragma unroll
    for (int a4 = 0; a4 < 4; ++a4) {
      const int j0 = qj * 32 + 8 * a4 + 4 * (lane >> 5);
      v4 x;
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const int j = j0 + b4;
        x[b4] = (T)((j <= i) ? s[4 * a4 + b4] * p.scale * __expf(gi - sGam[j]) : 0.f);
      }
      *(v4*)&sP[i * LDT + j0] = x;
    }
  }
  __syncthreads();

  const int trow = rw * 32 + (lane & 31);   // this lane's time row in the transposed output tiles
  f32x16 acc[TV];                           // acc[tv][4a+b] = o[trow][32 (cw TV + tv) + 8a + 4 (lane/32) + b]
#pragma unroll
  for (int tv = 0; tv < TV; ++tv) acc[tv] = zero16();
#pragma unroll
  for (int kt = 0; kt < KT32; ++kt)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v8 a = lds_frag32_perm<T>(sQ, LDK, rw * 32, kt * 32 + half * 16, lane);
#pragma unroll
      for (int tv = 0; tv < TV; ++tv) acc[tv] = Elem<T>::mfma32(hf[kt][tv][half], a, acc[tv]);
    }
  {
    const float rs = p.scale * __expf(sGam[trow]);
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[tv][r] *= rs;
  }
  const int jend = (rw + 1) * 32;
  for (int js = 0; js < jend; js += 16) {
    v8 a = lds_frag32<T>(sP, LDT, rw * 32, js, lane);
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
      acc[tv] = Elem<T>::mfma32(lds_frag32<T>(sVt, LDT, (cw * TV + tv) * 32, js, lane), a, acc[tv]);
  }
  __syncthreads();  // q is consumed: its tile carries the output
  constexpr int LDO = V + 8;
  static_assert(LDO <= 2 * LDK, "the output tile fits the q and k tiles");
  T* sO = sQK;  // [t][v]; with V > K it runs on into the k tile (P), which is consumed as well
#pragma unroll
  for (int tv = 0; tv < TV; ++tv)
#pragma unroll
    for (int a4 = 0; a4 < 4; ++a4) {
      v4 x;
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) x[b4] = (T)acc[tv][4 * a4 + b4];
      *(v4*)&sO[trow * LDO + (cw * TV + tv) * 32 + 8 * a4 + 4 * (lane >> 5)] = x;
    }
  __syncthreads();
  {
    constexpr int CV = V / 8;
    T* op = (T*)p.o + (row0 * H + hh) * (int64_t)V;
    for (int e = tid; e < BT * CV; e += 256) {
      const int row = e / CV, c8 = (e % CV) * 8;
      if (row < L) *(v8*)(op + (int64_t)row * H * V + c8) = *(const v8*)&sO[row * LDO + c8];
    }
  }
}

template <typename T>
int launch_wy(const WyParams& p, int K, int V, dim3 grid, hipStream_t st) {
#define FLA_CASE(KK, VV)                                                                \
  if (K == KK && V == VV) {                                                             \
    hipLaunchKernelGGL((gdr_fwd_wy_kernel<T, KK, VV>), grid, dim3(256), 0, st, p);      \
    FLA_CHECK_LAUNCH();                                                                 \
    return FLA_OK;                                                                      \
  }
  FLA_CASE(64, 64)
  FLA_CASE(128, 128)
  FLA_CASE(64, 128)
  FLA_CASE(128, 64)
  FLA_CASE(256, 64)
  FLA_CASE(256, 128)
#undef FLA_CASE
  return FLA_E_UNSUPPORTED;
}

template <typename T>
int launch_dh(const DHParams& p, int K, int h_dtype, int h_layout, hipStream_t st) {
  int64_t total = (int64_t)(p.V / 32) * p.N * p.H;
  if (total == 0) return FLA_OK;
  FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  dim3 grid((unsigned)total), block(256);
  int hl = (h_layout == FLA_H_FRAGMENT) ? 1 : (h_layout == FLA_H_FRAGMENT_T) ? 3 : (h_dtype == FLA_F32 ? 2 : 0);
#define FLA_CASE(KK, HL)                                                           \
  if (K == KK && hl == HL) {                                                       \
    if (p.v_new) hipLaunchKernelGGL((gdr_fwd_h_kernel<T, KK, HL, true>), grid, block, 0, st, p);   \
    else hipLaunchKernelGGL((gdr_fwd_h_kernel<T, KK, HL, false>), grid, block, 0, st, p);          \
    FLA_CHECK_LAUNCH();                                                            \
    return FLA_OK;                                                                 \
  }
  FLA_CASE(64, 0) FLA_CASE(64, 1) FLA_CASE(64, 2) FLA_CASE(64, 3)
  FLA_CASE(128, 0) FLA_CASE(128, 1) FLA_CASE(128, 2) FLA_CASE(128, 3)
  FLA_CASE(256, 0) FLA_CASE(256, 1) FLA_CASE(256, 2) FLA_CASE(256, 3)
#undef FLA_CASE
  return FLA_E_UNSUPPORTED;
}

template <typename T>
int launch_do(const DOParams& p, int K, int V, dim3 grid, hipStream_t st) {
#define FLA_CASE(KK, VV)                                                                \
  if (K == KK && V == VV) {                                                             \
    hipLaunchKernelGGL((chunk_fwd_o_kernel<T, KK, VV>), grid, dim3(256), 0, st, p);     \
    FLA_CHECK_LAUNCH();                                                                 \
    return FLA_OK;                                                                      \
  }
  FLA_CASE(64, 64)
  FLA_CASE(128, 128)
  FLA_CASE(64, 128)
  FLA_CASE(128, 64)
  FLA_CASE(256, 64)
  FLA_CASE(256, 128)
#undef FLA_CASE
  return FLA_E_UNSUPPORTED;
}

template <typename T>
int launch_prep(const PrepParams& p, int K, dim3 chunk_grid_, hipStream_t st) {
  // (chunk, head) items, head-fastest; as many workgroups as are resident at once, each walking its share of the items
  const int64_t total = (int64_t)chunk_grid_.x * chunk_grid_.y;
  const int64_t resident = (p.w ? kPrepResidentKeep : kPrepResident) * kNumCUs;
  dim3 grid((unsigned)(total < resident ? total : resident));
  if (p.l2_eps >= 0.f) {
    if (p.w) return FLA_E_UNSUPPORTED;
    if (K == 64) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 64, false, true>), grid, dim3(256), 0, st, p, total);
    else if (K == 128) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 128, false, true>), grid, dim3(256), 0, st, p, total);
    else return FLA_E_UNSUPPORTED;
  } else if (p.w) {
    if (K == 64) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 64, true>), grid, dim3(256), 0, st, p, total);
    else if (K == 128) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 128, true>), grid, dim3(256), 0, st, p, total);
    else return FLA_E_UNSUPPORTED;
  } else {
    if (K == 64) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 64, false>), grid, dim3(256), 0, st, p, total);
    else if (K == 128) hipLaunchKernelGGL((gdr_fwd_prep_kernel<T, 128, false>), grid, dim3(256), 0, st, p, total);
    else return FLA_E_UNSUPPORTED;
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

static int gdr_fwd_prep_impl(const void* k, const float* beta, const float* g, int g_is_cumsum,
                             float* g_cumsum_out, void* AT, void* w, void* Aw, const int64_t* offsets,
                             const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T, int64_t H,
                             int64_t K, float l2_eps, fla_stream_t stream, float* rk_out = nullptr) {
  FLA_REQUIRE(k && beta && AT, FLA_E_INVALID);
  FLA_REQUIRE((l2_eps >= 0.f) == (rk_out != nullptr), FLA_E_INVALID);
  FLA_REQUIRE((w == nullptr) == (Aw == nullptr), FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)AT | (uintptr_t)w | (uintptr_t)Aw) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  PrepParams p{k, beta, g, g_is_cumsum, g_cumsum_out, AT, offsets, indices, T, (int)H, ntfix, w, Aw, l2_eps, rk_out};
  if (qkv_dtype == FLA_BF16) return launch_prep<bf16>(p, (int)K, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_prep<f16>(p, (int)K, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_gdr_fwd_prep(const void* k, const float* beta, const float* g, int g_is_cumsum,
                                float* g_cumsum_out, void* AT, void* w, void* Aw, const int64_t* offsets,
                                const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T, int64_t H,
                                int64_t K, fla_stream_t stream) {
  return gdr_fwd_prep_impl(k, beta, g, g_is_cumsum, g_cumsum_out, AT, w, Aw, offsets, indices, NT, qkv_dtype, B, T,
                           H, K, -1.f, stream);
}

extern "C" int fla_gdr_fwd_prep_l2norm(const void* k, const float* beta, const float* g, int g_is_cumsum,
                                       float* g_cumsum_out, void* AT, float* k_rstd_out, const int64_t* offsets,
                                       const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T,
                                       int64_t H, int64_t K, float eps, fla_stream_t stream) {
  FLA_REQUIRE(eps >= 0.f && k_rstd_out, FLA_E_INVALID);
  return gdr_fwd_prep_impl(k, beta, g, g_is_cumsum, g_cumsum_out, AT, nullptr, nullptr, offsets, indices, NT,
                           qkv_dtype, B, T, H, K, eps, stream, k_rstd_out);
}

extern "C" int fla_gdr_fwd_wy(const void* k, const void* v, const float* beta, const float* g_cumsum, void* w, void* u,
                              void* Aw, void* Au, const int64_t* offsets, const int64_t* indices, int64_t NT,
                              int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                              fla_stream_t stream) {
  FLA_REQUIRE(k && v && beta && w, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)w | (uintptr_t)u | (uintptr_t)Aw | (uintptr_t)Au) % 16 == 0,
              FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  WyParams p{k, v, beta, g_cumsum, w, u, Aw, Au, offsets, indices, T, (int)H, ntfix, nullptr, nullptr};
  if (qkv_dtype == FLA_BF16) return launch_wy<bf16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_wy<f16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_fwd_recompute_w_u(const void* k, const void* v, const float* beta, const void* Aw, const void* Au,
                                     void* w, void* u, const int64_t* offsets, const int64_t* indices, int64_t NT,
                                     int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                     fla_stream_t stream) {
  FLA_REQUIRE(k && v && beta && Aw && Au && w && u, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)w | (uintptr_t)u | (uintptr_t)Aw | (uintptr_t)Au) % 16 == 0,
              FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  WyParams p{k, v, beta, nullptr, w, u, nullptr, nullptr, offsets, indices, T, (int)H, ntfix, Aw, Au};
  if (qkv_dtype == FLA_BF16) return launch_wy<bf16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_wy<f16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gated_delta_rule_fwd_h(const void* k, const void* w, const void* u, const float* g_cumsum,
                                                const float* h0, void* h, void* v_new, float* ht,
                                                const int64_t* offsets, const int64_t* chunk_offsets, int qkv_dtype,
                                                int h_dtype, int h_layout, int64_t B, int64_t T, int64_t H, int64_t K,
                                                int64_t V, int64_t N, fla_stream_t stream) {
  FLA_REQUIRE(k && w && u, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE(V % 32 == 0 && V <= 1024, FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(chunk_offsets != nullptr && B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  FLA_REQUIRE(h_layout == FLA_H_ROW_MAJOR || h_layout == FLA_H_FRAGMENT || h_layout == FLA_H_FRAGMENT_T,
              FLA_E_INVALID);
  if (h_layout != FLA_H_ROW_MAJOR) FLA_REQUIRE(h_dtype == qkv_dtype, FLA_E_UNSUPPORTED);
  else FLA_REQUIRE(h_dtype == qkv_dtype || h_dtype == FLA_F32, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)w | (uintptr_t)u | (uintptr_t)h | (uintptr_t)v_new) % 16 == 0,
              FLA_E_ALIGNMENT);
  DHParams p{k, w, u, g_cumsum, h0, h, v_new, ht, offsets, chunk_offsets, T, (int)H, (int)V, (int)N, nullptr};
  if (qkv_dtype == FLA_BF16) return launch_dh<bf16>(p, (int)K, h_dtype, h_layout, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_dh<f16>(p, (int)K, h_dtype, h_layout, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gated_delta_rule_fwd_h_both(const void* k, const void* w, const void* u,
                                                     const float* g_cumsum, const float* h0, void* h_frag,
                                                     void* h_frag_t, void* v_new, float* ht, const int64_t* offsets,
                                                     const int64_t* chunk_offsets, int qkv_dtype, int64_t B, int64_t T,
                                                     int64_t H, int64_t K, int64_t V, int64_t N, fla_stream_t stream) {
  FLA_REQUIRE(k && w && u && h_frag && h_frag_t, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE(V % 32 == 0 && V <= 1024, FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(chunk_offsets != nullptr && B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)w | (uintptr_t)u | (uintptr_t)h_frag | (uintptr_t)h_frag_t |
               (uintptr_t)v_new) % 16 == 0, FLA_E_ALIGNMENT);
  DHParams p{k, w, u, g_cumsum, h0, h_frag_t, v_new, ht, offsets, chunk_offsets, T, (int)H, (int)V, (int)N, h_frag};
  if (qkv_dtype == FLA_BF16) return launch_dh<bf16>(p, (int)K, qkv_dtype, FLA_H_FRAGMENT_T, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_dh<f16>(p, (int)K, qkv_dtype, FLA_H_FRAGMENT_T, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_fwd_o(const void* q, const void* k, const void* v, const float* g_cumsum, const void* h,
                               void* o, const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                               int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, float scale,
                               fla_stream_t stream) {
  FLA_REQUIRE(q && k && v && h && o, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)h | (uintptr_t)o) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  DOParams p{q, k, v, g_cumsum, h, o, offsets, indices, T, (int)H, ntfix, scale};
  if (qkv_dtype == FLA_BF16) return launch_do<bf16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_do<f16>(p, (int)K, (int)V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}
