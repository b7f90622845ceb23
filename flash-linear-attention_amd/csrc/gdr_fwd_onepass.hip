// Gated-delta-rule forward in ONE launch for gfx950: the chunk-local prefix sum of the gate, the scaled
// K K^T blocks and their triangular solve, the state scan and the output in a single pass over q, k, v.
// Nothing but o and the final state is written; no per-chunk tile crosses HBM.
//
// The workgroup is the one of gdr_fwd_scan_kernel (gdr_fwd_fused.hip): 8 waves per (sequence, head, 64 value
// columns), waves 4-7 staging q, k, v and the per-row scalars of the coming chunks, waves 0-3 each carrying 16
// value columns of the fp32 state in accumulators, one LDS-only barrier per chunk.  What differs is where the
// WY operator of a chunk comes from.  With M = strict_lower(diag(beta) K K^T * Gamma), Gamma_ij = e^{gamma_i -
// gamma_j} (fla/ops/gated_delta_rule/wy_fast.py:150-208), the scan needs
//     v_new = (I + M)^-1 diag(beta) (v - e^{gamma} * (k h))          (= u - e^{gamma} (w h), chunk_delta_h.py:101-110)
// The two-launch forward reads the 64x64 matrix (I + M)^-1 diag(beta) that fla_gdr_fwd_prep inverted.  Here the
// matrix waves solve the triangular system block by block instead, which needs no 64x64 inverse and therefore
// no exchange between waves inside a chunk period: in 16-row blocks,
//     y_i = D_i (beta_i r_i - sum_{j<i} M_ij y_j),   D_i = (I + M_ii)^-1   (16x16, unit lower triangular)
// While the workgroup works on chunk c, matrix wave w forms for chunk c + 1 (whose k rows are in LDS a chunk
// period early for the scores anyway): the diagonal block M_ww on the matrix pipe, D_w by forward substitution
// in fp32 (one column per lane, rows broadcast from a wave-private LDS scratch), one or two of the six
// off-diagonal blocks M_ij, and its share of the score blocks; all of it is published by the barrier that ends
// the period.  The solve is then eight dependent 16x16x32 products per wave and chunk instead of the six of the
// precomputed inverse.
#include "chunk_common.h"

namespace {

struct GdrOnepassParams {
  const void* q;
  const void* k;
  const void* v;
  const float* g;      // raw per-head log-gate [rows, H], or NULL
  const float* beta;   // [rows, H]
  const float* h0;
  void* o;
  float* ht;
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  const int64_t* seq_order;  // sequence ids, longest first (or NULL)
  int64_t T;
  int H, V, N;
  float scale;
  float l2_eps;     // L2N: q and k rows are l2-normalised (x / sqrt(sum x^2 + l2_eps)) as they are staged
};

// A operand (16 rows x 32 contraction indices) that holds one 16x16 block of a packed triangular tile in the
// first four indices of each group and zeros in the second four: the block times the first half of the other
// operand.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag_blk(const T* tile, int blk, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef __attribute__((address_space(3))) const volatile v4 lds_v4;
  const v4 lo = *(lds_v4*)(tile + blk * 256 + (lane & 15) * 16 + 4 * (lane >> 4));
  const v4 hi = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Two stacked 16-row accumulator tiles (or one and zeros) as the operand contracting over their rows.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 pack_rows(f32x4 a, f32x4 b) {
  typename Elem<T>::v8 x;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    x[r] = (T)a[r];
    x[4 + r] = (T)b[r];
  }
  return x;
}

constexpr int LDL = 20;   // row pitch (floats) of the wave-private 16x16 scratch of the substitution

template <typename T, int K, bool L2N>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gdr_fwd_onepass_kernel(
    GdrOnepassParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int BV = 64;
  constexpr int RV = BV / 16;   // v, o: rows of a staging lane's 4-column piece
  typedef T rvv __attribute__((ext_vector_type(RV)));
  constexpr int LDR = K + 8;  // pitch of the row-major k and q tiles
  constexpr int KS = K / 32;  // 32-wide contraction slices of the state
  constexpr int KT = K / 16;  // 16-row state tiles per matrix wave
  // k, q and the per-row scalars of a chunk are in LDS one chunk period before the rest of it (three buffers,
  // chunk modulo 3): the scores and the WY blocks of chunk c + 1 are formed from them while chunk c is in work.
  __shared__ __attribute__((aligned(16))) T sK[3][BT * LDR];     // k    [t][k]
  __shared__ __attribute__((aligned(16))) T sQ[3][BT * LDR];     // q    [t][k]
  __shared__ __attribute__((aligned(16))) T sVt[2][BV * LDT];    // v^T  [v][t], later o^T
  __shared__ __attribute__((aligned(16))) T sTB[2][kTriElems];   // D_i on the diagonal, M_ij below (packed blocks)
  __shared__ __attribute__((aligned(16))) T sP[2][kTriElems];    // Aqk, same packing
  __shared__ __attribute__((aligned(16))) float sGam[3][BT];     // gamma_t
  __shared__ __attribute__((aligned(16))) float sEg[3][BT];      // e^{gamma_t}
  __shared__ __attribute__((aligned(16))) float sEd[3][BT];      // e^{gamma_last - gamma_t}
  __shared__ __attribute__((aligned(16))) float sBeta[3][BT];    // beta_t (zero past the end of a short chunk)
  __shared__ __attribute__((aligned(16))) float sL[4][16 * LDL]; // per matrix wave: its diagonal block, fp32
  __shared__ float sDec[3];                                      // e^{gamma_last}

  const int tid = threadIdx.x, lane = tid & 63;
  // wave-uniform by construction: keeps the role split and the barriers on scalar branches
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = p.H, V = p.V;
  const int nvb = V / BV;
  const ScanItem wi = scan_item(nvb);
  const int vb = wi.slab;
  const int hh = (int)(wi.item % H);
  const int n = p.seq_order ? (int)p.seq_order[wi.item / H] : (int)(wi.item / H);
  const int nh = n * H + hh;
  const int vbase = vb * BV;
  SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int nchunks = (int)((sp.len + BT - 1) / BT);

  // Aqk = scale tril(q k^T * Gamma) of the chunk whose tiles are in buffer b3, shared out over waves 0-3 by 16x16
  // block: a block is computed transposed (k rows against q rows), which leaves every lane with four adjacent
  // entries of one row - an 8-byte piece of the packed tile frag_tri() reads.  Rows past the end of a short
  // chunk are zero in the q and k tiles.
  auto compute_p = [&](int b3, int pb) __attribute__((always_inline)) {
    const T* Kr = sK[b3];
    const T* Q = sQ[b3];
    T* Po = sP[pb];
    const int c = lane & 15, g = lane >> 4;
    // (row block, column block) of this wave's blocks, a nibble each, first in the low bits
    const int tis = wave == 0 ? 0x33 : wave == 1 ? 0x33 : wave == 2 ? 0x222 : 0x011;
    const int tjs = wave == 0 ? 0x10 : wave == 1 ? 0x32 : wave == 2 ? 0x210 : 0x010;
    const int cnt = wave < 2 ? 2 : 3;
    v8 fq[KS];
    int cur = -1;
#pragma unroll
    for (int n2 = 0; n2 < 3; ++n2) {
      if (n2 < cnt) {
        const int ti = (tis >> (4 * n2)) & 15, tj = (tjs >> (4 * n2)) & 15;
        if (ti != cur) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) fq[ks] = frag16<T>(Q, LDR, 16 * ti, 32 * ks, lane);
          cur = ti;
        }
        f32x4 sc = zero4();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) sc = Elem<T>::mfma16(frag16<T>(Kr, LDR, 16 * tj, 32 * ks, lane), fq[ks], sc);
        const float gi = sGam[b3][16 * ti + c];
        const f32x4 gj = *(const f32x4*)&sGam[b3][16 * tj + 4 * g];
        v4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          o[r] = (T)((ti > tj || 4 * g + r <= c) ? p.scale * sc[r] * __expf(gi - gj[r]) : 0.f);
        *(v4*)&Po[(ti * (ti + 1) / 2 + tj) * 256 + c * 16 + 4 * g] = o;
      }
    }
  };

  // The WY blocks of the chunk whose tiles are in buffer b3: M = strict_lower(diag(beta) k k^T * Gamma).  This wave's
  // one or two off-diagonal blocks M_ij go to the packed tile as they are; its diagonal block M_ww goes to the
  // wave's fp32 scratch, is inverted there, D_w = (I + M_ww)^-1, and D_w takes the diagonal place of the tile.
  auto compute_tb = [&](int b3, int pb) __attribute__((always_inline)) {
    const T* Kr = sK[b3];
    T* Tb = sTB[pb];
    const int c = lane & 15, g = lane >> 4;
    // waves 0 and 1 form two score blocks each and take two off-diagonal blocks, waves 2 and 3 (three score
    // blocks) one: (1,0) (2,0) | (2,1) (3,0) | (3,1) | (3,2)
    const int tis = wave == 0 ? 0x21 : wave == 1 ? 0x32 : 0x3;
    const int tjs = wave == 0 ? 0x00 : wave == 1 ? 0x01 : wave == 2 ? 0x1 : 0x2;
    const int cnt = wave < 2 ? 2 : 1;
#pragma unroll
    for (int n2 = 0; n2 < 2; ++n2) {
      if (n2 < cnt) {
        const int ti = (tis >> (4 * n2)) & 15, tj = (tjs >> (4 * n2)) & 15;
        f32x4 sc = zero4();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          sc = Elem<T>::mfma16(frag16<T>(Kr, LDR, 16 * tj, 32 * ks, lane), frag16<T>(Kr, LDR, 16 * ti, 32 * ks, lane), sc);
        const float gi = sGam[b3][16 * ti + c], bi = sBeta[b3][16 * ti + c];
        const f32x4 gj = *(const f32x4*)&sGam[b3][16 * tj + 4 * g];
        v4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (T)(bi * sc[r] * __expf(gi - gj[r]));
        *(v4*)&Tb[(ti * (ti + 1) / 2 + tj) * 256 + c * 16 + 4 * g] = o;
      }
    }
    {
      const int ti = wave;
      f32x4 sc = zero4();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const v8 f = frag16<T>(Kr, LDR, 16 * ti, 32 * ks, lane);
        sc = Elem<T>::mfma16(f, f, sc);
      }
      // lane (c, g) holds entries (i = c, j = 4 g + r) of the block
      const float gi = sGam[b3][16 * ti + c], bi = sBeta[b3][16 * ti + c];
      const f32x4 gj = *(const f32x4*)&sGam[b3][16 * ti + 4 * g];
      f32x4 m;
#pragma unroll
      for (int r = 0; r < 4; ++r) m[r] = (4 * g + r < c) ? bi * sc[r] * __expf(gi - gj[r]) : 0.f;
      float* L = sL[wave];
      *(f32x4*)&L[c * LDL + 4 * g] = m;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's own writes, read back below
      // X = (I + L)^-1 by forward substitution, one column per lane (the four rows of 16 lanes work alike):
      // x_i = [i == col] - sum_{j<i} L_ij x_j, the rows of L broadcast from the scratch
      float x[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float row[16];
#pragma unroll
        for (int q4 = 0; 4 * q4 < i; ++q4) *(f32x4*)&row[4 * q4] = *(const f32x4*)&L[i * LDL + 4 * q4];
        float s = (i == c) ? 1.f : 0.f;
#pragma unroll
        for (int j = 0; j < i; ++j) s = fmaf(-row[j], x[j], s);
        x[i] = s;
        if ((i & 3) == 3) __builtin_amdgcn_sched_barrier(0);   // keeps the row loads of later rows from piling up in registers
      }
      if (g == 0) {
        T* D = Tb + (ti * (ti + 1) / 2 + ti) * 256 + c;
#pragma unroll
        for (int i = 0; i < 16; ++i) D[i * 16] = (T)x[i];
      }
    }
  };

  if (wave >= 4) {
    // =========================== staging waves ===========================
    if (nchunks == 0) return;
    const int st = tid - 256;
    constexpr int C8 = K / 8, NPW = BT * C8 / 256;           // 16-byte pieces per row / per lane (q)
    const int urg = st / (BV / 4), uc4 = (st % (BV / 4)) * 4;   // v, o: a lane owns RV rows x 4 columns
    const uint32_t HK = (uint32_t)H * K, HV = (uint32_t)H * V;
    auto q_row = [&](int e) { return e / C8; };
    auto q_col = [&](int e) { return (e % C8) * 8; };
    struct Regs {
      v8 q[NPW], k[NPW];
      v4 v[RV];
      uint32_t g, beta;  // fp32 bits: this lane's row
    };
    // The steady state carries no address arithmetic: byte offsets of this lane's pieces from the
    // chunk's first row are computed once and the chunk base pointers advance by constant strides.
    uint32_t offq[NPW], offv[RV];
#pragma unroll
    for (int i = 0; i < NPW; ++i) offq[i] = 2 * ((uint32_t)q_row(st + 256 * i) * HK + q_col(st + 256 * i));
#pragma unroll
    for (int i = 0; i < RV; ++i) offv[i] = 2 * ((uint32_t)(urg * RV + i) * HV + uc4);
    const uint32_t offg = 4 * (uint32_t)lane * H;
    const int64_t row00 = sp.bos * H + hh;
    const char* lq = (const char*)p.q + row00 * K * 2;
    const char* lk = (const char*)p.k + row00 * K * 2;
    const char* lv = (const char*)p.v + (row00 * V + vbase) * 2;
    // The per-row loads are unconditional (a load under a branch would make the wave drain its whole load
    // queue at the join); without gates the gate load reads the beta row and the bits are masked to zero.
    const uint32_t gmask = p.g ? 0xffffffffu : 0u;
    const char* lb = (const char*)p.beta + row00 * 4;
    const char* lg = p.g ? (const char*)p.g + row00 * 4 : lb;
    char* so = (char*)p.o + (row00 * V + vbase) * 2;
    const int64_t strk = (int64_t)BT * HK * 2, strv = (int64_t)BT * HV * 2;
    const int64_t strg = (int64_t)BT * H * 4;
    const int Llast = (int)(sp.len - (int64_t)(nchunks - 1) * BT);
    // Every memory operation of the steady state is unconditional: the wait counts the compiler places
    // in front of a register's first use then count the loads of the other register sets and the output
    // stores issued since as still in flight.  Rows past the end of a sequence's last chunk are redirected to
    // its last row by one unsigned minimum per load (zeroed before use), and past the last chunk the pointers
    // stay on it.
    const uint32_t limq_full = 2 * ((uint32_t)(BT - 1) * HK), limq_last = 2 * ((uint32_t)(Llast - 1) * HK);
    const uint32_t limv_full = 2 * ((uint32_t)(BT - 1) * HV), limv_last = 2 * ((uint32_t)(Llast - 1) * HV);
    const uint32_t colq = 2 * (uint32_t)q_col(st), colv = 2 * (uint32_t)uc4;
    // k, q and the per-row scalars run one chunk ahead of v: register set j holds k, q, g, beta of chunk j + 1 and
    // v of chunk j.
    int lcq = 0, lcv = 0;  // chunks the two groups of load pointers are on
    auto load_kq = [&](Regs& R) __attribute__((always_inline)) {
      const bool last = lcq >= nchunks - 1;
      const uint32_t limq = (last ? limq_last : limq_full) + colq;
      const uint32_t limg = 4 * (uint32_t)((last ? Llast : BT) - 1) * H;
#pragma unroll
      for (int i = 0; i < NPW; ++i) {
        const uint32_t o = offq[i] < limq ? offq[i] : limq;
        R.q[i] = *(const v8*)(lq + o);
        R.k[i] = *(const v8*)(lk + o);
      }
      const uint32_t og = offg < limg ? offg : limg;
      R.g = *(const uint32_t*)(lg + og);
      R.beta = *(const uint32_t*)(lb + og);
      if (lcq + 1 < nchunks) {
        lq += strk;
        lk += strk;
        lg += strg;
        lb += strg;
      }
      ++lcq;
    };
    auto load = [&](Regs& R) __attribute__((always_inline)) {
      const bool last = lcv >= nchunks - 1;
      const uint32_t limv = (last ? limv_last : limv_full) + colv;
#pragma unroll
      for (int i = 0; i < RV; ++i) R.v[i] = *(const v4*)(lv + (offv[i] < limv ? offv[i] : limv));
      if (lcv + 1 < nchunks) lv += strv;
      ++lcv;
      load_kq(R);
    };
    // LDS destinations of this lane (element offsets inside a tile)
    int dq[NPW], dv[4];
#pragma unroll
    for (int i = 0; i < NPW; ++i) dq[i] = q_row(st + 256 * i) * LDR + q_col(st + 256 * i);
#pragma unroll
    for (int j = 0; j < 4; ++j) dv[j] = (uc4 + j) * LDT + swz_t(uc4 + j, urg * RV);
    // Rows past the end of a sequence's last, short chunk are zeroed on the way to LDS.  (What a set holds
    // beyond the last chunk is that chunk again; nothing reads the buffer it goes to.)
    int wq = 0, wq3 = 0;  // next chunk whose k, q, per-row scalars are written, and its buffer
    auto write_kq = [&](Regs& R) __attribute__((always_inline)) {
      const int Lc = wq >= nchunks - 1 ? Llast : BT;
      if (wq == nchunks - 1 && Llast < BT) {
#pragma unroll
        for (int i = 0; i < NPW; ++i)
          if (q_row(st + 256 * i) >= Llast)
#pragma unroll
            for (int j = 0; j < 8; ++j) R.q[i][j] = R.k[i][j] = (T)0.f;
      }
      if constexpr (L2N) {
#pragma unroll
        for (int i = 0; i < NPW; ++i) {
          R.q[i] = l2norm_piece<T, K / 8>(R.q[i], p.l2_eps);
          R.k[i] = l2norm_piece<T, K / 8>(R.k[i], p.l2_eps);
        }
      }
#pragma unroll
      for (int i = 0; i < NPW; ++i) *(v8*)&sQ[wq3][dq[i]] = R.q[i];
#pragma unroll
      for (int i = 0; i < NPW; ++i) *(v8*)&sK[wq3][dq[i]] = R.k[i];
      if (wave == 4) {
        // the chunk-local inclusive prefix sum of the gate over the 64 rows: a DPP scan inside each row of 16
        // lanes plus the totals of the earlier rows; rows past the end of a short chunk add zero, so they carry
        // the last valid row's sum (and beta = 0 there)
        const bool ok = lane < Lc;
        const float x = row_prefix16(ok ? __uint_as_float(R.g & gmask) : 0.f);
        const float t0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 15));
        const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 31));
        const float t2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 47));
        const int r = lane >> 4;
        const float gam = x + (r >= 1 ? t0 : 0.f) + (r >= 2 ? t1 : 0.f) + (r >= 3 ? t2 : 0.f);
        const float glast = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gam), 63));
        sGam[wq3][lane] = gam;
        sEg[wq3][lane] = __expf(gam);
        sEd[wq3][lane] = __expf(glast - gam);
        sBeta[wq3][lane] = ok ? __uint_as_float(R.beta) : 0.f;
        if (lane == 0) sDec[wq3] = __expf(glast);
      }
      ++wq;
      wq3 = wq3 == 2 ? 0 : wq3 + 1;
    };
    int wc = 0;  // next chunk whose v is written
    auto write = [&](Regs& R) __attribute__((always_inline)) {
      const int b = wc & 1;
      if (wc == nchunks - 1 && Llast < BT) {
#pragma unroll
        for (int i = 0; i < RV; ++i)
          if (urg * RV + i >= Llast) R.v[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rvv vc;
#pragma unroll
        for (int i = 0; i < RV; ++i) vc[i] = R.v[i][j];
        *(rvv*)&sVt[b][dv[j]] = vc;
      }
      ++wc;
      write_kq(R);
    };
    // The matrix waves left o^T of a chunk where v^T of that chunk was; each lane reads back
    // exactly the addresses it writes in write(), so the tile can be refilled right after.
    int oc = 0;  // next chunk whose output is stored
    auto store_o = [&](auto maybe_last) __attribute__((always_inline)) {
      const int b = oc & 1;
      rvv x[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) x[j] = *(const rvv*)&sVt[b][dv[j]];
      bool full = true;
      if constexpr (decltype(maybe_last)::value) full = oc != nchunks - 1 || Llast == BT;
      if (full) {
#pragma unroll
        for (int i = 0; i < RV; ++i) *(v4*)(so + offv[i]) = v4{x[0][i], x[1][i], x[2][i], x[3][i]};
      } else {
#pragma unroll
        for (int i = 0; i < RV; ++i)
          if (urg * RV + i < Llast) *(v4*)(so + offv[i]) = v4{x[0][i], x[1][i], x[2][i], x[3][i]};
      }
      so += strv;
      ++oc;
    };
    // Three register sets: a set is loaded three iterations before it is written to LDS, so its loads have two
    // chunk periods to land.  Iteration c (the matrix waves work on chunk c and prepare chunk c + 1) stores
    // the output of chunk c-1, writes set c + 1 (k, q, scalars of chunk c + 2; v of chunk c + 1) and loads set
    // c + 4 into the registers just emptied; sets rotate R1, R2, R0.  The steady-state loop runs whole rotations
    // over the iterations that touch neither the first nor the last chunk and leaves only at its latch.
    constexpr std::true_type any_chunk{};
    constexpr std::false_type inner_chunk{};
    Regs R0, R1, R2;
    load_kq(R0);              // k, q, scalars of chunk 0 on their own
    write_kq(R0);
    load(R0);
    load(R1);
    load(R2);
    lds_barrier();            // the scores and WY blocks of chunk 0 can be formed
    write(R0);
    load(R0);
    lds_barrier();
    if (nchunks > 1) {
      write(R1);              // iteration 0
      load(R1);
      lds_barrier();
      auto iter = [&](Regs& R) __attribute__((always_inline)) {
        store_o(inner_chunk);
        write(R);
        load(R);
        lds_barrier();
      };
      const int inner = nchunks > 3 ? nchunks - 3 : 0;   // iterations 1 .. nchunks - 3
      for (int trips = inner / 3; trips > 0; --trips) {
        iter(R2);
        iter(R0);
        iter(R1);
      }
      const int rem = inner % 3;
      if (rem >= 1) iter(R2);
      if (rem >= 2) iter(R0);
      if (nchunks > 2) {      // iteration nchunks - 2 writes the last chunk's v
        store_o(inner_chunk);
        if (rem == 0) write(R2);
        else if (rem == 1) write(R0);
        else write(R1);
        lds_barrier();
      }
      store_o(inner_chunk);   // iteration nchunks - 1: the output of chunk nchunks - 2
    }
    lds_barrier();
    store_o(any_chunk);
  } else {
    // =========================== matrix waves ===========================
    const int cb = 16 * wave;  // first of this wave's 16 columns within the slab
    const int c = lane & 15, g = lane >> 4;
    f32x4 acc[KT];  // acc[kt][r] = h[16 kt + 4 g + r][cb + c]
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      acc[kt] = zero4();
      if (p.h0) {
        const float* h0p = p.h0 + (int64_t)nh * K * V + vbase + cb + c;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[kt][r] = h0p[(int64_t)(16 * kt + 4 * g + r) * V];
      }
    }
    if (nchunks > 0) {
      lds_barrier();
      compute_p(0, 0);
      compute_tb(0, 0);
      lds_barrier();
      int b3 = 0;   // ci modulo 3
      for (int ci = 0; ci < nchunks; ++ci) {
        const int b = ci & 1;
        const int n3 = b3 == 2 ? 0 : b3 + 1;
        const T* Kr = sK[b3];
        const T* Q = sQ[b3];
        const T* Tb = sTB[b];
        const T* P = sP[b];
        if (ci + 1 < nchunks) {
          compute_p(n3, b ^ 1);
          compute_tb(n3, b ^ 1);
        }
        const int vrow = cb + c;
        T* vt = &sVt[b][vrow * LDT];
        // LDS reads are issued a group ahead of the MFMAs that consume them; the scheduling
        // fences keep the compiler from sinking them back next to their use.
        v8 fa[2 * KS], fb[2 * KS];
        auto load_kq = [&](int tt, v8* f) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            f[ks] = frag16<T>(Kr, LDR, 16 * tt, 32 * ks, lane);
            f[KS + ks] = frag16<T>(Q, LDR, 16 * tt, 32 * ks, lane);
          }
        };
        auto load_kt = [&](int half, v8* f) {
#pragma unroll
          for (int i = 0; i < KT / 2; ++i)
#pragma unroll
            for (int s = 0; s < 2; ++s) f[2 * i + s] = frag16_tr<T>(Kr, LDR, 16 * (half * (KT / 2) + i), 32 * s, lane);
        };
        load_kq(0, fa);
        load_kq(1, fb);
        __builtin_amdgcn_sched_barrier(0);
        // the state as the other MFMA operand: two stacked accumulators per 32-slice
        v8 hb[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) hb[ks] = pack_rows<T>(acc[2 * ks], acc[2 * ks + 1]);
        f32x4 d[4], oq[4];
        auto mm_kq = [&](int tt, const v8* f) {
          d[tt] = zero4();
          oq[tt] = zero4();
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            d[tt] = Elem<T>::mfma16(f[ks], hb[ks], d[tt]);
            oq[tt] = Elem<T>::mfma16(f[KS + ks], hb[ks], oq[tt]);
          }
        };
        mm_kq(0, fa);
        __builtin_amdgcn_sched_barrier(0);
        load_kq(2, fa);
        __builtin_amdgcn_sched_barrier(0);
        mm_kq(1, fb);
        __builtin_amdgcn_sched_barrier(0);
        load_kq(3, fb);
        __builtin_amdgcn_sched_barrier(0);
        mm_kq(2, fa);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 eg[4], ed[4], bt[4];
        v4 vv[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          eg[tt] = *(const f32x4*)&sEg[b3][16 * tt + 4 * g];
          ed[tt] = *(const f32x4*)&sEd[b3][16 * tt + 4 * g];
          bt[tt] = *(const f32x4*)&sBeta[b3][16 * tt + 4 * g];
          vv[tt] = *(const v4*)(vt + swz_t(vrow, 16 * tt + 4 * g));
        }
        const float dec = sDec[b3];
        // the WY blocks: D_i, the off-diagonal M_i0 on their own and the pairs (M_i0 | M_i1)
        const v8 fD0 = frag_blk<T>(Tb, 0, lane), fD1 = frag_blk<T>(Tb, 2, lane), fD2 = frag_blk<T>(Tb, 5, lane),
                 fD3 = frag_blk<T>(Tb, 9, lane);
        const v8 fM10 = frag_blk<T>(Tb, 1, lane), fM2 = frag_tri<T>(Tb, 2, 0, lane), fM3 = frag_tri<T>(Tb, 3, 0, lane),
                 fM32 = frag_blk<T>(Tb, 8, lane);
        __builtin_amdgcn_sched_barrier(0);
        mm_kq(3, fb);
        __builtin_amdgcn_sched_barrier(0);
        v8 fp[6];
        fp[0] = frag_tri<T>(P, 0, 0, lane);
        fp[1] = frag_tri<T>(P, 1, 0, lane);
        fp[2] = frag_tri<T>(P, 2, 0, lane);
        fp[3] = frag_tri<T>(P, 2, 1, lane);
        fp[4] = frag_tri<T>(P, 3, 0, lane);
        fp[5] = frag_tri<T>(P, 3, 1, lane);
        __builtin_amdgcn_sched_barrier(0);
        // rhs = beta (v - e^{gamma} (k h)), block by block; y = (I + M)^-1 rhs by block forward substitution
        f32x4 rhs[4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
          for (int r = 0; r < 4; ++r) rhs[tt][r] = bt[tt][r] * ((float)vv[tt][r] - d[tt][r] * eg[tt][r]);
        const f32x4 z4 = zero4();
        f32x4 vn[4];
        vn[0] = Elem<T>::mfma16(fD0, pack_rows<T>(rhs[0], z4), z4);
        {
          const f32x4 t = Elem<T>::mfma16(fM10, pack_rows<T>(vn[0], z4), z4);
          f32x4 x;
#pragma unroll
          for (int r = 0; r < 4; ++r) x[r] = rhs[1][r] - t[r];
          vn[1] = Elem<T>::mfma16(fD1, pack_rows<T>(x, z4), z4);
        }
        const v8 y01 = pack_rows<T>(vn[0], vn[1]);
        {
          const f32x4 t = Elem<T>::mfma16(fM2, y01, z4);
          f32x4 x;
#pragma unroll
          for (int r = 0; r < 4; ++r) x[r] = rhs[2][r] - t[r];
          vn[2] = Elem<T>::mfma16(fD2, pack_rows<T>(x, z4), z4);
        }
        {
          f32x4 t = Elem<T>::mfma16(fM3, y01, z4);
          t = Elem<T>::mfma16(fM32, pack_rows<T>(vn[2], z4), t);
          f32x4 x;
#pragma unroll
          for (int r = 0; r < 4; ++r) x[r] = rhs[3][r] - t[r];
          vn[3] = Elem<T>::mfma16(fD3, pack_rows<T>(x, z4), z4);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_kt(0, fa);     // behind the solve (which needs its registers): the score products below cover the latency
        __builtin_amdgcn_sched_barrier(0);
        v8 vnb[2], vsb[2];  // v_new and its decayed copy as operands contracting over time
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            vnb[tt >> 1][(tt & 1) * 4 + r] = (T)vn[tt][r];
            vsb[tt >> 1][(tt & 1) * 4 + r] = (T)(vn[tt][r] * ed[tt][r]);
            oq[tt][r] *= p.scale * eg[tt][r];
          }
        }
        oq[0] = Elem<T>::mfma16(fp[0], vnb[0], oq[0]);
        oq[1] = Elem<T>::mfma16(fp[1], vnb[0], oq[1]);
        oq[2] = Elem<T>::mfma16(fp[2], vnb[0], oq[2]);
        oq[3] = Elem<T>::mfma16(fp[4], vnb[0], oq[3]);
        oq[2] = Elem<T>::mfma16(fp[3], vnb[1], oq[2]);
        oq[3] = Elem<T>::mfma16(fp[5], vnb[1], oq[3]);
        __builtin_amdgcn_sched_barrier(0);
        load_kt(1, fb);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[kt][r] *= dec;
#pragma unroll
        for (int i = 0; i < KT / 2; ++i)
#pragma unroll
          for (int s = 0; s < 2; ++s) acc[i] = Elem<T>::mfma16(fa[2 * i + s], vsb[s], acc[i]);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          v4 ov;
#pragma unroll
          for (int r = 0; r < 4; ++r) ov[r] = (T)oq[tt][r];
          *(v4*)(vt + swz_t(vrow, 16 * tt + 4 * g)) = ov;
        }
#pragma unroll
        for (int i = 0; i < KT / 2; ++i)
#pragma unroll
          for (int s = 0; s < 2; ++s) acc[KT / 2 + i] = Elem<T>::mfma16(fb[2 * i + s], vsb[s], acc[KT / 2 + i]);
        lds_barrier();
        b3 = n3;
      }
    }
    if (p.ht) {
      float* htp = p.ht + (int64_t)nh * K * V + vbase + cb + c;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) htp[(int64_t)(16 * kt + 4 * g + r) * V] = acc[kt][r];
    }
  }
}

template <typename T>
int launch_onepass(const GdrOnepassParams& p, int K, hipStream_t st) {
  const int64_t nblk = (int64_t)p.N * p.H * (p.V / 64);
  FLA_REQUIRE(nblk <= 0x7fffffffLL / 2, FLA_E_UNSUPPORTED);
  if (nblk == 0) return FLA_OK;
  dim3 grid((unsigned)nblk), block(512);
  const bool l2n = p.l2_eps >= 0.f;
  if (K == 128 && l2n) hipLaunchKernelGGL((gdr_fwd_onepass_kernel<T, 128, true>), grid, block, 0, st, p);
  else if (K == 128) hipLaunchKernelGGL((gdr_fwd_onepass_kernel<T, 128, false>), grid, block, 0, st, p);
  else if (K == 64 && l2n) hipLaunchKernelGGL((gdr_fwd_onepass_kernel<T, 64, true>), grid, block, 0, st, p);
  else if (K == 64) hipLaunchKernelGGL((gdr_fwd_onepass_kernel<T, 64, false>), grid, block, 0, st, p);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

extern "C" int fla_chunk_gated_delta_rule_fwd_onepass(const void* q, const void* k, const void* v, const float* g,
                                                      const float* beta, const float* h0, void* o, float* ht,
                                                      const int64_t* offsets, const int64_t* chunk_offsets,
                                                      const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T,
                                                      int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                                      int qk_l2norm, float l2norm_eps, fla_stream_t stream) {
  FLA_REQUIRE(q && k && v && beta && o, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE(offsets ? B == 1 : N == B, FLA_E_INVALID);
  FLA_REQUIRE(V % 64 == 0 && H <= 0x7fffff, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(!qk_l2norm || l2norm_eps >= 0.f, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) % 16 == 0, FLA_E_ALIGNMENT);
  GdrOnepassParams p{q, k, v, g, beta, h0, o, ht, offsets, chunk_offsets, seq_order, T, (int)H, (int)V, (int)N, scale,
                     qk_l2norm ? l2norm_eps : -1.f};
  if (qkv_dtype == FLA_BF16) return launch_onepass<bf16>(p, (int)K, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_onepass<f16>(p, (int)K, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}
