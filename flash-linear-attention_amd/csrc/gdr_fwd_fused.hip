// One-pass gated-delta-rule forward for gfx950: state scan and output in one launch; neither w, u,
// v_new nor the per-chunk states exist in memory.
//
// Inputs are q, k, v, the chunk-local gate prefix sums gamma and the packed triangular 64x64 tile per
// (chunk, head) that fla_gdr_fwd_prep leaves: Tu = (Aw * Gamma) diag(beta).  One workgroup of 8 waves owns
// one (sequence, head, 64 value columns) and walks the chunks serially:
//   waves 4-7 ("staging")  copy k, q and the gate row of chunk c+2 and the triangular tile of chunk c+1 to
//                          LDS, transpose v of chunk c+1 into a time-contiguous tile, and write the
//                          finished o tile of chunk c-1 to global memory (k is staged row-major only: the
//                          state update reads its transposed operand from that tile with the transposing
//                          LDS load);
//   waves 0-3 ("matrix")   each own 16 value columns of the fp32 state (all K rows, in 16x16
//                          accumulator tiles).  The delta rule is independent per value column, so a
//                          matrix wave exchanges one thing with the others: the gated causal scores
//                          Aqk = s tril(q k^T * Gamma) of the *next* chunk, of whose ten 16x16 blocks each
//                          wave forms two or three while it works on the current chunk (k and q are in LDS
//                          a chunk period early for that; the barrier that ends the period publishes them):
//                            v_new = Tu (v - e^{gamma} * (k h))
//                            o     = s e^{gamma} * (q h) + Aqk v_new
//                            h    <- e^{gamma_last} h + k^T (e^{gamma_last - gamma} * v_new)
//                          (fla/ops/common/chunk_delta_h.py:71-119, chunk_o.py:68-101; v_new equals the
//                          reference's u - e^{gamma} (w h), see gdr_fwd.hip).  State, k h, the residual
//                          and v_new go from accumulators straight back into MFMA operands: the
//                          contraction index of the LDS-side operand is permuted to the accumulator
//                          row order instead.
// Operand tiles are double-buffered (k, q and the gate rows: three buffers) and the two groups meet at one
// barrier per chunk.  The o tile
// takes the place of the v tile it was computed from (same lanes, same addresses), so it needs no
// storage of its own.
// The KEEP instantiation serves a forward pass that will be differentiated: the matrix waves also write
// v_new and the state entering every chunk (FLA_H_FRAGMENT_T order, what the backward kernels read).  Both
// sit in registers as MFMA operands with a lane per value column, four consecutive time rows / key rows
// per register quad; a product with a permuted identity turns them round on the matrix pipe (exact for
// 16-bit values), after which a lane holds four consecutive value columns of one row; a lane-swap between
// the halves (state) or neighbouring rows of 16 lanes (v_new) pairs them up into 16-byte stores (a store
// instruction costs the CU's memory pipeline the same whatever its width, and that pipeline is what bounds
// the scan).
#include "chunk_common.h"

namespace {

// Per chunk and workgroup the kernel reads q, k (16 KB each at K=128), its 64 value columns (8 KB) and
// 5 KB of triangular blocks, and its time follows those bytes: the launch is bound by the rate at which
// data reaches the CUs through L2, both value-column slabs of a head pulling q, k and the tiles.
struct GdrScanParams {
  const void* q;
  const void* k;
  const void* v;
  const void* AT;   // [chunks, H, 10, 16, 16]: Tu
  const float* gam;
  const float* h0;
  void* o;
  float* ht;
  void* v_new;      // KEEP: [rows, H, V]
  void* h_frag_t;   // KEEP: [chunks, H, K*V], FLA_H_FRAGMENT_T
  void* Aqk_out;    // KEEP: [chunks, H, 10, 16, 16], the gated scores (or NULL)
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  const int64_t* seq_order;  // sequence ids, longest first (or NULL)
  int64_t T;
  int H, V, N;
  float scale;
  float l2_eps;     // L2N: q and k are un-normalised; the launch works with x / sqrt(sum x^2 + l2_eps) ...
  const float* rk;  //      ... the factors of k, fp32 [rows, H], come from fla_gdr_fwd_prep_l2norm
};

// Two 4-element results per lane (16-bit after conversion) -> one 8-element vector per lane: lanes 0-31 keep
// their own a and receive a of lane + 32, lanes 32-63 receive b of lane - 32 and keep their own b.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 pair_halves(f32x4 a, f32x4 b) {
  typedef typename Elem<T>::v4 v4;
  typedef typename Elem<T>::v8 v8;
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const u2 ua = __builtin_bit_cast(u2, v4{(T)a[0], (T)a[1], (T)a[2], (T)a[3]});
  const u2 ub = __builtin_bit_cast(u2, v4{(T)b[0], (T)b[1], (T)b[2], (T)b[3]});
  const auto lo = __builtin_amdgcn_permlane32_swap(ua[0], ub[0], false, false);
  const auto hi = __builtin_amdgcn_permlane32_swap(ua[1], ub[1], false, false);
  return __builtin_bit_cast(v8, u4{lo[0], hi[0], lo[1], hi[1]});
}

// The same between neighbouring rows of 16 lanes: even rows keep their own a and receive a of lane + 16,
// odd rows receive b of lane - 16 and keep their own b.
template <typename T>
FLA_DEVICE typename Elem<T>::v8 pair_rows(f32x4 a, f32x4 b) {
  typedef typename Elem<T>::v4 v4;
  typedef typename Elem<T>::v8 v8;
  typedef uint32_t u2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const u2 ua = __builtin_bit_cast(u2, v4{(T)a[0], (T)a[1], (T)a[2], (T)a[3]});
  const u2 ub = __builtin_bit_cast(u2, v4{(T)b[0], (T)b[1], (T)b[2], (T)b[3]});
  const auto lo = __builtin_amdgcn_permlane16_swap(ua[0], ub[0], false, false);
  const auto hi = __builtin_amdgcn_permlane16_swap(ua[1], ub[1], false, false);
  return __builtin_bit_cast(v8, u4{lo[0], hi[0], lo[1], hi[1]});
}

// NMW: matrix waves that carry state, 16 value columns each; the workgroup's slab is 16 NMW columns wide.  Four
// (64 columns) is the form described above; two (32 columns, waves 2-3 only keep the barriers) doubles the number of
// workgroups where 64-column slabs would leave half the CUs without one - a CU is fed at a fixed rate, and a
// 32-column workgroup needs three quarters of the bytes of a 64-column one per chunk.
// L2N: q and k arrive un-normalised (the two l2_norm launches in front of the operator,
// fla/layers/gated_deltanet.py:234-235, are not run).  The rows are not rewritten: with q^ = rq q and k^ = rk k per row,
// every place the normalised rows enter is linear in them, so the factors ride on quantities that are scaled anyway -
// rk on e^{gamma} in front of (k h) and on e^{gamma_last - gamma} in the state update, rq and rk on the rows and
// columns of the score blocks, rq on the scale of the inter-chunk output.  rk comes from the first launch; rq is formed
// by the staging lanes from the q pieces they hold (a row sits in K / 8 adjacent lanes: four packed dot products and
// four lane exchanges per piece).
// DELTA = false: the same scan without the delta rule - v_new = v, no (k h) correction, no Tu tile - which is
// chunk_simple_gla (fla/ops/simple_gla/chunk.py:16-131): h <- e^{g_last} h + (k e^{g_last - g})^T v,
// o = s e^{g} (q h) + s tril(q k^T * Gamma) v.  p.gam then holds the RAW per-head log-gates and the staging wave that
// owns the gate row forms the chunk-local prefix sum itself (64 lanes, DPP row scans).
template <typename T, int K, bool KEEP, int NMW = 4, bool L2N = false, bool DELTA = true>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gdr_fwd_scan_kernel(
    GdrScanParams p) {
  static_assert(!(KEEP && L2N), "a forward that keeps its intermediates takes normalised q and k");
  static_assert(DELTA || (!KEEP && !L2N), "the plain scan: forward only, no l2 norm");
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int BV = 16 * NMW;
  constexpr int RV = BV / 16;   // v, o: rows of a staging lane's 4-column piece
  typedef T rvv __attribute__((ext_vector_type(RV)));
  constexpr int LDR = K + 8;  // pitch of the row-major k and q tiles
  constexpr int KS = K / 32;  // 32-wide contraction slices of the state
  constexpr int KT = K / 16;  // 16-row state tiles per matrix wave
  constexpr int ATS = kTriElems;  // elements per (chunk, head) in AT
  // k, q and the gate rows of a chunk are in LDS one chunk period before the rest of it (three buffers, chunk
  // modulo 3): Aqk of chunk c + 1 is formed from them while chunk c is in work.
  __shared__ __attribute__((aligned(16))) T sK[3][BT * LDR];     // k    [t][k]
  __shared__ __attribute__((aligned(16))) T sQ[3][BT * LDR];     // q    [t][k]
  __shared__ __attribute__((aligned(16))) T sVt[2][BV * LDT];    // v^T  [v][t], later o^T
  __shared__ __attribute__((aligned(16))) T sAT[2][kTriElems];   // Tu (packed triangular tile)
  __shared__ __attribute__((aligned(16))) T sP[2][kTriElems];    // Aqk, same packing
  __shared__ __attribute__((aligned(16))) float sGam[3][BT];     // gamma_t
  __shared__ __attribute__((aligned(16))) float sEg[3][BT];      // e^{gamma_t}
  __shared__ __attribute__((aligned(16))) float sEd[3][BT];      // e^{gamma_last - gamma_t}
  __shared__ float sDec[3];                                      // e^{gamma_last}
  __shared__ __attribute__((aligned(16))) float sRq[L2N ? 3 : 1][L2N ? BT : 4];    // L2N: 1 / |q_t|
  __shared__ __attribute__((aligned(16))) float sRk[L2N ? 3 : 1][L2N ? BT : 4];    // L2N: 1 / |k_t|
  __shared__ __attribute__((aligned(16))) float sEgk[L2N ? 3 : 1][L2N ? BT : 4];   // L2N: e^{gamma_t} / |k_t|

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
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);

  // Aqk = scale tril(q k^T * Gamma) of the chunk whose tiles are in buffer b, shared out over waves 0-3 by 16x16
  // block: a block is computed transposed (k rows against q rows), which leaves every lane with four
  // adjacent entries of one row of Aqk - an 8-byte piece of the packed tile frag_tri() reads.  Rows past the
  // end of a short chunk are zero in the q and k tiles.
  auto compute_p = [&](int b3, int pb, int chunk) __attribute__((always_inline)) {
    const T* Kr = sK[b3];
    const T* Q = sQ[b3];
    T* Po = sP[pb];
    // KEEP: the first value slab of a head also leaves the tile in memory for the backward pass
    T* Pg = nullptr;
    if constexpr (KEEP) {
      if (vb == 0 && p.Aqk_out) Pg = (T*)p.Aqk_out + ((chunk0 + chunk) * H + hh) * (int64_t)kTriElems;
    }
    const int c = lane & 15, g = lane >> 4;
    // (row block, column block) of this wave's blocks, a nibble each, first in the low bits: two or three
    // blocks for each of the four waves, or five for each of the two waves that carry no state
    int tis, tjs, cnt;
    if constexpr (NMW == 4) {
      tis = wave == 0 ? 0x33 : wave == 1 ? 0x33 : wave == 2 ? 0x222 : 0x011;
      tjs = wave == 0 ? 0x10 : wave == 1 ? 0x32 : wave == 2 ? 0x210 : 0x010;
      cnt = wave < 2 ? 2 : 3;
    } else {
      tis = wave == 2 ? 0x03333 : 0x11222;
      tjs = wave == 2 ? 0x03210 : 0x10210;
      cnt = wave >= 2 ? 5 : 0;
    }
    v8 fq[KS];
    int cur = -1;
#pragma unroll
    for (int n = 0; n < (NMW == 4 ? 3 : 5); ++n) {
      if (n < cnt) {
        const int ti = (tis >> (4 * n)) & 15, tj = (tjs >> (4 * n)) & 15;
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
        if constexpr (L2N) {
          const float ri = sRq[b3][16 * ti + c];
          const f32x4 rj = *(const f32x4*)&sRk[b3][16 * tj + 4 * g];
#pragma unroll
          for (int r = 0; r < 4; ++r) sc[r] *= ri * rj[r];
        }
        v4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          o[r] = (T)((ti > tj || 4 * g + r <= c) ? p.scale * sc[r] * __expf(gi - gj[r]) : 0.f);
        *(v4*)&Po[(ti * (ti + 1) / 2 + tj) * 256 + c * 16 + 4 * g] = o;
        if constexpr (KEEP) {
          if (Pg) *(v4*)&Pg[(ti * (ti + 1) / 2 + tj) * 256 + c * 16 + 4 * g] = o;
        }
      }
    }
  };

  if (wave >= 4) {
    // =========================== staging waves ===========================
    if (nchunks == 0) return;
    const int st = tid - 256;
    constexpr int C8 = K / 8, NPW = BT * C8 / 256;           // 16-byte pieces per row / per lane (q)
    static_assert(kTriElems == 8 * (256 + 64), "Tu: a 16-byte piece per staging lane and 64 more");
    const int urg = st / (BV / 4), uc4 = (st % (BV / 4)) * 4;   // v, o: a lane owns RV rows x 4 columns
    const uint32_t HK = (uint32_t)H * K, HV = (uint32_t)H * V;
    auto q_row = [&](int e) { return e / C8; };
    auto q_col = [&](int e) { return (e % C8) * 8; };
    struct Regs {
      v8 q[NPW], k[NPW];
      v8 a0, a1;
      v4 v[RV];
      uint32_t gam;  // fp32 bits
      uint32_t rk;   // L2N: fp32 bits
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
    const char* la = (const char*)p.AT + (chunk0 * H + hh) * (int64_t)ATS * 2;
    const uint32_t offa0 = 16 * (uint32_t)st, offa1 = 16 * (uint32_t)(256 + lane);
    // The gate load is unconditional (a load under a branch would make the wave drain its whole load
    // queue at the join); without gates it reads a dummy address and the bits are masked to zero.
    const uint32_t gmask = p.gam ? 0xffffffffu : 0u;
    const char* lg = p.gam ? (const char*)p.gam + row00 * 4 : lq;
    const char* lr = L2N ? (const char*)p.rk + row00 * 4 : lq;
    const int64_t strr = (int64_t)BT * H * 4;
    char* so = (char*)p.o + (row00 * V + vbase) * 2;
    const int64_t strk = (int64_t)BT * HK * 2, strv = (int64_t)BT * HV * 2;
    const int64_t stra = (int64_t)H * ATS * 2;
    const int64_t strg = p.gam ? (int64_t)BT * H * 4 : 0;
    const int Llast = (int)(sp.len - (int64_t)(nchunks - 1) * BT);
    // Every memory operation of the steady state is unconditional: the wait counts the compiler places
    // in front of a register's first use then count the loads of the other register sets and the output
    // stores issued since as still in flight.  (With a load or store under a branch it has to assume the
    // path that skipped it, and the wave waits for everything it issued, the stores of a moment ago
    // included.)  Rows past the end of a sequence's last chunk are redirected to its last row by one
    // unsigned minimum per load (zeroed before use), and past the last chunk the pointers stay on it.
    const uint32_t limq_full = 2 * ((uint32_t)(BT - 1) * HK), limq_last = 2 * ((uint32_t)(Llast - 1) * HK);
    const uint32_t limv_full = 2 * ((uint32_t)(BT - 1) * HV), limv_last = 2 * ((uint32_t)(Llast - 1) * HV);
    static_assert(RV == 4 || RV == 2, "slab of 64 or 32 value columns");
    const uint32_t colq = 2 * (uint32_t)q_col(st), colv = 2 * (uint32_t)uc4;
    // k, q and the gate run one chunk ahead of v and Tu: register set j holds k, q, gamma of chunk j + 1 and
    // v, Tu of chunk j.
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
      R.gam = *(const uint32_t*)(lg + (offg < limg ? offg : limg));
      if constexpr (L2N) R.rk = *(const uint32_t*)(lr + (offg < limg ? offg : limg));
      if (lcq + 1 < nchunks) {
        lq += strk;
        lk += strk;
        lg += strg;
        if constexpr (L2N) lr += strr;
      }
      ++lcq;
    };
    auto load = [&](Regs& R) __attribute__((always_inline)) {
      const bool last = lcv >= nchunks - 1;
      const uint32_t limv = (last ? limv_last : limv_full) + colv;
      if constexpr (DELTA) {
        R.a0 = *(const v8*)(la + offa0);   // a full tile whatever the chunk length
        R.a1 = *(const v8*)(la + offa1);   // its last 64 pieces: every wave loads them, the first one writes them
      }
#pragma unroll
      for (int i = 0; i < RV; ++i) R.v[i] = *(const v4*)(lv + (offv[i] < limv ? offv[i] : limv));
      if (lcv + 1 < nchunks) {
        lv += strv;
        la += stra;
      }
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
    int wq = 0, wq3 = 0;  // next chunk whose k, q, gate rows are written, and its buffer
    auto write_kq = [&](Regs& R) __attribute__((always_inline)) {
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
          const float rq = l2norm_rstd<T, K / 8>(R.q[i], p.l2_eps);
          if (st % C8 == 0) sRq[wq3][q_row(st + 256 * i)] = rq;
        }
      }
#pragma unroll
      for (int i = 0; i < NPW; ++i) *(v8*)&sQ[wq3][dq[i]] = R.q[i];
#pragma unroll
      for (int i = 0; i < NPW; ++i) *(v8*)&sK[wq3][dq[i]] = R.k[i];
      if (wave == 4) {
        // lanes past the end of a short chunk carry the last row's gate
        float gam = __uint_as_float(R.gam & gmask);
        if constexpr (!DELTA) {
          // raw gates: inclusive prefix sum over the 64 rows (rows past the end add zero)
          const int Lw = wq == nchunks - 1 ? Llast : BT;
          const float x = row_prefix16(lane < Lw ? gam : 0.f);
          const float t0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 15));
          const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 31));
          const float t2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 47));
          const int rr = lane >> 4;
          gam = x + (rr >= 1 ? t0 : 0.f) + (rr >= 2 ? t1 : 0.f) + (rr >= 3 ? t2 : 0.f);
        }
        const float glast = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(gam), 63));
        sGam[wq3][lane] = gam;
        sEg[wq3][lane] = __expf(gam);
        if constexpr (L2N) {
          const float rk = __uint_as_float(R.rk);
          sRk[wq3][lane] = rk;
          sEgk[wq3][lane] = __expf(gam) * rk;
          sEd[wq3][lane] = __expf(glast - gam) * rk;
        } else {
          sEd[wq3][lane] = __expf(glast - gam);
        }
        if (lane == 0) sDec[wq3] = __expf(glast);
      }
      ++wq;
      wq3 = wq3 == 2 ? 0 : wq3 + 1;
    };
    int wc = 0;  // next chunk whose v, Tu are written
    auto write = [&](Regs& R) __attribute__((always_inline)) {
      const int b = wc & 1;
      if (wc == nchunks - 1 && Llast < BT) {
#pragma unroll
        for (int i = 0; i < RV; ++i)
          if (urg * RV + i >= Llast) R.v[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      }
      if constexpr (DELTA) {
        *(v8*)&sAT[b][st * 8] = R.a0;
        if (wave == 4) *(v8*)&sAT[b][2048 + lane * 8] = R.a1;
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
    // chunk periods to land.  Iteration c (the matrix waves work on chunk c and form Aqk of chunk c + 1) stores
    // the output of chunk c-1, writes set c + 1 (k, q, gamma of chunk c + 2; v, Tu of chunk c + 1) and loads set
    // c + 4 into the registers just emptied; sets rotate R1, R2, R0.  The steady-state loop runs whole rotations
    // over the iterations that touch neither the first nor the last chunk and leaves only at its latch.
    constexpr std::true_type any_chunk{};
    constexpr std::false_type inner_chunk{};
    Regs R0, R1, R2;
    load_kq(R0);              // k, q, gamma of chunk 0 on their own
    write_kq(R0);
    load(R0);
    load(R1);
    load(R2);
    lds_barrier();            // Aqk of chunk 0 can be formed
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
      if (nchunks > 2) {      // iteration nchunks - 2 writes the last chunk's v and Tu
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
  } else if (wave >= NMW) {
    // waves without a share of the state form their share of the scores and keep the barrier count
    if (nchunks > 0) {
      lds_barrier();
      compute_p(0, 0, 0);
      lds_barrier();
      int b3 = 0;
      for (int ci = 0; ci < nchunks; ++ci) {
        const int n3 = b3 == 2 ? 0 : b3 + 1;
        if (ci + 1 < nchunks) compute_p(n3, (ci + 1) & 1, ci + 1);
        lds_barrier();
        b3 = n3;
      }
    }
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
    // KEEP: the identity in the contraction order of an accumulator pair, one operand per 16-wide half of
    // a 32-slice, and this lane's places in the two outputs
    v8 eye[2];
    // wave-uniform bases (advanced chunk by chunk) and one 32-bit byte offset per lane for each output
    char* hT_base = nullptr;
    char* vn_base = nullptr;
    uint32_t hT_lane = 0, vn_lane = 0;
    if constexpr (KEEP) {
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int e = 0; e < 8; ++e) eye[half][e] = (T)(((e >> 2) == half && 4 * g + (e & 3) == c) ? 1.f : 0.f);
      // state tile (value block of 32, key block ks): lane (g & 1) * 32 + 16 half + c, slots 4 (2 (wave & 1) + g / 2) ..
      hT_base = (char*)p.h_frag_t +
                ((chunk0 * H + hh) * (int64_t)K * V + (int64_t)((vbase + cb) / 32) * (K / 32) * 64 * 16) * (int64_t)sizeof(T);
      hT_lane = (uint32_t)((((g & 1) * 32 + 16 * (g >> 1) + c) * 16 + 8 * (wave & 1)) * sizeof(T));
      vn_base = (char*)p.v_new + ((sp.bos * H + hh) * (int64_t)V + vbase + cb) * (int64_t)sizeof(T);
      vn_lane = (uint32_t)(((16 * (g & 1) + c) * H * V + 8 * (g >> 1)) * sizeof(T));
    }
    const int Llast = (int)(sp.len - (int64_t)(nchunks - 1) * BT);
    if (nchunks > 0) {
      lds_barrier();
      if constexpr (NMW == 4) compute_p(0, 0, 0);
      lds_barrier();
      int b3 = 0;   // ci modulo 3
      for (int ci = 0; ci < nchunks; ++ci) {
        const int b = ci & 1;
        const int n3 = b3 == 2 ? 0 : b3 + 1;
        const T* Kr = sK[b3];
        const T* Q = sQ[b3];
        const T* Tu = sAT[b];
        const T* P = sP[b];
        if constexpr (NMW == 4) {
          if (ci + 1 < nchunks) compute_p(n3, b ^ 1, ci + 1);   // with 32-column slabs the two other waves form the scores
        }
        const int vrow = cb + c;
        T* vt = &sVt[b][vrow * LDT];
        // LDS reads are issued a group ahead of the MFMAs that consume them; the scheduling
        // fences keep the compiler from sinking them back next to their use.
        v8 fa[2 * KS], fb[2 * KS];
        auto load_kq = [&](int tt, v8* f) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            if constexpr (DELTA) f[ks] = frag16<T>(Kr, LDR, 16 * tt, 32 * ks, lane);
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
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            hb[ks][e] = (T)acc[2 * ks][e];
            hb[ks][4 + e] = (T)acc[2 * ks + 1][e];
          }
        if constexpr (KEEP) {
          // the state entering this chunk, transposed tile by tile
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            // lanes 0-31 end up with key row 32 ks + c, lanes 32-63 with 32 ks + 16 + c, eight value columns each
            const f32x4 t0 = Elem<T>::mfma16(hb[ks], eye[0], zero4());
            const f32x4 t1 = Elem<T>::mfma16(hb[ks], eye[1], zero4());
            *(v8*)(hT_base + hT_lane + ks * 64 * 16 * sizeof(T)) = pair_halves<T>(t0, t1);
          }
          hT_base += (int64_t)H * K * V * (int64_t)sizeof(T);
        }
        f32x4 d[4], oq[4];
        auto mm_kq = [&](int tt, const v8* f) {
          d[tt] = zero4();
          oq[tt] = zero4();
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            if constexpr (DELTA) d[tt] = Elem<T>::mfma16(f[ks], hb[ks], d[tt]);
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
        f32x4 eg[4], ed[4];
        v4 vv[4];
        v8 ft[6];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
          if constexpr (L2N) eg[tt] = *(const f32x4*)&sEgk[b3][16 * tt + 4 * g];   // e^{gamma} / |k|, for the (k h) term
          else eg[tt] = *(const f32x4*)&sEg[b3][16 * tt + 4 * g];
          ed[tt] = *(const f32x4*)&sEd[b3][16 * tt + 4 * g];
          vv[tt] = *(const v4*)(vt + swz_t(vrow, 16 * tt + 4 * g));
        }
        const float dec = sDec[b3];
        if constexpr (DELTA) {
          ft[0] = frag_tri<T>(Tu, 0, 0, lane);
          ft[1] = frag_tri<T>(Tu, 1, 0, lane);
          ft[2] = frag_tri<T>(Tu, 2, 0, lane);
          ft[3] = frag_tri<T>(Tu, 2, 1, lane);
          ft[4] = frag_tri<T>(Tu, 3, 0, lane);
          ft[5] = frag_tri<T>(Tu, 3, 1, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        mm_kq(3, fb);
        __builtin_amdgcn_sched_barrier(0);
        load_kt(0, fa);
        v8 fp[6];
        fp[0] = frag_tri<T>(P, 0, 0, lane);
        fp[1] = frag_tri<T>(P, 1, 0, lane);
        fp[2] = frag_tri<T>(P, 2, 0, lane);
        fp[3] = frag_tri<T>(P, 2, 1, lane);
        fp[4] = frag_tri<T>(P, 3, 0, lane);
        fp[5] = frag_tri<T>(P, 3, 1, lane);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 vn[4];
        if constexpr (DELTA) {
          // r = v - e^{gamma} (k h), as the operand contracting over time
          v8 rb[2];
#pragma unroll
          for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) rb[tt >> 1][(tt & 1) * 4 + r] = (T)((float)vv[tt][r] - d[tt][r] * eg[tt][r]);
          // v_new = Tu r; Tu is lower triangular: row tiles 0 and 1 only meet the first 32 rows of r
          vn[0] = Elem<T>::mfma16(ft[0], rb[0], zero4());
          vn[1] = Elem<T>::mfma16(ft[1], rb[0], zero4());
          vn[2] = Elem<T>::mfma16(ft[2], rb[0], zero4());
          vn[3] = Elem<T>::mfma16(ft[4], rb[0], zero4());
          vn[2] = Elem<T>::mfma16(ft[3], rb[1], vn[2]);
          vn[3] = Elem<T>::mfma16(ft[5], rb[1], vn[3]);
        } else {
#pragma unroll
          for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) vn[tt][r] = (float)vv[tt][r];
        }
        if constexpr (L2N) {
          // the (q h) term carries e^{gamma} / |q| instead
#pragma unroll
          for (int tt = 0; tt < 4; ++tt) {
            const f32x4 e = *(const f32x4*)&sEg[b3][16 * tt + 4 * g];
            const f32x4 rq = *(const f32x4*)&sRq[b3][16 * tt + 4 * g];
#pragma unroll
            for (int r = 0; r < 4; ++r) eg[tt][r] = e[r] * rq[r];
          }
        }
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
        if constexpr (KEEP) {
          // v_new of this chunk, turned round the same way (here, where few registers are live)
          const int Lc = ci == nchunks - 1 ? Llast : BT;
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            // even rows of 16 lanes end up with time row 32 s2 + c, odd ones with 32 s2 + 16 + c
            const f32x4 t0 = Elem<T>::mfma16(vnb[s2], eye[0], zero4());
            const f32x4 t1 = Elem<T>::mfma16(vnb[s2], eye[1], zero4());
            const v8 x = pair_rows<T>(t0, t1);
            if (32 * s2 + 16 * (g & 1) + c < Lc) *(v8*)(vn_base + vn_lane + (int64_t)(32 * s2) * H * V * (int64_t)sizeof(T)) = x;
          }
          vn_base += (int64_t)BT * H * V * (int64_t)sizeof(T);
        }
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
int launch_scan(const GdrScanParams& p, int K, hipStream_t st) {
  int64_t nblk = (int64_t)p.N * p.H * (p.V / 64);
  FLA_REQUIRE(nblk <= 0x7fffffffLL / 2, FLA_E_UNSUPPORTED);
  if (nblk == 0) return FLA_OK;
  // 32-column slabs while they still give every workgroup a CU of its own
  const bool narrow = 2 * nblk <= kNumCUs;
  if (narrow) nblk *= 2;
  dim3 grid((unsigned)nblk), block(512);
  const bool keep = p.v_new != nullptr;
  if (!p.AT) {
    // the plain scan (no delta rule, raw per-head gates)
    if (keep || p.l2_eps >= 0.f) return FLA_E_UNSUPPORTED;
#define FLA_SCAN_PLAIN(KK)                                                                                     \
  if (narrow) hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, false, 2, false, false>), grid, block, 0, st, p);  \
  else hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, false, 4, false, false>), grid, block, 0, st, p);
    if (K == 64) { FLA_SCAN_PLAIN(64) }
    else if (K == 128) { FLA_SCAN_PLAIN(128) }
    else return FLA_E_UNSUPPORTED;
#undef FLA_SCAN_PLAIN
    FLA_CHECK_LAUNCH();
    return FLA_OK;
  }
#define FLA_SCAN(KK, KEEPV)                                                                              \
  if (narrow) hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, KEEPV, 2>), grid, block, 0, st, p);          \
  else hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, KEEPV, 4>), grid, block, 0, st, p);
#define FLA_SCAN_L2N(KK)                                                                                 \
  if (narrow) hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, false, 2, true>), grid, block, 0, st, p);    \
  else hipLaunchKernelGGL((gdr_fwd_scan_kernel<T, KK, false, 4, true>), grid, block, 0, st, p);
  if (p.l2_eps >= 0.f) {
    if (keep) return FLA_E_UNSUPPORTED;
    if (K == 64) { FLA_SCAN_L2N(64) }
    else if (K == 128) { FLA_SCAN_L2N(128) }
    else return FLA_E_UNSUPPORTED;
  } else
  if (K == 64 && keep) { FLA_SCAN(64, true) }
  else if (K == 64) { FLA_SCAN(64, false) }
  else if (K == 128 && keep) { FLA_SCAN(128, true) }
  else if (K == 128) { FLA_SCAN(128, false) }
  else return FLA_E_UNSUPPORTED;
#undef FLA_SCAN
#undef FLA_SCAN_L2N
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

static int gdr_fwd_scan_impl(const void* q, const void* k, const void* v, const void* AT, const float* g_cumsum,
                             const float* h0, void* o, float* ht, void* v_new, void* h_frag_t, void* Aqk_out,
                             const int64_t* offsets, const int64_t* chunk_offsets, const int64_t* seq_order,
                             int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                             float scale, float l2_eps, fla_stream_t stream, const float* k_rstd = nullptr) {
  FLA_REQUIRE(q && k && v && o, FLA_E_INVALID);   // AT == NULL: the plain scan (fla_chunk_simple_gla_fwd_scan)
  FLA_REQUIRE((l2_eps >= 0.f) == (k_rstd != nullptr), FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE(offsets ? (B == 1 && chunk_offsets != nullptr) : N == B, FLA_E_INVALID);
  FLA_REQUIRE(V % 64 == 0 && H <= 0x7fffff, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((v_new == nullptr) == (h_frag_t == nullptr), FLA_E_INVALID);
  FLA_REQUIRE(Aqk_out == nullptr || v_new != nullptr, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)AT | (uintptr_t)o | (uintptr_t)v_new |
               (uintptr_t)h_frag_t | (uintptr_t)Aqk_out) % 16 == 0, FLA_E_ALIGNMENT);
  GdrScanParams p{q, k, v, AT, g_cumsum, h0, o, ht, v_new, h_frag_t, Aqk_out, offsets, chunk_offsets, seq_order, T,
                  (int)H, (int)V, (int)N, scale, l2_eps, k_rstd};
  if (qkv_dtype == FLA_BF16) return launch_scan<bf16>(p, (int)K, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_scan<f16>(p, (int)K, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gated_delta_rule_fwd_scan(const void* q, const void* k, const void* v, const void* AT,
                                                   const float* g_cumsum, const float* h0, void* o, float* ht,
                                                   void* v_new, void* h_frag_t, void* Aqk_out, const int64_t* offsets, const int64_t* chunk_offsets,
                                                   const int64_t* seq_order, int qkv_dtype, int64_t B, int64_t T,
                                                   int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                                   fla_stream_t stream) {
  FLA_REQUIRE(AT, FLA_E_INVALID);
  return gdr_fwd_scan_impl(q, k, v, AT, g_cumsum, h0, o, ht, v_new, h_frag_t, Aqk_out, offsets, chunk_offsets,
                           seq_order, qkv_dtype, B, T, H, K, V, N, scale, -1.f, stream);
}

extern "C" int fla_chunk_gated_delta_rule_fwd_scan_l2norm(const void* q, const void* k, const void* v, const void* AT,
                                                          const float* g_cumsum, const float* k_rstd, const float* h0,
                                                          void* o, float* ht,
                                                          const int64_t* offsets, const int64_t* chunk_offsets,
                                                          const int64_t* seq_order, int qkv_dtype, int64_t B,
                                                          int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                                          float scale, float eps, fla_stream_t stream) {
  FLA_REQUIRE(eps >= 0.f && k_rstd, FLA_E_INVALID);
  return gdr_fwd_scan_impl(q, k, v, AT, g_cumsum, h0, o, ht, nullptr, nullptr, nullptr, offsets, chunk_offsets,
                           seq_order, qkv_dtype, B, T, H, K, V, N, scale, eps, stream, k_rstd);
}

extern "C" int fla_chunk_simple_gla_fwd_scan(const void* q, const void* k, const void* v, const float* g,
                                             const float* h0, void* o, float* ht, const int64_t* offsets,
                                             const int64_t* chunk_offsets, const int64_t* seq_order, int qkv_dtype,
                                             int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                             float scale, fla_stream_t stream) {
  return gdr_fwd_scan_impl(q, k, v, nullptr, g, h0, o, ht, nullptr, nullptr, nullptr, offsets, chunk_offsets,
                           seq_order, qkv_dtype, B, T, H, K, V, N, scale, -1.f, stream);
}
