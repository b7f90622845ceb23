// Fused chunked GLA forward for K = V = 128: one workgroup per (sequence, head) covering all 128 value
// columns, so that q, k and the gates of a head reach a CU once (the 64-column kernel has two workgroups
// per head, each pulling them through L2).  Same mathematics, staging waves and barrier protocol as
// gla_fwd_fused_kernel; what differs is how the matrix waves hold the state:
//   waves 0-3 ("matrix")   wave w owns value columns 32w .. 32w+31 of the fp32 state (all 128 key rows, in
//                          16x16 accumulator tiles).  The recurrence is independent per value column, so
//                          apart from the score tile a matrix wave exchanges nothing with the others:
//                            o_inter = q~ h            state straight from the accumulators (the LDS-side
//                                                      operand is read in accumulator-row order)
//                            P       = tril(q~ k~^T)   ten 16x16 blocks shared out over the four waves,
//                                                      exchanged through LDS (packed triangular tile)
//                            o       = s (o_inter + P v)
//                            h      <- diag(e^{G_last}) h + k^^T v
//                          The finished o tile takes the place of the wave's own columns of the v tile
//                          (time-contiguous); after the next barrier the matrix lanes write it to memory
//                          from there, each lane reading exactly the addresses it then refills with v of
//                          the chunk after next.  Neither a state tile nor an output tile of its own in LDS.
//   waves 4-7 ("staging")  gla_stage_waves.
#pragma once
#include "gla_fused_staging.h"

namespace {

// 16x16x32 operand from a swz_rm row-major tile (16 rows from row0, contraction slice [k0, k0 + 32) in
// accumulator-row order: indices 4g.., 16+4g.. for lane group g)
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag16_rm(const T* tile, int ld, int row0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  typedef __attribute__((address_space(3))) const volatile v4 lds_v4;
  const int row = row0 + (lane & 15), c = k0 + 4 * (lane >> 4);
  const T* p = tile + row * ld;
  v4 lo = *(lds_v4*)(p + swz_rm(row, c));
  v4 hi = *(lds_v4*)(p + swz_rm(row, c + 16));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <typename T, typename GT, bool SG>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gla_fwd_fused_wide_kernel(
    FusedParams p) {
  static_assert(!SG || sizeof(GT) == 4, "per-head gates are fp32");
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int K = 128, V = 128, NSTG = 4;
  constexpr int LDK = K + 8;
  constexpr int KS = K / 32;   // 32-wide contraction slices of the state
  constexpr int KT = K / 16;   // 16-row state tiles per column block
  __shared__ __attribute__((aligned(16))) T sQ[2][BT * LDK];     // q~  [t][k]
  __shared__ __attribute__((aligned(16))) T sK[2][BT * LDK];     // k~  [t][k]
  __shared__ __attribute__((aligned(16))) T sKh[2][K * LDT];     // k^  [k][t]
  __shared__ __attribute__((aligned(16))) T sVt[2][V * LDT];     // v   [v][t] (swz_t), later o [v][t]
  __shared__ __attribute__((aligned(16))) float sDecay[2][K];
  __shared__ __attribute__((aligned(16))) T sP[kTriElems];       // tril(S), packed 16x16 blocks
  __shared__ int sWide[2][NSTG];                                   // per staging wave: gates out of range

  const int tid = threadIdx.x, lane = tid & 63;
  // wave-uniform by construction: keeps the role split and the barriers on scalar branches
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int H = p.H;
  const int64_t item = blockIdx.x;
  const int hh = (int)(item % H);
  const int n = p.seq_order ? (int)p.seq_order[item / H] : (int)(item / H);
  const int nh = n * H + hh;
  SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);

  if (wave >= 4) {
    StageLds<T> L{{sQ[0], sQ[1]}, {sK[0], sK[1]}, {sKh[0], sKh[1]}, {sDecay[0], sDecay[1]}, {sWide[0], sWide[1]},
                  nullptr};
    gla_stage_waves<T, GT, K, NSTG, SG, false>(p, L, sp, nchunks, hh, 0, wave, lane, tid);
    return;
  }
  // =========================== matrix waves ===========================
  const int cb = 32 * wave;                 // first of this wave's 32 value columns
  const int c = lane & 15, g = lane >> 4;
  f32x4 acc[2][KT];                         // acc[nb][kt][r] = h[16 kt + 4 g + r][cb + 16 nb + c]
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      acc[nb][kt] = zero4();
      if (p.h0) {
        const float* h0p = p.h0 + (int64_t)nh * K * V + cb + 16 * nb + c;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[nb][kt][r] = h0p[(int64_t)(16 * kt + 4 * g + r) * V];
      }
    }
  // The matrix lanes stage the value tile (time-contiguous) of the next chunk and write the output tile of
  // the previous one: a lane owns 8 rows x 4 columns of both, loaded one chunk period ahead.
  const int vr = tid >> 5, vc4 = (tid & 31) * 4;
  const uint32_t vpitch = (uint32_t)H * V * (uint32_t)sizeof(T);
  const char* lv = (const char*)p.v + (sp.bos * H + hh) * (int64_t)V * (int64_t)sizeof(T);
  char* po = (char*)p.o + (sp.bos * H + hh) * (int64_t)V * (int64_t)sizeof(T);
  const int64_t strv = (int64_t)BT * vpitch;
  const int Llast = (int)(sp.len - (nchunks - 1) * BT);
  uint32_t offv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) offv[i] = (uint32_t)(vr * 8 + i) * vpitch + (uint32_t)vc4 * (uint32_t)sizeof(T);
  const uint32_t vlim_full = (uint32_t)(BT - 1) * vpitch, vlim_last = (uint32_t)(Llast - 1) * vpitch;
  int dvt[4];   // LDS slots of this lane: column vc4 + j, rows 8 vr .. 8 vr + 7
#pragma unroll
  for (int j = 0; j < 4; ++j) dvt[j] = (vc4 + j) * LDT + swz_t(vc4 + j, vr * 8);
  int64_t lvc = 0;  // chunk the value pointer is on (stays on the last one)
  v4 vreg[8];
  auto load_v = [&]() __attribute__((always_inline)) {
    const uint32_t lim = (lvc >= nchunks - 1 ? vlim_last : vlim_full) + (uint32_t)vc4 * (uint32_t)sizeof(T);
#pragma unroll
    for (int i = 0; i < 8; ++i) vreg[i] = *(const v4*)(lv + (offv[i] < lim ? offv[i] : lim));
    if (lvc + 1 < nchunks) lv += strv;
    ++lvc;
  };
  auto stage_v = [&](int buf, int64_t cidx) __attribute__((always_inline)) {
    const int64_t rem = sp.len - cidx * BT;
    const int L = (int)(rem < BT ? rem : BT);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v8 x;
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = (L < BT && vr * 8 + i >= L) ? (T)0.f : vreg[i][j];
      *(v8*)&sVt[buf][dvt[j]] = x;
    }
  };
  // output tile of chunk `oc` (left in the v tile by the matrix waves): LDS -> registers, registers -> memory
  int64_t oc = 0;
  v8 oreg[4];
  auto read_o = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j) oreg[j] = *(const v8*)&sVt[buf][dvt[j]];
  };
  auto store_o = [&]() __attribute__((always_inline)) {
    const int Lc = oc == nchunks - 1 ? Llast : BT;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (vr * 8 + i < Lc) *(v4*)(po + offv[i]) = v4{oreg[0][i], oreg[1][i], oreg[2][i], oreg[3][i]};
    po += strv;
    ++oc;
  };
  if (nchunks > 0) {
    load_v();
    stage_v(0, 0);
    load_v();
  }
  for (int64_t ci = 0; ci < nchunks; ++ci) {
    const int buf = (int)(ci & 1);
    lds_barrier();  // B1(ci): tiles of chunk ci and the output tile of chunk ci-1 are visible
    const T* Q = sQ[buf];
    const T* Kr = sK[buf];
    const T* Kh = sKh[buf];
    T* Vt = sVt[buf];
    // LDS reads are issued a group ahead of the MFMAs that consume them (the scheduling fences keep the
    // compiler from sinking them back next to their use); the value / output shuffling of the matrix lanes
    // runs while the first fragments are on their way.
    v8 fa[KS], fb[KS];
    auto load_q = [&](int tt, v8* f) __attribute__((always_inline)) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) f[ks] = frag16_rm<T>(Q, LDK, 16 * tt, 32 * ks, lane);
    };
    auto load_k = [&](int bj, v8* f) __attribute__((always_inline)) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) f[ks] = frag16_rm<T>(Kr, LDK, 16 * bj, 32 * ks, lane);
    };
    load_q(0, fa);
    load_q(1, fb);
    __builtin_amdgcn_sched_barrier(0);
    // stores before the next loads: the wait for those loads at the top of the next chunk then asks for
    // nothing younger than what it needs
    if (ci >= 1) read_o(buf ^ 1);
    if (ci + 1 < nchunks) stage_v(buf ^ 1, ci + 1);
    if (ci >= 1) store_o();
    if (ci + 1 < nchunks) load_v();
    if (p.wide) {
      int wide = 0;
#pragma unroll
      for (int w2 = 0; w2 < NSTG; ++w2) wide |= sWide[buf][w2];
      if (tid == 0) p.wide[(chunk0 + ci) * H + hh] = wide;
      if (wide) {
        // hand the state entering this chunk to the exact kernel: [V][K], 16-bit
        T* hw = (T*)p.hwide + ((chunk0 + ci) * H + hh) * (int64_t)K * V;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int kt = 0; kt < KT; ++kt) {
            v4 x;
#pragma unroll
            for (int r = 0; r < 4; ++r) x[r] = (T)acc[nb][kt][r];
            *(v4*)(hw + (int64_t)(cb + 16 * nb + c) * K + 16 * kt + 4 * g) = x;
          }
      }
    }
    // the state as the other MFMA operand: two stacked accumulators per 32-slice
    v8 hb[2][KS];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          hb[nb][ks][e] = (T)acc[nb][2 * ks][e];
          hb[nb][ks][4 + e] = (T)acc[nb][2 * ks + 1][e];
        }
    // ---- o_inter = q~ h, row tile by row tile
    f32x4 o[4][2];
    auto mm_q = [&](int tt, const v8* f) __attribute__((always_inline)) {
      o[tt][0] = zero4();
      o[tt][1] = zero4();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        o[tt][0] = Elem<T>::mfma16(f[ks], hb[0][ks], o[tt][0]);
        o[tt][1] = Elem<T>::mfma16(f[ks], hb[1][ks], o[tt][1]);
      }
    };
    __builtin_amdgcn_sched_barrier(0);
    mm_q(0, fa);
    __builtin_amdgcn_sched_barrier(0);
    load_q(2, fa);
    __builtin_amdgcn_sched_barrier(0);
    mm_q(1, fb);
    __builtin_amdgcn_sched_barrier(0);
    load_q(3, fb);
    __builtin_amdgcn_sched_barrier(0);
    mm_q(2, fa);
    __builtin_amdgcn_sched_barrier(0);
    // ---- the score blocks of this wave (transposed, k~ q~^T: a lane ends up with four consecutive
    // columns j of one row i): waves 0..3 take (0,0) (1,0) (1,1) | (2,0) (2,1) (2,2) | (3,0) (3,1) | (3,2) (3,3)
    {
      const int bi0 = wave == 0 ? 0 : wave == 1 ? 2 : 3;           // row block of the first score block
      const int bj0 = wave == 3 ? 2 : 0;
      load_q(bi0, fa);                                              // fa is free again
      __builtin_amdgcn_sched_barrier(0);
      mm_q(3, fb);
      __builtin_amdgcn_sched_barrier(0);
      v8 fk0[KS], fk1[KS];                                          // the state operand is dead by now
      load_k(bj0, fk0);
      auto score = [&](int bi, int bj, const v8* fq, const v8* fk) __attribute__((always_inline)) {
        f32x4 s = zero4();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = Elem<T>::mfma16(fk[ks], fq[ks], s);
        v4 x;
#pragma unroll
        for (int r = 0; r < 4; ++r) x[r] = (T)((bj < bi || 4 * g + r <= c) ? s[r] : 0.f);
        *(v4*)&sP[(bi * (bi + 1) / 2 + bj) * 256 + c * 16 + 4 * g] = x;
      };
      if (wave == 0) {
        load_q(1, fb);
        load_k(1, fk1);
        __builtin_amdgcn_sched_barrier(0);
        score(0, 0, fa, fk0);
        score(1, 0, fb, fk0);
        score(1, 1, fb, fk1);
      } else if (wave == 1) {
        load_k(1, fk1);
        __builtin_amdgcn_sched_barrier(0);
        score(2, 0, fa, fk0);
        load_k(2, fk0);
        __builtin_amdgcn_sched_barrier(0);
        score(2, 1, fa, fk1);
        score(2, 2, fa, fk0);
      } else if (wave == 2) {
        load_k(1, fk1);
        __builtin_amdgcn_sched_barrier(0);
        score(3, 0, fa, fk0);
        score(3, 1, fa, fk1);
      } else {
        load_k(3, fk1);
        __builtin_amdgcn_sched_barrier(0);
        score(3, 2, fa, fk0);
        score(3, 3, fa, fk1);
      }
    }
    lds_barrier();  // B2(ci): P visible
    // ---- o += P v (row tiles 0 and 1 only meet the first 32 columns of P), this wave's two column blocks
    v8 vb[2][2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int s = 0; s < 2; ++s) vb[nb][s] = frag16_t<T>(Vt, cb + 16 * nb, 32 * s, lane);
    v8 fp[6];
    fp[0] = frag_tri<T>(sP, 0, 0, lane);
    fp[1] = frag_tri<T>(sP, 1, 0, lane);
    fp[2] = frag_tri<T>(sP, 2, 0, lane);
    fp[3] = frag_tri<T>(sP, 2, 1, lane);
    fp[4] = frag_tri<T>(sP, 3, 0, lane);
    fp[5] = frag_tri<T>(sP, 3, 1, lane);
    // the first two state tiles' k^ fragments behind them
    v8 ka[2], kb[2];
    auto load_kh = [&](int kt, v8* f) __attribute__((always_inline)) {
#pragma unroll
      for (int s = 0; s < 2; ++s) f[s] = frag16<T>(Kh, LDT, 16 * kt, 32 * s, lane);
    };
    load_kh(0, ka);
    load_kh(1, kb);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      o[0][nb] = Elem<T>::mfma16(fp[0], vb[nb][0], o[0][nb]);
      o[1][nb] = Elem<T>::mfma16(fp[1], vb[nb][0], o[1][nb]);
      o[2][nb] = Elem<T>::mfma16(fp[2], vb[nb][0], o[2][nb]);
      o[3][nb] = Elem<T>::mfma16(fp[4], vb[nb][0], o[3][nb]);
      o[2][nb] = Elem<T>::mfma16(fp[3], vb[nb][1], o[2][nb]);
      o[3][nb] = Elem<T>::mfma16(fp[5], vb[nb][1], o[3][nb]);
    }
    __builtin_amdgcn_sched_barrier(0);
    // ---- state update: h <- diag(e^{G_last}) h + k^^T v, two state tiles per step, the next two in flight
    auto upd = [&](int kt, const v8* f) __attribute__((always_inline)) {
      const f32x4 d = *(const f32x4*)&sDecay[buf][16 * kt + 4 * g];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[nb][kt][r] *= d[r];
#pragma unroll
        for (int s = 0; s < 2; ++s) acc[nb][kt] = Elem<T>::mfma16(f[s], vb[nb][s], acc[nb][kt]);
      }
    };
#pragma unroll
    for (int kt = 0; kt < KT; kt += 2) {
      upd(kt, ka);
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 2 < KT) load_kh(kt + 2, ka);
      __builtin_amdgcn_sched_barrier(0);
      upd(kt + 1, kb);
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 3 < KT) load_kh(kt + 3, kb);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- the output tile takes the place of this wave's columns of the v tile (nobody else reads them)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int row = cb + 16 * nb + c;
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        v4 ov;
#pragma unroll
        for (int r = 0; r < 4; ++r) ov[r] = (T)(o[tt][nb][r] * p.scale);
        *(v4*)(Vt + row * LDT + swz_t(row, 16 * tt + 4 * g)) = ov;
      }
    }
  }
  if (nchunks > 0) {
    lds_barrier();  // the last output tile is visible
    read_o((int)((nchunks - 1) & 1));
    store_o();
  }
  if (p.ht) {
    float* htp = p.ht + (int64_t)nh * K * V + cb + c;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) htp[(int64_t)(16 * kt + 4 * g + r) * V + 16 * nb] = acc[nb][kt][r];
  }
}

}  // namespace
