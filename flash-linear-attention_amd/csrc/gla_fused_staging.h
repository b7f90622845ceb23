// Shared parts of the fused GLA forward kernels: launch parameters, the swizzled row-major operand
// tiles, and the work of the staging waves (loads, prefix sums of the log-gates, gated operand tiles).
#pragma once
#include "chunk_common.h"

namespace {

struct FusedParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const float* h0;
  void* o;
  float* ht;
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  const int64_t* seq_order;  // sequence ids, longest first (or NULL)
  int* wide;        // [chunks, H]: 1 where a chunk's gates leave the single-reference range
  void* hwide;      // states entering those chunks, FLA_H_FRAGMENT order, [chunks, H, K*V]
  int64_t T;
  int H, V, N;
  float scale;
  void* hT;         // HT variant: the state entering every chunk, FLA_H_FRAGMENT_T order, [chunks, H, K*V]
  void* qg;         // HT variant, optional: the gated queries q e^{G} as staged, [rows, H, K] in the q dtype
  float* decay;     //   and e^{G_last} of every chunk, [chunks, H, K] (both or neither)
  void* kh_t;       // with qg, optional: k^ = k e^{G_last - G} per chunk as staged, [chunks, H, K, 64] (key-major) ...
  void* scores;     //   ... and the chunk's causal score tile tril(q~ k~^T), [chunks, H, 64, 64] (both or neither)
  // LOGITS form: p.g holds the gate projection's output x and the log-gate is max(logsigmoid(x) * gate_inv_norm,
  // gate_clamp_min) (fla/layers/gla.py:214-217), formed by the staging waves on the way to the prefix sums
  float gate_inv_norm;
  float gate_clamp_min;   // -inf: no clamp
  // the workgroup redoes the output rows of its own flagged chunks after its last chunk (the 64- and 32-column
  // kernels; otherwise a second launch does)
  int exact_tail;
};

// log2(sigmoid(x)) * inv_norm, clamped from below at clamp2 (both in the log2 domain): two transcendental
// instructions per element.  log2(1 + e) keeps an absolute error of 1e-7, far below what a log-gate needs;
// x = +inf gives exactly 0 (the value rows past the end of a short chunk are set to).
FLA_DEVICE float log2_sigmoid_gate(float x, float inv_norm, float clamp2) {
  constexpr float LOG2E = 1.4426950408889634f;
  const float t = x * LOG2E;
  const float e = __builtin_amdgcn_exp2f(-fabsf(t));
  const float l = __builtin_amdgcn_logf(1.f + e);
  return fmaxf((fminf(t, 0.f) - l) * inv_norm, clamp2);
}

// The row-major q~ / k~ tiles are written by lanes that own four adjacent rows each, i.e.
// with a row stride of four between neighbouring lanes (64 bytes modulo 256: measured 2.5x
// slower than conflict-free writes).  XOR-ing row bits 4-5 into the 16-byte chunk index
// spreads the writes over all banks; every fragment read stays one (or two half-) chunk reads.
FLA_DEVICE int swz_rm(int row, int col) { return col ^ (((row >> 4) & 3) << 3); }

template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag32_swz(const T* tile, int ld, int row0, int k0, int lane) {
  const int row = row0 + (lane & 31);
  return *(const typename Elem<T>::v8*)(tile + row * ld + swz_rm(row, k0 + 8 * (lane >> 5)));
}
// lds_frag32_perm on a swizzled tile
template <typename T>
FLA_DEVICE typename Elem<T>::v8 frag32_perm_swz(const T* tile, int ld, int row0, int k0, int lane) {
  typedef typename Elem<T>::v4 v4;
  const int row = row0 + (lane & 31), c = k0 + 4 * (lane >> 5);
  const T* p = tile + row * ld;
  v4 lo = *(const v4*)(p + swz_rm(row, c));
  v4 hi = *(const v4*)(p + swz_rm(row, c + 8));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// LDS tiles the staging waves fill (two buffers each) and, for kernels whose staging waves also write the
// output, the finished output tile they read.
template <typename T>
struct StageLds {
  T* q[2];        // q~  [t][k], pitch K + 8, swz_rm
  T* k[2];        // k~  [t][k]
  T* kh[2];       // k^  [k][t], pitch LDT
  float* decay[2];
  int* wide[2];   // per staging wave: gates out of range
  const T* o;     // finished output tile [t][v] of 64 value columns, pitch LDT (STORE_O only)
};

// The staging waves (waves 4 .. 4 + NSTG - 1 of the workgroup) of one (sequence, head):
// load chunk c+1 (refilling each register as it is consumed), form the chunk-local prefix sum G of the
// log-gates with DPP row scans, and write the gated operand tiles of chunk c+1 to LDS:
//   q~ = q e^{G}, k~ = k e^{-G} (row-major), k^ = k e^{G_last-G} (time-contiguous), e^{G_last}.
// Barrier protocol with the matrix waves, per chunk c: B1(c) publishes the tiles of chunk c; B2(c) sits in the
// middle of staging chunk c+1.  STORE_O: after B1(c) the staging waves also write the output tile of chunk c-1
// (left in L.o by the matrix waves) to memory as whole rows, and one more barrier + store follows the last chunk.
// SG: one log-gate per (token, head), p.g is fp32 [B*T, H]: a lane loads one word per row and uses it for all
// its key channels, so the prefix sums and exponentials of a row are formed once.
// keep(buf, c): called right behind B1(c), while the tiles of chunk c sit complete in buffer buf (kernels that leave
// copies of them in memory for a backward pass do it there; the tiles are next written after B1(c+1)).
struct NoKeep {
  FLA_DEVICE void operator()(int, int64_t) const {}
};
template <typename T, typename GT, int K, int NSTG, bool SG, bool STORE_O, int BV = 64, bool LOGITS = false,
          typename KeepFn = NoKeep>
FLA_DEVICE void gla_stage_waves(const FusedParams& p, const StageLds<T>& L, const SeqSpan& sp, int64_t nchunks,
                                int hh, int vbase, int wave, int lane, int tid, KeepFn keep = KeepFn()) {
  typedef typename Elem<T>::v8 v8;
  constexpr int LDK = K + 8;
  constexpr int CPW = K / NSTG;                // key columns per staging wave
  constexpr int CPL = CPW / 4;                 // key columns per staging lane (8 for K=128, 4 for K=64)
  static_assert(CPL == 8 || CPL == 4, "staging lane tiling");
  constexpr float LOG2E = 1.4426950408889634f;
  const int H = p.H, V = p.V;
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };
  // A staging wave owns CPW key columns; a lane owns CPL adjacent columns of 4 rows.  The 16
  // row groups of a column block sit in the 16 lanes of one DPP row, so the prefix sum over
  // time is register adds plus DPP row shifts.
  constexpr int RPT = 4;                // rows per lane
  const int pw = wave - 4;
  const int rg = lane & 15;
  const int kc = pw * CPW + (lane >> 4) * CPL;
  typedef GT gvec __attribute__((ext_vector_type(CPL)));
  typedef T kvec __attribute__((ext_vector_type(CPL)));
  struct Regs {
    gvec g[RPT];
    kvec q[RPT];
    kvec k[RPT];
  };
  // A wave issues at most one instruction every few cycles and this path is arithmetic-bound,
  // so the steady state carries no address arithmetic: the byte offsets of this lane's rows
  // from the first row of a chunk are computed once, the (uniform) chunk base pointers are
  // advanced by a constant stride, and rows past the end of a sequence's last chunk are
  // redirected to its last row by one unsigned minimum (they are zeroed before use).
  // Loads are unconditional, so the compiler is free to batch and interleave them; past the
  // last chunk the pointers stay on it.
  constexpr int GSH = sizeof(GT) == 4 ? 1 : 0;   // gate bytes = q/k bytes << GSH
  const uint32_t pitch = (uint32_t)H * K * (uint32_t)sizeof(T);
  uint32_t offk[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) offk[i] = (uint32_t)(rg * RPT + i) * pitch + (uint32_t)kc * (uint32_t)sizeof(T);
  const int64_t row00 = (sp.bos * H + hh) * (int64_t)K;
  const char* lq = (const char*)p.q + row00 * (int64_t)sizeof(T);
  const char* lk = (const char*)p.k + row00 * (int64_t)sizeof(T);
  const char* lg = SG ? (const char*)p.g + (sp.bos * H + hh) * (int64_t)sizeof(float)
                      : (const char*)p.g + row00 * (int64_t)sizeof(GT);
  const int64_t strk = (int64_t)BT * pitch;
  const uint32_t gpitch = (uint32_t)H * (uint32_t)sizeof(float);   // SG: row pitch of the gates
  const int64_t strg = SG ? (int64_t)BT * gpitch : (strk << (sizeof(GT) == 4 ? 1 : 0));
  uint32_t offg[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) offg[i] = (uint32_t)(rg * RPT + i) * gpitch;
  const int Llast = (int)(sp.len - (nchunks - 1) * BT);
  const uint32_t lim_full = (uint32_t)(BT - 1) * pitch, lim_last = (uint32_t)(Llast - 1) * pitch;
  int64_t lc = 0;  // chunk the load pointers are on
  uint32_t lim = 0, limg = 0;
  auto begin_loads = [&]() __attribute__((always_inline)) {
    lim = (lc >= nchunks - 1 ? lim_last : lim_full) + (uint32_t)kc * (uint32_t)sizeof(T);
    if (SG) limg = (uint32_t)((lc >= nchunks - 1 ? Llast : BT) - 1) * gpitch;
  };
  auto load_g = [&](Regs& R, int i) __attribute__((always_inline)) {
    if constexpr (SG) {
      const float x = *(const float*)(lg + (offg[i] < limg ? offg[i] : limg));
#pragma unroll
      for (int j = 0; j < CPL; ++j) R.g[i][j] = x;
    } else {
      uint32_t o = offk[i] < lim ? offk[i] : lim;
      R.g[i] = *(const gvec*)(lg + (o << GSH));
    }
  };
  auto load_qk = [&](Regs& R, int i) __attribute__((always_inline)) {
    uint32_t o = offk[i] < lim ? offk[i] : lim;
    R.q[i] = *(const kvec*)(lq + o);
    R.k[i] = *(const kvec*)(lk + o);
  };
  auto end_loads = [&]() __attribute__((always_inline)) {
    if (lc + 1 < nchunks) {
      lq += strk;
      lk += strk;
      lg += strg;
    }
    ++lc;
  };
  auto mask_tail = [&](Regs& R, int L) __attribute__((always_inline)) {
    if (L < BT) {
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        if (rg * RPT + i >= L) {
#pragma unroll
          for (int j = 0; j < CPL; ++j) {
            R.g[i][j] = LOGITS ? (GT)INFINITY : (GT)0.f;   // a log-gate of exactly zero either way
            R.q[i][j] = (T)0.f;
            R.k[i][j] = (T)0.f;
          }
        }
      }
    }
  };
  // LDS destinations of this lane
  int dq[RPT], dkh[CPL];
#pragma unroll
  for (int i = 0; i < RPT; ++i) dq[i] = (rg * RPT + i) * LDK + swz_rm(rg * RPT + i, kc);
#pragma unroll
  for (int j = 0; j < CPL; ++j) dkh[j] = (kc + j) * LDT + rg * RPT;
  // Stage the tiles of chunk c (held in R) into buffer `buf` and refill R, register by
  // register as each is consumed, with the chunk two further on: the loads of that chunk are
  // spread through the arithmetic of this one.  mid_barrier() is called half way through; in the
  // steady state it is the workgroup barrier between the two halves of the matrix waves' chunk.
  auto stage = [&](Regs& R, int buf, int64_t c, auto mid_barrier) __attribute__((always_inline)) {
    mask_tail(R, chunk_len(c));
    begin_loads();
    float G[RPT][CPL], glast[CPL];
    float gabs = 0.f;
    [[maybe_unused]] const float clamp2 = p.gate_clamp_min * LOG2E;
    if constexpr (SG) {
      // one gate per row: a single prefix sum, shared by all key channels of the lane (the
      // exponentials below then collapse to one pair per row)
      float run = 0.f, Gs[RPT];
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        run = fmaf((float)R.g[i][0], LOG2E, run);
        Gs[i] = run;
      }
      const float pre = row_prefix16(run);
      const float tot = pre - run;
      const float gl = dpp_f32<0x15f>(pre);
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        Gs[i] += tot;
        gabs = fmaxf(gabs, fabsf(Gs[i]));
      }
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        glast[j] = gl;
#pragma unroll
        for (int i = 0; i < RPT; ++i) G[i][j] = Gs[i];
      }
    } else
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
      float run = 0.f;
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        if constexpr (LOGITS) run += log2_sigmoid_gate((float)R.g[i][j], p.gate_inv_norm, clamp2);
        else run = fmaf((float)R.g[i][j], LOG2E, run);   // prefix sums in the log2 domain
        G[i][j] = run;
      }
      const float pre = row_prefix16(run);
      const float tot = pre - run;                             // gates of the earlier row groups
      glast[j] = dpp_f32<0x15f>(pre);                          // G_last: lane 15 of the row, broadcast
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        G[i][j] += tot;
        gabs = fmaxf(gabs, fabsf(G[i][j]));
      }
    }
    // The scores use one reference point per chunk (e^{G} on q, e^{-G} on k), exact while
    // |G| stays below InvDecayLimit<T>::value.  Chunks beyond that are flagged and recomputed by
    // the exact routine afterwards (their q~, k~ tiles may hold infinities: only the scores
    // use them, and those are recomputed).
    const int out_of_range = __any(gabs > InvDecayLimit<T>::value * LOG2E);  // wave-uniform
    if (lane == 0) L.wide[buf][pw] = out_of_range;
    float eglast[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) eglast[j] = __builtin_amdgcn_exp2f(glast[j]);
#pragma unroll
    for (int i = 0; i < RPT; ++i) load_g(R, i);
    T khat[CPL][RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      kvec qv, kv;
      float kt[CPL];
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        const float e = __builtin_amdgcn_exp2f(G[i][j]);       // e^{G}
        const float einv = __builtin_amdgcn_exp2f(-G[i][j]);   // e^{-G}
        kt[j] = (float)R.k[i][j] * einv;
        qv[j] = (T)((float)R.q[i][j] * e);   // the matrix waves apply the scale to the fp32 output
        kv[j] = (T)kt[j];
      }
      // k^ = k e^{G_last-G}: inside the guarded range the product of the two factors is exact
      // to rounding; beyond it e^{-G} may overflow, so the exponent (always <= 0 for
      // non-positive gates) is formed directly (wave-uniform branch, rare)
      if (out_of_range) {
#pragma unroll
        for (int j = 0; j < CPL; ++j)
          khat[j][i] = (T)((float)R.k[i][j] * __builtin_amdgcn_exp2f(glast[j] - G[i][j]));
      } else {
#pragma unroll
        for (int j = 0; j < CPL; ++j) khat[j][i] = (T)(kt[j] * eglast[j]);
      }
      load_qk(R, i);
      *(kvec*)&L.q[buf][dq[i]] = qv;
      *(kvec*)&L.k[buf][dq[i]] = kv;
      if (i == RPT / 2 - 1) mid_barrier();
    }
    end_loads();
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
      typedef T rvec __attribute__((ext_vector_type(RPT)));
      rvec x;
#pragma unroll
      for (int i = 0; i < RPT; ++i) x[i] = khat[j][i];
      *(rvec*)&L.kh[buf][dkh[j]] = x;
    }
    if (rg == 0) {
#pragma unroll
      for (int j = 0; j < CPL; ++j) L.decay[buf][kc + j] = eglast[j];
    }
  };

  // The matrix waves leave each finished output tile in LDS; the staging waves write it to
  // memory one chunk period later as whole rows of the slab (BV / 8 lanes x 16 bytes per row).
  constexpr int NPO = BT * (BV / 8) / (64 * NSTG);
  static_assert(NPO >= 1, "output pieces per staging lane");
  const uint32_t opitch = (uint32_t)H * V * (uint32_t)sizeof(T);
  uint32_t offo[NPO];
  int ldo[NPO];
  const int ocol = (tid & (BV / 8 - 1)) * 8;   // element offset inside a row: the same for every piece of a lane
#pragma unroll
  for (int i = 0; i < NPO; ++i) {
    const int orow = ((tid - 256) + 64 * NSTG * i) / (BV / 8);
    ldo[i] = orow * LDT + ocol;
    offo[i] = (uint32_t)orow * opitch + (uint32_t)ocol * (uint32_t)sizeof(T);
  }
  char* po = (char*)p.o + ((sp.bos * H + hh) * (int64_t)V + vbase) * (int64_t)sizeof(T);
  const int64_t stro = (int64_t)BT * opitch;
  int64_t oc = 0;  // chunk whose output tile is stored next
  // Rows past the end of a short last chunk are redirected to its last row (LDS source and
  // destination alike, so the duplicates rewrite the same bytes): the stores stay unconditional
  // and the compiler's wait counts around them exact.
  auto store_o = [&]() __attribute__((always_inline)) {
    if constexpr (!STORE_O) return;
    const int Lc = oc == nchunks - 1 ? Llast : BT;
#pragma unroll
    for (int i = 0; i < NPO; ++i) {
      const int ls = min(ldo[i], (Lc - 1) * LDT + ocol);
      const uint32_t os = min(offo[i], (uint32_t)(Lc - 1) * opitch + (uint32_t)ocol * (uint32_t)sizeof(T));
      const v8 x = *(const v8*)&L.o[ls];
      __builtin_nontemporal_store(x, (v8*)(po + os));   // written once, never read here: keep it out of the L2's way
    }
    po += stro;
    ++oc;
  };

  if (nchunks > 0) {
    // Two register sets, used alternately: the loads refilling a set have two chunk periods
    // to land before it is staged again.
    Regs RA, RB;
    begin_loads();
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      load_g(RA, i);
      load_qk(RA, i);
    }
    end_loads();
    begin_loads();
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      load_g(RB, i);
      load_qk(RB, i);
    }
    end_loads();
    stage(RA, 0, 0, [] {});
    // Chunk c: B1(c) publishes its tiles and the output tile of chunk c-1, then the tiles of
    // chunk c+1 are staged around B2(c).  The steady-state loop runs whole pairs of chunks and
    // leaves only at its latch (the odd chunk out is handled after it): every path round it
    // issues the same loads, so the wait counts keep the two register sets two chunk periods
    // apart instead of waiting for the set that was refilled last.
    lds_barrier();  // B1(0)
    keep(0, 0);
    if (nchunks > 1) {
      stage(RB, 1, 1, [] { lds_barrier(); });  // contains B2(0)
      int64_t c = 1;
      for (int64_t pairs = (nchunks - 2) >> 1; pairs > 0; --pairs, c += 2) {
        lds_barrier();  // B1(c), c odd
        store_o();
        keep(1, c);
        stage(RA, 0, c + 1, [] { lds_barrier(); });  // contains B2(c)
        lds_barrier();  // B1(c+1)
        store_o();
        keep(0, c + 1);
        stage(RB, 1, c + 2, [] { lds_barrier(); });  // contains B2(c+1)
      }
      lds_barrier();  // B1(c)
      store_o();
      keep(1, c);
      if (c + 1 < nchunks) {
        stage(RA, 0, c + 1, [] { lds_barrier(); });  // contains B2(c)
        lds_barrier();  // B1(c+1)
        store_o();
        keep(0, c + 1);
      }
      lds_barrier();  // B2 of the last chunk
    } else {
      lds_barrier();  // B2(0)
    }
    lds_barrier();  // the last output tile is published
    store_o();
  }
}

}  // namespace
