// Fused chunked GLA forward for gfx950: one pass over q, k, v, g produces o and the
// final state; the per-chunk states never leave the chip.
//
// One workgroup of 8 or 12 waves owns one (sequence, head, 64 value columns) and walks the
// chunks serially.  The waves are specialised:
//   waves 4..   ("staging")  load chunk c+1 (refilling each register as it is consumed), form the
//                          chunk-local prefix sum G of the log-gates with wave shuffles,
//                          and write the gated operand tiles of chunk c+1 to LDS:
//                          q~ = s q e^{G}, k~ = k e^{-G} (row-major), k^ = k e^{G_last-G}
//                          and v (time-contiguous), e^{G_last};
//   waves 0-3 ("matrix")   for chunk c:  S = q~ k~^T,  P = tril(S),
//                          o = q~ h + P v,  h <- diag(e^{G_last}) h + k^^T v,
//                          with the fp32 state in MFMA accumulators.
// Every SIMD therefore hosts one matrix wave and one or two staging waves, so the transcendental
// and LDS-write work of the next chunk overlaps the MFMAs of the current one.  Operand
// tiles are double-buffered; both groups meet at two workgroup barriers per chunk.
// The state is handed from the accumulators to the q~ h product in MFMA-fragment order
// through LDS (each lane writes and reads its own 32 contiguous bytes per tile).
//
// Math: fla/ops/common/chunk_h.py:73-137, fla/ops/gla/chunk.py:29-170 and :320-393.
// HBM traffic is the operator's floor (q, k, v, g read once per 64-column slab, o
// written once, h0/ht once) instead of that plus a [B,NT,H,K,V] state round trip.
#include "gla_fused_staging.h"
#include "gla_fwd_fused_wide.h"

namespace {

// Exact recomputation of the output rows of flagged chunks: the scores
//   A_ij = s sum_k q_ik k_jk e^{G_ik - G_jk}   (j <= i)
// are evaluated pair by pair in fp32 with every exponent <= 0, as the reference does on its
// diagonal sub-blocks (fla/ops/gla/chunk.py:113-170), then o = (s q e^{G}) h_c + A v on MFMA.
struct ExactParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const int* wide;
  const void* hwide;
  void* o;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  float scale;
  int64_t total;   // (chunk, head) pairs
  int head_gates;  // g is fp32 [B*T, H]: one log-gate per (token, head)
  int hwide_vk;    // hwide holds [V][K] tiles (the 128-column kernel) instead of fragment-order ones
  int gate_logits; // g holds gate logits: the log-gate is max(logsigmoid(g) * gate_inv_norm, gate_clamp_min)
  float gate_inv_norm, gate_clamp_min;
};

// LDS tiles of one flagged chunk
template <typename T>
struct ExactLds {
  float* g;      // G     [t][k], pitch K + 4
  T* q;          // q, later s q e^{G}  [t][k], pitch K + 8
  T* k;          // k     [t][k]
  T* vt;         // v     [v][t], VS rows, pitch LDT
  T* p;          // A     [i][j], pitch LDT
  float* part;   // gate sums of the row groups, [256 / (K / 4)][K]
};

// One flagged chunk of head hh: output rows of the value columns vbase .. vbase + VS - 1 (V columns per row in
// memory).  Called by all NTHR threads of a workgroup (NTHR = 256 or 512): the first four waves load, stage and run
// the matrix products, every thread takes a share of the pairwise scores; the barriers are reached by all.
template <typename T, typename GT, int K, int VS, int NTHR>
FLA_DEVICE void gla_exact_chunk(const ExactParams& p, const ExactLds<T>& S, const ChunkLoc& cl, int hh, int V, int vbase,
                                int tid) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int LDG = K + 4;
  constexpr int CG = K / 4, RG = 256 / CG, RPT = BT / RG;
  constexpr int CGV = VS / 4, RGV = 256 / CGV, RPTV = BT / RGV;
  constexpr int KT32 = K / 32, TV = VS >= 64 ? VS / 64 : 1;
  static_assert(NTHR == 256 || NTHR == 512, "threads of the calling workgroup");
  const int H = p.H;
  const int lane = tid & 63, wave = tid >> 6;
  const bool worker = wave < 4;   // wave-uniform
  const int L = cl.L;
  const int64_t row0 = cl.row0;
  const int rg = (tid & 255) / CG, c4 = ((tid & 255) % CG) * 4;
  float G[RPT][4];
  v4 qreg[RPT], kreg[RPT];
  if (worker) {
    float gq[RPT][4];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      int row = rg * RPT + i;
      if (row < L) {
        int64_t off = ((row0 + row) * H + hh) * (int64_t)K + c4;
        if (p.head_gates) {
          const float x = ((const float*)p.g)[(row0 + row) * H + hh];
#pragma unroll
          for (int j = 0; j < 4; ++j) gq[i][j] = x;
        } else {
          Load<GT>::x4((const GT*)p.g + off, gq[i]);
          if (p.gate_logits) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              gq[i][j] = log2_sigmoid_gate(gq[i][j], p.gate_inv_norm, p.gate_clamp_min * 1.4426950408889634f) *
                         0.6931471805599453f;
          }
        }
        qreg[i] = *(const v4*)((const T*)p.q + off);
        kreg[i] = *(const v4*)((const T*)p.k + off);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) gq[i][j] = 0.f;
        qreg[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
        kreg[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      }
    }
    const int rgv = tid / CGV, cv4 = (tid % CGV) * 4;
#pragma unroll
    for (int i = 0; i < RPTV; ++i) {
      int row = rgv * RPTV + i;
      v4 x = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      if (row < L) x = *(const v4*)((const T*)p.v + ((row0 + row) * H + hh) * (int64_t)V + vbase + cv4);
#pragma unroll
      for (int j = 0; j < 4; ++j) S.vt[(cv4 + j) * LDT + row] = x[j];
    }
    float run[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < RPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        run[j] += gq[i][j];
        G[i][j] = run[j];
      }
    *(f32x4*)&S.part[rg * K + c4] = f32x4{run[0], run[1], run[2], run[3]};
  }
  __syncthreads();
  if (worker) {
    float off[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r = 0; r < rg; ++r) {
      f32x4 pr = *(const f32x4*)&S.part[r * K + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) off[j] += pr[j];
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      int row = rg * RPT + i;
      *(f32x4*)&S.g[row * LDG + c4] = f32x4{G[i][0] + off[0], G[i][1] + off[1], G[i][2] + off[2], G[i][3] + off[3]};
      *(v4*)&S.q[row * LDK + c4] = qreg[i];
      *(v4*)&S.k[row * LDK + c4] = kreg[i];
    }
  }
  __syncthreads();
  // ---- exact scores: a thread handles row i and every NQ-th column j <= i
  {
    constexpr int NQ = NTHR / BT;
    const int i = tid / NQ, jq = tid % NQ;
    for (int j = jq; j < BT; j += NQ) {
      float a = 0.f;
      if (j <= i) {
        for (int kk = 0; kk < K; kk += 4) {
          f32x4 gi = *(const f32x4*)&S.g[i * LDG + kk];
          f32x4 gj = *(const f32x4*)&S.g[j * LDG + kk];
          v4 qv = *(const v4*)&S.q[i * LDK + kk];
          v4 kv = *(const v4*)&S.k[j * LDK + kk];
#pragma unroll
          for (int e = 0; e < 4; ++e) a += (float)qv[e] * (float)kv[e] * __expf(gi[e] - gj[e]);
        }
      }
      S.p[i * LDT + j] = (T)(a * p.scale);
    }
  }
  __syncthreads();
  // ---- q~ = s q e^{G} over the raw q tile (every lane rewrites exactly what it reads)
  if (worker) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      int row = rg * RPT + i;
      f32x4 gg = *(const f32x4*)&S.g[row * LDG + c4];
      v4 qv = *(const v4*)&S.q[row * LDK + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) qv[j] = (T)((float)qv[j] * p.scale * __expf(gg[j]));
      *(v4*)&S.q[row * LDK + c4] = qv;
    }
  }
  __syncthreads();
  const int rw = wave >> 1, cw = wave & 1;
  if (worker && cw * TV * 32 < VS) {
    f32x16 acc[TV];
#pragma unroll
    for (int tv = 0; tv < TV; ++tv) acc[tv] = zero16();
    const T* hp = (const T*)p.hwide + (cl.cglob * H + hh) * (int64_t)K * V;
#pragma unroll
    for (int kt = 0; kt < KT32; ++kt)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (p.hwide_vk) {   // [V][K]: a lane reads 8 consecutive key channels of its value column
          v8 a = lds_frag32<T>(S.q, LDK, rw * 32, kt * 32 + half * 16, lane);
#pragma unroll
          for (int tv = 0; tv < TV; ++tv) {
            v8 b = *(const v8*)(hp + (int64_t)(vbase + (cw * TV + tv) * 32 + (lane & 31)) * K + kt * 32 + half * 16 + 8 * (lane >> 5));
            acc[tv] = Elem<T>::mfma32(a, b, acc[tv]);
          }
        } else {
          v8 a = lds_frag32_perm<T>(S.q, LDK, rw * 32, kt * 32 + half * 16, lane);
#pragma unroll
          for (int tv = 0; tv < TV; ++tv) {
            v8 b = *(const v8*)(hp + (((int64_t)kt * (V / 32) + (vbase / 32 + cw * TV + tv)) * 64 + lane) * 16 + half * 8);
            acc[tv] = Elem<T>::mfma32(a, b, acc[tv]);
          }
        }
      }
    const int jend = (rw + 1) * 32;
    for (int js = 0; js < jend; js += 16) {
      v8 a = lds_frag32<T>(S.p, LDT, rw * 32, js, lane);
#pragma unroll
      for (int tv = 0; tv < TV; ++tv)
        acc[tv] = Elem<T>::mfma32(a, lds_frag32<T>(S.vt, LDT, (cw * TV + tv) * 32, js, lane), acc[tv]);
    }
    T* op = (T*)p.o + (row0 * H + hh) * (int64_t)V + vbase;
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int i = rw * 32 + c32_row(r, lane);
        if (i < L) op[(int64_t)i * H * V + (cw * TV + tv) * 32 + (lane & 31)] = (T)acc[tv][r];
      }
  }
  __syncthreads();   // the tiles are free for the next flagged chunk
}

// NSTG: number of staging waves (4 or 8); the workgroup has 4 + NSTG waves.
// HT: the matrix waves also write the state entering every chunk to p.hT, transposed (what the backward
// kernels contract over v with), for a forward pass whose states are kept instead of being recomputed by
// the backward pass.
// SG: one log-gate per (token, head), p.g is fp32 [B*T, H] (the simple-GLA / RetNet-style decay): a lane loads one
// word per row and uses it for all its key channels, so the prefix sums and exponentials of a row are formed once.
// NVT: 32-column value tiles of the workgroup's slab.  Two (64 columns) is the form described above; one (32 columns,
// the matrix waves with cw = 1 only form their score quadrant) doubles the number of workgroups where 64-column slabs
// would leave half the CUs without one: a CU is fed at a fixed rate, and a 32-column workgroup needs five sixths of
// the bytes of a 64-column one per chunk (three quarters when it also writes the states).
// LOGITS: p.g holds gate logits; the staging waves apply logsigmoid / normalizer (and the clamp) themselves.
template <typename T, typename GT, int K, int NSTG, bool HT, bool SG = false, int NVT = 2, bool LOGITS = false>
__global__ __launch_bounds__(256 + 64 * NSTG) void gla_fwd_fused_kernel(FusedParams p) {
  static_assert(!SG || sizeof(GT) == 4, "per-head gates are fp32");
  static_assert(!LOGITS || (!SG && !HT), "gate logits: per-key gates, forward without kept states");
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  typedef T t2 __attribute__((ext_vector_type(2)));
  constexpr int BV = 32 * NVT;
  constexpr int LDK = K + 8;
  constexpr int KT32 = K / 32;                 // 32-row state tiles
  constexpr int NKT = (KT32 + 3) / 4;          // state tiles per matrix wave (x2 value tiles)
  constexpr int CPW = K / NSTG;                // key columns per staging wave
  constexpr int CPL = CPW / 4;                 // key columns per staging lane (8 for K=128, 4 for K=64)
  static_assert(CPL == 8 || CPL == 4, "staging lane tiling");
  constexpr float LOG2E = 1.4426950408889634f;
  __shared__ __attribute__((aligned(16))) T sQ[2][BT * LDK];     // q~  [t][k]
  __shared__ __attribute__((aligned(16))) T sK[2][BT * LDK];     // k~  [t][k]
  __shared__ __attribute__((aligned(16))) T sKh[2][K * LDT];     // k^  [k][t]
  __shared__ __attribute__((aligned(16))) T sVt[2][BV * LDT];    // v   [v][t]
  __shared__ __attribute__((aligned(16))) float sDecay[2][K];
  __shared__ __attribute__((aligned(16))) T sP[BT * LDT];        // tril(S) [i][j]
  __shared__ __attribute__((aligned(16))) T sHf[KT32 * NVT * 64 * 16];  // state, fragment order [kt][vt][lane][16]
  __shared__ __attribute__((aligned(16))) T sO[BT * LDT];        // finished output tile [t][v]
  __shared__ int sWide[2][NSTG];                                   // per staging wave: gates out of range

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
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };

  // HT: the gated queries of a chunk and its decay factors, as the staging waves left them in LDS, for a
  // backward pass whose reverse state scan then streams them instead of forming prefix sums and exponentials
  // of its own.  The slabs of a head share the rows out; rows past the end of a short chunk are not written.
  auto store_qg = [&](int buf, int64_t c) __attribute__((always_inline)) {
    const int tid = (int)(threadIdx.x & 255);   // the staging waves run it, 256 threads like the matrix waves
    if constexpr (HT) {
      if (p.qg) {
        constexpr int C8 = K / 8;
        const int nrow = BT / nvb > 0 ? BT / nvb : 0, r0 = vb * nrow;
        const int L = chunk_len(c);
        T* qb = (T*)p.qg + ((sp.bos + c * BT) * H + hh) * (int64_t)K;
        for (int e = tid; e < nrow * C8; e += 256) {
          const int row = r0 + e / C8, c8 = (e % C8) * 8;
          if (row < L) *(v8*)(qb + (int64_t)row * H * K + c8) = *(const v8*)&sQ[buf][row * LDK + swz_rm(row, c8)];
        }
        if (vb == 0 && tid < K) p.decay[((chunk0 + c) * H + hh) * (int64_t)K + tid] = sDecay[buf][tid];
      }
      if (p.kh_t) {
        // k^ of the chunk, key-major as staged (rows of 64 time steps; zero past the end of a short chunk): the
        // slabs share the key rows out
        const int nrow = K / nvb, r0 = vb * nrow;
        T* kb = (T*)p.kh_t + ((chunk0 + c) * H + hh) * (int64_t)K * BT;
        for (int e = tid; e < nrow * (BT / 8); e += 256) {
          const int row = r0 + e / (BT / 8), c8 = (e % (BT / 8)) * 8;
          *(v8*)(kb + row * BT + c8) = *(const v8*)&sKh[buf][row * LDT + c8];
        }
      }
    }
  };
  int any_wide = 0;   // matrix waves: some chunk of this workgroup was flagged
  if (wave >= 4) {
    // staging waves: see gla_fused_staging.h
    StageLds<T> L{{sQ[0], sQ[1]}, {sK[0], sK[1]}, {sKh[0], sKh[1]}, {sDecay[0], sDecay[1]}, {sWide[0], sWide[1]}, sO};
    // (the copies of q~ and k^ a backward pass reads are theirs: the matrix waves are the critical path of a forward
    // that keeps its activations)
    gla_stage_waves<T, GT, K, NSTG, SG, true, BV, LOGITS>(p, L, sp, nchunks, hh, vbase, wave, lane, tid, store_qg);
  } else {
    // =========================== matrix waves ===========================
    const int rw = wave >> 1, cw = wave & 1;   // output tile: rows 32rw.., value columns 32cw..
    f32x16 acc[NKT][NVT];                       // state tiles kt = wave + 4a, value tiles 0 .. NVT-1
#pragma unroll
    for (int a = 0; a < NKT; ++a)
#pragma unroll
      for (int vt = 0; vt < NVT; ++vt) {
        acc[a][vt] = zero16();
        int kt = wave + 4 * a;
        if (p.h0 && kt < KT32) {
          const float* h0p = p.h0 + (int64_t)nh * K * V;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[a][vt][r] = h0p[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + vt * 32 + (lane & 31)];
        }
      }
    // HT: the state entering chunk c in transposed fragment order (rows v, columns k: what the backward kernels
    // contract over v with).  A tile in accumulator order, converted to 16 bits and read as the first operand, is
    // its own transpose (lane = row index of the product, registers = contraction index in accumulator-row
    // order); multiplied by the identity in the same permuted order the product comes out in accumulator order
    // with lanes and registers exchanged: two matrix instructions per tile instead of a second set of
    // accumulators that is updated alongside the first.
    v8 eye[2];
    if constexpr (HT) {
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          eye[half][e] = (T)(((lane & 31) == 16 * half + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3)) ? 1.f : 0.f);
    }
    auto store_ht = [&](int64_t c) {
      if constexpr (HT) {
        T* hb = (T*)p.hT + ((chunk0 + c) * H + hh) * (int64_t)K * V;
#pragma unroll
        for (int a = 0; a < NKT; ++a) {
          int kt = wave + 4 * a;
          if (kt < KT32) {
#pragma unroll
            for (int vt = 0; vt < NVT; ++vt) {
              v8 lo, hi;
#pragma unroll
              for (int r = 0; r < 8; ++r) {
                lo[r] = (T)acc[a][vt][r];
                hi[r] = (T)acc[a][vt][r + 8];
              }
              f32x16 t = Elem<T>::mfma32(lo, eye[0], zero16());
              t = Elem<T>::mfma32(hi, eye[1], t);
#pragma unroll
              for (int r = 0; r < 8; ++r) {
                lo[r] = (T)t[r];
                hi[r] = (T)t[r + 8];
              }
              T* dst = hb + (((int64_t)(vbase / 32 + vt) * (K / 32) + kt) * 64 + lane) * 16;
              *(v8*)dst = lo;
              *(v8*)(dst + 8) = hi;
            }
          }
        }
      }
    };
    // the score tile of chunk c, once every wave has written its quadrant (rows shared out over the slabs)
    auto store_scores = [&](int64_t c) {
      if constexpr (HT) {
        if (p.scores) {
          const int nrow = BT / nvb, r0 = vb * nrow;
          T* pb = (T*)p.scores + ((chunk0 + c) * H + hh) * (int64_t)BT * BT;
          for (int e = tid; e < nrow * (BT / 8); e += 256) {
            const int row = r0 + e / (BT / 8), c8 = (e % (BT / 8)) * 8;
            *(v8*)(pb + row * BT + c8) = *(const v8*)&sP[row * LDT + c8];
          }
        }
      }
    };
    auto publish_state = [&]() {
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int vt = 0; vt < NVT; ++vt) {
            v8 lo, hi;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
              lo[r] = (T)acc[a][vt][r];
              hi[r] = (T)acc[a][vt][r + 8];
            }
            T* dst = &sHf[((kt * NVT + vt) * 64 + lane) * 16];
            *(v8*)dst = lo;
            *(v8*)(dst + 8) = hi;
          }
        }
      }
    };
    publish_state();
    // The matrix waves also stage the value tile (time-contiguous) of the next chunk: RPV rows x
    // 2 columns per lane, loaded one chunk period ahead.
    constexpr int RPV = BV / 8;   // 8 rows of 64 columns, 4 rows of 32
    typedef T rpv __attribute__((ext_vector_type(RPV)));
    const int vrg = tid / (BV / 2), vc = (tid % (BV / 2)) * 2;
    const uint32_t vpitch = (uint32_t)H * V * (uint32_t)sizeof(T);
    const char* lv = (const char*)p.v + ((sp.bos * H + hh) * (int64_t)V + vbase) * (int64_t)sizeof(T);
    const int64_t strv = (int64_t)BT * vpitch;
    const int Llast = (int)(sp.len - (nchunks - 1) * BT);
    uint32_t offv[RPV];
#pragma unroll
    for (int i = 0; i < RPV; ++i) offv[i] = (uint32_t)(vrg * RPV + i) * vpitch + (uint32_t)vc * (uint32_t)sizeof(T);
    const uint32_t vlim_full = (uint32_t)(BT - 1) * vpitch, vlim_last = (uint32_t)(Llast - 1) * vpitch;
    int64_t lvc = 0;  // chunk the value pointer is on (stays on the last one)
    t2 vreg[RPV];
    auto load_v = [&]() __attribute__((always_inline)) {
      const uint32_t lim = (lvc >= nchunks - 1 ? vlim_last : vlim_full) + (uint32_t)vc * (uint32_t)sizeof(T);
#pragma unroll
      for (int i = 0; i < RPV; ++i)   // read once by this workgroup only (q, k, g are read by every slab of a head)
        vreg[i] = __builtin_nontemporal_load((const t2*)(lv + (offv[i] < lim ? offv[i] : lim)));
      if (lvc + 1 < nchunks) lv += strv;
      ++lvc;
    };
    const int dv0 = (vc + 0) * LDT + vrg * RPV, dv1 = (vc + 1) * LDT + vrg * RPV;
    auto stage_v = [&](int buf, int64_t c) __attribute__((always_inline)) {
      const int L = chunk_len(c);
      rpv a, b;
#pragma unroll
      for (int i = 0; i < RPV; ++i) {
        a[i] = vreg[i][0];
        b[i] = vreg[i][1];
      }
      if (L < BT) {
#pragma unroll
        for (int i = 0; i < RPV; ++i)
          if (vrg * RPV + i >= L) a[i] = b[i] = (T)0.f;
      }
      *(rpv*)&sVt[buf][dv0] = a;
      *(rpv*)&sVt[buf][dv1] = b;
    };
    if (nchunks > 0) {
      load_v();
      stage_v(0, 0);
      load_v();
    }
    for (int64_t c = 0; c < nchunks; ++c) {
      const int buf = (int)(c & 1);
      lds_barrier();  // B1(c)
      // the next chunk's values first: the wait for their loads then covers no store issued after them
      if (c + 1 < nchunks) {
        stage_v(buf ^ 1, c + 1);
        load_v();
      }
      store_ht(c);  // unconditional and a whole chunk period ahead of the next wait for the value loads
      if (p.wide) {
        int wide = 0;
#pragma unroll
        for (int w2 = 0; w2 < NSTG; ++w2) wide |= sWide[buf][w2];
        if (tid == 0) p.wide[(chunk0 + c) * H + hh] = wide;
        any_wide |= wide;
        if (wide) {
          // hand over the state entering this chunk for the exact recomputation (fragment order, this slab's columns)
          T* hw = (T*)p.hwide + ((chunk0 + c) * H + hh) * (int64_t)K * V;
          for (int e = tid; e < KT32 * NVT * 64 * 2; e += 256) {
            int piece = e & 1, ln = (e >> 1) & 63, tile = e >> 7;  // tile = kt*NVT + vt
            int kt = tile / NVT, vt = tile % NVT;
            v8 x = *(const v8*)&sHf[(tile * 64 + ln) * 16 + piece * 8];
            *(v8*)(hw + (((int64_t)kt * (V / 32) + (vbase / 32 + vt)) * 64 + ln) * 16 + piece * 8) = x;
          }
        }
      }
      // ---- scores on the lower-triangular quadrants and the inter-chunk part of o
      const int qi = wave >> 1, qj = wave & 1;
      // transposed scores (k~ q~^T): a lane ends up with one row i of P and four consecutive
      // columns j per register quad, so P is written with 8-byte stores
      f32x16 s = zero16();
      if (qj <= qi) {
#pragma unroll
        for (int ks = 0; ks < K; ks += 16)
          s = Elem<T>::mfma32(frag32_swz<T>(sK[buf], LDK, qj * 32, ks, lane),
                              frag32_swz<T>(sQ[buf], LDK, qi * 32, ks, lane), s);
      }
      f32x16 o = zero16();
      if (cw < NVT) {
#pragma unroll
      for (int kt = 0; kt < KT32; ++kt) {
        const T* hf = &sHf[((kt * NVT + cw) * 64 + lane) * 16];
        v8 h0v = *(const v8*)hf, h1v = *(const v8*)(hf + 8);
        // transposed product (h^T q~^T): a lane ends up with four consecutive value columns of one row
        o = Elem<T>::mfma32(h0v, frag32_perm_swz<T>(sQ[buf], LDK, rw * 32, kt * 32, lane), o);
        o = Elem<T>::mfma32(h1v, frag32_perm_swz<T>(sQ[buf], LDK, rw * 32, kt * 32 + 16, lane), o);
      }
      }
      {
        const int i = qi * 32 + (lane & 31);
        T* prow = &sP[i * LDT + qj * 32 + 4 * (lane >> 5)];
        if (qi == qj) {            // diagonal quadrant: keep j <= i
          const int il = (lane & 31) - 4 * (lane >> 5);
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            v4 x;
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = (T)((8 * r4 + e <= il) ? s[4 * r4 + e] : 0.f);
            *(v4*)(prow + 8 * r4) = x;
          }
        } else {                   // below the diagonal, or the all-zero quadrant above it
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            v4 x;
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = (T)s[4 * r4 + e];
            *(v4*)(prow + 8 * r4) = x;
          }
        }
      }
      lds_barrier();  // B2(c): P visible; nobody reads the state fragments any more
      store_scores(c);
      if (cw < NVT) {
      if (rw == 0) {
#pragma unroll
        for (int js = 0; js < 32; js += 16)
          o = Elem<T>::mfma32(lds_frag32<T>(sVt[buf], LDT, cw * 32, js, lane), lds_frag32<T>(sP, LDT, 0, js, lane), o);
      } else {
#pragma unroll
        for (int js = 0; js < 64; js += 16)
          o = Elem<T>::mfma32(lds_frag32<T>(sVt[buf], LDT, cw * 32, js, lane), lds_frag32<T>(sP, LDT, 32, js, lane), o);
      }
      {
        // o^T tile: lane <-> time row, registers <-> value columns 8 (r/4) + 4 (lane/32) + r%4.
        // Left in LDS for the staging waves (rows past the end of a short chunk are not stored).
        T* orow_ = &sO[(rw * 32 + (lane & 31)) * LDT + cw * 32 + 4 * (lane >> 5)];
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          v4 ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = (T)(o[4 * r4 + e] * p.scale);
          *(v4*)(orow_ + 8 * r4) = ov;
        }
      }
      }
      // ---- state update
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            f32x4 d = *(const f32x4*)&sDecay[buf][kt * 32 + 8 * q4 + 4 * (lane >> 5)];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
#pragma unroll
              for (int vt = 0; vt < NVT; ++vt) acc[a][vt][4 * q4 + b] *= d[b];
            }
          }
#pragma unroll
          for (int ts = 0; ts < BT; ts += 16) {
            v8 fk = lds_frag32<T>(sKh[buf], LDT, kt * 32, ts, lane);
#pragma unroll
            for (int vt = 0; vt < NVT; ++vt)
              acc[a][vt] = Elem<T>::mfma32(fk, lds_frag32<T>(sVt[buf], LDT, 32 * vt, ts, lane), acc[a][vt]);
          }
        }
      }
      publish_state();
    }
    if (nchunks > 0) lds_barrier();  // hands the last output tile to the staging waves
    if (p.ht) {
      float* htp = p.ht + (int64_t)nh * K * V;
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int vt = 0; vt < NVT; ++vt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              htp[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + vt * 32 + (lane & 31)] = acc[a][vt][r];
        }
      }
    }
  }
  // Flagged chunks (rare: chunk-cumulative log-gates beyond the single-reference range): the workgroup redoes the
  // output rows of its own slab from the states it handed over, in the tiles the scan no longer needs, so the
  // operator needs no second launch.  Both wave groups take part; every barrier below is reached by all waves.
  if (p.exact_tail) {
    if (tid == 0) sWide[0][0] = any_wide;
    __syncthreads();   // also completes this workgroup's stores: the states handed over and the rows about to be rewritten
    if (sWide[0][0]) {
      const ExactParams e{p.q, p.k, p.v, p.g, p.wide, p.hwide, p.o, nullptr, nullptr, p.T, H, 0, p.scale, 0,
                          SG ? 1 : 0, 0, LOGITS ? 1 : 0, p.gate_inv_norm, p.gate_clamp_min};
      const ExactLds<T> S{(float*)&sQ[0][0], sK[0], sK[1], sVt[0], sP, (float*)&sKh[0][0]};
      static_assert(sizeof(sQ) >= BT * (K + 4) * sizeof(float) && sizeof(sKh[0]) >= (256 / (K / 4)) * K * sizeof(float),
                    "tiles of the exact recomputation fit the scan's");
      for (int64_t c = 0; c < nchunks; ++c) {
        // this workgroup's own flag, read past the caches other workgroups' flags of the same line may sit in
        if (__hip_atomic_load(&p.wide[(chunk0 + c) * H + hh], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) continue;
        const ChunkLoc cl{sp.bos + c * BT, chunk_len(c), chunk0 + c};
        gla_exact_chunk<T, GT, K, BV, 256 + 64 * NSTG>(e, S, cl, hh, V, vbase, tid);
      }
    }
  }
}

// The second launch of the operator where the scan does not redo its flagged chunks itself (the 128-column kernel).
template <typename T, typename GT, int K, int V>
__global__ __launch_bounds__(256) void gla_fwd_o_exact_kernel(ExactParams p) {
  constexpr int LDK = K + 8;
  constexpr int LDG = K + 4;
  constexpr int RG = 256 / (K / 4);
  const int H = p.H;
  // A few hundred workgroups walk the (chunk, head) flags: almost always none is set, and a
  // launch of one workgroup per chunk would cost more than the scan.  The lanes first read all flags
  // of the workgroup side by side (one memory latency instead of one per flag) and leave if none is set.
  {
    int any = 0;
    for (int64_t lin = blockIdx.x + (int64_t)threadIdx.x * gridDim.x; lin < p.total; lin += (int64_t)256 * gridDim.x)
      any |= p.wide[lin];
    if (!__syncthreads_or(any)) return;
  }
  __shared__ __attribute__((aligned(16))) float sG[BT * LDG];
  __shared__ __attribute__((aligned(16))) T sQ[BT * LDK];
  __shared__ __attribute__((aligned(16))) T sK[BT * LDK];
  __shared__ __attribute__((aligned(16))) T sVt[V * LDT];
  __shared__ __attribute__((aligned(16))) T sP[BT * LDT];
  __shared__ __attribute__((aligned(16))) float sPart[RG * K];
  const ExactLds<T> S{sG, sQ, sK, sVt, sP, sPart};
  for (int64_t lin = blockIdx.x; lin < p.total; lin += gridDim.x) {
    if (p.wide[lin] == 0) continue;  // workgroup-uniform
    int hh;
    ChunkLoc cl = locate_chunk_at(lin, p.offsets, p.indices, p.T, p.NTfix, H, &hh);
    gla_exact_chunk<T, GT, K, V, 256>(p, S, cl, hh, V, 0, (int)threadIdx.x);
  }
}

template <typename T, typename GT>
int launch_exact(const ExactParams& p, int K, int V, dim3 grid, hipStream_t st) {
#define FLA_CASE(KK, VV)                                                                              \
  if (K == KK && V == VV) {                                                                           \
    hipLaunchKernelGGL((gla_fwd_o_exact_kernel<T, GT, KK, VV>), grid, dim3(256), 0, st, p);           \
    FLA_CHECK_LAUNCH();                                                                               \
    return FLA_OK;                                                                                    \
  }
  FLA_CASE(64, 64)
  FLA_CASE(128, 128)
  FLA_CASE(64, 128)
  FLA_CASE(128, 64)
#undef FLA_CASE
  return FLA_E_UNSUPPORTED;
}

// K = V = 128 without kept states goes to the 128-column kernel (one workgroup per (sequence, head)) once the
// 64-column kernel would put more than one workgroup on a CU (256 CUs): 336 against 380 us at 256 heads of
// 4096 tokens.  Below that the 64-column kernel spreads a head over two CUs and is the faster one (190
// against 238 us at 128 heads).
constexpr int64_t kWideMinHeads = 128;
inline bool use_wide_kernel(const FusedParams& p, int K) {
  return K == 128 && p.V == 128 && !p.hT && (int64_t)p.N * p.H > kWideMinHeads;
}

template <typename T, typename GT, bool SG = false>
int launch_fused(const FusedParams& p, int K, hipStream_t st, bool logits = false) {
  int64_t total = (int64_t)(p.V / 64) * p.N * p.H;
  if (total == 0) return FLA_OK;
  FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  if constexpr (!SG) {
    if (logits) {
      FLA_REQUIRE(!p.hT, FLA_E_UNSUPPORTED);
      dim3 grid((unsigned)total);
      if (K == 128) hipLaunchKernelGGL((gla_fwd_fused_kernel<T, GT, 128, 4, false, false, 2, true>), grid, dim3(512), 0, st, p);
      else if (K == 64) hipLaunchKernelGGL((gla_fwd_fused_kernel<T, GT, 64, 4, false, false, 2, true>), grid, dim3(512), 0, st, p);
      else return FLA_E_UNSUPPORTED;
      FLA_CHECK_LAUNCH();
      return FLA_OK;
    }
  }
  if (use_wide_kernel(p, K)) {
    hipLaunchKernelGGL((gla_fwd_fused_wide_kernel<T, GT, SG>), dim3((unsigned)(p.N * p.H)), dim3(512), 0, st, p);
    FLA_CHECK_LAUNCH();
    return FLA_OK;
  }
  // 32-column slabs for a forward that keeps the states, while they still give every workgroup a CU of its own
  // (205 -> 187 us at B=4, H=16, T=4096; without the state stores the chunk period is set by the gating work of
  // the staging waves, which does not shrink with the slab: 157 against 158 us)
  const bool narrow = p.hT != nullptr && 2 * total <= kNumCUs;
  if (narrow) total *= 2;
  dim3 grid((unsigned)total);
#define FLA_FUSED(KK, HTV)                                                                                     \
  if (narrow) hipLaunchKernelGGL((gla_fwd_fused_kernel<T, GT, KK, 4, HTV, SG, 1>), grid, dim3(512), 0, st, p);  \
  else hipLaunchKernelGGL((gla_fwd_fused_kernel<T, GT, KK, 4, HTV, SG, 2>), grid, dim3(512), 0, st, p);
  if (p.hT) {
    if (K == 128) { FLA_FUSED(128, true) }
    else if (K == 64) { FLA_FUSED(64, true) }
    else return FLA_E_UNSUPPORTED;
  } else {
    if (K == 128) { FLA_FUSED(128, false) }
    else if (K == 64) { FLA_FUSED(64, false) }
    else return FLA_E_UNSUPPORTED;
  }
#undef FLA_FUSED
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

static int gla_fwd_fused_impl(const void* q, const void* k, const void* v, const void* gates, const float* h0,
                              void* o, float* ht, int* ws_wide, void* ws_hwide, void* h_frag_t, void* qg,
                              float* decay, const int64_t* offsets,
                              const int64_t* indices, const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                              int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K,
                              int64_t V, int64_t N, float scale, fla_stream_t stream, bool head_gates = false,
                              bool exact_pass = true, void* kh_t = nullptr, void* scores = nullptr,
                              bool logits = false, float gate_inv_norm = 1.f, float gate_clamp_min = -INFINITY) {
  FLA_REQUIRE(q && k && v && gates && o, FLA_E_INVALID);
  if (logits) FLA_REQUIRE(!head_gates && !h_frag_t, FLA_E_UNSUPPORTED);
  if (head_gates) FLA_REQUIRE(gate_dtype == FLA_F32, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE((K == 64 || K == 128) && V % 64 == 0 && V <= 1024, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((ws_wide == nullptr) == (ws_hwide == nullptr), FLA_E_INVALID);
  if (offsets) FLA_REQUIRE(B == 1 && (!ws_wide || (indices && chunk_offsets)), FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  if (ws_wide) FLA_REQUIRE(V <= 128, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)gates | (uintptr_t)o | (uintptr_t)ws_hwide) % 16 == 0,
              FLA_E_ALIGNMENT);
  if (h_frag_t) {
    FLA_REQUIRE((uintptr_t)h_frag_t % 16 == 0, FLA_E_ALIGNMENT);
    if (offsets) FLA_REQUIRE(chunk_offsets != nullptr, FLA_E_INVALID);
  }
  FLA_REQUIRE((qg == nullptr) == (decay == nullptr), FLA_E_INVALID);
  if (qg) {
    FLA_REQUIRE(h_frag_t != nullptr, FLA_E_INVALID);
    // the value slabs of a head share the rows of the kept tiles out evenly: 1, 2 or 4 slabs (8 in the narrow form)
    FLA_REQUIRE(V == 64 || V == 128 || V == 256, FLA_E_UNSUPPORTED);
    FLA_REQUIRE((uintptr_t)qg % 16 == 0, FLA_E_ALIGNMENT);
  }
  FLA_REQUIRE((kh_t == nullptr) == (scores == nullptr), FLA_E_INVALID);
  if (kh_t) {
    FLA_REQUIRE(qg != nullptr, FLA_E_INVALID);
    FLA_REQUIRE(V <= 128, FLA_E_UNSUPPORTED);   // what fla_chunk_gla_bwd_kept reads them for
    FLA_REQUIRE(((uintptr_t)kh_t | (uintptr_t)scores) % 16 == 0, FLA_E_ALIGNMENT);
  }
  FusedParams p{q, k, v, gates, h0, o, ht, offsets, chunk_offsets, seq_order, ws_wide, ws_hwide,
                T, (int)H, (int)V, (int)N, scale, h_frag_t, qg, decay, kh_t, scores, gate_inv_norm, gate_clamp_min, 0};
  hipStream_t st = (hipStream_t)stream;
  dim3 grid;
  int ntfix = 0;
  if (ws_wide) {
    int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
    if (rc) return rc;
  }
  ExactParams e{q, k, v, gates, ws_wide, ws_hwide, o, offsets, indices, T, (int)H, ntfix, scale,
                (int64_t)grid.x * grid.y, head_gates ? 1 : 0, (!logits && use_wide_kernel(p, (int)K)) ? 1 : 0,
                logits ? 1 : 0, gate_inv_norm, gate_clamp_min};
  if (ws_wide) grid = dim3((unsigned)(e.total < 512 ? e.total : 512));
  // the 64- and 32-column kernels redo flagged chunks themselves; the 128-column kernel leaves them to a second launch
  p.exact_tail = ws_wide && exact_pass && !(!logits && use_wide_kernel(p, (int)K)) ? 1 : 0;
  if (p.exact_tail) exact_pass = false;
#define FLA_FUSED(TT, GG)                                                \
  {                                                                      \
    int rc = launch_fused<TT, GG>(p, (int)K, st, logits);                \
    if (rc || !ws_wide || grid.x == 0 || !exact_pass) return rc;         \
    return launch_exact<TT, GG>(e, (int)K, (int)V, grid, st);            \
  }
  if (head_gates) {
#define FLA_FUSED_SG(TT)                                                 \
  {                                                                      \
    int rc = launch_fused<TT, float, true>(p, (int)K, st);               \
    if (rc || !ws_wide || grid.x == 0 || !exact_pass) return rc;         \
    return launch_exact<TT, float>(e, (int)K, (int)V, grid, st);         \
  }
    if (qkv_dtype == FLA_BF16) FLA_FUSED_SG(bf16)
    if (qkv_dtype == FLA_F16) FLA_FUSED_SG(f16)
#undef FLA_FUSED_SG
    return FLA_E_UNSUPPORTED;
  }
  if (qkv_dtype == FLA_BF16 && gate_dtype == FLA_F32) FLA_FUSED(bf16, float)
  if (qkv_dtype == FLA_BF16 && gate_dtype == FLA_BF16) FLA_FUSED(bf16, bf16)
  if (qkv_dtype == FLA_F16 && gate_dtype == FLA_F32) FLA_FUSED(f16, float)
  if (qkv_dtype == FLA_F16 && gate_dtype == FLA_F16) FLA_FUSED(f16, f16)
#undef FLA_FUSED
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gla_fwd_fused(const void* q, const void* k, const void* v, const void* gates, const float* h0,
                                       void* o, float* ht, int* ws_wide, void* ws_hwide, const int64_t* offsets,
                                       const int64_t* indices, const int64_t* chunk_offsets,
                                       const int64_t* seq_order, int64_t NT,
                                       int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K,
                                       int64_t V, int64_t N, float scale, fla_stream_t stream) {
  return gla_fwd_fused_impl(q, k, v, gates, h0, o, ht, ws_wide, ws_hwide, nullptr, nullptr, nullptr, offsets, indices, chunk_offsets,
                            seq_order, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream);
}

extern "C" int fla_chunk_gla_fwd_fused_first_launch(const void* q, const void* k, const void* v, const void* gates,
                                                    const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                                    const int64_t* offsets, const int64_t* indices,
                                                    const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                                    int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H,
                                                    int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream) {
  return gla_fwd_fused_impl(q, k, v, gates, h0, o, ht, ws_wide, ws_hwide, nullptr, nullptr, nullptr, offsets, indices, chunk_offsets,
                            seq_order, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream, false, false);
}

extern "C" int fla_chunk_gla_fwd_fused_states(const void* q, const void* k, const void* v, const void* gates,
                                              const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                              void* h_frag_t, const int64_t* offsets, const int64_t* indices,
                                              const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                              int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H,
                                              int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream) {
  FLA_REQUIRE(h_frag_t, FLA_E_INVALID);
  return gla_fwd_fused_impl(q, k, v, gates, h0, o, ht, ws_wide, ws_hwide, h_frag_t, nullptr, nullptr, offsets, indices, chunk_offsets,
                            seq_order, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream);
}

extern "C" int fla_chunk_gla_fwd_fused_kept(const void* q, const void* k, const void* v, const void* gates,
                                            const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                            void* h_frag_t, void* q_gated, float* chunk_decay, void* khat_t,
                                            void* scores, const int64_t* offsets,
                                            const int64_t* indices, const int64_t* chunk_offsets,
                                            const int64_t* seq_order, int64_t NT, int qkv_dtype, int gate_dtype,
                                            int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                            float scale, fla_stream_t stream) {
  FLA_REQUIRE(h_frag_t && q_gated && chunk_decay, FLA_E_INVALID);
  return gla_fwd_fused_impl(q, k, v, gates, h0, o, ht, ws_wide, ws_hwide, h_frag_t, q_gated, chunk_decay, offsets,
                            indices, chunk_offsets, seq_order, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream,
                            false, true, khat_t, scores);
}

extern "C" int fla_chunk_simple_gla_fwd_fused(const void* q, const void* k, const void* v, const float* g,
                                              const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                              void* h_frag_t, void* q_gated, float* chunk_decay, void* khat_t,
                                              void* scores, const int64_t* offsets, const int64_t* indices,
                                              const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                              int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                              int64_t N, float scale, fla_stream_t stream) {
  return gla_fwd_fused_impl(q, k, v, g, h0, o, ht, ws_wide, ws_hwide, h_frag_t, q_gated, chunk_decay, offsets, indices, chunk_offsets,
                            seq_order, NT, qkv_dtype, FLA_F32, B, T, H, K, V, N, scale, stream, true, true, khat_t, scores);
}

extern "C" int fla_chunk_gla_fwd_fused_logits(const void* q, const void* k, const void* v, const void* gate_logits,
                                              const float* h0, void* o, float* ht, int* ws_wide, void* ws_hwide,
                                              const int64_t* offsets, const int64_t* indices,
                                              const int64_t* chunk_offsets, const int64_t* seq_order, int64_t NT,
                                              int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H,
                                              int64_t K, int64_t V, int64_t N, float scale, float normalizer,
                                              int has_clamp, float clamp_min, fla_stream_t stream) {
  FLA_REQUIRE(normalizer != 0.f, FLA_E_INVALID);
  return gla_fwd_fused_impl(q, k, v, gate_logits, h0, o, ht, ws_wide, ws_hwide, nullptr, nullptr, nullptr, offsets,
                            indices, chunk_offsets, seq_order, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale,
                            stream, false, true, nullptr, nullptr, true, 1.f / normalizer,
                            has_clamp ? clamp_min : -INFINITY);
}
