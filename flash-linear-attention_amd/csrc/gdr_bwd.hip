// Chunked gated delta rule backward for gfx950 (chunk size 64).
//
// Notation (per chunk and head): gamma = chunk-local prefix sum of g, Gamma_ij =
// e^{gamma_i-gamma_j} (j<=i), kb = beta*k, vb = beta*v, M = strict_lower(kb k^T),
// Aw = (I+M)^-1, Au = Aw*Gamma, w = Aw kb, u = Au vb, v_new = u - (w e^gamma) h_c,
// dH_c = gradient w.r.t. the state LEAVING chunk c.  Follows
// fla/ops/gated_delta_rule/chunk.py:76-177:
//
//   gdr_bwd_dvlocal_kernel   dv_loc = (s tril(q k^T * Gamma))^T do               (chunk_o.py:379-441)
//   gdr_bwd_dhu_kernel       reverse scan per (sequence, head, 32 value columns):
//                              store dH_c;  dv2 = dv_loc + (k e^{gamma_last-gamma}) dH_c;
//                              dH <- e^{gamma_last} dH + (s q e^gamma)^T do - (w e^gamma)^T dv2
//                                                                                (chunk_delta_h.py:136-237)
//   gdr_bwd_dqkwg_kernel     per (chunk, head, 64-wide half of K):
//                              ds = s tril((do v_new^T) * Gamma)
//                              dq = s e^gamma (do h_c^T) + ds k
//                              dk = e^{gamma_last-gamma} (v_new dH_c^T) + ds^T q
//                              dw = -e^gamma (dv2 h_c^T)
//                              dgamma_i = sum_k (q*dq - k*dk + w*dw)_ik
//                                         + [i last] (sum_jk k*dk_inter + e^{gamma_last} <h_c, dH_c>)
//                            (chunk_o.py:118-265; the row/column sums of ds*(q k^T) there equal
//                            sum_k q*dq_intra - k*dk_intra, so no second score matrix is formed)
//   gdr_bwd_wy_kernel        gradient through the WY representation:
//                              d(kb) = Aw^T dw, d(vb) = Au^T du,
//                              dAw = strict_lower(dw kb^T) + strict_lower(du vb^T) * Gamma,
//                              dM = -strict_lower(Aw^T dAw Aw^T),
//                              d(kb) += dM k, dk = beta d(kb) + dM^T kb, dv = beta d(vb),
//                              dbeta = sum d(kb)*k + sum d(vb)*v,
//                              dgamma_i += rowsum_i(X) - colsum_i(X), X = strict_lower(du vb^T) * Au
//                            (wy_fast.py:440-562, written for the single inverse Aw).
#include <type_traits>

#include "chunk_common.h"

namespace {

// ---------------------------------------------------------------------------
struct DvlParams {
  const void* q;
  const void* k;
  const void* dout;
  const float* gam;
  void* dvl;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  float scale;
};

template <typename T, int K, int V>
__global__ __launch_bounds__(256) void gdr_bwd_dvlocal_kernel(DvlParams p, uint32_t nitems) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int C8 = K / 8, NP = BT * C8 / 256;
  constexpr int CGV = V / 4, RGV = 256 / CGV, RPTV = BT / RGV;
  constexpr int TV = V / 64;
  constexpr int LDV = V + 8;
  __shared__ __attribute__((aligned(16))) T sQ[BT * (K > V ? LDK : LDV)];   // q; later the dv tile [t][v]
  __shared__ __attribute__((aligned(16))) T sK[BT * LDK];
  __shared__ __attribute__((aligned(16))) T sDt[V * LDT];
  __shared__ __attribute__((aligned(16))) T sPT[BT * LDT];
  __shared__ float sGam[BT];
  const int tid0 = threadIdx.x;
  const int H = p.H;
  // A workgroup walks (chunk, head) items with a stride of the grid size; the rows of the next item are
  // requested as soon as those of the current one are in LDS (32-bit offsets off wave-uniform bases; rows past
  // the end of a short chunk re-read its last row and are masked at use, so no load sits under a branch).
  struct Item {
    ChunkLoc cl;
    int hh;
  };
  auto locate = [&](uint32_t it) {
    Item r;
    r.cl = locate_chunk_at32(it, p.offsets, p.indices, p.T, p.NTfix, H, &r.hh);
    return r;
  };
  struct Raw {
    v8 q[NP], k[NP];
    v4 d[RPTV];
    float gam;
  };
  const uint32_t pitchk = (uint32_t)H * K * (uint32_t)sizeof(T), pitchv = (uint32_t)H * V * (uint32_t)sizeof(T);
  uint32_t offk[NP], offv[RPTV];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid0 + 256 * i;
    offk[i] = (uint32_t)(e / C8) * pitchk + (uint32_t)((e % C8) * 8) * (uint32_t)sizeof(T);
  }
#pragma unroll
  for (int i = 0; i < RPTV; ++i)
    offv[i] = (uint32_t)((tid0 / CGV) * RPTV + i) * pitchv + (uint32_t)((tid0 % CGV) * 4) * (uint32_t)sizeof(T);
  const uint32_t colk = (uint32_t)((tid0 % C8) * 8) * (uint32_t)sizeof(T), colv = (uint32_t)((tid0 % CGV) * 4) * (uint32_t)sizeof(T);
  auto request = [&](const Item& im, Raw& R) __attribute__((always_inline)) {
    const uint32_t last = (uint32_t)(im.cl.L - 1);
    const int64_t r0h = im.cl.row0 * H + im.hh;
    const char* qb = (const char*)p.q + r0h * K * (int64_t)sizeof(T);
    const char* kb = (const char*)p.k + r0h * K * (int64_t)sizeof(T);
    const char* db = (const char*)p.dout + r0h * V * (int64_t)sizeof(T);
    const uint32_t limk = last * pitchk + colk, limv = last * pitchv + colv;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const uint32_t o = offk[i] < limk ? offk[i] : limk;
      R.q[i] = *(const v8*)(qb + o);
      R.k[i] = *(const v8*)(kb + o);
    }
#pragma unroll
    for (int i = 0; i < RPTV; ++i) R.d[i] = *(const v4*)(db + (offv[i] < limv ? offv[i] : limv));
    const uint32_t grow = (uint32_t)(tid0 & (BT - 1)) < last ? (uint32_t)(tid0 & (BT - 1)) : last;
    R.gam = p.gam ? p.gam[(im.cl.row0 + grow) * H + im.hh] : 0.f;
  };
  uint32_t it = blockIdx.x;
  if (it >= nitems) return;
  Item im = locate(it);
  Raw R;
  request(im, R);
  const v8 z8 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};
  for (;;) {
  // (the lane id goes through an opaque copy once per item, so that the LDS addresses of the body are formed
  // where they are used instead of being hoisted out of the loop into long-lived registers)
  int tid = tid0;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = im.hh;
  const int L = im.cl.L;
  const int64_t row0 = im.cl.row0;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    *(v8*)&sQ[row * LDK + c8] = row < L ? R.q[i] : z8;
    *(v8*)&sK[row * LDK + c8] = row < L ? R.k[i] : z8;
  }
  const int rgv = tid / CGV, cv4 = (tid % CGV) * 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    T* dst = &sDt[(cv4 + j) * LDT + rgv * RPTV];
#pragma unroll
    for (int i = 0; i < RPTV; ++i) dst[i] = rgv * RPTV + i < L ? R.d[i][j] : (T)0.f;
  }
  if (tid < BT) sGam[tid] = R.gam;
  const uint32_t nit = it + gridDim.x;
  const bool more = nit < nitems;   // workgroup-uniform
  const Item nim = locate(more ? nit : it);   // (past the last item the request repeats it)
  request(nim, R);
  __syncthreads();
  {
    const int qi = wave >> 1, qj = wave & 1;
    if (qj <= qi) {
      f32x16 s = zero16();
#pragma unroll
      for (int ks = 0; ks < K; ks += 16)
        s = Elem<T>::mfma32(lds_frag32<T>(sQ, LDK, qi * 32, ks, lane), lds_frag32<T>(sK, LDK, qj * 32, ks, lane), s);
      const int j = qj * 32 + (lane & 31);
      const float gj = sGam[j];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int i0 = qi * 32 + 8 * a + 4 * (lane >> 5);
        v4 x;
#pragma unroll
        for (int b = 0; b < 4; ++b)
          x[b] = (T)((j <= i0 + b) ? s[4 * a + b] * p.scale * __expf(sGam[i0 + b] - gj) : 0.f);
        *(v4*)&sPT[j * LDT + i0] = x;
      }
    }
  }
  __syncthreads();
  const int rw = wave >> 1, cw = wave & 1;
  f32x16 acc[TV];
#pragma unroll
  for (int tv = 0; tv < TV; ++tv) acc[tv] = zero16();
  // transposed product (do^T A): a lane ends up with one time row and four consecutive value
  // columns per register quad; the tile leaves through LDS (the q tile is dead) as whole rows
  for (int is = rw * 32; is < BT; is += 16) {
    v8 a = lds_frag32<T>(sPT, LDT, rw * 32, is, lane);
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
      acc[tv] = Elem<T>::mfma32(lds_frag32<T>(sDt, LDT, (cw * TV + tv) * 32, is, lane), a, acc[tv]);
  }
  T* sO = sQ;
  {
    T* orow = &sO[(rw * 32 + (lane & 31)) * LDV + cw * TV * 32 + 4 * (lane >> 5)];
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        v4 x;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = (T)acc[tv][4 * r4 + e];
        *(v4*)(orow + tv * 32 + 8 * r4) = x;
      }
  }
  __syncthreads();
  constexpr int C8V = V / 8;
  T* op = (T*)p.dvl + (row0 * H + hh) * (int64_t)V;
#pragma unroll
  for (int i = 0; i < BT * C8V / 256; ++i) {
    const int e = tid + 256 * i, row = e / C8V, c8 = (e % C8V) * 8;
    if (row < L) *(v8*)(op + (int64_t)row * H * V + c8) = *(const v8*)&sO[row * LDV + c8];
  }
  if (!more) break;
  __syncthreads();  // the dv tile is on its way: the next item's tiles may be written
  it = nit;
  im = nim;
  }
}

// ---------------------------------------------------------------------------
struct DhuParams {
  const void* q;
  const void* k;
  const void* w;
  const void* dout;
  const void* dvl;
  const void* Aqk;   // FROMP: the packed score tiles the forward kept, [chunks, H, 10, 16, 16] (dvl unused)
  const float* gam;
  const float* dht;
  void* dv2;
  void* dhtf;   // dH, FLA_H_FRAGMENT_T
  float* dh0;
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  int64_t T;
  int H, V, N;
  float scale;
};

// One workgroup of eight waves: all K rows x 32 value columns of one (sequence, head).
// Waves 0-3 ("matrix") carry the state gradient and do the two products of a chunk; waves 4-7 ("staging") load
// the next chunk's rows, write the operand tiles and store dv2.  (With one four-wave workgroup per CU every SIMD
// held a single wave that alternated between the two kinds of work: 55 % of a chunk period went into staging
// while the matrix pipe idled, and two workgroups per CU overlapped perfectly - so the second wave per SIMD is
// brought along instead.)  Per chunk c (walking backwards) the groups meet twice:
//   B1(c)  k, dv_loc and the gates of chunk c and the 16-bit dH are in LDS
//          matrix:  dv2 = dv_loc + e^{gamma_last-gamma} * (k dH) -> LDS, and -e^{gamma} * dv2 beside it
//          staging: q, w and s e^{gamma} * do of chunk c -> LDS
//   B2(c)  matrix:  dH <- e^{gamma_last} dH + q^T (s e^{gamma} * do) + w^T (-e^{gamma} * dv2); publishes dH
//          staging: dv2 of chunk c -> memory; k, dv_loc, gates of chunk c-1 -> LDS
// Each tile is written in the half of the period in which the matrix waves read the other kind, so nothing is
// double-buffered.  The gates are per (token, head): as row scalings they commute out of the K-wide operands
// onto the 32-column ones (do, dv2) and onto the product k dH, so q, w and k are staged as plain 16-byte copies -
// the staging waves are bound by the instructions they issue (a memory instruction costs the issuing wave about
// 70 cycles once the CU's memory pipeline is full), the matrix waves have time to spare - and every transposed
// operand is read from a row-major tile with the transposing LDS load.
// FROMP: dv_loc = Aqk^T do is not read from memory but formed here from the packed score tile Aqk the forward
// kept (5 KB per chunk and head) and the raw do rows, which then travel with the k group: four more small
// matrix products per wave and chunk instead of a launch that reads q, k, do and writes dv_loc.
template <typename T, int K, bool FROMP>
__global__ __launch_bounds__(512) void gdr_bwd_dhu_kernel(DhuParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int BV = 32;
  constexpr int LDK = K + 8;
  constexpr int LDV = BV + 8;
  constexpr int C8 = K / 8, NP = BT * C8 / 256;   // q, w, k: 16-byte pieces per row / per staging lane
  constexpr int PR = 256 / C8;                    // rows between two pieces of a lane
  constexpr int KT32 = K / 32;
  constexpr int NKT = (KT32 + 3) / 4;
  __shared__ __attribute__((aligned(16))) T sK[BT * LDK];      // k, row-major
  __shared__ __attribute__((aligned(16))) T sQ[BT * LDK];      // q, row-major
  __shared__ __attribute__((aligned(16))) T sW[BT * LDK];      // w, row-major
  __shared__ __attribute__((aligned(16))) T sDo[BT * LDV];     // s e^{gamma} * do, row-major [t][v]
  __shared__ __attribute__((aligned(16))) T sDvl[BT * LDV];    // dv_loc (FROMP: do), row-major [t][v]
  __shared__ __attribute__((aligned(16))) T sP[FROMP ? kTriElems : 8];   // FROMP: Aqk, packed triangular tile
  __shared__ __attribute__((aligned(16))) T sDHt[BV * LDK];    // dH^T in 16-bit
  __shared__ __attribute__((aligned(16))) T sDv2T[BV * LDT];   // dv2^T
  __shared__ __attribute__((aligned(16))) T sDv2s[BV * LDT];   // (-e^{gamma} * dv2)^T
  __shared__ __attribute__((aligned(16))) float sEg[BT];       // e^{gamma_t} (0 past the end of a short chunk)
  __shared__ __attribute__((aligned(16))) float sEd[BT];       // e^{gamma_last - gamma_t} (0 past the end)
  __shared__ float sDec[2];                                     // e^{gamma_last} of chunk c at [c & 1]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };

  if (wave >= 4) {
    // =========================== staging waves ===========================
    if (nchunks == 0) return;
    const int st = tid - 256;
    const int prow = st / C8, c8 = (st % C8) * 8;   // piece i of a lane: row prow + PR i, columns c8 ..
    const int vrow = st >> 2, vc8 = (st & 3) * 8;   // do, dv_loc, dv2: one row, 8 of the 32 columns
    struct XRegs {
      v8 q[NP];
      v8 w[NP];
      v8 d;
    };
    struct YRegs {
      v8 k[NP];
      v8 dvl;       // FROMP: do
      v8 a0, a1;    // FROMP: pieces of the score tile
      float gam, glast;
    };
    // Loads are unconditional (a load under a branch makes the wave drain its whole load queue at the
    // join): byte offsets of this lane's rows from the first row of a chunk are computed once, rows past
    // the end of a short chunk are redirected to its last row, chunks before the first one to chunk 0.
    // What a redirected row holds never counts: its gate factors are zero.
    const uint32_t pitchK = (uint32_t)H * K * (uint32_t)sizeof(T), pitchV = (uint32_t)H * V * (uint32_t)sizeof(T);
    const uint32_t pitchG = (uint32_t)H * 4u;
    uint32_t offk[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) offk[i] = (uint32_t)(prow + PR * i) * pitchK + (uint32_t)c8 * (uint32_t)sizeof(T);
    const uint32_t offv = (uint32_t)vrow * pitchV + (uint32_t)vc8 * (uint32_t)sizeof(T);
    const uint32_t offg = (uint32_t)vrow * pitchG;
    const char* gq = (const char*)p.q + (sp.bos * H + hh) * (int64_t)K * (int64_t)sizeof(T);
    const char* gk = (const char*)p.k + (sp.bos * H + hh) * (int64_t)K * (int64_t)sizeof(T);
    const char* gw = (const char*)p.w + (sp.bos * H + hh) * (int64_t)K * (int64_t)sizeof(T);
    const char* gd = (const char*)p.dout + ((sp.bos * H + hh) * (int64_t)V + vbase) * (int64_t)sizeof(T);
    const char* gl = FROMP ? gd : (const char*)p.dvl + ((sp.bos * H + hh) * (int64_t)V + vbase) * (int64_t)sizeof(T);
    const char* ga = FROMP ? (const char*)p.Aqk + (chunk0 * H + hh) * (int64_t)kTriElems * (int64_t)sizeof(T) : nullptr;
    const uint32_t offa0 = 16 * (uint32_t)st, offa1 = 16 * (uint32_t)(256 + (st & 63));
    // without gates every gate load reads one zero word (no select on the loaded value: it would
    // make the wave wait for the load where it is issued)
    const char* gg = p.gam ? (const char*)p.gam + (sp.bos * H + hh) * 4 : (const char*)&kZeroWord;
    auto load_x = [&](int64_t c, XRegs& R) __attribute__((always_inline)) {
      c = c < 0 ? 0 : c;
      const uint32_t last = (uint32_t)(chunk_len(c) - 1);
      const int64_t ck = c * BT * (int64_t)pitchK, cv = c * BT * (int64_t)pitchV;
      const uint32_t lk = last * pitchK + (uint32_t)c8 * (uint32_t)sizeof(T);
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        const uint32_t o = offk[i] < lk ? offk[i] : lk;
        R.q[i] = *(const v8*)(gq + ck + o);
        R.w[i] = *(const v8*)(gw + ck + o);
      }
      if constexpr (!FROMP) {
        const uint32_t lv = last * pitchV + (uint32_t)vc8 * (uint32_t)sizeof(T);
        R.d = *(const v8*)(gd + cv + (offv < lv ? offv : lv));
      }
    };
    auto load_y = [&](int64_t c, YRegs& R) __attribute__((always_inline)) {
      c = c < 0 ? 0 : c;
      const uint32_t last = (uint32_t)(chunk_len(c) - 1);
      const int64_t ck = c * BT * (int64_t)pitchK, cv = c * BT * (int64_t)pitchV, cg = p.gam ? c * BT * (int64_t)pitchG : 0;
      const uint32_t lk = last * pitchK + (uint32_t)c8 * (uint32_t)sizeof(T);
#pragma unroll
      for (int i = 0; i < NP; ++i) R.k[i] = *(const v8*)(gk + ck + (offk[i] < lk ? offk[i] : lk));
      const uint32_t lv = last * pitchV + (uint32_t)vc8 * (uint32_t)sizeof(T);
      R.dvl = *(const v8*)(gl + cv + (offv < lv ? offv : lv));
      if constexpr (FROMP) {
        const char* pa = ga + c * (int64_t)H * kTriElems * (int64_t)sizeof(T);
        R.a0 = *(const v8*)(pa + offa0);
        R.a1 = *(const v8*)(pa + offa1);   // the last 64 pieces: every wave loads them, the first one writes them
      }
      const uint32_t og = offg < last * pitchG ? offg : last * pitchG;
      R.gam = *(const float*)(gg + cg + (p.gam ? og : 0u));
      R.glast = *(const float*)(gg + cg + (p.gam ? last * pitchG : 0u));
    };
    // s e^{gamma} of this lane's do row in the chunk held in X (zero past its end): formed when the same chunk
    // is staged as Y, half a period earlier, so that nothing loop-carried depends on a load in flight
    float egx = 0.f;
    v8 dkeep;   // FROMP: this lane's do piece of the chunk last staged as Y
    auto stage_x = [&](const XRegs& R) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < NP; ++i) {
        *(v8*)&sQ[(prow + PR * i) * LDK + c8] = R.q[i];
        *(v8*)&sW[(prow + PR * i) * LDK + c8] = R.w[i];
      }
      v8 x;
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = (T)((float)(FROMP ? dkeep[j] : R.d[j]) * egx);
      *(v8*)&sDo[vrow * LDV + vc8] = x;
    };
    auto stage_y = [&](const YRegs& R, int64_t c) __attribute__((always_inline)) {
      const int L = chunk_len(c);
#pragma unroll
      for (int i = 0; i < NP; ++i) *(v8*)&sK[(prow + PR * i) * LDK + c8] = R.k[i];
      *(v8*)&sDvl[vrow * LDV + vc8] = R.dvl;
      if constexpr (FROMP) {
        dkeep = R.dvl;
        *(v8*)&sP[st * 8] = R.a0;
        if (wave == 4) *(v8*)&sP[2048 + lane * 8] = R.a1;
      }
      const float eg = vrow < L ? __expf(R.gam) : 0.f;
      egx = p.scale * eg;
      if ((st & 3) == 0) {
        sEg[vrow] = eg;
        sEd[vrow] = vrow < L ? __expf(R.glast - R.gam) : 0.f;
      }
      if (st == 0) sDec[c & 1] = __expf(R.glast);
    };
    // dv2 of chunk c leaves as whole rows, 16 bytes per lane: a 16-lane group turns a block of 8 value columns x
    // 16 time rows of the transposed tile round with two transposing LDS loads (lane j ends up with time row
    // 16 tb + j, columns 8 vb ..).  Only a sequence's last chunk (the first one processed) can be short: it takes
    // the variant with the masked store, the steady state stores unconditionally.
    const int dgrp = st >> 4, dtb = dgrp >> 2, dvb = dgrp & 3, dj = st & 15;
    const int dsrc = (8 * dvb + (dj >> 2)) * LDT + 16 * dtb + 4 * (dj & 3);
    auto store_dv2 = [&](int64_t c, auto maybe_short) __attribute__((always_inline)) {
      typedef short s4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) s4 lds_s4;
      s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sDv2T[dsrc]);
      s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sDv2T[dsrc + 4 * LDT]);
      const v8 x = __builtin_shufflevector(__builtin_bit_cast(v4, lo), __builtin_bit_cast(v4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
      const int row = 16 * dtb + dj;
      T* dst = (T*)p.dv2 + ((sp.bos + c * BT + row) * H + hh) * (int64_t)V + vbase + 8 * dvb;
      if constexpr (decltype(maybe_short)::value) {
        if (row < chunk_len(c)) *(v8*)dst = x;
      } else {
        *(v8*)dst = x;
      }
    };
    XRegs X;
    YRegs Y;
    load_x(nchunks - 1, X);
    load_y(nchunks - 1, Y);
    stage_y(Y, nchunks - 1);
    load_y(nchunks - 2, Y);
    // The first chunk of the sequence (processed last) and its last one (processed first, possibly short) are
    // peeled off so that the steady-state loop has no memory operation under a branch.
    if (nchunks > 1) {
      lds_barrier();  // B1(nchunks - 1)
      stage_x(X);
      load_x(nchunks - 2, X);
      lds_barrier();  // B2(nchunks - 1)
      store_dv2(nchunks - 1, std::true_type{});
      stage_y(Y, nchunks - 2);
      load_y(nchunks - 3, Y);
      for (int64_t c = nchunks - 2; c >= 1; --c) {
        lds_barrier();  // B1(c)
        stage_x(X);
        load_x(c - 1, X);
        lds_barrier();  // B2(c)
        store_dv2(c, std::false_type{});
        stage_y(Y, c - 1);
        load_y(c - 2, Y);
      }
    }
    lds_barrier();  // B1(0)
    stage_x(X);
    lds_barrier();  // B2(0)
    store_dv2(0, std::true_type{});
  } else {
    // =========================== matrix waves ===========================
    f32x16 acc[NKT], acct[NKT];
#pragma unroll
    for (int a = 0; a < NKT; ++a) {
      acc[a] = zero16();
      acct[a] = zero16();
      int kt = wave + 4 * a;
      if (p.dht && kt < KT32) {
        const float* d0 = p.dht + (int64_t)nh * K * V;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[a][r] = d0[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)];
          acct[a][r] = d0[(int64_t)(kt * 32 + (lane & 31)) * V + vbase + c32_row(r, lane)];
        }
      }
    }
    // gradient w.r.t. the state leaving chunk c: 16-bit transpose in LDS, FRAGMENT_T copy in HBM
    auto publish = [&](int64_t c) __attribute__((always_inline)) {
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            v4 x;
#pragma unroll
            for (int b = 0; b < 4; ++b) x[b] = (T)acc[a][4 * q4 + b];
            *(v4*)&sDHt[(lane & 31) * LDK + kt * 32 + 8 * q4 + 4 * (lane >> 5)] = x;
          }
          v8 lo, hi;
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            lo[r] = (T)acct[a][r];
            hi[r] = (T)acct[a][r + 8];
          }
          T* hp = (T*)p.dhtf + ((chunk0 + c) * H + hh) * (int64_t)K * V + (((int64_t)vt * (K / 32) + kt) * 64 + lane) * 16;
          *(v8*)hp = lo;
          *(v8*)(hp + 8) = hi;
        }
      }
    };
    if (nchunks > 0) publish(nchunks - 1);
    for (int64_t c = nchunks - 1; c >= 0; --c) {
      lds_barrier();  // B1(c)
      // ---- dv2 = dv_loc + e^{gamma_last-gamma} * (k dH): wave w owns rows 16w..16w+15, two 16-column tiles
      {
        f32x4 d[2] = {zero4(), zero4()};
#pragma unroll
        for (int ks = 0; ks < K; ks += 32) {
          v8 a = lds_frag16<T>(sK, LDK, wave * 16, ks, lane);
#pragma unroll
          for (int j = 0; j < 2; ++j) d[j] = Elem<T>::mfma16(a, lds_frag16<T>(sDHt, LDK, j * 16, ks, lane), d[j]);
        }
        const int tr = wave * 16 + 4 * (lane >> 4);
        const f32x4 ed = *(const f32x4*)&sEd[tr], eg = *(const f32x4*)&sEg[tr];
        f32x4 dl[2] = {zero4(), zero4()};
        if constexpr (FROMP) {
          // dv_loc rows 16 wave ..: sum over the time rows i of Aqk[i][t] do[i][v]; Aqk^T comes out of the
          // row-major 16x16 blocks (row blocks 2s and 2s+1 of column block `wave`) through the transposing load,
          // blocks above the diagonal are not stored
          typedef short s4 __attribute__((ext_vector_type(4)));
          typedef __attribute__((address_space(3))) s4 lds_s4;
          const int jj = lane & 15, gg = lane >> 4;
          const int off = (4 * gg + (jj >> 2)) * 16 + 4 * (jj & 3);
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int t0 = 2 * s, t1 = 2 * s + 1;
            if (t1 < wave) continue;   // wave-uniform
            s4 lo = {0, 0, 0, 0};
            if (t0 >= wave) lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sP[(t0 * (t0 + 1) / 2 + wave) * 256 + off]);
            s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sP[(t1 * (t1 + 1) / 2 + wave) * 256 + off]);
            const v8 a = __builtin_shufflevector(__builtin_bit_cast(v4, lo), __builtin_bit_cast(v4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int j = 0; j < 2; ++j) dl[j] = Elem<T>::mfma16(a, frag16_tr<T>(sDvl, LDV, 16 * j, 32 * s, lane), dl[j]);
          }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          int vc = j * 16 + (lane & 15);
          v4 o, os;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x = (FROMP ? dl[j][r] : (float)sDvl[(tr + r) * LDV + vc]) + ed[r] * d[j][r];
            o[r] = (T)x;
            os[r] = (T)(-eg[r] * x);
          }
          *(v4*)&sDv2T[vc * LDT + tr] = o;
          *(v4*)&sDv2s[vc * LDT + tr] = os;
        }
      }
      lds_barrier();  // B2(c)
      // ---- dH <- e^{gamma_last} dH + q^T (s e^gamma * do) + w^T (-e^gamma * dv2), in both orientations
      const float dec_c = sDec[c & 1];
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            acc[a][r] *= dec_c;
            acct[a][r] *= dec_c;
          }
#pragma unroll
          for (int s = 0; s < BT; s += 16) {
            v8 fq = frag32_tr<T>(sQ, LDK, kt * 32, s, lane);
            v8 fd = frag32_tr<T>(sDo, LDV, 0, s, lane);
            v8 fw = frag32_tr<T>(sW, LDK, kt * 32, s, lane);
            v8 f2 = lds_frag32<T>(sDv2s, LDT, 0, s, lane);
            acc[a] = Elem<T>::mfma32(fq, fd, acc[a]);
            acc[a] = Elem<T>::mfma32(fw, f2, acc[a]);
            acct[a] = Elem<T>::mfma32(fd, fq, acct[a]);
            acct[a] = Elem<T>::mfma32(f2, fw, acct[a]);
          }
        }
      }
      if (c > 0) publish(c - 1);
    }
    if (p.dh0) {
      float* o = p.dh0 + (int64_t)nh * K * V;
#pragma unroll
      for (int a = 0; a < NKT; ++a) {
        int kt = wave + 4 * a;
        if (kt < KT32) {
#pragma unroll
          for (int r = 0; r < 16; ++r) o[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] = acc[a][r];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
struct DqkwgParams {
  const void* q;
  const void* k;
  const void* vnew;
  const void* w;
  const void* dout;
  const void* dv2;
  const float* gam;
  const void* hT;     // forward states, FLA_H_FRAGMENT_T
  const void* dhtf;   // dH, FLA_H_FRAGMENT_T
  void* dq;
  void* dk;           // partial: everything except the WY path
  void* dw;
  float* dgam;        // [K/64][B*T][H] partial per key slice
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int64_t total_rows;
  int H, K, NTfix;
  float scale;
};

template <typename T, int V>
__global__ __launch_bounds__(256, 2) void gdr_bwd_dqkwg_kernel(DqkwgParams p, int64_t pairs) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDV = V + 8;
  constexpr int C8 = V / 8, NP = BT * C8 / 256;
  constexpr int VT32 = V / 32;
  constexpr int ROWB = BT * LDV * 2;
  constexpr int STG = BT * LDM * 4;
  constexpr int REG_A = ROWB > STG ? ROWB : STG;
  constexpr int REG_C = (2 * BT * LDT * 2 > STG) ? 2 * BT * LDT * 2 : STG;
  __shared__ __attribute__((aligned(16))) char sRA[REG_A];  // do row-major -> dv2 row-major -> staging (dq)
  __shared__ __attribute__((aligned(16))) char sRB[REG_A];  // v_new row-major -> staging (dk intra)
  __shared__ __attribute__((aligned(16))) char sRC[REG_C];  // k^T | q^T -> staging (dk inter)
  __shared__ __attribute__((aligned(16))) char sRD[REG_C];  // ds | ds^T -> staging (dw)
  __shared__ __attribute__((aligned(16))) float sGam[BT];
  T* sDo = (T*)sRA;
  T* sVn = (T*)sRB;
  T* sKT = (T*)sRC;
  T* sQT = sKT + BT * LDT;
  T* sDs = (T*)sRD;
  T* sDsT = sDs + BT * LDT;
  float* stA = (float*)sRA;
  float* stB = (float*)sRB;
  float* stC = (float*)sRC;
  float* stD = (float*)sRD;

  const int tid0 = threadIdx.x;
  const int H = p.H, K = p.K;
  // A workgroup walks items (chunk, head, key slice) with a stride of the grid size.  The key slices of one
  // (chunk, head) share do, v_new and dv2: where the counts allow, they are items 8 apart, i.e. they run at the
  // same time on the same XCD, and the second slice finds those tiles in that XCD's L2.
  const int nz = K / 64;
  const uint32_t nitems = (uint32_t)pairs * (uint32_t)nz;   // < 2^31, checked by the launcher
  const bool paired = nitems % (8 * nz) == 0 && gridDim.x % (8 * nz) == 0;
  struct Item {
    ChunkLoc cl;
    int hh, kb;
  };
  auto locate = [&](uint32_t it) {
    Item r;
    const uint32_t unz = (uint32_t)nz;
    const uint32_t pair = paired ? (it / (8 * unz)) * 8 + it % 8 : it / unz;
    r.kb = (int)(paired ? (it / 8) % unz : it % unz) * 64;
    r.cl = locate_chunk_at32(pair, p.offsets, p.indices, p.T, p.NTfix, H, &r.hh);
    return r;
  };
  // The rows an item starts with (q, k, w slice: 4 rows x 4 columns per lane; do, v_new: whole rows in 16-byte
  // pieces) are requested while the item before it is in its epilogue; rows past the end of a short chunk
  // re-read its last row (masked at use), so no load sits under a branch.
  const int rg0 = tid0 >> 4, c40 = (tid0 & 15) * 4;
  struct Raw {
    v4 q[4], k[4], w[4];
    v8 d[NP], v[NP];
    float gam;   // the gate row of lane % 64
  };
  // byte offsets of this lane's pieces from the first row of a chunk (32-bit, off wave-uniform base pointers)
  const uint32_t pitchk = (uint32_t)H * K * (uint32_t)sizeof(T), pitchv = (uint32_t)H * V * (uint32_t)sizeof(T);
  uint32_t offk[4], offv[NP];
#pragma unroll
  for (int i = 0; i < 4; ++i) offk[i] = (uint32_t)(rg0 * 4 + i) * pitchk + (uint32_t)c40 * (uint32_t)sizeof(T);
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid0 + 256 * i;
    offv[i] = (uint32_t)(e / C8) * pitchv + (uint32_t)((e % C8) * 8) * (uint32_t)sizeof(T);
  }
  const uint32_t colk = (uint32_t)c40 * (uint32_t)sizeof(T), colv = (uint32_t)((tid0 % C8) * 8) * (uint32_t)sizeof(T);
  auto request = [&](const Item& im, Raw& R) __attribute__((always_inline)) {
    const uint32_t last = (uint32_t)(im.cl.L - 1);
    const int64_t r0h = im.cl.row0 * H + im.hh;
    const char* qb = (const char*)p.q + (r0h * K + im.kb) * (int64_t)sizeof(T);
    const char* kb_ = (const char*)p.k + (r0h * K + im.kb) * (int64_t)sizeof(T);
    const char* wb = (const char*)p.w + (r0h * K + im.kb) * (int64_t)sizeof(T);
    const char* db = (const char*)p.dout + r0h * V * (int64_t)sizeof(T);
    const char* vb = (const char*)p.vnew + r0h * V * (int64_t)sizeof(T);
    const uint32_t limk = last * pitchk + colk, limv = last * pitchv + colv;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t o = offk[i] < limk ? offk[i] : limk;
      R.q[i] = *(const v4*)(qb + o);
      R.k[i] = *(const v4*)(kb_ + o);
      R.w[i] = *(const v4*)(wb + o);
    }
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const uint32_t o = offv[i] < limv ? offv[i] : limv;
      R.d[i] = *(const v8*)(db + o);
      R.v[i] = *(const v8*)(vb + o);
    }
    // with the rows, not behind the state fragments the item itself asks for: a value that goes to LDS right away
    // would otherwise wait for every load queued in front of it (without gates: one zero word, no branch)
    const uint32_t grow = (uint32_t)(tid0 & (BT - 1)) < last ? (uint32_t)(tid0 & (BT - 1)) : last;
    R.gam = *(p.gam ? p.gam + (im.cl.row0 + grow) * H + im.hh : &kZeroWord);
  };
  uint32_t it = blockIdx.x;
  if (it >= nitems) return;
  Item im = locate(it);
  Raw R;
  request(im, R);
  const v8 z8 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};
  for (;;) {
  // The lane id goes through an opaque copy once per item: the LDS addresses of the body are then formed where
  // they are used instead of being hoisted out of the loop into a hundred long-lived registers.
  int tid = tid0;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rg = tid >> 4, c4 = (tid & 15) * 4;
  const int hh = im.hh, kb = im.kb;
  const ChunkLoc cl = im.cl;
  const int L = cl.L;
  const int64_t row0 = cl.row0;
  // this item's q, k, w slice stays in storage precision until the epilogue (rows past the end zero)
  v4 cq[4], ck[4], cww[4];
  {
    const v4 z4 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = rg * 4 + i < L;
      cq[i] = ok ? R.q[i] : z4;
      ck[i] = ok ? R.k[i] : z4;
      cww[i] = ok ? R.w[i] : z4;
    }
  }
  v8 dreg[NP], vreg[NP], d2reg[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    dreg[i] = row < L ? R.d[i] : z8;
    vreg[i] = row < L ? R.v[i] : z8;
    const uint32_t limv = (uint32_t)(L - 1) * pitchv + colv;
    d2reg[i] = *(const v8*)((const char*)p.dv2 + (row0 * H + hh) * (int64_t)V * (int64_t)sizeof(T) + (offv[i] < limv ? offv[i] : limv));
  }
  const int rw = wave >> 1, cw = wave & 1;
  const int kt32 = kb / 32 + cw;
  v8 hf[VT32][2], dhf[VT32][2];
  {
    const int64_t blk = (cl.cglob * H + hh) * (int64_t)K * V * (int64_t)sizeof(T);
    const char* hb = (const char*)p.hT + blk;
    const char* dhb = (const char*)p.dhtf + blk;
#pragma unroll
    for (int vt = 0; vt < VT32; ++vt) {
      const uint32_t o = (uint32_t)(((vt * (K / 32) + kt32) * 64 + lane) * 16) * (uint32_t)sizeof(T);
      hf[vt][0] = *(const v8*)(hb + o);
      hf[vt][1] = *(const v8*)(hb + o + 16);
      dhf[vt][0] = *(const v8*)(dhb + o);
      dhf[vt][1] = *(const v8*)(dhb + o + 16);
    }
  }
  if (tid < BT) sGam[tid] = R.gam;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    *(v8*)&sDo[row * LDV + c8] = dreg[i];
    *(v8*)&sVn[row * LDV + c8] = vreg[i];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v4 kt, qt;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      kt[i] = ck[i][j];
      qt[i] = cq[i][j];
    }
    *(v4*)&sKT[(c4 + j) * LDT + rg * 4] = kt;
    *(v4*)&sQT[(c4 + j) * LDT + rg * 4] = qt;
  }
  __syncthreads();
  // ---- ds = s tril((do v_new^T) * Gamma), both orientations
  {
    const int ib = wave >> 1, jb = wave & 1;
    if (jb <= ib) {
      f32x16 s1 = zero16(), s2 = zero16();
#pragma unroll
      for (int vs = 0; vs < V; vs += 16) {
        v8 fd = lds_frag32<T>(sDo, LDV, ib * 32, vs, lane);
        v8 fv = lds_frag32<T>(sVn, LDV, jb * 32, vs, lane);
        s1 = Elem<T>::mfma32(fd, fv, s1);  // rows i, cols j
        s2 = Elem<T>::mfma32(fv, fd, s2);  // rows j, cols i
      }
      const int c = lane & 31;
      const float gj1 = sGam[jb * 32 + c], gi2 = sGam[ib * 32 + c];
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int r0 = 8 * a + 4 * (lane >> 5);
        const f32x4 gi1 = *(const f32x4*)&sGam[ib * 32 + r0], gj2 = *(const f32x4*)&sGam[jb * 32 + r0];
        v4 x1, x2;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          int i1 = ib * 32 + r0 + b, j1 = jb * 32 + c;
          x1[b] = (T)((j1 <= i1) ? s1[4 * a + b] * p.scale * __expf(gi1[b] - gj1) : 0.f);
          int j2 = jb * 32 + r0 + b, i2 = ib * 32 + c;
          x2[b] = (T)((j2 <= i2) ? s2[4 * a + b] * p.scale * __expf(gi2 - gj2[b]) : 0.f);
        }
        *(v4*)&sDsT[(jb * 32 + c) * LDT + ib * 32 + r0] = x1;
        *(v4*)&sDs[(ib * 32 + c) * LDT + jb * 32 + r0] = x2;
      }
    }
  }
  __syncthreads();
  // ---- dq = s e^gamma (do h^T) + ds k ; dk_intra = ds^T q ; dk_inter = v_new dH^T
  f32x16 aq = zero16(), ak1 = zero16(), ak2 = zero16(), aw = zero16();
  const float glast = sGam[L - 1];
  // <h_c, dH_c> over this wave's tiles (same fragment order on both sides); here, where the fragments are first
  // needed, and not at the top of the item, where they have just been asked for
  float hd = 0.f;
#pragma unroll
  for (int vt = 0; vt < VT32; ++vt)
#pragma unroll
    for (int half = 0; half < 2; ++half) hd = Elem<T>::dot8(hf[vt][half], dhf[vt][half], hd);
#pragma unroll
  for (int vt = 0; vt < VT32; ++vt)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      // transposed products (the state fragment as the first operand): a lane ends up with one time row and, per
      // register quad, four adjacent key channels - the per-row factors are one exponential per lane, and the
      // accumulators leave as 16-byte pieces
      aq = Elem<T>::mfma32(hf[vt][half], lds_frag32_perm<T>(sDo, LDV, rw * 32, vt * 32 + half * 16, lane), aq);
      ak2 = Elem<T>::mfma32(dhf[vt][half], lds_frag32_perm<T>(sVn, LDV, rw * 32, vt * 32 + half * 16, lane), ak2);
    }
  const float gm = sGam[rw * 32 + (lane & 31)];   // this lane's time row
  {
    const float eq = p.scale * __expf(gm), ek = __expf(glast - gm);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      aq[r] *= eq;
      ak2[r] *= ek;
    }
  }
  const int jend = (rw + 1) * 32;
  for (int js = 0; js < jend; js += 16)
    aq = Elem<T>::mfma32(lds_frag32<T>(sKT, LDT, cw * 32, js, lane), lds_frag32<T>(sDs, LDT, rw * 32, js, lane), aq);
  for (int is = rw * 32; is < BT; is += 16)
    ak1 = Elem<T>::mfma32(lds_frag32<T>(sQT, LDT, cw * 32, is, lane), lds_frag32<T>(sDsT, LDT, rw * 32, is, lane), ak1);
  __syncthreads();  // do is consumed: its tile takes dv2
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    *(v8*)&sDo[row * LDV + c8] = row < L ? d2reg[i] : z8;
  }
  __syncthreads();
  // ---- dw = -e^gamma (dv2 h^T)
#pragma unroll
  for (int vt = 0; vt < VT32; ++vt)
#pragma unroll
    for (int half = 0; half < 2; ++half)
      aw = Elem<T>::mfma32(hf[vt][half], lds_frag32_perm<T>(sDo, LDV, rw * 32, vt * 32 + half * 16, lane), aw);
  {
    const float ew = -__expf(gm);
#pragma unroll
    for (int r = 0; r < 16; ++r) aw[r] *= ew;
  }
  __syncthreads();  // all operand reads done: tiles become fp32 staging
#pragma unroll
  for (int a4 = 0; a4 < 4; ++a4) {
    const int o = (rw * 32 + (lane & 31)) * LDM + cw * 32 + 8 * a4 + 4 * (lane >> 5);
    *(f32x4*)&stA[o] = f32x4{aq[4 * a4], aq[4 * a4 + 1], aq[4 * a4 + 2], aq[4 * a4 + 3]};
    *(f32x4*)&stB[o] = f32x4{ak1[4 * a4], ak1[4 * a4 + 1], ak1[4 * a4 + 2], ak1[4 * a4 + 3]};
    *(f32x4*)&stC[o] = f32x4{ak2[4 * a4], ak2[4 * a4 + 1], ak2[4 * a4 + 2], ak2[4 * a4 + 3]};
    *(f32x4*)&stD[o] = f32x4{aw[4 * a4], aw[4 * a4 + 1], aw[4 * a4 + 2], aw[4 * a4 + 3]};
  }
  // the next item's first rows are requested now: the accumulators are in LDS, the epilogue needs few registers
  const uint32_t nit = it + gridDim.x;
  const bool more = nit < nitems;   // workgroup-uniform
  const Item nim = locate(more ? nit : it);   // (past the last item the request repeats it: no load under a branch)
  request(nim, R);
  // <h, dH> of the whole key slice: reduce over the 4 waves through LDS
  __shared__ float sHd[4];
  hd = wave_sum_lane63(hd);
  if (lane == 63) sHd[wave] = hd;
  __syncthreads();
  // waves (rw=0,cw) and (rw=1,cw) loaded the same fragments: count each key tile once
  const float hd_all = sHd[0] + sHd[1];
  // ---- epilogue in the load mapping (4 rows x 4 key channels per lane)
  float rowsum[4], kin = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = rg * 4 + i;
    f32x4 a = *(const f32x4*)&stA[row * LDM + c4];
    f32x4 b = *(const f32x4*)&stB[row * LDM + c4];
    f32x4 c = *(const f32x4*)&stC[row * LDM + c4];
    f32x4 d = *(const f32x4*)&stD[row * LDM + c4];
    v4 dqv, dkv, dwv;
    float rs = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float dk = b[j] + c[j];
      dqv[j] = (T)a[j];
      dkv[j] = (T)dk;
      dwv[j] = (T)d[j];
      rs += (float)cq[i][j] * a[j] - (float)ck[i][j] * dk + (float)cww[i][j] * d[j];
      kin += (float)ck[i][j] * c[j];
    }
    rowsum[i] = rs;
    if (row < L) {
      int64_t off = ((row0 + row) * H + hh) * (int64_t)K + kb + c4;
      *(v4*)((T*)p.dq + off) = dqv;
      *(v4*)((T*)p.dk + off) = dkv;
      *(v4*)((T*)p.dw + off) = dwv;
    }
  }
  // row sums over the 16 lanes that share a row group; total of k*dk_inter over the workgroup
#pragma unroll
  for (int i = 0; i < 4; ++i) rowsum[i] = group_allsum<16>(rowsum[i]);
  kin = wave_sum_lane63(kin);
  __shared__ float sKin[4];
  if (lane == 63) sKin[wave] = kin;
  __syncthreads();
  const float kin_all = sKin[0] + sKin[1] + sKin[2] + sKin[3];
  if ((tid & 15) == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int row = rg * 4 + i;
      if (row < L) {
        float val = rowsum[i];
        if (row == L - 1) val += kin_all + __expf(glast) * hd_all;
        p.dgam[((int64_t)(kb / 64) * p.total_rows + row0 + row) * H + hh] = val;
      }
    }
  }
  if (!more) break;
  __syncthreads();  // the staging tiles are consumed: the next item's operand tiles may be written
  it = nit;
  im = nim;
  }
}

// ---------------------------------------------------------------------------
struct WyBwdParams {
  const void* k;
  const void* v;
  const float* beta;
  const float* gam;
  const void* Aw;
  const void* dw;
  const void* du;
  const void* dk_in;   // partial dk from the dq/dk/dw kernel, added to this launch's (rounded) part on the way out
  void* dk;
  void* dv;
  float* dbeta;
  float* dgam2;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  // With dgam_part (fp32 [nparts, total_rows, H], the gate-gradient partial sums of the dq/dk/dw launch) dgam2
  // receives the gradient of the raw gate itself: the reverse chunk-local cumulative sum of (sum of the parts +
  // this launch's own terms), as chunk_local_cumsum(reverse=True) leaves it (fla/ops/gated_delta_rule/chunk.py:170-171).
  const float* dgam_part;
  int nparts;
  int64_t total_rows;
};

// Transposed 64 x N product: acc[t] (+)= X^T-tile A^T, i.e. C[column][time row] with
//   X^T  [columns][ldx]  (contraction contiguous), columns col0 + 32 t ..
//   A    [64][lda]       (rows = output time rows 32 rw .., contraction contiguous).
// A lane ends up with one time row (32 rw + lane % 32) and, per tile, registers
// r <-> column col0 + 32 t + 8 (r/4) + 4 (lane/32) + r%4: four consecutive columns per
// register quad, so the epilogues use 8-byte accesses and row sums stay in the lane.
template <typename T, int NT_>
FLA_DEVICE void mm64t(const T* Xt, int ldx, int col0, const T* A, int lda, int rw, int c_begin, int c_end, int lane,
                      f32x16* acc) {
  typedef typename Elem<T>::v8 v8;
  for (int cs = c_begin; cs < c_end; cs += 16) {
    v8 a = lds_frag32<T>(A, lda, rw * 32, cs, lane);
#pragma unroll
    for (int t = 0; t < NT_; ++t) acc[t] = Elem<T>::mfma32(lds_frag32<T>(Xt, ldx, col0 + t * 32, cs, lane), a, acc[t]);
  }
}

// A thread of the tile loaders owns RPT rows x 4 columns of a [64][DIM] tile: 8-byte global
// loads, 8-byte row-major LDS writes and time-contiguous vectors for the transposed copy.
template <typename T, int DIM>
struct TileIO {
  typedef typename Elem<T>::v4 v4;
  static constexpr int CG = DIM / 4, RG = 256 / CG, RPT = BT / RG;
  typedef T tvec __attribute__((ext_vector_type(RPT)));
  // Unconditional: rows past the end of a short chunk re-read its last row (a load under a branch makes the
  // compiler wait for it, and for everything issued before it, at the join); zero_tail() clears them before use.
  static FLA_DEVICE void load(const void* src, int64_t row0, int L, int H, int hh, int tid, v4* reg) {
    const int rg = tid / CG, c4 = (tid % CG) * 4;
    const char* p = (const char*)((const T*)src + (row0 * H + hh) * (int64_t)DIM + c4);
    const uint32_t pitch = (uint32_t)H * DIM * (uint32_t)sizeof(T), lim = (uint32_t)(L - 1) * pitch;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const uint32_t o = (uint32_t)(rg * RPT + i) * pitch;
      reg[i] = *(const v4*)(p + (o < lim ? o : lim));
    }
  }
  static FLA_DEVICE void zero_tail(int L, int tid, v4* reg) {
    const int rg = tid / CG;
#pragma unroll
    for (int i = 0; i < RPT; ++i)
      if (rg * RPT + i >= L) reg[i] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
  }
  static FLA_DEVICE void put_rows(T* dst, int ld, int tid, const v4* reg) {
    const int rg = tid / CG, c4 = (tid % CG) * 4;
#pragma unroll
    for (int i = 0; i < RPT; ++i) *(v4*)&dst[(rg * RPT + i) * ld + c4] = reg[i];
  }
  static FLA_DEVICE void put_tr(T* dst, int tid, const v4* reg) {
    const int rg = tid / CG, c4 = (tid % CG) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      tvec x;
#pragma unroll
      for (int i = 0; i < RPT; ++i) x[i] = reg[i][j];
      *(tvec*)&dst[(c4 + j) * LDT + rg * RPT] = x;
    }
  }
};

template <typename T, int K, int V>
__global__ __launch_bounds__(256, K <= 128 ? 2 : 1) void gdr_bwd_wy_kernel(WyBwdParams p, uint32_t nitems) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int D = K > V ? K : V;
  constexpr int LDD = D + 8;
  constexpr int TK = K / 64, TV = V / 64;
  typedef TileIO<T, K> IOK;
  typedef TileIO<T, V> IOV;
  typedef TileIO<T, BT> IOA;
  __shared__ __attribute__((aligned(16))) T sRow1[BT * LDD];   // du, then dw          row-major [t][d]; later sS2
  __shared__ __attribute__((aligned(16))) T sRow2[BT * LDD];   // v,  then k           row-major
  __shared__ __attribute__((aligned(16))) T sTr1[D * LDT];     // du^T, dw^T, k^T      [d][t]
  __shared__ __attribute__((aligned(16))) T sAw[BT * LDT];     // Aw [i][j]
  __shared__ __attribute__((aligned(16))) T sAwT[BT * LDT];    // Aw^T
  __shared__ __attribute__((aligned(16))) T sS1[BT * LDT];     // Au^T -> dA^T (masked) -> dM
  __shared__ float sBeta[BT], sGam[BT];
  // Partial sums of dbeta and dgamma, one slot per contributing wave and step, added in a fixed order at the
  // end (no atomics: the gradients are bit-reproducible from run to run).  Slots 0-3: dbeta from the value
  // side / key side x the two column halves; 4-5: dgamma row sums from the two column blocks; 6-7: dgamma
  // column sums from the two row blocks.  They live in the 16 bytes of padding behind every row of the
  // transposed tile (and of the Aw tile where that one has only 64 rows), which no tile access touches, so
  // that two workgroups still fit a CU.
  auto slot = [&](int s_, int r) -> float& {
    T* base = s_ < 4 ? &sTr1[r * LDT + BT] : (D >= 128 ? &sTr1[(r + BT) * LDT + BT] : &sAw[r * LDT + BT]);
    return ((float*)base)[s_ & 3];
  };
  // X1^T, then dM^T diag(beta): lives in the du/dw tile, which is dead once dA has been formed
  // (two workgroups then fit a CU)
  T* sS2 = sRow1;

  const int tid0 = threadIdx.x;
  const int H = p.H;
  // A workgroup walks (chunk, head) items with a stride of the grid size; the rows an item starts with (du, v,
  // Aw, beta, gamma) are requested as soon as those of the item before it are in LDS (32-bit offsets off
  // wave-uniform bases; rows past the end of a short chunk re-read its last row and are masked at use, so no
  // load sits under a branch).
  struct Item {
    ChunkLoc cl;
    int hh;
  };
  auto locate = [&](uint32_t it) {
    Item r;
    r.cl = locate_chunk_at32(it, p.offsets, p.indices, p.T, p.NTfix, H, &r.hh);
    return r;
  };
  struct Raw {
    v4 du[IOV::RPT], v[IOV::RPT], a[IOA::RPT];
    float beta, gam;
  };
  const uint32_t pitchv = (uint32_t)H * V * (uint32_t)sizeof(T), pitcha = (uint32_t)H * BT * (uint32_t)sizeof(T);
  const uint32_t colv = (uint32_t)((tid0 % IOV::CG) * 4) * (uint32_t)sizeof(T), cola = (uint32_t)((tid0 % IOA::CG) * 4) * (uint32_t)sizeof(T);
  uint32_t offv[IOV::RPT], offa[IOA::RPT];
#pragma unroll
  for (int i = 0; i < IOV::RPT; ++i) offv[i] = (uint32_t)((tid0 / IOV::CG) * IOV::RPT + i) * pitchv + colv;
#pragma unroll
  for (int i = 0; i < IOA::RPT; ++i) offa[i] = (uint32_t)((tid0 / IOA::CG) * IOA::RPT + i) * pitcha + cola;
  auto request = [&](const Item& im, Raw& R) __attribute__((always_inline)) {
    const uint32_t last = (uint32_t)(im.cl.L - 1);
    const int64_t r0h = im.cl.row0 * H + im.hh;
    const char* dub = (const char*)p.du + r0h * V * (int64_t)sizeof(T);
    const char* vb = (const char*)p.v + r0h * V * (int64_t)sizeof(T);
    const char* ab = (const char*)p.Aw + r0h * BT * (int64_t)sizeof(T);
    const uint32_t limv = last * pitchv + colv, lima = last * pitcha + cola;
#pragma unroll
    for (int i = 0; i < IOV::RPT; ++i) {
      const uint32_t o = offv[i] < limv ? offv[i] : limv;
      R.du[i] = *(const v4*)(dub + o);
      R.v[i] = *(const v4*)(vb + o);
    }
#pragma unroll
    for (int i = 0; i < IOA::RPT; ++i) R.a[i] = *(const v4*)(ab + (offa[i] < lima ? offa[i] : lima));
    const uint32_t row = (uint32_t)(tid0 & (BT - 1)) < last ? (uint32_t)(tid0 & (BT - 1)) : last;
    R.beta = p.beta[(im.cl.row0 + row) * H + im.hh];
    // without gates the load reads one zero word (no branch round a load)
    R.gam = *(p.gam ? p.gam + (im.cl.row0 + row) * H + im.hh : &kZeroWord);
  };
  uint32_t it = blockIdx.x;
  if (it >= nitems) return;
  Item im = locate(it);
  Raw R;
  request(im, R);
  for (;;) {
  // (the lane id goes through an opaque copy once per item, so that the LDS addresses of the body are formed
  // where they are used instead of being hoisted out of the loop into long-lived registers)
  int tid = tid0;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = im.hh;
  const ChunkLoc cl = im.cl;
  const int L = cl.L;
  const int64_t row0 = cl.row0;
  const int rw = wave >> 1, cw = wave & 1;

  // ---- the value side and Aw, rows past the end of the chunk zero (Aw: identity, below)
  v4 rdu[IOV::RPT], rv[IOV::RPT], ra[IOA::RPT];
  {
    const v4 z4 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
    for (int i = 0; i < IOV::RPT; ++i) {
      const bool ok = (tid / IOV::CG) * IOV::RPT + i < L;
      rdu[i] = ok ? R.du[i] : z4;
      rv[i] = ok ? R.v[i] : z4;
    }
#pragma unroll
    for (int i = 0; i < IOA::RPT; ++i) ra[i] = R.a[i];
  }
  if (tid < BT) {
    sBeta[tid] = tid < L ? R.beta : 0.f;
    sGam[tid] = R.gam;
    // the quadrant above the diagonal contributes nothing: its slots stay zero
    slot(5, tid) = 0.f;
    slot(6, tid) = 0.f;
  }
  {
    // rows beyond L: identity
    const int rg = tid / IOA::CG, c4 = (tid % IOA::CG) * 4;
#pragma unroll
    for (int i = 0; i < IOA::RPT; ++i) {
      int row = rg * IOA::RPT + i;
      if (row >= L)
#pragma unroll
        for (int j = 0; j < 4; ++j) ra[i][j] = (T)((c4 + j == row) ? 1.f : 0.f);
    }
  }
  IOA::put_rows(sAw, LDT, tid, ra);
  IOA::put_tr(sAwT, tid, ra);
  IOV::put_rows(sRow1, LDD, tid, rdu);
  IOV::put_tr(sTr1, tid, rdu);
  IOV::put_rows(sRow2, LDD, tid, rv);
  // the key side is loaded while the value side computes
  v4 rdw[IOK::RPT], rk[IOK::RPT];
  IOK::load(p.dw, row0, L, H, hh, tid, rdw);
  IOK::load(p.k, row0, L, H, hh, tid, rk);
  const uint32_t nit = it + gridDim.x;
  const bool more = nit < nitems;   // workgroup-uniform
  const Item nim = locate(more ? nit : it);   // (past the last item the request repeats it)
  __syncthreads();
  {
    // Au^T[j][i] = Aw^T[j][i] * e^{gamma_i - gamma_j}, i >= j
    const int j = tid >> 2, i0 = (tid & 3) * 16;
    const float gj = sGam[j];
#pragma unroll
    for (int h8 = 0; h8 < 2; ++h8) {
      v8 a = *(const v8*)&sAwT[j * LDT + i0 + 8 * h8], o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        int i = i0 + 8 * h8 + e;
        o[e] = (T)((i >= j) ? (float)a[e] * __expf(sGam[i] - gj) : 0.f);
      }
      *(v8*)&sS1[j * LDT + i0 + 8 * h8] = o;
    }
  }
  __syncthreads();

  const int jrow = rw * 32 + (lane & 31);      // this lane's time row in the transposed products
  const float bj = sBeta[jrow];
  // ================= value side: d(vb) = Au^T du ; dAu = (du v^T) diag(beta)
  const int ib = wave >> 1, jb = wave & 1;     // score quadrants: waves 0,2,3 -> (0,0),(1,0),(1,1)
  f32x16 dAu = zero16();
  v4 dvst[TV][4];
  {
    f32x16 dvb[TV];
#pragma unroll
    for (int t = 0; t < TV; ++t) dvb[t] = zero16();
    // Au^T is upper triangular: row j contracts over i >= j
    mm64t<T, TV>(sTr1, LDT, cw * TV * 32, sS1, LDT, rw, rw * 32, BT, lane, dvb);
    if (jb <= ib) {
      for (int vs = 0; vs < V; vs += 16)
        dAu = Elem<T>::mfma32(lds_frag32<T>(sRow1, LDD, ib * 32, vs, lane), lds_frag32<T>(sRow2, LDD, jb * 32, vs, lane),
                              dAu);
      const float bcol = sBeta[jb * 32 + (lane & 31)];
#pragma unroll
      for (int r = 0; r < 16; ++r) dAu[r] *= bcol;
    }
    // dv = beta d(vb), kept in registers until the tiles are free to carry it to whole-row stores;
    // dbeta += sum_v d(vb) * v
    float part = 0.f;
#pragma unroll
    for (int t = 0; t < TV; ++t)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int col = (cw * TV + t) * 32 + 8 * r4 + 4 * (lane >> 5);
        v4 vv = *(const v4*)&sRow2[jrow * LDD + col], o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float d = dvb[t][4 * r4 + e];
          part += d * (float)vv[e];
          o[e] = (T)(d * bj);
        }
        dvst[t][r4] = o;
      }
    part += __shfl_xor(part, 32, 64);
    if (lane < 32) slot(cw, jrow) = part;
  }
  __syncthreads();  // the value tiles and Au^T are consumed
  // ================= key side: d(kb)_1 = Aw^T dw ; dAw_1 = (dw k^T) diag(beta)
  IOK::zero_tail(L, tid, rdw);
  IOK::zero_tail(L, tid, rk);
  IOK::put_rows(sRow1, LDD, tid, rdw);
  IOK::put_tr(sTr1, tid, rdw);
  IOK::put_rows(sRow2, LDD, tid, rk);
  __syncthreads();
  request(nim, R);  // the next item's first rows
  // the partial dk of the previous launch is needed only in the last step: fetched now, so that its
  // latency hides behind the products
  // In the mapping of the final stores (whole rows, 16 bytes per lane: a lane per accumulator row would touch 32
  // cache lines per instruction).  Unconditional, at a row inside the chunk, masked where they are used: a load under
  // a branch is waited for at the join; without a partial dk the rows of k are read.
  constexpr int CKs = K / 8, NDI = BT * CKs / 256;
  v8 dinr[NDI];
  {
    const T* dip = (p.dk_in ? (const T*)p.dk_in : (const T*)p.k) + (row0 * H + hh) * (int64_t)K;
#pragma unroll
    for (int i = 0; i < NDI; ++i) {
      const int e = tid + 256 * i, row = e / CKs, c8 = (e % CKs) * 8;
      dinr[i] = *(const v8*)(dip + (int64_t)(row < L ? row : L - 1) * H * K + c8);
    }
  }
  // the gate-gradient partial sums of the launch before, for the last step as well (wave 0, one row per lane)
  float dgpv[4];   // (at most four key slices of 64 channels; no branch round the loads)
  {
    const int rl = (tid & (BT - 1)) < L ? (tid & (BT - 1)) : L - 1;
    const float* gp0 = p.dgam_part ? p.dgam_part + (row0 + rl) * H + hh : &kZeroWord;
    const int64_t zs = p.dgam_part ? p.total_rows * H : 0;
#pragma unroll
    for (int z = 0; z < 4; ++z) dgpv[z] = gp0[(z < p.nparts ? z : 0) * zs];
  }
  f32x16 dkb[TK];   // d(kb)^T: columns (cw*TK+t)*32.., time row jrow
#pragma unroll
  for (int t = 0; t < TK; ++t) dkb[t] = zero16();
  mm64t<T, TK>(sTr1, LDT, cw * TK * 32, sAwT, LDT, rw, rw * 32, BT, lane, dkb);
  f32x16 dA = zero16();
  if (jb <= ib) {
    for (int ks = 0; ks < K; ks += 16)
      dA = Elem<T>::mfma32(lds_frag32<T>(sRow1, LDD, ib * 32, ks, lane), lds_frag32<T>(sRow2, LDD, jb * 32, ks, lane), dA);
    const float bcol = sBeta[jb * 32 + (lane & 31)];
#pragma unroll
    for (int r = 0; r < 16; ++r) dA[r] *= bcol;
  }
  // ================= dA_total (strictly lower) and the gate gradient through Gamma
  if (jb <= ib) {
    const int j = jb * 32 + (lane & 31);
    const float gj = sGam[j];
    float colsum = 0.f;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      int i0 = ib * 32 + 8 * a + 4 * (lane >> 5);
      // this lane's four rows of column j are adjacent in the transposed tiles: one 8-byte access each for Aw and
      // for dA, which is left transposed (dA^T[j][i]; the product below reads it through the transposing load)
      const f32x4 gi4 = *(const f32x4*)&sGam[i0];
      const v4 aw4 = *(const v4*)&sAwT[j * LDT + i0];
      v4 tot4;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int i = i0 + b, r = 4 * a + b;
        bool low = j < i;
        float gamma = low ? __expf(gi4[b] - gj) : 0.f;
        float au = (float)aw4[b] * gamma;                   // Au_ij
        float x = low ? dAu[r] * au : 0.f;                  // dAu * Au
        float tot = low ? dA[r] + dAu[r] * gamma : 0.f;     // dAw total
        tot4[b] = (T)tot;
        // row sums over the 32 lanes holding the same row: inside each row of 16 lanes on the data-parallel path,
        // then the first row's total handed to the second (sixteen butterflies through the LDS crossbar per lane
        // were a third of this kernel's time)
        const float rs = half_wave_sum_hi(x);
        if ((lane & 31) == 16) slot(4 + jb, i) = rs;
        colsum += x;
      }
      *(v4*)&sS1[j * LDT + i0] = tot4;                       // dA^T (masked) [j][i]
    }
    colsum += __shfl_xor(colsum, 32, 64);
    if (lane < 32) slot(6 + ib, j) = -colsum;
  } else {
    // quadrant (0,1) lies strictly above the diagonal (rows 32.. of the transposed tile, columns 0..31)
    for (int e = lane; e < 32 * 32; e += 64) sS1[(32 + (e >> 5)) * LDT + (e & 31)] = (T)0.f;
  }
  __syncthreads();  // dA complete; dw^T consumed
  IOK::put_tr(sTr1, tid, rk);   // k^T
  // ================= X1 = dA Aw^T  (stored transposed), dM = -strict_lower(Aw^T X1)
  {
    // wave (rw, cw): rows a = 32rw.., cols j = 32cw..  ; contraction over b
    f32x16 x1 = zero16();
    for (int bs = 0; bs < BT; bs += 16)
      x1 = Elem<T>::mfma32(frag32_tr<T>(sS1, LDT, rw * 32, bs, lane), lds_frag32<T>(sAw, LDT, cw * 32, bs, lane), x1);
    const int j = cw * 32 + (lane & 31);
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      int a0 = rw * 32 + 8 * a + 4 * (lane >> 5);
      v4 x;
#pragma unroll
      for (int b = 0; b < 4; ++b) x[b] = (T)x1[4 * a + b];
      *(v4*)&sS2[j * LDT + a0] = x;   // X1^T[j][a]
    }
  }
  __syncthreads();
  {
    // both orientations of Aw^T X1 so that dM and dM^T are written with 8-byte vectors
    f32x16 m = zero16(), mt = zero16();
    for (int as = 0; as < BT; as += 16) {
      v8 fa = lds_frag32<T>(sAwT, LDT, rw * 32, as, lane), fx = lds_frag32<T>(sS2, LDT, cw * 32, as, lane);
      m = Elem<T>::mfma32(fa, fx, m);     // rows i = 32rw.. (registers), column j = 32cw + lane%32
      mt = Elem<T>::mfma32(fx, fa, mt);   // rows j = 32cw.. (registers), column i = 32rw + lane%32
    }
    __syncthreads();  // every wave has read dA (sS1) and X1^T (sS2)
    {
      const int j = cw * 32 + (lane & 31);
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int i0 = rw * 32 + 8 * a + 4 * (lane >> 5);
        v4 x;
#pragma unroll
        for (int b = 0; b < 4; ++b) x[b] = (T)((j < i0 + b) ? -m[4 * a + b] * sBeta[i0 + b] : 0.f);
        *(v4*)&sS2[j * LDT + i0] = x;           // (dM^T diag(beta))[j][i]
      }
      const int i = rw * 32 + (lane & 31);
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int j0 = cw * 32 + 8 * a + 4 * (lane >> 5);
        v4 x;
#pragma unroll
        for (int b = 0; b < 4; ++b) x[b] = (T)((j0 + b < i) ? -mt[4 * a + b] : 0.f);
        *(v4*)&sS1[i * LDT + j0] = x;           // dM[i][j]
      }
    }
  }
  __syncthreads();
  // ================= d(kb) += dM k ; dk = beta d(kb) + (dM^T diag(beta)) k ; dbeta += sum_k d(kb) * k
  // dM is strictly lower: row i contracts over j < i ; dM^T row j contracts over i > j
  mm64t<T, TK>(sTr1, LDT, cw * TK * 32, sS1, LDT, rw, 0, (rw + 1) * 32, lane, dkb);
  f32x16 dk2[TK];
#pragma unroll
  for (int t = 0; t < TK; ++t) dk2[t] = zero16();
  mm64t<T, TK>(sTr1, LDT, cw * TK * 32, sS2, LDT, rw, rw * 32, BT, lane, dk2);
  {
    float part = 0.f;
#pragma unroll
    for (int t = 0; t < TK; ++t)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int col = (cw * TK + t) * 32 + 8 * r4 + 4 * (lane >> 5);
        v4 kk = *(const v4*)&sRow2[jrow * LDD + col], o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float d = dkb[t][4 * r4 + e];
          part += d * (float)kk[e];
          o[e] = (T)(d * bj + dk2[t][4 * r4 + e]);
        }
        // dk takes the place of the k element this lane has just read (nobody else reads the tile any more)
        *(v4*)&sRow2[jrow * LDD + col] = o;
      }
    part += __shfl_xor(part, 32, 64);
    if (lane < 32) slot(2 + cw, jrow) = part;
  }
  __syncthreads();  // every wave is past its last read of X1^T / dM^T, which share storage with the dv tile
  if (tid < BT) {   // wave 0: one row per lane
    const bool ok = tid < L;
    if (ok) p.dbeta[(row0 + tid) * H + hh] = (slot(0, tid) + slot(1, tid)) + (slot(2, tid) + slot(3, tid));
    float dgm = ok ? (slot(4, tid) + slot(5, tid)) + (slot(6, tid) + slot(7, tid)) : 0.f;
    if (p.dgam_part) {
      float dgp = 0.f;
#pragma unroll
      for (int z = 0; z < 4; ++z) dgp += z < p.nparts ? dgpv[z] : 0.f;
      dgm += ok ? dgp : 0.f;
      // inclusive suffix sum over the 64 rows: DPP row scans plus the totals of the later rows of 16
      float x = row_suffix16(dgm);
      const float t1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 16));
      const float t2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 32));
      const float t3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 48));
      const int r = lane >> 4;
      dgm = x + (r < 1 ? t1 : 0.f) + (r < 2 ? t2 : 0.f) + (r < 3 ? t3 : 0.f);
    }
    if (ok) p.dgam2[(row0 + tid) * H + hh] = dgm;
  }
#pragma unroll
  for (int t = 0; t < TV; ++t)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
      *(v4*)&sRow1[jrow * LDD + (cw * TV + t) * 32 + 8 * r4 + 4 * (lane >> 5)] = dvst[t][r4];
  __syncthreads();
  // dk and dv leave as whole rows, 16 bytes per lane (8-byte pieces scattered over 32 rows cost
  // several times their bytes)
  {
    constexpr int CK = K / 8, CV = V / 8;
    // dk = this launch's part (rounded once into the tile) + the partial dk of the launch before
#pragma unroll
    for (int i = 0; i < NDI; ++i) {
      const int e = tid + 256 * i, row = e / CK, c8 = (e % CK) * 8;
      v8 x = *(const v8*)&sRow2[row * LDD + c8];
      if (p.dk_in) {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = (T)((float)x[j] + (float)dinr[i][j]);
      }
      if (row < L) *(v8*)((T*)p.dk + ((row0 + row) * H + hh) * (int64_t)K + c8) = x;
    }
    for (int e = tid; e < BT * CV; e += 256) {
      const int row = e / CV, c8 = (e % CV) * 8;
      if (row < L) *(v8*)((T*)p.dv + ((row0 + row) * H + hh) * (int64_t)V + c8) = *(const v8*)&sRow1[row * LDD + c8];
    }
  }
  if (!more) break;
  __syncthreads();  // dk and dv are on their way: the next item's tiles may be written
  it = nit;
  im = nim;
  }
}

#define FLA_KV(STMT)                                   \
  if (K == 64 && V == 64) { STMT(64, 64) }             \
  else if (K == 128 && V == 128) { STMT(128, 128) }    \
  else if (K == 64 && V == 128) { STMT(64, 128) }      \
  else if (K == 128 && V == 64) { STMT(128, 64) }      \
  else if (K == 256 && V == 64) { STMT(256, 64) }      \
  else if (K == 256 && V == 128) { STMT(256, 128) }    \
  else return FLA_E_UNSUPPORTED;

template <typename T>
int launch_dv_local(const DvlParams& p, int64_t K, int64_t V, dim3 grid, hipStream_t st) {
  // as many workgroups as are resident at once, each walking its share of the (chunk, head) items
  const int64_t total = (int64_t)grid.x * grid.y;
  FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
#define L1(KK, VV)                                                                                        \
  {                                                                                                       \
    const int64_t res = resident_workgroups(gdr_bwd_dvlocal_kernel<T, KK, VV>);                           \
    hipLaunchKernelGGL((gdr_bwd_dvlocal_kernel<T, KK, VV>), dim3((unsigned)(total < res ? total : res)), dim3(256), 0, st, \
                       p, (uint32_t)total);                                                               \
  }
  FLA_KV(L1)
#undef L1
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

// reverse state scan: one workgroup per (sequence, head, 32 value columns)
template <typename T>
int launch_dhu(const DhuParams& p, int64_t K, hipStream_t st) {
  const int64_t total = (int64_t)(p.V / 32) * p.N * p.H;
  FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  if (total == 0) return FLA_OK;
  if (p.Aqk) {
    if (K == 64) hipLaunchKernelGGL((gdr_bwd_dhu_kernel<T, 64, true>), dim3((unsigned)total), dim3(512), 0, st, p);
    else if (K == 128) hipLaunchKernelGGL((gdr_bwd_dhu_kernel<T, 128, true>), dim3((unsigned)total), dim3(512), 0, st, p);
    else return FLA_E_UNSUPPORTED;
  } else if (K == 64) hipLaunchKernelGGL((gdr_bwd_dhu_kernel<T, 64, false>), dim3((unsigned)total), dim3(512), 0, st, p);
  else if (K == 256) hipLaunchKernelGGL((gdr_bwd_dhu_kernel<T, 256, false>), dim3((unsigned)total), dim3(512), 0, st, p);
  else if (K == 128) hipLaunchKernelGGL((gdr_bwd_dhu_kernel<T, 128, false>), dim3((unsigned)total), dim3(512), 0, st, p);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

// one workgroup per (chunk, head, 64 key channels)
template <typename T>
int launch_dqkwg(const DqkwgParams& p, int64_t V, dim3 grid, hipStream_t st) {
  // as many workgroups as are resident at once (two per CU), each walking its share of the items
  const int64_t pairs = (int64_t)grid.x * grid.y, nwg = pairs * (p.K / 64);
  FLA_REQUIRE(nwg <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  dim3 g3((unsigned)(nwg < 2 * kNumCUs ? nwg : 2 * kNumCUs));
  if (V == 64) hipLaunchKernelGGL((gdr_bwd_dqkwg_kernel<T, 64>), g3, dim3(256), 0, st, p, pairs);
  else if (V == 128) hipLaunchKernelGGL((gdr_bwd_dqkwg_kernel<T, 128>), g3, dim3(256), 0, st, p, pairs);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

template <typename T>
int launch_wy_bwd(const WyBwdParams& p, int64_t K, int64_t V, dim3 grid, hipStream_t st) {
  // as many workgroups as are resident at once, each walking its share of the (chunk, head) items
  const int64_t total = (int64_t)grid.x * grid.y;
  FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
#define L4(KK, VV)                                                                                   \
  {                                                                                                  \
    const int64_t res = resident_workgroups(gdr_bwd_wy_kernel<T, KK, VV>);                           \
    hipLaunchKernelGGL((gdr_bwd_wy_kernel<T, KK, VV>), dim3((unsigned)(total < res ? total : res)), dim3(256), 0, st, p, \
                       (uint32_t)total);                                                             \
  }
  FLA_KV(L4)
#undef L4
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}
#undef FLA_KV

template <typename T>
int launch_gdr_bwd(const void* q, const void* k, const void* v, const void* w, const void* vnew, const float* beta,
                   const float* gam, const void* Aw, const void* dout, const float* dht, const void* hT,
                   const void* Aqk, void* dvl, void* dv2, void* dhtf, void* dw, void* dkp, float* dgam_part, void* dq, void* dk, void* dv,
                   float* dbeta, float* dgam2, float* dh0, const int64_t* offsets, const int64_t* indices,
                   const int64_t* chunk_offsets, int64_t NT, int64_t B, int64_t T_, int64_t H, int64_t K, int64_t V,
                   int64_t N, float scale, hipStream_t st) {
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T_, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return copy_or_zero(dht, dh0, N * H * K * V, st);   // no chunk at all: d h0 = d ht
  if (!Aqk) {   // dv_loc by a launch of its own unless the forward kept its score tiles
    DvlParams p1{q, k, dout, gam, dvl, offsets, indices, T_, (int)H, ntfix, scale};
    if ((rc = launch_dv_local<T>(p1, K, V, grid, st))) return rc;
  }
  DhuParams p2{q, k, w, dout, dvl, Aqk, gam, dht, dv2, dhtf, dh0, offsets, chunk_offsets, T_, (int)H, (int)V, (int)N, scale};
  if ((rc = launch_dhu<T>(p2, K, st))) return rc;
  DqkwgParams p3{q, k, vnew, w, dout, dv2, gam, hT, dhtf, dq, dkp, dw, dgam_part, offsets, indices, T_,
                 B * T_, (int)H, (int)K, ntfix, scale};
  if ((rc = launch_dqkwg<T>(p3, V, grid, st))) return rc;
  WyBwdParams p4{k, v, beta, gam, Aw, dw, dv2, dkp, dk, dv, dbeta, dgam2, offsets, indices, T_, (int)H, ntfix,
                 gam ? dgam_part : nullptr, (int)(K / 64), B * T_};
  return launch_wy_bwd<T>(p4, K, V, grid, st);
}

}  // namespace

extern "C" int fla_chunk_bwd_dv_local(const void* q, const void* k, const float* g_cumsum, const void* dout, void* dv,
                                      const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype,
                                      int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, float scale,
                                      fla_stream_t stream) {
  FLA_REQUIRE(q && k && dout && dv, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)dout | (uintptr_t)dv) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  DvlParams p{q, k, dout, g_cumsum, dv, offsets, indices, T, (int)H, ntfix, scale};
  if (qkv_dtype == FLA_BF16) return launch_dv_local<bf16>(p, K, V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_dv_local<f16>(p, K, V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gated_delta_rule_bwd(
    const void* q, const void* k, const void* v, const void* w, const void* v_new, const float* beta,
    const float* g_cumsum, const void* Aw, const void* dout, const float* dht, const void* hT, const void* Aqk,
    void* ws_dv_local, void* ws_dv2, void* ws_dh_frag_t, void* ws_dw, void* ws_dk_partial, float* ws_dgam_partial,
    void* dq, void* dk, void* dv, float* dbeta, float* dgam2, float* dh0,
    const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT, int qkv_dtype,
    int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N, float scale, fla_stream_t stream) {
  FLA_REQUIRE(q && k && v && w && v_new && beta && Aw && dout && hT && (ws_dv_local || Aqk) && ws_dv2 && ws_dh_frag_t &&
                  ws_dw && ws_dk_partial && ws_dgam_partial && dq && dk && dv && dbeta && dgam2,
              FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE((K == 64 || K == 128 || K == 256) && (V == 64 || V == 128), FLA_E_UNSUPPORTED);
  if (Aqk) FLA_REQUIRE(K <= 128 && (uintptr_t)Aqk % 16 == 0, FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(indices && chunk_offsets && B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  hipStream_t st = (hipStream_t)stream;
  if (qkv_dtype == FLA_BF16)
    return launch_gdr_bwd<bf16>(q, k, v, w, v_new, beta, g_cumsum, Aw, dout, dht, hT, Aqk, ws_dv_local, ws_dv2,
                                ws_dh_frag_t, ws_dw, ws_dk_partial, ws_dgam_partial, dq, dk, dv, dbeta, dgam2, dh0,
                                offsets, indices, chunk_offsets, NT, B, T, H, K, V, N, scale, st);
  if (qkv_dtype == FLA_F16)
    return launch_gdr_bwd<f16>(q, k, v, w, v_new, beta, g_cumsum, Aw, dout, dht, hT, Aqk, ws_dv_local, ws_dv2,
                               ws_dh_frag_t, ws_dw, ws_dk_partial, ws_dgam_partial, dq, dk, dv, dbeta, dgam2, dh0,
                               offsets, indices, chunk_offsets, NT, B, T, H, K, V, N, scale, st);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gated_delta_rule_bwd_dhu(const void* q, const void* k, const void* w, const float* g_cumsum,
                                                  const float* dht, const void* dout, const void* dv, void* dh_frag_t,
                                                  void* dv2, float* dh0, const int64_t* offsets,
                                                  const int64_t* chunk_offsets, int qkv_dtype, int64_t B, int64_t T,
                                                  int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                                  fla_stream_t stream) {
  FLA_REQUIRE(q && k && w && dout && dv && dh_frag_t && dv2, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE((K == 64 || K == 128 || K == 256) && V % 32 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(offsets ? (B == 1 && chunk_offsets != nullptr) : N == B, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)w | (uintptr_t)dout | (uintptr_t)dv | (uintptr_t)dh_frag_t |
               (uintptr_t)dv2) % 16 == 0, FLA_E_ALIGNMENT);
  hipStream_t st = (hipStream_t)stream;
  if (N == 0 || T == 0) return copy_or_zero(dht, dh0, N * H * K * V, st);
  DhuParams p{q, k, w, dout, dv, nullptr, g_cumsum, dht, dv2, dh_frag_t, dh0, offsets, chunk_offsets, T, (int)H, (int)V, (int)N,
              scale};
  if (qkv_dtype == FLA_BF16) return launch_dhu<bf16>(p, K, st);
  if (qkv_dtype == FLA_F16) return launch_dhu<f16>(p, K, st);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_bwd_dqkwg(const void* q, const void* k, const void* v_new, const void* w,
                                   const float* g_cumsum, const void* h_frag_t, const void* dh_frag_t, const void* dout,
                                   const void* dv, void* dq, void* dk, void* dw, float* dg_partial,
                                   const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B,
                                   int64_t T, int64_t H, int64_t K, int64_t V, float scale, fla_stream_t stream) {
  FLA_REQUIRE(q && k && v_new && w && h_frag_t && dh_frag_t && dout && dv && dq && dk && dw && dg_partial,
              FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(K % 64 == 0 && (V == 64 || V == 128), FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v_new | (uintptr_t)w | (uintptr_t)h_frag_t |
               (uintptr_t)dh_frag_t | (uintptr_t)dout | (uintptr_t)dv | (uintptr_t)dq | (uintptr_t)dk |
               (uintptr_t)dw) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  DqkwgParams p{q, k, v_new, w, dout, dv, g_cumsum, h_frag_t, dh_frag_t, dq, dk, dw, dg_partial, offsets, indices, T,
                B * T, (int)H, (int)K, ntfix, scale};
  if (qkv_dtype == FLA_BF16) return launch_dqkwg<bf16>(p, V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_dqkwg<f16>(p, V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_bwd_prepare_wy_repr(const void* k, const void* v, const float* beta, const float* g_cumsum,
                                       const void* Aw, const void* dw, const void* du, const void* dk_in, void* dk,
                                       void* dv, float* dbeta, float* dg, const int64_t* offsets,
                                       const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T,
                                       int64_t H, int64_t K, int64_t V, fla_stream_t stream) {
  FLA_REQUIRE(k && v && beta && Aw && dw && du && dk && dv && dbeta && dg, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)k | (uintptr_t)v | (uintptr_t)Aw | (uintptr_t)dw | (uintptr_t)du | (uintptr_t)dk_in |
               (uintptr_t)dk | (uintptr_t)dv) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  WyBwdParams p{k, v, beta, g_cumsum, Aw, dw, du, dk_in, dk, dv, dbeta, dg, offsets, indices, T, (int)H, ntfix, nullptr, 0, 0};
  if (qkv_dtype == FLA_BF16) return launch_wy_bwd<bf16>(p, K, V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_wy_bwd<f16>(p, K, V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}
