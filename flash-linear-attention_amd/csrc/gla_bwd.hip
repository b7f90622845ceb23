// Chunked GLA backward for gfx950 (chunk size 64, 16-bit q/k/v/do, fp32 state).
//
// With G the chunk-local prefix sum of the log-gates, q~ = s q e^{G},
// k^ = k e^{G_last-G}, A = tril(q~ (k e^{-G})^T), dH_c the gradient w.r.t. the state
// LEAVING chunk c (fla/ops/gla/chunk.py:1217-1320, fla/ops/common/chunk_h.py:156-271):
//
//   gla_bwd_dh_kernel    reverse state scan:  store dH_c;  dH <- diag(e^{G_last}) dH + q~^T do.
//                        The tile is kept and stored transposed ([V,K], MFMA-fragment order), the
//                        orientation dk contracts it in; also emits dh0.
//   gla_bwd_dh_qg_kernel the same scan on the gated queries q e^{G} and the chunk decays e^{G_last} a
//                        states-keeping forward left: no prefix sums, no exponentials, 16-byte row pieces.
//   gla_bwd_dv_kernel    per (chunk, head):  dv = A^T do + k^ dH_c.  dv contracts dH over K: the
//                        stored [V,K] fragments are turned round on the matrix pipe (a product with a
//                        permuted identity is a transposition of the accumulator layout, exact for
//                        16-bit values).
//   gla_bwd_dqkg_kernel  per (chunk, head, 64-wide half of K):
//                          dA = tril(do v^T)
//                          dq = s e^{G}  * (dA (k e^{-G}) + do h_c^T)
//                          dk = s e^{-G} * (dA^T (q e^{G})) + e^{G_last-G} * (v dH_c^T)
//                          dg = reverse-cumsum(q*dq - k*dk) + sum_t k*dk_inter + e^{G_last} sum_v h_c*dH_c
//                          (the last sum from the h_c and dH_c fragments the kernel holds anyway)
//                        (fla/ops/gla/chunk.py:409-567 intra, :726-837 inter incl. the dg formula
//                        :818-823).  As in the forward, one reference point per chunk replaces
//                        the 16x16 sub-block scheme.
// The chunk-parallel kernels also exist for one gate per (token, head) (chunk_simple_gla's backward,
// fla/ops/simple_gla/chunk.py:134-210): the gate word of a row is broadcast over the lane's key channels and dg
// leaves as its sum over the key channels.
#include <type_traits>

#include "chunk_common.h"

namespace {

// Gate operand of the chunk-parallel kernels: GT is the element type of per-key log-gates [rows, H, K], or
// HeadGate for one fp32 log-gate per (token, head), [rows, H], which a lane broadcasts over its key channels.
struct HeadGate {};
template <typename GT> struct GateOf { typedef GT elem; static constexpr bool per_head = false; };
template <> struct GateOf<HeadGate> { typedef float elem; static constexpr bool per_head = true; };

struct BDhParams {
  const void* q;
  const void* g;
  const void* dout;
  const float* dht;
  void* dhtf;         // out: dH, FLA_H_FRAGMENT_T
  float* dh0;         // out: fp32 [N,H,K,V] or null
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  int64_t T;
  int64_t total_chunks;
  int H, K, V, N;
  float scale;
  const void* qg;      // optional: the gated queries q e^{G} the forward staged, [rows, H, K] in the q dtype
  const float* decay;  //   and e^{G_last} per chunk, [chunks, H, K]
};

// The same scan from what a states-keeping forward left behind: dH_c = e^{G_last} dH_{c+1} + s (q e^{G})^T do with
// the gated queries and the decay factors read back instead of being formed from q and g again - no prefix sums,
// no exponentials, 16-byte loads (5 memory instructions per lane and chunk instead of 24) and half the bytes.  The
// tiles are plain row-major copies; both operands of the update contract over time, i.e. over the tiles' rows,
// and come out of LDS through the transposing load.  The scale is kept out of the operands: the accumulators
// carry dH / s (the incoming d ht is divided by s, every copy that leaves is multiplied by it).
template <typename T>
__global__ __launch_bounds__(256) void gla_bwd_dh_qg_kernel(BDhParams p) {
  typedef typename Elem<T>::v8 v8;
  __shared__ __attribute__((aligned(16))) T sQ[2][64 * LDT];  // [t][k] q e^{G}
  __shared__ __attribute__((aligned(16))) T sD[2][64 * LDT];  // [t][v] do
  __shared__ __attribute__((aligned(16))) float sDecay[2][64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = p.H, K = p.K, V = p.V;
  const int nkt = K / 64, nvt = V / 64, ntile = nkt * nvt;
  int64_t id = xcd_remap(blockIdx.x, gridDim.x);
  const int tile = (int)(id % ntile);
  const int nh = (int)(id / ntile);
  const int n = nh / H, hh = nh % H;
  const int kbase = (tile % nkt) * 64, vbase = (tile / nkt) * 64;
  SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);

  // a lane owns two 16-byte pieces of each tile: rows prow and prow + 32, columns c8 ..
  const int prow = tid >> 3, c8 = (tid & 7) * 8;
  const char* qp = (const char*)((const T*)p.qg + (sp.bos * H + hh) * (int64_t)K + kbase + c8);
  const char* dp = (const char*)((const T*)p.dout + (sp.bos * H + hh) * (int64_t)V + vbase + c8);
  const float* cp = p.decay + (chunk0 * H + hh) * (int64_t)K + kbase + (tid & 63);
  const uint32_t pitchK = (uint32_t)H * K * (uint32_t)sizeof(T), pitchV = (uint32_t)H * V * (uint32_t)sizeof(T);
  const int64_t strideC = (int64_t)H * K;

  const int kq = wave & 1, vq = wave >> 1;
  const int kt32 = kbase / 32 + kq, vt32 = vbase / 32 + vq;
  const int kcol = kbase + kq * 32 + (lane & 31);
  // An empty sequence hands d ht through to d h0 bit for bit: no factor goes on and off it.
  const float scale = nchunks > 0 ? p.scale : 1.f, inv_scale = 1.f / scale;
  f32x16 acc2 = zero16();  // rows v, cols k: dH / s
  if (p.dht) {
    const float* dp0 = p.dht + (int64_t)nh * K * V;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc2[r] = dp0[(int64_t)kcol * V + vbase + vq * 32 + c32_row(r, lane)] * inv_scale;
  }
  struct Regs {
    v8 q[2], d[2];
    float dec;
  };
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };
  // Every load is unconditional: rows past the end of a short (last) chunk are redirected to its last row and
  // their do rows zeroed where they are staged (the forward did not write gated queries there).
  auto load_chunk = [&](int64_t c, Regs& R) {
    const uint32_t last = (uint32_t)(chunk_len(c) - 1);
    const char* qb = qp + c * BT * (int64_t)pitchK;
    const char* db = dp + c * BT * (int64_t)pitchV;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t row = (uint32_t)(prow + 32 * i) < last ? (uint32_t)(prow + 32 * i) : last;
      R.q[i] = *(const v8*)(qb + row * pitchK);
      R.d[i] = *(const v8*)(db + row * pitchV);
    }
    R.dec = cp[c * strideC];
  };
  // One barrier per chunk, tiles double-buffered in LDS; two register sets, each refilled right after the
  // staging step that consumed it.
  auto step = [&](int64_t c, Regs& R, auto more) {
    const int buf = (int)(c & 1);
    const int L = chunk_len(c);
    // ---- gradient w.r.t. the state leaving chunk c, transposed fragment order
    {
      int64_t blk = ((chunk0 + c) * H + hh) * (int64_t)K * V;
      v8 lo, hi;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        lo[r] = (T)(acc2[r] * scale);
        hi[r] = (T)(acc2[r + 8] * scale);
      }
      T* o2 = (T*)p.dhtf + blk + (((int64_t)vt32 * (K / 32) + kt32) * 64 + lane) * 16;
      *(v8*)o2 = lo;
      *(v8*)(o2 + 8) = hi;
    }
    const v8 z8 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = prow + 32 * i;
      *(v8*)&sQ[buf][row * LDT + c8] = R.q[i];
      *(v8*)&sD[buf][row * LDT + c8] = row < L ? R.d[i] : z8;
    }
    if (tid < 64) sDecay[buf][tid] = R.dec;
    if constexpr (decltype(more)::value) {
      load_chunk(c >= 2 ? c - 2 : 0, R);
      asm volatile("" ::: "memory");  // the loads stay here, ahead of the barrier
    }
    lds_barrier();
    {
      const float d = sDecay[buf][kq * 32 + (lane & 31)];
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[r] *= d;
    }
#pragma unroll
    for (int s = 0; s < BT; s += 16) {
      v8 fq = frag32_tr<T>(sQ[buf], LDT, kq * 32, s, lane);
      v8 fd = frag32_tr<T>(sD[buf], LDT, vq * 32, s, lane);
      acc2 = Elem<T>::mfma32(fd, fq, acc2);
    }
  };
  Regs R0, R1;
  if (nchunks > 0) {
    load_chunk(nchunks - 1, R0);
    asm volatile("" ::: "memory");
    load_chunk(nchunks > 1 ? nchunks - 2 : 0, R1);
    asm volatile("" ::: "memory");
    int64_t c = nchunks - 1;
    for (; c >= 3; c -= 2) {
      step(c, R0, std::true_type{});
      step(c - 1, R1, std::true_type{});
    }
    if (c == 2) {
      step(2, R0, std::true_type{});
      step(1, R1, std::false_type{});
      step(0, R0, std::false_type{});
    } else {
      step(c, R0, std::false_type{});
      if (c == 1) step(0, R1, std::false_type{});
    }
  }
  if (p.dh0) {
    float* o = p.dh0 + (int64_t)nh * K * V;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
      *(f32x4*)&o[(int64_t)kcol * V + vbase + vq * 32 + 8 * r4 + 4 * (lane >> 5)] =
          f32x4{acc2[4 * r4] * scale, acc2[4 * r4 + 1] * scale, acc2[4 * r4 + 2] * scale, acc2[4 * r4 + 3] * scale};
  }
}

// ---------------------------------------------------------------------------
// Reverse state scan and dv in one pass, from what a states-keeping forward left: the gated queries q e^{G}, the
// chunk decays e^{G_last}, k^ = k e^{G_last-G} (key-major tiles) and the causal score tile P = tril(q~ k~^T):
//   dv_c = s P_c^T do_c + k^_c dH_c          dH_{c-1} = e^{G_last} dH_c + s (q e^{G})_c^T do_c
// (fla/ops/gla/chunk.py:1037-1061 with fla/ops/common/chunk_h.py:338-402).  dH never comes back from memory for dv,
// and neither q, k nor the gates are read.  One workgroup of eight waves per (sequence, head, 32 value columns):
// waves 4-7 ("staging") load the next chunk's tiles, write them to LDS and store dv; waves 0-3 ("matrix") carry
// dH / s in accumulators (both orientations: the fragment-order copy for the dq/dk launch is the transposed one)
// and do the products.  Per chunk c (walking backwards) the groups meet twice:
//   B1(c)  k^, P, do of chunk c and the 16-bit dH_c are in LDS
//          matrix:  dv = s P^T do + k^ dH -> LDS (transposed)           staging: q e^{G}, decay, do of chunk c -> LDS
//   B2(c)  matrix:  dH <- decay * dH + (q e^{G})^T do; publishes dH     staging: dv of chunk c -> memory; chunk c-1 -> LDS
// Chunks whose cumulative log-gate left the single-reference range (flagged) get their intra-chunk term from the exact
// kernel: P is skipped for them (k^ and q e^{G} are exact for any gate).
struct BDhvParams {
  const void* qg;       // [rows, H, K]
  const void* kh_t;     // [chunks, H, K, 64]
  const void* scores;   // [chunks, H, 64, 64]
  const float* decay;   // [chunks, H, K]
  const void* dout;     // [rows, H, V]
  const float* dht;     // [N, H, K, V] or null
  const int* wide;      // [chunks, H] or null
  void* dhtf;           // out: dH, FLA_H_FRAGMENT_T
  void* dv;             // out: [rows, H, V]
  float* dh0;           // out: [N, H, K, V] or null
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  int64_t T;
  int H, V, N;
  float scale;
};

template <typename T, int K>
__global__ __launch_bounds__(512) void gla_bwd_dhv_kernel(BDhvParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int BV = 32;
  constexpr int LDK = K + 8;
  constexpr int LDV = BV + 8;
  constexpr int C8 = K / 8, NP = BT * C8 / 256;   // q e^{G}: 16-byte pieces per row / per staging lane
  constexpr int PR = 256 / C8;                    // rows between two pieces of a lane
  constexpr int NKH = K * (BT / 8) / 256;         // k^ tile: pieces per staging lane (the tile is contiguous in memory)
  constexpr int NPP = BT * (BT / 8) / 256;        // score tile: pieces per staging lane
  constexpr int KT32 = K / 32;
  static_assert(KT32 <= 4, "one 32-row block of the state per matrix wave");
  __shared__ __attribute__((aligned(16))) T sKh[K * LDT];      // k^, key-major [k][t]
  __shared__ __attribute__((aligned(16))) T sQ[BT * LDK];      // q e^{G}, row-major [t][k]
  __shared__ __attribute__((aligned(16))) T sP[BT * LDT];      // P [i][j]
  __shared__ __attribute__((aligned(16))) T sDoY[BT * LDV];    // do [t][v], for the dv products
  __shared__ __attribute__((aligned(16))) T sDoX[BT * LDV];    // do [t][v], for the update
  __shared__ __attribute__((aligned(16))) T sDHt[BV * LDK];    // dH^T in 16-bit [v][k]
  __shared__ __attribute__((aligned(16))) T sDvT[BV * LDT];    // dv^T [v][t]
  __shared__ __attribute__((aligned(16))) float sDec[K];       // e^{G_last} of the chunk being folded in
  __shared__ int sFlag;

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
  // An empty sequence hands d ht through to d h0 bit for bit: no factor goes on and off it.
  const float scale = nchunks > 0 ? p.scale : 1.f, inv_scale = 1.f / scale;

  if (wave >= 4) {
    // =========================== staging waves ===========================
    if (nchunks == 0) return;
    const int st = tid - 256;
    const int prow = st / C8, c8 = (st % C8) * 8;   // q e^{G}: piece i of a lane is row prow + PR i, columns c8 ..
    const int vrow = st >> 2, vc8 = (st & 3) * 8;   // do, dv: one row, 8 of the 32 columns
    struct XRegs {
      v8 q[NP];
      float dec;
    };
    struct YRegs {
      v8 kh[NKH];
      v8 pp[NPP];
      v8 d;
      int flag;
    };
    // Every load is unconditional: rows past the end of a short chunk are redirected to its last row (their do rows
    // are zeroed where they are staged), chunks before the first one to chunk 0.
    const uint32_t pitchK = (uint32_t)H * K * (uint32_t)sizeof(T), pitchV = (uint32_t)H * V * (uint32_t)sizeof(T);
    uint32_t offk[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) offk[i] = (uint32_t)(prow + PR * i) * pitchK + (uint32_t)c8 * (uint32_t)sizeof(T);
    const uint32_t offv = (uint32_t)vrow * pitchV + (uint32_t)vc8 * (uint32_t)sizeof(T);
    const char* gq = (const char*)p.qg + (sp.bos * H + hh) * (int64_t)K * (int64_t)sizeof(T);
    const char* gd = (const char*)p.dout + ((sp.bos * H + hh) * (int64_t)V + vbase) * (int64_t)sizeof(T);
    const char* gk = (const char*)p.kh_t + (chunk0 * H + hh) * (int64_t)K * BT * (int64_t)sizeof(T) + 16 * st;
    const char* gp = (const char*)p.scores + (chunk0 * H + hh) * (int64_t)BT * BT * (int64_t)sizeof(T) + 16 * st;
    const float* gdec = p.decay + (chunk0 * H + hh) * (int64_t)K + (st & (K - 1));
    const int* gf = p.wide ? p.wide + chunk0 * H + hh : (const int*)&kZeroWord;
    const int64_t strKh = (int64_t)H * K * BT * (int64_t)sizeof(T), strP = (int64_t)H * BT * BT * (int64_t)sizeof(T);
    auto load_x = [&](int64_t c, XRegs& R) __attribute__((always_inline)) {
      c = c < 0 ? 0 : c;
      const uint32_t last = (uint32_t)(chunk_len(c) - 1);
      const int64_t ck = c * BT * (int64_t)pitchK;
      const uint32_t lk = last * pitchK + (uint32_t)c8 * (uint32_t)sizeof(T);
#pragma unroll
      for (int i = 0; i < NP; ++i) R.q[i] = *(const v8*)(gq + ck + (offk[i] < lk ? offk[i] : lk));
      R.dec = gdec[c * (int64_t)H * K];
    };
    auto load_y = [&](int64_t c, YRegs& R) __attribute__((always_inline)) {
      c = c < 0 ? 0 : c;
      const uint32_t last = (uint32_t)(chunk_len(c) - 1);
#pragma unroll
      for (int i = 0; i < NKH; ++i) R.kh[i] = *(const v8*)(gk + c * strKh + 4096 * i);
#pragma unroll
      for (int i = 0; i < NPP; ++i) R.pp[i] = *(const v8*)(gp + c * strP + 4096 * i);
      const uint32_t lv = last * pitchV + (uint32_t)vc8 * (uint32_t)sizeof(T);
      R.d = *(const v8*)(gd + c * BT * (int64_t)pitchV + (offv < lv ? offv : lv));
      R.flag = gf[p.wide ? c * H : 0];
    };
    v8 dkeep;   // this lane's do piece of the chunk last staged as Y (zero past the end of the chunk)
    auto stage_x = [&](const XRegs& R) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < NP; ++i) *(v8*)&sQ[(prow + PR * i) * LDK + c8] = R.q[i];
      *(v8*)&sDoX[vrow * LDV + vc8] = dkeep;
      if (st < K) sDec[st] = R.dec;
    };
    auto stage_y = [&](const YRegs& R, int64_t c) __attribute__((always_inline)) {
      const int L = chunk_len(c);
#pragma unroll
      for (int i = 0; i < NKH; ++i) {
        const int e = st + 256 * i;
        *(v8*)&sKh[(e >> 3) * LDT + (e & 7) * 8] = R.kh[i];
      }
#pragma unroll
      for (int i = 0; i < NPP; ++i) {
        const int e = st + 256 * i;
        *(v8*)&sP[(e >> 3) * LDT + (e & 7) * 8] = R.pp[i];
      }
      const v8 z8 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};
      dkeep = vrow < L ? R.d : z8;
      *(v8*)&sDoY[vrow * LDV + vc8] = dkeep;
      if (st == 0) sFlag = R.flag;
    };
    // dv of chunk c leaves as whole rows, 16 bytes per lane: a 16-lane group turns a block of 8 value columns x
    // 16 time rows of the transposed tile round with two transposing LDS loads.  Only a sequence's last chunk (the
    // first one processed) can be short: it takes the variant with the masked store.
    const int dgrp = st >> 4, dtb = dgrp >> 2, dvb = dgrp & 3, dj = st & 15;
    const int dsrc = (8 * dvb + (dj >> 2)) * LDT + 16 * dtb + 4 * (dj & 3);
    auto store_dv = [&](int64_t c, auto maybe_short) __attribute__((always_inline)) {
      typedef short s4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) s4 lds_s4;
      s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sDvT[dsrc]);
      s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)&sDvT[dsrc + 4 * LDT]);
      const v8 x = __builtin_shufflevector(__builtin_bit_cast(v4, lo), __builtin_bit_cast(v4, hi), 0, 1, 2, 3, 4, 5, 6, 7);
      const int row = 16 * dtb + dj;
      T* dst = (T*)p.dv + ((sp.bos + c * BT + row) * H + hh) * (int64_t)V + vbase + 8 * dvb;
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
    if (nchunks > 1) {
      lds_barrier();  // B1(nchunks - 1)
      stage_x(X);
      load_x(nchunks - 2, X);
      lds_barrier();  // B2(nchunks - 1)
      store_dv(nchunks - 1, std::true_type{});
      stage_y(Y, nchunks - 2);
      load_y(nchunks - 3, Y);
      for (int64_t c = nchunks - 2; c >= 1; --c) {
        lds_barrier();  // B1(c)
        stage_x(X);
        load_x(c - 1, X);
        lds_barrier();  // B2(c)
        store_dv(c, std::false_type{});
        stage_y(Y, c - 1);
        load_y(c - 2, Y);
      }
    }
    lds_barrier();  // B1(0)
    stage_x(X);
    lds_barrier();  // B2(0)
    store_dv(0, std::true_type{});
  } else {
    // =========================== matrix waves ===========================
    const int kt = wave;   // this wave's 32 key rows of the state gradient
    f32x16 acc = zero16(), acct = zero16();   // dH / s: rows k x columns v, and transposed
    if (p.dht && kt < KT32) {
      const float* d0 = p.dht + (int64_t)nh * K * V;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[r] = d0[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] * inv_scale;
        acct[r] = d0[(int64_t)(kt * 32 + (lane & 31)) * V + vbase + c32_row(r, lane)] * inv_scale;
      }
    }
    // gradient w.r.t. the state leaving chunk c: 16-bit transpose in LDS, FRAGMENT_T copy in memory
    auto publish = [&](int64_t c) __attribute__((always_inline)) {
      if (kt < KT32) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          v4 x;
#pragma unroll
          for (int b = 0; b < 4; ++b) x[b] = (T)(acc[4 * q4 + b] * scale);
          *(v4*)&sDHt[(lane & 31) * LDK + kt * 32 + 8 * q4 + 4 * (lane >> 5)] = x;
        }
        v8 lo, hi;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          lo[r] = (T)(acct[r] * scale);
          hi[r] = (T)(acct[r + 8] * scale);
        }
        T* hp = (T*)p.dhtf + ((chunk0 + c) * H + hh) * (int64_t)K * V + (((int64_t)vt * (K / 32) + kt) * 64 + lane) * 16;
        *(v8*)hp = lo;
        *(v8*)(hp + 8) = hi;
      }
    };
    if (nchunks > 0) publish(nchunks - 1);
    for (int64_t c = nchunks - 1; c >= 0; --c) {
      lds_barrier();  // B1(c)
      // ---- dv = s P^T do + k^ dH: wave w owns time rows 16w .. 16w+15, two 16-column tiles
      {
        f32x4 d[2] = {zero4(), zero4()}, dl[2] = {zero4(), zero4()};
#pragma unroll
        for (int ks = 0; ks < K; ks += 32) {
          const v8 a = frag16_tr<T>(sKh, LDT, wave * 16, ks, lane);
#pragma unroll
          for (int j = 0; j < 2; ++j) d[j] = Elem<T>::mfma16(a, frag16<T>(sDHt, LDK, j * 16, ks, lane), d[j]);
        }
        if (!sFlag) {
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            if (32 * s + 31 < 16 * wave) continue;   // P is lower triangular (wave-uniform)
            const v8 a = frag16_tr<T>(sP, LDT, wave * 16, 32 * s, lane);
#pragma unroll
            for (int j = 0; j < 2; ++j) dl[j] = Elem<T>::mfma16(a, frag16_tr<T>(sDoY, LDV, 16 * j, 32 * s, lane), dl[j]);
          }
        }
        const int tr = wave * 16 + 4 * (lane >> 4);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int vc = j * 16 + (lane & 15);
          v4 o;
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r] = (T)(scale * dl[j][r] + d[j][r]);
          *(v4*)&sDvT[vc * LDT + tr] = o;
        }
      }
      lds_barrier();  // B2(c)
      // ---- dH / s <- decay * dH / s + (q e^{G})^T do, in both orientations
      if (kt < KT32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] *= sDec[kt * 32 + c32_row(r, lane)];
        const float dt = sDec[kt * 32 + (lane & 31)];
#pragma unroll
        for (int r = 0; r < 16; ++r) acct[r] *= dt;
#pragma unroll
        for (int s = 0; s < BT; s += 16) {
          const v8 fq = frag32_tr<T>(sQ, LDK, kt * 32, s, lane);
          const v8 fd = frag32_tr<T>(sDoX, LDV, 0, s, lane);
          acc = Elem<T>::mfma32(fq, fd, acc);
          acct = Elem<T>::mfma32(fd, fq, acct);
        }
      }
      if (c > 0) publish(c - 1);
    }
    if (p.dh0 && kt < KT32) {
      float* o = p.dh0 + (int64_t)nh * K * V;
#pragma unroll
      for (int r = 0; r < 16; ++r) o[(int64_t)(kt * 32 + c32_row(r, lane)) * V + vbase + (lane & 31)] = acc[r] * scale;
    }
  }
}

template <typename T, typename GT>
__global__ __launch_bounds__(256) void gla_bwd_dh_kernel(BDhParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef T t2 __attribute__((ext_vector_type(2)));
  typedef GT g2 __attribute__((ext_vector_type(2)));
  __shared__ __attribute__((aligned(16))) T sQt[2][64 * LDT];  // [k][t] s q e^{G}
  __shared__ __attribute__((aligned(16))) T sDt[2][64 * LDT];  // [v][t] do
  __shared__ __attribute__((aligned(16))) float sDecay[2][64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = p.H, K = p.K, V = p.V;
  const int nkt = K / 64, nvt = V / 64, ntile = nkt * nvt;
  int64_t id = xcd_remap(blockIdx.x, gridDim.x);
  const int tile = (int)(id % ntile);
  const int nh = (int)(id / ntile);
  const int n = nh / H, hh = nh % H;
  const int kbase = (tile % nkt) * 64, vbase = (tile / nkt) * 64;
  SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t chunk0 = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);

  const int rg = lane >> 3, c2 = wave * 16 + (lane & 7) * 2;
  const T* qp = (const T*)p.q + (sp.bos * H + hh) * (int64_t)K + kbase + c2;
  const GT* gp = (const GT*)p.g + (sp.bos * H + hh) * (int64_t)K + kbase + c2;
  const T* dp = (const T*)p.dout + (sp.bos * H + hh) * (int64_t)V + vbase + c2;
  const int64_t kstride = (int64_t)H * K, vstride = (int64_t)H * V;

  const int kq = wave & 1, vq = wave >> 1;
  const int kt32 = kbase / 32 + kq, vt32 = vbase / 32 + vq;
  const int vcol = vbase + vq * 32 + (lane & 31), kcol = kbase + kq * 32 + (lane & 31);
  f32x16 acc2 = zero16();  // rows v, cols k
  if (p.dht) {
    const float* dp0 = p.dht + (int64_t)nh * K * V;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc2[r] = dp0[(int64_t)kcol * V + vbase + vq * 32 + c32_row(r, lane)];
  }

  struct Regs {
    g2 g[8];
    t2 q[8];
    t2 d[8];
  };
  auto chunk_len = [&](int64_t c) {
    int64_t rem = sp.len - c * BT;
    return (int)(rem < BT ? rem : BT);
  };
  // Every load is unconditional: rows past the end of a short (last) chunk are redirected to its
  // last row (one unsigned minimum on a byte offset) and masked where they are used.
  const uint32_t pitchK = (uint32_t)kstride * sizeof(T), pitchG = (uint32_t)kstride * sizeof(GT);
  const uint32_t pitchV = (uint32_t)vstride * sizeof(T);
  auto load_chunk = [&](int64_t c, Regs& R) {
    const uint32_t last = (uint32_t)(chunk_len(c) - 1);
    const uint32_t limk = last * pitchK, limg = last * pitchG, limv = last * pitchV;
    const char* qb = (const char*)(qp + c * BT * kstride);
    const char* gb = (const char*)(gp + c * BT * kstride);
    const char* db = (const char*)(dp + c * BT * vstride);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t row = (uint32_t)(rg * 8 + i);
      uint32_t ok = row * pitchK, og = row * pitchG, ov = row * pitchV;
      R.g[i] = *(const g2*)(gb + (og < limg ? og : limg));
      R.q[i] = *(const t2*)(qb + (ok < limk ? ok : limk));
      R.d[i] = *(const t2*)(db + (ov < limv ? ov : limv));
    }
  };

  // One barrier per chunk, operand tiles double-buffered in LDS.  Two register sets, each
  // refilled right after the staging step that consumed it: a chunk is in flight for almost two
  // iterations and no register copy sits between a load and its use.
  auto step = [&](int64_t c, Regs& R, auto more) {
    const int buf = (int)(c & 1);
    const int L = chunk_len(c);
    // ---- gradient w.r.t. the state leaving chunk c, transposed fragment order
    {
      int64_t blk = ((chunk0 + c) * H + hh) * (int64_t)K * V;
      v8 lo, hi;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        lo[r] = (T)acc2[r];
        hi[r] = (T)acc2[r + 8];
      }
      T* o2 = (T*)p.dhtf + blk + (((int64_t)vt32 * (K / 32) + kt32) * 64 + lane) * 16;
      *(v8*)o2 = lo;
      *(v8*)(o2 + 8) = hi;
    }
    // ---- chunk-local prefix sums of the gates
    float G[8][2], glast0, glast1;
    {
      float r0 = 0.f, r1 = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        bool valid = (rg * 8 + i) < L;
        r0 += valid ? (float)R.g[i][0] : 0.f;
        r1 += valid ? (float)R.g[i][1] : 0.f;
        G[i][0] = r0;
        G[i][1] = r1;
      }
      float s0 = r0, s1 = r1;
#pragma unroll
      for (int d = 8; d < 64; d <<= 1) {
        float u0 = __shfl_up(s0, d, 64), u1 = __shfl_up(s1, d, 64);
        if (lane >= d) {
          s0 += u0;
          s1 += u1;
        }
      }
      float off0 = s0 - r0, off1 = s1 - r1;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        G[i][0] += off0;
        G[i][1] += off1;
      }
      glast0 = __shfl(s0, 56 + (lane & 7), 64);
      glast1 = __shfl(s1, 56 + (lane & 7), 64);
    }
    {
      v8 qa, qb, da, db;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        bool valid = (rg * 8 + i) < L;
        qa[i] = (T)(valid ? (float)R.q[i][0] * p.scale * __expf(G[i][0]) : 0.f);
        qb[i] = (T)(valid ? (float)R.q[i][1] * p.scale * __expf(G[i][1]) : 0.f);
        da[i] = R.d[i][0];
        db[i] = R.d[i][1];
      }
      *(v8*)&sQt[buf][(c2 + 0) * LDT + rg * 8] = qa;
      *(v8*)&sQt[buf][(c2 + 1) * LDT + rg * 8] = qb;
      *(v8*)&sDt[buf][(c2 + 0) * LDT + rg * 8] = da;
      *(v8*)&sDt[buf][(c2 + 1) * LDT + rg * 8] = db;
      if (rg == 0) *(f32x2*)&sDecay[buf][c2] = f32x2{__expf(glast0), __expf(glast1)};
    }
    if constexpr (decltype(more)::value) {
      load_chunk(c >= 2 ? c - 2 : 0, R);
      asm volatile("" ::: "memory");  // the loads stay here, ahead of the barrier
    }
    lds_barrier();
    {
      const float d = sDecay[buf][kq * 32 + (lane & 31)];
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[r] *= d;
    }
#pragma unroll
    for (int s = 0; s < BT; s += 16) {
      v8 fq = lds_frag32<T>(sQt[buf], LDT, kq * 32, s, lane);
      v8 fd = lds_frag32<T>(sDt[buf], LDT, vq * 32, s, lane);
      acc2 = Elem<T>::mfma32(fd, fq, acc2);
    }
  };
  Regs R0, R1;
  if (nchunks > 0) {
    load_chunk(nchunks - 1, R0);
    asm volatile("" ::: "memory");  // the two sets are issued one after the other, as in the loop:
    load_chunk(nchunks > 1 ? nchunks - 2 : 0, R1);  // interleaved, the loop's first wait would cover both
    asm volatile("" ::: "memory");
    int64_t c = nchunks - 1;
    for (; c >= 3; c -= 2) {
      step(c, R0, std::true_type{});
      step(c - 1, R1, std::true_type{});
    }
    // the last one to three chunks: nothing is left to prefetch for the final two
    if (c == 2) {
      step(2, R0, std::true_type{});
      step(1, R1, std::false_type{});
      step(0, R0, std::false_type{});
    } else {
      step(c, R0, std::false_type{});
      if (c == 1) step(0, R1, std::false_type{});
    }
  }
  if (p.dh0) {
    float* o = p.dh0 + (int64_t)nh * K * V;
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
      *(f32x4*)&o[(int64_t)kcol * V + vbase + vq * 32 + 8 * r4 + 4 * (lane >> 5)] =
          f32x4{acc2[4 * r4], acc2[4 * r4 + 1], acc2[4 * r4 + 2], acc2[4 * r4 + 3]};
  }
}

// ---------------------------------------------------------------------------
struct BDvParams {
  const void* q;
  const void* k;
  const void* g;
  const void* dout;
  const void* dhtf;  // dH, FLA_H_FRAGMENT_T
  const int* wide;   // [chunks, H] or null: chunks whose intra-chunk part is left to the exact kernel
  void* dv;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  float scale;
};

template <typename T, typename GT, int K, int V>
__global__ __launch_bounds__(256, 2) void gla_bwd_dv_kernel(BDvParams p, uint32_t nitems) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  constexpr int CG = K / 4, RG = 256 / CG, RPT = BT / RG;
  constexpr int CGV = V / 4, RGV = 256 / CGV, RPTV = BT / RGV;
  constexpr int KT32 = K / 32, TV = V / 64;
  constexpr int LDV = V + 8;
  __shared__ __attribute__((aligned(16))) T sQ[BT * (K > V ? LDK : LDV)];   // s q e^{G-G_last}; later the dv tile [t][v]
  __shared__ __attribute__((aligned(16))) T sKh[BT * LDK];   // k e^{G_last-G}
  __shared__ __attribute__((aligned(16))) T sDt[V * LDT];    // do^T [v][i]
  __shared__ __attribute__((aligned(16))) T sPT[BT * LDT];   // A^T [j][i]
  __shared__ __attribute__((aligned(16))) float sPart[RG * K];

  const int tid0 = threadIdx.x;
  const int H = p.H;
  // A workgroup walks (chunk, head) items with a stride of the grid size; the q, k, g and do rows of the next
  // item are requested as soon as those of the current one are in LDS (32-bit offsets off wave-uniform bases;
  // rows past the end of a short chunk re-read its last row and are masked at use, so no load sits under a
  // branch).
  struct Item {
    ChunkLoc cl;
    int hh;
  };
  auto locate = [&](uint32_t it) {
    Item r;
    r.cl = locate_chunk_at32(it, p.offsets, p.indices, p.T, p.NTfix, H, &r.hh);
    return r;
  };
  typedef typename GateOf<GT>::elem GE;
  constexpr bool PER_HEAD = GateOf<GT>::per_head;
  typedef GE g4 __attribute__((ext_vector_type(4)));
  struct Raw {
    g4 g[RPT];
    v4 q[RPT], k[RPT], d[RPTV];
  };
  constexpr int GSH = sizeof(GE) == 4 ? 1 : 0;   // gate bytes = q/k bytes << GSH
  const uint32_t pitchk = (uint32_t)H * K * (uint32_t)sizeof(T), pitchv = (uint32_t)H * V * (uint32_t)sizeof(T);
  const uint32_t colk = (uint32_t)((tid0 % CG) * 4) * (uint32_t)sizeof(T), colv = (uint32_t)((tid0 % CGV) * 4) * (uint32_t)sizeof(T);
  uint32_t offk[RPT], offv[RPTV];
#pragma unroll
  for (int i = 0; i < RPT; ++i) offk[i] = (uint32_t)((tid0 / CG) * RPT + i) * pitchk + colk;
#pragma unroll
  for (int i = 0; i < RPTV; ++i) offv[i] = (uint32_t)((tid0 / CGV) * RPTV + i) * pitchv + colv;
  auto request = [&](const Item& im, Raw& R) __attribute__((always_inline)) {
    const uint32_t last = (uint32_t)(im.cl.L - 1);
    const int64_t r0h = im.cl.row0 * H + im.hh;
    const char* qb = (const char*)p.q + r0h * K * (int64_t)sizeof(T);
    const char* kb = (const char*)p.k + r0h * K * (int64_t)sizeof(T);
    const char* gb = (const char*)p.g + r0h * (PER_HEAD ? 1 : K) * (int64_t)sizeof(GE);
    const char* db = (const char*)p.dout + r0h * V * (int64_t)sizeof(T);
    const uint32_t limk = last * pitchk + colk, limv = last * pitchv + colv;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const uint32_t o = offk[i] < limk ? offk[i] : limk;
      if constexpr (PER_HEAD) {
        const uint32_t row = (uint32_t)((tid0 / CG) * RPT + i);
        const float x = *(const float*)(gb + (row < last ? row : last) * (uint32_t)H * 4u);
        R.g[i] = g4{x, x, x, x};
      } else {
        R.g[i] = *(const g4*)(gb + (o << GSH));
      }
      R.q[i] = *(const v4*)(qb + o);
      R.k[i] = *(const v4*)(kb + o);
    }
#pragma unroll
    for (int i = 0; i < RPTV; ++i) R.d[i] = *(const v4*)(db + (offv[i] < limv ? offv[i] : limv));
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

  // gates beyond the single-reference range: the scores are left out here and added by
  // gla_bwd_intra_exact_kernel
  const bool flagged = p.wide && p.wide[cl.cglob * H + hh];
  const int rg = tid / CG, c4 = (tid % CG) * 4;
  float gq[RPT][4], qq[RPT][4], kk[RPT][4];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const bool ok = rg * RPT + i < L;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      gq[i][j] = ok ? (float)R.g[i][j] : 0.f;
      qq[i][j] = ok ? (float)R.q[i][j] : 0.f;
      kk[i][j] = ok ? (float)R.k[i][j] : 0.f;
    }
  }
  const int rgv = tid / CGV, cv4 = (tid % CGV) * 4;
  v4 dreg[RPTV];
#pragma unroll
  for (int i = 0; i < RPTV; ++i) dreg[i] = rgv * RPTV + i < L ? R.d[i] : v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
  const int rw = wave >> 1, cw = wave & 1;
  // ---- prefix sums and G_last
  float G[RPT][4], glast[4];
  {
    float run[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < RPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        run[j] += gq[i][j];
        G[i][j] = run[j];
      }
    *(f32x4*)&sPart[rg * K + c4] = f32x4{run[0], run[1], run[2], run[3]};
    __syncthreads();
    float off[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) glast[j] = 0.f;
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      f32x4 pr = *(const f32x4*)&sPart[r * K + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (r < rg) off[j] += pr[j];
        glast[j] += pr[j];
      }
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) G[i][j] += off[j];
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    int row = rg * RPT + i;
    v4 qv, kv;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float up = fminf(G[i][j] - glast[j], InvDecayLimit<T>::value);
      qv[j] = (T)(qq[i][j] * p.scale * __expf(up));
      kv[j] = (T)(kk[i][j] * __expf(glast[j] - G[i][j]));
    }
    *(v4*)&sQ[row * LDK + c4] = qv;
    *(v4*)&sKh[row * LDK + c4] = kv;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    T* dst = &sDt[(cv4 + j) * LDT + rgv * RPTV];
#pragma unroll
    for (int i = 0; i < RPTV; ++i) dst[i] = dreg[i][j];
  }
  const uint32_t nit = it + gridDim.x;
  const bool more = nit < nitems;   // workgroup-uniform
  const Item nim = locate(more ? nit : it);   // (past the last item the request repeats it)
  request(nim, R);
  // dH tiles as stored: rows v, columns k (a lane holds one key column); on their way during the score phase
  v8 hf[KT32][TV][2];
  {
    const char* hp = (const char*)p.dhtf + (cl.cglob * H + hh) * (int64_t)K * V * (int64_t)sizeof(T);
#pragma unroll
    for (int kt = 0; kt < KT32; ++kt)
#pragma unroll
      for (int tv = 0; tv < TV; ++tv) {
        const uint32_t o = (uint32_t)((((cw * TV + tv) * KT32 + kt) * 64 + lane) * 16) * (uint32_t)sizeof(T);
        hf[kt][tv][0] = *(const v8*)(hp + o);
        hf[kt][tv][1] = *(const v8*)(hp + o + 16);
      }
  }
  __syncthreads();
  // ---- A^T on the lower-triangular quadrants
  {
    const int qi = wave >> 1, qj = wave & 1;
    if (qj <= qi) {
      f32x16 s = zero16();
#pragma unroll
      for (int ks = 0; ks < K; ks += 16)
        s = Elem<T>::mfma32(lds_frag32<T>(sQ, LDK, qi * 32, ks, lane), lds_frag32<T>(sKh, LDK, qj * 32, ks, lane), s);
      const int j = qj * 32 + (lane & 31);
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int i0 = qi * 32 + 8 * a + 4 * (lane >> 5);
        v4 x;
#pragma unroll
        for (int b = 0; b < 4; ++b) x[b] = (T)((j <= i0 + b && !flagged) ? s[4 * a + b] : 0.f);
        *(v4*)&sPT[j * LDT + i0] = x;
      }
    }
  }
  __syncthreads();
  // ---- dv^T = do^T A + dH^T k^^T (transposed products: a lane ends up with one time row and four
  // consecutive value columns per register quad)
  f32x16 acc[TV];
#pragma unroll
  for (int tv = 0; tv < TV; ++tv) acc[tv] = zero16();
  for (int is = rw * 32; is < BT; is += 16) {
    v8 a = lds_frag32<T>(sPT, LDT, rw * 32, is, lane);
#pragma unroll
    for (int tv = 0; tv < TV; ++tv)
      acc[tv] = Elem<T>::mfma32(lds_frag32<T>(sDt, LDT, (cw * TV + tv) * 32, is, lane), a, acc[tv]);
  }
  // The state term contracts over k, so the tiles are needed with a lane per value column.  A tile in
  // accumulator order is, read as the first operand, its own transpose (lane = row index of the product,
  // registers = contraction index in accumulator-row order); multiplied by the identity in the same
  // permuted order the product comes out in accumulator order with lanes and registers exchanged.
  v8 eye[2];
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      eye[half][e] = (T)(((lane & 31) == 16 * half + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3)) ? 1.f : 0.f);
#pragma unroll
  for (int kt = 0; kt < KT32; ++kt) {
    v8 ht[TV][2];
#pragma unroll
    for (int tv = 0; tv < TV; ++tv) {
      f32x16 t = Elem<T>::mfma32(hf[kt][tv][0], eye[0], zero16());
      t = Elem<T>::mfma32(hf[kt][tv][1], eye[1], t);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ht[tv][0][e] = (T)t[e];
        ht[tv][1][e] = (T)t[8 + e];
      }
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v8 a = lds_frag32_perm<T>(sKh, LDK, rw * 32, kt * 32 + half * 16, lane);
#pragma unroll
      for (int tv = 0; tv < TV; ++tv) acc[tv] = Elem<T>::mfma32(ht[tv][half], a, acc[tv]);
    }
  }
  // the q tile is dead since the score phase: the dv tile goes through it and leaves as whole rows
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
  T* op = (T*)p.dv + (row0 * H + hh) * (int64_t)V;
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
struct BDqkgParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const void* dout;
  const void* hT;     // forward states, FLA_H_FRAGMENT_T
  const void* dhtf;   // dH, FLA_H_FRAGMENT_T
  const int* wide;    // [chunks, H] or null: chunks whose intra-chunk part is left to the exact kernel
  void* dq;
  void* dk;
  float* dg;
  float* dg_head;   // or: fp32 [rows, H], zeroed by the caller, receives the sums of dg over the key channels (dg unused)
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int64_t total_chunks;
  int H, K, NTfix;
  float scale;
};

// grid (chunks, H, K/64): one workgroup per 64-wide slice of the key dim.
template <typename T, typename GT, int V>
__global__ __launch_bounds__(256, 2) void gla_bwd_dqkg_kernel(BDqkgParams p, int64_t pairs) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDV = V + 8;
  constexpr int C8 = V / 8, NP = BT * C8 / 256;
  constexpr int VT32 = V / 32;
  constexpr int ROWB = BT * LDV * 2;                       // bytes of one row-major [64][V] tile
  constexpr int STG = BT * LDM * 4;                        // bytes of one fp32 [64][64] staging tile
  constexpr int REG_A = ROWB > STG ? ROWB : STG;
  constexpr int REG_C = (2 * BT * LDT * 2 > STG) ? 2 * BT * LDT * 2 : STG;
  __shared__ __attribute__((aligned(16))) char sRA[REG_A];   // do row-major; later staging of the dq accumulators
  __shared__ __attribute__((aligned(16))) char sRB[REG_A];   // v row-major;  later staging of the intra dk accumulators
  __shared__ __attribute__((aligned(16))) char sRC[REG_C];   // (k e^{-G})^T | (q e^{G})^T; later staging of the inter dk acc
  __shared__ __attribute__((aligned(16))) T sdA[BT * LDT];   // dA  [i][j]
  __shared__ __attribute__((aligned(16))) T sdAT[BT * LDT];  // dA^T [j][i]
  __shared__ __attribute__((aligned(16))) float sPart[16 * 64];
  __shared__ __attribute__((aligned(16))) float sPart2[16 * 64];
  __shared__ float sHd[64];                                   // sum_v h_c * dH_c per key channel of the slice
  T* sDo = (T*)sRA;
  T* sV = (T*)sRB;
  T* sKtT = (T*)sRC;
  T* sQtT = sKtT + BT * LDT;
  float* stA = (float*)sRA;
  float* stB = (float*)sRB;
  float* stC = (float*)sRC;

  const int tid0 = threadIdx.x;
  const int H = p.H, K = p.K;
  // A workgroup walks items (chunk, head, key slice) with a stride of the grid size.  The key slices of one
  // (chunk, head) share v and do: where the counts allow, they are items 8 apart, i.e. they run at the same
  // time on the same XCD, and the second slice finds those tiles in that XCD's L2.
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
  // The rows an item starts with (do, v: whole rows in 16-byte pieces) are requested while the item before it
  // is in its epilogue; its q, k, g slice (4 rows x 4 columns per lane) and its state fragments are requested at
  // its top and arrive behind the dA products, which need do and v only.  All of it at 32-bit offsets from
  // wave-uniform base pointers; rows past the end of a short chunk re-read its last row (masked at use), so no
  // load sits under a branch.
  typedef typename GateOf<GT>::elem GE;
  constexpr bool PER_HEAD = GateOf<GT>::per_head;
  typedef GE g4 __attribute__((ext_vector_type(4)));
  struct Raw {
    v8 d[NP], v[NP];
  };
  const int rg0 = tid0 >> 4, c40 = (tid0 & 15) * 4;
  const uint32_t pitchk = (uint32_t)H * K * (uint32_t)sizeof(T), pitchv = (uint32_t)H * V * (uint32_t)sizeof(T);
  constexpr int GSH = sizeof(GE) == 4 ? 1 : 0;   // gate bytes = q/k bytes << GSH
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
    const char* db = (const char*)p.dout + r0h * V * (int64_t)sizeof(T);
    const char* vb = (const char*)p.v + r0h * V * (int64_t)sizeof(T);
    const uint32_t limv = last * pitchv + colv;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const uint32_t o = offv[i] < limv ? offv[i] : limv;
      R.d[i] = *(const v8*)(db + o);
      R.v[i] = *(const v8*)(vb + o);
    }
  };
  uint32_t it = blockIdx.x;
  if (it >= nitems) return;
  Item im = locate(it);
  Raw R;
  request(im, R);
  const v8 z8 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f, (T)0.f};
  for (;;) {
  // The lane id goes through an opaque copy once per item: the LDS addresses of the body are then formed where
  // they are used instead of being hoisted out of the loop into long-lived registers.
  int tid = tid0;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rg = tid >> 4, c4 = (tid & 15) * 4;
  const int hh = im.hh, kb = im.kb;
  const ChunkLoc cl = im.cl;
  const int L = cl.L;
  const int64_t row0 = cl.row0;

  // gates beyond the single-reference range: dA is left out here and the intra-chunk terms are
  // added by gla_bwd_intra_exact_kernel
  const bool flagged = p.wide && p.wide[cl.cglob * H + hh];
  // ---- do, v row-major (rows past the end zero)
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int e = tid + 256 * i, row = e / C8, c8 = (e % C8) * 8;
    *(v8*)&sDo[row * LDV + c8] = row < L ? R.d[i] : z8;
    *(v8*)&sV[row * LDV + c8] = row < L ? R.v[i] : z8;
  }
  // ---- this item's q, k, g slice and state fragments: on their way during the dA products
  g4 cg[4];
  v4 cq[4], ck[4];
  {
    const int64_t r0h = row0 * H + hh;
    const char* qb = (const char*)p.q + (r0h * K + kb) * (int64_t)sizeof(T);
    const char* kb_ = (const char*)p.k + (r0h * K + kb) * (int64_t)sizeof(T);
    const char* gb = PER_HEAD ? (const char*)p.g + r0h * 4 : (const char*)p.g + (r0h * K + kb) * (int64_t)sizeof(GE);
    const uint32_t limk = (uint32_t)(L - 1) * pitchk + colk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t o = offk[i] < limk ? offk[i] : limk;
      if constexpr (PER_HEAD) {
        const uint32_t row = (uint32_t)(rg0 * 4 + i), last = (uint32_t)(L - 1);
        const float x = *(const float*)(gb + (row < last ? row : last) * (uint32_t)H * 4u);
        cg[i] = g4{x, x, x, x};
      } else {
        cg[i] = *(const g4*)(gb + (o << GSH));
      }
      cq[i] = *(const v4*)(qb + o);
      ck[i] = *(const v4*)(kb_ + o);
    }
  }
  // operand fragments: wave (rw, cw) produces rows 32rw.., key columns kb + 32cw..
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
  __syncthreads();
  // ---- dA = tril(do v^T) in both orientations (each gives 8-byte LDS writes)
  {
    const int ib = wave >> 1, jb = wave & 1;
    if (jb <= ib) {
      f32x16 s1 = zero16(), s2 = zero16();
#pragma unroll
      for (int vs = 0; vs < V; vs += 16) {
        v8 fd = lds_frag32<T>(sDo, LDV, ib * 32, vs, lane);
        v8 fv = lds_frag32<T>(sV, LDV, jb * 32, vs, lane);
        s1 = Elem<T>::mfma32(fd, fv, s1);  // rows i, cols j
        s2 = Elem<T>::mfma32(fv, fd, s2);  // rows j, cols i
      }
      const int c = lane & 31;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        int r0 = 8 * a + 4 * (lane >> 5);
        v4 x1, x2;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          int i1 = ib * 32 + r0 + b, j1 = jb * 32 + c;      // s1 element (i1, j1)
          x1[b] = (T)((j1 <= i1 && !flagged) ? s1[4 * a + b] : 0.f);
          int j2 = jb * 32 + r0 + b, i2 = ib * 32 + c;      // s2 element (j2, i2)
          x2[b] = (T)((j2 <= i2 && !flagged) ? s2[4 * a + b] : 0.f);
        }
        *(v4*)&sdAT[(jb * 32 + c) * LDT + ib * 32 + r0] = x1;  // dA^T[j][i..i+3]
        *(v4*)&sdA[(ib * 32 + c) * LDT + jb * 32 + r0] = x2;   // dA[i][j..j+3]
      }
    } else {
      // quadrant (i block 0, j block 1) is strictly above the diagonal
      for (int e = lane; e < 32 * 8; e += 64) {
        int r = e >> 3, c = (e & 7) * 4;
        *(v4*)&sdA[r * LDT + 32 + c] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
        *(v4*)&sdAT[(32 + r) * LDT + c] = v4{(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      }
    }
  }
  // ---- prefix sums of the gates over the 16 row groups (q, k of the slice stay in storage precision until
  // the epilogue; rows past the end zero)
  float G[4][4], glast[4];
  {
    const v4 z4 = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
    float run[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = rg * 4 + i < L;
      cq[i] = ok ? cq[i] : z4;
      ck[i] = ok ? ck[i] : z4;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        run[j] += ok ? (float)cg[i][j] : 0.f;
        G[i][j] = run[j];
      }
    }
    *(f32x4*)&sPart[rg * 64 + c4] = f32x4{run[0], run[1], run[2], run[3]};
    __syncthreads();   // also publishes dA
    float off[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) glast[j] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      f32x4 pr = *(const f32x4*)&sPart[r * 64 + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (r < rg) off[j] += pr[j];
        glast[j] += pr[j];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) G[i][j] += off[j];
  }
  // ---- gated operand tiles
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v4 kt, qt;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      kt[i] = (T)((float)ck[i][j] * __expf(fminf(-G[i][j], InvDecayLimit<T>::value)));   // e^{-G}, clamped
      qt[i] = (T)((float)cq[i][j] * __expf(G[i][j]));
    }
    *(v4*)&sKtT[(c4 + j) * LDT + rg * 4] = kt;
    *(v4*)&sQtT[(c4 + j) * LDT + rg * 4] = qt;
  }
  __syncthreads();
  // ---- accumulate: dq (intra + inter), dk intra, dk inter
  f32x16 aq = zero16(), ak1 = zero16(), ak2 = zero16();
  const int jend = (rw + 1) * 32;
  // (transposed products - the key-channel operand first: a lane ends up with one time row and, per register quad,
  // four adjacent key channels, so the accumulators leave for the staging tiles as 16-byte pieces)
  for (int js = 0; js < jend; js += 16)
    aq = Elem<T>::mfma32(lds_frag32<T>(sKtT, LDT, cw * 32, js, lane), lds_frag32<T>(sdA, LDT, rw * 32, js, lane), aq);
  for (int is = rw * 32; is < BT; is += 16)
    ak1 = Elem<T>::mfma32(lds_frag32<T>(sQtT, LDT, cw * 32, is, lane), lds_frag32<T>(sdAT, LDT, rw * 32, is, lane), ak1);
  // sum over the value columns of h_c * dH_c on the way: both sets of fragments hold one key column per
  // lane, and each pair is dead once its products are issued (the two row-block waves of a column block
  // hold the same fragments; one of them reports)
  float hd = 0.f;
#pragma unroll
  for (int vt = 0; vt < VT32; ++vt)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      aq = Elem<T>::mfma32(hf[vt][half], lds_frag32_perm<T>(sDo, LDV, rw * 32, vt * 32 + half * 16, lane), aq);
      ak2 = Elem<T>::mfma32(dhf[vt][half], lds_frag32_perm<T>(sV, LDV, rw * 32, vt * 32 + half * 16, lane), ak2);
      hd = Elem<T>::dot8(hf[vt][half], dhf[vt][half], hd);
      __builtin_amdgcn_sched_barrier(0);
    }
  hd += __shfl_xor(hd, 32, 64);
  if (rw == 0 && lane < 32) sHd[cw * 32 + lane] = hd;
  __syncthreads();  // every MFMA operand read is done: the tiles become fp32 staging
#pragma unroll
  for (int a4 = 0; a4 < 4; ++a4) {
    const int o = (rw * 32 + (lane & 31)) * LDM + cw * 32 + 8 * a4 + 4 * (lane >> 5);
    *(f32x4*)&stA[o] = f32x4{aq[4 * a4], aq[4 * a4 + 1], aq[4 * a4 + 2], aq[4 * a4 + 3]};
    *(f32x4*)&stB[o] = f32x4{ak1[4 * a4], ak1[4 * a4 + 1], ak1[4 * a4 + 2], ak1[4 * a4 + 3]};
    *(f32x4*)&stC[o] = f32x4{ak2[4 * a4], ak2[4 * a4 + 1], ak2[4 * a4 + 2], ak2[4 * a4 + 3]};
  }
  // the next item's first rows are requested now: the accumulators are in LDS, the epilogue needs few registers
  const uint32_t nit = it + gridDim.x;
  const bool more = nit < nitems;   // workgroup-uniform
  const Item nim = locate(more ? nit : it);   // (past the last item the request repeats it: no load under a branch)
  request(nim, R);
  __syncthreads();
  // ---- epilogue in the load mapping (4 rows x 4 key channels per lane)
  float x[4][4], ksum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = rg * 4 + i;
    f32x4 a = *(const f32x4*)&stA[row * LDM + c4];
    f32x4 b = *(const f32x4*)&stB[row * LDM + c4];
    f32x4 c = *(const f32x4*)&stC[row * LDM + c4];
    v4 dqv, dkv;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // (the gate factors go through an opaque copy: the rounded operands below are recomputed
      // here instead of being kept in registers from the staging step to this point)
      float gij = G[i][j];
      asm volatile("" : "+v"(gij));
      const float eg = __expf(gij), ei = __expf(fminf(-gij, InvDecayLimit<T>::value));
      const float qf = (float)cq[i][j], kf = (float)ck[i][j];
      float dq = p.scale * eg * a[j];
      float dki = __expf(glast[j] - gij) * c[j];
      float dk = p.scale * ei * b[j] + dki;
      dqv[j] = (T)dq;
      dkv[j] = (T)dk;
      // dg sums q*dq - k*dk over later rows: an intra-chunk pair (i, j) enters q*dq at row i and
      // k*dk at row j and cancels unless it straddles the row.  Formed with the rounded operands
      // the matrix products used, the two copies are equal and cancel exactly; with strong gates,
      // where dg is small against either sum, this is what keeps its error at rounding level.
      const float qr = (float)(T)(qf * eg);
      const float kr = (float)(T)(kf * ei);
      x[i][j] = p.scale * (qr * a[j] - kr * b[j]) - kf * dki;
      ksum[j] += kf * dki;
    }
    if (row < L) {
      int64_t off = ((row0 + row) * H + hh) * (int64_t)K + kb + c4;
      *(v4*)((T*)p.dq + off) = dqv;
      *(v4*)((T*)p.dk + off) = dkv;
    }
  }
  // reverse cumsum over rows + column sums of k*dk_inter
  float suf[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 3; i >= 0; --i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      suf[j] += x[i][j];
      x[i][j] = suf[j];
    }
  *(f32x4*)&sPart[rg * 64 + c4] = f32x4{suf[0], suf[1], suf[2], suf[3]};
  *(f32x4*)&sPart2[rg * 64 + c4] = f32x4{ksum[0], ksum[1], ksum[2], ksum[3]};
  __syncthreads();
  float add[4] = {0.f, 0.f, 0.f, 0.f};
  // (four row groups at a time: all 32 reads in flight at once would take 128 registers from the rows that
  // are on their way for the next item)
#pragma unroll
  for (int r0 = 0; r0 < 16; r0 += 4) {
#pragma unroll
    for (int r = r0; r < r0 + 4; ++r) {
      f32x4 s1 = *(const f32x4*)&sPart[r * 64 + c4];
      f32x4 s2 = *(const f32x4*)&sPart2[r * 64 + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (r > rg) add[j] += s1[j];
        add[j] += s2[j];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) add[j] += __expf(glast[j]) * sHd[c4 + j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = rg * 4 + i;
    f32x4 o = {x[i][0] + add[0], x[i][1] + add[1], x[i][2] + add[2], x[i][3] + add[3]};
    if (p.dg_head) {
      // one gate per (token, head): the sum over this slice's 64 key channels, which sit in the 16 lanes of a DPP
      // row; the slices of a head (and the exact kernel, a launch later) add up in a fixed order
      const float tot = row_prefix16((o[0] + o[1]) + (o[2] + o[3]));
      if ((tid & 15) == 15 && row < L) atomicAdd(p.dg_head + (row0 + row) * H + hh, tot);
    } else if (row < L) {
      *(f32x4*)(p.dg + ((row0 + row) * H + hh) * (int64_t)K + kb + c4) = o;
    }
  }
  if (!more) break;
  __syncthreads();  // the staging tiles are consumed: the next item's operand tiles may be written
  it = nit;
  im = nim;
  }
}

// ---------------------------------------------------------------------------
// Intra-chunk part of the backward for chunks whose cumulative log-gate leaves the range in
// which one reference point per chunk is exact.  gla_bwd_dv_kernel and gla_bwd_dqkg_kernel
// leave the score terms of such chunks out; this kernel adds them with pairwise exponents
// G_i - G_j <= 0, the arithmetic of the reference's diagonal sub-blocks
// (fla/ops/gla/chunk.py:409-567):
//   A_ij  = s sum_k q_ik k_jk e^{G_ik-G_jk},  dA_ij = do_i . v_j            (j <= i)
//   dv_j += sum_{i>=j} A_ij do_i
//   dq_ik += s sum_{j<=i} dA_ij k_jk e^{G_ik-G_jk},  dk_jk += s sum_{i>=j} dA_ij q_ik e^{G_ik-G_jk}
//   dg_ik += sum_{t>=i} (q_tk dq'_tk - k_tk dk'_tk)          (dq', dk': the terms added here)
// Plain fp32 arithmetic on the vector ALU: it only runs for flagged chunks.
struct BExactParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const void* dout;
  const int* wide;
  void* dq;
  void* dk;
  void* dv;
  float* dg;
  float* dg_head;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int H, NTfix;
  float scale;
  int64_t total;   // (chunk, head) pairs
};

template <typename T, typename GT, int K, int V>
__global__ __launch_bounds__(256) void gla_bwd_intra_exact_kernel(BExactParams p) {
  typedef typename Elem<T>::v4 v4;
  constexpr int LDG = K + 1, LDQ = K + 8, LDVV = V + 8, LDA = BT + 1;
  constexpr int VD_BYTES = 2 * BT * LDVV * 2;
  constexpr int X_BYTES = BT * LDG * 4;
  const int H = p.H;
  // A few hundred workgroups walk the (chunk, head) flags (almost always none is set).  The lanes first read
  // all flags of the workgroup side by side (one memory latency instead of one per flag) and leave if none is set.
  {
    int any = 0;
    for (int64_t lin = blockIdx.x + (int64_t)threadIdx.x * gridDim.x; lin < p.total; lin += (int64_t)256 * gridDim.x)
      any |= p.wide[lin];
    if (!__syncthreads_or(any)) return;
  }
  for (int64_t lin = blockIdx.x; lin < p.total; lin += gridDim.x) {
  if (p.wide[lin] == 0) continue;  // workgroup-uniform
  __syncthreads();                 // the tiles of the previous flagged chunk are free
  int hh;
  ChunkLoc cl = locate_chunk_at(lin, p.offsets, p.indices, p.T, p.NTfix, H, &hh);
  __shared__ float sG[BT * LDG];
  __shared__ __attribute__((aligned(16))) T sQ[BT * LDQ];
  __shared__ __attribute__((aligned(16))) T sK[BT * LDQ];
  __shared__ __attribute__((aligned(16))) char sVD[VD_BYTES > X_BYTES ? VD_BYTES : X_BYTES];  // v | do, later x
  __shared__ float sA[BT * LDA];
  __shared__ float sdA[BT * LDA];
  T* sV = (T*)sVD;
  T* sDo = sV + BT * LDVV;
  float* sX = (float*)sVD;
  const int tid = threadIdx.x;
  const int L = cl.L;
  const int64_t row0 = cl.row0;
  const int64_t strideK = (int64_t)H * K, strideV = (int64_t)H * V;
  const int64_t baseK = (row0 * H + hh) * (int64_t)K, baseV = (row0 * H + hh) * (int64_t)V;

  for (int e = tid; e < BT * (K / 4); e += 256) {
    int row = e / (K / 4), c4 = (e % (K / 4)) * 4;
    float gv[4] = {0.f, 0.f, 0.f, 0.f};
    v4 qv = {(T)0.f, (T)0.f, (T)0.f, (T)0.f}, kv = qv;
    if (row < L) {
      int64_t off = baseK + row * strideK + c4;
      if constexpr (GateOf<GT>::per_head) {
        gv[0] = gv[1] = gv[2] = gv[3] = ((const float*)p.g)[(row0 + row) * H + hh];
      } else {
        Load<GT>::x4((const GT*)p.g + off, gv);
      }
      qv = *(const v4*)((const T*)p.q + off);
      kv = *(const v4*)((const T*)p.k + off);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) sG[row * LDG + c4 + j] = gv[j];
    *(v4*)&sQ[row * LDQ + c4] = qv;
    *(v4*)&sK[row * LDQ + c4] = kv;
  }
  for (int e = tid; e < BT * (V / 4); e += 256) {
    int row = e / (V / 4), c4 = (e % (V / 4)) * 4;
    v4 vv = {(T)0.f, (T)0.f, (T)0.f, (T)0.f}, dv = vv;
    if (row < L) {
      int64_t off = baseV + row * strideV + c4;
      vv = *(const v4*)((const T*)p.v + off);
      dv = *(const v4*)((const T*)p.dout + off);
    }
    *(v4*)&sV[row * LDVV + c4] = vv;
    *(v4*)&sDo[row * LDVV + c4] = dv;
  }
  __syncthreads();
  // prefix sums of the gates along time, one channel per thread
  for (int c = tid; c < K; c += 256) {
    float run = 0.f;
    for (int t = 0; t < BT; ++t) {
      run += sG[t * LDG + c];
      sG[t * LDG + c] = run;
    }
  }
  __syncthreads();
  // A and dA, one (i, j) pair at a time
  for (int e = tid; e < BT * BT; e += 256) {
    int i = e >> 6, j = e & 63;
    float a = 0.f, da = 0.f;
    if (j <= i && i < L) {
      for (int c = 0; c < K; ++c)
        a += (float)sQ[i * LDQ + c] * (float)sK[j * LDQ + c] * __expf(sG[i * LDG + c] - sG[j * LDG + c]);
      for (int c = 0; c < V; ++c) da += (float)sDo[i * LDVV + c] * (float)sV[j * LDVV + c];
    }
    sA[i * LDA + j] = a * p.scale;
    sdA[i * LDA + j] = da * p.scale;
  }
  __syncthreads();
  // dv_j += sum_{i>=j} A_ij do_i
  for (int e = tid; e < BT * (V / 4); e += 256) {
    int j = e / (V / 4), c4 = (e % (V / 4)) * 4;
    if (j >= L) continue;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i = j; i < L; ++i) {
      float a = sA[i * LDA + j];
      v4 d = *(const v4*)&sDo[i * LDVV + c4];
#pragma unroll
      for (int x = 0; x < 4; ++x) acc[x] += a * (float)d[x];
    }
    T* dst = (T*)p.dv + baseV + j * strideV + c4;
    v4 old = *(const v4*)dst, nw;
#pragma unroll
    for (int x = 0; x < 4; ++x) nw[x] = (T)((float)old[x] + acc[x]);
    *(v4*)dst = nw;
  }
  __syncthreads();  // v and do are consumed: their storage becomes x = q dq' - k dk'
  for (int e = tid; e < BT * (K / 4); e += 256) {
    int r = e / (K / 4), c4 = (e % (K / 4)) * 4;
    float xq[4] = {0.f, 0.f, 0.f, 0.f}, xk[4] = {0.f, 0.f, 0.f, 0.f};
    if (r < L) {
      float dq[4] = {0.f, 0.f, 0.f, 0.f}, dk[4] = {0.f, 0.f, 0.f, 0.f};
      float gr[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) gr[x] = sG[r * LDG + c4 + x];
      for (int j = 0; j <= r; ++j) {       // row r as the query row i
        float da = sdA[r * LDA + j];
        v4 kj = *(const v4*)&sK[j * LDQ + c4];
#pragma unroll
        for (int x = 0; x < 4; ++x) dq[x] += da * (float)kj[x] * __expf(gr[x] - sG[j * LDG + c4 + x]);
      }
      for (int i = r; i < L; ++i) {        // row r as the key row j
        float da = sdA[i * LDA + r];
        v4 qi = *(const v4*)&sQ[i * LDQ + c4];
#pragma unroll
        for (int x = 0; x < 4; ++x) dk[x] += da * (float)qi[x] * __expf(sG[i * LDG + c4 + x] - gr[x]);
      }
      v4 qr = *(const v4*)&sQ[r * LDQ + c4], kr = *(const v4*)&sK[r * LDQ + c4];
      T* dqp = (T*)p.dq + baseK + r * strideK + c4;
      T* dkp = (T*)p.dk + baseK + r * strideK + c4;
      v4 oq = *(const v4*)dqp, ok = *(const v4*)dkp, nq, nk;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        nq[x] = (T)((float)oq[x] + dq[x]);
        nk[x] = (T)((float)ok[x] + dk[x]);
        xq[x] = (float)qr[x] * dq[x];
        xk[x] = (float)kr[x] * dk[x];
      }
      *(v4*)dqp = nq;
      *(v4*)dkp = nk;
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) sX[r * LDG + c4 + x] = xq[x] - xk[x];
  }
  __syncthreads();
  // dg_ik += sum_{t>=i} x_tk, one channel per thread
  for (int c = tid; c < K; c += 256) {
    float run = 0.f;
    for (int t = L - 1; t >= 0; --t) {
      run += sX[t * LDG + c];
      if (p.dg_head) sX[t * LDG + c] = run;
      else p.dg[baseK + t * strideK + c] += run;
    }
  }
  if (p.dg_head) {
    // one gate per (token, head): a row's channels are summed in a fixed order, one addition per row
    __syncthreads();
    for (int t = tid; t < L; t += 256) {
      float sum = 0.f;
      for (int c = 0; c < K; ++c) sum += sX[t * LDG + c];
      atomicAdd(p.dg_head + (cl.row0 + t) * H + hh, sum);
    }
  }
  }
}

template <typename T, typename GT>
int launch_bwd(const void* q, const void* k, const void* v, const void* g, const void* dout, const float* dht,
               const void* hT, const void* qg, const float* decay, void* dhtf, void* dq, void* dk, void* dv, float* dg,
               float* dg_head, float* dh0, const int* wide,
               const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT, int64_t B,
               int64_t T_, int64_t H, int64_t K, int64_t V, int64_t N, float scale, hipStream_t st,
               const void* kh_t = nullptr, const void* scores = nullptr) {
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T_, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return copy_or_zero(dht, dh0, N * H * K * V, st);   // no chunk at all: d h0 = d ht
  const int64_t total_chunks = grid.x;
  const bool fused_dv = qg && kh_t && scores;   // the reverse state scan also forms dv
  if (fused_dv) {
    BDhvParams p{qg, kh_t, scores, decay, dout, dht, wide, dhtf, dv, dh0, offsets, chunk_offsets, T_, (int)H, (int)V, (int)N,
                 scale};
    const int64_t total = (V / 32) * N * H;
    FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
    if (K == 64) hipLaunchKernelGGL((gla_bwd_dhv_kernel<T, 64>), dim3((unsigned)total), dim3(512), 0, st, p);
    else if (K == 128) hipLaunchKernelGGL((gla_bwd_dhv_kernel<T, 128>), dim3((unsigned)total), dim3(512), 0, st, p);
    else return FLA_E_UNSUPPORTED;
    FLA_CHECK_LAUNCH();
  } else {
    BDhParams p{q, g, dout, dht, dhtf, dh0, offsets, chunk_offsets, T_, total_chunks,
                (int)H, (int)K, (int)V, (int)N, scale, qg, decay};
    int64_t total = (K / 64) * (V / 64) * N * H;
    FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
    if (qg) hipLaunchKernelGGL((gla_bwd_dh_qg_kernel<T>), dim3((unsigned)total), dim3(256), 0, st, p);
    else if constexpr (GateOf<GT>::per_head) return FLA_E_INVALID;   // per-head gates come with kept gated queries
    else hipLaunchKernelGGL((gla_bwd_dh_kernel<T, GT>), dim3((unsigned)total), dim3(256), 0, st, p);
    FLA_CHECK_LAUNCH();
  }
  if (!fused_dv) {
    BDvParams p{q, k, g, dout, dhtf, wide, dv, offsets, indices, T_, (int)H, ntfix, scale};
    // as many workgroups as are resident at once, each walking its share of the (chunk, head) items
    const int64_t total = (int64_t)grid.x * grid.y;
    FLA_REQUIRE(total <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
#define FLA_CASE(KK, VV)                                                                            \
  if (K == KK && V == VV) {                                                                         \
    const int64_t res = resident_workgroups(gla_bwd_dv_kernel<T, GT, KK, VV>);                      \
    hipLaunchKernelGGL((gla_bwd_dv_kernel<T, GT, KK, VV>), dim3((unsigned)(total < res ? total : res)), dim3(256), 0, st, p, \
                       (uint32_t)total);                                                            \
  }
    FLA_CASE(64, 64) else FLA_CASE(128, 128) else FLA_CASE(64, 128) else FLA_CASE(128, 64) else return FLA_E_UNSUPPORTED;
#undef FLA_CASE
    FLA_CHECK_LAUNCH();
  }
  {
    BDqkgParams p{q, k, v, g, dout, hT, dhtf, wide, dq, dk, dg, dg_head, offsets, indices, T_, total_chunks,
                  (int)H, (int)K, ntfix, scale};
    // as many workgroups as are resident at once (two per CU), each walking its share of the items
    const int64_t pairs = (int64_t)grid.x * grid.y, nwg = pairs * (K / 64);
    FLA_REQUIRE(nwg <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
    dim3 g3((unsigned)(nwg < 2 * kNumCUs ? nwg : 2 * kNumCUs));
    if (V == 64) hipLaunchKernelGGL((gla_bwd_dqkg_kernel<T, GT, 64>), g3, dim3(256), 0, st, p, pairs);
    else if (V == 128) hipLaunchKernelGGL((gla_bwd_dqkg_kernel<T, GT, 128>), g3, dim3(256), 0, st, p, pairs);
    else return FLA_E_UNSUPPORTED;
    FLA_CHECK_LAUNCH();
  }
  if (wide) {
    BExactParams p{q, k, v, g, dout, wide, dq, dk, dv, dg, dg_head, offsets, indices, T_, (int)H, ntfix, scale,
                   (int64_t)grid.x * grid.y};
    const dim3 gx((unsigned)(p.total < 512 ? p.total : 512));
#define FLA_CASE(KK, VV)                                                                                      \
  if (K == KK && V == VV) hipLaunchKernelGGL((gla_bwd_intra_exact_kernel<T, GT, KK, VV>), gx, dim3(256), 0, st, p);
    FLA_CASE(64, 64) else FLA_CASE(128, 128) else FLA_CASE(64, 128) else FLA_CASE(128, 64) else return FLA_E_UNSUPPORTED;
#undef FLA_CASE
    FLA_CHECK_LAUNCH();
  }
  return FLA_OK;
}

}  // namespace

static int gla_bwd_impl(const void* q, const void* k, const void* v, const void* gates, const void* dout,
                        const float* dht, const void* hT, const void* q_gated, const float* chunk_decay,
                        void* dh_frag_t, void* dq, void* dk, void* dv, float* dg, float* dg_head, float* dh0,
                        const int* wide,
                        const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                        int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                        int64_t N, float scale, fla_stream_t stream, bool head_gates = false,
                        const void* kh_t = nullptr, const void* scores = nullptr) {
  FLA_REQUIRE(q && k && v && gates && dout && hT && dh_frag_t && dq && dk && dv && (dg || dg_head),
              FLA_E_INVALID);
  if (head_gates) FLA_REQUIRE(q_gated && dg_head, FLA_E_INVALID);
  FLA_REQUIRE((kh_t == nullptr) == (scores == nullptr) && (kh_t == nullptr || q_gated != nullptr), FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)kh_t | (uintptr_t)scores) % 16 == 0, FLA_E_ALIGNMENT);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(K % 64 == 0 && V % 64 == 0 && K <= 128 && V <= 128, FLA_E_UNSUPPORTED);
  if (offsets) FLA_REQUIRE(indices && chunk_offsets && B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  FLA_REQUIRE((q_gated == nullptr) == (chunk_decay == nullptr), FLA_E_INVALID);
  if (q_gated) FLA_REQUIRE(scale != 0.f, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (head_gates ? 0 : (uintptr_t)gates) | (uintptr_t)dout |
               (uintptr_t)hT | (uintptr_t)dh_frag_t | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv |
               (uintptr_t)dg | (uintptr_t)q_gated) % 16 == 0,
              FLA_E_ALIGNMENT);
  hipStream_t st = (hipStream_t)stream;
#define FLA_BWD(TT, GG)                                                                                           \
  return launch_bwd<TT, GG>(q, k, v, gates, dout, dht, hT, q_gated, chunk_decay, dh_frag_t, dq, dk, dv, dg, dg_head, dh0, wide,   \
                            offsets, indices, chunk_offsets, NT, B, T, H, K, V, N, scale, st, kh_t, scores)
  if (head_gates && qkv_dtype == FLA_BF16) FLA_BWD(bf16, HeadGate);
  if (head_gates && qkv_dtype == FLA_F16) FLA_BWD(f16, HeadGate);
  if (head_gates) return FLA_E_UNSUPPORTED;
  if (qkv_dtype == FLA_BF16 && gate_dtype == FLA_F32) FLA_BWD(bf16, float);
  if (qkv_dtype == FLA_BF16 && gate_dtype == FLA_BF16) FLA_BWD(bf16, bf16);
  if (qkv_dtype == FLA_F16 && gate_dtype == FLA_F32) FLA_BWD(f16, float);
  if (qkv_dtype == FLA_F16 && gate_dtype == FLA_F16) FLA_BWD(f16, f16);
#undef FLA_BWD
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_gla_bwd(const void* q, const void* k, const void* v, const void* gates, const void* dout,
                                 const float* dht, const void* hT, void* dh_frag_t,
                                 void* dq, void* dk, void* dv, float* dg, float* dh0, const int* wide,
                                 const int64_t* offsets, const int64_t* indices, const int64_t* chunk_offsets,
                                 int64_t NT, int qkv_dtype,
                                 int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, int64_t N,
                                 float scale, fla_stream_t stream) {
  return gla_bwd_impl(q, k, v, gates, dout, dht, hT, nullptr, nullptr, dh_frag_t, dq, dk, dv, dg, nullptr, dh0, wide, offsets,
                      indices, chunk_offsets, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream);
}

extern "C" int fla_chunk_gla_bwd_kept(const void* q, const void* k, const void* v, const void* gates,
                                      const void* dout, const float* dht, const void* hT, const void* q_gated,
                                      const float* chunk_decay, const void* khat_t, const void* scores,
                                      void* dh_frag_t, void* dq, void* dk, void* dv,
                                      float* dg, float* dh0, const int* wide, const int64_t* offsets,
                                      const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                                      int qkv_dtype, int gate_dtype, int64_t B, int64_t T, int64_t H, int64_t K,
                                      int64_t V, int64_t N, float scale, fla_stream_t stream) {
  FLA_REQUIRE(q_gated && chunk_decay, FLA_E_INVALID);
  return gla_bwd_impl(q, k, v, gates, dout, dht, hT, q_gated, chunk_decay, dh_frag_t, dq, dk, dv, dg, nullptr, dh0, wide,
                      offsets, indices, chunk_offsets, NT, qkv_dtype, gate_dtype, B, T, H, K, V, N, scale, stream, false,
                      khat_t, scores);
}

extern "C" int fla_chunk_simple_gla_bwd(const void* q, const void* k, const void* v, const float* g, const void* dout,
                                        const float* dht, const void* hT, const void* q_gated,
                                        const float* chunk_decay, const void* khat_t, const void* scores,
                                        void* dh_frag_t, void* dq, void* dk, void* dv, float* dg, float* dh0, const int* wide, const int64_t* offsets,
                                        const int64_t* indices, const int64_t* chunk_offsets, int64_t NT,
                                        int qkv_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                        int64_t N, float scale, fla_stream_t stream) {
  FLA_REQUIRE(q_gated && chunk_decay && dg, FLA_E_INVALID);
  return gla_bwd_impl(q, k, v, g, dout, dht, hT, q_gated, chunk_decay, dh_frag_t, dq, dk, dv, nullptr, dg, dh0, wide,
                      offsets, indices, chunk_offsets, NT, qkv_dtype, FLA_F32, B, T, H, K, V, N, scale, stream, true,
                      khat_t, scores);
}
