// The chunk-parallel stages of gated linear attention under the operand layouts of the
// reference's internal functions, for sibling operators that compute the intra-chunk scores A
// and the per-chunk states themselves (RWKV6 calls them this way, fla/ops/rwkv6/chunk.py:1163,
// 1227, 1236): A is [B, T, H, 64] and the states h / dh are row-major [chunks, H, K, V].
//
//   fla_chunk_gla_fwd_o_gk : o  = (s q e^{g}) h + tril(A) v            fla/ops/gla/chunk.py:320-393
//   fla_chunk_gla_bwd_dA   : dA = s tril(do v^T)                       fla/ops/gla/chunk.py:582-624
//   fla_chunk_gla_bwd_dv   : dv = triu(A^T) do + (k e^{g_last-g}) dh   fla/ops/gla/chunk.py:642-710
//   fla_chunk_bwd_dh       : the reverse state scan with row-major dh  fla/ops/common/chunk_h.py:146-262
//
// The operator's own forward and backward never take this route (they keep the states in MFMA
// fragment order and recompute A on the fly); these are one workgroup per (chunk, head[, 64 value
// columns]) with every operand staged once through LDS, contraction index contiguous.
#include "chunk_common.h"

namespace {

struct PieceParams {
  const void* x;     // q (output stage) or k (dv stage), [B*T, H, K]
  const float* g;    // chunk-cumulative log-gates, [B*T, H, K]
  const void* A;     // intra-chunk scores, [B*T, H, 64]
  const void* m;     // h (output stage) or dh (dv stage), [chunks, H, K, V]
  const void* y;     // v (output stage) or do (dv stage), [B*T, H, V]
  void* out;         // o or dv, [B*T, H, V]
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int ntfix;
  int H;
  int V;
  float scale;
  int a_is_f32;
  int m_is_f32;
};

// eight consecutive elements of a tensor that is either fp32 or 16-bit, as fp32
template <typename T>
FLA_DEVICE void load8_as_f32(const void* base, int64_t idx, bool is_f32, float* o) {
  if (is_f32) {
    Load<float>::x4((const float*)base + idx, o);
    Load<float>::x4((const float*)base + idx + 4, o + 4);
  } else {
    Load<T>::x4((const T*)base + idx, o);
    Load<T>::x4((const T*)base + idx + 4, o + 4);
  }
}

template <typename T>
FLA_DEVICE void store_pair(T* dst, float a, float b) {
  typedef T t2 __attribute__((ext_vector_type(2)));
  t2 x;
  x[0] = (T)a;
  x[1] = (T)b;
  *(t2*)dst = x;
}

// DV == false: out[t][v] = sum_k X[t][k] M[k][v] + sum_{j<=t} A[t][j] Y[j][v],   X = s q e^{g}
// DV == true : out[j][v] = sum_k X[j][k] M[k][v] + sum_{i>=j} A[i][j] Y[i][v],   X = k e^{g_last-g}
template <typename T, int K, bool DV>
__global__ __launch_bounds__(256) void gla_piece_kernel(PieceParams p) {
  typedef typename Elem<T>::v8 v8;
  typedef typename Elem<T>::v4 v4;
  constexpr int LDK = K + 8;
  __shared__ __attribute__((aligned(16))) T sX[BT * LDK];    // [row][k]
  __shared__ __attribute__((aligned(16))) T sMt[64 * LDK];   // [v][k]
  __shared__ __attribute__((aligned(16))) T sS[BT * LDT];    // [row][contraction row]
  __shared__ __attribute__((aligned(16))) T sYt[64 * LDT];   // [v][contraction row]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // 1-D grid, value slabs of one (chunk, head) side by side on one XCD: the second slab finds the
  // q/k and gate rows of the first in that XCD's L2
  int hh;
  const int nslab = p.V / 64;
  const int64_t lid = xcd_remap(blockIdx.x, gridDim.x);
  const ChunkLoc cl = locate_chunk_at(lid / nslab, p.offsets, p.indices, p.T, p.ntfix, p.H, &hh);
  const int H = p.H, V = p.V, L = cl.L;
  const int vbase = (int)(lid % nslab) * 64;

  // X: 8 key channels of one row per unit
  {
    const T* x = (const T*)p.x;
    constexpr int UPR = K / 8;
    for (int u = tid; u < BT * UPR; u += 256) {
      const int row = u / UPR, kc = (u % UPR) * 8;
      v8 w;
      if (row < L) {
        const int64_t idx = ((cl.row0 + row) * H + hh) * (int64_t)K + kc;
        float xv[8], gv[8];
        Load<T>::x4(x + idx, xv);
        Load<T>::x4(x + idx + 4, xv + 4);
        Load<float>::x4(p.g + idx, gv);
        Load<float>::x4(p.g + idx + 4, gv + 4);
        if (DV) {
          float gn[8];
          const int64_t idn = ((cl.row0 + L - 1) * H + hh) * (int64_t)K + kc;
          Load<float>::x4(p.g + idn, gn);
          Load<float>::x4(p.g + idn + 4, gn + 4);
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e] = (T)(xv[e] * __expf(gn[e] - gv[e]));
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e] = (T)(xv[e] * p.scale * __expf(gv[e]));
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = (T)0.f;
      }
      *(v8*)&sX[row * LDK + kc] = w;
    }
  }
  // M^T: two state rows x 8 value columns per unit, written as (k, k+1) pairs
  {
    const int64_t mbase = (cl.cglob * H + hh) * (int64_t)K * V + vbase;
    for (int u = tid; u < (K / 2) * 8; u += 256) {
      const int kp = u >> 3, vc = (u & 7) * 8;
      float a[8], b[8];
      load8_as_f32<T>(p.m, mbase + (int64_t)(2 * kp) * V + vc, p.m_is_f32, a);
      load8_as_f32<T>(p.m, mbase + (int64_t)(2 * kp + 1) * V + vc, p.m_is_f32, b);
#pragma unroll
      for (int e = 0; e < 8; ++e) store_pair<T>(&sMt[(vc + e) * LDK + 2 * kp], a[e], b[e]);
    }
  }
  // S: the causal part of A, contraction index contiguous
  if (!DV) {
    for (int u = tid; u < BT * 8; u += 256) {
      const int i = u >> 3, jc = (u & 7) * 8;
      v8 w;
      if (i < L) {
        float a[8];
        load8_as_f32<T>(p.A, ((cl.row0 + i) * H + hh) * (int64_t)BT + jc, p.a_is_f32, a);
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = (T)(jc + e <= i ? a[e] : 0.f);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = (T)0.f;
      }
      *(v8*)&sS[i * LDT + jc] = w;
    }
  } else {
    const int ip = tid >> 3, jc = (tid & 7) * 8;   // rows 2ip, 2ip+1 of A, transposed on the way in
    float a[8], b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = b[e] = 0.f;
    if (2 * ip < L) load8_as_f32<T>(p.A, ((cl.row0 + 2 * ip) * H + hh) * (int64_t)BT + jc, p.a_is_f32, a);
    if (2 * ip + 1 < L) load8_as_f32<T>(p.A, ((cl.row0 + 2 * ip + 1) * H + hh) * (int64_t)BT + jc, p.a_is_f32, b);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      store_pair<T>(&sS[(jc + e) * LDT + 2 * ip], jc + e <= 2 * ip ? a[e] : 0.f, jc + e <= 2 * ip + 1 ? b[e] : 0.f);
  }
  // Y^T: two rows x 8 value columns per thread
  {
    const T* y = (const T*)p.y;
    const int tp = tid >> 3, vc = (tid & 7) * 8;
    float a[8], b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = b[e] = 0.f;
    if (2 * tp < L) {
      const int64_t idx = ((cl.row0 + 2 * tp) * H + hh) * (int64_t)V + vbase + vc;
      Load<T>::x4(y + idx, a);
      Load<T>::x4(y + idx + 4, a + 4);
    }
    if (2 * tp + 1 < L) {
      const int64_t idx = ((cl.row0 + 2 * tp + 1) * H + hh) * (int64_t)V + vbase + vc;
      Load<T>::x4(y + idx, b);
      Load<T>::x4(y + idx + 4, b + 4);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) store_pair<T>(&sYt[(vc + e) * LDT + 2 * tp], a[e], b[e]);
  }
  __syncthreads();

  // Transposed products (value columns as MFMA rows): a lane ends up with one output row and four
  // consecutive value columns per register quad, so the stores are 8 bytes wide.
  const int rw = wave >> 1, cw = wave & 1;
  f32x16 acc = zero16();
#pragma unroll
  for (int ks = 0; ks < K; ks += 16)
    acc = Elem<T>::mfma32(lds_frag32<T>(sMt, LDK, cw * 32, ks, lane), lds_frag32<T>(sX, LDK, rw * 32, ks, lane), acc);
  const int s0 = DV ? rw * 32 : 0, s1 = DV ? BT : (rw + 1) * 32;   // the other rows of S are zero
  for (int ss = s0; ss < s1; ss += 16)
    acc = Elem<T>::mfma32(lds_frag32<T>(sYt, LDT, cw * 32, ss, lane), lds_frag32<T>(sS, LDT, rw * 32, ss, lane), acc);
  const int row = rw * 32 + (lane & 31);
  if (row < L) {
    T* orow = (T*)p.out + ((cl.row0 + row) * H + hh) * (int64_t)V + vbase + cw * 32 + 4 * (lane >> 5);
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      v4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = (T)acc[4 * r4 + e];
      *(v4*)(orow + 8 * r4) = w;
    }
  }
}

struct DAParams {
  const void* v;
  const void* dout;
  float* dA;
  const int64_t* offsets;
  const int64_t* indices;
  int64_t T;
  int ntfix;
  int H;
  float scale;
};

template <typename T, int V>
__global__ __launch_bounds__(256) void gla_bwd_dA_kernel(DAParams p) {
  typedef typename Elem<T>::v8 v8;
  constexpr int LDV = V + 8;
  __shared__ __attribute__((aligned(16))) T sDo[BT * LDV];
  __shared__ __attribute__((aligned(16))) T sV[BT * LDV];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int hh;
  const ChunkLoc cl = locate_chunk(p.offsets, p.indices, p.T, p.ntfix, p.H, &hh);
  const int H = p.H, L = cl.L;
  constexpr int UPR = V / 8;
  for (int u = tid; u < BT * UPR; u += 256) {
    const int row = u / UPR, vc = (u % UPR) * 8;
    v8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = b[e] = (T)0.f;
    if (row < L) {
      const int64_t idx = ((cl.row0 + row) * H + hh) * (int64_t)V + vc;
      a = *(const v8*)((const T*)p.dout + idx);
      b = *(const v8*)((const T*)p.v + idx);
    }
    *(v8*)&sDo[row * LDV + vc] = a;
    *(v8*)&sV[row * LDV + vc] = b;
  }
  __syncthreads();
  const int rw = wave >> 1, cw = wave & 1;   // rows i, columns j
  f32x16 acc = zero16();
  if (cw <= rw) {
#pragma unroll
    for (int vs = 0; vs < V; vs += 16)
      acc = Elem<T>::mfma32(lds_frag32<T>(sV, LDV, cw * 32, vs, lane), lds_frag32<T>(sDo, LDV, rw * 32, vs, lane), acc);
  }
  const int i = rw * 32 + (lane & 31);
  if (i < L) {
    float* drow = p.dA + ((cl.row0 + i) * H + hh) * (int64_t)BT + cw * 32 + 4 * (lane >> 5);
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int j0 = cw * 32 + 8 * r4 + 4 * (lane >> 5);
      f32x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = j0 + e <= i ? acc[4 * r4 + e] * p.scale : 0.f;
      *(f32x4*)(drow + 8 * r4) = w;
    }
  }
}

// ---------------------------------------------------------------------------
// Reverse state scan with row-major output (chunk_bwd_kernel_dh, fla/ops/common/chunk_h.py:146-262):
// for c = last .. 0:  store dh_c;  dh <- e^{g_last} diag(e^{gk_last}) dh + (s q e^{g} e^{gk})^T do.
// One workgroup per (sequence, head, 64 key channels x 64 value columns), serial over chunks.
struct RowDhParams {
  const void* q;
  const float* g;     // [B*T, H] or null
  const float* gk;    // [B*T, H, K] or null
  const void* dout;
  const float* dht;   // [N, H, K, V] or null
  void* dh;           // [chunks, H, K, V]
  float* dh0;         // [N, H, K, V] or null
  const int64_t* offsets;
  const int64_t* chunk_offsets;
  int64_t T;
  int H, K, V;
  float scale;
  int dh_is_f32;
};

template <typename T>
__global__ __launch_bounds__(256) void chunk_bwd_dh_rowmajor_kernel(RowDhParams p) {
  __shared__ __attribute__((aligned(16))) T sQt[64 * LDT];   // [k][t]
  __shared__ __attribute__((aligned(16))) T sDt[64 * LDT];   // [v][t]
  __shared__ float sDecay[64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = p.H, K = p.K, V = p.V;
  // 1-D grid, the tiles of one (sequence, head) side by side on one XCD (they share q, do and the gates)
  const int nv = V / 64, ntile = (K / 64) * nv;
  const int64_t lid = xcd_remap(blockIdx.x, gridDim.x);
  const int tile = (int)(lid % ntile);
  const int kbase = (tile / nv) * 64, vbase = (tile % nv) * 64;
  const int n = (int)((lid / ntile) / H), hh = (int)((lid / ntile) % H);
  const SeqSpan sp = seq_span(p.offsets, n, p.T);
  const int64_t nchunks = (sp.len + BT - 1) / BT;
  const int64_t boh = p.chunk_offsets ? p.chunk_offsets[n] : (int64_t)n * ((p.T + BT - 1) / BT);
  const int kq = wave >> 1, vq = wave & 1;
  const int vcol = vbase + vq * 32 + (lane & 31);
  f32x16 acc = zero16();
  if (p.dht) {
    const float* s = p.dht + ((int64_t)n * H + hh) * K * V;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = s[(int64_t)(kbase + kq * 32 + c32_row(r, lane)) * V + vcol];
  }
  const int tp = tid >> 3, c8 = (tid & 7) * 8;
  for (int64_t c = nchunks - 1; c >= 0; --c) {
    const int64_t row0 = sp.bos + c * BT;
    const int L = (int)(sp.len - c * BT < BT ? sp.len - c * BT : BT);
    {
      const int64_t base = ((boh + c) * H + hh) * (int64_t)K * V;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t idx = base + (int64_t)(kbase + kq * 32 + c32_row(r, lane)) * V + vcol;
        if (p.dh_is_f32) ((float*)p.dh)[idx] = acc[r];
        else ((T*)p.dh)[idx] = (T)acc[r];
      }
    }
    // q~^T and do^T, two rows x 8 columns per thread, written as (t, t+1) pairs
    float qa[8], qb[8], da[8], db[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qa[e] = qb[e] = da[e] = db[e] = 0.f;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int t = 2 * tp + half;
      if (t < L) {
        float* qo = half ? qb : qa;
        float* dd = half ? db : da;
        const int64_t tok = (row0 + t) * H + hh;
        Load<T>::x4((const T*)p.q + tok * K + kbase + c8, qo);
        Load<T>::x4((const T*)p.q + tok * K + kbase + c8 + 4, qo + 4);
        Load<T>::x4((const T*)p.dout + tok * V + vbase + c8, dd);
        Load<T>::x4((const T*)p.dout + tok * V + vbase + c8 + 4, dd + 4);
        float gs = p.scale;
        if (p.g) gs *= __expf(p.g[tok]);
        float gv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) gv[e] = 0.f;
        if (p.gk) {
          Load<float>::x4(p.gk + tok * K + kbase + c8, gv);
          Load<float>::x4(p.gk + tok * K + kbase + c8 + 4, gv + 4);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) qo[e] *= gs * __expf(gv[e]);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      store_pair<T>(&sQt[(c8 + e) * LDT + 2 * tp], qa[e], qb[e]);
      store_pair<T>(&sDt[(c8 + e) * LDT + 2 * tp], da[e], db[e]);
    }
    if (tid < 64) {
      const int64_t tok = (row0 + L - 1) * H + hh;
      float d = p.g ? p.g[tok] : 0.f;
      if (p.gk) d += p.gk[tok * K + kbase + tid];
      sDecay[tid] = __expf(d);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] *= sDecay[kq * 32 + c32_row(r, lane)];
#pragma unroll
    for (int s = 0; s < BT; s += 16)
      acc = Elem<T>::mfma32(lds_frag32<T>(sQt, LDT, kq * 32, s, lane), lds_frag32<T>(sDt, LDT, vq * 32, s, lane), acc);
    __syncthreads();
  }
  if (p.dh0) {
    float* o = p.dh0 + ((int64_t)n * H + hh) * K * V;
#pragma unroll
    for (int r = 0; r < 16; ++r) o[(int64_t)(kbase + kq * 32 + c32_row(r, lane)) * V + vcol] = acc[r];
  }
}


// ---------------------------------------------------------------------------
// Row-major [K, V] state tiles -> MFMA fragment order (FLA_H_FRAGMENT, or FLA_H_FRAGMENT_T with
// every 32x32 tile transposed), 16-bit: what the output-stage and backward kernels read.  One
// wave per 32x32 tile; lane l, slot r holds element (32 kt + row(r, l), 32 vt + l % 32) of the
// tile, row(r, l) = 8 (r / 4) + 4 (l / 32) + r % 4 (the accumulator order of the 32x32 MFMA).
template <typename T>
__global__ __launch_bounds__(256) void states_to_fragments_kernel(const void* src, int src_is_f32, T* dst, int K, int V,
                                                                  int transposed, int64_t total_tiles) {
  typedef typename Elem<T>::v8 v8;
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= total_tiles) return;
  const int nkt = K / 32, nvt = V / 32;
  const int64_t state = tile / (nkt * nvt);
  const int t = (int)(tile % (nkt * nvt)), kt = t / nvt, vt = t % nvt;
  const int64_t blk = state * (int64_t)K * V;
  v8 lo, hi;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int kk = kt * 32 + (transposed ? (lane & 31) : c32_row(r, lane));
    const int vv = vt * 32 + (transposed ? c32_row(r, lane) : (lane & 31));
    const int64_t idx = blk + (int64_t)kk * V + vv;
    const float x = src_is_f32 ? ((const float*)src)[idx] : (float)((const T*)src)[idx];
    if (r < 8) lo[r] = (T)x;
    else hi[r - 8] = (T)x;
  }
  T* d = dst + blk + ((transposed ? (int64_t)vt * nkt + kt : (int64_t)kt * nvt + vt) * 64 + lane) * 16;
  *(v8*)d = lo;
  *(v8*)(d + 8) = hi;
}

// The inverse: fragment order (16-bit) back to row-major, 16-bit or fp32.
template <typename T>
__global__ __launch_bounds__(256) void fragments_to_states_kernel(const T* src, void* dst, int dst_is_f32, int K, int V,
                                                                  int transposed, int64_t total_tiles) {
  typedef typename Elem<T>::v8 v8;
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= total_tiles) return;
  const int nkt = K / 32, nvt = V / 32;
  const int64_t state = tile / (nkt * nvt);
  const int t = (int)(tile % (nkt * nvt)), kt = t / nvt, vt = t % nvt;
  const int64_t blk = state * (int64_t)K * V;
  const T* s = src + blk + ((transposed ? (int64_t)vt * nkt + kt : (int64_t)kt * nvt + vt) * 64 + lane) * 16;
  const v8 lo = *(const v8*)s, hi = *(const v8*)(s + 8);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int kk = kt * 32 + (transposed ? (lane & 31) : c32_row(r, lane));
    const int vv = vt * 32 + (transposed ? c32_row(r, lane) : (lane & 31));
    const int64_t idx = blk + (int64_t)kk * V + vv;
    const T x = r < 8 ? lo[r] : hi[r - 8];
    if (dst_is_f32) ((float*)dst)[idx] = (float)x;
    else ((T*)dst)[idx] = x;
  }
}


template <typename T, bool DV>
int launch_piece(const PieceParams& p, int K, dim3 grid, hipStream_t stream) {
  switch (K) {
    case 64: gla_piece_kernel<T, 64, DV><<<grid, 256, 0, stream>>>(p); break;
    case 128: gla_piece_kernel<T, 128, DV><<<grid, 256, 0, stream>>>(p); break;
    case 256: gla_piece_kernel<T, 256, DV><<<grid, 256, 0, stream>>>(p); break;
    default: return FLA_E_UNSUPPORTED;
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

template <typename T>
int launch_dA(const DAParams& p, int V, dim3 grid, hipStream_t stream) {
  switch (V) {
    case 64: gla_bwd_dA_kernel<T, 64><<<grid, 256, 0, stream>>>(p); break;
    case 128: gla_bwd_dA_kernel<T, 128><<<grid, 256, 0, stream>>>(p); break;
    case 256: gla_bwd_dA_kernel<T, 256><<<grid, 256, 0, stream>>>(p); break;
    default: return FLA_E_UNSUPPORTED;
  }
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

int is_f32_code(int dtype, int qkv_dtype, int* is_f32) {
  if (dtype == FLA_F32) *is_f32 = 1;
  else if (dtype == qkv_dtype) *is_f32 = 0;
  else return FLA_E_UNSUPPORTED;
  return FLA_OK;
}

int piece_entry(bool dv, const void* x, const float* g, const void* A, const void* m, const void* y, void* out,
                const int64_t* offsets, const int64_t* indices, int64_t NT, int qkv_dtype, int a_dtype, int m_dtype,
                int64_t B, int64_t T, int64_t H, int64_t K, int64_t V, float scale, hipStream_t stream) {
  FLA_REQUIRE(x && g && A && m && y && out, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(V % 64 == 0 && V / 64 <= 65535, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)x | (uintptr_t)g | (uintptr_t)A | (uintptr_t)m | (uintptr_t)y | (uintptr_t)out) % 16 == 0,
              FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  const int64_t nwg = (int64_t)grid.x * grid.y * (V / 64);
  FLA_REQUIRE(nwg <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  grid = dim3((unsigned)nwg);
  PieceParams p{x, g, A, m, y, out, offsets, indices, T, ntfix, (int)H, (int)V, scale, 0, 0};
  if ((rc = is_f32_code(a_dtype, qkv_dtype, &p.a_is_f32))) return rc;
  if ((rc = is_f32_code(m_dtype, qkv_dtype, &p.m_is_f32))) return rc;
  if (qkv_dtype == FLA_BF16)
    return dv ? launch_piece<bf16, true>(p, (int)K, grid, stream) : launch_piece<bf16, false>(p, (int)K, grid, stream);
  if (qkv_dtype == FLA_F16)
    return dv ? launch_piece<f16, true>(p, (int)K, grid, stream) : launch_piece<f16, false>(p, (int)K, grid, stream);
  return FLA_E_UNSUPPORTED;
}

}  // namespace

extern "C" int fla_chunk_gla_fwd_o_gk(const void* q, const void* v, const float* g_cumsum, const void* A, const void* h,
                                      void* o, const int64_t* offsets, const int64_t* indices, int64_t NT,
                                      int qkv_dtype, int a_dtype, int h_dtype, int64_t B, int64_t T, int64_t H,
                                      int64_t K, int64_t V, float scale, fla_stream_t stream) {
  return piece_entry(false, q, g_cumsum, A, h, v, o, offsets, indices, NT, qkv_dtype, a_dtype, h_dtype, B, T, H, K, V,
                     scale, (hipStream_t)stream);
}

extern "C" int fla_chunk_gla_bwd_dv(const void* k, const float* g_cumsum, const void* A, const void* dout,
                                    const void* dh, void* dv, const int64_t* offsets, const int64_t* indices,
                                    int64_t NT, int qkv_dtype, int a_dtype, int dh_dtype, int64_t B, int64_t T,
                                    int64_t H, int64_t K, int64_t V, fla_stream_t stream) {
  return piece_entry(true, k, g_cumsum, A, dh, dout, dv, offsets, indices, NT, qkv_dtype, a_dtype, dh_dtype, B, T, H, K,
                     V, 1.f, (hipStream_t)stream);
}

extern "C" int fla_chunk_gla_bwd_dA(const void* v, const void* dout, float* dA, const int64_t* offsets,
                                    const int64_t* indices, int64_t NT, int qkv_dtype, int64_t B, int64_t T,
                                    int64_t H, int64_t V, float scale, fla_stream_t stream) {
  FLA_REQUIRE(v && dout && dA, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && V > 0 && NT >= 0, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)v | (uintptr_t)dout | (uintptr_t)dA) % 16 == 0, FLA_E_ALIGNMENT);
  dim3 grid;
  int ntfix;
  int rc = chunk_grid(offsets, indices, B, T, H, NT, &grid, &ntfix);
  if (rc) return rc;
  if (grid.x == 0) return FLA_OK;
  DAParams p{v, dout, dA, offsets, indices, T, ntfix, (int)H, scale};
  if (qkv_dtype == FLA_BF16) return launch_dA<bf16>(p, (int)V, grid, (hipStream_t)stream);
  if (qkv_dtype == FLA_F16) return launch_dA<f16>(p, (int)V, grid, (hipStream_t)stream);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_chunk_bwd_dh(const void* q, const float* g, const float* gk, const void* dout, const float* dht,
                                void* dh, float* dh0, const int64_t* offsets, const int64_t* chunk_offsets,
                                int qkv_dtype, int dh_dtype, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                                int64_t N, float scale, fla_stream_t stream) {
  FLA_REQUIRE(q && dout && dh, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  FLA_REQUIRE(K % 64 == 0 && V % 64 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(offsets ? (B == 1 && chunk_offsets != nullptr) : N == B, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)q | (uintptr_t)gk | (uintptr_t)dout | (uintptr_t)dh) % 16 == 0, FLA_E_ALIGNMENT);
  const int64_t tiles = (K / 64) * (V / 64);
  FLA_REQUIRE(tiles * N * H <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  if (N == 0 || T == 0) return FLA_OK;
  RowDhParams p{q, g, gk, dout, dht, dh, dh0, offsets, chunk_offsets, T, (int)H, (int)K, (int)V, scale, 0};
  int rc = is_f32_code(dh_dtype, qkv_dtype, &p.dh_is_f32);
  if (rc) return rc;
  dim3 grid((unsigned)(tiles * N * H));
  if (qkv_dtype == FLA_BF16) chunk_bwd_dh_rowmajor_kernel<bf16><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  else if (qkv_dtype == FLA_F16) chunk_bwd_dh_rowmajor_kernel<f16><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

extern "C" int fla_states_to_fragments(const void* h_row_major, void* h_frag, int src_dtype, int dst_dtype,
                                       int transposed, int64_t n_states, int64_t K, int64_t V, fla_stream_t stream) {
  FLA_REQUIRE(h_row_major && h_frag && h_row_major != h_frag, FLA_E_INVALID);
  FLA_REQUIRE(n_states >= 0 && K > 0 && V > 0, FLA_E_INVALID);
  FLA_REQUIRE(K % 32 == 0 && V % 32 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((uintptr_t)h_frag % 16 == 0, FLA_E_ALIGNMENT);
  int src_is_f32;
  int rc = is_f32_code(src_dtype, dst_dtype, &src_is_f32);
  if (rc) return rc;
  const int64_t tiles = n_states * (K / 32) * (V / 32);
  if (tiles == 0) return FLA_OK;
  const int64_t blocks = (tiles + 3) / 4;
  FLA_REQUIRE(blocks <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  if (dst_dtype == FLA_BF16)
    states_to_fragments_kernel<bf16><<<dim3((unsigned)blocks), 256, 0, (hipStream_t)stream>>>(
        h_row_major, src_is_f32, (bf16*)h_frag, (int)K, (int)V, transposed, tiles);
  else if (dst_dtype == FLA_F16)
    states_to_fragments_kernel<f16><<<dim3((unsigned)blocks), 256, 0, (hipStream_t)stream>>>(
        h_row_major, src_is_f32, (f16*)h_frag, (int)K, (int)V, transposed, tiles);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

extern "C" int fla_fragments_to_states(const void* h_frag, void* h_row_major, int src_dtype, int dst_dtype,
                                       int transposed, int64_t n_states, int64_t K, int64_t V, fla_stream_t stream) {
  FLA_REQUIRE(h_row_major && h_frag && h_row_major != h_frag, FLA_E_INVALID);
  FLA_REQUIRE(n_states >= 0 && K > 0 && V > 0, FLA_E_INVALID);
  FLA_REQUIRE(K % 32 == 0 && V % 32 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((uintptr_t)h_frag % 16 == 0, FLA_E_ALIGNMENT);
  int dst_is_f32;
  int rc = is_f32_code(dst_dtype, src_dtype, &dst_is_f32);
  if (rc) return rc;
  const int64_t tiles = n_states * (K / 32) * (V / 32);
  if (tiles == 0) return FLA_OK;
  const int64_t blocks = (tiles + 3) / 4;
  FLA_REQUIRE(blocks <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  if (src_dtype == FLA_BF16)
    fragments_to_states_kernel<bf16><<<dim3((unsigned)blocks), 256, 0, (hipStream_t)stream>>>(
        (const bf16*)h_frag, h_row_major, dst_is_f32, (int)K, (int)V, transposed, tiles);
  else if (src_dtype == FLA_F16)
    fragments_to_states_kernel<f16><<<dim3((unsigned)blocks), 256, 0, (hipStream_t)stream>>>(
        (const f16*)h_frag, h_row_major, dst_is_f32, (int)K, (int)V, transposed, tiles);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}
