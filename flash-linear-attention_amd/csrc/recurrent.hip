// Token-by-token recurrences (prefill of short prompts and the T = 1 decode
// step) for GLA-style gated linear attention and the gated delta rule.
//
// The step is a read-modify-write of the fp32 [K,V] state of every
// (sequence, head): pure HBM streaming.  One workgroup owns a [K, BV] slab of
// one state; lane (rg, c4) holds rows rg, rg+RG, ... and 4 adjacent value
// columns, so every state access is a 16-byte load/store and a wave touches
// whole 512-byte rows.  All state loads are issued before anything else, the
// per-token vectors are staged once in LDS, and o is a single cross-row-group
// LDS reduction: no fp32 partial-output tensor and no second pass as in the
// reference (fla/ops/common/fused_recurrent.py:349,377).  The final state may
// be written over the initial one (in-place decode).
//
// GLA   (fla/ops/common/fused_recurrent.py:98-114):
//     h <- h * e^{gk}[:,None] * e^{gv}[None,:] * e^{g} + k v^T ;  o = (s q)^T h
// GDR   (fla/ops/gated_delta_rule/fused_recurrent.py:83-99):
//     h <- e^{g} h ;  v' = beta (v - h^T k) ;  h <- h + k v'^T ;  o = (s q)^T h
//   computed in one sweep as  o = s (h_d^T q + (q.k) v')  with h_d the decayed
//   state, so the state is traversed once per token.
#include "fla_common.h"

namespace {

struct RParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;     // [B,T,H]
  const void* gk;    // [B,T,H,K]   (GLA)
  const void* gv;    // [B,T,H,V]   (GLA)
  const void* beta;  // [B,T,H] or [B,T,H,V]  (GDR)
  void* o;
  const float* h0;
  float* ht;
  const int64_t* offsets;
  int64_t T;
  int H, K, V;
  float scale;
  int reverse;
  int beta_per_value;
  float l2_eps;   // GDR, >= 0: q and k enter as x / sqrt(sum x^2 + l2_eps) (the l2 norm the layer applies in front of the step)
};

template <typename X>
FLA_DEVICE float ld(const void* p, int64_t i) { return (float)((const X*)p)[i]; }

template <typename X>
FLA_DEVICE void st(void* p, int64_t i, float x) { ((X*)p)[i] = (X)x; }

// KP: padded key dim (rows), BV: value columns per workgroup, GDR: delta rule.
template <typename T, typename GT, typename OT, int KP, int BV, bool GDR>
__global__ __launch_bounds__(256) void recurrent_fwd_kernel(RParams p) {
  constexpr int CG = BV / 4;       // column groups (4 columns each)
  constexpr int RG = 256 / CG;     // row groups
  constexpr int NR = KP / RG;      // rows per lane
  static_assert(KP % RG == 0, "row tiling");
  __shared__ __attribute__((aligned(16))) float sq[2][KP];
  __shared__ __attribute__((aligned(16))) float sk[2][KP];
  __shared__ __attribute__((aligned(16))) float sdk[2][KP];  // e^{gk}
  __shared__ __attribute__((aligned(16))) float sv[2][BV];
  __shared__ __attribute__((aligned(16))) float sdv[2][BV];  // e^{gv} (GLA) or beta (GDR)
  __shared__ __attribute__((aligned(16))) float sred[2][2][RG][BV];
  __shared__ float sscal[2][4];  // e^{g}, q.k, 1/|q|, 1/|k| (the last two 1 unless the rows are normalised here)

  const int tid = threadIdx.x;
  const int H = p.H, K = p.K, V = p.V;
  const int nvb = (V + BV - 1) / BV;
  const int vb = blockIdx.x % nvb;
  const int nh = blockIdx.x / nvb;
  const int n = nh / H, hh = nh % H;
  const int c4 = (tid % CG) * 4, rg = tid / CG;
  const int vcol = vb * BV + c4;
  const bool colok = vcol < V;  // V % 4 == 0
  SeqSpan sp = seq_span(p.offsets, n, p.T);

  // ---- state slab, all loads in flight at once
  f32x4 h[NR];
  {
    const float* h0p = p.h0 ? p.h0 + (int64_t)nh * K * V + vcol : nullptr;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      int row = rg + RG * i;
      if (h0p && colok && row < K) h[i] = __builtin_nontemporal_load((const f32x4*)(h0p + (int64_t)row * V));
      else h[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }

  auto stage = [&](int64_t step, int buf) {
    int64_t t = p.reverse ? (sp.len - 1 - step) : step;
    int64_t row = sp.bos + t;
    int64_t qk = (row * H + hh) * (int64_t)K;
    int64_t vv = (row * H + hh) * (int64_t)V;
    for (int i = tid; i < KP; i += 256) {
      bool ok = i < K;
      float qv = ok ? ld<T>(p.q, qk + i) * p.scale : 0.f;
      float kv = ok ? ld<T>(p.k, qk + i) : 0.f;
      sq[buf][i] = qv;
      sk[buf][i] = kv;
      if (!GDR) sdk[buf][i] = (ok && p.gk) ? __expf(ld<GT>(p.gk, qk + i)) : 1.f;
    }
    for (int i = tid; i < BV; i += 256) {
      int c = vb * BV + i;
      bool ok = c < V;
      sv[buf][i] = ok ? ld<T>(p.v, vv + c) : 0.f;
      if (!GDR) {
        sdv[buf][i] = (ok && p.gv) ? __expf(ld<GT>(p.gv, vv + c)) : 1.f;
      } else {
        float b = 1.f;
        if (p.beta) b = p.beta_per_value ? (ok ? ld<GT>(p.beta, vv + c) : 0.f) : ld<GT>(p.beta, row * H + hh);
        sdv[buf][i] = b;
      }
    }
    if (tid == 0) sscal[buf][0] = p.g ? __expf(ld<GT>(p.g, row * H + hh)) : 1.f;
    if (GDR && tid < 64) {
      // q.k (and, where the rows are normalised here, q.q and k.k) over the whole key dim, reduced inside wave 0
      float acc = 0.f, aq = 0.f, ak = 0.f;
      for (int i = tid; i < K; i += 64) {
        const float qx = ld<T>(p.q, qk + i), kx = ld<T>(p.k, qk + i);
        acc += qx * p.scale * kx;
        aq += qx * qx;
        ak += kx * kx;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        acc += __shfl_down(acc, off, 64);
        aq += __shfl_down(aq, off, 64);
        ak += __shfl_down(ak, off, 64);
      }
      if (tid == 0) {
        const bool l2 = p.l2_eps >= 0.f;
        const float rq = l2 ? rsqrtf(aq + p.l2_eps) : 1.f, rk = l2 ? rsqrtf(ak + p.l2_eps) : 1.f;
        sscal[buf][1] = acc * rq * rk;
        sscal[buf][2] = rq;
        sscal[buf][3] = rk;
      }
    }
  };

  if (sp.len > 0) stage(0, 0);
  __syncthreads();
  for (int64_t step = 0; step < sp.len; ++step) {
    const int buf = (int)(step & 1);
    int64_t t = p.reverse ? (sp.len - 1 - step) : step;
    int64_t orow = ((sp.bos + t) * H + hh) * (int64_t)V;
    const float eg = sscal[buf][0];
    f32x4 vv = *(const f32x4*)&sv[buf][c4];
    f32x4 dv = *(const f32x4*)&sdv[buf][c4];
    f32x4 pq = {0.f, 0.f, 0.f, 0.f}, pk = {0.f, 0.f, 0.f, 0.f};
    // Everything read from the staging buffers is taken before the barrier:
    // the next step restages this buffer before its own barrier.
    const float qk = GDR ? sscal[buf][1] : 0.f;
    const float rq = GDR ? sscal[buf][2] : 1.f, rk = GDR ? sscal[buf][3] : 1.f;
    float krow[NR];
    if (!GDR) {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        int row = rg + RG * i;
        float dk = sdk[buf][row] * eg, kr = sk[buf][row], qr = sq[buf][row];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h[i][j] = h[i][j] * (dk * dv[j]) + kr * vv[j];
          pq[j] += h[i][j] * qr;
        }
      }
      *(f32x4*)&sred[buf][0][rg][c4] = pq;
    } else {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        int row = rg + RG * i;
        float kr = sk[buf][row] * rk, qr = sq[buf][row] * rq;
        krow[i] = kr;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          h[i][j] *= eg;
          pk[j] += h[i][j] * kr;
          pq[j] += h[i][j] * qr;
        }
      }
      *(f32x4*)&sred[buf][0][rg][c4] = pq;
      *(f32x4*)&sred[buf][1][rg][c4] = pk;
    }
    if (step + 1 < sp.len) stage(step + 1, buf ^ 1);
    __syncthreads();
    if (!GDR) {
      if (rg == 0 && colok) {
        f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < RG; ++r) tot += *(const f32x4*)&sred[buf][0][r][c4];
        typedef OT ov4 __attribute__((ext_vector_type(4)));
        ov4 ov;
#pragma unroll
        for (int j = 0; j < 4; ++j) ov[j] = (OT)tot[j];
        *(ov4*)((OT*)p.o + orow + vcol) = ov;
      }
    } else {
      f32x4 tq = {0.f, 0.f, 0.f, 0.f}, tk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RG; ++r) {
        tq += *(const f32x4*)&sred[buf][0][r][c4];
        tk += *(const f32x4*)&sred[buf][1][r][c4];
      }
      f32x4 vn;
#pragma unroll
      for (int j = 0; j < 4; ++j) vn[j] = (vv[j] - tk[j]) * dv[j];
#pragma unroll
      for (int i = 0; i < NR; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) h[i][j] += krow[i] * vn[j];
      }
      if (rg == 0 && colok) {
        typedef OT ov4 __attribute__((ext_vector_type(4)));
        ov4 ov;
#pragma unroll
        for (int j = 0; j < 4; ++j) ov[j] = (OT)(tq[j] + qk * vn[j]);
        *(ov4*)((OT*)p.o + orow + vcol) = ov;
      }
    }
  }
  if (p.ht && colok) {
    float* htp = p.ht + (int64_t)nh * K * V + vcol;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      int row = rg + RG * i;
      if (row < K) __builtin_nontemporal_store(h[i], (f32x4*)(htp + (int64_t)row * V));
    }
  }
}

template <typename T, typename GT, typename OT, bool GDR>
int launch_r(const RParams& p, int64_t NH, hipStream_t st) {
  const int K = p.K, V = p.V;
  FLA_REQUIRE(K <= 256 && V % 4 == 0, FLA_E_UNSUPPORTED);
  // Value columns per workgroup: whole rows when there are enough (n,h) pairs
  // to fill 256 CUs several times over, narrower slabs otherwise.
  int bv = 128;
  if (V <= 32 || NH * ((V + 127) / 128) < 1024) bv = 32;
  if (V > 32 && V <= 64 && bv == 128) bv = 64;
  int64_t nblk = NH * ((V + bv - 1) / bv);
  if (nblk == 0) return FLA_OK;
  FLA_REQUIRE(nblk <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  dim3 grid((unsigned)nblk), block(256);
  int kp = K <= 64 ? 64 : (K <= 128 ? 128 : 256);
#define FLA_R_CASE(KP_, BV_)                                                                          \
  if (kp == KP_ && bv == BV_) {                                                                       \
    hipLaunchKernelGGL((recurrent_fwd_kernel<T, GT, OT, KP_, BV_, GDR>), grid, block, 0, st, p);      \
    FLA_CHECK_LAUNCH();                                                                               \
    return FLA_OK;                                                                                    \
  }
  FLA_R_CASE(64, 32)
  FLA_R_CASE(64, 64)
  FLA_R_CASE(64, 128)
  FLA_R_CASE(128, 32)
  FLA_R_CASE(128, 64)
  FLA_R_CASE(128, 128)
  FLA_R_CASE(256, 32)
  FLA_R_CASE(256, 64)
  FLA_R_CASE(256, 128)
#undef FLA_R_CASE
  return FLA_E_UNSUPPORTED;
}

template <bool GDR>
int dispatch_r(const RParams& p, int qkv_dtype, int gate_dtype, int o_dtype, int64_t NH, hipStream_t st) {
  // The gate dtype only matters when a gate tensor is present.
#define FLA_R_DT(QT, QE, GT_, GE, OT_, OE) \
  if (qkv_dtype == QE && gate_dtype == GE && o_dtype == OE) return launch_r<QT, GT_, OT_, GDR>(p, NH, st);
  FLA_R_DT(bf16, FLA_BF16, bf16, FLA_BF16, bf16, FLA_BF16)
  FLA_R_DT(bf16, FLA_BF16, float, FLA_F32, bf16, FLA_BF16)
  FLA_R_DT(bf16, FLA_BF16, bf16, FLA_BF16, float, FLA_F32)
  FLA_R_DT(bf16, FLA_BF16, float, FLA_F32, float, FLA_F32)
  FLA_R_DT(f16, FLA_F16, f16, FLA_F16, f16, FLA_F16)
  FLA_R_DT(f16, FLA_F16, float, FLA_F32, f16, FLA_F16)
  FLA_R_DT(f16, FLA_F16, f16, FLA_F16, float, FLA_F32)
  FLA_R_DT(f16, FLA_F16, float, FLA_F32, float, FLA_F32)
  FLA_R_DT(float, FLA_F32, float, FLA_F32, float, FLA_F32)
#undef FLA_R_DT
  return FLA_E_UNSUPPORTED;
}

int check_common(const void* q, const void* k, const void* v, void* o, const int64_t* offsets, int64_t B, int64_t T,
                 int64_t H, int64_t K, int64_t V, int64_t N) {
  FLA_REQUIRE(q && k && v && o, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  if (offsets) FLA_REQUIRE(B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  FLA_REQUIRE(((uintptr_t)o | (uintptr_t)v) % 8 == 0, FLA_E_ALIGNMENT);
  return FLA_OK;
}

}  // namespace

extern "C" int fla_fused_recurrent_fwd(const void* q, const void* k, const void* v, const void* g, const void* gk,
                                       const void* gv, void* o, const float* h0, float* ht, const int64_t* offsets,
                                       int qkv_dtype, int gate_dtype, int o_dtype, int64_t B, int64_t T, int64_t H,
                                       int64_t K, int64_t V, int64_t N, float scale, int reverse,
                                       fla_stream_t stream) {
  int rc = check_common(q, k, v, o, offsets, B, T, H, K, V, N);
  if (rc) return rc;
  FLA_REQUIRE((((uintptr_t)h0) | ((uintptr_t)ht)) % 16 == 0, FLA_E_ALIGNMENT);
  RParams p{q, k, v, g, gk, gv, nullptr, o, h0, ht, offsets, T, (int)H, (int)K, (int)V, scale, reverse, 0, -1.f};
  if (!g && !gk && !gv) gate_dtype = FLA_F32;
  return dispatch_r<false>(p, qkv_dtype, gate_dtype, o_dtype, N * H, (hipStream_t)stream);
}

static int recurrent_gdr_impl(const void* q, const void* k, const void* v, const void* g, const void* beta, void* o,
                              const float* h0, float* ht, const int64_t* offsets, int qkv_dtype, int gate_dtype,
                              int o_dtype, int beta_per_value, int64_t B, int64_t T, int64_t H, int64_t K, int64_t V,
                              int64_t N, float scale, float l2_eps, fla_stream_t stream) {
  int rc = check_common(q, k, v, o, offsets, B, T, H, K, V, N);
  if (rc) return rc;
  FLA_REQUIRE((((uintptr_t)h0) | ((uintptr_t)ht)) % 16 == 0, FLA_E_ALIGNMENT);
  RParams p{q, k, v, g, nullptr, nullptr, beta, o, h0, ht, offsets, T, (int)H, (int)K, (int)V, scale, 0, beta_per_value,
            l2_eps};
  if (!g && !beta) gate_dtype = FLA_F32;
  return dispatch_r<true>(p, qkv_dtype, gate_dtype, o_dtype, N * H, (hipStream_t)stream);
}

extern "C" int fla_fused_recurrent_gated_delta_rule_fwd(const void* q, const void* k, const void* v, const void* g,
                                                        const void* beta, void* o, const float* h0, float* ht,
                                                        const int64_t* offsets, int qkv_dtype, int gate_dtype,
                                                        int o_dtype, int beta_per_value, int64_t B, int64_t T,
                                                        int64_t H, int64_t K, int64_t V, int64_t N, float scale,
                                                        fla_stream_t stream) {
  return recurrent_gdr_impl(q, k, v, g, beta, o, h0, ht, offsets, qkv_dtype, gate_dtype, o_dtype, beta_per_value, B, T, H,
                            K, V, N, scale, -1.f, stream);
}

extern "C" int fla_fused_recurrent_gated_delta_rule_fwd_l2norm(const void* q, const void* k, const void* v,
                                                               const void* g, const void* beta, void* o,
                                                               const float* h0, float* ht, const int64_t* offsets,
                                                               int qkv_dtype, int gate_dtype, int o_dtype,
                                                               int beta_per_value, int64_t B, int64_t T, int64_t H,
                                                               int64_t K, int64_t V, int64_t N, float scale,
                                                               float l2norm_eps, fla_stream_t stream) {
  FLA_REQUIRE(l2norm_eps >= 0.f, FLA_E_INVALID);
  return recurrent_gdr_impl(q, k, v, g, beta, o, h0, ht, offsets, qkv_dtype, gate_dtype, o_dtype, beta_per_value, B, T, H,
                            K, V, N, scale, l2norm_eps, stream);
}
