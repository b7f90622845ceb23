// Token-by-token backward of the gated linear-attention recurrence
//     h_t = h_{t-1} * e^{g_t} * e^{gk_t}[:,None] * e^{gv_t}[None,:] + k_t v_t^T ,   o_t = (s q_t)^T h_t
// (fla/ops/common/fused_recurrent.py:381-468, kernel :131-319), in fp32 whatever the storage type.
//
// One workgroup owns all K rows and 64 value columns of one (sequence, head) state and makes two
// passes over the tokens, as the reference does:
//   pass 1, in the direction of the recurrence: rebuild h_t and emit  dq_t = s h_t do_t ;
//   pass 2, against it:  dh += (s q_t) do_t^T ;  dk_t = dh v_t ;  dv_t = dh^T k_t ;  dh *= decay_t ;
//   what is left of dh after the first token is the gradient of the initial state.
// Lane (rg, c4) holds rows rg, rg+16, ... and 4 adjacent columns of the slab (the layout of the
// forward kernel).  Sums over the slab's columns (dq, dk) and over the rows (dv) go through LDS;
// sums over the column slabs of a head are left to the caller as partial tensors [V/64, ...],
// like the reference's (fla/ops/common/fused_recurrent.py:405-407, :445-447).
#include "fla_common.h"

namespace {

struct RBParams {
  const void* q;
  const void* k;
  const void* v;
  const void* g;     // [B,T,H]
  const void* gk;    // [B,T,H,K]
  const void* gv;    // [B,T,H,V]
  const float* h0;
  const void* dout;
  const float* dht;
  float* dq;         // [NV, B*T, H, K]
  float* dk;         // [NV, B*T, H, K]
  float* dv;         // [B*T, H, V]
  float* dh0;
  const int64_t* offsets;
  int64_t T, rows;   // rows = B*T: stride between the partial tensors
  int H, K, V;
  float scale;
  int reverse;
};

template <typename X>
FLA_DEVICE float ldf(const void* p, int64_t i) { return (float)((const X*)p)[i]; }

constexpr int BV = 64, CG = BV / 4, RG = 256 / CG;   // 16 column groups x 16 row groups

template <typename T, typename GT, int KP>
__global__ __launch_bounds__(256) void recurrent_bwd_kernel(RBParams p) {
  constexpr int NR = KP / RG;   // rows per lane
  __shared__ __attribute__((aligned(16))) float sq[2][KP];
  __shared__ __attribute__((aligned(16))) float sk[2][KP];
  __shared__ __attribute__((aligned(16))) float sdk[2][KP];   // e^{g + gk}
  __shared__ __attribute__((aligned(16))) float sv[2][BV];
  __shared__ __attribute__((aligned(16))) float sdo[2][BV];
  __shared__ __attribute__((aligned(16))) float sdv[2][BV];   // e^{gv}
  __shared__ __attribute__((aligned(16))) float srow[2][KP][CG + 4];   // per-row partial sums, one per column group
  __shared__ __attribute__((aligned(16))) float scol[2][RG][BV];       // per-column partial sums, one per row group

  const int tid = threadIdx.x;
  const int H = p.H, K = p.K, V = p.V;
  const int nvb = (V + BV - 1) / BV;
  const int vb = blockIdx.x % nvb;
  const int nh = blockIdx.x / nvb;
  const int n = nh / H, hh = nh % H;
  const int cg = tid % CG, c4 = cg * 4, rg = tid / CG;
  const int vcol = vb * BV + c4;
  const bool colok = vcol < V;   // V % 4 == 0
  SeqSpan sp = seq_span(p.offsets, n, p.T);

  // token `step` of a pass that walks the sequence forwards (fwd_dir) or backwards
  auto token = [&](int64_t step, bool fwd_dir) { return fwd_dir ? step : sp.len - 1 - step; };
  auto stage = [&](int64_t t, int buf) {
    const int64_t row = sp.bos + t;
    const int64_t qk = (row * H + hh) * (int64_t)K;
    const int64_t vv = (row * H + hh) * (int64_t)V;
    const float gs = p.g ? ldf<GT>(p.g, row * H + hh) : 0.f;
    for (int i = tid; i < KP; i += 256) {
      const bool ok = i < K;
      sq[buf][i] = ok ? ldf<T>(p.q, qk + i) * p.scale : 0.f;
      sk[buf][i] = ok ? ldf<T>(p.k, qk + i) : 0.f;
      sdk[buf][i] = __expf(gs + ((ok && p.gk) ? ldf<GT>(p.gk, qk + i) : 0.f));
    }
    for (int i = tid; i < BV; i += 256) {
      const int c = vb * BV + i;
      const bool ok = c < V;
      sv[buf][i] = ok ? ldf<T>(p.v, vv + c) : 0.f;
      sdo[buf][i] = ok ? ldf<T>(p.dout, vv + c) : 0.f;
      sdv[buf][i] = (ok && p.gv) ? __expf(ldf<GT>(p.gv, vv + c)) : 1.f;
    }
  };
  // sum of a row's CG partials
  auto row_total = [&](int buf, int row) {
    float t = 0.f;
#pragma unroll
    for (int c = 0; c < CG; c += 4) {
      const f32x4 x = *(const f32x4*)&srow[buf][row][c];
      t += (x[0] + x[1]) + (x[2] + x[3]);
    }
    return t;
  };

  // ---- pass 1: h_t, dq_t
  f32x4 h[NR];
  {
    const float* h0p = p.h0 ? p.h0 + (int64_t)nh * K * V + vcol : nullptr;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = rg + RG * i;
      if (h0p && colok && row < K) h[i] = *(const f32x4*)(h0p + (int64_t)row * V);
      else h[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  const bool dir1 = !p.reverse;
  if (sp.len > 0) stage(token(0, dir1), 0);
  __syncthreads();
  for (int64_t step = 0; step < sp.len; ++step) {
    const int buf = (int)(step & 1);
    const int64_t t = token(step, dir1);
    const f32x4 vv = *(const f32x4*)&sv[buf][c4];
    const f32x4 dov = *(const f32x4*)&sdo[buf][c4];
    const f32x4 dcv = *(const f32x4*)&sdv[buf][c4];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = rg + RG * i;
      const float dk_ = sdk[buf][row], kr = sk[buf][row];
      float pq = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        h[i][j] = h[i][j] * (dk_ * dcv[j]) + kr * vv[j];
        pq += h[i][j] * dov[j];
      }
      srow[buf][row][cg] = pq;
    }
    if (step + 1 < sp.len) stage(token(step + 1, dir1), buf ^ 1);
    __syncthreads();
    if (tid < K) p.dq[((int64_t)vb * p.rows + sp.bos + t) * H * K + (int64_t)hh * K + tid] = p.scale * row_total(buf, tid);
  }
  __syncthreads();

  // ---- pass 2: dh, dk_t, dv_t
  f32x4 dh[NR];
  {
    const float* dp = p.dht ? p.dht + (int64_t)nh * K * V + vcol : nullptr;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = rg + RG * i;
      if (dp && colok && row < K) dh[i] = *(const f32x4*)(dp + (int64_t)row * V);
      else dh[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
  const bool dir2 = !dir1;
  if (sp.len > 0) stage(token(0, dir2), 0);
  __syncthreads();
  for (int64_t step = 0; step < sp.len; ++step) {
    const int buf = (int)(step & 1);
    const int64_t t = token(step, dir2);
    const f32x4 vv = *(const f32x4*)&sv[buf][c4];
    const f32x4 dov = *(const f32x4*)&sdo[buf][c4];
    const f32x4 dcv = *(const f32x4*)&sdv[buf][c4];
    f32x4 pv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = rg + RG * i;
      const float qr = sq[buf][row], kr = sk[buf][row], dk_ = sdk[buf][row];
      float pk = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dh[i][j] += qr * dov[j];
        pk += dh[i][j] * vv[j];
        pv[j] += dh[i][j] * kr;
        dh[i][j] *= dk_ * dcv[j];
      }
      srow[buf][row][cg] = pk;
    }
    *(f32x4*)&scol[buf][rg][c4] = pv;
    if (step + 1 < sp.len) stage(token(step + 1, dir2), buf ^ 1);
    __syncthreads();
    if (tid < K) p.dk[((int64_t)vb * p.rows + sp.bos + t) * H * K + (int64_t)hh * K + tid] = row_total(buf, tid);
    if (rg == RG - 1 && colok) {   // another wave than the one that writes dk
      f32x4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RG; ++r) tot += *(const f32x4*)&scol[buf][r][c4];
      *(f32x4*)(p.dv + ((sp.bos + t) * H + hh) * (int64_t)V + vcol) = tot;
    }
  }
  if (p.dh0 && colok) {
    float* dp = p.dh0 + (int64_t)nh * K * V + vcol;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = rg + RG * i;
      if (row < K) *(f32x4*)(dp + (int64_t)row * V) = dh[i];
    }
  }
}

template <typename T, typename GT>
int launch_rb(const RBParams& p, int64_t NH, hipStream_t st) {
  const int64_t nblk = NH * ((p.V + BV - 1) / BV);
  if (nblk == 0) return FLA_OK;
  FLA_REQUIRE(nblk <= 0x7fffffffLL, FLA_E_UNSUPPORTED);
  dim3 grid((unsigned)nblk), block(256);
  if (p.K <= 64) hipLaunchKernelGGL((recurrent_bwd_kernel<T, GT, 64>), grid, block, 0, st, p);
  else if (p.K <= 128) hipLaunchKernelGGL((recurrent_bwd_kernel<T, GT, 128>), grid, block, 0, st, p);
  else if (p.K <= 256) hipLaunchKernelGGL((recurrent_bwd_kernel<T, GT, 256>), grid, block, 0, st, p);
  else return FLA_E_UNSUPPORTED;
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

}  // namespace

extern "C" int fla_fused_recurrent_bwd(const void* q, const void* k, const void* v, const void* g, const void* gk,
                                       const void* gv, const float* h0, const void* dout, const float* dht,
                                       float* dq_partial, float* dk_partial, float* dv, float* dh0,
                                       const int64_t* offsets, int qkv_dtype, int gate_dtype, int64_t B, int64_t T,
                                       int64_t H, int64_t K, int64_t V, int64_t N, float scale, int reverse,
                                       fla_stream_t stream) {
  FLA_REQUIRE(q && k && v && dout && dq_partial && dk_partial && dv, FLA_E_INVALID);
  FLA_REQUIRE(B >= 0 && T >= 0 && H > 0 && K > 0 && V > 0 && N >= 0, FLA_E_INVALID);
  if (offsets) FLA_REQUIRE(B == 1, FLA_E_INVALID);
  else FLA_REQUIRE(N == B, FLA_E_INVALID);
  FLA_REQUIRE(K <= 256 && V % 4 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)h0 | (uintptr_t)dht | (uintptr_t)dh0 | (uintptr_t)dv) % 16 == 0, FLA_E_ALIGNMENT);
  RBParams p{q, k, v, g, gk, gv, h0, dout, dht, dq_partial, dk_partial, dv, dh0, offsets, T, B * T,
             (int)H, (int)K, (int)V, scale, reverse};
  if (!g && !gk && !gv) gate_dtype = FLA_F32;
  hipStream_t st = (hipStream_t)stream;
#define FLA_RB_DT(QT, QE, GT_, GE) \
  if (qkv_dtype == QE && gate_dtype == GE) return launch_rb<QT, GT_>(p, N * H, st);
  FLA_RB_DT(bf16, FLA_BF16, bf16, FLA_BF16)
  FLA_RB_DT(bf16, FLA_BF16, float, FLA_F32)
  FLA_RB_DT(f16, FLA_F16, f16, FLA_F16)
  FLA_RB_DT(f16, FLA_F16, float, FLA_F32)
  FLA_RB_DT(float, FLA_F32, float, FLA_F32)
#undef FLA_RB_DT
  return FLA_E_UNSUPPORTED;
}
