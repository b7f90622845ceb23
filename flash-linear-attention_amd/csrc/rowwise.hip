// Row-wise normalisations that sit either side of the chunk operators inside the layers:
//   l2norm            y = x / sqrt(sum x^2 + eps)                       (q, k before the gated delta rule)
//                     fla/modules/l2norm.py:18-40 (forward), :52-88 (backward)
//   norm + swish gate y = norm(x) * w (+ b) * g * sigmoid(g)            (o after the operator)
//                     fla/modules/fused_norm_gate.py:114-183 (forward), :198-330 (backward)
//
// HBM-streaming kernels.  A row of N elements is held by LPR adjacent lanes, 8 elements (one
// or two 16-byte loads) per lane and column pass, so a wave reads 64*8 contiguous elements
// when N == 8*LPR; sums over a row are butterfly exchanges inside the lane group.  Rows are
// walked with a grid-stride loop so that the per-column weight/bias gradients of the gated
// norm are accumulated in registers and leave the chip once per workgroup.
#include "fla_common.h"

namespace {

constexpr int VEC = 8;

template <typename T>
struct Row8;
template <>
struct Row8<float> {
  struct raw {
    f32x4 a, b;
  };
  static FLA_DEVICE raw load_raw(const float* p) { return raw{*(const f32x4*)p, *(const f32x4*)(p + 4)}; }
  static FLA_DEVICE void unpack(const raw& r, float* o) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = r.a[i];
      o[4 + i] = r.b[i];
    }
  }
  static FLA_DEVICE void load(const float* p, float* o) {
    f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = a[i];
      o[4 + i] = b[i];
    }
  }
  static FLA_DEVICE void store(float* p, const float* v) {
    *(f32x4*)p = f32x4{v[0], v[1], v[2], v[3]};
    *(f32x4*)(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
  }
};
template <>
struct Row8<bf16> {
  typedef bf16x8 raw;
  static FLA_DEVICE raw load_raw(const bf16* p) { return *(const bf16x8*)p; }
  static FLA_DEVICE void unpack(const raw& r, float* o) {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)r[i];
  }
  static FLA_DEVICE void load(const bf16* p, float* o) {
    bf16x8 a = *(const bf16x8*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)a[i];
  }
  static FLA_DEVICE void store(bf16* p, const float* v) {
    bf16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = (bf16)v[i];
    *(bf16x8*)p = a;
  }
};
template <>
struct Row8<f16> {
  typedef f16x8 raw;
  static FLA_DEVICE raw load_raw(const f16* p) { return *(const f16x8*)p; }
  static FLA_DEVICE void unpack(const raw& r, float* o) {
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)r[i];
  }
  static FLA_DEVICE void load(const f16* p, float* o) {
    f16x8 a = *(const f16x8*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)a[i];
  }
  static FLA_DEVICE void store(f16* p, const float* v) {
    f16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = (f16)v[i];
    *(f16x8*)p = a;
  }
};

// sum over the LPR lanes of a group (LPR a power of two <= 64), result in every lane
template <int LPR>
FLA_DEVICE float group_sum(float x) {
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

// the hardware reciprocal (1 ulp) instead of an IEEE division: ten instructions less per element
FLA_DEVICE float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

// ------------------------------------------------------------------ l2norm
// NP column passes of 8*LPR elements cover a row; lanes past the end of the row idle.
template <typename TX, typename TY, int LPR, int NP>
__global__ __launch_bounds__(256) void l2norm_fwd_kernel(const TX* __restrict__ x, TY* __restrict__ y, int64_t M, int N,
                                                         float eps) {
  constexpr int RPW = 256 / LPR;
  const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
  for (int64_t row = (int64_t)blockIdx.x * RPW + rl; row < M; row += (int64_t)gridDim.x * RPW) {
    float v[NP][VEC];
    float ss = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
        Row8<TX>::load(x + row * N + col, v[pss]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) ss = fmaf(v[pss][i], v[pss][i], ss);
      }
    }
    ss = group_sum<LPR>(ss);
    const float rstd = __builtin_amdgcn_rsqf(ss + eps);  // hardware reciprocal square root (1 ulp)
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[pss][i] *= rstd;
        Row8<TY>::store(y + row * N + col, v[pss]);
      }
    }
  }
}

template <typename TX, typename TD, int LPR, int NP>
__global__ __launch_bounds__(256) void l2norm_bwd_kernel(const TX* __restrict__ x, const TD* __restrict__ dy,
                                                         TX* __restrict__ dx, int64_t M, int N, float eps) {
  constexpr int RPW = 256 / LPR;
  const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
  for (int64_t row = (int64_t)blockIdx.x * RPW + rl; row < M; row += (int64_t)gridDim.x * RPW) {
    float v[NP][VEC], g[NP][VEC];
    float ss = 0.f, sd = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
        Row8<TX>::load(x + row * N + col, v[pss]);
        Row8<TD>::load(dy + row * N + col, g[pss]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          ss = fmaf(v[pss][i], v[pss][i], ss);
          sd = fmaf(v[pss][i], g[pss][i], sd);
        }
      }
    }
    ss = group_sum<LPR>(ss);
    sd = group_sum<LPR>(sd);
    const float rstd = __builtin_amdgcn_rsqf(ss + eps);
    const float c = sd * rstd * rstd * rstd;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) g[pss][i] = g[pss][i] * rstd - c * v[pss][i];
        Row8<TX>::store(dx + row * N + col, g[pss]);
      }
    }
  }
}

// ------------------------------------------------------------------ norm + swish gate
struct NormGateParams {
  const void* x;
  const void* gate;
  const float* w;     // [N] or NULL
  const float* b;     // [N] or NULL
  void* y;
  float* mean;        // [M], layer norm only
  float* rstd;        // [M]
  // backward
  const void* dy;
  void* dx;
  void* dgate;
  float* dw_part;     // [gridDim.x, N] or NULL
  float* db_part;     // [gridDim.x, N] or NULL
  int64_t M;
  int N;
  float eps;
  // residual / prenorm variants (fla/modules/fused_norm_gate.py:68-74, :265-271).  Forward: the row that is
  // normalised is x + res, and that sum is kept in res_out; backward: `x` is that kept sum, dres the gradient that
  // arrives for it (prenorm), dres_in a copy of dx in the kept sum's type.  *_f32: fp32 instead of the type T.
  const void* res;
  void* res_out;
  const void* dres;
  void* dres_in;
  int res_f32, res_out_f32;   // forward
  int x_f32;                  // backward: type of x, dres and dres_in
};

// 8 elements of a row whose storage type is T or, when f32 is set (workgroup-uniform), fp32
template <typename T>
FLA_DEVICE void load8_as(const void* base, int f32, int64_t idx, float* o) {
  if (f32) Row8<float>::load((const float*)base + idx, o);
  else Row8<T>::load((const T*)base + idx, o);
}
template <typename T>
FLA_DEVICE void store8_as(void* base, int f32, int64_t idx, const float* v) {
  if (f32) Row8<float>::store((float*)base + idx, v);
  else Row8<T>::store((T*)base + idx, v);
}

template <typename T, bool RMS, int LPR, int NP>
__global__ __launch_bounds__(256) void norm_gate_fwd_kernel(NormGateParams p) {
  constexpr int RPW = 256 / LPR;
  const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
  const int N = p.N;
  float w[NP][VEC], b[NP][VEC];
#pragma unroll
  for (int pss = 0; pss < NP; ++pss) {
    const int col = (pss * LPR + sub) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      w[pss][i] = (p.w && col < N) ? p.w[col + i] : 1.f;
      b[pss][i] = (p.b && col < N) ? p.b[col + i] : 0.f;
    }
  }
  const float invN = 1.f / (float)N;
  // The rows of the next pass are fetched (in storage precision) before this pass computes, so
  // that a lane always has two passes of loads in flight; past the last row the fetch repeats it.
  typedef typename Row8<T>::raw raw_t;
  const int64_t step = (int64_t)gridDim.x * RPW;
  const int64_t first = (int64_t)blockIdx.x * RPW + rl;
  raw_t nx[NP], ng[NP];
  auto fetch = [&](int64_t row) {
    const int64_t r = row < p.M ? row : p.M - 1;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      const int c = col < N ? col : 0;
      nx[pss] = Row8<T>::load_raw((const T*)p.x + r * N + c);
      ng[pss] = Row8<T>::load_raw((const T*)p.gate + r * N + c);
    }
  };
  fetch(first);
  for (int64_t row = first; row < p.M; row += step) {
    float v[NP][VEC], g[NP][VEC];
    float s1 = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      Row8<T>::unpack(nx[pss], v[pss]);
      Row8<T>::unpack(ng[pss], g[pss]);
      if (col < N) {
        if (p.res) {
          float r8[VEC];
          load8_as<T>(p.res, p.res_f32, row * N + col, r8);
#pragma unroll
          for (int i = 0; i < VEC; ++i) v[pss][i] += r8[i];
        }
        if (p.res_out) store8_as<T>(p.res_out, p.res_out_f32, row * N + col, v[pss]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) s1 += v[pss][i];
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[pss][i] = g[pss][i] = 0.f;
      }
    }
    fetch(row + step);
    float mean = 0.f;
    if (!RMS) mean = group_sum<LPR>(s1) * invN;
    float ss = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          v[pss][i] -= mean;
          ss = fmaf(v[pss][i], v[pss][i], ss);
        }
      }
    }
    ss = group_sum<LPR>(ss) * invN;
    const float rstd = __builtin_amdgcn_rsqf(ss + p.eps);  // hardware reciprocal square root (1 ulp)
    if (sub == 0) {
      p.rstd[row] = rstd;
      if (!RMS) p.mean[row] = mean;
    }
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const float yv = fmaf(v[pss][i] * rstd, w[pss][i], b[pss][i]);
          v[pss][i] = yv * g[pss][i] * sigmoidf(g[pss][i]);
        }
        Row8<T>::store((T*)p.y + row * N + col, v[pss]);
      }
    }
  }
}

template <typename T, bool RMS, int LPR, int NP>
__global__ __launch_bounds__(256) void norm_gate_bwd_kernel(NormGateParams p) {
  constexpr int RPW = 256 / LPR;
  const int sub = threadIdx.x % LPR, rl = threadIdx.x / LPR;
  const int N = p.N;
  __shared__ float sred[RPW][LPR * VEC + 1];
  float w[NP][VEC], b[NP][VEC], dw[NP][VEC], db[NP][VEC];
#pragma unroll
  for (int pss = 0; pss < NP; ++pss) {
    const int col = (pss * LPR + sub) * VEC;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      w[pss][i] = (p.w && col < N) ? p.w[col + i] : 1.f;
      b[pss][i] = (p.b && col < N) ? p.b[col + i] : 0.f;
      dw[pss][i] = db[pss][i] = 0.f;
    }
  }
  const float invN = 1.f / (float)N;
  for (int64_t row = (int64_t)blockIdx.x * RPW + rl; row < p.M; row += (int64_t)gridDim.x * RPW) {
    float xh[NP][VEC], g[NP][VEC], d[NP][VEC];
    const float rstd = p.rstd[row];
    const float mean = RMS ? 0.f : p.mean[row];
    float c1 = 0.f, c2 = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
        load8_as<T>(p.x, p.x_f32, row * N + col, xh[pss]);
        Row8<T>::load((const T*)p.gate + row * N + col, g[pss]);
        Row8<T>::load((const T*)p.dy + row * N + col, d[pss]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const float xhat = (xh[pss][i] - mean) * rstd;
          const float yv = fmaf(xhat, w[pss][i], b[pss][i]);
          const float o = g[pss][i], sg = sigmoidf(o);
          const float dyv = d[pss][i];
          g[pss][i] = dyv * yv * (sg + o * sg * (1.f - sg));   // gradient of the gate
          const float dyn = dyv * o * sg;                      // gradient of the normalised, affine value
          dw[pss][i] = fmaf(dyn, xhat, dw[pss][i]);
          db[pss][i] += dyn;
          const float wdy = dyn * w[pss][i];
          c1 = fmaf(xhat, wdy, c1);
          c2 += wdy;
          xh[pss][i] = xhat;
          d[pss][i] = wdy;
        }
      }
    }
    c1 = group_sum<LPR>(c1) * invN;
    if (!RMS) c2 = group_sum<LPR>(c2) * invN;
    else c2 = 0.f;
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      const int col = (pss * LPR + sub) * VEC;
      if (col < N) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) d[pss][i] = (d[pss][i] - (xh[pss][i] * c1 + c2)) * rstd;
        if (p.dres) {
          float r8[VEC];
          load8_as<T>(p.dres, p.x_f32, row * N + col, r8);
#pragma unroll
          for (int i = 0; i < VEC; ++i) d[pss][i] += r8[i];
        }
        if (p.dres_in) store8_as<T>(p.dres_in, p.x_f32, row * N + col, d[pss]);
        Row8<T>::store((T*)p.dx + row * N + col, d[pss]);
        Row8<T>::store((T*)p.dgate + row * N + col, g[pss]);
      }
    }
  }
  // per-workgroup column sums of the weight / bias gradients
  for (int which = 0; which < 2; ++which) {
    float* part = which ? p.db_part : p.dw_part;
    if (!part) continue;  // uniform
#pragma unroll
    for (int pss = 0; pss < NP; ++pss) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < VEC; ++i) sred[rl][sub * VEC + i] = which ? db[pss][i] : dw[pss][i];
      __syncthreads();
      for (int c = threadIdx.x; c < LPR * VEC; c += 256) {
        float t = 0.f;
#pragma unroll
        for (int r = 0; r < RPW; ++r) t += sred[r][c];
        const int col = pss * LPR * VEC + c;
        if (col < N) part[(int64_t)blockIdx.x * N + col] = t;
      }
    }
  }
}

int rows_grid(int64_t M, int rpw, int cap) {
  int64_t g = fla_cdiv(M, rpw);
  return (int)(g < cap ? (g < 1 ? 1 : g) : cap);
}

#define FLA_ROW_SHAPES(CALL)            \
  if (N <= 64) CALL(8, 1)               \
  else if (N <= 128) CALL(16, 1)        \
  else if (N <= 256) CALL(32, 1)        \
  else if (N <= 512) CALL(64, 1)        \
  else if (N <= 1024) CALL(64, 2)       \
  else CALL(64, 4)

template <typename TX, typename TY>
int launch_l2_fwd(const void* x, void* y, int64_t M, int N, float eps, hipStream_t st) {
#define CALL(LPR, NP)                                                                                        \
  hipLaunchKernelGGL((l2norm_fwd_kernel<TX, TY, LPR, NP>), dim3(rows_grid(M, 256 / LPR, 1 << 20)), dim3(256), 0, st, \
                     (const TX*)x, (TY*)y, M, N, eps);
  FLA_ROW_SHAPES(CALL)
#undef CALL
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

template <typename TX, typename TD>
int launch_l2_bwd(const void* x, const void* dy, void* dx, int64_t M, int N, float eps, hipStream_t st) {
#define CALL(LPR, NP)                                                                                        \
  hipLaunchKernelGGL((l2norm_bwd_kernel<TX, TD, LPR, NP>), dim3(rows_grid(M, 256 / LPR, 1 << 20)), dim3(256), 0, st, \
                     (const TX*)x, (const TD*)dy, (TX*)dx, M, N, eps);
  FLA_ROW_SHAPES(CALL)
#undef CALL
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

template <typename T, bool RMS>
int launch_ng(const NormGateParams& p, bool bwd, int grid, hipStream_t st) {
  const int N = p.N;
#define CALL(LPR, NP)                                                                                   \
  {                                                                                                     \
    if (bwd) hipLaunchKernelGGL((norm_gate_bwd_kernel<T, RMS, LPR, NP>), dim3(grid), dim3(256), 0, st, p); \
    else hipLaunchKernelGGL((norm_gate_fwd_kernel<T, RMS, LPR, NP>), dim3(grid), dim3(256), 0, st, p);  \
  }
  FLA_ROW_SHAPES(CALL)
#undef CALL
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

int rpw_of(int N) { return N <= 64 ? 32 : N <= 128 ? 16 : N <= 256 ? 8 : 4; }

}  // namespace

extern "C" int fla_l2norm_fwd(const void* x, void* y, int64_t M, int64_t N, float eps, int x_dtype, int y_dtype,
                              fla_stream_t stream) {
  FLA_REQUIRE(x && y && M >= 0 && N > 0, FLA_E_INVALID);
  FLA_REQUIRE(N % 8 == 0 && N <= 2048, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)y)) % 16 == 0, FLA_E_ALIGNMENT);
  if (M == 0) return FLA_OK;
  hipStream_t st = (hipStream_t)stream;
#define D(XE, XT, YE, YT) \
  if (x_dtype == XE && y_dtype == YE) return launch_l2_fwd<XT, YT>(x, y, M, (int)N, eps, st);
  D(FLA_BF16, bf16, FLA_BF16, bf16)
  D(FLA_F16, f16, FLA_F16, f16)
  D(FLA_F32, float, FLA_F32, float)
  D(FLA_F32, float, FLA_BF16, bf16)
  D(FLA_F32, float, FLA_F16, f16)
  D(FLA_BF16, bf16, FLA_F32, float)
  D(FLA_F16, f16, FLA_F32, float)
#undef D
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t M, int64_t N, float eps, int x_dtype,
                              int dy_dtype, fla_stream_t stream) {
  FLA_REQUIRE(x && dy && dx && M >= 0 && N > 0, FLA_E_INVALID);
  FLA_REQUIRE(N % 8 == 0 && N <= 2048, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)dy) | ((uintptr_t)dx)) % 16 == 0, FLA_E_ALIGNMENT);
  if (M == 0) return FLA_OK;
  hipStream_t st = (hipStream_t)stream;
#define D(XE, XT, YE, YT) \
  if (x_dtype == XE && dy_dtype == YE) return launch_l2_bwd<XT, YT>(x, dy, dx, M, (int)N, eps, st);
  D(FLA_BF16, bf16, FLA_BF16, bf16)
  D(FLA_F16, f16, FLA_F16, f16)
  D(FLA_F32, float, FLA_F32, float)
  D(FLA_F32, float, FLA_BF16, bf16)
  D(FLA_F32, float, FLA_F16, f16)
  D(FLA_BF16, bf16, FLA_F32, float)
  D(FLA_F16, f16, FLA_F32, float)
#undef D
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_norm_swish_gate_workgroups(int64_t M, int64_t N) {
  if (M <= 0 || N <= 0) return 1;
  return rows_grid(M, rpw_of((int)N), 2048);
}

extern "C" int fla_norm_swish_gate_residual_fwd(const void* x, const void* gate, const float* weight, const float* bias,
                                                const void* residual, int residual_dtype, void* y, void* residual_out,
                                                int residual_out_dtype, float* mean, float* rstd, int64_t M, int64_t N,
                                                float eps, int is_rms_norm, int dtype, fla_stream_t stream) {
  FLA_REQUIRE(x && gate && y && rstd && M >= 0 && N > 0, FLA_E_INVALID);
  FLA_REQUIRE(is_rms_norm || mean, FLA_E_INVALID);
  FLA_REQUIRE(N % 8 == 0 && N <= 2048, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)gate) | ((uintptr_t)y) | ((uintptr_t)residual) | ((uintptr_t)residual_out)) % 16 == 0,
              FLA_E_ALIGNMENT);
  if (residual) FLA_REQUIRE(residual_dtype == dtype || residual_dtype == FLA_F32, FLA_E_UNSUPPORTED);
  if (residual_out) FLA_REQUIRE(residual_out_dtype == dtype || residual_out_dtype == FLA_F32, FLA_E_UNSUPPORTED);
  if (M == 0) return FLA_OK;
  NormGateParams p{x, gate, weight, bias, y, mean, rstd, nullptr, nullptr, nullptr, nullptr, nullptr, M, (int)N, eps,
                   residual, residual_out, nullptr, nullptr,
                   residual && residual_dtype == FLA_F32, residual_out && residual_out_dtype == FLA_F32, 0};
  const int grid = rows_grid(M, rpw_of((int)N), 4096);   // grid-stride: weights are loaded once per lane
  hipStream_t st = (hipStream_t)stream;
#define D(E, TT)                                                         \
  if (dtype == E) {                                                      \
    if (is_rms_norm) return launch_ng<TT, true>(p, false, grid, st);     \
    return launch_ng<TT, false>(p, false, grid, st);                     \
  }
  D(FLA_BF16, bf16)
  D(FLA_F16, f16)
  D(FLA_F32, float)
#undef D
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_norm_swish_gate_fwd(const void* x, const void* gate, const float* weight, const float* bias, void* y,
                                       float* mean, float* rstd, int64_t M, int64_t N, float eps, int is_rms_norm,
                                       int dtype, fla_stream_t stream) {
  return fla_norm_swish_gate_residual_fwd(x, gate, weight, bias, nullptr, dtype, y, nullptr, dtype, mean, rstd, M, N, eps,
                                          is_rms_norm, dtype, stream);
}

extern "C" int fla_norm_swish_gate_residual_bwd(const void* dy, const void* x, int x_dtype, const void* gate,
                                                const float* weight, const float* bias, const float* mean,
                                                const float* rstd, const void* dresidual, void* dx, void* dgate,
                                                void* dresidual_in, float* dw_partial, float* db_partial, int64_t M,
                                                int64_t N, float eps, int is_rms_norm, int dtype, fla_stream_t stream) {
  FLA_REQUIRE(dy && x && gate && rstd && dx && dgate && M >= 0 && N > 0, FLA_E_INVALID);
  FLA_REQUIRE(is_rms_norm || mean, FLA_E_INVALID);
  FLA_REQUIRE(N % 8 == 0 && N <= 2048, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(x_dtype == dtype || x_dtype == FLA_F32, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)gate) | ((uintptr_t)dy) | ((uintptr_t)dx) | ((uintptr_t)dgate) |
               ((uintptr_t)dresidual) | ((uintptr_t)dresidual_in)) % 16 == 0,
              FLA_E_ALIGNMENT);
  if (M == 0) return FLA_OK;
  NormGateParams p{x, gate, weight, bias, nullptr, (float*)mean, (float*)rstd, dy, dx, dgate, dw_partial, db_partial,
                   M, (int)N, eps, nullptr, nullptr, dresidual, dresidual_in, 0, 0, x_dtype == FLA_F32};
  const int grid = fla_norm_swish_gate_workgroups(M, N);
  hipStream_t st = (hipStream_t)stream;
#define D(E, TT)                                                        \
  if (dtype == E) {                                                     \
    if (is_rms_norm) return launch_ng<TT, true>(p, true, grid, st);     \
    return launch_ng<TT, false>(p, true, grid, st);                     \
  }
  D(FLA_BF16, bf16)
  D(FLA_F16, f16)
  D(FLA_F32, float)
#undef D
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_norm_swish_gate_bwd(const void* dy, const void* x, const void* gate, const float* weight,
                                       const float* bias, const float* mean, const float* rstd, void* dx, void* dgate,
                                       float* dw_partial, float* db_partial, int64_t M, int64_t N, float eps,
                                       int is_rms_norm, int dtype, fla_stream_t stream) {
  return fla_norm_swish_gate_residual_bwd(dy, x, dtype, gate, weight, bias, mean, rstd, nullptr, dx, dgate, nullptr,
                                          dw_partial, db_partial, M, N, eps, is_rms_norm, dtype, stream);
}
