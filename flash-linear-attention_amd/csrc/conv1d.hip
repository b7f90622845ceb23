// Depthwise causal short convolution over time in the layers' own [B,T,D] layout (channels
// last), with optional bias and SiLU:  y[b,t,d] = act(bias[d] + sum_i w[d,i] x[b,t-(W-1)+i,d]).
// Replaces the external causal_conv1d package the reference's ShortConvolution needs
// (fla/modules/convolution.py:79-211; forward :171-186, single-token step :188-211).
//
// HBM-streaming kernels: a lane owns 8 (backward: 4) adjacent channels (one 16-byte access per
// row for 16-bit storage) and walks a tile of consecutive time steps with the last W inputs (and, in
// backward, the last W pre-activation gradients) in registers, so every input row is read
// once per tile plus a (W-1)-row halo that the neighbouring tile has just pulled into L2.
// The weight/bias gradients are accumulated in registers over all tiles a lane visits, summed
// over the workgroup's tile slots in LDS and written once per workgroup (the host adds the
// per-workgroup partial sums: deterministic, no atomics).
#include "fla_common.h"

namespace {

constexpr int TT = 16;   // time steps per tile

// A lane's slice of one row: N adjacent channels, kept in storage precision until use so that
// a whole tile of rows can be in flight at once.
template <typename T, int N>
struct Chan {
  typedef T raw __attribute__((ext_vector_type(N)));
  static FLA_DEVICE raw load(const T* p) { return *(const raw*)p; }
  static FLA_DEVICE raw zero() {
    raw r;
#pragma unroll
    for (int i = 0; i < N; ++i) r[i] = (T)0.f;
    return r;
  }
  static FLA_DEVICE void to_f32(raw r, float* o) {
#pragma unroll
    for (int i = 0; i < N; ++i) o[i] = (float)r[i];
  }
  static FLA_DEVICE void store(T* p, const float* v) {
    raw r;
#pragma unroll
    for (int i = 0; i < N; ++i) r[i] = (T)v[i];
    *(raw*)p = r;
  }
};

struct ConvParams {
  const void* x;       // [B,T,D]
  const float* w;      // [D,W] fp32
  const float* bias;   // [D] fp32 or NULL
  void* y;             // [B,T,D]
  const void* dy;      // backward
  void* dx;
  float* dw;           // [gridDim.y, D, W] fp32 partial sums
  float* dbias;        // [gridDim.y, D] fp32 partial sums or NULL
  int64_t B, T;
  int D, silu;
};

FLA_DEVICE float silu_f(float z) { return z * __builtin_amdgcn_rcpf(1.f + __expf(-z)); }
FLA_DEVICE float silu_grad(float z) {
  const float s = __builtin_amdgcn_rcpf(1.f + __expf(-z));  // hardware reciprocal (1 ulp), not an IEEE division
  return s * (1.f + z * (1.f - s));
}

// block (64, 4): x = channel vector, y = tile slot; grid (channel blocks, tile groups): the
// workgroups that share rows of x are adjacent in dispatch order
template <typename T, int W>
__global__ __launch_bounds__(256) void conv_fwd_kernel(ConvParams p) {
  constexpr int CV = 8;
  typedef Chan<T, CV> C;
  const int dv = blockIdx.x * 64 + threadIdx.x;
  const int D = p.D;
  if (dv * CV >= D) return;
  const int d0 = dv * CV;
  float w[W][CV], bias[CV];
#pragma unroll
  for (int j = 0; j < CV; ++j) {
#pragma unroll
    for (int i = 0; i < W; ++i) w[i][j] = p.w[(int64_t)(d0 + j) * W + i];
    bias[j] = p.bias ? p.bias[d0 + j] : 0.f;
  }
  const int64_t tiles_per_seq = (p.T + TT - 1) / TT, ntiles = p.B * tiles_per_seq;
  for (int64_t tile = (int64_t)blockIdx.y * 4 + threadIdx.y; tile < ntiles; tile += (int64_t)gridDim.y * 4) {
    const int64_t b = tile / tiles_per_seq, t0 = (tile % tiles_per_seq) * TT;
    const T* xb = (const T*)p.x + (b * p.T) * D + d0;
    T* yb = (T*)p.y + (b * p.T) * D + d0;
    // rows t0-(W-1) .. t0+TT-1, all loads in flight at once; rows outside the sequence read
    // row 0 (always valid here) and are zeroed
    typename C::raw rows[TT + W - 1];
#pragma unroll
    for (int s = 0; s < TT + W - 1; ++s) {
      const int64_t t = t0 - (W - 1) + s;
      rows[s] = C::load(xb + ((t >= 0 && t < p.T) ? t : 0) * D);
    }
    float win[W][CV];   // win[i] = x[t - (W-1) + i]
#pragma unroll
    for (int s = 0; s < TT + W - 1; ++s) {
      const int64_t t = t0 - (W - 1) + s;
#pragma unroll
      for (int i = 0; i < W - 1; ++i)
#pragma unroll
        for (int j = 0; j < CV; ++j) win[i][j] = win[i + 1][j];
      C::to_f32((t >= 0 && t < p.T) ? rows[s] : C::zero(), win[W - 1]);
      if (s >= W - 1 && t < p.T) {
        float out[CV];
#pragma unroll
        for (int j = 0; j < CV; ++j) {
          float acc = bias[j];
#pragma unroll
          for (int i = 0; i < W; ++i) acc = fmaf(w[i][j], win[i][j], acc);
          out[j] = p.silu ? silu_f(acc) : acc;
        }
        C::store(yb + t * D, out);
      }
    }
  }
}

// Backward: a lane owns 4 channels (the running state is four times the forward's).
template <typename T, int W>
__global__ __launch_bounds__(256) void conv_bwd_kernel(ConvParams p) {
  constexpr int CV = 4;
  typedef Chan<T, CV> C;
  __shared__ float sred[4][64][(W + 1) * CV + 1];
  const int dv = blockIdx.x * 64 + threadIdx.x;
  const int D = p.D;
  const bool active = dv * CV < D;   // idle lanes still take part in the reduction barrier
  const int d0 = active ? dv * CV : 0;
  float w[W][CV], bias[CV], dw[W][CV], db[CV];
#pragma unroll
  for (int j = 0; j < CV; ++j) {
#pragma unroll
    for (int i = 0; i < W; ++i) {
      w[i][j] = p.w[(int64_t)(d0 + j) * W + i];
      dw[i][j] = 0.f;
    }
    bias[j] = p.bias ? p.bias[d0 + j] : 0.f;
    db[j] = 0.f;
  }
  const int64_t tiles_per_seq = (p.T + TT - 1) / TT, ntiles = active ? p.B * tiles_per_seq : 0;
  for (int64_t tile = (int64_t)blockIdx.y * 4 + threadIdx.y; tile < ntiles; tile += (int64_t)gridDim.y * 4) {
    const int64_t b = tile / tiles_per_seq, t0 = (tile % tiles_per_seq) * TT;
    const T* xb = (const T*)p.x + (b * p.T) * D + d0;
    const T* gb = (const T*)p.dy + (b * p.T) * D + d0;
    T* dxb = (T*)p.dx + (b * p.T) * D + d0;
    // x rows t0-(W-1) .. t0+TT+W-2 and dy rows t0 .. t0+TT+W-2, all loads in flight at once
    // (rows outside the sequence read row 0 and are zeroed)
    typename C::raw xr[TT + 2 * (W - 1)], gr[TT + W - 1];
#pragma unroll
    for (int s = 0; s < TT + 2 * (W - 1); ++s) {
      const int64_t t = t0 - (W - 1) + s;
      xr[s] = C::load(xb + ((t >= 0 && t < p.T) ? t : 0) * D);
    }
#pragma unroll
    for (int s = 0; s < TT + W - 1; ++s) {
      const int64_t t = t0 + s;
      gr[s] = C::load(gb + (t < p.T ? t : 0) * D);
    }
    float win[W][CV];   // inputs   x[t-(W-1) .. t]
    float dpw[W][CV];   // pre-activation gradients of steps t-(W-1) .. t
#pragma unroll
    for (int i = 0; i < W; ++i)
#pragma unroll
      for (int j = 0; j < CV; ++j) dpw[i][j] = 0.f;
#pragma unroll
    for (int i = 0; i < W - 1; ++i) C::to_f32((t0 - (W - 1) + i >= 0) ? xr[i] : C::zero(), win[i + 1]);
    // step s (time t0+s) forms the pre-activation gradient of its own time step; the input
    // gradient of time t0+s-(W-1) is complete once the W steps ahead of it are known
#pragma unroll
    for (int s = 0; s < TT + W - 1; ++s) {
      const int64_t t = t0 + s;
      const bool live = t < p.T;
      float gs[CV];
#pragma unroll
      for (int i = 0; i < W - 1; ++i)
#pragma unroll
        for (int j = 0; j < CV; ++j) {
          win[i][j] = win[i + 1][j];
          dpw[i][j] = dpw[i + 1][j];
        }
      C::to_f32(live ? xr[s + W - 1] : C::zero(), win[W - 1]);
      C::to_f32(live ? gr[s] : C::zero(), gs);
#pragma unroll
      for (int j = 0; j < CV; ++j) {
        float dp = gs[j];
        if (p.silu) {
          float pre = bias[j];
#pragma unroll
          for (int i = 0; i < W; ++i) pre = fmaf(w[i][j], win[i][j], pre);
          dp *= silu_grad(pre);
        }
        dpw[W - 1][j] = dp;
      }
      if (s < TT && live) {   // own time step: weight and bias gradients
#pragma unroll
        for (int j = 0; j < CV; ++j) {
#pragma unroll
          for (int i = 0; i < W; ++i) dw[i][j] = fmaf(dpw[W - 1][j], win[i][j], dw[i][j]);
          db[j] += dpw[W - 1][j];
        }
      }
      if (s >= W - 1) {
        const int64_t to = t - (W - 1);
        if (to < p.T) {
          float out[CV];
#pragma unroll
          for (int j = 0; j < CV; ++j) {
            float acc = 0.f;
            // dx[to] = sum_i w[i] dpre[to + (W-1) - i]; dpw[m] holds dpre[to + m]
#pragma unroll
            for (int i = 0; i < W; ++i) acc = fmaf(w[i][j], dpw[W - 1 - i][j], acc);
            out[j] = acc;
          }
          C::store(dxb + to * D, out);
        }
      }
    }
  }
  // sum the four tile slots of the workgroup, then one partial per workgroup
#pragma unroll
  for (int j = 0; j < CV; ++j) {
#pragma unroll
    for (int i = 0; i < W; ++i) sred[threadIdx.y][threadIdx.x][j * W + i] = dw[i][j];
    sred[threadIdx.y][threadIdx.x][W * CV + j] = db[j];
  }
  __syncthreads();
  if (threadIdx.y == 0 && active) {
    float* dwp = p.dw + ((int64_t)blockIdx.y * D + d0) * W;
#pragma unroll
    for (int e = 0; e < W * CV; ++e)
      dwp[e] = sred[0][threadIdx.x][e] + sred[1][threadIdx.x][e] + sred[2][threadIdx.x][e] + sred[3][threadIdx.x][e];
    if (p.dbias) {
      float* dbp = p.dbias + (int64_t)blockIdx.y * D + d0;
#pragma unroll
      for (int j = 0; j < CV; ++j) {
        const int e = W * CV + j;
        dbp[j] = sred[0][threadIdx.x][e] + sred[1][threadIdx.x][e] + sred[2][threadIdx.x][e] + sred[3][threadIdx.x][e];
      }
    }
  }
}

// single-token step: shift the cache [B,D,W] left by one, append x, y = act(bias + sum cache * w)
template <typename T, int W>
__global__ __launch_bounds__(256) void conv_update_kernel(const T* __restrict__ x, T* __restrict__ cache,
                                                          const float* __restrict__ w, const float* __restrict__ bias,
                                                          T* __restrict__ y, int64_t BD, int D, int silu) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= BD) return;
  const int d = (int)(i % D);
  T c[W];
#pragma unroll
  for (int k = 0; k < W; ++k) c[k] = cache[i * W + k];
#pragma unroll
  for (int k = 0; k < W - 1; ++k) c[k] = c[k + 1];
  c[W - 1] = x[i];
  float acc = bias ? bias[d] : 0.f;
#pragma unroll
  for (int k = 0; k < W; ++k) {
    acc = fmaf((float)c[k], w[(int64_t)d * W + k], acc);
    cache[i * W + k] = c[k];
  }
  y[i] = (T)(silu ? silu_f(acc) : acc);
}

// backward: few enough workgroups that the partial sums stay small, enough to fill the chip
int64_t conv_bwd_parts(int64_t B, int64_t T) {
  const int64_t g = fla_cdiv(B * fla_cdiv(T, TT), 4);
  return g < 1 ? 1 : (g > 128 ? 128 : g);
}

template <typename T, int W>
int launch_conv(const ConvParams& p, bool bwd, hipStream_t st) {
  const int64_t ntiles = p.B * fla_cdiv(p.T, TT);
  const int64_t cblocks = fla_cdiv(p.D / (bwd ? 4 : 8), 64);
  int64_t gy = fla_cdiv(ntiles, 4);
  if (bwd) gy = conv_bwd_parts(p.B, p.T);
  else if (gy * cblocks > 4096) gy = fla_cdiv(4096, cblocks);   // a few tiles per lane: weights are loaded once
  if (gy < 1) gy = 1;
  if (gy > 65535) gy = 65535;
  dim3 grid((unsigned)cblocks, (unsigned)gy), block(64, 4);
  if (bwd) hipLaunchKernelGGL((conv_bwd_kernel<T, W>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((conv_fwd_kernel<T, W>), grid, block, 0, st, p);
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

template <typename T>
int dispatch_conv(const ConvParams& p, int W, bool bwd, hipStream_t st) {
  if (W == 2) return launch_conv<T, 2>(p, bwd, st);
  if (W == 3) return launch_conv<T, 3>(p, bwd, st);
  if (W == 4) return launch_conv<T, 4>(p, bwd, st);
  return FLA_E_UNSUPPORTED;
}

template <typename T>
int dispatch_update(const void* x, void* cache, const float* w, const float* bias, void* y, int64_t BD, int D, int W,
                    int silu, hipStream_t st) {
  dim3 grid((unsigned)fla_cdiv(BD, 256));
#define U(WW)                                                                                                    \
  if (W == WW) {                                                                                                 \
    hipLaunchKernelGGL((conv_update_kernel<T, WW>), grid, dim3(256), 0, st, (const T*)x, (T*)cache, w, bias, (T*)y, \
                       BD, D, silu);                                                                             \
    FLA_CHECK_LAUNCH();                                                                                          \
    return FLA_OK;                                                                                               \
  }
  U(2) U(3) U(4)
#undef U
  return FLA_E_UNSUPPORTED;
}

}  // namespace

extern "C" int fla_causal_conv1d_fwd(const void* x, const float* weight, const float* bias, void* y, int64_t B, int64_t T,
                                     int64_t D, int64_t W, int silu, int dtype, fla_stream_t stream) {
  FLA_REQUIRE(x && weight && y && B >= 0 && T >= 0 && D > 0, FLA_E_INVALID);
  FLA_REQUIRE(D % 8 == 0 && W >= 2 && W <= 4, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)y)) % 16 == 0, FLA_E_ALIGNMENT);
  if (B == 0 || T == 0) return FLA_OK;
  ConvParams p{x, weight, bias, y, nullptr, nullptr, nullptr, nullptr, B, T, (int)D, silu};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == FLA_BF16) return dispatch_conv<bf16>(p, (int)W, false, st);
  if (dtype == FLA_F16) return dispatch_conv<f16>(p, (int)W, false, st);
  if (dtype == FLA_F32) return dispatch_conv<float>(p, (int)W, false, st);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_causal_conv1d_bwd_partials(int64_t B, int64_t T) { return (int)conv_bwd_parts(B, T); }

extern "C" int fla_causal_conv1d_bwd(const void* x, const float* weight, const float* bias, const void* dy, void* dx,
                                     float* dw_partial, float* db_partial, int64_t B, int64_t T, int64_t D, int64_t W,
                                     int silu, int dtype, fla_stream_t stream) {
  float* dweight = dw_partial;
  float* dbias = db_partial;
  FLA_REQUIRE(x && weight && dy && dx && dweight && B >= 0 && T >= 0 && D > 0, FLA_E_INVALID);
  FLA_REQUIRE(D % 8 == 0 && W >= 2 && W <= 4, FLA_E_UNSUPPORTED);
  FLA_REQUIRE((((uintptr_t)x) | ((uintptr_t)dy) | ((uintptr_t)dx)) % 16 == 0, FLA_E_ALIGNMENT);
  if (B == 0 || T == 0) return FLA_OK;
  ConvParams p{x, weight, bias, nullptr, dy, dx, dweight, dbias, B, T, (int)D, silu};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == FLA_BF16) return dispatch_conv<bf16>(p, (int)W, true, st);
  if (dtype == FLA_F16) return dispatch_conv<f16>(p, (int)W, true, st);
  if (dtype == FLA_F32) return dispatch_conv<float>(p, (int)W, true, st);
  return FLA_E_UNSUPPORTED;
}

extern "C" int fla_causal_conv1d_update(const void* x, void* cache, const float* weight, const float* bias, void* y,
                                        int64_t B, int64_t D, int64_t W, int silu, int dtype, fla_stream_t stream) {
  FLA_REQUIRE(x && cache && weight && y && B >= 0 && D > 0, FLA_E_INVALID);
  FLA_REQUIRE(W >= 2 && W <= 4, FLA_E_UNSUPPORTED);
  if (B == 0) return FLA_OK;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == FLA_BF16) return dispatch_update<bf16>(x, cache, weight, bias, y, B * D, (int)D, (int)W, silu, st);
  if (dtype == FLA_F16) return dispatch_update<f16>(x, cache, weight, bias, y, B * D, (int)D, (int)W, silu, st);
  if (dtype == FLA_F32) return dispatch_update<float>(x, cache, weight, bias, y, B * D, (int)D, (int)W, silu, st);
  return FLA_E_UNSUPPORTED;
}
