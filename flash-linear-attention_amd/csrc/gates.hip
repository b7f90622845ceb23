// Gate pre-activations of the layers that call the chunk operators:
//   GLA             gk = logsigmoid(x) / normalizer, optionally clamped from below
//                   (fla/layers/gla.py:214-217)
//   gated DeltaNet  g = -exp(A_log) * softplus(a + dt_bias), beta = sigmoid(b)
//                   (fla/layers/gated_deltanet.py:236-237)
// forward and backward.  Elementwise HBM streams: 8 elements (16 or 32 bytes) per lane and step.
// The per-head parameter gradients of the second form (dA_log, d dt_bias) are per-workgroup partial
// sums in a fixed order, added by the caller: no atomics, bit-reproducible.
#include "fla_common.h"

namespace {

// log(1 + e) for 0 <= e: the alternating series where 1 + e would round the small term away (four terms are
// exact to 1e-8 relative below 2^-6), the hardware logarithm above (relative error below 4e-6 there).  The
// library's log1p costs several times the instructions and made these kernels issue-bound.
FLA_DEVICE float log1p_pos(float e) {
  const float series = e * (1.f - e * (0.5f - e * (1.f / 3.f - 0.25f * e)));
  return e < 0.015625f ? series : __logf(1.f + e);
}

// log(sigmoid(x)) = min(x, 0) - log1p(e^{-|x|})
FLA_DEVICE float log_sigmoid(float x) { return fminf(x, 0.f) - log1p_pos(__expf(-fabsf(x))); }

// torch.nn.functional.softplus with its defaults (beta = 1, threshold = 20)
FLA_DEVICE float softplus(float x) { return x > 20.f ? x : log1p_pos(__expf(x)); }

FLA_DEVICE float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

template <typename T>
struct Vec8 {
  typedef typename Elem<T>::v8 raw;
  static FLA_DEVICE void load(const T* p, float* o) {
    const raw a = *(const raw*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)a[i];
  }
  static FLA_DEVICE void store(T* p, const float* v) {
    raw a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = (T)v[i];
    *(raw*)p = a;
  }
};
template <>
struct Vec8<float> {
  static FLA_DEVICE void load(const float* p, float* o) {
    const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
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

// y = max(logsigmoid(x) * inv_norm, clamp_min)   (clamp_min = -inf: no clamp); n % 8 == 0
template <typename TX, typename TY>
__global__ __launch_bounds__(256) void gate_logsigmoid_fwd_kernel(const TX* __restrict__ x, TY* __restrict__ y,
                                                                  int64_t n8, float inv_norm, float clamp_min) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    float v[8];
    Vec8<TX>::load(x + 8 * i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fmaxf(log_sigmoid(v[j]) * inv_norm, clamp_min);
    Vec8<TY>::store(y + 8 * i, v);
  }
}

// dx = dy * inv_norm * sigmoid(-x) where the clamp did not bind, 0 where it did
template <typename TX, typename TD>
__global__ __launch_bounds__(256) void gate_logsigmoid_bwd_kernel(const TX* __restrict__ x, const TD* __restrict__ dy,
                                                                  TX* __restrict__ dx, int64_t n8, float inv_norm,
                                                                  float clamp_min) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    float v[8], d[8];
    Vec8<TX>::load(x + 8 * i, v);
    Vec8<TD>::load(dy + 8 * i, d);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool open = log_sigmoid(v[j]) * inv_norm >= clamp_min;
      d[j] = open ? d[j] * inv_norm * sigmoidf(-v[j]) : 0.f;
    }
    Vec8<TX>::store(dx + 8 * i, d);
  }
}

// Elements of [M, H] are walked with a stride that is a multiple of H, so a thread keeps one head.
struct HeadWalk {
  int64_t first, stride;
  int h;
  bool active;
};
FLA_DEVICE HeadWalk head_walk(int H) {
  const int64_t nthr = (int64_t)gridDim.x * 256;
  HeadWalk w;
  w.stride = nthr / H * H;
  w.first = (int64_t)blockIdx.x * 256 + threadIdx.x;
  w.active = w.first < w.stride;
  w.h = (int)(w.first % H);
  return w;
}

template <typename TA, typename TB>
__global__ __launch_bounds__(256) void gdn_gate_fwd_kernel(const TA* __restrict__ a, const TB* __restrict__ b,
                                                           const float* __restrict__ A_log,
                                                           const float* __restrict__ dt_bias, float* __restrict__ g,
                                                           TB* __restrict__ beta, int64_t n, int H) {
  const HeadWalk w = head_walk(H);
  if (!w.active) return;
  const float neg_A = -__expf(A_log[w.h]);
  const float bias = dt_bias ? dt_bias[w.h] : 0.f;
  for (int64_t i = w.first; i < n; i += w.stride) {
    g[i] = neg_A * softplus((float)a[i] + bias);
    if (b) beta[i] = (TB)sigmoidf((float)b[i]);
  }
}

// da = dg * (-e^{A_log}) * softplus'(a + dt_bias), db = dbeta * beta (1 - beta);
// part[block][0][h] = sum dg * g (the gradient of A_log), part[block][1][h] = sum da (that of dt_bias)
template <typename TA, typename TB>
__global__ __launch_bounds__(256) void gdn_gate_bwd_kernel(const TA* __restrict__ a, const TB* __restrict__ b,
                                                           const float* __restrict__ A_log,
                                                           const float* __restrict__ dt_bias,
                                                           const float* __restrict__ dg, const TB* __restrict__ dbeta,
                                                           TA* __restrict__ da, TB* __restrict__ db,
                                                           float* __restrict__ part, int64_t n, int H) {
  __shared__ float sA[256], sB[256];
  const HeadWalk w = head_walk(H);
  float accA = 0.f, accB = 0.f;
  if (w.active) {
    const float neg_A = -__expf(A_log[w.h]);
    const float bias = dt_bias ? dt_bias[w.h] : 0.f;
    for (int64_t i = w.first; i < n; i += w.stride) {
      const float x = (float)a[i] + bias;
      const float d = dg[i];
      const float dx = d * neg_A * (x > 20.f ? 1.f : sigmoidf(x));
      da[i] = (TA)dx;
      accA += d * neg_A * softplus(x);
      accB += dx;
      if (b) {
        const float s = sigmoidf((float)b[i]);
        db[i] = (TB)((float)dbeta[i] * s * (1.f - s));
      }
    }
  }
  sA[threadIdx.x] = accA;
  sB[threadIdx.x] = accB;
  __syncthreads();
  // threads t, t + H', t + 2H', ... of a block share a head when 256 % H == 0; in general the head of
  // thread t is (blockIdx.x * 256 + t) % H
  if ((int)threadIdx.x < H) {
    const int hh = threadIdx.x;
    float tA = 0.f, tB = 0.f;
    const int first = (int)(((int64_t)hh - (int64_t)blockIdx.x * 256 % H + H) % H);
    for (int t = first; t < 256; t += H) {
      tA += sA[t];
      tB += sB[t];
    }
    part[((int64_t)blockIdx.x * 2 + 0) * H + hh] = tA;
    part[((int64_t)blockIdx.x * 2 + 1) * H + hh] = tB;
  }
}

int stream_blocks(int64_t n_items) {
  const int64_t want = fla_cdiv(n_items, 256);
  return (int)(want < 1 ? 1 : want > 2048 ? 2048 : want);
}

}  // namespace

extern "C" int fla_gate_logsigmoid_fwd(const void* x, void* y, int64_t n, float normalizer, int has_clamp,
                                       float clamp_min, int x_dtype, int y_dtype, fla_stream_t stream) {
  FLA_REQUIRE(n >= 0 && normalizer != 0.f, FLA_E_INVALID);
  if (n == 0) return FLA_OK;
  FLA_REQUIRE(x && y, FLA_E_INVALID);
  FLA_REQUIRE(n % 8 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)x | (uintptr_t)y) % 16 == 0, FLA_E_ALIGNMENT);
  const float inv = 1.f / normalizer, cm = has_clamp ? clamp_min : -INFINITY;
  const int64_t n8 = n / 8;
  dim3 grid(stream_blocks(n8)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define FLA_GATE(TX, TY) \
  hipLaunchKernelGGL((gate_logsigmoid_fwd_kernel<TX, TY>), grid, block, 0, st, (const TX*)x, (TY*)y, n8, inv, cm)
  if (x_dtype == FLA_F32 && y_dtype == FLA_F32) FLA_GATE(float, float);
  else if (x_dtype == FLA_BF16 && y_dtype == FLA_F32) FLA_GATE(bf16, float);
  else if (x_dtype == FLA_F16 && y_dtype == FLA_F32) FLA_GATE(f16, float);
  else if (x_dtype == FLA_BF16 && y_dtype == FLA_BF16) FLA_GATE(bf16, bf16);
  else if (x_dtype == FLA_F16 && y_dtype == FLA_F16) FLA_GATE(f16, f16);
  else return FLA_E_UNSUPPORTED;
#undef FLA_GATE
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

extern "C" int fla_gate_logsigmoid_bwd(const void* x, const void* dy, void* dx, int64_t n, float normalizer,
                                       int has_clamp, float clamp_min, int x_dtype, int dy_dtype,
                                       fla_stream_t stream) {
  FLA_REQUIRE(n >= 0 && normalizer != 0.f, FLA_E_INVALID);
  if (n == 0) return FLA_OK;
  FLA_REQUIRE(x && dy && dx, FLA_E_INVALID);
  FLA_REQUIRE(n % 8 == 0, FLA_E_UNSUPPORTED);
  FLA_REQUIRE(((uintptr_t)x | (uintptr_t)dy | (uintptr_t)dx) % 16 == 0, FLA_E_ALIGNMENT);
  const float inv = 1.f / normalizer, cm = has_clamp ? clamp_min : -INFINITY;
  const int64_t n8 = n / 8;
  dim3 grid(stream_blocks(n8)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define FLA_GATE(TX, TD)                                                                                       \
  hipLaunchKernelGGL((gate_logsigmoid_bwd_kernel<TX, TD>), grid, block, 0, st, (const TX*)x, (const TD*)dy, \
                     (TX*)dx, n8, inv, cm)
  if (x_dtype == FLA_F32 && dy_dtype == FLA_F32) FLA_GATE(float, float);
  else if (x_dtype == FLA_BF16 && dy_dtype == FLA_F32) FLA_GATE(bf16, float);
  else if (x_dtype == FLA_F16 && dy_dtype == FLA_F32) FLA_GATE(f16, float);
  else if (x_dtype == FLA_BF16 && dy_dtype == FLA_BF16) FLA_GATE(bf16, bf16);
  else if (x_dtype == FLA_F16 && dy_dtype == FLA_F16) FLA_GATE(f16, f16);
  else return FLA_E_UNSUPPORTED;
#undef FLA_GATE
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

extern "C" int fla_gdn_gate_workgroups(int64_t M, int64_t H) {
  if (M < 0 || H <= 0 || H > 256) return 0;
  return stream_blocks(M * H);
}

extern "C" int fla_gdn_gate_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g,
                                void* beta, int64_t M, int64_t H, int a_dtype, int b_dtype, fla_stream_t stream) {
  FLA_REQUIRE(M >= 0 && H > 0, FLA_E_INVALID);
  FLA_REQUIRE(H <= 256, FLA_E_UNSUPPORTED);
  if (M == 0) return FLA_OK;
  FLA_REQUIRE(a && A_log && g && ((b == nullptr) == (beta == nullptr)), FLA_E_INVALID);
  dim3 grid(stream_blocks(M * H)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define FLA_GATE(TA, TB)                                                                                    \
  hipLaunchKernelGGL((gdn_gate_fwd_kernel<TA, TB>), grid, block, 0, st, (const TA*)a, (const TB*)b, A_log, \
                     dt_bias, g, (TB*)beta, M * H, (int)H)
  if (a_dtype == FLA_F32 && b_dtype == FLA_F32) FLA_GATE(float, float);
  else if (a_dtype == FLA_BF16 && b_dtype == FLA_BF16) FLA_GATE(bf16, bf16);
  else if (a_dtype == FLA_F16 && b_dtype == FLA_F16) FLA_GATE(f16, f16);
  else return FLA_E_UNSUPPORTED;
#undef FLA_GATE
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}

extern "C" int fla_gdn_gate_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias,
                                const float* dg, const void* dbeta, void* da, void* db, float* partials, int64_t M,
                                int64_t H, int a_dtype, int b_dtype, fla_stream_t stream) {
  FLA_REQUIRE(M >= 0 && H > 0, FLA_E_INVALID);
  FLA_REQUIRE(H <= 256, FLA_E_UNSUPPORTED);
  if (M == 0) return FLA_OK;
  FLA_REQUIRE(a && A_log && dg && da && partials, FLA_E_INVALID);
  FLA_REQUIRE((b == nullptr) == (db == nullptr) && (b == nullptr) == (dbeta == nullptr), FLA_E_INVALID);
  dim3 grid(stream_blocks(M * H)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define FLA_GATE(TA, TB)                                                                                    \
  hipLaunchKernelGGL((gdn_gate_bwd_kernel<TA, TB>), grid, block, 0, st, (const TA*)a, (const TB*)b, A_log, \
                     dt_bias, dg, (const TB*)dbeta, (TA*)da, (TB*)db, partials, M * H, (int)H)
  if (a_dtype == FLA_F32 && b_dtype == FLA_F32) FLA_GATE(float, float);
  else if (a_dtype == FLA_BF16 && b_dtype == FLA_BF16) FLA_GATE(bf16, bf16);
  else if (a_dtype == FLA_F16 && b_dtype == FLA_F16) FLA_GATE(f16, f16);
  else return FLA_E_UNSUPPORTED;
#undef FLA_GATE
  FLA_CHECK_LAUNCH();
  return FLA_OK;
}
