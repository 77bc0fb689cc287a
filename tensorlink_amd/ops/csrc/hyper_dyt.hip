// Hyper-connection stream update fused with the Dynamic-Tanh norm (gfx950).
//
// A hyper-connected residual keeps `ns` fp32 copies X_1..X_ns of the
// residual stream. Around a sublayer with output y:
//     X_t <- sum_s mix[s,t] X_s + out[t] * y          (all t from the old X)
// and the NEXT sublayer reads u = sum_s in[s] X_s through a Dynamic-Tanh
// norm h = tanh(alpha * u) * w + b, which needs no row statistics. Both are
// elementwise over (token, column), so one pass over the fp32 streams does
// the update of sublayer q and the read+norm of sublayer q+1: the streams
// make one HBM round trip per sublayer instead of three.
//
// Every stage is optional:  y == null  -> no update (first sublayer);
//                           inw == null -> u is the plain sum of streams;
//                           w == null   -> no norm, h is not written
//                           usum != null -> u is also stored in fp32.
// Also here: relu(x)^2 activation for the expert feed-forward.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int MAX_STREAMS = 8;

template <typename T> DEVINLINE float ld(const T* p, int64_t i);
template <> DEVINLINE float ld<float>(const float* p, int64_t i) { return p[i]; }
template <> DEVINLINE float ld<bf16>(const bf16* p, int64_t i) { return bf2f(p[i]); }
template <typename T> DEVINLINE void st(T* p, int64_t i, float v);
template <> DEVINLINE void st<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> DEVINLINE void st<bf16>(bf16* p, int64_t i, float v) { p[i] = f2bf(v); }

// NS is the compile-time stream count (loops unroll, the copies stay in
// registers); NS == MAX_STREAMS also serves any smaller runtime count.
template <typename T, int NS>
__global__ __launch_bounds__(BLOCK) void hyper_dyt_kernel(
    float* __restrict__ X,            // [ns, TW]
    const T* __restrict__ y,          // [TW] or null
    const float* __restrict__ mix,    // [ns, ns] (from, to)
    const float* __restrict__ outw,   // [ns]
    const float* __restrict__ inw,    // [ns] or null
    const float* __restrict__ alpha,  // [1]
    const float* __restrict__ w,      // [W] or null
    const float* __restrict__ b,      // [W]
    T* __restrict__ h,                // [TW]
    float* __restrict__ usum,         // [TW] or null
    int ns, int64_t TW, int W) {
  float mx[NS * NS], ow[NS], iw[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const bool on = s < ns;
    ow[s] = (y != nullptr && on) ? outw[s] : 0.f;
    iw[s] = on ? (inw ? inw[s] : 1.f) : 0.f;
#pragma unroll
    for (int t = 0; t < NS; ++t)
      mx[s * NS + t] = (y != nullptr && on && t < ns) ? mix[s * ns + t] : 0.f;
  }
  const float al = w ? alpha[0] : 0.f;
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < TW;
       i += (int64_t)gridDim.x * BLOCK) {
    float x[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
      x[s] = (s < ns) ? X[(int64_t)s * TW + i] : 0.f;
    if (y != nullptr) {
      const float yv = ld<T>(y, i);
      float nx[NS];
#pragma unroll
      for (int t = 0; t < NS; ++t) {
        float a = ow[t] * yv;
#pragma unroll
        for (int s = 0; s < NS; ++s) a += mx[s * NS + t] * x[s];
        nx[t] = a;
      }
#pragma unroll
      for (int t = 0; t < NS; ++t) {
        x[t] = nx[t];
        if (t < ns) X[(int64_t)t * TW + i] = nx[t];
      }
    }
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) u += iw[s] * x[s];
    if (usum) usum[i] = u;
    if (w) {
      const int c = (int)(i % W);
      st<T>(h, i, tanhf(al * u) * w[c] + b[c]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void relu_sq_kernel(
    const T* __restrict__ x, T* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * BLOCK) {
    const float v = fmaxf(ld<T>(x, i), 0.f);
    st<T>(out, i, v * v);
  }
}

int grid_for(int64_t n) {
  int64_t g = (n + BLOCK - 1) / BLOCK;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

extern "C" {

void tl_hyper_dyt(void* X, const void* y, const void* mix, const void* outw,
                  const void* inw, const void* alpha, const void* w,
                  const void* b, void* h, void* usum, int ns, int64_t TW,
                  int W, int is_f32, hipStream_t stream) {
  dim3 grid(grid_for(TW)), block(BLOCK);
#define TL_HD_LAUNCH(TT, NS)                                                \
  hipLaunchKernelGGL((hyper_dyt_kernel<TT, NS>), grid, block, 0, stream,    \
                     (float*)X, (const TT*)y, (const float*)mix,            \
                     (const float*)outw, (const float*)inw,                 \
                     (const float*)alpha, (const float*)w, (const float*)b, \
                     (TT*)h, (float*)usum, ns, TW, W)
#define TL_HD_NS(TT)                                  \
  switch (ns) {                                       \
    case 1: TL_HD_LAUNCH(TT, 1); break;               \
    case 2: TL_HD_LAUNCH(TT, 2); break;               \
    case 3: TL_HD_LAUNCH(TT, 3); break;               \
    case 4: TL_HD_LAUNCH(TT, 4); break;               \
    default: TL_HD_LAUNCH(TT, MAX_STREAMS); break;    \
  }
  if (is_f32) {
    TL_HD_NS(float)
  } else {
    TL_HD_NS(bf16)
  }
#undef TL_HD_NS
#undef TL_HD_LAUNCH
}

void tl_relu_sq(const void* x, void* out, int64_t n, int is_f32,
                hipStream_t stream) {
  dim3 grid(grid_for(n)), block(BLOCK);
  if (is_f32)
    hipLaunchKernelGGL(relu_sq_kernel<float>, grid, block, 0, stream,
                       (const float*)x, (float*)out, n);
  else
    hipLaunchKernelGGL(relu_sq_kernel<bf16>, grid, block, 0, stream,
                       (const bf16*)x, (bf16*)out, n);
}

}  // extern "C"
