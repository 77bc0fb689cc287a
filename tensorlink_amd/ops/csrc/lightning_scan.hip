// Lightning (decayed linear) attention over ragged sequences (gfx950).
//
// Per head, with one fixed decay a in (0, 1]:
//     S_t = a S_(t-1) + k_t v_t^T        (S is [D, V], fp32, per slot)
//     o_t = S_t^T q_t
// q, k, v are silu of columns of the fused projection (bf16 or fp32),
// evaluated in fp32. One block per (sequence, head) walks the sequence's
// new tokens in order; the state comes from the sequence's slot (zeros when
// it has no cached tokens) and goes back there, so prompt portions of any
// size and single decoded tokens run the same arithmetic in the same
// order. The read-out is stored raw in fp32; the norm over all heads and
// the output gate follow in tl_rms_scale.
//
// Register form: thread (c, g) owns column c of S for the rows
// d = g, g + DG, g + 2 DG, ... (DR of them, VR columns c + r*VT per
// thread), so a token costs DR*VR FMAs per thread for the update and as
// many for the read-out; the DG partial read-outs of a column meet in LDS.
// Tokens are staged in rounds of RT so a round needs three barriers.
// Shapes whose state does not fit the register budget take the generic
// kernel, which keeps S in the slot's memory.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;
constexpr int RT = 8;  // tokens per round

template <typename T> DEVINLINE float ldf(const T* p) ;
template <> DEVINLINE float ldf<float>(const float* p) { return *p; }
template <> DEVINLINE float ldf<bf16>(const bf16* p) { return bf2f(*p); }

DEVINLINE float silu(float z) { return z / (1.f + expf(-z)); }

template <typename T, int DR, int VR>
__global__ __launch_bounds__(BLOCK) void lightning_scan_kernel(
    const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
    const float* __restrict__ decay, float* __restrict__ S,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ pos0, float* __restrict__ out, int H, int D,
    int V, int VT, int DG) {
  extern __shared__ float lds[];
  // lds: qs[RT][D] | ks[RT][D] | vs[RT][V] | part[RT][DG][V]
  float* qs = lds;
  float* ks = qs + RT * D;
  float* vs = ks + RT * D;
  float* part = vs + RT * V;
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  const int c0 = threadIdx.x % VT, g = threadIdx.x / VT;
  const float a = decay[h];
  float* Sh = S + ((int64_t)slots[b] * H + h) * D * V;
  float st[DR][VR];
  const bool fresh = pos0[b] == 0;
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = g + r * DG;
#pragma unroll
    for (int u = 0; u < VR; ++u) {
      const int c = c0 + u * VT;
      st[r][u] = (!fresh && d < D && c < V) ? Sh[(int64_t)d * V + c] : 0.f;
    }
  }
  for (int tb = t0; tb < t1; tb += RT) {
    const int nt = min(RT, t1 - tb);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * D; i += BLOCK) {
      const int tt = i / D, d = i - tt * D;
      const T* row = proj + (int64_t)(tb + tt) * ld;
      qs[tt * D + d] = silu(ldf<T>(row + q_off + h * D + d));
      ks[tt * D + d] = silu(ldf<T>(row + k_off + h * D + d));
    }
    for (int i = threadIdx.x; i < nt * V; i += BLOCK) {
      const int tt = i / V, c = i - tt * V;
      vs[tt * V + c] =
          silu(ldf<T>(proj + (int64_t)(tb + tt) * ld + v_off + h * V + c));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      float vv[VR], acc[VR];
#pragma unroll
      for (int u = 0; u < VR; ++u) {
        const int c = c0 + u * VT;
        vv[u] = c < V ? vs[tt * V + c] : 0.f;
        acc[u] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < DR; ++r) {
        const int d = g + r * DG;
        const float kd = d < D ? ks[tt * D + d] : 0.f;
        const float qd = d < D ? qs[tt * D + d] : 0.f;
#pragma unroll
        for (int u = 0; u < VR; ++u) {
          st[r][u] = a * st[r][u] + kd * vv[u];
          acc[u] += st[r][u] * qd;
        }
      }
#pragma unroll
      for (int u = 0; u < VR; ++u) {
        const int c = c0 + u * VT;
        if (c < V) part[(tt * DG + g) * V + c] = acc[u];
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * V; i += BLOCK) {
      const int tt = i / V, c = i - tt * V;
      float o = 0.f;
      for (int gg = 0; gg < DG; ++gg) o += part[(tt * DG + gg) * V + c];
      out[((int64_t)(tb + tt) * H + h) * V + c] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < DR; ++r) {
    const int d = g + r * DG;
#pragma unroll
    for (int u = 0; u < VR; ++u) {
      const int c = c0 + u * VT;
      if (d < D && c < V) Sh[(int64_t)d * V + c] = st[r][u];
    }
  }
}

// Any head size: the state stays in the slot's memory; thread c owns the
// columns c, c + BLOCK, ... and walks all rows for every token.
template <typename T>
__global__ __launch_bounds__(BLOCK) void lightning_scan_generic_kernel(
    const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
    const float* __restrict__ decay, float* __restrict__ S,
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ pos0, float* __restrict__ out, int H, int D,
    int V) {
  extern __shared__ float lds[];  // qs[D] | ks[D]
  float* qs = lds;
  float* ks = lds + D;
  const int b = blockIdx.x, h = blockIdx.y;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  const float a = decay[h];
  float* Sh = S + ((int64_t)slots[b] * H + h) * D * V;
  if (pos0[b] == 0)
    for (int i = threadIdx.x; i < D * V; i += BLOCK) Sh[i] = 0.f;
  for (int t = t0; t < t1; ++t) {
    __syncthreads();
    const T* row = proj + (int64_t)t * ld;
    for (int d = threadIdx.x; d < D; d += BLOCK) {
      qs[d] = silu(ldf<T>(row + q_off + h * D + d));
      ks[d] = silu(ldf<T>(row + k_off + h * D + d));
    }
    __syncthreads();
    for (int c = threadIdx.x; c < V; c += BLOCK) {
      const float vv = silu(ldf<T>(row + v_off + h * V + c));
      float acc = 0.f;
      for (int d = 0; d < D; ++d) {
        const float s = a * Sh[(int64_t)d * V + c] + ks[d] * vv;
        Sh[(int64_t)d * V + c] = s;
        acc += s * qs[d];
      }
      out[((int64_t)t * H + h) * V + c] = acc;
    }
  }
}

}  // namespace

extern "C" {

// returns 0 on success, 1 if the launch cannot be made
int tl_lightning_scan(const void* proj, int ld, int q_off, int k_off,
                      int v_off, const void* decay, void* S, const void* cu,
                      const void* slots, const void* pos0, void* out, int B,
                      int H, int D, int V, int is_f32, hipStream_t stream) {
  if (B <= 0 || H <= 0 || D <= 0 || V <= 0) return 1;
  dim3 grid(B, H), block(BLOCK);
  // column threads: the smallest power of two >= V, at most the block
  int VT = 1;
  while (VT < V && VT < BLOCK) VT <<= 1;
  const int DG = BLOCK / VT;
  const int vr = (V + VT - 1) / VT;
  const int dr = (D + DG - 1) / DG;
  const size_t smem = sizeof(float) * ((size_t)RT * (2 * D + V) +
                                       (size_t)RT * DG * V);
#define TL_LS(TT, DRR, VRR)                                                  \
  hipLaunchKernelGGL((lightning_scan_kernel<TT, DRR, VRR>), grid, block,     \
                     smem, stream, (const TT*)proj, ld, q_off, k_off, v_off, \
                     (const float*)decay, (float*)S, (const int*)cu,         \
                     (const int*)slots, (const int*)pos0, (float*)out, H, D, \
                     V, VT, DG)
#define TL_LS_T(DRR, VRR)     \
  do {                        \
    if (is_f32)               \
      TL_LS(float, DRR, VRR); \
    else                      \
      TL_LS(bf16, DRR, VRR);  \
    return 0;                 \
  } while (0)
  if (smem <= 64 * 1024) {
    if (vr == 1) {
      if (dr <= 8) TL_LS_T(8, 1);
      if (dr <= 16) TL_LS_T(16, 1);
      if (dr <= 32) TL_LS_T(32, 1);
      if (dr <= 64) TL_LS_T(64, 1);
      if (dr <= 128) TL_LS_T(128, 1);
    } else if (vr == 2) {
      if (dr <= 32) TL_LS_T(32, 2);
      if (dr <= 64) TL_LS_T(64, 2);
    }
  }
#undef TL_LS_T
#undef TL_LS
  const size_t gsmem = sizeof(float) * 2 * (size_t)D;
  if (gsmem > 64 * 1024) return 1;
  if (is_f32)
    hipLaunchKernelGGL(lightning_scan_generic_kernel<float>, grid, block,
                       gsmem, stream, (const float*)proj, ld, q_off, k_off,
                       v_off, (const float*)decay, (float*)S, (const int*)cu,
                       (const int*)slots, (const int*)pos0, (float*)out, H,
                       D, V);
  else
    hipLaunchKernelGGL(lightning_scan_generic_kernel<bf16>, grid, block,
                       gsmem, stream, (const bf16*)proj, ld, q_off, k_off,
                       v_off, (const float*)decay, (float*)S, (const int*)cu,
                       (const int*)slots, (const int*)pos0, (float*)out, H,
                       D, V);
  return 0;
}

}  // extern "C"
