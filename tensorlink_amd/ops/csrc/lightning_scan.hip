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
//
// Long prompt portions take the chunk form instead. With chunks of C
// tokens, S0 the state before a chunk and i, j indices inside it:
//     o_i = a^(i+1) S0^T q_i + sum_{j<=i} a^(i-j) (q_i . k_j) v_j
//     S1  = a^n S0 + sum_j a^(n-1-j) k_j v_j^T           (n tokens in it)
// so every chunk needs four small matrix products (Q K^T, (A o M) V,
// Kw^T V, Qd S0), all chunks at once as batched fp32 GEMMs of the vendor
// library, and only the chain S0 -> S1 over a sequence's chunks is
// sequential, an elementwise pass. The kernels here do what is not a
// matrix product: tl_lightning_chunk_prep lays out silu(q), silu(k),
// silu(v) per (chunk, head), zero-padded, with the decay-weighted copies
// Qd = a^(i+1) q and Kw = a^(n-1-j) k; tl_lightning_decay_mask applies
// M[i][j] = a^(i-j) (j <= i, else 0); tl_lightning_chain turns the chunk
// summaries into the state before each chunk and leaves the final state
// in the slot. Everything is fp32.

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

// grid (chunks, H); outputs [chunk][h][C][D|V] fp32, rows >= n are zero
template <typename T>
__global__ __launch_bounds__(BLOCK) void lightning_chunk_prep_kernel(
    const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
    const float* __restrict__ decay, const int* __restrict__ cu_c,
    float* __restrict__ Qs, float* __restrict__ Qd, float* __restrict__ Ks,
    float* __restrict__ Kw, float* __restrict__ Vs, int H, int D, int V,
    int C) {
  extern __shared__ float pw[];            // a^0 .. a^C
  const int c = blockIdx.x, h = blockIdx.y;
  const int t0 = cu_c[c], n = cu_c[c + 1] - t0;
  const float a = decay[h];
  for (int i = threadIdx.x; i <= C; i += BLOCK) pw[i] = powf(a, (float)i);
  __syncthreads();
  const int64_t base = ((int64_t)c * H + h) * C;
  for (int i = threadIdx.x; i < C * D; i += BLOCK) {
    const int r = i / D, d = i - r * D;
    float qv = 0.f, kv = 0.f, qd = 0.f, kw = 0.f;
    if (r < n) {
      const T* row = proj + (int64_t)(t0 + r) * ld;
      qv = silu(ldf<T>(row + q_off + h * D + d));
      kv = silu(ldf<T>(row + k_off + h * D + d));
      qd = qv * pw[r + 1];
      kw = kv * pw[n - 1 - r];
    }
    const int64_t o = (base + r) * D + d;
    Qs[o] = qv;
    Qd[o] = qd;
    Ks[o] = kv;
    Kw[o] = kw;
  }
  for (int i = threadIdx.x; i < C * V; i += BLOCK) {
    const int r = i / V, e = i - r * V;
    float vv = 0.f;
    if (r < n)
      vv = silu(ldf<T>(proj + (int64_t)(t0 + r) * ld + v_off + h * V + e));
    Vs[(base + r) * V + e] = vv;
  }
}

// A [chunks*H][C][C] in place: A[i][j] *= a^(i-j) for j <= i, else 0
__global__ __launch_bounds__(BLOCK) void lightning_decay_mask_kernel(
    float* __restrict__ A, const float* __restrict__ decay, int H, int C) {
  extern __shared__ float pw[];
  const int h = blockIdx.x % H;
  const float a = decay[h];
  for (int i = threadIdx.x; i < C; i += BLOCK) pw[i] = powf(a, (float)i);
  __syncthreads();
  float* Ab = A + (int64_t)blockIdx.x * C * C;
  for (int i = threadIdx.x; i < C * C; i += BLOCK) {
    const int r = i / C, j = i - r * C;
    Ab[i] = j <= r ? Ab[i] * pw[r - j] : 0.f;
  }
}

// grid (B, H, ceil(D*V / BLOCK)): U [chunks][H][D*V] holds the chunk
// summaries on entry and the state BEFORE each chunk on exit; the slot
// receives the state after the sequence's last chunk.
__global__ __launch_bounds__(BLOCK) void lightning_chain_kernel(
    float* __restrict__ U, float* __restrict__ S,
    const float* __restrict__ decay, const int* __restrict__ cu_c,
    const int* __restrict__ chunk_base, const int* __restrict__ n_chunks,
    const int* __restrict__ slots, const int* __restrict__ pos0, int H,
    int DV) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * BLOCK + threadIdx.x;
  const int nc = n_chunks[b];
  if (e >= DV || nc <= 0) return;
  const float a = decay[h];
  float* Sp = S + ((int64_t)slots[b] * H + h) * DV + e;
  float s = pos0[b] == 0 ? 0.f : *Sp;
  const int c0 = chunk_base[b];
  for (int c = c0; c < c0 + nc; ++c) {
    float* up = U + ((int64_t)c * H + h) * DV + e;
    const float u = *up;
    *up = s;
    s = powf(a, (float)(cu_c[c + 1] - cu_c[c])) * s + u;
  }
  *Sp = s;
}

}  // namespace

extern "C" {

void tl_lightning_chunk_prep(const void* proj, int ld, int q_off, int k_off,
                             int v_off, const void* decay, const void* cu_c,
                             void* Qs, void* Qd, void* Ks, void* Kw, void* Vs,
                             int NC, int H, int D, int V, int C, int is_f32,
                             hipStream_t stream) {
  if (NC <= 0) return;
  dim3 grid(NC, H), block(BLOCK);
  const size_t smem = sizeof(float) * (C + 1);
  if (is_f32)
    hipLaunchKernelGGL(lightning_chunk_prep_kernel<float>, grid, block, smem,
                       stream, (const float*)proj, ld, q_off, k_off, v_off,
                       (const float*)decay, (const int*)cu_c, (float*)Qs,
                       (float*)Qd, (float*)Ks, (float*)Kw, (float*)Vs, H, D,
                       V, C);
  else
    hipLaunchKernelGGL(lightning_chunk_prep_kernel<bf16>, grid, block, smem,
                       stream, (const bf16*)proj, ld, q_off, k_off, v_off,
                       (const float*)decay, (const int*)cu_c, (float*)Qs,
                       (float*)Qd, (float*)Ks, (float*)Kw, (float*)Vs, H, D,
                       V, C);
}

void tl_lightning_decay_mask(void* A, const void* decay, int NCH, int H,
                             int C, hipStream_t stream) {
  if (NCH <= 0) return;
  hipLaunchKernelGGL(lightning_decay_mask_kernel, dim3(NCH), dim3(BLOCK),
                     sizeof(float) * C, stream, (float*)A,
                     (const float*)decay, H, C);
}

void tl_lightning_chain(void* U, void* S, const void* decay, const void* cu_c,
                        const void* chunk_base, const void* n_chunks,
                        const void* slots, const void* pos0, int B, int H,
                        int DV, hipStream_t stream) {
  if (B <= 0) return;
  dim3 grid(B, H, (DV + BLOCK - 1) / BLOCK);
  hipLaunchKernelGGL(lightning_chain_kernel, grid, dim3(BLOCK), 0, stream,
                     (float*)U, (float*)S, (const float*)decay,
                     (const int*)cu_c, (const int*)chunk_base,
                     (const int*)n_chunks, (const int*)slots,
                     (const int*)pos0, H, DV);
}

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
