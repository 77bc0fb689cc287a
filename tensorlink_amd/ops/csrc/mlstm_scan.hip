// Matrix-memory (mLSTM) recurrence over ragged sequences (gfx950).
//
// Per head the state is a matrix S [D, V], a normaliser n [D] and a running
// log-scale m, all fp32 and resident in a slot pool between steps. For a
// token with log gates (li, lf), key k, value v and scaled query q:
//     m' = max(lf + m, li)
//     S' = exp(lf + m - m') S + exp(li - m') k v^T       (n' likewise, v = 1)
//     o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// followed, fused here, by the per-head unit-RMS norm, the norm weight and
// the sigmoid output gate. The raw gate pre-activations arrive in fp32 and
// are soft-capped in-kernel: li = cap*tanh(gi/cap),
// lf = logsigmoid(cap*tanh(gf/cap)).
//
// One block serves one (sequence, head) and walks the sequence's tokens in
// order, so the same kernel is the decode step (one token) and the exact
// sequential prefill. Column thread c < V owns column c of S in registers
// (split over DG thread groups along D); column thread c == V owns n (the
// column a constant value 1 would produce), so n . q falls out of the same
// dot product. A sequence whose cached length is zero
// starts from the zero state without reading its slot: a reused slot needs
// no clearing.

#include "common.hpp"

namespace {

template <typename T> DEVINLINE float ldv(const T* p);
template <> DEVINLINE float ldv<float>(const float* p) { return *p; }
template <> DEVINLINE float ldv<bf16>(const bf16* p) { return bf2f(*p); }
template <typename T> DEVINLINE void stv(T* p, float v);
template <> DEVINLINE void stv<float>(float* p, float v) { *p = v; }
template <> DEVINLINE void stv<bf16>(bf16* p, float v) { *p = f2bf(v); }

DEVINLINE float log_sigmoid(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// TB tokens are staged per round: their q/k rows and capped gates go to
// LDS in one sweep (one global-memory latency per round instead of one per
// token), v and the output gate wait in registers, and the per-token
// normaliser / RMS reductions of the whole round share the barriers.
// DG thread groups split the D rows of every column (DMAX/DG state
// registers per thread, DG times the waves to hide latency); their partial
// read-outs meet in LDS once per round.
template <typename T, int DMAX, int TB, int DG>
__global__ __launch_bounds__(1024) void mlstm_seq_kernel(
    const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
    int g_off,
    const float* __restrict__ gates,   // [Ttot, 2H] raw (input | forget)
    const float* __restrict__ norm_w,  // [H*V]
    float* __restrict__ S_pool,        // [slots, H, D, V]
    float* __restrict__ n_pool,        // [slots, H, D]
    float* __restrict__ m_pool,        // [slots, H]
    const int* __restrict__ cu, const int* __restrict__ slots,
    const int* __restrict__ pos0, T* __restrict__ out, int H, int D, int V,
    float cap, float qscale, float eps,
    float* __restrict__ F_pool,        // [slots, H] (summary mode) or null
    int summary) {
  // summary mode: the block runs its tokens from the EMPTY state with
  // m = -inf, writes no output, and leaves in its slot the tokens' joint
  // contribution (S, n scaled by exp(-m), m = their own maximum) plus the
  // sum of their log forget gates in F_pool: one link of the chunk chain.
  constexpr int DPER = DMAX / DG;
  extern __shared__ __align__(16) float lds[];
  const int h = blockIdx.x, b = blockIdx.y;
  const int nt = blockDim.x;
  const int nc = nt / DG;                 // column threads per group
  const int c = threadIdx.x % nc, dg = threadIdx.x / nc;
  const int nw = nc / WAVE_SIZE;
  const int lane = c & (WAVE_SIZE - 1), wave = c / WAVE_SIZE;
  // lds: q[TB][DMAX] | k[TB][DMAX] | li[TB] | lf[TB] | nq[TB] | a[TB] |
  //      b[TB] | em[TB] | m_end | red[TB][nw] | pnum[TB][DG][nc]
  // (rows padded with zeros to DMAX: the inner loop carries no d < D test
  // and reads float4; state entries beyond D stay zero)
  float* lq = lds;
  float* lk = lq + TB * DMAX;
  float* lli = lk + TB * DMAX;
  float* llf = lli + TB;
  float* lnq = llf + TB;
  float* la = lnq + TB;      // per token: exp(lf + m_prev - m), exp(li - m),
  float* lb = la + TB;       //            exp(-m); then the round's last m
  float* lem = lb + TB;
  float* lmend = lem + TB;   // [0] round's last m, [1] running sum of lf
  float* red = lmend + 2;
  float* pnum = red + TB * nw;

  const int t0 = cu[b], t1 = cu[b + 1];
  if (t0 >= t1) return;
  const int slot = slots[b];
  const bool fresh = summary || pos0[b] == 0;
  const bool is_col = c < V, is_n = c == V;
  const int d0 = dg * DPER;
  if (threadIdx.x == 0) lmend[1] = 0.f;

  float s[DPER];
  float* S_base = S_pool + ((int64_t)slot * H + h) * (int64_t)D * V;
  float* n_base = n_pool + ((int64_t)slot * H + h) * D;
#pragma unroll
  for (int i = 0; i < DPER; ++i) {
    float v = 0.f;
    if (!fresh && d0 + i < D) {
      if (is_col) v = S_base[(int64_t)(d0 + i) * V + c];
      else if (is_n) v = n_base[d0 + i];
    }
    s[i] = v;
  }
  float m = summary ? -INFINITY
                    : (fresh ? 0.f : m_pool[(int64_t)slot * H + h]);
  const float nw_c = is_col ? norm_w[h * V + c] : 0.f;

  for (int tb0 = t0; tb0 < t1; tb0 += TB) {
    const int cnt = min(TB, t1 - tb0);
    // ---- stage the round
    for (int i = threadIdx.x; i < cnt * DMAX; i += nt) {
      const int tt = i / DMAX, d = i - tt * DMAX;
      const T* row = proj + (int64_t)(tb0 + tt) * ld;
      const bool in = d < D;
      lq[i] = in ? ldv<T>(row + q_off + h * D + d) * qscale : 0.f;
      lk[i] = in ? ldv<T>(row + k_off + h * D + d) : 0.f;
    }
    if (threadIdx.x < cnt) {
      const int tt = threadIdx.x;
      const float gi = gates[(int64_t)(tb0 + tt) * 2 * H + h];
      const float gf = gates[(int64_t)(tb0 + tt) * 2 * H + H + h];
      lli[tt] = cap * tanhf(gi / cap);
      llf[tt] = log_sigmoid(cap * tanhf(gf / cap));
    }
    float vreg[TB], greg[TB], num[TB], em[TB];
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      vreg[tt] = is_n ? 1.f : 0.f;
      greg[tt] = 0.f;
      if (tt < cnt && is_col) {
        const T* row = proj + (int64_t)(tb0 + tt) * ld;
        vreg[tt] = ldv<T>(row + v_off + h * V + c);
        if (dg == 0) greg[tt] = ldv<T>(row + g_off + h * V + c);
      }
    }
    __syncthreads();
    // ---- the round's scale recurrence, once, by one thread per token
    // (thread tt replays m over tokens 0..tt: at most TB cheap steps)
    // instead of three exponentials per token in EVERY thread
    if (threadIdx.x < cnt) {
      const int tt = threadIdx.x;
      float mp = m, mc = m;          // m before / after token tt
      for (int j = 0; j <= tt; ++j) {
        mp = mc;
        mc = fmaxf(llf[j] + mc, lli[j]);
      }
      la[tt] = expf(llf[tt] + mp - mc);
      lb[tt] = expf(lli[tt] - mc);
      lem[tt] = expf(-mc);
      if (tt == cnt - 1) {
        lmend[0] = mc;
        float f = lmend[1];
        for (int j = 0; j < cnt; ++j) f += llf[j];
        lmend[1] = f;
      }
    }
    __syncthreads();
    m = lmend[0];
    // ---- the recurrence, token by token, no barrier inside
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      num[tt] = 0.f;
      em[tt] = 0.f;
      if (tt < cnt) {
        const float a = la[tt];
        const float bv = lb[tt] * vreg[tt];
        em[tt] = lem[tt];
        const float4* qq =
            reinterpret_cast<const float4*>(lq + tt * DMAX + d0);
        const float4* kk =
            reinterpret_cast<const float4*>(lk + tt * DMAX + d0);
        float ac0 = 0.f, ac1 = 0.f, ac2 = 0.f, ac3 = 0.f;
#pragma unroll
        for (int d4 = 0; d4 < DPER / 4; ++d4) {
          const float4 k4 = kk[d4], q4 = qq[d4];
          s[d4 * 4 + 0] = a * s[d4 * 4 + 0] + bv * k4.x;
          s[d4 * 4 + 1] = a * s[d4 * 4 + 1] + bv * k4.y;
          s[d4 * 4 + 2] = a * s[d4 * 4 + 2] + bv * k4.z;
          s[d4 * 4 + 3] = a * s[d4 * 4 + 3] + bv * k4.w;
          ac0 += s[d4 * 4 + 0] * q4.x;
          ac1 += s[d4 * 4 + 1] * q4.y;
          ac2 += s[d4 * 4 + 2] * q4.z;
          ac3 += s[d4 * 4 + 3] * q4.w;
        }
        num[tt] = (ac0 + ac1) + (ac2 + ac3);
      }
    }
    if (summary) {           // block-uniform: no read-out, next round
      __syncthreads();
      continue;
    }
    // ---- the groups' partial read-outs meet
    if (DG > 1) {
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) pnum[(tt * DG + dg) * nc + c] = num[tt];
      __syncthreads();
      if (dg == 0) {
#pragma unroll
        for (int tt = 0; tt < TB; ++tt) {
          float a = 0.f;
#pragma unroll
          for (int gq = 0; gq < DG; ++gq) a += pnum[(tt * DG + gq) * nc + c];
          num[tt] = a;
        }
      }
    }
    // ---- reductions of the whole round behind one barrier
    if (dg == 0) {
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) {
        const float sq = wave_reduce_sum(is_col ? num[tt] * num[tt] : 0.f);
        if (lane == 0) red[tt * nw + wave] = sq;
        if (is_n) lnq[tt] = num[tt];
      }
    }
    __syncthreads();
    if (dg == 0 && is_col) {
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) {
        if (tt < cnt) {
          float ss = 0.f;
          for (int w = 0; w < nw; ++w) ss += red[tt * nw + w];
          const float den = fmaxf(fabsf(lnq[tt]), em[tt]) + 1e-6f;
          const float o = num[tt] / den;
          const float r = rsqrtf(ss / (den * den) / (float)V + eps);
          const float sg = 1.f / (1.f + expf(-greg[tt]));
          stv<T>(out + (int64_t)(tb0 + tt) * H * V + h * V + c,
                 o * r * nw_c * sg);
        }
      }
    }
    __syncthreads();     // LDS is rewritten by the next round
  }
#pragma unroll
  for (int i = 0; i < DPER; ++i) {
    if (d0 + i < D) {
      if (is_col) S_base[(int64_t)(d0 + i) * V + c] = s[i];
      else if (is_n) n_base[d0 + i] = s[i];
    }
  }
  if (threadIdx.x == 0) {
    m_pool[(int64_t)slot * H + h] = m;
    if (summary) F_pool[(int64_t)slot * H + h] = lmend[1];
  }
}

// Chain the chunk summaries of every sequence: walking a sequence's chunks
// in order with the running state (S, n, m) — the slot's, or empty —
//     m' = max(F_c + m, m_c)
//     X' = exp(F_c + m - m') X + exp(m_c - m') dX_c          (X = S and n)
// where (dX_c, m_c, F_c) is chunk c's summary. Each chunk's entry is
// REPLACED by the state BEFORE the chunk (what the read-out pass of that
// chunk starts from); the state after the last chunk goes to the slot.
// The same m as token-by-token: max is associative. One block per
// (head, sequence); threads own elements, chunks are walked sequentially.
constexpr int CHAIN_MAX = 2048;

__global__ __launch_bounds__(256) void mlstm_chain_kernel(
    float* __restrict__ S_tmp, float* __restrict__ n_tmp,
    float* __restrict__ m_tmp, const float* __restrict__ F_tmp,
    float* __restrict__ S_pool, float* __restrict__ n_pool,
    float* __restrict__ m_pool, const int* __restrict__ chunk_base,
    const int* __restrict__ n_chunks, const int* __restrict__ slots,
    const int* __restrict__ pos0, int H, int D, int V) {
  __shared__ float ca[CHAIN_MAX], cb[CHAIN_MAX];
  const int h = blockIdx.x, b = blockIdx.y;
  const int c0 = chunk_base[b], C = n_chunks[b];
  if (C <= 0) return;
  const int slot = slots[b];
  const bool fresh = pos0[b] == 0;
  if (threadIdx.x == 0) {
    float m = fresh ? 0.f : m_pool[(int64_t)slot * H + h];
    for (int c = 0; c < C; ++c) {
      const int64_t ci = (int64_t)(c0 + c) * H + h;
      const float mc = m_tmp[ci], f = F_tmp[ci];
      const float mn = fmaxf(f + m, mc);
      ca[c] = expf(f + m - mn);
      cb[c] = expf(mc - mn);
      m_tmp[ci] = m;                 // scale before the chunk
      m = mn;
    }
    m_pool[(int64_t)slot * H + h] = m;
  }
  __syncthreads();
  const int DV = D * V;
  for (int e = threadIdx.x; e < DV + D; e += blockDim.x) {
    const bool isS = e < DV;
    float* pool = isS ? S_pool + ((int64_t)slot * H + h) * DV + e
                      : n_pool + ((int64_t)slot * H + h) * D + (e - DV);
    float x = fresh ? 0.f : *pool;
    for (int c = 0; c < C; ++c) {
      const int64_t ci = (int64_t)(c0 + c) * H + h;
      float* t = isS ? S_tmp + ci * DV + e : n_tmp + ci * D + (e - DV);
      const float d = *t;
      *t = x;
      x = ca[c] * x + cb[c] * d;
    }
    *pool = x;
  }
}

}  // namespace

extern "C" {

// returns 0 on success, 1 if the shape is outside what the kernel serves
int tl_mlstm_seq(const void* proj, int ld, int q_off, int k_off, int v_off,
                 int g_off, const void* gates, const void* norm_w, void* S,
                 void* n, void* m, const void* cu, const void* slots,
                 const void* pos0, void* out, int B, int H, int D, int V,
                 float cap, float qscale, float eps, void* F, int summary,
                 int is_f32, hipStream_t stream) {
  if (summary && !F) return 1;
  if (D > 256 || V + 1 > 1024 || B < 1) return 1;
  const int nc = ((V + 1 + WAVE_SIZE - 1) / WAVE_SIZE) * WAVE_SIZE;
  const int nw = nc / WAVE_SIZE;
  dim3 grid(H, B);
#define TL_ML_LAUNCH(TT, DM, TBB, DGG)                                       \
  do {                                                                       \
    const size_t smem = sizeof(float) * (2 * TBB * DM + 6 * TBB + 8 + TBB * nw + \
                                         (DGG > 1 ? TBB * DGG * nc : 0));    \
    hipLaunchKernelGGL((mlstm_seq_kernel<TT, DM, TBB, DGG>), grid,           \
                       dim3(nc * DGG), smem, stream, (const TT*)proj, ld,    \
                       q_off, k_off, v_off, g_off, (const float*)gates,      \
                       (const float*)norm_w, (float*)S, (float*)n,           \
                       (float*)m, (const int*)cu, (const int*)slots,         \
                       (const int*)pos0, (TT*)out, H, D, V, cap, qscale,     \
                       eps, (float*)F, summary);                             \
  } while (0)
// up to 256 column threads: four D-groups per column; wider heads keep one
// group and short rounds
#define TL_ML_D(TT)                                                \
  if (nc > 256) {                                                  \
    if (D <= 64) TL_ML_LAUNCH(TT, 64, 4, 1);                       \
    else TL_ML_LAUNCH(TT, 256, 4, 1);                              \
  } else if (D <= 32) TL_ML_LAUNCH(TT, 32, 8, 4);                  \
  else if (D <= 64) TL_ML_LAUNCH(TT, 64, 8, 4);                    \
  else if (D <= 128) TL_ML_LAUNCH(TT, 128, 8, 4);                  \
  else TL_ML_LAUNCH(TT, 256, 8, 4);
  if (is_f32) {
    TL_ML_D(float)
  } else {
    TL_ML_D(bf16)
  }
#undef TL_ML_D
#undef TL_ML_LAUNCH
  return 0;
}

// chunk_base/n_chunks/slots/pos0 are per sequence; returns 1 if a sequence
// has more chunks than the kernel's table holds
int tl_mlstm_chain(void* S_tmp, void* n_tmp, void* m_tmp, const void* F_tmp,
                   void* S, void* n, void* m, const void* chunk_base,
                   const void* n_chunks, const void* slots, const void* pos0,
                   int B, int max_chunks, int H, int D, int V,
                   hipStream_t stream) {
  if (max_chunks > CHAIN_MAX || B < 1) return 1;
  hipLaunchKernelGGL(mlstm_chain_kernel, dim3(H, B), dim3(256), 0, stream,
                     (float*)S_tmp, (float*)n_tmp, (float*)m_tmp,
                     (const float*)F_tmp, (float*)S, (float*)n, (float*)m,
                     (const int*)chunk_base, (const int*)n_chunks,
                     (const int*)slots, (const int*)pos0, H, D, V);
  return 0;
}

}  // extern "C"
