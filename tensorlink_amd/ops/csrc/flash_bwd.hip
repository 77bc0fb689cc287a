// Causal GQA flash-attention BACKWARD on gfx950 MFMA (training path).
//
// Replaces the earlier torch-SDPA composition for training attention:
// two kernels recompute P from the forward's
// saved logsumexp and produce the three gradients:
//
//   dKV kernel — grid (kv_tiles, Hkv, B): a block owns 64 keys of one
//   kv head; for every query head of the GQA group and every
//   intersecting 64-row q tile it computes (per wave = 16 keys)
//     S^T = K Q^T            P^T = exp(S^T*scale - L[q])
//     dP^T = V dO^T          dS^T = P^T (dP^T - Delta[q]) * scale
//     dV += P^T dO           dK += dS^T Q
//   with the contractions over q running through LDS round trips
//   (C-layout -> A-fragments) against tr16 panels of Q / dO — the same
//   fragment idioms as the forward (prefill_attn.hip).
//
//   dQ kernel — grid (q_tiles, Hq, B): a block owns 64 query rows; per
//   64-key tile
//     S = Q K^T   P = exp(S*scale - L)   dP = dO V^T
//     dS = P (dP - Delta) * scale        dQ += dS K
//
// Delta[b,h,i] = rowsum(dO_i * O_i) is precomputed (torch, f32).
// All accumulation in f32; inputs/outputs bf16 except lse/delta f32.

#include "common.hpp"

namespace {

constexpr int BLOCK = 256;   // 4 waves
constexpr int BT = 64;       // tile size (keys and q rows)
constexpr int PPAD = 8;

using f32x4 = __attribute__((ext_vector_type(4))) float;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int PSTRIDE = 32 * 16 + 8;

// stage a [BT][D] tile as both padded rows and tr16 panels
template <int D, bool ROWS, bool PANELS>
DEVINLINE void stage_tile(const bf16* __restrict__ src, int64_t base,
                          int64_t row_stride, int first, int limit,
                          bf16 (*rows_lds)[D + 8], bf16* pan_lds) {
  for (int i = threadIdx.x * 8; i < BT * D; i += BLOCK * 8) {
    const int row = i / D, c = i % D;
    const int idx = first + row;
    const int64_t off = base + (int64_t)min(idx, limit - 1) * row_stride + c;
    bf16x8_t val = *reinterpret_cast<const bf16x8_t*>(src + off);
    if (idx >= limit) {
#pragma unroll
      for (int j = 0; j < 8; ++j) val[j] = (__bf16)0.f;
    }
    if (ROWS)
      *reinterpret_cast<bf16x8_t*>(&rows_lds[row][c]) = val;
    if (PANELS) {
      const int pan = (row >> 5) * (D / 16) + (c >> 4);
      *reinterpret_cast<bf16x8_t*>(
          &pan_lds[pan * PSTRIDE + (row & 31) * 16 + (c & 15)]) = val;
    }
  }
}

// ------------------------------ dK / dV ------------------------------
template <int D>
__global__ __launch_bounds__(BLOCK) void attn_bwd_dkv_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k,
    const bf16* __restrict__ v, const bf16* __restrict__ dout,
    const float* __restrict__ lse, const float* __restrict__ delta,
    bf16* __restrict__ dk, bf16* __restrict__ dv, int B, int S, int Hq,
    int Hkv, float scale, int causal) {
  constexpr int KCH = D / 32;
  constexpr int ND = D / 16;
  const int kt = blockIdx.x;
  const int hkv = blockIdx.y;
  const int b = blockIdx.z;
  const int G = Hq / Hkv;
  const int k0 = kt * BT;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15;
  const int quad = lane >> 4;
  const int mykey = k0 + wave * 16 + col;   // this lane's key row (A-frag)

  __shared__ bf16 q_lds[BT][D + 8];
  __shared__ bf16 q_pan[(BT / 32) * ND * PSTRIDE];
  __shared__ bf16 do_lds[BT][D + 8];
  __shared__ bf16 do_pan[(BT / 32) * ND * PSTRIDE];
  __shared__ bf16 p_lds[4][16][BT + PPAD];   // per-wave P^T tile
  __shared__ bf16 s_lds[4][16][BT + PPAD];   // per-wave dS^T tile
  __shared__ float ld_lds[2][BT];            // L and Delta for the q tile

  // K/V fragments for this wave's 16 keys stay in registers
  bf16x8_t kfrag[KCH], vfrag[KCH];
  {
    const int safe = min(mykey, S - 1);
    const int64_t off = (((int64_t)b * S + safe) * Hkv + hkv) * D;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      kfrag[c] = *reinterpret_cast<const bf16x8_t*>(k + off + c * 32 +
                                                    quad * 8);
      vfrag[c] = *reinterpret_cast<const bf16x8_t*>(v + off + c * 32 +
                                                    quad * 8);
      if (mykey >= S) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          kfrag[c][j] = (__bf16)0.f;
          vfrag[c][j] = (__bf16)0.f;
        }
      }
    }
  }

  f32x4 dk_acc[ND], dv_acc[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) {
    dk_acc[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
    dv_acc[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  const int qt_start = causal ? (k0 / BT) : 0;
  for (int g = 0; g < G; ++g) {
    const int h = hkv * G + g;
    const int64_t qbase = ((int64_t)b * S) * Hq * D + (int64_t)h * D;
    for (int qt = qt_start; qt * BT < S; ++qt) {
      const int q0 = qt * BT;
      // ---- stage Q and dO (rows + panels), L and Delta ----
      stage_tile<D, true, true>(q, qbase, (int64_t)Hq * D, q0, S, q_lds,
                                q_pan);
      stage_tile<D, true, true>(dout, qbase, (int64_t)Hq * D, q0, S,
                                do_lds, do_pan);
      for (int i = threadIdx.x; i < BT; i += BLOCK) {
        const int row = min(q0 + i, S - 1);
        const int64_t lb = ((int64_t)b * Hq + h) * S + row;
        ld_lds[0][i] = lse[lb];
        ld_lds[1][i] = delta[lb];
      }
      __syncthreads();

      // ---- per 16-q subtile: S^T, P^T, dP^T, dS^T; accumulate ----
#pragma unroll
      for (int qs = 0; qs < BT / 16; ++qs) {
        f32x4 st = (f32x4){0.f, 0.f, 0.f, 0.f};
        f32x4 dpt = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
          bf16x8_t qb = *reinterpret_cast<const bf16x8_t*>(
              &q_lds[qs * 16 + col][c * 32 + quad * 8]);
          bf16x8_t dob = *reinterpret_cast<const bf16x8_t*>(
              &do_lds[qs * 16 + col][c * 32 + quad * 8]);
          st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kfrag[c], qb, st,
                                                       0, 0, 0);
          dpt = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfrag[c], dob,
                                                        dpt, 0, 0, 0);
        }
        // C layout: row = key (quad*4+r within wave's 16), col = q
        const int qcol = q0 + qs * 16 + col;
        const float L = ld_lds[0][qs * 16 + col];
        const float Dl = ld_lds[1][qs * 16 + col];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = k0 + wave * 16 + quad * 4 + r;
          const bool masked = (qcol >= S) || key >= S ||
                              (causal && key > qcol) || L <= -1e29f;
          const float p = masked ? 0.f : __expf(st[r] * scale - L);
          const float ds = p * (dpt[r] - Dl) * scale;
          p_lds[wave][quad * 4 + r][qs * 16 + col] = f2bf(p);
          s_lds[wave][quad * 4 + r][qs * 16 + col] = f2bf(ds);
        }
        // ---- contractions run per 32-q chunk (mfma K=32), i.e. after
        // each odd subtile; same-wave ds_write -> ds_read ordering is
        // by lgkmcnt (each wave owns its [wave] slabs) ----
        if (qs & 1) {
          const int ks32 = (qs - 1) * 16;   // start q of the 32-chunk
#pragma unroll
          for (int n = 0; n < ND; ++n) {
            bf16x8_t pa = *reinterpret_cast<const bf16x8_t*>(
                &p_lds[wave][col][ks32 + quad * 8]);
            const unsigned pan_base = (unsigned)(uintptr_t)(
                &do_pan[((ks32 >> 5) * ND + n) * PSTRIDE]);
            bf16x8_t db = (bf16x8_t)ds_read_tr16_frag(
                tr16_frag_addr(pan_base, lane));
            dv_acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                pa, db, dv_acc[n], 0, 0, 0);
            bf16x8_t sa = *reinterpret_cast<const bf16x8_t*>(
                &s_lds[wave][col][ks32 + quad * 8]);
            const unsigned qpan_base = (unsigned)(uintptr_t)(
                &q_pan[((ks32 >> 5) * ND + n) * PSTRIDE]);
            bf16x8_t qb = (bf16x8_t)ds_read_tr16_frag(
                tr16_frag_addr(qpan_base, lane));
            dk_acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                sa, qb, dk_acc[n], 0, 0, 0);
          }
        }
      }
      __syncthreads();   // tile done before next q tile restages
    }
  }

  // ---- store dK/dV: C layout row = key quad*4+r, col -> d = n*16+col
  {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = k0 + wave * 16 + quad * 4 + r;
      if (key < S) {
        const int64_t off = (((int64_t)b * S + key) * Hkv + hkv) * D;
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          dk[off + n * 16 + col] = f2bf(dk_acc[n][r]);
          dv[off + n * 16 + col] = f2bf(dv_acc[n][r]);
        }
      }
    }
  }
}

// -------------------------------- dQ ---------------------------------
template <int D>
__global__ __launch_bounds__(BLOCK) void attn_bwd_dq_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k,
    const bf16* __restrict__ v, const bf16* __restrict__ dout,
    const float* __restrict__ lse, const float* __restrict__ delta,
    bf16* __restrict__ dq, int B, int S, int Hq, int Hkv, float scale,
    int causal) {
  constexpr int KCH = D / 32;
  constexpr int ND = D / 16;
  const int qt = blockIdx.x;
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int hkv = h / (Hq / Hkv);
  const int q0 = qt * BT;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15;
  const int quad = lane >> 4;
  const int myrow = q0 + wave * 16 + col;   // this lane's q row (A-frag)

  __shared__ bf16 k_lds[BT][D + 8];
  __shared__ bf16 v_lds[BT][D + 8];
  __shared__ bf16 k_pan[(BT / 32) * ND * PSTRIDE];
  __shared__ bf16 t_lds[4][16][BT + PPAD];   // per-wave dS tile

  // Q and dO fragments for this wave's 16 rows in registers
  bf16x8_t qfrag[KCH], dofrag[KCH];
  float L, Dl;
  {
    const int safe = min(myrow, S - 1);
    const int64_t off = (((int64_t)b * S + safe) * Hq + h) * D;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      qfrag[c] = *reinterpret_cast<const bf16x8_t*>(q + off + c * 32 +
                                                    quad * 8);
      dofrag[c] = *reinterpret_cast<const bf16x8_t*>(dout + off + c * 32 +
                                                     quad * 8);
    }
  }
  // L/Delta are per C-ROW (quad*4+r); load via lane col==row trick later
  const int64_t lbase = ((int64_t)b * Hq + h) * S;

  f32x4 dq_acc[ND];
#pragma unroll
  for (int n = 0; n < ND; ++n) dq_acc[n] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int kv_end = causal ? min(S, q0 + BT) : S;
  const int64_t kbase = ((int64_t)b * S) * Hkv * D + (int64_t)hkv * D;
  for (int kt0 = 0; kt0 < kv_end; kt0 += BT) {
    stage_tile<D, true, false>(k, kbase, (int64_t)Hkv * D, kt0, S, k_lds,
                               nullptr);
    stage_tile<D, false, true>(k, kbase, (int64_t)Hkv * D, kt0, S,
                               nullptr, k_pan);
    stage_tile<D, true, false>(v, kbase, (int64_t)Hkv * D, kt0, S, v_lds,
                               nullptr);
    __syncthreads();

#pragma unroll
    for (int ks = 0; ks < BT / 16; ++ks) {
      f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
      f32x4 dp = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        bf16x8_t kb = *reinterpret_cast<const bf16x8_t*>(
            &k_lds[ks * 16 + col][c * 32 + quad * 8]);
        bf16x8_t vb = *reinterpret_cast<const bf16x8_t*>(
            &v_lds[ks * 16 + col][c * 32 + quad * 8]);
        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[c], kb, s, 0, 0,
                                                    0);
        dp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(dofrag[c], vb, dp, 0,
                                                     0, 0);
      }
      // C layout: row = q (quad*4+r), col = key
      const int kcol = kt0 + ks * 16 + col;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int qrow = q0 + wave * 16 + quad * 4 + r;
        const int safe = min(qrow, S - 1);
        const float Lr = lse[lbase + safe];
        const float Dr = delta[lbase + safe];
        const bool masked = (qrow >= S) || (kcol >= S) ||
                            (causal && kcol > qrow) || Lr <= -1e29f;
        const float p = masked ? 0.f : __expf(s[r] * scale - Lr);
        const float ds = p * (dp[r] - Dr) * scale;
        t_lds[wave][quad * 4 + r][ks * 16 + col] = f2bf(ds);
      }
      if (ks & 1) {
        const int kk32 = (ks - 1) * 16;
#pragma unroll
        for (int n = 0; n < ND; ++n) {
          bf16x8_t pa = *reinterpret_cast<const bf16x8_t*>(
              &t_lds[wave][col][kk32 + quad * 8]);
          const unsigned pan_base = (unsigned)(uintptr_t)(
              &k_pan[((kk32 >> 5) * ND + n) * PSTRIDE]);
          bf16x8_t kb = (bf16x8_t)ds_read_tr16_frag(
              tr16_frag_addr(pan_base, lane));
          dq_acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              pa, kb, dq_acc[n], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int qrow = q0 + wave * 16 + quad * 4 + r;
      if (qrow < S) {
        const int64_t off = (((int64_t)b * S + qrow) * Hq + h) * D;
#pragma unroll
        for (int n = 0; n < ND; ++n)
          dq[off + n * 16 + col] = f2bf(dq_acc[n][r]);
      }
    }
  }
}

}  // namespace

extern "C" {

void tl_attn_bwd(const void* q, const void* k, const void* v,
                 const void* dout, const void* lse, const void* delta,
                 void* dq, void* dk, void* dv, int B, int S, int Hq,
                 int Hkv, int D, float scale, int causal,
                 hipStream_t stream) {
  dim3 block(BLOCK);
  dim3 gkv((S + BT - 1) / BT, Hkv, B);
  dim3 gq((S + BT - 1) / BT, Hq, B);
#define L2(KER, GRID, ...)                                                  \
  hipLaunchKernelGGL(KER, GRID, block, 0, stream, (const bf16*)q,           \
                     (const bf16*)k, (const bf16*)v, (const bf16*)dout,     \
                     (const float*)lse, (const float*)delta, __VA_ARGS__,   \
                     B, S, Hq, Hkv, scale, causal)
  if (D == 128) {
    L2((attn_bwd_dkv_kernel<128>), gkv, (bf16*)dk, (bf16*)dv);
    L2((attn_bwd_dq_kernel<128>), gq, (bf16*)dq);
  } else if (D == 64) {
    L2((attn_bwd_dkv_kernel<64>), gkv, (bf16*)dk, (bf16*)dv);
    L2((attn_bwd_dq_kernel<64>), gq, (bf16*)dq);
  }
#undef L2
}

}  // extern "C"
