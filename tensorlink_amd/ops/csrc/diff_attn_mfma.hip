// Differential attention, prompt portions, on MFMA (gfx950, bf16).
//
// One block = 64 consecutive query tokens of one sequence (16 per wave) and
// one query head; keys/values come from the paged pool through the
// sequence's block-table row. Both softmax maps of the head are carried
// side by side (two score tiles, two running max/sum pairs, two output
// accumulators over the SAME value tile).
//
// The products are arranged so that nothing is transposed through LDS:
//   S^T[key][q] = K Q^T      A = K rows (16 keys x 32 d), B = Q^T
//   O^T[v][q]  += V^T P^T    A = V^T (16 v x 32 keys),    B = P^T
// With mfma_f32_16x16x32_bf16 a lane's C fragment of S^T holds 4 keys of
// query (lane & 15); two 16-key tiles give the 8 values that are exactly
// its B fragment of P^T for a 32-key step (the k-slot order is a free
// choice as long as A agrees: slot (quad, j) = key 16*(j/4) + 4*quad + j%4,
// which V^T reads from LDS as two 8-byte loads). Query (lane & 15) is also
// the column of the O^T fragment, so online-softmax rescaling is lane-local.
// Scores, softmax statistics and accumulators are fp32; P is rounded to
// bf16 only as the MFMA operand.
//
// Only V is staged through LDS (transposed, [V][64 keys]); K fragments are
// 16-byte global loads that the four waves of a block share through L1/L2.

#include "common.hpp"

namespace {

constexpr int PAGE = 128;
constexpr int QT = 64;           // queries per block
constexpr int KT = 64;           // keys per round
constexpr int VLD = KT + 8;      // LDS row stride of V^T (bf16 elements)

using f32x4 = __attribute__((ext_vector_type(4))) float;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));

DEVINLINE bf16x8_t zero8() {
  bf16x8_t z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

DEVINLINE float quad_max(float x) {
  x = fmaxf(x, __shfl_xor(x, 16, WAVE_SIZE));
  return fmaxf(x, __shfl_xor(x, 32, WAVE_SIZE));
}
DEVINLINE float quad_sum(float x) {
  x += __shfl_xor(x, 16, WAVE_SIZE);
  return x + __shfl_xor(x, 32, WAVE_SIZE);
}

template <int DC, int VTMAX>
__global__ __launch_bounds__(256) void diff_attn_tile_kernel(
    const bf16* __restrict__ q, int ldq, int q_off,
    const bf16* __restrict__ kpool, const bf16* __restrict__ vpool,
    const int* __restrict__ tiles,   // [n][4]: seq, first token, count, pos
    const int* __restrict__ table, int P, const float* __restrict__ lam_p,
    bf16* __restrict__ out, int H, int G, int D, int V, float scale,
    float diff, float eps) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16* vt_lds = reinterpret_cast<bf16*>(smem_raw);     // [V][VLD]

  const int h = blockIdx.y;
  const int g = h / (H / G);
  const int seq = tiles[blockIdx.x * 4 + 0];
  const int tok0 = tiles[blockIdx.x * 4 + 1];
  const int n = tiles[blockIdx.x * 4 + 2];
  const int p0 = tiles[blockIdx.x * 4 + 3];
  const int* tab = table + (int64_t)seq * P;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, quad = lane >> 4;
  const int DK = 2 * D;
  const int nvt = V / 16;

  const int qi = wave * 16 + col;
  const bool q_valid = qi < n;
  const int qc = min(qi, n - 1);
  const int tok = tok0 + qc;
  const int qpos = p0 + qc;
  const int k_end = p0 + n;                             // keys of the block
  const int wave_last = p0 + min(wave * 16 + 15, n - 1);
  const bool wave_on = wave * 16 < n;

  // query fragments: Q[q = col][d = c*32 + quad*8 ..]
  bf16x8_t qf[2][DC];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      const int d = c * 32 + quad * 8;
      qf[mp][c] = (d < D)
          ? *reinterpret_cast<const bf16x8_t*>(
                q + (int64_t)tok * ldq + q_off + h * DK + mp * D + d)
          : zero8();
    }

  f32x4 acc[2][VTMAX];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int vt = 0; vt < VTMAX; ++vt)
      acc[mp][vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float mrun[2] = {-INFINITY, -INFINITY}, lrun[2] = {0.f, 0.f};

  const int vchunks = V / 8;                // 16-byte chunks per value row
  for (int k0 = 0; k0 < k_end; k0 += KT) {
    __syncthreads();                        // previous round's reads done
    for (int i = threadIdx.x; i < KT * vchunks; i += 256) {
      const int kk = i / vchunks, c8 = i - kk * vchunks;
      const int j = min(k0 + kk, k_end - 1);
      const int page = tab[j / PAGE];
      const bf16x8 v8 = *reinterpret_cast<const bf16x8*>(
          vpool + (((int64_t)page * G + g) * PAGE + (j % PAGE)) * V + c8 * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) vt_lds[(c8 * 8 + e) * VLD + kk] = v8.v[e];
    }
    __syncthreads();
    if (!wave_on || k0 > wave_last) continue;   // wave-uniform

#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int kb = k0 + sub * 32;
      if (kb > wave_last) break;                // wave-uniform
      // ---- S^T for two 16-key tiles, both maps
      f32x4 st[2][2];
#pragma unroll
      for (int t16 = 0; t16 < 2; ++t16) {
        const int j = min(kb + t16 * 16 + col, k_end - 1);
        const int page = tab[j / PAGE];
        const bf16* kr =
            kpool + (((int64_t)page * G + g) * PAGE + (j % PAGE)) * DK;
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
          f32x4 sacc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < DC; ++c) {
            const int d = c * 32 + quad * 8;
            const bf16x8_t kf =
                (d < D) ? *reinterpret_cast<const bf16x8_t*>(kr + mp * D + d)
                        : zero8();
            sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[mp][c],
                                                           sacc, 0, 0, 0);
          }
          st[mp][t16] = sacc;
        }
      }
      // ---- online softmax per map (query = col; keys over r and quads)
      bf16x8_t pf[2];
#pragma unroll
      for (int mp = 0; mp < 2; ++mp) {
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int t16 = 0; t16 < 2; ++t16)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = kb + t16 * 16 + quad * 4 + r;
            const float s =
                key <= qpos ? st[mp][t16][r] * scale : -INFINITY;
            sv[t16 * 4 + r] = s;
            mx = fmaxf(mx, s);
          }
        mx = quad_max(mx);
        const float m_new = fmaxf(mrun[mp], mx);
        const float corr = __expf(mrun[mp] - m_new);
        mrun[mp] = m_new;
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __expf(sv[i] - m_new);
          ps += p;
          pf[mp][i] = (__bf16)p;
        }
        lrun[mp] = lrun[mp] * corr + ps;
#pragma unroll
        for (int vt = 0; vt < VTMAX; ++vt)
          if (vt < nvt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mp][vt][r] *= corr;
          }
      }
      // ---- O^T += V^T P^T
#pragma unroll
      for (int vt = 0; vt < VTMAX; ++vt)
        if (vt < nvt) {
          const bf16* vr = vt_lds + (vt * 16 + col) * VLD + sub * 32 + quad * 4;
          const bf16x4_t lo = *reinterpret_cast<const bf16x4_t*>(vr);
          const bf16x4_t hi = *reinterpret_cast<const bf16x4_t*>(vr + 16);
          bf16x8_t vf;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            vf[i] = lo[i];
            vf[4 + i] = hi[i];
          }
          acc[0][vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              vf, pf[0], acc[0][vt], 0, 0, 0);
          acc[1][vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              vf, pf[1], acc[1][vt], 0, 0, 0);
        }
    }
  }

  if (!wave_on) return;
  const float l1 = quad_sum(lrun[0]), l2 = quad_sum(lrun[1]);
  const float lam = lam_p[0];
  const float i1 = 1.f / l1, i2 = lam / l2;
  float ss = 0.f;
#pragma unroll
  for (int vt = 0; vt < VTMAX; ++vt)
    if (vt < nvt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float o = acc[0][vt][r] * i1 - acc[1][vt][r] * i2;
        acc[0][vt][r] = o;
        ss += o * o;
      }
    }
  ss = quad_sum(ss);
  const float rn = rsqrtf(ss / (float)V + eps) * (1.f - diff);
  if (q_valid) {
    bf16* orow = out + ((int64_t)tok * H + h) * V;
#pragma unroll
    for (int vt = 0; vt < VTMAX; ++vt)
      if (vt < nvt) {
        bf16x4_t o4;
#pragma unroll
        for (int r = 0; r < 4; ++r) o4[r] = (__bf16)(acc[0][vt][r] * rn);
        *reinterpret_cast<bf16x4_t*>(orow + vt * 16 + quad * 4) = o4;
      }
  }
}

}  // namespace

extern "C" {

// returns 0 on success, 1 if the shape is outside what this kernel serves
// (the caller then uses the row kernel)
int tl_diff_attn_tiles(const void* q, int ldq, int q_off, const void* kpool,
                       const void* vpool, const void* tiles, int n_tiles,
                       const void* table, int P, const void* lam, void* out,
                       int H, int G, int D, int V, float scale, float diff,
                       float eps, hipStream_t stream) {
  if (D % 8 != 0 || D > 128 || V % 16 != 0 || V > 256 || H % G != 0 ||
      ldq % 8 != 0 || q_off % 8 != 0 || n_tiles <= 0)
    return 1;
  const size_t smem = sizeof(bf16) * (size_t)V * VLD;
  dim3 grid(n_tiles, H), block(256);
  const int dc = (D + 31) / 32, nvt = V / 16;
#define TL_DT_LAUNCH(DCC, VTM)                                               \
  hipLaunchKernelGGL((diff_attn_tile_kernel<DCC, VTM>), grid, block, smem,   \
                     stream, (const bf16*)q, ldq, q_off, (const bf16*)kpool, \
                     (const bf16*)vpool, (const int*)tiles,                  \
                     (const int*)table, P, (const float*)lam, (bf16*)out, H, \
                     G, D, V, scale, diff, eps)
#define TL_DT_V(DCC)                          \
  if (nvt <= 4) TL_DT_LAUNCH(DCC, 4);         \
  else if (nvt <= 8) TL_DT_LAUNCH(DCC, 8);    \
  else TL_DT_LAUNCH(DCC, 16);
  if (dc <= 1) { TL_DT_V(1) }
  else if (dc <= 2) { TL_DT_V(2) }
  else { TL_DT_V(4) }
#undef TL_DT_V
#undef TL_DT_LAUNCH
  return 0;
}

}  // extern "C"
