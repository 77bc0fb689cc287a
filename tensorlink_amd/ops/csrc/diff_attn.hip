// Differential attention over a paged KV pool, ragged batches (gfx950).
//
// Every query head carries TWO softmax maps over the same values: the
// query row is [map 1 | map 2] (2*D), so is the key row, and
//     o = a1 - lambda * a2,   a_i = softmax(q_i . k_i * scale) V
// followed, fused here, by the unit-RMS norm over the head's V values and
// the constant (1 - diff). Keys and values live in page pools
// [pages, G, PAGE, 2D] / [pages, G, PAGE, V] addressed through each
// sequence's block-table row; a layer may read another layer's pools
// (cross-layer KV sharing), which only changes the pointers passed in.
//
// tl_kv_append scatters the new tokens' key/value rows into their pages.
// tl_diff_attn_rows serves one query token per block row: each of the four
// waves strides over 64-key tiles (one key per lane for the two score dot
// products, one value column per lane for P.V), keeps online-softmax
// statistics for both maps, and the waves merge through LDS. It is exact
// for any query position, so it is both the decode kernel and the plain
// prefill path; scores, softmax weights and the accumulators are fp32.

#include "common.hpp"

namespace {

constexpr int PAGE = 128;
static_assert(PAGE % WAVE_SIZE == 0, "a key tile must not straddle pages");
constexpr int NWAVE = 4;
constexpr int BLOCK = NWAVE * WAVE_SIZE;

template <typename T> DEVINLINE float ldv(const T* p);
template <> DEVINLINE float ldv<float>(const float* p) { return *p; }
template <> DEVINLINE float ldv<bf16>(const bf16* p) { return bf2f(*p); }
template <typename T> DEVINLINE void stv(T* p, float v);
template <> DEVINLINE void stv<float>(float* p, float v) { *p = v; }
template <> DEVINLINE void stv<bf16>(bf16* p, float v) { *p = f2bf(v); }

template <typename T>
__global__ __launch_bounds__(256) void kv_append_kernel(
    const T* __restrict__ proj, int ld, int k_off, int v_off,
    T* __restrict__ kpool, T* __restrict__ vpool,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int P, int G, int DK, int V) {
  const int t = blockIdx.x;
  const int seq = tok_seq[t], pos = tok_pos[t];
  const int page = table[(int64_t)seq * P + pos / PAGE];
  const int r = pos % PAGE;
  const T* row = proj + (int64_t)t * ld;
  for (int i = threadIdx.x; i < G * DK; i += blockDim.x) {
    const int g = i / DK, e = i % DK;
    kpool[(((int64_t)page * G + g) * PAGE + r) * DK + e] = row[k_off + i];
  }
  for (int i = threadIdx.x; i < G * V; i += blockDim.x) {
    const int g = i / V, e = i % V;
    vpool[(((int64_t)page * G + g) * PAGE + r) * V + e] = row[v_off + i];
  }
}

template <typename T, int VR>
__global__ __launch_bounds__(BLOCK) void diff_attn_row_kernel(
    const T* __restrict__ q, int ldq, int q_off,
    const T* __restrict__ kpool, const T* __restrict__ vpool,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ table, int P, const float* __restrict__ lam_p,
    T* __restrict__ out, float* __restrict__ part, int H, int G, int D,
    int V, float scale, float diff, float eps) {
  extern __shared__ float lds[];
  const int t = blockIdx.x, h = blockIdx.y;
  const int ns = gridDim.z, z = blockIdx.z;   // key splits (flash-decode)
  const int g = h / (H / G);
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  const int DK = 2 * D;
  // lds: qs[2D] | stat[NWAVE][4] | acc[NWAVE][2][V] | red[NWAVE]
  float* qs = lds;
  float* stat = lds + DK;
  float* accs = stat + NWAVE * 4;
  float* red = accs + NWAVE * 2 * V;

  const int seq = tok_seq[t], pos = tok_pos[t];
  const int* tab = table + (int64_t)seq * P;
  for (int i = threadIdx.x; i < DK; i += BLOCK)
    qs[i] = ldv<T>(q + (int64_t)t * ldq + q_off + h * DK + i) * scale;
  __syncthreads();

  float m1 = -INFINITY, m2 = -INFINITY, l1 = 0.f, l2 = 0.f;
  float a1[VR], a2[VR];
#pragma unroll
  for (int r = 0; r < VR; ++r) a1[r] = a2[r] = 0.f;

  const bool vec8 = (D % 8) == 0 && sizeof(T) == 2;
  for (int j0 = (z * NWAVE + wave) * WAVE_SIZE; j0 <= pos;
       j0 += ns * NWAVE * WAVE_SIZE) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s1 = -INFINITY, s2 = -INFINITY;
    // a 64-key tile starts at a multiple of 64 and so lies inside ONE
    // 128-position page: one table lookup per tile, and the value loads
    // below do not wait on per-key lookups
    const int64_t tile_row =
        ((int64_t)tab[j0 / PAGE] * G + g) * PAGE + (j0 % PAGE);
    if (valid) {
      const T* kr = kpool + (tile_row + lane) * DK;
      float x1 = 0.f, x2 = 0.f;
      if (vec8) {
        // 16-byte loads of 8 bf16 (rows are 16-byte aligned when D % 8 == 0)
        const bf16x8* k8 = reinterpret_cast<const bf16x8*>(kr);
        for (int d8 = 0; d8 < D / 8; ++d8) {
          const bf16x8 a = k8[d8], b = k8[D / 8 + d8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            x1 += qs[d8 * 8 + e] * bf2f(a.v[e]);
            x2 += qs[D + d8 * 8 + e] * bf2f(b.v[e]);
          }
        }
      } else {
        for (int d = 0; d < D; ++d) {
          x1 += qs[d] * ldv<T>(kr + d);
          x2 += qs[D + d] * ldv<T>(kr + D + d);
        }
      }
      s1 = x1;
      s2 = x2;
    }
    const float n1 = fmaxf(m1, wave_reduce_max(s1));
    const float n2 = fmaxf(m2, wave_reduce_max(s2));
    const float c1 = expf(m1 - n1), c2 = expf(m2 - n2);
    const float p1 = valid ? expf(s1 - n1) : 0.f;
    const float p2 = valid ? expf(s2 - n2) : 0.f;
    l1 = l1 * c1 + wave_reduce_sum(p1);
    l2 = l2 * c2 + wave_reduce_sum(p2);
    m1 = n1;
    m2 = n2;
#pragma unroll
    for (int r = 0; r < VR; ++r) {
      a1[r] *= c1;
      a2[r] *= c2;
    }
    const int cnt = min(WAVE_SIZE, pos + 1 - j0);
    const T* vtile = vpool + tile_row * V;
#pragma unroll 8
    for (int jj = 0; jj < cnt; ++jj) {
      const float w1 = __shfl(p1, jj, WAVE_SIZE);
      const float w2 = __shfl(p2, jj, WAVE_SIZE);
      const T* vr = vtile + (int64_t)jj * V;
#pragma unroll
      for (int r = 0; r < VR; ++r) {
        const int c = lane + r * WAVE_SIZE;
        if (c < V) {
          const float vv = ldv<T>(vr + c);
          a1[r] += w1 * vv;
          a2[r] += w2 * vv;
        }
      }
    }
  }
  if (lane == 0) {
    stat[wave * 4 + 0] = m1;
    stat[wave * 4 + 1] = l1;
    stat[wave * 4 + 2] = m2;
    stat[wave * 4 + 3] = l2;
  }
#pragma unroll
  for (int r = 0; r < VR; ++r) {
    const int c = lane + r * WAVE_SIZE;
    if (c < V) {
      accs[(wave * 2 + 0) * V + c] = a1[r];
      accs[(wave * 2 + 1) * V + c] = a2[r];
    }
  }
  __syncthreads();
  float M1 = -INFINITY, M2 = -INFINITY;
  for (int w = 0; w < NWAVE; ++w) {
    M1 = fmaxf(M1, stat[w * 4 + 0]);
    M2 = fmaxf(M2, stat[w * 4 + 2]);
  }
  float f1[NWAVE], f2[NWAVE], L1 = 0.f, L2 = 0.f;
  for (int w = 0; w < NWAVE; ++w) {
    const float mm1 = stat[w * 4 + 0], mm2 = stat[w * 4 + 2];
    f1[w] = (mm1 == -INFINITY) ? 0.f : expf(mm1 - M1);
    f2[w] = (mm2 == -INFINITY) ? 0.f : expf(mm2 - M2);
    L1 += f1[w] * stat[w * 4 + 1];
    L2 += f2[w] * stat[w * 4 + 3];
  }
  if (ns > 1) {
    // partial of this key split: (M1, L1, M2, L2 | A1[V] | A2[V]); the
    // merge kernel finishes the row
    float* pr = part + (((int64_t)t * H + h) * ns + z) * (4 + 2 * V);
    if (threadIdx.x == 0) {
      pr[0] = M1;
      pr[1] = L1;
      pr[2] = M2;
      pr[3] = L2;
    }
    for (int c = threadIdx.x; c < V; c += BLOCK) {
      float A1 = 0.f, A2 = 0.f;
      for (int w = 0; w < NWAVE; ++w) {
        A1 += f1[w] * accs[(w * 2 + 0) * V + c];
        A2 += f2[w] * accs[(w * 2 + 1) * V + c];
      }
      pr[4 + c] = A1;
      pr[4 + V + c] = A2;
    }
    return;
  }
  const float lam = lam_p[0];
  // at most VR*64/BLOCK columns per thread; VR <= 8 -> 2
  float o[2];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = threadIdx.x + r * BLOCK;
    o[r] = 0.f;
    if (c < V) {
      float A1 = 0.f, A2 = 0.f;
      for (int w = 0; w < NWAVE; ++w) {
        A1 += f1[w] * accs[(w * 2 + 0) * V + c];
        A2 += f2[w] * accs[(w * 2 + 1) * V + c];
      }
      o[r] = A1 / L1 - lam * (A2 / L2);
      ss += o[r] * o[r];
    }
  }
  ss = wave_reduce_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  float tot = 0.f;
  for (int w = 0; w < NWAVE; ++w) tot += red[w];
  const float rn = rsqrtf(tot / (float)V + eps) * (1.f - diff);
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = threadIdx.x + r * BLOCK;
    if (c < V) stv<T>(out + ((int64_t)t * H + h) * V + c, o[r] * rn);
  }
}

// Merge the key splits of one (token, head): rescale every split's sums to
// the common maximum, then lambda, unit RMS and (1 - diff) as in the row
// kernel. One block of 256 threads per row; V <= 512.
template <typename T>
__global__ __launch_bounds__(BLOCK) void diff_attn_merge_kernel(
    const float* __restrict__ part, const float* __restrict__ lam_p,
    T* __restrict__ out, int ns, int V, float diff, float eps) {
  __shared__ float red[NWAVE];
  const int64_t row = blockIdx.x;
  const float* pr = part + row * ns * (4 + 2 * V);
  const int lane = threadIdx.x & (WAVE_SIZE - 1);
  const int wave = threadIdx.x / WAVE_SIZE;
  float M1 = -INFINITY, M2 = -INFINITY;
  for (int z = 0; z < ns; ++z) {
    M1 = fmaxf(M1, pr[z * (4 + 2 * V) + 0]);
    M2 = fmaxf(M2, pr[z * (4 + 2 * V) + 2]);
  }
  float L1 = 0.f, L2 = 0.f;
  float o[2] = {0.f, 0.f}, a1[2] = {0.f, 0.f}, a2[2] = {0.f, 0.f};
  for (int z = 0; z < ns; ++z) {
    const float* pz = pr + z * (4 + 2 * V);
    const float f1 = pz[0] == -INFINITY ? 0.f : expf(pz[0] - M1);
    const float f2 = pz[2] == -INFINITY ? 0.f : expf(pz[2] - M2);
    L1 += f1 * pz[1];
    L2 += f2 * pz[3];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int c = threadIdx.x + r * BLOCK;
      if (c < V) {
        a1[r] += f1 * pz[4 + c];
        a2[r] += f2 * pz[4 + V + c];
      }
    }
  }
  const float lam = lam_p[0];
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = threadIdx.x + r * BLOCK;
    if (c < V) {
      o[r] = a1[r] / L1 - lam * (a2[r] / L2);
      ss += o[r] * o[r];
    }
  }
  ss = wave_reduce_sum(ss);
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  float tot = 0.f;
  for (int w = 0; w < NWAVE; ++w) tot += red[w];
  const float rn = rsqrtf(tot / (float)V + eps) * (1.f - diff);
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = threadIdx.x + r * BLOCK;
    if (c < V) stv<T>(out + row * V + c, o[r] * rn);
  }
}

}  // namespace

extern "C" {

void tl_kv_append(const void* proj, int ld, int k_off, int v_off, void* kpool,
                  void* vpool, const void* tok_seq, const void* tok_pos,
                  const void* table, int P, int T, int G, int DK, int V,
                  int is_f32, hipStream_t stream) {
  if (T <= 0) return;
  dim3 grid(T), block(256);
  if (is_f32)
    hipLaunchKernelGGL(kv_append_kernel<float>, grid, block, 0, stream,
                       (const float*)proj, ld, k_off, v_off, (float*)kpool,
                       (float*)vpool, (const int*)tok_seq,
                       (const int*)tok_pos, (const int*)table, P, G, DK, V);
  else
    hipLaunchKernelGGL(kv_append_kernel<bf16>, grid, block, 0, stream,
                       (const bf16*)proj, ld, k_off, v_off, (bf16*)kpool,
                       (bf16*)vpool, (const int*)tok_seq,
                       (const int*)tok_pos, (const int*)table, P, G, DK, V);
}

// returns 0 on success, 1 if the shape is outside what the kernel serves
int tl_diff_attn_rows(const void* q, int ldq, int q_off, const void* kpool,
                      const void* vpool, const void* tok_seq,
                      const void* tok_pos, const void* table, int P,
                      const void* lam, void* out, void* part, int ns, int T,
                      int H, int G, int D, int V, float scale, float diff,
                      float eps, int is_f32, hipStream_t stream) {
  if (V > 512 || T <= 0 || H % G != 0 || ns < 1 || (ns > 1 && !part))
    return 1;
  const size_t smem =
      sizeof(float) * (2 * D + NWAVE * 4 + NWAVE * 2 * V + NWAVE);
  if (smem > 64 * 1024) return 1;
  dim3 grid(T, H, ns), block(BLOCK);
  const int vr = (V + WAVE_SIZE - 1) / WAVE_SIZE;
#define TL_DA_LAUNCH(TT, VRR)                                                \
  hipLaunchKernelGGL((diff_attn_row_kernel<TT, VRR>), grid, block, smem,     \
                     stream, (const TT*)q, ldq, q_off, (const TT*)kpool,     \
                     (const TT*)vpool, (const int*)tok_seq,                  \
                     (const int*)tok_pos, (const int*)table, P,              \
                     (const float*)lam, (TT*)out, (float*)part, H, G, D, V,  \
                     scale, diff, eps)
#define TL_DA_V(TT)                          \
  if (vr <= 1) TL_DA_LAUNCH(TT, 1);          \
  else if (vr <= 2) TL_DA_LAUNCH(TT, 2);     \
  else if (vr <= 4) TL_DA_LAUNCH(TT, 4);     \
  else TL_DA_LAUNCH(TT, 8);
  if (is_f32) {
    TL_DA_V(float)
  } else {
    TL_DA_V(bf16)
  }
#undef TL_DA_V
#undef TL_DA_LAUNCH
  if (ns > 1) {
    dim3 mgrid(T * H);
    if (is_f32)
      hipLaunchKernelGGL(diff_attn_merge_kernel<float>, mgrid, block, 0,
                         stream, (const float*)part, (const float*)lam,
                         (float*)out, ns, V, diff, eps);
    else
      hipLaunchKernelGGL(diff_attn_merge_kernel<bf16>, mgrid, block, 0,
                         stream, (const float*)part, (const float*)lam,
                         (bf16*)out, ns, V, diff, eps);
  }
  return 0;
}

}  // extern "C"
