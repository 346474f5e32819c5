// Latent attention on the matrix cores (bf16 activations, fp32 scores / softmax / sums).
// Same inputs and outputs as latent_attn.hip: queries arrive in latent space (qa = W_uk^T q), a score
// is scale * qa . c_j over the cached latents of the causal sliding window, the softmax
// denominator also holds exp(sink_h) (no sink given: an ordinary softmax), and the result is
// sum_j p_j c_j per head.
//
// Every head attends to the same latents, so (row, head) pairs are the M dimension: one
// wavefront owns 16 pairs -- RW consecutive rows of one sequence portion x HS head slots --
// and walks the union of their windows 32 keys at a time:
//   S^T[16 keys x 16 pairs] = C[16 keys x rank] . Q^T      rank/32 x mfma_16x16x32_bf16, twice
//   online softmax in the accumulator layout (a pair's 32 scores sit in 4 lanes x 8 values)
//   O[16 pairs x rank]     += P[16 pairs x 32 keys] . C     rank/16 x mfma_16x16x32_bf16
// The latents of a tile are loaded once from the paged pool as A operands of S^T and written
// transposed to LDS, where the second product reads them as B operands.  One wavefront per
// workgroup, no cross-wave synchronisation.  `units` (int32 x 2: first row, rows) lists the
// row groups; a group never spans two portions.
#include "common.h"
using namespace sm;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define LM_LDK 36   // keys per transposed row in LDS (32 + padding), in bf16: rows 72 bytes apart
                    // spread the four key-index slices over different banks

template <int NT2>  // rank padded to NT2 * 32
__global__ void __launch_bounds__(64)
latent_attn_mfma_k(const bf16* __restrict__ qa, long sqh, long sqr, const bf16* __restrict__ cache,
                   const int* __restrict__ bt, int max_pages, const int* __restrict__ row_ent,
                   const int* __restrict__ pos, const int* __restrict__ units,
                   const float* __restrict__ sink, float scale, int win, bf16* __restrict__ out,
                   long soh, long sor, int H, int rank, int page, int HS, int splits,
                   float* __restrict__ part) {
  constexpr int RP = NT2 * 32;       // padded rank
  constexpr int NT = NT2 * 2;        // 16-wide output column tiles
  constexpr int LDQ = RP + 8;
  extern __shared__ unsigned short lds[];
  unsigned short* sQ = lds;                 // [16 pairs][LDQ]
  unsigned short* sC = lds + 16 * LDQ;      // [RP][LM_LDK]  latents of the tile, transposed
  const int lane = threadIdx.x, n16 = lane & 15, quad = lane >> 4;
  const int r0 = units[2 * blockIdx.x], nr = units[2 * blockIdx.x + 1];
  const int h0 = blockIdx.y * HS;
  // this lane's pair (as a column of S^T and a row of P)
  const int prow = n16 / HS, ph = h0 + n16 % HS;
  const bool pvalid = prow < nr && ph < H;
  const int ppos = pvalid ? pos[r0 + prow] : -1;
  const int* pages = bt + (size_t)row_ent[r0] * max_pages;
  int j_lo = max(0, pos[r0] - win + 1), j_hi = pos[r0 + nr - 1];
  if (splits > 1) {
    // this block takes one run of 32-key tiles of the window; partial results go to `part`
    int tiles = (j_hi - j_lo) / 32 + 1;
    int per = (tiles + splits - 1) / splits;
    int lo = j_lo + blockIdx.z * per * 32;
    j_hi = min(j_hi, lo + per * 32 - 1);
    j_lo = lo;
  }
  const bool first = blockIdx.z == 0;   // the sink is counted by the first run only

  // queries -> LDS (zero rows for unused pairs, zero columns beyond the rank)
  for (int idx = lane; idx < 16 * (RP / 8); idx += 64) {
    int m = idx / (RP / 8), c8 = (idx % (RP / 8)) * 8;
    int mr = m / HS, mh = h0 + m % HS;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (mr < nr && mh < H && c8 < rank)
      v = *(const uint4*)(qa + (size_t)mh * sqh + (size_t)(r0 + mr) * sqr + c8);
    *(uint4*)(sQ + m * LDQ + c8) = v;
  }
  __syncthreads();

  const bool sunk = first && sink != nullptr;   // no sink: an ordinary softmax
  float m_run = pvalid ? (sunk ? sink[ph] : -1e30f) : 0.0f;
  float l_part = (pvalid && quad == 0 && sunk) ? 1.0f : 0.0f;
  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int j0 = j_lo; j0 <= j_hi; j0 += 32) {
    f32x4 s[2];
#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
      int j = j0 + sub * 16 + n16;   // the key this lane loads
      const bf16* crow = nullptr;
      if (j <= j_hi) crow = cache + ((size_t)pages[j / page] * page + (j % page)) * rank;
      uint4 cf[NT2];
#pragma unroll
      for (int kk = 0; kk < NT2; kk++) {
        int c8 = kk * 32 + quad * 8;
        cf[kk] = (crow && c8 < rank) ? *(const uint4*)(crow + c8) : make_uint4(0, 0, 0, 0);
      }
      f32x4 sa = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NT2; kk++) {
        bf16x8 a = __builtin_bit_cast(bf16x8, cf[kk]);
        bf16x8 b = __builtin_bit_cast(bf16x8, *(const uint4*)(sQ + n16 * LDQ + kk * 32 + quad * 8));
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, sa, 0, 0, 0);
      }
      s[sub] = sa;
      // transposed copy for the second product: sC[rank index][key in tile]
#pragma unroll
      for (int kk = 0; kk < NT2; kk++) {
        unsigned int w[4] = {cf[kk].x, cf[kk].y, cf[kk].z, cf[kk].w};
        unsigned short* dst = sC + (kk * 32 + quad * 8) * LM_LDK + sub * 16 + n16;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          dst[(2 * i) * LM_LDK] = (unsigned short)(w[i] & 0xffffu);
          dst[(2 * i + 1) * LM_LDK] = (unsigned short)(w[i] >> 16);
        }
      }
    }
    // scores of pair n16: keys j0 + sub*16 + quad*4 + i
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 2; sub++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        int j = j0 + sub * 16 + quad * 4 + i;
        bool ok = pvalid && j <= ppos && j > ppos - win;
        float v = ok ? s[sub][i] * scale : -INFINITY;
        sv[sub * 4 + i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    float m_new = fmaxf(m_run, tmax);
    float alpha = expf(m_run - m_new);
    m_run = m_new;
    float psum = 0.0f;
    bf16x8 pf;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float p = expf(sv[i] - m_new);   // exp(-inf) = 0 for masked keys
      psum += p;
      pf[i] = (__bf16)p;
    }
    l_part = l_part * alpha + psum;
    // the accumulators hold pairs quad*4 + i: fetch their rescale factors
    bool any = __any(alpha != 1.0f);
    if (any) {
      float al[4];
#pragma unroll
      for (int i = 0; i < 4; i++) al[i] = __shfl(alpha, quad * 4 + i, 64);
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[t][i] *= al[i];
    }
    __syncthreads();   // the tile's latents are in LDS
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const unsigned short* src = sC + (t * 16 + n16) * LM_LDK + quad * 4;
      uint2 lo = *(const uint2*)src, hi = *(const uint2*)(src + 16);
      bf16x8 b = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, b, acc[t], 0, 0, 0);
    }
    __syncthreads();   // before the next tile overwrites sC
  }
  float l = l_part + __shfl_xor(l_part, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (splits > 1) {
    // partial record of this run: [pair][RP + 2] = unnormalised sums, running max, running sum
    float* rec = part + (((size_t)blockIdx.x * gridDim.y + blockIdx.y) * splits + blockIdx.z) *
                            16 * (RP + 2);
    if (quad == 0) {
      rec[n16 * (RP + 2) + RP] = m_run;
      rec[n16 * (RP + 2) + RP + 1] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int t = 0; t < NT; t++) rec[(quad * 4 + i) * (RP + 2) + t * 16 + n16] = acc[t][i];
    return;
  }
  float inv[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float li = __shfl(l, quad * 4 + i, 64);
    inv[i] = li > 0.0f ? 1.0f / li : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int m = quad * 4 + i;
    int mr = m / HS, mh = h0 + m % HS;
    if (mr < nr && mh < H) {
      bf16* o = out + (size_t)mh * soh + (size_t)(r0 + mr) * sor;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        int c = t * 16 + n16;
        if (c < rank) o[c] = __float2bfloat16(acc[t][i] * inv[i]);
      }
    }
  }
}

// Merges the runs of a split window: out = sum_z e^(m_z - M) acc_z / sum_z e^(m_z - M) l_z.
// One block per (unit, head group, pair); the weights of the runs are formed once in LDS.
__global__ void latent_attn_merge_k(const float* __restrict__ part, const int* __restrict__ units,
                                    bf16* __restrict__ out, long soh, long sor, int H, int rank,
                                    int HS, int splits, int RP) {
  __shared__ float sw[65];
  const int r0 = units[2 * blockIdx.x], nr = units[2 * blockIdx.x + 1];
  const int m = blockIdx.z;
  const int mr = m / HS, mh = blockIdx.y * HS + m % HS;
  if (mr >= nr || mh >= H) return;
  const float* rec = part + ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * splits * 16 * (RP + 2) +
                     (size_t)m * (RP + 2);
  const size_t zs = (size_t)16 * (RP + 2);   // stride between runs
  if (threadIdx.x < 64) {
    int z = threadIdx.x;
    float mz = z < splits ? rec[z * zs + RP] : -INFINITY;
    float M = mz;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
    float w = z < splits ? expf(mz - M) : 0.0f;
    float d = z < splits ? w * rec[z * zs + RP + 1] : 0.0f;
    d = wave_sum(d);
    sw[z] = w;
    if (z == 0) sw[64] = d > 0.0f ? 1.0f / d : 0.0f;
  }
  __syncthreads();
  float inv = sw[64];
  bf16* o = out + (size_t)mh * soh + (size_t)(r0 + mr) * sor;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) {
    float num = 0.0f;
    for (int z = 0; z < splits; z++) num += sw[z] * rec[z * zs + c];
    o[c] = __float2bfloat16(num * inv);
  }
}

// the P operand's key order: slot quad*8 + i holds key quad*4 + i (i < 4) or 16 + quad*4 + i - 4;
// the B operand above reads sC with the same order (src and src + 16).

extern "C" {

// 1 when the matrix-core kernel serves this shape (bf16 only): rank a multiple of 8, <= 512
int p2p_sm_latent_attn_mfma_ok(int H, int rank) { return H >= 1 && rank >= 8 && rank % 8 == 0 && rank <= 512; }

// rows one wavefront takes for H heads
int p2p_sm_latent_attn_mfma_rows(int H) {
  int hs = 1;
  while (hs < H && hs < 16) hs *= 2;
  return 16 / hs;
}

// floats of workspace for `splits` runs per window (0 when splits <= 1)
long p2p_sm_latent_attn_mfma_ws(int U, int H, int rank, int splits) {
  if (splits <= 1) return 0;
  int HS = 16 / p2p_sm_latent_attn_mfma_rows(H);
  int n = (rank + 31) / 32;
  int N = n <= 1 ? 1 : n <= 2 ? 2 : n <= 4 ? 4 : n <= 8 ? 8 : 16;
  return (long)U * ((H + HS - 1) / HS) * splits * 16 * (N * 32 + 2);
}

// splits > 1: each window is cut into that many runs of key tiles (decode steps: few rows,
// long windows), partial results in `part` (p2p_sm_latent_attn_mfma_ws floats), then merged
int p2p_sm_latent_attn_mfma(const void* qa, long sqh, long sqr, const void* cache, const int* bt,
                            int max_pages, const int* row_ent, const int* pos, const int* units,
                            int U, const float* sink, float scale, int win, void* out, long soh,
                            long sor, int H, int rank, int page, int splits, float* part,
                            hipStream_t st) {
  if (U <= 0) return 0;
  if (!p2p_sm_latent_attn_mfma_ok(H, rank) || win < 1) return (int)hipErrorInvalidValue;
  if (splits < 1 || splits > 64 || (splits > 1 && !part)) return (int)hipErrorInvalidValue;
  int HS = 16 / p2p_sm_latent_attn_mfma_rows(H);
  dim3 grid(U, (H + HS - 1) / HS, splits), block(64);
#define LM(N)                                                                                  \
  do {                                                                                         \
    size_t shm = (size_t)(16 * (N * 32 + 8) + N * 32 * LM_LDK) * 2;                            \
    hipLaunchKernelGGL((latent_attn_mfma_k<N>), grid, block, shm, st, (const bf16*)qa, sqh,    \
                       sqr, (const bf16*)cache, bt, max_pages, row_ent, pos, units, sink,      \
                       scale, win, (bf16*)out, soh, sor, H, rank, page, HS, splits, part);     \
    if (splits > 1)                                                                            \
      hipLaunchKernelGGL(latent_attn_merge_k, dim3(grid.x, grid.y, 16), dim3(128), 0, st, part, \
                         units, (bf16*)out, soh, sor, H, rank, HS, splits, N * 32);            \
  } while (0)
  int n = (rank + 31) / 32;
  if (n <= 1) LM(1);
  else if (n <= 2) LM(2);
  else if (n <= 4) LM(4);
  else if (n <= 8) LM(8);
  else LM(16);
#undef LM
  return (int)hipGetLastError();
}

}  // extern "C"
