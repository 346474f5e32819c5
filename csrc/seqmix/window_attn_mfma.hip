// Grouped-query window attention on the matrix cores (bf16 activations, fp32 scores / softmax /
// sums).  Same inputs and outputs as window_attn_k: pool row = [k of G heads | v of G heads],
// query head h reads key/value head h / (H/G), causal sliding window of `win` keys, softmax
// denominator with one more term exp(sink_h); optionally scores capped by cap * tanh(s / cap),
// a per-head penalty r1_h * ln(1 + r2_h * distance) taken off them, and every head's result
// multiplied by sigmoid(gate[row, head]).
//
// The query heads of one key/value head attend to the same keys, so (row, head) pairs are the M
// dimension: one wavefront owns 16 pairs -- RW consecutive rows of one sequence portion x HS
// head slots of one key/value head -- and walks the union of their windows 32 keys at a time:
//   S^T[16 keys x 16 pairs] = K[16 keys x D] . Q^T        D/32 x mfma_16x16x32_bf16, twice
//   online softmax in the accumulator layout (a pair's 32 scores sit in 4 lanes x 8 values)
//   O[16 pairs x V]        += P[16 pairs x 32 keys] . V    V/16 x mfma_16x16x32_bf16
// Keys go from the paged pool straight into A fragments; values are written transposed to LDS,
// where the second product reads them as B fragments.  One wavefront per workgroup.  `units`
// (int32 x 2: first row, rows) lists the row groups; a group never spans two portions.  Few
// row groups with long windows (decode) cut every window into runs of key tiles over
// gridDim.z; a second kernel merges the runs.
#include "common.h"
using namespace sm;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// cap * tanh(v / cap) and ln(1 + x) on the hardware's exp2 / log2 / reciprocal units: a prompt
// evaluates them once per (query, key, head), where the library forms (tanhf, log1pf) cost more
// than the matrix products; their error is far below the bf16 rounding of the probabilities.
__device__ __forceinline__ float fast_tanh(float x) {
  float t = __expf(2.0f * x);                       // inf for large x -> 1, 0 for small x -> -1
  return 1.0f - 2.0f * __frcp_rn(t + 1.0f);
}

#define WM_LDK 36   // keys per transposed value row in LDS (32 + padding), in bf16

template <int NK, int NV2>  // D padded to NK * 32, V padded to NV2 * 32
__global__ void __launch_bounds__(64)
window_attn_mfma_k(const bf16* __restrict__ q, int ldq, const bf16* __restrict__ pool,
                   const int* __restrict__ bt, int max_pages, const int* __restrict__ row_ent,
                   const int* __restrict__ pos, const int* __restrict__ units,
                   const float* __restrict__ sink, float scale, int win, bf16* __restrict__ out,
                   int ldo, int H, int G, int D, int V, int page, int HS, int splits,
                   float* __restrict__ part, float out_scale, float cap,
                   const float* __restrict__ r1, const float* __restrict__ r2,
                   const bf16* __restrict__ gate, int ldg) {
  constexpr int DP = NK * 32;        // padded key size
  constexpr int VP = NV2 * 32;       // padded value size
  constexpr int NT = NV2 * 2;        // 16-wide output column tiles
  constexpr int LDQ = DP + 8;
  extern __shared__ unsigned short lds[];
  unsigned short* sQ = lds;                 // [16 pairs][LDQ]
  unsigned short* sV = lds + 16 * LDQ;      // [VP][WM_LDK]  values of the tile, transposed
  const int lane = threadIdx.x, n16 = lane & 15, quad = lane >> 4;
  const int r0 = units[2 * blockIdx.x], nr = units[2 * blockIdx.x + 1];
  const int HG = H / G, hblocks = (HG + HS - 1) / HS;
  const int g = blockIdx.y / hblocks, hb0 = (blockIdx.y % hblocks) * HS;   // head slots hb0 ..
  const int ldpool = G * (D + V);
  const bf16* kbase = pool + (size_t)g * D;
  const bf16* vbase = pool + (size_t)G * D + (size_t)g * V;
  // this lane's pair (as a column of S^T and a row of P)
  const int prow = n16 / HS, phs = hb0 + n16 % HS;
  const bool pvalid = prow < nr && phs < HG;
  const int ph = g * HG + phs;
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

  // queries -> LDS (zero rows for unused pairs, zero columns beyond D)
  for (int idx = lane; idx < 16 * (DP / 8); idx += 64) {
    int m = idx / (DP / 8), c8 = (idx % (DP / 8)) * 8;
    int mr = m / HS, ms = hb0 + m % HS;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (mr < nr && ms < HG && c8 < D)
      v = *(const uint4*)(q + (size_t)(r0 + mr) * ldq + (size_t)(g * HG + ms) * D + c8);
    *(uint4*)(sQ + m * LDQ + c8) = v;
  }
  __syncthreads();

  const float pr1 = (pvalid && r1) ? r1[ph] : 0.0f, pr2 = (pvalid && r1) ? r2[ph] : 0.0f;
  const float inv_cap = cap > 0.0f ? 1.0f / cap : 0.0f;
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
      size_t tok = 0;
      bool have = j <= j_hi;
      if (have) tok = ((size_t)pages[j / page] * page + (j % page)) * ldpool;
      uint4 kf[NK], vf[NV2];
#pragma unroll
      for (int kk = 0; kk < NK; kk++) {
        int c8 = kk * 32 + quad * 8;
        kf[kk] = (have && c8 < D) ? *(const uint4*)(kbase + tok + c8) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int kk = 0; kk < NV2; kk++) {
        int c8 = kk * 32 + quad * 8;
        vf[kk] = (have && c8 < V) ? *(const uint4*)(vbase + tok + c8) : make_uint4(0, 0, 0, 0);
      }
      f32x4 sa = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NK; kk++) {
        if (kk * 32 < D) {
          bf16x8 a = __builtin_bit_cast(bf16x8, kf[kk]);
          bf16x8 b = __builtin_bit_cast(bf16x8, *(const uint4*)(sQ + n16 * LDQ + kk * 32 + quad * 8));
          sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, sa, 0, 0, 0);
        }
      }
      s[sub] = sa;
      // transposed copy for the second product: sV[value channel][key in tile]
#pragma unroll
      for (int kk = 0; kk < NV2; kk++) {
        unsigned int w[4] = {vf[kk].x, vf[kk].y, vf[kk].z, vf[kk].w};
        unsigned short* dst = sV + (kk * 32 + quad * 8) * WM_LDK + sub * 16 + n16;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          dst[(2 * i) * WM_LDK] = (unsigned short)(w[i] & 0xffffu);
          dst[(2 * i + 1) * WM_LDK] = (unsigned short)(w[i] >> 16);
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
        bool ok = pvalid && j <= ppos && j > ppos - win && j <= j_hi;
        float v = -INFINITY;
        if (ok) {
          v = s[sub][i] * scale;
          if (cap > 0.0f) v = cap * fast_tanh(v * inv_cap);
          if (r1) v -= pr1 * __logf(1.0f + pr2 * (float)(ppos - j));
        }
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
    __syncthreads();   // the tile's values are in LDS
#pragma unroll
    for (int t = 0; t < NT; t++) {
      if (t * 16 < V) {
        const unsigned short* src = sV + (t * 16 + n16) * WM_LDK + quad * 4;
        uint2 lo = *(const uint2*)src, hi = *(const uint2*)(src + 16);
        bf16x8 b = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, b, acc[t], 0, 0, 0);
      }
    }
    __syncthreads();   // before the next tile overwrites sV
  }
  float l = l_part + __shfl_xor(l_part, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (splits > 1) {
    // partial record of this run: [pair][VP + 2] = unnormalised sums, running max, running sum
    float* rec = part + (((size_t)blockIdx.x * gridDim.y + blockIdx.y) * splits + blockIdx.z) *
                            16 * (VP + 2);
    if (quad == 0) {
      rec[n16 * (VP + 2) + VP] = m_run;
      rec[n16 * (VP + 2) + VP + 1] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int t = 0; t < NT; t++) rec[(quad * 4 + i) * (VP + 2) + t * 16 + n16] = acc[t][i];
    return;
  }
  float inv[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    float li = __shfl(l, quad * 4 + i, 64);
    inv[i] = li > 0.0f ? out_scale / li : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int m = quad * 4 + i;
    int mr = m / HS, ms = hb0 + m % HS;
    if (mr < nr && ms < HG) {
      bf16* o = out + (size_t)(r0 + mr) * ldo + (size_t)(g * HG + ms) * V;
      float gv = inv[i];
      if (gate) gv *= sigmoidf_(__bfloat162float(gate[(size_t)(r0 + mr) * ldg + g * HG + ms]));
#pragma unroll
      for (int t = 0; t < NT; t++) {
        int c = t * 16 + n16;
        if (c < V) o[c] = __float2bfloat16(acc[t][i] * gv);
      }
    }
  }
}

// Merges the runs of a split window: out = sum_z e^(m_z - M) acc_z / sum_z e^(m_z - M) l_z.
// One block per (unit, head block, pair); the weights of the runs are formed once in LDS.
__global__ void window_attn_merge_k(const float* __restrict__ part, const int* __restrict__ units,
                                    bf16* __restrict__ out, int ldo, int H, int G, int V, int HS,
                                    int splits, int VP, float out_scale,
                                    const bf16* __restrict__ gate, int ldg) {
  __shared__ float sw[65];
  const int r0 = units[2 * blockIdx.x], nr = units[2 * blockIdx.x + 1];
  const int HG = H / G, hblocks = (HG + HS - 1) / HS;
  const int g = blockIdx.y / hblocks, hb0 = (blockIdx.y % hblocks) * HS;
  const int m = blockIdx.z;
  const int mr = m / HS, ms = hb0 + m % HS;
  if (mr >= nr || ms >= HG) return;
  const float* rec = part + ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * splits * 16 * (VP + 2) +
                     (size_t)m * (VP + 2);
  const size_t zs = (size_t)16 * (VP + 2);   // stride between runs
  if (threadIdx.x < 64) {
    int z = threadIdx.x;
    float mz = z < splits ? rec[z * zs + VP] : -INFINITY;
    float M = mz;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
    float w = z < splits ? expf(mz - M) : 0.0f;
    float d = z < splits ? w * rec[z * zs + VP + 1] : 0.0f;
    d = wave_sum(d);
    sw[z] = w;
    if (z == 0) {
      float gv = gate ? sigmoidf_(__bfloat162float(gate[(size_t)(r0 + mr) * ldg + g * HG + ms])) : 1.0f;
      sw[64] = d > 0.0f ? out_scale * gv / d : 0.0f;
    }
  }
  __syncthreads();
  float inv = sw[64];
  bf16* o = out + (size_t)(r0 + mr) * ldo + (size_t)(g * HG + ms) * V;
  for (int c = threadIdx.x; c < V; c += blockDim.x) {
    float num = 0.0f;
    for (int z = 0; z < splits; z++) num += sw[z] * rec[z * zs + c];
    o[c] = __float2bfloat16(num * inv);
  }
}

static int pad32(int n) {   // 32-channel steps the kernel is instantiated for
  int s = (n + 31) / 32;
  return s <= 1 ? 1 : s <= 2 ? 2 : s <= 4 ? 4 : 8;
}

static int head_slots(int HG) {
  int hs = 1;
  while (hs < HG && hs < 16) hs *= 2;
  return hs;
}

extern "C" {

// floats of workspace for `splits` runs per window (0 when splits <= 1)
long p2p_sm_window_attn_mfma_ws(int U, int H, int G, int V, int splits) {
  if (splits <= 1 || G < 1 || H % G) return 0;
  int HG = H / G, HS = head_slots(HG);
  return (long)U * G * ((HG + HS - 1) / HS) * splits * 16 * (pad32(V) * 32 + 2);
}

int p2p_sm_window_attn_mfma(const void* q, int ldq, const void* pool, const int* bt,
                            int max_pages, const int* row_ent, const int* pos, const int* units,
                            int U, const float* sink, float scale, int win, void* out, int ldo,
                            int H, int G, int D, int V, int page, int splits, float* part,
                            float out_scale, float cap, const float* r1, const float* r2,
                            const void* gate, int ldg, hipStream_t st) {
  if (U <= 0) return 0;
  if (H < 1 || G < 1 || H % G || D < 8 || D > 256 || D % 8 || V < 8 || V > 256 || V % 8 ||
      win < 1 || ldq % 8 || (r1 && !r2) || cap < 0.0f)
    return (int)hipErrorInvalidValue;
  if (splits < 1 || splits > 64 || (splits > 1 && !part)) return (int)hipErrorInvalidValue;
  int HG = H / G, HS = head_slots(HG);
  dim3 grid(U, G * ((HG + HS - 1) / HS), splits), block(64);
  int nk = pad32(D), nv = pad32(V);
#define WM(NKK, NVV)                                                                           \
  do {                                                                                         \
    size_t shm = (size_t)(16 * (NKK * 32 + 8) + NVV * 32 * WM_LDK) * 2;                        \
    hipLaunchKernelGGL((window_attn_mfma_k<NKK, NVV>), grid, block, shm, st, (const bf16*)q,   \
                       ldq, (const bf16*)pool, bt, max_pages, row_ent, pos, units, sink,       \
                       scale, win, (bf16*)out, ldo, H, G, D, V, page, HS, splits, part,        \
                       out_scale, cap, r1, r2, (const bf16*)gate, ldg);                        \
    if (splits > 1)                                                                            \
      hipLaunchKernelGGL(window_attn_merge_k, dim3(grid.x, grid.y, 16), dim3(128), 0, st,      \
                         part, units, (bf16*)out, ldo, H, G, V, HS, splits, NVV * 32,          \
                         out_scale, (const bf16*)gate, ldg);                                   \
  } while (0)
#define WMV(NKK)                 \
  do {                           \
    if (nv == 1) WM(NKK, 1);     \
    else if (nv == 2) WM(NKK, 2);\
    else if (nv == 4) WM(NKK, 4);\
    else WM(NKK, 8);             \
  } while (0)
  if (nk == 1) WMV(1);
  else if (nk == 2) WMV(2);
  else if (nk == 4) WMV(4);
  else WMV(8);
#undef WMV
#undef WM
  return (int)hipGetLastError();
}

}  // extern "C"
