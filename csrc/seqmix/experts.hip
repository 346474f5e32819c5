// Mixture of experts: the router with a group-limited choice, the expert matrix products over
// the routed rows, and the weighted sum of the chosen experts' outputs.
//
// group_route_k: z = h . Wr^T in fp32, s = sigmoid(z) or softmax(z) over all experts; the
// choice is made on s plus an optional per-expert correction.  The E experts are cut into
// `groups` contiguous blocks of equal size; a block is ranked by the sum of its two best choice
// scores or by its best one; experts outside the `keep` best blocks are struck out, and the
// `top` largest remaining choice scores win (ties: the lower index).  The weights are the
// winners' s (without the correction), not rescaled.  A token r routed to its k-th expert is slot
// r * top + k; every expert gets the list of its slots (cnt / rows).
//
// expert_gemm: for expert e and each of its slots s: out[s] = x[s / x_div] . W_e^T.  Rows are
// gathered through the slot lists, so only experts with rows read their weights.  bf16 runs
// on the matrix cores (a 16 x 64 tile with K split over the wavefronts for decode-sized steps,
// an LDS-staged 128 x 128 tile for prompts); fp32 and odd shapes run a tiled FMA kernel.  A
// slot's result does not depend on which other slots share its tile.
#include "common.h"
using namespace sm;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// best (value, index) over the wavefront; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(v, o, 64);
    int oi = __shfl_xor(i, o, 64);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// orders one wavefront's LDS writes before its later reads by other lanes
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// score: 0 sigmoid, 1 softmax over all experts, 2 the logits themselves for the choice and the
// softmax over the chosen logits as weights.  bias (optional, [E]): added to the logits.
// corr (optional, [E]): added to the scores for the choice only.  gscore: a group is ranked by 0 the sum of its two best choice scores, 1 its
// best choice score.
template <typename T>
__global__ void __launch_bounds__(256)
group_route_k(const T* __restrict__ h, int ldh, const float* __restrict__ wr, int W, int E, int top,
              int groups, int keep, int score, const float* __restrict__ corr, int gscore,
              int* __restrict__ ids, float* __restrict__ wts, int* __restrict__ cnt,
              int* __restrict__ rows, int ldr, const float* __restrict__ bias) {
  extern __shared__ float smem[];
  float* sh = smem;          // [W] the row in fp32
  float* ss = sh + W;        // [E] scores (the weights of the chosen)
  float* sc = ss + E;        // [E] choice scores; -inf marks "cannot be chosen (any more)"
  float* sgs = sc + E;       // [groups] group scores
  float* stop = sgs + groups;   // [top] the chosen logits (score 2)
  const int r = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int i = threadIdx.x; i < W; i += blockDim.x) sh[i] = ldf(h, (size_t)r * ldh + i);
  __syncthreads();
  // four experts at a time per wavefront: their weight loads are independent and go out together
  for (int e0 = wave * 4; e0 < E; e0 += nw * 4) {
    const float* w0 = wr + (size_t)e0 * W;
    const float* w1 = wr + (size_t)min(e0 + 1, E - 1) * W;
    const float* w2 = wr + (size_t)min(e0 + 2, E - 1) * W;
    const float* w3 = wr + (size_t)min(e0 + 3, E - 1) * W;
    float d0 = 0.0f, d1 = 0.0f, d2 = 0.0f, d3 = 0.0f;
#pragma unroll 4
    for (int i = lane; i < W; i += 64) {
      float x = sh[i];
      d0 += x * w0[i];
      d1 += x * w1[i];
      d2 += x * w2[i];
      d3 += x * w3[i];
    }
    d0 = wave_sum(d0);
    d1 = wave_sum(d1);
    d2 = wave_sum(d2);
    d3 = wave_sum(d3);
    if (lane == 0) {
      if (bias) {
        d0 += bias[e0];
        d1 += bias[min(e0 + 1, E - 1)];
        d2 += bias[min(e0 + 2, E - 1)];
        d3 += bias[min(e0 + 3, E - 1)];
      }
      ss[e0] = score ? d0 : sigmoidf_(d0);
      if (e0 + 1 < E) ss[e0 + 1] = score ? d1 : sigmoidf_(d1);
      if (e0 + 2 < E) ss[e0 + 2] = score ? d2 : sigmoidf_(d2);
      if (e0 + 3 < E) ss[e0 + 3] = score ? d3 : sigmoidf_(d3);
    }
  }
  __syncthreads();
  if (wave != 0) return;
  if (score == 1) {   // softmax over all experts
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, ss[e]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float sum = 0.0f;
    for (int e = lane; e < E; e += 64) {
      float v = expf(ss[e] - mx);
      ss[e] = v;
      sum += v;
    }
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) ss[e] = ss[e] / sum;
  }
  for (int e = lane; e < E; e += 64) sc[e] = corr ? ss[e] + corr[e] : ss[e];
  wave_sync();
  const int per = E / groups;
  if (keep < groups) {
    for (int g = lane; g < groups; g += 64) {
      float b1 = -INFINITY, b2 = -INFINITY;   // top-2 of the block
      for (int i = 0; i < per; i++) {
        float v = sc[g * per + i];
        if (v > b1) { b2 = b1; b1 = v; }
        else if (v > b2) b2 = v;
      }
      sgs[g] = b1 + ((per > 1 && gscore == 0) ? b2 : 0.0f);
    }
    wave_sync();
    // keep the best groups: pick `keep` times, then strike out the experts of the others
    for (int k = 0; k < keep; k++) {
      float bv = -INFINITY;
      int bi = 1 << 30;
      for (int g = lane; g < groups; g += 64) {
        float v = sgs[g];
        if (v > bv) { bv = v; bi = g; }     // ascending g: the first of equals stays
      }
      wave_argmax(bv, bi);
      if (lane == 0) sgs[bi] = -INFINITY;   // marks "kept"
      wave_sync();
    }
    for (int e = lane; e < E; e += 64)
      if (sgs[e / per] != -INFINITY) sc[e] = -INFINITY;
    wave_sync();
  }
  for (int k = 0; k < top; k++) {
    float bv = -INFINITY;
    int bi = 1 << 30;
    for (int e = lane; e < E; e += 64) {
      float v = sc[e];
      if (v > bv) { bv = v; bi = e; }
    }
    wave_argmax(bv, bi);
    if (lane == 0) {
      sc[bi] = -INFINITY;
      int slot = r * top + k;
      ids[slot] = bi;
      if (score == 2) stop[k] = ss[bi];
      else wts[slot] = ss[bi];
      int at = atomicAdd(&cnt[bi], 1);
      rows[(size_t)bi * ldr + at] = slot;
    }
    wave_sync();
  }
  if (score == 2) {   // the weights become the softmax over the chosen logits
    float mx = -INFINITY;
    for (int k = lane; k < top; k += 64) mx = fmaxf(mx, stop[k]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float sum = 0.0f;
    for (int k = lane; k < top; k += 64) sum += expf(stop[k] - mx);
    sum = wave_sum(sum);
    for (int k = lane; k < top; k += 64) wts[r * top + k] = expf(stop[k] - mx) / sum;
  }
}

// The grid is sized for the most row tiles the experts can have together (total slots / BM + E,
// since every expert wastes at most one partial tile), one-dimensional, and workgroups go to
// the 8 XCDs round-robin: block L runs on XCD L % 8.  A block counts the row tiles that exist,
// deals them to the XCDs in contiguous runs of equal length (XCD j takes row tiles
// j*pr .. j*pr+pr-1 and all column tiles, so its L2 holds the gathered rows of few experts and
// streams only those experts' weights), and finds its expert and first slot by walking the
// counts.  Blocks beyond the tiles that exist leave at once.
__device__ __forceinline__ bool find_tile(const int* __restrict__ cnt, int E, int BM,
                                          int row_tiles_pad, int& e, int& m0, int& nt) {
  // every wavefront does this for itself, 64 experts at a time: one vector load of the counts,
  // sums and prefix sums by lane shuffles (a scalar walk over the counts costs a dependent
  // load per expert, which a decode-sized launch cannot hide)
  const int lane = threadIdx.x & 63;
  int total = 0;
  for (int base = 0; base < E; base += 64) {
    int i = base + lane;
    int n = i < E ? (cnt[i] + BM - 1) / BM : 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) n += __shfl_xor(n, o, 64);
    total += n;
  }
  const int j = blockIdx.x & 7, s = blockIdx.x >> 3, pm = row_tiles_pad >> 3;
  const int pr = (total + 7) >> 3, li = s % pm;
  nt = s / pm;
  const int t = j * pr + li;
  if (li >= pr || t >= total) return false;
  int acc = 0, fe = -1, fm = 0;
  for (int base = 0; base < E && fe < 0; base += 64) {
    int i = base + lane;
    int n = i < E ? (cnt[i] + BM - 1) / BM : 0;
    int incl = n;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      int v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    int excl = acc + incl - n;
    bool hit = n > 0 && t >= excl && t < excl + n;
    unsigned long long mask = __ballot(hit);
    if (mask) {
      int src = __ffsll((long long)mask) - 1;
      fe = base + src;
      fm = (t - __shfl(excl, src, 64)) * BM;
    }
    acc += __shfl(incl, 63, 64);
  }
  // the same for every lane: keep them in scalar registers
  e = __builtin_amdgcn_readfirstlane(fe);
  m0 = __builtin_amdgcn_readfirstlane(fm);
  return e >= 0;
}

// Epilogue with the experts' activation (epi = 1): the weight rows of the first product are
// stored as 16 gate rows, their 16 up rows, the next 16 gate rows, ..., so a thread that holds
// output column c of a 16-column tile holds the matching up value in the next tile, and
//   y = min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, -limit, limit) + 1)
// is written to column (tile / 2) * 16 + c of an output half as wide.
__device__ __forceinline__ float expert_act(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoidf_(alpha * g) * (u + 1.0f);
}

// epi = 3: the same layout with y = g * sigmoid(g) * u
__device__ __forceinline__ float glu_epi(float g, float u, int epi, float limit, float alpha) {
  return epi == 3 ? g * sigmoidf_(g) * u : expert_act(g, u, limit, alpha);
}

// epi = 2: an ungated unit, every product passes relu(.)^2; epi = 0: the products themselves
__device__ __forceinline__ float plain_epi(float v, int epi) {
  if (epi == 2) {
    v = fmaxf(v, 0.0f);
    v *= v;
  }
  return v;
}

// bf16 on the matrix cores, few slots per expert (decode-sized steps): a block takes 16 slots x
// 64 output columns of one expert and its four wavefronts split K among themselves, so the
// chain of dependent loads is a quarter as long; each wavefront walks its share in steps of 32
// with one A fragment (the gathered rows) and four B fragments (16 weight rows each), the next
// step's fragments in flight while the current products run; the four partial tiles are
// added through LDS.
__global__ void __launch_bounds__(256)
expert_gemm_mfma_k(const bf16* __restrict__ x, int ldx, int x_div, const bf16* __restrict__ w,
                   const int* __restrict__ cnt, const int* __restrict__ rows, int ldr,
                   bf16* __restrict__ out, int ldo, int N, int K, int E, int TMP, int epi, float limit, float alpha) {
  __shared__ f32x4 red[3][4][64];
  int e, m0, nt;
  if (!find_tile(cnt, E, 16, TMP, e, m0, nt)) return;
  const int c = cnt[e], n0 = nt * 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n16 = lane & 15, quad = lane >> 4;
  const int mi = m0 + n16;
  const int slot = mi < c ? rows[(size_t)e * ldr + mi] : -1;
  const int kq = ((K + 127) / 128) * 32;          // K per wavefront, a multiple of 32
  const int kb = wave * kq, ke = min(K, kb + kq);
  const bf16* xa = slot >= 0 ? x + (size_t)(slot / x_div) * ldx + quad * 8 : nullptr;
  const bf16* wb[4];
#pragma unroll
  for (int t = 0; t < 4; t++) {
    int n = n0 + t * 16 + n16;
    wb[t] = n < N ? w + ((size_t)e * N + n) * K + quad * 8 : nullptr;
  }
  f32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const uint4 zero = make_uint4(0, 0, 0, 0);
  uint4 av, bv[4];
  {
    bool kin = kb + quad * 8 < ke;                 // K is a multiple of 8
    av = (xa && kin) ? *(const uint4*)(xa + kb) : zero;
#pragma unroll
    for (int t = 0; t < 4; t++) bv[t] = (wb[t] && kin) ? *(const uint4*)(wb[t] + kb) : zero;
  }
  for (int k0 = kb; k0 < ke; k0 += 32) {
    const int kn = k0 + 32;
    const bool nin = kn + quad * 8 < ke;
    uint4 an = (xa && nin) ? *(const uint4*)(xa + kn) : zero;
    uint4 bn[4];
#pragma unroll
    for (int t = 0; t < 4; t++) bn[t] = (wb[t] && nin) ? *(const uint4*)(wb[t] + kn) : zero;
    bf16x8 af = __builtin_bit_cast(bf16x8, av);
#pragma unroll
    for (int t = 0; t < 4; t++)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, __builtin_bit_cast(bf16x8, bv[t]),
                                                        acc[t], 0, 0, 0);
    av = an;
#pragma unroll
    for (int t = 0; t < 4; t++) bv[t] = bn[t];
  }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < 4; t++) red[wave - 1][t][lane] = acc[t];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int u = 0; u < 3; u++) acc[t] += red[u][t][lane];
  // accumulator layout: row quad*4 + i of the 16 slots, column n16 of each tile
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int so = __shfl(slot, quad * 4 + i, 64);
    if (so < 0) continue;
    if (epi == 1 || epi == 3) {
#pragma unroll
      for (int t = 0; t < 4; t += 2) {
        int n = n0 + t * 16;
        if (n + 16 + n16 < N)
          out[(size_t)so * ldo + n / 2 + n16] =
              __float2bfloat16(glu_epi(acc[t][i], acc[t + 1][i], epi, limit, alpha));
      }
      continue;
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
      int n = n0 + t * 16 + n16;
      if (n < N) out[(size_t)so * ldo + n] = __float2bfloat16(plain_epi(acc[t][i], epi));
    }
  }
}

// Many slots per expert (prompts): a block of 2 x 2 wavefronts takes 128 slots x 128 columns
// and walks K in steps of 64.  The gathered A rows and the weight rows of a step are loaded
// with coalesced 16-byte reads (8 threads per row), kept in registers while the previous step
// computes, and handed to the MFMA fragments through LDS (rows 144 bytes apart).  Each
// wavefront owns 64 x 64 (4 x 4 MFMA tiles); 16-slot tiles beyond the expert's count are skipped.
#define EB_LD 72   // bf16 per LDS row: 64 + 8
__global__ void __launch_bounds__(256)
expert_gemm_mfma_big_k(const bf16* __restrict__ x, int ldx, int x_div, const bf16* __restrict__ w,
                       const int* __restrict__ cnt, const int* __restrict__ rows, int ldr,
                       bf16* __restrict__ out, int ldo, int N, int K, int E, int TMP, int epi, float limit, float alpha) {
  __shared__ __align__(16) unsigned short sA[128 * EB_LD];
  __shared__ __align__(16) unsigned short sB[128 * EB_LD];
  __shared__ int sslot[128];
  int e, m0, nt;
  if (!find_tile(cnt, E, 128, TMP, e, m0, nt)) return;
  const int c = cnt[e], n0 = nt * 128;
  const int tid = threadIdx.x;
  if (tid < 128) sslot[tid] = m0 + tid < c ? rows[(size_t)e * ldr + m0 + tid] : -1;
  __syncthreads();
  const int lane = tid & 63, wave = tid >> 6, n16 = lane & 15, quad = lane >> 4;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int nmt = max(0, min(4, (c - (m0 + wm) + 15) / 16));
  // this thread's four 16-byte pieces of the A and B tiles: row = (tid + 256 u) / 8
  const int c8 = (tid & 7) * 8;
  const bf16* pa[4];
  const bf16* pb[4];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    int r = (tid + 256 * u) >> 3;
    int sl = sslot[r];
    pa[u] = sl >= 0 ? x + (size_t)(sl / x_div) * ldx + c8 : nullptr;
    pb[u] = n0 + r < N ? w + ((size_t)e * N + n0 + r) * K + c8 : nullptr;
  }
  const uint4 zero = make_uint4(0, 0, 0, 0);
  uint4 ra[4], rb[4];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    bool kin = c8 < K;
    ra[u] = (pa[u] && kin) ? *(const uint4*)pa[u] : zero;
    rb[u] = (pb[u] && kin) ? *(const uint4*)pb[u] : zero;
  }
  f32x4 acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int b = 0; b < 4; b++) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 64) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
      int r = (tid + 256 * u) >> 3;
      *(uint4*)(sA + r * EB_LD + c8) = ra[u];
      *(uint4*)(sB + r * EB_LD + c8) = rb[u];
    }
    __syncthreads();
    const int kn = k0 + 64;
    if (kn < K) {
      bool kin = kn + c8 < K;
#pragma unroll
      for (int u = 0; u < 4; u++) {
        ra[u] = (pa[u] && kin) ? *(const uint4*)(pa[u] + kn) : zero;
        rb[u] = (pb[u] && kin) ? *(const uint4*)(pb[u] + kn) : zero;
      }
    }
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      bf16x8 bfr[4];
#pragma unroll
      for (int b = 0; b < 4; b++)
        bfr[b] = __builtin_bit_cast(bf16x8, *(const uint4*)(sB + (wn + b * 16 + n16) * EB_LD +
                                                             kk * 32 + quad * 8));
#pragma unroll
      for (int a = 0; a < 4; a++) {
        if (a < nmt) {
          bf16x8 av = __builtin_bit_cast(bf16x8, *(const uint4*)(sA + (wm + a * 16 + n16) * EB_LD +
                                                                  kk * 32 + quad * 8));
#pragma unroll
          for (int b = 0; b < 4; b++)
            acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bfr[b], acc[a][b], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 4; a++) {
    if (a >= nmt) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int so = sslot[wm + a * 16 + quad * 4 + i];
      if (so < 0) continue;
      if (epi == 1 || epi == 3) {
#pragma unroll
        for (int b = 0; b < 4; b += 2) {
          int n = n0 + wn + b * 16;
          if (n + 16 + n16 < N)
            out[(size_t)so * ldo + n / 2 + n16] =
                __float2bfloat16(glu_epi(acc[a][b][i], acc[a][b + 1][i], epi, limit, alpha));
        }
        continue;
      }
#pragma unroll
      for (int b = 0; b < 4; b++) {
        int n = n0 + wn + b * 16 + n16;
        if (n < N) out[(size_t)so * ldo + n] = __float2bfloat16(plain_epi(acc[a][b][i], epi));
      }
    }
  }
}

// any type, any shape: 32 slots x 64 columns per block, K staged through LDS 32 at a time
#define EG_KT 32
template <typename T>
__global__ void __launch_bounds__(256)
expert_gemm_fma_k(const T* __restrict__ x, int ldx, int x_div, const T* __restrict__ w,
                  const int* __restrict__ cnt, const int* __restrict__ rows, int ldr,
                  T* __restrict__ out, int ldo, int N, int K, int E, int TMP, int epi, float limit, float alpha) {
  __shared__ float sx[32][EG_KT + 1];
  __shared__ float sw[64][EG_KT + 1];
  __shared__ int sslot[32];
  int e, m0, nt;
  if (!find_tile(cnt, E, 32, TMP, e, m0, nt)) return;
  const int c = cnt[e], n0 = nt * 64;
  const int tid = threadIdx.x;
  if (tid < 32) sslot[tid] = m0 + tid < c ? rows[(size_t)e * ldr + m0 + tid] : -1;
  __syncthreads();
  // thread (ty, tx): slots ty*2 .. ty*2+1, columns tx + 16*u
  const int tx = tid & 15, ty = tid >> 4;
  float acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int u = 0; u < 4; u++) acc[a][u] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += EG_KT) {
    for (int idx = tid; idx < 32 * EG_KT; idx += 256) {
      int m = idx / EG_KT, k = idx % EG_KT;
      int s = sslot[m];
      sx[m][k] = (s >= 0 && k0 + k < K) ? ldf(x, (size_t)(s / x_div) * ldx + k0 + k) : 0.0f;
    }
    for (int idx = tid; idx < 64 * EG_KT; idx += 256) {
      int n = idx / EG_KT, k = idx % EG_KT;
      sw[n][k] = (n0 + n < N && k0 + k < K) ? ldf(w, ((size_t)e * N + n0 + n) * K + k0 + k) : 0.0f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < EG_KT; k++) {
      float xa = sx[ty * 2][k], xb = sx[ty * 2 + 1][k];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        float wv = sw[tx + 16 * u][k];
        acc[0][u] += xa * wv;
        acc[1][u] += xb * wv;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 2; a++) {
    int s = sslot[ty * 2 + a];
    if (s < 0) continue;
    if (epi == 1 || epi == 3) {
#pragma unroll
      for (int u = 0; u < 4; u += 2) {
        int n = n0 + 16 * u;
        if (n + 16 + tx < N)
          stf(out, (size_t)s * ldo + n / 2 + tx,
              glu_epi(acc[a][u], acc[a][u + 1], epi, limit, alpha));
      }
      continue;
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      int n = n0 + tx + 16 * u;
      if (n < N) stf(out, (size_t)s * ldo + n, plain_epi(acc[a][u], epi));
    }
  }
}

// out[r] = sum_k wts[r, k] * y[r * top + k]; a slot whose expert index is >= n_real (ids given)
// stands for an expert that hands its input back: its term is wts * x[r]
template <typename T>
__global__ void expert_combine_k(const T* __restrict__ y, int ldy, const float* __restrict__ wts,
                                 T* __restrict__ out, int ldo, int top, int n,
                                 const int* __restrict__ ids, int n_real, const T* __restrict__ x,
                                 int ldx) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= n) return;
  float s = 0.0f;
  for (int k = 0; k < top; k++) {
    bool same = ids && ids[r * top + k] >= n_real;
    float v = same ? ldf(x, (size_t)r * ldx + c) : ldf(y, (size_t)(r * top + k) * ldy + c);
    s += wts[r * top + k] * v;
  }
  stf(out, (size_t)r * ldo + c, s);
}

extern "C" {

// cnt must be zero on entry
int p2p_sm_group_route(const void* h, int ldh, const float* wr, int R, int W, int E, int top,
                       int groups, int keep, int score, const float* corr, int gscore, int* ids,
                       float* wts, int* cnt, int* rows, int ldr, const float* bias, int f32,
                       hipStream_t st) {
  if (R <= 0) return 0;
  if (E < 1 || groups < 1 || E % groups || keep < 1 || keep > groups || top < 1 ||
      top > keep * (E / groups) || ldr < R * top)
    return (int)hipErrorInvalidValue;
  size_t shm = (size_t)(W + 2 * E + groups + top) * 4;
  if (shm > 64 * 1024) return (int)hipErrorInvalidValue;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(group_route_k<T>, dim3(R), dim3(256), shm, st,
                                         (const T*)h, ldh, wr, W, E, top, groups, keep, score, corr,
                                         gscore, ids, wts, cnt, rows, ldr, bias));
  return (int)hipGetLastError();
}

// total_slots: slots over all experts (rows * top; every slot is in exactly one list).
// epi = 1: w holds gate / up rows interleaved in groups of 16 (N = 2F rows, a multiple of 32)
// and out [slots, F] receives the experts' activation instead of the raw products.
int p2p_sm_expert_gemm(const void* x, int ldx, int x_div, const void* w, const int* cnt,
                       const int* rows, int ldr, void* out, int ldo, int E, int N, int K,
                       int total_slots, int epi, float limit, float alpha, int f32,
                       hipStream_t st) {
  if (total_slots <= 0 || E <= 0) return 0;
  if (x_div < 1 || N < 1 || K < 1 || ((epi == 1 || epi == 3) && N % 32))
    return (int)hipErrorInvalidValue;
  if (!f32 && K % 8 == 0 && ldx % 8 == 0 && ((size_t)x & 15) == 0 && ((size_t)w & 15) == 0) {
    if (total_slots >= 64 * E) {   // prompts: the large tile
      int tmp = (((total_slots + 127) / 128 + E) + 7) & ~7;
      dim3 grid(tmp * ((N + 127) / 128));
      hipLaunchKernelGGL(expert_gemm_mfma_big_k, grid, dim3(256), 0, st, (const bf16*)x, ldx, x_div,
                         (const bf16*)w, cnt, rows, ldr, (bf16*)out, ldo, N, K, E, tmp, epi, limit, alpha);
      return (int)hipGetLastError();
    }
    int tmp = (((total_slots + 15) / 16 + E) + 7) & ~7;
    dim3 grid(tmp * ((N + 63) / 64));
    hipLaunchKernelGGL(expert_gemm_mfma_k, grid, dim3(256), 0, st, (const bf16*)x, ldx, x_div,
                       (const bf16*)w, cnt, rows, ldr, (bf16*)out, ldo, N, K, E, tmp, epi, limit, alpha);
    return (int)hipGetLastError();
  }
  int tmp = (((total_slots + 31) / 32 + E) + 7) & ~7;
  dim3 grid(tmp * ((N + 63) / 64));
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(expert_gemm_fma_k<T>, grid, dim3(256), 0, st,
                                         (const T*)x, ldx, x_div, (const T*)w, cnt, rows, ldr,
                                         (T*)out, ldo, N, K, E, tmp, epi, limit, alpha));
  return (int)hipGetLastError();
}

int p2p_sm_expert_combine(const void* y, int ldy, const float* wts, void* out, int ldo, int R,
                          int top, int n, const int* ids, int n_real, const void* x, int ldx,
                          int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (ids && !x) return (int)hipErrorInvalidValue;
  dim3 g((n + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(expert_combine_k<T>, g, b, 0, st, (const T*)y, ldy, wts,
                                         (T*)out, ldo, top, n, ids, n_real, (const T*)x, ldx));
  return (int)hipGetLastError();
}

}  // extern "C"
