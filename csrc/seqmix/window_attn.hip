// Grouped-query attention over a paged key/value pool: the pass that prepares its inputs and
// the attention kernel in fp32 arithmetic (float32 models, shapes the matrix-core kernel does
// not take).
//
// qk_norm_rope_store_k: one projection buffer holds q (H heads x D) | k (G x D) | v (G x V) of a
// row.  q and k are RMS-normalised and weighted -- with one mean square per row (heads not
// separated, a weight per channel of the row) or, `per_head`, one per head and a weight of D
// channels that the heads share -- and nrot channel pairs of every head, (2i, 2i+1) or, `half`,
// (i, i + nrot), are turned by the angle pos * inv_freq[i]:
// (a, b) -> (a cos - b sin, b cos + a sin).  q goes to its own buffer, k | v to the row of the
// paged pool that the token owns; a layer that reads another layer's keys and values passes no
// pool and only its queries are prepared.  Norm, angle and rotation are fp32.
//
// window_attn_k: pool row = [k of G heads | v of G heads]; query head h reads key/value head
// h / (H/G).  Causal sliding window: position i sees j with 0 <= i - j < win.  The softmax
// denominator holds one more term exp(sink_h) that adds nothing to the numerator: the running
// maximum starts at sink_h and the running sum at 1 (without a sink: an ordinary softmax).
// Optional steps on a score s of query position i and key position j, in this order:
// cap * tanh(s / cap) (cap > 0), and s - r1_h * ln(1 + r2_h * (i - j)) (r1, r2 given).  Optional
// head gate: head h of row r leaves multiplied by sigmoid(gate[r, h]).  One block per (query
// row, key/value head): the heads of the group share the key and value tiles, which stream
// through LDS with an online softmax.
//
// rope_rows_k: turns the channel pairs (2i, 2i+1) of a stretch of every head by pos * inv_freq[i]
// and writes them to another place (its own rows or scattered ones).  qtemp_kv_store_k: the
// input pass of attention without rotation: q times the temperature of its position,
// 1 + coef * ln(floor((p + 1) / every) + 1), to its own buffer, k | v to the token's pool row.
#include "common.h"
using namespace sm;

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_k(const T* __restrict__ proj, int ldp, int H, int G, int D, int V,
                     const float* __restrict__ qw, const float* __restrict__ kw,
                     const float* __restrict__ inv_freq, int nrot, const int* __restrict__ pos,
                     const int* __restrict__ cache_rows, T* __restrict__ pool, float eps,
                     T* __restrict__ q_out, int ldq, int per_head, int half) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const int nq = H * D, nk = G * D, nv = G * V;
  const int heads = pool ? H + G : H;     // without a pool only the queries are prepared
  const T* row = proj + (size_t)r * ldp;
  float rq = 0.0f, rk = 0.0f;
  if (!per_head) {
    float sq = 0.0f, sk = 0.0f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      float v = ldf(row, i);
      sq += v * v;
    }
    if (pool)
      for (int i = threadIdx.x; i < nk; i += blockDim.x) {
        float v = ldf(row, nq + i);
        sk += v * v;
      }
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    rq = 1.0f / sqrtf(sq / (float)nq + eps);
    rk = 1.0f / sqrtf(sk / (float)nk + eps);
  }
  const float p = (float)pos[r];
  T* crow = pool ? pool + (size_t)cache_rows[r] * (nk + nv) : nullptr;
  T* qrow = q_out + (size_t)r * ldq;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  // one wavefront per head: q heads, then k heads
  for (int hh = wave; hh < heads; hh += nw) {
    const bool isq = hh < H;
    const int hd = isq ? hh : hh - H;
    const T* src = row + (isq ? 0 : nq) + hd * D;
    const float* w = (isq ? qw : kw) + (per_head ? 0 : hd * D);
    T* dst = (isq ? qrow : crow) + hd * D;
    float rs = isq ? rq : rk;
    if (per_head) {
      float ss = 0.0f;
      for (int i = lane; i < D; i += 64) {
        float v = ldf(src, i);
        ss += v * v;
      }
      ss = wave_sum(ss);
      rs = 1.0f / sqrtf(ss / (float)D + eps);
    }
    for (int j = lane; j < nrot; j += 64) {
      int ca = half ? j : 2 * j, cb = half ? j + nrot : 2 * j + 1;
      float a = ldf(src, ca) * rs * w[ca], b = ldf(src, cb) * rs * w[cb];
      float sn, cs;
      sincosf(p * inv_freq[j], &sn, &cs);
      stf(dst, ca, a * cs - b * sn);
      stf(dst, cb, b * cs + a * sn);
    }
    for (int c = 2 * nrot + lane; c < D; c += 64) stf(dst, c, ldf(src, c) * rs * w[c]);
  }
  if (pool)
    for (int i = threadIdx.x; i < nv; i += blockDim.x) crow[nk + i] = row[nq + nk + i];
}

template <typename T>
__global__ void rope_rows_k(const T* __restrict__ src, int lds_, int heads, int src_hs,
                            const float* __restrict__ inv_freq, int nrot,
                            const int* __restrict__ pos, const int* __restrict__ out_rows,
                            T* __restrict__ dst, long ldd, long dst_hs) {
  const int r = blockIdx.x;
  const float p = (float)pos[r];
  const long ro = out_rows ? out_rows[r] : r;
  if (ro < 0) return;
  const T* s = src + (size_t)r * lds_;
  T* d = dst + ro * ldd;
  for (int idx = threadIdx.x; idx < heads * nrot; idx += blockDim.x) {
    int h = idx / nrot, i = idx % nrot;
    float a = ldf(s, (size_t)h * src_hs + 2 * i), b = ldf(s, (size_t)h * src_hs + 2 * i + 1);
    float sn, cs;
    sincosf(p * inv_freq[i], &sn, &cs);
    stf(d, (size_t)(h * dst_hs + 2 * i), a * cs - b * sn);
    stf(d, (size_t)(h * dst_hs + 2 * i + 1), b * cs + a * sn);
  }
}

// Input pass of latent attention with low-rank queries: one projection row holds the query
// latent (nq numbers), the key/value latent (nc) and a key part to be rotated (2 * nrot and what
// follows it up to nr channels, unrotated).  Both latents are RMS-normalised by themselves and
// weighted; the query latent goes to its own buffer, the key/value latent and the rotated part
// to the token's row of the paged pool ([nc | nr]).  Wavefront 0 takes the query latent,
// wavefront 1 the key/value latent, wavefront 2 the rotation.
#define LP_NV 24   // values a lane keeps in registers: latents of up to 1536 numbers are read once
template <typename T>
__global__ void __launch_bounds__(192)
latent_prep_k(const T* __restrict__ proj, int ldp, int nq, int nc, int nr,
              const float* __restrict__ qw, const float* __restrict__ cw,
              const float* __restrict__ inv_freq, int nrot, const int* __restrict__ pos,
              const int* __restrict__ cache_rows, T* __restrict__ pool, float eps,
              T* __restrict__ cq, int ldq) {
  const int r = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* row = proj + (size_t)r * ldp;
  T* crow = pool + (size_t)cache_rows[r] * (nc + nr);
  if (wave < 2) {
    const T* src = row + (wave ? nq : 0);
    const int n = wave ? nc : nq;
    const float* w = wave ? cw : qw;
    T* dst = wave ? crow : cq + (size_t)r * ldq;
    float ss = 0.0f;
    if (n <= 64 * LP_NV) {
      // the latent and its weights are read once, all loads in flight together
      float v[LP_NV], wv[LP_NV];
#pragma unroll
      for (int k = 0; k < LP_NV; k++) {
        int i = lane + 64 * k;
        v[k] = i < n ? ldf(src, i) : 0.0f;
        wv[k] = i < n ? w[i] : 0.0f;
        ss += v[k] * v[k];
      }
      ss = wave_sum(ss);
      const float rs = 1.0f / sqrtf(ss / (float)n + eps);
#pragma unroll
      for (int k = 0; k < LP_NV; k++) {
        int i = lane + 64 * k;
        if (i < n) stf(dst, i, v[k] * rs * wv[k]);
      }
      return;
    }
    for (int i = lane; i < n; i += 64) {
      float v = ldf(src, i);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)n + eps);
    for (int i = lane; i < n; i += 64) stf(dst, i, ldf(src, i) * rs * w[i]);
    return;
  }
  const T* src = row + nq + nc;
  T* dst = crow + nc;
  const float p = (float)pos[r];
  for (int i = lane; i < nrot; i += 64) {
    float a = ldf(src, 2 * i), b = ldf(src, 2 * i + 1);
    float sn, cs;
    sincosf(p * inv_freq[i], &sn, &cs);
    stf(dst, 2 * i, a * cs - b * sn);
    stf(dst, 2 * i + 1, b * cs + a * sn);
  }
  for (int i = 2 * nrot + lane; i < nr; i += 64) dst[i] = src[i];
}

template <typename T>
__global__ void qtemp_kv_store_k(const T* __restrict__ proj, int ldp, int nq, int nkv, float coef,
                                 int every, const int* __restrict__ pos,
                                 const int* __restrict__ cache_rows, T* __restrict__ pool,
                                 T* __restrict__ q_out, int ldq) {
  const int r = blockIdx.x;
  const T* row = proj + (size_t)r * ldp;
  const float temp = 1.0f + coef * logf((float)((pos[r] + 1) / every + 1));
  for (int i = threadIdx.x; i < nq; i += blockDim.x)
    stf(q_out, (size_t)r * ldq + i, ldf(row, i) * temp);
  T* crow = pool + (size_t)cache_rows[r] * nkv;
  for (int i = threadIdx.x; i < nkv; i += blockDim.x) crow[i] = row[nq + i];
}

#define WA_TK 32       // keys per tile at most
#define WA_THREADS 256
#define WA_ACC 16      // (head, value channel) pairs per thread at most

template <typename T>
__global__ void __launch_bounds__(WA_THREADS)
window_attn_k(const T* __restrict__ q, int ldq, const T* __restrict__ pool,
              const int* __restrict__ bt, int max_pages, const int* __restrict__ row_ent,
              const int* __restrict__ pos, const float* __restrict__ sink, float scale, int win,
              T* __restrict__ out, int ldo, int H, int G, int D, int V, int page, int TK,
              float out_scale, int HB, float cap, const float* __restrict__ r1,
              const float* __restrict__ r2, const T* __restrict__ gate, int ldg) {
  extern __shared__ float smem[];
  // a block takes up to HB query heads of one key/value head (all of them when they fit)
  const int nhb = (H / G + HB - 1) / HB;
  const int g = blockIdx.y / nhb, hb0 = (blockIdx.y % nhb) * HB;
  const int h0 = g * (H / G) + hb0, HG = min(HB, H / G - hb0);
  const int ldk = D + 1, ldv = V + 1, ldpool = G * (D + V);
  float* sq = smem;                      // [HB][D]
  float* sk = sq + HB * D;               // [TK][D + 1]
  float* sv = sk + TK * ldk;             // [TK][V + 1]
  float* sp = sv + TK * ldv;             // [HB][TK]
  float* sm_ = sp + HB * TK;             // [HB] running max
  float* sl = sm_ + HB;                  // [HB] running sum
  float* sal = sl + HB;                  // [HB] rescale of this tile
  const int r = blockIdx.x, tid = threadIdx.x;
  const int p = pos[r];
  const int* pages = bt + (size_t)row_ent[r] * max_pages;
  const int j_lo = max(0, p - win + 1);
  for (int idx = tid; idx < HG * D; idx += WA_THREADS)
    sq[idx] = ldf(q, (size_t)r * ldq + (size_t)h0 * D + idx);
  if (tid < HG) {
    sm_[tid] = sink ? sink[h0 + tid] : -1e30f;   // no sink: an ordinary softmax
    sl[tid] = sink ? 1.0f : 0.0f;
  }
  float acc[WA_ACC];
#pragma unroll
  for (int a = 0; a < WA_ACC; a++) acc[a] = 0.0f;
  const int npair = HG * V;
  for (int j0 = j_lo; j0 <= p; j0 += TK) {
    int nk = min(TK, p + 1 - j0);
    __syncthreads();  // previous tile fully consumed (and sq / sm_ / sl initialised)
    for (int idx = tid; idx < nk * D; idx += WA_THREADS) {
      int jj = idx / D, c = idx % D;
      int j = j0 + jj;
      size_t tok = (size_t)pages[j / page] * page + (j % page);
      sk[jj * ldk + c] = ldf(pool, tok * ldpool + (size_t)g * D + c);
    }
    for (int idx = tid; idx < nk * V; idx += WA_THREADS) {
      int jj = idx / V, c = idx % V;
      int j = j0 + jj;
      size_t tok = (size_t)pages[j / page] * page + (j % page);
      sv[jj * ldv + c] = ldf(pool, tok * ldpool + (size_t)G * D + (size_t)g * V + c);
    }
    __syncthreads();
    for (int idx = tid; idx < HG * TK; idx += WA_THREADS) {
      int h = idx / TK, jj = idx % TK;
      float s = -INFINITY;
      if (jj < nk) {
        const float* qh = sq + h * D;
        const float* kr = sk + jj * ldk;
        float d = 0.0f;
        for (int i = 0; i < D; i++) d += qh[i] * kr[i];
        s = d * scale;
        if (cap > 0.0f) s = cap * tanhf(s / cap);
        if (r1) s -= r1[h0 + h] * log1pf(r2[h0 + h] * (float)(p - (j0 + jj)));
      }
      sp[idx] = s;
    }
    __syncthreads();
    if (tid < HG) {
      float mt = sm_[tid];
      float mo = mt;
      for (int jj = 0; jj < nk; jj++) mt = fmaxf(mt, sp[tid * TK + jj]);
      sal[tid] = expf(mo - mt);
      sm_[tid] = mt;
    }
    __syncthreads();
    for (int idx = tid; idx < HG * TK; idx += WA_THREADS) {
      int h = idx / TK, jj = idx % TK;
      sp[idx] = jj < nk ? expf(sp[idx] - sm_[h]) : 0.0f;
    }
    __syncthreads();
    if (tid < HG) {
      float l = sl[tid] * sal[tid];
      for (int jj = 0; jj < nk; jj++) l += sp[tid * TK + jj];
      sl[tid] = l;
    }
#pragma unroll
    for (int a = 0; a < WA_ACC; a++) {
      int idx = tid + a * WA_THREADS;
      if (idx < npair) {
        int h = idx / V, c = idx % V;
        float v = acc[a] * sal[h];
        const float* pr = sp + h * TK;
        for (int jj = 0; jj < nk; jj++) v += pr[jj] * sv[jj * ldv + c];
        acc[a] = v;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int a = 0; a < WA_ACC; a++) {
    int idx = tid + a * WA_THREADS;
    if (idx < npair) {
      int h = idx / V;
      float o = acc[a] / sl[h] * out_scale;
      if (gate) o *= sigmoidf_(ldf(gate, (size_t)r * ldg + h0 + h));
      stf(out, (size_t)r * ldo + (size_t)h0 * V + idx, o);
    }
  }
}

extern "C" {

int p2p_sm_qk_norm_rope_store(const void* proj, int ldp, int H, int G, int D, int V,
                              const float* qw, const float* kw, const float* inv_freq, int nrot,
                              const int* pos, const int* cache_rows, void* pool, float eps,
                              void* q_out, int ldq, int R, int per_head, int half, int f32,
                              hipStream_t st) {
  if (R <= 0) return 0;
  if (H < 1 || G < 1 || D < 1 || V < 1 || nrot < 0 || 2 * nrot > D) return (int)hipErrorInvalidValue;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(qk_norm_rope_store_k<T>, dim3(R), dim3(256), 0, st,
                                         (const T*)proj, ldp, H, G, D, V, qw, kw, inv_freq, nrot,
                                         pos, cache_rows, (T*)pool, eps, (T*)q_out, ldq, per_head,
                                         half));
  return (int)hipGetLastError();
}

int p2p_sm_rope_rows(const void* src, int lds_, int heads, int src_hs, const float* inv_freq,
                     int nrot, const int* pos, const int* out_rows, void* dst, long ldd,
                     long dst_hs, int R, int f32, hipStream_t st) {
  if (R <= 0 || heads <= 0 || nrot <= 0) return 0;
  int threads = heads * nrot >= 256 ? 256 : 64;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(rope_rows_k<T>, dim3(R), dim3(threads), 0, st,
                                         (const T*)src, lds_, heads, src_hs, inv_freq, nrot, pos,
                                         out_rows, (T*)dst, ldd, dst_hs));
  return (int)hipGetLastError();
}

int p2p_sm_latent_prep(const void* proj, int ldp, int nq, int nc, int nr, const float* qw,
                       const float* cw, const float* inv_freq, int nrot, const int* pos,
                       const int* cache_rows, void* pool, float eps, void* cq, int ldq, int R,
                       int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (nq < 1 || nc < 1 || nr < 0 || nrot < 0 || 2 * nrot > nr) return (int)hipErrorInvalidValue;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(latent_prep_k<T>, dim3(R), dim3(192), 0, st,
                                         (const T*)proj, ldp, nq, nc, nr, qw, cw, inv_freq, nrot,
                                         pos, cache_rows, (T*)pool, eps, (T*)cq, ldq));
  return (int)hipGetLastError();
}

int p2p_sm_qtemp_kv_store(const void* proj, int ldp, int nq, int nkv, float coef, int every,
                          const int* pos, const int* cache_rows, void* pool, void* q_out, int ldq,
                          int R, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (nq < 1 || nkv < 1 || every < 1) return (int)hipErrorInvalidValue;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(qtemp_kv_store_k<T>, dim3(R), dim3(256), 0, st,
                                         (const T*)proj, ldp, nq, nkv, coef, every, pos,
                                         cache_rows, (T*)pool, (T*)q_out, ldq));
  return (int)hipGetLastError();
}

int p2p_sm_window_attn(const void* q, int ldq, const void* pool, const int* bt, int max_pages,
                       const int* row_ent, const int* pos, const float* sink, float scale, int win,
                       void* out, int ldo, int R, int H, int G, int D, int V, int page,
                       float out_scale, float cap, const float* r1, const float* r2,
                       const void* gate, int ldg, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (H < 1 || G < 1 || H % G || D < 1 || V < 1 || win < 1 || (r1 && !r2) || cap < 0.0f)
    return (int)hipErrorInvalidValue;
  int HG = H / G, TK = WA_TK, HB = HG;
  auto lds = [&](int tk, int hb) {
    return ((size_t)hb * D + (size_t)tk * (D + 1) + (size_t)tk * (V + 1) + (size_t)hb * tk +
            3 * hb) * 4;
  };
  // heads per block: as many of the group as the accumulators and the LDS hold
  while (HB > 1 && ((long)HB * V > (long)WA_ACC * WA_THREADS || HB > WA_THREADS ||
                    lds(8, HB) > 64 * 1024))
    HB = (HB + 1) / 2;
  while (TK > 2 && lds(TK, HB) > 64 * 1024) TK /= 2;
  if ((long)HB * V > (long)WA_ACC * WA_THREADS || lds(TK, HB) > 64 * 1024)
    return (int)hipErrorInvalidValue;
  dim3 grid(R, G * ((HG + HB - 1) / HB));
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(window_attn_k<T>, grid, dim3(WA_THREADS), lds(TK, HB), st,
                                         (const T*)q, ldq, (const T*)pool, bt, max_pages, row_ent,
                                         pos, sink, scale, win, (T*)out, ldo, H, G, D, V, page, TK,
                                         out_scale, HB, cap, r1, r2, (const T*)gate, ldg));
  return (int)hipGetLastError();
}

}  // extern "C"
