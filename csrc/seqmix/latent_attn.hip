// Latent attention over a paged cache of per-token latents c (one vector of `rank` numbers
// per token, shared by all heads).  The key and value up-projections are applied outside:
// the query arrives already multiplied by W_uk (qa = W_uk^T q per head), so a score is
// scale * qa . c, and the kernel returns sum_j p_j c_j per head, to be multiplied by W_uv.
// Causal sliding window: position i sees j with 0 <= i - j < win.  The softmax denominator
// holds one more term exp(sink_h) with no key and no value: the running maximum starts at
// sink_h and the running sum at 1.
// One block per (query row, group of heads); keys stream through LDS in tiles with an online
// softmax in fp32.  The group size and the key tile are chosen so that a block's LDS fits.
#include "common.h"
using namespace sm;

#define LA_TK 32       // keys per tile at most
#define LA_THREADS 256
#define LA_ACC 32      // (head, latent channel) pairs per thread at most

template <typename T>
__global__ void __launch_bounds__(LA_THREADS)
latent_attn_k(const T* __restrict__ qa, long sqh, long sqr, const T* __restrict__ cache,
              const int* __restrict__ bt, int max_pages, const int* __restrict__ row_ent,
              const int* __restrict__ pos, const float* __restrict__ sink, float scale, int win,
              T* __restrict__ out, long soh, long sor, int Hall, int rank, int page, int HG,
              int TK) {
  extern __shared__ float smem[];
  int ldc = rank + 1;
  int h0 = blockIdx.y * HG;
  int H = min(HG, Hall - h0);            // heads of this block
  qa += (size_t)h0 * sqh;
  out += (size_t)h0 * soh;
  if (sink) sink += h0;
  float* sq = smem;                      // [H][rank]
  float* sc = sq + HG * rank;            // [TK][rank + 1]
  float* sp = sc + TK * ldc;             // [H][TK]
  float* sm_ = sp + HG * TK;             // [H] running max
  float* sl = sm_ + HG;                  // [H] running sum
  float* sal = sl + HG;                  // [H] rescale of this tile
  int r = blockIdx.x, tid = threadIdx.x;
  int p = pos[r];
  const int* pages = bt + (size_t)row_ent[r] * max_pages;
  int j_lo = max(0, p - win + 1);
  for (int idx = tid; idx < H * rank; idx += LA_THREADS) {
    int h = idx / rank, c = idx % rank;
    sq[idx] = ldf(qa, (size_t)h * sqh + (size_t)r * sqr + c);
  }
  if (tid < H) {
    sm_[tid] = sink ? sink[tid] : -1e30f;   // no sink: an ordinary softmax
    sl[tid] = sink ? 1.0f : 0.0f;
  }
  float acc[LA_ACC];
#pragma unroll
  for (int a = 0; a < LA_ACC; a++) acc[a] = 0.0f;
  int npair = H * rank;
  for (int j0 = j_lo; j0 <= p; j0 += TK) {
    int nk = min(TK, p + 1 - j0);
    __syncthreads();  // previous tile fully consumed (and sq / sm_ / sl initialised)
    for (int idx = tid; idx < nk * rank; idx += LA_THREADS) {
      int jj = idx / rank, c = idx % rank;
      int j = j0 + jj;
      size_t tok = (size_t)pages[j / page] * page + (j % page);
      sc[jj * ldc + c] = ldf(cache, tok * rank + c);
    }
    __syncthreads();
    for (int idx = tid; idx < H * TK; idx += LA_THREADS) {
      int h = idx / TK, jj = idx % TK;
      float s = -INFINITY;
      if (jj < nk) {
        const float* q = sq + h * rank;
        const float* c = sc + jj * ldc;
        float d = 0.0f;
        for (int i = 0; i < rank; i++) d += q[i] * c[i];
        s = d * scale;
      }
      sp[idx] = s;
    }
    __syncthreads();
    if (tid < H) {
      float mt = sm_[tid];
      float mo = mt;
      for (int jj = 0; jj < nk; jj++) mt = fmaxf(mt, sp[tid * TK + jj]);
      sal[tid] = expf(mo - mt);
      sm_[tid] = mt;
    }
    __syncthreads();
    for (int idx = tid; idx < H * TK; idx += LA_THREADS) {
      int h = idx / TK, jj = idx % TK;
      sp[idx] = jj < nk ? expf(sp[idx] - sm_[h]) : 0.0f;
    }
    __syncthreads();
    if (tid < H) {
      float l = sl[tid] * sal[tid];
      for (int jj = 0; jj < nk; jj++) l += sp[tid * TK + jj];
      sl[tid] = l;
    }
#pragma unroll
    for (int a = 0; a < LA_ACC; a++) {
      int idx = tid + a * LA_THREADS;
      if (idx < npair) {
        int h = idx / rank, c = idx % rank;
        float v = acc[a] * sal[h];
        const float* pr = sp + h * TK;
        for (int jj = 0; jj < nk; jj++) v += pr[jj] * sc[jj * ldc + c];
        acc[a] = v;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int a = 0; a < LA_ACC; a++) {
    int idx = tid + a * LA_THREADS;
    if (idx < npair) {
      int h = idx / rank, c = idx % rank;
      stf(out, (size_t)h * soh + (size_t)r * sor + c, acc[a] / sl[h]);
    }
  }
}

extern "C" int p2p_sm_latent_attn(const void* qa, long sqh, long sqr, const void* cache,
                                  const int* bt, int max_pages, const int* row_ent,
                                  const int* pos, const float* sink, float scale, int win,
                                  void* out, long soh, long sor, int R, int H, int rank, int page,
                                  int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (H < 1 || rank < 1 || win < 1) return (int)hipErrorInvalidValue;
  // heads per block and keys per tile: the largest that fit the accumulators and 64 KB of LDS
  int HG = H < LA_THREADS ? H : LA_THREADS, TK = LA_TK;
  auto lds = [&](int hg, int tk) {
    return ((size_t)hg * rank + (size_t)tk * (rank + 1) + (size_t)hg * tk + 3 * hg) * 4;
  };
  while (HG > 1 && ((long)HG * rank > (long)LA_ACC * LA_THREADS || lds(HG, TK) > 64 * 1024))
    HG = (HG + 1) / 2;
  while (TK > 4 && lds(HG, TK) > 64 * 1024) TK /= 2;
  if ((long)HG * rank > (long)LA_ACC * LA_THREADS || lds(HG, TK) > 64 * 1024)
    return (int)hipErrorInvalidValue;
  size_t shm = lds(HG, TK);
  dim3 grid(R, (H + HG - 1) / HG);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(latent_attn_k<T>, grid, dim3(LA_THREADS), shm, st,
                                         (const T*)qa, sqh, sqr, (const T*)cache, bt, max_pages,
                                         row_ent, pos, sink, scale, win, (T*)out, soh, sor, H,
                                         rank, page, HG, TK));
  return (int)hipGetLastError();
}
