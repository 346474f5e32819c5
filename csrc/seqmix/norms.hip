// Embedding with learned positions, RMS norms over fp32 or activation-typed rows (whole
// row or equal parts, optional scatter of the rows), and the post-sublayer passes on the fp32
// residual stream: norm + layer scale + residual add, and the gated form
// x += N(y * sigmoid(g + b)) * w with the norm N taken over equal parts of the row.
#include "common.h"
using namespace sm;

template <typename T>
__global__ void embed_pos_k(const T* __restrict__ embed, const T* __restrict__ ptab,
                            const int* __restrict__ ids, const int* __restrict__ pos,
                            float* __restrict__ out, int W, int has_pos) {
  int r = blockIdx.x;
  size_t eo = (size_t)ids[r] * W, po = (size_t)pos[r] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = ldf(embed, eo + i);
    if (has_pos) v += ldf(ptab, po + i);
    out[(size_t)r * W + i] = v;
  }
}

#define NV 16   // values a thread keeps in registers: rows of up to 256 * NV numbers are read once

// one block per (row, part): out = x / sqrt(mean(x^2) + eps) * w
template <typename TI, typename TO>
__global__ void rmsnorm_k(const TI* __restrict__ x, int ldx, const float* __restrict__ w,
                          TO* __restrict__ out, int ldo, const int* __restrict__ in_rows,
                          const int* __restrict__ out_rows, int n, int parts, float eps) {
  __shared__ float red[16];
  int r = blockIdx.x / parts, g = blockIdx.x % parts;
  int np = n / parts;
  int ri = in_rows ? in_rows[r] : r;
  int ro = out_rows ? out_rows[r] : r;
  const TI* xr = x + (size_t)ri * ldx + (size_t)g * np;
  const float* wp = w ? w + g * np : nullptr;
  if (np <= NV * (int)blockDim.x) {
    // the row and its weights are loaded once, before the reduction
    float v[NV], wv[NV];
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      v[k] = i < np ? ldf(xr, i) : 0.0f;
      wv[k] = (wp && i < np) ? wp[i] : 1.0f;
      ss += v[k] * v[k];
    }
    ss = block_sum(ss, red);
    if (ro < 0) return;
    float rs = 1.0f / sqrtf(ss / (float)np + eps);
    TO* o = out + (size_t)ro * ldo + (size_t)g * np;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      if (i < np) stf(o, i, v[k] * rs * wv[k]);
    }
    return;
  }
  float ss = 0.0f;
  for (int i = threadIdx.x; i < np; i += blockDim.x) {
    float v = ldf(xr, i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  if (ro < 0) return;
  float rs = 1.0f / sqrtf(ss / (float)np + eps);
  TO* o = out + (size_t)ro * ldo + (size_t)g * np;
  for (int i = threadIdx.x; i < np; i += blockDim.x) {
    float v = ldf(xr, i) * rs;
    if (wp) v *= wp[i];
    stf(o, i, v);
  }
}

// x += y / sqrt(mean(y^2) + eps) * w * ls   (x fp32 residual); with w2 also the next
// sublayer's input h = x / sqrt(mean(x^2) + eps) * w2 from the updated row
template <typename T>
__global__ void norm_scale_add_k(float* __restrict__ x, const T* __restrict__ y, int ldy,
                                 const float* __restrict__ w, const float* __restrict__ ls,
                                 int n, float eps, const float* __restrict__ w2,
                                 T* __restrict__ h, int ldh) {
  __shared__ float red[16];
  int r = blockIdx.x;
  const T* yr = y + (size_t)r * ldy;
  float* xr = x + (size_t)r * n;
  if (n <= NV * (int)blockDim.x) {
    // y, the weights and the residual are loaded once, before the reduction
    float v[NV], wv[NV], xv[NV];
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      bool ok = i < n;
      v[k] = ok ? ldf(yr, i) : 0.0f;
      wv[k] = ok ? (ls ? w[i] * ls[i] : w[i]) : 0.0f;
      xv[k] = ok ? xr[i] : 0.0f;
      ss += v[k] * v[k];
    }
    ss = block_sum(ss, red);
    float rs = 1.0f / sqrtf(ss / (float)n + eps);
    float s2 = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      xv[k] = xv[k] + v[k] * rs * wv[k];
      if (i < n) xr[i] = xv[k];
      s2 += xv[k] * xv[k];
    }
    if (!w2) return;
    s2 = block_sum(s2, red);
    float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      if (i < n) stf(h, (size_t)r * ldh + i, xv[k] * r2 * w2[i]);
    }
    return;
  }
  float ss = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = ldf(yr, i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  float rs = 1.0f / sqrtf(ss / (float)n + eps);
  float s2 = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float v = xr[i] + ldf(yr, i) * rs * (ls ? w[i] * ls[i] : w[i]);
    xr[i] = v;
    s2 += v * v;
  }
  if (!w2) return;
  s2 = block_sum(s2, red);
  float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x)   // each thread re-reads its own writes
    stf(h, (size_t)r * ldh + i, xr[i] * r2 * w2[i]);
}

// x += a (+ b) on the fp32 residual, the addends summed first (fp32); with w2 also the next
// layer's input h = x / sqrt(mean(x^2) + eps) * w2 from the updated row
template <typename T>
__global__ void add_norm_k(float* __restrict__ x, const T* __restrict__ a, int lda,
                           const T* __restrict__ b, int ldb, int n, float eps,
                           const float* __restrict__ w2, T* __restrict__ h, int ldh) {
  __shared__ float red[16];
  int r = blockIdx.x;
  const T* ar = a + (size_t)r * lda;
  const T* br = b ? b + (size_t)r * ldb : nullptr;
  float* xr = x + (size_t)r * n;
  if (n <= NV * (int)blockDim.x) {
    // every load goes out before the first store (a store to x in between would hold back
    // the later loads of x)
    float xv[NV], wv[NV], yv[NV];
    float s2 = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      bool ok = i < n;
      int ic = ok ? i : 0;
      float y = ldf(ar, ic);
      if (br) y += ldf(br, ic);
      yv[k] = ok ? y : 0.0f;
      wv[k] = (ok && w2) ? w2[ic] : 0.0f;
      xv[k] = ok ? xr[ic] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      xv[k] += yv[k];
      if (i < n) xr[i] = xv[k];
      s2 += xv[k] * xv[k];
    }
    if (!w2) return;
    s2 = block_sum(s2, red);
    float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      if (i < n) stf(h, (size_t)r * ldh + i, xv[k] * r2 * wv[k]);
    }
    return;
  }
  float s2 = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float y = ldf(ar, i);
    if (br) y += ldf(br, i);
    float v = xr[i] + y;
    xr[i] = v;
    s2 += v * v;
  }
  if (!w2) return;
  s2 = block_sum(s2, red);
  float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x)   // each thread re-reads its own writes
    stf(h, (size_t)r * ldh + i, xr[i] * r2 * w2[i]);
}

// x += a + b + rows + vec + sum_k cw[r, k] * cy[r * top + k] on the fp32 residual (each addend
// optional; a, b, cy activation typed, rows fp32 [R, n], vec fp32 [n], cw fp32 [R, top]: the
// weighted sum of a token's routed expert outputs; summed first, in fp32), then up to two normed copies of the
// updated row, h_i = x / sqrt(mean(x^2) + eps) * w_i, where w_i is a vector (ws_i = 1) or one
// number for all channels (ws_i = 0): two sublayers that read the same row through norms of
// their own get their inputs from one pass over it.
template <typename T, int NR>   // NR: values a thread keeps (rows of up to 256 * NR numbers are read once)
__global__ void add_norm2_k(float* __restrict__ x, const T* __restrict__ a, int lda,
                            const T* __restrict__ b, int ldb, const float* __restrict__ rows,
                            const float* __restrict__ vec, int n, float eps,
                            const float* __restrict__ w1, int ws1, T* __restrict__ h1, int ld1,
                            const float* __restrict__ w2, int ws2, T* __restrict__ h2, int ld2,
                            const T* __restrict__ cy, int ldcy, const float* __restrict__ cw,
                            int top) {
  __shared__ float red[16];
  int r = blockIdx.x;
  const T* cyr = cy ? cy + (size_t)r * top * ldcy : nullptr;
  const float* cwr = cy ? cw + (size_t)r * top : nullptr;
  const T* ar = a ? a + (size_t)r * lda : nullptr;
  const T* br = b ? b + (size_t)r * ldb : nullptr;
  const float* er = rows ? rows + (size_t)r * n : nullptr;
  float* xr = x + (size_t)r * n;
  const bool adds = ar || br || er || vec || cyr;
  // weights that are one number are read before the reduction
  const float g1 = (w1 && !ws1) ? w1[0] : 1.0f, g2 = (w2 && !ws2) ? w2[0] : 1.0f;
  if (n <= NR * (int)blockDim.x) {
    // every load goes out before the first store; each addend's loads form one batch (the
    // tests for the optional addends stay outside the unrolled loops)
    float xv[NR], yv[NR];
    float s2 = 0.0f;
#pragma unroll
    for (int k = 0; k < NR; k++) {
      int i = threadIdx.x + k * blockDim.x;
      xv[k] = xr[i < n ? i : 0];
      yv[k] = 0.0f;
    }
    if (ar) {
#pragma unroll
      for (int k = 0; k < NR; k++) {
        int i = threadIdx.x + k * blockDim.x;
        yv[k] = ldf(ar, i < n ? i : 0);
      }
    }
    if (br) {
#pragma unroll
      for (int k = 0; k < NR; k++) {
        int i = threadIdx.x + k * blockDim.x;
        yv[k] += ldf(br, i < n ? i : 0);
      }
    }
    if (er) {
#pragma unroll
      for (int k = 0; k < NR; k++) {
        int i = threadIdx.x + k * blockDim.x;
        yv[k] += er[i < n ? i : 0];
      }
    }
    if (vec) {
#pragma unroll
      for (int k = 0; k < NR; k++) {
        int i = threadIdx.x + k * blockDim.x;
        yv[k] += vec[i < n ? i : 0];
      }
    }
    if (cyr) {
      // two experts at a time, so that a choice of two is one batch of loads
      for (int t = 0; t < top; t += 2) {
        const bool two = t + 1 < top;
        const float wa = cwr[t], wb = two ? cwr[t + 1] : 0.0f;
        const T* ya = cyr + (size_t)t * ldcy;
        const T* yb = cyr + (size_t)(two ? t + 1 : t) * ldcy;
#pragma unroll
        for (int k = 0; k < NR; k++) {
          int i = threadIdx.x + k * blockDim.x;
          int ic = i < n ? i : 0;
          yv[k] += wa * ldf(ya, ic) + wb * ldf(yb, ic);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < NR; k++) {
      int i = threadIdx.x + k * blockDim.x;
      xv[k] = i < n ? xv[k] + yv[k] : 0.0f;
      if (adds && i < n) xr[i] = xv[k];
      s2 += xv[k] * xv[k];
    }
    if (!w1) return;
    s2 = block_sum(s2, red);
    float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
#pragma unroll
    for (int k = 0; k < NR; k++) {
      int i = threadIdx.x + k * blockDim.x;
      if (i < n) {
        float v = xv[k] * r2;
        stf(h1, (size_t)r * ld1 + i, v * (ws1 ? w1[i] : g1));
        if (w2) stf(h2, (size_t)r * ld2 + i, v * (ws2 ? w2[i] : g2));
      }
    }
    return;
  }
  float s2 = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    float y = 0.0f;
    if (ar) y += ldf(ar, i);
    if (br) y += ldf(br, i);
    if (er) y += er[i];
    if (vec) y += vec[i];
    if (cyr)
      for (int t = 0; t < top; t++) y += cwr[t] * ldf(cyr, (size_t)t * ldcy + i);
    float v = xr[i] + y;
    if (adds) xr[i] = v;
    s2 += v * v;
  }
  if (!w1) return;
  s2 = block_sum(s2, red);
  float r2 = 1.0f / sqrtf(s2 / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) {   // each thread re-reads its own writes
    float v = xr[i] * r2;
    stf(h1, (size_t)r * ld1 + i, v * (ws1 ? w1[i] : g1));
    if (w2) stf(h2, (size_t)r * ld2 + i, v * (ws2 ? w2[i] : g2));
  }
}

// out[r] = embed[ids[r]] * scale as fp32, and (optionally) the same row in the activation type
template <typename T>
__global__ void embed_rows_k(const T* __restrict__ embed, const int* __restrict__ ids,
                             float* __restrict__ out, T* __restrict__ h, int ldh, int W,
                             float scale) {
  int r = blockIdx.x;
  size_t eo = (size_t)ids[r] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = ldf(embed, eo + i) * scale;
    out[(size_t)r * W + i] = v;
    if (h) stf(h, (size_t)r * ldh + i, v);
  }
}

// one block per (row, part): x += v / sqrt(mean(v^2) + eps) * w with v = y * sigmoid(g + gb),
// the mean over the part; h (optional) receives the updated residual in the activation type
template <typename T>
__global__ void gate_norm_add_k(float* __restrict__ x, const T* __restrict__ y, int ldy,
                                const T* __restrict__ g, int ldg, const float* __restrict__ gb,
                                const float* __restrict__ w, int n, int parts, float eps,
                                T* __restrict__ h, int ldh) {
  __shared__ float red[16];
  int r = blockIdx.x / parts, p = blockIdx.x % parts;
  int np = n / parts, c0 = p * np;
  const T* yr = y + (size_t)r * ldy + c0;
  const T* gr = g + (size_t)r * ldg + c0;
  float* xr = x + (size_t)r * n + c0;
  if (np <= NV * (int)blockDim.x) {
    float v[NV], wv[NV], xv[NV];
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      bool ok = i < np;
      float yv = ok ? ldf(yr, i) : 0.0f;
      float gv = ok ? ldf(gr, i) + gb[c0 + i] : 0.0f;
      wv[k] = ok ? w[c0 + i] : 0.0f;
      xv[k] = ok ? xr[i] : 0.0f;
      v[k] = yv * sigmoidf_(gv);
      ss += v[k] * v[k];
    }
    ss = block_sum(ss, red);
    float rs = 1.0f / sqrtf(ss / (float)np + eps);
#pragma unroll
    for (int k = 0; k < NV; k++) {
      int i = threadIdx.x + k * blockDim.x;
      if (i < np) {
        float nv = xv[k] + v[k] * rs * wv[k];
        xr[i] = nv;
        if (h) stf(h, (size_t)r * ldh + c0 + i, nv);
      }
    }
    return;
  }
  float ss = 0.0f;
  for (int i = threadIdx.x; i < np; i += blockDim.x) {
    float v = ldf(yr, i) * sigmoidf_(ldf(gr, i) + gb[c0 + i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  float rs = 1.0f / sqrtf(ss / (float)np + eps);
  for (int i = threadIdx.x; i < np; i += blockDim.x) {
    float v = ldf(yr, i) * sigmoidf_(ldf(gr, i) + gb[c0 + i]);
    float nv = xr[i] + v * rs * w[c0 + i];
    xr[i] = nv;
    if (h) stf(h, (size_t)r * ldh + c0 + i, nv);
  }
}

extern "C" {

int p2p_sm_embed_rows(const void* embed, const int* ids, float* out, void* h, int ldh, int R,
                      int W, float scale, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(embed_rows_k<T>, dim3(R), dim3(256), 0, st,
                                         (const T*)embed, ids, out, (T*)h, ldh, W, scale));
  return (int)hipGetLastError();
}

// h (optional) has the activation type of y and g
int p2p_sm_gate_norm_add(float* x, const void* y, int ldy, const void* g, int ldg,
                         const float* gb, const float* w, int R, int n, int parts, float eps,
                         void* h, int ldh, int h_f32, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (parts <= 0 || n % parts || (h && h_f32 != f32)) return (int)hipErrorInvalidValue;
  // many short parts (prompts): one wavefront per (row, part), so the reduction needs no other
  // wave and more parts are in flight; few rows (decode) keep four wavefronts per part
  const int threads = (n / parts <= 1024 && R * parts >= 1024) ? 64 : 256;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(gate_norm_add_k<T>, dim3(R * parts), dim3(threads), 0, st, x,
                                         (const T*)y, ldy, (const T*)g, ldg, gb, w, n, parts, eps,
                                         (T*)h, ldh));
  return (int)hipGetLastError();
}

int p2p_sm_embed_pos(const void* embed, const void* ptab, const int* ids, const int* pos,
                     float* out, int R, int W, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(embed_pos_k<T>, dim3(R), dim3(256), 0, st,
                                         (const T*)embed, (const T*)ptab, ids, pos, out, W,
                                         ptab != nullptr));
  return (int)hipGetLastError();
}

int p2p_sm_rmsnorm(const void* x, int ldx, int in_f32, const float* w, void* out, int ldo,
                   int out_f32, const int* in_rows, const int* out_rows, int R, int n, int parts,
                   float eps, hipStream_t st) {
  if (R <= 0) return 0;
  if (parts <= 0 || n % parts) return (int)hipErrorInvalidValue;
  dim3 g(R * parts), b(256);
#define RN(TI, TO)                                                                          \
  hipLaunchKernelGGL((rmsnorm_k<TI, TO>), g, b, 0, st, (const TI*)x, ldx, w, (TO*)out, ldo, \
                     in_rows, out_rows, n, parts, eps)
  if (in_f32 && out_f32) RN(float, float);
  else if (in_f32) RN(float, bf16);
  else if (out_f32) RN(bf16, float);
  else RN(bf16, bf16);
#undef RN
  return (int)hipGetLastError();
}

int p2p_sm_norm_scale_add(float* x, const void* y, int ldy, const float* w, const float* ls,
                          int R, int n, float eps, const float* w2, void* h, int ldh, int f32,
                          hipStream_t st) {
  if (R <= 0) return 0;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(norm_scale_add_k<T>, dim3(R), dim3(256), 0, st, x,
                                         (const T*)y, ldy, w, ls, n, eps, w2, (T*)h, ldh));
  return (int)hipGetLastError();
}

int p2p_sm_add_norm2(float* x, const void* a, int lda, const void* b, int ldb, const float* rows,
                     const float* vec, int R, int n, float eps, const float* w1, int ws1, void* h1,
                     int ld1, const float* w2, int ws2, void* h2, int ld2, const void* cy, int ldcy,
                     const float* cw, int top, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if ((w1 && !h1) || (w2 && (!h2 || !w1)) || (b && !a) || (cy && (!cw || top < 1)))
    return (int)hipErrorInvalidValue;
#define AN2(NR)                                                                                 \
  SM_DISPATCH_T(f32, hipLaunchKernelGGL((add_norm2_k<T, NR>), dim3(R), dim3(256), 0, st, x,     \
                                         (const T*)a, lda, (const T*)b, ldb, rows, vec, n, eps,  \
                                         w1, ws1, (T*)h1, ld1, w2, ws2, (T*)h2, ld2,             \
                                         (const T*)cy, ldcy, cw, top))
  // the smallest instance whose registers hold the row: no loads of padding, less code to fetch
  if (n <= 256 * 4) AN2(4);
  else if (n <= 256 * 8) AN2(8);
  else AN2(16);
#undef AN2
  return (int)hipGetLastError();
}

int p2p_sm_add_norm(float* x, const void* a, int lda, const void* b, int ldb, int R, int n,
                    float eps, const float* w2, void* h, int ldh, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(add_norm_k<T>, dim3(R), dim3(256), 0, st, x, (const T*)a,
                                         lda, (const T*)b, ldb, n, eps, w2, (T*)h, ldh));
  return (int)hipGetLastError();
}

}  // extern "C"
