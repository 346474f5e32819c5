// Pointwise pieces between the matrix products: tanh in place, sigmoid output gates with
// arbitrary input strides, the clamped gated feed-forward activation
//   g = min(gate, limit), u = clamp(up, -limit, limit), y = g * sigmoid(1.702 g) * (u + 1),
// the silu-gated one, silu(gate) * up, and the tanh cap of the logits.
#include "common.h"
using namespace sm;

template <typename T>
__global__ void tanh_k(T* x, int ld, int n, int R) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c < n) stf(x, (size_t)r * ld + c, tanhf(ldf(x, (size_t)r * ld + c)));
}

// out[r, h * V + v] = o[h * soh + r * sor + v] * sigmoid(g[r * ldg + h * V + v])
template <typename T>
__global__ void sigmoid_gate_k(const T* __restrict__ o, long soh, long sor, const T* __restrict__ g,
                               int ldg, T* __restrict__ out, int ldo, int H, int V,
                               int per_head) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= H * V) return;
  int h = c / V, v = c % V;
  float x = ldf(o, (size_t)h * soh + (size_t)r * sor + v);
  stf(out, (size_t)r * ldo + c, x * sigmoidf_(ldf(g, (size_t)r * ldg + (per_head ? h : c))));
}

template <typename T>
__global__ void ff_act_k(const T* __restrict__ gu, int ld, T* __restrict__ out, int ldo, int F,
                         float limit, float alpha) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= F) return;
  float g = fminf(ldf(gu, (size_t)r * ld + c), limit);
  float u = fminf(fmaxf(ldf(gu, (size_t)r * ld + F + c), -limit), limit);
  stf(out, (size_t)r * ldo + c, g * sigmoidf_(alpha * g) * (u + 1.0f));
}

// tanh form of gelu: 0.5 z (1 + tanh(y)), y = sqrt(2/pi) (z + 0.044715 z^3), evaluated as
// z * sigmoid(2 y), which is the same function (1 + tanh(y) = 2 sigmoid(2 y))
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return z * sigmoidf_(1.5957691216057308f * (z + 0.044715f * z * z * z));
}

// [gate | up] -> act(gate) * up; act: 0 silu, 1 gelu (tanh form)
template <typename T>
__global__ void glu_act_k(const T* __restrict__ gu, int ld, T* __restrict__ out, int ldo, int F,
                          int act) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= F) return;
  float g = ldf(gu, (size_t)r * ld + c);
  float a = act == 1 ? gelu_tanhf_(g) : g * sigmoidf_(g);
  stf(out, (size_t)r * ldo + c, a * ldf(gu, (size_t)r * ld + F + c));
}

// out[r, c] = relu(u[r, c])^2 * sigmoid(g[r]): an ungated squared-relu unit whose result is
// weighted by one gate per row (g == nullptr: no gate)
template <typename T>
__global__ void relu2_gate_k(const T* __restrict__ u, int ld, const T* __restrict__ g, int ldg,
                             T* __restrict__ out, int ldo, int F) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= F) return;
  float v = fmaxf(ldf(u, (size_t)r * ld + c), 0.0f);
  float w = g ? sigmoidf_(ldf(g, (size_t)r * ldg)) : 1.0f;
  stf(out, (size_t)r * ldo + c, v * v * w);
}

template <typename T>
__global__ void softcap_k(const T* __restrict__ y, int ld, float* __restrict__ out, int n,
                          float cap, float scale) {
  int c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
  if (c >= n) return;
  float z = ldf(y, (size_t)r * ld + c) * scale;
  out[(size_t)r * n + c] = cap > 0.0f ? cap * tanhf(z / cap) : z;
}

extern "C" {

int p2p_sm_glu_act(const void* gu, int ld, void* out, int ldo, int R, int F, int act, int f32,
                   hipStream_t st) {
  if (R <= 0) return 0;
  dim3 g((F + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(glu_act_k<T>, g, b, 0, st, (const T*)gu, ld, (T*)out, ldo, F,
                                         act));
  return (int)hipGetLastError();
}

int p2p_sm_relu2_gate(const void* u, int ld, const void* gt, int ldg, void* out, int ldo, int R,
                      int F, int f32, hipStream_t st) {
  if (R <= 0 || F <= 0) return 0;
  dim3 g((F + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(relu2_gate_k<T>, g, b, 0, st, (const T*)u, ld,
                                         (const T*)gt, ldg, (T*)out, ldo, F));
  return (int)hipGetLastError();
}

int p2p_sm_softcap(const void* y, int ld, float* out, int R, int n, float cap, float scale,
                   int f32, hipStream_t st) {
  if (R <= 0 || n <= 0) return 0;
  dim3 g((n + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(softcap_k<T>, g, b, 0, st, (const T*)y, ld, out, n, cap,
                                         scale));
  return (int)hipGetLastError();
}

int p2p_sm_tanh(void* x, int ld, int n, int R, int f32, hipStream_t st) {
  if (R <= 0 || n <= 0) return 0;
  dim3 g((n + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(tanh_k<T>, g, b, 0, st, (T*)x, ld, n, R));
  return (int)hipGetLastError();
}

int p2p_sm_sigmoid_gate(const void* o, long soh, long sor, const void* gt, int ldg, void* out,
                        int ldo, int R, int H, int V, int per_head, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  dim3 g((H * V + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(sigmoid_gate_k<T>, g, b, 0, st, (const T*)o, soh, sor,
                                         (const T*)gt, ldg, (T*)out, ldo, H, V, per_head));
  return (int)hipGetLastError();
}

int p2p_sm_ff_act(const void* gu, int ld, void* out, int ldo, int R, int F, float limit,
                  float alpha, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  dim3 g((F + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(ff_act_k<T>, g, b, 0, st, (const T*)gu, ld, (T*)out, ldo,
                                         F, limit, alpha));
  return (int)hipGetLastError();
}

}  // extern "C"
