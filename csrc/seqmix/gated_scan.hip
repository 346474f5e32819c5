// Gated linear scans: per head a D x V fp32 state S (key channel i, value channel j) and one
// step per token,
//   S <- diag(g) S
//   u = v                        plain write   (HGRN2: g = f, k = 1 - f)
//   u = beta * (v - S^T k)       delta rule    (the write corrects what the key reads)
//   S <- S + k u^T,  o = S^T q   (o is formed from the updated S)
// followed by the head's RMS norm over V, a weight shared by the heads and, for the delta
// rule, a sigmoid output gate.
//
// The matrix memory of the mLSTM is the plain write with a scalar decay per head and a
// normaliser: with log gates i_t, f_t and the running maximum m_t = max(f_t + m_(t-1), i_t)
// (m_0 = 0),  a_t = exp(f_t + m_(t-1) - m_t),  b_t = exp(i_t - m_t),
//   S <- a_t S + (b_t k) v^T,  n <- a_t n + b_t k,  o = S^T q / (max(|n . q|, exp(-m_t)) + 1e-6).
// m_t depends on the gates alone, so a small kernel walks it first (mlstm_gates_k: a_t, b_t and
// exp(-m_t) per token and head, the slot keeps m); with these coefficients the recurrence is
// linear in (S, n) and runs here.  n is stored as one more value column of the state (column V
// of V + 1) but not carried by the wavefronts that hold S: after a staged chunk's tokens have
// gone through S, thread i walks n_i through the same tokens and leaves n_i q_i in place of q_i
// in LDS, and the epilogue sums them per token.  The head's o is RMS-normalised, weighted per
// channel of the head and gated by a sigmoid.
//
// The value columns of S are independent.  A wavefront covers 16 columns x 4 slices of the key
// index; lane (c, s) keeps rows s*DQ .. s*DQ+DQ-1 of column c in registers (NC columns, 16
// apart, in the general form of the kernel), and the sums over the key index (S^T k before
// the write, S^T q after it) are finished with two lane shuffles.
// The tokens of a sequence portion are walked in order; their vectors are staged through LDS
// a chunk at a time and everything that enters the recurrence is evaluated in fp32 while
// staging: HGRN2's silu(q) and f = lower + (1 - lower) sigmoid(. + b); the delta rule's unit q
// and k (x / sqrt(|x|^2 + 1e-6), q also times D^-1/2), beta = sigmoid(.) and the decay
// g = exp(-exp(A_log_h) softplus(. + dt_bias)).
//
// Long portions run as chunks side by side (the recurrences are linear in the state):
//   local pass   every chunk from a zero state; its end state, and what carries a state across
//                the chunk: the product of its decays per key channel (plain write) or the
//                D x D transition obtained by running the recurrence without values on the
//                identity (delta rule);
//   chain        init_{c+1} = T_c init_c + local_c over each portion's chunks, from the slot's
//                state (or zero at position 0); the last one is the slot's new state;
//   output pass  every chunk again from its true initial state, with the outputs.
#include "common.h"
using namespace sm;

struct ScanArgs {
  // HGRN2: proj = [q (H*D) | f (H*D) | v (H*V)] in the activation type
  const void* proj; int ldp;
  const float* lower; const float* fb;
  // delta rule: conv fp32 = [q (G*D) | k (G*D) | v (H*V)], decay logits, beta logits, gate logits
  const float* conv; int ldc;
  const void* araw; int lda;
  const void* braw; int ldb;
  const void* gate; int ldg;
  const float* A_log; const float* dt_bias;
  // matrix memory: proj = [q (H*D) | k (H*D) | v (H*V) | gate (H*V) | ...] and the
  // coefficients (a_t, b_t, exp(-m_t)) fp32 [rows, H, 3]
  const float* coef;
  int VS;   // value columns of the state: V, or V + 1 with the normaliser
  // common
  const float* normw; float* state; const int* ent; void* out; int ldo;
  int H, G, D, V, CT;
  float eps, out_scale;
  // 0: portions from their slots' states, states written back.  Chunk modes (`ent` lists chunks,
  // its slot field is the chunk index into the buffers below): 1: from zero, end state ->
  // chunk_state (and the decay product -> chunk_decay for the plain write); 2: from
  // chunk_state, outputs only; 3 (delta rule): the transition on the identity -> chunk_trans.
  int mode;
  float* chunk_state;   // [chunks, H, D, V]
  float* chunk_decay;   // [chunks, H, D]
  float* chunk_trans;   // [chunks, H, D, D]
};

template <typename T, int DQ, int KIND, int NC>   // KIND 0: plain write (HGRN2), 1: delta rule, 2: matrix memory
__global__ void __launch_bounds__(1024 / NC) gated_scan_k(ScanArgs a) {
  constexpr bool DELTA = KIND == 1, MEM = KIND == 2;
  constexpr int DKP = 4 * DQ;   // padded key index (zero filled in LDS)
  constexpr int WC = 16 * NC;   // columns per wavefront: a lane keeps NC columns, 16 apart
  const int H = a.H, D = a.D, V = a.V, VS = a.VS, CT = a.CT, mode = a.mode;
  const int e = blockIdx.x / H, h = blockIdx.x % H;
  const Entry en = load_entry(a.ent, e);
  if (en.n <= 0) return;
  const bool trans = mode == 3;
  const int NCOL = trans ? D : V;              // columns of the matrix the wavefronts carry
  const int SST = trans ? D : VS;              // columns of a state row in memory
  constexpr int NI = (DKP + 63) / 64;          // normaliser channels per thread at most
  const int nw = blockDim.x >> 6, VP = nw * WC;
  extern __shared__ __align__(16) float smem[];
  float* sq = smem;                  // [CT][DKP]
  float* sk = sq + CT * DKP;
  float* sg = sk + CT * DKP;
  float* sv = sg + CT * DKP;         // [CT][VP]
  float* so = sv + CT * VP;          // [CT][VP]
  float* sb = so + CT * VP;          // [CT]
  float* sP = sb + CT;               // [DKP] product of the chunk's decays (mode 1, plain write)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int is = lane >> 4, i0 = is * DQ;
  int j[NC], jc[NC];
  bool act[NC];
#pragma unroll
  for (int c = 0; c < NC; c++) {
    j[c] = wave * WC + c * 16 + (lane & 15);
    act[c] = j[c] < NCOL;
    jc[c] = min(j[c], NCOL - 1);
  }
  const int hk = DELTA ? h / (H / a.G) : h;    // the q/k head this head reads
  const T* proj = (const T*)a.proj;
  const T* araw = (const T*)a.araw;
  const T* braw = (const T*)a.braw;
  const T* gate = (const T*)a.gate;
  T* out = (T*)a.out;
  float S[NC][DQ];
  float* Sg = mode == 0 ? a.state + ((size_t)en.slot * H + h) * D * VS
            : trans     ? a.chunk_trans + ((size_t)en.slot * H + h) * D * D
                        : a.chunk_state + ((size_t)en.slot * H + h) * D * VS;
  const bool from_state = mode == 2 || (mode == 0 && en.start > 0);
#pragma unroll
  for (int c = 0; c < NC; c++)
#pragma unroll
    for (int q = 0; q < DQ; q++) {
      // loads at clamped addresses, selected afterwards, so that they go out together
      float v0 = (trans && i0 + q == j[c]) ? 1.0f : 0.0f;
      float vv = from_state ? Sg[(size_t)min(i0 + q, D - 1) * SST + jc[c]] : v0;
      S[c][q] = (act[c] && i0 + q < D) ? vv : 0.0f;
    }
  float nr[NI];   // matrix memory: the normaliser's channels threadIdx.x + k * blockDim.x
#pragma unroll
  for (int k = 0; k < NI; k++) {
    int i = threadIdx.x + k * blockDim.x;
    nr[k] = (MEM && from_state && i < D) ? Sg[(size_t)i * SST + V] : 0.0f;
  }
  if (!DELTA && mode == 1)
    for (int i = threadIdx.x; i < DKP; i += blockDim.x) sP[i] = 1.0f;
  const float negA = DELTA ? -expf(a.A_log[h]) : 0.0f;
  const float qscale = (DELTA || MEM) ? 1.0f / sqrtf((float)D) : 1.0f;
  for (int t0 = 0; t0 < en.n; t0 += CT) {
    const int ct = min(CT, en.n - t0);
    for (int idx = threadIdx.x; idx < ct * DKP; idx += blockDim.x) {
      int t = idx / DKP, i = idx % DKP;
      float vq = 0.f, vk = 0.f, vg = 0.f;
      if (i < D) {
        size_t row = (size_t)(en.row0 + t0 + t);
        if (DELTA) {
          vq = a.conv[row * a.ldc + hk * D + i];
          vk = a.conv[row * a.ldc + a.G * D + hk * D + i];
          float dt = softplusf_(ldf(araw, row * a.lda + h * D + i) + a.dt_bias[h * D + i]);
          vg = expf(negA * dt);
        } else if (MEM) {
          const float* cf = a.coef + (row * H + h) * 3;
          vq = ldf(proj, row * a.ldp + h * D + i) * qscale;
          vk = cf[1] * ldf(proj, row * a.ldp + H * D + h * D + i);
          vg = cf[0];
        } else {
          float qr = ldf(proj, row * a.ldp + h * D + i);
          vq = qr * sigmoidf_(qr);
          float lo = a.lower[h * D + i];
          vg = lo + (1.0f - lo) * sigmoidf_(ldf(proj, row * a.ldp + H * D + h * D + i) + a.fb[h * D + i]);
          vk = 1.0f - vg;
        }
      }
      sq[idx] = vq; sk[idx] = vk; sg[idx] = vg;
    }
    if (!trans)
      for (int idx = threadIdx.x; idx < ct * VP; idx += blockDim.x) {
        int t = idx / VP, i = idx % VP;
        size_t row = (size_t)(en.row0 + t0 + t);
        float vv = 0.0f;
        if (i < V) vv = DELTA ? a.conv[row * a.ldc + 2 * a.G * D + h * V + i]
                              : ldf(proj, row * a.ldp + 2 * H * D + h * V + i);
        sv[idx] = vv;
      }
    if (DELTA) {
      for (int t = threadIdx.x; t < ct; t += blockDim.x)
        sb[t] = sigmoidf_(ldf(braw, (size_t)(en.row0 + t0 + t) * a.ldb + h));
      __syncthreads();
      // unit q and k: one wavefront per token
      for (int t = wave; t < ct; t += nw) {
        float s1 = 0.0f, s2 = 0.0f;
        for (int i = lane; i < D; i += 64) {
          float x = sq[t * DKP + i], y = sk[t * DKP + i];
          s1 += x * x;
          s2 += y * y;
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        float r1 = qscale / sqrtf(s1 + 1e-6f), r2 = 1.0f / sqrtf(s2 + 1e-6f);
        for (int i = lane; i < D; i += 64) {
          sq[t * DKP + i] *= r1;
          sk[t * DKP + i] *= r2;
        }
      }
    }
    __syncthreads();
    if (!DELTA && mode == 1)
      for (int i = threadIdx.x; i < D; i += blockDim.x) {
        float p = sP[i];
        for (int t = 0; t < ct; t++) p *= sg[t * DKP + i];
        sP[i] = p;
      }
    for (int t = 0; t < ct; t++) {   // every lane takes part (the shuffles need all of them)
      const float4* k4 = (const float4*)(sk + t * DKP + i0);
      const float4* g4 = (const float4*)(sg + t * DKP + i0);
      const float4* q4 = (const float4*)(sq + t * DKP + i0);
      float u[NC];
#pragma unroll
      for (int c = 0; c < NC; c++) u[c] = trans ? 0.0f : sv[t * VP + jc[c]];
      if (DELTA) {
        float d0[NC], d1[NC];   // two chains per column instead of one
#pragma unroll
        for (int c = 0; c < NC; c++) d0[c] = d1[c] = 0.0f;
#pragma unroll
        for (int q = 0; q < DQ / 4; q++) {
          float4 g = g4[q], k = k4[q];
#pragma unroll
          for (int c = 0; c < NC; c++) {
            S[c][4 * q] *= g.x; S[c][4 * q + 1] *= g.y; S[c][4 * q + 2] *= g.z; S[c][4 * q + 3] *= g.w;
            d0[c] += k.x * S[c][4 * q] + k.z * S[c][4 * q + 2];
            d1[c] += k.y * S[c][4 * q + 1] + k.w * S[c][4 * q + 3];
          }
        }
#pragma unroll
        for (int c = 0; c < NC; c++) {
          float d = d0[c] + d1[c];
          d += __shfl_xor(d, 16, 64);
          d += __shfl_xor(d, 32, 64);
          u[c] = sb[t] * (u[c] - d);
        }
      } else {
#pragma unroll
        for (int q = 0; q < DQ / 4; q++) {
          float4 g = g4[q];
#pragma unroll
          for (int c = 0; c < NC; c++) {
            S[c][4 * q] *= g.x; S[c][4 * q + 1] *= g.y; S[c][4 * q + 2] *= g.z; S[c][4 * q + 3] *= g.w;
          }
        }
      }
      float o0[NC], o1[NC];
#pragma unroll
      for (int c = 0; c < NC; c++) o0[c] = o1[c] = 0.0f;
#pragma unroll
      for (int q = 0; q < DQ / 4; q++) {
        float4 k = k4[q], qv = q4[q];
#pragma unroll
        for (int c = 0; c < NC; c++) {
          S[c][4 * q] += k.x * u[c]; S[c][4 * q + 1] += k.y * u[c];
          S[c][4 * q + 2] += k.z * u[c]; S[c][4 * q + 3] += k.w * u[c];
          o0[c] += S[c][4 * q] * qv.x + S[c][4 * q + 2] * qv.z;
          o1[c] += S[c][4 * q + 1] * qv.y + S[c][4 * q + 3] * qv.w;
        }
      }
      if (mode == 0 || mode == 2) {
#pragma unroll
        for (int c = 0; c < NC; c++) {
          float o = o0[c] + o1[c];
          o += __shfl_xor(o, 16, 64);
          o += __shfl_xor(o, 32, 64);
          if (is == 0) so[t * VP + j[c]] = act[c] ? o : 0.0f;
        }
      }
    }
    __syncthreads();
    if (MEM) {
      // the normaliser through the chunk's tokens; n_i q_i replaces q_i for the epilogue
#pragma unroll
      for (int k = 0; k < NI; k++) {
        int i = threadIdx.x + k * blockDim.x;
        if (i < D) {
          float n = nr[k];
          for (int t = 0; t < ct; t++) {
            n = sg[t * DKP + i] * n + sk[t * DKP + i];
            if (mode != 1) sq[t * DKP + i] *= n;
          }
          nr[k] = n;
        }
      }
      __syncthreads();
    }
    if (mode == 0 || mode == 2)
    for (int t = wave; t < ct; t += nw) {
      size_t row = (size_t)(en.row0 + t0 + t);
      float den = 1.0f;
      if (MEM) {
        float nq = 0.0f;
        for (int i = lane; i < D; i += 64) nq += sq[t * DKP + i];
        nq = wave_sum(nq);
        den = fmaxf(fabsf(nq), a.coef[(row * H + h) * 3 + 2]) + 1e-6f;
      }
      float ss = 0.0f;
      for (int i = lane; i < V; i += 64) {
        float o = MEM ? so[t * VP + i] / den : so[t * VP + i];
        ss += o * o;
      }
      ss = wave_sum(ss);
      float rs = a.out_scale / sqrtf(ss / (float)V + a.eps);
      for (int i = lane; i < V; i += 64) {
        float y;
        if (MEM) {
          y = so[t * VP + i] / den * rs * a.normw[h * V + i];
          y *= sigmoidf_(ldf(proj, row * a.ldp + 2 * H * D + H * V + h * V + i));
        } else {
          y = so[t * VP + i] * rs * a.normw[i];
          if (DELTA) y *= sigmoidf_(ldf(gate, row * a.ldg + h * V + i));
        }
        stf(out, row * a.ldo + h * V + i, y);
      }
    }
    // the next staging writes sq .. sb, whose readers passed the barrier above; `so` is
    // written again only after the next staging barrier, which every wave reaches after its
    // share of this chunk's outputs (the matrix memory's epilogue reads sq as well)
    if (MEM) __syncthreads();
  }
  if (mode != 2) {
#pragma unroll
    for (int c = 0; c < NC; c++)
      if (act[c]) {
#pragma unroll
        for (int q = 0; q < DQ; q++)
          if (i0 + q < D) Sg[(size_t)(i0 + q) * SST + j[c]] = S[c][q];
      }
    if (MEM) {
#pragma unroll
      for (int k = 0; k < NI; k++) {
        int i = threadIdx.x + k * blockDim.x;
        if (i < D) Sg[(size_t)i * SST + V] = nr[k];
      }
    }
  }
  if (!DELTA && mode == 1) {
    __syncthreads();
    for (int i = threadIdx.x; i < D; i += blockDim.x)
      a.chunk_decay[((size_t)en.slot * H + h) * D + i] = sP[i];
  }
}

// Chain of the plain write: the transition of a chunk is diagonal.  One thread per state
// element walks its portion's chunks: init_c replaces local_c in `cs`, the end goes to the slot.
__global__ void __launch_bounds__(256)
diag_chain_k(float* __restrict__ cs, const float* __restrict__ decay, float* __restrict__ state,
             const int* __restrict__ cent, int H, int D, int V) {
  const int e = blockIdx.y / H, h = blockIdx.y % H;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= D * V) return;
  const int i = idx / V;
  const int c0 = cent[4 * e], nc = cent[4 * e + 1], start = cent[4 * e + 2], slot = cent[4 * e + 3];
  float* sg = state + ((size_t)slot * H + h) * D * V + idx;
  float cur = start > 0 ? *sg : 0.0f;
  for (int c = c0; c < c0 + nc; c++) {
    float* p = cs + ((size_t)c * H + h) * D * V + idx;
    float local = *p;
    *p = cur;
    cur = decay[((size_t)c * H + h) * D + i] * cur + local;
  }
  *sg = cur;
}

// Chain of the delta rule: init_{c+1} = T_c . init_c + local_c with a dense D x D transition.
// The columns of the state are independent: one block per (portion, head, 8 columns), the
// current columns in LDS, thread (column, row group) forms every 32nd row of the product.
#define DC_COLS 8
#define DC_RG 32     // row groups: 256 threads / DC_COLS
#define DC_ROWS 8    // rows per thread at most (D <= 256)
__global__ void __launch_bounds__(256)
dense_chain_k(float* __restrict__ cs, const float* __restrict__ trans, float* __restrict__ state,
              const int* __restrict__ cent, int H, int D, int V) {
  extern __shared__ float scur[];   // [D][DC_COLS + 1]
  constexpr int LD = DC_COLS + 1;
  const int e = blockIdx.y / H, h = blockIdx.y % H;
  const int col = threadIdx.x % DC_COLS, rg = threadIdx.x / DC_COLS;
  const int j = blockIdx.x * DC_COLS + col;
  const bool act = j < V;
  const int jc = min(j, V - 1);
  const int c0 = cent[4 * e], nc = cent[4 * e + 1], start = cent[4 * e + 2], slot = cent[4 * e + 3];
  float* sg = state + ((size_t)slot * H + h) * D * V;
  for (int i = rg; i < D; i += DC_RG)
    scur[i * LD + col] = (start > 0 && act) ? sg[(size_t)i * V + jc] : 0.0f;
  __syncthreads();
  for (int c = c0; c < c0 + nc; c++) {
    float* loc = cs + ((size_t)c * H + h) * D * V;
    const float* Tc = trans + ((size_t)c * H + h) * D * D;
    float nv[DC_ROWS];
#pragma unroll
    for (int r = 0; r < DC_ROWS; r++) {
      int i = rg + DC_RG * r;
      if (i < D) {
        float acc0 = loc[(size_t)i * V + jc], acc1 = 0.0f;
        const float* Ti = Tc + (size_t)i * D;
        int k = 0;
        for (; k + 3 < D; k += 4) {
          acc0 += Ti[k] * scur[k * LD + col] + Ti[k + 2] * scur[(k + 2) * LD + col];
          acc1 += Ti[k + 1] * scur[(k + 1) * LD + col] + Ti[k + 3] * scur[(k + 3) * LD + col];
        }
        for (; k < D; k++) acc0 += Ti[k] * scur[k * LD + col];
        nv[r] = acc0 + acc1;
      }
    }
    __syncthreads();   // every thread has read the old columns
#pragma unroll
    for (int r = 0; r < DC_ROWS; r++) {
      int i = rg + DC_RG * r;
      if (i < D) {
        if (act) loc[(size_t)i * V + j] = scur[i * LD + col];   // init_c replaces local_c
        scur[i * LD + col] = nv[r];
      }
    }
    __syncthreads();
  }
  if (act)
    for (int i = rg; i < D; i += DC_RG) sg[(size_t)i * V + j] = scur[i * LD + col];
}

// Log gates of the matrix memory and their running maximum, one block per (portion, head):
//   i_t = cap tanh((zi_t + bi) / cap),  f_t = logsigmoid(cap tanh((zf_t + bf) / cap)),
//   m_t = max(f_t + m_(t-1), i_t)  (m = 0 before position 0; the slot keeps it between steps),
//   coef[t] = (exp(f_t + m_(t-1) - m_t), exp(i_t - m_t), exp(-m_t)).
// A token is the map m -> max(F + m, I) with (F, I) = (f_t, i_t); maps compose as
// (F2, I2) o (F1, I1) = (F1 + F2, max(I1 + F2, I2)).  Every wavefront takes 64 tokens: an
// inclusive scan of the maps by lane shuffles, the 64-token composite to LDS; one lane walks
// m through the composites of the block's wavefronts; then every lane applies its prefix map
// to the m at its group's start.  Any rounding of m only moves the scale on which S and n are
// kept: the coefficients are formed from the same m values, so S e^m and n e^m stay exact.
__device__ __forceinline__ float logsigmoidf_(float x) {
  return fminf(x, 0.0f) - log1pf(expf(-fabsf(x)));
}

template <typename T>
__global__ void __launch_bounds__(1024)
mlstm_gates_k(const T* __restrict__ proj, int ldp, int off_i, int off_f,
              const float* __restrict__ bi, const float* __restrict__ bf, float cap,
              float* __restrict__ mstate, const int* __restrict__ ent, float* __restrict__ coef,
              int H) {
  __shared__ float cF[16], cI[16], cM[17];
  const int e = blockIdx.x / H, h = blockIdx.x % H;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const Entry en = load_entry(ent, e);
  if (en.n <= 0) return;
  float* mg = mstate + (size_t)en.slot * H + h;
  float m0 = en.start > 0 ? *mg : 0.0f;
  const float bih = bi[h], bfh = bf[h];
  for (int t0 = 0; t0 < en.n; t0 += 64 * nw) {
    const int t = t0 + wave * 64 + lane;
    const bool ok = t < en.n;
    const size_t row = (size_t)(en.row0 + min(t, en.n - 1));
    float it = cap * tanhf((ldf(proj, row * ldp + off_i + h) + bih) / cap);
    float ft = logsigmoidf_(cap * tanhf((ldf(proj, row * ldp + off_f + h) + bfh) / cap));
    // tokens beyond the portion are the identity map
    float F = ok ? ft : 0.0f, I = ok ? it : -INFINITY;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      float Fp = __shfl_up(F, o, 64), Ip = __shfl_up(I, o, 64);
      if (lane >= o) {
        I = fmaxf(Ip + F, I);
        F = Fp + F;
      }
    }
    if (lane == 63) {
      cF[wave] = F;
      cI[wave] = I;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float mm = m0;
      for (int w = 0; w < nw; w++) {
        cM[w] = mm;
        mm = fmaxf(cF[w] + mm, cI[w]);
      }
      cM[nw] = mm;
    }
    __syncthreads();
    const float ms = cM[wave];              // m before this wavefront's first token
    float mn = fmaxf(F + ms, I);            // m_t
    float mp = __shfl_up(mn, 1, 64);        // m_(t-1)
    if (lane == 0) mp = ms;
    if (ok) {
      float* cf = coef + (row * H + h) * 3;
      cf[0] = expf(ft + mp - mn);
      cf[1] = expf(it - mn);
      cf[2] = expf(-mn);
    }
    m0 = cM[nw];
    __syncthreads();
  }
  if (threadIdx.x == 0) *mg = m0;
}

template <int KIND>
static int launch_scan(ScanArgs a, int E, int f32, hipStream_t st) {
  if (E <= 0) return 0;
  if (KIND != 2) a.VS = a.V;
  if (a.H < 1 || a.D < 1 || a.V < 1 || a.D > 256 || a.V > 256 || a.G < 1 || a.H % a.G)
    return (int)hipErrorInvalidValue;
  int cols = a.mode == 3 ? a.D : a.V;
  int dq = a.D <= 32 ? 8 : a.D <= 64 ? 16 : a.D <= 128 ? 32 : 64;
  // one column per lane: two (NC = 2) halve the wavefronts that read the staged vectors from
  // LDS but measured no faster (120 us against 110 us per 64-token pass at 128 x 128 states)
  const int nc = 1;
  int nw = (cols + 16 * nc - 1) / (16 * nc);
  int per_tok = 3 * 4 * dq + 2 * nw * 16 * nc + 1;
  int CT = 16;
  while (CT > 2 && (size_t)(CT * per_tok + 4 * dq) * 4 > 48 * 1024) CT /= 2;
  a.CT = CT;
  size_t shm = (size_t)(CT * per_tok + 4 * dq) * 4;
  dim3 grid(E * a.H), block(64 * nw);
#define GS(DQ, NC)                                                                            \
  SM_DISPATCH_T(f32, hipLaunchKernelGGL((gated_scan_k<T, DQ, KIND, NC>), grid, block, shm, st, a))
  if (dq == 8) GS(8, 1);
  else if (dq == 16) GS(16, 1);
  else if (dq == 32) GS(32, 1);
  else GS(64, 1);
#undef GS
  return (int)hipGetLastError();
}

// the three passes over `NV` chunks (vent) of `E` portions (cent = first chunk, chunks, first
// position, slot); cs [NV, H, D, V], cd [NV, H, D] (plain write) or ct [NV, H, D, D] (delta rule)
template <int KIND>
static int launch_chunked(ScanArgs a, const int* vent, int NV, const int* cent, int E, float* cs,
                          float* cd, float* ct, int f32, hipStream_t st) {
  constexpr bool DELTA = KIND == 1;
  if (NV <= 0 || E <= 0) return 0;
  if (KIND != 2) a.VS = a.V;
  float* state = a.state;
  a.ent = vent;
  a.chunk_state = cs; a.chunk_decay = cd; a.chunk_trans = ct;
  a.mode = 1;
  int err = launch_scan<KIND>(a, NV, f32, st);
  if (err) return err;
  if (DELTA) {
    a.mode = 3;
    if ((err = launch_scan<KIND>(a, NV, f32, st))) return err;
    hipLaunchKernelGGL(dense_chain_k, dim3((a.V + DC_COLS - 1) / DC_COLS, E * a.H), dim3(256),
                       (size_t)a.D * (DC_COLS + 1) * 4, st, cs, ct, state, cent, a.H, a.D, a.V);
  } else {
    hipLaunchKernelGGL(diag_chain_k, dim3((a.D * a.VS + 255) / 256, E * a.H), dim3(256), 0, st, cs,
                       cd, state, cent, a.H, a.D, a.VS);
  }
  if ((err = (int)hipGetLastError())) return err;
  a.mode = 2;
  return launch_scan<KIND>(a, NV, f32, st);
}

extern "C" {

int p2p_sm_hgrn2_scan(const void* proj, int ldp, const float* lower, const float* fb,
                      const float* normw, float* state, const int* ent, int E, void* out, int ldo,
                      int H, int D, int V, float eps, float out_scale, int f32, hipStream_t st) {
  ScanArgs a = {};
  a.proj = proj; a.ldp = ldp; a.lower = lower; a.fb = fb;
  a.normw = normw; a.state = state; a.ent = ent; a.out = out; a.ldo = ldo;
  a.H = H; a.G = H; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  return launch_scan<0>(a, E, f32, st);
}

int p2p_sm_gated_delta_scan(const float* conv, int ldc, const void* araw, int lda,
                            const void* braw, int ldb, const void* gate, int ldg,
                            const float* A_log, const float* dt_bias, const float* normw,
                            float* state, const int* ent, int E, void* out, int ldo, int H, int G,
                            int D, int V, float eps, float out_scale, int f32, hipStream_t st) {
  ScanArgs a = {};
  a.conv = conv; a.ldc = ldc; a.araw = araw; a.lda = lda; a.braw = braw; a.ldb = ldb;
  a.gate = gate; a.ldg = ldg; a.A_log = A_log; a.dt_bias = dt_bias;
  a.normw = normw; a.state = state; a.ent = ent; a.out = out; a.ldo = ldo;
  a.H = H; a.G = G; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  return launch_scan<1>(a, E, f32, st);
}

int p2p_sm_hgrn2_scan_chunked(const void* proj, int ldp, const float* lower, const float* fb,
                              const float* normw, float* state, float* cs, float* cd,
                              const int* vent, int NV, const int* cent, int E, void* out, int ldo,
                              int H, int D, int V, float eps, float out_scale, int f32,
                              hipStream_t st) {
  ScanArgs a = {};
  a.proj = proj; a.ldp = ldp; a.lower = lower; a.fb = fb;
  a.normw = normw; a.state = state; a.out = out; a.ldo = ldo;
  a.H = H; a.G = H; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  return launch_chunked<0>(a, vent, NV, cent, E, cs, cd, nullptr, f32, st);
}

int p2p_sm_gated_delta_scan_chunked(const float* conv, int ldc, const void* araw, int lda,
                                    const void* braw, int ldb, const void* gate, int ldg,
                                    const float* A_log, const float* dt_bias, const float* normw,
                                    float* state, float* cs, float* ct, const int* vent, int NV,
                                    const int* cent, int E, void* out, int ldo, int H, int G,
                                    int D, int V, float eps, float out_scale, int f32,
                                    hipStream_t st) {
  ScanArgs a = {};
  a.conv = conv; a.ldc = ldc; a.araw = araw; a.lda = lda; a.braw = braw; a.ldb = ldb;
  a.gate = gate; a.ldg = ldg; a.A_log = A_log; a.dt_bias = dt_bias;
  a.normw = normw; a.state = state; a.out = out; a.ldo = ldo;
  a.H = H; a.G = G; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  return launch_chunked<1>(a, vent, NV, cent, E, cs, nullptr, ct, f32, st);
}

// Matrix memory: proj = [q (H*D) | k (H*D) | v (H*V) | gate (H*V) | zi (H) | zf (H)] in the
// activation type; state fp32 [slots, H, D, V + 1] (column V: the normaliser), mstate fp32
// [slots, H]; coef fp32 [rows, H, 3] scratch; normw fp32 [H*V]; max_n: rows of the longest
// portion (sizes the gates' blocks).  With NV > 0 the portions run
// as chunks (vent / cent / cs [NV, H, D, V+1] / cd [NV, H, D]), else in one pass over `ent`.
int p2p_sm_mlstm_scan(const void* proj, int ldp, const float* bi, const float* bf, float cap,
                      const float* normw, float* state, float* mstate, float* coef,
                      const int* ent, int E, float* cs, float* cd, const int* vent, int NV,
                      const int* cent, void* out, int ldo, int H, int D, int V, float eps,
                      float out_scale, int max_n, int f32, hipStream_t st) {
  if (E <= 0) return 0;
  if (H < 1 || D < 1 || V < 1 || D > 256 || V > 256 || cap <= 0.0f) return (int)hipErrorInvalidValue;
  const int off_i = 2 * H * D + 2 * H * V, off_f = off_i + H;
  // wavefronts per (portion, head): one per 64 tokens of the longest portion, 16 at most
  const int gw = max(1, min(16, (max_n + 63) / 64));
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(mlstm_gates_k<T>, dim3(E * H), dim3(64 * gw), 0, st,
                                         (const T*)proj, ldp, off_i, off_f, bi, bf, cap, mstate,
                                         ent, coef, H));
  int err = (int)hipGetLastError();
  if (err) return err;
  ScanArgs a = {};
  a.proj = proj; a.ldp = ldp; a.coef = coef; a.VS = V + 1;
  a.normw = normw; a.state = state; a.ent = ent; a.out = out; a.ldo = ldo;
  a.H = H; a.G = H; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  if (NV > 0) return launch_chunked<2>(a, vent, NV, cent, E, cs, cd, nullptr, f32, st);
  return launch_scan<2>(a, E, f32, st);
}

}  // extern "C"
