// Gated linear scans: per head a D x V fp32 state S (key channel i, value channel j) and one
// step per token,
//   S <- diag(g) S
//   u = v                        plain write   (HGRN2: g = f, k = 1 - f)
//   u = beta * (v - S^T k)       delta rule    (the write corrects what the key reads)
//   S <- S + k u^T,  o = S^T q   (the read-out sees the token's own write)
// followed by the head's RMS norm over V, a weight shared by the heads and, for the delta
// rule, a sigmoid output gate.
//
// The value columns of S are independent.  A wavefront covers 16 columns x 4 slices of the key
// index; lane (c, s) keeps rows s*DQ .. s*DQ+DQ-1 of column c in registers, and the sums over
// the key index (S^T k before the write, S^T q after it) are finished with two lane shuffles.
// The tokens of a sequence portion are walked in order; their vectors are staged through LDS
// a chunk at a time and everything that enters the recurrence is evaluated in fp32 while
// staging: HGRN2's silu(q) and f = lower + (1 - lower) sigmoid(. + b); the delta rule's unit q
// and k (x / sqrt(|x|^2 + 1e-6), q also times D^-1/2), beta = sigmoid(.) and the decay
// g = exp(-exp(A_log_h) softplus(. + dt_bias)).
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
  // common
  const float* normw; float* state; const int* ent; void* out; int ldo;
  int H, G, D, V, CT;
  float eps, out_scale;
};

template <typename T, int DQ, bool DELTA>
__global__ void __launch_bounds__(1024) gated_scan_k(ScanArgs a) {
  constexpr int DKP = 4 * DQ;   // padded key index (zero filled in LDS)
  const int H = a.H, D = a.D, V = a.V, CT = a.CT;
  const int e = blockIdx.x / H, h = blockIdx.x % H;
  const Entry en = load_entry(a.ent, e);
  if (en.n <= 0) return;
  const int nw = blockDim.x >> 6, VP = nw * 16;
  extern __shared__ float smem[];
  float* sq = smem;                  // [CT][DKP]
  float* sk = sq + CT * DKP;
  float* sg = sk + CT * DKP;
  float* sv = sg + CT * DKP;         // [CT][VP]
  float* so = sv + CT * VP;          // [CT][VP]
  float* sb = so + CT * VP;          // [CT]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = wave * 16 + (lane & 15), is = lane >> 4, i0 = is * DQ;
  const bool act = j < V;
  const int jc = min(j, V - 1);
  const int hk = DELTA ? h / (H / a.G) : h;    // the q/k head this head reads
  const T* proj = (const T*)a.proj;
  const T* araw = (const T*)a.araw;
  const T* braw = (const T*)a.braw;
  const T* gate = (const T*)a.gate;
  T* out = (T*)a.out;
  float S[DQ];
  float* Sg = a.state + ((size_t)en.slot * H + h) * D * V;
#pragma unroll
  for (int q = 0; q < DQ; q++) {
    // loads at clamped addresses, selected afterwards, so that they go out together
    float vv = en.start > 0 ? Sg[(size_t)min(i0 + q, D - 1) * V + jc] : 0.0f;
    S[q] = (act && i0 + q < D) ? vv : 0.0f;
  }
  const float negA = DELTA ? -expf(a.A_log[h]) : 0.0f;
  const float qscale = DELTA ? 1.0f / sqrtf((float)D) : 1.0f;
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
    for (int t = 0; t < ct; t++) {   // every lane takes part (the shuffles need all of them)
      const float* kr = sk + t * DKP + i0;
      const float* gr = sg + t * DKP + i0;
      const float* qr = sq + t * DKP + i0;
      float u = sv[t * VP + jc];
      if (DELTA) {
        float d = 0.0f;
#pragma unroll
        for (int q = 0; q < DQ; q++) {
          S[q] *= gr[q];
          d += kr[q] * S[q];
        }
        d += __shfl_xor(d, 16, 64);
        d += __shfl_xor(d, 32, 64);
        u = sb[t] * (u - d);
      } else {
#pragma unroll
        for (int q = 0; q < DQ; q++) S[q] *= gr[q];
      }
      float o = 0.0f;
#pragma unroll
      for (int q = 0; q < DQ; q++) {
        S[q] += kr[q] * u;
        o += S[q] * qr[q];
      }
      o += __shfl_xor(o, 16, 64);
      o += __shfl_xor(o, 32, 64);
      if (is == 0) so[t * VP + j] = act ? o : 0.0f;
    }
    __syncthreads();
    for (int t = wave; t < ct; t += nw) {
      float ss = 0.0f;
      for (int i = lane; i < V; i += 64) ss += so[t * VP + i] * so[t * VP + i];
      ss = wave_sum(ss);
      float rs = a.out_scale / sqrtf(ss / (float)V + a.eps);
      size_t row = (size_t)(en.row0 + t0 + t);
      for (int i = lane; i < V; i += 64) {
        float y = so[t * VP + i] * rs * a.normw[i];
        if (DELTA) y *= sigmoidf_(ldf(gate, row * a.ldg + h * V + i));
        stf(out, row * a.ldo + h * V + i, y);
      }
    }
    // the next staging writes sq .. sb, whose readers passed the barrier above; `so` is
    // written again only after the next staging barrier, which every wave reaches after its
    // share of this chunk's outputs
  }
  if (act) {
#pragma unroll
    for (int q = 0; q < DQ; q++)
      if (i0 + q < D) Sg[(size_t)(i0 + q) * V + j] = S[q];
  }
}

template <bool DELTA>
static int launch_scan(ScanArgs a, int E, int f32, hipStream_t st) {
  if (E <= 0) return 0;
  if (a.H < 1 || a.D < 1 || a.V < 1 || a.D > 256 || a.V > 256 || a.G < 1 || a.H % a.G)
    return (int)hipErrorInvalidValue;
  int nw = (a.V + 15) / 16;
  int dq = a.D <= 32 ? 8 : a.D <= 64 ? 16 : a.D <= 128 ? 32 : 64;
  int per_tok = 3 * 4 * dq + 2 * nw * 16 + 1;
  int CT = 16;
  while (CT > 2 && (size_t)CT * per_tok * 4 > 48 * 1024) CT /= 2;
  a.CT = CT;
  size_t shm = (size_t)CT * per_tok * 4;
  dim3 grid(E * a.H), block(64 * nw);
#define GS(DQ)                                                                              \
  SM_DISPATCH_T(f32, hipLaunchKernelGGL((gated_scan_k<T, DQ, DELTA>), grid, block, shm, st, a))
  if (dq == 8) GS(8);
  else if (dq == 16) GS(16);
  else if (dq == 32) GS(32);
  else GS(64);
#undef GS
  return (int)hipGetLastError();
}

extern "C" {

int p2p_sm_hgrn2_scan(const void* proj, int ldp, const float* lower, const float* fb,
                      const float* normw, float* state, const int* ent, int E, void* out, int ldo,
                      int H, int D, int V, float eps, float out_scale, int f32, hipStream_t st) {
  ScanArgs a = {};
  a.proj = proj; a.ldp = ldp; a.lower = lower; a.fb = fb;
  a.normw = normw; a.state = state; a.ent = ent; a.out = out; a.ldo = ldo;
  a.H = H; a.G = H; a.D = D; a.V = V; a.eps = eps; a.out_scale = out_scale;
  return launch_scan<false>(a, E, f32, st);
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
  return launch_scan<true>(a, E, f32, st);
}

}  // extern "C"
