// Generalized delta rule: per head a D x D fp32 state S (key index i, value index j),
//   S <- diag(w) S - (a * u)(u^T S) + k v^T,   o = S^T r,   u = k / sqrt(|k|^2 + 1e-6),
// decay and removal both applied to the state as it was before the token.  Value columns are independent, so one thread
// owns column j of S in registers and walks the tokens of its sequence portion in order;
// the per-token vectors (r, k, v, decay w, removal rate a) are staged through LDS a chunk
// of tokens at a time, with the decay and the rate evaluated while staging.  The head's
// outputs are RMS-normalised, weighted and gated as each chunk finishes.
#include "common.h"
using namespace sm;

#define GD_DECAY_SCALE 0.6065306597126334f  // exp(-1/2)

template <typename T, int DKP>
__global__ void __launch_bounds__(256)
gdelta_scan_k(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
              const T* __restrict__ g, const T* __restrict__ a, int ld,
              const T* __restrict__ lo, int ldlo, const float* __restrict__ w0,
              const float* __restrict__ ab, const float* __restrict__ normw,
              float* __restrict__ state, const int* __restrict__ ent, T* __restrict__ out,
              int ldo, int H, int D, float eps, int CT) {
  int e = blockIdx.x / H, h = blockIdx.x % H;
  Entry en = load_entry(ent, e);
  if (en.n <= 0) return;
  extern __shared__ float smem[];
  float* sr = smem;                 // [CT][DKP]
  float* sk = sr + CT * DKP;
  float* sv = sk + CT * DKP;
  float* sw = sv + CT * DKP;
  float* sa = sw + CT * DKP;
  float* so = sa + CT * DKP;
  int j = threadIdx.x;
  bool act = j < D;
  float S[DKP];
  float* Sg = state + ((size_t)en.slot * H + h) * D * D;
#pragma unroll
  for (int i = 0; i < DKP; i++) S[i] = (act && i < D && en.start > 0) ? Sg[(size_t)i * D + j] : 0.0f;
  int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int t0 = 0; t0 < en.n; t0 += CT) {
    int ct = min(CT, en.n - t0);
    for (int idx = threadIdx.x; idx < ct * DKP; idx += blockDim.x) {
      int t = idx / DKP, i = idx % DKP;
      float vr = 0.f, vk = 0.f, vv = 0.f, vw = 0.f, va = 0.f;
      if (i < D) {
        size_t row = (size_t)(en.row0 + t0 + t);
        int col = h * D + i;
        vr = ldf(r, row * ld + col);
        vk = ldf(k, row * ld + col);
        vv = ldf(v, row * ld + col);
        vw = expf(-GD_DECAY_SCALE * sigmoidf_(ldf(lo, row * ldlo + col) + w0[col]));
        va = sigmoidf_(ldf(a, row * ld + col) + ab[col]);
      }
      sr[idx] = vr; sk[idx] = vk; sv[idx] = vv; sw[idx] = vw; sa[idx] = va;
    }
    __syncthreads();
    if (act) {
      for (int t = 0; t < ct; t++) {
        const float* kr = sk + t * DKP;
        float kk = 0.0f, d = 0.0f;
#pragma unroll
        for (int i = 0; i < DKP; i++) {
          float ki = kr[i];
          kk += ki * ki;
          d += ki * S[i];
        }
        float rs = 1.0f / sqrtf(kk + 1e-6f);
        float dot = d * rs;            // u^T S (column j)
        float vj = sv[t * DKP + j];
        float o = 0.0f;
#pragma unroll
        for (int i = 0; i < DKP; i++) {
          float ki = kr[i];
          float ui = ki * rs;
          S[i] = sw[t * DKP + i] * S[i] - (sa[t * DKP + i] * ui) * dot + ki * vj;
          o += S[i] * sr[t * DKP + i];
        }
        so[t * DKP + j] = o;
      }
    }
    __syncthreads();
    for (int t = wave; t < ct; t += nw) {
      float ss = 0.0f;
      for (int i = lane; i < D; i += 64) ss += so[t * DKP + i] * so[t * DKP + i];
      ss = wave_sum(ss);
      float rs = 1.0f / sqrtf(ss / (float)D + eps);
      size_t row = (size_t)(en.row0 + t0 + t);
      for (int i = lane; i < D; i += 64) {
        int col = h * D + i;
        float gv = sigmoidf_(ldf(g, row * ld + col));
        stf(out, row * ldo + col, so[t * DKP + i] * rs * normw[col] * gv);
      }
    }
    // the next staging writes sr..sa (their readers passed the second barrier); `so` is
    // written again only after the next first barrier, which every wave reaches after its
    // share of this chunk's outputs
  }
  if (act) {
#pragma unroll
    for (int i = 0; i < DKP; i++)
      if (i < D) Sg[(size_t)i * D + j] = S[i];
  }
}

template <typename T, int DKP>
static int launch_gd(const void* r, const void* k, const void* v, const void* g, const void* a,
                     int ld, const void* lo, int ldlo, const float* w0, const float* ab,
                     const float* normw, float* state, const int* ent, int E, void* out, int ldo,
                     int H, int D, float eps, hipStream_t st) {
  int threads = ((D + 63) / 64) * 64;
  int CT = (48 * 1024) / (6 * DKP * 4);
  if (CT > 32) CT = 32;
  if (CT < 1) CT = 1;
  size_t shm = (size_t)6 * CT * DKP * 4;
  hipLaunchKernelGGL((gdelta_scan_k<T, DKP>), dim3(E * H), dim3(threads), shm, st, (const T*)r,
                     (const T*)k, (const T*)v, (const T*)g, (const T*)a, ld, (const T*)lo, ldlo,
                     w0, ab, normw, state, ent, (T*)out, ldo, H, D, eps, CT);
  return (int)hipGetLastError();
}

extern "C" int p2p_sm_gdelta_scan(const void* r, const void* k, const void* v, const void* g,
                                  const void* a, int ld, const void* lo, int ldlo,
                                  const float* w0, const float* ab, const float* normw,
                                  float* state, const int* ent, int E, void* out, int ldo, int H,
                                  int D, float eps, int f32, hipStream_t st) {
  if (E <= 0) return 0;
  if (D < 1 || D > 256) return (int)hipErrorInvalidValue;
#define GD(P)                                                                                   \
  SM_DISPATCH_T(f32, return (launch_gd<T, P>(r, k, v, g, a, ld, lo, ldlo, w0, ab, normw, state, \
                                             ent, E, out, ldo, H, D, eps, st)))
  if (D <= 32) GD(32);
  else if (D <= 64) GD(64);
  else if (D <= 128) GD(128);
  else GD(256);
#undef GD
  return 0;
}
