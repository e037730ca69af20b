// Generalized delta rule: per head a D x D fp32 state S (key index i, value index j),
//   S <- diag(w) S - (a * u)(u^T S) + k v^T,   o = S^T r,   u = k / sqrt(|k|^2 + 1e-6),
// decay and removal both applied to the state as it was before the token.  The value columns
// of S are independent; the state sits in registers and the tokens of a sequence portion are
// walked in order.  The per-token vectors (r, k, v, decay w, removal rate a) are staged
// through LDS a chunk of tokens at a time, with the decay and the rate evaluated while
// staging.  The head's outputs are RMS-normalised, weighted and gated as each chunk
// finishes.  Long portions run as chunks side by side (modes 1 and 2 + gdelta_combine_k).
#include "common.h"
using namespace sm;

#define GD_DECAY_SCALE 0.6065306597126334f  // exp(-1/2)

// Thread layout: a wavefront covers 16 value columns x 4 slices of the key index; lane
// (c, s) holds rows s * DQ .. s * DQ + DQ - 1 of column c.  The two sums a token needs over
// the whole key index (|k|^2 and u^T S before the update, S^T r after it) are finished with
// two lane shuffles, so a token costs DQ steps instead of D.
template <typename T, int DQ>
__global__ void __launch_bounds__(1024)
gdelta_scan_k(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v,
              const T* __restrict__ g, const T* __restrict__ a, int ld,
              const T* __restrict__ lo, int ldlo, const float* __restrict__ w0,
              const float* __restrict__ ab, const float* __restrict__ normw,
              float* __restrict__ state, const int* __restrict__ ent, T* __restrict__ out,
              int ldo, int H, int D, float eps, int CT, int mode, float* __restrict__ state2) {
  // mode 0: a portion from its slot's state (or zero at position 0), state written back.
  // mode 1: a chunk alone, no outputs: blockIdx.y = 0 runs it from a zero state and leaves the
  //         end state in state[slot]; blockIdx.y = 1 runs only the state transition on the
  //         identity (no k v^T term) and leaves the chunk's transition matrix in state2[slot].
  // mode 2: a chunk from state[slot], outputs only.
  constexpr int DKP = 4 * DQ;   // padded key index (zero filled in LDS)
  int e = blockIdx.x / H, h = blockIdx.x % H;
  const bool trans = mode == 1 && blockIdx.y == 1;
  Entry en = load_entry(ent, e);
  if (en.n <= 0) return;
  extern __shared__ float smem[];
  float* sr = smem;                 // [CT][DKP]
  float* sk = sr + CT * DKP;
  float* sv = sk + CT * DKP;
  float* sw = sv + CT * DKP;
  float* sa = sw + CT * DKP;
  float* so = sa + CT * DKP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int j = wave * 16 + (lane & 15), is = lane >> 4, i0 = is * DQ;
  const bool act = j < D;
  const int jc = min(j, D - 1);
  float S[DQ];
  float* Sg = (trans ? state2 : state) + ((size_t)en.slot * H + h) * D * D;
  const bool from_state = mode == 2 || (mode == 0 && en.start > 0);
#pragma unroll
  for (int q = 0; q < DQ; q++) {
    // loads at clamped addresses, selected afterwards: the loads stay independent of the
    // bounds tests and go out together
    float v0 = (trans && i0 + q == j) ? 1.0f : 0.0f;
    float vv = from_state ? Sg[(size_t)min(i0 + q, D - 1) * D + jc] : v0;
    S[q] = (act && i0 + q < D) ? vv : 0.0f;
  }
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
    for (int t = 0; t < ct; t++) {   // every lane takes part (the shuffles need all of them)
      const float* kr = sk + t * DKP + i0;
      float kk = 0.0f, d = 0.0f;
#pragma unroll
      for (int q = 0; q < DQ; q++) {
        float ki = kr[q];
        kk += ki * ki;
        d += ki * S[q];
      }
      kk += __shfl_xor(kk, 16, 64);
      d += __shfl_xor(d, 16, 64);
      kk += __shfl_xor(kk, 32, 64);
      d += __shfl_xor(d, 32, 64);
      float rs = 1.0f / sqrtf(kk + 1e-6f);
      float dot = d * rs;            // u^T S (column j)
      float vj = trans ? 0.0f : sv[t * DKP + jc];
      float o = 0.0f;
#pragma unroll
      for (int q = 0; q < DQ; q++) {
        float ki = kr[q];
        float ui = ki * rs;
        S[q] = sw[t * DKP + i0 + q] * S[q] - (sa[t * DKP + i0 + q] * ui) * dot + ki * vj;
        o += S[q] * sr[t * DKP + i0 + q];
      }
      o += __shfl_xor(o, 16, 64);
      o += __shfl_xor(o, 32, 64);
      if (is == 0 && act) so[t * DKP + j] = o;
    }
    __syncthreads();
    if (mode != 1)
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
  if (act && mode != 2) {
#pragma unroll
    for (int q = 0; q < DQ; q++)
      if (i0 + q < D) Sg[(size_t)(i0 + q) * D + j] = S[q];
  }
}

// Chains the chunks of each portion: init_{c+1} = trans_c . init_c + local_c (D x D products
// on the key index).  One block per (portion, head), one thread per value column.  `init`
// receives init_c for every chunk, the portion's slot its final state.
template <int DKP>
__global__ void __launch_bounds__(256)
gdelta_combine_k(const float* __restrict__ local, const float* __restrict__ trans,
                 float* __restrict__ init, float* __restrict__ state,
                 const int* __restrict__ cent, int H, int D, int TI) {
  extern __shared__ float sP[];   // [TI (+3)][DS] rows of the transition matrix, zero padded
  const int DS = (D + 3) & ~3;
  int e = blockIdx.x / H, h = blockIdx.x % H;
  int c0 = cent[4 * e], nc = cent[4 * e + 1], start = cent[4 * e + 2], slot = cent[4 * e + 3];
  // the block is NW groups of TD threads: every group holds all columns (thread j of a
  // group owns column j) and takes every NW-th set of four rows
  const int TD = ((D + 63) / 64) * 64, NW = blockDim.x / TD;
  int j = threadIdx.x % TD, w = threadIdx.x / TD;
  bool act = j < D;
  int jc = min(j, D - 1);
  size_t DD = (size_t)D * D;
  float* sg = state + ((size_t)slot * H + h) * DD;
  float cur[DKP];
#pragma unroll
  for (int k = 0; k < DKP; k++) {
    float v = start > 0 ? sg[(size_t)min(k, D - 1) * D + jc] : 0.0f;
    cur[k] = (act && k < D) ? v : 0.0f;
  }
  __syncthreads();   // every group has read the slot before a single-chunk portion rewrites it
  for (int c = c0; c < c0 + nc; c++) {
    size_t off = ((size_t)c * H + h) * DD;
    if (act && w == 0) {
#pragma unroll
      for (int k = 0; k < DKP; k++)
        if (k < D) init[off + (size_t)k * D + j] = cur[k];
    }
    float* dst = (c + 1 < c0 + nc) ? init + ((size_t)(c + 1) * H + h) * DD : sg;
    for (int i0 = 0; i0 < D; i0 += TI) {
      int ti = min(TI, D - i0);
      __syncthreads();
      for (int idx = threadIdx.x; idx < (ti + 3) * DS; idx += blockDim.x) {
        int i = idx / DS, k = idx % DS;
        sP[idx] = (i < ti && k < D) ? trans[off + (size_t)(i0 + i) * D + k] : 0.0f;
      }
      __syncthreads();
      if (act) {
        for (int i = 4 * w; i < ti; i += 4 * NW) {   // four rows at a time: independent sums
          float a[4];
#pragma unroll
          for (int u = 0; u < 4; u++)
            a[u] = local[off + (size_t)min(i0 + i + u, D - 1) * D + j];
#pragma unroll
          for (int k = 0; k < DKP; k += 4) {
            if (k < DS) {
#pragma unroll
              for (int u = 0; u < 4; u++) {
                const float4 p = *(const float4*)(sP + (i + u) * DS + k);
                a[u] += p.x * cur[k] + p.y * cur[k + 1] + p.z * cur[k + 2] + p.w * cur[k + 3];
              }
            }
          }
#pragma unroll
          for (int u = 0; u < 4; u++)
            if (i + u < ti) dst[(size_t)(i0 + i + u) * D + j] = a[u];
        }
      }
    }
    __syncthreads();   // the groups' rows of the new state are all written
#pragma unroll
    for (int k = 0; k < DKP; k++) {
      float v = dst[(size_t)min(k, D - 1) * D + jc];   // column j, written by this block
      cur[k] = (act && k < D) ? v : 0.0f;
    }
  }
}

template <typename T, int DQ>
static int launch_gd(const void* r, const void* k, const void* v, const void* g, const void* a,
                     int ld, const void* lo, int ldlo, const float* w0, const float* ab,
                     const float* normw, float* state, const int* ent, int E, void* out, int ldo,
                     int H, int D, float eps, int mode, float* state2, hipStream_t st) {
  constexpr int DKP = 4 * DQ;
  int threads = ((D + 15) / 16) * 64;   // a wavefront per 16 value columns
  int CT = (48 * 1024) / (6 * DKP * 4);
  if (CT > 32) CT = 32;
  if (CT < 1) CT = 1;
  size_t shm = (size_t)6 * CT * DKP * 4;
  hipLaunchKernelGGL((gdelta_scan_k<T, DQ>), dim3(E * H, mode == 1 ? 2 : 1), dim3(threads), shm,
                     st, (const T*)r, (const T*)k, (const T*)v, (const T*)g, (const T*)a, ld,
                     (const T*)lo, ldlo, w0, ab, normw, state, ent, (T*)out, ldo, H, D, eps, CT,
                     mode, state2);
  return (int)hipGetLastError();
}

extern "C" {

int p2p_sm_gdelta_scan_mode(const void* r, const void* k, const void* v, const void* g,
                            const void* a, int ld, const void* lo, int ldlo, const float* w0,
                            const float* ab, const float* normw, float* state, const int* ent,
                            int E, void* out, int ldo, int H, int D, float eps, int mode,
                            float* state2, int f32, hipStream_t st) {
  if (E <= 0) return 0;
  if (D < 1 || D > 256) return (int)hipErrorInvalidValue;
#define GD(P)                                                                                   \
  SM_DISPATCH_T(f32, return (launch_gd<T, P>(r, k, v, g, a, ld, lo, ldlo, w0, ab, normw, state, \
                                             ent, E, out, ldo, H, D, eps, mode, state2, st)))
  if (D <= 32) GD(8);
  else if (D <= 64) GD(16);
  else if (D <= 128) GD(32);
  else GD(64);
#undef GD
  return 0;
}

int p2p_sm_gdelta_scan(const void* r, const void* k, const void* v, const void* g, const void* a,
                       int ld, const void* lo, int ldlo, const float* w0, const float* ab,
                       const float* normw, float* state, const int* ent, int E, void* out,
                       int ldo, int H, int D, float eps, int f32, hipStream_t st) {
  return p2p_sm_gdelta_scan_mode(r, k, v, g, a, ld, lo, ldlo, w0, ab, normw, state, ent, E, out,
                                 ldo, H, D, eps, 0, nullptr, f32, st);
}

// Long portions in chunks that run side by side: every chunk's local end state and transition
// matrix, a chain over each portion's chunks, then every chunk again from its true initial
// state.  vent: the chunks as entries (row0, n, 1, chunk index); tmp: 3 fp32 buffers of
// [chunks, H, D, D] (local, transition, init); cent: per portion (first chunk, chunks, first
// position, slot).
int p2p_sm_gdelta_scan_chunked(const void* r, const void* k, const void* v, const void* g,
                               const void* a, int ld, const void* lo, int ldlo, const float* w0,
                               const float* ab, const float* normw, float* state, float* tmp,
                               const int* vent, int NV, const int* cent, int E, void* out,
                               int ldo, int H, int D, float eps, int f32, hipStream_t st) {
  if (E <= 0 || NV <= 0) return 0;
  size_t sz = (size_t)NV * H * D * D;
  float *loc = tmp, *trn = tmp + sz, *ini = tmp + 2 * sz;
  int err = p2p_sm_gdelta_scan_mode(r, k, v, g, a, ld, lo, ldlo, w0, ab, normw, loc, vent, NV, out,
                                    ldo, H, D, eps, 1, trn, f32, st);
  if (err) return err;
  int threads = ((D + 63) / 64) * 64;
  int DS = (D + 3) & ~3;
  int TI = ((32 * 1024) / (DS * 4)) & ~3;
  if (TI > D) TI = D;
  if (TI < 4) TI = 4;
  size_t shm = (size_t)(TI + 3) * DS * 4;
  int nw = 256 / threads;   // groups of `threads` per block
#define GC(P) hipLaunchKernelGGL((gdelta_combine_k<P>), dim3(E * H), dim3(threads * nw), shm, st, loc, trn, ini, state, cent, H, D, TI)
  if (D <= 32) GC(32);
  else if (D <= 64) GC(64);
  else if (D <= 128) GC(128);
  else GC(256);
#undef GC
  err = (int)hipGetLastError();
  if (err) return err;
  return p2p_sm_gdelta_scan_mode(r, k, v, g, a, ld, lo, ldlo, w0, ab, normw, ini, vent, NV, out,
                                 ldo, H, D, eps, 2, nullptr, f32, st);
}

}  // extern "C"
