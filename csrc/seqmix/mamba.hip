// Mamba-2 (state-space duality) layer pieces.
//   conv : causal per-channel convolution over the x|B|C channels + bias + silu; the inputs
//          before a portion's first token come from the sequence's saved tail (the last
//          taps-1 raw inputs), or are zero at the start of a sequence.
//   scan : per head an N x P fp32 state, S <- exp(-exp(A_log) dt) S + dt B x^T,
//          y = S^T C + D x, y *= silu(z); dt = softplus(raw + bias).  The state sits in
//          registers (a thread holds a run of state rows of one value column); B, C, x, z,
//          dt of a chunk of tokens go through LDS.  Long portions run as chunks side by
//          side (modes 1 and 2 + mamba_combine_k).
//   tail : rolls the convolution tail forward after the scan.
#include "common.h"
using namespace sm;

template <typename T>
__global__ void mamba_conv_k(const T* __restrict__ zx, int ldz, int xoff,
                             const float* __restrict__ cw, const float* __restrict__ cb,
                             const float* __restrict__ tail, const int* __restrict__ ent,
                             const int* __restrict__ row_ent, float* __restrict__ out, int R,
                             int C, int K) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  int r = blockIdx.y;
  if (c >= C) return;
  Entry en = load_entry(ent, row_ent[r]);
  int t = r - en.row0;
  float acc = cb[c];
  for (int kk = 0; kk < K; kk++) {
    int q = t - (K - 1) + kk;
    float val = 0.0f;
    if (q >= 0) val = ldf(zx, (size_t)(en.row0 + q) * ldz + xoff + c);
    else if (en.start > 0) val = tail[((size_t)en.slot * (K - 1) + (K - 1 + q)) * C + c];
    acc += cw[(size_t)c * K + kk] * val;
  }
  out[(size_t)r * C + c] = acc * sigmoidf_(acc);
}

// One thread owns NSUB consecutive state rows of one value column: thread (p, ns) holds
// S[ns * NSUB + q][p].  Per token it updates them and leaves its share of y = S^T C in LDS;
// the shares are added, D x and the gate applied, once per staged chunk of tokens.
template <typename T, int NSUB>
__global__ void __launch_bounds__(1024)
mamba_scan_k(const float* __restrict__ conv, int C, const T* __restrict__ zx, int ldz, int xoff,
             int dtoff, const float* __restrict__ dt_bias, const float* __restrict__ A_log,
             const float* __restrict__ Dp, float* __restrict__ state, float* __restrict__ tail,
             const int* __restrict__ ent, float* __restrict__ y, int H, int P, int N, int G,
             int K, int CT, int mode, float* __restrict__ decay_out, int TP, int NS) {
  // mode 0: a portion from its slot's state (or zero at position 0), state written back.
  // mode 1: a chunk from a zero state: no outputs; the end state goes to `state[slot]` and
  //         the product of the chunk's decays to decay_out[entry, head].
  // mode 2: a chunk from `state[slot]`, outputs only.
  int e = blockIdx.x / H, h = blockIdx.x % H;
  Entry en = load_entry(ent, e);
  if (en.n <= 0) return;
  extern __shared__ float smem[];
  const int NPAD = NS * NSUB;
  float* sB = smem;                  // [CT][NPAD]
  float* sC = sB + CT * NPAD;        // [CT][NPAD]
  float* sx = sC + CT * NPAD;        // [CT][P]
  float* sz = sx + CT * P;           // [CT][P]
  float* sy = sz + CT * P;           // [CT][NS][P] shares of y
  float* sdt = sy + CT * NS * P;     // [CT]
  float* sdA = sdt + CT;             // [CT]
  int inner = H * P;
  int g = h / (H / G);
  const int p = threadIdx.x % TP, ns = threadIdx.x / TP;
  const bool act = p < P;
  const int n0 = ns * NSUB;
  float S[NSUB];
  float* Sg = state + ((size_t)en.slot * H + h) * N * P;
  const bool from_state = mode == 2 || (mode == 0 && en.start > 0);
#pragma unroll
  for (int q = 0; q < NSUB; q++) {
    // loads at clamped addresses, selected afterwards: the loads stay independent of the
    // bounds tests and go out together
    float v = from_state ? Sg[(size_t)min(n0 + q, N - 1) * P + min(p, P - 1)] : 0.0f;
    S[q] = (act && n0 + q < N) ? v : 0.0f;
  }
  float A = -expf(A_log[h]), Dh = Dp[h], bias = dt_bias[h];
  float dtsum = 0.0f;
  for (int t0 = 0; t0 < en.n; t0 += CT) {
    int ct = min(CT, en.n - t0);
    __syncthreads();   // the previous chunk's outputs have been read
    for (int idx = threadIdx.x; idx < ct * NPAD; idx += blockDim.x) {
      int t = idx / NPAD, n = idx % NPAD;
      size_t row = (size_t)(en.row0 + t0 + t);
      float b = 0.f, c = 0.f;
      if (n < N) {
        b = conv[row * C + inner + g * N + n];
        c = conv[row * C + inner + G * N + g * N + n];
      }
      sB[idx] = b; sC[idx] = c;
    }
    for (int idx = threadIdx.x; idx < ct * P; idx += blockDim.x) {
      int t = idx / P, q = idx % P;
      size_t row = (size_t)(en.row0 + t0 + t);
      sx[idx] = conv[row * C + h * P + q];
      sz[idx] = ldf(zx, row * ldz + h * P + q);
    }
    for (int t = threadIdx.x; t < ct; t += blockDim.x) {
      size_t row = (size_t)(en.row0 + t0 + t);
      float dt = softplusf_(ldf(zx, row * ldz + dtoff + h) + bias);
      sdt[t] = dt;
      sdA[t] = expf(A * dt);
    }
    __syncthreads();
    if (act) {
      for (int t = 0; t < ct; t++) {
        float dA = sdA[t];
        float dx = sdt[t] * sx[t * P + p];
        dtsum += sdt[t];
        const float* bb = sB + t * NPAD + n0;
        const float* cc = sC + t * NPAD + n0;
        float acc = 0.0f;
#pragma unroll
        for (int q = 0; q < NSUB; q++) {
          S[q] = dA * S[q] + dx * bb[q];
          acc += S[q] * cc[q];
        }
        sy[(t * NS + ns) * P + p] = acc;
      }
    }
    __syncthreads();
    if (mode != 1) {
      for (int idx = threadIdx.x; idx < ct * P; idx += blockDim.x) {
        int t = idx / P, q = idx % P;
        float acc = 0.0f;
        for (int k = 0; k < NS; k++) acc += sy[(t * NS + k) * P + q];
        acc += Dh * sx[idx];
        float z = sz[idx];
        y[(size_t)(en.row0 + t0 + t) * inner + h * P + q] = acc * (z * sigmoidf_(z));
      }
    }
  }
  if (act && mode != 2) {
#pragma unroll
    for (int q = 0; q < NSUB; q++)
      if (n0 + q < N) Sg[(size_t)(n0 + q) * P + p] = S[q];
  }
  if (mode == 1 && threadIdx.x == 0) decay_out[(size_t)e * H + h] = expf(A * dtsum);
}

// Chains the chunks of each portion: chunk c starts from init_c, init_{c+1} = decay_c * init_c
// + local_c.  `tmp` holds local_c on entry and init_c on exit; the portion's final state goes
// to its slot.  cent: per portion (first chunk, chunks, first position, slot).
__global__ void mamba_combine_k(float* __restrict__ tmp, const float* __restrict__ decay,
                                float* __restrict__ state, const int* __restrict__ cent, int H,
                                int NPsz) {
  int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= NPsz) return;
  int h = blockIdx.y, e = blockIdx.z;
  int c0 = cent[4 * e], nc = cent[4 * e + 1], start = cent[4 * e + 2], slot = cent[4 * e + 3];
  float* sg = state + ((size_t)slot * H + h) * NPsz + idx;
  float cur = start > 0 ? *sg : 0.0f;
  for (int c = c0; c < c0 + nc; c++) {
    float* t = tmp + ((size_t)c * H + h) * NPsz + idx;
    float loc = *t;
    *t = cur;
    cur = decay[(size_t)c * H + h] * cur + loc;
  }
  *sg = cur;
}

// new tail = the last K-1 raw inputs of (old tail ++ this portion): one thread per (entry,
// channel); slot j reads old slot j + n or a row of the portion, so ascending j never reads
// a slot it has already written
template <typename T>
__global__ void mamba_tail_k(const T* __restrict__ zx, int ldz, int xoff, float* __restrict__ tail,
                             const int* __restrict__ ent, int C, int K) {
  int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  Entry en = load_entry(ent, blockIdx.y);
  if (en.n <= 0) return;
  float* tl = tail + (size_t)en.slot * (K - 1) * C;
  for (int j = 0; j < K - 1; j++) {
    int q = en.n + j - (K - 1);
    float val;
    if (q >= 0) val = ldf(zx, (size_t)(en.row0 + q) * ldz + xoff + c);
    else val = en.start > 0 ? tl[(size_t)(K - 1 + q) * C + c] : 0.0f;
    tl[(size_t)j * C + c] = val;
  }
}

template <typename T, int NSUB>
static int launch_ms(const float* conv, int C, const void* zx, int ldz, int xoff, int dtoff,
                     const float* dt_bias, const float* A_log, const float* Dp, float* state,
                     float* tail, const int* ent, int E, float* y, int H, int P, int N, int G,
                     int K, int mode, float* decay_out, hipStream_t st) {
  int TP = ((P + 63) / 64) * 64;
  int NS = (N + NSUB - 1) / NSUB;
  int per = 2 * NS * NSUB + 2 * P + NS * P + 2;
  int CT = (48 * 1024) / (per * 4);
  if (CT > 32) CT = 32;
  if (CT < 1) CT = 1;
  size_t shm = (size_t)CT * per * 4;
  hipLaunchKernelGGL((mamba_scan_k<T, NSUB>), dim3(E * H), dim3(TP * NS), shm, st, conv, C,
                     (const T*)zx, ldz, xoff, dtoff, dt_bias, A_log, Dp, state, tail, ent, y, H,
                     P, N, G, K, CT, mode, decay_out, TP, NS);
  return (int)hipGetLastError();
}

extern "C" {

int p2p_sm_mamba_conv(const void* zx, int ldz, int xoff, const float* cw, const float* cb,
                      const float* tail, const int* ent, const int* row_ent, float* out, int R,
                      int C, int K, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  dim3 g((C + 255) / 256, R), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(mamba_conv_k<T>, g, b, 0, st, (const T*)zx, ldz, xoff, cw,
                                         cb, tail, ent, row_ent, out, R, C, K));
  return (int)hipGetLastError();
}

int p2p_sm_mamba_scan_mode(const float* conv, int C, const void* zx, int ldz, int xoff,
                           int dtoff, const float* dt_bias, const float* A_log, const float* Dp,
                           float* state, float* tail, const int* ent, int E, float* y, int H,
                           int P, int N, int G, int K, int mode, float* decay_out, int f32,
                           hipStream_t st) {
  if (E <= 0) return 0;
  if (N < 1 || N > 256 || P < 1 || P > 256 || G < 1 || H % G) return (int)hipErrorInvalidValue;
#define MS(NPV)                                                                               \
  SM_DISPATCH_T(f32, return (launch_ms<T, NPV>(conv, C, zx, ldz, xoff, dtoff, dt_bias, A_log, \
                                               Dp, state, tail, ent, E, y, H, P, N, G, K, mode, \
                                               decay_out, st)))
  // state rows per thread: 32 where the block (value columns x row slices) fits 1024 threads
  int TPv = ((P + 63) / 64) * 64;
  // (value and state sizes are at most 256, so 64 rows per thread always fit)
  if (TPv * ((N + 31) / 32) <= 1024) MS(32);
  else MS(64);
#undef MS
  return 0;
}

int p2p_sm_mamba_scan(const float* conv, int C, const void* zx, int ldz, int xoff, int dtoff,
                      const float* dt_bias, const float* A_log, const float* Dp, float* state,
                      float* tail, const int* ent, int E, float* y, int H, int P, int N, int G,
                      int K, int f32, hipStream_t st) {  return p2p_sm_mamba_scan_mode(conv, C, zx, ldz, xoff, dtoff, dt_bias, A_log, Dp, state, tail,
                                ent, E, y, H, P, N, G, K, 0, nullptr, f32, st);
}

// Long portions in chunks that run side by side: local states of every chunk from zero, a
// chain over each portion's chunks, then every chunk again from its true initial state.
// vent: the chunks as entries (row0, n, 1, chunk index); tmp fp32 [chunks, H, N, P];
// decay fp32 [chunks, H]; cent: see mamba_combine_k.
int p2p_sm_mamba_scan_chunked(const float* conv, int C, const void* zx, int ldz, int xoff,
                              int dtoff, const float* dt_bias, const float* A_log,
                              const float* Dp, float* state, float* tmp, float* decay,
                              const int* vent, int NV, const int* cent, int E, float* y, int H,
                              int P, int N, int G, int f32, hipStream_t st) {
  if (E <= 0 || NV <= 0) return 0;
  int err = p2p_sm_mamba_scan_mode(conv, C, zx, ldz, xoff, dtoff, dt_bias, A_log, Dp, tmp,
                                   nullptr, vent, NV, y, H, P, N, G, 1, 1, decay, f32, st);
  if (err) return err;
  dim3 g((N * P + 255) / 256, H, E);
  hipLaunchKernelGGL(mamba_combine_k, g, dim3(256), 0, st, tmp, decay, state, cent, H, N * P);
  err = (int)hipGetLastError();
  if (err) return err;
  return p2p_sm_mamba_scan_mode(conv, C, zx, ldz, xoff, dtoff, dt_bias, A_log, Dp, tmp, nullptr,
                                vent, NV, y, H, P, N, G, 1, 2, nullptr, f32, st);
}

int p2p_sm_mamba_tail(const void* zx, int ldz, int xoff, float* tail, const int* ent, int E, int C,
                      int K, int f32, hipStream_t st) {
  if (E <= 0 || K <= 1) return 0;
  dim3 g((C + 255) / 256, E), b(256);
  SM_DISPATCH_T(f32, hipLaunchKernelGGL(mamba_tail_k<T>, g, b, 0, st, (const T*)zx, ldz, xoff, tail,
                                        ent, C, K));
  return (int)hipGetLastError();
}

}  // extern "C"
