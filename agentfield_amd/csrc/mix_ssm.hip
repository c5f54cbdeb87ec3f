// Selective state-space mixer (Mamba-1 form) over packed row chunks: the
// depthwise causal convolution with its carried inputs, and the token-serial
// selective scan with one fp32 state matrix [channels, N] per sequence slot.
//
// Storage dtype S is bf16 (raw u16) or fp32.  Step sizes (softplus), decays
// (exp), the state and its update are fp32; the scan walks tokens strictly
// in order, so results do not depend on where a sequence was cut.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// exp for decays: hardware exp2 when the inputs already carry bf16 rounding,
// the precise library form for fp32 storage
template <typename S> __device__ __forceinline__ float decay_exp(float v);
template <> __device__ __forceinline__ float decay_exp<u16>(float v) { return __expf(v); }
template <> __device__ __forceinline__ float decay_exp<float>(float v) { return expf(v); }

// ------------------------------------------------------------- convolution
// out[t, c] = silu(b[c] + sum_j w[c, j] * in[t - (taps-1-j), c]).  Inputs
// before the chunk come from the sequence's slot of `state`
// [slots, taps-1, C] (the taps-1 inputs before the chunk, oldest first),
// inputs before position 0 are zero.  One thread per (row, channel).
template <typename S>
__global__ void __launch_bounds__(256) causal_conv_kernel(
    S* __restrict__ out, const S* __restrict__ in, i64 ldi,
    const S* __restrict__ w, const S* __restrict__ bias,
    const S* __restrict__ state, const i32* __restrict__ row_seq,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, i64 n, int C, int taps, int silu) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const int t = (int)(i / C), c = (int)(i % C);
    const int b = row_seq[t];
    const int r0 = cu[b];
    const int k = t - r0;                 // row inside the chunk
    const int pos = q_start[b] + k;
    const S* st = state + (size_t)sslot[b] * (taps - 1) * C;
    float acc = bias ? ldf<S>(bias + c) : 0.f;
    for (int l = 0; l < taps; ++l) {      // lag
      if (pos - l < 0) break;
      const float wv = ldf<S>(w + (size_t)c * taps + (taps - 1 - l));
      float v;
      if (l <= k) v = ldf<S>(in + (size_t)(t - l) * ldi + c);
      else v = ldf<S>(st + (size_t)(taps - 1 - (l - k)) * C + c);
      acc += wv * v;
    }
    if (silu) acc = acc / (1.0f + expf(-acc));
    stf<S>(out + (size_t)t * C + c, acc);
  }
}

// After the chunk: the slot keeps the last taps-1 inputs of the sequence.
// One thread per (sequence, channel); entry i takes old entry i + L when
// the chunk (L rows) is shorter than the history, read before it is written.
template <typename S>
__global__ void __launch_bounds__(256) conv_state_kernel(
    S* __restrict__ state, const S* __restrict__ in, i64 ldi,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int B, int C, int taps) {
  const i64 n = (i64)B * C;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const int b = (int)(i / C), c = (int)(i % C);
    const int r0 = cu[b], L = cu[b + 1] - r0;
    if (L == 0) continue;
    const int start = q_start[b];
    S* st = state + (size_t)sslot[b] * (taps - 1) * C;
    const int hist = taps - 1;
    for (int j = 0; j < hist; ++j) {
      // entry j holds position end - hist + j
      const int k = L - hist + j;         // row inside the chunk
      float v = 0.f;
      if (k >= 0) v = ldf<S>(in + (size_t)(r0 + k) * ldi + c);
      else if (start + k >= 0) v = ldf<S>(st + (size_t)(j + L) * C + c);
      stf<S>(st + (size_t)j * C + c, v);
    }
  }
}

// ---------------------------------------------------------- selective scan
// Workgroup = (block of CB = 16 channels, sequence); 256 threads = 16
// channels x 16 state lanes, lane l keeping states n = l, l+16, ... (PER of
// them) of its channel in registers.  Tokens are staged TB at a time into
// LDS (step size after softplus, input, silu(z), B and C rows), then walked serially:
//   S[c,n] = exp(dt_c A[c,n]) S[c,n] + dt_c x_c B_n ;  y_c = sum_n S[c,n] C_n
// with the sum over the 16 lanes taken by shuffles.  The output is
// (y + D x) * silu(z) in the storage dtype.
constexpr int SCAN_CB = 16;
constexpr int SCAN_TB = 16;

template <typename S, int PER>
__global__ void __launch_bounds__(256) selective_scan_kernel(
    S* __restrict__ out, float* __restrict__ state, const S* __restrict__ x,
    const S* __restrict__ dtp, const S* __restrict__ dt_bias,
    const S* __restrict__ bc, i64 ldbc, const S* __restrict__ z, i64 ldz,
    const float* __restrict__ A, const float* __restrict__ D,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int C, int N) {
  extern __shared__ float sh[];
  float* s_dt = sh;                              // [TB][CB]
  float* s_x = s_dt + SCAN_TB * SCAN_CB;         // [TB][CB]
  float* s_b = s_x + SCAN_TB * SCAN_CB;          // [TB][N]
  float* s_c = s_b + SCAN_TB * N;                // [TB][N]
  float* s_z = s_c + SCAN_TB * N;                // [TB][CB], silu(z)
  const int b = blockIdx.y;
  const int r0 = cu[b], L = cu[b + 1] - r0;
  if (L == 0) return;
  const int c0 = blockIdx.x * SCAN_CB;
  const int cl = threadIdx.x >> 4, lane = threadIdx.x & 15;
  const int c = c0 + cl;
  const bool okc = c < C;
  float* sb = state + ((size_t)sslot[b] * C + (okc ? c : 0)) * N;
  float st[PER], a[PER];
  const bool fresh = q_start[b] == 0;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = lane + 16 * j;
    const bool ok = okc && n < N;
    st[j] = (ok && !fresh) ? sb[n] : 0.f;
    a[j] = ok ? A[(size_t)c * N + n] : 0.f;
  }
  const float dcoef = okc ? D[c] : 0.f;
  for (int tb = 0; tb < L; tb += SCAN_TB) {
    const int nt = min(SCAN_TB, L - tb);
    __syncthreads();                   // previous block fully consumed
    {
      const int tt = threadIdx.x >> 4, cc = threadIdx.x & 15;   // [TB][CB]
      if (tt < nt && c0 + cc < C) {
        const size_t row = (size_t)(r0 + tb + tt);
        const float v = ldf<S>(dtp + row * C + c0 + cc) +
                        ldf<S>(dt_bias + c0 + cc);
        s_dt[tt * SCAN_CB + cc] = v > 20.f ? v : log1pf(expf(v));
        s_x[tt * SCAN_CB + cc] = ldf<S>(x + row * C + c0 + cc);
        const float zv = ldf<S>(z + row * ldz + c0 + cc);
        s_z[tt * SCAN_CB + cc] = zv / (1.0f + expf(-zv));
      }
      for (int i = threadIdx.x; i < nt * N; i += 256) {
        const int t2 = i / N, n = i % N;
        const S* rowp = bc + (size_t)(r0 + tb + t2) * ldbc;
        s_b[t2 * N + n] = ldf<S>(rowp + n);
        s_c[t2 * N + n] = ldf<S>(rowp + N + n);
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dt = s_dt[tt * SCAN_CB + cl];
      const float xv = s_x[tt * SCAN_CB + cl];
      const float dx = dt * xv;
      float y = 0.f;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const int n = lane + 16 * j;
        if (n < N) {
          st[j] = decay_exp<S>(dt * a[j]) * st[j] + dx * s_b[tt * N + n];
          y += st[j] * s_c[tt * N + n];
        }
      }
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) y += __shfl_xor(y, o, 64);
      if (lane == 0 && okc) {
        stf<S>(out + (size_t)(r0 + tb + tt) * C + c,
               (y + dcoef * xv) * s_z[tt * SCAN_CB + cl]);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = lane + 16 * j;
    if (okc && n < N) sb[n] = st[j];
  }
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace

AF_EXPORT int afm_causal_conv(void* out, const void* in, i64 ldi,
                              const void* w, const void* bias, void* state,
                              const void* row_seq, const void* cu,
                              const void* q_start, const void* sslot, int T,
                              int B, int C, int taps, int silu, int dt,
                              void* stream) {
  if (T == 0) return 0;
  if (taps < 1 || (taps > 1 && !state)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const i64 n = (i64)T * C;
#define CONV(ST)                                                             \
  do {                                                                       \
    causal_conv_kernel<ST><<<grid_for(n), 256, 0, s>>>((ST*)out,             \
        (const ST*)in, ldi, (const ST*)w, (const ST*)bias, (const ST*)state, \
        (const i32*)row_seq, (const i32*)cu, (const i32*)q_start,            \
        (const i32*)sslot, n, C, taps, silu);                                \
    if (taps > 1)                                                            \
      conv_state_kernel<ST><<<grid_for((i64)B * C), 256, 0, s>>>(            \
          (ST*)state, (const ST*)in, ldi, (const i32*)cu,                    \
          (const i32*)q_start, (const i32*)sslot, B, C, taps);               \
  } while (0)
  if (dt == 0) CONV(u16);
  else if (dt == 1) CONV(float);
  else return 9002;
#undef CONV
  return af_last_err();
}

AF_EXPORT int afm_selective_scan(void* out, void* state, const void* x,
                                 const void* dtp, const void* dt_bias,
                                 const void* bc, i64 ldbc, const void* z,
                                 i64 ldz, const void* A, const void* D,
                                 const void* cu, const void* q_start,
                                 const void* sslot, int B, int C, int N,
                                 int dt, void* stream) {
  if (B == 0) return 0;
  if (N < 1 || N > 256) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const size_t sm = (size_t)SCAN_TB * (3 * SCAN_CB + 2 * N) * sizeof(float);
  dim3 grid((C + SCAN_CB - 1) / SCAN_CB, B);
  const int per = (N + 15) / 16;
#define SCAN(ST, P)                                                           \
  selective_scan_kernel<ST, P><<<grid, 256, sm, s>>>((ST*)out, (float*)state, \
      (const ST*)x, (const ST*)dtp, (const ST*)dt_bias, (const ST*)bc, ldbc,  \
      (const ST*)z, ldz, (const float*)A, (const float*)D, (const i32*)cu,    \
      (const i32*)q_start, (const i32*)sslot, C, N)
#define SCAN_PER(ST)                          \
  do {                                        \
    if (per <= 1) SCAN(ST, 1);                \
    else if (per <= 2) SCAN(ST, 2);           \
    else if (per <= 4) SCAN(ST, 4);           \
    else if (per <= 8) SCAN(ST, 8);           \
    else SCAN(ST, 16);                        \
  } while (0)
  if (dt == 0) SCAN_PER(u16);
  else if (dt == 1) SCAN_PER(float);
  else return 9002;
#undef SCAN_PER
#undef SCAN
  return af_last_err();
}
