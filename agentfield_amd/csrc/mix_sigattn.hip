// Sigmoid attention over the paged cache: per-head unit-RMS q and k, a
// position-dependent query temperature, value mixing with an earlier
// layer's values, a learned bucketed distance bias, mixing of the heads'
// scores (talking heads), un-normalised sigmoid weights, per-head output gate.
//
// Storage dtype S is bf16 (raw u16) or fp32; norms, temperatures, scores,
// the head mix and the weights are fp32.  Because weights are not normalised
// over keys, partial sums over key ranges simply add: a row's keys may be cut
// over several workgroups and merged by the gate kernel in a fixed order.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// 16 bytes of storage -> EPL floats
template <typename S> struct Epl { static constexpr int n = 16 / (int)sizeof(S); };
template <typename S, bool VEC>
__device__ __forceinline__ void ld16(const S* p, float* o) {
  if constexpr (!VEC) {
    o[0] = ldf<S>(p);
  } else if constexpr (sizeof(S) == 2) {
    const s16x8 v = *reinterpret_cast<const s16x8*>(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = bf2f((u16)v[j]);
  } else {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = v[j];
  }
}

// ------------------------------------------------------------ q/k/v intake
// One workgroup per row, one wave per head in turn.  q and k heads are
// divided by their root mean square (no weight); q is then multiplied by
// 1 + coef * ln(floor((p + 1) / every) + 1); v becomes (1-lam) v + lam
// v_first when v_first is given.  k and v go to the pages at `slots`.
template <typename S>
__global__ void __launch_bounds__(256) qk_unit_cache_kernel(
    S* __restrict__ qout, const S* __restrict__ q, i64 ldq,
    const S* __restrict__ k, i64 ldk, const S* __restrict__ v, i64 ldv,
    const S* __restrict__ vfirst, i64 ldvf, float lam, S* __restrict__ kc,
    S* __restrict__ vc, const i64* __restrict__ slots,
    const i32* __restrict__ positions, float eps, float t_coef, int t_every,
    int H, int G, int dk, int dv, int page) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const i64 sl = slots[t];
  const i64 pg = sl >= 0 ? sl / page : 0, off = sl >= 0 ? sl % page : 0;
  float temp = 1.0f;
  if (t_every > 0)
    temp = 1.0f + t_coef * logf((float)((positions[t] + 1) / t_every) + 1.0f);
  for (int hh = wave; hh < H + G; hh += 4) {
    const bool isq = hh < H;
    const S* src = isq ? q + (size_t)t * ldq + (size_t)hh * dk
                       : k + (size_t)t * ldk + (size_t)(hh - H) * dk;
    float ss = 0.f;
    for (int d = lane; d < dk; d += 64) {
      const float x = ldf<S>(src + d);
      ss += x * x;
    }
    ss = wave_sum_f32(ss);
    float r = 1.0f / sqrtf(ss / (float)dk + eps);
    if (isq) {
      r *= temp;
      S* dst = qout + ((size_t)t * H + hh) * dk;
      for (int d = lane; d < dk; d += 64) stf<S>(dst + d, ldf<S>(src + d) * r);
    } else if (sl >= 0) {
      S* dst = kc + (((size_t)pg * G + (hh - H)) * page + off) * dk;
      for (int d = lane; d < dk; d += 64) stf<S>(dst + d, ldf<S>(src + d) * r);
    }
  }
  if (sl < 0) return;
  for (int i = threadIdx.x; i < G * dv; i += 256) {
    const int g = i / dv, d = i % dv;
    float x = ldf<S>(v + (size_t)t * ldv + i);
    if (vfirst)
      x = (1.0f - lam) * x + lam * ldf<S>(vfirst + (size_t)t * ldvf + i);
    stf<S>(vc + (((size_t)pg * G + g) * page + off) * dv + d, x);
  }
}

// The same with 16-byte accesses: LPH = dk / EPL lanes share a head (a power
// of two), a wave takes 64 / LPH heads per pass.
template <typename S>
__device__ __forceinline__ void st16(S* p, const float* o) {
  if constexpr (sizeof(S) == 2) {
    s16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (short)f2bf(o[j]);
    *reinterpret_cast<s16x8*>(p) = v;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
  }
}

template <typename S>
__global__ void __launch_bounds__(256) qk_unit_cache_vec_kernel(
    S* __restrict__ qout, const S* __restrict__ q, i64 ldq,
    const S* __restrict__ k, i64 ldk, const S* __restrict__ v, i64 ldv,
    const S* __restrict__ vfirst, i64 ldvf, float lam, S* __restrict__ kc,
    S* __restrict__ vc, const i64* __restrict__ slots,
    const i32* __restrict__ positions, float eps, float t_coef, int t_every,
    int H, int G, int dk, int dv, int page, int lph) {
  constexpr int EPL = Epl<S>::n;
  const int t = blockIdx.x;
  const i64 sl = slots[t];
  const i64 pg = sl >= 0 ? sl / page : 0, off = sl >= 0 ? sl % page : 0;
  float temp = 1.0f;
  if (t_every > 0)
    temp = 1.0f + t_coef * logf((float)((positions[t] + 1) / t_every) + 1.0f);
  const int hpp = 256 / lph;                  // heads per pass
  const int sub = threadIdx.x % lph;
  for (int hh = threadIdx.x / lph; hh < H + G; hh += hpp) {
    const bool isq = hh < H;
    const S* src = (isq ? q + (size_t)t * ldq + (size_t)hh * dk
                        : k + (size_t)t * ldk + (size_t)(hh - H) * dk) +
                   sub * EPL;
    float x[EPL];
    ld16<S, true>(src, x);
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) ss += x[j] * x[j];
    for (int o = lph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    float r = 1.0f / sqrtf(ss / (float)dk + eps);
    if (isq) r *= temp;
#pragma unroll
    for (int j = 0; j < EPL; ++j) x[j] *= r;
    if (isq)
      st16<S>(qout + ((size_t)t * H + hh) * dk + sub * EPL, x);
    else if (sl >= 0)
      st16<S>(kc + (((size_t)pg * G + (hh - H)) * page + off) * dk + sub * EPL,
              x);
  }
  if (sl < 0) return;
  for (int i = threadIdx.x * EPL; i < G * dv; i += 256 * EPL) {
    const int g = i / dv, d = i % dv;
    float x[EPL];
    ld16<S, true>(v + (size_t)t * ldv + i, x);
    if (vfirst) {
      float f[EPL];
      ld16<S, true>(vfirst + (size_t)t * ldvf + i, f);
#pragma unroll
      for (int j = 0; j < EPL; ++j) x[j] = (1.0f - lam) * x[j] + lam * f[j];
    }
    st16<S>(vc + (((size_t)pg * G + g) * page + off) * dv + d, x);
  }
}

// --------------------------------------------------------------- attention
// One workgroup per (row, key split).  Keys are walked in tiles of KT:
//   A. one key per thread: its K rows are dotted with every head's query
//      (queries in LDS, read as broadcasts; up to 8 heads of a K/V group
//      share each 16-byte K load); score = q.k * scale + rel[bucket(i-j), h]
//      goes to LDS, one column per key;
//   B. the same thread mixes its column over heads, m_h = sum_g T[h,g] s_g,
//      and leaves w_h = sigmoid(m_h + pb[h]) (0 for keys that do not exist);
//   C. W.V: thread = (key group, 16-byte slice of one head's output); the
//      key groups' partial sums are added through LDS at the end.
// Partial outputs are fp32 [T, nsplit, H*dv].
// output slices per thread when H*dv/EPL > 256 (more in the scalar build)
template <bool VEC> struct Accr { static constexpr int n = VEC ? 4 : 16; };

template <typename S, int KT, bool VEC>
__global__ void __launch_bounds__(256) sigmoid_attention_kernel(
    float* __restrict__ part, const S* __restrict__ q,
    const S* __restrict__ kc, const S* __restrict__ vc,
    const i32* __restrict__ bt, const i32* __restrict__ row_seq,
    const i32* __restrict__ positions, const float* __restrict__ rel,
    const i32* __restrict__ bucket_tab, int n_tab, int RB,
    const float* __restrict__ talk, const float* __restrict__ pb, float scale,
    int H, int G, int dk, int dv, int page, int maxp, int nsplit,
    int window) {
  constexpr int EPL = VEC ? Epl<S>::n : 1;
  constexpr int ACCR = Accr<VEC>::n;
  extern __shared__ float sh[];
  float* qs = sh;                         // [H*dk]
  float* sc = qs + H * dk;                // [H][KT]
  float* wt = sc + H * KT;                // [H][KT]
  float* talk_s = wt + H * KT;            // [H*H]
  float* pb_s = talk_s + H * H;           // [H]
  float* rel_s = pb_s + H;                // [RB*H]
  i32* koff = (i32*)(rel_s + RB * H);     // [KT]
  float* red = (float*)(koff + KT);       // [256*EPL]

  const int t = blockIdx.x, split = blockIdx.y, tid = threadIdx.x;
  const int seq = row_seq[t];
  const int qi = positions[t];
  const int rep = H / G;
  for (int i = tid; i < H * dk; i += 256) qs[i] = ldf<S>(q + (size_t)t * H * dk + i);
  for (int i = tid; i < H * H; i += 256) talk_s[i] = talk ? talk[i] : 0.f;
  for (int i = tid; i < H; i += 256) pb_s[i] = pb ? pb[i] : 0.f;
  for (int i = tid; i < RB * H; i += 256) rel_s[i] = rel[i];

  const int lo_all = window > 0 ? max(0, qi - window + 1) : 0;
  const int n_keys = qi + 1 - lo_all;
  // even key ranges per split, in steps of 32 keys
  const int per = ((n_keys + nsplit - 1) / nsplit + 31) / 32 * 32;
  const int lo = lo_all + split * per;
  const int hi = min(qi + 1, lo + per);

  const int NE = H * dv / EPL;
  const int NEb = NE < 256 ? NE : 256;
  const int KG = 256 / NEb;
  const int kg = tid / NEb, es = tid % NEb;
  float acc[ACCR][EPL];
#pragma unroll
  for (int r = 0; r < ACCR; ++r)
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[r][e] = 0.f;
  const i32* btr = bt + (size_t)seq * maxp;

  // tile width actually walked: the split's keys, 32 .. KT (a power of two)
  int ktw = 32;
  while (ktw < KT && ktw < hi - lo) ktw <<= 1;
  const int ngs = 256 / ktw;

  for (int j0 = lo; j0 < hi; j0 += ktw) {
    const int cnt = min(ktw, hi - j0);
    __syncthreads();            // previous tile's wt/koff consumed; qs ready
    {
      // thread = (key kk, group slice gs): with a narrow tile the K/V groups
      // of one key are dotted by 256 / KT threads side by side
      const int NGS = ngs;
      const int kk = tid % ktw, gs = tid / ktw;
      const int j = j0 + kk;
      if (kk < cnt) {
        const int pg = btr[j / page], off = j % page;
        const int base = pg * G * page + off;
        if (gs == 0) koff[kk] = base;
        int bk = 0;
        if (RB > 0) {
          const int n = qi - j;
          bk = n < n_tab ? bucket_tab[n] : RB - 1;
        }
        for (int g = gs; g < G; g += NGS) {
          const S* kp = kc + (size_t)(base + g * page) * dk;
          for (int r0 = 0; r0 < rep; r0 += 8) {
            float a8[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) a8[r] = 0.f;
            for (int d0 = 0; d0 < dk; d0 += EPL) {
              float kv[EPL];
              ld16<S, VEC>(kp + d0, kv);
#pragma unroll
              for (int r = 0; r < 8; ++r) {
                if (r0 + r < rep) {
                  const float* qp = qs + (size_t)(g * rep + r0 + r) * dk + d0;
#pragma unroll
                  for (int e = 0; e < EPL; ++e) a8[r] += qp[e] * kv[e];
                }
              }
            }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
              if (r0 + r < rep) {
                const int h = g * rep + r0 + r;
                sc[h * KT + kk] =
                    a8[r] * scale + (RB > 0 ? rel_s[bk * H + h] : 0.f);
              }
            }
          }
        }
      }
      if (NGS > 1) __syncthreads();   // a key's scores come from NGS threads
      // the mix: thread = (key kk, heads gs, gs + NGS, ...)
      for (int h = gs; h < H; h += NGS) {
        float w = 0.f;
        if (kk < cnt) {
          float m = pb_s[h];
          if (talk) {
            for (int g2 = 0; g2 < H; ++g2)
              m += talk_s[h * H + g2] * sc[g2 * KT + kk];
          } else {
            m += sc[h * KT + kk];
          }
          w = 1.0f / (1.0f + expf(-m));
        }
        wt[h * KT + kk] = w;
      }
    }
    __syncthreads();
    if (kg < KG) {
#pragma unroll
      for (int r = 0; r < ACCR; ++r) {
        const int e = es + r * 256;
        if (e < NE) {
          const int h = (e * EPL) / dv, d = (e * EPL) % dv;
          const int g = h / rep;
          const float* wh = wt + h * KT;
          const S* vbase = vc + (size_t)g * page * dv + d;
          int jj = kg;
          // four value rows in flight per thread
          for (; jj + 3 * KG < cnt; jj += 4 * KG) {
            float v0[EPL], v1[EPL], v2[EPL], v3[EPL];
            ld16<S, VEC>(vbase + (size_t)koff[jj] * dv, v0);
            ld16<S, VEC>(vbase + (size_t)koff[jj + KG] * dv, v1);
            ld16<S, VEC>(vbase + (size_t)koff[jj + 2 * KG] * dv, v2);
            ld16<S, VEC>(vbase + (size_t)koff[jj + 3 * KG] * dv, v3);
            const float w0 = wh[jj], w1 = wh[jj + KG], w2 = wh[jj + 2 * KG],
                        w3 = wh[jj + 3 * KG];
#pragma unroll
            for (int x = 0; x < EPL; ++x) {
              acc[r][x] += w0 * v0[x];
              acc[r][x] += w1 * v1[x];
              acc[r][x] += w2 * v2[x];
              acc[r][x] += w3 * v3[x];
            }
          }
          for (; jj < cnt; jj += KG) {
            float vv[EPL];
            ld16<S, VEC>(vbase + (size_t)koff[jj] * dv, vv);
            const float w = wh[jj];
#pragma unroll
            for (int x = 0; x < EPL; ++x) acc[r][x] += w * vv[x];
          }
        }
      }
    }
  }
  float* dst = part + ((size_t)t * nsplit + split) * H * dv;
  if (KG == 1) {
#pragma unroll
    for (int r = 0; r < ACCR; ++r) {
      const int e = es + r * 256;
      if (e < NE && kg == 0)
#pragma unroll
        for (int x = 0; x < EPL; ++x) dst[e * EPL + x] = acc[r][x];
    }
    return;
  }
  __syncthreads();
#pragma unroll
  for (int x = 0; x < EPL; ++x) red[tid * EPL + x] = acc[0][x];
  __syncthreads();
  if (tid < NEb) {
#pragma unroll
    for (int x = 0; x < EPL; ++x) {
      float s = 0.f;
      for (int g2 = 0; g2 < KG; ++g2) s += red[(g2 * NEb + tid) * EPL + x];
      dst[tid * EPL + x] = s;
    }
  }
}

// out[t, h, :] = sigmoid(glog[t, h]) * sum_s part[t, s, h, :]
template <typename S>
__global__ void __launch_bounds__(256) gate_heads_kernel(
    S* __restrict__ out, const float* __restrict__ part, int nsplit,
    const S* __restrict__ glog, i64 ldg, i64 n, int H, int dv) {
  const int HD = H * dv;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const i64 t = i / HD;
    const int e = (int)(i % HD);
    float s = 0.f;
    for (int k = 0; k < nsplit; ++k) s += part[(t * nsplit + k) * HD + e];
    if (glog) {
      const float gv = ldf<S>(glog + t * ldg + e / dv);
      s *= 1.0f / (1.0f + expf(-gv));
    }
    stf<S>(out + i, s);
  }
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

template <typename S, int KT, bool VEC>
int launch_sig(float* part, const void* q, const void* kc, const void* vc,
               const void* bt, const void* row_seq, const void* positions,
               const void* rel, const void* tab, int n_tab, int RB,
               const void* talk, const void* pb, float scale, int T, int H,
               int G, int dk, int dv, int page, int maxp, int nsplit,
               int window, size_t sm, hipStream_t s) {
  auto kern = sigmoid_attention_kernel<S, KT, VEC>;
  if (sm > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(
        (const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm);
    if (e != hipSuccess) return (int)e;
  }
  kern<<<dim3(T, nsplit), 256, sm, s>>>(
      part, (const S*)q, (const S*)kc, (const S*)vc, (const i32*)bt,
      (const i32*)row_seq, (const i32*)positions, (const float*)rel,
      (const i32*)tab, n_tab, RB, (const float*)talk, (const float*)pb, scale,
      H, G, dk, dv, page, maxp, nsplit, window);
  return af_last_err();
}

template <typename S>
int dispatch_sig(float* part, const void* q, const void* kc, const void* vc,
                 const void* bt, const void* row_seq, const void* positions,
                 const void* rel, const void* tab, int n_tab, int RB,
                 const void* talk, const void* pb, float scale, int T, int H,
                 int G, int dk, int dv, int page, int maxp, int nsplit,
                 int window, hipStream_t s) {
  constexpr int EPLV = Epl<S>::n;
  const bool vec = dk % EPLV == 0 && dv % EPLV == 0 &&
                   (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0;
  const int epl = vec ? EPLV : 1;
  if ((i64)H * dv > (i64)256 * (vec ? Accr<true>::n : Accr<false>::n) * epl)
    return 9004;
  auto lds = [&](int kt) {
    return ((size_t)H * dk + 2 * (size_t)H * kt + (size_t)H * H + H +
            (size_t)RB * H + kt + 256 * (size_t)epl) * sizeof(float);
  };
  int kt = 256;
  while (kt > 32 && lds(kt) > 64 * 1024) kt >>= 1;
  const size_t sm = lds(kt);
  if (sm > 160 * 1024) return 9004;
#define SIG(KT, V)                                                            \
  return launch_sig<S, KT, V>(part, q, kc, vc, bt, row_seq, positions, rel,   \
                              tab, n_tab, RB, talk, pb, scale, T, H, G, dk,   \
                              dv, page, maxp, nsplit, window, sm, s)
  if (vec) {
    if (kt == 256) SIG(256, true);
    if (kt == 128) SIG(128, true);
    if (kt == 64) SIG(64, true);
    SIG(32, true);
  }
  if (kt == 256) SIG(256, false);
  if (kt == 128) SIG(128, false);
  if (kt == 64) SIG(64, false);
  SIG(32, false);
#undef SIG
}

}  // namespace

AF_EXPORT int afm_qk_unit_cache(
    void* qout, const void* q, i64 ldq, const void* k, i64 ldk, const void* v,
    i64 ldv, const void* vfirst, i64 ldvf, float lam, void* kc, void* vc,
    const void* slots, const void* positions, float eps, float t_coef,
    int t_every, int T, int H, int G, int dk, int dv, int page, int dt,
    void* stream) {
  if (T == 0) return 0;
  if (H < 1 || G < 1 || H % G != 0) return 9003;
  hipStream_t s = (hipStream_t)stream;
  auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
#define QKU(ST)                                                              \
  do {                                                                       \
    constexpr int E = 16 / (int)sizeof(ST);                                  \
    const int lph = dk / E;                                                  \
    const bool vec = dk % E == 0 && dv % E == 0 && lph >= 1 && lph <= 64 && \
                     (lph & (lph - 1)) == 0 && ldq % E == 0 &&               \
                     ldk % E == 0 && ldv % E == 0 && ldvf % E == 0 &&        \
                     al(qout) && al(q) && al(k) && al(v) && al(vfirst) &&    \
                     al(kc) && al(vc);                                       \
    if (vec)                                                                 \
      qk_unit_cache_vec_kernel<ST><<<T, 256, 0, s>>>((ST*)qout,              \
          (const ST*)q, ldq, (const ST*)k, ldk, (const ST*)v, ldv,           \
          (const ST*)vfirst, ldvf, lam, (ST*)kc, (ST*)vc,                    \
          (const i64*)slots, (const i32*)positions, eps, t_coef, t_every,    \
          H, G, dk, dv, page, lph);                                          \
    else                                                                     \
      qk_unit_cache_kernel<ST><<<T, 256, 0, s>>>((ST*)qout, (const ST*)q,    \
          ldq, (const ST*)k, ldk, (const ST*)v, ldv, (const ST*)vfirst,      \
          ldvf, lam, (ST*)kc, (ST*)vc, (const i64*)slots,                    \
          (const i32*)positions, eps, t_coef, t_every, H, G, dk, dv, page);  \
  } while (0)
  if (dt == 0) QKU(u16);
  else if (dt == 1) QKU(float);
  else return 9002;
#undef QKU
  return af_last_err();
}

// part: fp32 scratch [T, nsplit, H*dv]; glog: per-head output gate logits
// [T, H] with row stride ldg (optional).
AF_EXPORT int afm_sigmoid_attention(
    void* out, void* part, const void* q, const void* kc, const void* vc,
    const void* bt, const void* row_seq, const void* positions,
    const void* rel, const void* bucket_tab, int n_tab, int RB,
    const void* talk, const void* pb, const void* glog, i64 ldg, float scale,
    int T, int H, int G, int dk, int dv, int page, int maxp, int nsplit,
    int window, int dt, void* stream) {
  if (T == 0) return 0;
  if (H < 1 || G < 1 || H % G != 0 || nsplit < 1 || !part) return 9003;
  if (RB > 0 && (!rel || !bucket_tab)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (dt == 0)
    rc = dispatch_sig<u16>((float*)part, q, kc, vc, bt, row_seq, positions,
                           rel, bucket_tab, n_tab, RB, talk, pb, scale, T, H,
                           G, dk, dv, page, maxp, nsplit, window, s);
  else if (dt == 1)
    rc = dispatch_sig<float>((float*)part, q, kc, vc, bt, row_seq, positions,
                             rel, bucket_tab, n_tab, RB, talk, pb, scale, T,
                             H, G, dk, dv, page, maxp, nsplit, window, s);
  else
    return 9002;
  if (rc != 0) return rc;
  const i64 n = (i64)T * H * dv;
  if (dt == 0)
    gate_heads_kernel<u16><<<grid_for(n), 256, 0, s>>>(
        (u16*)out, (const float*)part, nsplit, (const u16*)glog, ldg, n, H, dv);
  else
    gate_heads_kernel<float><<<grid_for(n), 256, 0, s>>>(
        (float*)out, (const float*)part, nsplit, (const float*)glog, ldg, n, H,
        dv);
  return af_last_err();
}
