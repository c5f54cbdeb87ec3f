// Sigmoid attention with head mixing for prompt portions on the matrix
// cores, bf16 storage, head sizes up to 128 (any size; multiples of 8 take
// vector loads).  Scores, the distance bias, the head mix, the sigmoid and
// the output accumulators are fp32; Q.K^T and W.V run as MFMA 16x16x32 bf16.
//
// The head mix needs the scores of ALL heads for a (row, key) pair before
// any weight is known, and the output accumulators of all heads for a row
// tile must stay on chip over the whole key walk.  So a workgroup takes 16
// consecutive rows of one sequence and all heads; wave w (of up to 8) owns HPW
// consecutive heads (scores, weights and outputs of those heads).  Per tile
// of 32 keys:
//   1. every wave stages V of its K/V groups transposed into a private LDS
//      tile and computes S_h = Q_h K^T for its heads, K fragments read
//      straight from the pages (a fragment is 16 contiguous bytes of a K row);
//      S_h * scale + rel[bucket(i-j), h] goes to a workgroup-wide LDS array
//      in MFMA C layout (one 16-byte slot per lane, head and sub-tile);
//   2. after a barrier each wave reads all heads' slots of its own lanes and
//      forms m_h = pb[h] + sum_g T[h, g] s_g for its heads (T in LDS, read
//      as broadcasts), w = sigmoid(m) for visible keys, else 0;
//   3. w goes through a private LDS tile to become an MFMA A fragment and
//      O_h += W_h V.
// Weights are not normalised over keys, so there is no running maximum or
// rescaling.  The epilogue multiplies by the per-head output gate.
//
// Fragment layouts of v_mfma_f32_16x16x32_bf16 (64-lane wave):
//   A: lane holds A[m = lane&15][k = (lane>>4)*8 + j], j = 0..7
//   B: lane holds B[k = (lane>>4)*8 + j][n = lane&15]
//   C: lane reg r holds C[m = (lane>>4)*4 + r][n = lane&15]
#include "common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__device__ __forceinline__ bf16x8 as_bf16x8(s16x8 v) {
  union { s16x8 s; bf16x8 b; } u;
  u.s = v;
  return u.b;
}

template <bool VEC>
__device__ __forceinline__ s16x8 load8(const u16* row, int e0, int n) {
  s16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (VEC) {
    if (e0 < n) v = *reinterpret_cast<const s16x8*>(row + e0);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (e0 + j < n) v[j] = (short)row[e0 + j];
  }
  return v;
}

constexpr int KT = 32;    // keys per tile
constexpr int VS = 40;    // LDS row stride of V^T / W tiles (32 keys + pad)

// LDS, not registers, bounds residency here: MAXT = 256 (up to four waves,
// one per SIMD) leaves the whole register file to a wave, MAXT = 512 (up to
// eight waves) half of it.
template <int DKC, int DVT, int HPW, bool VEC, int MAXT>
__global__ void __launch_bounds__(MAXT) sigattn_prefill_mfma_kernel(
    u16* __restrict__ out, const u16* __restrict__ q,
    const u16* __restrict__ kc, const u16* __restrict__ vc,
    const i32* __restrict__ bt, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ tile_seq,
    const i32* __restrict__ tile_q0, const float* __restrict__ rel,
    const i32* __restrict__ bucket_tab, int n_tab, int RB,
    const float* __restrict__ talk, const float* __restrict__ pb,
    const u16* __restrict__ glog, i64 ldg, float scale, int H, int G, int dk,
    int dv, int page, int maxp, int ngw, int talk_lds) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  f32x4* s_x = reinterpret_cast<f32x4*>(smem);            // [H][2][64]
  u16* v_all = reinterpret_cast<u16*>(s_x + (size_t)H * 2 * 64);
  const int vwave = ngw * DVT * 16 * VS;                  // elements per wave
  const int nwv = blockDim.x >> 6;                        // waves: 1..8
  u16* p_all = v_all + nwv * vwave;                       // [nwv][16][VS]
  float* rel_s = reinterpret_cast<float*>(p_all + nwv * 16 * VS);  // [RB*H]
  i32* tab_s = reinterpret_cast<i32*>(rel_s + RB * H);            // [n_tab]
  float* talk_s = reinterpret_cast<float*>(tab_s + n_tab);        // [H*H]

  const int tile = blockIdx.x;
  const int wid = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int b = tile_seq[tile];
  const int r0 = cu[b];
  const int len = cu[b + 1] - r0;
  const int q0 = tile_q0[tile];
  const int nrows = min(16, len - q0);
  const int p0 = q_start[b] + q0;           // position of the tile's first row
  const int p_last = p0 + nrows - 1;
  const i32* btr = bt + (size_t)b * maxp;
  const int rep = H / G;
  const int h0 = wid * HPW;                 // this wave's first head
  const int nh = max(0, min(HPW, H - h0));  // and how many it has
  const int g0 = min(h0, H - 1) / rep;      // first K/V group it touches

  for (int i = threadIdx.x; i < RB * H; i += blockDim.x) rel_s[i] = rel[i];
  for (int i = threadIdx.x; i < n_tab; i += blockDim.x)
    tab_s[i] = bucket_tab[i];
  // the head-mix matrix sits in LDS when there is room, else it is read
  // through the scalar cache (wave-uniform addresses)
  if (talk && talk_lds)
    for (int i = threadIdx.x; i < H * H; i += blockDim.x) talk_s[i] = talk[i];
  const float* tmat = talk_lds ? talk_s : talk;

  s16x8 q_frag[HPW][DKC];
  {
    const int row = min(q0 + (lane & 15), len - 1);
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const int h = min(h0 + hh, H - 1);
      const u16* qr = q + ((size_t)(r0 + row) * H + h) * dk;
#pragma unroll
      for (int c = 0; c < DKC; ++c)
        q_frag[hh][c] = load8<VEC>(qr, c * 32 + (lane >> 4) * 8, dk);
    }
  }
  f32x4 o_acc[HPW][DVT];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) o_acc[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  u16* vw = v_all + wid * vwave;
  u16* pw = p_all + wid * 16 * VS;

  // Page indices of this lane's keys (two for K sub-tiles, two for its V
  // token pair), looked up one tile ahead so that no K or V load waits for a
  // block-table read.
  const int tp_lane = lane & 15;
  auto pages_of = [&](int kv0, int (&pk)[2], int (&pv)[2]) {
#pragma unroll
    for (int st = 0; st < 2; ++st)
      pk[st] = btr[min(kv0 + st * 16 + (lane & 15), p_last) / page];
    pv[0] = btr[min(kv0 + tp_lane * 2, p_last) / page];
    pv[1] = btr[min(kv0 + tp_lane * 2 + 1, p_last) / page];
  };
  int pgk[2], pgv[2];
  pages_of(0, pgk, pgv);

  // Where registers allow (the whole file to a wave, or few heads per wave)
  // the K fragments and the raw V rows of the NEXT tile, for the first PFG
  // groups of the wave,
  // are fetched into registers while the current tile is mixed and
  // multiplied, so a tile starts with its operands already on chip.
  constexpr bool PF = MAXT == 256 || HPW <= 2;
  constexpr int PFG = HPW <= 2 ? 1 : 2;
  constexpr int VIT = DVT / 2;             // V staging iterations per group
  s16x8 kpf[PF ? PFG : 1][2][DKC];
  s16x8 vpf[PF ? PFG : 1][VIT][2];
  const int n_groups_w = nh > 0 ? (h0 + nh - 1) / rep - g0 + 1 : 0;
  auto prefetch = [&](int kv0, const int (&pk)[2], const int (&pv)[2]) {
#pragma unroll
    for (int gi = 0; gi < PFG; ++gi) {
      if (gi < n_groups_w) {
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const int jc = min(kv0 + st * 16 + (lane & 15), p_last);
          const u16* krow = kc + (((size_t)pk[st] * G + g0 + gi) * page +
                                  (jc % page)) * dk;
#pragma unroll
          for (int c = 0; c < DKC; ++c)
            kpf[gi][st][c] = load8<VEC>(krow, c * 32 + (lane >> 4) * 8, dk);
        }
        const int j0 = min(kv0 + tp_lane * 2, p_last);
        const int j1 = min(kv0 + tp_lane * 2 + 1, p_last);
#pragma unroll
        for (int it = 0; it < VIT; ++it) {
          const int e0 = ((lane >> 4) + 4 * it) * 8;
          vpf[gi][it][0] = load8<VEC>(
              vc + (((size_t)pv[0] * G + g0 + gi) * page + (j0 % page)) * dv,
              e0, dv);
          vpf[gi][it][1] = load8<VEC>(
              vc + (((size_t)pv[1] * G + g0 + gi) * page + (j1 % page)) * dv,
              e0, dv);
        }
      }
    }
  };
  if (PF) prefetch(0, pgk, pgv);

  for (int kv0 = 0; kv0 <= p_last; kv0 += KT) {
    int nk[2], nv[2];
    pages_of(min(kv0 + KT, p_last), nk, nv);   // next tile's, in flight
    __syncthreads();   // s_x of the previous tile is consumed; tables loaded
    // ---- stage V^T of this wave's groups: token pairs -> 32-bit writes ----
    // keys past the tile's last row are clamped to it: their weights are
    // zero, and unconditional loads can all be in flight at once
    {
      const int j0 = min(kv0 + tp_lane * 2, p_last);
      const int j1 = min(kv0 + tp_lane * 2 + 1, p_last);
#pragma unroll
      for (int gi = 0; gi < HPW; ++gi) {     // a wave touches <= HPW groups
        if (gi < n_groups_w) {
          u16* vg = vw + gi * DVT * 16 * VS;
#pragma unroll
          for (int it = 0; it < VIT; ++it) {
            const int e0 = ((lane >> 4) + 4 * it) * 8;
            s16x8 a, c8;
            if constexpr (PF) {
              if (gi < PFG) {
                a = vpf[gi < PFG ? gi : 0][it][0];
                c8 = vpf[gi < PFG ? gi : 0][it][1];
              } else {
                a = load8<VEC>(vc + (((size_t)pgv[0] * G + g0 + gi) * page +
                                     (j0 % page)) * dv, e0, dv);
                c8 = load8<VEC>(vc + (((size_t)pgv[1] * G + g0 + gi) * page +
                                      (j1 % page)) * dv, e0, dv);
              }
            } else {
              a = load8<VEC>(vc + (((size_t)pgv[0] * G + g0 + gi) * page +
                                   (j0 % page)) * dv, e0, dv);
              c8 = load8<VEC>(vc + (((size_t)pgv[1] * G + g0 + gi) * page +
                                    (j1 % page)) * dv, e0, dv);
            }
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
              const uint32_t packed = (uint32_t)(unsigned short)a[jj] |
                                      ((uint32_t)(unsigned short)c8[jj] << 16);
              *reinterpret_cast<uint32_t*>(vg + (e0 + jj) * VS + tp_lane * 2) =
                  packed;
            }
          }
        }
      }
    }
    // ---- S_h = Q_h K^T (+ bias) for this wave's heads -> s_x ----
    int bk[2][4];
    size_t kbase[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int j = kv0 + st * 16 + (lane & 15);
      const int jc = min(j, p_last);     // clamped like V: masked later
      kbase[st] = (size_t)pgk[st] * G * page + (jc % page);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int dist = p0 + (lane >> 4) * 4 + r - j;
        bk[st][r] = (dist >= 0 && dist < n_tab) ? tab_s[dist] : RB - 1;
      }
    }
    // K fragments of one group serve all its heads of this wave; they are
    // the prefetched ones, or 2*DKC loads issued before the first MFMA
    auto scores_of_group = [&](const s16x8 (&kfr)[2][DKC], int g) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        const int h = h0 + hh;
        if (hh < nh && h / rep == g) {
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DKC; ++c)
              acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  as_bf16x8(q_frag[hh][c]), as_bf16x8(kfr[st][c]), acc, 0, 0,
                  0);
#pragma unroll
            for (int r = 0; r < 4; ++r)
              acc[r] = acc[r] * scale +
                       (RB > 0 ? rel_s[bk[st][r] * H + h] : 0.f);
            s_x[((size_t)h * 2 + st) * 64 + lane] = acc;
          }
        }
      }
    };
#pragma unroll
    for (int gi = 0; gi < HPW; ++gi) {
      if (gi < n_groups_w) {
        const int g = g0 + gi;
        bool done = false;
        if constexpr (PF) {
          if (gi < PFG) {
            scores_of_group(kpf[gi < PFG ? gi : 0], g);
            done = true;
          }
        }
        if (!done) {
          s16x8 kf[2][DKC];
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            const u16* krow = kc + (kbase[st] + (size_t)g * page) * dk;
#pragma unroll
            for (int c = 0; c < DKC; ++c)
              kf[st][c] = load8<VEC>(krow, c * 32 + (lane >> 4) * 8, dk);
          }
          scores_of_group(kf, g);
        }
      }
    }
    __syncthreads();
    if (PF && kv0 + KT <= p_last) prefetch(kv0 + KT, nk, nv);
    if (nh == 0) {           // a wave without heads only keeps the barriers
      pgk[0] = nk[0]; pgk[1] = nk[1];
      pgv[0] = nv[0]; pgv[1] = nv[1];
      continue;
    }
    // ---- head mix, sigmoid ----
    f32x4 m_acc[HPW][2];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      const float b0 = (pb && hh < nh) ? pb[h0 + hh] : 0.f;
      m_acc[hh][0] = m_acc[hh][1] = f32x4{b0, b0, b0, b0};
    }
    if (talk) {
      for (int g = 0; g < H; ++g) {
        const f32x4 s0 = s_x[((size_t)g * 2) * 64 + lane];
        const f32x4 s1 = s_x[((size_t)g * 2 + 1) * 64 + lane];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
          const float tw = hh < nh ? tmat[(h0 + hh) * H + g] : 0.f;
          m_acc[hh][0] += tw * s0;
          m_acc[hh][1] += tw * s1;
        }
      }
    } else {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        if (hh < nh) {
          m_acc[hh][0] += s_x[((size_t)(h0 + hh) * 2) * 64 + lane];
          m_acc[hh][1] += s_x[((size_t)(h0 + hh) * 2 + 1) * 64 + lane];
        }
      }
    }
    // ---- per head: weights -> A fragment, O += W V ----
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      if (hh < nh) {
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = (lane >> 4) * 4 + r;
            const int j = kv0 + st * 16 + (lane & 15);
            // hardware reciprocal and bf16 conversion: the weight is
            // rounded to bf16 for the matrix cores anyway
            const float w = (j <= p0 + m && m < nrows)
                                ? __builtin_amdgcn_rcpf(
                                      1.0f + __expf(-m_acc[hh][st][r]))
                                : 0.f;
            pw[m * VS + st * 16 + (lane & 15)] =
                __builtin_bit_cast(unsigned short, static_cast<__bf16>(w));
          }
        __builtin_amdgcn_wave_barrier();
        const s16x8 pf = *reinterpret_cast<const s16x8*>(
            pw + (lane & 15) * VS + (lane >> 4) * 8);
        __builtin_amdgcn_wave_barrier();
        const u16* vg = vw + ((h0 + hh) / rep - g0) * DVT * 16 * VS;
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) {
          const s16x8 vf = *reinterpret_cast<const s16x8*>(
              vg + (dt * 16 + (lane & 15)) * VS + (lane >> 4) * 8);
          o_acc[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              as_bf16x8(pf), as_bf16x8(vf), o_acc[hh][dt], 0, 0, 0);
        }
      }
    }
    pgk[0] = nk[0]; pgk[1] = nk[1];
    pgv[0] = nv[0]; pgv[1] = nv[1];
  }

#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    if (hh >= nh) continue;
    const int h = h0 + hh;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = q0 + (lane >> 4) * 4 + r;
      if (row >= len) continue;
      float gate = 1.0f;
      if (glog) {
        const float gv = bf2f(glog[(size_t)(r0 + row) * ldg + h]);
        gate = 1.0f / (1.0f + __expf(-gv));
      }
      u16* op = out + ((size_t)(r0 + row) * H + h) * dv;
#pragma unroll
      for (int dt = 0; dt < DVT; ++dt) {
        const int d = dt * 16 + (lane & 15);
        if (d < dv) op[d] = f2bf(o_acc[hh][dt][r] * gate);
      }
    }
  }
}

}  // namespace

// q [T, H*dk] bf16 contiguous (already unit-normed and temperature-scaled);
// caches [P, G, page, dk|dv] bf16; tile map (tile_seq, tile_q0): workgroup i
// covers chunk rows [q0, q0 + 16) of sequence tile_seq[i]; rel [RB, H],
// talk [H, H], pb [H] fp32 (each optional); glog [T, H] gate logits at row
// stride ldg (optional).  out [T, H*dv] bf16.
AF_EXPORT int afm_sigattn_prefill_mfma(
    void* out, const void* q, const void* kc, const void* vc, const void* bt,
    const void* cu, const void* q_start, const void* tile_seq,
    const void* tile_q0, const void* rel, const void* bucket_tab, int n_tab,
    int RB, const void* talk, const void* pb, const void* glog, i64 ldg,
    float scale, int ntiles, int H, int G, int dk, int dv, int page, int maxp,
    void* stream) {
  if (ntiles == 0) return 0;
  if (G <= 0 || H % G || dk < 1 || dv < 1 || dk > 128 || dv > 128 || H > 32)
    return 9003;
  if (RB > 0 && (!rel || !bucket_tab)) return 9003;
  const bool vec = (dk % 8 == 0) && (dv % 8 == 0) &&
                   ((uintptr_t)q % 16 == 0) && ((uintptr_t)kc % 16 == 0) &&
                   ((uintptr_t)vc % 16 == 0);
  // up to eight waves: two waves per SIMD hide each other's LDS and MFMA waits
  const int hpw = H <= 8 ? 1 : H <= 16 ? 2 : 4;
  const int nwv = (H + hpw - 1) / hpw;      // waves per workgroup, <= 8
  const int rep = H / G;
  int ngw = 1;
  for (int w = 0; w < nwv; ++w) {
    const int h0 = w * hpw, nh = H - h0 < hpw ? H - h0 : hpw;
    if (nh > 0) {
      const int n = (h0 + nh - 1) / rep - h0 / rep + 1;
      if (n > ngw) ngw = n;
    }
  }
  const bool small = dk <= 64 && dv <= 64;
  const int dvt = small ? 4 : 8;
  size_t sm = (size_t)H * 2 * 64 * 16 +
              (size_t)nwv * ngw * dvt * 16 * VS * 2 +
              (size_t)nwv * 16 * VS * 2 +
              (size_t)RB * H * 4 + (size_t)n_tab * 4 + 16;
  const int talk_lds = sm + (size_t)H * H * 4 <= 160 * 1024 ? 1 : 0;
  if (talk_lds) sm += (size_t)H * H * 4;
  if (sm > 160 * 1024) return 9004;
  hipStream_t s = (hipStream_t)stream;
#define SPM(DKC, DVT, HPW, VEC)                                               \
  do {                                                                        \
    auto kern = nwv <= 4                                                      \
        ? sigattn_prefill_mfma_kernel<DKC, DVT, HPW, VEC, 256>                \
        : sigattn_prefill_mfma_kernel<DKC, DVT, HPW, VEC, 512>;               \
    if (sm > 64 * 1024) {                                                     \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                   \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)sm);               \
      if (e != hipSuccess) return (int)e;                                     \
    }                                                                         \
    kern<<<ntiles, 64 * nwv, sm, s>>>((u16*)out, (const u16*)q, (const u16*)kc,    \
        (const u16*)vc, (const i32*)bt, (const i32*)cu, (const i32*)q_start,  \
        (const i32*)tile_seq, (const i32*)tile_q0, (const float*)rel,         \
        (const i32*)bucket_tab, n_tab, RB, (const float*)talk,                \
        (const float*)pb, (const u16*)glog, ldg, scale, H, G, dk, dv, page,   \
        maxp, ngw, talk_lds);                                                 \
  } while (0)
#define SPM_H(DKC, DVT, VEC)                       \
  do {                                             \
    if (hpw == 1) SPM(DKC, DVT, 1, VEC);           \
    else if (hpw == 2) SPM(DKC, DVT, 2, VEC);      \
    else SPM(DKC, DVT, 4, VEC);                    \
  } while (0)
  if (small && vec) SPM_H(2, 4, true);
  else if (small) SPM_H(2, 4, false);
  else if (vec) SPM_H(4, 8, true);
  else SPM_H(4, 8, false);
#undef SPM_H
#undef SPM
  return af_last_err();
}
