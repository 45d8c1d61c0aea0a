// Softmax attention forward for gfx950 (online softmax, causal / cached-prefix
// masks, grouped KV heads), with the KeyFormer perturbed log-sum-exp fused in.
//
// Orientation.  Scores are computed transposed, S^T[key, query] = K . Q^T, so
// each accumulator lane owns ONE query (column l % 32) and sixteen keys: the
// running max / sum of the online softmax are per-lane scalars (one exchange
// with lane l ^ 32), and the probabilities already sit in the register layout
// MFMA source 1 needs for O^T[d, query] += V^T[d, key] . P^T[key, query]
// (the k index of that product is permuted identically on both operands).
// V stays [key][d] in LDS; its transposed fragments come from LDS transpose
// reads.
//
// Workgroup = 4 waves x (32 * QT) queries of one query head; K/V tiles of 64
// keys are double-buffered in LDS and prefetched through registers.
#include "common.h"
#include "launch.h"
#include "philox.h"

namespace tri {

constexpr int kKeyTile = 64;

template <int D>
struct AttnLds {
  static constexpr int KS = D + 8;    // K tile row stride (halfs): 16-byte reads conflict-free
  static constexpr int VS = D + 32;   // V tile row stride: transpose reads conflict-free
  static constexpr int K_HALFS = kKeyTile * KS, V_HALFS = kKeyTile * VS;
  static constexpr int STAGE_HALFS = K_HALFS + V_HALFS;
  static constexpr int BYTES = 2 * STAGE_HALFS * 2;
  static constexpr int CH = kKeyTile * D / 8 / 256;  // 16-byte chunks per thread per tile (K and V each)
};

template <int D, int QT, bool KEYFORMER>
__global__ __launch_bounds__(256) void attn_fwd_kernel(AttnArgs a) {
  using L = AttnLds<D>;
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  constexpr int BQ = 4 * 32 * QT;
  constexpr int KSTEPS = D / 16, DT = D / 32;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int nqb = (a.S + BQ - 1) / BQ;
  const int qb = nqb - 1 - (int)blockIdx.x;  // latest (heaviest under the causal mask) blocks first
  const int h = blockIdx.y;
  const int hk = h / (a.Hq / a.Hkv);
  const int Ltot = a.P + a.S;
  const int q0 = qb * BQ;
  const int qw0 = q0 + wave * 32 * QT;

  // ---- Q fragments (source 1 of S^T = K . Q^T), kept for the whole kernel
  half8v qf[QT][KSTEPS];
  int qidx[QT];
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    int q = qw0 + nt * 32 + l32;
    qidx[nt] = q;
    q = q < a.S ? q : a.S - 1;
    const half_t* qp = a.q + (int64_t)q * a.ldq + h * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[nt][ks] = *reinterpret_cast<const half8v*>(qp + ks * 16);
  }

  // ---- key range of this workgroup
  const int qlast = min(q0 + BQ, a.S) - 1;
  const int kend = a.causal ? min(Ltot, a.P + qlast + 1) : Ltot;  // keys [0, kend)
  const int nkt = (kend + kKeyTile - 1) / kKeyTile;
  const int wave_qmax = min(qw0 + 32 * QT, a.S) - 1;  // last real query of this wave (may be < qw0)

  // ---- global -> LDS staging of K/V tiles
  const half_t* kbase = a.k + (int64_t)hk * a.k_sh;
  const half_t* vbase = a.v + (int64_t)hk * a.v_sh;
  constexpr int CPR = D / 8;  // chunks per row
  uint4v kreg[L::CH], vreg[L::CH];
  auto load_global = [&](int kt) {
#pragma unroll
    for (int i = 0; i < L::CH; ++i) {
      const int id = i * 256 + t;
      const int row = id / CPR, c = id % CPR;
      int key = kt * kKeyTile + row;
      key = key < Ltot ? key : Ltot - 1;
      kreg[i] = *reinterpret_cast<const uint4v*>(kbase + (int64_t)key * a.k_sr + c * 8);
      vreg[i] = *reinterpret_cast<const uint4v*>(vbase + (int64_t)key * a.v_sr + c * 8);
    }
  };
  auto store_lds = [&](int stage) {
    half_t* ks = lds + stage * L::STAGE_HALFS;
    half_t* vs = ks + L::K_HALFS;
#pragma unroll
    for (int i = 0; i < L::CH; ++i) {
      const int id = i * 256 + t;
      const int row = id / CPR, c = id % CPR;
      *reinterpret_cast<uint4v*>(ks + row * L::KS + c * 8) = kreg[i];
      *reinterpret_cast<uint4v*>(vs + row * L::VS + c * 8) = vreg[i];
    }
  };

  // ---- softmax state (log2 domain)
  const float c2 = a.scale * kLog2e;
  const float cp2 = kLog2e / a.tau;  // perturbed logits: (scale * qk + g) * cp2
  float m_i[QT], l_i[QT], mp_i[QT], lp_i[QT];
  float16v o[DT][QT];
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    m_i[nt] = -INFINITY; l_i[nt] = 0.f; mp_i[nt] = -INFINITY; lp_i[nt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][nt][r] = 0.f;
  }

  const int kfrag = l32 * L::KS + g * 8;
  const int vfrag = (4 * g + ((lane & 15) >> 2)) * L::VS + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);

  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < nkt; ++kt) {
    const bool more = (kt + 1) < nkt;
    if (more) load_global(kt + 1);
    const half_t* ks_ = lds + (kt & 1) * L::STAGE_HALFS;
    const half_t* vs_ = ks_ + L::K_HALFS;
    const int key0 = kt * kKeyTile;
    // a wave whose queries all precede this tile has nothing to add
    const bool active = !a.causal || key0 <= a.P + wave_qmax;
    if (active) {
      // ---- S^T = K . Q^T
      float16v st[2][QT];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < QT; ++nt)
#pragma unroll
          for (int r = 0; r < 16; ++r) st[mt][nt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        half8v kf[2];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) kf[mt] = lds_read8(ks_ + kfrag + mt * 32 * L::KS + ks * 16);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int nt = 0; nt < QT; ++nt) st[mt][nt] = mfma32(kf[mt], qf[nt][ks], st[mt][nt]);
      }
      const bool need_mask = (key0 + kKeyTile > Ltot) || (a.causal && key0 + kKeyTile - 1 > a.P + qw0);
      half8v pf[QT][2][2];
#pragma unroll
      for (int nt = 0; nt < QT; ++nt) {
        const int qlim = a.causal ? a.P + min(qidx[nt], a.S - 1) : Ltot;  // last visible key
        if (KEYFORMER) {
          // perturbed logits feed only their own running max / sum
          float sp[2][16];
          float mx = -INFINITY;
          const int qq = min(qidx[nt], a.S - 1);
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
              const int key = key0 + mt * 32 + rq * 8 + g * 4;
              float gn[4];
              if (a.noise != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const int kk = min(key + e, Ltot - 1);
                  gn[e] = (float)a.noise[((int64_t)h * a.S + qq) * Ltot + kk];
                }
              } else {
                uint32_t rnd[4];
                philox4x32_10((uint32_t)(key >> 2), (uint32_t)qq, (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
                for (int e = 0; e < 4; ++e) gn[e] = gumbel_from_bits(rnd[e]);
              }
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float v = (st[mt][nt][rq * 4 + e] * a.scale + gn[e]) * cp2;
                if (need_mask && (key + e > qlim || key + e >= Ltot)) v = -INFINITY;
                sp[mt][rq * 4 + e] = v;
                mx = fmaxf(mx, v);
              }
            }
          mx = pair_max(mx);
          const float mnew = fmaxf(mp_i[nt], mx);
          float sum = 0.f;
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += fast_exp2(sp[mt][r] - mnew);
          lp_i[nt] = lp_i[nt] * fast_exp2(mp_i[nt] - mnew) + sum;
          mp_i[nt] = mnew;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float v = st[mt][nt][r] * c2;
            if (need_mask) {
              const int key = key0 + mt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
              if (key > qlim || key >= Ltot) v = -INFINITY;
            }
            st[mt][nt][r] = v;
            mx = fmaxf(mx, v);
          }
        mx = pair_max(mx);
        const float mnew = fmaxf(m_i[nt], mx);
        const float alpha = fast_exp2(m_i[nt] - mnew);
        m_i[nt] = mnew;
        float sum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh) {
            half8v pk;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float p = fast_exp2(st[mt][nt][hh * 8 + e] - mnew);
              sum += p;
              pk[e] = (half_t)p;
            }
            pf[nt][mt][hh] = pk;
          }
        l_i[nt] = l_i[nt] * alpha + sum;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[dt][nt][r] *= alpha;
      }
      // ---- O^T += V^T . P^T
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const half_t* vp = vs_ + vfrag + (mt * 32 + hh * 16) * L::VS + dt * 32;
            const half8v vf = cat8(lds_read_tr16(vp), lds_read_tr16(vp + 8 * L::VS));
#pragma unroll
            for (int nt = 0; nt < QT; ++nt) o[dt][nt] = mfma32(vf, pf[nt][mt][hh], o[dt][nt]);
          }
    }
    if (more) store_lds((kt + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    const float l = pair_sum(l_i[nt]);
    const float lp = KEYFORMER ? pair_sum(lp_i[nt]) : 1.0f;
    const float inv = 1.0f / l;
    const int q = qidx[nt];
    if (q >= a.S) continue;
    half_t* op = a.out + (int64_t)q * a.ldo + h * D + g * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4v hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = (half_t)(o[dt][nt][rq * 4 + e] * inv);
        *reinterpret_cast<half4v*>(op + dt * 32 + rq * 8) = hv;
      }
    if (g == 0) {
      if (a.lse != nullptr) a.lse[(int64_t)h * a.S + q] = (m_i[nt] + fast_log2(l)) * kLn2;
    }
    if (KEYFORMER && g == 0 && a.lse_pert != nullptr)
      a.lse_pert[(int64_t)h * a.S + q] = (mp_i[nt] + fast_log2(lp)) * kLn2;
  }
}

template <int D, int QT, bool KF>
static int launch_attn_t(const AttnArgs& a, hipStream_t stream) {
  using L = AttnLds<D>;
  constexpr int BQ = 4 * 32 * QT;
  auto kern = attn_fwd_kernel<D, QT, KF>;
  static bool attr_done = false;
  if (!attr_done) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            L::BYTES) != hipSuccess)
      return -1;
    attr_done = true;
  }
  const dim3 grid((a.S + BQ - 1) / BQ, a.Hq);
  hipLaunchKernelGGL(kern, grid, dim3(256), L::BYTES, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_attention(const AttnArgs& a, hipStream_t stream) {
  if (a.S <= 0) return 0;
  const bool kf = a.lse_pert != nullptr;
  if (a.D == 128) return kf ? launch_attn_t<128, 1, true>(a, stream) : launch_attn_t<128, 1, false>(a, stream);
  if (a.D == 64) return kf ? launch_attn_t<64, 1, true>(a, stream) : launch_attn_t<64, 1, false>(a, stream);
  return -1;
}

}  // namespace tri
