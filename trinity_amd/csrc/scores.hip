// Per-key accumulators over queries for RoCo (sum p, sum p^2) and KeyFormer
// (sum of the noise-perturbed probabilities).
//
// Key-major column reduction: a workgroup owns 128 keys of one query head
// (4 waves x 32 keys, K fragments held in registers) and walks the query axis
// in tiles of 64 staged through LDS.  The score tile is recomputed with MFMA
// in the transposed orientation S^T[key, query], the row normaliser comes from
// the log-sum-exp written by the attention kernel, and each lane accumulates
// its sixteen keys over all queries it meets; one cross-lane reduction at the
// very end.  Nothing of size [heads, S, S] ever reaches HBM.
#include "common.h"
#include "launch.h"
#include "philox.h"

namespace tri {

constexpr int kQTile = 64;

template <int D, int MODE>
__global__ __launch_bounds__(256) void score_kernel(ScoreArgs a) {
  constexpr int QS = D + 8;  // LDS row stride (halfs)
  constexpr int STAGE = kQTile * QS;
  constexpr int KSTEPS = D / 16;
  constexpr int CPR = D / 8, CH = kQTile * D / 8 / 256;
  __shared__ __attribute__((aligned(16))) half_t lds[2 * STAGE];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int h = blockIdx.y, hk = h / (a.Hq / a.Hkv);
  const int Ltot = a.P + a.S;
  const int kb0 = blockIdx.x * 128;
  const int kw0 = kb0 + wave * 32;

  // K fragments: MFMA source 0, rows = this wave's 32 keys
  half8v kf[KSTEPS];
  {
    int key = kw0 + l32;
    key = key < Ltot ? key : Ltot - 1;
    const half_t* kp = a.k + (int64_t)hk * a.k_sh + (int64_t)key * a.k_sr + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = *reinterpret_cast<const half8v*>(kp + ks * 16);
  }

  // queries that can see any key of this workgroup
  int qstart = 0;
  if (a.causal) {
    qstart = kb0 - a.P;
    qstart = qstart > 0 ? (qstart / kQTile) * kQTile : 0;
  }
  const int nqt = qstart < a.S ? (a.S - qstart + kQTile - 1) / kQTile : 0;

  uint4v qreg[CH];
  auto load_global = [&](int qt) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int id = i * 256 + t;
      const int row = id / CPR, c = id % CPR;
      int q = qstart + qt * kQTile + row;
      q = q < a.S ? q : a.S - 1;
      qreg[i] = *reinterpret_cast<const uint4v*>(a.q + (int64_t)q * a.ldq + h * D + c * 8);
    }
  };
  auto store_lds = [&](int stage) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int id = i * 256 + t;
      const int row = id / CPR, c = id % CPR;
      *reinterpret_cast<uint4v*>(lds + stage * STAGE + row * QS + c * 8) = qreg[i];
    }
  };

  float acc1[16], acc2[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc1[r] = 0.f; acc2[r] = 0.f; }
  const float c2 = a.scale * kLog2e;
  const float cp2 = kLog2e / a.tau;
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);
  const int qfrag = l32 * QS + g * 8;

  if (nqt > 0) {
    load_global(0);
    store_lds(0);
  }
  __syncthreads();
  for (int qt = 0; qt < nqt; ++qt) {
    const bool more = (qt + 1) < nqt;
    if (more) load_global(qt + 1);
    const half_t* qs = lds + (qt & 1) * STAGE;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int qbase = qstart + qt * kQTile + nt * 32;
      // whole 32x32 tile hidden by the causal mask, or past the end
      if (qbase >= a.S || (a.causal && kw0 > a.P + qbase + 31) || kw0 >= Ltot) continue;
      float16v st;
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        st = mfma32(kf[ks], lds_read8(qs + qfrag + nt * 32 * QS + ks * 16), st);
      const int q = qbase + l32;
      const bool qok = q < a.S;
      const int qq = qok ? q : a.S - 1;
      const float lse2 = a.lse[(int64_t)h * a.S + qq] * kLog2e;
      const int qlim = a.causal ? a.P + qq : Ltot;
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int key = kw0 + rq * 8 + g * 4;
        float gn[4] = {0.f, 0.f, 0.f, 0.f};
        if (MODE == 1) {
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
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = rq * 4 + e;
          float x;
          if (MODE == 1) x = (st[r] * a.scale + gn[e]) * cp2 - lse2;
          else x = st[r] * c2 - lse2;
          float p = fast_exp2(x);
          if (!qok || key + e > qlim || key + e >= Ltot) p = 0.f;
          acc1[r] += p;
          if (MODE == 0) acc2[r] = fmaf(p, p, acc2[r]);
        }
      }
    }
    if (more) store_lds((qt + 1) & 1);
    __syncthreads();
  }

  // ---- reduce over the 32 query lanes; lane (l32 == 0) of each half writes
  const float invS = 1.0f / (float)a.S;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float s1 = half_wave_sum(acc1[r]);
    const float s2 = (MODE == 0) ? half_wave_sum(acc2[r]) : 0.f;
    const int key = kw0 + (r >> 2) * 8 + g * 4 + (r & 3);
    if (l32 == 0 && key < Ltot) {
      if (MODE == 0) {
        if (a.mean_var) {
          const float mean = s1 * invS;
          a.o1[(int64_t)h * a.ldo1 + key] = mean;
          a.o2[(int64_t)h * a.ldo2 + key] = s2 * invS - mean * mean;
        } else {
          a.o1[(int64_t)h * a.ldo1 + key] = s1;
          a.o2[(int64_t)h * a.ldo2 + key] = s2;
        }
      } else {
        a.o1[(int64_t)h * a.ldo1 + key] = s1;
      }
    }
  }
}

int launch_scores(const ScoreArgs& a, hipStream_t stream) {
  if (a.S <= 0) return 0;
  const int Ltot = a.P + a.S;
  const dim3 grid((Ltot + 127) / 128, a.Hq), block(256);
  if (a.D == 128) {
    if (a.mode == 0) hipLaunchKernelGGL((score_kernel<128, 0>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((score_kernel<128, 1>), grid, block, 0, stream, a);
  } else if (a.D == 64) {
    if (a.mode == 0) hipLaunchKernelGGL((score_kernel<64, 0>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((score_kernel<64, 1>), grid, block, 0, stream, a);
  } else {
    return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tri
