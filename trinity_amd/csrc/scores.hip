// Per-key accumulators over queries for RoCo (sum p, sum p^2) and KeyFormer
// (sum of the noise-perturbed probabilities).
//
// Key-major column reduction: a workgroup owns 128 keys of one query head
// (4 waves x 32 keys, K fragments held in registers) and walks the query axis
// in tiles of 64 that go global -> LDS directly.  The score tile is recomputed
// with MFMA in the transposed orientation S^T[key, query], the row normaliser
// comes from the log-sum-exp written by the attention kernel, and each lane
// accumulates its sixteen keys over all queries it meets; one cross-lane
// reduction at the very end.  Nothing of size [heads, S, S] ever reaches HBM.
//
// Under the causal mask key block b only meets queries >= its first key, so
// the work per block falls linearly with b; every workgroup therefore takes
// block b and block (n - 1 - b), which makes all workgroups equally long.
#include "common.h"
#include "launch.h"
#include "philox.h"


namespace tri {

constexpr int kQTile = 64;
constexpr int kKeysPerWg = 128;

// MODE_ 0: RoCo; 1: KeyFormer; 2: KeyFormer with seeded noise at temperature 1 (a compile-time variant: left as
// a run-time flag, the compiler computes both noise transforms for every element and selects)
template <int D, int MODE_>
__device__ __forceinline__ void score_body(const ScoreArgs& a, half_t* lds) {
  constexpr int MODE = MODE_ == 0 ? 0 : 1;
  constexpr bool kf_fast = MODE_ == 2;  // seeded noise at temperature 1: exp(s + g) = exp(s) / (-ln u)
  constexpr int STAGE = kQTile * D;  // halfs; unpadded, XOR-swizzled (chunk c of row r at slot c ^ f(r))
  constexpr int KSTEPS = D / 16;
  constexpr int CPR = D / 8, INSTR = kQTile * D * 2 / 1024 / 4;
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int h = blockIdx.y, hk = h / (a.Hq / a.Hkv);
  const int Ltot = a.P + a.S;
  const int nkb = (Ltot + kKeysPerWg - 1) / kKeysPerWg;
  const float c2 = a.scale * kLog2e;
  const float cp2 = kLog2e / a.tau;
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);
  auto swz = [](int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); };

  // Q tiles: buffer-descriptor loads straight into LDS; rows past S read as zero
  const __amdgpu_buffer_rsrc_t qrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<half_t*>(a.q + h * D), 0, (int)(((int64_t)(a.S - 1) * a.ldq + D) * 2), 0x00020000);
  int ld_off[INSTR];
#pragma unroll
  for (int i = 0; i < INSTR; ++i) {
    const int p = (i * 4 + wave) * 64 + lane;
    const int row = p / CPR, slot = p % CPR;
    ld_off[i] = (row * (int)a.ldq + (slot ^ swz(row)) * 8) * 2;
  }
  const int qtile_bytes = kQTile * (int)a.ldq * 2;
  int qoff[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) qoff[ks] = l32 * D + (((ks * 2 + g) ^ swz(l32)) << 3);

  for (int half = 0; half < 2; ++half) {
    // the two key blocks of this workgroup: b and n-1-b (the middle one only once)
    const int kb = half == 0 ? (int)blockIdx.x : nkb - 1 - (int)blockIdx.x;
    if (half == 1 && kb <= (int)blockIdx.x) break;
    const int kb0 = kb * kKeysPerWg;
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
    // queries that can see any key of this block
    int qstart = 0;
    if (a.causal) {
      qstart = kb0 - a.P;
      qstart = qstart > 0 ? (qstart / kQTile) * kQTile : 0;
    }
    const int nqt = qstart < a.S ? (a.S - qstart + kQTile - 1) / kQTile : 0;
    auto issue = [&](int qt) {
#pragma unroll
      for (int i = 0; i < INSTR; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(qrsrc, (TRI_LDS void*)(lds + (qt & 1) * STAGE + (i * 4 + wave) * 512), 16,
                                                 ld_off[i] + (qstart / kQTile + qt) * qtile_bytes, 0, 0, 0);
    };
    auto load_lse = [&](int qt, float (&v)[2]) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        int q = qstart + qt * kQTile + nt * 32 + l32;
        q = q < a.S ? q : a.S - 1;
        v[nt] = a.lse[(int64_t)h * a.S + q] * kLog2e;
      }
    };

    float acc1[16], acc2[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc1[r] = 0.f; acc2[r] = 0.f; }

    auto tile = [&](int qt, const float (&lse2)[2], const bool MASK) __attribute__((always_inline)) {
      const half_t* qs = lds + (qt & 1) * STAGE;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const int qbase = qstart + qt * kQTile + nt * 32;
        // whole 32x32 tile hidden by the causal mask, or past the end (wave-uniform)
        if (MASK && (qbase >= a.S || (a.causal && kw0 > a.P + qbase + 31) || kw0 >= Ltot)) continue;
        float16v st;
#pragma unroll
        for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) st = mfma32(kf[ks], lds_read8(qs + qoff[ks] + nt * 32 * D), st);
        const int q = qbase + l32;
        const int qq = q < a.S ? q : a.S - 1;
        const int qlim = a.causal ? a.P + qq : Ltot;
        // the lane's keys kw0 + 8 rq + 4 g + e: groups rq = 2 rp and 2 rp + 1 are the two halves of one
        // generator call
#pragma unroll
        for (int rp = 0; rp < 2; ++rp) {
          uint32_t rnd[4] = {0u, 0u, 0u, 0u};
          if (MODE == 1 && (kf_fast || a.noise == nullptr))
            philox4x32_10(noise_counter(kw0 + rp * 16 + g * 4), (uint32_t)qq, (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int rq = rp * 2 + half;
            const int key = kw0 + rq * 8 + g * 4;
            float gn[4] = {0.f, 0.f, 0.f, 0.f};
            if (MODE == 1) {
              if (!kf_fast && a.noise != nullptr) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const int kk = min(key + e, Ltot - 1);
                  gn[e] = (float)a.noise[((int64_t)h * a.S + qq) * Ltot + kk];
                }
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const uint32_t bits = half ? (rnd[e] >> 16) : (rnd[e] & 0xFFFFu);
                  gn[e] = kf_fast ? inv_log2_uniform(bits) : gumbel_from_bits(bits);
                }
              }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = rq * 4 + e;
              float x;
              if (MODE == 1 && !kf_fast) x = (st[r] * a.scale + gn[e]) * cp2 - lse2[nt];
              else x = fmaf(st[r], c2, -lse2[nt]);
              float p = fast_exp2(x);
              if (MODE == 1 && kf_fast) p *= gn[e];
              if (MASK && (q >= a.S || key + e > qlim || key + e >= Ltot)) p = 0.f;
              acc1[r] += p;
              if (MODE == 0) acc2[r] = fmaf(p, p, acc2[r]);
            }
          }
        }
      }
    };

    float lse_cur[2] = {0.f, 0.f}, lse_nxt[2] = {0.f, 0.f};
    __builtin_amdgcn_s_barrier();  // the previous key block's last tile is no longer read by anyone
    if (nqt > 0) {
      issue(0);
      load_lse(0, lse_cur);
    }
    for (int qt = 0; qt < nqt; ++qt) {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): own loads of tile qt (and its lse values) have landed
      __builtin_amdgcn_s_barrier();
      if (qt + 1 < nqt) {
        issue(qt + 1);
        load_lse(qt + 1, lse_nxt);
      }
      const int qbase = qstart + qt * kQTile;
      // masking is needed where the causal diagonal crosses this wave's keys, at the ragged ends, and
      // whenever part of the tile must be skipped
      const bool need_mask = (qbase + kQTile > a.S) || (kw0 + 32 > Ltot) || (a.causal && kw0 + 31 > a.P + qbase);
      if (need_mask) tile(qt, lse_cur, true);
      else tile(qt, lse_cur, false);
      lse_cur[0] = lse_nxt[0];
      lse_cur[1] = lse_nxt[1];
    }

    // ---- reduce over the 32 query lanes; lane (l32 == 0) of each half writes
    const float invS = 1.0f / (float)a.S;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float s1 = half_wave_sum(acc1[r]) * ((MODE == 1 && kf_fast) ? kInvNegLnScale : 1.0f);
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
}

// (body in a device function: see the note at attn_fwd_kernel)
template <int D, int MODE>
__global__ __launch_bounds__(256) void score_kernel(ScoreArgs a) {
  __shared__ __attribute__((aligned(16))) half_t lds[2 * kQTile * D];
  score_body<D, MODE>(a, lds);
}

int launch_scores(const ScoreArgs& a, hipStream_t stream) {
  if (a.S <= 0) return 0;
  if (a.S <= kFewMaxQueries) {
    const int r = launch_scores_few(a, stream);
    if (r <= 0) return r;
  }
  const int Ltot = a.P + a.S;
  const int nkb = (Ltot + kKeysPerWg - 1) / kKeysPerWg;
  const dim3 grid((nkb + 1) / 2, a.Hq), block(256);
  const bool fast = a.mode == 1 && a.noise == nullptr && a.tau == 1.0f;
  if (a.D == 128) {
    if (a.mode == 0) hipLaunchKernelGGL((score_kernel<128, 0>), grid, block, 0, stream, a);
    else if (fast) hipLaunchKernelGGL((score_kernel<128, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((score_kernel<128, 1>), grid, block, 0, stream, a);
  } else if (a.D == 64) {
    if (a.mode == 0) hipLaunchKernelGGL((score_kernel<64, 0>), grid, block, 0, stream, a);
    else if (fast) hipLaunchKernelGGL((score_kernel<64, 2>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((score_kernel<64, 1>), grid, block, 0, stream, a);
  } else {
    return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tri
