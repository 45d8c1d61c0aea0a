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

constexpr int kScoreStages = 4;  // Q tiles in LDS

// s_waitcnt vmcnt(n) leaving the other counters unconstrained (gfx9 encoding)
#define TRI_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)

// x + (x of the lane that the DPP pattern CTRL names); rows outside ROW_MASK keep x
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float x) {
  return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROW_MASK, 0xF, true));
}

// Sum over the 32 lanes of each half of the wave, in lanes 16..31 of the half (the other lanes hold the sum of
// their own 16).  Five vector instructions with lane patterns; the same through __shfl_xor is five LDS
// permutes, each with a wait for the LDS, and a key block ends with 32 such sums per lane.
__device__ __forceinline__ float half_wave_sum_dpp(float x) {
  x = dpp_add<0xB1, 0xF>(x);   // quad_perm [1,0,3,2]
  x = dpp_add<0x4E, 0xF>(x);   // quad_perm [2,3,0,1]
  x = dpp_add<0x141, 0xF>(x);  // row_half_mirror: the other quad of the eight
  x = dpp_add<0x140, 0xF>(x);  // row_mirror: the other eight of the row of 16
  x = dpp_add<0x142, 0xA>(x);  // row_bcast:15 into rows 1 and 3: the sum of the row before
  return x;
}

// MODE_ 0: RoCo; 1: KeyFormer; 2: KeyFormer with seeded noise at temperature 1 (a compile-time variant: left as
// a run-time flag, the compiler computes both noise transforms for every element and selects)
//
// Schedule.  A wave's unit of work is a half tile: S^T of its 32 keys against 32 queries (a chain of D / 16
// MFMAs into one accumulator) and the exponentials and sums of those 16 scores per lane.  The MFMA chain of half
// tile n + 1 is interleaved, instruction slot by slot, with the vector arithmetic of half tile n: one MFMA, the
// LDS read of a Q fragment three slots ahead, two scores' worth of arithmetic, and a scheduling fence - left to
// itself the compiler puts all MFMAs of a tile first, each waiting for its LDS read, and the arithmetic after.
// The chain of (tile t + 1, first half) runs during step t, so a Q tile must be in LDS one step before its own:
// four LDS stages, tiles loaded three steps ahead (tiles past the last one read as zero and are never used).
template <int D, int MODE_>
__device__ __forceinline__ void score_body(const ScoreArgs& a, half_t* lds) {
  constexpr int MODE = MODE_ == 0 ? 0 : 1;
  constexpr bool kf_fast = MODE_ == 2;  // seeded noise at temperature 1: exp(s + g) = exp(s) / (-ln u)
  constexpr int STAGE = kQTile * D;  // halfs; unpadded, XOR-swizzled (chunk c of row r at slot c ^ f(r))
  constexpr int KSTEPS = D / 16;
  constexpr int CPR = D / 8, INSTR = kQTile * D * 2 / 1024 / 4;
  constexpr int PD = 3, RING = 4;  // LDS reads run PD slots ahead of their MFMAs
  constexpr int GPS = 8 / KSTEPS;  // groups of two scores per MFMA slot
  static_assert(KSTEPS % RING == 0 && PD < KSTEPS, "the fragment ring keeps its phase from chain to chain");
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int Ltot = a.P + a.S;
  const int nkb = (Ltot + kKeysPerWg - 1) / kKeysPerWg;
  // Linear workgroup id -> (head, pair of key blocks).  Workgroups go to the eight XCDs round-robin by id; with a
  // multiple of eight heads XCD x takes heads [x Hq / 8, (x + 1) Hq / 8), so that its L2 streams the Q rows of
  // those heads only (all workgroups of a head read the same Q).
  const int nbx = (nkb + 1) / 2;
  int h, bx;
  if (a.Hq % 8 == 0) {
    const int x = (int)blockIdx.x % 8, sidx = (int)blockIdx.x / 8;
    h = x * (a.Hq / 8) + sidx / nbx;
    bx = sidx % nbx;
  } else {
    h = (int)blockIdx.x / nbx;
    bx = (int)blockIdx.x % nbx;
  }
  const int hk = h / (a.Hq / a.Hkv);
  // the wave's slot on its SIMD (HW_ID bits 3:0): the waves that share a SIMD differ in it
  const int slot = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (3 << 11));
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
  // Q fragment of k step ks: chunk (2 ks + g) ^ swz of row l32 - the k step only flips bits of the chunk index.
  // (Byte offsets, one register per k step behind an empty asm statement: the compiler would otherwise keep one
  // per (k step, half, stage).)
  int qb[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    qb[ks] = (l32 * D + (((ks * 2 + g) ^ swz(l32)) << 3)) * 2;
    asm volatile("" : "+v"(qb[ks]));
  }
  const char* const ldsb = reinterpret_cast<const char*>(lds);
  // fragment (tile qt, query half u, k step ks)
  auto frag = [&](int qt, int u, int ks) {
    return *reinterpret_cast<const half8v*>(ldsb + qb[ks] + ((qt & (kScoreStages - 1)) * STAGE + u * 32 * D) * 2);
  };

  for (int half = 0; half < 2; ++half) {
    // the two key blocks of this workgroup: b and n-1-b (the middle one only once)
    const int kb = half == 0 ? bx : nkb - 1 - bx;
    if (half == 1 && kb <= bx) break;
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
    auto issue = [&](int qt) {   // (qt may lie past the last tile: those rows are past S and read as zero)
#pragma unroll
      for (int i = 0; i < INSTR; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            qrsrc, (TRI_LDS void*)(lds + (qt & (kScoreStages - 1)) * STAGE + (i * 4 + wave) * 512), 16,
            // (unsigned: tiles up to three past the last one are issued, and for a Q buffer close to 2 GiB their
            // offsets pass 2^31; they stay beyond the descriptor's size and read as zero)
            (int)((uint32_t)ld_off[i] + (uint32_t)(qstart / kQTile + qt) * (uint32_t)qtile_bytes), 0, 0, 0);
    };
    auto load_lse = [&](int qt, float (&v)[2]) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        int q = qstart + qt * kQTile + nt * 32 + l32;
        q = q < a.S ? q : a.S - 1;
        v[nt] = a.lse[(int64_t)h * a.S + q];
      }
    };

    float acc1[16], acc2[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc1[r] = 0.f; acc2[r] = 0.f; }

    // vector arithmetic of scores 2 i and 2 i + 1 of a half tile (tile qt, query half u); st: its S^T block
    uint32_t rnd[4] = {0u, 0u, 0u, 0u};
    auto group = [&](const float16v& st, int qt, int u, float lse_q, int i, const bool MASK) {
      const int q = qstart + qt * kQTile + u * 32 + l32;
      const int qq = q < a.S ? q : a.S - 1;
      const int qlim = a.causal ? a.P + qq : Ltot;
      const float lse2 = lse_q * kLog2e;
      const int rq = i / 2, rp = i / 4;  // the lane's keys kw0 + 8 rq + 4 g + e; groups rq = 2 rp and 2 rp + 1 are
                                         // the two halves of one generator call
      if (MODE == 1 && (i % 4) == 0 && (kf_fast || a.noise == nullptr))
        philox4x32(noise_counter(kw0 + rp * 16 + g * 4), (uint32_t)qq, (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
      for (int x = 0; x < 2; ++x) {
        const int r = 2 * i + x, e = r % 4;
        const int key = kw0 + rq * 8 + g * 4 + e;
        float gn = 0.f;
        if (MODE == 1) {
          if (!kf_fast && a.noise != nullptr) {
            gn = (float)a.noise[((int64_t)h * a.S + qq) * Ltot + min(key, Ltot - 1)];
          } else {
            const uint32_t bits = (rq % 2) ? (rnd[e] >> 16) : (rnd[e] & 0xFFFFu);
            gn = kf_fast ? inv_log2_uniform(bits) : gumbel_from_bits(bits);
          }
        }
        float v;
        if (MODE == 1 && !kf_fast) v = (st[r] * a.scale + gn) * cp2 - lse2;
        else v = fmaf(st[r], c2, -lse2);
        float p = fast_exp2(v);
        if (MODE == 1 && kf_fast) p *= gn;
        if (MASK && (q >= a.S || key > qlim || key >= Ltot)) p = 0.f;
        acc1[r] += p;
        if (MODE == 0) acc2[r] = fmaf(p, p, acc2[r]);
      }
    };

    if (nqt > 0) {
      float lse_cur[2], lse_nxt[2];
      half8v fr[RING];
      float16v sa, sb;
      __builtin_amdgcn_s_barrier();  // the previous key block's tiles are no longer read by anyone
      load_lse(0, lse_cur);
      issue(0);
      issue(1);
      issue(2);
      TRI_WAIT_VMCNT(2 * INSTR);     // lse(0) and this wave's share of tile 0
      __builtin_amdgcn_s_barrier();
      // ---- S^T of (tile 0, first half) on its own; the first fragments of its second half
#pragma unroll
      for (int r = 0; r < 16; ++r) sa[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) sa = mfma32(kf[ks], frag(0, 0, ks), sa);
#pragma unroll
      for (int j = 0; j < PD; ++j) fr[j] = frag(0, 1, j);

      // One step: [chain (qt, second half) beside the arithmetic of (qt, first half)], then
      // [chain (qt + 1, first half) beside the arithmetic of (qt, second half)].
      auto step = [&](int qt, const bool MASK) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sb[r] = 0.f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < KSTEPS; ++i) {
          fr[(i + PD) % RING] = (i + PD < KSTEPS) ? frag(qt, 1, i + PD) : frag(qt + 1, 0, i + PD - KSTEPS);
          sb = mfma32(kf[i], fr[i % RING], sb);
#pragma unroll
          for (int x = 0; x < GPS; ++x) group(sa, qt, 0, lse_cur[0], i * GPS + x, MASK);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) sa[r] = 0.f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < KSTEPS; ++i) {
          fr[(i + PD) % RING] = (i + PD < KSTEPS) ? frag(qt + 1, 0, i + PD) : frag(qt + 1, 1, i + PD - KSTEPS);
          sa = mfma32(kf[i], fr[i % RING], sa);
#pragma unroll
          for (int x = 0; x < GPS; ++x) group(sb, qt, 1, lse_cur[1], i * GPS + x, MASK);
          __builtin_amdgcn_sched_barrier(0);
        }
      };

      // Tiles [q0, q1), every one with or every one without masking.  The walk over the tiles is cut into such
      // runs - the tiles on the causal diagonal come first, a ragged last tile last, and in between nothing is
      // masked - because one loop that chose between the two copies of the step tile by tile made the compiler keep
      // the sums and the S^T blocks in different registers in the two copies and move them at every turn: 62
      // register moves per tile beside 128 instructions of arithmetic (RoCo, S = 4096: 448 -> 440 us).
      auto run = [&](int q0, int q1, const bool MASK) __attribute__((always_inline)) {
        for (int qt = q0; qt < q1; ++qt) {
          // Two workgroups share a CU, and a SIMD serves the older of its two waves first whenever both are ready:
          // left alone, the older workgroup runs at the pace of a lone one, the younger on what is left, and then
          // finishes on its own, one wave per SIMD (S = 4096: one done after 76 us, the other after 110 us).  So the
          // two waves of a SIMD take turns at the higher priority, tile by tile, and stay side by side.
          if ((qt ^ slot) & 1) __builtin_amdgcn_s_setprio(1);
          else __builtin_amdgcn_s_setprio(0);
          // this wave's share of tile qt + 1 has landed (the loads of a wave complete in order; those of tile
          // qt + 2 may still be in flight)
          TRI_WAIT_VMCNT(INSTR);
          __builtin_amdgcn_s_barrier();  // ... and everybody's; tile qt - 1 is retired
          load_lse(qt + 1, lse_nxt);
          issue(qt + 3);
          step(qt, MASK);
          lse_cur[0] = lse_nxt[0];
          lse_cur[1] = lse_nxt[1];
        }
      };
      // masking is needed where the causal diagonal crosses this wave's keys - tile qt with
      // kw0 + 31 > P + qstart + 64 qt - and at the ragged ends (keys past the last one: every tile; queries past
      // S: the last tile).  Every wave walks all nqt tiles, one barrier each, whatever its runs are.
      int n_diag = 0;
      if (kw0 + 32 > Ltot) n_diag = nqt;
      else if (a.causal) n_diag = min(nqt, max(0, (kw0 + 31 - a.P - qstart + kQTile - 1) / kQTile));
      const int n_plain_end = max(n_diag, (qstart + nqt * kQTile > a.S) ? nqt - 1 : nqt);
      run(0, n_diag, true);
      run(n_diag, n_plain_end, false);
      run(n_plain_end, nqt, true);
      __builtin_amdgcn_s_setprio(0);
      TRI_WAIT_VMCNT(0);  // (the loads past the last tile)
    }

    // ---- reduce over the 32 query lanes; lane (l32 == 16) of each half writes
    const float invS = 1.0f / (float)a.S;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float s1 = half_wave_sum_dpp(acc1[r]) * ((MODE == 1 && kf_fast) ? kInvNegLnScale : 1.0f);
      const float s2 = (MODE == 0) ? half_wave_sum_dpp(acc2[r]) : 0.f;
      const int key = kw0 + (r >> 2) * 8 + g * 4 + (r & 3);
      if (l32 == 16 && key < Ltot) {
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
  __shared__ __attribute__((aligned(16))) half_t lds[kScoreStages * kQTile * D];
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
  const dim3 grid(((nkb + 1) / 2) * a.Hq), block(256);
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
