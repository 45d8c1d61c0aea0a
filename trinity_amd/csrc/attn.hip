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
// keys go global -> LDS directly (no register staging) into two stages, the
// loads of tile t+1 overlapping the work on tile t.  Two workgroups share a CU
// (two waves per SIMD), so one wave's softmax arithmetic overlaps the other's
// MFMAs.
#include <type_traits>

#include "common.h"
#include "launch.h"
#include "philox.h"


namespace tri {

constexpr int kKeyTile = 64;

// s_waitcnt vmcnt(n) leaving the other counters unconstrained (gfx9 encoding)
#define TRI_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)

// LDS tiles are filled by direct-to-LDS loads (1 KB of contiguous LDS per wave
// instruction), so they are unpadded and XOR-swizzled at 16-byte granularity:
//   K tile [64][D]: chunk c of key row r at slot c ^ fk(r)   (16-byte fragment reads conflict-free)
//   V tile [64][D]: chunk c of key row r at slot c ^ fv(r)   (transpose reads conflict-free)
template <int D>
struct AttnLds {
  static constexpr int CPR = D / 8;                     // 16-byte chunks per row
  static constexpr int K_HALFS = kKeyTile * D, V_HALFS = kKeyTile * D;
  static constexpr int STAGE_HALFS = K_HALFS + V_HALFS;
  static constexpr int BYTES = 2 * STAGE_HALFS * 2;     // two stages
  static constexpr int INSTR = kKeyTile * D * 2 / 1024 / 4;  // wave-level loads per wave per tile (K and V each)
  __device__ static __forceinline__ int fk(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
  __device__ static __forceinline__ int fv(int row) { return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
};

template <int D>
constexpr int kAttnStageRow = D + 8;  // halfs per row of an output tile staged in LDS

// The running maximum is only raised when some query of the wave exceeds it by
// more than this many powers of two: probabilities then stay below 2^kLazyMax
// (exact in fp32, far inside fp16 range) and the O accumulators are rescaled
// rarely instead of once per key tile.  The final normalisation uses the sum
// taken against the same reference value, so the result is unchanged.
constexpr float kLazyMax = 8.0f;
constexpr int kTwoWayMaxWorkgroups = 256, kTwoWayMinKeys = 640;  // when the eight-wave variant runs
constexpr int kEightGroupMinWorkgroups = 129, kEightGroupMaxWorkgroups = 256;  // (of 256 queries each)
constexpr int kWideMinWorkgroups = 768;  // 64 queries per wave (head dimension 64) from this many workgroups on

// Linear workgroup id -> (query block, head).  Workgroups go to the eight XCDs round-robin by id, and each XCD
// has its own 4 MB L2: with a multiple of eight heads, XCD x gets heads [x Hq / 8, (x + 1) Hq / 8) - for grouped
// KV heads those share K / V (Llama-3-8B: one KV head, 2 MB of K and V at 4096 keys, per XCD instead of four of
// them).  On every XCD the latest query blocks come first: under the causal mask those are the longest, so the
// hardware's in-order dispatch becomes longest-job-first; consecutive ids of an XCD are heads of one query block.
__device__ __forceinline__ void attn_wg_map(int id, int Hq, int nqb, int& qb, int& h) {
  if (Hq % 8 == 0) {
    const int hx = Hq / 8, x = id % 8, s = id / 8;
    qb = nqb - 1 - s / hx;
    h = x * hx + s % hx;
  } else {
    qb = nqb - 1 - id / Hq;
    h = id % Hq;
  }
}

// KF 0: plain attention; 1: KeyFormer (perturbed log-sum-exp on the side); 2: KeyFormer with seeded noise at
// temperature 1 (compile-time, so that neither variant carries the other's arithmetic)
//
// KW = 2: eight waves - the four query groups twice - take alternate key tiles (a stage holds two tiles) and merge
// their (max, sum, O) through LDS at the end.  A workgroup then walks its keys in half as many steps: for short
// sequences, where the kernel's time is the chain of dependent tile steps of its longest workgroup rather than
// the chip's throughput.
//
// SPLIT: few new tokens against a long cached prefix (16-bit caches: every variant; fp8 caches: plain attention).  The query heads that share a KV head
// are stacked along the query axis - row j of a KV head is (head hk * group + j / S, token j % S) - so K / V are read
// once per 128 rows instead of once per head, and the key axis is cut into runs of a.split_tiles tiles per
// workgroup; the unnormalised (O, max, sum) of every run go to the workspace in the layout of the few-query kernel
// and are merged by its combine kernel.
// With FP8 (SPLIT only) K and V come from fp8 (e4m3) caches: a tile travels global -> registers while the tile
// before it is worked on, and is converted to the 16-bit element type on its way into the same swizzled LDS places
// (exact; the scales ride on a.scale and a.out_scale).
template <int D, int QT, int KF, int KW, bool SPLIT = false, bool FP8 = false>
__device__ __forceinline__ void attn_fwd_body(const AttnArgs& a, half_t* lds, const half_t* __restrict__ qglob) {
  // (qglob = a.q; the qualifier is what keeps the compiler from waiting for the loads in flight before the
  // first LDS transpose read of a tile - see attn_fwd_pipe_body)
  static_assert(!SPLIT || (QT == 1 && KW == 1), "the split variant is the four-wave kernel");
  static_assert(!FP8 || SPLIT, "fp8 caches are read by the split variant only");
  constexpr bool KEYFORMER = KF != 0;
  constexpr bool kf_fast = KF == 2;
  // a wave may meet tiles without a visible key before it has met one (its state is then still -inf / 0)
  constexpr bool GUARD = KW > 1 || SPLIT;
  using L = AttnLds<D>;
  constexpr int BQ = 4 * 32 * QT;
  constexpr int NWAVE = 4 * KW;
  constexpr int KSTEPS = D / 16, DT = D / 32;
  const int t = threadIdx.x, lane = t & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(t >> 6);
  // query group; which of the stage's tiles.  (Eight waves: the two key ways of a query group sit on SIMDs
  // 2 w and 2 w + 1, so that every SIMD holds one of the groups 0, 1 and one of the groups 2, 3 - see FOLD.)
  static_assert(KW == 1 || QT == 1, "eight waves: 32 queries per wave");
  const int wave = KW == 2 ? wave_all / 2 : wave_all % 4, kway = KW == 2 ? wave_all % 2 : wave_all / 4;
  const int l32 = lane & 31, g = lane >> 5;
  const int group = a.Hq / a.Hkv;
  const int rows = SPLIT ? group * a.S : a.S;  // length of the query axis
  const int nqb = (rows + BQ - 1) / BQ;
  int qb, h, hk, split = 0;
  if (SPLIT) {  // linear workgroup id -> (key run, row block, KV head)
    hk = (int)blockIdx.x % a.Hkv;
    qb = ((int)blockIdx.x / a.Hkv) % nqb;
    split = (int)blockIdx.x / a.Hkv / nqb;
    h = hk * group;  // (first head of the group; rows carry their own)
  } else {
    attn_wg_map((int)blockIdx.x, a.Hq, nqb, qb, h);
    hk = h / group;
  }
  const int Ltot = a.P + a.S;
  int qw0 = qb * BQ + wave * 32 * QT;  // first query of this wave
  int qend = qb * BQ + BQ;              // the workgroup's key range is that of query qend - 1
  if (KW == 2 && a.causal) {
    // FOLD: under the causal mask the late query blocks have many key tiles and the early ones few, and this
    // variant runs where there is one workgroup per CU at most - nothing evens that out.  So a workgroup takes
    // two 64-query half blocks that add up to the same work everywhere: groups 0, 1 the half block nhb - 1 - qb
    // (long), groups 2, 3 the half block qb (short).  They share the K / V tiles in LDS (the short half block
    // drops out of the walk when its keys end), and every SIMD runs one long and one short wave.
    const int nhb = (a.S + 63) / 64, hb_long = nhb - 1 - qb, hb_short = qb;
    // (an odd number of half blocks: the middle one is its own partner, and groups 2, 3 stay empty)
    qw0 = wave < 2 ? hb_long * 64 + wave * 32 : (hb_short < hb_long ? hb_short * 64 + (wave - 2) * 32 : a.S);
    qend = hb_long * 64 + 64;
  }

  // ---- Q fragments (source 1 of S^T = K . Q^T), kept for the whole kernel
  half8v qf[QT][KSTEPS];
  int qidx[QT];   // position on the query axis (may lie past its end)
  int qtok[QT];   // the token it stands for, clamped to a real one
  int qhead[QT];  // ... and its head
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    int q = qw0 + nt * 32 + l32;
    qidx[nt] = q;
    q = q < rows ? q : rows - 1;
    qtok[nt] = SPLIT ? q % a.S : q;
    qhead[nt] = SPLIT ? h + q / a.S : h;
    const half_t* qp = qglob + (int64_t)qtok[nt] * a.ldq + qhead[nt] * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[nt][ks] = *reinterpret_cast<const half8v*>(qp + ks * 16);
  }

  // ---- key range of this workgroup
  const int qlast = min(qend, a.S) - 1;
  const int kend = (a.causal && !SPLIT) ? min(Ltot, a.P + qlast + 1) : Ltot;  // keys [0, kend)
  const int nkt_all = (kend + kKeyTile - 1) / kKeyTile;
  const int kt_begin = SPLIT ? split * a.split_tiles : 0;                      // tiles [kt_begin, nkt)
  const int nkt = SPLIT ? min(nkt_all, kt_begin + a.split_tiles) : nkt_all;
  const int wave_qmax = min(qw0 + 32 * QT, a.S) - 1;  // last real query of this wave (may be < qw0)

  // ---- global -> LDS loads of K/V tiles through buffer descriptors: the per-thread byte offset is fixed
  // (a thread always fetches the same logical chunk) and rows past the last key read as zero instead of
  // faulting.
  const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<half_t*>(a.k + (int64_t)hk * a.k_sh), 0, (int)((int64_t)Ltot * a.k_sr * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<half_t*>(a.v + (int64_t)hk * a.v_sh), 0, (int)((int64_t)Ltot * a.v_sr * 2), 0x00020000);
  // a stage holds KW tiles, [K][V] each; load instruction i of a wave fetches chunk (i * NWAVE + wave_all) * 64 +
  // lane of the stage's KW * 64 * CPR chunks (per K and V)
  constexpr int kInstrPerTile = kKeyTile * L::CPR / 64;  // wave-level instructions per tile
  int ld_koff[L::INSTR], ld_voff[L::INSTR];
#pragma unroll
  for (int i = 0; i < L::INSTR; ++i) {
    const int p = ((i * NWAVE + wave_all) % kInstrPerTile) * 64 + lane;  // chunk within its tile
    const int row = p / L::CPR, slot = p % L::CPR;
    ld_koff[i] = (row * (int)a.k_sr + (slot ^ L::fk(row)) * 8) * 2;
    ld_voff[i] = (row * (int)a.v_sr + (slot ^ L::fv(row)) * 8) * 2;
  }
  const int ktile_bytes = kKeyTile * (int)a.k_sr * 2, vtile_bytes = kKeyTile * (int)a.v_sr * 2;
  auto issue = [&](int step) {  // tiles step * KW .. step * KW + KW - 1
    half_t* st = lds + (step & 1) * (KW * L::STAGE_HALFS);
#pragma unroll
    for (int i = 0; i < L::INSTR; ++i) {
      const int ti = (i * NWAVE + wave_all) / kInstrPerTile;         // tile within the stage (wave-uniform)
      const int wi = (i * NWAVE + wave_all) % kInstrPerTile;         // 1 KB slice within the tile
      const int kt = kt_begin + step * KW + ti;
      half_t* ks = st + ti * L::STAGE_HALFS;
      half_t* vs = ks + L::K_HALFS;
      // the tile advance goes into the per-lane offset: the scalar offset of a buffer load is not range-checked
      __builtin_amdgcn_raw_ptr_buffer_load_lds(krsrc, (TRI_LDS void*)(ks + wi * 512), 16,
                                               ld_koff[i] + kt * ktile_bytes, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(vrsrc, (TRI_LDS void*)(vs + wi * 512), 16,
                                               ld_voff[i] + kt * vtile_bytes, 0, 0, 0);
    }
  };

  // ---- fp8 caches: 16-byte pieces (sixteen values: two chunks) of a tile, D / 64 per thread for K and V each
  constexpr int PIECES = D / 64, PPR = D / 16;  // pieces per thread; per row
  uint4v kraw[PIECES], vraw[PIECES];
  auto fetch8 = [&](int step) {
    const int kt = kt_begin + step;
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int piece = i * 256 + t;
      const int key = kt * kKeyTile + piece / PPR, j = piece % PPR;
      kraw[i] = uint4v{0u, 0u, 0u, 0u};  // fp8 zeros past the last key
      vraw[i] = uint4v{0u, 0u, 0u, 0u};
      if (key < Ltot) {
        kraw[i] = *reinterpret_cast<const uint4v*>(a.k8 + (int64_t)hk * a.k8_sh + (int64_t)key * a.k8_sr + j * 16);
        vraw[i] = *reinterpret_cast<const uint4v*>(a.v8 + (int64_t)hk * a.v8_sh + (int64_t)key * a.v8_sr + j * 16);
      }
    }
  };
  auto commit8 = [&](int step) {
    half_t* ks = lds + (step & 1) * L::STAGE_HALFS;
    half_t* vs = ks + L::K_HALFS;
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int piece = i * 256 + t;
      const int row = piece / PPR, j = piece % PPR;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int chunk = 2 * j + c;
        *reinterpret_cast<half8v*>(ks + row * D + ((chunk ^ L::fk(row)) << 3)) = fp8x8_to_half8(uint2v{kraw[i][2 * c], kraw[i][2 * c + 1]});
        *reinterpret_cast<half8v*>(vs + row * D + ((chunk ^ L::fv(row)) << 3)) = fp8x8_to_half8(uint2v{vraw[i][2 * c], vraw[i][2 * c + 1]});
      }
    }
  };

  // ---- fragment read offsets (halfs)
  int koff[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) koff[ks] = l32 * D + (((ks * 2 + g) ^ L::fk(l32)) << 3);
  const int j4 = (lane & 15) >> 2;
  int voff[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int chunk = dt * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    voff[dt] = L::K_HALFS + (4 * g + j4) * D + ((chunk ^ L::fv(j4)) << 3) + (lane & 1) * 4;
  }

  // ---- softmax state (log2 domain, reference value m_i is lazily raised)
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
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);
  // Seeded noise at temperature 1: exp(s + g) with g = -ln(-ln u) is exp(s) / (-ln u), so the perturbed sum is
  // the plain probabilities weighted by 1 / (-ln u) - one logarithm and one reciprocal per element instead of
  // two logarithms, an exponential and a second running maximum.

  // One key tile.  The body is inlined once per value of MASK, so that full (unmasked) tiles carry no
  // masking arithmetic at all.
  auto tile = [&](int kt, const bool MASK) __attribute__((always_inline)) {
    // MASK is wave-uniform; the empty asm statements keep the masking code behind real branches (left alone,
    // the compiler turns it into per-element selects that every full tile would pay for)
    const half_t* ks_ = lds + (((kt - kt_begin) / KW) & 1) * (KW * L::STAGE_HALFS) + kway * L::STAGE_HALFS;
    const int key0 = kt * kKeyTile;
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
      for (int mt = 0; mt < 2; ++mt) kf[mt] = lds_read8(ks_ + koff[ks] + mt * 32 * D);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < QT; ++nt) st[mt][nt] = mfma32(kf[mt], qf[nt][ks], st[mt][nt]);
    }
    half8v pf[QT][2][2];
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      const int qlim = a.causal ? a.P + qtok[nt] : Ltot;  // last visible key
      if (KEYFORMER && !kf_fast) {
        // perturbed logits feed only their own running max / sum
        float sp[2][16];
        float mx = -INFINITY;
        const int qq = qtok[nt];
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
                gn[e] = (float)a.noise[((int64_t)qhead[nt] * a.S + qq) * Ltot + kk];
              }
            } else {
              gumbel4(key, qq, qhead[nt], seed_lo, seed_hi, gn);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float v = (st[mt][nt][rq * 4 + e] * a.scale + gn[e]) * cp2;
              if (MASK && (key + e > qlim || key + e >= Ltot)) v = -INFINITY;
              sp[mt][rq * 4 + e] = v;
              mx = fmaxf(mx, v);
            }
          }
        mx = pair_max(mx);
        const float mnew = fmaxf(mp_i[nt], mx);
        // (a wave's first tiles may hold no visible key of some query: keep the exponents defined)
        const float mref = (GUARD && mnew == -INFINITY) ? 0.f : mnew;
        float sum = 0.f;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int r = 0; r < 16; ++r) sum += fast_exp2(sp[mt][r] - mref);
        lp_i[nt] = lp_i[nt] * fast_exp2(mp_i[nt] - mref) + sum;
        mp_i[nt] = mnew;
      }
      // ---- plain softmax: mask, tile max of the raw scores, lazy reference update
      if (MASK) {
        asm volatile("");
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key0 + mt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
            if (key > qlim || key >= Ltot) st[mt][nt][r] = -INFINITY;
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[mt][nt][r]);
      mx = pair_max(mx) * c2;  // scale > 0
      if (__builtin_amdgcn_ballot_w64(mx > m_i[nt] + kLazyMax) != 0) {  // wave-uniform
        const float mnew = fmaxf(m_i[nt], mx);
        const float alpha = (GUARD && mnew == -INFINITY) ? 1.0f : fast_exp2(m_i[nt] - mnew);
        m_i[nt] = mnew;
        l_i[nt] *= alpha;
        if (KEYFORMER && kf_fast) lp_i[nt] *= alpha;  // the fast path keeps its sum against m_i
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt][nt] = o[dt][nt] * alpha;
      }
      const float nm = (GUARD && m_i[nt] == -INFINITY) ? 0.f : -m_i[nt];
      float sum = 0.f, sump = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          float wgt[8];
          if (KEYFORMER && kf_fast) {
            // the lane's eight keys of this (mt, hh) block are the two groups of one generator call
            const int qq = qtok[nt];
            const int key = key0 + mt * 32 + hh * 16 + g * 4;
            uint32_t rnd[4];
            philox4x32(noise_counter(key), (uint32_t)qq, (uint32_t)qhead[nt], 0u, seed_lo, seed_hi, rnd);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              wgt[e] = inv_log2_uniform(rnd[e] & 0xFFFFu);
              wgt[4 + e] = inv_log2_uniform(rnd[e] >> 16);
            }
          }
          half8v pk;
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const float p0 = fast_exp2(fmaf(st[mt][nt][hh * 8 + e], c2, nm));
            const float p1 = fast_exp2(fmaf(st[mt][nt][hh * 8 + e + 1], c2, nm));
            sum += p0 + p1;
            if (KEYFORMER && kf_fast) sump = fmaf(p0, wgt[e], fmaf(p1, wgt[e + 1], sump));
            const half2v h2 = pack_prob(p0, p1);
            pk[e] = h2[0];
            pk[e + 1] = h2[1];
          }
          pf[nt][mt][hh] = pk;
        }
      l_i[nt] += sum;
      if (KEYFORMER && kf_fast) lp_i[nt] += sump;
    }
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const half_t* vp = ks_ + voff[dt] + (mt * 32 + hh * 16) * D;
          const half8v vf = cat8(lds_read_tr16(vp), lds_read_tr16(vp + 8 * D));
#pragma unroll
          for (int nt = 0; nt < QT; ++nt) o[dt][nt] = mfma32(vf, pf[nt][mt][hh], o[dt][nt]);
        }
  };

  const int nsteps = (nkt - kt_begin + KW - 1) / KW;  // (> 0: the launcher starts no workgroup without tiles)
  if (FP8) fetch8(0);
  else issue(0);
  for (int step = 0; step < nsteps; ++step) {
    if (FP8) {
      commit8(step);  // (waits for its loads; the stage was last read two steps ago, before the previous barrier)
      __syncthreads();
      if (step + 1 < nsteps) fetch8(step + 1);
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of the stage has landed
      __builtin_amdgcn_s_barrier();        // ... and everybody's; the stage before is retired
      if (step + 1 < nsteps) issue(step + 1);
    }
    const int kt = kt_begin + step * KW + kway;
    const int key0 = kt * kKeyTile;
    // a wave whose queries all precede this tile has nothing to add (nor has one past the last tile); with
    // stacked heads every wave that has rows at all holds every token
    const bool active = SPLIT ? qw0 < rows
                              : (kt < nkt && !(a.causal && key0 > a.P + wave_qmax) && !(KW == 2 && qw0 >= a.S));
    const bool need_mask = (key0 + kKeyTile > Ltot) || (a.causal && key0 + kKeyTile - 1 > a.P + (SPLIT ? 0 : qw0));
    if (active) tile(kt, need_mask);
  }

  // ---- KW > 1: the waves of the second key way hand their state over through LDS (lane for lane); those of
  // the first merge it into theirs and go on to the epilogue
  if (KW > 1) {
    constexpr int REG = QT * (DT * 16 + 4);  // floats per lane
    float* mg = reinterpret_cast<float*>(lds) + wave * REG * 64 + lane;
    __syncthreads();  // every wave is done with the K/V stages
    if (kway == 1) {
#pragma unroll
      for (int nt = 0; nt < QT; ++nt) {
        float* r = mg + nt * (DT * 16 + 4) * 64;
        r[0] = m_i[nt]; r[64] = l_i[nt]; r[128] = mp_i[nt]; r[192] = lp_i[nt];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) r[(4 + dt * 16 + e) * 64] = o[dt][nt][e];
      }
    }
    __syncthreads();
    if (kway == 1) return;
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      const float* r = mg + nt * (DT * 16 + 4) * 64;
      const float m1 = r[0], mp1 = r[128];
      const float m = fmaxf(m_i[nt], m1), mp = fmaxf(mp_i[nt], mp1);
      const float a0 = m_i[nt] == -INFINITY ? 0.f : fast_exp2(m_i[nt] - m);
      const float a1 = m1 == -INFINITY ? 0.f : fast_exp2(m1 - m);
      l_i[nt] = l_i[nt] * a0 + r[64] * a1;
      if (KEYFORMER) {
        if (kf_fast) {
          lp_i[nt] = lp_i[nt] * a0 + r[192] * a1;
        } else {
          const float b0 = mp_i[nt] == -INFINITY ? 0.f : fast_exp2(mp_i[nt] - mp);
          const float b1 = mp1 == -INFINITY ? 0.f : fast_exp2(mp1 - mp);
          lp_i[nt] = lp_i[nt] * b0 + r[192] * b1;
          mp_i[nt] = mp;
        }
      }
      m_i[nt] = m;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][nt][e] = o[dt][nt][e] * a0 + r[(4 + dt * 16 + e) * 64] * a1;
    }
  }

  if (SPLIT) {
    // ---- this run's unnormalised result: O [Hq][runs][S][D], then (max, sum, perturbed max, perturbed sum)
    // [Hq][runs][S][4]
    const int nsplit = (nkt_all + a.split_tiles - 1) / a.split_tiles;
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      const float l = pair_sum(l_i[nt]);
      const float lp = KEYFORMER ? pair_sum(lp_i[nt]) * (kf_fast ? kInvNegLnScale : 1.0f) : 0.f;
      if (qidx[nt] >= rows) continue;
      const int64_t row = ((int64_t)qhead[nt] * nsplit + split) * a.S + qtok[nt];
      float* po = a.ws + row * D + g * 4;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const float4v v = {o[dt][nt][rq * 4], o[dt][nt][rq * 4 + 1], o[dt][nt][rq * 4 + 2], o[dt][nt][rq * 4 + 3]};
          *reinterpret_cast<float4v*>(po + dt * 32 + rq * 8) = v;
        }
      if (g == 0) {
        // (a run whose keys are all hidden from a token leaves max = -inf, sum = 0: stored as the few-query kernel's
        // "no key seen" pair, which the merge weighs with zero)
        const float mpr = kf_fast ? m_i[nt] : mp_i[nt];  // (the seeded fast path keeps its sum against the plain maximum)
        const float4v st4 = {m_i[nt] == -INFINITY ? -1.0e30f : m_i[nt], l,
                             (!KEYFORMER || mpr == -INFINITY) ? -1.0e30f : mpr, lp};
        *reinterpret_cast<float4v*>(a.ws + (int64_t)a.Hq * nsplit * a.S * D + row * 4) = st4;
      }
    }
    return;
  }

  // ---- epilogue
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    const float l = pair_sum(l_i[nt]);
    const float lp = KEYFORMER ? pair_sum(lp_i[nt]) * (kf_fast ? kInvNegLnScale : 1.0f) : 1.0f;
    const float inv = a.out_scale / l;
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
      a.lse_pert[(int64_t)h * a.S + q] = ((kf_fast ? m_i[nt] : mp_i[nt]) + fast_log2(lp)) * kLn2;
  }
}

// ---------------------------------------------------------------------------
// The prefill kernel at 32 queries per wave (four waves, or eight as two key
// ways or eight query groups), software-pipelined inside each wave: while the
// probabilities of key tile t are computed (vector arithmetic), the matrix
// pipe already works on S^T of tile t + 1, and the running maximum of tile
// t + 1 is folded while O += V^T . P^T of tile t runs.  Every slot below holds
// the MFMAs of one K / V fragment, the LDS read of a fragment PD slots ahead
// and its share of the vector arithmetic; a scheduling fence after each slot
// keeps that order.  K(t + 1) and V(t) are read during step t, so K tiles
// are loaded two steps ahead and V tiles one (two LDS buffers each).
// Same arithmetic per element as attn_fwd_body (KF 0 and 2; not SPLIT).
// ---------------------------------------------------------------------------
template <int D, int QT, int KF, int KW, int QW>
__device__ __forceinline__ void attn_fwd_pipe_body(const AttnArgs& a, half_t* lds, const half_t* __restrict__ qglob) {
  // (qglob = a.q.  The qualifier matters beyond Q: inlined, every LDS access of this function carries "does not
  // alias Q", and an LDS read that carries alias information is not made to wait for the global -> LDS loads in
  // flight - without it the compiler puts s_waitcnt vmcnt(0) before the first transpose read after every load.
  // The barrier and the explicit wait at the top of a step are what orders loads and reads here.)
  static_assert(KF == 0 || KF == 2, "plain attention and KeyFormer with seeded noise at temperature 1");
  static_assert(KW == 1 || (KW == 2 && QT == 1), "eight waves: 32 queries per wave, two key ways");
  static_assert(QW == 1 || (QW == 2 && KW == 1 && QT == 1), "eight waves: 32 queries per wave, eight query groups");
  constexpr bool KFN = KF == 2;
  using L = AttnLds<D>;
  constexpr int BQ = 4 * 32 * QT;
  constexpr int KSTEPS = D / 16, DT = D / 32;
  constexpr int NKF = 2 * KSTEPS, NVF = 4 * DT;  // K / V fragments per tile, QT MFMAs each
  constexpr int GPS = 16 * QT / NKF;             // softmax groups (two keys each) per S^T slot
  constexpr int EPS = 32 * QT / NVF;             // scores folded into the running maximum per O^T slot
  constexpr int PD = 3, RING = 4;                // LDS reads run PD slots ahead of their MFMAs
  static_assert(GPS * NKF == 16 * QT && EPS * NVF == 32 * QT && PD < RING && PD < NKF && PD < NVF, "slot plan");
  const int t = threadIdx.x, lane = t & 63;
  // KW = 2: eight waves, the four query groups twice; the wave of key way w takes the tiles KW * step + w, a step
  // moves KW tiles through LDS, and the ways' (max, sum, O) are merged at the end (see attn_fwd_body, also for
  // the order of the waves and the folded query blocks)
  // QW = 2 (causal only): eight waves, eight query groups of 32 - four half blocks of 64 queries, two late ones
  // (waves 0 - 3) and two early ones (waves 4 - 7, one of them on each SIMD beside a late one), that walk the same
  // K / V tiles.  Every workgroup then has the same work, every SIMD a long and a short wave, and a K / V tile
  // serves 256 queries.  Meant for launches of one round (up to one workgroup per CU), where the four-wave
  // kernel's time is the chain of its longest workgroup, which shares its SIMDs with another long one.
  constexpr int NWAVE = 4 * KW * QW;
  const int wave_all = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wave = KW == 2 ? wave_all / 2 : wave_all, kway = KW == 2 ? wave_all % 2 : 0;
  const int l32 = lane & 31, g = lane >> 5;
  const int group = a.Hq / a.Hkv;
  const int nqb = (a.S + QW * BQ - 1) / (QW * BQ);
  int qb, h;
  attn_wg_map((int)blockIdx.x, a.Hq, nqb, qb, h);
  const int hk = h / group;
  const int Ltot = a.P + a.S;
  int qw0 = qb * BQ + wave * 32 * QT, qend = qb * BQ + BQ;
  if (KW == 2 && a.causal) {  // the folded half blocks of attn_fwd_body
    const int nhb = (a.S + 63) / 64, hb_long = nhb - 1 - qb, hb_short = qb;
    qw0 = wave < 2 ? hb_long * 64 + wave * 32 : (hb_short < hb_long ? hb_short * 64 + (wave - 2) * 32 : a.S);
    qend = hb_long * 64 + 64;
  }
  if (QW == 2) {
    // workgroup qb takes what the workgroups before it left, from both ends: half blocks hi, lo, hi - 1, lo + 1
    // (in this order, as far as they exist)
    const int nhb = (a.S + 63) / 64, lo = 2 * qb, hi = nhb - 1 - 2 * qb;
    const int r = (wave_all % 4) / 2;                              // first or second of its kind
    const bool late = wave_all < 4;
    const int order = late ? 2 * r : 2 * r + 1, hb = late ? hi - r : lo + r;
    qw0 = order < hi - lo + 1 ? hb * 64 + (wave_all % 2) * 32 : a.S;
    qend = hi * 64 + 64;
  }

  half8v qf[QT][KSTEPS];
  int qidx[QT], qtok[QT];
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    int q = qw0 + nt * 32 + l32;
    qidx[nt] = q;
    q = q < a.S ? q : a.S - 1;
    qtok[nt] = q;
    const half_t* qp = qglob + (int64_t)q * a.ldq + h * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[nt][ks] = *reinterpret_cast<const half8v*>(qp + ks * 16);
  }

  const int qlast = min(qend, a.S) - 1;
  const int kend = a.causal ? min(Ltot, a.P + qlast + 1) : Ltot;
  const int nkt = (kend + kKeyTile - 1) / kKeyTile;   // tiles of the workgroup (> 0)
  const int nsteps = (nkt + KW - 1) / KW;
  const int wave_qmax = min(qw0 + 32 * QT, a.S) - 1;
  // tiles [0, nact_tiles) hold a key some query of this wave sees; the wave's own tiles among them are those of
  // its steps [0, nact)
  const int nact_tiles = qw0 >= a.S ? 0 : (a.causal ? min(nkt, (a.P + wave_qmax) / kKeyTile + 1) : nkt);
  const int nact = max(0, (nact_tiles - kway + KW - 1) / KW);
  // (a wave of the second way may meet rows without a visible key before any other: their state is still -inf / 0)
  constexpr bool GUARD = KW > 1;

  // K / V tiles go global -> LDS through buffer descriptors, one per tile: base and size move with the tile
  // (scalar arithmetic), the per-lane offsets stay fixed, and rows past the last key read as zero
  half_t* const kglob = const_cast<half_t*>(a.k + (int64_t)hk * a.k_sh);
  half_t* const vglob = const_cast<half_t*>(a.v + (int64_t)hk * a.v_sh);
  constexpr int kInstrPerTile = kKeyTile * L::CPR / 64;  // wave-level load instructions per tile
  int ld_koff[L::INSTR], ld_voff[L::INSTR];
#pragma unroll
  for (int i = 0; i < L::INSTR; ++i) {
    static_assert(kInstrPerTile % NWAVE == 0, "a load instruction's tile is known at compile time");
    const int p = ((i % (kInstrPerTile / NWAVE)) * NWAVE + wave_all) * 64 + lane;  // chunk within its tile
    const int row = p / L::CPR, slot = p % L::CPR;
    ld_koff[i] = (row * (int)a.k_sr + (slot ^ L::fk(row)) * 8) * 2;
    ld_voff[i] = (row * (int)a.v_sr + (slot ^ L::fv(row)) * 8) * 2;
  }
  // the K tiles of step st (way w) at kbase + ((st & 1) * KW + w) * K_HALFS, the V tiles likewise from vbase
  half_t* const kbase = lds;
  half_t* const vbase = lds + 2 * KW * L::K_HALFS;
  constexpr int kIpt = kInstrPerTile / NWAVE;  // load instructions of a wave per tile
  auto load_k = [&](int st) {
#pragma unroll
    for (int w = 0; w < KW; ++w) {
      half_t* dst = kbase + ((st & 1) * KW + w) * L::K_HALFS;
      const int key0 = (st * KW + w) * kKeyTile;  // (past the last key: the size below is <= 0, everything reads as zero)
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
          kglob + (int64_t)key0 * a.k_sr, 0, (int)max((int64_t)0, (int64_t)(Ltot - key0) * a.k_sr * 2), 0x00020000);
#pragma unroll
      for (int i = 0; i < kIpt; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (TRI_LDS void*)(dst + (i * NWAVE + wave_all) * 512), 16,
                                                 ld_koff[w * kIpt + i], 0, 0, 0);
    }
  };
  auto load_v = [&](int st) {
#pragma unroll
    for (int w = 0; w < KW; ++w) {
      half_t* dst = vbase + ((st & 1) * KW + w) * L::V_HALFS;
      const int key0 = (st * KW + w) * kKeyTile;
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
          vglob + (int64_t)key0 * a.v_sr, 0, (int)max((int64_t)0, (int64_t)(Ltot - key0) * a.v_sr * 2), 0x00020000);
#pragma unroll
      for (int i = 0; i < kIpt; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (TRI_LDS void*)(dst + (i * NWAVE + wave_all) * 512), 16,
                                                 ld_voff[w * kIpt + i], 0, 0, 0);
    }
  };

  // Fragment addresses: one per-lane byte offset per k step (K) and per d block (V), kept in registers behind an
  // empty asm statement; buffer parity, key half and key quarter are compile-time constants of an unrolled step
  // and go into the offset fields of the LDS reads - no address arithmetic in the loop.
  int kbyte[KSTEPS], vbyte[DT];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    kbyte[ks] = (kway * L::K_HALFS + l32 * D + (((ks * 2 + g) ^ L::fk(l32)) << 3)) * 2;
    asm volatile("" : "+v"(kbyte[ks]));
  }
  const int j4 = (lane & 15) >> 2;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int chunk = dt * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    vbyte[dt] = (int)(uint32_t)(uintptr_t)lds +
                (2 * KW * L::K_HALFS + kway * L::V_HALFS + (4 * g + j4) * D + ((chunk ^ L::fv(j4)) << 3) + (lane & 1) * 4) * 2;
    // (an LDS address; the start of the V tiles is part of it because an LDS instruction's offset field ends at 64 KB)
    asm volatile("" : "+v"(vbyte[dt]));
  }
  const char* const ldsb = reinterpret_cast<const char*>(lds);
  // K fragment j = (k step j / 2, key half j % 2); V fragment v = (key half, key quarter, d block)
  // K fragment j = (k step j / 2, key half j % 2) of the K buffer `par`; V fragment v = (key half, key quarter, d block)
  auto read_kf = [&](int par, int j) {
    return *reinterpret_cast<const half8v*>(ldsb + kbyte[j / 2] + (par * KW * L::K_HALFS + (j % 2) * 32 * D) * 2);
  };
  auto read_vf = [&](int par, int v) {
    // (pointer arithmetic in the LDS address space, so that the constant part lands in the instruction's offset field)
    TRI_LDS char* vp = (TRI_LDS char*)(uintptr_t)(uint32_t)vbyte[v % DT] +
                       (par * KW * L::V_HALFS + ((v / (2 * DT)) * 32 + ((v / DT) % 2) * 16) * D) * 2;
    const short4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS short4s*)vp);
    const short4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS short4s*)(vp + 8 * D * 2));
    half4v hl, hh;
    __builtin_memcpy(&hl, &lo, 8);
    __builtin_memcpy(&hh, &hi, 8);
    return cat8(hl, hh);
  };

  const float c2 = a.scale * kLog2e;
  float m_i[QT], l_i[QT], lp_i[QT];
  float16v o[DT][QT];
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    m_i[nt] = -INFINITY; l_i[nt] = 0.f; lp_i[nt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][nt][r] = 0.f;
  }
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);

  auto need_mask = [&](int kt) {
    const int key0 = kt * kKeyTile;
    return (key0 + kKeyTile > Ltot) || (a.causal && key0 + kKeyTile - 1 > a.P + qw0);
  };
  auto apply_mask = [&](float16v (&s)[2][QT], int kt) {
    const int key0 = kt * kKeyTile;
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      const int qlim = a.causal ? a.P + qtok[nt] : Ltot;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + mt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
          if (key > qlim || key >= Ltot) s[mt][nt][r] = -INFINITY;
        }
    }
  };
  auto tile_max = [&](const float16v (&s)[2][QT], float (&mx)[QT]) {
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      float m = -INFINITY;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) m = fmaxf(m, s[mt][nt][r]);
      mx[nt] = m;
    }
  };
  // the lazily raised reference value (see kLazyMax); mx: the lane's maximum of the raw scores of the tile
  auto raise = [&](const float (&mx)[QT]) {
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      const float m = pair_max(mx[nt]) * c2;  // scale > 0
      if (__builtin_amdgcn_ballot_w64(m > m_i[nt] + kLazyMax) != 0) {  // wave-uniform
        const float mnew = fmaxf(m_i[nt], m);
        const float alpha = (GUARD && mnew == -INFINITY) ? 1.0f : fast_exp2(m_i[nt] - mnew);
        m_i[nt] = mnew;
        l_i[nt] *= alpha;
        if (KFN) lp_i[nt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[dt][nt] = o[dt][nt] * alpha;
      }
    }
  };
  auto zero_scores = [&](float16v (&s)[2][QT]) {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < QT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[mt][nt][r] = 0.f;
  };

  // softmax group gi of tile kt: two keys of one query -> two probabilities, packed for O^T's MFMA
  half8v pf[QT][2][2];
  float sum[QT], sump[QT], nm[QT], wgt[8];
  auto softmax_group = [&](const float16v (&s)[2][QT], int kt, int gi) {
    const int nt = gi / 16, mt = (gi / 8) % 2, hh = (gi / 4) % 2, e = (gi % 4) * 2;
    if (KFN && e == 0) {
      // the lane's eight keys of this (mt, hh) block are the two groups of one generator call
      const int key = kt * kKeyTile + mt * 32 + hh * 16 + g * 4;
      uint32_t rnd[4];
      philox4x32(noise_counter(key), (uint32_t)qtok[nt], (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        wgt[x] = inv_log2_uniform(rnd[x] & 0xFFFFu);
        wgt[4 + x] = inv_log2_uniform(rnd[x] >> 16);
      }
    }
    const float p0 = fast_exp2(fmaf(s[mt][nt][hh * 8 + e], c2, nm[nt]));
    const float p1 = fast_exp2(fmaf(s[mt][nt][hh * 8 + e + 1], c2, nm[nt]));
    sum[nt] += p0 + p1;
    if (KFN) sump[nt] = fmaf(p0, wgt[e], fmaf(p1, wgt[e + 1], sump[nt]));
    const half2v h2 = pack_prob(p0, p1);
    pf[nt][mt][hh][e] = h2[0];
    pf[nt][mt][hh][e + 1] = h2[1];
  };
  auto begin_tile = [&]() {
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      sum[nt] = 0.f;
      sump[nt] = 0.f;
      nm[nt] = (GUARD && m_i[nt] == -INFINITY) ? 0.f : -m_i[nt];
    }
  };
  auto end_tile = [&]() {
#pragma unroll
    for (int nt = 0; nt < QT; ++nt) {
      l_i[nt] += sum[nt];
      if (KFN) lp_i[nt] += sump[nt];
    }
  };

  half8v fr[RING];  // fragment ring: the K fragments of a step, then its V fragments

  // One step.  cur: S^T of the wave's tile of step st (masked, its maximum already folded into m_i); next: receives
  // S^T of its tile of step st + 1.  (PAR = st & 1, a compile-time constant of each unrolled copy)
  auto step = [&](int st, auto parc, float16v (&cur)[2][QT], float16v (&next)[2][QT]) __attribute__((always_inline)) {
    constexpr int PAR = decltype(parc)::value;
    const int kt = st * KW + kway;  // the wave's tile of this step
    TRI_WAIT_VMCNT(0);              // this wave's share of K(st + 1) and V(st) has landed
    __builtin_amdgcn_s_barrier();   // ... and everybody's; K(st) and V(st - 1) are retired
    if (st + 2 < nsteps) load_k(st + 2);
    if (st + 1 < nsteps) load_v(st + 1);
    if (st < nact) {
      // ---- S^T(kt + 1) = K . Q^T beside the probabilities of tile kt.  (On the wave's last tile the product
      // is not used - K(kt + 1) may not even have been loaded - and costs sixteen idle MFMAs per workgroup;
      // a second copy of the step without it costs the registers of a second set of O accumulators.)
#pragma unroll
      for (int j = 0; j < PD; ++j) fr[j] = read_kf(PAR ^ 1, j);
      zero_scores(next);
      begin_tile();
      // The wave takes issue priority over the SIMD's other wave (another workgroup) while its slots mix MFMAs
      // and vector arithmetic, and gives it back for the MFMA-only phase, which then fills the other wave's
      // gaps: Llama S = 4096 165 -> 154 us.  (Priority in both phases, or in the second only: 167, 164 us.)
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < NKF; ++j) {
        if (j + PD < NKF) fr[(j + PD) % RING] = read_kf(PAR ^ 1, j + PD);
        else fr[(j + PD) % RING] = read_vf(PAR, j + PD - NKF);   // the first V fragments
#pragma unroll
        for (int nt = 0; nt < QT; ++nt) next[j % 2][nt] = mfma32(fr[j % RING], qf[nt][j / 2], next[j % 2][nt]);
#pragma unroll
        for (int x = 0; x < GPS; ++x) softmax_group(cur, kt, j * GPS + x);
        __builtin_amdgcn_sched_barrier(0);
      }
      // ---- O^T += V^T . P^T of tile kt beside the maximum of tile kt + 1
      float mx[QT];
#pragma unroll
      for (int nt = 0; nt < QT; ++nt) mx[nt] = -INFINITY;
      __builtin_amdgcn_s_setprio(0);
#pragma unroll
      for (int v = 0; v < NVF; ++v) {
        if (v + PD < NVF) fr[(NKF + v + PD) % RING] = read_vf(PAR, v + PD);
#pragma unroll
        for (int nt = 0; nt < QT; ++nt)
          o[v % DT][nt] = mfma32(fr[(NKF + v) % RING], pf[nt][v / (2 * DT)][(v / DT) % 2], o[v % DT][nt]);
#pragma unroll
        for (int x = 0; x < EPS; ++x) {
          const int idx = v * EPS + x;  // (query block, key half, register) of the scores
          mx[idx / 32] = fmaxf(mx[idx / 32], next[(idx / 16) % 2][idx / 32][idx % 16]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      end_tile();
      if (st + 1 < nact) {
        if (need_mask(kt + KW)) {  // wave-uniform; the diagonal and the last tile only
          asm volatile("");
          apply_mask(next, kt + KW);
          tile_max(next, mx);
        }
        raise(mx);
      }
    }
  };

  // ---- prologue: K(0), K(1), V(0); S^T of tile 0
  load_k(0);
  if (1 < nsteps) load_k(1);
  load_v(0);
  TRI_WAIT_VMCNT(0);
  __builtin_amdgcn_s_barrier();
  float16v sa[2][QT], sb[2][QT];
  if (0 < nact) {
    zero_scores(sa);
#pragma unroll
    for (int j = 0; j < NKF; ++j) {
      const half8v kf = read_kf(0, j);
#pragma unroll
      for (int nt = 0; nt < QT; ++nt) sa[j % 2][nt] = mfma32(kf, qf[nt][j / 2], sa[j % 2][nt]);
    }
    if (need_mask(kway)) {
      asm volatile("");
      apply_mask(sa, kway);
    }
    float mx[QT];
    tile_max(sa, mx);
    raise(mx);
  }
  for (int st = 0; st < nsteps; st += 2) {
    step(st, std::integral_constant<int, 0>{}, sa, sb);
    if (st + 1 < nsteps) step(st + 1, std::integral_constant<int, 1>{}, sb, sa);
  }

  // ---- KW = 2: the waves of the second key way hand their state over through LDS (lane for lane); those of the
  // first merge it into theirs and go on to the epilogue
  if (KW > 1) {
    constexpr int REG = DT * 16 + 4;  // floats per lane
    float* mg = reinterpret_cast<float*>(lds) + wave * REG * 64 + lane;
    __syncthreads();  // every wave is done with the K/V tiles
    if (kway == 1) {
      mg[0] = m_i[0]; mg[64] = l_i[0]; mg[128] = lp_i[0];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) mg[(4 + dt * 16 + e) * 64] = o[dt][0][e];
    }
    __syncthreads();
    if (kway == 1) return;
    const float m1 = mg[0];
    const float m = fmaxf(m_i[0], m1);
    const float a0 = m_i[0] == -INFINITY ? 0.f : fast_exp2(m_i[0] - m);
    const float a1 = m1 == -INFINITY ? 0.f : fast_exp2(m1 - m);
    l_i[0] = l_i[0] * a0 + mg[64] * a1;
    if (KFN) lp_i[0] = lp_i[0] * a0 + mg[128] * a1;
    m_i[0] = m;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[dt][0][e] = o[dt][0][e] * a0 + mg[(4 + dt * 16 + e) * 64] * a1;
  }

  // ---- epilogue
  if (KW > 1 || QW > 1) {
    // Eight waves run with one workgroup per CU, so nothing hides the epilogue: stored straight from the
    // accumulators, an instruction writes 16 bytes to each of 32 rows, and the 8 MB of Llama-3-8B's S = 1024
    // output take 3.5 us as half a million partial-line writes.  Each wave turns its 32 x D tile around in LDS
    // instead - the part of the merge area only it has read, or with QW = 2 a region of its own behind the K / V
    // tiles - and stores whole rows, 16 bytes per lane.
    constexpr int LDO = kAttnStageRow<D>;  // halfs per staged row (the padding spreads the rows over the banks)
    static_assert(32 * LDO * 2 <= (DT * 16 + 4) * 64 * 4, "the staged tile fits the wave's merge area");
    half_t* stage = QW > 1 ? lds + L::BYTES / 2 + wave_all * 32 * LDO
                           : reinterpret_cast<half_t*>(reinterpret_cast<float*>(lds) + wave * (DT * 16 + 4) * 64);
    const float l = pair_sum(l_i[0]);
    const float lp = KFN ? pair_sum(lp_i[0]) * kInvNegLnScale : 1.0f;
    const float inv = a.out_scale / l;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4v hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] = (half_t)(o[dt][0][rq * 4 + e] * inv);
        *reinterpret_cast<half4v*>(stage + l32 * LDO + dt * 32 + rq * 8 + g * 4) = hv;
      }
    // (the wave's own LDS writes are visible to its own reads after the wait the compiler places; no barrier)
    constexpr int CPRO = D / 8;          // 16-byte chunks per row
    constexpr int RPI = 64 / CPRO;       // rows per store instruction
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
      const int row = i * RPI + lane / CPRO, chunk = lane % CPRO;
      const half8v v = *reinterpret_cast<const half8v*>(stage + row * LDO + chunk * 8);
      const int q = qw0 + row;
      if (q < a.S) *reinterpret_cast<half8v*>(a.out + (int64_t)q * a.ldo + h * D + chunk * 8) = v;
    }
    const int q = qidx[0];
    if (q < a.S && g == 0) {
      if (a.lse != nullptr) a.lse[(int64_t)h * a.S + q] = (m_i[0] + fast_log2(l)) * kLn2;
      if (KFN && a.lse_pert != nullptr) a.lse_pert[(int64_t)h * a.S + q] = (m_i[0] + fast_log2(lp)) * kLn2;
    }
    return;
  }
#pragma unroll
  for (int nt = 0; nt < QT; ++nt) {
    const float l = pair_sum(l_i[nt]);
    const float lp = KFN ? pair_sum(lp_i[nt]) * kInvNegLnScale : 1.0f;
    const float inv = a.out_scale / l;
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
      if (KFN && a.lse_pert != nullptr) a.lse_pert[(int64_t)h * a.S + q] = (m_i[nt] + fast_log2(lp)) * kLn2;
    }
  }
}

// The body lives in a device function: it uses device-only types (buffer descriptors) that the host pass
// of the compiler must not be asked to instantiate.
// which instantiations run the pipelined body, and its LDS (two K tiles, two V tiles)
template <int QT, int KF, int KW>
constexpr bool kAttnPipe = QT == 1 && KF != 1;
// (QW = 2: the K / V tiles, then a staged output tile per wave)
template <int D, int KW, int QW>
constexpr int kAttnPipeLds = KW * AttnLds<D>::BYTES + (QW > 1 ? 8 * 32 * kAttnStageRow<D> * 2 : 0);

template <int D, int QT, int KF, int KW, int QW = 1>
__global__ __launch_bounds__(256 * KW * QW) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_fwd_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  if constexpr (kAttnPipe<QT, KF, KW>) attn_fwd_pipe_body<D, QT, KF, KW, QW>(a, lds, a.q);
  else attn_fwd_body<D, QT, KF, KW>(a, lds, a.q);
}

template <int D, int KF, bool FP8>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_split_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  attn_fwd_body<D, 1, KF, 1, true, FP8>(a, lds, a.q);
}

template <int D, int QT, int KF, int KW, int QW = 1>
static int launch_attn_t(const AttnArgs& a, hipStream_t stream) {
  using L = AttnLds<D>;
  static_assert(QW == 1 || kAttnPipe<QT, KF, KW>, "eight query groups: the pipelined body");
  constexpr int BQ = 4 * 32 * QT * QW;
  constexpr int LDS = kAttnPipe<QT, KF, KW> ? kAttnPipeLds<D, KW, QW> : KW * L::BYTES;
  static_assert(KW == 1 || 4 * QT * (D / 2 + 4) * 64 * 4 <= LDS, "the merge area fits the K/V stages");
  constexpr auto kern = attn_fwd_kernel<D, QT, KF, KW, QW>;
  if (set_max_lds<kern, LDS>() != 0) return -1;
  const dim3 grid(((a.S + BQ - 1) / BQ) * a.Hq);
  hipLaunchKernelGGL(kern, grid, dim3(256 * KW * QW), LDS, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int D, int KW>
static int launch_attn_kf(const AttnArgs& a, int kf, hipStream_t stream) {
  return kf == 0 ? launch_attn_t<D, 1, 0, KW>(a, stream)
                 : (kf == 1 ? launch_attn_t<D, 1, 1, KW>(a, stream) : launch_attn_t<D, 1, 2, KW>(a, stream));
}

// Few new tokens against a long prefix; returns 1 when the call is not of that kind.
// Workgroups aimed at (two per CU) and the most runs the key axis is cut into: every run adds a partial result per
// (head, token) that the merge kernel reads, eight runs per round trip.  16 tokens, 32768 keys: Llama-3-8B's 8 KV
// heads 57.8 us with 64 runs, 52.8 us with 32; 32 KV heads want the 512 workgroups (134 us; 148 us with 256)
constexpr int kSplitTargetWorkgroups = 512;
constexpr int kSplitMaxRuns = 32;
constexpr int kSplitMinTiles = 4;            // key tiles per workgroup, at least
template <int D, int KF, bool FP8>
static int launch_attn_split_t(const AttnArgs& a, int nwg, hipStream_t stream) {
  using L = AttnLds<D>;
  constexpr auto kern = attn_split_kernel<D, KF, FP8>;
  if (set_max_lds<kern, L::BYTES>() != 0) return -1;
  hipLaunchKernelGGL(kern, dim3(nwg), dim3(256), L::BYTES, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// Key tiles per workgroup and number of runs for a call, 0 = the call is not of this kind: at least kSplitMinKeys
// keys and either few new tokens or so few that the prefill kernel would start at most kSplitMaxPrefillWorkgroups
// workgroups, each walking the whole key axis alone (chunks of a long prompt, speculative tokens).
// (Llama-3-8B heads: 64 tokens against 4096 keys 81.5 -> 41.8 us for the whole block, 128 against 8192 166 -> 87 us,
// 512 against 32768 506 -> 364 us; 512 against 2048 level)
constexpr int kSplitMaxPrefillWorkgroups = 128;
static int split_plan(int S, int Hq, int Hkv, int Ltot, int* nsplit) {
  *nsplit = 0;
  if (S < 1 || Ltot < kSplitMinKeys) return 0;
  const bool few = S <= kFewMaxQueries;
  if (!few && (int64_t)((S + 127) / 128) * Hq > kSplitMaxPrefillWorkgroups) return 0;
  const int rows = (Hq / Hkv) * S;
  const int base = ((rows + 127) / 128) * Hkv;  // workgroups per run of keys
  const int nkt = (Ltot + kKeyTile - 1) / kKeyTile;
  int runs = kSplitTargetWorkgroups / base;
  runs = runs < 1 ? 1 : (runs > kSplitMaxRuns ? kSplitMaxRuns : runs);
  if (!few && runs < 2) return 0;
  int tiles = (nkt + runs - 1) / runs;
  tiles = tiles < kSplitMinTiles ? kSplitMinTiles : tiles;
  *nsplit = (nkt + tiles - 1) / tiles;
  return tiles;
}

int64_t split_attn_workspace_bytes(int S, int Hq, int Hkv, int D, int Ltot) {
  int nsplit;
  if ((D != 64 && D != 128) || Hkv < 1 || split_plan(S, Hq, Hkv, Ltot, &nsplit) == 0) return 0;
  return (int64_t)Hq * nsplit * S * (D + 4) * 4;
}

static int launch_attn_split(const AttnArgs& a, hipStream_t stream) {
  const int Ltot = a.P + a.S;
  const int kf = a.lse_pert == nullptr ? 0 : ((a.noise == nullptr && a.tau == 1.0f) ? 2 : 1);
  if (a.pj != nullptr || a.ws == nullptr || (a.D != 64 && a.D != 128) || (a.k8 != nullptr && (a.v8 == nullptr || kf != 0)))
    return 1;
  int nsplit;
  const int tiles = split_plan(a.S, a.Hq, a.Hkv, Ltot, &nsplit);
  if (tiles == 0) return 1;
  const int base = (((a.Hq / a.Hkv) * a.S + 127) / 128) * a.Hkv;
  if (a.ws_bytes < (int64_t)a.Hq * nsplit * a.S * (a.D + 4) * 4) return 1;
  AttnArgs b = a;
  b.split_tiles = tiles;
  const int nwg = nsplit * base;
  int rc;
  if (a.D == 128) {
    if (a.k8 != nullptr) rc = launch_attn_split_t<128, 0, true>(b, nwg, stream);
    else rc = kf == 0 ? launch_attn_split_t<128, 0, false>(b, nwg, stream)
                      : (kf == 1 ? launch_attn_split_t<128, 1, false>(b, nwg, stream) : launch_attn_split_t<128, 2, false>(b, nwg, stream));
  } else {
    if (a.k8 != nullptr) rc = launch_attn_split_t<64, 0, true>(b, nwg, stream);
    else rc = kf == 0 ? launch_attn_split_t<64, 0, false>(b, nwg, stream)
                      : (kf == 1 ? launch_attn_split_t<64, 1, false>(b, nwg, stream) : launch_attn_split_t<64, 2, false>(b, nwg, stream));
  }
  if (rc != 0) return rc;
  return launch_attention_few_combine(b, nsplit, stream);
}

int launch_attention(const AttnArgs& a, hipStream_t stream) {
  if (a.S <= 0) return 0;
  {
    const int r = launch_attn_split(a, stream);
    if (r <= 0) return r;
  }
  if (a.S <= kFewMaxQueries) {
    const int r = launch_attention_few(a, stream);
    if (r <= 0) return r;
  }
  if (a.k == nullptr || a.v == nullptr) return -1;  // (fp8 caches are read by the two variants above only)
  const int kf = a.lse_pert == nullptr ? 0 : ((a.noise == nullptr && a.tau == 1.0f) ? 2 : 1);
  // At most one workgroup per CU and a long key axis: eight waves per workgroup walk the keys two tiles at a
  // time (Llama-3-8B, four-wave -> eight-wave kernel: S = 1024 26 -> 20.8 us, S = 768 20.0 -> 17.5 us, S = 512
  // 14.4 -> 14.3 us, S = 256 9.6 -> 11.0 us; with more than one workgroup per CU the four-wave kernel is ahead:
  // S = 1280 33 vs 43 us)
  const int64_t wgs = (int64_t)((a.S + 127) / 128) * a.Hq;
  const bool two = wgs <= kTwoWayMaxWorkgroups && a.P + a.S >= kTwoWayMinKeys;
  // One round of four-wave workgroups under a causal mask: eight query groups per workgroup instead (128-wide
  // heads; with 64-wide heads it is level at best: 71 heads S = 768 17.2 -> 17.7 us, 32 heads S = 2048 36.3 -> 35.5)
  const int64_t wgs8 = (int64_t)((a.S + 255) / 256) * a.Hq;
  const bool eight = a.causal && kf != 1 && !two && wgs8 >= kEightGroupMinWorkgroups && wgs8 <= kEightGroupMaxWorkgroups;
  if (a.D == 128) {
    if (eight) return kf == 0 ? launch_attn_t<128, 1, 0, 1, 2>(a, stream) : launch_attn_t<128, 1, 2, 1, 2>(a, stream);
    return two ? launch_attn_kf<128, 2>(a, kf, stream) : launch_attn_kf<128, 1>(a, kf, stream);
  }
  if (a.D == 64) {
    // 64-wide heads leave registers for 64 queries per wave: half the LDS reads and K/V loads per flop.  It pays
    // once the twice-as-large workgroups still fill the chip three times over (S = 3072 x 71 heads: 138.4 ->
    // 133.7 us, S = 4096: 235 -> 224 us, S = 8192: 782 -> 718 us; S = 2048: 62.3 -> 67.5 us)
    const int64_t wgs2 = (int64_t)((a.S + 255) / 256) * a.Hq;
    // (the general KeyFormer variant has no registers for it)
    if (kf != 1 && wgs2 >= kWideMinWorkgroups)
      return kf == 0 ? launch_attn_t<64, 2, 0, 1>(a, stream) : launch_attn_t<64, 2, 2, 1>(a, stream);
    return two ? launch_attn_kf<64, 2>(a, kf, stream) : launch_attn_kf<64, 1>(a, kf, stream);
  }
  return -1;
}

}  // namespace tri
