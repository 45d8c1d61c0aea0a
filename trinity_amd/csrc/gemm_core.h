// Tiled fp16 MFMA GEMM main loops for gfx950, shared by the FFN and the
// QKV-projection kernels.  Two loops live here: `gemm_mainloop_dma`, the fast
// path (K a multiple of 32: global -> LDS without passing through registers,
// four stages), and `gemm_mainloop`, the general one (any K that is a multiple
// of 8, register-staged, two stages).
//
// Roles.  The weight tile W[k, n] (row-major, n contiguous) feeds MFMA source 0
// through LDS transpose reads, the activation tile X[m, k] feeds source 1, so
// every accumulator lane owns one token (column l % 32) and four consecutive
// output columns per register quad.  Per-token epilogue factors (RMSNorm row
// scale, per-head RMS of q/k) are therefore per-lane scalars, and stores are
// 8 bytes per lane with lanes l / l^32 adjacent.
//
// LDS layout per stage (padding chosen so that the reads below are free of
// bank conflicts):
//   X tile [BM][64 + 8] halfs  - 16-byte reads, row stride 144 B
//   W tile [64][BN + 32] halfs - transpose reads touch 4 rows x 64 B per
//                                half-wave, row stride = 64 B mod 256 B
// Two stages; global loads for tile t+1 are issued into registers before the
// MFMAs of tile t and written to the other stage afterwards (one barrier per
// k-tile).
#if (defined(TRI_BF16) && !defined(TRI_GEMM_CORE_H_BF16)) || (!defined(TRI_BF16) && !defined(TRI_GEMM_CORE_H_F16))
#ifdef TRI_BF16
#define TRI_GEMM_CORE_H_BF16
#else
#define TRI_GEMM_CORE_H_F16
#endif
#include "common.h"

namespace tri {

template <int BM_, int BN_, int WM_, int WN_>
struct GemmTile {
  static constexpr bool kDma = false;
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int BK = 64;
  static constexpr int NT = WM * WN * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int XS = BK + 8;
  static constexpr int WS = BN + 32;
  static constexpr int X_HALFS = BM * XS, W_HALFS = BK * WS;
  static constexpr int STAGE_HALFS = X_HALFS + W_HALFS;
  static constexpr int LDS_BYTES = 2 * STAGE_HALFS * 2;
  static constexpr int XCH = BM * BK / 8 / NT;
  static constexpr int WCH = BK * BN / 8 / NT;
  static constexpr int XROWS_PER_PASS = NT / 8;          // X rows covered by one chunk pass
  static constexpr int WROWS_PER_PASS = NT / (BN / 8);   // W k-rows covered by one chunk pass
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tiles are multiples of 32");
  static_assert(NT % (BN / 8) == 0 && (BM * BK / 8) % NT == 0 && (BK * BN / 8) % NT == 0, "chunk mapping");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

// ---- activation functions of the epilogues
// GELU(a) = a * Phi(a) with the normal distribution function from Abramowitz & Stegun 26.2.17:
//   Q(t) = Phi(-t) = phi(t) * (b1 u + ... + b5 u^5), u = 1 / (1 + p t), |error| < 7.5e-8 for t >= 0.
// Branch-free and a fifth of the instructions of erff(); the absolute error of |a| * 7.5e-8 is far below the
// fp16 spacing of the result everywhere.
__device__ __forceinline__ float gelu_erf(float a) {
  const float t = fabsf(a);
  const float u = __builtin_amdgcn_rcpf(fmaf(0.2316419f, t, 1.0f));
  float poly = fmaf(u, 1.330274429f, -1.821255978f);
  poly = fmaf(u, poly, 1.781477937f);
  poly = fmaf(u, poly, -0.356563782f);
  poly = fmaf(u, poly, 0.319381530f);
  // phi(t) = exp(-t^2 / 2) / sqrt(2 pi)
  const float q = poly * u * 0.3989422804014327f * fast_exp2(t * t * -0.72134752044448170f);
  return a * (a >= 0.f ? 1.0f - q : q);
}
// silu(a) = a / (1 + exp(-a)) with the hardware reciprocal (1 ulp) in place of an IEEE division
__device__ __forceinline__ float silu(float a) {
  return a * __builtin_amdgcn_rcpf(1.0f + fast_exp2(a * -1.4426950408889634f));
}

// Map a linear workgroup id to a tile: first undo the round-robin of
// workgroups over the 8 XCDs (so one XCD's L2 sees a contiguous tile range),
// then walk tiles in groups of `group_m` token tiles per weight tile.
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int per = total >> 3, rem = total & 7;
  const int xcd = pid & 7, idx = pid >> 3;
  const int p = xcd * per + (xcd < rem ? xcd : rem) + idx;
  const int in_group = group_m * tiles_n;
  const int gid = p / in_group;
  const int first_m = gid * group_m;
  const int gsm = min(tiles_m - first_m, group_m);
  const int r = p - gid * in_group;
  tm = first_m + r % gsm;
  tn = r / gsm;
}

// acc[ni][mi] += W-tile^T x X-tile over the whole K range.
//   xbase        X + m0 * ldx (row clamping is applied here)
//   colmap(chunk, ldw) -> pointer to row 0 of the weight column that LDS
//   column chunk `chunk` (8 columns) holds, clamped to a valid column.
// Rows of X past M are clamped, k past K reads as zero (K % 8 == 0).
template <class T, class ColMap>
__device__ __forceinline__ void gemm_mainloop(const half_t* __restrict__ x, int64_t ldx, int m0, int M, int K,
                                              ColMap colmap, half_t* lds, float16v (&acc)[T::NI][T::MI]) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;

  // ---- global -> register staging coordinates
  const int xkc = t & 7;            // k chunk (8 halfs) inside the 64-wide k tile
  const int xr0 = t >> 3;           // first X row of this thread
  const int wcc = t % (T::BN / 8);  // weight column chunk
  const int wk0 = t / (T::BN / 8);  // first weight k row of this thread
  int64_t ldw = 0;
  const half_t* wcol = colmap(wcc, ldw);
  const half_t* xp[T::XCH];
#pragma unroll
  for (int i = 0; i < T::XCH; ++i) {
    int row = m0 + xr0 + i * T::XROWS_PER_PASS;
    row = row < M ? row : M - 1;
    xp[i] = x + (int64_t)row * ldx + xkc * 8;
  }
  uint4v xreg[T::XCH], wreg[T::WCH];
  const uint4v zero4 = {0u, 0u, 0u, 0u};

  auto load_global = [&](int k0) {
    const bool xok = (k0 + xkc * 8) < K;
#pragma unroll
    for (int i = 0; i < T::XCH; ++i) xreg[i] = xok ? *reinterpret_cast<const uint4v*>(xp[i] + k0) : zero4;
#pragma unroll
    for (int i = 0; i < T::WCH; ++i) {
      const int kr = k0 + wk0 + i * T::WROWS_PER_PASS;
      wreg[i] = kr < K ? *reinterpret_cast<const uint4v*>(wcol + (int64_t)kr * ldw) : zero4;
    }
  };
  auto store_lds = [&](int stage) {
    half_t* xs = lds + stage * T::STAGE_HALFS;
    half_t* ws = xs + T::X_HALFS;
#pragma unroll
    for (int i = 0; i < T::XCH; ++i)
      *reinterpret_cast<uint4v*>(xs + (xr0 + i * T::XROWS_PER_PASS) * T::XS + xkc * 8) = xreg[i];
#pragma unroll
    for (int i = 0; i < T::WCH; ++i)
      *reinterpret_cast<uint4v*>(ws + (wk0 + i * T::WROWS_PER_PASS) * T::WS + wcc * 8) = wreg[i];
  };

  // ---- LDS fragment read offsets (halfs)
  const int xfrag = (wm * T::TM + l32) * T::XS + g * 8;
  const int wfrag = (g * 8 + ((lane & 15) >> 2)) * T::WS + wn * T::TN + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;

  const int KT = (K + T::BK - 1) / T::BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = (kt + 1) < KT;
    if (more) load_global((kt + 1) * T::BK);
    const half_t* xs = lds + (kt & 1) * T::STAGE_HALFS;
    const half_t* ws = xs + T::X_HALFS;
#pragma unroll
    for (int kk = 0; kk < T::BK / 16; ++kk) {
      half8v wf[T::NI], xf[T::MI];
#pragma unroll
      for (int ni = 0; ni < T::NI; ++ni) {
        const half_t* p = ws + wfrag + kk * 16 * T::WS + ni * 32;
        wf[ni] = cat8(lds_read_tr16(p), lds_read_tr16(p + 4 * T::WS));
      }
#pragma unroll
      for (int mi = 0; mi < T::MI; ++mi) xf[mi] = lds_read8(xs + xfrag + mi * 32 * T::XS + kk * 16);
#pragma unroll
      for (int ni = 0; ni < T::NI; ++ni)
#pragma unroll
        for (int mi = 0; mi < T::MI; ++mi) acc[ni][mi] = mfma32(wf[ni], xf[mi], acc[ni][mi]);
    }
    if (more) store_lds((kt + 1) & 1);
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Fast path: direct-to-LDS loads, BK = 32, four stages.
//
// `global_load_lds_dwordx4` writes the 64 lanes' 16-byte chunks to 1 KB of
// contiguous LDS, so LDS tiles cannot be padded; they are XOR-swizzled
// instead, by choosing which global chunk each lane fetches:
//   X tile [BM][32] halfs (4 chunks / row): chunk c of row r sits at slot
//       c ^ ((r >> 2) & 3)            -> 16-byte fragment reads conflict-free
//   W tile [32][BN] halfs (BN/8 chunks / row): chunk c of row k sits at slot
//       c ^ ((k & 3) << 2)            -> transpose reads conflict-free
// Schedule per 32-wide k tile t (one barrier):
//   MFMAs of k16-step 0 while reading the fragments of step 1;
//   wait for this wave's own loads of tile t+1, barrier (publishes tile t+1
//   and retires tile t-1 for everybody);
//   issue the loads of tile t+3 into the stage tile t-1 used, read the first
//   fragments of tile t+1, MFMAs of step 1.
// Loads therefore have two full tiles of MFMA time to land.
// ---------------------------------------------------------------------------
// WLD_ is the width of the weight tile's LDS rows (128 or 256 columns); BN_ may be smaller, in which case the
// columns past BN_ are simply never loaded (their lanes are switched off): that gives tile widths of any multiple
// of 32 for shapes whose column count fills the chip badly with 128 / 256 wide tiles.
template <int BM_, int BN_, int WM_, int WN_, int WLD_ = BN_>
struct DmaTile {
  static constexpr bool kDma = true;
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, WLD = WLD_;
  static constexpr int BK = 32, NSTAGE = 4;
  static constexpr int NW = WM * WN, NT = NW * 64;
  static constexpr int TM = BM / WM, TN = BN / WN;
  static constexpr int MI = TM / 32, NI = TN / 32;
  static constexpr int X_HALFS = BM * BK, W_HALFS = BK * WLD;
  static constexpr int STAGE_HALFS = X_HALFS + W_HALFS;
  // the 64-deep loop of the 256- and 128-row tiles (gemm_mainloop_dma64) keeps 2 activation and 3 weight buffers
  // (3 and 3 for wave tiles of few MFMAs per k16 step, see there)
  static constexpr bool DEEP = MI * NI <= 6;
  static constexpr int K64_BYTES = (BM == 256 || BM == 128) ? ((DEEP ? 3 : 2) * BM * 64 + 3 * WLD * 64) * 2 : 0;
  static constexpr int LDS_BYTES = NSTAGE * STAGE_HALFS * 2 > K64_BYTES ? NSTAGE * STAGE_HALFS * 2 : K64_BYTES;
  static constexpr int X_INSTR = BM / 16 / NW;   // wave-level load instructions per wave per tile (X)
  static constexpr int W_INSTR = WLD / 16 / NW;  // (W)
  static constexpr int CPRW = WLD / 8;           // 16-byte chunk slots per W row in LDS
  static constexpr int CHUNKS = BN / 8;          // chunks per row that hold data
  static constexpr int LOADS_PER_TILE = X_INSTR + W_INSTR;
  static_assert(BM % (16 * NW) == 0 && WLD % (16 * NW) == 0 && BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile split");
  static_assert(CPRW == 16 || CPRW == 32, "LDS rows are 128 or 256 columns wide");
  static_assert(BN <= WLD && BN % 8 == 0, "logical width fits the LDS row");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

__device__ __forceinline__ void load_to_lds16(const half_t* g, half_t* l) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g,
                                   (__attribute__((address_space(3))) void*)l, 16, 0, 0);
}

// s_waitcnt vmcnt(n) leaving the other counters unconstrained (gfx9 encoding)
#define TRI_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | 0x0F70)
#define TRI_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)

// ---------------------------------------------------------------------------
// 64-deep k tiles for the 256- and 128-row tiles (K % 64 == 0).
//
// A load instruction then fetches 8 rows x 128 bytes of the activations - whole cache lines - where the 32-deep
// loop fetches 16 rows x 64 bytes: a half line costs the L1 a whole line's fill, and with half lines the fills
// (64 bytes per clock and CU) take as long as the MFMAs of the tile.  One barrier serves 64 MFMAs per wave
// instead of 32.  The activation tile [256][64] sits in 2 buffers, the weight tile in 3 (row-major weights:
// [64][WLD]; K-contiguous weights: [WLD][64], the activation tile's format): the loads of activations for tile
// t + 2 are issued in the last k16 step of tile t (right after the barrier that frees the buffer), the loads of
// weights for tile t + 2 in its first, and the wait before the barrier leaves the weight loads in flight.  256 x 256: 160 KB of LDS; 256 x 128: 112 KB.
//   row-major [2048, 4096] x [4096, 28672]: 488 -> 460 us; K-contiguous weights: 493 -> 451 us (same box,
//   alternating launches, both with the compiler's schedule; the explicit schedule below takes off another 5 %)
// Chunk c of activation row r (8 chunks of 16 bytes) sits at slot c ^ ((r >> 1) & 7): two rows span the 64 banks.
// The MFMAs of a k16 step walk the accumulators in a serpentine, so that consecutive instructions always share
// one source operand.
//   wmap: NTL ? rowmap(nloc) : colmap(chunk, ldw), as in the 32-deep loops.
// ---------------------------------------------------------------------------
template <class T>
constexpr bool kHasK64 = T::kDma && (T::WLD == 256 || T::WLD == 128) &&
                         ((T::BM == 256 && ((T::WM == 2 && T::WN == 2) || (T::WM == 4 && T::WN == 1))) || (T::BM == 128 && T::WM == 2 && T::WN == 2));

template <class T, bool NTL, bool SWAP, class WMap>
__device__ __forceinline__ void gemm_mainloop_dma64(const half_t* __restrict__ x, int64_t ldx, int m0, int M, int K,
                                                    WMap wmap, half_t* lds, float16v (&acc)[T::NI][T::MI]) {
  static_assert(kHasK64<T>, "256-row tiles with 2 x 2 or 4 x 1 waves, 128-row tiles with 2 x 2");
  constexpr int NW = 4, BK = 64, WLD = T::WLD;
  constexpr int XB = T::BM * BK, WB = WLD * BK;            // halfs per buffer
  constexpr int XI = T::BM / 8 / NW;                       // 1 KB load instructions per wave and activation tile
  constexpr int W_INSTR = WB / 512 / NW;                   // 1 KB load instructions per wave and weight tile
  constexpr bool DEEP = T::DEEP;
  constexpr int NXB = DEEP ? 3 : 2;  // activation buffers
  static_assert((NXB * XB + 3 * WB) * 2 <= T::LDS_BYTES, "LDS budget of the 64-deep loop");
  half_t* xbuf = lds;
  half_t* wbuf = lds + NXB * XB;
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  const int KT = K / BK;

  const half_t* xsrc[XI];
  const half_t* wsrc[W_INSTR];
  int64_t ldw = 0;
  bool wlive = true;  // this lane's chunk holds data (always, unless the tile is narrower than its LDS rows)
#pragma unroll
  for (int i = 0; i < XI; ++i) {
    const int rloc = (i * NW + wave) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ ((rloc >> 1) & 7);
    int row = m0 + rloc;
    row = row < M ? row : M - 1;
    xsrc[i] = x + (int64_t)row * ldx + c * 8;
  }
#pragma unroll
  for (int i = 0; i < W_INSTR; ++i) {
    if constexpr (NTL) {
      const int nloc = (i * NW + wave) * 8 + (lane >> 3);
      wsrc[i] = wmap(nloc) + ((lane & 7) ^ ((nloc >> 1) & 7)) * 8;
    } else {
      const int p = (i * NW + wave) * 64 + lane;
      const int krow = p / T::CPRW, slot = p % T::CPRW;
      const int chunk = slot ^ ((krow & 3) << 2);
      if (T::CHUNKS < T::CPRW) wlive = chunk < T::CHUNKS;  // the same for every i: a lane keeps its column chunk
      wsrc[i] = wmap(chunk < T::CHUNKS ? chunk : 0, ldw) + (int64_t)krow * ldw;
    }
  }
  const int64_t wstep = NTL ? (int64_t)BK : (int64_t)BK * ldw;   // halfs per k tile (wave-uniform)
  // load instruction i of a tile step: the XI activation loads of tile kt_x, then the weight loads of tile kt_w
  auto load_one = [&](int kt_x, int xbn, int kt_w, int wbn, int i) {
    if (i < XI) load_to_lds16(xsrc[i] + (int64_t)kt_x * BK, xbuf + xbn * XB + (i * NW + wave) * 512);
    else if (wlive) load_to_lds16(wsrc[i - XI] + (int64_t)kt_w * wstep, wbuf + wbn * WB + ((i - XI) * NW + wave) * 512);
  };

  // ---- fragment read offsets (halfs)
  const int sx = (l32 >> 1) & 7;
  int xoff[4], woff_t[4], woff_n[T::NI];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) {
    xoff[kk] = (wm * T::TM + l32) * BK + (((kk * 2 + g) ^ sx) << 3);
    woff_t[kk] = (wn * T::TN + l32) * BK + (((kk * 2 + g) ^ sx) << 3);
  }
  const int j4 = (lane & 15) >> 2;
#pragma unroll
  for (int ni = 0; ni < T::NI; ++ni) {
    const int chunk = (wn * T::TN + ni * 32) / 8 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    woff_n[ni] = (g * 8 + j4) * WLD + ((chunk ^ (j4 << 2)) << 3) + (lane & 1) * 4;
  }
  // Wave tiles of few MFMAs per k16 step (DEEP) read their fragments two steps ahead into four register sets:
  // one step - six MFMAs, 200 cycles, for the 64 x 96 wave tile - is shorter than an LDS read takes under load,
  // and every step then began by waiting for its fragments.
  constexpr int NFB = DEEP ? 4 : 2;
  half8v wf[NFB][T::NI], xf[NFB][T::MI];
  // fragment i of k16 step kk of the tile in buffers (xb, wb): the weight fragments first, then the activations'
  auto read_one = [&](int xb, int wb, int kk, int buf, int i) {
    if (i < T::NI) {
      const half_t* ws = wbuf + wb * WB;
      if constexpr (NTL) {
        wf[buf][i] = lds_read8(ws + woff_t[kk] + i * 32 * BK);
      } else {
        const half_t* p = ws + woff_n[i] + kk * 16 * WLD;
        wf[buf][i] = cat8(lds_read_tr16(p), lds_read_tr16(p + 4 * WLD));
      }
    } else {
      xf[buf][i - T::NI] = lds_read8(xbuf + xb * XB + xoff[kk] + (i - T::NI) * 32 * BK);
    }
  };
  auto mfma_one = [&](int buf, int i) {
    const int ni = i / T::MI, mq = i % T::MI;
    const int mi = (ni & 1) ? T::MI - 1 - mq : mq;
    acc[ni][mi] = SWAP ? mfma32(xf[buf][mi], wf[buf][ni], acc[ni][mi]) : mfma32(wf[buf][ni], xf[buf][mi], acc[ni][mi]);
  };
  constexpr int NMFMA = T::NI * T::MI, NFRAG = T::NI + T::MI, L = XI + W_INSTR;
  static_assert(NFRAG <= NMFMA, "a fragment read per MFMA slot");
  // One k16 step, instruction by instruction: MFMA i, then its share of the tile step's loads (first step only)
  // and fragment read i of the next k16 step, with a schedule fence after every slot.  Left to the compiler (with
  // or without sched_group_barrier hints) the loads - each a chain of an M0 write, an address add and the load -
  // bunch up between two MFMAs and the matrix pipe idles: 488 -> 462 us for [2048, 4096] x [4096, 28672].
  // `loads`: 0 none, 1 the weight loads (tile kt_w into buffer wbn), 2 the activation loads (tile kt_x into xbn)
  auto step = [&](int buf, int loads, int kt_x, int xbn, int kt_w, int wbn, int rxb, int rwb, int rkk) {
    const int first = loads == 1 ? XI : 0, n = loads == 1 ? W_INSTR : loads == 2 ? XI : 0;
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      mfma_one(buf, i);
#pragma unroll
      for (int j = i * n / NMFMA; j < (i + 1) * n / NMFMA; ++j) load_one(kt_x, xbn, kt_w, wbn, first + j);
      if (i < NFRAG) read_one(rxb, rwb, rkk, buf ^ 1, i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto clampt = [&](int kt) { return kt < KT ? kt : KT - 1; };

  // issue order: X(0) W(0) X(1) W(1) | W(2) X(2) | W(3) X(3) | ...
#pragma unroll
  for (int i = 0; i < L; ++i) load_one(0, 0, 0, 0, i);
#pragma unroll
  for (int i = 0; i < L; ++i) load_one(clampt(1), 1, clampt(1), 1, i);
  TRI_WAIT_VMCNT(L);
  __builtin_amdgcn_s_barrier();
  if constexpr (DEEP) {
    // Fragment set kk holds k16 step kk of a tile; step (kt, kk) reads the fragments of the step two later, so all
    // reads of tile kt are over after its second step and the barrier sits in the middle of the tile.  These tiles
    // move many bytes per MFMA (256 x 96: 44 KB per 24 MFMAs of a wave, as long on the L1's 64 bytes per clock
    // as on the matrix pipe), and a wave that issues loads faster than they drain stalls with its MFMAs behind
    // it: with a third activation buffer nothing ties the loads of tile kt + 2 to a barrier any more, and they
    // are spread evenly over the four steps of tile kt.
    static_assert(L % 4 == 0, "the same number of loads in every k16 step");
    constexpr int LPS = L / 4;
#pragma unroll
    for (int i = 0; i < NFRAG; ++i) read_one(0, 0, 0, 0, i);
#pragma unroll
    for (int i = 0; i < NFRAG; ++i) read_one(0, 0, 1, 1, i);
    int xb = 0, wb = 0;  // buffers of tile kt
    // step `q` of a tile: MFMAs on fragment set q, loads [q LPS, (q + 1) LPS) of tile kt2 into (xb2, wb2), reads of
    // k16 step rkk of the tile in (rxb, rwb) into set (q + 2) % 4
    auto step4 = [&](int q, int kt2, int xb2, int wb2, int rxb, int rwb, int rkk) {
#pragma unroll
      for (int i = 0; i < NMFMA; ++i) {
        mfma_one(q, i);
#pragma unroll
        for (int j = q * LPS + i * LPS / NMFMA; j < q * LPS + (i + 1) * LPS / NMFMA; ++j) load_one(kt2, xb2, kt2, wb2, j);
        if (i < NFRAG) read_one(rxb, rwb, rkk, (q + 2) % 4, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    for (int kt = 0; kt < KT; ++kt) {
      const int xb1 = xb == 2 ? 0 : xb + 1, xb2 = xb1 == 2 ? 0 : xb1 + 1;
      const int wb1 = wb == 2 ? 0 : wb + 1, wb2 = wb1 == 2 ? 0 : wb1 + 1;
      const int kt2 = clampt(kt + 2);  // (past the end the loop keeps its load count, see below)
      __builtin_amdgcn_sched_barrier(0);
      step4(0, kt2, xb2, wb2, xb, wb, 2);
      step4(1, kt2, xb2, wb2, xb, wb, 3);
      // tile kt + 1 has landed (this wave's share; the barrier adds everybody's), half of tile kt + 2 is in flight
      __builtin_amdgcn_s_waitcnt(((2 * LPS) & 15) | 0x0070);  // vmcnt(2 LPS) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      step4(2, kt2, xb2, wb2, xb1, wb1, 0);
      step4(3, kt2, xb2, wb2, xb1, wb1, 1);
      xb = xb1;
      wb = wb1;
    }
    TRI_WAIT_VMCNT(0);
    return;
  }
#pragma unroll
  for (int i = 0; i < NFRAG; ++i) read_one(0, 0, 0, 0, i);
  int xb = 0, wb = 0;  // buffers of tile kt
  for (int kt = 0; kt < KT; ++kt) {
    const int wb1 = wb == 2 ? 0 : wb + 1, wb2 = wb1 == 2 ? 0 : wb1 + 1;
    // past the last tile the loop keeps its load count (the wait below assumes it): the last tile is fetched
    // again, into buffers that nobody reads any more
    const int kt2 = clampt(kt + 2);
    __builtin_amdgcn_sched_barrier(0);
    step(0, 1, 0, 0, kt2, wb2, xb, wb, 1);   // weights of tile kt + 2 into the buffer tile kt - 1 left
    step(1, 0, 0, 0, 0, 0, xb, wb, 2);
    step(0, 0, 0, 0, 0, 0, xb, wb, 3);
    // this wave's reads of tile kt are in its registers (other waves overwrite the tile's buffers right after
    // the barrier) and the loads of tile kt + 1 have landed; the weight loads of tile kt + 2 stay in flight
    __builtin_amdgcn_s_waitcnt((W_INSTR & 15) | 0x0070);  // vmcnt(W_INSTR) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // activations of tile kt + 2 into the buffer tile kt has just left: issued here, a k16 step before the top of
    // the next tile, they have four steps to land instead of three (the loop waits for them, not for the MFMAs)
    step(1, 2, kt2, xb, 0, 0, xb ^ 1, wb1, 0);
    xb ^= 1;
    wb = wb1;
  }
  TRI_WAIT_VMCNT(0);
}

// acc[ni][mi] += W-tile^T x X-tile over K (K % 32 == 0).
//   colmap(chunk, ldw) -> pointer to row 0 of the weight column that LDS
//   column chunk `chunk` (8 columns) holds, clamped to a valid column.
// SWAP exchanges the MFMA operands: acc[ni][mi] then holds X-tile x W-tile (rows = tokens in the registers,
// columns = weight columns across the lanes), the orientation in which fp32 partial tiles store coalesced.
template <class T, class ColMap, bool SWAP = false>
__device__ __forceinline__ void gemm_mainloop_dma(const half_t* __restrict__ x, int64_t ldx, int m0, int M, int K,
                                                  ColMap colmap, half_t* lds, float16v (&acc)[T::NI][T::MI]) {
  if constexpr (kHasK64<T>) {
    if (K % 64 == 0) {
      gemm_mainloop_dma64<T, false, SWAP>(x, ldx, m0, M, K, colmap, lds, acc);
      return;
    }
  }
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  const int KT = K / T::BK;

  // ---- load sources: every thread fetches the same logical chunk in all its instructions
  const half_t* xsrc[T::X_INSTR];
#pragma unroll
  for (int i = 0; i < T::X_INSTR; ++i) {
    const int rloc = (i * T::NW + wave) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ ((rloc >> 2) & 3);
    int row = m0 + rloc;
    row = row < M ? row : M - 1;
    xsrc[i] = x + (int64_t)row * ldx + c * 8;
  }
  const half_t* wsrc[T::W_INSTR];
  int64_t ldw = 0;
  bool wlive = true;  // this lane's chunk holds data (always, unless the tile is narrower than its LDS rows)
#pragma unroll
  for (int i = 0; i < T::W_INSTR; ++i) {
    const int p = (i * T::NW + wave) * 64 + lane;
    const int krow = p / T::CPRW, slot = p % T::CPRW;
    const int chunk = slot ^ ((krow & 3) << 2);
    if (T::CHUNKS < T::CPRW) wlive = chunk < T::CHUNKS;  // the same for every i (see above)
    wsrc[i] = colmap(chunk < T::CHUNKS ? chunk : 0, ldw) + (int64_t)krow * ldw;
  }
  // load instruction i of k tile `kt` into the stage of tile `slot` (slot == kt except past the end, see clampt):
  // the activation loads first, then the weight loads
  auto load_one = [&](int kt, int slot, int i) {
    half_t* st = lds + (slot & 3) * T::STAGE_HALFS;
    const int k0 = kt * T::BK;
    if (i < T::X_INSTR) {
      load_to_lds16(xsrc[i] + k0, st + (i * T::NW + wave) * 512);
    } else if (wlive) {
      const int j = i - T::X_INSTR;
      load_to_lds16(wsrc[j] + (int64_t)k0 * ldw, st + T::X_HALFS + (j * T::NW + wave) * 512);
    }
  };

  // ---- fragment read offsets (halfs)
  const int sx = (l32 >> 2) & 3;
  int xoff[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) xoff[kk] = (wm * T::TM + l32) * 32 + (((kk * 2 + g) ^ sx) << 3);
  const int j4 = (lane & 15) >> 2;
  int woff[T::NI];
#pragma unroll
  for (int ni = 0; ni < T::NI; ++ni) {
    const int chunk = (wn * T::TN + ni * 32) / 8 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    woff[ni] = T::X_HALFS + (g * 8 + j4) * T::WLD + ((chunk ^ (j4 << 2)) << 3) + (lane & 1) * 4;
  }
  half8v wf[2][T::NI], xf[2][T::MI];
  // fragment i of k16 step kk of tile kt: the weight fragments first, then the activations'
  auto read_one = [&](int kt, int kk, int buf, int i) {
    const half_t* base = lds + (kt & 3) * T::STAGE_HALFS;
    if (i < T::NI) {
      const half_t* p = base + woff[i] + kk * 16 * T::WLD;
      wf[buf][i] = cat8(lds_read_tr16(p), lds_read_tr16(p + 4 * T::WLD));
    } else {
      xf[buf][i - T::NI] = lds_read8(base + xoff[kk] + (i - T::NI) * 32 * 32);
    }
  };
  auto mfma_one = [&](int buf, int i) {
    const int ni = i / T::MI, mq = i % T::MI;
    const int mi = (ni & 1) ? T::MI - 1 - mq : mq;  // serpentine: consecutive MFMAs share a source operand
    acc[ni][mi] = SWAP ? mfma32(xf[buf][mi], wf[buf][ni], acc[ni][mi]) : mfma32(wf[buf][ni], xf[buf][mi], acc[ni][mi]);
  };
  constexpr int NMFMA = T::NI * T::MI, NFRAG = T::NI + T::MI, L = T::LOADS_PER_TILE;
  // One k16 step, instruction by instruction (see gemm_mainloop_dma64): MFMA i, its share of the tile's loads
  // (second step only) and of the fragment reads of the next k16 step, a schedule fence after every slot.
  auto step = [&](int buf, int load_kt, int load_slot, int rkt, int rkk) {
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      mfma_one(buf, i);
      if (load_slot >= 0) {
#pragma unroll
        for (int j = i * L / NMFMA; j < (i + 1) * L / NMFMA; ++j) load_one(load_kt, load_slot, j);
      }
#pragma unroll
      for (int j = i * NFRAG / NMFMA; j < (i + 1) * NFRAG / NMFMA; ++j) read_one(rkt, rkk, buf ^ 1, j);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // past the last tile the loop keeps its load count per iteration (the vmcnt waits assume it): the last tile is
  // fetched again, into the stage the tile past the end would have used - a stage nobody reads any more
  auto clampt = [&](int kt) { return kt < KT ? kt : KT - 1; };

#pragma unroll
  for (int i = 0; i < L; ++i) load_one(0, 0, i);
#pragma unroll
  for (int i = 0; i < L; ++i) load_one(clampt(1), 1, i);
#pragma unroll
  for (int i = 0; i < L; ++i) load_one(clampt(2), 2, i);
  TRI_WAIT_VMCNT(2 * L);
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < NFRAG; ++i) read_one(0, 0, 0, i);
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_sched_barrier(0);
    step(0, 0, -1, kt, 1);
    TRI_WAIT_VMCNT(L);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    step(1, clampt(kt + 3), kt + 3, kt + 1, 0);
  }
  TRI_WAIT_VMCNT(0);
}

// ---------------------------------------------------------------------------
// Fast path for K-contiguous weights (W stored as W^T [N][K], i.e. a [K, N] tensor whose stride along K is 1).
// Both operands are then rows of 32 consecutive k: the weight tile gets the activation tile's LDS format
// ([BN][32] halfs, chunk c of row n at slot c ^ ((n >> 2) & 3)) and both MFMA sources are filled by plain 16-byte
// LDS reads - no transpose reads.  Stages, schedule and accumulator layout are those of gemm_mainloop_dma, so the
// epilogues are shared.
//   rowmap(nloc) -> pointer to k = 0 of the weight column that LDS row `nloc` of the weight tile holds (clamped to
//   a valid column).
// ---------------------------------------------------------------------------
template <class T, class RowMap>
__device__ __forceinline__ void gemm_mainloop_dma_wt(const half_t* __restrict__ x, int64_t ldx, int m0, int M, int K,
                                                     RowMap rowmap, half_t* lds, float16v (&acc)[T::NI][T::MI]) {
  static_assert(T::WLD == T::BN && T::BN % (16 * T::NW) == 0, "whole 16-row load instructions per wave");
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  const int KT = K / T::BK;
  constexpr int WT_INSTR = T::BN / 16 / T::NW;
  constexpr int WT_HALFS = T::BN * T::BK;
  constexpr int STAGE = T::X_HALFS + WT_HALFS;
  static_assert(T::NSTAGE * STAGE * 2 <= T::LDS_BYTES, "the weight tile is no larger than in the row-major layout");
  if constexpr (kHasK64<T>) {
    if (K % 64 == 0) {
      gemm_mainloop_dma64<T, true, false>(x, ldx, m0, M, K, rowmap, lds, acc);
      return;
    }
  }

  const half_t* xsrc[T::X_INSTR];
#pragma unroll
  for (int i = 0; i < T::X_INSTR; ++i) {
    const int rloc = (i * T::NW + wave) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ ((rloc >> 2) & 3);
    int row = m0 + rloc;
    row = row < M ? row : M - 1;
    xsrc[i] = x + (int64_t)row * ldx + c * 8;
  }
  const half_t* wsrc[WT_INSTR];
#pragma unroll
  for (int i = 0; i < WT_INSTR; ++i) {
    const int nloc = (i * T::NW + wave) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ ((nloc >> 2) & 3);
    wsrc[i] = rowmap(nloc) + c * 8;
  }
  auto issue = [&](int kt, int slot) {
    half_t* st = lds + (slot & 3) * STAGE;
    const int k0 = kt * T::BK;
#pragma unroll
    for (int i = 0; i < T::X_INSTR; ++i) load_to_lds16(xsrc[i] + k0, st + (i * T::NW + wave) * 512);
#pragma unroll
    for (int i = 0; i < WT_INSTR; ++i) load_to_lds16(wsrc[i] + k0, st + T::X_HALFS + (i * T::NW + wave) * 512);
  };

  const int sx = (l32 >> 2) & 3;
  int xoff[2], woff[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    xoff[kk] = (wm * T::TM + l32) * 32 + (((kk * 2 + g) ^ sx) << 3);
    woff[kk] = T::X_HALFS + (wn * T::TN + l32) * 32 + (((kk * 2 + g) ^ sx) << 3);
  }
  half8v wf[2][T::NI], xf[2][T::MI];
  auto read_frags = [&](int kt, int kk, int buf) {
    const half_t* base = lds + (kt & 3) * STAGE;
#pragma unroll
    for (int ni = 0; ni < T::NI; ++ni) wf[buf][ni] = lds_read8(base + woff[kk] + ni * 32 * 32);
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi) xf[buf][mi] = lds_read8(base + xoff[kk] + mi * 32 * 32);
  };
  auto mfmas = [&](int buf) {
#pragma unroll
    for (int ni = 0; ni < T::NI; ++ni)
#pragma unroll
      for (int mi = 0; mi < T::MI; ++mi) acc[ni][mi] = mfma32(wf[buf][ni], xf[buf][mi], acc[ni][mi]);
  };
  constexpr int NMFMA = T::NI * T::MI, NREAD = T::NI + T::MI, L = T::X_INSTR + WT_INSTR;
  auto clampt = [&](int kt) { return kt < KT ? kt : KT - 1; };

  issue(0, 0);
  issue(clampt(1), 1);
  issue(clampt(2), 2);
  TRI_WAIT_VMCNT(2 * L);
  __builtin_amdgcn_s_barrier();
  read_frags(0, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_sched_barrier(0);
    read_frags(kt, 1, 1);
    mfmas(0);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      TRI_SGB(0x008, 1);
      if (i < NREAD) TRI_SGB(0x100, 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    TRI_WAIT_VMCNT(L);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    issue(clampt(kt + 3), kt + 3);
    read_frags(kt + 1, 0, 0);
    mfmas(1);
#pragma unroll
    for (int i = 0; i < NMFMA; ++i) {
      TRI_SGB(0x008, 1);
      if (i < L) TRI_SGB(0x020, 1);
      if (i < NREAD) TRI_SGB(0x100, 1);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  TRI_WAIT_VMCNT(0);
}

}  // namespace tri

#endif  // once per element type
