// Tiled fp16 MFMA GEMM main loop for gfx950, shared by the FFN and the
// QKV-projection kernels.
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
#pragma once
#include "common.h"

namespace tri {

template <int BM_, int BN_, int WM_, int WN_>
struct GemmTile {
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
//   wcol / ldw   this thread's weight column chunk at k = 0 (nullptr: the
//                chunk lies outside the matrix and reads as zero)
//   kscale       optional [K] factor applied to X along k (PreNorm weight)
template <class T, bool KSCALE>
__device__ __forceinline__ void gemm_mainloop(const half_t* __restrict__ x, int64_t ldx, int m0, int M, int K,
                                              const half_t* __restrict__ wcol, int64_t ldw,
                                              const half_t* __restrict__ kscale, half_t* lds,
                                              float16v (&acc)[T::NI][T::MI]) {
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;

  // ---- global -> register staging coordinates
  const int xkc = t & 7;            // k chunk (8 halfs) inside the 64-wide k tile
  const int xr0 = t >> 3;           // first X row of this thread
  const int wcc = t % (T::BN / 8);  // weight column chunk
  const int wk0 = t / (T::BN / 8);  // first weight k row of this thread
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
    half8v ks;
    if (KSCALE) {
      uint4v kv = xok ? *reinterpret_cast<const uint4v*>(kscale + k0 + xkc * 8) : zero4;
      __builtin_memcpy(&ks, &kv, 16);
    }
#pragma unroll
    for (int i = 0; i < T::XCH; ++i) {
      xreg[i] = xok ? *reinterpret_cast<const uint4v*>(xp[i] + k0) : zero4;
      if (KSCALE) {
        half8v h;
        __builtin_memcpy(&h, &xreg[i], 16);
        h = h * ks;
        __builtin_memcpy(&xreg[i], &h, 16);
      }
    }
#pragma unroll
    for (int i = 0; i < T::WCH; ++i) {
      const int kr = k0 + wk0 + i * T::WROWS_PER_PASS;
      wreg[i] = (wcol != nullptr && kr < K) ? *reinterpret_cast<const uint4v*>(wcol + (int64_t)kr * ldw) : zero4;
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

}  // namespace tri
