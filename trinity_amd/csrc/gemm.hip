// FFN GEMMs (plain / GELU / SwiGLU epilogues, optional row scale and residual)
// and the fused QKV projection (per-head QKNorm, head-major scatter into the
// KV cache rows).
#include <type_traits>

#include "gemm_core.h"
#include "launch.h"

namespace tri {



__device__ __forceinline__ void store4(half_t* p, float a, float b, float c, float d) {
  half4v h = {(half_t)a, (half_t)b, (half_t)c, (half_t)d};
  *reinterpret_cast<half4v*>(p) = h;
}

template <class T>
__device__ __forceinline__ void zero_acc(float16v (&acc)[T::NI][T::MI]) {
#pragma unroll
  for (int ni = 0; ni < T::NI; ++ni)
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0.f;
}

template <class T, class ColMap>
__device__ __forceinline__ void run_mainloop(const half_t* x, int64_t ldx, int m0, int M, int K, ColMap colmap,
                                             half_t* lds, float16v (&acc)[T::NI][T::MI]) {
  zero_acc<T>(acc);
  if constexpr (T::kDma) gemm_mainloop_dma<T>(x, ldx, m0, M, K, colmap, lds, acc);
  else gemm_mainloop<T>(x, ldx, m0, M, K, colmap, lds, acc);
}

// ---------------------------------------------------------------------------
// out = act(rowscale * X.W) [+ residual] over output columns [col0, col0 + ncols).
// EPI_SWIGLU: a workgroup produces BN/2 output columns; the LDS weight tile
// holds, for every wave, TN/2 gate columns followed by the matching TN/2 up
// columns, so gate and up of one output element sit in the same lane.
// ---------------------------------------------------------------------------
// Token tiles per group in the tile order: an XCD round of 32 workgroups covers `group` token tiles x 32 / group
// weight tiles and streams that many activation and weight panels through its L2.  Square tiles are level at
// 8 x 4 and 4 x 8; a tile half as wide has weight panels half as large, and 4 x 8 reads a fifth less (Llama-3-8B
// down projection: 587 -> 470 MB per launch at the L2 / fabric boundary; gate/up 471 -> 461 us, down 246 -> 244 us).
template <class T>
constexpr int kGroupM = T::BN >= 256 ? 8 : 4;

// WT: the weights are K-contiguous (a.ldw / a.ldw2 are then the strides between weight columns).
template <class T, int EPI, bool WT = false>
__device__ __forceinline__ void gemm_tile(const GemmArgs& a, int pid, int col0, int ncols, half_t* lds) {
  constexpr int OUT_BN = (EPI == EPI_SWIGLU) ? T::BN / 2 : T::BN;
  constexpr int OUT_TN = (EPI == EPI_SWIGLU) ? T::TN / 2 : T::TN;
  const int tiles_m = (a.M + T::BM - 1) / T::BM, tiles_n = (ncols + OUT_BN - 1) / OUT_BN;
  int tm, tn;
  tile_coords(pid, tiles_m, tiles_n, kGroupM<T>, tm, tn);
  const int m0 = tm * T::BM, n0 = col0 + tn * OUT_BN;
  const int nend = col0 + ncols;

  // LDS column chunk (8 columns) -> weight column it holds
  auto colmap = [&](int chunk, int64_t& ldw) -> const half_t* {
    const int c = chunk * 8;
    int col;
    const half_t* base = a.w;
    ldw = a.ldw;
    if (EPI == EPI_SWIGLU) {
      const int wv = c / T::TN, within = c % T::TN;
      const int up = within / OUT_TN, jj = within % OUT_TN;
      col = n0 + wv * OUT_TN + jj;
      if (up) { base = a.w2; ldw = a.ldw2; }
    } else {
      col = n0 + c;
    }
    return base + (col < nend ? col : n0);
  };

  // the same mapping per LDS row of a K-contiguous weight tile: row -> start of that weight column's k run
  auto rowmap = [&](int nloc) -> const half_t* {
    int col;
    const half_t* base = a.w;
    int64_t ldw = a.ldw;
    if (EPI == EPI_SWIGLU) {
      const int wv = nloc / T::TN, within = nloc % T::TN;
      const int up = within / OUT_TN, jj = within % OUT_TN;
      col = n0 + wv * OUT_TN + jj;
      if (up) { base = a.w2; ldw = a.ldw2; }
    } else {
      col = n0 + nloc;
    }
    return base + (int64_t)(col < nend ? col : n0) * ldw;
  };

  float16v acc[T::NI][T::MI];
  if constexpr (WT) {
    zero_acc<T>(acc);
    gemm_mainloop_dma_wt<T>(a.x, a.ldx, m0, a.M, a.K, rowmap, lds, acc);
  } else {
    run_mainloop<T>(a.x, a.ldx, m0, a.M, a.K, colmap, lds, acc);
  }

  // ---- epilogue.  A lane owns one token and four consecutive columns per register quad: stored straight from
  // the registers, a store instruction touches 32 rows with 16 bytes each.  Every wave therefore turns its tile
  // around in LDS (free after the main loop; a wave's own region, so no barrier between its writes and reads) and
  // stores rows of OUT_TN contiguous columns, 16 bytes per lane: [2048, 4096] x [4096, 28672] spent 44 of 467 us
  // on its stores before and 15 us after.  The arithmetic (row scale, activation, residual, one rounding) is
  // unchanged and still per lane.
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  constexpr int ONI = (EPI == EPI_SWIGLU) ? T::NI / 2 : T::NI;
  constexpr int RS = OUT_TN + 8;  // halfs per staged row
  static_assert(T::WM * T::WN * T::TM * RS * 2 <= T::LDS_BYTES, "the staged output tile fits the main loop's LDS");
  __syncthreads();  // every wave is done with the main loop's LDS tiles (and every load into them has landed)
  half_t* stg = lds + wave * (T::TM * RS);
  // (Two copies, with and without the row scale: one wave per SIMD issues an instruction every five cycles or so,
  // nothing else runs beside the epilogue, and the two multiplications by a scale of one were a quarter of the
  // gated epilogue's 9.5 vector instructions per output.)
  auto to_stage = [&](auto with_rowscale) __attribute__((always_inline)) {
    constexpr bool ROWSCALE = decltype(with_rowscale)::value;
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi) {
      const int m = m0 + wm * T::TM + mi * 32 + l32;
      const bool mok = m < a.M;
      const float rs = (ROWSCALE && mok) ? a.rowscale[m] : 1.0f;
#pragma unroll
      for (int ni = 0; ni < ONI; ++ni) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int nloc = ni * 32 + rq * 8 + g * 4;
          const int n = n0 + wn * OUT_TN + nloc;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float c = acc[ni][mi][rq * 4 + e];
            if (ROWSCALE) c *= rs;
            if (EPI == EPI_GELU) c = gelu_erf(c);
            if (EPI == EPI_SWIGLU) {
              float u = acc[ni + ONI][mi][rq * 4 + e];
              if (ROWSCALE) u *= rs;
              c = silu(c) * u;
            }
            v[e] = c;
          }
          if (a.residual != nullptr && mok && n < nend) {
            const half4v rr = *reinterpret_cast<const half4v*>(a.residual + (int64_t)m * a.ldr + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += (float)rr[e];
          }
          store4(stg + (mi * 32 + l32) * RS + nloc, v[0], v[1], v[2], v[3]);
        }
      }
    }
  };
  if (a.rowscale != nullptr) to_stage(std::true_type{});
  else to_stage(std::false_type{});
  constexpr int LPR = OUT_TN / 8;  // 16-byte chunks per staged row
#pragma unroll 4
  for (int idx = lane; idx < T::TM * LPR; idx += 64) {
    const int row = idx / LPR, ch = idx % LPR;
    const int m = m0 + wm * T::TM + row, n = n0 + wn * OUT_TN + ch * 8;
    const half8v v = *reinterpret_cast<const half8v*>(stg + row * RS + ch * 8);
    // (column counts are multiples of eight: a chunk lies wholly inside or wholly outside)
    if (m < a.M && n < nend) *reinterpret_cast<half8v*>(a.out + (int64_t)m * a.ldo + n) = v;
  }
}

// One launch covers two column ranges: workgroups [0, n_big) run big tiles
// over columns [0, big_cols), the rest run the smaller tile over the remaining
// columns (the partial last round of big tiles would leave CUs idle).
template <class Big, class Mid, int EPI, bool WT = false>
__global__ __launch_bounds__(Big::NT) void gemm_epi_kernel(GemmArgs a) {
  static_assert(Big::NT == Mid::NT, "both tile shapes use the same workgroup size");
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  if ((int)blockIdx.x < a.n_big) gemm_tile<Big, EPI, WT>(a, blockIdx.x, 0, a.big_cols, lds);
  else gemm_tile<Mid, EPI, WT>(a, blockIdx.x - a.n_big, a.big_cols, a.N - a.big_cols, lds);
}

// ---------------------------------------------------------------------------
// Fused QKV projection.  Logical output columns: [0, Hq*D) -> Q,
// [Hq*D, Hq*D + Hkv*D) -> K, then V.  A wave tile (128 columns) holds whole
// heads, so QKNorm reduces inside one lane pair.
// ---------------------------------------------------------------------------
template <class T, int D, bool WT = false>
__device__ __forceinline__ void qkv_tile(const QkvProjArgs& a, int pid, int col_begin, int col_end, half_t* lds) {
  const int nq = a.Hq * D, nkv = a.Hkv * D, ntot = col_end;
  const int tiles_m = (a.S + T::BM - 1) / T::BM, tiles_n = (col_end - col_begin + T::BN - 1) / T::BN;
  int tm, tn;
  tile_coords(pid, tiles_m, tiles_n, kGroupM<T>, tm, tn);
  const int m0 = tm * T::BM, n0 = col_begin + tn * T::BN;

  auto colmap = [&](int chunk, int64_t& ldw) -> const half_t* {
    int col = n0 + chunk * 8;
    col = col < ntot ? col : 0;
    if (col < nq) { ldw = a.ldwq; return a.wq + col; }
    if (col < nq + nkv) { ldw = a.ldwk; return a.wk + (col - nq); }
    ldw = a.ldwv;
    return a.wv + (col - nq - nkv);
  };

  // K-contiguous weights: LDS row of the weight tile -> start of that logical column's k run
  auto rowmap = [&](int nloc) -> const half_t* {
    int col = n0 + nloc;
    col = col < ntot ? col : 0;
    if (col < nq) return a.wq + (int64_t)col * a.ldwq;
    if (col < nq + nkv) return a.wk + (int64_t)(col - nq) * a.ldwk;
    return a.wv + (int64_t)(col - nq - nkv) * a.ldwv;
  };

  float16v acc[T::NI][T::MI];
  if constexpr (WT) {
    zero_acc<T>(acc);
    gemm_mainloop_dma_wt<T>(a.x, a.ldx, m0, a.S, a.K, rowmap, lds, acc);
  } else {
    run_mainloop<T>(a.x, a.ldx, m0, a.S, a.K, colmap, lds, acc);
  }

  // ---- epilogue: per-head QKNorm in the registers, then the wave's tile goes through LDS (as in gemm_tile) and
  // leaves as 16-byte pieces of rows: q rows [S, Hq * D], K / V rows of one head [.., D] contiguous.
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  constexpr int RS = T::TN + 8;  // halfs per staged row
  static_assert(T::WM * T::WN * T::TM * RS * 2 <= T::LDS_BYTES, "the staged output tile fits the main loop's LDS");
  __syncthreads();  // every wave is done with the main loop's LDS tiles
  half_t* stg = lds + wave * (T::TM * RS);
  if constexpr (T::TN % D == 0) {
    // wave tiles of whole heads: per-head RMS norm (QKNorm) reduces inside the lane pair
    constexpr int NIH = D / 32;         // 32-column tiles per head
    constexpr int HEADS = T::TN / D;    // heads per wave tile
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi) {
#pragma unroll
      for (int hh = 0; hh < HEADS; ++hh) {
        const int col0 = n0 + wn * T::TN + hh * D;  // first logical column of this head
        if (col0 >= ntot) continue;                 // uniform across the wave
        const bool norm = a.qknorm && col0 < nq + nkv;  // uniform across the wave
        float nrm = 1.0f;
        if (norm) {
          // the oracle squares the fp16-rounded projection
          float ss = 0.f;
#pragma unroll
          for (int ni = 0; ni < NIH; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float h = (float)(half_t)acc[hh * NIH + ni][mi][r];
              ss = fmaf(h, h, ss);
            }
          ss = pair_sum(ss);
          nrm = rsqrtf(ss / (float)D + a.eps);
        }
#pragma unroll
        for (int ni = 0; ni < NIH; ++ni)
#pragma unroll
          for (int rq = 0; rq < 4; ++rq) {
            half4v o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const half_t h = (half_t)acc[hh * NIH + ni][mi][rq * 4 + e];
              o[e] = norm ? (half_t)((float)h * nrm) : h;
            }
            *reinterpret_cast<half4v*>(stg + (mi * 32 + l32) * RS + hh * D + ni * 32 + rq * 8 + g * 4) = o;
          }
      }
    }
  } else {
    // wave tiles that cut heads: no QKNorm (it needs whole heads: the host never pairs it with such a tile)
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < T::NI; ++ni)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          half4v o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (half_t)acc[ni][mi][rq * 4 + e];
          *reinterpret_cast<half4v*>(stg + (mi * 32 + l32) * RS + ni * 32 + rq * 8 + g * 4) = o;
        }
  }
  constexpr int LPR = T::TN / 8;  // 16-byte chunks per staged row
#pragma unroll 4
  for (int idx = lane; idx < T::TM * LPR; idx += 64) {
    const int row = idx / LPR, ch = idx % LPR;
    const int m = m0 + wm * T::TM + row;
    const int col = n0 + wn * T::TN + ch * 8;  // logical column; a chunk never straddles a head (D % 32 == 0)
    if (m >= a.S || col >= ntot) continue;
    half_t* dst;
    if (col < nq) {
      dst = a.q + (int64_t)m * a.ldq + col;
    } else if (col < nq + nkv) {
      const int c = col - nq;
      dst = a.k + (int64_t)(c / D) * a.k_sh + (int64_t)(a.P + m) * a.k_sr + c % D;
    } else {
      const int c = col - nq - nkv;
      dst = a.v + (int64_t)(c / D) * a.v_sh + (int64_t)(a.P + m) * a.v_sr + c % D;
    }
    *reinterpret_cast<half8v*>(dst) = *reinterpret_cast<const half8v*>(stg + row * RS + ch * 8);
  }
}

// One launch covers two column ranges (as gemm_epi_kernel): workgroups [0, n_big) run the big tile over logical
// columns [0, big_cols), the rest run the smaller tile over the remaining columns.
template <class Big, class Mid, int D, bool WT = false>
__global__ __launch_bounds__(Big::NT) void qkv_proj_kernel(QkvProjArgs a) {
  static_assert(Big::NT == Mid::NT, "both tile shapes use the same workgroup size");
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  const int ntot = (a.Hq + 2 * a.Hkv) * D;
  if ((int)blockIdx.x < a.n_big) qkv_tile<Big, D, WT>(a, blockIdx.x, 0, a.big_cols, lds);
  else qkv_tile<Mid, D, WT>(a, blockIdx.x - a.n_big, a.big_cols, ntot, lds);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
typedef DmaTile<256, 256, 2, 2> FastBig;    // 256 tokens x 256 columns, 4 waves of 128 x 128
typedef DmaTile<256, 128, 2, 2> FastMidN;   // 256 tokens x 128 columns, 4 waves of 128 x 64
typedef DmaTile<128, 256, 2, 2> FastMidM;   // 128 tokens x 256 columns, 4 waves of 64 x 128
typedef GemmTile<256, 256, 2, 2> SlowBig;   // general-K counterparts
typedef GemmTile<256, 128, 2, 2> SlowMidN;
typedef GemmTile<128, 256, 2, 2> SlowMidM;

constexpr int kCUs = 256;

// Tile plan: 256 x 256 tiles for whole rounds of 256 workgroups over the first columns, the remaining columns
// with a second tile shape, both in one launch.  The second shape is chosen per call from a small family
// (256 x 128 in the 2 x 2 wave arrangement, 256 x 64 / 96 / 160 / 192 with four waves stacked over the rows) so
// that the last, partial round costs as little as possible; the whole matrix may also go to the second shape.
struct TilePlan {
  int n_big, big_cols, n_mid;
  double cost;  // in units of one round of 256 x 256 tiles
};

static TilePlan make_plan(int M, int N, int out_big, int mid_bm, int out_mid, double mid_cost, bool use_big) {
  TilePlan p = {0, 0, 0, 0.0};
  const int tiles_m = (M + 255) / 256;
  const int ct_big = (N + out_big - 1) / out_big;  // column tiles if everything were big
  const int total_big = tiles_m * ct_big;
  int full_ct = 0;                                 // column tiles that make whole rounds of big tiles
  if (use_big && total_big >= kCUs) {
    full_ct = ((total_big / kCUs) * kCUs) / tiles_m;
    if (full_ct > ct_big || total_big % kCUs == 0) full_ct = ct_big;
  }
  p.big_cols = full_ct * out_big < N ? full_ct * out_big : N;
  p.n_big = tiles_m * full_ct;
  const int rest = N - p.big_cols;
  p.n_mid = ((M + mid_bm - 1) / mid_bm) * ((rest + out_mid - 1) / out_mid);
  p.cost = (p.n_big + kCUs - 1) / kCUs + mid_cost * ((p.n_mid + kCUs - 1) / kCUs);
  return p;
}

template <class Big, class Mid, int EPI, bool WT = false>
static int launch_gemm_plan(GemmArgs a, const TilePlan& p, hipStream_t stream) {
  a.big_cols = p.big_cols;
  a.n_big = p.n_big;
  constexpr int LDS = Big::LDS_BYTES > Mid::LDS_BYTES ? Big::LDS_BYTES : Mid::LDS_BYTES;
  constexpr auto kern = gemm_epi_kernel<Big, Mid, EPI, WT>;
  if (set_max_lds<kern, LDS>() != 0) return -1;
  hipLaunchKernelGGL(kern, dim3(p.n_big + p.n_mid), dim3(Big::NT), LDS, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

typedef DmaTile<256, 64, 4, 1, 128> Fit64;    // four waves of 64 x 64 (LDS weight rows 128 wide)
typedef DmaTile<256, 96, 4, 1, 128> Fit96;    // four waves of 64 x 96
typedef DmaTile<256, 160, 4, 1, 256> Fit160;  // four waves of 64 x 160
typedef DmaTile<256, 192, 4, 1, 256> Fit192;  // four waves of 64 x 192
// cost of one round of each second shape relative to a round of 256 x 256 tiles (measured)
constexpr double kCostMidN = 0.55, kCostMidM = 0.50, kCostFit96 = 0.47, kCostFit160 = 0.72, kCostFit192 = 0.84;
constexpr double kCostFit64 = 0.43;

// the cheapest plan of the family for plain / GELU epilogues; `which` = 2 * shape + (no big segment)
static TilePlan best_plan(int M, int N, int& which) {
  TilePlan best = make_plan(M, N, 256, 256, 128, kCostMidN, true);
  which = 0;
  auto consider = [&](int id, int out_mid, double c, bool use_big) {
    const TilePlan p = make_plan(M, N, 256, 256, out_mid, c, use_big);
    if (p.cost < best.cost - 1e-9) { best = p; which = id; }
  };
  consider(1, 128, kCostMidN, false);
  consider(2, 96, kCostFit96, true);
  consider(3, 96, kCostFit96, false);
  consider(4, 160, kCostFit160, true);
  consider(5, 160, kCostFit160, false);
  consider(6, 192, kCostFit192, true);
  consider(7, 192, kCostFit192, false);
  consider(8, 64, kCostFit64, true);
  consider(9, 64, kCostFit64, false);
  return best;
}

// Split factor for an [M, K] x [K, N] product with many rows, 1 = a tile plan is at least as good.  Split-K
// runs all of N as 256 x 128 tiles in `s` parts each and pays for writing and reading the fp32 partials
// (taken at 4 TB/s against 3.9 TFLOP/s per CU); it wins only when even the best tile plan leaves most of the
// chip idle and K is deep.
static int plan_large_split(int M, int K, int N) {
  if (M <= kSkinnyMaxRows || skinny_workspace_bytes(M, K, N) > 0 || K % 32 != 0 || K < 2048 || N % 8 != 0) return 1;
  int which;
  const double base = best_plan(M, N, which).cost;
  const int mid_all = ((M + 255) / 256) * ((N + 127) / 128);
  const double t_big = 2.0 * 65536.0 * K / 3.9e12;
  int best = 1;
  double best_cost = base * 0.8;  // worth it only for a clear gain
  for (int s = 2; s <= 16; ++s) {  // (Llama-3-8B FFN at 128 rows: 149.5 us with at most 4 parts, 133.2 us with up to 16)
    if (K / 32 / s < 16) break;
    const double cost = 0.65 / s * ((mid_all * s + kCUs - 1) / kCUs) + (2.0 * s * M * (double)N * 4 / 4e12) / t_big;
    if (cost < best_cost) { best_cost = cost; best = s; }
  }
  return best;
}

int64_t large_split_workspace_bytes(int M, int K, int N) {
  const int s = plan_large_split(M, K, N);
  return s > 1 ? (int64_t)s * M * N * 4 : 0;
}

// plain and GELU epilogues on the direct-to-LDS path: pick the cheapest plan
template <int EPI>
static int launch_gemm_fast(const GemmArgs& a, hipStream_t stream) {
  static_assert(EPI != EPI_SWIGLU, "the gated epilogue keeps the two-shape plan");
  int which;
  const TilePlan best = best_plan(a.M, a.N, which);
  switch (which >> 1) {
    case 0: return launch_gemm_plan<FastBig, FastMidN, EPI>(a, best, stream);
    case 1: return launch_gemm_plan<FastBig, Fit96, EPI>(a, best, stream);
    case 2: return launch_gemm_plan<FastBig, Fit160, EPI>(a, best, stream);
    case 3: return launch_gemm_plan<FastBig, Fit192, EPI>(a, best, stream);
    default: return launch_gemm_plan<FastBig, Fit64, EPI>(a, best, stream);
  }
}

int launch_gemm(const GemmArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0) return 0;
  if (a.w_kcontig) {
    // K-contiguous weights: the two-shape plan (256 x 256 rounds, then 256 x 128 tiles) on the direct-to-LDS loop
    if (a.K % 32 != 0 || a.K < 32) return -1;  // (refused by the entry points before any launch)
    const TilePlan two = make_plan(a.M, a.N, a.epi == EPI_SWIGLU ? 128 : 256, 256, a.epi == EPI_SWIGLU ? 64 : 128,
                                   kCostMidN, true);
    switch (a.epi) {
      case EPI_NONE: return launch_gemm_plan<FastBig, FastMidN, EPI_NONE, true>(a, two, stream);
      case EPI_GELU: return launch_gemm_plan<FastBig, FastMidN, EPI_GELU, true>(a, two, stream);
      case EPI_SWIGLU: return launch_gemm_plan<FastBig, FastMidN, EPI_SWIGLU, true>(a, two, stream);
    }
    return -1;
  }
  if (a.M <= kSkinnyWideMaxRows) {  // few rows: stream the weights with the split-K kernels when shape and workspace allow
    const int r = launch_skinny_gemm(a, stream);
    if (r <= 0) return r;
  }
  if (a.M > kSkinnyMaxRows && a.ws != nullptr && a.epi != EPI_SWIGLU) {
    const int s = plan_large_split(a.M, a.K, a.N);
    if (s > 1 && a.ws_bytes >= (int64_t)s * a.M * a.N * 4) return launch_gemm_splitk(a, s, stream);
  }
  const bool fast = (a.K % 32 == 0) && a.K >= 32;
  const int out_mid = a.epi == EPI_SWIGLU ? 64 : 128;
  const TilePlan two = make_plan(a.M, a.N, a.epi == EPI_SWIGLU ? 128 : 256, 256, out_mid, kCostMidN, true);
  switch (a.epi) {
    case EPI_NONE:
      return fast ? launch_gemm_fast<EPI_NONE>(a, stream) : launch_gemm_plan<SlowBig, SlowMidN, EPI_NONE>(a, two, stream);
    case EPI_GELU:
      return fast ? launch_gemm_fast<EPI_GELU>(a, stream) : launch_gemm_plan<SlowBig, SlowMidN, EPI_GELU>(a, two, stream);
    case EPI_SWIGLU:
      return fast ? launch_gemm_plan<FastBig, FastMidN, EPI_SWIGLU>(a, two, stream)
                  : launch_gemm_plan<SlowBig, SlowMidN, EPI_SWIGLU>(a, two, stream);
  }
  return -1;
}

// Tile plan of the projection: as for the GEMMs, full rounds of 256 x 256 tiles plus a second shape for the
// remaining columns (or for everything), chosen by cost.  QKNorm needs wave tiles of whole heads.
template <class Big, class Mid, int D, bool WT = false>
static int launch_qkv_t(QkvProjArgs a, const TilePlan& p, hipStream_t stream) {
  a.big_cols = p.big_cols;
  a.n_big = p.n_big;
  constexpr int LDS = Big::LDS_BYTES > Mid::LDS_BYTES ? Big::LDS_BYTES : Mid::LDS_BYTES;
  constexpr auto kern = qkv_proj_kernel<Big, Mid, D, WT>;
  if (set_max_lds<kern, LDS>() != 0) return -1;
  hipLaunchKernelGGL(kern, dim3(p.n_big + p.n_mid), dim3(Big::NT), LDS, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

template <int D>
static int launch_qkv_d(const QkvProjArgs& a, hipStream_t stream) {
  const int ntot = (a.Hq + 2 * a.Hkv) * D;
  const bool fast = (a.K % 32 == 0) && a.K >= 32;
  TilePlan best = make_plan(a.S, ntot, 256, 128, 256, kCostMidM, true);
  if (a.w_kcontig) {
    // K-contiguous weights (K % 32 == 0, checked at the boundary): 256 x 256 rounds and / or 128 x 256 tiles, whose
    // wave tiles are 128 columns - whole heads - so QKNorm needs no other shape
    if (!fast) return -1;
    const TilePlan all_mid = make_plan(a.S, ntot, 256, 128, 256, kCostMidM, false);
    return launch_qkv_t<FastBig, FastMidM, D, true>(a, all_mid.cost < best.cost - 1e-9 ? all_mid : best, stream);
  }
  if (!fast) return launch_qkv_t<SlowBig, SlowMidM, D>(a, best, stream);
  int which = 0;
  auto consider = [&](int id, int mid_bm, int out_mid, double c, bool use_big) {
    if (a.qknorm && out_mid % D != 0) return;  // the wave tile (all columns of the shape) must hold whole heads
    const TilePlan p = make_plan(a.S, ntot, 256, mid_bm, out_mid, c, use_big);
    if (p.cost < best.cost - 1e-9) { best = p; which = id; }
  };
  consider(1, 128, 256, kCostMidM, false);
  consider(2, 256, 96, kCostFit96, true);
  consider(3, 256, 96, kCostFit96, false);
  consider(4, 256, 160, kCostFit160, true);
  consider(5, 256, 160, kCostFit160, false);
  consider(6, 256, 192, kCostFit192, true);
  consider(7, 256, 192, kCostFit192, false);
  switch (which >> 1) {
    case 0: return launch_qkv_t<FastBig, FastMidM, D>(a, best, stream);
    case 1: return launch_qkv_t<FastBig, Fit96, D>(a, best, stream);
    case 2: return launch_qkv_t<FastBig, Fit160, D>(a, best, stream);
    default: return launch_qkv_t<FastBig, Fit192, D>(a, best, stream);
  }
}

int launch_qkv_proj(const QkvProjArgs& a, hipStream_t stream, int* deferred_ksplit) {
  if (deferred_ksplit != nullptr) *deferred_ksplit = 0;
  if (a.S <= 0) return 0;
  if (a.S <= kSkinnyWideMaxRowsQkv && !a.w_kcontig) {  // (the few-row split-K kernels read row-major weights)
    const int r = launch_skinny_qkv(a, stream, deferred_ksplit);
    if (r <= 0) return r;
  }
  if (a.D == 128) return launch_qkv_d<128>(a, stream);
  if (a.D == 64) return launch_qkv_d<64>(a, stream);
  return -1;
}

}  // namespace tri
