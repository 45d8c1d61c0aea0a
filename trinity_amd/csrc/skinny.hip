// GEMMs with few rows (M <= 64): the reference's own regime (16 new tokens
// against 4096-wide weights), where the job is to stream the weight matrices
// from HBM once at full bandwidth.
//
// Phase 1 (skinny_partial_kernel): the K axis is split so that a few hundred
// workgroups share the job; each workgroup streams a [k range] x
// [128 columns] slab of the (concatenated) weights through the same
// direct-to-LDS pipeline as the large GEMMs and writes its fp32 partial
// products to the workspace, laid out [split][row][column].  Workgroups that
// run at the same time read neighbouring column ranges of the same weight
// rows, so DRAM pages are consumed whole.
// Phase 2 (finalize kernels): sum over the splits in a fixed order (results do
// not depend on scheduling), apply the epilogue (row scale, GELU, SwiGLU,
// residual; or per-head QKNorm and the head-major scatter of the QKV
// projection) and round to fp16.
#include "gemm_core.h"
#include "launch.h"

namespace tri {

typedef DmaTile<64, 128, 1, 4> SkinnyTile;  // 64 rows x 128 columns, 4 waves of 64 x 32

struct SkinnyArgs {
  const half_t* x;
  int64_t ldx;
  const half_t* w[3];  // column segments, concatenated logically
  int64_t ldw[3];
  int seg_begin[3];    // first logical column of each segment (unused segments start at ntot)
  int M, K, ntot;
  int kt_per_split;    // k tiles (32 deep) per split
  float* partial;      // [ksplit][M][ntot]
};

__global__ __launch_bounds__(256) void skinny_partial_kernel(SkinnyArgs a) {
  using T = SkinnyTile;
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  // linear id -> (row block of 64, column tile, split), row blocks fastest: the workgroups that stream the same
  // weight slab for different rows start together
  const int tiles_n = (a.ntot + T::BN - 1) / T::BN, nrb = (a.M + T::BM - 1) / T::BM;
  const int rb = (int)blockIdx.x % nrb, rest = (int)blockIdx.x / nrb;
  const int tn = rest % tiles_n, split = rest / tiles_n;
  const int n0 = tn * T::BN, m0 = rb * T::BM;
  const int KT = a.K / T::BK;
  const int kt0 = split * a.kt_per_split;
  const int nkt = min(KT - kt0, a.kt_per_split);
  const int64_t k0 = (int64_t)kt0 * T::BK;

  auto colmap = [&](int chunk, int64_t& ldw) -> const half_t* {
    int col = n0 + chunk * 8;
    col = col < a.ntot ? col : 0;
    const int seg = col >= a.seg_begin[2] ? 2 : (col >= a.seg_begin[1] ? 1 : 0);
    ldw = a.ldw[seg];
    return a.w[seg] + (col - a.seg_begin[seg]) + k0 * ldw;
  };

  float16v acc[T::NI][T::MI];
#pragma unroll
  for (int mi = 0; mi < T::MI; ++mi)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][mi][r] = 0.f;
  gemm_mainloop_dma<T>(a.x + k0, a.ldx, m0, a.M, nkt * T::BK, colmap, lds, acc);

  const int lane = threadIdx.x & 63, wn = threadIdx.x >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  float* base = a.partial + (int64_t)split * a.M * a.ntot;
#pragma unroll
  for (int mi = 0; mi < T::MI; ++mi) {
    const int m = m0 + mi * 32 + l32;
    if (m >= a.M) continue;
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const int n = n0 + wn * T::TN + rq * 8 + g * 4;
      if (n >= a.ntot) continue;
      float4v v = {acc[0][mi][rq * 4], acc[0][mi][rq * 4 + 1], acc[0][mi][rq * 4 + 2], acc[0][mi][rq * 4 + 3]};
      *reinterpret_cast<float4v*>(base + (int64_t)m * a.ntot + n) = v;
    }
  }
}

// out[m, n..n+3] for one thread; the arithmetic mirrors the epilogue of the large-tile GEMM
template <int EPI>
__device__ __forceinline__ void finalize_group(const GemmArgs& a, const float* partial, int ksplit, int m, int n, float rs) {
  const int ntot = EPI == EPI_SWIGLU ? 2 * a.N : a.N;
  const int64_t stride = (int64_t)a.M * ntot, off = (int64_t)m * ntot + n;
  float4v v = sum_splits(partial, ksplit, stride, off);
  float4v u = {0.f, 0.f, 0.f, 0.f};
  if (EPI == EPI_SWIGLU) u = sum_splits(partial, ksplit, stride, off + a.N);
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float c = v[e] * rs;
    if (EPI == EPI_GELU) c = gelu_erf(c);
    if (EPI == EPI_SWIGLU) c = silu(c) * (u[e] * rs);
    o[e] = c;
  }
  if (a.residual != nullptr) {
    const half4v rr = *reinterpret_cast<const half4v*>(a.residual + (int64_t)m * a.ldr + n);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] += (float)rr[e];
  }
  half4v h = {(half_t)o[0], (half_t)o[1], (half_t)o[2], (half_t)o[3]};
  *reinterpret_cast<half4v*>(a.out + (int64_t)m * a.ldo + n) = h;
}

template <int EPI>
__global__ __launch_bounds__(256) void skinny_finalize_kernel(GemmArgs a, const float* partial, int ksplit) {
  const int groups = a.N / 4;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.M * groups) return;
  const int m = idx / groups, n = (idx % groups) * 4;
  finalize_group<EPI>(a, partial, ksplit, m, n, a.rowscale != nullptr ? a.rowscale[m] : 1.0f);
}

// The same with the row scale computed on the way: blockIdx.y = row; every workgroup first reduces
// rownorm_src[m, :] (a few KB, L2-resident) to rsqrt(mean(x^2)).
template <int EPI>
__global__ __launch_bounds__(256) void skinny_finalize_rownorm_kernel(GemmArgs a, const float* partial, int ksplit) {
  __shared__ float part[4];
  const int m = blockIdx.y, t = threadIdx.x;
  const half_t* src = a.rownorm_src + (int64_t)m * a.rownorm_ld;
  float ss = 0.f;
  for (int i = t * 8; i < a.rownorm_n; i += 256 * 8) {
    const half8v x = *reinterpret_cast<const half8v*>(src + i);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf((float)x[e], (float)x[e], ss);
  }
  ss = wave_sum(ss);
  if ((t & 63) == 0) part[t >> 6] = ss;
  __syncthreads();
  const float rs = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)a.rownorm_n);
  if (blockIdx.x == 0 && t == 0 && a.rownorm_out != nullptr) a.rownorm_out[m] = rs;
  const int g = blockIdx.x * 256 + t;
  if (g < a.N / 4) finalize_group<EPI>(a, partial, ksplit, m, g * 4, rs);
}

// One group of D/4 consecutive lanes per (row, head): sum the splits, round to fp16, optionally RMS-normalise
// the head (Q and K only), scatter to q / the cache rows.
template <int D>
__global__ __launch_bounds__(256) void skinny_finalize_qkv_kernel(QkvProjArgs a, const float* partial, int ksplit) {
  constexpr int LPH = D / 4;  // lanes per head
  const int nq = a.Hq * D, nkv = a.Hkv * D, ntot = nq + 2 * nkv;
  const int heads = a.Hq + 2 * a.Hkv;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int grp = idx / LPH, li = idx % LPH;
  const bool live = grp < a.S * heads;
  const int m = live ? grp / heads : 0, hc = live ? grp % heads : 0;
  const int col0 = hc * D;
  float4v v = sum_splits(partial, live ? ksplit : 0, (int64_t)a.S * ntot, (int64_t)m * ntot + col0 + li * 4);
  half_t* dst;
  int seg;
  if (col0 < nq) { seg = 0; dst = a.q + (int64_t)m * a.ldq + col0; }
  else if (col0 < nq + nkv) { seg = 1; dst = a.k + (int64_t)((col0 - nq) / D) * a.k_sh + (int64_t)(a.P + m) * a.k_sr; }
  else { seg = 2; dst = a.v + (int64_t)((col0 - nq - nkv) / D) * a.v_sh + (int64_t)(a.P + m) * a.v_sr; }
  half4v h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
  if (a.qknorm) {  // uniform; every lane takes part in the reduction
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) ss = fmaf((float)h[e], (float)h[e], ss);
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (seg < 2) {
      const float nrm = rsqrtf(ss / (float)D + a.eps);
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = (half_t)((float)h[e] * nrm);
    }
  }
  if (live) *reinterpret_cast<half4v*>(dst + li * 4) = h;
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// Workgroups aimed at.  A compute-free kernel streams the same slabs at the same 5.3-5.5 TB/s with anything from
// 670 to 2500 workgroups, so the count is set by what follows: every split adds 4 * M * N_cols bytes of partial
// sums that the merge kernel (or the attention kernel) reads back.  Whole blocks at 16 rows: 256-384 workgroups
// are 4-10 % faster than 768 (384 taken) (Llama-3-8B FFN block 102.6 -> 97 us, Falcon-7B 60.4 -> 54 us, attention blocks
// 38.5 -> 36.5 and 42.8 -> 39.9 us).
constexpr int kTargetWorkgroups = 384;

// k tiles per split for an [M, K] x [K, ncols] product
static int plan_kt_per_split(int M, int K, int ncols) {
  const int KT = K / 32;
  const int tiles_n = (ncols + SkinnyTile::BN - 1) / SkinnyTile::BN;
  int ksplit = (kTargetWorkgroups + tiles_n - 1) / tiles_n;
  // partial sums cost 8 * M bytes per split and column against 2 * K bytes of weights: keep them under a quarter
  const int cap = K / (16 * M) > 1 ? K / (16 * M) : 1;
  ksplit = ksplit < cap ? ksplit : cap;
  ksplit = ksplit < KT / 4 ? ksplit : (KT / 4 > 1 ? KT / 4 : 1);  // at least four k tiles per workgroup
  return (KT + ksplit - 1) / ksplit;
}

static bool skinny_shape(int M, int K, int ncols, bool qkv) {
  if (M < 1 || K % 32 != 0 || K < 32 || ncols < 1) return false;
  const int64_t bytes = 2 * (int64_t)K * ncols;
  if (M <= kSkinnyMaxRows) return true;
  // (two row blocks of a Q/K/V projection still gain with up to 160 MB of weights: 32 KV heads, 100 MB, 128 rows
  // 61.8 -> 51.8 us; four blocks do not: 256 rows 68.1 -> 86.2 us)
  if (qkv && M <= kSkinnyWideMaxRows && bytes <= (kSkinnyWideMaxBytes / 2) * 5) return true;
  return M <= (qkv ? kSkinnyWideMaxRowsQkv : kSkinnyWideMaxRows) && bytes <= kSkinnyWideMaxBytes;
}

int64_t skinny_workspace_bytes(int M, int K, int ncols, bool qkv) {
  if (!skinny_shape(M, K, ncols, qkv)) return 0;
  const int ktps = plan_kt_per_split(M, K, ncols);
  const int ksplit = (K / 32 + ktps - 1) / ktps;
  return (int64_t)ksplit * M * ncols * 4;
}

static int launch_partial(const SkinnyArgs& s, int ksplit, hipStream_t stream) {
  if (set_max_lds<skinny_partial_kernel, SkinnyTile::LDS_BYTES>() != 0) return -1;
  const int tiles_n = (s.ntot + SkinnyTile::BN - 1) / SkinnyTile::BN;
  const int nrb = (s.M + SkinnyTile::BM - 1) / SkinnyTile::BM;
  hipLaunchKernelGGL(skinny_partial_kernel, dim3(nrb * tiles_n * ksplit), dim3(256), SkinnyTile::LDS_BYTES, stream, s);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

bool skinny_gemm_applies(const GemmArgs& a) {
  const int ncols = a.epi == EPI_SWIGLU ? 2 * a.N : a.N;
  if (!skinny_shape(a.M, a.K, ncols, false) || a.N % 8 != 0 || a.ws == nullptr) return false;
  const int64_t need = skinny_workspace_bytes(a.M, a.K, ncols);
  return need != 0 && a.ws_bytes >= need;
}

// returns 1 when the shape / workspace does not allow the split-K path (the caller then uses the large tiles)
int launch_skinny_gemm(const GemmArgs& a, hipStream_t stream) {
  const int ncols = a.epi == EPI_SWIGLU ? 2 * a.N : a.N;
  if (!skinny_gemm_applies(a)) return 1;
  SkinnyArgs s = {};
  s.x = a.x; s.ldx = a.ldx; s.M = a.M; s.K = a.K; s.ntot = ncols; s.partial = a.ws;
  s.w[0] = a.w; s.ldw[0] = a.ldw; s.seg_begin[0] = 0;
  s.w[1] = a.epi == EPI_SWIGLU ? a.w2 : a.w; s.ldw[1] = a.epi == EPI_SWIGLU ? a.ldw2 : a.ldw;
  s.seg_begin[1] = a.epi == EPI_SWIGLU ? a.N : ncols;
  s.w[2] = s.w[1]; s.ldw[2] = s.ldw[1]; s.seg_begin[2] = ncols;
  s.kt_per_split = plan_kt_per_split(a.M, a.K, ncols);
  const int ksplit = (a.K / 32 + s.kt_per_split - 1) / s.kt_per_split;
  if (launch_partial(s, ksplit, stream) != 0) return -1;
  if (a.rownorm_src != nullptr) {  // (8 elements at a time: the caller passes 16-byte aligned rows of a multiple of 8)
    const dim3 grid((a.N / 4 + 255) / 256, a.M);
    switch (a.epi) {
      case EPI_NONE: hipLaunchKernelGGL(skinny_finalize_rownorm_kernel<EPI_NONE>, grid, dim3(256), 0, stream, a, a.ws, ksplit); break;
      case EPI_GELU: hipLaunchKernelGGL(skinny_finalize_rownorm_kernel<EPI_GELU>, grid, dim3(256), 0, stream, a, a.ws, ksplit); break;
      case EPI_SWIGLU: hipLaunchKernelGGL(skinny_finalize_rownorm_kernel<EPI_SWIGLU>, grid, dim3(256), 0, stream, a, a.ws, ksplit); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
  }
  const int blocks = (a.M * (a.N / 4) + 255) / 256;
  switch (a.epi) {
    case EPI_NONE: hipLaunchKernelGGL(skinny_finalize_kernel<EPI_NONE>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit); break;
    case EPI_GELU: hipLaunchKernelGGL(skinny_finalize_kernel<EPI_GELU>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit); break;
    case EPI_SWIGLU: hipLaunchKernelGGL(skinny_finalize_kernel<EPI_SWIGLU>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// ---------------------------------------------------------------------------
// Split-K for many-row GEMMs whose tile count fills the chip badly (e.g. 2048 x 4544 outputs over K = 18176:
// 288 tiles of 256 x 128 are two rounds on 256 CUs, the second one nearly empty).  Each 256 x 128 tile is
// computed in `ksplit` parts by different workgroups, fp32 partial tiles go to the workspace in the plain
// [split][row][column] layout (the MFMA operands are swapped so that lanes run along the columns and the
// stores coalesce), and the finalize kernel above adds them and applies the epilogue.
// ---------------------------------------------------------------------------
typedef DmaTile<256, 128, 2, 2> SplitTile;

struct SplitArgs {
  const half_t* x;
  int64_t ldx;
  const half_t* w;
  int64_t ldw;
  float* partial;  // [ksplit][M][N]
  int M, N, K, kt_per_split;
};

__global__ __launch_bounds__(256) void gemm_splitk_partial_kernel(SplitArgs a) {
  using T = SplitTile;
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  const int tiles_m = (a.M + T::BM - 1) / T::BM, tiles_n = (a.N + T::BN - 1) / T::BN;
  const int tiles = tiles_m * tiles_n;
  const int split = blockIdx.x / tiles;
  int tm, tn;
  tile_coords(blockIdx.x % tiles, tiles_m, tiles_n, 8, tm, tn);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int KT = a.K / T::BK;
  const int kt0 = split * a.kt_per_split;
  const int nkt = min(KT - kt0, a.kt_per_split);
  const int64_t k0 = (int64_t)kt0 * T::BK;
  auto colmap = [&](int chunk, int64_t& ldw) -> const half_t* {
    const int col = n0 + chunk * 8;
    ldw = a.ldw;
    return a.w + (col < a.N ? col : n0) + k0 * a.ldw;
  };
  float16v acc[T::NI][T::MI];
#pragma unroll
  for (int ni = 0; ni < T::NI; ++ni)
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ni][mi][r] = 0.f;
  gemm_mainloop_dma<T, decltype(colmap), true>(a.x + k0, a.ldx, m0, a.M, nkt * T::BK, colmap, lds, acc);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % T::WM, wn = wave / T::WM;
  const int l32 = lane & 31, g = lane >> 5;
  float* base = a.partial + (int64_t)split * a.M * a.N;
#pragma unroll
  for (int ni = 0; ni < T::NI; ++ni) {
    const int n = n0 + wn * T::TN + ni * 32 + l32;
    if (n >= a.N) continue;
#pragma unroll
    for (int mi = 0; mi < T::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * T::TM + mi * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (m < a.M) base[(int64_t)m * a.N + n] = acc[ni][mi][r];
      }
  }
}

// `s` parts per tile (chosen by the caller, who has checked the workspace)
int launch_gemm_splitk(const GemmArgs& a, int s, hipStream_t stream) {
  if (a.epi == EPI_SWIGLU || a.ws == nullptr || s < 2 || a.ws_bytes < (int64_t)s * a.M * a.N * 4) return -1;
  SplitArgs p = {};
  p.x = a.x; p.ldx = a.ldx; p.w = a.w; p.ldw = a.ldw; p.partial = a.ws;
  p.M = a.M; p.N = a.N; p.K = a.K;
  p.kt_per_split = (a.K / 32 + s - 1) / s;
  const int ksplit = (a.K / 32 + p.kt_per_split - 1) / p.kt_per_split;
  if (set_max_lds<gemm_splitk_partial_kernel, SplitTile::LDS_BYTES>() != 0) return -1;
  const int tiles = ((a.M + 255) / 256) * ((a.N + 127) / 128);
  hipLaunchKernelGGL(gemm_splitk_partial_kernel, dim3(tiles * ksplit), dim3(256), SplitTile::LDS_BYTES, stream, p);
  if (hipGetLastError() != hipSuccess) return -1;
  const int blocks = (a.M * (a.N / 4) + 255) / 256;
  if (a.epi == EPI_NONE) hipLaunchKernelGGL(skinny_finalize_kernel<EPI_NONE>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit);
  else hipLaunchKernelGGL(skinny_finalize_kernel<EPI_GELU>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_skinny_qkv(const QkvProjArgs& a, hipStream_t stream, int* deferred_ksplit) {
  if (deferred_ksplit != nullptr) *deferred_ksplit = 0;
  const int nq = a.Hq * a.D, nkv = a.Hkv * a.D, ntot = nq + 2 * nkv;
  if (!skinny_shape(a.S, a.K, ntot, true) || a.ws == nullptr || (a.D != 64 && a.D != 128)) return 1;
  const int64_t need = skinny_workspace_bytes(a.S, a.K, ntot, true);
  if (need == 0 || a.ws_bytes < need) return 1;
  SkinnyArgs s = {};
  s.x = a.x; s.ldx = a.ldx; s.M = a.S; s.K = a.K; s.ntot = ntot; s.partial = a.ws;
  s.w[0] = a.wq; s.ldw[0] = a.ldwq; s.seg_begin[0] = 0;
  s.w[1] = a.wk; s.ldw[1] = a.ldwk; s.seg_begin[1] = nq;
  s.w[2] = a.wv; s.ldw[2] = a.ldwv; s.seg_begin[2] = nq + nkv;
  s.kt_per_split = plan_kt_per_split(a.S, a.K, ntot);
  const int ksplit = (a.K / 32 + s.kt_per_split - 1) / s.kt_per_split;
  if (launch_partial(s, ksplit, stream) != 0) return -1;
  if (deferred_ksplit != nullptr) {
    *deferred_ksplit = ksplit;
    return 0;
  }
  const int heads = a.Hq + 2 * a.Hkv;
  const int threads = a.S * heads * (a.D / 4);
  const int blocks = (threads + 255) / 256;
  if (a.D == 128) hipLaunchKernelGGL(skinny_finalize_qkv_kernel<128>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit);
  else hipLaunchKernelGGL(skinny_finalize_qkv_kernel<64>, dim3(blocks), dim3(256), 0, stream, a, a.ws, ksplit);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tri
