// Standalone RMSNorm and the per-row rsqrt(mean(x^2)+eps) statistic.
//
// One wavefront owns one row: the row is read once with 16-byte
// loads, kept in registers, reduced with wave shuffles (no LDS, no barrier)
// and written once.  HBM traffic per row = 2 * n * 2 bytes (+ the weight
// vector, which each wave loads once and keeps in registers).
#include "common.h"
#include "launch.h"

namespace tri {

// One wave per row, nothing loops: every load of the row is issued at once, the row stays in registers, and the
// workgroups are small (two waves), so the hardware keeps every CU topped up with rows whose loads are all in
// flight while older rows reduce and store.  4096 x 4096 over buffers that do not fit the Infinity Cache
// (rmsnorm_wave_full_kernel below): 11.1 us (6.05 TB/s) against 15.4 us for a persistent wave per CU slot that
// prefetches one row ahead, 11.7 us with three rows ahead, 13.1 us for a 256-thread workgroup per row and 14.0 us
// for a device-to-device copy of the same 64 MB.
// (The second launch bound asks for four waves per SIMD, i.e. at most 128 registers: left alone the compiler
// spreads the widest row over 226 and halves the rows in flight - 24.8 us.)
constexpr int kWaveRowThreads = 128;
template <int CH, bool HAS_W, bool STORE>  // HAS_W: multiply by w; STORE: write y (otherwise only the row statistic)
__global__ __launch_bounds__(kWaveRowThreads, 4) void rmsnorm_wave_kernel(const half_t* __restrict__ x, int64_t ldx,
                                                                       const half_t* __restrict__ w,
                                                                       half_t* __restrict__ y, int64_t ldy,
                                                                       float* __restrict__ rstd_out, int rows, int n,
                                                                       float eps) {
  const int lane = threadIdx.x & 63;
  const int nch = n >> 3;
  const int row = blockIdx.x * (kWaveRowThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  uint4v v[CH], wv[CH];
  const uint4v* xr = reinterpret_cast<const uint4v*>(x + (int64_t)row * ldx);
  // chunks past the end of the row re-read its last chunk and are zeroed by a select: every load is issued
  // unconditionally (a branch around each load makes the compiler wait for it before the next one)
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int idx = c * 64 + lane;
    v[c] = __builtin_nontemporal_load(xr + (idx < nch ? idx : nch - 1));
  }
  if (HAS_W && STORE) {
    const uint4v* wr = reinterpret_cast<const uint4v*>(w);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      wv[c] = wr[idx < nch ? idx : nch - 1];
    }
  }
  // every load of the wave is on its way before anything waits for one (the weights come out of L2 while the
  // row is still travelling)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int c = 0; c < CH; ++c)
    if (c * 64 + lane >= nch) v[c] = uint4v{0u, 0u, 0u, 0u};
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    half8v h;
    __builtin_memcpy(&h, &v[c], 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)h[e];
      ss = fmaf(f, f, ss);
    }
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)n + eps);
  if (!STORE) {
    if (rstd_out != nullptr && lane == 0) rstd_out[row] = r;
    return;
  }
  // the row (and the weights) stay packed in their 16-bit form across the reduction: without this fence the
  // compiler keeps the 64 converted floats of the first pass (and converts the weights early) and runs out of the
  // 128 registers that four waves per SIMD leave it
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    asm volatile("" : "+v"(v[c]));
    if (HAS_W) asm volatile("" : "+v"(wv[c]));
  }
  uint4v* yr = reinterpret_cast<uint4v*>(y + (int64_t)row * ldy);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int idx = c * 64 + lane;
    if (idx < nch) {
      half8v h, o;
      __builtin_memcpy(&h, &v[c], 16);
      if (HAS_W) {
        half8v wh;
        __builtin_memcpy(&wh, &wv[c], 16);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)h[e] * r * (float)wh[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)h[e] * r);
      }
      uint4v ov;
      __builtin_memcpy(&ov, &o, 16);
      __builtin_nontemporal_store(ov, yr + idx);
    }
  }
  // last: a store behind a branch in the middle makes the compiler's wait counts after it pessimistic, and the y
  // stores then wait for one another
  if (rstd_out != nullptr && lane == 0) rstd_out[row] = r;
}

// Any n (rows longer than 8192 elements, or n not a multiple of 8): one
// workgroup per row, two sweeps (the second one hits L2).
__global__ __launch_bounds__(256) void rmsnorm_row_kernel(const half_t* __restrict__ x, int64_t ldx,
                                                          const half_t* __restrict__ w, half_t* __restrict__ y,
                                                          int64_t ldy, float* __restrict__ rstd_out, int rows, int n,
                                                          float eps) {
  __shared__ float part[4];
  const int row = blockIdx.x;
  const half_t* xr = x + (int64_t)row * ldx;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float f = (float)xr[i];
    ss = fmaf(f, f, ss);
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float r = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)n + eps);
  if (rstd_out != nullptr && threadIdx.x == 0) rstd_out[row] = r;
  if (y == nullptr) return;
  half_t* yr = y + (int64_t)row * ldy;
  for (int i = threadIdx.x; i < n; i += 256) {
    float f = (float)xr[i] * r;
    if (w != nullptr) f *= (float)w[i];
    yr[i] = (half_t)f;
  }
}

// Few rows (fewer than there are waves on the chip): one 256-thread workgroup per row, the row read once with
// 16-byte loads (up to 4 chunks per thread: n <= 8192) and kept in registers.  With `b` the row is
// a[m] + b[m] * bscale[m] (the trailing residual of the Falcon-shaped FFN block,
// baseline/ffn_ref.py:114-121 in the reference) before it is normalised.
template <int CH, bool ADD>
__global__ __launch_bounds__(256) void rmsnorm_block_kernel(const half_t* __restrict__ x, int64_t ldx,
                                                            const half_t* __restrict__ b, int64_t ldb,
                                                            const float* __restrict__ bscale,
                                                            const half_t* __restrict__ w, half_t* __restrict__ y,
                                                            int64_t ldy, float* __restrict__ rstd_out, int n, float eps) {
  __shared__ float part[4];
  const int row = blockIdx.x, t = threadIdx.x;
  const int nch = n >> 3;
  const uint4v* xr = reinterpret_cast<const uint4v*>(x + (int64_t)row * ldx);
  const uint4v* br = ADD ? reinterpret_cast<const uint4v*>(b + (int64_t)row * ldb) : nullptr;
  const float bs = ADD ? bscale[row] : 0.f;
  float f[CH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = c * 256 + t;
    uint4v xv = {0u, 0u, 0u, 0u}, bv = {0u, 0u, 0u, 0u};
    if (i < nch) {
      xv = xr[i];
      if (ADD) bv = br[i];
    }
    const half8v xh = __builtin_bit_cast(half8v, xv), bh = __builtin_bit_cast(half8v, bv);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      f[c][e] = ADD ? (float)xh[e] + (float)bh[e] * bs : (float)xh[e];
      ss = fmaf(f[c][e], f[c][e], ss);
    }
  }
  ss = wave_sum(ss);
  if ((t & 63) == 0) part[t >> 6] = ss;
  __syncthreads();
  const float r = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)n + eps);
  if (rstd_out != nullptr && t == 0) rstd_out[row] = r;
  if (y == nullptr) return;
  uint4v* yr = reinterpret_cast<uint4v*>(y + (int64_t)row * ldy);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = c * 256 + t;
    if (i >= nch) continue;
    half8v o;
    if (w != nullptr) {
      const half8v wh = __builtin_bit_cast(half8v, reinterpret_cast<const uint4v*>(w)[i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (half_t)(f[c][e] * r * (float)wh[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (half_t)(f[c][e] * r);
    }
    yr[i] = __builtin_bit_cast(uint4v, o);
  }
}

template <bool ADD>
static void launch_block_rows(const half_t* x, int64_t ldx, const half_t* b, int64_t ldb, const float* bscale,
                              const half_t* w, half_t* y, int64_t ldy, float* rstd_out, int rows, int n, float eps,
                              hipStream_t stream) {
  const int ch = (n / 8 + 255) / 256;
#define TRI_RMSB(C)                                                                                                \
  hipLaunchKernelGGL((rmsnorm_block_kernel<C, ADD>), dim3(rows), dim3(256), 0, stream, x, ldx, b, ldb, bscale, w, y, ldy, \
                     rstd_out, n, eps)
  if (ch <= 1) TRI_RMSB(1);
  else if (ch <= 2) TRI_RMSB(2);
  else if (ch <= 3) TRI_RMSB(3);
  else TRI_RMSB(4);
#undef TRI_RMSB
}

// Rows of exactly CH * 512 elements with a weight vector (n = 4096: the benchmark's shape): the same wave per row
// with nothing conditional in it.  Whether the row statistic is stored is a template parameter: behind a run-time
// branch (never taken when the pointer is null) the possible store made the compiler's wait counts after the join
// pessimistic - each y store then waited for all but three earlier memory operations, i.e. for earlier stores to
// be acknowledged: 12.9 us against 11.3 us without the branch (4096 x 4096).
template <int CH, bool RSTD>
__global__ __launch_bounds__(kWaveRowThreads) void rmsnorm_wave_full_kernel(const half_t* __restrict__ x, int64_t ldx,
                                                                          const half_t* __restrict__ w,
                                                                          half_t* __restrict__ y, int64_t ldy,
                                                                          float* __restrict__ rstd_out, int rows,
                                                                          float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (kWaveRowThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint4v* xr = reinterpret_cast<const uint4v*>(x + (int64_t)row * ldx) + lane;
  uint4v v[CH], wv[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) v[c] = __builtin_nontemporal_load(xr + c * 64);
  const uint4v* wr = reinterpret_cast<const uint4v*>(w) + lane;
#pragma unroll
  for (int c = 0; c < CH; ++c) wv[c] = wr[c * 64];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    half8v h;
    __builtin_memcpy(&h, &v[c], 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)h[e];
      ss = fmaf(f, f, ss);
    }
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)(CH * 512) + eps);
  uint4v* yr = reinterpret_cast<uint4v*>(y + (int64_t)row * ldy) + lane;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    half8v h, o, wh;
    __builtin_memcpy(&h, &v[c], 16);
    __builtin_memcpy(&wh, &wv[c], 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (half_t)((float)h[e] * r * (float)wh[e]);
    uint4v ov;
    __builtin_memcpy(&ov, &o, 16);
    __builtin_nontemporal_store(ov, yr + c * 64);
  }
  if (RSTD && lane == 0) rstd_out[row] = r;
}

static int num_cus() {
  static int n = 0;  // benign race: every thread computes the same value
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    n = v;
  }
  return n;
}

int launch_rmsnorm(const half_t* x, int64_t ldx, const half_t* w, half_t* y, int64_t ldy, float* rstd_out, int rows,
                   int n, float eps, hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  const bool vec = (n % 8 == 0) && (ldx % 8 == 0) && (y == nullptr || ldy % 8 == 0) &&
                   ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)w % 16 == 0) && n <= 8192;
  if (vec && (rows < 16 * num_cus() || n > 4096)) {
    // up to a few thousand rows a workgroup per row finishes sooner than a wave per row (measured: 1024 x 4544
    // 4.9 against 7.6 us, 3072 x 4096 9.4 against 10.0 us; from 4096 rows on the wave kernel is ahead), and so
    // does a row of more than 4096 elements, which a single wave cannot hold in registers without spilling
    // (4096 x 4544: 13.5 against 14.1 us)
    launch_block_rows<false>(x, ldx, nullptr, 0, nullptr, w, y, ldy, rstd_out, rows, n, eps, stream);
  } else if (vec) {
    const int nch = n / 8;
    const int ch = (nch + 63) / 64;
    constexpr int per = kWaveRowThreads / 64;
    const dim3 grid((rows + per - 1) / per), block(kWaveRowThreads);
#define TRI_RMS_LAUNCH(C, W, S)                                                                                \
  hipLaunchKernelGGL((rmsnorm_wave_kernel<C, W, S>), grid, block, 0, stream, x, ldx, w, y, ldy, rstd_out, rows, n, eps)
#define TRI_RMS_CASE(C)                                                                                         \
  do {                                                                                                          \
    if (y == nullptr) TRI_RMS_LAUNCH(C, false, false);                                                          \
    else if (w != nullptr && nch == C * 64 && rstd_out == nullptr)                                              \
      hipLaunchKernelGGL((rmsnorm_wave_full_kernel<C, false>), grid, block, 0, stream, x, ldx, w, y, ldy, rstd_out, \
                         rows, eps);                                                                            \
    else if (w != nullptr && nch == C * 64)                                                                     \
      hipLaunchKernelGGL((rmsnorm_wave_full_kernel<C, true>), grid, block, 0, stream, x, ldx, w, y, ldy, rstd_out, \
                         rows, eps);                                                                            \
    else if (w != nullptr) TRI_RMS_LAUNCH(C, true, true);                                                       \
    else TRI_RMS_LAUNCH(C, false, true);                                                                        \
  } while (0)
    if (ch <= 1) TRI_RMS_CASE(1);
    else if (ch <= 2) TRI_RMS_CASE(2);
    else if (ch <= 4) TRI_RMS_CASE(4);
    else TRI_RMS_CASE(8);
#undef TRI_RMS_CASE
#undef TRI_RMS_LAUNCH
  } else {
    hipLaunchKernelGGL(rmsnorm_row_kernel, dim3(rows), dim3(256), 0, stream, x, ldx, w, y, ldy, rstd_out, rows, n, eps);
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// y[m, :] = rmsnorm(a[m, :] + b[m, :] * bscale[m])  (no weight, eps = 0): the
// trailing residual + RMSNorm of the Falcon-shaped FFN block
// (baseline/ffn_ref.py:114-121 in the reference).
__global__ __launch_bounds__(256) void add_scaled_rmsnorm_kernel(const half_t* __restrict__ a, int64_t lda,
                                                                 const half_t* __restrict__ b, int64_t ldb,
                                                                 const float* __restrict__ bscale,
                                                                 half_t* __restrict__ y, int64_t ldy, int n) {
  __shared__ float part[4];
  const int row = blockIdx.x;
  const half_t* ar = a + (int64_t)row * lda;
  const half_t* br = b + (int64_t)row * ldb;
  const float bs = bscale[row];
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float f = (float)ar[i] + (float)br[i] * bs;
    ss = fmaf(f, f, ss);
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float r = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)n);
  half_t* yr = y + (int64_t)row * ldy;
  for (int i = threadIdx.x; i < n; i += 256) yr[i] = (half_t)(((float)ar[i] + (float)br[i] * bs) * r);
}

int launch_add_scaled_rmsnorm(const half_t* a, int64_t lda, const half_t* b, int64_t ldb, const float* bscale,
                              half_t* y, int64_t ldy, int rows, int n, hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  const bool vec = (n % 8 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) && (ldy % 8 == 0) && ((uintptr_t)a % 16 == 0) &&
                   ((uintptr_t)b % 16 == 0) && ((uintptr_t)y % 16 == 0) && n <= 8192;
  if (vec) launch_block_rows<true>(a, lda, b, ldb, bscale, nullptr, y, ldy, nullptr, rows, n, 0.f, stream);
  else hipLaunchKernelGGL(add_scaled_rmsnorm_kernel, dim3(rows), dim3(256), 0, stream, a, lda, b, ldb, bscale, y, ldy, n);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tri
