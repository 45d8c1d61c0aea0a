// Two probes that measure the chip instead of computing anything for a caller.
//
// Issue probe: how many vector instructions hide under one MFMA on a gfx950 SIMD.  Every wave loops over a group of
// one v_mfma_f32_32x32x16_f16 (or none), n independent v_fma_f32 and t v_exp_f32, with a scheduling fence between
// groups.  One workgroup per CU (it asks for most of the LDS), four to sixteen waves, i.e. one to four waves per SIMD.
// The kernel measures itself: s_memtime ticks and 100 MHz ticks around the loop (to the moment the workgroup's last
// wave is through), per workgroup.  The softmax kernels of this library are bound by exactly this mix (an MFMA per
// 16 scores against a handful of vector instructions and an exponential per score), and the figures this probe
// gives are what the issue-bound estimate of bench.py is built from.  Its operands are constants: the chip runs at
// its full clock.
//
// Power probe (further down): the same kind of loop on random operands, long enough for the clock to settle at what
// the board's power limit leaves, with LDS reads and global -> LDS loads beside the MFMA as well: there a group's
// time is the energy it draws.
#include "../../include/trinity_amd.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kProbeLds = 96 * 1024;  // more than half of a CU's LDS: one workgroup per CU

// The instruction counts are template parameters: behind run-time counts every instruction of the group would sit
// behind a scalar branch of its own.
template <bool MFMA, int NV, int NT>
__global__ __launch_bounds__(1024) void issue_probe_kernel(int iters, int64_t* ticks, float* sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int t = threadIdx.x;
  if (t == 0) lds[0] = 1;  // the LDS request is what keeps a second workgroup off the CU
  float16v acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc0[r] = 0.f, acc1[r] = 0.f;
  half8v a = {1, 1, 1, 1, 1, 1, 1, 1}, b = {1, 1, 1, 1, 1, 1, 1, 1};
  asm volatile("" : "+v"(a), "+v"(b));  // operands the compiler cannot fold or rematerialise inside the loop
  float f[NV + 1], e[NT + 1];
#pragma unroll
  for (int i = 0; i < NV; ++i) f[i] = 0.001f * (float)(t + i);
#pragma unroll
  for (int i = 0; i < NT; ++i) e[i] = -0.001f * (float)(t + i);
  float m = 0.999f, c = 0.0005f;
  asm volatile("" : "+v"(m), "+v"(c));
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  // eight groups per trip (a taken branch costs a lone wave some twenty cycles), alternating between two
  // accumulators so that no MFMA waits for the result of the one before it
  for (int it = 0; it < iters; it += 8) {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      if (MFMA) {
        if (g & 1) acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc1, 0, 0, 0);
        else acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc0, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < NV; ++i) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[i]) : "v"(m), "v"(c));
#pragma unroll
      for (int i = 0; i < NT; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(e[i]));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // the SIMD serves its oldest wave first: the time of the group is the time until every wave is through
  __syncthreads();
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 16; ++r) s += acc0[r] + acc1[r];
#pragma unroll
  for (int i = 0; i < NV; ++i) s += f[i];
#pragma unroll
  for (int i = 0; i < NT; ++i) s += e[i];
  if (s == 12345.678f) sink[0] = s;  // keeps the arithmetic alive; never true in practice
  if (t == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;
    ticks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

template <bool MFMA, int NV, int NT>
int launch_probe(int waves_per_simd, int iters, int workgroups, int64_t* tk, float* sink, hipStream_t st) {
  auto kern = issue_probe_kernel<MFMA, NV, NT>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeLds) != hipSuccess)
    return TRI_ERR_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(workgroups), dim3(256 * waves_per_simd), kProbeLds, st, iters, tk, sink);
  return hipGetLastError() == hipSuccess ? TRI_OK : TRI_ERR_LAUNCH;
}

template <bool MFMA, int NV>
int launch_probe_nt(int n_trans, int w, int iters, int wgs, int64_t* tk, float* sink, hipStream_t st) {
  switch (n_trans) {
    case 0: return launch_probe<MFMA, NV, 0>(w, iters, wgs, tk, sink, st);
    case 1: return launch_probe<MFMA, NV, 1>(w, iters, wgs, tk, sink, st);
    case 2: return launch_probe<MFMA, NV, 2>(w, iters, wgs, tk, sink, st);
    case 4: return launch_probe<MFMA, NV, 4>(w, iters, wgs, tk, sink, st);
    default: return TRI_ERR_UNSUPPORTED;
  }
}

template <bool MFMA>
int launch_probe_nv(int n_valu, int n_trans, int w, int iters, int wgs, int64_t* tk, float* sink, hipStream_t st) {
  switch (n_valu) {
    case 0: return launch_probe_nt<MFMA, 0>(n_trans, w, iters, wgs, tk, sink, st);
    case 2: return launch_probe_nt<MFMA, 2>(n_trans, w, iters, wgs, tk, sink, st);
    case 4: return launch_probe_nt<MFMA, 4>(n_trans, w, iters, wgs, tk, sink, st);
    case 6: return launch_probe_nt<MFMA, 6>(n_trans, w, iters, wgs, tk, sink, st);
    case 8: return launch_probe_nt<MFMA, 8>(n_trans, w, iters, wgs, tk, sink, st);
    case 12: return launch_probe_nt<MFMA, 12>(n_trans, w, iters, wgs, tk, sink, st);
    case 16: return launch_probe_nt<MFMA, 16>(n_trans, w, iters, wgs, tk, sink, st);
    default: return TRI_ERR_UNSUPPORTED;
  }
}

// Power probe.  Under the board's power limit a kernel's time is the energy it draws: this kernel repeats a group
// of one MFMA on random (or zero) operands with LDS reads, v_fma_f32 and v_exp_f32 beside it, two waves per SIMD,
// long enough for the clock to settle, and reports both clocks.  Random operands: the pure MFMA loop already sits
// at the limit (about 1.7 GHz of 2.4), and every further instruction shows as time.  Zero operands: the same
// instruction streams at the full clock - what the issue limits alone allow.
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// the source of the probe's global -> LDS loads: small enough to stay in every L2
constexpr int kProbeSrcHalfs = 256 * 1024;
__device__ __attribute__((aligned(256))) _Float16 g_probe_src[kProbeSrcHalfs];

__global__ void power_probe_fill_kernel(_Float16* src, int random) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < kProbeSrcHalfs)
    src[i] = random ? (_Float16)((float)(int)(probe_hash(0x20000u + i) & 0xFFFFu) * (1.0f / 32768.0f) - 1.0f) : (_Float16)0.f;
}

// NL2: ds_read_b128 per two groups; NG8: global -> LDS loads (16 bytes per lane) per eight groups
template <int NL2, int NG8, int NV, int NT>
__global__ __launch_bounds__(512) void power_probe_kernel(int iters, int random, const _Float16* gsrc, int64_t* ticks,
                                                          float* sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int t = threadIdx.x;
  auto value = [&](uint32_t i) {   // fp16 in [-1, 1), or zero
    return random ? (_Float16)((float)(int)(probe_hash(i) & 0xFFFFu) * (1.0f / 32768.0f) - 1.0f) : (_Float16)0.f;
  };
  for (int i = t; i < 64 * 1024 / 2; i += 512) reinterpret_cast<_Float16*>(lds)[i] = value(0x10000u + i);
  half8v a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[i][e] = value((uint32_t)(t * 64 + i * 8 + e));
      b[i][e] = value((uint32_t)(t * 64 + 32 + i * 8 + e));
    }
  float16v acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  float f[NV + 1], e[NT + 1];
#pragma unroll
  for (int i = 0; i < NV; ++i) f[i] = (float)a[i % 4][i % 8] + 0.37f * (float)i;
#pragma unroll
  for (int i = 0; i < NT; ++i) e[i] = 0.f;
  float m = -1.0001f, c = 0.013f;  // the values change sign at every turn
  asm volatile("" : "+v"(m), "+v"(c));
  uint32_t addr = (uint32_t)(uintptr_t)lds + (t & 63) * 16 + (t >> 6) * 4096;  // a wave reads 1 KB in a row
  asm volatile("" : "+v"(addr));
  float4v l[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) l[i] = float4v{0.f, 0.f, 0.f, 0.f};
  // global -> LDS: a wave's load brings 1 KB in a row (of the wave's 4 KB of the source) to a place of its own
  // behind the 64 KB that are read
  const _Float16* gp = gsrc + ((int)(blockIdx.x % 16) * 8 + (t >> 6)) * 2048 + (t & 63) * 8;
  __attribute__((address_space(3))) unsigned char* ldst =
      (__attribute__((address_space(3))) unsigned char*)(uintptr_t)((uint32_t)(uintptr_t)lds + 64 * 1024 + (t >> 6) * 4096);
  __syncthreads();
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it += 8) {
#pragma unroll
    for (int i = 0; i < NG8; ++i)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gp + ((i + ((it >> 3) & 1) * NG8) % 4) * 512),
                                       (__attribute__((address_space(3))) void*)(ldst + i * 1024), 16, 0, 0);
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      acc[g & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[g & 3], b[(g >> 1) & 3], acc[g & 3], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < (NL2 + (g & 1)) / 2; ++i)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(l[(g + i) & 3]) : "v"(addr), "n"(((g * 2 + i) & 15) * 1024));
#pragma unroll
      for (int i = 0; i < NV; ++i) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[i]) : "v"(m), "v"(c));
#pragma unroll
      for (int i = 0; i < NT; ++i) asm volatile("v_exp_f32 %0, %1" : "=v"(e[i]) : "v"(f[i % (NV ? NV : 1)]));
      __builtin_amdgcn_sched_barrier(0);
    }
    // (the LDS reads of this trip; of the global loads all but those of the last two trips)
    if (NG8 > 0) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * NG8) : "memory");
    else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
    s += l[i][0] + l[i][1] + l[i][2] + l[i][3];
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) s += f[i];
#pragma unroll
  for (int i = 0; i < NT; ++i) s += e[i];
  if (s == 12345.678f) sink[0] = s;  // keeps the arithmetic alive; never true in practice
  if (t == 0) {
    ticks[2 * blockIdx.x] = c1 - c0;
    ticks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

template <int NL2, int NG8, int NV, int NT>
int launch_power(int iters, int random, int workgroups, int64_t* tk, float* sink, hipStream_t st) {
  auto kern = power_probe_kernel<NL2, NG8, NV, NT>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeLds) != hipSuccess)
    return TRI_ERR_LAUNCH;
  _Float16* src = nullptr;
  if (hipGetSymbolAddress((void**)&src, HIP_SYMBOL(g_probe_src)) != hipSuccess) return TRI_ERR_LAUNCH;
  hipLaunchKernelGGL(power_probe_fill_kernel, dim3(kProbeSrcHalfs / 256), dim3(256), 0, st, src, random);
  hipLaunchKernelGGL(kern, dim3(workgroups), dim3(512), kProbeLds, st, iters, random, src, tk, sink);
  return hipGetLastError() == hipSuccess ? TRI_OK : TRI_ERR_LAUNCH;
}

template <int NL2, int NG8>
int launch_power_nv(int n_valu, int n_trans, int iters, int random, int wgs, int64_t* tk, float* sink, hipStream_t st) {
  switch (n_valu * 2 + n_trans) {
    case 0: return launch_power<NL2, NG8, 0, 0>(iters, random, wgs, tk, sink, st);
    case 8: return launch_power<NL2, NG8, 4, 0>(iters, random, wgs, tk, sink, st);
    case 9: return launch_power<NL2, NG8, 4, 1>(iters, random, wgs, tk, sink, st);
    case 7: return launch_power<NL2, NG8, 3, 1>(iters, random, wgs, tk, sink, st);
    default: return TRI_ERR_UNSUPPORTED;
  }
}

template <int NG8>
int launch_power_nl(int nl2, int n_valu, int n_trans, int iters, int random, int wgs, int64_t* tk, float* sink,
                    hipStream_t st) {
  switch (nl2) {
    case 0: return launch_power_nv<0, NG8>(n_valu, n_trans, iters, random, wgs, tk, sink, st);
    case 1: return launch_power_nv<1, NG8>(n_valu, n_trans, iters, random, wgs, tk, sink, st);
    case 2: return launch_power_nv<2, NG8>(n_valu, n_trans, iters, random, wgs, tk, sink, st);
    case 4: return launch_power_nv<4, NG8>(n_valu, n_trans, iters, random, wgs, tk, sink, st);
    default: return TRI_ERR_UNSUPPORTED;
  }
}

}  // namespace

extern "C" int tri_diag_power_probe(int32_t lds_reads_per_two_groups, int32_t dma_loads_per_eight_groups, int32_t n_valu,
                                    int32_t n_trans, int32_t random_operands, int32_t iters, int32_t workgroups,
                                    tri_tensor* ticks, void* hip_stream) {
  if (ticks == nullptr || ticks->ptr == nullptr) return TRI_ERR_NULL;
  if (iters < 8 || iters % 8 != 0 || iters > (1 << 22) || workgroups < 1 || workgroups > 4096) return TRI_ERR_SHAPE;
  if (ticks->dtype != TRI_U8 || ticks->ndim != 1 || ticks->shape[0] < (int64_t)workgroups * 16 + 16) return TRI_ERR_SHAPE;
  if (((uintptr_t)ticks->ptr & 15u) != 0) return TRI_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  int64_t* tk = static_cast<int64_t*>(ticks->ptr);
  float* sink = reinterpret_cast<float*>(tk + 2 * (int64_t)workgroups);
  const int rnd = random_operands != 0, nl = lds_reads_per_two_groups;
  switch (dma_loads_per_eight_groups) {
    case 0: return launch_power_nl<0>(nl, n_valu, n_trans, iters, rnd, workgroups, tk, sink, st);
    case 2: return launch_power_nl<2>(nl, n_valu, n_trans, iters, rnd, workgroups, tk, sink, st);
    case 4: return launch_power_nl<4>(nl, n_valu, n_trans, iters, rnd, workgroups, tk, sink, st);
    default: return TRI_ERR_UNSUPPORTED;
  }
}

extern "C" int tri_diag_issue_probe(int32_t with_mfma, int32_t n_valu, int32_t n_trans, int32_t waves_per_simd,
                                    int32_t iters, int32_t workgroups, tri_tensor* ticks, void* hip_stream) {
  if (ticks == nullptr || ticks->ptr == nullptr) return TRI_ERR_NULL;
  if (waves_per_simd < 1 || waves_per_simd > 4) return TRI_ERR_UNSUPPORTED;
  if (iters < 8 || iters % 8 != 0 || iters > (1 << 20) || workgroups < 1 || workgroups > 4096) return TRI_ERR_SHAPE;
  // ticks: an int64 pair per workgroup, then sixteen bytes the kernel never writes in practice
  if (ticks->dtype != TRI_U8 || ticks->ndim != 1 || ticks->shape[0] < (int64_t)workgroups * 16 + 16) return TRI_ERR_SHAPE;
  if (((uintptr_t)ticks->ptr & 15u) != 0) return TRI_ERR_ALIGN;
  hipStream_t st = static_cast<hipStream_t>(hip_stream);
  int64_t* tk = static_cast<int64_t*>(ticks->ptr);
  float* sink = reinterpret_cast<float*>(tk + 2 * (int64_t)workgroups);
  return with_mfma ? launch_probe_nv<true>(n_valu, n_trans, waves_per_simd, iters, workgroups, tk, sink, st)
                   : launch_probe_nv<false>(n_valu, n_trans, waves_per_simd, iters, workgroups, tk, sink, st);
}
