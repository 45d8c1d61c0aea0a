// Issue probe: how many vector instructions hide under one MFMA on a gfx950 SIMD.
//
// Every wave loops over a group of one v_mfma_f32_32x32x16_f16 (or none), n independent v_fma_f32 and t
// v_exp_f32, with a scheduling fence between groups.  One workgroup per CU (it asks for most of the LDS), four
// or eight waves, i.e. one or two waves per SIMD.  The kernel measures itself: s_memtime ticks and 100 MHz
// ticks around the loop (to the moment the workgroup's last wave is through), per workgroup.  The softmax kernels of this library are bound by exactly this mix (an
// MFMA per 16 scores against a handful of vector instructions and an exponential per score), and the figures this
// probe gives are what the issue-bound estimate of bench.py is built from.
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
__global__ __launch_bounds__(512) void issue_probe_kernel(int iters, int64_t* ticks, float* sink) {
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

}  // namespace

extern "C" int tri_diag_issue_probe(int32_t with_mfma, int32_t n_valu, int32_t n_trans, int32_t waves_per_simd,
                                    int32_t iters, int32_t workgroups, tri_tensor* ticks, void* hip_stream) {
  if (ticks == nullptr || ticks->ptr == nullptr) return TRI_ERR_NULL;
  if (waves_per_simd != 1 && waves_per_simd != 2) return TRI_ERR_UNSUPPORTED;
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
