// KV caches held as OCP fp8 (e4m3, one fp32 scale per tensor): value = scale * fp8.
//
//   kv_quant_append_kernel   rows [P, P+S) of the caches = fp8(new k / k_scale), fp8(new v / v_scale), read from
//                            the fp16 rows the projection has just written (round to nearest even, saturating
//                            at +-448)
//   kv_dequant_kernel        rows [0, rows) of the caches as 16-bit elements WITHOUT the scale (every e4m3 value
//                            is exact in fp16 and bf16): the attention kernels fold k_scale into the softmax
//                            scale and v_scale into the final normalisation, so nothing is rounded twice
//
// The few-query attention kernel reads the fp8 rows directly (attn_few.hip); these two kernels serve the append
// and the kernels that want 16-bit K / V tiles.
#include "common.h"
#include "launch.h"

namespace tri {

// one thread per eight elements of one row; blockIdx.y = 0: K, 1: V
__global__ __launch_bounds__(256) void kv_quant_append_kernel(KvQuantArgs a) {
  const int cpr = a.D / 8;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.Hkv * a.S * cpr) return;
  const int c = idx % cpr, m = (idx / cpr) % a.S, hk = idx / (cpr * a.S);
  const bool isv = blockIdx.y != 0;
  const half_t* src = isv ? a.v + (int64_t)hk * a.v_sh + (int64_t)m * a.v_sr : a.k + (int64_t)hk * a.k_sh + (int64_t)m * a.k_sr;
  uint8_t* dst = isv ? a.vc + (int64_t)hk * a.vc_sh + (int64_t)(a.P + m) * a.vc_sr
                     : a.kc + (int64_t)hk * a.kc_sh + (int64_t)(a.P + m) * a.kc_sr;
  const float scale = isv ? a.v_scale : a.k_scale;
  const half8v x = *reinterpret_cast<const half8v*>(src + c * 8);
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = fminf(fmaxf((float)x[e] / scale, -448.0f), 448.0f);
  uint2v out;
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
  out[0] = (uint32_t)w;
  w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w, true);
  out[1] = (uint32_t)w;
  *reinterpret_cast<uint2v*>(dst + c * 8) = out;
}

__global__ __launch_bounds__(256) void kv_dequant_kernel(KvDequantArgs a) {
  const int cpr = a.D / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)a.Hkv * a.rows * cpr) return;
  const int c = (int)(idx % cpr), m = (int)((idx / cpr) % a.rows), hk = (int)(idx / ((int64_t)cpr * a.rows));
  const bool isv = blockIdx.y != 0;
  const uint8_t* src = isv ? a.vc + (int64_t)hk * a.vc_sh + (int64_t)m * a.vc_sr : a.kc + (int64_t)hk * a.kc_sh + (int64_t)m * a.kc_sr;
  half_t* dst = (isv ? a.v : a.k) + ((int64_t)hk * a.rows + m) * a.D;
  *reinterpret_cast<half8v*>(dst + c * 8) = fp8x8_to_half8(*reinterpret_cast<const uint2v*>(src + c * 8));
}

int launch_kv_quant_append(const KvQuantArgs& a, hipStream_t stream) {
  if (a.S <= 0) return 0;
  const int threads = a.Hkv * a.S * (a.D / 8);
  hipLaunchKernelGGL(kv_quant_append_kernel, dim3((threads + 255) / 256, 2), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_kv_dequant(const KvDequantArgs& a, hipStream_t stream) {
  if (a.rows <= 0) return 0;
  const int64_t threads = (int64_t)a.Hkv * a.rows * (a.D / 8);
  hipLaunchKernelGGL(kv_dequant_kernel, dim3((unsigned)((threads + 255) / 256), 2), dim3(256), 0, stream, a);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tri
