// Device-side helpers shared by the gfx950 kernels: vector types, MFMA
// wrappers, LDS transpose reads, wavefront reductions.
//
// The kernels exist twice: once for fp16 and once for bf16 elements.  The bf16 copy is the same source compiled
// with -DTRI_BF16 -Dtri=tri_bf16 (every `namespace tri` / `tri::` then names the second namespace), so the
// headers may be included once per element type; `half_t` is "the 16-bit element type" of the copy.
#include <hip/hip_runtime.h>
#include <stdint.h>

#if (defined(TRI_BF16) && !defined(TRI_COMMON_H_BF16)) || (!defined(TRI_BF16) && !defined(TRI_COMMON_H_F16))
#ifdef TRI_BF16
#define TRI_COMMON_H_BF16
#else
#define TRI_COMMON_H_F16
#endif

namespace tri {

#ifdef TRI_BF16
typedef __bf16 half_t;
typedef __bf16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 half4v __attribute__((ext_vector_type(4)));
typedef __bf16 half8v __attribute__((ext_vector_type(8)));
#else
typedef _Float16 half_t;
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
#endif
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef short short4s __attribute__((__vector_size__(4 * sizeof(short))));

#define TRI_LDS __attribute__((address_space(3)))

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// D[32x32] += A[32x16] * B[16x32].  Lane l supplies row (l % 32) of A and
// column (l % 32) of B, eight consecutive k each, k-group (l / 32).  Lane l
// receives column (l % 32) of D; register r is row 8*(r/4) + 4*(l/32) + r%4.
__device__ __forceinline__ float16v mfma32(half8v a, half8v b, float16v c) {
#ifdef TRI_BF16
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#endif
}

// two probabilities (non-negative, at most 2^8) to the element type: fp16 truncates (one instruction), bf16 rounds
__device__ __forceinline__ half2v pack_prob(float a, float b) {
#ifdef TRI_BF16
  half2v h = {(half_t)a, (half_t)b};
  return h;
#else
  return __builtin_bit_cast(half2v, __builtin_amdgcn_cvt_pkrtz(a, b));
#endif
}

// eight OCP fp8 (e4m3) values to the 16-bit element type (exact: e4m3 has 3 mantissa bits and |x| <= 448)
__device__ __forceinline__ half8v fp8x8_to_half8(uint2v w) {
  typedef float float2v __attribute__((ext_vector_type(2)));
  const float2v f0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[0], false), f1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[0], true);
  const float2v f2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[1], false), f3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[1], true);
  const half2v p0 = pack_prob(f0[0], f0[1]), p1 = pack_prob(f1[0], f1[1]);
  const half2v p2 = pack_prob(f2[0], f2[1]), p3 = pack_prob(f3[0], f3[1]);
  const half8v h = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  return h;
}

// LDS transpose read: a 16-lane block reads a [4 rows][16 columns] patch of
// 16-bit elements, lane j of the block addressing row j/4, columns 4*(j%4)..+3;
// lane j receives column j of the patch, rows 0..3.
__device__ __forceinline__ half4v lds_read_tr16(const half_t* p) {
  short4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS short4s*)(uintptr_t)(p));
  half4v h;
  __builtin_memcpy(&h, &v, 8);
  return h;
}

__device__ __forceinline__ half8v cat8(half4v lo, half4v hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ half8v lds_read8(const half_t* p) { return *(const half8v*)p; }

// Exchange between lane l and lane l ^ 32 folded into a reduction.
__device__ __forceinline__ float pair_max(float x) {
  uint2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  uint2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}

// sum over the 32 lanes that share (lane / 32)
__device__ __forceinline__ float half_wave_sum(float x) {
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Sum of the `ksplit` fp32 partial results of a split-K product for four consecutive columns: split i holds them at
// partial + i * split_stride + off.
__device__ __forceinline__ float4v sum_splits(const float* partial, int ksplit, int64_t split_stride, int64_t off) {
  // eight splits at a time with all loads in flight together (past the last split the last one is re-read and
  // ignored); the order of the additions is fixed
  float4v s = {0.f, 0.f, 0.f, 0.f};
  for (int i0 = 0; i0 < ksplit; i0 += 8) {
    float4v p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j < ksplit ? i0 + j : ksplit - 1;
      p[j] = *reinterpret_cast<const float4v*>(partial + i * split_stride + off);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (i0 + j < ksplit) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] += p[j][e];
      }
  }
  return s;
}

}  // namespace tri

#endif  // once per element type
