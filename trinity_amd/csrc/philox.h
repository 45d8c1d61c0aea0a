// Philox4x32-10 (Salmon et al., Random123) and the Gumbel transform used by
// the KeyFormer score path.  One call yields the noise of four consecutive
// keys of one (head, query) row:
//   counter = (key / 4, query, head, 0), key = (seed lo, seed hi).
#if (defined(TRI_BF16) && !defined(TRI_PHILOX_H_BF16)) || (!defined(TRI_BF16) && !defined(TRI_PHILOX_H_F16))
#ifdef TRI_BF16
#define TRI_PHILOX_H_BF16
#else
#define TRI_PHILOX_H_F16
#endif
#include "common.h"

namespace tri {

__host__ __device__ inline void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t out[4]) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// u = (top 23 bits + 0.5) * 2^-23 lies strictly inside (0, 1) and is exact in
// fp32; g = -ln(-ln(u)).
__device__ __forceinline__ float gumbel_from_bits(uint32_t x) {
  const float u = ((float)(x >> 9) + 0.5f) * 0x1p-23f;
  const float t = -kLn2 * fast_log2(u);
  return -kLn2 * fast_log2(t);
}

// 1 / (-ln u) for the same u: exp(g) of the Gumbel variate above
__device__ __forceinline__ float inv_neg_log_uniform(uint32_t x) {
  const float u = ((float)(x >> 9) + 0.5f) * 0x1p-23f;
  return __builtin_amdgcn_rcpf(-kLn2 * fast_log2(u));
}

}  // namespace tri

#endif  // once per element type
