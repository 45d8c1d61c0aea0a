// Philox4x32-7 (Salmon et al., Random123: the 4 x 32 generator at seven rounds,
// the fewest at which it passes BigCrush - their Table 2; ten is the library's
// default with a safety margin) and the Gumbel transform used by the KeyFormer
// score path.  The generator is most of what the seeded noise costs, and on this
// chip a round is two quarter-rate 32 x 32 -> 64 multiplies: seven rounds instead
// of ten take 21 us off the 572 us KeyFormer block at S = 4096.  One call yields sixteen random bits for each of
// eight keys of one (head, query) row - two groups of four consecutive keys,
// eight apart, which is what one lane of the score tiles holds:
//   counter = (2 * (key / 16) + (key / 4) % 2, query, head, 0), key = (seed lo, seed hi);
//   key k takes word k % 4 of the output, its low half if (k / 8) % 2 == 0, else its high half.
// (The reference feeds the noise as an fp16 tensor, 11 significant bits; sixteen-bit uniforms are finer than
// that and halve the generator's cost, which dominates the seeded kernels.)
#if (defined(TRI_BF16) && !defined(TRI_PHILOX_H_BF16)) || (!defined(TRI_BF16) && !defined(TRI_PHILOX_H_F16))
#ifdef TRI_BF16
#define TRI_PHILOX_H_BF16
#else
#define TRI_PHILOX_H_F16
#endif
#include "common.h"

namespace tri {

constexpr int kPhiloxRounds = 7;

__device__ __forceinline__ void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                           uint32_t k1, uint32_t out[4]) {
#pragma unroll
  for (int r = 0; r < kPhiloxRounds; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    // hi ^ counter ^ key in one three-input bit operation (truth table 0x96 = a ^ b ^ c)
    const uint32_t n0 = __builtin_amdgcn_bitop3_b32((uint32_t)(p1 >> 32), c1, k0, 0x96);
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = __builtin_amdgcn_bitop3_b32((uint32_t)(p0 >> 32), c3, k1, 0x96);
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// counter word 0 of the call that covers `key`
__device__ __forceinline__ uint32_t noise_counter(int key) { return (uint32_t)((key >> 4) * 2 + ((key >> 2) & 1)); }
// the sixteen bits of `key` out of the four output words of its call
__device__ __forceinline__ uint32_t noise_bits(const uint32_t rnd[4], int key) {
  const uint32_t w = rnd[key & 3];
  return ((key >> 3) & 1) ? (w >> 16) : (w & 0xFFFFu);
}

// u = (bits + 0.5) * 2^-16 lies strictly inside (0, 1) and is exact in fp32;
// g = -ln(-ln(u)).
__device__ __forceinline__ float gumbel_from_bits(uint32_t bits16) {
  const float u = ((float)bits16 + 0.5f) * 0x1p-16f;
  const float t = -kLn2 * fast_log2(u);
  return -kLn2 * fast_log2(t);
}

// exp(g) of the Gumbel variate above is 1 / (-ln u) = kInvNegLnScale / log2(u): the callers sum
// probability * inv_log2_uniform(bits) and apply the constant factor once per sum.
constexpr float kInvNegLnScale = -1.4426950408889634f;  // -1 / ln 2
__device__ __forceinline__ float inv_log2_uniform(uint32_t bits16) {
  return __builtin_amdgcn_rcpf(fast_log2(fmaf((float)bits16, 0x1p-16f, 0x1p-17f)));
}

// Gumbel noise of the four consecutive keys key .. key + 3 (key % 4 == 0) - for the paths that do not hold both
// groups of a call in one lane
__device__ __forceinline__ void gumbel4(int key, int q, int h, uint32_t seed_lo, uint32_t seed_hi, float gn[4]) {
  uint32_t rnd[4];
  philox4x32(noise_counter(key), (uint32_t)q, (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
  for (int e = 0; e < 4; ++e) gn[e] = gumbel_from_bits(((key >> 3) & 1) ? (rnd[e] >> 16) : (rnd[e] & 0xFFFFu));
}

}  // namespace tri

#endif  // once per element type
