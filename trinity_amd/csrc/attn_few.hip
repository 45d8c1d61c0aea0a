// Attention for few queries (S <= 32) against a long key axis: the reference's
// own regime (16 new tokens, 1024 cached keys per head), where the kernel is
// bound by reading the K/V cache once.
//
// The key axis is split over workgroups of 256 keys; each of the four waves
// of a workgroup owns ONE tile of 64 keys, so nothing loops: a wave issues all
// its loads at once (V straight into its private LDS tile, K rows straight
// into MFMA source registers: [key][d] is already the layout source 0 of
// S^T = K . Q^T wants), does one exact softmax over its tile, and the four
// waves merge their (max, sum, O) through LDS.  A second small kernel merges
// the workgroups' partial results and writes O2, the log-sum-exp, and (for
// KeyFormer) the log-sum-exp of the noise-perturbed logits.
//
// Partial results in the workspace (fp32): O [Hq][nsplit][S][D] unnormalised,
// stats [Hq][nsplit][S][4] = (max, sum, perturbed max, perturbed sum), log2 units.
#include "common.h"
#include "launch.h"
#include "philox.h"

namespace tri {

constexpr int kFewTile = 64;        // keys per wave
constexpr int kFewKeysPerWg = 256;  // keys per workgroup
constexpr float kNegBig = -1.0e30f; // "no key seen yet" (finite, so that differences stay defined)
constexpr int kFewWaves = kFewKeysPerWg / kFewTile;

template <int D>
__device__ __forceinline__ int few_fv(int row) { return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }

// Merge of a split-K projection for this workgroup: rows [0, S) x D columns of `nseg` column blocks (q head; new k
// rows; new v rows) starting at columns col0[], each the sum of the splits in a fixed order, rounded to the element
// type, RMS-normalised per row when `norm` (q and k only) - the arithmetic of the projection's own merge kernel -
// stored to LDS dst_lds[seg] [row][D] and, where dst_g[seg] is given, to global rows of stride g_stride[seg].
// Every thread takes up to R groups of four columns and has the loads of all of them in flight together: the
// partial sums sit in other XCDs' caches, one round trip instead of one per block.  Called by all NT threads of the workgroup.
template <int D, int R, int NT>
__device__ __forceinline__ void few_merge_projection(const AttnArgs& a, int nseg, const int (&col0)[3], bool norm,
                                                     half_t* const (&dst_lds)[3], half_t* const (&dst_g)[3],
                                                     const int64_t (&g_stride)[3]) {
  constexpr int LPH = D / 4;  // lanes per row
  const int per = a.S * LPH, total = nseg * per;
  const int64_t split_stride = (int64_t)a.S * a.pj_ntot;
  for (int base = 0; base < total; base += NT * R) {
    bool live[R];
    int seg[R], m[R], li[R];
    const float* src[R];
    float4v acc[R];
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int idx = base + u * NT + (int)threadIdx.x;
      live[u] = idx < total;
      seg[u] = live[u] ? idx / per : 0;
      const int rem = live[u] ? idx - seg[u] * per : 0;
      m[u] = rem / LPH;
      li[u] = rem % LPH;
      const int c0 = seg[u] == 0 ? col0[0] : (seg[u] == 1 ? col0[1] : col0[2]);
      src[u] = a.pj + (int64_t)m[u] * a.pj_ntot + c0 + li[u] * 4;
      acc[u] = float4v{0.f, 0.f, 0.f, 0.f};
    }
    // eight splits at a time (past the last split the last one is re-read and ignored)
    for (int i0 = 0; i0 < a.pj_ksplit; i0 += 8) {
      float4v p[R][8];
#pragma unroll
      for (int u = 0; u < R; ++u)
        if (live[u]) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int i = i0 + j < a.pj_ksplit ? i0 + j : a.pj_ksplit - 1;
            p[u][j] = *reinterpret_cast<const float4v*>(src[u] + i * split_stride);
          }
        }
#pragma unroll
      for (int u = 0; u < R; ++u)
        if (live[u]) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (i0 + j < a.pj_ksplit) {
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[u][e] += p[u][j][e];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
      half4v h = {(half_t)acc[u][0], (half_t)acc[u][1], (half_t)acc[u][2], (half_t)acc[u][3]};
      if (norm) {  // uniform; every lane takes part in the reduction
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) ss = fmaf((float)h[e], (float)h[e], ss);
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        if (seg[u] < 2) {
          const float nrm = rsqrtf(ss / (float)D + a.eps);
#pragma unroll
          for (int e = 0; e < 4; ++e) h[e] = (half_t)((float)h[e] * nrm);
        }
      }
      if (live[u]) {
        half_t* dl = seg[u] == 0 ? dst_lds[0] : (seg[u] == 1 ? dst_lds[1] : dst_lds[2]);
        half_t* dg = seg[u] == 0 ? dst_g[0] : (seg[u] == 1 ? dst_g[1] : dst_g[2]);
        const int64_t gs = seg[u] == 0 ? g_stride[0] : (seg[u] == 1 ? g_stride[1] : g_stride[2]);
        *reinterpret_cast<half4v*>(dl + m[u] * D + li[u] * 4) = h;
        if (dg != nullptr) *reinterpret_cast<half4v*>(dg + (int64_t)m[u] * gs + li[u] * 4) = h;
      }
    }
  }
}

// FP8: K and V come from fp8 (e4m3) caches (a.k8 / a.v8) and are converted on the way in - K rows in registers, V
// rows while they are staged in LDS; their scales are folded into a.scale and a.out_scale by the caller.
// FUSED: q and the new rows of k / v come from the partial sums of a split-K projection (AttnArgs::pj): every
// workgroup merges its head's q rows, the workgroups whose keys include new ones merge those k / v rows too, all
// into LDS; one workgroup per q head / kv head also stores them where the unfused projection would have.
// NW: waves (tiles of 64 keys) per workgroup.
template <int D, bool KEYFORMER, bool FP8, bool FUSED, int NW>
__device__ __forceinline__ void attn_few_body(const AttnArgs& a, half_t* lds) {
  constexpr int KPW = NW * kFewTile;  // keys per workgroup
  static_assert(!(FP8 && FUSED), "the fused merge writes 16-bit caches");
  constexpr int KSTEPS = D / 16, DT = D / 32, CPR = D / 8;
  constexpr int VINSTR = kFewTile * D * 2 / 1024;  // 1 KB per wave-level load
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int split = blockIdx.x, nsplit = gridDim.x, h = blockIdx.y;
  const int hk = h / (a.Hq / a.Hkv);
  const int Ltot = a.P + a.S;
  const int key0 = split * KPW + wave * kFewTile;
  half_t* vs = lds + wave * kFewTile * D;  // this wave's V tile, later its O tile
  const bool live = key0 < Ltot;           // wave-uniform

  float m = kNegBig, l = 0.f, mp = kNegBig, lp = 0.f;
  float16v o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;

  // FUSED: merged rows [32][D] of q, new k, new v behind the V tiles and the statistics
  half_t* stage_q = lds + NW * kFewTile * D + NW * 32 * 4 * 2;
  half_t* stage_k = stage_q + 32 * D;
  half_t* stage_v = stage_k + 32 * D;
  const int qq = l32 < a.S ? l32 : a.S - 1;
  half8v qf[KSTEPS], kf[2][KSTEPS];

  if (live) {
    // ---- V tile -> LDS (rows past the last key read as zero), XOR-swizzled for the transpose reads
    if (FP8) {
      const uint8_t* vbase = a.v8 + (int64_t)hk * a.v8_sh;
      uint2v raw[VINSTR];
#pragma unroll
      for (int i = 0; i < VINSTR; ++i) {
        const int p = i * 64 + lane;
        const int row = p / CPR, slot = p % CPR;
        const int key = key0 + row;
        raw[i] = uint2v{0u, 0u};  // fp8 zero
        if (key < Ltot)
          raw[i] = *reinterpret_cast<const uint2v*>(vbase + (int64_t)key * a.v8_sr + (slot ^ few_fv<D>(row)) * 8);
      }
#pragma unroll
      for (int i = 0; i < VINSTR; ++i) *reinterpret_cast<half8v*>(vs + i * 512 + lane * 8) = fp8x8_to_half8(raw[i]);
    } else {
      const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<half_t*>(a.v + (int64_t)hk * a.v_sh), 0, (int)((int64_t)Ltot * a.v_sr * 2), 0x00020000);
#pragma unroll
      for (int i = 0; i < VINSTR; ++i) {
        const int p = i * 64 + lane;
        const int row = p / CPR, slot = p % CPR;
        const int off = ((key0 + row) * (int)a.v_sr + (slot ^ few_fv<D>(row)) * 8) * 2;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(vrsrc, (TRI_LDS void*)(vs + i * 512), 16, off, 0, 0, 0);
      }
    }
    // ---- Q (source 1) and K (source 0) fragments straight from global memory
    {
      if (!FUSED) {
        const half_t* qp = a.q + (int64_t)qq * a.ldq + h * D + g * 8;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const half8v*>(qp + ks * 16);
      }
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        int key = key0 + mt * 32 + l32;
        key = key < Ltot ? key : Ltot - 1;
        if (FP8) {
          const uint8_t* kp = a.k8 + (int64_t)hk * a.k8_sh + (int64_t)key * a.k8_sr + g * 8;
          uint2v raw[KSTEPS];
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) raw[ks] = *reinterpret_cast<const uint2v*>(kp + ks * 16);
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) kf[mt][ks] = fp8x8_to_half8(raw[ks]);
        } else {
          const half_t* kp = a.k + (int64_t)hk * a.k_sh + (int64_t)key * a.k_sr + g * 8;
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks) kf[mt][ks] = *reinterpret_cast<const half8v*>(kp + ks * 16);
        }
      }
    }
  }

  if (FUSED) {
    // (the loads above stay in flight meanwhile; rows >= P of the K / V buffers hold stale values until the
    // writer workgroups below have run, and are replaced from LDS further down)
    const int group = a.Hq / a.Hkv, nq = a.Hq * D, nkv = a.Hkv * D;
    // the k / v rows too when some of this workgroup's keys are new
    const bool kv = split * KPW < Ltot && (split + 1) * KPW > a.P;
    const bool writer = split == a.P / KPW && h % group == 0;
    const int col0[3] = {h * D, nq + hk * D, nq + nkv + hk * D};
    half_t* const dst_lds[3] = {stage_q, stage_k, stage_v};
    half_t* const dst_g[3] = {(split == 0 && a.q_w != nullptr) ? a.q_w + h * D : nullptr,
                              writer ? a.k_w + (int64_t)hk * a.k_sh + (int64_t)a.P * a.k_sr : nullptr,
                              writer ? a.v_w + (int64_t)hk * a.v_sh + (int64_t)a.P * a.v_sr : nullptr};
    const int64_t g_stride[3] = {a.ldq, a.k_sr, a.v_sr};
    few_merge_projection<D, 3, NW * 64>(a, kv ? 3 : 1, col0, a.qknorm != 0, dst_lds, dst_g, g_stride);
    __syncthreads();
  }

  if (live) {
    if (FUSED) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const half8v*>(stage_q + qq * D + g * 8 + ks * 16);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        int key = key0 + mt * 32 + l32;
        key = key < Ltot ? key : Ltot - 1;
        if (key >= a.P) {
#pragma unroll
          for (int ks = 0; ks < KSTEPS; ++ks)
            kf[mt][ks] = *reinterpret_cast<const half8v*>(stage_k + (key - a.P) * D + g * 8 + ks * 16);
        }
      }
    }
    float16v st[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[mt][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) st[mt] = mfma32(kf[mt][ks], qf[ks], st[mt]);

    // ---- one exact softmax over the tile (log2 units); lane = query, registers = keys
    const float c2 = a.scale * kLog2e;
    const int qlim = a.causal ? a.P + qq : Ltot;  // last visible key
    if (KEYFORMER) {
      const float cp2 = kLog2e / a.tau;  // perturbed logits: (scale * qk + g) * cp2
      const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);
      const bool vec = (Ltot & 3) == 0;  // rows of the noise tensor keep groups of four keys 8-byte aligned
      float sp[2][16];
      float mx = kNegBig;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int rp = 0; rp < 2; ++rp) {
          // key groups rq = 2 rp and 2 rp + 1 (eight keys apart) are the two halves of one generator call
          uint32_t rnd[4] = {0u, 0u, 0u, 0u};
          if (a.noise == nullptr)
            philox4x32(noise_counter(key0 + mt * 32 + rp * 16 + g * 4), (uint32_t)qq, (uint32_t)h, 0u, seed_lo, seed_hi, rnd);
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int rq = rp * 2 + half;
            const int key = key0 + mt * 32 + rq * 8 + g * 4;
            float gn[4];
            if (a.noise != nullptr) {
              const half_t* np = a.noise + ((int64_t)h * a.S + qq) * Ltot;
              if (vec) {
                const half4v n4 = *reinterpret_cast<const half4v*>(np + (key < Ltot ? key : Ltot - 4));
#pragma unroll
                for (int e = 0; e < 4; ++e) gn[e] = (float)n4[e];
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) gn[e] = (float)np[key + e < Ltot ? key + e : Ltot - 1];
              }
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) gn[e] = gumbel_from_bits(half ? (rnd[e] >> 16) : (rnd[e] & 0xFFFFu));
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float v = (st[mt][rq * 4 + e] * a.scale + gn[e]) * cp2;
              if (key + e > qlim || key + e >= Ltot) v = -INFINITY;
              sp[mt][rq * 4 + e] = v;
              mx = fmaxf(mx, v);
            }
          }
        }
      mp = pair_max(mx);
      float sum = 0.f;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += fast_exp2(sp[mt][r] - mp);
      lp = pair_sum(sum);
    }
    float mx = kNegBig;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = key0 + mt * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
        float s = st[mt][r] * c2;
        if (key > qlim || key >= Ltot) s = -INFINITY;
        st[mt][r] = s;
        mx = fmaxf(mx, s);
      }
    m = pair_max(mx);
    half8v pf[2][2];
    float sum = 0.f;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        half8v pk;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float p0 = fast_exp2(st[mt][hh * 8 + e] - m);
          const float p1 = fast_exp2(st[mt][hh * 8 + e + 1] - m);
          sum += p0 + p1;
          const half2v h2 = pack_prob(p0, p1);
          pk[e] = h2[0];
          pk[e + 1] = h2[1];
        }
        pf[mt][hh] = pk;
      }
    l = pair_sum(sum);

    // ---- O^T = V^T . P^T
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the V tile has landed (wave-private, no barrier needed)
    if (FUSED) {  // rows of new keys: from the merged rows, into the same swizzled places
      const int r0 = a.P > key0 ? a.P - key0 : 0;
      const int r1 = Ltot - key0 < kFewTile ? Ltot - key0 : kFewTile;
      for (int p = r0 * CPR + lane; p < r1 * CPR; p += 64) {
        const int row = p / CPR, slot = p % CPR;
        *reinterpret_cast<half8v*>(vs + row * D + slot * 8) =
            *reinterpret_cast<const half8v*>(stage_v + (key0 + row - a.P) * D + ((slot ^ few_fv<D>(row)) << 3));
      }
    }
    const int j4 = (lane & 15) >> 2;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const int chunk = dt * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
          const half_t* vp = vs + (mt * 32 + hh * 16 + 4 * g + j4) * D + ((chunk ^ few_fv<D>(j4)) << 3) + (lane & 1) * 4;
          const half8v vf = cat8(lds_read_tr16(vp), lds_read_tr16(vp + 8 * D));
          o[dt] = mfma32(vf, pf[mt][hh], o[dt]);
        }
  }

  // ---- merge the waves through LDS: O tiles as [d / 4][query] float4 (in place of the V tiles),
  // statistics behind them
  float* ow = reinterpret_cast<float*>(vs);
  float* stats = reinterpret_cast<float*>(lds + NW * kFewTile * D);  // [wave][query][4]
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const int d4 = dt * 8 + rq * 2 + g;
      const float4v v = {o[dt][rq * 4], o[dt][rq * 4 + 1], o[dt][rq * 4 + 2], o[dt][rq * 4 + 3]};
      *reinterpret_cast<float4v*>(ow + (d4 * 32 + l32) * 4) = v;
    }
  if (g == 0) {
    const float4v v = {m, l, mp, lp};
    *reinterpret_cast<float4v*>(stats + (wave * 32 + l32) * 4) = v;
  }
  __syncthreads();
  const int q = t & 31;
  float sc[NW];
  float4v tot;
  {
    float4v s4[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) s4[w] = *reinterpret_cast<const float4v*>(stats + (w * 32 + q) * 4);
    float M = s4[0][0], Mp = s4[0][2];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
      M = fmaxf(M, s4[w][0]);
      Mp = fmaxf(Mp, s4[w][2]);
    }
    float L = 0.f, Lp = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      sc[w] = fast_exp2(s4[w][0] - M);
      L = fmaf(s4[w][1], sc[w], L);
      Lp = fmaf(s4[w][3], fast_exp2(s4[w][2] - Mp), Lp);
    }
    tot = float4v{M, L, Mp, Lp};
  }
  if (q < a.S) {
    const int64_t row = ((int64_t)h * nsplit + split) * a.S + q;
    float* po = a.ws + row * D;
    const float* o_lds = reinterpret_cast<const float*>(lds);
#pragma unroll
    for (int j = 0; j < (D / 4) / (NW * 2); ++j) {
      const int d4 = (t >> 5) + NW * 2 * j;  // NW * 2 groups of 32 threads share the D / 4 column groups
      float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float4v v = *reinterpret_cast<const float4v*>(o_lds + w * (kFewTile * D / 2) + (d4 * 32 + q) * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(v[e], sc[w], acc[e]);
      }
      *reinterpret_cast<float4v*>(po + d4 * 4) = acc;
    }
    if ((t >> 5) == 0)
      *reinterpret_cast<float4v*>(a.ws + (int64_t)a.Hq * nsplit * a.S * D + row * 4) = tot;
  }
}

// (body in a device function: device-only types must not reach the host pass of the compiler)
template <int D, bool KEYFORMER, bool FP8, bool FUSED, int NW>
__global__ __launch_bounds__(NW * 64) void attn_few_kernel(AttnArgs a) {
  extern __shared__ __attribute__((aligned(16))) half_t lds[];
  attn_few_body<D, KEYFORMER, FP8, FUSED, NW>(a, lds);
}

// One thread per (head, query, four output columns): merge the splits.
template <int D>
__global__ __launch_bounds__(256) void attn_few_combine_kernel(AttnArgs a, int nsplit) {
  constexpr int LPQ = D / 4;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int pair = idx / LPQ, d4 = idx % LPQ;
  if (pair >= a.Hq * a.S) return;
  const int h = pair / a.S, q = pair % a.S;
  const float* stats = a.ws + (int64_t)a.Hq * nsplit * a.S * D;
  // splits are taken eight at a time with all their loads (statistics and O rows) in flight together (past the
  // last split the last one is re-read and ignored), in a fixed order; the running maxima are raised between the
  // groups of eight, so up to eight splits cost one round trip
  float M = kNegBig, Mp = kNegBig, L = 0.f, Lp = 0.f;
  float4v acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < nsplit; s0 += 8) {
    float4v v[8], ov[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < nsplit ? s0 + j : nsplit - 1;
      const int64_t row = ((int64_t)h * nsplit + s) * a.S + q;
      v[j] = *reinterpret_cast<const float4v*>(stats + row * 4);
      ov[j] = *reinterpret_cast<const float4v*>(a.ws + row * D + d4 * 4);
    }
    float Mn = M, Mpn = Mp;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      Mn = fmaxf(Mn, v[j][0]);
      Mpn = fmaxf(Mpn, v[j][2]);
    }
    const float r = fast_exp2(M - Mn), rp = fast_exp2(Mp - Mpn);  // (1 when nothing changed, 0 at the first group)
    L *= r;
    Lp *= rp;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] *= r;
    M = Mn;
    Mp = Mpn;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (s0 + j < nsplit) {
        const float w = fast_exp2(v[j][0] - M);
        L = fmaf(v[j][1], w, L);
        Lp = fmaf(v[j][3], fast_exp2(v[j][2] - Mp), Lp);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(ov[j][e], w, acc[e]);
      }
    }
  }
  const float inv = a.out_scale / L;
  half4v hv;
#pragma unroll
  for (int e = 0; e < 4; ++e) hv[e] = (half_t)(acc[e] * inv);
  *reinterpret_cast<half4v*>(a.out + (int64_t)q * a.ldo + h * D + d4 * 4) = hv;
  if (d4 == 0) {
    if (a.lse != nullptr) a.lse[(int64_t)h * a.S + q] = (M + fast_log2(L)) * kLn2;
    if (a.lse_pert != nullptr) a.lse_pert[(int64_t)h * a.S + q] = (Mp + fast_log2(Lp)) * kLn2;
  }
}

// Per-key accumulators over few queries (RoCo sum p / sum p^2, KeyFormer sum of perturbed probabilities).
// Scores are computed as S[query, key] = Q . K^T, so a lane owns ONE key and sixteen queries: the sum over
// queries is a sum over registers plus one exchange with lane l ^ 32.  A wave covers 64 keys.
// MODE_ 0: RoCo; 1: KeyFormer with a noise tensor; 2: KeyFormer with seeded noise
// SHARED: the four waves are four query heads that share a KV head, all on the same 64 keys, whose K rows go
// global -> LDS once for the workgroup (long prefixes with grouped heads: the K rows are then read from memory once
// per group instead of once per head).  Otherwise the waves are four 64-key tiles of one head, K rows straight into
// registers.
template <int D>
__device__ __forceinline__ int few_fk(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }

template <int D, int MODE_, bool SHARED>
__global__ __launch_bounds__(256) void score_few_kernel(ScoreArgs a) {
  constexpr int MODE = MODE_ == 0 ? 0 : 1;
  constexpr bool SEEDED = MODE_ == 2;
  constexpr int KSTEPS = D / 16, CPR = D / 8;
  __shared__ __attribute__((aligned(16))) half_t ktile[SHARED ? kFewTile * D : 8];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  // SHARED: blockIdx.y = (KV head, chunk of four of its query heads); a wave past the group's last head only helps
  // with the loads
  const int group = a.Hq / a.Hkv, chunks = (group + 3) / 4;
  const int hk = SHARED ? (int)blockIdx.y / chunks : (int)blockIdx.y / group;
  const int h = SHARED ? hk * group + ((int)blockIdx.y % chunks) * 4 + wave : (int)blockIdx.y;
  const bool idle = SHARED && h >= (hk + 1) * group;
  const int Ltot = a.P + a.S;
  const int key0 = SHARED ? (int)blockIdx.x * kFewTile : (int)blockIdx.x * kFewKeysPerWg + wave * kFewTile;
  if (key0 >= Ltot) return;  // wave-uniform (SHARED: the same for the whole workgroup, which has one barrier below)
  half8v qf[KSTEPS], kf[2][KSTEPS];
  {
    const int qq = l32 < a.S ? l32 : a.S - 1;
    const half_t* qp = a.q + (int64_t)qq * a.ldq + (idle ? 0 : h) * D + g * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[ks] = *reinterpret_cast<const half8v*>(qp + ks * 16);
    if (SHARED) {
      // rows past the last key read as zero; chunk c of row r sits at slot c ^ few_fk(r) (fragment reads conflict-free)
      const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<half_t*>(a.k + (int64_t)hk * a.k_sh), 0, (int)((int64_t)Ltot * a.k_sr * 2), 0x00020000);
      constexpr int INSTR = kFewTile * D * 2 / 1024 / 4;
#pragma unroll
      for (int i = 0; i < INSTR; ++i) {
        const int p = (i * 4 + wave) * 64 + lane;
        const int row = p / CPR, slot = p % CPR;
        const int off = ((key0 + row) * (int)a.k_sr + (slot ^ few_fk<D>(row)) * 8) * 2;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(krsrc, (TRI_LDS void*)(ktile + (i * 4 + wave) * 512), 16, off, 0, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      __syncthreads();
      if (idle) return;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks)
          kf[nt][ks] = lds_read8(ktile + (nt * 32 + l32) * D + (((ks * 2 + g) ^ few_fk<D>(nt * 32 + l32)) << 3));
    } else {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        int key = key0 + nt * 32 + l32;
        key = key < Ltot ? key : Ltot - 1;
        const half_t* kp = a.k + (int64_t)hk * a.k_sh + (int64_t)key * a.k_sr + g * 8;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) kf[nt][ks] = *reinterpret_cast<const half8v*>(kp + ks * 16);
      }
    }
  }
  // register r of an accumulator holds query 8 * (r / 4) + 4 * g + r % 4
  float lse2[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int q = 8 * (r >> 2) + 4 * g + (r & 3);
    lse2[r] = a.lse[(int64_t)h * a.S + (q < a.S ? q : a.S - 1)] * kLog2e;
  }
  const float c2 = a.scale * kLog2e, cp2 = kLog2e / a.tau;
  const uint32_t seed_lo = (uint32_t)a.seed, seed_hi = (uint32_t)(a.seed >> 32);
  const float invS = 1.0f / (float)a.S;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    float16v st;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) st = mfma32(qf[ks], kf[nt][ks], st);
    const int key = key0 + nt * 32 + l32;
    const int kc = key < Ltot ? key : Ltot - 1;
    // Seeded noise: one generator call covers eight keys - lanes that differ in bits 0, 1 and 3 - for one query.
    // Each of those eight lanes makes the calls of two of the sixteen queries and the words travel by lane
    // exchange: two calls per lane instead of sixteen.  (The counter comes from the unclamped key: lanes past the
    // last key still serve their group.)
    uint32_t mine[2][4];
    if (SEEDED) {
      const int j = ((lane >> 3) & 1) * 4 + (lane & 3);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int r = 2 * j + u;
        const int q = 8 * (r >> 2) + 4 * g + (r & 3);
        philox4x32(noise_counter(key), (uint32_t)(q < a.S ? q : a.S - 1), (uint32_t)h, 0u, seed_lo, seed_hi, mine[u]);
      }
    }
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int q = 8 * (r >> 2) + 4 * g + (r & 3);
      const int qq = q < a.S ? q : a.S - 1;
      float x;
      if (MODE == 1) {
        float gn;
        if (!SEEDED) {
          gn = (float)a.noise[((int64_t)h * a.S + qq) * Ltot + kc];
        } else {
          const int src = (lane & ~11) | (((r >> 1) >> 2) << 3) | ((r >> 1) & 3);  // the lane that made query r's call
          const uint32_t w0 = __shfl(mine[r & 1][0], src, 64), w1 = __shfl(mine[r & 1][1], src, 64);
          const uint32_t w2 = __shfl(mine[r & 1][2], src, 64), w3 = __shfl(mine[r & 1][3], src, 64);
          const int e = key & 3;
          const uint32_t w = e == 0 ? w0 : (e == 1 ? w1 : (e == 2 ? w2 : w3));
          gn = gumbel_from_bits(((key >> 3) & 1) ? (w >> 16) : (w & 0xFFFFu));
        }
        x = (st[r] * a.scale + gn) * cp2 - lse2[r];
      } else {
        x = fmaf(st[r], c2, -lse2[r]);
      }
      float p = fast_exp2(x);
      if (q >= a.S || key >= Ltot || (a.causal && key > a.P + q)) p = 0.f;
      s1 += p;
      if (MODE == 0) s2 = fmaf(p, p, s2);
    }
    s1 = pair_sum(s1);
    if (MODE == 0) s2 = pair_sum(s2);
    if (g == 0 && key < Ltot) {
      if (MODE == 0 && a.mean_var) {
        const float mean = s1 * invS;
        a.o1[(int64_t)h * a.ldo1 + key] = mean;
        a.o2[(int64_t)h * a.ldo2 + key] = s2 * invS - mean * mean;
      } else {
        a.o1[(int64_t)h * a.ldo1 + key] = s1;
        if (MODE == 0) a.o2[(int64_t)h * a.ldo2 + key] = s2;
      }
    }
  }
}

template <int D, bool SHARED>
static void launch_scores_few_t(const ScoreArgs& a, dim3 grid, hipStream_t stream) {
  const dim3 block(256);
  if (a.mode == 0) hipLaunchKernelGGL((score_few_kernel<D, 0, SHARED>), grid, block, 0, stream, a);
  else if (a.noise != nullptr) hipLaunchKernelGGL((score_few_kernel<D, 1, SHARED>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((score_few_kernel<D, 2, SHARED>), grid, block, 0, stream, a);
}

// returns 1 when there are too many queries for this kernel
int launch_scores_few(const ScoreArgs& a, hipStream_t stream) {
  if (a.S < 1 || a.S > kFewMaxQueries || (a.D != 64 && a.D != 128)) return 1;
  const int Ltot = a.P + a.S;
  // grouped heads against a long prefix: four heads of a group per workgroup, K rows through LDS
  const int group = a.Hq / a.Hkv;
  const bool shared = group >= 4 && Ltot >= kSplitMinKeys;
  if (shared) {
    const dim3 grid((Ltot + kFewTile - 1) / kFewTile, a.Hkv * ((group + 3) / 4));
    if (a.D == 128) launch_scores_few_t<128, true>(a, grid, stream);
    else launch_scores_few_t<64, true>(a, grid, stream);
  } else {
    const dim3 grid((Ltot + kFewKeysPerWg - 1) / kFewKeysPerWg, a.Hq);
    if (a.D == 128) launch_scores_few_t<128, false>(a, grid, stream);
    else launch_scores_few_t<64, false>(a, grid, stream);
  }
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int64_t few_attn_workspace_bytes(int S, int Hq, int D, int Ltot) {
  if (S < 1 || S > kFewMaxQueries || (D != 64 && D != 128) || Ltot < 1) return 0;
  const int64_t nsplit = (Ltot + kFewKeysPerWg - 1) / kFewKeysPerWg;
  return (int64_t)Hq * nsplit * S * (D + 4) * 4;
}

template <int D, bool KF, bool FP8, bool FUSED = false, int NW = kFewWaves>
static int launch_few_t(const AttnArgs& a, hipStream_t stream) {
  constexpr int LDS = NW * kFewTile * D * 2 + NW * 32 * 4 * 4 + (FUSED ? 3 * 32 * D * 2 : 0);
  const int nsplit = (a.P + a.S + NW * kFewTile - 1) / (NW * kFewTile);
  constexpr auto kern = attn_few_kernel<D, KF, FP8, FUSED, NW>;
  if (set_max_lds<kern, LDS>() != 0) return -1;
  hipLaunchKernelGGL(kern, dim3(nsplit, a.Hq), dim3(NW * 64), LDS, stream, a);
  if (hipGetLastError() != hipSuccess) return -1;
  const int threads = a.Hq * a.S * (D / 4);
  hipLaunchKernelGGL(attn_few_combine_kernel<D>, dim3((threads + 255) / 256), dim3(256), 0, stream, a, nsplit);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_attention_few_combine(const AttnArgs& a, int nsplit, hipStream_t stream) {
  const int threads = a.Hq * a.S * (a.D / 4);
  if (a.D == 128) hipLaunchKernelGGL(attn_few_combine_kernel<128>, dim3((threads + 255) / 256), dim3(256), 0, stream, a, nsplit);
  else hipLaunchKernelGGL(attn_few_combine_kernel<64>, dim3((threads + 255) / 256), dim3(256), 0, stream, a, nsplit);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// returns 1 when the shape / workspace does not allow this path (the caller then uses the general kernel)
int launch_attention_few(const AttnArgs& a, hipStream_t stream) {
  const int Ltot = a.P + a.S;
  const int64_t need = few_attn_workspace_bytes(a.S, a.Hq, a.D, Ltot);
  if (need == 0 || a.ws == nullptr || a.ws_bytes < need) return 1;
  const bool kf = a.lse_pert != nullptr;
  if (a.k8 != nullptr) {  // fp8 caches: plain attention only
    if (kf || a.v8 == nullptr) return 1;
    return a.D == 128 ? launch_few_t<128, false, true>(a, stream) : launch_few_t<64, false, true>(a, stream);
  }
  if (a.pj != nullptr) {  // q and the new k / v rows are still partial sums of the projection
    if (a.pj_ksplit < 1 || a.k_w == nullptr || a.v_w == nullptr) return -1;
    if (a.D == 128)
      return kf ? launch_few_t<128, true, false, true>(a, stream) : launch_few_t<128, false, false, true>(a, stream);
    return kf ? launch_few_t<64, true, false, true>(a, stream) : launch_few_t<64, false, false, true>(a, stream);
  }
  if (a.D == 128)
    return kf ? launch_few_t<128, true, false>(a, stream) : launch_few_t<128, false, false>(a, stream);
  return kf ? launch_few_t<64, true, false>(a, stream) : launch_few_t<64, false, false>(a, stream);
}

}  // namespace tri
