// Internal launcher prototypes (host side).  Every launcher enqueues on
// `stream`, allocates nothing, and returns 0 or -1 (the runtime refused).
#if (defined(TRI_BF16) && !defined(TRI_LAUNCH_H_BF16)) || (!defined(TRI_BF16) && !defined(TRI_LAUNCH_H_F16))
#ifdef TRI_BF16
#define TRI_LAUNCH_H_BF16
#else
#define TRI_LAUNCH_H_F16
#endif
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "common.h"

#ifndef TRI_LDS_ATTR_REGISTRY
#define TRI_LDS_ATTR_REGISTRY
// One node per kernel that needs the large-LDS attribute (see LdsAttr below); shared by the fp16 and bf16 copies of
// the kernels, defined in abi.hip.
struct TriLdsAttr;
__attribute__((visibility("hidden"))) void tri_lds_attr_register(TriLdsAttr* node);
__attribute__((visibility("hidden"))) int tri_lds_attr_apply(TriLdsAttr* node);  // current device; 0 or -1
struct TriLdsAttr {
  const void* kern;
  int bytes;
  std::atomic<uint64_t> done{0};
  TriLdsAttr* next = nullptr;
  TriLdsAttr(const void* k, int b) : kern(k), bytes(b) { tri_lds_attr_register(this); }
};
#endif

namespace tri {

// A kernel that wants more than 64 KB of dynamic LDS has to be told so once per device before its first launch.
// Every such kernel owns one TriLdsAttr (a static member of LdsAttr<kernel, bytes>, constructed when the library
// is loaded), which links itself into a list: tri_prepare() walks the list and sets the attribute of every kernel
// for the current device, and a launcher whose kernel has not been prepared on its device does so itself on the
// first call.  Bit d of `done` is set once device d has the attribute; threads racing on the first call repeat
// the same idempotent runtime call.
template <auto Kern, int Bytes>
struct LdsAttr {
  static TriLdsAttr once;
};
template <auto Kern, int Bytes>
TriLdsAttr LdsAttr<Kern, Bytes>::once(reinterpret_cast<const void*>(Kern), Bytes);

template <auto Kern, int Bytes>
inline int set_max_lds() {
  return tri_lds_attr_apply(&LdsAttr<Kern, Bytes>::once);
}

int launch_rmsnorm(const half_t* x, int64_t ldx, const half_t* w, half_t* y, int64_t ldy, float* rstd_out, int rows,
                   int n, float eps, hipStream_t stream);

int launch_add_scaled_rmsnorm(const half_t* a, int64_t lda, const half_t* b, int64_t ldb, const float* bscale,
                              half_t* y, int64_t ldy, int rows, int n, hipStream_t stream);

enum GemmEpi { EPI_NONE = 0, EPI_GELU = 1, EPI_SWIGLU = 2 };

// out[M, N] = act(rowscale[m] * (X[M,K] . W[K,N])) + residual[M,N]
// EPI_SWIGLU: out[M, N] = silu(X.W) * (X.W2), W and W2 both [K, N].
struct GemmArgs {
  const half_t* x;
  int64_t ldx;
  const half_t* w;
  int64_t ldw;
  const half_t* w2;
  int64_t ldw2;
  // weights stored K-contiguous (W^T [N][K]): ldw / ldw2 are then the strides between weight columns.  Needs
  // K % 32 == 0; takes the large-tile kernels whatever M (the few-row and split-K paths read row-major weights).
  int w_kcontig;
  const float* rowscale;   // nullable, [M]
  const half_t* residual;  // nullable
  int64_t ldr;
  half_t* out;
  int64_t ldo;
  int M, N, K;
  int epi;
  int n_big, big_cols;  // tile plan (filled in by launch_gemm): workgroups and columns covered by big tiles
  float* ws;            // nullable: fp32 workspace for the split-K path taken when M <= kSkinnyMaxRows
  int64_t ws_bytes;
  // Few-row path only (set when skinny_gemm_applies(args)): the merge kernel computes the row scale itself,
  // rowscale[m] = rsqrt(mean(rownorm_src[m, 0..rownorm_n)^2)), and also stores it to rownorm_out[m] - the
  // RMSNorm statistic of the FFN block without a kernel of its own.
  const half_t* rownorm_src;
  int64_t rownorm_ld;
  int rownorm_n;
  float* rownorm_out;
};
int launch_gemm(const GemmArgs& a, hipStream_t stream);

// Few-row GEMMs (M <= kSkinnyMaxRows) are bound by streaming the weights once from HBM.  They run as a
// split-K kernel (many workgroups, each a [k range] x [128 columns] slab, fp32 partial sums into the
// workspace) followed by a finalize kernel that adds the partials and applies the epilogue.
constexpr int kSkinnyMaxRows = 64;
// ... and more rows when the weights are small enough to stay in the 256 MB Infinity Cache while the workgroups of
// the different 64-row blocks stream them (each block reads every slab again): up to 128 rows for plain products
// (beyond that the large tiles' split-K plan is ahead: 4544 x 4544 at 256 rows 34.5 against 45.9 us), up to 256 for
// the Q/K/V projection, which has no such plan (Llama-3-8B heads, 50 MB of weights: 128 rows 59.3 -> 35.9 us, 256
// rows 65.3 -> 54.3 us; with 100 MB of weights the gain is gone at 256 rows, hence the limit on the bytes)
constexpr int kSkinnyWideMaxRows = 128, kSkinnyWideMaxRowsQkv = 256;
constexpr int64_t kSkinnyWideMaxBytes = (int64_t)64 << 20;
// bytes of workspace that guarantee the split-K path for an [M, K] x [K, ncols] product (ncols counts gate and
// up columns separately for SwiGLU); 0 when the shape never takes that path
int64_t skinny_workspace_bytes(int M, int K, int ncols, bool qkv = false);  // qkv: the Q/K/V projection's row limit
int launch_skinny_gemm(const GemmArgs& a, hipStream_t stream);
bool skinny_gemm_applies(const GemmArgs& a);  // launch_gemm(a) will take the few-row path
// Many rows, but a tile count that fills the chip badly and a deep K: split-K over half-size tiles with the
// same workspace and finalize kernels (plain and GELU epilogues).  0 bytes = never taken for this shape.
int64_t large_split_workspace_bytes(int M, int K, int N);
int launch_gemm_splitk(const GemmArgs& a, int s, hipStream_t stream);  // s parts per 256 x 128 tile

// [Q | K | V] = X . [Wq | Wk | Wv], optional per-head RMSNorm of Q and K,
// scattered to q [S, Hq*D] and the head-major k/v buffers.
struct QkvProjArgs {
  const half_t* x;
  int64_t ldx;
  const half_t *wq, *wk, *wv;
  int64_t ldwq, ldwk, ldwv;
  half_t* q;  // [S, Hq*D]
  int64_t ldq;
  half_t *k, *v;            // element (h, row, d) at h*stride_h + row*stride_r + d
  int64_t k_sh, k_sr, v_sh, v_sr;
  int S, K, Hq, Hkv, D, P;
  int qknorm;
  float eps;
  float* ws;  // nullable: split-K workspace (see skinny_workspace_bytes), used when S <= kSkinnyMaxRows
  int64_t ws_bytes;
  int n_big, big_cols;  // tile plan (filled in by launch_qkv_proj)
  int w_kcontig;        // the three weight matrices are K-contiguous (ldwq / ldwk / ldwv: strides between columns)
};
// deferred_ksplit (nullable): when given and the few-row path runs, its merge kernel is left out - q, k and v stay
// fp32 partial results ws [ksplit][S][(Hq + 2 Hkv) * D] for the attention kernel to merge - and the number of
// splits is stored there; 0 is stored when the projection finished the job itself.
int launch_skinny_qkv(const QkvProjArgs& a, hipStream_t stream, int* deferred_ksplit = nullptr);
int launch_qkv_proj(const QkvProjArgs& a, hipStream_t stream, int* deferred_ksplit = nullptr);

struct AttnArgs {
  const half_t* q;  // [S, Hq*D]
  int64_t ldq;
  const half_t *k, *v;  // head-major, rows [0, P+S)
  int64_t k_sh, k_sr, v_sh, v_sr;
  half_t* out;  // [S, Hq*D]
  int64_t ldo;
  float* lse;       // nullable [Hq, S], natural log
  float* lse_pert;  // nullable [Hq, S]: logsumexp of the perturbed logits (KeyFormer)
  const half_t* noise;  // nullable [Hq, S, P+S]
  int S, P, Hq, Hkv, D;
  float scale, tau;
  int causal;
  uint64_t seed;
  float* ws;  // nullable: workspace of the few-query path (few_attn_workspace_bytes)
  int64_t ws_bytes;
  float out_scale;  // multiplies the normalised output (v_scale of an fp8 cache; 1 otherwise)
  // fp8 (e4m3) caches read directly - few-query path only; k / v are then unused.  Strides in elements = bytes.
  const uint8_t *k8, *v8;
  int64_t k8_sh, k8_sr, v8_sh, v8_sr;
  // Few-query path fused with the merge of a split-K projection (pj != nullptr; launch_attention_few only): q and
  // the S new rows of k / v are not read from memory but summed from the projection's partial results
  // pj [pj_ksplit][S][pj_ntot] (columns [q heads | k heads | v heads]), rounded, RMS-normalised per head when
  // qknorm (q and k), and stored to q_w and to rows [P, P+S) of k_w / v_w (the buffers k / v point to) on the way.
  int split_tiles;  // set by launch_attention for its long-prefix variant: key tiles (64 keys) per workgroup
  const float* pj;
  int pj_ksplit, pj_ntot, qknorm;
  float eps;
  half_t *q_w, *k_w, *v_w;
};
int launch_attention(const AttnArgs& a, hipStream_t stream);

// With at most kFewMaxQueries queries attention is bound by reading the K/V cache once; it then runs split
// over the key axis (partial results in the workspace) followed by a merge kernel.
constexpr int kFewMaxQueries = 32;
int64_t few_attn_workspace_bytes(int S, int Hq, int D, int Ltot);
int launch_attention_few(const AttnArgs& a, hipStream_t stream);
int launch_attention_few_combine(const AttnArgs& a, int nsplit, hipStream_t stream);  // the merge kernel alone
// workspace of launch_attention's long-prefix variant for a call (0 when it does not take it)
int64_t split_attn_workspace_bytes(int S, int Hq, int Hkv, int D, int Ltot);
// From this many keys on, plain attention for few new tokens leaves the one-tile-per-wave kernel for one that
// loops over its keys with the query heads of a KV head stacked along the query axis (launch_attention decides).
// 16 tokens: at 1040 keys the two are level, at 2064 keys the looping kernel is 2-5 us ahead, at 32784 keys
// 2.3x (8 KV heads, head dimension 128) to 3x (1 KV head, 64) on the whole block.
constexpr int kSplitMinKeys = 2048;

// fp8 (OCP e4m3) KV caches, value = scale * fp8: append of the new rows, and 16-bit copies (without the scale)
// for the kernels that read 16-bit K / V tiles.
struct KvQuantArgs {
  const half_t *k, *v;  // new rows [Hkv][S][D] as written by the projection
  int64_t k_sh, k_sr, v_sh, v_sr;
  uint8_t *kc, *vc;  // caches; rows [P, P+S) are written
  int64_t kc_sh, kc_sr, vc_sh, vc_sr;
  int S, P, Hkv, D;
  float k_scale, v_scale;
};
int launch_kv_quant_append(const KvQuantArgs& a, hipStream_t stream);
struct KvDequantArgs {
  const uint8_t *kc, *vc;
  int64_t kc_sh, kc_sr, vc_sh, vc_sr;
  half_t *k, *v;  // [Hkv][rows][D] contiguous
  int rows, Hkv, D;
};
int launch_kv_dequant(const KvDequantArgs& a, hipStream_t stream);

// Per-key accumulators over queries.  mode 0: RoCo (o1 = sum p, o2 = sum p^2,
// or mean / variance when mean_var); mode 1: KeyFormer (o1 = sum p_perturbed).
struct ScoreArgs {
  const half_t* q;
  int64_t ldq;
  const half_t* k;
  int64_t k_sh, k_sr;
  const float* lse;  // [Hq, S]: plain (mode 0) or perturbed (mode 1)
  const half_t* noise;
  float *o1, *o2;  // [Hq, P+S]
  int64_t ldo1, ldo2;
  int S, P, Hq, Hkv, D;
  float scale, tau;
  int causal, mode, mean_var;
  uint64_t seed;
};
int launch_scores(const ScoreArgs& a, hipStream_t stream);
int launch_scores_few(const ScoreArgs& a, hipStream_t stream);  // S <= kFewMaxQueries; 1 = not applicable

}  // namespace tri

#endif  // once per element type
