/*
 * trinity_amd.h - C ABI of libtrinity_amd.so (gfx950 / MI355X).
 *
 * These entry points are what the `forward(...)` of a generated module binds
 * instead of launching Triton kernels.  Reference interface being replaced:
 * the per-kernel launches `kernel_i[grid](ptr, strides..., BLOCK_*, D, H, M, N, P)`
 * emitted by codegen/TritonGen.py:543-716 (instance:
 * evaluation/vanilla/vanilla_falcon_benchmark28173.py:151-209).
 *
 * Conventions (all entry points):
 *   - return TRI_OK (0) or a negative tri_status; every argument is checked
 *     before anything is launched, so a failed call enqueues nothing;
 *   - never allocate, never synchronise, never throw; kernels are enqueued on
 *     `hip_stream` (a hipStream_t, NULL = the default stream) and the call is
 *     legal under stream capture;
 *   - the caller owns every buffer including scratch (size queries below); the tensors of a call are distinct
 *     buffers - outputs, scratch and workspace overlap neither one another nor an input (the reference's callers
 *     allocate each tensor on its own, convert_eval_rms.py:141-176); the KV caches are the one in/out pair;
 *   - tensors are fp16 (the reference's type) unless stated, or bf16: a call is
 *     fp16 or bf16 throughout, decided by its first activation tensor, and every
 *     other 16-bit tensor of the call (weights, caches, noise, outputs) must
 *     have the same element type (TRI_ERR_DTYPE otherwise); accumulation,
 *     softmax statistics and score outputs are fp32 either way; the innermost
 *     dimension must be contiguous (stride 1) and every row start 16-byte
 *     aligned;
 *   - the weight matrices of tri_ffn_swiglu, tri_ffn_gelu, tri_gateup_swiglu, tri_matmul and of the three QKV
 *     entry points (w_q / w_k / w_v; tri_qkv_attention_static too) ([K, N], K = the contracted dimension) may
 *     instead be K-contiguous: stride[0] == 1 and stride[1] >= K, a multiple of 8 - the
 *     transpose view of a row-major [N, K] tensor, the layout torch.nn.Linear keeps its weight in (the reference
 *     passes every stride of every tensor to its kernels, codegen/TritonGen.py:656-669).  K must then be a
 *     multiple of 32 (TRI_ERR_UNSUPPORTED otherwise), w_gate and w_up must share one layout and so must w_q, w_k
 *     and w_v (TRI_ERR_STRIDE), and the product runs on the large-tile kernels whatever the row count (both
 *     operands then reach the matrix cores through plain LDS reads, about a tenth faster at many rows; with few
 *     rows the row-major layout - and for the FFN a workspace - is the fast path).  The weights of tri_ffn_block
 *     are row-major;
 *   - tri_rmsnorm and the FFN entry points accept an empty batch (0 rows; the
 *     pointer of a 0-row tensor may be NULL) and then launch nothing; an empty
 *     (0-byte) workspace counts as none;
 *   - each tri_validate_* takes the same arguments as its launcher, touches no
 *     GPU state and returns the status the launcher would return.
 */
#ifndef TRINITY_AMD_H
#define TRINITY_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 6: the seeded KeyFormer noise (noise == NULL) comes from seven generator rounds instead of ten: same
 * signatures, a different noise stream for a given seed.
 * 7: tri_diag_issue_probe added; nothing else changed.
 * 8: tri_diag_power_probe added; nothing else changed. */
#define TRI_ABI_VERSION 8

typedef enum tri_dtype {
  TRI_F16 = 0,
  TRI_BF16 = 1,
  TRI_F32 = 2,
  TRI_U8 = 3,
  TRI_FP8_E4M3 = 4 /* OCP e4m3 (no infinities, +-448 largest): KV caches only */
} tri_dtype;

typedef enum tri_status {
  TRI_OK = 0,
  TRI_ERR_NULL = -1,      /* required pointer is NULL */
  TRI_ERR_DTYPE = -2,     /* unsupported element type */
  TRI_ERR_SHAPE = -3,     /* dimensions inconsistent between arguments */
  TRI_ERR_STRIDE = -4,    /* innermost stride != 1, or a stride not a multiple of 8 elements */
  TRI_ERR_ALIGN = -5,     /* base pointer not 16-byte aligned */
  TRI_ERR_UNSUPPORTED = -6, /* legal but not implemented (e.g. head_dim not 64/128) */
  TRI_ERR_SCRATCH = -7,   /* scratch buffer too small */
  TRI_ERR_LAUNCH = -8     /* the HIP runtime refused a launch */
} tri_status;

typedef struct tri_tensor {
  void* ptr;
  int64_t shape[4];
  int64_t stride[4]; /* in elements */
  int32_t ndim;
  int32_t dtype; /* tri_dtype */
} tri_tensor;

/* Parameters of the QKV-projection + attention block.  The reference's point
 * (baseline/ref_rms.py:28-82, convert_eval_rms.py:32-59) is
 * {H, H, D, M, P, 1.0f, 0, 0.0f, prenorm?, qknorm?, 1.5f, 0};
 * the benchmark's point is {Hq, Hkv, D, S, 0, 1/sqrt(D), 1, 1e-5f, ., ., 1.0f, seed}. */
typedef struct tri_attn_params {
  int32_t n_q_heads;
  int32_t n_kv_heads;
  int32_t head_dim;   /* 64 or 128 */
  int32_t seq;        /* S: rows of X = new tokens; S * n_q_heads * head_dim < 2^30 elements (else TRI_ERR_UNSUPPORTED) */
  int32_t kv_prefix;  /* P: keys already in the caches */
  float scale;        /* multiplies q.k before the softmax; must be > 0 */
  int32_t causal;     /* key j visible to query i iff j <= P + i */
  float rms_eps;      /* eps of PreNorm and QKNorm */
  int32_t prenorm;    /* RMSNorm(X [, norm_w]) before the projections */
  int32_t qknorm;     /* per-head RMSNorm over head_dim of q and k */
  float tau;          /* KeyFormer temperature; must be > 0 */
  uint64_t noise_seed; /* KeyFormer: Philox4x32-7 key when no noise tensor is given */
  int32_t kv_fp8;     /* 1: k_cache / v_cache hold TRI_FP8_E4M3 values, cached value = scale * fp8 */
  float k_scale;      /* per-tensor scales of the fp8 caches; must be > 0 when kv_fp8 */
  float v_scale;
} tri_attn_params;

int tri_abi_version(void);
const char* tri_status_string(int status);

/* Optional set-up for the current HIP device: every kernel of the library that needs more than 64 KB of LDS is
 * given that attribute now (hipFuncSetAttribute) instead of on its first launch; nothing is launched or allocated.
 * A caller that captures its first call of an entry point into a HIP graph calls this once per device beforehand,
 * outside the capture (the reference warms its modules up before capturing, convert_eval_rms.py:253-263; with
 * this call the warm-up is not needed for the capture to be legal).  Idempotent and thread-safe.
 * Returns TRI_OK or TRI_ERR_LAUNCH. */
int tri_prepare(void);

/* Standalone RMSNorm: y[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) [* w].
 * Replaces evaluation/ffn/ffn_falcon/rms_ref.py:13-71 and ffn_benchmark7777.py:5-29
 * (oracle: baseline/ref_rms.py:101-102).  x, y [rows, n]; w [n] or NULL. */
int tri_rmsnorm(const tri_tensor* x, const tri_tensor* w, tri_tensor* y, float eps, void* hip_stream);
int tri_validate_rmsnorm(const tri_tensor* x, const tri_tensor* w, const tri_tensor* y, float eps);

/* SwiGLU FFN: out = (silu(x.w_gate) * (x.w_up)).w_down.  Replaces kernels
 * K7+K8 of evaluation/ffn/ffn_llama/ffn_llama_benchmark2248.py:80-185
 * (oracle: baseline/ffn_ref.py:37-50, w_gate = WFF1b, w_up = WFF1a, w_down = WFF2).
 * x [T, N]; w_gate, w_up [N, F]; w_down [F, N2]; hidden scratch [T, F]; out [T, N2]. */
int tri_ffn_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                   const tri_tensor* w_down, tri_tensor* hidden, tri_tensor* out,
                   tri_tensor* workspace /* nullable */, void* hip_stream);
int tri_validate_ffn_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                            const tri_tensor* w_down, const tri_tensor* hidden, const tri_tensor* out,
                            const tri_tensor* workspace);

/* Workspace of the few-row path.  With at most 64 rows (the reference's own
 * regime: M = 16 new tokens, convert_eval_rms.py:61-107; up to 128 rows when w
 * is at most 64 MB) a product x.w is bound
 * by streaming w from HBM once; the library then splits the K axis over many
 * workgroups, which needs room for fp32 partial sums.  Every FFN entry point
 * takes that room as `workspace`, a 1-D byte buffer (TRI_U8, 16-byte aligned)
 * or NULL; without it, or when it is too small, the large-tile kernels run
 * (same results to rounding, slower for few rows).  tri_gemm_workspace_bytes
 * sizes it for one product [M, K] x [K, ncols] (ncols = 2 F for the gate/up
 * pair); tri_ffn_workspace_bytes for a whole FFN (x [M, N], hidden width F,
 * including the N x N output projection of tri_ffn_block).  Both return 0 when
 * the shape never takes the few-row path.  The attention entry points carry
 * the same room inside their scratch buffer (tri_qkv_scratch_bytes), next to
 * the partial results of their key-split attention kernels (few new tokens,
 * or a chunk of tokens against thousands of cached keys). */
int64_t tri_gemm_workspace_bytes(int64_t m, int64_t k, int64_t ncols);
int64_t tri_ffn_workspace_bytes(int64_t m, int64_t n, int64_t f);

/* The two halves of tri_ffn_swiglu as separate launches, as the reference's generated module
 * launches them (kernel K7 "gate/up GEMM + SwiGLU", ffn_llama_benchmark2248.py:80-130, and K6/K8
 * "GEMM [+ residual]", :19-62 and :148-185):
 *   tri_gateup_swiglu: hidden = silu(rs * x.w_gate) * (rs * x.w_up), row_scale fp32 [T] or NULL;
 *   tri_matmul:        out = x.w [+ residual], residual [T, N2] or NULL. */
int tri_gateup_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                      const tri_tensor* row_scale, tri_tensor* hidden, tri_tensor* workspace /* nullable */,
                      void* hip_stream);
int tri_matmul(const tri_tensor* x, const tri_tensor* w, const tri_tensor* residual, tri_tensor* out,
               tri_tensor* workspace /* nullable */, void* hip_stream);

/* GELU(erf) FFN: out = gelu(x.w1).w2 (the Falcon-7B MLP of the benchmark
 * configuration; the reference has no counterpart).  Shapes as above. */
int tri_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2, tri_tensor* hidden,
                 tri_tensor* out, tri_tensor* workspace /* nullable */, void* hip_stream);
int tri_validate_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2,
                          const tri_tensor* hidden, const tri_tensor* out, const tri_tensor* workspace);

/* The reference-shaped FFN block (kernels K6-K9,
 * evaluation/ffn/ffn_llama/ffn_llama_benchmark2248.py:19-185,
 * evaluation/ffn/ffn_falcon/ffn_benchmark428.py:103-168; oracle baseline/ffn_ref.py:24-52, :114-121):
 *   attn_o2 = o2.wo + x ; norm = attn_o2 / sqrt(sum(attn_o2^2)/N) ;
 *   ff1 = (norm.wff1a) * silu(norm.wff1b) ; ff2 = ff1.wff2 ;
 *   o_ff_norm (optional, Falcon) = rmsnorm(ff2 + norm).
 * o2, x, attn_o2, ff2, o_ff_norm [M, N]; wo [N, N]; wff1a, wff1b [N, F]; wff2 [F, N];
 * ff1 [M, F]; row_scratch fp32 [M]. */
int tri_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x, const tri_tensor* wff1a,
                  const tri_tensor* wff1b, const tri_tensor* wff2, tri_tensor* attn_o2, tri_tensor* row_scratch,
                  tri_tensor* ff1, tri_tensor* ff2, tri_tensor* o_ff_norm /* nullable */,
                  tri_tensor* workspace /* nullable */, void* hip_stream);
int tri_validate_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x,
                           const tri_tensor* wff1a, const tri_tensor* wff1b, const tri_tensor* wff2,
                           const tri_tensor* attn_o2, const tri_tensor* row_scratch, const tri_tensor* ff1,
                           const tri_tensor* ff2, const tri_tensor* o_ff_norm, const tri_tensor* workspace);

/* Bytes of scratch tri_qkv_attention / tri_keyformer / tri_roco need for the
 * given parameters (n_model = columns of X).  Negative = tri_status.  The
 * attention entry points want at least one new token: p->seq < 1 is
 * TRI_ERR_SHAPE here and there. */
int64_t tri_qkv_scratch_bytes(const tri_attn_params* p, int64_t n_model);

/* Fused QKV projection + KV-cache append + softmax attention: Vanilla,
 * PreNorm (p->prenorm), QKNorm (p->qknorm) and their combination.  Replaces
 * kernel_0/kernel_1 of evaluation/vanilla/vanilla_falcon_benchmark28173.py:19-144,
 * evaluation/prenorm/prenorm_falcon_benchmark579.py:19-120,
 * evaluation/qknorm/qknorm_falcon_benchmark40460.py:19-143
 * (oracles: baseline/ref_rms.py:28-126, :221-314).
 *   x [S, N]; norm_w [N] or NULL; wq [N, Hq*D]; wk, wv [N, Hkv*D];
 *   k_cache, v_cache [Hkv, >= P+S, D] in/out, both NULL only when P == 0
 *   (rows [P, P+S) are written; under QKNorm the normalised k is written).
 *   With p->kv_fp8 the caches are TRI_FP8_E4M3 (required, also when P == 0), rows of a
 *   multiple of 16 bytes: the new rows are appended as fp8(k / k_scale), fp8(v / v_scale)
 *   (round to nearest even, saturating at +-448) and attention then reads every key,
 *   cached or new, from the fp8 rows - with at most 32 new tokens straight from the cache
 *   (half the bytes of a 16-bit cache), otherwise through a 16-bit copy in the scratch
 *   buffer; the scales are applied in fp32 (k_scale with the softmax scale, v_scale with
 *   the final normalisation).  No counterpart in the reference, whose caches are fp16;
 *   scratch: 1-D byte buffer (tri_qkv_scratch_bytes), 256-byte aligned; lse fp32 [Hq, S] or NULL;
 *   out [S, Hq*D]. */
int tri_qkv_attention(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                      const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch,
                      tri_tensor* lse, tri_tensor* out, const tri_attn_params* p, void* hip_stream);
int tri_validate_qkv_attention(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                               const tri_tensor* wk, const tri_tensor* wv, const tri_tensor* k_cache,
                               const tri_tensor* v_cache, const tri_tensor* scratch, const tri_tensor* lse,
                               const tri_tensor* out, const tri_attn_params* p);

/* tri_qkv_attention for callers that cannot provide scratch memory because they cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its
 * callers allocate every buffer, convert_eval_rms.py:141-176).  Same arguments and results as tri_qkv_attention
 * without `scratch`: the library keeps that memory itself, TRI_STATIC_SCRATCH_BYTES of device memory per GPU,
 * held from the moment the library is loaded on that GPU until the process ends.  A call whose
 * tri_qkv_scratch_bytes exceeds it returns TRI_ERR_SCRATCH and launches nothing (64 MiB hold e.g. the Llama-3-8B
 * block up to 4096 new tokens and every reference-shaped call).  The call allocates nothing; its first use on a
 * device looks the array's address up (tri_prepare does the same ahead of time).  All calls on one GPU share
 * the one array: calls that may overlap in time (different streams, different threads) race - serialise them. */
#define TRI_STATIC_SCRATCH_BYTES (64 * 1024 * 1024)
int tri_qkv_attention_static(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                             const tri_tensor* wk, const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache,
                             tri_tensor* lse, tri_tensor* out, const tri_attn_params* p, void* hip_stream);

/* KeyFormer: the block above plus score[h, j] = sum_i softmax_j((scale*q_i.k_j + g[h,i,j]) / tau).
 * Replaces evaluation/keyformer/keyformer_falcon_benchmark4358.py:19-147 (oracle lines
 * baseline/ref_rms.py:163-166).  noise fp16 [Hq, S, P+S] or NULL (then Gumbel noise is
 * generated in-kernel from p->noise_seed: Philox4x32 at seven rounds, key = the seed and counter
 * (2 * (k / 16) + (k / 4) % 2, query, head, 0); key k takes word k % 4 of the output, its low
 * sixteen bits if (k / 8) % 2 == 0, else its high sixteen; u = (bits + 0.5) * 2^-16,
 * g = -ln(-ln u)); score fp32 [Hq, P+S]. */
int tri_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                  const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch,
                  const tri_tensor* noise, tri_tensor* out, tri_tensor* score, const tri_attn_params* p,
                  void* hip_stream);
int tri_validate_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                           const tri_tensor* wk, const tri_tensor* wv, const tri_tensor* k_cache,
                           const tri_tensor* v_cache, const tri_tensor* scratch, const tri_tensor* noise,
                           const tri_tensor* out, const tri_tensor* score, const tri_attn_params* p);

/* RoCo: the block above plus s1[h, j] = sum_i p[h,i,j], s2[h, j] = sum_i p[h,i,j]^2
 * (as_mean_var != 0: s1/S and s2/S - (s1/S)^2).  Replaces
 * evaluation/roco/roco_falcon_benchmark2470.py:19-139 (oracle lines baseline/ref_rms.py:349-352).
 * sum_out, sumsq_out fp32 [Hq, P+S]. */
int tri_roco(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
             const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch, tri_tensor* out,
             tri_tensor* sum_out, tri_tensor* sumsq_out, int32_t as_mean_var, const tri_attn_params* p,
             void* hip_stream);
int tri_validate_roco(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                      const tri_tensor* wv, const tri_tensor* k_cache, const tri_tensor* v_cache,
                      const tri_tensor* scratch, const tri_tensor* out, const tri_tensor* sum_out,
                      const tri_tensor* sumsq_out, int32_t as_mean_var, const tri_attn_params* p);

/* Issue probe (measurement only; no counterpart in the reference).  Launches `workgroups` workgroups of
 * 4 * waves_per_simd waves, one workgroup per CU, every wave looping `iters` times (a multiple of 8) over a group
 * of one v_mfma_f32_32x32x16_f16 (with_mfma != 0), n_valu independent v_fma_f32 (0, 2, 4, 6, 8, 12 or 16) and
 * n_trans v_exp_f32 (0, 1, 2 or 4), a scheduling fence between groups.  Each workgroup writes two int64 to
 * `ticks` (TRI_U8, 1-D, at least 16 * workgroups + 16 bytes, 16-byte aligned): s_memtime ticks and 100 MHz ticks
 * from the start of its loops to the end of its last wave's.  The softmax kernels are bound by this instruction
 * mix; bench.py --microbench prints what a group costs.  waves_per_simd 1 to 4; counts outside the lists return
 * TRI_ERR_UNSUPPORTED. */
int tri_diag_issue_probe(int32_t with_mfma, int32_t n_valu, int32_t n_trans, int32_t waves_per_simd, int32_t iters,
                         int32_t workgroups, tri_tensor* ticks, void* hip_stream);

/* Power probe (measurement only; no counterpart in the reference).  `workgroups` workgroups of eight waves (two per
 * SIMD, one workgroup per CU), every wave looping `iters` times (a multiple of 8, at most 2^22) over a group of one
 * v_mfma_f32_32x32x16_f16 on random fp16 operands (random_operands != 0) or zeros, and beside it
 * lds_reads_per_two_groups (0, 1, 2 or 4) ds_read_b128 per two groups, dma_loads_per_eight_groups (0, 2 or 4)
 * global -> LDS loads of 16 bytes per lane per eight groups (from half a megabyte that stays in the L2), and per
 * group (n_valu v_fma_f32, n_trans v_exp_f32) = (0, 0), (4, 0), (4, 1) or (3, 1).  `ticks` as for
 * tri_diag_issue_probe.  Long loops on random operands run at the board's power limit, where a kernel's time is
 * the energy it draws: the time per group, less that of the MFMA alone, is what the added instructions cost
 * there; on zeros the same streams run at the full clock.  bench.py --microbench prints both.  Counts outside the
 * lists return TRI_ERR_UNSUPPORTED. */
int tri_diag_power_probe(int32_t lds_reads_per_two_groups, int32_t dma_loads_per_eight_groups, int32_t n_valu,
                         int32_t n_trans, int32_t random_operands, int32_t iters, int32_t workgroups,
                         tri_tensor* ticks, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* TRINITY_AMD_H */
