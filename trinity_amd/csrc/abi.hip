// C ABI of libtrinity_amd.so: argument validation (pure host code, usable
// without a GPU) and the launch sequences behind each entry point.
#include "../../include/trinity_amd.h"

#include "launch.h"

using namespace tri;

namespace {

struct Scratch {
  int64_t q_off, k_off, v_off, xn_off, lse_off, lsep_off, ws_off, ws_bytes, total;
};

inline int64_t align256(int64_t x) { return (x + 255) & ~(int64_t)255; }

Scratch scratch_layout(const tri_attn_params* p, int64_t n_model) {
  Scratch s{};
  const int64_t S = p->seq, Hq = p->n_q_heads, Hkv = p->n_kv_heads, D = p->head_dim;
  int64_t off = 0;
  s.q_off = off; off = align256(off + S * Hq * D * 2);
  s.k_off = off; off = align256(off + Hkv * S * D * 2);
  s.v_off = off; off = align256(off + Hkv * S * D * 2);
  s.xn_off = off; off = align256(off + (p->prenorm ? S * n_model * 2 : 0));
  s.lse_off = off; off = align256(off + Hq * S * 4);
  s.lsep_off = off; off = align256(off + Hq * S * 4);
  // few new tokens: room for the split-K partial sums of the projection, reused afterwards for the partial
  // results of the key-split attention
  s.ws_bytes = skinny_workspace_bytes((int)S, (int)n_model, (int)((Hq + 2 * Hkv) * D));
  const int64_t few = few_attn_workspace_bytes((int)S, (int)Hq, (int)D, (int)(p->kv_prefix + S));
  s.ws_bytes = s.ws_bytes > few ? s.ws_bytes : few;
  s.ws_off = off; off = align256(off + s.ws_bytes);
  s.total = off;
  return s;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// fp16 matrix [rows, cols] with unit inner stride and 16-byte aligned rows
int check_mat(const tri_tensor* t, int64_t rows, int64_t cols, int dtype = TRI_F16) {
  if (t == nullptr) return TRI_ERR_NULL;
  // an empty batch (no rows) is legal and carries no storage; the entry points then launch nothing
  if (t->ptr == nullptr && !(t->ndim == 2 && t->shape[0] == 0)) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (t->ndim != 2) return TRI_ERR_SHAPE;
  if (rows >= 0 && t->shape[0] != rows) return TRI_ERR_SHAPE;
  if (cols >= 0 && t->shape[1] != cols) return TRI_ERR_SHAPE;
  if (t->shape[0] < 0 || t->shape[1] < 0) return TRI_ERR_SHAPE;
  if (t->stride[1] != 1) return TRI_ERR_STRIDE;
  if (t->shape[0] > 1 && t->stride[0] < t->shape[1]) return TRI_ERR_STRIDE;
  if (dtype == TRI_F16) {
    if (t->stride[0] % 8 != 0 || t->shape[1] % 8 != 0) return TRI_ERR_STRIDE;
    if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  }
  return TRI_OK;
}

int check_vec(const tri_tensor* t, int64_t n, int dtype) {
  if (t == nullptr || t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (t->ndim != 1 || t->shape[0] != n) return TRI_ERR_SHAPE;
  if (n > 1 && t->stride[0] != 1) return TRI_ERR_STRIDE;
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

// head-major [H, rows >= min_rows, D] fp16 with contiguous d
int check_cache(const tri_tensor* t, int64_t H, int64_t min_rows, int64_t D) {
  if (t == nullptr || t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != TRI_F16) return TRI_ERR_DTYPE;
  if (t->ndim != 3 || t->shape[0] != H || t->shape[1] < min_rows || t->shape[2] != D) return TRI_ERR_SHAPE;
  if (t->stride[2] != 1 || t->stride[1] % 8 != 0 || t->stride[0] % 8 != 0 || t->stride[1] < D) return TRI_ERR_STRIDE;
  if (t->shape[1] * t->stride[1] * 2 >= ((int64_t)1 << 31)) return TRI_ERR_UNSUPPORTED;  // per-head extent fits a buffer descriptor
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

// optional split-K workspace: 1-D bytes
int check_ws(const tri_tensor* t) {
  if (t == nullptr) return TRI_OK;
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != TRI_U8) return TRI_ERR_DTYPE;
  if (t->ndim != 1 || t->shape[0] < 0) return TRI_ERR_SHAPE;
  if (t->shape[0] > 1 && t->stride[0] != 1) return TRI_ERR_STRIDE;
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

inline void set_ws(GemmArgs& g, const tri_tensor* ws) {
  g.ws = ws != nullptr ? static_cast<float*>(ws->ptr) : nullptr;
  g.ws_bytes = ws != nullptr ? ws->shape[0] : 0;
}

#define TRI_TRY(expr)            \
  do {                           \
    const int st__ = (expr);     \
    if (st__ != TRI_OK) return st__; \
  } while (0)

inline const half_t* H(const tri_tensor* t) { return t != nullptr ? static_cast<const half_t*>(t->ptr) : nullptr; }
inline half_t* HM(tri_tensor* t) { return t != nullptr ? static_cast<half_t*>(t->ptr) : nullptr; }

int validate_rmsnorm(const tri_tensor* x, const tri_tensor* w, const tri_tensor* y) {
  if (x == nullptr || y == nullptr) return TRI_ERR_NULL;
  if (x->dtype != TRI_F16 || y->dtype != TRI_F16) return TRI_ERR_DTYPE;
  if (x->ndim != 2 || y->ndim != 2) return TRI_ERR_SHAPE;
  if ((x->ptr == nullptr || y->ptr == nullptr) && x->shape[0] != 0) return TRI_ERR_NULL;  // no rows: no storage
  if (x->shape[0] != y->shape[0] || x->shape[1] != y->shape[1]) return TRI_ERR_SHAPE;
  if (x->stride[1] != 1 || y->stride[1] != 1) return TRI_ERR_STRIDE;
  if (x->shape[0] > 1 && (x->stride[0] < x->shape[1] || y->stride[0] < y->shape[1])) return TRI_ERR_STRIDE;
  if (w != nullptr) {
    if (w->ptr == nullptr) return TRI_ERR_NULL;
    if (w->dtype != TRI_F16) return TRI_ERR_DTYPE;
    if (w->ndim != 1 || w->shape[0] != x->shape[1]) return TRI_ERR_SHAPE;
    if (w->shape[0] > 1 && w->stride[0] != 1) return TRI_ERR_STRIDE;
  }
  return TRI_OK;
}

int validate_ffn2(const tri_tensor* x, const tri_tensor* wa, const tri_tensor* wb, const tri_tensor* wd,
                  const tri_tensor* hidden, const tri_tensor* out) {
  if (x == nullptr || wa == nullptr || wd == nullptr || hidden == nullptr || out == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_mat(x, -1, -1));
  const int64_t T = x->shape[0], N = x->shape[1];
  TRI_TRY(check_mat(wa, N, -1));
  const int64_t F = wa->shape[1];
  if (wb != nullptr) TRI_TRY(check_mat(wb, N, F));
  TRI_TRY(check_mat(wd, F, -1));
  TRI_TRY(check_mat(hidden, T, F));
  TRI_TRY(check_mat(out, T, wd->shape[1]));
  return TRI_OK;
}

int validate_qkv_common(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                        const tri_tensor* wv, const tri_tensor* k_cache, const tri_tensor* v_cache,
                        const tri_tensor* scratch, const tri_tensor* out, const tri_attn_params* p) {
  if (p == nullptr) return TRI_ERR_NULL;
  if (p->head_dim != 64 && p->head_dim != 128) return TRI_ERR_UNSUPPORTED;
  if (p->n_q_heads <= 0 || p->n_kv_heads <= 0 || p->n_q_heads % p->n_kv_heads != 0) return TRI_ERR_SHAPE;
  if (p->seq <= 0 || p->kv_prefix < 0) return TRI_ERR_SHAPE;
  if (!(p->tau > 0.f) || !(p->scale > 0.f)) return TRI_ERR_UNSUPPORTED;
  const int64_t S = p->seq, D = p->head_dim, Hq = p->n_q_heads, Hkv = p->n_kv_heads, P = p->kv_prefix;
  TRI_TRY(check_mat(x, S, -1));
  const int64_t N = x->shape[1];
  if (norm_w != nullptr) {
    if (!p->prenorm) return TRI_ERR_SHAPE;
    TRI_TRY(check_vec(norm_w, N, TRI_F16));
  }
  TRI_TRY(check_mat(wq, N, Hq * D));
  TRI_TRY(check_mat(wk, N, Hkv * D));
  TRI_TRY(check_mat(wv, N, Hkv * D));
  if ((k_cache == nullptr) != (v_cache == nullptr)) return TRI_ERR_NULL;
  if (k_cache == nullptr && P > 0) return TRI_ERR_NULL;
  if (k_cache != nullptr) {
    TRI_TRY(check_cache(k_cache, Hkv, P + S, D));
    TRI_TRY(check_cache(v_cache, Hkv, P + S, D));
  }
  if (scratch == nullptr || scratch->ptr == nullptr) return TRI_ERR_NULL;
  if (scratch->ndim != 1 || (scratch->shape[0] > 1 && scratch->stride[0] != 1)) return TRI_ERR_STRIDE;
  {
    const int64_t esz = (scratch->dtype == TRI_U8) ? 1 : (scratch->dtype == TRI_F32 ? 4 : 2);
    if (scratch->shape[0] * esz < scratch_layout(p, N).total) return TRI_ERR_SCRATCH;
    if (((uintptr_t)scratch->ptr & 255u) != 0) return TRI_ERR_ALIGN;
  }
  TRI_TRY(check_mat(out, S, Hq * D));
  return TRI_OK;
}

int check_f32_mat(const tri_tensor* t, int64_t rows, int64_t cols) {
  if (t == nullptr || t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != TRI_F32) return TRI_ERR_DTYPE;
  if (t->ndim != 2 || t->shape[0] != rows || t->shape[1] != cols) return TRI_ERR_SHAPE;
  if (t->stride[1] != 1 || (rows > 1 && t->stride[0] < cols)) return TRI_ERR_STRIDE;
  return TRI_OK;
}

int check_noise(const tri_tensor* t, int64_t Hq, int64_t S, int64_t L) {
  if (t == nullptr) return TRI_OK;
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != TRI_F16) return TRI_ERR_DTYPE;
  if (t->ndim != 3 || t->shape[0] != Hq || t->shape[1] != S || t->shape[2] != L) return TRI_ERR_SHAPE;
  if (t->stride[2] != 1 || t->stride[1] != L || t->stride[0] != S * L) return TRI_ERR_STRIDE;
  return TRI_OK;
}

// projection + attention shared by the three QKV entry points
struct QkvPlan {
  const half_t* q;
  const half_t *k, *v;
  int64_t k_sh, k_sr, v_sh, v_sr;
  float *lse, *lse_pert;
};

int run_qkv(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
            const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch, float* lse_user,
            tri_tensor* out, const tri_attn_params* p, bool need_lse, bool keyformer, const half_t* noise,
            hipStream_t stream, QkvPlan* plan) {
  const int S = p->seq, D = p->head_dim, Hq = p->n_q_heads, Hkv = p->n_kv_heads, P = p->kv_prefix;
  const int N = (int)x->shape[1];
  const Scratch sl = scratch_layout(p, N);
  char* sb = static_cast<char*>(scratch->ptr);
  half_t* q = reinterpret_cast<half_t*>(sb + sl.q_off);

  QkvProjArgs pa{};
  pa.x = H(x); pa.ldx = x->stride[0];
  if (p->prenorm) {
    // PreNorm: the normalised activations are materialised once (fp16, as the
    // reference's X_norm) and the projection reads them.
    half_t* xn = reinterpret_cast<half_t*>(sb + sl.xn_off);
    if (launch_rmsnorm(H(x), x->stride[0], H(norm_w), xn, N, nullptr, S, N, p->rms_eps, stream) != 0)
      return TRI_ERR_LAUNCH;
    pa.x = xn; pa.ldx = N;
  }
  pa.wq = H(wq); pa.wk = H(wk); pa.wv = H(wv);
  pa.ldwq = wq->stride[0]; pa.ldwk = wk->stride[0]; pa.ldwv = wv->stride[0];
  pa.q = q; pa.ldq = (int64_t)Hq * D;
  if (k_cache != nullptr) {
    pa.k = HM(k_cache); pa.k_sh = k_cache->stride[0]; pa.k_sr = k_cache->stride[1];
    pa.v = HM(v_cache); pa.v_sh = v_cache->stride[0]; pa.v_sr = v_cache->stride[1];
  } else {
    pa.k = reinterpret_cast<half_t*>(sb + sl.k_off); pa.k_sh = (int64_t)S * D; pa.k_sr = D;
    pa.v = reinterpret_cast<half_t*>(sb + sl.v_off); pa.v_sh = (int64_t)S * D; pa.v_sr = D;
  }
  pa.S = S; pa.K = N; pa.Hq = Hq; pa.Hkv = Hkv; pa.D = D; pa.P = P;
  pa.qknorm = p->qknorm; pa.eps = p->rms_eps;
  pa.ws = sl.ws_bytes > 0 ? reinterpret_cast<float*>(sb + sl.ws_off) : nullptr;
  pa.ws_bytes = sl.ws_bytes;
  if (launch_qkv_proj(pa, stream) != 0) return TRI_ERR_LAUNCH;

  AttnArgs aa{};
  aa.q = q; aa.ldq = pa.ldq;
  aa.k = pa.k; aa.v = pa.v; aa.k_sh = pa.k_sh; aa.k_sr = pa.k_sr; aa.v_sh = pa.v_sh; aa.v_sr = pa.v_sr;
  aa.out = HM(out); aa.ldo = out->stride[0];
  aa.lse = lse_user != nullptr ? lse_user : (need_lse ? reinterpret_cast<float*>(sb + sl.lse_off) : nullptr);
  aa.lse_pert = keyformer ? reinterpret_cast<float*>(sb + sl.lsep_off) : nullptr;
  aa.noise = noise;
  aa.S = S; aa.P = P; aa.Hq = Hq; aa.Hkv = Hkv; aa.D = D;
  aa.scale = p->scale; aa.tau = p->tau; aa.causal = p->causal; aa.seed = p->noise_seed;
  aa.ws = sl.ws_bytes > 0 ? reinterpret_cast<float*>(sb + sl.ws_off) : nullptr;
  aa.ws_bytes = sl.ws_bytes;
  if (launch_attention(aa, stream) != 0) return TRI_ERR_LAUNCH;
  if (plan != nullptr) {
    plan->q = q; plan->k = pa.k; plan->v = pa.v;
    plan->k_sh = pa.k_sh; plan->k_sr = pa.k_sr; plan->v_sh = pa.v_sh; plan->v_sr = pa.v_sr;
    plan->lse = aa.lse; plan->lse_pert = aa.lse_pert;
  }
  return TRI_OK;
}

}  // namespace

extern "C" {

int tri_abi_version(void) { return TRI_ABI_VERSION; }

const char* tri_status_string(int status) {
  switch (status) {
    case TRI_OK: return "ok";
    case TRI_ERR_NULL: return "required pointer is NULL";
    case TRI_ERR_DTYPE: return "unsupported element type";
    case TRI_ERR_SHAPE: return "inconsistent shapes";
    case TRI_ERR_STRIDE: return "unsupported strides (inner stride must be 1, rows multiples of 8 elements)";
    case TRI_ERR_ALIGN: return "pointer not sufficiently aligned";
    case TRI_ERR_UNSUPPORTED: return "unsupported configuration";
    case TRI_ERR_SCRATCH: return "scratch buffer too small";
    case TRI_ERR_LAUNCH: return "HIP launch failed";
    default: return "unknown status";
  }
}

// ------------------------------------------------------------------ RMSNorm
int tri_validate_rmsnorm(const tri_tensor* x, const tri_tensor* w, const tri_tensor* y, float /*eps*/) {
  return validate_rmsnorm(x, w, y);
}

int tri_rmsnorm(const tri_tensor* x, const tri_tensor* w, tri_tensor* y, float eps, void* hip_stream) {
  TRI_TRY(validate_rmsnorm(x, w, y));
  const int rc = launch_rmsnorm(H(x), x->stride[0], H(w), HM(y), y->stride[0], nullptr, (int)x->shape[0],
                                (int)x->shape[1], eps, static_cast<hipStream_t>(hip_stream));
  return rc == 0 ? TRI_OK : TRI_ERR_LAUNCH;
}

// ---------------------------------------------------------------------- FFN
int tri_validate_ffn_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                            const tri_tensor* w_down, const tri_tensor* hidden, const tri_tensor* out,
                            const tri_tensor* workspace) {
  if (w_up == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_ws(workspace));
  return validate_ffn2(x, w_gate, w_up, w_down, hidden, out);
}

int64_t tri_gemm_workspace_bytes(int64_t m, int64_t k, int64_t ncols) {
  if (m <= 0 || k <= 0 || ncols <= 0 || m >= ((int64_t)1 << 31) || k >= ((int64_t)1 << 31) || ncols >= ((int64_t)1 << 31))
    return 0;
  if (m > kSkinnyMaxRows) return large_split_workspace_bytes((int)m, (int)k, (int)ncols);
  return skinny_workspace_bytes((int)m, (int)k, (int)ncols);
}

int64_t tri_ffn_workspace_bytes(int64_t m, int64_t n, int64_t f) {
  int64_t need = tri_gemm_workspace_bytes(m, n, 2 * f);
  const int64_t b = tri_gemm_workspace_bytes(m, n, f), c = tri_gemm_workspace_bytes(m, f, n),
                d = tri_gemm_workspace_bytes(m, n, n);
  need = need > b ? need : b;
  need = need > c ? need : c;
  return need > d ? need : d;
}

int tri_ffn_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up, const tri_tensor* w_down,
                   tri_tensor* hidden, tri_tensor* out, tri_tensor* workspace, void* hip_stream) {
  TRI_TRY(tri_validate_ffn_swiglu(x, w_gate, w_up, w_down, hidden, out, workspace));
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  GemmArgs g{};
  g.x = H(x); g.ldx = x->stride[0];
  g.w = H(w_gate); g.ldw = w_gate->stride[0];
  g.w2 = H(w_up); g.ldw2 = w_up->stride[0];
  g.out = HM(hidden); g.ldo = hidden->stride[0];
  g.M = (int)x->shape[0]; g.K = (int)x->shape[1]; g.N = (int)w_gate->shape[1];
  g.epi = EPI_SWIGLU;
  set_ws(g, workspace);
  if (launch_gemm(g, stream) != 0) return TRI_ERR_LAUNCH;
  GemmArgs d{};
  d.x = H(hidden); d.ldx = hidden->stride[0];
  d.w = H(w_down); d.ldw = w_down->stride[0];
  d.out = HM(out); d.ldo = out->stride[0];
  d.M = g.M; d.K = g.N; d.N = (int)w_down->shape[1];
  d.epi = EPI_NONE;
  set_ws(d, workspace);
  if (launch_gemm(d, stream) != 0) return TRI_ERR_LAUNCH;
  return TRI_OK;
}

int tri_gateup_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                      const tri_tensor* row_scale, tri_tensor* hidden, tri_tensor* workspace, void* hip_stream) {
  if (x == nullptr || w_gate == nullptr || w_up == nullptr || hidden == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_ws(workspace));
  TRI_TRY(check_mat(x, -1, -1));
  TRI_TRY(check_mat(w_gate, x->shape[1], -1));
  TRI_TRY(check_mat(w_up, x->shape[1], w_gate->shape[1]));
  TRI_TRY(check_mat(hidden, x->shape[0], w_gate->shape[1]));
  if (row_scale != nullptr) TRI_TRY(check_vec(row_scale, x->shape[0], TRI_F32));
  GemmArgs g{};
  g.x = H(x); g.ldx = x->stride[0];
  g.w = H(w_gate); g.ldw = w_gate->stride[0];
  g.w2 = H(w_up); g.ldw2 = w_up->stride[0];
  g.rowscale = row_scale != nullptr ? static_cast<const float*>(row_scale->ptr) : nullptr;
  g.out = HM(hidden); g.ldo = hidden->stride[0];
  g.M = (int)x->shape[0]; g.K = (int)x->shape[1]; g.N = (int)w_gate->shape[1];
  g.epi = EPI_SWIGLU;
  set_ws(g, workspace);
  return launch_gemm(g, static_cast<hipStream_t>(hip_stream)) == 0 ? TRI_OK : TRI_ERR_LAUNCH;
}

int tri_matmul(const tri_tensor* x, const tri_tensor* w, const tri_tensor* residual, tri_tensor* out,
               tri_tensor* workspace, void* hip_stream) {
  if (x == nullptr || w == nullptr || out == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_ws(workspace));
  TRI_TRY(check_mat(x, -1, -1));
  TRI_TRY(check_mat(w, x->shape[1], -1));
  TRI_TRY(check_mat(out, x->shape[0], w->shape[1]));
  if (residual != nullptr) TRI_TRY(check_mat(residual, x->shape[0], w->shape[1]));
  GemmArgs d{};
  d.x = H(x); d.ldx = x->stride[0];
  d.w = H(w); d.ldw = w->stride[0];
  d.residual = H(residual); d.ldr = residual != nullptr ? residual->stride[0] : 0;
  d.out = HM(out); d.ldo = out->stride[0];
  d.M = (int)x->shape[0]; d.K = (int)x->shape[1]; d.N = (int)w->shape[1];
  d.epi = EPI_NONE;
  set_ws(d, workspace);
  return launch_gemm(d, static_cast<hipStream_t>(hip_stream)) == 0 ? TRI_OK : TRI_ERR_LAUNCH;
}

int tri_validate_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2, const tri_tensor* hidden,
                          const tri_tensor* out, const tri_tensor* workspace) {
  TRI_TRY(check_ws(workspace));
  return validate_ffn2(x, w1, nullptr, w2, hidden, out);
}

int tri_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2, tri_tensor* hidden, tri_tensor* out,
                 tri_tensor* workspace, void* hip_stream) {
  TRI_TRY(tri_validate_ffn_gelu(x, w1, w2, hidden, out, workspace));
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  GemmArgs g{};
  g.x = H(x); g.ldx = x->stride[0];
  g.w = H(w1); g.ldw = w1->stride[0];
  g.out = HM(hidden); g.ldo = hidden->stride[0];
  g.M = (int)x->shape[0]; g.K = (int)x->shape[1]; g.N = (int)w1->shape[1];
  g.epi = EPI_GELU;
  set_ws(g, workspace);
  if (launch_gemm(g, stream) != 0) return TRI_ERR_LAUNCH;
  GemmArgs d{};
  d.x = H(hidden); d.ldx = hidden->stride[0];
  d.w = H(w2); d.ldw = w2->stride[0];
  d.out = HM(out); d.ldo = out->stride[0];
  d.M = g.M; d.K = g.N; d.N = (int)w2->shape[1];
  d.epi = EPI_NONE;
  set_ws(d, workspace);
  if (launch_gemm(d, stream) != 0) return TRI_ERR_LAUNCH;
  return TRI_OK;
}

int tri_validate_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x, const tri_tensor* wff1a,
                           const tri_tensor* wff1b, const tri_tensor* wff2, const tri_tensor* attn_o2,
                           const tri_tensor* row_scratch, const tri_tensor* ff1, const tri_tensor* ff2,
                           const tri_tensor* o_ff_norm, const tri_tensor* workspace) {
  TRI_TRY(check_ws(workspace));
  TRI_TRY(check_mat(o2, -1, -1));
  const int64_t M = o2->shape[0], N = o2->shape[1];
  TRI_TRY(check_mat(wo, N, N));
  TRI_TRY(check_mat(x, M, N));
  TRI_TRY(check_mat(wff1a, N, -1));
  const int64_t F = wff1a->shape[1];
  TRI_TRY(check_mat(wff1b, N, F));
  TRI_TRY(check_mat(wff2, F, N));
  TRI_TRY(check_mat(attn_o2, M, N));
  TRI_TRY(check_vec(row_scratch, M, TRI_F32));
  TRI_TRY(check_mat(ff1, M, F));
  TRI_TRY(check_mat(ff2, M, N));
  if (o_ff_norm != nullptr) TRI_TRY(check_mat(o_ff_norm, M, N));
  return TRI_OK;
}

int tri_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x, const tri_tensor* wff1a,
                  const tri_tensor* wff1b, const tri_tensor* wff2, tri_tensor* attn_o2, tri_tensor* row_scratch,
                  tri_tensor* ff1, tri_tensor* ff2, tri_tensor* o_ff_norm, tri_tensor* workspace, void* hip_stream) {
  TRI_TRY(tri_validate_ffn_block(o2, wo, x, wff1a, wff1b, wff2, attn_o2, row_scratch, ff1, ff2, o_ff_norm,
                                 workspace));
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const int M = (int)o2->shape[0], N = (int)o2->shape[1], F = (int)wff1a->shape[1];
  float* rs = static_cast<float*>(row_scratch->ptr);
  // attn_o2 = o2 . wo + x
  GemmArgs a{};
  a.x = H(o2); a.ldx = o2->stride[0];
  a.w = H(wo); a.ldw = wo->stride[0];
  a.residual = H(x); a.ldr = x->stride[0];
  a.out = HM(attn_o2); a.ldo = attn_o2->stride[0];
  a.M = M; a.K = N; a.N = N; a.epi = EPI_NONE;
  set_ws(a, workspace);
  if (launch_gemm(a, stream) != 0) return TRI_ERR_LAUNCH;
  // rs[m] = rsqrt(mean(attn_o2[m]^2))
  if (launch_rmsnorm(H(attn_o2), attn_o2->stride[0], nullptr, nullptr, 0, rs, M, N, 0.f, stream) != 0)
    return TRI_ERR_LAUNCH;
  // ff1 = silu(rs * attn_o2 . wff1b) * (rs * attn_o2 . wff1a)
  GemmArgs g{};
  g.x = H(attn_o2); g.ldx = attn_o2->stride[0];
  g.w = H(wff1b); g.ldw = wff1b->stride[0];
  g.w2 = H(wff1a); g.ldw2 = wff1a->stride[0];
  g.rowscale = rs;
  g.out = HM(ff1); g.ldo = ff1->stride[0];
  g.M = M; g.K = N; g.N = F; g.epi = EPI_SWIGLU;
  set_ws(g, workspace);
  if (launch_gemm(g, stream) != 0) return TRI_ERR_LAUNCH;
  // ff2 = ff1 . wff2
  GemmArgs d{};
  d.x = H(ff1); d.ldx = ff1->stride[0];
  d.w = H(wff2); d.ldw = wff2->stride[0];
  d.out = HM(ff2); d.ldo = ff2->stride[0];
  d.M = M; d.K = F; d.N = N; d.epi = EPI_NONE;
  set_ws(d, workspace);
  if (launch_gemm(d, stream) != 0) return TRI_ERR_LAUNCH;
  if (o_ff_norm != nullptr) {
    if (launch_add_scaled_rmsnorm(H(ff2), ff2->stride[0], H(attn_o2), attn_o2->stride[0], rs, HM(o_ff_norm),
                                  o_ff_norm->stride[0], M, N, stream) != 0)
      return TRI_ERR_LAUNCH;
  }
  return TRI_OK;
}

// ---------------------------------------------------------------- attention
int64_t tri_qkv_scratch_bytes(const tri_attn_params* p, int64_t n_model) {
  if (p == nullptr) return TRI_ERR_NULL;
  if (p->seq <= 0 || p->n_q_heads <= 0 || p->n_kv_heads <= 0 || p->head_dim <= 0 || n_model < 0) return TRI_ERR_SHAPE;
  return scratch_layout(p, n_model).total;
}

int tri_validate_qkv_attention(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                               const tri_tensor* wk, const tri_tensor* wv, const tri_tensor* k_cache,
                               const tri_tensor* v_cache, const tri_tensor* scratch, const tri_tensor* lse,
                               const tri_tensor* out, const tri_attn_params* p) {
  TRI_TRY(validate_qkv_common(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, p));
  if (lse != nullptr) TRI_TRY(check_f32_mat(lse, p->n_q_heads, p->seq));
  if (lse != nullptr && lse->stride[0] != p->seq) return TRI_ERR_STRIDE;
  return TRI_OK;
}

int tri_qkv_attention(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                      const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch,
                      tri_tensor* lse, tri_tensor* out, const tri_attn_params* p, void* hip_stream) {
  TRI_TRY(tri_validate_qkv_attention(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, lse, out, p));
  return run_qkv(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch,
                 lse != nullptr ? static_cast<float*>(lse->ptr) : nullptr, out, p, false, false, nullptr,
                 static_cast<hipStream_t>(hip_stream), nullptr);
}

int tri_validate_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                           const tri_tensor* wk, const tri_tensor* wv, const tri_tensor* k_cache,
                           const tri_tensor* v_cache, const tri_tensor* scratch, const tri_tensor* noise,
                           const tri_tensor* out, const tri_tensor* score, const tri_attn_params* p) {
  TRI_TRY(validate_qkv_common(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, p));
  TRI_TRY(check_noise(noise, p->n_q_heads, p->seq, (int64_t)p->kv_prefix + p->seq));
  TRI_TRY(check_f32_mat(score, p->n_q_heads, (int64_t)p->kv_prefix + p->seq));
  return TRI_OK;
}

int tri_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                  const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch,
                  const tri_tensor* noise, tri_tensor* out, tri_tensor* score, const tri_attn_params* p,
                  void* hip_stream) {
  TRI_TRY(tri_validate_keyformer(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, noise, out, score, p));
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  QkvPlan plan{};
  TRI_TRY(run_qkv(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, nullptr, out, p, false, true, H(noise), stream,
                  &plan));
  ScoreArgs sa{};
  sa.q = plan.q; sa.ldq = (int64_t)p->n_q_heads * p->head_dim;
  sa.k = plan.k; sa.k_sh = plan.k_sh; sa.k_sr = plan.k_sr;
  sa.lse = plan.lse_pert;
  sa.noise = H(noise);
  sa.o1 = static_cast<float*>(score->ptr); sa.ldo1 = score->stride[0];
  sa.o2 = nullptr; sa.ldo2 = 0;
  sa.S = p->seq; sa.P = p->kv_prefix; sa.Hq = p->n_q_heads; sa.Hkv = p->n_kv_heads; sa.D = p->head_dim;
  sa.scale = p->scale; sa.tau = p->tau; sa.causal = p->causal; sa.mode = 1; sa.mean_var = 0;
  sa.seed = p->noise_seed;
  if (launch_scores(sa, stream) != 0) return TRI_ERR_LAUNCH;
  return TRI_OK;
}

int tri_validate_roco(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                      const tri_tensor* wv, const tri_tensor* k_cache, const tri_tensor* v_cache,
                      const tri_tensor* scratch, const tri_tensor* out, const tri_tensor* sum_out,
                      const tri_tensor* sumsq_out, int32_t /*as_mean_var*/, const tri_attn_params* p) {
  TRI_TRY(validate_qkv_common(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, p));
  TRI_TRY(check_f32_mat(sum_out, p->n_q_heads, (int64_t)p->kv_prefix + p->seq));
  TRI_TRY(check_f32_mat(sumsq_out, p->n_q_heads, (int64_t)p->kv_prefix + p->seq));
  return TRI_OK;
}

int tri_roco(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
             const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch, tri_tensor* out,
             tri_tensor* sum_out, tri_tensor* sumsq_out, int32_t as_mean_var, const tri_attn_params* p,
             void* hip_stream) {
  TRI_TRY(tri_validate_roco(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, sum_out, sumsq_out, as_mean_var, p));
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  QkvPlan plan{};
  TRI_TRY(run_qkv(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, nullptr, out, p, true, false, nullptr, stream,
                  &plan));
  ScoreArgs sa{};
  sa.q = plan.q; sa.ldq = (int64_t)p->n_q_heads * p->head_dim;
  sa.k = plan.k; sa.k_sh = plan.k_sh; sa.k_sr = plan.k_sr;
  sa.lse = plan.lse;
  sa.noise = nullptr;
  sa.o1 = static_cast<float*>(sum_out->ptr); sa.ldo1 = sum_out->stride[0];
  sa.o2 = static_cast<float*>(sumsq_out->ptr); sa.ldo2 = sumsq_out->stride[0];
  sa.S = p->seq; sa.P = p->kv_prefix; sa.Hq = p->n_q_heads; sa.Hkv = p->n_kv_heads; sa.D = p->head_dim;
  sa.scale = p->scale; sa.tau = p->tau; sa.causal = p->causal; sa.mode = 0; sa.mean_var = as_mean_var != 0;
  sa.seed = 0;
  if (launch_scores(sa, stream) != 0) return TRI_ERR_LAUNCH;
  return TRI_OK;
}

}  // extern "C"
