// C ABI of libtrinity_amd.so: argument validation (pure host code, usable
// without a GPU) and the launch sequences behind each entry point.
#include "../../include/trinity_amd.h"

#include "launch.h"  // fp16 kernels: namespace tri
#define TRI_BF16
#define tri tri_bf16
#include "launch.h"  // bf16 kernels: namespace tri_bf16 (the same sources compiled a second time)
#undef tri
#undef TRI_BF16

// ------------------------------------------------- kernels that need the large-LDS attribute (see launch.h)
namespace {
TriLdsAttr* g_lds_attr_head = nullptr;  // filled while the library is loaded (static constructors, one thread)
}
void tri_lds_attr_register(TriLdsAttr* node) {
  node->next = g_lds_attr_head;
  g_lds_attr_head = node;
}
int tri_lds_attr_apply(TriLdsAttr* node) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  const uint64_t bit = 1ull << (dev & 63);
  if (node->done.load(std::memory_order_acquire) & bit) return 0;
  if (hipFuncSetAttribute(node->kern, hipFuncAttributeMaxDynamicSharedMemorySize, node->bytes) != hipSuccess) return -1;
  node->done.fetch_or(bit, std::memory_order_release);
  return 0;
}

// ------------------------------------------------- scratch memory of the entry point that allocates nothing
// tri_qkv_attention_static keeps what tri_qkv_attention takes as its `scratch` argument (q / k / v rows, split-K
// partial sums, partial attention results, log-sum-exp rows) in this array.  Every GPU the library runs on holds
// its own copy, at its own address, until the process ends.  In host code the array's name only stands for the
// symbol: the address kernels can use is the one hipGetSymbolAddress returns with that device current, looked up
// once per device and kept in g_static_scratch_ptr.
constexpr int64_t kStaticScratchBytes = TRI_STATIC_SCRATCH_BYTES;
constexpr int kStaticScratchMaxDevices = 64;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];
namespace {
std::atomic<unsigned char*> g_static_scratch_ptr[kStaticScratchMaxDevices];

// address of the current device's copy; threads racing on the first call look the same address up twice
int static_scratch_ptr(unsigned char** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return TRI_ERR_LAUNCH;
  if (dev < 0 || dev >= kStaticScratchMaxDevices) return TRI_ERR_UNSUPPORTED;
  unsigned char* ptr = g_static_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_static_scratch)) != hipSuccess || sym == nullptr) return TRI_ERR_LAUNCH;
    ptr = static_cast<unsigned char*>(sym);
    g_static_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return TRI_OK;
}
}  // namespace

using tri::few_attn_workspace_bytes;
using tri::split_attn_workspace_bytes;
using tri::kSkinnyMaxRows;
using tri::large_split_workspace_bytes;
using tri::skinny_workspace_bytes;

namespace {

struct Scratch {
  int64_t q_off, k_off, v_off, xn_off, lse_off, lsep_off, ws_off, ws_bytes, aws_off, aws_bytes, kd_off, vd_off, total;
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
  // few new tokens: room for the split-K partial sums of the projection and for the partial results of the
  // key-split attention (separate: the attention kernel merges the former while it writes the latter)
  s.ws_bytes = skinny_workspace_bytes((int)S, (int)n_model, (int)((Hq + 2 * Hkv) * D), true);
  s.ws_off = off; off = align256(off + s.ws_bytes);
  s.aws_bytes = few_attn_workspace_bytes((int)S, (int)Hq, (int)D, (int)(p->kv_prefix + S));
  {
    const int64_t split = split_attn_workspace_bytes((int)S, (int)Hq, (int)Hkv, (int)D, (int)(p->kv_prefix + S));
    s.aws_bytes = s.aws_bytes > split ? s.aws_bytes : split;
  }
  s.aws_off = off; off = align256(off + s.aws_bytes);
  // fp8 caches: 16-bit copies of all P + S rows for the kernels that read 16-bit K / V tiles
  const int64_t copy = p->kv_fp8 ? Hkv * ((int64_t)p->kv_prefix + S) * D * 2 : 0;
  s.kd_off = off; off = align256(off + copy);
  s.vd_off = off; off = align256(off + copy);
  s.total = off;
  return s;
}

// element type of a call: fp16 or bf16, taken from its first activation tensor (every other 16-bit tensor of the
// call must match)
inline int elem_dtype(const tri_tensor* t) { return (t != nullptr && t->dtype == TRI_BF16) ? TRI_BF16 : TRI_F16; }

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// fp16 matrix [rows, cols] with unit inner stride and 16-byte aligned rows
int check_mat(const tri_tensor* t, int64_t rows, int64_t cols, int dtype) {
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
  if (dtype == TRI_F16 || dtype == TRI_BF16) {
    if (t->stride[0] % 8 != 0 || t->shape[1] % 8 != 0) return TRI_ERR_STRIDE;
    if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  }
  return TRI_OK;
}

// A weight matrix [K, N] may also be stored K-contiguous (stride[0] == 1: the transpose view of a row-major [N, K]
// tensor, the layout of torch.nn.Linear.weight).
inline bool is_kcontig(const tri_tensor* t) {
  return t != nullptr && t->ndim == 2 && t->stride[0] == 1 && t->stride[1] != 1 && t->shape[0] > 1;
}
int check_wmat(const tri_tensor* t, int64_t rows, int64_t cols, int dtype) {
  if (!is_kcontig(t)) return check_mat(t, rows, cols, dtype);
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (rows >= 0 && t->shape[0] != rows) return TRI_ERR_SHAPE;
  if (cols >= 0 && t->shape[1] != cols) return TRI_ERR_SHAPE;
  if (t->shape[1] < 0) return TRI_ERR_SHAPE;
  if (t->stride[1] < t->shape[0] || t->stride[1] % 8 != 0 || t->shape[1] % 8 != 0) return TRI_ERR_STRIDE;
  if (t->shape[0] % 32 != 0) return TRI_ERR_UNSUPPORTED;  // this layout runs on the direct-to-LDS loop only
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

int check_vec(const tri_tensor* t, int64_t n, int dtype) {
  if (t == nullptr) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (t->ndim != 1 || t->shape[0] != n) return TRI_ERR_SHAPE;
  if (n == 0) return TRI_OK;  // no elements: no storage (the vector of an empty batch)
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (n > 1 && t->stride[0] != 1) return TRI_ERR_STRIDE;
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

// head-major [H, rows >= min_rows, D] fp16 with contiguous d
int check_cache(const tri_tensor* t, int64_t H, int64_t min_rows, int64_t D, int dtype) {
  if (t == nullptr || t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (t->ndim != 3 || t->shape[0] != H || t->shape[1] < min_rows || t->shape[2] != D) return TRI_ERR_SHAPE;
  const int64_t q = dtype == TRI_FP8_E4M3 ? 16 : 8;  // rows start on 16-byte boundaries
  if (t->stride[2] != 1 || t->stride[1] % q != 0 || t->stride[0] % q != 0 || t->stride[1] < D) return TRI_ERR_STRIDE;
  if (t->shape[1] * t->stride[1] * 2 >= ((int64_t)1 << 31)) return TRI_ERR_UNSUPPORTED;  // per-head extent fits a buffer descriptor
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

// optional split-K workspace: 1-D bytes
int check_ws(const tri_tensor* t) {
  if (t == nullptr) return TRI_OK;
  if (t->dtype != TRI_U8) return TRI_ERR_DTYPE;
  if (t->ndim != 1 || t->shape[0] < 0) return TRI_ERR_SHAPE;
  if (t->shape[0] == 0) return TRI_OK;  // an empty workspace is no workspace (its pointer may be NULL)
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->shape[0] > 1 && t->stride[0] != 1) return TRI_ERR_STRIDE;
  if (!aligned16(t->ptr)) return TRI_ERR_ALIGN;
  return TRI_OK;
}

#define TRI_TRY(expr)            \
  do {                           \
    const int st__ = (expr);     \
    if (st__ != TRI_OK) return st__; \
  } while (0)

int validate_rmsnorm(const tri_tensor* x, const tri_tensor* w, const tri_tensor* y) {
  if (x == nullptr || y == nullptr) return TRI_ERR_NULL;
  const int dt = elem_dtype(x);
  if (x->dtype != dt || y->dtype != dt) return TRI_ERR_DTYPE;
  if (x->ndim != 2 || y->ndim != 2) return TRI_ERR_SHAPE;
  if ((x->ptr == nullptr || y->ptr == nullptr) && x->shape[0] != 0) return TRI_ERR_NULL;  // no rows: no storage
  if (x->shape[0] != y->shape[0] || x->shape[1] != y->shape[1]) return TRI_ERR_SHAPE;
  if (x->stride[1] != 1 || y->stride[1] != 1) return TRI_ERR_STRIDE;
  if (x->shape[0] > 1 && (x->stride[0] < x->shape[1] || y->stride[0] < y->shape[1])) return TRI_ERR_STRIDE;
  if (w != nullptr) {
    if (w->ptr == nullptr) return TRI_ERR_NULL;
    if (w->dtype != dt) return TRI_ERR_DTYPE;
    if (w->ndim != 1 || w->shape[0] != x->shape[1]) return TRI_ERR_SHAPE;
    if (w->shape[0] > 1 && w->stride[0] != 1) return TRI_ERR_STRIDE;
  }
  return TRI_OK;
}

int validate_ffn2(const tri_tensor* x, const tri_tensor* wa, const tri_tensor* wb, const tri_tensor* wd,
                  const tri_tensor* hidden, const tri_tensor* out) {
  if (x == nullptr || wa == nullptr || wd == nullptr || hidden == nullptr || out == nullptr) return TRI_ERR_NULL;
  const int dt = elem_dtype(x);
  TRI_TRY(check_mat(x, -1, -1, dt));
  const int64_t T = x->shape[0], N = x->shape[1];
  TRI_TRY(check_wmat(wa, N, -1, dt));
  const int64_t F = wa->shape[1];
  if (wb != nullptr) TRI_TRY(check_wmat(wb, N, F, dt));
  if (wb != nullptr && is_kcontig(wa) != is_kcontig(wb)) return TRI_ERR_STRIDE;  // gate and up share one layout
  TRI_TRY(check_wmat(wd, F, -1, dt));
  TRI_TRY(check_mat(hidden, T, F, dt));
  TRI_TRY(check_mat(out, T, wd->shape[1], dt));
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
  // the projected queries [S, Hq * D] are addressed through a 32-bit buffer descriptor
  if (S * Hq * D * 2 >= ((int64_t)1 << 31)) return TRI_ERR_UNSUPPORTED;
  const int dt = elem_dtype(x);
  TRI_TRY(check_mat(x, S, -1, dt));
  const int64_t N = x->shape[1];
  if (norm_w != nullptr) {
    if (!p->prenorm) return TRI_ERR_SHAPE;
    TRI_TRY(check_vec(norm_w, N, dt));
  }
  // row-major [N, heads * D] (the reference's X.W) or K-contiguous (see is_kcontig), all three alike
  TRI_TRY(check_wmat(wq, N, Hq * D, dt));
  TRI_TRY(check_wmat(wk, N, Hkv * D, dt));
  TRI_TRY(check_wmat(wv, N, Hkv * D, dt));
  if (is_kcontig(wq) != is_kcontig(wk) || is_kcontig(wq) != is_kcontig(wv)) return TRI_ERR_STRIDE;
  if ((k_cache == nullptr) != (v_cache == nullptr)) return TRI_ERR_NULL;
  if (k_cache == nullptr && (P > 0 || p->kv_fp8)) return TRI_ERR_NULL;
  if (p->kv_fp8 && (!(p->k_scale > 0.f) || !(p->v_scale > 0.f))) return TRI_ERR_UNSUPPORTED;
  if (k_cache != nullptr) {
    const int cdt = p->kv_fp8 ? (int)TRI_FP8_E4M3 : dt;
    TRI_TRY(check_cache(k_cache, Hkv, P + S, D, cdt));
    TRI_TRY(check_cache(v_cache, Hkv, P + S, D, cdt));
  }
  if (scratch == nullptr || scratch->ptr == nullptr) return TRI_ERR_NULL;
  if (scratch->ndim != 1 || (scratch->shape[0] > 1 && scratch->stride[0] != 1)) return TRI_ERR_STRIDE;
  {
    const int64_t esz = (scratch->dtype == TRI_U8) ? 1 : (scratch->dtype == TRI_F32 ? 4 : 2);
    if (scratch->shape[0] * esz < scratch_layout(p, N).total) return TRI_ERR_SCRATCH;
    if (((uintptr_t)scratch->ptr & 255u) != 0) return TRI_ERR_ALIGN;
  }
  TRI_TRY(check_mat(out, S, Hq * D, dt));
  return TRI_OK;
}

int check_f32_mat(const tri_tensor* t, int64_t rows, int64_t cols) {
  if (t == nullptr || t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != TRI_F32) return TRI_ERR_DTYPE;
  if (t->ndim != 2 || t->shape[0] != rows || t->shape[1] != cols) return TRI_ERR_SHAPE;
  if (t->stride[1] != 1 || (rows > 1 && t->stride[0] < cols)) return TRI_ERR_STRIDE;
  return TRI_OK;
}

int check_noise(const tri_tensor* t, int64_t Hq, int64_t S, int64_t L, int dtype) {
  if (t == nullptr) return TRI_OK;
  if (t->ptr == nullptr) return TRI_ERR_NULL;
  if (t->dtype != dtype) return TRI_ERR_DTYPE;
  if (t->ndim != 3 || t->shape[0] != Hq || t->shape[1] != S || t->shape[2] != L) return TRI_ERR_SHAPE;
  if (t->stride[2] != 1 || t->stride[1] != L || t->stride[0] != S * L) return TRI_ERR_STRIDE;
  return TRI_OK;
}

}  // namespace

// The launch sequences exist once per element type: the same text, compiled against the fp16 kernels
// (namespace tri) and against the bf16 kernels (namespace tri_bf16).
namespace f16 {
using namespace tri;
#include "abi_impl.inc"
}  // namespace f16
namespace bf16 {
using namespace tri_bf16;
#include "abi_impl.inc"
}  // namespace bf16

#define TRI_DISPATCH(t, call) ((t)->dtype == TRI_BF16 ? bf16::call : f16::call)

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

int tri_prepare(void) {
  for (TriLdsAttr* n = g_lds_attr_head; n != nullptr; n = n->next)
    if (tri_lds_attr_apply(n) != 0) return TRI_ERR_LAUNCH;
  unsigned char* ptr = nullptr;
  return static_scratch_ptr(&ptr);  // the current device's scratch array of tri_qkv_attention_static
}

// ------------------------------------------------------------------ RMSNorm
int tri_validate_rmsnorm(const tri_tensor* x, const tri_tensor* w, const tri_tensor* y, float /*eps*/) {
  return validate_rmsnorm(x, w, y);
}

int tri_rmsnorm(const tri_tensor* x, const tri_tensor* w, tri_tensor* y, float eps, void* hip_stream) {
  TRI_TRY(validate_rmsnorm(x, w, y));
  return TRI_DISPATCH(x, impl_rmsnorm(x, w, y, eps, hip_stream));
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
  const int64_t few = skinny_workspace_bytes((int)m, (int)k, (int)ncols);
  return few > 0 ? few : large_split_workspace_bytes((int)m, (int)k, (int)ncols);
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
  return TRI_DISPATCH(x, impl_ffn_swiglu(x, w_gate, w_up, w_down, hidden, out, workspace, hip_stream));
}

int tri_gateup_swiglu(const tri_tensor* x, const tri_tensor* w_gate, const tri_tensor* w_up,
                      const tri_tensor* row_scale, tri_tensor* hidden, tri_tensor* workspace, void* hip_stream) {
  if (x == nullptr || w_gate == nullptr || w_up == nullptr || hidden == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_ws(workspace));
  const int dt = elem_dtype(x);
  TRI_TRY(check_mat(x, -1, -1, dt));
  TRI_TRY(check_wmat(w_gate, x->shape[1], -1, dt));
  TRI_TRY(check_wmat(w_up, x->shape[1], w_gate->shape[1], dt));
  if (is_kcontig(w_gate) != is_kcontig(w_up)) return TRI_ERR_STRIDE;
  TRI_TRY(check_mat(hidden, x->shape[0], w_gate->shape[1], dt));
  if (row_scale != nullptr) TRI_TRY(check_vec(row_scale, x->shape[0], TRI_F32));
  return TRI_DISPATCH(x, impl_gateup_swiglu(x, w_gate, w_up, row_scale, hidden, workspace, hip_stream));
}

int tri_matmul(const tri_tensor* x, const tri_tensor* w, const tri_tensor* residual, tri_tensor* out,
               tri_tensor* workspace, void* hip_stream) {
  if (x == nullptr || w == nullptr || out == nullptr) return TRI_ERR_NULL;
  TRI_TRY(check_ws(workspace));
  const int dt = elem_dtype(x);
  TRI_TRY(check_mat(x, -1, -1, dt));
  TRI_TRY(check_wmat(w, x->shape[1], -1, dt));
  TRI_TRY(check_mat(out, x->shape[0], w->shape[1], dt));
  if (residual != nullptr) TRI_TRY(check_mat(residual, x->shape[0], w->shape[1], dt));
  return TRI_DISPATCH(x, impl_matmul(x, w, residual, out, workspace, hip_stream));
}

int tri_validate_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2, const tri_tensor* hidden,
                          const tri_tensor* out, const tri_tensor* workspace) {
  TRI_TRY(check_ws(workspace));
  return validate_ffn2(x, w1, nullptr, w2, hidden, out);
}

int tri_ffn_gelu(const tri_tensor* x, const tri_tensor* w1, const tri_tensor* w2, tri_tensor* hidden, tri_tensor* out,
                 tri_tensor* workspace, void* hip_stream) {
  TRI_TRY(tri_validate_ffn_gelu(x, w1, w2, hidden, out, workspace));
  return TRI_DISPATCH(x, impl_ffn_gelu(x, w1, w2, hidden, out, workspace, hip_stream));
}

int tri_validate_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x, const tri_tensor* wff1a,
                           const tri_tensor* wff1b, const tri_tensor* wff2, const tri_tensor* attn_o2,
                           const tri_tensor* row_scratch, const tri_tensor* ff1, const tri_tensor* ff2,
                           const tri_tensor* o_ff_norm, const tri_tensor* workspace) {
  TRI_TRY(check_ws(workspace));
  const int dt = elem_dtype(o2);
  TRI_TRY(check_mat(o2, -1, -1, dt));
  const int64_t M = o2->shape[0], N = o2->shape[1];
  TRI_TRY(check_mat(wo, N, N, dt));
  TRI_TRY(check_mat(x, M, N, dt));
  TRI_TRY(check_mat(wff1a, N, -1, dt));
  const int64_t F = wff1a->shape[1];
  TRI_TRY(check_mat(wff1b, N, F, dt));
  TRI_TRY(check_mat(wff2, F, N, dt));
  TRI_TRY(check_mat(attn_o2, M, N, dt));
  TRI_TRY(check_vec(row_scratch, M, TRI_F32));
  TRI_TRY(check_mat(ff1, M, F, dt));
  TRI_TRY(check_mat(ff2, M, N, dt));
  if (o_ff_norm != nullptr) TRI_TRY(check_mat(o_ff_norm, M, N, dt));
  return TRI_OK;
}

int tri_ffn_block(const tri_tensor* o2, const tri_tensor* wo, const tri_tensor* x, const tri_tensor* wff1a,
                  const tri_tensor* wff1b, const tri_tensor* wff2, tri_tensor* attn_o2, tri_tensor* row_scratch,
                  tri_tensor* ff1, tri_tensor* ff2, tri_tensor* o_ff_norm, tri_tensor* workspace, void* hip_stream) {
  TRI_TRY(tri_validate_ffn_block(o2, wo, x, wff1a, wff1b, wff2, attn_o2, row_scratch, ff1, ff2, o_ff_norm,
                                 workspace));
  return TRI_DISPATCH(o2, impl_ffn_block(o2, wo, x, wff1a, wff1b, wff2, attn_o2, row_scratch, ff1, ff2, o_ff_norm, workspace, hip_stream));
}

// ---------------------------------------------------------------- attention
int64_t tri_qkv_scratch_bytes(const tri_attn_params* p, int64_t n_model) {
  if (p == nullptr) return TRI_ERR_NULL;
  // the limits of validate_qkv_common, so that a size is only returned for parameters the launchers accept
  if (p->head_dim != 64 && p->head_dim != 128) return TRI_ERR_UNSUPPORTED;
  if (p->seq <= 0 || p->kv_prefix < 0 || p->n_q_heads <= 0 || p->n_kv_heads <= 0 ||
      p->n_q_heads % p->n_kv_heads != 0 || n_model < 0 || n_model >= ((int64_t)1 << 31))
    return TRI_ERR_SHAPE;
  const int64_t S = p->seq, D = p->head_dim, L = (int64_t)p->kv_prefix + S;
  if (S * p->n_q_heads * D * 2 >= ((int64_t)1 << 31)) return TRI_ERR_UNSUPPORTED;
  if (L * D * 2 >= ((int64_t)1 << 31)) return TRI_ERR_UNSUPPORTED;  // a head's cache rows fit a buffer descriptor
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
  return TRI_DISPATCH(x, impl_qkv_attention(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, lse, out, p, hip_stream));
}

int tri_qkv_attention_static(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                             const tri_tensor* wk, const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache,
                             tri_tensor* lse, tri_tensor* out, const tri_attn_params* p, void* hip_stream) {
  if (x == nullptr || p == nullptr) return TRI_ERR_NULL;
  if (x->ndim != 2) return TRI_ERR_SHAPE;
  // the size first: a call that does not fit the array is refused before anything else is looked at
  const int64_t need = tri_qkv_scratch_bytes(p, x->shape[1]);
  if (need < 0) return (int)need;
  if (need > kStaticScratchBytes) return TRI_ERR_SCRATCH;
  // every other argument is checked against a stand-in for the array (right size and alignment, never
  // dereferenced), so that a bad call fails without touching the GPU
  tri_tensor scratch{};
  scratch.ptr = reinterpret_cast<void*>(static_cast<uintptr_t>(256));
  scratch.shape[0] = kStaticScratchBytes;
  scratch.stride[0] = 1;
  scratch.ndim = 1;
  scratch.dtype = TRI_U8;
  TRI_TRY(tri_validate_qkv_attention(x, norm_w, wq, wk, wv, k_cache, v_cache, &scratch, lse, out, p));
  unsigned char* ptr = nullptr;
  TRI_TRY(static_scratch_ptr(&ptr));
  scratch.ptr = ptr;
  return TRI_DISPATCH(x, impl_qkv_attention(x, norm_w, wq, wk, wv, k_cache, v_cache, &scratch, lse, out, p, hip_stream));
}

int tri_validate_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq,
                           const tri_tensor* wk, const tri_tensor* wv, const tri_tensor* k_cache,
                           const tri_tensor* v_cache, const tri_tensor* scratch, const tri_tensor* noise,
                           const tri_tensor* out, const tri_tensor* score, const tri_attn_params* p) {
  TRI_TRY(validate_qkv_common(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, p));
  TRI_TRY(check_noise(noise, p->n_q_heads, p->seq, (int64_t)p->kv_prefix + p->seq, elem_dtype(x)));
  TRI_TRY(check_f32_mat(score, p->n_q_heads, (int64_t)p->kv_prefix + p->seq));
  return TRI_OK;
}

int tri_keyformer(const tri_tensor* x, const tri_tensor* norm_w, const tri_tensor* wq, const tri_tensor* wk,
                  const tri_tensor* wv, tri_tensor* k_cache, tri_tensor* v_cache, tri_tensor* scratch,
                  const tri_tensor* noise, tri_tensor* out, tri_tensor* score, const tri_attn_params* p,
                  void* hip_stream) {
  TRI_TRY(tri_validate_keyformer(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, noise, out, score, p));
  return TRI_DISPATCH(x, impl_keyformer(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, noise, out, score, p, hip_stream));
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
  return TRI_DISPATCH(x, impl_roco(x, norm_w, wq, wk, wv, k_cache, v_cache, scratch, out, sum_out, sumsq_out, as_mean_var, p, hip_stream));
}

}  // extern "C"
