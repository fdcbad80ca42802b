// C ABI of libautograd_hip.so: context, memory, passes, the typed entry points
// and the name-based dispatcher that plays the role of
// MetalContext.dispatch_with_args_3d (metal_ext.mm:559-590).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "launch.hpp"

struct agrad_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    // The word kernels set when they see a token id or a class label out of range.  It lives in
    // pinned host memory that the GPU writes directly: the pass boundary reads it without a copy
    // (a blocking device-to-host copy per end_pass was a tenth of a small training step).
    int* err_flag = nullptr;               // the GPU's address of the word
    volatile int* err_host = nullptr;      // the host's address of the same word
    uint64_t total_mem = 0;
    std::mutex mu;
    std::map<uint64_t, uint64_t> allocs;   // base address -> bytes
    bool capturing = false;                // between agrad_graph_begin and agrad_graph_end
    std::map<uint64_t, hipGraphExec_t> graphs;
    uint64_t next_graph = 1;
    // column sums (dgamma / dbeta, bias gradients) that backward calls with AGRAD_DEFER_PARAM_GRAD
    // left unfolded: their partial rows wait in the callers' workspaces for agrad_finalize_param_grads
    std::vector<agrad::ColsumJob> pending;
    // counters and (max, sum) pairs of the workgroup teams of the fused cross-entropy (long rows)
    void* ce_scratch = nullptr;
    uint32_t team_polls = 0;               // 0: the kernels' own bound on a team member's wait
};

namespace agrad {

static thread_local std::string g_last_error;

int set_error(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

static thread_local bool g_capturing = false;
void set_capturing(bool on) { g_capturing = on; }
bool is_capturing() { return g_capturing; }

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return AGRAD_OK;
    return set_error(AGRAD_EHIP, "%s: %s", what, hipGetErrorString(e));
}

namespace {

struct DeviceGuard {
    explicit DeviceGuard(agrad_ctx* c) { (void)hipSetDevice(c->device); }
};

// Resolve (buffer id, byte offset) to a device address and check that `need`
// bytes from there lie inside one allocation made through this context.
int resolve(agrad_ctx* ctx, uint64_t id, uint64_t off, uint64_t need, const char* what, void** out) {
    if (id == 0) {
        *out = nullptr;
        return need == 0 ? AGRAD_OK : set_error(AGRAD_EINVAL, "%s: null buffer", what);
    }
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->allocs.upper_bound(id);
    if (it == ctx->allocs.begin()) return set_error(AGRAD_EINVAL, "%s: buffer id 0x%llx is not an allocation of this context", what, (unsigned long long)id);
    --it;
    const uint64_t base = it->first, size = it->second;
    if (id < base || id >= base + size)
        return set_error(AGRAD_EINVAL, "%s: buffer id 0x%llx is not an allocation of this context", what, (unsigned long long)id);
    const uint64_t begin = (id - base) + off;
    if (begin > size || need > size - begin)
        return set_error(AGRAD_EINVAL, "%s: range [%llu, +%llu) outside a %llu-byte buffer", what,
                         (unsigned long long)begin, (unsigned long long)need, (unsigned long long)size);
    *out = reinterpret_cast<void*>(id + off);
    return AGRAD_OK;
}

int no_capture(agrad_ctx* ctx, const char* what) {
    if (ctx->capturing) return set_error(AGRAD_EINVAL, "%s cannot be recorded into a graph (it waits for the GPU)", what);
    return AGRAD_OK;
}

// folds every pending column sum (one launch per kFinalizeManyJobs of them)
int flush_pending(agrad_ctx* ctx) {
    if (ctx->pending.empty()) return AGRAD_OK;
    const int rc = launch_colsum_finalize_many(ctx->stream, ctx->pending.data(), ctx->pending.size());
    ctx->pending.clear();
    return rc;
}

// a backward entry point's scope: with AGRAD_DEFER_PARAM_GRAD in its flags, the finalize
// launches it would make are appended to the context's pending list instead
struct DeferScope : ColsumDefer {
    DeferScope(agrad_ctx* ctx, uint32_t flags) : ColsumDefer((flags & AGRAD_DEFER_PARAM_GRAD) ? &ctx->pending : nullptr) {}
};

int finish_stream(agrad_ctx* ctx) {
    if (int rc = no_capture(ctx, "synchronize / end_pass")) return rc;
    if (int rc = flush_pending(ctx)) return rc;      // nothing a caller waits for stays unfolded
    if (int rc = check_hip(hipStreamSynchronize(ctx->stream), "stream synchronize")) return rc;
    if (ctx->err_host[1] != 0) {               // (the stream has drained: every kernel's write has landed)
        ctx->err_host[0] = ctx->err_host[1] = 0;
        return set_error(AGRAD_EHIP, "fused cross-entropy: a team of workgroups did not assemble in time; the gradient "
                                     "it left is not valid");
    }
    if (*ctx->err_host != 0) {
        *ctx->err_host = 0;
        return set_error(AGRAD_EINDEX, "index out of range on the device (a token id or a class label)");
    }
    return AGRAD_OK;
}

// ---- name-based dispatch table ------------------------------------------------
struct Operand {
    void* p;
};
struct Call {
    agrad_ctx* ctx;
    const uint64_t* ids;
    const uint64_t* offs;
    int nbuf;
    const uint32_t* a;
    int nargs;
};
typedef int (*Handler)(const Call&);
struct Entry {
    const char* name;
    int nbuf, nargs;
    const char* signature;
    Handler fn;
};

inline uint64_t u64(const uint32_t* a, int lo) { return (uint64_t)a[lo] | ((uint64_t)a[lo + 1] << 32); }
inline float f32(uint32_t bits) { float f; std::memcpy(&f, &bits, 4); return f; }
inline bool dtype_ok(uint32_t d) { return d == AGRAD_F32 || d == AGRAD_BF16; }

#define RESOLVE(i, need, var)                                                             \
    void* var = nullptr;                                                                  \
    if (int rc_ = resolve(c.ctx, c.ids[i], c.offs[i], (need), #var, &var)) return rc_;
#define RESOLVE_IF(cond, i, need, var)                                                    \
    void* var = nullptr;                                                                  \
    if (cond) { if (int rc_ = resolve(c.ctx, c.ids[i], c.offs[i], (need), #var, &var)) return rc_; }
#define NEED_DTYPE(d) if (!dtype_ok(d)) return set_error(AGRAD_EINVAL, "unknown dtype %u", (unsigned)(d));

int h_fill(const Call& c) {
    const uint64_t n = u64(c.a, 1);
    RESOLVE(0, n * 4, out)
    return launch_fill(c.ctx->stream, out, c.a[0], 4, n);
}
int h_fill2(const Call& c) {
    const uint32_t itemsize = c.a[1];
    if (itemsize != 1 && itemsize != 2 && itemsize != 4) return set_error(AGRAD_EINVAL, "fill: itemsize %u", itemsize);
    const uint64_t n = u64(c.a, 2);
    RESOLVE(0, n * itemsize, out)
    return launch_fill(c.ctx->stream, out, c.a[0], (int)itemsize, n);
}
int h_copy(const Call& c) {
    const uint64_t n = u64(c.a, 0);
    RESOLVE(0, n, src) RESOLVE(1, n, dst)
    return launch_copy(c.ctx->stream, src, dst, n);
}
int h_add_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 1), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, x) RESOLVE(1, bytes, y) RESOLVE(2, bytes, out)
    return launch_add(c.ctx->stream, c.a[0], x, y, out, n);
}
int h_add_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 2), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, src) RESOLVE(1, bytes, dst)
    return launch_accumulate(c.ctx->stream, c.a[0], src, dst, n, c.a[1]);
}
// buffers x, y, out | args dtype, lead lo, hi, inner lo, hi
int h_bcast_add(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t lead = u64(c.a, 1), inner = u64(c.a, 3), es = dtype_size(c.a[0]);
    RESOLVE(0, lead * inner * es, x) RESOLVE(1, inner * es, y) RESOLVE(2, lead * inner * es, out)
    return launch_broadcast_add(c.ctx->stream, (int)c.a[0], x, y, out, lead, inner);
}
// buffers g, dy, workspace | args dtype, lead lo, hi, inner lo, hi, flags, ws lo, hi, present_mask
int h_bcast_grad(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t lead = u64(c.a, 1), inner = u64(c.a, 3), es = dtype_size(c.a[0]), wsb = u64(c.a, 6);
    RESOLVE(0, lead * inner * es, g) RESOLVE(1, inner * ((c.a[5] & AGRAD_PARAM_GRAD_BF16) ? 2 : es), dy)
    RESOLVE_IF(c.a[8] & 4u, 2, wsb, ws)
    DeferScope defer(c.ctx, c.a[5]);
    return launch_broadcast_grad(c.ctx->stream, (int)c.a[0], g, dy, ws, ws ? wsb : 0, lead, inner, c.a[5]);
}
// buffers x, y | args dtype, op, n lo, hi
int h_unary_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 2), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, x) RESOLVE(1, bytes, y)
    return launch_unary_fwd(c.ctx->stream, (int)c.a[1], (int)c.a[0], x, y, n);
}
// buffers dy, saved, dx | args dtype, op, flags, n lo, hi
int h_unary_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 3), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, dy) RESOLVE(1, bytes, saved) RESOLVE(2, bytes, dx)
    return launch_unary_bwd(c.ctx->stream, (int)c.a[1], (int)c.a[0], dy, saved, dx, n, c.a[2]);
}
inline uint64_t mul_small_elems(uint32_t kind, uint64_t lead, uint64_t inner) {
    return kind == AGRAD_MUL_SAME ? lead * inner : kind == AGRAD_MUL_ROW ? inner : kind == AGRAD_MUL_COL ? lead : 1;
}
// buffers x, y, out | args dtype, kind, lead lo, hi, inner lo, hi
int h_mul_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    if (c.a[1] > AGRAD_MUL_SCALAR) return set_error(AGRAD_EINVAL, "mul: unknown broadcast kind %u", c.a[1]);
    const uint64_t lead = u64(c.a, 2), inner = u64(c.a, 4), es = dtype_size(c.a[0]);
    RESOLVE(0, lead * inner * es, x) RESOLVE(1, mul_small_elems(c.a[1], lead, inner) * es, y) RESOLVE(2, lead * inner * es, out)
    return launch_mul_fwd(c.ctx->stream, (int)c.a[0], (int)c.a[1], x, y, out, lead, inner);
}
// buffers g, x, y, dx, dy, workspace | args dtype, kind, lead lo, hi, inner lo, hi, flags, ws lo, hi, present_mask
int h_mul_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    if (c.a[1] > AGRAD_MUL_SCALAR) return set_error(AGRAD_EINVAL, "mul backward: unknown broadcast kind %u", c.a[1]);
    const uint64_t lead = u64(c.a, 2), inner = u64(c.a, 4), es = dtype_size(c.a[0]), wsb = u64(c.a, 7);
    const uint64_t big = lead * inner * es, small = mul_small_elems(c.a[1], lead, inner) * es;
    const uint32_t mask = c.a[9];
    RESOLVE(0, big, g)
    RESOLVE_IF(mask & 2u, 1, big, x) RESOLVE_IF(mask & 4u, 2, small, y)
    RESOLVE_IF(mask & 8u, 3, big, dx) RESOLVE_IF(mask & 16u, 4, small, dy)
    RESOLVE_IF(mask & 32u, 5, wsb, ws)
    DeferScope defer(c.ctx, c.a[6]);
    return launch_mul_bwd(c.ctx->stream, (int)c.a[0], (int)c.a[1], g, x, y, dx, dy, ws, ws ? wsb : 0, lead, inner, c.a[6]);
}
// buffers x, y | args dtype, rows lo, hi, V
int h_softmax_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1), bytes = rows * c.a[3] * dtype_size(c.a[0]);
    RESOLVE(0, bytes, x) RESOLVE(1, bytes, y)
    return launch_softmax_fwd(c.ctx->stream, (int)c.a[0], x, y, rows, c.a[3]);
}
// buffers y, dy, dx | args dtype, rows lo, hi, V, flags
int h_softmax_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1), bytes = rows * c.a[3] * dtype_size(c.a[0]);
    RESOLVE(0, bytes, y) RESOLVE(1, bytes, dy) RESOLVE(2, bytes, dx)
    return launch_softmax_bwd(c.ctx->stream, (int)c.a[0], y, dy, dx, rows, c.a[3], c.a[4]);
}
int h_cast_down(const Call& c) {
    const uint64_t n = u64(c.a, 1);
    RESOLVE(0, n * 4, src) RESOLVE(1, n * 2, dst)
    return launch_cast_f32_bf16(c.ctx->stream, src, dst, n, c.a[0] != 0);
}
// buffers src, dst | args dtype, flags, ndim, shape[8], (stride lo, hi)[8]; slots past ndim are ignored
int h_strided_copy(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint32_t ndim = c.a[2];
    if (ndim > AGRAD_MAX_DIMS) return set_error(AGRAD_EINVAL, "strided copy: %u dimensions (at most %d)", ndim, AGRAD_MAX_DIMS);
    uint32_t shape[AGRAD_MAX_DIMS];
    uint64_t strides[AGRAD_MAX_DIMS];
    uint64_t numel = 1;
    for (uint32_t i = 0; i < ndim; ++i) {
        shape[i] = c.a[3 + i];
        strides[i] = u64(c.a, 3 + AGRAD_MAX_DIMS + 2 * (int)i);
        if (shape[i] != 0 && numel > 0xffffffffffffull / shape[i]) return set_error(AGRAD_EINVAL, "strided copy: shape too large");
        numel *= shape[i];
        if (shape[i] > 1 && strides[i] > 0xffffffffffffull / shape[i]) return set_error(AGRAD_EINVAL, "strided copy: stride too large");
    }
    if (numel == 0) return AGRAD_OK;
    const uint64_t es = dtype_size(c.a[0]);
    RESOLVE(0, strided_extent((int)ndim, shape, strides) * es, src) RESOLVE(1, numel * es, dst)
    return launch_strided_copy(c.ctx->stream, (int)c.a[0], src, dst, (int)ndim, shape, strides, c.a[1]);
}
int h_cast_up(const Call& c) {
    const uint64_t n = u64(c.a, 0);
    RESOLVE(0, n * 2, src) RESOLVE(1, n * 4, dst)
    return launch_cast_bf16_f32(c.ctx->stream, src, dst, n);
}

// buffers x, residual, gamma, beta, h, y | args dtype, rows, C, eps_bits, present
template <int KIND>
int h_norm_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = c.a[1];
    const uint32_t C = c.a[2], present = c.a[4];
    const uint64_t act = rows * C * dtype_size(c.a[0]), par = (uint64_t)C * 4;
    RESOLVE(0, act, x)
    RESOLVE_IF(present & 2u, 1, act, res)
    RESOLVE_IF(present & 4u, 2, par, gamma)
    RESOLVE_IF(present & 8u, 3, par, beta)
    RESOLVE_IF(present & 16u, 4, act, h)
    RESOLVE(5, act, y)
    return launch_norm_fwd(c.ctx->stream, KIND, c.a[0], x, res, (const float*)gamma, (const float*)beta,
                           h, y, rows, C, f32(c.a[3]));
}

// buffers x, dy, gamma, dres, dx, dx2, dgamma, dbeta, workspace
// args dtype, rows, C, eps_bits, flags, present, ws_bytes lo, hi
template <int KIND>
int h_norm_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = c.a[1];
    const uint32_t C = c.a[2], flags = c.a[4], present = c.a[5];
    const uint64_t ws_bytes = u64(c.a, 6);
    const uint64_t act = rows * C * dtype_size(c.a[0]), par = (uint64_t)C * 4;
    const uint64_t gpar = (flags & AGRAD_PARAM_GRAD_BF16) ? (uint64_t)C * 2 : par;     // dgamma / dbeta element size
    RESOLVE(0, act, x) RESOLVE(1, act, dy)
    RESOLVE_IF(present & 4u, 2, par, gamma)
    RESOLVE_IF(present & 8u, 3, act, dres)
    RESOLVE_IF(present & 16u, 4, act, dx)
    RESOLVE_IF(present & 32u, 5, act, dx2)
    RESOLVE_IF(present & 64u, 6, gpar, dgamma)
    RESOLVE_IF(present & 128u, 7, gpar, dbeta)
    RESOLVE_IF(present & 256u, 8, ws_bytes, ws)
    DeferScope defer(c.ctx, flags);
    return launch_norm_bwd(c.ctx->stream, KIND, c.a[0], x, dy, (const float*)gamma, dres, dx, dx2,
                           (float*)dgamma, (float*)dbeta, ws, ws ? ws_bytes : 0, rows, C, f32(c.a[3]), flags);
}

// buffers x, y | args dtype, n lo, hi
template <int WHICH>
int h_act_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 1), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, x) RESOLVE(1, bytes, y)
    return WHICH == 0 ? launch_gelu_fwd(c.ctx->stream, c.a[0], x, y, n)
                      : launch_relu2_fwd(c.ctx->stream, c.a[0], x, y, n);
}
// buffers dy, x, dx (the reference's order, backend.py:2951-2955) | args dtype, flags, n lo, hi
template <int WHICH>
int h_act_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t n = u64(c.a, 2), bytes = n * dtype_size(c.a[0]);
    RESOLVE(0, bytes, dy) RESOLVE(1, bytes, x) RESOLVE(2, bytes, dx)
    return WHICH == 0 ? launch_gelu_bwd(c.ctx->stream, c.a[0], x, dy, dx, n, c.a[1])
                      : launch_relu2_bwd(c.ctx->stream, c.a[0], x, dy, dx, n, c.a[1]);
}
// buffers h, b, out (the reference's order, metal_ops.metal:3737-3744) | args dtype, rows lo, hi, C
int h_gelu_bias_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1), es = dtype_size(c.a[0]);
    RESOLVE(0, rows * c.a[3] * es, h) RESOLVE(1, (uint64_t)c.a[3] * es, b) RESOLVE(2, rows * c.a[3] * es, out)
    return launch_gelu_bias_fwd(c.ctx->stream, (int)c.a[0], h, b, out, rows, c.a[3]);
}
// buffers dy, h, b, dh (the reference's order, metal_ops.metal:3753-3760), db, workspace
// args dtype, rows lo, hi, C, flags, ws lo, hi, present_mask
int h_gelu_bias_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1), es = dtype_size(c.a[0]), wsb = u64(c.a, 5);
    const uint64_t big = rows * c.a[3] * es, small = (uint64_t)c.a[3] * es;
    RESOLVE(0, big, dy) RESOLVE(1, big, h) RESOLVE(2, small, b) RESOLVE_IF(c.a[7] & 8u, 3, big, dh)
    RESOLVE_IF(c.a[7] & 16u, 4, (c.a[4] & AGRAD_PARAM_GRAD_BF16) ? (uint64_t)c.a[3] * 2 : small, db) RESOLVE_IF(c.a[7] & 32u, 5, wsb, ws)
    DeferScope defer(c.ctx, c.a[4]);
    return launch_gelu_bias_bwd(c.ctx->stream, (int)c.a[0], dy, h, b, dh, db, ws, ws ? wsb : 0, rows, c.a[3], c.a[4]);
}
// buffers gu, h | args dtype, rows, H
int h_swiglu_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = c.a[1], hb = rows * c.a[2] * dtype_size(c.a[0]);
    RESOLVE(0, 2 * hb, gu) RESOLVE(1, hb, h)
    return launch_swiglu_fwd(c.ctx->stream, c.a[0], gu, h, rows, c.a[2]);
}
// buffers gu, hidden_tile | args dtype, then the reference's N, H, h0, h (backend.py:3910-3913)
int h_swiglu_tile(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = c.a[1], es = dtype_size(c.a[0]);
    RESOLVE(0, rows * 2 * c.a[2] * es, gu) RESOLVE(1, rows * c.a[4] * es, tile)
    return launch_swiglu_fwd_tile(c.ctx->stream, c.a[0], gu, tile, rows, c.a[2], c.a[3], c.a[4]);
}
// buffers gu, dh, dgu | args dtype, rows, H, flags
int h_swiglu_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = c.a[1], hb = rows * c.a[2] * dtype_size(c.a[0]);
    RESOLVE(0, 2 * hb, gu) RESOLVE(1, hb, dh) RESOLVE(2, 2 * hb, dgu)
    return launch_swiglu_bwd(c.ctx->stream, c.a[0], gu, dh, dgu, rows, c.a[2], c.a[3]);
}
// buffers q, k, cos, sin | args dtype, B, T, H, HKV, D, hf_sign, backward, present
template <int BHTD>
int h_rope(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint32_t B = c.a[1], T = c.a[2], H = c.a[3], HKV = c.a[4], D = c.a[5], present = c.a[8];
    const uint64_t tok = (uint64_t)B * T, es = dtype_size(c.a[0]);
    RESOLVE(0, tok * H * D * es, q)
    RESOLVE_IF(present & 2u, 1, tok * HKV * D * es, k)
    RESOLVE(2, (uint64_t)T * (D / 2) * 4, cs) RESOLVE(3, (uint64_t)T * (D / 2) * 4, sn)
    return launch_rope(c.ctx->stream, c.a[0], q, k, (const float*)cs, (const float*)sn, B, T, H, HKV, D,
                       c.a[6] ? 1 : -1, c.a[7] != 0, BHTD);
}
// buffers ids, W, out | args dtype, N, C, V
int h_gather_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1], es = dtype_size(c.a[0]);
    const uint32_t C = c.a[2], V = c.a[3];
    RESOLVE(0, N * 4, ids) RESOLVE(1, (uint64_t)V * C * es, W) RESOLVE(2, N * C * es, out)
    return launch_gather_fwd(c.ctx->stream, c.a[0], (const int32_t*)ids, W, nullptr, out, N, 1, C, V, c.ctx->err_flag);
}
// buffers ids, W, wpe, out | args dtype, N, T, C, V
int h_embed_sum_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1], es = dtype_size(c.a[0]);
    const uint32_t T = c.a[2], C = c.a[3], V = c.a[4];
    RESOLVE(0, N * 4, ids) RESOLVE(1, (uint64_t)V * C * es, W) RESOLVE(2, (uint64_t)T * C * es, wpe)
    RESOLVE(3, N * C * es, out)
    return launch_gather_fwd(c.ctx->stream, c.a[0], (const int32_t*)ids, W, wpe, out, N, T, C, V, c.ctx->err_flag);
}
// buffers ids, dY, dW, workspace | args dtype, N, C, V, flags, ws_bytes lo, hi
int h_gather_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1], es = dtype_size(c.a[0]), ws_bytes = u64(c.a, 5);
    const uint32_t C = c.a[2], V = c.a[3];
    const uint64_t gs = (c.a[4] & AGRAD_PARAM_GRAD_BF16) ? 2 : es;      // element size of the table gradient
    RESOLVE(0, N * 4, ids) RESOLVE(1, N * C * es, dY) RESOLVE(2, (uint64_t)V * C * gs, dW)
    RESOLVE(3, ws_bytes, ws)
    return launch_embedding_bwd(c.ctx->stream, c.a[0], (const int32_t*)ids, dY, dW, ws, ws_bytes, N, C, V,
                                c.a[4], c.ctx->err_flag);
}
// buffers ids, W, wpe, out, order, sort_ws, kept_ids | args dtype, N, T, C, V, ws lo, hi, present_mask
int h_gather_fwd_sorted(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1], es = dtype_size(c.a[0]), wsb = u64(c.a, 5);
    const uint32_t T = c.a[2], C = c.a[3], V = c.a[4], mask = c.a[7];
    RESOLVE(0, N * 4, ids) RESOLVE(1, (uint64_t)V * C * es, W)
    RESOLVE_IF(mask & 4u, 2, (uint64_t)T * C * es, wpe)
    RESOLVE(3, N * C * es, out) RESOLVE(4, (N * 6 + 128) * 4, order) RESOLVE(5, wsb, ws)
    RESOLVE_IF(mask & 64u, 6, N * 4, kept)
    return launch_gather_fwd_sorted(c.ctx->stream, (int)c.a[0], (const int32_t*)ids, W, wpe, out, N, T, C, V,
                                    (uint32_t*)order, ws, wsb, c.ctx->err_flag, (int32_t*)kept);
}
// buffers order, dY, dW, workspace, dwpe | args dtype, N, C, V, flags, ws lo, hi, T, present mask
int h_gather_bwd_sorted(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1], es = dtype_size(c.a[0]), wsb = u64(c.a, 5);
    const uint32_t C = c.a[2], V = c.a[3], T = c.a[7], mask = c.a[8];
    const uint64_t gs = (c.a[4] & AGRAD_PARAM_GRAD_BF16) ? 2 : es;      // element size of the table gradients
    RESOLVE(0, (N * 6 + 128) * 4, order) RESOLVE(1, N * C * es, dY) RESOLVE(2, (uint64_t)V * C * gs, dW) RESOLVE(3, wsb, ws)
    RESOLVE_IF(mask & 16u, 4, (uint64_t)T * C * gs, dwpe)
    return launch_embedding_bwd_sorted(c.ctx->stream, (int)c.a[0], (uint32_t*)order, dY, dW, dwpe, ws, wsb, N, T,
                                       C, V, c.a[4]);
}
// buffers dY, dwpe | args dtype, B, T, C, flags
int h_pos_grad(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t es = dtype_size(c.a[0]), tc = (uint64_t)c.a[2] * c.a[3] * es;
    RESOLVE(0, tc * c.a[1], dY) RESOLVE(1, (c.a[4] & AGRAD_PARAM_GRAD_BF16) ? tc / es * 2 : tc, dwpe)
    return launch_pos_embedding_bwd(c.ctx->stream, c.a[0], dY, dwpe, c.a[1], c.a[2], c.a[3], c.a[4]);
}

// buffers logits, labels, loss, lse | args dtype, rows lo, hi, V, present_mask
int h_ce_fwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1);
    const uint32_t V = c.a[3], mask = c.a[4];
    RESOLVE(0, rows * V * dtype_size(c.a[0]), logits) RESOLVE(1, rows * 4, labels) RESOLVE(2, rows * 4, loss)
    RESOLVE_IF(mask & 8u, 3, rows * 4, lse)
    return launch_ce_fwd(c.ctx->stream, (int)c.a[0], logits, (const int32_t*)labels, (float*)loss, (float*)lse,
                         rows, V, c.ctx->err_flag);
}
// buffers logits, labels, dloss, lse, dlogits | args dtype, rows lo, hi, V, flags, present_mask
int h_ce_bwd(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t rows = u64(c.a, 1);
    const uint32_t V = c.a[3], mask = c.a[5];
    const uint64_t bytes = rows * V * dtype_size(c.a[0]);
    RESOLVE(0, bytes, logits) RESOLVE(1, rows * 4, labels) RESOLVE(2, rows * 4, dloss)
    RESOLVE_IF(mask & 8u, 3, rows * 4, lse)
    RESOLVE(4, bytes, dlogits)
    return launch_ce_bwd(c.ctx->stream, (int)c.a[0], logits, (const int32_t*)labels, (const float*)dloss,
                         (const float*)lse, dlogits, rows, V, c.a[4], c.ctx->err_flag);
}
// buffers logits, targets, row_loss, lse_out (the reference's order, metal_ops.metal:8808-8817), then row_scale when ROW_SCALED
// args rows, V, row_base, scale_bits (ROW_SCALED: total_rows, unused), write_grad, dtype, present_mask
template <bool ROW_SCALED>
int h_ce_fused(const Call& c) {
    NEED_DTYPE(c.a[5])
    const uint64_t rows = c.a[0], row_base = c.a[2];
    const uint32_t V = c.a[1], mask = c.a[6];
    const uint64_t upto = (row_base + rows) * 4;
    RESOLVE(0, rows * V * dtype_size(c.a[5]), logits) RESOLVE(1, upto, targets)
    RESOLVE_IF(mask & 4u, 2, upto, row_loss) RESOLVE_IF(mask & 8u, 3, upto, lse)
    void* row_scale = nullptr;
    if (ROW_SCALED) { if (int rc_ = resolve(c.ctx, c.ids[4], c.offs[4], upto, "row_scale", &row_scale)) return rc_; }
    return launch_ce_fused(c.ctx->stream, (int)c.a[5], logits, (const int32_t*)targets, (float*)row_loss, (float*)lse,
                           (const float*)row_scale, rows, V, row_base, ROW_SCALED ? 1.0f : f32(c.a[3]), c.a[4], c.ctx->ce_scratch, c.ctx->err_flag, c.ctx->team_polls);
}
// buffers ids, order, sort_workspace, zero_dst | args N, V, ws_lo, ws_hi, zero_lo, zero_hi, present_mask
int h_emb_order(const Call& c) {
    const uint64_t N = c.a[0], wsb = u64(c.a, 2), zb = u64(c.a, 4);
    RESOLVE(0, N * 4, ids) RESOLVE(1, embedding_order_bytes(N), order) RESOLVE(2, wsb, ws)
    RESOLVE_IF(c.a[6] & 8u, 3, zb, zero_dst)
    return launch_embedding_order(c.ctx->stream, (const int32_t*)ids, (uint32_t*)order, ws, wsb, N, c.a[1], zero_dst,
                                  zero_dst ? zb : 0, c.ctx->err_flag);
}
// buffers rows, dW | args dtype, N, C, V
int h_emb_grad_reset(const Call& c) {
    NEED_DTYPE(c.a[0])
    const uint64_t N = c.a[1];
    RESOLVE(0, N * 4, rows) RESOLVE(1, (uint64_t)c.a[2] * c.a[3] * dtype_size(c.a[0]), dW)
    return launch_embedding_grad_reset(c.ctx->stream, (int)c.a[0], (const int32_t*)rows, N, dW, c.a[2], c.a[3]);
}
// buffers p, g, m, v | args (float bits) lr_wd, b1, 1-b1, b2, 1-b2, eps, step_lr, inv_sqrt_bc2, grad_scale,
//                       then numel lo, hi, decay_numel lo, hi, grad dtype
int h_adamw(const Call& c) {
    NEED_DTYPE(c.a[13])
    const uint64_t n = u64(c.a, 9), dn = u64(c.a, 11);
    RESOLVE(0, n * 4, p) RESOLVE(1, n * dtype_size(c.a[13]), g) RESOLVE(2, n * 4, m) RESOLVE(3, n * 4, v)
    return launch_adamw(c.ctx->stream, (int)c.a[13], (float*)p, g, (float*)m, (float*)v, n, dn, f32(c.a[0]),
                        f32(c.a[1]), f32(c.a[2]), f32(c.a[3]), f32(c.a[4]), f32(c.a[5]), f32(c.a[6]),
                        f32(c.a[7]), f32(c.a[8]));
}
// buffers p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v; args decay, lr_bc1, b1, b2, eps (float
// bits), numel, decay_numel, first_step, inv_sqrt_bc2 (bits), grad_bf16, clip_coef (bits) -- the
// reference's own list (Backend.adamw8bit_step, backend.py:5142-5151)
int h_adamw8bit(const Call& c) {
    const uint64_t n = c.a[5], blocks = (n + 255) / 256;
    const int gd = c.a[9] ? AGRAD_BF16 : AGRAD_F32;
    RESOLVE(0, n * 4, p) RESOLVE(1, n * dtype_size(gd), g) RESOLVE(2, n, qm) RESOLVE(3, n, qv)
    RESOLVE(4, blocks * 4, am) RESOLVE(5, blocks * 4, av) RESOLVE(6, 1024, mapm) RESOLVE(7, 1024, mapv)
    return launch_adamw8bit(c.ctx->stream, gd, (float*)p, g, (uint8_t*)qm, (uint8_t*)qv, (float*)am, (float*)av,
                            (const float*)mapm, (const float*)mapv, n, c.a[6], f32(c.a[0]), f32(c.a[1]), f32(c.a[2]),
                            f32(c.a[3]), f32(c.a[4]), f32(c.a[8]), f32(c.a[10]), (int)c.a[7]);
}
// buffers g, partial | args numel lo, hi, dtype
int h_grad_norm(const Call& c) {
    NEED_DTYPE(c.a[2])
    const uint64_t n = u64(c.a, 0);
    RESOLVE(0, n * dtype_size(c.a[2]), g) RESOLVE(1, grad_norm_groups(n) * 4, partial)
    return launch_grad_norm_sq(c.ctx->stream, (int)c.a[2], g, (float*)partial, n);
}

const Entry kTable[] = {
    {"fill_scalar_kernel", 1, 3, "out | bits, n_lo, n_hi", h_fill},
    {"fill_scalar_kernel2", 1, 4, "out | bits, itemsize, n_lo, n_hi", h_fill2},
    {"copy_kernel", 2, 2, "src, dst | nbytes_lo, nbytes_hi", h_copy},
    {"add_residual_forward", 3, 3, "x, y, out | dtype, n_lo, n_hi", h_add_fwd},
    {"add_residual_backward", 2, 4, "g, dst | dtype, flags, n_lo, n_hi", h_add_bwd},
    {"add_broadcast_forward", 3, 5, "x, y, out | dtype, lead_lo, lead_hi, inner_lo, inner_hi", h_bcast_add},
    {"add_broadcast_backward", 3, 9, "g, dy, workspace | dtype, lead_lo, lead_hi, inner_lo, inner_hi, flags, ws_lo, ws_hi, present_mask", h_bcast_grad},
    {"fp32_to_bf16", 2, 3, "src, dst | accumulate, n_lo, n_hi", h_cast_down},
    {"bf16_to_fp32", 2, 2, "src, dst | n_lo, n_hi", h_cast_up},
    {"unary_forward", 2, 4, "x, y | dtype, op, n_lo, n_hi", h_unary_fwd},
    {"unary_backward", 3, 5, "dy, saved, dx | dtype, op, flags, n_lo, n_hi", h_unary_bwd},
    {"mul_forward_kernel", 3, 6, "x, y, out | dtype, kind, lead_lo, lead_hi, inner_lo, inner_hi", h_mul_fwd},
    {"mul_backward_kernel", 6, 10, "g, x, y, dx, dy, workspace | dtype, kind, lead_lo, lead_hi, inner_lo, inner_hi, flags, ws_lo, ws_hi, present_mask", h_mul_bwd},
    {"softmax_forward", 2, 4, "x, y | dtype, rows_lo, rows_hi, V", h_softmax_fwd},
    {"softmax_backward", 3, 5, "y, dy, dx | dtype, rows_lo, rows_hi, V, flags", h_softmax_bwd},
    {"contiguous_forward_kernel", 2, 27, "src, dst | dtype, flags, ndim, shape[8], stride_lo_hi[8]", h_strided_copy},
    {"strided_add_backward_kernel", 2, 27, "src, dst | dtype, flags, ndim, shape[8], stride_lo_hi[8]", h_strided_copy},
    {"layernorm_forward", 6, 5, "x, residual, gamma, beta, h, y | dtype, rows, C, eps_bits, present_mask", h_norm_fwd<AGRAD_NORM_LAYER>},
    {"rmsnorm_forward", 6, 5, "x, residual, gamma, beta, h, y | dtype, rows, C, eps_bits, present_mask", h_norm_fwd<AGRAD_NORM_RMS>},
    {"layernorm_backward_kernel", 9, 8, "x, dy, gamma, dres, dx, dx2, dgamma, dbeta, workspace | dtype, rows, C, eps_bits, flags, present_mask, ws_lo, ws_hi", h_norm_bwd<AGRAD_NORM_LAYER>},
    {"rmsnorm_backward", 9, 8, "x, dy, gamma, dres, dx, dx2, dgamma, dbeta, workspace | dtype, rows, C, eps_bits, flags, present_mask, ws_lo, ws_hi", h_norm_bwd<AGRAD_NORM_RMS>},
    {"gelu_forward_kernel", 2, 3, "x, y | dtype, n_lo, n_hi", h_act_fwd<0>},
    {"gelu_backward_kernel", 3, 4, "dy, x, dx | dtype, flags, n_lo, n_hi", h_act_bwd<0>},
    {"gelu_add_bias_kernel", 3, 4, "h, b, out | dtype, rows_lo, rows_hi, C", h_gelu_bias_fwd},
    {"gelu_backward_bias_kernel", 6, 8, "dy, h, b, dh, db, workspace | dtype, rows_lo, rows_hi, C, flags, ws_lo, ws_hi, present_mask", h_gelu_bias_bwd},
    {"relu2_forward_kernel", 2, 3, "x, y | dtype, n_lo, n_hi", h_act_fwd<1>},
    {"relu2_backward_kernel", 3, 4, "dy, x, dx | dtype, flags, n_lo, n_hi", h_act_bwd<1>},
    {"swiglu_forward_kernel", 2, 3, "gu, h | dtype, rows, H", h_swiglu_fwd},
    {"swiglu_forward_tile_kernel", 2, 5, "gu, hidden_tile | dtype, rows, H, h0, h", h_swiglu_tile},
    {"swiglu_backward_kernel", 3, 4, "gu, dh, dgu | dtype, rows, H, flags", h_swiglu_bwd},
    {"rope_qk_inplace", 4, 9, "q, k, cos, sin | dtype, B, T, H, HKV, D, hf_sign, backward, present_mask", h_rope<0>},
    {"rope_qk_inplace_bhtd", 4, 9, "q, k, cos, sin | dtype, B, T, H, HKV, D, hf_sign, backward, present_mask", h_rope<1>},
    {"gather_forward_kernel", 3, 4, "ids, W, out | dtype, N, C, V", h_gather_fwd},
    {"embedding_sum_forward", 4, 5, "ids, W, wpe, out | dtype, N, T, C, V", h_embed_sum_fwd},
    {"gather_backward_kernel", 4, 7, "ids, dY, dW, workspace | dtype, N, C, V, flags, ws_lo, ws_hi", h_gather_bwd},
    {"gather_forward_sorted", 7, 8, "ids, W, wpe, out, order, sort_workspace, kept_ids | dtype, N, T, C, V, ws_lo, ws_hi, present_mask", h_gather_fwd_sorted},
    {"gather_backward_sorted", 5, 9, "order, dY, dW, workspace, dwpe | dtype, N, C, V, flags, ws_lo, ws_hi, T, present_mask", h_gather_bwd_sorted},
    {"pos_emb_grad", 2, 5, "dY, dwpe | dtype, B, T, C, flags", h_pos_grad},
    {"cross_entropy_forward", 4, 5, "logits, labels, loss, lse | dtype, rows_lo, rows_hi, V, present_mask", h_ce_fwd},
    {"cross_entropy_backward", 5, 6, "logits, labels, dloss, lse, dlogits | dtype, rows_lo, rows_hi, V, flags, present_mask", h_ce_bwd},
    {"fused_linear_ce_logits_to_dlogits", 4, 7, "logits (in place), targets, row_loss, lse_out | rows, V, row_base, scale_bits, write_grad, dtype, present_mask", h_ce_fused<false>},
    {"fused_linear_ce_logits_to_dlogits_row_scaled", 5, 7, "logits (in place), targets, row_loss, lse_out, row_scale | rows, V, row_base, total_rows, write_grad, dtype, present_mask", h_ce_fused<true>},
    {"embedding_order", 4, 7, "ids, order, sort_workspace, zero_dst | N, V, ws_lo, ws_hi, zero_lo, zero_hi, present_mask", h_emb_order},
    {"embedding_grad_reset", 2, 4, "rows, dW | dtype, N, C, V", h_emb_grad_reset},
    {"adamw_step", 4, 14, "p, g, m, v | lr_wd, b1, one_minus_b1, b2, one_minus_b2, eps, step_lr, inv_sqrt_bc2, grad_scale (float bits), n_lo, n_hi, decay_lo, decay_hi, grad_dtype", h_adamw},
    {"adamw8bit_step", 8, 11, "p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v | decay, lr_bc1, b1, b2, eps (float bits), numel, decay_numel, first_step, inv_sqrt_bc2 (bits), grad_bf16, clip_coef (bits)", h_adamw8bit},
    {"grad_norm_sq", 2, 3, "g, partial | n_lo, n_hi, dtype", h_grad_norm},
};
constexpr int kTableSize = (int)(sizeof(kTable) / sizeof(kTable[0]));

const Entry* find_entry(const char* name) {
    if (name == nullptr) return nullptr;
    for (int i = 0; i < kTableSize; ++i)
        if (std::strcmp(kTable[i].name, name) == 0) return &kTable[i];
    return nullptr;
}

}  // namespace
}  // namespace agrad

using namespace agrad;

#define CTX_OR_FAIL(ctx) \
    if ((ctx) == nullptr) return set_error(AGRAD_EINVAL, "null context"); \
    DeviceGuard guard_(ctx);

extern "C" {

const char* agrad_last_error(void) { return g_last_error.c_str(); }

int agrad_device_count(int* count) {
    if (count == nullptr) return set_error(AGRAD_EINVAL, "null count");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { *count = 0; return check_hip(e, "hipGetDeviceCount"); }
    *count = n;
    return AGRAD_OK;
}

int agrad_ctx_create(int device, agrad_ctx** out) {
    if (out == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *out = nullptr;
    int n = 0;
    if (int rc = check_hip(hipGetDeviceCount(&n), "hipGetDeviceCount")) return rc;
    if (device < 0 || device >= n) return set_error(AGRAD_EINVAL, "device %d out of range (%d visible)", device, n);
    if (int rc = check_hip(hipSetDevice(device), "hipSetDevice")) return rc;
    hipDeviceProp_t prop;
    if (int rc = check_hip(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties")) return rc;
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(AGRAD_EHIP, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    if (int rc = norm_noalloc_setup(device)) return rc;   // this GPU's address of the fixed scratch array
    agrad_ctx* c = new agrad_ctx();
    c->device = device;
    c->total_mem = prop.totalGlobalMem;
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_start);
    if (e == hipSuccess) e = hipEventCreate(&c->ev_stop);
    void* pinned = nullptr;
    if (e == hipSuccess) e = hipHostMalloc(&pinned, 256, hipHostMallocMapped);
    if (e == hipSuccess) {
        std::memset(pinned, 0, 256);
        c->err_host = static_cast<volatile int*>(pinned);
        e = hipHostGetDevicePointer((void**)&c->err_flag, pinned, 0);
    }
    if (e == hipSuccess) e = hipMalloc(&c->ce_scratch, ce_fused_scratch_bytes());
    if (e != hipSuccess) {
        agrad_ctx_destroy(c);
        return check_hip(e, "context setup");
    }
    *out = c;
    return AGRAD_OK;
}

int agrad_ctx_destroy(agrad_ctx* ctx) {
    if (ctx == nullptr) return AGRAD_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (auto& kv : ctx->graphs) (void)hipGraphExecDestroy(kv.second);
    for (auto& kv : ctx->allocs) (void)hipFree(reinterpret_cast<void*>(kv.first));
    if (ctx->ce_scratch) (void)hipFree(ctx->ce_scratch);
    if (ctx->err_host) (void)hipHostFree(const_cast<int*>(ctx->err_host));
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return AGRAD_OK;
}

int agrad_max_buffer_length(agrad_ctx* ctx, uint64_t* bytes) {
    CTX_OR_FAIL(ctx)
    if (bytes == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *bytes = ctx->total_mem;
    return AGRAD_OK;
}

int agrad_alloc(agrad_ctx* ctx, uint64_t bytes, uint64_t* buffer_id) {
    CTX_OR_FAIL(ctx)
    if (buffer_id == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *buffer_id = 0;
    void* p = nullptr;
    const uint64_t want = bytes ? bytes : 1;
    if (int rc = check_hip(hipMalloc(&p, want), "hipMalloc")) return rc;
    std::lock_guard<std::mutex> lock(ctx->mu);
    ctx->allocs[reinterpret_cast<uint64_t>(p)] = want;
    *buffer_id = reinterpret_cast<uint64_t>(p);
    return AGRAD_OK;
}

int agrad_free(agrad_ctx* ctx, uint64_t buffer_id) {
    CTX_OR_FAIL(ctx)
    if (int rc = no_capture(ctx, "free")) return rc;
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        auto it = ctx->allocs.find(buffer_id);
        if (it == ctx->allocs.end()) return set_error(AGRAD_EINVAL, "free: 0x%llx is not a live buffer id", (unsigned long long)buffer_id);
        ctx->allocs.erase(it);
    }
    if (int rc = check_hip(hipStreamSynchronize(ctx->stream), "stream synchronize")) return rc;
    return check_hip(hipFree(reinterpret_cast<void*>(buffer_id)), "hipFree");
}

int agrad_begin_pass(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    return AGRAD_OK;  // kernels are enqueued eagerly on the in-order stream
}

int agrad_end_pass(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    return finish_stream(ctx);
}

int agrad_synchronize(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    return finish_stream(ctx);
}

int agrad_copy_from_host(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset, const void* src, uint64_t nbytes) {
    CTX_OR_FAIL(ctx)
    if (nbytes == 0) return AGRAD_OK;
    if (src == nullptr) return set_error(AGRAD_EINVAL, "copy_from_host: null source");
    if (int rc = no_capture(ctx, "copy_from_host")) return rc;
    void* dst = nullptr;
    if (int rc = resolve(ctx, buffer_id, offset, nbytes, "copy_from_host", &dst)) return rc;
    if (int rc = check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, ctx->stream), "hipMemcpyAsync H2D")) return rc;
    return check_hip(hipStreamSynchronize(ctx->stream), "stream synchronize");
}

int agrad_copy_to_host(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset, void* dst, uint64_t nbytes) {
    CTX_OR_FAIL(ctx)
    if (nbytes == 0) return AGRAD_OK;
    if (dst == nullptr) return set_error(AGRAD_EINVAL, "copy_to_host: null destination");
    if (int rc = no_capture(ctx, "copy_to_host")) return rc;
    void* src = nullptr;
    if (int rc = resolve(ctx, buffer_id, offset, nbytes, "copy_to_host", &src)) return rc;
    if (int rc = check_hip(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, ctx->stream), "hipMemcpyAsync D2H")) return rc;
    return check_hip(hipStreamSynchronize(ctx->stream), "stream synchronize");
}

int agrad_fill(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset, uint32_t bits, int itemsize, uint64_t n) {
    CTX_OR_FAIL(ctx)
    if (itemsize != 1 && itemsize != 2 && itemsize != 4) return set_error(AGRAD_EINVAL, "fill: itemsize %d not in {1, 2, 4}", itemsize);
    void* dst = nullptr;
    if (int rc = resolve(ctx, buffer_id, offset, n * (uint64_t)itemsize, "fill", &dst)) return rc;
    return launch_fill(ctx->stream, dst, bits, itemsize, n);
}

int agrad_stream(agrad_ctx* ctx, void** stream) {
    CTX_OR_FAIL(ctx)
    if (stream == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *stream = (void*)ctx->stream;
    return AGRAD_OK;
}

int agrad_timer_start(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    if (int rc = no_capture(ctx, "timer")) return rc;
    return check_hip(hipEventRecord(ctx->ev_start, ctx->stream), "hipEventRecord");
}

int agrad_timer_stop(agrad_ctx* ctx, float* elapsed_ms) {
    CTX_OR_FAIL(ctx)
    if (elapsed_ms == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    if (int rc = no_capture(ctx, "timer")) return rc;
    if (int rc = check_hip(hipEventRecord(ctx->ev_stop, ctx->stream), "hipEventRecord")) return rc;
    if (int rc = check_hip(hipEventSynchronize(ctx->ev_stop), "hipEventSynchronize")) return rc;
    return check_hip(hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop), "hipEventElapsedTime");
}

// ---- graphs: record the launches between begin and end once, replay them as one submission ----
int agrad_graph_begin(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    if (ctx->capturing) return set_error(AGRAD_EINVAL, "graph capture is already open");
    if (int rc = flush_pending(ctx)) return rc;     // what was left pending before the recording is not part of it
    // relaxed mode: allocations and queries made by other code meanwhile stay legal
    if (int rc = check_hip(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture")) return rc;
    ctx->capturing = true;
    set_capturing(true);
    return AGRAD_OK;
}

int agrad_graph_end(agrad_ctx* ctx, uint64_t* graph_id) {
    CTX_OR_FAIL(ctx)
    if (graph_id == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *graph_id = 0;
    if (!ctx->capturing) return set_error(AGRAD_EINVAL, "no graph capture is open");
    const int flush_rc = flush_pending(ctx);       // column sums left pending inside the recording are folded inside it
    ctx->capturing = false;
    set_capturing(false);
    hipGraph_t graph = nullptr;
    if (int rc = check_hip(hipStreamEndCapture(ctx->stream, &graph), "hipStreamEndCapture")) return rc;
    if (flush_rc != AGRAD_OK) { if (graph) (void)hipGraphDestroy(graph); return flush_rc; }
    if (graph == nullptr) return set_error(AGRAD_EHIP, "graph capture was invalidated");
    hipGraphExec_t exec = nullptr;
    const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (int rc = check_hip(e, "hipGraphInstantiate")) return rc;
    std::lock_guard<std::mutex> lock(ctx->mu);
    const uint64_t id = ctx->next_graph++;
    ctx->graphs[id] = exec;
    *graph_id = id;
    return AGRAD_OK;
}

int agrad_graph_launch(agrad_ctx* ctx, uint64_t graph_id) {
    CTX_OR_FAIL(ctx)
    if (int rc = no_capture(ctx, "graph launch")) return rc;
    hipGraphExec_t exec = nullptr;
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        auto it = ctx->graphs.find(graph_id);
        if (it == ctx->graphs.end()) return set_error(AGRAD_EINVAL, "graph %llu does not exist", (unsigned long long)graph_id);
        exec = it->second;
    }
    return check_hip(hipGraphLaunch(exec, ctx->stream), "hipGraphLaunch");
}

int agrad_graph_destroy(agrad_ctx* ctx, uint64_t graph_id) {
    CTX_OR_FAIL(ctx)
    if (int rc = no_capture(ctx, "graph destroy")) return rc;
    hipGraphExec_t exec = nullptr;
    {
        std::lock_guard<std::mutex> lock(ctx->mu);
        auto it = ctx->graphs.find(graph_id);
        if (it == ctx->graphs.end()) return set_error(AGRAD_EINVAL, "graph %llu does not exist", (unsigned long long)graph_id);
        exec = it->second;
        ctx->graphs.erase(it);
    }
    if (int rc = check_hip(hipStreamSynchronize(ctx->stream), "stream synchronize")) return rc;
    return check_hip(hipGraphExecDestroy(exec), "hipGraphExecDestroy");
}

int agrad_dispatch(agrad_ctx* ctx, const char* name, const uint64_t* buffer_ids, const uint64_t* offsets,
                   int n_buffers, const uint32_t* args, int n_args,
                   uint64_t gx, uint64_t gy, uint64_t gz, uint64_t tg) {
    (void)gx; (void)gy; (void)gz; (void)tg;
    CTX_OR_FAIL(ctx)
    const Entry* e = find_entry(name);
    if (e == nullptr) return set_error(AGRAD_ENOKERNEL, "no kernel named '%s'", name ? name : "(null)");
    if (n_buffers != e->nbuf || n_args != e->nargs)
        return set_error(AGRAD_EINVAL, "%s expects %d buffers and %d args (%s), got %d and %d", e->name,
                         e->nbuf, e->nargs, e->signature, n_buffers, n_args);
    if ((n_buffers > 0 && (buffer_ids == nullptr || offsets == nullptr)) || (n_args > 0 && args == nullptr))
        return set_error(AGRAD_EINVAL, "%s: null argument list", e->name);
    Call c{ctx, buffer_ids, offsets, n_buffers, args, n_args};
    return e->fn(c);
}

int agrad_kernel_count(void) { return kTableSize; }
const char* agrad_kernel_name(int index) { return (index >= 0 && index < kTableSize) ? kTable[index].name : nullptr; }
const char* agrad_kernel_signature(const char* name) {
    const Entry* e = find_entry(name);
    return e ? e->signature : nullptr;
}

// ---- typed entry points --------------------------------------------------------

int agrad_add_forward(agrad_ctx* ctx, int dtype, const void* x, const void* y, void* out, uint64_t n) {
    CTX_OR_FAIL(ctx)
    return launch_add(ctx->stream, dtype, x, y, out, n);
}
int agrad_grad_accumulate(agrad_ctx* ctx, int dtype, const void* src, void* dst, uint64_t n, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_accumulate(ctx->stream, dtype, src, dst, n, flags);
}
int agrad_cast_f32_to_bf16(agrad_ctx* ctx, const void* src, void* dst, uint64_t n, int accumulate) {
    CTX_OR_FAIL(ctx)
    return launch_cast_f32_bf16(ctx->stream, src, dst, n, accumulate);
}
int agrad_unary_forward(agrad_ctx* ctx, int op, int dtype, const void* x, void* y, uint64_t n) {
    CTX_OR_FAIL(ctx)
    return launch_unary_fwd(ctx->stream, op, dtype, x, y, n);
}
int agrad_unary_backward(agrad_ctx* ctx, int op, int dtype, const void* dy, const void* saved, void* dx, uint64_t n,
                         uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_unary_bwd(ctx->stream, op, dtype, dy, saved, dx, n, flags);
}
int agrad_mul_forward(agrad_ctx* ctx, int dtype, int kind, const void* x, const void* y, void* out, uint64_t lead,
                      uint64_t inner) {
    CTX_OR_FAIL(ctx)
    return launch_mul_fwd(ctx->stream, dtype, kind, x, y, out, lead, inner);
}
uint64_t agrad_mul_backward_workspace_bytes(int kind, uint64_t lead, uint64_t inner) {
    return mul_bwd_workspace_bytes(kind, lead, inner);
}
int agrad_mul_backward(agrad_ctx* ctx, int dtype, int kind, const void* g, const void* x, const void* y, void* dx,
                       void* dy, void* workspace, uint64_t workspace_bytes, uint64_t lead, uint64_t inner,
                       uint32_t flags) {
    CTX_OR_FAIL(ctx)
    DeferScope defer(ctx, flags);
    return launch_mul_bwd(ctx->stream, dtype, kind, g, x, y, dx, dy, workspace, workspace_bytes, lead, inner, flags);
}
int agrad_softmax_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t rows, uint32_t V) {
    CTX_OR_FAIL(ctx)
    return launch_softmax_fwd(ctx->stream, dtype, x, y, rows, V);
}
int agrad_softmax_backward(agrad_ctx* ctx, int dtype, const void* y, const void* dy, void* dx, uint64_t rows,
                           uint32_t V, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_softmax_bwd(ctx->stream, dtype, y, dy, dx, rows, V, flags);
}
int agrad_strided_copy(agrad_ctx* ctx, int dtype, const void* src, void* dst, int ndim, const uint32_t* shape,
                       const uint64_t* strides, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    if (!dtype_ok((uint32_t)dtype)) return set_error(AGRAD_EINVAL, "unknown dtype %d", dtype);
    return launch_strided_copy(ctx->stream, dtype, src, dst, ndim, shape, strides, flags);
}
int agrad_cast_bf16_to_f32(agrad_ctx* ctx, const void* src, void* dst, uint64_t n) {
    CTX_OR_FAIL(ctx)
    return launch_cast_bf16_f32(ctx->stream, src, dst, n);
}
int agrad_copy(agrad_ctx* ctx, const void* src, void* dst, uint64_t nbytes) {
    CTX_OR_FAIL(ctx)
    return launch_copy(ctx->stream, src, dst, nbytes);
}

int agrad_norm_forward(agrad_ctx* ctx, int kind, int dtype, const void* x, const void* residual,
                       const float* gamma, const float* beta, void* h_out, void* y,
                       uint64_t rows, uint32_t C, float eps) {
    CTX_OR_FAIL(ctx)
    return launch_norm_fwd(ctx->stream, kind, dtype, x, residual, gamma, beta, h_out, y, rows, C, eps);
}
uint64_t agrad_norm_backward_workspace_bytes(uint64_t rows, uint32_t C, int dtype) {
    return norm_bwd_workspace_bytes(rows, C, dtype);
}
int agrad_norm_backward(agrad_ctx* ctx, int kind, int dtype, const void* x, const void* dy,
                        const float* gamma, const void* dres_in, void* dx, void* dx2,
                        float* dgamma, float* dbeta, void* workspace, uint64_t workspace_bytes,
                        uint64_t rows, uint32_t C, float eps, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    DeferScope defer(ctx, flags);
    return launch_norm_bwd(ctx->stream, kind, dtype, x, dy, gamma, dres_in, dx, dx2, dgamma, dbeta,
                           workspace, workspace_bytes, rows, C, eps, flags);
}
int agrad_norm_backward_noalloc(agrad_ctx* ctx, int kind, int dtype, const void* x, const void* dy,
                                const float* gamma, const void* dres_in, void* dx, void* dx2,
                                float* dgamma, float* dbeta, uint64_t rows, uint32_t C, float eps, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    if (flags & AGRAD_DEFER_PARAM_GRAD)
        return set_error(AGRAD_EINVAL, "norm backward (no allocation): the partial rows share one fixed array, so the "
                                       "column sums cannot be left pending (AGRAD_DEFER_PARAM_GRAD)");
    return launch_norm_bwd_noalloc(ctx->stream, ctx->device, kind, dtype, x, dy, gamma, dres_in, dx, dx2,
                                   dgamma, dbeta, rows, C, eps, flags);
}

int agrad_pending_param_grads(agrad_ctx* ctx, uint32_t* count) {
    CTX_OR_FAIL(ctx)
    if (count == nullptr) return set_error(AGRAD_EINVAL, "null out pointer");
    *count = (uint32_t)ctx->pending.size();
    return AGRAD_OK;
}
int agrad_finalize_param_grads(agrad_ctx* ctx) {
    CTX_OR_FAIL(ctx)
    return flush_pending(ctx);
}
int agrad_colsum_finalize_many(agrad_ctx* ctx, const agrad_colsum_job* jobs, uint32_t n_jobs) {
    CTX_OR_FAIL(ctx)
    if (n_jobs == 0) return AGRAD_OK;
    if (jobs == nullptr) return set_error(AGRAD_EINVAL, "column-sum finalize: null job list");
    std::vector<ColsumJob> list(n_jobs);
    for (uint32_t i = 0; i < n_jobs; ++i) {
        const agrad_colsum_job& j = jobs[i];
        if ((j.partial_a != nullptr) != (j.out_a != nullptr) || (j.partial_b != nullptr) != (j.out_b != nullptr))
            return set_error(AGRAD_EINVAL, "column-sum finalize: job %u has partial rows without a destination or the reverse", i);
        if (j.flags & ~(uint32_t)(AGRAD_ACC_PARAM_GRAD | AGRAD_PARAM_GRAD_BF16))
            return set_error(AGRAD_EINVAL, "column-sum finalize: job %u has unknown flag bits 0x%x", i, j.flags);
        list[i] = ColsumJob{j.partial_a, j.partial_b, j.out_a, j.out_b, j.partial_rows, j.C,
                            (j.flags & AGRAD_ACC_PARAM_GRAD) ? 1u : 0u, (j.flags & AGRAD_PARAM_GRAD_BF16) ? 1u : 0u};
    }
    return launch_colsum_finalize_many(ctx->stream, list.data(), list.size());
}
int agrad_norm_backward_partial(agrad_ctx* ctx, int kind, int dtype, const void* x, const void* dy,
                                const float* gamma, const void* dres_in, void* dx, void* dx2,
                                float* dgamma, float* dbeta, void* workspace, uint64_t workspace_bytes,
                                uint64_t rows, uint32_t C, float eps, uint32_t flags, agrad_colsum_job* job) {
    CTX_OR_FAIL(ctx)
    if (job == nullptr) return set_error(AGRAD_EINVAL, "norm backward (partial): null job pointer");
    std::memset(job, 0, sizeof(*job));
    std::vector<ColsumJob> sink;
    int rc;
    {
        ColsumDefer defer(&sink);
        rc = launch_norm_bwd(ctx->stream, kind, dtype, x, dy, gamma, dres_in, dx, dx2, dgamma, dbeta,
                             workspace, workspace_bytes, rows, C, eps, flags);
    }
    if (rc != AGRAD_OK || sink.empty()) return rc;        // (no dgamma / dbeta, or no rows: nothing is left to fold)
    const ColsumJob& j = sink[0];
    job->partial_a = j.pa; job->partial_b = j.pb; job->out_a = j.out_a; job->out_b = j.out_b;
    job->partial_rows = j.P; job->C = j.C;
    job->flags = (j.accumulate ? AGRAD_ACC_PARAM_GRAD : 0u) | (j.out_bf16 ? AGRAD_PARAM_GRAD_BF16 : 0u);
    return AGRAD_OK;
}

int agrad_gelu_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t n) {
    CTX_OR_FAIL(ctx)
    return launch_gelu_fwd(ctx->stream, dtype, x, y, n);
}
int agrad_gelu_bias_forward(agrad_ctx* ctx, int dtype, const void* h, const void* b, void* y, uint64_t rows, uint32_t C) {
    CTX_OR_FAIL(ctx)
    return launch_gelu_bias_fwd(ctx->stream, dtype, h, b, y, rows, C);
}
uint64_t agrad_gelu_bias_backward_workspace_bytes(uint64_t rows, uint32_t C) {
    return gelu_bias_backward_workspace_bytes(rows, C);
}
int agrad_gelu_bias_backward(agrad_ctx* ctx, int dtype, const void* dy, const void* h, const void* b, void* dh, void* db,
                             void* workspace, uint64_t workspace_bytes, uint64_t rows, uint32_t C, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    DeferScope defer(ctx, flags);
    return launch_gelu_bias_bwd(ctx->stream, dtype, dy, h, b, dh, db, workspace, workspace_bytes, rows, C, flags);
}
int agrad_gelu_backward(agrad_ctx* ctx, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_gelu_bwd(ctx->stream, dtype, x, dy, dx, n, flags);
}
int agrad_relu2_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t n) {
    CTX_OR_FAIL(ctx)
    return launch_relu2_fwd(ctx->stream, dtype, x, y, n);
}
int agrad_relu2_backward(agrad_ctx* ctx, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_relu2_bwd(ctx->stream, dtype, x, dy, dx, n, flags);
}
int agrad_swiglu_forward(agrad_ctx* ctx, int dtype, const void* gu, void* h, uint64_t rows, uint32_t H) {
    CTX_OR_FAIL(ctx)
    return launch_swiglu_fwd(ctx->stream, dtype, gu, h, rows, H);
}
int agrad_swiglu_forward_tile(agrad_ctx* ctx, int dtype, const void* gu, void* tile, uint64_t rows, uint32_t H,
                              uint32_t h0, uint32_t h) {
    CTX_OR_FAIL(ctx)
    return launch_swiglu_fwd_tile(ctx->stream, dtype, gu, tile, rows, H, h0, h);
}
int agrad_swiglu_backward(agrad_ctx* ctx, int dtype, const void* gu, const void* dh, void* dgu,
                          uint64_t rows, uint32_t H, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_swiglu_bwd(ctx->stream, dtype, gu, dh, dgu, rows, H, flags);
}

int agrad_rope_qk(agrad_ctx* ctx, int dtype, void* q, void* k, const float* cos_table, const float* sin_table,
                  uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D, int rope_sign, int backward) {
    CTX_OR_FAIL(ctx)
    return launch_rope(ctx->stream, dtype, q, k, cos_table, sin_table, B, T, H, HKV, D, rope_sign, backward);
}
int agrad_rope_qk_bhtd(agrad_ctx* ctx, int dtype, void* q, void* k, const float* cos_table, const float* sin_table,
                       uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D, int rope_sign, int backward) {
    CTX_OR_FAIL(ctx)
    return launch_rope(ctx->stream, dtype, q, k, cos_table, sin_table, B, T, H, HKV, D, rope_sign, backward, 1);
}

int agrad_gather_forward(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* W, const void* wpe,
                         void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V) {
    CTX_OR_FAIL(ctx)
    return launch_gather_fwd(ctx->stream, dtype, ids, W, wpe, out, N, T, C, V, ctx->err_flag);
}
uint64_t agrad_embedding_backward_workspace_bytes(uint64_t N, uint32_t C, uint32_t V, int dtype) {
    return embedding_bwd_workspace_bytes(N, C, V, dtype);
}
int agrad_embedding_backward(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* dY, void* dW,
                             void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t C,
                             uint32_t V, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_embedding_bwd(ctx->stream, dtype, ids, dY, dW, workspace, workspace_bytes, N, C, V,
                                flags, ctx->err_flag);
}
uint64_t agrad_embedding_sort_workspace_bytes(uint64_t N, uint32_t V) { return embedding_sort_workspace_bytes(N, V); }
int agrad_gather_forward_sorted(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* W, const void* wpe,
                                void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V,
                                uint32_t* order, void* sort_workspace, uint64_t sort_workspace_bytes) {
    CTX_OR_FAIL(ctx)
    return launch_gather_fwd_sorted(ctx->stream, dtype, ids, W, wpe, out, N, T, C, V, order, sort_workspace,
                                    sort_workspace_bytes, ctx->err_flag);
}
int agrad_gather_forward_sorted_kept(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* W, const void* wpe,
                                     void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V, uint32_t* order,
                                     void* sort_workspace, uint64_t sort_workspace_bytes, int32_t* ids_kept) {
    CTX_OR_FAIL(ctx)
    if (ids_kept == nullptr) return set_error(AGRAD_EINVAL, "gather: null buffer for the kept ids");
    return launch_gather_fwd_sorted(ctx->stream, dtype, ids, W, wpe, out, N, T, C, V, order, sort_workspace,
                                    sort_workspace_bytes, ctx->err_flag, ids_kept);
}
int agrad_embedding_order(agrad_ctx* ctx, const int32_t* ids, uint64_t N, uint32_t V, uint32_t* order,
                          void* sort_workspace, uint64_t sort_workspace_bytes, void* zero_dst, uint64_t zero_bytes) {
    CTX_OR_FAIL(ctx)
    return launch_embedding_order(ctx->stream, ids, order, sort_workspace, sort_workspace_bytes, N, V, zero_dst, zero_bytes,
                                  ctx->err_flag);
}
int agrad_embedding_grad_reset(agrad_ctx* ctx, int dtype, const int32_t* rows, uint64_t N, void* dW, uint32_t C,
                               uint32_t V) {
    CTX_OR_FAIL(ctx)
    return launch_embedding_grad_reset(ctx->stream, dtype, rows, N, dW, C, V);
}
uint64_t agrad_embedding_backward_sorted_workspace_bytes(uint64_t N, uint32_t C) {
    return embedding_bwd_sorted_workspace_bytes(N, C);
}
int agrad_embedding_backward_sorted(agrad_ctx* ctx, int dtype, uint32_t* order, const void* dY, void* dW,
                                    void* dwpe, void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t T,
                                    uint32_t C, uint32_t V, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_embedding_bwd_sorted(ctx->stream, dtype, order, dY, dW, dwpe, workspace, workspace_bytes, N, T, C, V,
                                       flags);
}
int agrad_pos_embedding_backward(agrad_ctx* ctx, int dtype, const void* dY, void* dwpe, uint32_t B,
                                 uint32_t T, uint32_t C, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_pos_embedding_bwd(ctx->stream, dtype, dY, dwpe, B, T, C, flags);
}

int agrad_broadcast_add_forward(agrad_ctx* ctx, int dtype, const void* x, const void* y, void* out,
                                uint64_t lead, uint64_t inner) {
    CTX_OR_FAIL(ctx)
    return launch_broadcast_add(ctx->stream, dtype, x, y, out, lead, inner);
}
uint64_t agrad_broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner) {
    return broadcast_grad_workspace_bytes(lead, inner);
}
int agrad_broadcast_add_backward(agrad_ctx* ctx, int dtype, const void* g, void* dy, void* workspace,
                                 uint64_t workspace_bytes, uint64_t lead, uint64_t inner, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    DeferScope defer(ctx, flags);
    return launch_broadcast_grad(ctx->stream, dtype, g, dy, workspace, workspace_bytes, lead, inner, flags);
}

int agrad_cross_entropy_forward(agrad_ctx* ctx, int dtype, const void* logits, const int32_t* labels,
                                float* loss, float* lse_out, uint64_t rows, uint32_t V) {
    CTX_OR_FAIL(ctx)
    return launch_ce_fwd(ctx->stream, dtype, logits, labels, loss, lse_out, rows, V, ctx->err_flag);
}
int agrad_cross_entropy_fused(agrad_ctx* ctx, int dtype, void* logits, const int32_t* targets, float* row_loss,
                              float* lse, const float* row_scale, uint64_t rows, uint32_t V, uint64_t row_base,
                              float scale, uint32_t write_grad) {
    CTX_OR_FAIL(ctx)
    return launch_ce_fused(ctx->stream, dtype, logits, targets, row_loss, lse, row_scale, rows, V, row_base, scale, write_grad,
                           ctx->ce_scratch, ctx->err_flag, ctx->team_polls);
}
int agrad_set_team_wait_polls(agrad_ctx* ctx, uint32_t polls) {
    CTX_OR_FAIL(ctx)
    ctx->team_polls = polls;
    return AGRAD_OK;
}
int agrad_cross_entropy_backward(agrad_ctx* ctx, int dtype, const void* logits, const int32_t* labels,
                                 const float* dloss, const float* lse, void* dlogits,
                                 uint64_t rows, uint32_t V, uint32_t flags) {
    CTX_OR_FAIL(ctx)
    return launch_ce_bwd(ctx->stream, dtype, logits, labels, dloss, lse, dlogits, rows, V, flags, ctx->err_flag);
}

int agrad_adamw8bit_step(agrad_ctx* ctx, int grad_dtype, float* p, const void* g, uint8_t* qm, uint8_t* qv,
                         float* absmax_m, float* absmax_v, const float* qmap_m, const float* qmap_v,
                         uint64_t numel, uint64_t decay_numel, float decay, float lr_bc1, float b1, float b2,
                         float eps, float inv_sqrt_bc2, float clip_coef, int first_step) {
    CTX_OR_FAIL(ctx)
    return launch_adamw8bit(ctx->stream, grad_dtype, p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v, numel,
                            decay_numel, decay, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip_coef, first_step);
}
int agrad_adamw_step(agrad_ctx* ctx, int grad_dtype, float* p, const void* g, float* m, float* v,
                     uint64_t numel, uint64_t decay_numel, float lr_wd, float b1, float one_minus_b1,
                     float b2, float one_minus_b2, float eps, float step_lr, float inv_sqrt_bc2,
                     float grad_scale) {
    CTX_OR_FAIL(ctx)
    return launch_adamw(ctx->stream, grad_dtype, p, g, m, v, numel, decay_numel, lr_wd, b1, one_minus_b1, b2,
                        one_minus_b2, eps, step_lr, inv_sqrt_bc2, grad_scale);
}
uint64_t agrad_grad_norm_groups(uint64_t numel) { return grad_norm_groups(numel); }
int agrad_grad_norm_sq(agrad_ctx* ctx, int dtype, const void* g, float* partial, uint64_t numel) {
    CTX_OR_FAIL(ctx)
    return launch_grad_norm_sq(ctx->stream, dtype, g, partial, numel);
}

}  // extern "C"
