/*
 * autograd_hip.h -- C ABI of libautograd_hip.so: the MI355X (gfx950) native layer
 * that takes the place of the reference's Metal extension for the fused
 * layer-op path (norms, activations, rotary, embedding gather / grad).
 *
 * Everything crosses the boundary as plain pointers, sizes and 32-bit words.
 * Device buffers are addressed the way the reference addresses Metal buffers:
 * an opaque buffer id (here: the device address returned by agrad_alloc) plus a
 * byte offset (storage.py:66-90).  All work is enqueued on the context's single
 * in-order HIP stream; agrad_end_pass / agrad_synchronize block until it drains
 * (metal_ext.mm:202-213, 763-767).
 *
 * Every function returns AGRAD_OK (0) or a negative AGRAD_E* code; the message
 * of the last failure on the calling thread is agrad_last_error().
 */
#ifndef AUTOGRAD_HIP_H
#define AUTOGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct agrad_ctx agrad_ctx;

enum {
    AGRAD_OK = 0,
    AGRAD_EINVAL = -1,      /* bad argument, shape or alignment            */
    AGRAD_EHIP = -2,        /* a HIP runtime call failed                   */
    AGRAD_ENOKERNEL = -3,   /* agrad_dispatch: unknown kernel name         */
    AGRAD_EINDEX = -4,      /* a token id outside [0, V) was seen on device */
    AGRAD_EWORKSPACE = -5   /* workspace too small                         */
};

/* Storage type of the large operands.  Arithmetic is always fp32.            */
enum { AGRAD_F32 = 0, AGRAD_BF16 = 1 };

/* Norm flavour.                                                              */
enum { AGRAD_NORM_LAYER = 0, AGRAD_NORM_RMS = 1 };

/* Flag bits for backward entry points.                                       */
enum {
    AGRAD_ACC_INPUT_GRAD = 1u, /* dx += ... (CPU semantics, backend.py:414,477-487); else dx = ... */
    AGRAD_ACC_PARAM_GRAD = 2u, /* dgamma/dbeta/dW += ...; else =                                   */
    AGRAD_ACC_INPUT_GRAD2 = 4u, /* norm backward: the same choice for the second output dx2        */
    AGRAD_ACC_PARAM_GRAD2 = 8u, /* sorted embedding backward: the same choice for dwpe             */
    AGRAD_PARAM_GRAD_BF16 = 16u, /* parameter gradients stored as bf16: the embedding backward with an fp32
                                 * upstream gradient (dW and dwpe; gather_backward_bf16_kernel,
                                 * metal_ops.metal:12395-12446) and the norm backward (dgamma and dbeta then
                                 * point at bf16; the bf16 option of rmsnorm_weighted_dgamma and
                                 * gqa_rms_dgamma_bf16, metal_ops.metal:12448-12479, 14541-14746), and the column
                                 * sums agrad_broadcast_add_backward / agrad_pos_embedding_backward / db of
                                 * agrad_gelu_bias_backward (bias_grad_reduce_bf16, metal_ops.metal:12101).  A sum is finished in fp32,
                                 * added to the stored value and rounded once */
    AGRAD_DEFER_PARAM_GRAD = 32u /* agrad_norm_backward, agrad_broadcast_add_backward, agrad_gelu_bias_backward and
                                 * agrad_mul_backward (row operand): the column sum over rows is left UNFOLDED -- the
                                 * partial rows stay in the call's workspace, the context remembers the job, and
                                 * agrad_finalize_param_grads folds all remembered jobs in one launch (see there).
                                 * The reference splits dgamma off the same way (rmsnorm_weighted_dgamma,
                                 * metal_ops.metal:14541-14746) */
};

/* ---- context, memory, passes --------------------------------------------
 * Replaces MetalContext() / alloc / free / max_buffer_length / begin_pass /
 * end_pass / synchronize / copy_* / fill_scalar* (metal_ext.mm:33-213, 444-510,
 * 723-767). */
const char* agrad_last_error(void);
int agrad_device_count(int* count);
int agrad_ctx_create(int device, agrad_ctx** out);
int agrad_ctx_destroy(agrad_ctx* ctx);
int agrad_max_buffer_length(agrad_ctx* ctx, uint64_t* bytes);
int agrad_alloc(agrad_ctx* ctx, uint64_t bytes, uint64_t* buffer_id);
int agrad_free(agrad_ctx* ctx, uint64_t buffer_id);
int agrad_begin_pass(agrad_ctx* ctx);
/* Blocks until the stream drains; returns AGRAD_EINDEX if any kernel since the
 * last check saw an out-of-range token id (numpy raises IndexError there,
 * backend.py:525-538). */
int agrad_end_pass(agrad_ctx* ctx);
int agrad_synchronize(agrad_ctx* ctx);
int agrad_copy_from_host(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset,
                         const void* src, uint64_t nbytes);
int agrad_copy_to_host(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset,
                       void* dst, uint64_t nbytes);
/* fill n items of itemsize 1, 2 or 4 bytes with the low bits of `bits`
 * (fill_scalar_kernel / fill_scalar_kernel2, metal_ops.metal:122-144). */
int agrad_fill(agrad_ctx* ctx, uint64_t buffer_id, uint64_t offset,
               uint32_t bits, int itemsize, uint64_t n);
/* The HIP stream of the context as a hipStream_t cast to void*.              */
int agrad_stream(agrad_ctx* ctx, void** stream);
/* Event timing on the context's stream (the role of begin_pass_profiled /
 * end_pass_profiled, metal_ext.mm:215-286): elapsed GPU ms between the two. */
int agrad_timer_start(agrad_ctx* ctx);
int agrad_timer_stop(agrad_ctx* ctx, float* elapsed_ms);

/* ---- name-based launch ----------------------------------------------------
 * Replaces MetalContext.dispatch_with_args_3d (metal_ext.mm:559-590): a kernel
 * name, parallel lists of buffer ids and byte offsets, and uint32 arguments
 * (floats travel as their bit pattern, backend.py:2916).  The launch geometry
 * is chosen here from the shape arguments; gx/gy/gz/tg are accepted so call
 * sites keep the reference's signature, and are ignored.  Unknown names fail
 * with AGRAD_ENOKERNEL (the reference silently binds a nil pipeline,
 * metal_ext.mm:567).  Kernel names and their operand lists are given by
 * agrad_kernel_signature. */
int agrad_dispatch(agrad_ctx* ctx, const char* name,
                   const uint64_t* buffer_ids, const uint64_t* offsets, int n_buffers,
                   const uint32_t* args, int n_args,
                   uint64_t gx, uint64_t gy, uint64_t gz, uint64_t tg);
int agrad_kernel_count(void);
const char* agrad_kernel_name(int index);
/* Human-readable "buffers | args" description of a kernel, or NULL.          */
const char* agrad_kernel_signature(const char* name);

/* ---- graphs -----------------------------------------------------------------
 * Launch-bound chains (ops of a few MB, where the ~4 us per launch dominates) can
 * be recorded once and replayed as one submission.  Between agrad_graph_begin
 * and agrad_graph_end every launch on the context's stream is recorded instead
 * of run; calls that wait for the GPU (synchronize, end_pass, host copies,
 * timers, free) fail with AGRAD_EINVAL, as does an embedding backward too large
 * for the one-launch sort.  Run the chain once eagerly first (kernels are loaded
 * on first use).  The recorded launches keep their addresses and sizes: replay
 * with the same buffers.  No counterpart in the reference (Metal command buffers
 * are re-encoded every pass, metal_ext.mm:202-213). */
int agrad_graph_begin(agrad_ctx* ctx);
int agrad_graph_end(agrad_ctx* ctx, uint64_t* graph_id);
int agrad_graph_launch(agrad_ctx* ctx, uint64_t graph_id);
int agrad_graph_destroy(agrad_ctx* ctx, uint64_t graph_id);

/* ---- typed entry points (device addresses, already offset) ----------------
 * `dtype` is the storage type of activations / gradients / embedding tables;
 * gamma, beta, dgamma, dbeta, cos, sin are always fp32; ids are int32.       */

/* out[i] = x[i] + y[i]  (cpu_add_forward, backend.py:74-76; add_residual_forward,
 * metal_ops.metal:161-181). */
int agrad_add_forward(agrad_ctx* ctx, int dtype, const void* x, const void* y, void* out, uint64_t n);
/* out[l, j] = x[l, j] + y[j] for x [lead, inner] and y of the trailing shape [inner]
 * (a bias, or a position table added to every batch entry: the broadcasting branch
 * of cpu_add_forward, backend.py:74-76; add_pos_forward, metal_ops.metal:205-218). */
int agrad_broadcast_add_forward(agrad_ctx* ctx, int dtype, const void* x, const void* y, void* out,
                                uint64_t lead, uint64_t inner);
/* dy[j] (+)= sum_l g[l, j], l ascending within a fixed two-level order (the
 * broadcasting branch of cpu_add_backward, backend.py:78-105; pos_emb_grad and
 * the bias-gradient column reductions, metal_ops.metal:220-234, 1002-1193).
 * AGRAD_ACC_PARAM_GRAD accumulates into dy.  With more than 64 leading rows the sum
 * runs in two stages through a workspace of agrad_broadcast_grad_workspace_bytes(lead,
 * inner) bytes (16-byte aligned; bf16 sums are finished in fp32 and rounded once).
 * fp32 needs it then; a bf16 call may pass NULL and gets a one-thread-per-column sum. */
uint64_t agrad_broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner);
int agrad_broadcast_add_backward(agrad_ctx* ctx, int dtype, const void* g, void* dy,
                                 void* workspace, uint64_t workspace_bytes,
                                 uint64_t lead, uint64_t inner, uint32_t flags);
/* dst[i] (+)= src[i]  (same-shape branch of cpu_add_backward, backend.py:78-105). */
int agrad_grad_accumulate(agrad_ctx* ctx, int dtype, const void* src, void* dst, uint64_t n, uint32_t flags);
/* dst_bf16[i] = rne(src_f32[i]) (+ dst if accumulate) (fp32_to_bf16, metal_ops.metal:12010-12041). */
int agrad_cast_f32_to_bf16(agrad_ctx* ctx, const void* src, void* dst, uint64_t n, int accumulate);
int agrad_cast_bf16_to_f32(agrad_ctx* ctx, const void* src, void* dst, uint64_t n);
/* The element-wise primitives Exp, Log and Rsqrt (op.py:187-204).
 *   forward   y = exp(x) | log(x) | 1 / sqrt(x)                  (cpu_exp_forward, cpu_log_forward,
 *                                                                  cpu_rsqrt_forward, backend.py:320-345)
 *   backward  dx (+)= dy * y | dy / x | (((dy * -0.5) * y) * y) * y;  `saved` is y for exp
 *             and rsqrt and x for log (cpu_*_backward, backend.py:324-352).
 * AGRAD_ACC_INPUT_GRAD accumulates into dx. */
enum { AGRAD_UNARY_EXP = 0, AGRAD_UNARY_LOG = 1, AGRAD_UNARY_RSQRT = 2 };
int agrad_unary_forward(agrad_ctx* ctx, int op, int dtype, const void* x, void* y, uint64_t n);
int agrad_unary_backward(agrad_ctx* ctx, int op, int dtype, const void* dy, const void* saved, void* dx,
                         uint64_t n, uint32_t flags);

/* Mul with the reference's broadcast kinds (mul_bcast_kind, utils.py:134-143): x is
 * [lead, inner]; y is the same shape (SAME), [inner] (ROW), [lead] -- one factor per
 * row (COL) -- or one element (SCALAR).  out = x * y (cpu_mul_forward, backend.py:107-111).
 * Backward (cpu_mul_backward, backend.py:113-146): dx (+)= g * y and dy (+)= the
 * product g * x summed over what y was broadcast along, in a fixed order; either may
 * be NULL.  AGRAD_ACC_INPUT_GRAD accumulates into dx, AGRAD_ACC_INPUT_GRAD2 into dy.
 * ROW (fp32, more than 64 rows) and SCALAR need agrad_mul_backward_workspace_bytes
 * bytes of 16-byte aligned workspace. */
enum { AGRAD_MUL_SAME = 0, AGRAD_MUL_ROW = 1, AGRAD_MUL_COL = 2, AGRAD_MUL_SCALAR = 3 };
int agrad_mul_forward(agrad_ctx* ctx, int dtype, int kind, const void* x, const void* y, void* out,
                      uint64_t lead, uint64_t inner);
uint64_t agrad_mul_backward_workspace_bytes(int kind, uint64_t lead, uint64_t inner);
int agrad_mul_backward(agrad_ctx* ctx, int dtype, int kind, const void* g, const void* x, const void* y,
                       void* dx, void* dy, void* workspace, uint64_t workspace_bytes,
                       uint64_t lead, uint64_t inner, uint32_t flags);

/* Softmax over the last axis of x[rows, V] (SoftmaxOp(dim=-1), op.py:205-218):
 *   forward   y = exp(x - max) / sum exp(x - max)    (cpu_softmax_forward, backend.py:354-362)
 *   backward  dx (+)= y * (dy - sum(dy * y))          (cpu_softmax_backward, backend.py:364-374)
 * y may be x (in place).  AGRAD_ACC_INPUT_GRAD accumulates into dx. */
int agrad_softmax_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t rows, uint32_t V);
int agrad_softmax_backward(agrad_ctx* ctx, int dtype, const void* y, const void* dy, void* dx,
                           uint64_t rows, uint32_t V, uint32_t flags);

/* Strided gather into a dense tensor: dst[dense index over shape] (+)=
 * src[sum_i coord_i * strides[i]], strides in elements (0 broadcasts), ndim <=
 * AGRAD_MAX_DIMS.  Contiguous forward of a permuted / transposed view and the
 * Permute / Transpose gradients (contiguous_forward_kernel and
 * strided_add_backward_kernel, metal_ops.metal:429-449, 1002-1023, bound through
 * dispatch_contiguous / dispatch_strided, metal_ext.mm:512-557; CPU:
 * cpu_permute_backward, cpu_transpose_backward, cpu_contiguous_forward,
 * backend.py:286-313).  Overwriting moves raw bits of any 2-byte (AGRAD_BF16) or
 * 4-byte (AGRAD_F32) element; AGRAD_ACC_INPUT_GRAD adds onto dst, as the CPU
 * backward kernels do.  src and dst may not overlap. */
#define AGRAD_MAX_DIMS 8
int agrad_strided_copy(agrad_ctx* ctx, int dtype, const void* src, void* dst, int ndim,
                       const uint32_t* shape, const uint64_t* strides, uint32_t flags);
/* plain device copy kernel; the calibration kernel for bandwidth and counters. */
int agrad_copy(agrad_ctx* ctx, const void* src, void* dst, uint64_t nbytes);

/* LayerNorm / RMSNorm forward over rows of width C.
 *   residual != NULL: h = x + residual is normalised; h is stored to h_out if non-NULL.
 *   gamma / beta may be NULL (weightless RMSNorm, backend.py:1097-1105).
 * LayerNorm: cpu_layernorm_forward (backend.py:416-433), layernorm_forward
 * (metal_ops.metal:3539-3649).  RMSNorm: backend.py:1097-1108, 1737-1745;
 * rmsnorm_forward / rmsnorm_weighted_forward (metal_ops.metal:3412-3537). */
int agrad_norm_forward(agrad_ctx* ctx, int kind, int dtype,
                       const void* x, const void* residual,
                       const float* gamma, const float* beta,
                       void* h_out, void* y,
                       uint64_t rows, uint32_t C, float eps);

/* Bytes of workspace agrad_norm_backward needs for the column reductions.    */
uint64_t agrad_norm_backward_workspace_bytes(uint64_t rows, uint32_t C, int dtype);
/* Norm backward.  x is the tensor that was normalised (h when a residual was
 * fused).  dx = [dx if ACC_INPUT_GRAD] + ([dres_in] + dnorm); dx2 (optional, the
 * second operand of a fused residual add) = [dx2 if ACC_INPUT_GRAD2] + the same.
 * dres_in may be the same buffer as dx or dx2 only when that output is stored.
 * dgamma / dbeta (optional) are reduced over rows in two deterministic stages.
 * cpu_layernorm_backward (backend.py:435-487); RMSNorm slices backend.py:1228-1251,
 * 1990-2011; rmsnorm_backward's fused residual_grad (metal_ops.metal:8107-8257). */
int agrad_norm_backward(agrad_ctx* ctx, int kind, int dtype,
                        const void* x, const void* dy, const float* gamma,
                        const void* dres_in, void* dx, void* dx2,
                        float* dgamma, float* dbeta,
                        void* workspace, uint64_t workspace_bytes,
                        uint64_t rows, uint32_t C, float eps, uint32_t flags);

/* One column sum that is still to be folded: out_a[c] (+)= sum over partial_rows rows of
 * partial_a[partial_rows, C], and the same for partial_b -> out_b (either pair may be NULL).
 * flags: AGRAD_ACC_PARAM_GRAD (add to what out_* holds), AGRAD_PARAM_GRAD_BF16 (out_* are bf16). */
typedef struct agrad_colsum_job {
    const float* partial_a;
    const float* partial_b;
    void* out_a;
    void* out_b;
    uint32_t partial_rows, C, flags, reserved;
} agrad_colsum_job;

/* The second launch of a column sum, amortised.  Every backward kernel that reduces over rows
 * (dgamma / dbeta of the norms, bias gradients) leaves one partial row per workgroup and folds
 * them with a second, tiny launch, which on this GPU costs about 4 us of launch floor whatever
 * its size: a fifth of a norm backward at 16384 x 384.  A network has dozens of such sums
 * per backward pass and needs none of them before the pass ends, so:
 *   - a backward call with AGRAD_DEFER_PARAM_GRAD in its flags runs its main kernel only and
 *     leaves the job with the context.  Its workspace must stay untouched, and may not be
 *     shared with another deferred call, until the jobs have been folded;
 *   - agrad_finalize_param_grads folds every job the context holds, 32 to a launch
 *     (blockIdx.z = job), each with exactly the workgroups, loads and additions of its own
 *     second launch: the same bits.  Jobs are folded in the order they were left; two jobs that
 *     write the same gradient (a gamma tied between two norms: one call stores, the next adds)
 *     go into separate launches, one after the other.  agrad_end_pass, agrad_synchronize, agrad_graph_begin and
 *     agrad_graph_end fold what is pending first, so nothing a caller waits for stays unfolded;
 *   - agrad_pending_param_grads reports how many jobs wait.
 * agrad_norm_backward_partial / agrad_colsum_finalize_many are the same two halves for callers
 * that keep the job list themselves.  The reference's closest precedent is its separate dgamma
 * kernel (rmsnorm_weighted_dgamma, metal_ops.metal:14541-14746; backend.py:4053-4068). */
int agrad_pending_param_grads(agrad_ctx* ctx, uint32_t* count);
int agrad_finalize_param_grads(agrad_ctx* ctx);
int agrad_colsum_finalize_many(agrad_ctx* ctx, const agrad_colsum_job* jobs, uint32_t n_jobs);
/* agrad_norm_backward without the fold of dgamma / dbeta: *job receives what is left to do
 * (partial_rows == 0 when nothing is: no dgamma and dbeta asked for, or no rows). */
int agrad_norm_backward_partial(agrad_ctx* ctx, int kind, int dtype,
                                const void* x, const void* dy, const float* gamma,
                                const void* dres_in, void* dx, void* dx2,
                                float* dgamma, float* dbeta,
                                void* workspace, uint64_t workspace_bytes,
                                uint64_t rows, uint32_t C, float eps, uint32_t flags,
                                agrad_colsum_job* job);

/* agrad_norm_backward for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc): no workspace
 * argument; the partial dgamma / dbeta rows go to a fixed array of
 * AGRAD_NOALLOC_SCRATCH_BYTES that the library keeps in each GPU's memory for the
 * life of the process, and the call makes no hipMalloc / hipFree.  Same kernels,
 * same launch geometry and same results, bit for bit, as agrad_norm_backward.
 * A problem whose partial rows (agrad_norm_backward_workspace_bytes(rows, C, dtype))
 * exceed the array is refused with AGRAD_EINVAL; without dgamma and dbeta any size
 * runs.  All calls on one GPU share the array: calls that overlap there race.  A call from
 * another stream (another context) than the last one's, while that stream still has work in
 * flight, is refused with AGRAD_EINVAL; a replaying graph beside eager calls is the caller's
 * to keep apart.  This entry point has no counterpart in the reference. */
#define AGRAD_NOALLOC_SCRATCH_BYTES (32u * 1024u * 1024u)
int agrad_norm_backward_noalloc(agrad_ctx* ctx, int kind, int dtype,
                                const void* x, const void* dy, const float* gamma,
                                const void* dres_in, void* dx, void* dx2,
                                float* dgamma, float* dbeta,
                                uint64_t rows, uint32_t C, float eps, uint32_t flags);

/* tanh-GELU (cpu_gelu_forward / backward, backend.py:376-414).               */
int agrad_gelu_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t n);
int agrad_gelu_backward(agrad_ctx* ctx, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags);
/* The bias add of a linear layer folded into its GELU: y[r, c] = GELU(h[r, c] + b[c])
 * for h of shape [rows, C] (gelu_add_bias_kernel / gelu_backward_bias_kernel,
 * metal_ops.metal:3737-3773; on the CPU cpu_add_forward, backend.py:74-88, followed
 * by cpu_gelu_forward, backend.py:376-395).  Backward: dh (+)= dy * GELU'(h + b)
 * (AGRAD_ACC_INPUT_GRAD accumulates) and, when db is not NULL, db[c] (+)= the sum
 * over rows of the same terms in a fixed order (AGRAD_ACC_PARAM_GRAD accumulates;
 * the reference runs bias_grad_reduce, metal_ops.metal:1026-1193, over dh
 * afterwards).  Either of dh and db may be NULL, not both.  With db the call needs
 * a 16-byte aligned workspace of agrad_gelu_bias_backward_workspace_bytes(rows, C)
 * bytes; without, none. */
int agrad_gelu_bias_forward(agrad_ctx* ctx, int dtype, const void* h, const void* b, void* y, uint64_t rows, uint32_t C);
uint64_t agrad_gelu_bias_backward_workspace_bytes(uint64_t rows, uint32_t C);
int agrad_gelu_bias_backward(agrad_ctx* ctx, int dtype, const void* dy, const void* h, const void* b, void* dh, void* db,
                             void* workspace, uint64_t workspace_bytes, uint64_t rows, uint32_t C, uint32_t flags);
/* ReLU^2: y = max(x,0)^2, dx = 2 max(x,0) dy.  No counterpart in the reference. */
int agrad_relu2_forward(agrad_ctx* ctx, int dtype, const void* x, void* y, uint64_t n);
int agrad_relu2_backward(agrad_ctx* ctx, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags);
/* SwiGLU on gu[rows, 2H] (gate = first H columns, up = last H): h = silu(g)*u.
 * Backward writes dgu[rows, 2H] = [dg | du]; dgu may alias gu (in place).
 * backend.py:1113-1126, 1178-1217; swiglu_forward_kernel /
 * swiglu_backward_inplace_kernel (metal_ops.metal:3808-4017). */
int agrad_swiglu_forward(agrad_ctx* ctx, int dtype, const void* gu, void* h, uint64_t rows, uint32_t H);
/* A column tile of the same forward: tile[r, c] = silu(gu[r, h0 + c]) * gu[r, H + h0 + c] for
 * c < h, written densely as [rows, h] (swiglu_forward_tile_kernel, metal_ops.metal:12043-12088;
 * the recompute of the hidden activations in column tiles, backend.py:3906-3913). */
int agrad_swiglu_forward_tile(agrad_ctx* ctx, int dtype, const void* gu, void* tile, uint64_t rows, uint32_t H,
                              uint32_t h0, uint32_t h);
int agrad_swiglu_backward(agrad_ctx* ctx, int dtype, const void* gu, const void* dh, void* dgu,
                          uint64_t rows, uint32_t H, uint32_t flags);

/* Split-half rotary embedding applied in place to q[B,T,H,D] and k[B,T,HKV,D]
 * (k may be NULL) with fp32 tables cos/sin[T, D/2]:
 *   lo' = lo*c - s*(hi*sin),  hi' = hi*c + s*(lo*sin),  s = rope_sign (+1 HF, -1 nanochat);
 * backward != 0 applies the transpose (s negated).
 * apply_rope_np / apply_rope_backward_np (backend.py:1382-1417), GQA loops
 * (backend.py:1755-1782, 1937-1958); rope_qk_inplace / gqa_rope_inplace
 * (metal_ops.metal:7423-7491, 11732-11747). */
int agrad_rope_qk(agrad_ctx* ctx, int dtype, void* q, void* k,
                  const float* cos_table, const float* sin_table,
                  uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D,
                  int rope_sign, int backward);
/* The same rotation for q[B,H,T,D] and k[B,HKV,T,D], the layout the attention kernels
 * work in (the layout flag of rope_qk_inplace mode 0 / gqa_rope_inplace,
 * metal_ops.metal:7458-7465, 11741; call sites backend.py:3764-3767, 3816-3824). */
int agrad_rope_qk_bhtd(agrad_ctx* ctx, int dtype, void* q, void* k,
                       const float* cos_table, const float* sin_table,
                       uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D,
                       int rope_sign, int backward);

/* out[n,:] = W[ids[n],:] (+ wpe[n % T,:] if wpe != NULL).
 * cpu_gather_forward (backend.py:525-529), gather_forward_kernel
 * (metal_ops.metal:390-404), add_pos_forward (metal_ops.metal:205-218). */
int agrad_gather_forward(agrad_ctx* ctx, int dtype, const int32_t* ids,
                         const void* W, const void* wpe, void* out,
                         uint64_t N, uint32_t T, uint32_t C, uint32_t V);

/* Embedding gradient dW[ids[n],:] += dY[n,:], deterministic: the rows are ordered
 * so that each token's rows are adjacent and ascending, and one launch then reads dY
 * once.  One wave adds the rows of a token with up to 127 rows in ascending row
 * order -- the sequence of fp32 adds np.add.at makes
 * (cpu_gather_backward, backend.py:531-538; replaces the float-atomic
 * gather_backward_kernel, metal_ops.metal:406-427).  A token with more rows is cut
 * into chunks of 64 rows, summed in row order each; the chunk sums are added in
 * chunk order in groups of 16, the groups in group order.  No float atomics; every
 * table row is written once, with the same bits on every run.
 * Without AGRAD_ACC_PARAM_GRAD the touched rows of dW are overwritten (correct on
 * a table that was just zero-filled); untouched rows are never written.
 * workspace: agrad_embedding_backward_workspace_bytes(N, C, V, dtype) bytes, 256-byte
 * aligned (the order of the ids, the sort's scratch, partial rows of long runs). */
uint64_t agrad_embedding_backward_workspace_bytes(uint64_t N, uint32_t C, uint32_t V, int dtype);
int agrad_embedding_backward(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* dY, void* dW,
                             void* workspace, uint64_t workspace_bytes,
                             uint64_t N, uint32_t C, uint32_t V, uint32_t flags);
/* The same pair with the ordering of the ids done in the forward call, where it
 * is free: up to 65536 rows the gather and the ordering are ONE launch (the
 * ordering workgroups run beside the bandwidth-bound gather), and the backward
 * call is one launch that reads dY front to back.  The forward call also writes
 * `order`, 6N + 128 uint32, 16-byte aligned: order[0..N) = the rows (in the low 30
 * bits: N < 2^30), each token's rows adjacent and ascending; bit 31 marks the first
 * row of a run of 2..127 rows and the first row of each 64-row chunk of a longer run
 * (the run's last chunk takes the rest), bit 30 those of them that start more than
 * 10 rows: what the backward call hands out as tasks.  Then, from the next multiple of four words on, four
 * words for row n = 0..N-1: its token (V for an id outside the table), the place
 * in order[] where its token's run starts, and (R, x): R = 0 for a row with
 * nothing to do (a later row of a run of up to 127 rows, an id outside the table);
 * 1..127 for the first row of such a run, x = the run's second row or 0xFFFFFFFF
 * (not given: it is order[start + 1]); for a longer run its length, x = the row's
 * index in the run.  The words after that are arrival counters of the backward
 * call's long runs: zero after the forward call and after every backward call.
 * sort_workspace (256-byte aligned, agrad_embedding_sort_workspace_bytes(N, V)
 * bytes) is free again when the forward call's work has run; the backward call's
 * workspace (16-byte aligned, agrad_embedding_backward_sorted_workspace_bytes(N, C)
 * bytes) holds the fp32 partial rows of runs longer than 127 rows.  Backward calls
 * that share one order buffer must not overlap in time.
 * Same results, bit for bit, as agrad_gather_forward + agrad_embedding_backward.
 * (The reference orders nothing: np.add.at, backend.py:531-538, and float
 * atomics, metal_ops.metal:406-427.) */
uint64_t agrad_embedding_sort_workspace_bytes(uint64_t N, uint32_t V);
int agrad_gather_forward_sorted(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* W, const void* wpe,
                                void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V,
                                uint32_t* order, void* sort_workspace, uint64_t sort_workspace_bytes);
/* The same call, which also leaves a copy of the N ids it read in ids_kept (not the ids'
 * own buffer): the list agrad_embedding_grad_reset needs after the backward call of this
 * order, in memory the caller's next batch of ids does not overwrite. */
int agrad_gather_forward_sorted_kept(agrad_ctx* ctx, int dtype, const int32_t* ids, const void* W, const void* wpe,
                                     void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V,
                                     uint32_t* order, void* sort_workspace, uint64_t sort_workspace_bytes,
                                     int32_t* ids_kept);
/* The ordering alone: writes `order` (same layout, same bits as the forward call above
 * leaves) from the ids, and -- when zero_dst is not NULL -- clears zero_dst[0 .. zero_bytes)
 * in the same launch, for a caller that zero-fills the table's gradient and orders the ids
 * before its forward pass and then calls the plain agrad_gather_forward.  One launch when
 * N <= 65536 and zero_dst / zero_bytes are multiples of 16; otherwise a fill and the ordering
 * one after the other.  The ids must already be what the forward pass will read.  Measured on
 * MI355X the forward gather is the better host for the ordering workgroups (they cost it 1 to
 * 3 us; the fill, which runs best with few waves on a CU, 3 to 25 us), so
 * agrad_gather_forward_sorted stays the default; this call is for callers whose forward pass
 * must be the plain gather.  The reference clears the table inside its forward gather
 * (metal_gather_forward, backend.py:2781-2785) and orders nothing. */
int agrad_embedding_order(agrad_ctx* ctx, const int32_t* ids, uint64_t N, uint32_t V, uint32_t* order,
                          void* sort_workspace, uint64_t sort_workspace_bytes,
                          void* zero_dst, uint64_t zero_bytes);
/* Clears the rows of dW[V, C] that `rows[0 .. N)` names (ids outside [0, V) are skipped):
 * N*C items written where a fill of the table writes V*C.  An embedding table's gradient
 * is zero outside the rows its backward call stored, so a caller that keeps the ids of
 * the last backward call can bring the table back to all-zero with this call instead of
 * agrad_fill once the optimizer has read it -- 1/3 to 1/50 of the fill's bytes at the
 * benchmark shapes.  The caller answers for the list: rows a backward call wrote that it
 * does not name stay as they are.  The reference clears the whole table on every forward
 * gather (metal_gather_forward, backend.py:2781-2785). */
int agrad_embedding_grad_reset(agrad_ctx* ctx, int dtype, const int32_t* rows, uint64_t N, void* dW,
                               uint32_t C, uint32_t V);
uint64_t agrad_embedding_backward_sorted_workspace_bytes(uint64_t N, uint32_t C);
/* `order` is read AND written: the call counts arrivals in the counters at its end and leaves
 * them zero again; they must be zero on entry, which the calls that write an order guarantee
 * and an interrupted backward call does not (write the order again after one).
 * dwpe may be NULL; otherwise it is the [T, C] position table's gradient
 * dwpe[t,:] (+)= sum_b dY[b,t,:] (N = B*T rows, b ascending), added up from the
 * same loads of dY that feed the table rows; AGRAD_ACC_PARAM_GRAD2 accumulates
 * into it. */
int agrad_embedding_backward_sorted(agrad_ctx* ctx, int dtype, uint32_t* order, const void* dY, void* dW,
                                    void* dwpe, void* workspace, uint64_t workspace_bytes,
                                    uint64_t N, uint32_t T, uint32_t C, uint32_t V, uint32_t flags);
/* dwpe[t,:] (+)= sum_b dY[b,t,:], b ascending (pos_emb_grad, metal_ops.metal:220-234;
 * broadcast branch of cpu_add_backward, backend.py:78-105). */
int agrad_pos_embedding_backward(agrad_ctx* ctx, int dtype, const void* dY, void* dwpe,
                                 uint32_t B, uint32_t T, uint32_t C, uint32_t flags);

/* ---- cross-entropy over the last axis (the loss that produces the upstream gradient) ---- */

/* loss[r] = -((x[r, labels[r]] - max_r) - log(sum_v exp(x[r, v] - max_r))) for logits
 * x[rows, V] (fp32 or bf16) and int32 labels (cpu_crossentropy_forward,
 * backend.py:489-503; CrossEntropyLossOp, op.py:269-284).  loss is fp32.  If
 * lse_out is not NULL it receives max_r + log(sum) per row (fp32) for the
 * backward pass.  A label outside [0, V) sets the deferred index error
 * (reported by agrad_end_pass / agrad_synchronize) and that row's loss is 0. */
int agrad_cross_entropy_forward(agrad_ctx* ctx, int dtype, const void* logits, const int32_t* labels,
                                float* loss, float* lse_out, uint64_t rows, uint32_t V);
/* dlogits[r, v] (+)= (exp(x[r, v] - lse[r]) - [v == labels[r]]) * dloss[r]
 * (cpu_crossentropy_backward, backend.py:505-524).  lse may be NULL: the row's
 * log-sum-exp is then recomputed first (one more read of the logits).
 * AGRAD_ACC_INPUT_GRAD accumulates into dlogits, otherwise it is overwritten. */
int agrad_cross_entropy_backward(agrad_ctx* ctx, int dtype, const void* logits, const int32_t* labels,
                                 const float* dloss, const float* lse, void* dlogits,
                                 uint64_t rows, uint32_t V, uint32_t flags);

/* Loss and gradient of a chunk of rows in ONE launch, in place
 * (fused_linear_ce_logits_to_dlogits and ..._row_scaled, metal_ops.metal:8808-9152; called behind the
 * output projection, backend.py:3175-3179, 3337-3342).  For local row r of logits[rows, V] and
 * g = row_base + r:  row_loss[g] = lse - x[r, targets[g]],  lse[g] = max + log(sum exp(x - max)), and -- when
 * write_grad is 1 -- logits[r, :] is REPLACED by (softmax(x[r, :]) - onehot(targets[g])) * s, with
 * s = row_scale[g] when row_scale is given, else `scale`.  A target outside [0, V) (an ignored position)
 * or a row without a finite logit gives loss 0, lse 0 and a zero row, as in the reference; no index
 * error is raised.  row_loss and lse may be NULL.  The row is read from memory once: a workgroup holds
 * it in registers between the statistics and the rewrite while it has at most 81920 fp32 or 163840
 * bf16 classes, and a team of up to 32 workgroups holds a slice each beyond that (the members exchange
 * one (max, sum) pair per slice through memory that the context owns, and wait for each other a
 * bounded number of polls: if a team does not assemble in time the call still ends, the gradient it
 * left is not valid, and the next agrad_end_pass / agrad_synchronize returns AGRAD_EHIP).  Rows that
 * start at odd addresses or have fewer than 16 bytes of classes are read twice.  The fp16 gradient
 * store of the reference (write_grad bit 1, which feeds its fp16 GEMM) is not built. */
int agrad_cross_entropy_fused(agrad_ctx* ctx, int dtype, void* logits, const int32_t* targets,
                              float* row_loss, float* lse, const float* row_scale,
                              uint64_t rows, uint32_t V, uint64_t row_base, float scale, uint32_t write_grad);
/* How many times a member of such a team looks for the others' pairs before it gives up
 * (0 = the default, about a second).  No counterpart in the reference; for callers that want a
 * tighter bound on a launch's worst case, and for the test of the give-up path. */
int agrad_set_team_wait_polls(agrad_ctx* ctx, uint32_t polls);

/* ---- optimizer step over the parameter slab (the consumer of the gradients above) ---- */

/* One AdamW step on numel fp32 parameters with fp32 moments, in place; the
 * gradient is fp32 or bf16 (grad_dtype).  Per element, each operation rounded
 * once, in the order of cpu_adamw_step (backend.py:2013-2038):
 *     g *= grad_scale                               (skipped when grad_scale == 1)
 *     p -= p * lr_wd                                (elements [0, decay_numel) only, and only if lr_wd != 0)
 *     m  = m*b1 + g*one_minus_b1
 *     v  = v*b2 + (g*g)*one_minus_b2
 *     p -= (m / (sqrt(v)*inv_sqrt_bc2 + eps)) * step_lr      (the multiply is skipped when inv_sqrt_bc2 == 1)
 * The reference's CPU path calls this with lr_wd = lr*weight_decay, step_lr =
 * lr*sqrt(1-b2^t)/(1-b1^t), inv_sqrt_bc2 = grad_scale = 1 (optimizer.py:443-446,
 * 488-498); its Metal path (Backend.adamw_step, backend.py:5122-5140; adamw_step,
 * metal_ops.metal:10139-10228) with step_lr = lr/(1-b1^t), inv_sqrt_bc2 =
 * 1/sqrt(1-b2^t), grad_scale = the clip coefficient and decay_numel = the
 * matrix-shaped prefix of a merged slab (optimizer.py:97-140).
 * one_minus_b1 / one_minus_b2 are separate arguments because the reference
 * forms 1.0 - b in double precision before rounding to fp32. */
int agrad_adamw_step(agrad_ctx* ctx, int grad_dtype, float* p, const void* g, float* m, float* v,
                     uint64_t numel, uint64_t decay_numel, float lr_wd, float b1, float one_minus_b1,
                     float b2, float one_minus_b2, float eps, float step_lr, float inv_sqrt_bc2,
                     float grad_scale);

/* One AdamW step with 8-bit moments (adamw8bit_step, metal_ops.metal:10229-10361;
 * Backend.adamw8bit_step, backend.py:5142-5151; optimizer.py:143-232, 469-479).
 * qm / qv hold one byte per element: an index into the 256-entry sorted maps qmap_m
 * (values in [-1, 1]) and qmap_v ([0, 1]); absmax_m / absmax_v hold one fp32 scale per
 * block of 256 elements ((numel + 255) / 256 of them).  Per element, each operation
 * rounded once, in the Metal kernel's order:
 *     m = absmax_m[blk] * qmap_m[qm], v = absmax_v[blk] * qmap_v[qv]     (both 0 when first_step)
 *     g *= clip_coef;  p *= decay                     (decay on elements [0, decay_numel) only)
 *     m += (g - m) * (1 - b1);  v += (g*g - v) * (1 - b2)
 *     p += -(m / (sqrt(max(v, 0)) * inv_sqrt_bc2 + eps)) * lr_bc1
 * then absmax_m[blk] = max(max |m|, 1e-30), absmax_v[blk] = max(max v, 1e-30) over the
 * block, and qm / qv = the index of the map entry nearest to m / absmax_m and to
 * max(v, 0) / absmax_v (bisection for the first entry not below, then the nearer of it
 * and the entry below; a tie takes the lower).  The caller passes decay = 1 - lr *
 * weight_decay and lr_bc1 = lr / (1 - b1^t).  The gradient is fp32 or bf16. */
int agrad_adamw8bit_step(agrad_ctx* ctx, int grad_dtype, float* p, const void* g, uint8_t* qm, uint8_t* qv,
                         float* absmax_m, float* absmax_v, const float* qmap_m, const float* qmap_v,
                         uint64_t numel, uint64_t decay_numel, float decay, float lr_bc1, float b1, float b2,
                         float eps, float inv_sqrt_bc2, float clip_coef, int first_step);

/* partial[i] = sum of squares of g[256 i .. 256 i + 255] for i < agrad_grad_norm_groups(numel);
 * the caller adds the partials in double precision and takes the square root
 * (grad_norm_sq, metal_ops.metal:10103-10137; Backend.grad_norm_sq,
 * backend.py:5115-5120; the host side of optimizer.py:579-600). */
uint64_t agrad_grad_norm_groups(uint64_t numel);
int agrad_grad_norm_sq(agrad_ctx* ctx, int dtype, const void* g, float* partial, uint64_t numel);

#ifdef __cplusplus
}
#endif
#endif /* AUTOGRAD_HIP_H */
