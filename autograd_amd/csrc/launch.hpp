// Host-side launchers, one per op family.  Each validates shapes and alignment,
// picks the launch geometry, and enqueues on the given stream.  They return an
// AGRAD_* status and record a message with set_error on failure.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

#include "../../include/autograd_hip.h"

namespace agrad {

int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int check_hip(hipError_t e, const char* what);
// true while the calling thread records launches into a graph: launchers whose
// work is not a plain sequence of kernels on the stream refuse
void set_capturing(bool on);
bool is_capturing();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline uint32_t dtype_size(int dtype) { return dtype == AGRAD_BF16 ? 2u : 4u; }

// Upper bound on the number of row-partials the norm backward keeps per column.

// Bytes of dynamic LDS that a kernel of ONE-WAVE workgroups asks for and never touches, so that at
// most `per_cu` of its workgroups share a CU (streams of stores, or of many operands, run faster
// with fewer waves in flight): this GPU's LDS per CU divided by the count, in whole 512-byte
// granules, so the cap keeps its meaning on a part with another LDS size.  0 if the size is unknown.
uint32_t idle_lds_for(int per_cu);

// memops.hip
int launch_fill(hipStream_t s, void* dst, uint32_t bits, int itemsize, uint64_t n);
int launch_copy(hipStream_t s, const void* src, void* dst, uint64_t nbytes);
int launch_add(hipStream_t s, int dtype, const void* x, const void* y, void* out, uint64_t n);
int launch_accumulate(hipStream_t s, int dtype, const void* src, void* dst, uint64_t n, uint32_t flags);
int launch_cast_f32_bf16(hipStream_t s, const void* src, void* dst, uint64_t n, int accumulate);
int launch_cast_bf16_f32(hipStream_t s, const void* src, void* dst, uint64_t n);

// norm.hip
uint64_t norm_bwd_workspace_bytes(uint64_t rows, uint32_t C, int dtype);
int launch_norm_fwd(hipStream_t s, int kind, int dtype, const void* x, const void* residual,
                    const float* gamma, const float* beta, void* h_out, void* y,
                    uint64_t rows, uint32_t C, float eps);
int launch_norm_bwd(hipStream_t s, int kind, int dtype, const void* x, const void* dy,
                    const float* gamma, const void* dres_in, void* dx, void* dx2,
                    float* dgamma, float* dbeta, void* workspace, uint64_t workspace_bytes,
                    uint64_t rows, uint32_t C, float eps, uint32_t flags);
// the same with the partial rows in a fixed per-GPU array instead of a workspace;
// norm_noalloc_setup(device) runs once per GPU, with that GPU current, before it
int norm_noalloc_setup(int device);
int launch_norm_bwd_noalloc(hipStream_t s, int device, int kind, int dtype, const void* x, const void* dy,
                            const float* gamma, const void* dres_in, void* dx, void* dx2,
                            float* dgamma, float* dbeta, uint64_t rows, uint32_t C, float eps, uint32_t flags);

// out_a[c] (+)= sum over the P rows of pa[P, C] (same for pb -> out_b; either pair may be null)
// out_bf16: out_a / out_b point at bf16 elements (the sum is rounded once, after the optional accumulate)
int launch_colsum_finalize(hipStream_t s, const float* pa, const float* pb, uint32_t P, uint32_t C,
                           float* out_a, float* out_b, int accumulate, bool out_bf16 = false);

// One column sum left to fold: out_a[c] (+)= sum of the P rows of pa[P, C], the same for pb -> out_b.
struct ColsumJob {
    const float* pa; const float* pb;
    void* out_a; void* out_b;            // fp32, or bf16 when out_bf16
    uint32_t P, C, accumulate, out_bf16;
};
constexpr int kFinalizeManyJobs = 32;    // jobs one batched finalize launch takes (they travel as kernel arguments)
// While one of these lives on the calling thread (with a non-null sink), every
// launch_colsum_finalize on that thread -- the second launch of the norm backward, of the
// bias gradients and of Mul's row-operand gradient -- is appended to `sink` instead of
// launched; the partial rows it names must stay untouched until the sink has been folded.
class ColsumDefer {
public:
    explicit ColsumDefer(std::vector<ColsumJob>* sink);
    ~ColsumDefer();
    ColsumDefer(const ColsumDefer&) = delete;
    ColsumDefer& operator=(const ColsumDefer&) = delete;
private:
    std::vector<ColsumJob>* prev_;
};
// folds `n` pending column sums in as few launches as possible: the same bits as n launch_colsum_finalize calls
int launch_colsum_finalize_many(hipStream_t s, const ColsumJob* jobs, size_t n);

// reduce.hip
int launch_broadcast_add(hipStream_t s, int dtype, const void* x, const void* y, void* out, uint64_t lead, uint64_t inner);
int launch_gelu_bias_fwd(hipStream_t s, int dtype, const void* h, const void* b, void* y, uint64_t rows, uint32_t C);
uint64_t gelu_bias_backward_workspace_bytes(uint64_t rows, uint32_t C);
int launch_gelu_bias_bwd(hipStream_t s, int dtype, const void* dy, const void* h, const void* b, void* dh, void* db,
                         void* workspace, uint64_t workspace_bytes, uint64_t rows, uint32_t C, uint32_t flags);
uint64_t broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner);
int launch_broadcast_grad(hipStream_t s, int dtype, const void* g, void* dy, void* workspace, uint64_t workspace_bytes,
                          uint64_t lead, uint64_t inner, uint32_t flags);

// pointwise.hip
int launch_unary_fwd(hipStream_t s, int op, int dtype, const void* x, void* y, uint64_t n);
int launch_unary_bwd(hipStream_t s, int op, int dtype, const void* dy, const void* saved, void* dx, uint64_t n,
                     uint32_t flags);
int launch_mul_same(hipStream_t s, int dtype, const void* a, const void* b, void* out, uint64_t n, int accumulate);
// reduce.hip: Mul with a broadcast operand and its gradients
int launch_mul_fwd(hipStream_t s, int dtype, int kind, const void* x, const void* y, void* out, uint64_t lead, uint64_t inner);
uint64_t mul_bwd_workspace_bytes(int kind, uint64_t lead, uint64_t inner);
int launch_mul_bwd(hipStream_t s, int dtype, int kind, const void* g, const void* x, const void* y, void* dx, void* dy,
                   void* workspace, uint64_t workspace_bytes, uint64_t lead, uint64_t inner, uint32_t flags);
// loss.hip: softmax over the last axis
int launch_softmax_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t rows, uint32_t V);
int launch_softmax_bwd(hipStream_t s, int dtype, const void* y, const void* dy, void* dx, uint64_t rows, uint32_t V,
                       uint32_t flags);

// strided.hip
// elements spanned by the view: 1 + sum (shape[i] - 1) * strides[i]; 0 for an empty shape
uint64_t strided_extent(int ndim, const uint32_t* shape, const uint64_t* strides);
int launch_strided_copy(hipStream_t s, int dtype, const void* src, void* dst, int ndim, const uint32_t* shape,
                        const uint64_t* strides, uint32_t flags);

// activation.hip
int launch_gelu_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t n);
int launch_gelu_bwd(hipStream_t s, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags);
int launch_relu2_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t n);
int launch_relu2_bwd(hipStream_t s, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags);
int launch_swiglu_fwd(hipStream_t s, int dtype, const void* gu, void* h, uint64_t rows, uint32_t H);
int launch_swiglu_fwd_tile(hipStream_t s, int dtype, const void* gu, void* tile, uint64_t rows, uint32_t H,
                           uint32_t h0, uint32_t hw);
int launch_swiglu_bwd(hipStream_t s, int dtype, const void* gu, const void* dh, void* dgu,
                      uint64_t rows, uint32_t H, uint32_t flags);

// rope.hip
int launch_rope(hipStream_t s, int dtype, void* q, void* k, const float* cos_t, const float* sin_t,
                uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D, int sign, int backward, int bhtd = 0);

// embedding.hip
int launch_gather_fwd(hipStream_t s, int dtype, const int32_t* ids, const void* W, const void* wpe,
                      void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V, int* err_flag);
uint64_t embedding_bwd_workspace_bytes(uint64_t N, uint32_t C, uint32_t V, int dtype);
// the two halves of the embedding gradient, for callers that order the ids ahead of time
uint64_t embedding_order_bytes(uint64_t N);
uint64_t embedding_sort_workspace_bytes(uint64_t N, uint32_t V);
int launch_embedding_sort(hipStream_t s, const int32_t* ids, uint32_t* order, void* workspace,
                          uint64_t workspace_bytes, uint64_t N, uint32_t V, int* err_flag);
// the ordering alone, with the zero fill of [zero_dst, +zero_bytes) riding in the same launch when given
int launch_embedding_order(hipStream_t s, const int32_t* ids, uint32_t* order, void* sort_workspace,
                           uint64_t sort_workspace_bytes, uint64_t N, uint32_t V, void* zero_dst, uint64_t zero_bytes,
                           int* err_flag);
int launch_embedding_grad_reset(hipStream_t s, int dtype, const int32_t* rows, uint64_t N, void* dW,
                                uint32_t C, uint32_t V);
int launch_gather_fwd_sorted(hipStream_t s, int dtype, const int32_t* ids, const void* W, const void* wpe,
                             void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V, uint32_t* order,
                             void* sort_workspace, uint64_t sort_workspace_bytes, int* err_flag, int32_t* kept = nullptr);
uint64_t embedding_bwd_sorted_workspace_bytes(uint64_t N, uint32_t C);
// dwpe (optional, [T, C]): the position table's gradient sum_b dY[b, t, :] rides in the same launch
int launch_embedding_bwd_sorted(hipStream_t s, int dtype, uint32_t* order, const void* dY, void* dW,
                                void* dwpe, void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t T,
                                uint32_t C, uint32_t V, uint32_t flags);
int launch_embedding_bwd(hipStream_t s, int dtype, const int32_t* ids, const void* dY, void* dW,
                         void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t C,
                         uint32_t V, uint32_t flags, int* err_flag);
int launch_pos_embedding_bwd(hipStream_t s, int dtype, const void* dY, void* dwpe, uint32_t B,
                             uint32_t T, uint32_t C, uint32_t flags);

// optimizer.hip
int launch_adamw(hipStream_t s, int grad_dtype, float* p, const void* g, float* m, float* v,
                 uint64_t numel, uint64_t decay_numel, float lr_wd, float b1, float one_minus_b1,
                 float b2, float one_minus_b2, float eps, float step_lr, float inv_sqrt_bc2, float grad_scale);
int launch_adamw8bit(hipStream_t s, int grad_dtype, float* p, const void* g, uint8_t* qm, uint8_t* qv,
                     float* absmax_m, float* absmax_v, const float* qmap_m, const float* qmap_v,
                     uint64_t numel, uint64_t decay_numel, float decay, float lr_bc1, float b1, float b2, float eps,
                     float inv_sqrt_bc2, float clip_coef, int first_step);
uint64_t grad_norm_groups(uint64_t numel);
int launch_grad_norm_sq(hipStream_t s, int dtype, const void* g, float* partial, uint64_t numel);

// loss.hip
int launch_ce_fwd(hipStream_t s, int dtype, const void* logits, const int32_t* labels, float* loss,
                  float* lse_out, uint64_t rows, uint32_t V, int* err_flag);
int launch_ce_bwd(hipStream_t s, int dtype, const void* logits, const int32_t* labels, const float* dloss,
                  const float* lse, void* dlogits, uint64_t rows, uint32_t V, uint32_t flags, int* err_flag);
// loss and gradient in one launch, in place: logits[r, :] becomes (softmax - onehot) * scale (row_scale[row_base + r]
// when given), row_loss / lse [row_base + r] are written; a target outside [0, V) gives a zero row
int launch_ce_fused(hipStream_t s, int dtype, void* logits, const int32_t* targets, float* row_loss, float* lse,
                    const float* row_scale, uint64_t rows, uint32_t V, uint64_t row_base, float scale,
                    uint32_t write_grad, void* team_scratch, int* err_words, uint32_t team_polls = 0);
// bytes of team_scratch: arrival counters and (max, sum) pairs of the workgroup teams that share long rows
uint64_t ce_fused_scratch_bytes();

}  // namespace agrad
