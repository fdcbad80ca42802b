// Broadcast add and its gradient: out[l, j] = x[l, j] + y[j] for x of shape
// [lead, inner] and y of the trailing shape [inner] (a bias, or a position table
// added to every batch entry), and dy[j] (+)= sum_l g[l, j]
// (cpu_add_forward / cpu_add_backward, backend.py:74-105; add_pos_forward,
// pos_emb_grad and the bias-gradient column reductions of the Metal library,
// metal_ops.metal:205-234, 1002-1193).
//
// Forward is a stream: one 16-byte vector per thread, y through the caches.
// The gradient is a column sum.  With few leading rows (a [T, C] table under a
// batch of 16) a thread owns a column vector and adds the rows in order.  With
// many (a [C] bias under 16384 rows) that would be C/4 threads walking the whole
// tensor, so persistent workgroups each add a strided share of the rows into one
// partial row (read-only stream, several rows in flight per lane), and the
// column-sum finalize kernel of the norm backward folds the partial rows.
// Every sum has a fixed order.
#include "common.hpp"
#include "launch.hpp"

namespace agrad {

namespace {

constexpr int kBcastBlock = 64;
constexpr int kColBlock = 256;
constexpr int kColRows = 4;             // rows a lane keeps in flight
constexpr uint32_t kColMaxBlocks = 1024;
constexpr uint64_t kColDirectLead = 64; // up to this many leading rows a thread adds them itself

template <typename T, int VEC>
__global__ void __launch_bounds__(kBcastBlock)
bcast_add_kernel(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ out, uint64_t nvec, uint32_t inner_vec) {
    const uint64_t idx = (uint64_t)blockIdx.x * kBcastBlock + threadIdx.x;
    if (idx >= nvec) return;
    float a[VEC], b[VEC];
    VecIO<T, VEC>::load(x + idx * VEC, a);
    const uint32_t j = (uint32_t)(idx % inner_vec);
    // the small operand is re-read by every leading row: ordinary (cached) loads
    if constexpr (VEC == 1) {
        b[0] = sizeof(T) == 2 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(y)[j]) : reinterpret_cast<const float*>(y)[j];
    } else if constexpr (sizeof(T) == 4) {
        const float4 t = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(y) + (uint64_t)j * 4);
        b[0] = t.x; b[1] = t.y; b[2] = t.z; b[3] = t.w;
    } else {
        const uint4 t = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(y) + (uint64_t)j * 8);
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            b[2 * k] = __builtin_bit_cast(float, w[k] << 16);
            b[2 * k + 1] = __builtin_bit_cast(float, w[k] & 0xffff0000u);
        }
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) a[k] = a[k] + b[k];
    VecIO<T, VEC>::store(out + idx * VEC, a);
}

// partial[blockIdx.x, :] = sum over rows blockIdx.x, blockIdx.x + gridDim.x, ... of g[row, :]
template <typename T, int VEC>
__global__ void __launch_bounds__(kColBlock)
colsum_partial_kernel(const T* __restrict__ g, float* __restrict__ partial, uint64_t lead, uint32_t inner,
                      uint32_t inner_vec) {
    for (uint32_t cv = threadIdx.x; cv < inner_vec; cv += kColBlock) {
        const uint32_t col = cv * VEC;
        float acc[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
        for (uint64_t r0 = blockIdx.x; r0 < lead; r0 += (uint64_t)gridDim.x * kColRows) {
            float v[kColRows][VEC];
#pragma unroll
            for (int u = 0; u < kColRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * gridDim.x;
                if (r < lead) VecIO<T, VEC>::load(g + r * inner + col, v[u]);
            }
#pragma unroll
            for (int u = 0; u < kColRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * gridDim.x;
                if (r < lead) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] = acc[k] + v[u][k];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) partial[(uint64_t)blockIdx.x * inner + col + k] = acc[k];
    }
}

uint32_t colsum_blocks(uint64_t lead) { return (uint32_t)(lead < kColMaxBlocks ? lead : kColMaxBlocks); }

template <typename T>
int bcast_add_typed(hipStream_t s, const T* x, const T* y, T* out, uint64_t lead, uint64_t inner) {
    constexpr int WIDE = WideVec<T>::value;
    const uint64_t n = lead * inner;
    const bool wide = inner % WIDE == 0 && aligned16(x) && aligned16(y) && aligned16(out) && inner / WIDE < 0xffffffffull;
    const uint64_t nvec = wide ? n / WIDE : n;
    const uint64_t grid = (nvec + kBcastBlock - 1) / kBcastBlock;
    if (grid > 0x7fffffffull || inner >= 0xffffffffull) return set_error(AGRAD_EINVAL, "broadcast add: tensor too large");
    if (wide) hipLaunchKernelGGL((bcast_add_kernel<T, WIDE>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, x, y, out, nvec, (uint32_t)(inner / WIDE));
    else hipLaunchKernelGGL((bcast_add_kernel<T, 1>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, x, y, out, nvec, (uint32_t)inner);
    return check_hip(hipGetLastError(), "broadcast add launch");
}

}  // namespace

int launch_broadcast_add(hipStream_t s, int dtype, const void* x, const void* y, void* out, uint64_t lead, uint64_t inner) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "broadcast add: unknown dtype %d", dtype);
    if (lead == 0 || inner == 0) return AGRAD_OK;
    if (x == nullptr || y == nullptr || out == nullptr) return set_error(AGRAD_EINVAL, "broadcast add: null operand");
    if (dtype == AGRAD_F32) return bcast_add_typed<float>(s, (const float*)x, (const float*)y, (float*)out, lead, inner);
    return bcast_add_typed<bf16_t>(s, (const bf16_t*)x, (const bf16_t*)y, (bf16_t*)out, lead, inner);
}

uint64_t broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner) {
    if (lead <= kColDirectLead || inner == 0) return 0;
    return (uint64_t)colsum_blocks(lead) * inner * sizeof(float);
}

int launch_broadcast_grad(hipStream_t s, int dtype, const void* g, void* dy, void* workspace, uint64_t workspace_bytes,
                          uint64_t lead, uint64_t inner, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "broadcast gradient: unknown dtype %d", dtype);
    if (inner == 0) return AGRAD_OK;
    if (dy == nullptr) return set_error(AGRAD_EINVAL, "broadcast gradient: null destination");
    if (inner >= 0x7fffffffull || lead >= 0x7fffffffull) return set_error(AGRAD_EINVAL, "broadcast gradient: tensor too large");
    if (lead == 0) {
        // an empty sum: a stored gradient is zero, an accumulated one keeps its value
        if (!(flags & AGRAD_ACC_PARAM_GRAD)) return launch_fill(s, dy, 0, (int)dtype_size(dtype), inner);
        return AGRAD_OK;
    }
    if (g == nullptr) return set_error(AGRAD_EINVAL, "broadcast gradient: null operand");
    const uint64_t need = broadcast_grad_workspace_bytes(lead, inner);
    // the two-stage path produces fp32; a bf16 destination keeps the direct path
    if (need == 0 || dtype == AGRAD_BF16)
        return launch_pos_embedding_bwd(s, dtype, g, dy, (uint32_t)lead, 1, (uint32_t)inner, flags);
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "broadcast gradient: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "broadcast gradient: workspace must be 16-byte aligned");
    const uint32_t blocks = colsum_blocks(lead);
    float* partial = (float*)workspace;
    const bool wide = inner % 4 == 0 && aligned16(g);
    if (wide) hipLaunchKernelGGL((colsum_partial_kernel<float, 4>), dim3(blocks), dim3(kColBlock), 0, s, (const float*)g, partial, lead, (uint32_t)inner, (uint32_t)(inner / 4));
    else hipLaunchKernelGGL((colsum_partial_kernel<float, 1>), dim3(blocks), dim3(kColBlock), 0, s, (const float*)g, partial, lead, (uint32_t)inner, (uint32_t)inner);
    if (int rc = check_hip(hipGetLastError(), "broadcast gradient launch")) return rc;
    return launch_colsum_finalize(s, partial, nullptr, blocks, (uint32_t)inner, (float*)dy, nullptr,
                                  (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0);
}

}  // namespace agrad
