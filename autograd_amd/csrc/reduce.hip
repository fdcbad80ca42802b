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
//
// Broadcast Mul (cpu_mul_forward / cpu_mul_backward, backend.py:107-146) has the
// same shapes plus two more: out[l, j] = x[l, j] * y[..] with y[j] ("row"), y[l]
// ("col": one factor per row) or y[0] ("scalar").  dx (+)= g * y[..] is the forward
// kernel again; dy is a column sum, a row sum or a full sum of the product g * x,
// each in a fixed order.
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

// element i of a small operand that many rows re-read: an ordinary (cached) load
template <typename T> __device__ __forceinline__ float small_elem(const T* y, uint64_t i) {
    if constexpr (sizeof(T) == 2) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(y)[i]);
    else return reinterpret_cast<const float*>(y)[i];
}

// partial[p, :] = sum over rows p, p + P, p + 2P, ... of g[row, :] (* x2[row, :]), for P partial
// rows.  `lanes` threads share a row (a multiple of 64 that covers the row's vectors, at most
// the workgroup), so a workgroup of 256 takes 256 / lanes partial rows: narrow tensors
// (C = 384: 96 vectors) keep three quarters of their lanes busy instead of three eighths.
// With dx given the kernel also writes dx[row, :] (+)= g[row, :] * y[:] -- the other gradient
// of x * y[:], from the g it has in registers anyway.
template <typename T, int VEC>
__global__ void __launch_bounds__(kColBlock)
colsum_partial_kernel(const T* __restrict__ g, const T* __restrict__ x2, const T* __restrict__ ysmall, T* dx,
                      float* __restrict__ partial, uint64_t lead, uint32_t inner, uint32_t inner_vec, uint32_t lanes,
                      uint32_t P, int acc_dx) {
    const uint32_t sub = threadIdx.x / lanes, lane = threadIdx.x - sub * lanes;
    const uint32_t p = blockIdx.x * (blockDim.x / lanes) + sub;
    if (p >= P) return;
    for (uint32_t cv = lane; cv < inner_vec; cv += lanes) {
        const uint32_t col = cv * VEC;
        float acc[VEC], yv[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
        if (dx != nullptr) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) yv[k] = small_elem<T>(ysmall, col + k);
        }
        for (uint64_t r0 = p; r0 < lead; r0 += (uint64_t)P * kColRows) {
            float v[kColRows][VEC], w[kColRows][VEC], o[kColRows][VEC];
#pragma unroll
            for (int u = 0; u < kColRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * P;
                if (r < lead) {
                    VecIO<T, VEC>::load(g + r * inner + col, v[u]);
                    if (x2 != nullptr) VecIO<T, VEC>::load(x2 + r * inner + col, w[u]);   // uniform branches
                    if (dx != nullptr && acc_dx) VecIO<T, VEC>::load(dx + r * inner + col, o[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < kColRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * P;
                if (r < lead) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) acc[k] = acc[k] + (x2 != nullptr ? v[u][k] * w[u][k] : v[u][k]);
                    if (dx != nullptr) {
#pragma unroll
                        for (int k = 0; k < VEC; ++k) {
                            const float t = v[u][k] * yv[k];
                            o[u][k] = acc_dx ? (o[u][k] + t) : t;
                        }
                        VecIO<T, VEC>::store(dx + r * inner + col, o[u]);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) partial[(uint64_t)p * inner + col + k] = acc[k];
    }
}

// ---- broadcast Mul --------------------------------------------------------------
// out (+)= a[l, j] * y[..]: KIND AGRAD_MUL_ROW y[j], AGRAD_MUL_COL y[l], AGRAD_MUL_SCALAR y[0]

template <typename T, int VEC, int KIND>
__global__ void __launch_bounds__(kBcastBlock)
bcast_mul_kernel(const T* __restrict__ a, const T* __restrict__ y, T* out, uint64_t nvec, uint32_t inner_vec, int accumulate) {
    const uint64_t idx = (uint64_t)blockIdx.x * kBcastBlock + threadIdx.x;
    if (idx >= nvec) return;
    float v[VEC], b[VEC];
    VecIO<T, VEC>::load(a + idx * VEC, v);
    if constexpr (KIND == AGRAD_MUL_ROW) {
        // the small operand is re-read by every leading row: ordinary (cached) loads
        const uint64_t j = (idx % inner_vec) * VEC;
#pragma unroll
        for (int k = 0; k < VEC; ++k) b[k] = small_elem<T>(y, j + k);
    } else {
        const float f = small_elem<T>(y, KIND == AGRAD_MUL_COL ? idx / inner_vec : 0);
#pragma unroll
        for (int k = 0; k < VEC; ++k) b[k] = f;
    }
    float o[VEC];
    if (accumulate) VecIO<T, VEC>::load(out + idx * VEC, o);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        const float t = v[k] * b[k];
        o[k] = accumulate ? (o[k] + t) : t;
    }
    VecIO<T, VEC>::store(out + idx * VEC, o);
}

// dy[j] (+)= sum_l g[l, j] * x[l, j], l ascending: a thread owns a column vector (few
// leading rows, or bf16 storage, where the result is rounded once at the end)
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
colprod_direct_kernel(const T* __restrict__ g, const T* __restrict__ x, T* dy, uint64_t lead, uint32_t inner,
                      uint32_t inner_vec, int accumulate) {
    const uint32_t cv = blockIdx.x * 256 + threadIdx.x;
    if (cv >= inner_vec) return;
    const uint32_t col = cv * VEC;
    float acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
    for (uint64_t l0 = 0; l0 < lead; l0 += kColRows) {
        float v[kColRows][VEC], w[kColRows][VEC];
#pragma unroll
        for (int u = 0; u < kColRows; ++u)
            if (l0 + u < lead) {
                VecIO<T, VEC>::load(g + (l0 + u) * inner + col, v[u]);
                VecIO<T, VEC>::load(x + (l0 + u) * inner + col, w[u]);
            }
#pragma unroll
        for (int u = 0; u < kColRows; ++u)
            if (l0 + u < lead) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] = acc[k] + v[u][k] * w[u][k];
            }
    }
    if (accumulate) {
        float o[VEC];
        VecIO<T, VEC>::load(dy + col, o);
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = o[k] + acc[k];
    }
    VecIO<T, VEC>::store(dy + col, acc);
}

// One workgroup per row: dot[l] = sum_j g[l, j] * x[l, j].  Lanes add their strided
// share in order, the wave folds by xor butterflies, waves are added in index order.
// TO_F32: the dots go to an fp32 array (first stage of the full sum); otherwise they
// are the gradient of the per-row factor, dy[l] (+)= dot[l].
template <typename T, int VEC, int BLOCK, bool TO_F32>
__global__ void __launch_bounds__(BLOCK)
rowdot_kernel(const T* __restrict__ g, const T* __restrict__ x, void* dst, uint32_t inner, uint32_t inner_vec,
              int accumulate) {
    __shared__ float lds[BLOCK / kWave];
    const uint64_t row = blockIdx.x;
    const T* gr = g + row * inner;
    const T* xr = x + row * inner;
    float dot = 0.0f;
    for (uint32_t i0 = threadIdx.x; i0 < inner_vec; i0 += BLOCK * kColRows) {
        float v[kColRows][VEC], w[kColRows][VEC];
#pragma unroll
        for (int u = 0; u < kColRows; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < inner_vec) {
                VecIO<T, VEC>::load(gr + (uint64_t)i * VEC, v[u]);
                VecIO<T, VEC>::load(xr + (uint64_t)i * VEC, w[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kColRows; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < inner_vec) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) dot = dot + v[u][k] * w[u][k];
            }
        }
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) dot = dot + __shfl_xor(dot, off);
    if constexpr (BLOCK > kWave) {
        if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = dot;
        __syncthreads();
        dot = lds[0];
#pragma unroll
        for (int w = 1; w < BLOCK / kWave; ++w) dot = dot + lds[w];
    }
    if (threadIdx.x == 0) {
        if constexpr (TO_F32) {
            static_cast<float*>(dst)[row] = dot;
        } else {
            T* dy = static_cast<T*>(dst);
            float o[1] = {dot};
            if (accumulate) {
                float old[1];
                VecIO<T, 1>::load(dy + row, old);
                o[0] = old[0] + dot;
            }
            VecIO<T, 1>::store(dy + row, o);
        }
    }
}

// dy[0] (+)= sum of n fp32 values: one workgroup, thread t adds t, t + 1024, ... in
// order, then the 1024 sums fold as in rowdot_kernel
template <typename T>
__global__ void __launch_bounds__(1024)
sum_finalize_kernel(const float* __restrict__ part, T* dy, uint64_t n, int accumulate) {
    __shared__ float lds[1024 / kWave];
    float acc = 0.0f;
    for (uint64_t i = threadIdx.x; i < n; i += 1024) acc = acc + part[i];
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) acc = acc + __shfl_xor(acc, off);
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = lds[0];
        for (int w = 1; w < 1024 / kWave; ++w) t = t + lds[w];
        float o[1] = {t};
        if (accumulate) {
            float old[1];
            VecIO<T, 1>::load(dy, old);
            o[0] = old[0] + t;
        }
        VecIO<T, 1>::store(dy, o);
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

// partial rows, plus one fp32 row in which a bf16 destination's sum is finished before it is rounded
uint64_t broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner) {
    if (lead <= kColDirectLead || inner == 0) return 0;
    return ((uint64_t)colsum_blocks(lead) + 1) * inner * sizeof(float);
}

namespace {

// dy[j] (+)= sum_l g[l, j] (* x2[l, j]) in two stages through `workspace`; bf16 sums are
// finished in fp32 and rounded once
template <typename T>
int colsum_two_stage(hipStream_t s, const T* g, const T* x2, T* dy, void* workspace, uint64_t lead, uint64_t inner,
                     int accumulate, const T* ysmall = nullptr, T* dx = nullptr, int acc_dx = 0) {
    constexpr int WIDE = WideVec<T>::value;
    const uint32_t blocks = colsum_blocks(lead);     // partial rows
    float* partial = (float*)workspace;
    const bool wide = inner % WIDE == 0 && aligned16(g) && (!x2 || aligned16(x2)) && (!dx || aligned16(dx));
    const uint32_t iv = (uint32_t)(wide ? inner / WIDE : inner);
    uint32_t lanes = (iv + kWave - 1) / kWave * kWave;
    if (lanes > (uint32_t)kColBlock) lanes = kColBlock;
    const uint32_t per_wg = kColBlock / lanes;       // partial rows per workgroup
    const dim3 grid((blocks + per_wg - 1) / per_wg), block(lanes * per_wg);
    if (wide) hipLaunchKernelGGL((colsum_partial_kernel<T, WIDE>), grid, block, 0, s, g, x2, ysmall, dx, partial, lead, (uint32_t)inner, iv, lanes, blocks, acc_dx);
    else hipLaunchKernelGGL((colsum_partial_kernel<T, 1>), grid, block, 0, s, g, x2, ysmall, dx, partial, lead, (uint32_t)inner, iv, lanes, blocks, acc_dx);
    if (int rc = check_hip(hipGetLastError(), "column sum launch")) return rc;
    if constexpr (sizeof(T) == 4) {
        return launch_colsum_finalize(s, partial, nullptr, blocks, (uint32_t)inner, (float*)dy, nullptr, accumulate);
    } else {
        float* row = partial + (uint64_t)blocks * inner;
        if (int rc = launch_colsum_finalize(s, partial, nullptr, blocks, (uint32_t)inner, row, nullptr, 0)) return rc;
        return launch_cast_f32_bf16(s, row, dy, inner, accumulate);
    }
}

}  // namespace

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
    // few rows: a thread per column adds them itself.  (A bf16 caller without a workspace
    // gets the same kernel whatever the row count: correct, but one thread walks the column.)
    if (need == 0 || (dtype == AGRAD_BF16 && workspace == nullptr))
        return launch_pos_embedding_bwd(s, dtype, g, dy, (uint32_t)lead, 1, (uint32_t)inner, flags);
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "broadcast gradient: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "broadcast gradient: workspace must be 16-byte aligned");
    const int acc = (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0;
    if (dtype == AGRAD_F32) return colsum_two_stage<float>(s, (const float*)g, nullptr, (float*)dy, workspace, lead, inner, acc);
    return colsum_two_stage<bf16_t>(s, (const bf16_t*)g, nullptr, (bf16_t*)dy, workspace, lead, inner, acc);
}

namespace {

template <typename T, int KIND>
int bcast_mul_typed(hipStream_t s, const T* a, const T* y, T* out, uint64_t lead, uint64_t inner, int acc) {
    constexpr int WIDE = WideVec<T>::value;
    const uint64_t n = lead * inner;
    // a vector never straddles two rows, and the row operand is read at vector offsets
    const bool wide = inner % WIDE == 0 && aligned16(a) && aligned16(out);
    const uint64_t nvec = wide ? n / WIDE : n;
    const uint64_t inner_vec = wide ? inner / WIDE : inner;
    const uint64_t grid = (nvec + kBcastBlock - 1) / kBcastBlock;
    if (grid > 0x7fffffffull || inner_vec >= 0xffffffffull) return set_error(AGRAD_EINVAL, "broadcast mul: tensor too large");
    if (wide) hipLaunchKernelGGL((bcast_mul_kernel<T, WIDE, KIND>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, a, y, out, nvec, (uint32_t)inner_vec, acc);
    else hipLaunchKernelGGL((bcast_mul_kernel<T, 1, KIND>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, a, y, out, nvec, (uint32_t)inner_vec, acc);
    return check_hip(hipGetLastError(), "broadcast mul launch");
}

template <typename T>
int bcast_mul_kind(hipStream_t s, int kind, const void* a, const void* y, void* out, uint64_t lead, uint64_t inner, int acc) {
    switch (kind) {
        case AGRAD_MUL_ROW: return bcast_mul_typed<T, AGRAD_MUL_ROW>(s, (const T*)a, (const T*)y, (T*)out, lead, inner, acc);
        case AGRAD_MUL_COL: return bcast_mul_typed<T, AGRAD_MUL_COL>(s, (const T*)a, (const T*)y, (T*)out, lead, inner, acc);
        default: return bcast_mul_typed<T, AGRAD_MUL_SCALAR>(s, (const T*)a, (const T*)y, (T*)out, lead, inner, acc);
    }
}

template <typename T, bool TO_F32>
int rowdot_typed(hipStream_t s, const T* g, const T* x, void* dst, uint64_t lead, uint64_t inner, int acc) {
    constexpr int WIDE = WideVec<T>::value;
    if (lead > 0x7fffffffull || inner >= 0xffffffffull) return set_error(AGRAD_EINVAL, "mul backward: tensor too large");
    const bool wide = inner % WIDE == 0 && aligned16(g) && aligned16(x);
    const uint32_t iv = (uint32_t)(wide ? inner / WIDE : inner);
    const bool small = inner * sizeof(T) <= 4096;
    const dim3 grid((uint32_t)lead);
#define AGRAD_RD(VEC, BLOCK) hipLaunchKernelGGL((rowdot_kernel<T, VEC, BLOCK, TO_F32>), grid, dim3(BLOCK), 0, s, g, x, dst, (uint32_t)inner, iv, acc)
    if (wide && small) AGRAD_RD(WIDE, 64);
    else if (wide) AGRAD_RD(WIDE, 256);
    else if (small) AGRAD_RD(1, 64);
    else AGRAD_RD(1, 256);
#undef AGRAD_RD
    return check_hip(hipGetLastError(), "mul backward launch");
}

bool mul_kind_ok(int kind) { return kind >= AGRAD_MUL_SAME && kind <= AGRAD_MUL_SCALAR; }

}  // namespace

int launch_mul_fwd(hipStream_t s, int dtype, int kind, const void* x, const void* y, void* out, uint64_t lead, uint64_t inner) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "mul: unknown dtype %d", dtype);
    if (!mul_kind_ok(kind)) return set_error(AGRAD_EINVAL, "mul: unknown broadcast kind %d", kind);
    if (lead == 0 || inner == 0) return AGRAD_OK;
    if (x == nullptr || y == nullptr || out == nullptr) return set_error(AGRAD_EINVAL, "mul: null operand");
    if (kind == AGRAD_MUL_SAME) return launch_mul_same(s, dtype, x, y, out, lead * inner, 0);
    if (dtype == AGRAD_F32) return bcast_mul_kind<float>(s, kind, x, y, out, lead, inner, 0);
    return bcast_mul_kind<bf16_t>(s, kind, x, y, out, lead, inner, 0);
}

uint64_t mul_bwd_workspace_bytes(int kind, uint64_t lead, uint64_t inner) {
    if (kind == AGRAD_MUL_ROW) return broadcast_grad_workspace_bytes(lead, inner);
    if (kind == AGRAD_MUL_SCALAR) return (lead * sizeof(float) + 255) & ~255ull;
    return 0;
}

int launch_mul_bwd(hipStream_t s, int dtype, int kind, const void* g, const void* x, const void* y, void* dx, void* dy,
                   void* workspace, uint64_t workspace_bytes, uint64_t lead, uint64_t inner, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "mul backward: unknown dtype %d", dtype);
    if (!mul_kind_ok(kind)) return set_error(AGRAD_EINVAL, "mul backward: unknown broadcast kind %d", kind);
    const int acc_x = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    const int acc_y = (flags & AGRAD_ACC_INPUT_GRAD2) ? 1 : 0;
    const uint32_t es = dtype_size(dtype);
    if (lead == 0 || inner == 0) {
        // an empty product: stored gradients of the small operand become zero
        if (dy != nullptr && !acc_y && kind != AGRAD_MUL_SAME) {
            const uint64_t ny = kind == AGRAD_MUL_ROW ? inner : (kind == AGRAD_MUL_COL ? lead : 1);
            if (ny) return launch_fill(s, dy, 0, (int)es, ny);
        }
        return AGRAD_OK;
    }
    if (g == nullptr) return set_error(AGRAD_EINVAL, "mul backward: null upstream gradient");
    // x * y[:] with many rows and both gradients wanted: the column-sum kernel writes dx as
    // well, from the g it has loaded anyway (g is then read once, not twice)
    const bool fused = kind == AGRAD_MUL_ROW && dx != nullptr && dy != nullptr && x != nullptr && y != nullptr &&
                       mul_bwd_workspace_bytes(kind, lead, inner) > 0 && workspace != nullptr &&
                       workspace_bytes >= mul_bwd_workspace_bytes(kind, lead, inner) && aligned16(workspace) &&
                       inner < 0x7fffffffull && lead < 0x7fffffffull;
    if (fused) {
        if (dtype == AGRAD_F32)
            return colsum_two_stage<float>(s, (const float*)g, (const float*)x, (float*)dy, workspace, lead, inner, acc_y,
                                           (const float*)y, (float*)dx, acc_x);
        return colsum_two_stage<bf16_t>(s, (const bf16_t*)g, (const bf16_t*)x, (bf16_t*)dy, workspace, lead, inner, acc_y,
                                        (const bf16_t*)y, (bf16_t*)dx, acc_x);
    }
    if (dx != nullptr) {
        if (y == nullptr) return set_error(AGRAD_EINVAL, "mul backward: dx needs y");
        int rc;
        if (kind == AGRAD_MUL_SAME) rc = launch_mul_same(s, dtype, g, y, dx, lead * inner, acc_x);
        else if (dtype == AGRAD_F32) rc = bcast_mul_kind<float>(s, kind, g, y, dx, lead, inner, acc_x);
        else rc = bcast_mul_kind<bf16_t>(s, kind, g, y, dx, lead, inner, acc_x);
        if (rc) return rc;
    }
    if (dy == nullptr) return AGRAD_OK;
    if (x == nullptr) return set_error(AGRAD_EINVAL, "mul backward: dy needs x");
    if (kind == AGRAD_MUL_SAME) return launch_mul_same(s, dtype, g, x, dy, lead * inner, acc_y);
    if (kind == AGRAD_MUL_COL) {
        if (dtype == AGRAD_F32) return rowdot_typed<float, false>(s, (const float*)g, (const float*)x, dy, lead, inner, acc_y);
        return rowdot_typed<bf16_t, false>(s, (const bf16_t*)g, (const bf16_t*)x, dy, lead, inner, acc_y);
    }
    const uint64_t need = mul_bwd_workspace_bytes(kind, lead, inner);
    if (kind == AGRAD_MUL_SCALAR) {
        if (workspace == nullptr || workspace_bytes < need)
            return set_error(AGRAD_EWORKSPACE, "mul backward: workspace %llu < %llu bytes",
                             (unsigned long long)workspace_bytes, (unsigned long long)need);
        if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "mul backward: workspace must be 16-byte aligned");
        int rc = dtype == AGRAD_F32
                     ? rowdot_typed<float, true>(s, (const float*)g, (const float*)x, workspace, lead, inner, 0)
                     : rowdot_typed<bf16_t, true>(s, (const bf16_t*)g, (const bf16_t*)x, workspace, lead, inner, 0);
        if (rc) return rc;
        if (dtype == AGRAD_F32) hipLaunchKernelGGL((sum_finalize_kernel<float>), dim3(1), dim3(1024), 0, s, (const float*)workspace, (float*)dy, lead, acc_y);
        else hipLaunchKernelGGL((sum_finalize_kernel<bf16_t>), dim3(1), dim3(1024), 0, s, (const float*)workspace, (bf16_t*)dy, lead, acc_y);
        return check_hip(hipGetLastError(), "mul backward launch");
    }
    // AGRAD_MUL_ROW: a column sum of the product
    if (inner >= 0x7fffffffull || lead >= 0x7fffffffull) return set_error(AGRAD_EINVAL, "mul backward: tensor too large");
    if (need == 0) {
        if (dtype == AGRAD_F32) {
            const bool wide = inner % 4 == 0 && aligned16(g) && aligned16(x) && aligned16(dy);
            const uint32_t iv = (uint32_t)(wide ? inner / 4 : inner);
            if (wide) hipLaunchKernelGGL((colprod_direct_kernel<float, 4>), dim3((iv + 255) / 256), dim3(256), 0, s, (const float*)g, (const float*)x, (float*)dy, lead, (uint32_t)inner, iv, acc_y);
            else hipLaunchKernelGGL((colprod_direct_kernel<float, 1>), dim3((iv + 255) / 256), dim3(256), 0, s, (const float*)g, (const float*)x, (float*)dy, lead, (uint32_t)inner, iv, acc_y);
        } else {
            const bool wide = inner % 8 == 0 && aligned16(g) && aligned16(x) && aligned16(dy);
            const uint32_t iv = (uint32_t)(wide ? inner / 8 : inner);
            if (wide) hipLaunchKernelGGL((colprod_direct_kernel<bf16_t, 8>), dim3((iv + 255) / 256), dim3(256), 0, s, (const bf16_t*)g, (const bf16_t*)x, (bf16_t*)dy, lead, (uint32_t)inner, iv, acc_y);
            else hipLaunchKernelGGL((colprod_direct_kernel<bf16_t, 1>), dim3((iv + 255) / 256), dim3(256), 0, s, (const bf16_t*)g, (const bf16_t*)x, (bf16_t*)dy, lead, (uint32_t)inner, iv, acc_y);
        }
        return check_hip(hipGetLastError(), "mul backward launch");
    }
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "mul backward: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "mul backward: workspace must be 16-byte aligned");
    if (dtype == AGRAD_F32) return colsum_two_stage<float>(s, (const float*)g, (const float*)x, (float*)dy, workspace, lead, inner, acc_y);
    return colsum_two_stage<bf16_t>(s, (const bf16_t*)g, (const bf16_t*)x, (bf16_t*)dy, workspace, lead, inner, acc_y);
}

}  // namespace agrad
