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
// tensor, so workgroups each add a tile of rows into one partial row (several
// rows in flight per lane), and the column-sum finalize kernel of the norm
// backward folds the partial rows.
// Every sum has a fixed order.
//
// Broadcast Mul (cpu_mul_forward / cpu_mul_backward, backend.py:107-146) has the
// same shapes plus two more: out[l, j] = x[l, j] * y[..] with y[j] ("row"), y[l]
// ("col": one factor per row) or y[0] ("scalar").  dx (+)= g * y[..] is the forward
// kernel again; dy is a column sum, a row sum or a full sum of the product g * x,
// each in a fixed order.
#include <cstdlib>

#include "common.hpp"
#include "gelu_math.hpp"
#include "launch.hpp"

namespace agrad {

namespace {

constexpr int kBcastBlock = 64;
constexpr int kColRows = 4;             // rows a lane keeps in flight
constexpr uint32_t kColMaxBlocks = 1024;
constexpr uint64_t kColDirectLead = 64; // up to this many leading rows a thread adds them itself

// vector j (VEC elements) of a small operand that every leading row re-reads: one
// ordinary (cached) load; the operand is 16-byte aligned when VEC > 1
template <typename T, int VEC>
__device__ __forceinline__ void small_vec(const T* __restrict__ y, uint32_t j, float (&b)[VEC]) {
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
}

template <typename T, int VEC>
__global__ void __launch_bounds__(kBcastBlock)
bcast_add_kernel(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ out, uint64_t nvec, uint32_t inner_vec) {
    const uint64_t idx = (uint64_t)blockIdx.x * kBcastBlock + threadIdx.x;
    if (idx >= nvec) return;
    float a[VEC], b[VEC];
    VecIO<T, VEC>::load(x + idx * VEC, a);
    small_vec<T, VEC>(y, (uint32_t)(idx % inner_vec), b);
#pragma unroll
    for (int k = 0; k < VEC; ++k) a[k] = a[k] + b[k];
    VecIO<T, VEC>::store(out + idx * VEC, a);
}

// element i of a small operand that many rows re-read: an ordinary (cached) load
template <typename T> __device__ __forceinline__ float small_elem(const T* y, uint64_t i) {
    if constexpr (sizeof(T) == 2) return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(y)[i]);
    else return reinterpret_cast<const float*>(y)[i];
}

// partial[t % P, :] = sum over the rows of tile t of g[row, :] (* x2[row, :]).  A workgroup of
// 256 threads is `lanes` column vectors (32 or 64) wide and 256 / lanes row groups deep; every
// thread has kTileRows rows in flight, so a workgroup covers a tile of (256 / lanes) * kTileRows
// rows, adds its threads' sums through LDS and writes ONE partial row.  With more tiles than
// partial rows a workgroup walks tiles t, t + P, ...  Many short workgroups keep the loads,
// arithmetic and stores of different tiles overlapped (a persistent grid of P workgroups with
// strided rows ran its load / compute / store phases in step: 20.1 against 17.5 us at
// 16384 x 384 fp32, 46 against 34 us at 16384 x 1536 bf16).
// With dx given the kernel also writes dx[row, :] (+)= g[row, :] * y[:] -- the other gradient
// of x * y[:], from the g it has in registers anyway.
// STAGE kStageGeluBias is the backward of GELU(x2 + y[:]): the summed term is
// g * GELU'(x2 + y), and dx (+)= the same term.
constexpr int kStageSum = 0, kStageGeluBias = 1;
constexpr int kTileBlock = 256;
constexpr uint32_t kTileMaxPartials = 512;

template <typename T, int VEC, int STAGE, int kTileRows>
__global__ void __launch_bounds__(kTileBlock)
colsum_tile_kernel(const T* __restrict__ g, const T* __restrict__ x2, const T* __restrict__ ysmall, T* dx,
                   float* __restrict__ partial, uint64_t lead, uint32_t inner, uint32_t inner_vec, uint32_t lanes,
                   uint32_t tiles, int acc_dx) {
    __shared__ float part[kTileBlock * VEC];
    const uint32_t sub = threadIdx.x / lanes, lane = threadIdx.x - sub * lanes;
    const uint32_t subs = kTileBlock / lanes;
    const uint32_t tile_rows = subs * kTileRows;
    const uint32_t cv = blockIdx.x * lanes + lane;
    const bool live = cv < inner_vec;
    const uint32_t col = cv * VEC;
    float acc[VEC], yv[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) { acc[k] = 0.0f; yv[k] = 0.0f; }
    if (live && (STAGE == kStageGeluBias || dx != nullptr)) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) yv[k] = small_elem<T>(ysmall, col + k);
    }
    if (live) {
        for (uint32_t tile = blockIdx.y; tile < tiles; tile += gridDim.y) {
            const uint64_t r0 = (uint64_t)tile * tile_rows + sub;      // rows r0, r0 + subs, ...
            float v[kTileRows][VEC], w[kTileRows][VEC], o[kTileRows][VEC];
#pragma unroll
            for (int u = 0; u < kTileRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * subs;
                if (r < lead) {
                    VecIO<T, VEC>::load(g + r * inner + col, v[u]);
                    if (x2 != nullptr) VecIO<T, VEC>::load(x2 + r * inner + col, w[u]);   // uniform branches
                    if (dx != nullptr && acc_dx) VecIO<T, VEC>::load(dx + r * inner + col, o[u]);
                }
            }
#pragma unroll
            for (int u = 0; u < kTileRows; ++u) {
                const uint64_t r = r0 + (uint64_t)u * subs;
                if (r < lead) {
                    if constexpr (STAGE == kStageGeluBias) {
#pragma unroll
                        for (int k = 0; k < VEC; ++k) {
                            const float t = v[u][k] * gelu_slope(w[u][k] + yv[k]);
                            acc[k] = acc[k] + t;
                            o[u][k] = acc_dx ? (o[u][k] + t) : t;
                        }
                        if (dx != nullptr) VecIO<T, VEC>::store(dx + r * inner + col, o[u]);
                    } else {
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
        }
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) part[(sub * lanes + lane) * VEC + k] = acc[k];
    __syncthreads();
    if (sub == 0 && live) {
        float sum[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) sum[k] = acc[k];
        for (uint32_t q = 1; q < subs; ++q)
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum[k] = sum[k] + part[(q * lanes + lane) * VEC + k];
#pragma unroll
        for (int k = 0; k < VEC; ++k) partial[(uint64_t)blockIdx.y * inner + col + k] = sum[k];
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
template <typename T, int STAGE = kStageSum>
int colsum_two_stage(hipStream_t s, const T* g, const T* x2, T* dy, void* workspace, uint64_t lead, uint64_t inner,
                     int accumulate, const T* ysmall = nullptr, T* dx = nullptr, int acc_dx = 0, bool narrow_out = false) {
    constexpr int WIDE = WideVec<T>::value;
    float* partial = (float*)workspace;
    const bool wide = inner % WIDE == 0 && aligned16(g) && (!x2 || aligned16(x2)) && (!dx || aligned16(dx));
    const uint32_t iv = (uint32_t)(wide ? inner / WIDE : inner);
    uint32_t blocks;                                 // partial rows
    // 32 lanes when that leaves fewer of them idle in the last column group (96 vectors:
    // three full groups of 32, not one and a half of 64)
    const uint32_t lanes = (iv + 31) / 32 * 32 < (iv + 63) / 64 * 64 ? 32 : 64;
    // Four rows in flight per thread when one tile per workgroup then covers the tensor
    // within kTileMaxPartials partial rows; else two (fewer registers, more waves
    // resident) and a walk over several tiles.  Measured on 16384 rows, fp32 x 384 /
    // x 768 / bf16 x 1536: 17.5 / 30.4 / 34.0 us this way, 19.1 / 30.4 / 34.0 with two
    // everywhere, 17.4 / 33.1 / 36.6 with four and 1024 partial rows.
    const uint32_t subs = kTileBlock / lanes;
    const uint32_t cap = colsum_blocks(lead) < kTileMaxPartials ? colsum_blocks(lead) : kTileMaxPartials;
    const int R = (lead + subs * 4 - 1) / (subs * 4) <= cap ? 4 : 2;
    const uint32_t tile_rows = subs * R;
    const uint64_t tiles = (lead + tile_rows - 1) / tile_rows;
    blocks = (uint32_t)(tiles < cap ? tiles : cap);
    const dim3 grid((iv + lanes - 1) / lanes, blocks), block(kTileBlock);
#define AGRAD_TILE_LAUNCH(V, RR) hipLaunchKernelGGL((colsum_tile_kernel<T, V, STAGE, RR>), grid, block, 0, s, g, x2, ysmall, dx, partial, lead, (uint32_t)inner, iv, lanes, (uint32_t)tiles, acc_dx)
    if (wide) { if (R == 4) AGRAD_TILE_LAUNCH(WIDE, 4); else AGRAD_TILE_LAUNCH(WIDE, 2); }
    else { if (R == 4) AGRAD_TILE_LAUNCH(1, 4); else AGRAD_TILE_LAUNCH(1, 2); }
#undef AGRAD_TILE_LAUNCH
    if (int rc = check_hip(hipGetLastError(), "column sum launch")) return rc;
    if constexpr (sizeof(T) == 4) {
        // narrow_out: dy points at bf16 although the summed tensor is fp32
        return launch_colsum_finalize(s, partial, nullptr, blocks, (uint32_t)inner, (float*)dy, nullptr, accumulate, narrow_out);
    } else {
        return launch_colsum_finalize(s, partial, nullptr, blocks, (uint32_t)inner, reinterpret_cast<float*>(dy), nullptr, accumulate, true);
    }
}

}  // namespace

int launch_broadcast_grad(hipStream_t s, int dtype, const void* g, void* dy, void* workspace, uint64_t workspace_bytes,
                          uint64_t lead, uint64_t inner, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "broadcast gradient: unknown dtype %d", dtype);
    if (inner == 0) return AGRAD_OK;
    if (dy == nullptr) return set_error(AGRAD_EINVAL, "broadcast gradient: null destination");
    if (inner >= 0x7fffffffull || lead >= 0x7fffffffull) return set_error(AGRAD_EINVAL, "broadcast gradient: tensor too large");
    const bool narrow = (flags & AGRAD_PARAM_GRAD_BF16) != 0;      // fp32 rows summed into a bf16 gradient
    if (narrow && dtype != AGRAD_F32)
        return set_error(AGRAD_EINVAL, "broadcast gradient: AGRAD_PARAM_GRAD_BF16 goes with an fp32 upstream gradient");
    if (lead == 0) {
        // an empty sum: a stored gradient is zero, an accumulated one keeps its value
        if (!(flags & AGRAD_ACC_PARAM_GRAD)) return launch_fill(s, dy, 0, narrow ? 2 : (int)dtype_size(dtype), inner);
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
    if (dtype == AGRAD_F32)
        return colsum_two_stage<float>(s, (const float*)g, nullptr, (float*)dy, workspace, lead, inner, acc, nullptr, nullptr, 0, narrow);
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

// ---- bias + GELU: y = GELU(h + b[:]) and its backward ---------------------------
// The bias add of a linear layer folded into its activation: the [rows, C] tensor
// is read once instead of written and read again (gelu_add_bias_kernel /
// gelu_backward_bias_kernel, metal_ops.metal:3737-3773; on the CPU the composition
// of cpu_add_forward, backend.py:74-88, and cpu_gelu_forward, backend.py:376-395).
// The backward also owns the bias gradient -- the column sum of the very terms it
// writes to dh -- where the reference runs bias_grad_reduce over dh afterwards.

namespace {

template <typename T, int VEC, bool BACKWARD>
__global__ void __launch_bounds__(kBcastBlock)
gelu_bias_kernel(const T* __restrict__ h, const T* __restrict__ b, const T* __restrict__ dy, T* out, uint64_t nvec,
                 uint32_t inner_vec, FastDiv32 by_inner, int accumulate) {
    const uint64_t idx = (uint64_t)blockIdx.x * kBcastBlock + threadIdx.x;
    if (idx >= nvec) return;
    float v[VEC], g[VEC], o[VEC];
    VecIO<T, VEC>::load(h + idx * VEC, v);
    if constexpr (BACKWARD) {
        VecIO<T, VEC>::load(dy + idx * VEC, g);
        if (accumulate) VecIO<T, VEC>::load(out + idx * VEC, o);
    }
    // the transcendental leaves no room for an emulated divide: with idx % inner_vec the
    // forward ran at 0.66 of a copy (fp32, 16384 x 3072)
    float bv[VEC];
    small_vec<T, VEC>(b, nvec <= 0xffffffffull ? by_inner.mod((uint32_t)idx) : (uint32_t)(idx % inner_vec), bv);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        const float z = v[k] + bv[k];
        if constexpr (BACKWARD) {
            const float t = g[k] * gelu_slope(z);
            o[k] = accumulate ? (o[k] + t) : t;
        } else {
            o[k] = gelu_value(z);
        }
    }
    VecIO<T, VEC>::store(out + idx * VEC, o);
}

template <typename T, bool BACKWARD>
int gelu_bias_stream(hipStream_t s, const T* h, const T* b, const T* dy, T* out, uint64_t rows, uint64_t C, int acc) {
    constexpr int WIDE = WideVec<T>::value;
    const uint64_t n = rows * C;
    const bool wide = C % WIDE == 0 && aligned16(h) && aligned16(b) && aligned16(out) && (!BACKWARD || aligned16(dy));
    const uint64_t nvec = wide ? n / WIDE : n;
    const uint64_t inner_vec = wide ? C / WIDE : C;
    const uint64_t grid = (nvec + kBcastBlock - 1) / kBcastBlock;
    if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "bias gelu: tensor too large");
    const FastDiv32 by_inner((uint32_t)inner_vec);
    if (wide) hipLaunchKernelGGL((gelu_bias_kernel<T, WIDE, BACKWARD>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, h, b, dy, out, nvec, (uint32_t)inner_vec, by_inner, acc);
    else hipLaunchKernelGGL((gelu_bias_kernel<T, 1, BACKWARD>), dim3((uint32_t)grid), dim3(kBcastBlock), 0, s, h, b, dy, out, nvec, (uint32_t)inner_vec, by_inner, acc);
    return check_hip(hipGetLastError(), "bias gelu launch");
}

}  // namespace

int launch_gelu_bias_fwd(hipStream_t s, int dtype, const void* h, const void* b, void* y, uint64_t rows, uint32_t C) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "bias gelu: unknown dtype %d", dtype);
    if (rows == 0 || C == 0) return AGRAD_OK;
    if (h == nullptr || b == nullptr || y == nullptr) return set_error(AGRAD_EINVAL, "bias gelu: null operand");
    if (dtype == AGRAD_F32) return gelu_bias_stream<float, false>(s, (const float*)h, (const float*)b, nullptr, (float*)y, rows, C, 0);
    return gelu_bias_stream<bf16_t, false>(s, (const bf16_t*)h, (const bf16_t*)b, nullptr, (bf16_t*)y, rows, C, 0);
}

// partial rows, plus one fp32 row in which a bf16 bias gradient is finished before it is rounded
uint64_t gelu_bias_backward_workspace_bytes(uint64_t rows, uint32_t C) {
    if (rows == 0 || C == 0) return 0;
    return ((uint64_t)colsum_blocks(rows) + 1) * C * sizeof(float);
}

int launch_gelu_bias_bwd(hipStream_t s, int dtype, const void* dy, const void* h, const void* b, void* dh, void* db,
                         void* workspace, uint64_t workspace_bytes, uint64_t rows, uint32_t C, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "bias gelu backward: unknown dtype %d", dtype);
    if (C == 0) return AGRAD_OK;
    if (rows >= 0x7fffffffull) return set_error(AGRAD_EINVAL, "bias gelu backward: tensor too large");
    const int acc_db = (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0, acc_dh = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    const bool narrow = (flags & AGRAD_PARAM_GRAD_BF16) != 0;      // an fp32 tensor's bias gradient stored as bf16
    if (narrow && dtype != AGRAD_F32)
        return set_error(AGRAD_EINVAL, "bias gelu backward: AGRAD_PARAM_GRAD_BF16 goes with fp32 tensors");
    if (rows == 0) {
        // an empty sum: a stored bias gradient is zero, an accumulated one keeps its value
        if (db != nullptr && !acc_db) return launch_fill(s, db, 0, narrow ? 2 : (int)dtype_size(dtype), C);
        return AGRAD_OK;
    }
    if (dy == nullptr || h == nullptr || b == nullptr || (dh == nullptr && db == nullptr))
        return set_error(AGRAD_EINVAL, "bias gelu backward: null operand");
    if (db == nullptr) {
        if (dtype == AGRAD_F32) return gelu_bias_stream<float, true>(s, (const float*)h, (const float*)b, (const float*)dy, (float*)dh, rows, C, acc_dh);
        return gelu_bias_stream<bf16_t, true>(s, (const bf16_t*)h, (const bf16_t*)b, (const bf16_t*)dy, (bf16_t*)dh, rows, C, acc_dh);
    }
    const uint64_t need = gelu_bias_backward_workspace_bytes(rows, C);
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "bias gelu backward: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "bias gelu backward: workspace must be 16-byte aligned");
    if (dtype == AGRAD_F32)
        return colsum_two_stage<float, kStageGeluBias>(s, (const float*)dy, (const float*)h, (float*)db, workspace, rows, C,
                                                       acc_db, (const float*)b, (float*)dh, acc_dh, narrow);
    return colsum_two_stage<bf16_t, kStageGeluBias>(s, (const bf16_t*)dy, (const bf16_t*)h, (bf16_t*)db, workspace, rows, C,
                                                    acc_db, (const bf16_t*)b, (bf16_t*)dh, acc_dh);
}


}  // namespace agrad
