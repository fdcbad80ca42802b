// Fill, copy, add / accumulate and fp32 <-> bf16 casts.
//   fill        fill_scalar_kernel / fill_scalar_kernel2 (metal_ops.metal:122-144)
//   add         cpu_add_forward (backend.py:74-76), add_residual_forward (metal_ops.metal:161-181)
//   accumulate  same-shape branch of cpu_add_backward (backend.py:78-105)
//   casts       fp32_to_bf16 (metal_ops.metal:12010-12041)
#include "elementwise.hpp"

namespace agrad {

namespace {

// 16-byte body: every uint4 carries the item pattern replicated.
// One stream of stores runs fastest with five one-wave workgroups on a CU (148 -> 133 us for a 934 MB fill).
constexpr int kFillPerCu = 5;
static_assert(kEwBlock == kWave, "the occupancy cap below counts one-wave workgroups");

__global__ void __launch_bounds__(kEwBlock) fill16_kernel(u32x4* dst, u32x4 pattern, uint64_t nvec) {
    const uint64_t first = (uint64_t)blockIdx.x * (kEwBlock * 4) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint64_t idx = first + (uint64_t)u * kEwBlock;
        if (idx < nvec) __builtin_nontemporal_store(pattern, dst + idx);
    }
}

// item-wise fill for unaligned heads / short tails
__global__ void __launch_bounds__(kEwBlock)
fill_items_kernel(uint8_t* dst, uint32_t bits, uint32_t itemsize, uint64_t n) {
    const uint64_t id = (uint64_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (id >= n) return;
    if (itemsize == 4) {
        reinterpret_cast<uint32_t*>(dst)[id] = bits;
    } else if (itemsize == 2) {
        reinterpret_cast<uint16_t*>(dst)[id] = (uint16_t)bits;
    } else {
        dst[id] = (uint8_t)bits;
    }
}

__global__ void __launch_bounds__(kEwBlock)
copy16_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, uint64_t nvec) {
    const uint64_t idx = (uint64_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (idx < nvec) __builtin_nontemporal_store(__builtin_nontemporal_load(src + idx), dst + idx);
}

__global__ void __launch_bounds__(kEwBlock)
copy_bytes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, uint64_t n) {
    const uint64_t id = (uint64_t)blockIdx.x * kEwBlock + threadIdx.x;
    if (id < n) dst[id] = src[id];
}

struct AddFn {
    static __device__ __forceinline__ float apply(const float (&in)[2]) { return in[0] + in[1]; }
};
struct IdentityFn {
    static __device__ __forceinline__ float apply(const float (&in)[1]) { return in[0]; }
};

// 8 fp32 -> 8 bf16 per thread-vector (two 128-bit loads, one 128-bit store)
template <int VEC>
__global__ void __launch_bounds__(kEwBlock)
cast_f32_bf16_kernel(const float* __restrict__ src, bf16_t* dst, uint64_t nvec, int accumulate) {
    const uint64_t first = (uint64_t)blockIdx.x * (kEwBlock * 2) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint64_t idx = first + (uint64_t)u * kEwBlock;
        if (idx >= nvec) continue;
        float v[VEC];
        if constexpr (VEC == 8) {
            float a[4], b[4];
            VecIO<float, 4>::load(src + idx * 8, a);
            VecIO<float, 4>::load(src + idx * 8 + 4, b);
#pragma unroll
            for (int k = 0; k < 4; ++k) { v[k] = a[k]; v[4 + k] = b[k]; }
        } else {
            v[0] = src[idx];
        }
        if (accumulate) {
            float old[VEC];
            VecIO<bf16_t, VEC>::load(dst + idx * VEC, old);
#pragma unroll
            for (int k = 0; k < VEC; ++k) v[k] = v[k] + old[k];
        }
        VecIO<bf16_t, VEC>::store(dst + idx * VEC, v);
    }
}

template <int VEC>
__global__ void __launch_bounds__(kEwBlock)
cast_bf16_f32_kernel(const bf16_t* __restrict__ src, float* __restrict__ dst, uint64_t nvec) {
    const uint64_t first = (uint64_t)blockIdx.x * (kEwBlock * 2) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint64_t idx = first + (uint64_t)u * kEwBlock;
        if (idx >= nvec) continue;
        float v[VEC];
        VecIO<bf16_t, VEC>::load(src + idx * VEC, v);
        if constexpr (VEC == 8) {
            float a[4] = {v[0], v[1], v[2], v[3]}, b[4] = {v[4], v[5], v[6], v[7]};
            VecIO<float, 4>::store(dst + idx * 8, a);
            VecIO<float, 4>::store(dst + idx * 8 + 4, b);
        } else {
            dst[idx] = v[0];
        }
    }
}

inline int grid_for(uint64_t n, uint64_t per_block, uint32_t* grid) {
    const uint64_t g = (n + per_block - 1) / per_block;
    if (g > 0x7fffffffull) return set_error(AGRAD_EINVAL, "launch of %llu items is too large", (unsigned long long)n);
    *grid = (uint32_t)g;
    return AGRAD_OK;
}

}  // namespace

int launch_fill(hipStream_t s, void* dst, uint32_t bits, int itemsize, uint64_t n) {
    if (itemsize != 1 && itemsize != 2 && itemsize != 4)
        return set_error(AGRAD_EINVAL, "fill: itemsize %d not in {1, 2, 4}", itemsize);
    if (n == 0) return AGRAD_OK;
    if (dst == nullptr) return set_error(AGRAD_EINVAL, "fill: null destination");
    if (reinterpret_cast<uintptr_t>(dst) % (uintptr_t)itemsize != 0)
        return set_error(AGRAD_EINVAL, "fill: destination not aligned to the item size");
    uint32_t word = bits;
    if (itemsize == 2) word = (bits & 0xffffu) * 0x00010001u;
    if (itemsize == 1) word = (bits & 0xffu) * 0x01010101u;

    uint8_t* p = static_cast<uint8_t*>(dst);
    uint64_t items = n;
    uint32_t grid;
    // head: items before the first 16-byte boundary
    const uint64_t mis = reinterpret_cast<uintptr_t>(p) & 15u;
    if (mis != 0) {
        uint64_t head = (16 - mis) / itemsize;
        if (head > items) head = items;
        if (int rc = grid_for(head, kEwBlock, &grid)) return rc;
        hipLaunchKernelGGL(fill_items_kernel, dim3(grid), dim3(kEwBlock), 0, s, p, bits, (uint32_t)itemsize, head);
        p += head * itemsize;
        items -= head;
    }
    const uint64_t nvec = items * itemsize / 16;
    if (nvec > 0) {
        if (int rc = grid_for(nvec, kEwBlock * 4, &grid)) return rc;
        u32x4 pat; pat.x = pat.y = pat.z = pat.w = word;
        // (Dynamic LDS that the kernel never touches leaves a CU five of these one-wave
        // workgroups instead of thirty-two: a stream of stores alone runs 10 % faster with few
        // waves on it -- the 934 MB zero fill of a [151936, 1536] fp32 gradient 148 -> 132 us.)
        hipLaunchKernelGGL(fill16_kernel, dim3(grid), dim3(kEwBlock), idle_lds_for(kFillPerCu), s, reinterpret_cast<u32x4*>(p), pat, nvec);
        p += nvec * 16;
        items -= nvec * 16 / itemsize;
    }
    if (items > 0) {
        if (int rc = grid_for(items, kEwBlock, &grid)) return rc;
        hipLaunchKernelGGL(fill_items_kernel, dim3(grid), dim3(kEwBlock), 0, s, p, bits, (uint32_t)itemsize, items);
    }
    return check_hip(hipGetLastError(), "fill launch");
}

int launch_copy(hipStream_t s, const void* src, void* dst, uint64_t nbytes) {
    if (nbytes == 0) return AGRAD_OK;
    if (src == nullptr || dst == nullptr) return set_error(AGRAD_EINVAL, "copy: null operand");
    uint32_t grid;
    if (aligned16(src) && aligned16(dst)) {
        const uint64_t nvec = nbytes / 16;
        if (nvec > 0) {
            if (int rc = grid_for(nvec, kEwBlock, &grid)) return rc;
            hipLaunchKernelGGL(copy16_kernel, dim3(grid), dim3(kEwBlock), 0, s,
                               static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), nvec);
        }
        const uint64_t done = nvec * 16;
        if (done < nbytes) {
            hipLaunchKernelGGL(copy_bytes_kernel, dim3(1), dim3(kEwBlock), 0, s,
                               static_cast<const uint8_t*>(src) + done, static_cast<uint8_t*>(dst) + done,
                               nbytes - done);
        }
    } else {
        if (int rc = grid_for(nbytes, kEwBlock, &grid)) return rc;
        hipLaunchKernelGGL(copy_bytes_kernel, dim3(grid), dim3(kEwBlock), 0, s,
                           static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), nbytes);
    }
    return check_hip(hipGetLastError(), "copy launch");
}

int launch_add(hipStream_t s, int dtype, const void* x, const void* y, void* out, uint64_t n) {
    const void* in[2] = {x, y};
    return ew_launch<2, AddFn>(s, dtype, in, out, n, 0, "add forward");
}

int launch_accumulate(hipStream_t s, int dtype, const void* src, void* dst, uint64_t n, uint32_t flags) {
    const void* in[1] = {src};
    return ew_launch<1, IdentityFn>(s, dtype, in, dst, n, (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0, "grad accumulate");
}

int launch_cast_f32_bf16(hipStream_t s, const void* src, void* dst, uint64_t n, int accumulate) {
    if (n == 0) return AGRAD_OK;
    if (src == nullptr || dst == nullptr) return set_error(AGRAD_EINVAL, "cast: null operand");
    uint32_t grid;
    const uint64_t nvec = (aligned16(src) && aligned16(dst)) ? n / 8 : 0;
    if (nvec > 0) {
        if (int rc = grid_for(nvec, kEwBlock * 2, &grid)) return rc;
        hipLaunchKernelGGL((cast_f32_bf16_kernel<8>), dim3(grid), dim3(kEwBlock), 0, s,
                           static_cast<const float*>(src), static_cast<bf16_t*>(dst), nvec, accumulate);
    }
    const uint64_t done = nvec * 8;
    if (done < n) {
        if (int rc = grid_for(n - done, kEwBlock * 2, &grid)) return rc;
        hipLaunchKernelGGL((cast_f32_bf16_kernel<1>), dim3(grid), dim3(kEwBlock), 0, s,
                           static_cast<const float*>(src) + done, static_cast<bf16_t*>(dst) + done,
                           n - done, accumulate);
    }
    return check_hip(hipGetLastError(), "cast launch");
}

int launch_cast_bf16_f32(hipStream_t s, const void* src, void* dst, uint64_t n) {
    if (n == 0) return AGRAD_OK;
    if (src == nullptr || dst == nullptr) return set_error(AGRAD_EINVAL, "cast: null operand");
    uint32_t grid;
    const uint64_t nvec = (aligned16(src) && aligned16(dst)) ? n / 8 : 0;
    if (nvec > 0) {
        if (int rc = grid_for(nvec, kEwBlock * 2, &grid)) return rc;
        hipLaunchKernelGGL((cast_bf16_f32_kernel<8>), dim3(grid), dim3(kEwBlock), 0, s,
                           static_cast<const bf16_t*>(src), static_cast<float*>(dst), nvec);
    }
    const uint64_t done = nvec * 8;
    if (done < n) {
        if (int rc = grid_for(n - done, kEwBlock * 2, &grid)) return rc;
        hipLaunchKernelGGL((cast_bf16_f32_kernel<1>), dim3(grid), dim3(kEwBlock), 0, s,
                           static_cast<const bf16_t*>(src) + done, static_cast<float*>(dst) + done, n - done);
    }
    return check_hip(hipGetLastError(), "cast launch");
}

uint32_t idle_lds_for(int per_cu) {
    static const uint32_t lds_per_cu = [] {
        int dev = 0, bytes = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 0u;
        if (hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess) return 0u;
        return (uint32_t)(bytes > 0 ? bytes : 0);
    }();
    if (per_cu <= 0) return 0;
    return lds_per_cu / (uint32_t)per_cu / 512u * 512u;
}

}  // namespace agrad
