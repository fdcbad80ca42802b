// Streaming element-wise kernels: every thread moves UNROLL 128-bit vectors per
// operand, strided by the workgroup so each wave issues full 1 KiB requests,
// with all loads issued before the arithmetic.  64-bit element offsets.
// One vector per thread and many small workgroups is the fastest shape on
// MI355X for pure streaming (a copy reaches 6.5 TB/s; four vectors per thread
// 6.1, eight 4.2), so UNROLL is 1.
#pragma once

#include "common.hpp"
#include "launch.hpp"

namespace agrad {

constexpr int kEwBlock = 64;

template <typename T, int NIN>
struct EwArgs {
    const T* in[NIN];
    T* out;
    uint64_t nvec;  // number of VEC-element groups
    int acc;        // out = old_out + f(in)
};

// F::apply(const float (&in)[NIN]) -> float, applied lane-wise.
template <typename T, int VEC, int UNROLL, int NIN, typename F>
__global__ void __launch_bounds__(kEwBlock) ew_kernel(const EwArgs<T, NIN> a) {
    const uint64_t first = (uint64_t)blockIdx.x * (kEwBlock * UNROLL) + threadIdx.x;
    float v[UNROLL][NIN][VEC];
    float old[UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t idx = first + (uint64_t)u * kEwBlock;
        if (idx < a.nvec) {
#pragma unroll
            for (int j = 0; j < NIN; ++j) VecIO<T, VEC>::load(a.in[j] + idx * VEC, v[u][j]);
            if (a.acc) VecIO<T, VEC>::load(a.out + idx * VEC, old[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t idx = first + (uint64_t)u * kEwBlock;
        if (idx < a.nvec) {
            float o[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float in[NIN];
#pragma unroll
                for (int j = 0; j < NIN; ++j) in[j] = v[u][j][k];
                const float r = F::apply(in);
                o[k] = a.acc ? (old[u][k] + r) : r;
            }
            VecIO<T, VEC>::store(a.out + idx * VEC, o);
        }
    }
}

template <typename T, int NIN, typename F>
int ew_launch_typed(hipStream_t s, const void* const (&in)[NIN], void* out, uint64_t n, int acc) {
    if (n == 0) return AGRAD_OK;
    constexpr int VEC = WideVec<T>::value;
    constexpr int UNROLL = 1;
    bool ok = aligned16(out);
    for (int j = 0; j < NIN; ++j) ok = ok && aligned16(in[j]);
    const uint64_t nvec = ok ? n / VEC : 0;
    const uint64_t tail_start = nvec * VEC;
    if (nvec > 0) {
        EwArgs<T, NIN> a;
        for (int j = 0; j < NIN; ++j) a.in[j] = (const T*)in[j];
        a.out = (T*)out; a.nvec = nvec; a.acc = acc;
        const uint64_t per_block = (uint64_t)kEwBlock * UNROLL;
        const uint64_t grid = (nvec + per_block - 1) / per_block;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "element-wise: %llu elements is too many", (unsigned long long)n);
        hipLaunchKernelGGL((ew_kernel<T, VEC, UNROLL, NIN, F>), dim3((uint32_t)grid), dim3(kEwBlock), 0, s, a);
    }
    if (tail_start < n) {
        EwArgs<T, NIN> a;
        for (int j = 0; j < NIN; ++j) a.in[j] = (const T*)in[j] + tail_start;
        a.out = (T*)out + tail_start; a.nvec = n - tail_start; a.acc = acc;
        const uint64_t per_block = (uint64_t)kEwBlock * 4;
        const uint64_t grid = (a.nvec + per_block - 1) / per_block;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "element-wise: %llu elements is too many", (unsigned long long)n);
        hipLaunchKernelGGL((ew_kernel<T, 1, 4, NIN, F>), dim3((uint32_t)grid), dim3(kEwBlock), 0, s, a);
    }
    return check_hip(hipGetLastError(), "element-wise launch");
}

template <int NIN, typename F>
int ew_launch(hipStream_t s, int dtype, const void* const (&in)[NIN], void* out, uint64_t n, int acc,
              const char* what) {
    for (int j = 0; j < NIN; ++j)
        if (in[j] == nullptr && n > 0) return set_error(AGRAD_EINVAL, "%s: null input %d", what, j);
    if (out == nullptr && n > 0) return set_error(AGRAD_EINVAL, "%s: null output", what);
    if (dtype == AGRAD_F32) return ew_launch_typed<float, NIN, F>(s, in, out, n, acc);
    if (dtype == AGRAD_BF16) return ew_launch_typed<bf16_t, NIN, F>(s, in, out, n, acc);
    return set_error(AGRAD_EINVAL, "%s: unknown dtype %d", what, dtype);
}

}  // namespace agrad
