// AdamW over a flat fp32 parameter slab, and the per-group sums of squares the
// gradient-norm clip needs.  Both are pure streams: AdamW reads p, g, m, v and
// writes p, m, v (28 bytes per element with fp32 gradients, 26 with bf16), the
// norm reads g once.
//
// The update is the reference CPU kernel's sequence, one rounding per numpy
// call (cpu_adamw_step, backend.py:2013-2038):
//     p -= p * (lr*wd)                       (only where weight decay applies)
//     m  = m*b1 + g*(1-b1)
//     v  = v*b2 + (g*g)*(1-b2)
//     p -= (m / (sqrt(v) + eps)) * lr_t
// with the two extensions of the Metal kernel (adamw_step, metal_ops.metal:10139-10228):
// the gradient is first multiplied by grad_scale (the clip coefficient), sqrt(v)
// is multiplied by inv_sqrt_bc2 before eps is added, the first decay_numel
// elements of the slab are the decayed ones, and the gradient may be bf16.
// With grad_scale = inv_sqrt_bc2 = 1 those multiplies are exact and the result
// is the CPU kernel's bit for bit (division and square root are IEEE here).
#include "common.hpp"
#include "launch.hpp"

namespace agrad {

namespace {

constexpr int kOptBlock = 64;

struct AdamwArgs {
    float* p; const void* g; float* m; float* v;
    uint64_t n;            // elements (vector kernel: groups of 4)
    uint64_t decay_n;      // elements [0, decay_n) get weight decay
    float lr_wd, b1, one_minus_b1, b2, one_minus_b2, eps, step_lr, inv_sqrt_bc2, grad_scale;
};

__device__ __forceinline__ void adamw_one(float& p, float g, float& m, float& v, bool decay, const AdamwArgs& a) {
    if (a.grad_scale != 1.0f) g = g * a.grad_scale;
    if (decay) {
        const float t = p * a.lr_wd;
        p = p - t;
    }
    float t = g * a.one_minus_b1;
    m = m * a.b1;
    m = m + t;
    v = v * a.b2;
    t = g * g;
    t = t * a.one_minus_b2;
    v = v + t;
    t = sqrtf(v);
    if (a.inv_sqrt_bc2 != 1.0f) t = t * a.inv_sqrt_bc2;
    t = t + a.eps;
    t = m / t;
    t = t * a.step_lr;
    p = p - t;
}

template <typename G> __device__ __forceinline__ void load_grad4(const G* g, float (&v)[4]);
template <> __device__ __forceinline__ void load_grad4<float>(const float* g, float (&v)[4]) {
    VecIO<float, 4>::load(g, v);
}
template <> __device__ __forceinline__ void load_grad4<bf16_t>(const bf16_t* g, float (&v)[4]) {
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 r = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(g));
    v[0] = __builtin_bit_cast(float, r.x << 16);
    v[1] = __builtin_bit_cast(float, r.x & 0xffff0000u);
    v[2] = __builtin_bit_cast(float, r.y << 16);
    v[3] = __builtin_bit_cast(float, r.y & 0xffff0000u);
}

// one group of 4 elements per thread
template <typename G>
__global__ void __launch_bounds__(kOptBlock) adamw_vec_kernel(const AdamwArgs a) {
    const uint64_t idx = (uint64_t)blockIdx.x * kOptBlock + threadIdx.x;
    if (idx >= a.n) return;
    const uint64_t e0 = idx * 4;
    float p[4], g[4], m[4], v[4];
    VecIO<float, 4>::load(a.p + e0, p);
    load_grad4<G>(static_cast<const G*>(a.g) + e0, g);
    VecIO<float, 4>::load(a.m + e0, m);
    VecIO<float, 4>::load(a.v + e0, v);
    const bool wd = a.lr_wd != 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) adamw_one(p[k], g[k], m[k], v[k], wd && e0 + k < a.decay_n, a);
    VecIO<float, 4>::store(a.p + e0, p);
    VecIO<float, 4>::store(a.m + e0, m);
    VecIO<float, 4>::store(a.v + e0, v);
}

// element-wise variant for tails and unaligned slabs; `first` is the index of
// element 0 of this launch within the slab (for the decay boundary)
template <typename G>
__global__ void __launch_bounds__(kOptBlock) adamw_scalar_kernel(const AdamwArgs a, uint64_t first) {
    const uint64_t i = (uint64_t)blockIdx.x * kOptBlock + threadIdx.x;
    if (i >= a.n) return;
    float g[1];
    VecIO<G, 1>::load(static_cast<const G*>(a.g) + i, g);
    float p = a.p[i], m = a.m[i], v = a.v[i];
    adamw_one(p, g[0], m, v, a.lr_wd != 0.0f && first + i < a.decay_n, a);
    a.p[i] = p; a.m[i] = m; a.v[i] = v;
}

// partial[i] = sum of squares of elements [256 i, 256 i + 256)  (grad_norm_sq,
// metal_ops.metal:10103-10137: one partial per 256 elements, summed on the host
// in float64).  A lane reads 16 bytes at a time, so a group is 64 lanes of fp32
// or 32 lanes of bf16; a wave takes kNormChunks consecutive kilobytes with all
// its loads in flight, each lane adds its squares in element order, and the
// lanes of a group are added by the fixed cross-lane tree.
constexpr int kNormChunks = 4;

template <typename G>
__global__ void __launch_bounds__(256) grad_norm_sq_kernel(const G* __restrict__ g, float* __restrict__ partial,
                                                            uint64_t n, uint64_t groups) {
    constexpr int VEC = WideVec<G>::value;            // elements per 16-byte load
    constexpr int LANES = 256 / VEC;                  // lanes per group: 64 or 32
    constexpr int GPW = kWave / LANES;                // groups per wave per chunk: 1 or 2
    const uint64_t wave = (uint64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    const uint32_t lane = threadIdx.x % kWave;
    const uint64_t first_group = wave * (kNormChunks * GPW);
    if (first_group >= groups) return;                // whole waves leave together
    float x[kNormChunks][VEC];
#pragma unroll
    for (int c = 0; c < kNormChunks; ++c) {
        const uint64_t e0 = (first_group + (uint64_t)c * GPW) * 256 + (uint64_t)lane * VEC;
        if (e0 + VEC <= n) {
            VecIO<G, VEC>::load(g + e0, x[c]);
        } else {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float one[1] = {0.0f};
                if (e0 + k < n) VecIO<G, 1>::load(g + e0 + k, one);
                x[c][k] = one[0];
            }
        }
    }
#pragma unroll
    for (int c = 0; c < kNormChunks; ++c) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < VEC; ++k) s = s + x[c][k] * x[c][k];
        s = lanes_sum<LANES>(s);
        const uint64_t group = first_group + (uint64_t)c * GPW + lane / LANES;
        if (lane % LANES == 0 && group < groups) partial[group] = s;
    }
}

// any alignment: one wave per group, element-wise loads
template <typename G>
__global__ void __launch_bounds__(256) grad_norm_sq_scalar_kernel(const G* __restrict__ g, float* __restrict__ partial,
                                                                   uint64_t n, uint64_t groups) {
    const uint64_t group = (uint64_t)blockIdx.x * 4 + threadIdx.x / kWave;
    if (group >= groups) return;
    const uint32_t lane = threadIdx.x % kWave;
    float s = 0.0f;
    for (int k = 0; k < 4; ++k) {
        const uint64_t e = group * 256 + (uint64_t)lane * 4 + k;
        if (e < n) {
            float one[1];
            VecIO<G, 1>::load(g + e, one);
            s = s + one[0] * one[0];
        }
    }
    s = wave_sum(s);
    if (lane == 0) partial[group] = s;
}

template <typename G>
int adamw_typed(hipStream_t s, AdamwArgs a, uint64_t numel) {
    const bool vec = aligned16(a.p) && aligned16(a.m) && aligned16(a.v) &&
                     (reinterpret_cast<uintptr_t>(a.g) % (4 * sizeof(G)) == 0);
    const uint64_t nvec = vec ? numel / 4 : 0;
    if (nvec > 0) {
        const uint64_t grid = (nvec + kOptBlock - 1) / kOptBlock;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "adamw: %llu elements is too many for one call", (unsigned long long)numel);
        AdamwArgs b = a;
        b.n = nvec;
        hipLaunchKernelGGL((adamw_vec_kernel<G>), dim3((uint32_t)grid), dim3(kOptBlock), 0, s, b);
    }
    const uint64_t done = nvec * 4;
    if (done < numel) {
        AdamwArgs b = a;
        b.p += done; b.m += done; b.v += done;
        b.g = static_cast<const G*>(a.g) + done;
        b.n = numel - done;
        const uint64_t grid = (b.n + kOptBlock - 1) / kOptBlock;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "adamw: %llu elements is too many for one call", (unsigned long long)numel);
        hipLaunchKernelGGL((adamw_scalar_kernel<G>), dim3((uint32_t)grid), dim3(kOptBlock), 0, s, b, done);
    }
    return check_hip(hipGetLastError(), "adamw launch");
}

}  // namespace

int launch_adamw(hipStream_t s, int grad_dtype, float* p, const void* g, float* m, float* v,
                 uint64_t numel, uint64_t decay_numel, float lr_wd, float b1, float one_minus_b1,
                 float b2, float one_minus_b2, float eps, float step_lr, float inv_sqrt_bc2, float grad_scale) {
    if (grad_dtype != AGRAD_F32 && grad_dtype != AGRAD_BF16)
        return set_error(AGRAD_EINVAL, "adamw: unknown gradient dtype %d", grad_dtype);
    if (numel == 0) return AGRAD_OK;
    if (p == nullptr || g == nullptr || m == nullptr || v == nullptr) return set_error(AGRAD_EINVAL, "adamw: null operand");
    if (decay_numel > numel) return set_error(AGRAD_EINVAL, "adamw: decay_numel %llu > numel %llu",
                                              (unsigned long long)decay_numel, (unsigned long long)numel);
    AdamwArgs a{p, g, m, v, numel, decay_numel, lr_wd, b1, one_minus_b1, b2, one_minus_b2, eps, step_lr,
                inv_sqrt_bc2, grad_scale};
    if (grad_dtype == AGRAD_F32) return adamw_typed<float>(s, a, numel);
    return adamw_typed<bf16_t>(s, a, numel);
}

uint64_t grad_norm_groups(uint64_t numel) { return (numel + 255) / 256; }

int launch_grad_norm_sq(hipStream_t s, int dtype, const void* g, float* partial, uint64_t numel) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "grad norm: unknown dtype %d", dtype);
    if (numel == 0) return AGRAD_OK;
    if (g == nullptr || partial == nullptr) return set_error(AGRAD_EINVAL, "grad norm: null operand");
    const uint64_t groups = grad_norm_groups(numel);
    const int gpw = dtype == AGRAD_F32 ? 1 : 2;
    const bool vec = aligned16(g);
    const uint64_t waves = vec ? (groups + kNormChunks * gpw - 1) / (kNormChunks * gpw) : groups;
    const uint64_t grid = (waves + 3) / 4;
    if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "grad norm: %llu elements is too many for one call", (unsigned long long)numel);
    if (dtype == AGRAD_F32) {
        if (vec) hipLaunchKernelGGL((grad_norm_sq_kernel<float>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)g, partial, numel, groups);
        else hipLaunchKernelGGL((grad_norm_sq_scalar_kernel<float>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)g, partial, numel, groups);
    } else {
        if (vec) hipLaunchKernelGGL((grad_norm_sq_kernel<bf16_t>), dim3((uint32_t)grid), dim3(256), 0, s, (const bf16_t*)g, partial, numel, groups);
        else hipLaunchKernelGGL((grad_norm_sq_scalar_kernel<bf16_t>), dim3((uint32_t)grid), dim3(256), 0, s, (const bf16_t*)g, partial, numel, groups);
    }
    return check_hip(hipGetLastError(), "grad norm launch");
}

}  // namespace agrad
