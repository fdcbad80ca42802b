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
constexpr int kAdamwPerCu = 12;        // one-wave workgroups of the AdamW step that share a CU (seven streams: 5 to 7 % faster than 32)
static_assert(kOptBlock == kWave, "the occupancy cap counts one-wave workgroups");

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
        // (seven streams -- p, g, m, v in; p, m, v out: idle dynamic LDS caps a CU at twelve of
        // these one-wave workgroups, 3 to 4 % faster than with all thirty-two: see the SwiGLU backward)
        hipLaunchKernelGGL((adamw_vec_kernel<G>), dim3((uint32_t)grid), dim3(kOptBlock), idle_lds_for(kAdamwPerCu), s, b);
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

// ---- AdamW with 8-bit moments ----------------------------------------------------
// adamw8bit_step (metal_ops.metal:10229-10361; Backend.adamw8bit_step,
// backend.py:5142-5151; optimizer.py:143-232, 469-479): both moments are stored as
// one byte per element -- an index into a 256-entry sorted map of values in [-1, 1]
// (m) or [0, 1] (v) -- times one fp32 scale per block of 256 elements.  A step
// dequantises a block, applies the update with the operations and roundings of the
// Metal kernel, takes the block's new scales (max |m|, max v) and re-quantises each
// moment to the NEAREST map entry.  16 bytes of traffic per parameter instead of 28.
//
// One wave owns one block: lane l holds elements 4l .. 4l+3 (one 16-byte vector of
// p and of g, one 4-byte word of each code array), the block maximum is a wave
// reduction, and the maps sit in LDS for the code search.
//
// The step is bound by vector instructions, not by memory: about 150 per element
// (three correctly rounded divisions and a square root are 45 of them, the two code
// searches 40), 33 M wave instructions for 12.6 M parameters = 54 us of issue time
// on 1024 SIMDs, 62 us measured -- about the time of the fp32-moment step on the
// same parameters (58 us), for a quarter of its state memory.

constexpr uint64_t kAdamw8MaxGrid = 2048;     // workgroups (8 waves a SIMD; 1024 and 4096 were 10 % slower); each walks its share of the blocks

struct Adamw8Args {
    float* p; const void* g; uint8_t* qm; uint8_t* qv; float* absmax_m; float* absmax_v;
    const float* qmap_m; const float* qmap_v;
    uint64_t n, decay_n, nblocks;
    float decay, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip;
    int first_step, vec_ok;
};

namespace {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int mask = kWave / 2; mask >= 1; mask >>= 1) v = fmaxf(v, __shfl_xor(v, mask));
    return v;
}

// first index whose map entry is not below x, never past the last entry: eight
// bisection steps over the 256 sorted entries (metal_ops.metal:10326-10335)
__device__ __forceinline__ uint32_t first_not_below(const float* map, float x) {
    uint32_t lo = 0, hi = 255;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const uint32_t mid = (lo + hi) >> 1;
        if (map[mid] < x) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// The bisection costs eight dependent LDS reads and some fifty instructions per
// code, eight codes a lane.  So each workgroup first tabulates, for every
// "bucket" of float values (sign, exponent and five mantissa bits: 32 buckets an
// octave from 2^-27 up to 1), where the bisection would land for the bucket's
// lowest value; a code search then starts there and walks up -- at most three
// entries, since no bucket holds more of the map.  The result is the
// bisection's for ANY sorted map; only the speed assumes a map that is not
// much denser than 32 entries an octave.
constexpr uint32_t kBucketShift = 18;                          // float bits >> 18: exponent and 5 mantissa bits
constexpr uint32_t kBucketMin = (127 - 27) * 32;               // 2^-27
constexpr uint32_t kBuckets = 127 * 32 - kBucketMin + 1;       // up to 1.0, which has a bucket of its own

__device__ __forceinline__ uint32_t bucket_of(float magnitude) {
    const uint32_t key = __builtin_bit_cast(uint32_t, magnitude) >> kBucketShift;
    const uint32_t k = key > kBucketMin ? key - kBucketMin : 0u;
    return k < kBuckets ? k : kBuckets - 1;
}
__device__ __forceinline__ float bucket_floor(uint32_t k) {    // lowest magnitude of bucket k
    return k == 0 ? 0.0f : __builtin_bit_cast(float, (k + kBucketMin) << kBucketShift);
}

struct CodeTables {
    float map[256];
    uint8_t up[kBuckets];        // x >= 0 in bucket k: the search starts at up[k]
    uint8_t down[kBuckets];      // x < 0 with |x| in bucket k (values in (-ceil_k, -floor_k]): starts at down[k]
};

// Every thread of the workgroup; a barrier before and after belongs to the caller.  A
// thread takes a run of neighbouring buckets: the first by bisection, the others by
// walking on from it (the answers are monotone in the bucket and a step or two apart).
__device__ __forceinline__ void build_tables(CodeTables& t, bool is_signed) {
    const uint32_t per_thread = (kBuckets + blockDim.x - 1) / blockDim.x;
    const uint32_t k0 = threadIdx.x * per_thread;
    const uint32_t k1 = k0 + per_thread < kBuckets ? k0 + per_thread : kBuckets;
    if (k0 >= k1) return;
    uint32_t at = first_not_below(t.map, bucket_floor(k0));
    t.up[k0] = (uint8_t)at;
    for (uint32_t k = k0 + 1; k < k1; ++k) {                     // rising thresholds: walk up
        const float edge = bucket_floor(k);
        while (at < 255u && t.map[at] < edge) ++at;
        t.up[k] = (uint8_t)at;
    }
    if (!is_signed) return;
    // down[k] = first entry not below -bucket_floor(k + 1): falling thresholds, walk down
    at = k0 + 1 < kBuckets ? first_not_below(t.map, -bucket_floor(k0 + 1)) : 0u;
    t.down[k0] = (uint8_t)at;
    for (uint32_t k = k0 + 1; k < k1; ++k) {
        if (k + 1 < kBuckets) {
            const float edge = -bucket_floor(k + 1);
            while (at > 0u && !(t.map[at - 1] < edge)) --at;
        } else {
            at = 0u;
        }
        t.down[k] = (uint8_t)at;
    }
}

// Index of the map entry nearest to x: the first entry not below x, then the nearer of
// it and the entry below; a tie goes to the lower one (metal_ops.metal:10326-10343).
template <bool SIGNED>
__device__ __forceinline__ uint32_t nearest_code(const CodeTables& t, float x) {
    const uint32_t k = bucket_of(fabsf(x));
    uint32_t upper = (SIGNED && x < 0.0f) ? t.down[k] : t.up[k];
    // One step (two for the unsigned map, which is twice as dense) without a branch, so
    // that the searches of a lane's eight codes overlap their LDS reads; the loop behind
    // them only runs for a map denser than the usual one.
#pragma unroll
    for (int step = 0; step < (SIGNED ? 1 : 2); ++step) upper += (t.map[upper] < x && upper < 255u) ? 1u : 0u;
    float at_upper = t.map[upper];
    while (at_upper < x && upper < 255u) at_upper = t.map[++upper];
    const uint32_t lower = upper > 0 ? upper - 1 : 0;
    return fabsf(at_upper - x) < fabsf(t.map[lower] - x) ? upper : lower;
}

template <typename G> __device__ __forceinline__ float grad_elem(const void* g, uint64_t i);
template <> __device__ __forceinline__ float grad_elem<float>(const void* g, uint64_t i) { return static_cast<const float*>(g)[i]; }
template <> __device__ __forceinline__ float grad_elem<bf16_t>(const void* g, uint64_t i) {
    return bf16_bits_to_f32(static_cast<const bf16_t*>(g)[i]);
}

template <typename G>
__global__ void __launch_bounds__(256) adamw8bit_kernel(const Adamw8Args a) {
    __shared__ CodeTables tm, tv;
    tm.map[threadIdx.x] = a.qmap_m[threadIdx.x];
    tv.map[threadIdx.x] = a.qmap_v[threadIdx.x];
    __syncthreads();
    build_tables(tm, true);
    build_tables(tv, false);
    __syncthreads();
    const float* map_m = tm.map;
    const float* map_v = tv.map;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    // a workgroup walks blocks 4 apart per round of the grid, so that the tables above
    // are built a few thousand times per call, not once per four blocks
    for (uint64_t block = (uint64_t)blockIdx.x * (256 / kWave) + threadIdx.x / kWave; block < a.nblocks;
         block += (uint64_t)gridDim.x * (256 / kWave)) {
    const uint64_t e0 = block * 256 + (uint64_t)lane * 4;
    const uint32_t here = e0 >= a.n ? 0u : (a.n - e0 < 4 ? (uint32_t)(a.n - e0) : 4u);
    const bool vec = a.vec_ok && here == 4;
    const bool first = a.first_step != 0;

    float p[4] = {0.0f, 0.0f, 0.0f, 0.0f}, g[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t cm = 0, cv = 0;
    if (vec) {
        VecIO<float, 4>::load(a.p + e0, p);
        load_grad4<G>(static_cast<const G*>(a.g) + e0, g);
        if (!first) {
            cm = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(a.qm + e0));
            cv = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(a.qv + e0));
        }
    } else {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            if (k < here) {
                p[k] = a.p[e0 + k];
                g[k] = grad_elem<G>(a.g, e0 + k);
                if (!first) {
                    cm |= (uint32_t)a.qm[e0 + k] << (8 * k);
                    cv |= (uint32_t)a.qv[e0 + k] << (8 * k);
                }
            }
        }
    }
    const float old_m = first ? 0.0f : a.absmax_m[block], old_v = first ? 0.0f : a.absmax_v[block];
    const float one_minus_b1 = 1.0f - a.b1, one_minus_b2 = 1.0f - a.b2;
    float m[4], v[4], top_m = 0.0f, top_v = 0.0f;
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k) {
        m[k] = first ? 0.0f : old_m * map_m[(cm >> (8 * k)) & 255u];
        v[k] = first ? 0.0f : old_v * map_v[(cv >> (8 * k)) & 255u];
        if (k < here) {
            const float gk = g[k] * a.clip;
            p[k] = p[k] * (e0 + k < a.decay_n ? a.decay : 1.0f);
            const float dm = (gk - m[k]) * one_minus_b1;
            m[k] = m[k] + dm;
            const float gg = gk * gk;
            const float dv = (gg - v[k]) * one_minus_b2;
            v[k] = v[k] + dv;
            const float denom = sqrtf(fmaxf(v[k], 0.0f)) * a.inv_sqrt_bc2 + a.eps;
            const float dp = -(m[k] / denom) * a.lr_bc1;
            p[k] = p[k] + dp;
            top_m = fmaxf(top_m, fabsf(m[k]));
            top_v = fmaxf(top_v, fmaxf(v[k], 0.0f));
        }
    }
    const float scale_m = fmaxf(wave_max(top_m), 1.0e-30f);
    const float scale_v = fmaxf(wave_max(top_v), 1.0e-30f);
    if (lane == 0) {
        a.absmax_m[block] = scale_m;
        a.absmax_v[block] = scale_v;
    }
    uint32_t out_m = 0, out_v = 0;
#pragma unroll
    for (uint32_t k = 0; k < 4; ++k) {
        if (k < here) {
            const float mn = fminf(fmaxf(m[k] / scale_m, -1.0f), 1.0f);
            const float vn = fminf(fmaxf(fmaxf(v[k], 0.0f) / scale_v, 0.0f), 1.0f);
            out_m |= nearest_code<true>(tm, mn) << (8 * k);
            out_v |= nearest_code<false>(tv, vn) << (8 * k);
        }
    }
    if (vec) {
        VecIO<float, 4>::store(a.p + e0, p);
        __builtin_nontemporal_store(out_m, reinterpret_cast<uint32_t*>(a.qm + e0));
        __builtin_nontemporal_store(out_v, reinterpret_cast<uint32_t*>(a.qv + e0));
    } else {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            if (k < here) {
                a.p[e0 + k] = p[k];
                a.qm[e0 + k] = (uint8_t)(out_m >> (8 * k));
                a.qv[e0 + k] = (uint8_t)(out_v >> (8 * k));
            }
        }
    }
    }   // blocks of this wave
}

}  // namespace

int launch_adamw8bit(hipStream_t s, int grad_dtype, float* p, const void* g, uint8_t* qm, uint8_t* qv,
                     float* absmax_m, float* absmax_v, const float* qmap_m, const float* qmap_v,
                     uint64_t numel, uint64_t decay_numel, float decay, float lr_bc1, float b1, float b2, float eps,
                     float inv_sqrt_bc2, float clip_coef, int first_step) {
    if (grad_dtype != AGRAD_F32 && grad_dtype != AGRAD_BF16)
        return set_error(AGRAD_EINVAL, "adamw8bit: unknown gradient dtype %d", grad_dtype);
    if (numel == 0) return AGRAD_OK;
    if (p == nullptr || g == nullptr || qm == nullptr || qv == nullptr || absmax_m == nullptr || absmax_v == nullptr ||
        qmap_m == nullptr || qmap_v == nullptr)
        return set_error(AGRAD_EINVAL, "adamw8bit: null operand");
    if (decay_numel > numel) return set_error(AGRAD_EINVAL, "adamw8bit: decay_numel %llu > numel %llu",
                                              (unsigned long long)decay_numel, (unsigned long long)numel);
    Adamw8Args a{p, g, qm, qv, absmax_m, absmax_v, qmap_m, qmap_v, numel, decay_numel, (numel + 255) / 256,
                 decay, lr_bc1, b1, b2, eps, inv_sqrt_bc2, clip_coef, first_step ? 1 : 0, 0};
    a.vec_ok = aligned16(p) && aligned16(g) && ((uintptr_t)qm % 4 == 0) && ((uintptr_t)qv % 4 == 0) ? 1 : 0;
    uint64_t grid = (a.nblocks + 3) / 4;
    if (grid > kAdamw8MaxGrid) grid = kAdamw8MaxGrid;
    if (grad_dtype == AGRAD_F32) hipLaunchKernelGGL((adamw8bit_kernel<float>), dim3((uint32_t)grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((adamw8bit_kernel<bf16_t>), dim3((uint32_t)grid), dim3(256), 0, s, a);
    return check_hip(hipGetLastError(), "adamw8bit launch");
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
