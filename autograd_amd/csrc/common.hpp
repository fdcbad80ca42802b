// Device-side building blocks shared by every gfx950 kernel in this library:
// 128-bit vector I/O for fp32 and bf16 storage, the bf16 rounding rule, and
// wave64 / workgroup sum reductions built on DPP and ds_swizzle.
//
// All arithmetic is fp32 with contraction disabled at compile time
// (-ffp-contract=off): every multiply and add rounds separately, which is what
// the numpy CPU kernels of the reference do (backend.py:376-487, 1097-1126).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "fastdiv.hpp"

namespace agrad {

constexpr int kWave = 64;

typedef uint16_t bf16_t;  // raw bfloat16 storage bits

// fp32 -> bf16, round to nearest even; Inf kept; NaN keeps its high half with
// the quiet bit forced (reference rule: utils.py:20-27, metal_ops.metal:12010-12041).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    uint32_t special = (u >> 16) | ((u & 0x007fffffu) ? 0x0040u : 0u);
    return ((u & 0x7f800000u) == 0x7f800000u) ? special : rounded;
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) {
    return __uint_as_float(b << 16);
}

// exp(x) for fp32 streams: 2^(x * log2(e)) on the hardware exp2, with the rounding
// error of the product and the low part of the constant carried into a
// first-order correction.  Within ~1.5 ulp of exp(x) over the whole fp32 range, a
// third of the instructions of expf (which makes an fp32 softmax stream
// instruction-bound on this GPU).  Arguments below -200 give 0, above 89 +inf.
constexpr float kLog2eHi = 1.44269504088896341f;
constexpr float kLog2eLo = 1.92596299112661746e-8f;   // log2(e) - (float)log2(e)
constexpr float kLn2 = 0.693147180559945309f;
__device__ __forceinline__ float exp_compensated(float x) {
    x = fminf(fmaxf(x, -200.0f), 89.0f);   // keeps +-inf out of the fma; exp(-200) = 0, exp(89) = inf in fp32
    const float t = x * kLog2eHi;
    const float lo = __builtin_fmaf(x, kLog2eHi, -t) + x * kLog2eLo;
    const float r = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(r, lo * kLn2, r);
}

// Two fp32 -> one packed pair of bf16 (a in the low half).  gfx950 converts a
// pair with round-to-nearest-even in one instruction (v_cvt_pk_bf16_f32); that
// takes every finite value and the infinities exactly where the integer rule
// above takes them.  NaNs are re-done with the integer rule so that the kept
// payload bits are the reference's.
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    const f32x2_hw v = {a, b};
    uint32_t r = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_hw));
    if (__builtin_expect(a != a, 0)) r = (r & 0xffff0000u) | f32_to_bf16_bits(a);
    if (__builtin_expect(b != b, 0)) r = (r & 0x0000ffffu) | (f32_to_bf16_bits(b) << 16);
    return r;
}

// ---------------------------------------------------------------------------
// Vector I/O.  VecIO<T, V> moves V consecutive elements between memory and an
// fp32 register array.  (float,4) and (bf16,8) are one 128-bit access.
// ---------------------------------------------------------------------------
// Activations and gradients are touched once per kernel, so their accesses
// carry the non-temporal hint (measured on MI355X: a plain copy goes from 5.6 to
// 6.5 TB/s with it).  Small re-read operands (gamma, beta, rotary tables, token
// ids, partial sums) use ordinary loads and stay cached.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T, int V> struct VecIO;

template <> struct VecIO<float, 4> {
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        f32x4 t; t.x = v[0]; t.y = v[1]; t.z = v[2]; t.w = v[3];
        __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(p));
    }
};

template <> struct VecIO<float, 1> {
    static __device__ __forceinline__ void load(const float* p, float (&v)[1]) { v[0] = __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ void store(float* p, const float (&v)[1]) { __builtin_nontemporal_store(v[0], p); }
};

template <> struct VecIO<bf16_t, 8> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
        const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i]     = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
        u32x4 t; t.x = w[0]; t.y = w[1]; t.z = w[2]; t.w = w[3];
        __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
    }
};

// four bf16 values: one 8-byte access (the bf16 gradient row of an fp32 upstream)
template <> struct VecIO<bf16_t, 4> {
    typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
        const u32x2_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
        v[0] = __builtin_bit_cast(float, t.x << 16);
        v[1] = __builtin_bit_cast(float, t.x & 0xffff0000u);
        v[2] = __builtin_bit_cast(float, t.y << 16);
        v[3] = __builtin_bit_cast(float, t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
        u32x2_t t;
        t.x = f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16);
        t.y = f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16);
        __builtin_nontemporal_store(t, reinterpret_cast<u32x2_t*>(p));
    }
};

template <> struct VecIO<bf16_t, 1> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[1]) {
        v[0] = bf16_bits_to_f32(__builtin_nontemporal_load(p));
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[1]) {
        __builtin_nontemporal_store((bf16_t)f32_to_bf16_bits(v[0]), p);
    }
};

// Raw access: the bits of one vector as loaded, unpacked to fp32 later.  A
// kernel that prefetches the next row keeps it in this form, so the wait for
// the data sits where the values are first used, not where they were requested.
template <typename T, int V> struct RawVec;
template <> struct RawVec<float, 4> {
    typedef f32x4 type;
    static __device__ __forceinline__ type load(const float* p) { return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p)); }
    static __device__ __forceinline__ type zero() { return f32x4{0.0f, 0.0f, 0.0f, 0.0f}; }
    static __device__ __forceinline__ void unpack(const type& r, float (&v)[4]) { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
};
template <> struct RawVec<bf16_t, 8> {
    typedef u32x4 type;
    static __device__ __forceinline__ type load(const bf16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }
    static __device__ __forceinline__ type zero() { return u32x4{0u, 0u, 0u, 0u}; }
    static __device__ __forceinline__ void unpack(const type& r, float (&v)[8]) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i]     = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};

template <> struct RawVec<float, 1> {
    typedef float type;
    static __device__ __forceinline__ type load(const float* p) { return __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ type zero() { return 0.0f; }
    static __device__ __forceinline__ void unpack(const type& r, float (&v)[1]) { v[0] = r; }
};
template <> struct RawVec<bf16_t, 1> {
    typedef bf16_t type;
    static __device__ __forceinline__ type load(const bf16_t* p) { return __builtin_nontemporal_load(p); }
    static __device__ __forceinline__ type zero() { return 0; }
    static __device__ __forceinline__ void unpack(const type& r, float (&v)[1]) { v[0] = bf16_bits_to_f32(r); }
};

// Widest vector a dtype supports (16 bytes).
template <typename T> struct WideVec;
template <> struct WideVec<float>  { static constexpr int value = 4; };
template <> struct WideVec<bf16_t> { static constexpr int value = 8; };

// ---------------------------------------------------------------------------
// Cross-lane sums.  A wave64 is four DPP rows of 16 lanes: quad_perm and the
// row mirrors fold a row without touching LDS, ds_swizzle folds row pairs, and
// two readlanes fold the two 32-lane halves into a wave-uniform value.
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

constexpr int kDppQuadXor1      = 0xB1;   // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2      = 0x4E;   // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror     = 0x140;
constexpr int kSwizzleXor16     = 0x401F; // bit mode: and 0x1f, or 0, xor 0x10

// Sum over aligned groups of TPR lanes (TPR = 16, 32 or 64); every lane of a
// group receives the group's total.  A group never reads lanes outside itself,
// so neighbouring groups of one wave may be masked off independently.
template <int TPR>
__device__ __forceinline__ float lanes_sum(float v) {
    static_assert(TPR == 16 || TPR == 32 || TPR == 64, "lane group must be 16, 32 or 64");
    v = v + dpp_move<kDppQuadXor1>(v);
    v = v + dpp_move<kDppQuadXor2>(v);
    v = v + dpp_move<kDppRowHalfMirror>(v);
    v = v + dpp_move<kDppRowMirror>(v);
    if constexpr (TPR >= 32)
        v = v + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), kSwizzleXor16));
    if constexpr (TPR == 64) {
        const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
        const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
        v = lo + hi;
    }
    return v;
}

// Two independent sums folded together so their DPP chains interleave.
template <int TPR>
__device__ __forceinline__ void lanes_sum2(float& a, float& b) {
    static_assert(TPR == 16 || TPR == 32 || TPR == 64, "lane group must be 16, 32 or 64");
    a = a + dpp_move<kDppQuadXor1>(a);       b = b + dpp_move<kDppQuadXor1>(b);
    a = a + dpp_move<kDppQuadXor2>(a);       b = b + dpp_move<kDppQuadXor2>(b);
    a = a + dpp_move<kDppRowHalfMirror>(a);  b = b + dpp_move<kDppRowHalfMirror>(b);
    a = a + dpp_move<kDppRowMirror>(a);      b = b + dpp_move<kDppRowMirror>(b);
    if constexpr (TPR >= 32) {
        a = a + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, a), kSwizzleXor16));
        b = b + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, b), kSwizzleXor16));
    }
    if constexpr (TPR == 64) {
        const float a0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a), 0));
        const float a1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a), 32));
        const float b0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b), 0));
        const float b1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b), 32));
        a = a0 + a1;
        b = b0 + b1;
    }
}

__device__ __forceinline__ float wave_sum(float v) { return lanes_sum<kWave>(v); }
__device__ __forceinline__ void wave_sum2(float& a, float& b) { lanes_sum2<kWave>(a, b); }

// Sum over the TPR threads that share one row.  TPR <= 64: pure DPP.  TPR > 64:
// each wave's total is staged in LDS and every thread adds the staged totals in
// wave order.  `slot` selects one of a few LDS lines so that consecutive
// reductions need only one barrier each (a slot is kRowSumSlot*TPR/64 floats;
// rotate at least two slots).  Callers with TPR > 64 run exactly one row per workgroup, so
// the barrier is reached by the whole workgroup.
constexpr int kRowSumSlot = 3;   // values one reduction may stage per wave

template <int TPR>
__device__ __forceinline__ float row_sum(float v, float* lds, int slot) {
    if constexpr (TPR <= kWave) {
        return lanes_sum<TPR>(v);
    } else {
        v = wave_sum(v);
        constexpr int NW = TPR / kWave;
        float* line = lds + slot * kRowSumSlot * NW;
        if ((threadIdx.x & (kWave - 1)) == 0) line[threadIdx.x / kWave] = v;
        __syncthreads();
        float t = line[0];
#pragma unroll
        for (int w = 1; w < NW; ++w) t = t + line[w];
        return t;
    }
}

template <int TPR>
__device__ __forceinline__ void row_sum2(float& a, float& b, float* lds, int slot) {
    if constexpr (TPR <= kWave) {
        lanes_sum2<TPR>(a, b);
    } else {
        wave_sum2(a, b);
        constexpr int NW = TPR / kWave;
        float* line = lds + slot * kRowSumSlot * NW;
        if ((threadIdx.x & (kWave - 1)) == 0) {
            line[threadIdx.x / kWave] = a;
            line[NW + threadIdx.x / kWave] = b;
        }
        __syncthreads();
        float ta = line[0], tb = line[NW];
#pragma unroll
        for (int w = 1; w < NW; ++w) { ta = ta + line[w]; tb = tb + line[NW + w]; }
        a = ta; b = tb;
    }
}

// three sums in one phase (one barrier when TPR > 64)
template <int TPR>
__device__ __forceinline__ void row_sum3(float& a, float& b, float& c, float* lds, int slot) {
    if constexpr (TPR <= kWave) {
        lanes_sum2<TPR>(a, b);
        c = lanes_sum<TPR>(c);
    } else {
        wave_sum2(a, b);
        c = wave_sum(c);
        constexpr int NW = TPR / kWave;
        float* line = lds + slot * kRowSumSlot * NW;
        if ((threadIdx.x & (kWave - 1)) == 0) {
            line[threadIdx.x / kWave] = a;
            line[NW + threadIdx.x / kWave] = b;
            line[2 * NW + threadIdx.x / kWave] = c;
        }
        __syncthreads();
        float ta = line[0], tb = line[NW], tc = line[2 * NW];
#pragma unroll
        for (int w = 1; w < NW; ++w) { ta = ta + line[w]; tb = tb + line[NW + w]; tc = tc + line[2 * NW + w]; }
        a = ta; b = tb; c = tc;
    }
}

// Division of a 32-bit index by a divisor fixed at launch: one multiply-high and
// two shifts on the device (Granlund & Montgomery's round-up form) in place of
// the twenty-odd instructions of a hardware-less integer divide.  Exact for
// every n < 2^32 and 1 <= d < 2^32.
struct FastDiv32 {
    uint32_t d, mul, shift1, shift2;
    FastDiv32() : d(1), mul(1), shift1(0), shift2(0) {}
    explicit FastDiv32(uint32_t divisor) : d(divisor) {
        uint32_t l = 0;
        while (l < 32 && (1ull << l) < (uint64_t)divisor) ++l;          // ceil(log2 d)
        mul = (uint32_t)((((1ull << l) - divisor) << 32) / divisor + 1);
        shift1 = l < 1 ? l : 1;
        shift2 = l > 1 ? l - 1 : 0;
    }
    __device__ __forceinline__ uint32_t div(uint32_t n) const {
        const uint32_t t = __umulhi(mul, n);
        return (t + ((n - t) >> shift1)) >> shift2;
    }
    __device__ __forceinline__ uint32_t mod(uint32_t n) const { return n - div(n) * d; }
};

}  // namespace agrad
