// GELU-tanh, ReLU^2 and SwiGLU, forward and backward.  Pure streaming: the
// roofline is HBM bandwidth, the arithmetic is a few fp32 ops per element plus
// one tanhf / expf.
//
// Operation order is the reference CPU kernels' (each multiply / add rounds
// separately): GELU backend.py:376-414 with the constants of backend.py:18-20,
// SwiGLU backend.py:1113-1126 and 1206-1217.  ReLU^2 has no counterpart in the
// reference: y = max(x, 0)^2, dx = (2 max(x, 0)) dy.
#include "elementwise.hpp"
#include "gelu_math.hpp"

namespace agrad {

namespace {

struct GeluFwd {
    static __device__ __forceinline__ float apply(const float (&in)[1]) { return gelu_value(in[0]); }
};

// in[0] = x, in[1] = dy
struct GeluBwd {
    static __device__ __forceinline__ float apply(const float (&in)[2]) { return in[1] * gelu_slope(in[0]); }
};

struct Relu2Fwd {
    static __device__ __forceinline__ float apply(const float (&in)[1]) {
        const float r = in[0] > 0.0f ? in[0] : 0.0f;
        return r * r;
    }
};

struct Relu2Bwd {
    static __device__ __forceinline__ float apply(const float (&in)[2]) {
        const float r = in[0] > 0.0f ? in[0] : 0.0f;
        return (2.0f * r) * in[1];
    }
};

__device__ __forceinline__ float sigmoid_ref(float g) {
    float h = -g;
    h = expf(h);
    h = h + 1.0f;
    return 1.0f / h;
}

// The sigmoid by I/O type.  fp32 tensors get the reference's sequence (accurate
// expf, IEEE division: the fp32 kernels are memory-bound with it).  bf16 tensors round their result to 8 significant bits,
// and at 2 bytes per element the accurate sequence (about 25 instructions) makes
// the kernel instruction-bound rather than memory-bound; the hardware exp2 and
// reciprocal (1 ulp each) are indistinguishable after the bf16 rounding.
template <typename T> __device__ __forceinline__ float sigmoid_io(float g) { return sigmoid_ref(g); }
template <> __device__ __forceinline__ float sigmoid_io<bf16_t>(float g) {
    const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896341f);   // exp(-g); overflows to +inf -> result 0
    return __builtin_amdgcn_rcpf(1.0f + e);
}

// gu[rows, 2H] -> h[rows, HV * VEC]: columns h0 ... h0 + HV * VEC - 1 of the gate and up
// halves, written densely (the whole width when h0 = 0 and HV * VEC = H; a column tile
// otherwise: swiglu_forward_tile_kernel, metal_ops.metal:12043-12088).  A "vector" is VEC
// consecutive columns of one row.
template <typename T, int VEC, int UNROLL>
__global__ void __launch_bounds__(kEwBlock)
swiglu_fwd_kernel(const T* __restrict__ gu, T* __restrict__ h, uint32_t H, uint32_t h0, uint32_t HV, uint32_t nvec) {
    const uint32_t first = blockIdx.x * (kEwBlock * UNROLL) + threadIdx.x;
    float g[UNROLL][VEC], u[UNROLL][VEC];
    uint64_t off_out[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint32_t idx = first + j * kEwBlock;
        if (idx < nvec) {
            const uint32_t row = idx / HV;
            const uint32_t col = (idx - row * HV) * VEC;
            const uint64_t off_in = (uint64_t)row * 2 * H + h0 + col;
            off_out[j] = (uint64_t)row * HV * VEC + col;
            VecIO<T, VEC>::load(gu + off_in, g[j]);
            VecIO<T, VEC>::load(gu + off_in + H, u[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint32_t idx = first + j * kEwBlock;
        if (idx < nvec) {
            float o[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float t = sigmoid_io<T>(g[j][k]);
                t = g[j][k] * t;
                o[k] = t * u[j][k];
            }
            VecIO<T, VEC>::store(h + off_out[j], o);
        }
    }
}

// dgu[rows, 2H] = [dg | du] from gu and dh; dgu may be gu itself (each thread
// reads its g, u before it writes the same addresses).
template <typename T, int VEC, int UNROLL>
__global__ void __launch_bounds__(kEwBlock)
swiglu_bwd_kernel(const T* gu, const T* __restrict__ dh, T* dgu, uint32_t H, uint32_t HV,
                  uint32_t nvec, int acc) {
    const uint32_t first = blockIdx.x * (kEwBlock * UNROLL) + threadIdx.x;
    float g[UNROLL][VEC], u[UNROLL][VEC], d[UNROLL][VEC];
    uint64_t off_gu[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint32_t idx = first + j * kEwBlock;
        if (idx < nvec) {
            const uint32_t row = idx / HV;
            const uint32_t col = (idx - row * HV) * VEC;
            off_gu[j] = (uint64_t)row * 2 * H + col;
            VecIO<T, VEC>::load(gu + off_gu[j], g[j]);
            VecIO<T, VEC>::load(gu + off_gu[j] + H, u[j]);
            VecIO<T, VEC>::load(dh + (uint64_t)row * H + col, d[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint32_t idx = first + j * kEwBlock;
        if (idx < nvec) {
            float dg[VEC], du[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float sg = sigmoid_io<T>(g[j][k]);
                float t = 1.0f - sg;
                t = t * g[j][k];
                t = t + 1.0f;
                t = t * sg;
                t = t * u[j][k];
                dg[k] = t * d[j][k];
                float w = g[j][k] * sg;
                du[k] = w * d[j][k];
            }
            if (acc) {
                float og[VEC], ou[VEC];
                VecIO<T, VEC>::load(dgu + off_gu[j], og);
                VecIO<T, VEC>::load(dgu + off_gu[j] + H, ou);
#pragma unroll
                for (int k = 0; k < VEC; ++k) { dg[k] = og[k] + dg[k]; du[k] = ou[k] + du[k]; }
            }
            VecIO<T, VEC>::store(dgu + off_gu[j], dg);
            VecIO<T, VEC>::store(dgu + off_gu[j] + H, du);
        }
    }
}

// The backward kernel has five streams (gate, up and dh in; dgate and dup out), and with
// every wave slot of the GPU filled they reach 0.91 of what a two-stream copy reaches: the
// more loads and stores of five streams are in flight at once, the more DRAM pages they keep
// open against each other.  Dynamic LDS that the kernel never touches caps the workgroups
// (one wave each) of a CU at sixteen instead of thirty-two: 65536 x 14336 bf16 1513 -> 1400
// us, 16384 x 8960 fp32 469 -> 451 us, bf16 225 -> 220 us.  (Eight: 20 % slower -- the
// sigmoid needs waves to hide behind.  The forward kernel, three streams, gains nothing, and
// the two- and three-stream elementwise kernels lose from any cap.)
constexpr int kSwigluBwdPerCu = 16;
static_assert(kEwBlock == kWave, "the occupancy cap counts one-wave workgroups");

// Rows are processed in slabs small enough for 32-bit vector indices.
template <typename T, int VEC>
int swiglu_typed(hipStream_t s, const T* gu, const T* dh, T* out, uint64_t rows, uint32_t H,
                 bool backward, int acc, uint32_t h0 = 0, uint32_t hw = 0) {
    constexpr int UNROLL = 1;
    if (hw == 0) hw = H;                       // forward only: the column tile [h0, h0 + hw)
    const uint32_t HV = hw / VEC;
    const uint64_t max_rows = 0xf0000000ull / HV;
    for (uint64_t r0 = 0; r0 < rows; r0 += max_rows) {
        const uint64_t nr = rows - r0 < max_rows ? rows - r0 : max_rows;
        const uint32_t nvec = (uint32_t)(nr * HV);
        const uint32_t per_block = kEwBlock * UNROLL;
        const uint32_t grid = (nvec + per_block - 1) / per_block;
        if (!backward) {
            hipLaunchKernelGGL((swiglu_fwd_kernel<T, VEC, UNROLL>), dim3(grid), dim3(kEwBlock), 0, s,
                               gu + r0 * 2 * H, out + r0 * hw, H, h0, HV, nvec);
        } else {
            hipLaunchKernelGGL((swiglu_bwd_kernel<T, VEC, UNROLL>), dim3(grid), dim3(kEwBlock), VEC > 1 ? idle_lds_for(kSwigluBwdPerCu) : 0u, s,
                               gu + r0 * 2 * H, dh + r0 * H, out + r0 * 2 * H, H, HV, nvec, acc);
        }
    }
    return check_hip(hipGetLastError(), "swiglu launch");
}

template <typename T>
int swiglu_dispatch(hipStream_t s, const void* gu, const void* dh, void* out, uint64_t rows,
                    uint32_t H, bool backward, int acc) {
    constexpr int VEC = WideVec<T>::value;
    const bool wide = H % VEC == 0 && aligned16(gu) && aligned16(out) && (!dh || aligned16(dh));
    if (wide) return swiglu_typed<T, VEC>(s, (const T*)gu, (const T*)dh, (T*)out, rows, H, backward, acc);
    return swiglu_typed<T, 1>(s, (const T*)gu, (const T*)dh, (T*)out, rows, H, backward, acc);
}

template <typename T>
int swiglu_tile_dispatch(hipStream_t s, const void* gu, void* out, uint64_t rows, uint32_t H, uint32_t h0, uint32_t hw) {
    constexpr int VEC = WideVec<T>::value;
    const bool wide = H % VEC == 0 && h0 % VEC == 0 && hw % VEC == 0 && aligned16(gu) && aligned16(out);
    if (wide) return swiglu_typed<T, VEC>(s, (const T*)gu, nullptr, (T*)out, rows, H, false, 0, h0, hw);
    return swiglu_typed<T, 1>(s, (const T*)gu, nullptr, (T*)out, rows, H, false, 0, h0, hw);
}

}  // namespace

int launch_gelu_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t n) {
    const void* in[1] = {x};
    return ew_launch<1, GeluFwd>(s, dtype, in, y, n, 0, "gelu forward");
}
int launch_gelu_bwd(hipStream_t s, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags) {
    const void* in[2] = {x, dy};
    return ew_launch<2, GeluBwd>(s, dtype, in, dx, n, (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0, "gelu backward");
}
int launch_relu2_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t n) {
    const void* in[1] = {x};
    return ew_launch<1, Relu2Fwd>(s, dtype, in, y, n, 0, "relu2 forward");
}
int launch_relu2_bwd(hipStream_t s, int dtype, const void* x, const void* dy, void* dx, uint64_t n, uint32_t flags) {
    const void* in[2] = {x, dy};
    return ew_launch<2, Relu2Bwd>(s, dtype, in, dx, n, (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0, "relu2 backward");
}

int launch_swiglu_fwd(hipStream_t s, int dtype, const void* gu, void* h, uint64_t rows, uint32_t H) {
    if (rows == 0 || H == 0) return AGRAD_OK;
    if (gu == nullptr || h == nullptr) return set_error(AGRAD_EINVAL, "swiglu forward: null operand");
    if (dtype == AGRAD_F32) return swiglu_dispatch<float>(s, gu, nullptr, h, rows, H, false, 0);
    if (dtype == AGRAD_BF16) return swiglu_dispatch<bf16_t>(s, gu, nullptr, h, rows, H, false, 0);
    return set_error(AGRAD_EINVAL, "swiglu forward: unknown dtype %d", dtype);
}

int launch_swiglu_fwd_tile(hipStream_t s, int dtype, const void* gu, void* tile, uint64_t rows, uint32_t H,
                           uint32_t h0, uint32_t hw) {
    if ((uint64_t)h0 + hw > H) return set_error(AGRAD_EINVAL, "swiglu tile: columns %u..%u of %u", h0, h0 + hw, H);
    if (rows == 0 || hw == 0) return AGRAD_OK;
    if (gu == nullptr || tile == nullptr) return set_error(AGRAD_EINVAL, "swiglu tile: null operand");
    if (dtype == AGRAD_F32) return swiglu_tile_dispatch<float>(s, gu, tile, rows, H, h0, hw);
    if (dtype == AGRAD_BF16) return swiglu_tile_dispatch<bf16_t>(s, gu, tile, rows, H, h0, hw);
    return set_error(AGRAD_EINVAL, "swiglu tile: unknown dtype %d", dtype);
}

int launch_swiglu_bwd(hipStream_t s, int dtype, const void* gu, const void* dh, void* dgu,
                      uint64_t rows, uint32_t H, uint32_t flags) {
    if (rows == 0 || H == 0) return AGRAD_OK;
    if (gu == nullptr || dh == nullptr || dgu == nullptr)
        return set_error(AGRAD_EINVAL, "swiglu backward: null operand");
    const int acc = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    if (acc && gu == dgu) return set_error(AGRAD_EINVAL, "swiglu backward: in-place and accumulate are exclusive");
    if (dtype == AGRAD_F32) return swiglu_dispatch<float>(s, gu, dh, dgu, rows, H, true, acc);
    if (dtype == AGRAD_BF16) return swiglu_dispatch<bf16_t>(s, gu, dh, dgu, rows, H, true, acc);
    return set_error(AGRAD_EINVAL, "swiglu backward: unknown dtype %d", dtype);
}

}  // namespace agrad
