// Split-half rotary embedding on q[B,T,H,D] and k[B,T,HKV,D], in place, both
// tensors in one launch.  Tables cos/sin are fp32 [T, D/2] and stay L2-resident.
// The same for q[B,H,T,D] and k[B,HKV,T,D] (the layout attention works in; the
// layout flag of rope_qk_inplace / gqa_rope_inplace, metal_ops.metal:7458-7465,
// 11741): only the mapping from work item to position differs.
//
// A work item is one 128-bit vector of the low half of a head together with
// the matching vector of the high half, so each item is two loads and two
// stores of activations plus one vector each of cos and sin.
//
// Arithmetic order is the reference's GQA loop (backend.py:1761-1782; backward
// 1938-1958): p = lo*c; q = hi*s; lo' = p -/+ q; q = lo*s; hi' = hi*c +/- q.
// sign = +1 is the HF convention (rope_sign=1), sign = -1 reproduces
// apply_rope_np (backend.py:1382-1399); backward flips the sign
// (apply_rope_backward_np, backend.py:1401-1417).
#include "common.hpp"
#include "launch.hpp"

namespace agrad {

namespace {

constexpr int kRopeBlock = 256;

template <typename T>
struct RopeArgs {
    T* q; T* k; const float* cos_t; const float* sin_t;
    uint32_t T_len, H, HKV, D;
    uint32_t J;      // vectors per half head  = D/2/VEC
    uint32_t Iq;     // items per token in q   = H*J
    uint32_t I;      // items per token        = (H + HKV)*J
    uint32_t total;  // B*T*I
    float sgn;       // +1 or -1 (already includes the backward flip)
    uint32_t bhtd;   // 0: [B,T,heads,D]; 1: [B,heads,T,D]
    uint32_t q_rows; // bhtd: B*H*T rows of D elements belong to q, the rest to k
    FastDiv by_J, by_I, by_T;   // exact division by J, I and T_len
};

template <int VEC>
__device__ __forceinline__ void load_table(const float* p, float (&v)[VEC]) {
    if constexpr (VEC == 1) {
        v[0] = p[0];
    } else {
#pragma unroll
        for (int j = 0; j < VEC / 4; ++j) {
            const float4 t = *reinterpret_cast<const float4*>(p + 4 * j);
            v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
        }
    }
}

template <typename T, int VEC, int UNROLL>
__global__ void __launch_bounds__(kRopeBlock) rope_kernel(const RopeArgs<T> a) {
    const uint32_t first = blockIdx.x * (kRopeBlock * UNROLL) + threadIdx.x;
    const uint32_t half = a.D / 2;
    T* ptr[UNROLL];
    float lo[UNROLL][VEC], hi[UNROLL][VEC], c[UNROLL][VEC], s[UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kRopeBlock;
        ptr[u] = nullptr;
        if (idx < a.total) {
            uint32_t t, j;
            if (a.bhtd) {                       // uniform over the launch
                uint32_t row = a.by_J.divmod(idx, j);       // a row is one (batch, head, position)
                T* base = a.q;
                if (row >= a.q_rows) { base = a.k; row -= a.q_rows; }
                a.by_T.divmod(row, t);
                ptr[u] = base + (uint64_t)row * a.D + (uint64_t)j * VEC;
            } else {
                uint32_t r;
                const uint32_t token = a.by_I.divmod(idx, r);
                a.by_T.divmod(token, t);
                T* base;
                uint32_t heads;
                if (r < a.Iq) { base = a.q; heads = a.H; } else { base = a.k; heads = a.HKV; r -= a.Iq; }
                const uint32_t head = a.by_J.divmod(r, j);
                ptr[u] = base + ((uint64_t)token * heads + head) * a.D + (uint64_t)j * VEC;
            }
            VecIO<T, VEC>::load(ptr[u], lo[u]);
            VecIO<T, VEC>::load(ptr[u] + half, hi[u]);
            const uint32_t tab = t * half + j * VEC;
            load_table<VEC>(a.cos_t + tab, c[u]);
            load_table<VEC>(a.sin_t + tab, s[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        if (ptr[u] != nullptr) {
            float nlo[VEC], nhi[VEC];
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float p = lo[u][k] * c[u][k];
                float q = hi[u][k] * s[u][k];
                p = p - a.sgn * q;       // sgn = +-1: the product is exact
                q = lo[u][k] * s[u][k];
                float h = hi[u][k] * c[u][k];
                nhi[k] = h + a.sgn * q;
                nlo[k] = p;
            }
            VecIO<T, VEC>::store(ptr[u], nlo);
            VecIO<T, VEC>::store(ptr[u] + half, nhi);
        }
    }
}

template <typename T, int VEC>
int rope_typed(hipStream_t s, RopeArgs<T> a, uint32_t B) {
    constexpr int UNROLL = 1;
    a.J = a.D / 2 / VEC;
    a.Iq = a.H * a.J;
    a.I = (a.H + (a.k ? a.HKV : 0)) * a.J;
    const uint64_t total = (uint64_t)B * a.T_len * a.I;
    if (total >= 0xffff0000ull) return set_error(AGRAD_EINVAL, "rope: %llu work items exceed 32-bit indexing", (unsigned long long)total);
    a.total = (uint32_t)total;
    a.q_rows = B * a.T_len * a.H;
    a.by_J = FastDiv(a.J);
    a.by_I = FastDiv(a.I);
    a.by_T = FastDiv(a.T_len);
    const uint32_t per_block = kRopeBlock * UNROLL;
    const uint32_t grid = (a.total + per_block - 1) / per_block;
    hipLaunchKernelGGL((rope_kernel<T, VEC, UNROLL>), dim3(grid), dim3(kRopeBlock), 0, s, a);
    return check_hip(hipGetLastError(), "rope launch");
}

template <typename T>
int rope_dispatch(hipStream_t s, void* q, void* k, const float* cos_t, const float* sin_t,
                  uint32_t B, uint32_t T_len, uint32_t H, uint32_t HKV, uint32_t D, float sgn, int bhtd) {
    constexpr int VEC = WideVec<T>::value;
    RopeArgs<T> a{};
    a.q = (T*)q; a.k = (T*)k; a.cos_t = cos_t; a.sin_t = sin_t;
    a.T_len = T_len; a.H = H; a.HKV = HKV; a.D = D; a.sgn = sgn; a.bhtd = bhtd ? 1u : 0u;
    const bool wide = (D / 2) % VEC == 0 && aligned16(q) && (!k || aligned16(k)) &&
                      aligned16(cos_t) && aligned16(sin_t);
    if (wide) return rope_typed<T, VEC>(s, a, B);
    return rope_typed<T, 1>(s, a, B);
}

}  // namespace

int launch_rope(hipStream_t s, int dtype, void* q, void* k, const float* cos_t, const float* sin_t,
                uint32_t B, uint32_t T, uint32_t H, uint32_t HKV, uint32_t D, int sign, int backward, int bhtd) {
    if (sign != 1 && sign != -1) return set_error(AGRAD_EINVAL, "rope: rope_sign must be +1 or -1, got %d", sign);
    if (D == 0 || D % 2 != 0) return set_error(AGRAD_EINVAL, "rope: head_dim %u must be even and non-zero", D);
    if (B == 0 || T == 0 || (H == 0 && (k == nullptr || HKV == 0))) return AGRAD_OK;
    if (q == nullptr || cos_t == nullptr || sin_t == nullptr) return set_error(AGRAD_EINVAL, "rope: null operand");
    if (H == 0) return set_error(AGRAD_EINVAL, "rope: q must have at least one head");
    if (k != nullptr && HKV == 0) k = nullptr;
    const float sgn = (float)(backward ? -sign : sign);
    if (dtype == AGRAD_F32) return rope_dispatch<float>(s, q, k, cos_t, sin_t, B, T, H, HKV, D, sgn, bhtd);
    if (dtype == AGRAD_BF16) return rope_dispatch<bf16_t>(s, q, k, cos_t, sin_t, B, T, H, HKV, D, sgn, bhtd);
    return set_error(AGRAD_EINVAL, "rope: unknown dtype %d", dtype);
}

}  // namespace agrad
