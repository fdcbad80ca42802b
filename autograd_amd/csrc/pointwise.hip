// The element-wise primitives of the graph IR -- Exp, Log, Rsqrt and the
// same-shape Mul (op.py:61-69, 187-204) -- as functors over the streaming
// element-wise kernel: one 16-byte vector per thread per operand.
//
//   exp     y = exp(x)                dx (+)= dy * y                       (backend.py:320-329)
//   log     y = log(x)                dx (+)= dy / x                       (backend.py:331-340)
//   rsqrt   y = 1 / sqrt(x)           dx (+)= (((dy * -0.5) * y) * y) * y  (backend.py:342-352)
//   mul     out = x * y               dx (+)= g * y,  dy (+)= g * x        (backend.py:107-146)
//
// fp32 follows the CPU's operation order (sqrt then reciprocal, both correctly
// rounded, so rsqrt and mul are bit-identical to numpy; exp and log are libm-accurate).
// bf16 storage rounds once per result.
#include "elementwise.hpp"

#include <cmath>

namespace agrad {

namespace {

struct ExpFwd {
    static __device__ __forceinline__ float apply(const float (&in)[1]) { return expf(in[0]); }
};
struct LogFwd {
    static __device__ __forceinline__ float apply(const float (&in)[1]) { return logf(in[0]); }
};
struct RsqrtFwd {
    static __device__ __forceinline__ float apply(const float (&in)[1]) { return 1.0f / sqrtf(in[0]); }
};
// in[0] = dy, in[1] = the saved tensor (y for exp and rsqrt, x for log)
struct ExpBwd {
    static __device__ __forceinline__ float apply(const float (&in)[2]) { return in[0] * in[1]; }
};
struct LogBwd {
    static __device__ __forceinline__ float apply(const float (&in)[2]) { return in[0] / in[1]; }
};
struct RsqrtBwd {
    static __device__ __forceinline__ float apply(const float (&in)[2]) {
        float t = in[0] * -0.5f;
        t = t * in[1];
        t = t * in[1];
        return t * in[1];
    }
};
struct MulFn {
    static __device__ __forceinline__ float apply(const float (&in)[2]) { return in[0] * in[1]; }
};

}  // namespace

int launch_unary_fwd(hipStream_t s, int op, int dtype, const void* x, void* y, uint64_t n) {
    const void* in[1] = {x};
    switch (op) {
        case AGRAD_UNARY_EXP: return ew_launch<1, ExpFwd>(s, dtype, in, y, n, 0, "exp forward");
        case AGRAD_UNARY_LOG: return ew_launch<1, LogFwd>(s, dtype, in, y, n, 0, "log forward");
        case AGRAD_UNARY_RSQRT: return ew_launch<1, RsqrtFwd>(s, dtype, in, y, n, 0, "rsqrt forward");
    }
    return set_error(AGRAD_EINVAL, "unary forward: unknown op %d", op);
}

int launch_unary_bwd(hipStream_t s, int op, int dtype, const void* dy, const void* saved, void* dx, uint64_t n,
                     uint32_t flags) {
    const void* in[2] = {dy, saved};
    const int acc = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    switch (op) {
        case AGRAD_UNARY_EXP: return ew_launch<2, ExpBwd>(s, dtype, in, dx, n, acc, "exp backward");
        case AGRAD_UNARY_LOG: return ew_launch<2, LogBwd>(s, dtype, in, dx, n, acc, "log backward");
        case AGRAD_UNARY_RSQRT: return ew_launch<2, RsqrtBwd>(s, dtype, in, dx, n, acc, "rsqrt backward");
    }
    return set_error(AGRAD_EINVAL, "unary backward: unknown op %d", op);
}

// out (+)= a * b, all of one shape (Mul forward, and each of its two gradients)
int launch_mul_same(hipStream_t s, int dtype, const void* a, const void* b, void* out, uint64_t n, int accumulate) {
    const void* in[2] = {a, b};
    return ew_launch<2, MulFn>(s, dtype, in, out, n, accumulate, "mul");
}

}  // namespace agrad
