// Cross-entropy over the last axis of logits[rows, V] with integer labels.
//
//   forward   loss[r] = -((x[r, label] - max_r) - log(sum_v exp(x[r, v] - max_r)))
//             (cpu_crossentropy_forward, backend.py:489-503) and, optionally,
//             lse[r] = max_r + log(sum) for the backward pass;
//   backward  dlogits[r, v] (+)= (softmax(x[r, :])[v] - [v == label]) * dloss[r]
//             (cpu_crossentropy_backward, backend.py:505-524).
//
// Both are streams over [rows, V]: forward reads the logits once (running
// maximum and rescaled sum, so no second pass), backward reads them once and
// writes the gradient once when the forward pass left lse (otherwise it first
// recomputes it with a second read of the row, which the caches serve).
// One workgroup per row; a lane keeps kCeUnroll 16-byte vectors in flight.
// Rows of odd length (V = 50257) start at any element alignment, so each row is
// split into an element-wise head up to the next 16-byte boundary, a vector
// body and an element-wise tail.
//
// exp: fp32 logits use the hardware exp2 with a compensated argument (~1.5 ulp;
// expf itself made the fp32 forward kernel instruction-bound at 0.88 of a copy);
// bf16 logits use the bare hardware exp2 (the result is rounded to 8 bits
// anyway).  loss, lse and dloss are fp32 for both.
#include "common.hpp"
#include "launch.hpp"

#include <cmath>

namespace agrad {

namespace {

constexpr int kCeBlock = 256;
constexpr int kCeUnroll = 4;      // forward (read-only): vectors a lane keeps in flight
constexpr int kCeBwdUnroll = 2;   // backward (read + write)

template <typename T> __device__ __forceinline__ float exp_io(float x) { return exp_compensated(x); }
template <> __device__ __forceinline__ float exp_io<bf16_t>(float x) { return __builtin_amdgcn_exp2f(x * kLog2eHi); }

// The softmax quotient e / sum by I/O type, from `scale = row_scale<T>(sum)`.  fp32
// tensors divide, as the CPU does.  bf16 tensors multiply by the reciprocal of the sum
// (one correctly rounded division per row): a division per element is ten instructions
// of the twenty the bf16 kernel spent per element -- it issued vector instructions for
// 78 % of its run time -- and the two differ by an ulp of fp32, gone in the rounding to
// eight bits.
template <typename T> __device__ __forceinline__ float row_scale(float sum) { return sum; }
template <> __device__ __forceinline__ float row_scale<bf16_t>(float sum) { return 1.0f / sum; }
template <typename T> __device__ __forceinline__ float quotient_io(float e, float scale) { return e / scale; }
template <> __device__ __forceinline__ float quotient_io<bf16_t>(float e, float scale) { return e * scale; }

// running (maximum, sum of exp(x - maximum))
struct MaxSum {
    float m, s;
};

template <typename T>
__device__ __forceinline__ void absorb(MaxSum& a, float x) {
    if (x > a.m) {
        a.s = a.s * exp_io<T>(a.m - x) + 1.0f;   // exp(-inf) = 0 on the first element
        a.m = x;
    } else if (a.m > -INFINITY) {                // (-inf) - (-inf) would poison the sum
        a.s = a.s + exp_io<T>(x - a.m);
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void absorb_vec(MaxSum& a, const float (&v)[VEC]) {
    float vm = v[0];
#pragma unroll
    for (int k = 1; k < VEC; ++k) vm = fmaxf(vm, v[k]);
    if (vm > a.m) {
        a.s = a.s * exp_io<T>(a.m - vm);
        a.m = vm;
    }
    if (a.m > -INFINITY) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) a.s = a.s + exp_io<T>(v[k] - a.m);
    }
}

template <typename T>
__device__ __forceinline__ MaxSum merge(const MaxSum& a, const MaxSum& b) {
    MaxSum r;
    r.m = fmaxf(a.m, b.m);
    if (r.m == -INFINITY) { r.s = 0.0f; return r; }
    r.s = a.s * exp_io<T>(a.m - r.m) + b.s * exp_io<T>(b.m - r.m);
    return r;
}

// how a row of V elements starting at `base` splits into head / vectors / tail
template <typename T, int VEC>
struct RowSplit {
    uint32_t head, nvec, tail_start;
    __device__ __forceinline__ RowSplit(const T* base, uint32_t V) {
        if constexpr (VEC == 1) {
            head = 0; nvec = V; tail_start = V;
        } else {
            const uint32_t mis = (uint32_t)(reinterpret_cast<uintptr_t>(base) & 15u) / (uint32_t)sizeof(T);
            head = mis ? (uint32_t)(16 / sizeof(T)) - mis : 0;
            if (head > V) head = V;
            nvec = (V - head) / VEC;
            tail_start = head + nvec * VEC;
        }
    }
};

// (max, sum) of one row, identical in every thread of the workgroup (BLOCK threads) on return
template <typename T, int VEC, int BLOCK = kCeBlock>
__device__ __forceinline__ MaxSum row_max_sum(const T* base, uint32_t V, MaxSum* lds) {
    const RowSplit<T, VEC> sp(base, V);
    MaxSum acc{-INFINITY, 0.0f};
    if constexpr (VEC > 1) {
        // head and tail elements, one per thread (fewer than 2 * VEC of them)
        const uint32_t extra = sp.head + (V - sp.tail_start);
        if (threadIdx.x < extra) {
            const uint32_t e = threadIdx.x < sp.head ? threadIdx.x : sp.tail_start + (threadIdx.x - sp.head);
            float x[1];
            VecIO<T, 1>::load(base + e, x);
            absorb<T>(acc, x[0]);
        }
    }
    const T* body = base + sp.head;
    for (uint32_t i0 = threadIdx.x; i0 < sp.nvec; i0 += BLOCK * kCeUnroll) {
        float v[kCeUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) VecIO<T, VEC>::load(body + (uint64_t)i * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kCeUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) absorb_vec<T, VEC>(acc, v[u]);
        }
    }
    // lanes of a wave, then the waves through LDS; the order is fixed
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        MaxSum o{__shfl_xor(acc.m, off), __shfl_xor(acc.s, off)};
        acc = merge<T>(acc, o);
    }
    const int wave = threadIdx.x / kWave;
    if (threadIdx.x % kWave == 0) lds[wave] = acc;
    __syncthreads();
    MaxSum total = lds[0];
#pragma unroll
    for (int w = 1; w < BLOCK / kWave; ++w) total = merge<T>(total, lds[w]);
    __syncthreads();
    return total;
}

template <typename T, int VEC>
__global__ void __launch_bounds__(kCeBlock)
ce_fwd_kernel(const T* __restrict__ x, const int32_t* __restrict__ labels, float* __restrict__ loss,
              float* __restrict__ lse_out, uint32_t V, int* err_flag) {
    __shared__ MaxSum lds[kCeBlock / kWave];
    const uint64_t row = blockIdx.x;
    const T* base = x + row * V;
    const MaxSum t = row_max_sum<T, VEC>(base, V, lds);
    if (threadIdx.x == 0) {
        const float lg = logf(t.s);
        if (lse_out != nullptr) lse_out[row] = t.m + lg;
        const int32_t label = labels[row];
        if (label < 0 || (uint32_t)label >= V) {
            *err_flag = 1;
            loss[row] = 0.0f;
        } else {
            float xl[1];
            VecIO<T, 1>::load(base + label, xl);
            float f = xl[0] - t.m;
            f = f - lg;
            loss[row] = -f;
        }
    }
}

template <typename T, int VEC>
__device__ __forceinline__ void ce_grad_elems(const float (&xv)[VEC], float (&d)[VEC], float lse, float gl,
                                              uint32_t first_elem, uint32_t label) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        float p = exp_io<T>(xv[k] - lse);
        if (first_elem + k == label) p = p - 1.0f;
        d[k] = p * gl;
    }
}

template <typename T, int VEC>
__global__ void __launch_bounds__(kCeBlock)
ce_bwd_kernel(const T* __restrict__ x, const int32_t* __restrict__ labels, const float* __restrict__ dloss,
              const float* __restrict__ lse_in, T* dx, uint32_t V, int accumulate, int* err_flag) {
    __shared__ MaxSum lds[kCeBlock / kWave];
    const uint64_t row = blockIdx.x;
    const T* base = x + row * V;
    T* out = dx + row * V;
    float lse;
    if (lse_in != nullptr) {
        lse = lse_in[row];
    } else {
        const MaxSum t = row_max_sum<T, VEC>(base, V, lds);
        lse = t.m + logf(t.s);
    }
    const float gl = dloss[row];
    const int32_t lab = labels[row];
    uint32_t label = 0xffffffffu;          // matches no element: the row gets softmax * dloss
    if (lab < 0 || (uint32_t)lab >= V) {
        if (threadIdx.x == 0) *err_flag = 1;
    } else {
        label = (uint32_t)lab;
    }
    const RowSplit<T, VEC> sp(base, V);
    if constexpr (VEC > 1) {
        const uint32_t extra = sp.head + (V - sp.tail_start);
        if (threadIdx.x < extra) {
            const uint32_t e = threadIdx.x < sp.head ? threadIdx.x : sp.tail_start + (threadIdx.x - sp.head);
            float xv[1], d[1];
            VecIO<T, 1>::load(base + e, xv);
            ce_grad_elems<T, 1>(xv, d, lse, gl, e, label);
            if (accumulate) {
                float old[1];
                VecIO<T, 1>::load(out + e, old);
                d[0] = old[0] + d[0];
            }
            VecIO<T, 1>::store(out + e, d);
        }
    }
    const T* body = base + sp.head;
    T* obody = out + sp.head;
    for (uint32_t i0 = threadIdx.x; i0 < sp.nvec; i0 += kCeBlock * kCeBwdUnroll) {
        float v[kCeBwdUnroll][VEC], old[kCeBwdUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * kCeBlock;
            if (i < sp.nvec) {
                VecIO<T, VEC>::load(body + (uint64_t)i * VEC, v[u]);
                if (accumulate) VecIO<T, VEC>::load(obody + (uint64_t)i * VEC, old[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * kCeBlock;
            if (i < sp.nvec) {
                float d[VEC];
                ce_grad_elems<T, VEC>(v[u], d, lse, gl, sp.head + i * VEC, label);
                if (accumulate) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) d[k] = old[u][k] + d[k];
                }
                VecIO<T, VEC>::store(obody + (uint64_t)i * VEC, d);
            }
        }
    }
}

// The same gradient with the row's log-sum-exp given, as a one-shot grid over
// the flat [rows * V] array: a workgroup is one wave and takes 64 consecutive
// 16-byte vectors, one per lane, wherever row boundaries fall (a vector may
// straddle two rows; V >= 64 vectors, so a wave meets at most one boundary).
// Every access is 16-byte aligned whatever V is (50257 included), consecutive
// workgroups touch consecutive kilobytes, and no workgroup loops: measured on
// MI355X this streams 20-25% faster than a workgroup walking along its row.
constexpr int kCeFlatBlock = 64;

template <typename T, int VEC>
__global__ void __launch_bounds__(kCeFlatBlock)
ce_bwd_flat_kernel(const T* __restrict__ x, const int32_t* __restrict__ labels, const float* __restrict__ dloss,
                   const float* __restrict__ lse_in, T* dx, uint32_t V, uint32_t rows, uint32_t total,
                   int accumulate, int* err_flag) {
    // element indices fit 32 bits: the launcher cuts the tensor into slabs of rows
    const uint32_t e_wave = blockIdx.x * (uint32_t)(kCeFlatBlock * VEC);   // first element of this wave
    const uint32_t row0 = e_wave / V;
    const uint32_t rel0 = e_wave - row0 * V;
    const uint32_t e0 = e_wave + threadIdx.x * VEC;
    if (e0 >= total) return;
    const uint32_t rel = rel0 + threadIdx.x * VEC;
    const float lse_a = lse_in[row0];
    const float gl_a = dloss[row0];
    const int32_t lab_a = labels[row0];
    if (rel0 == 0 && threadIdx.x == 0 && (lab_a < 0 || (uint32_t)lab_a >= V)) *err_flag = 1;
    const bool whole = e_wave + kCeFlatBlock * VEC <= total;              // uniform: no partial vector here
    if (whole && rel0 + kCeFlatBlock * VEC <= V) {
        // the common case: the whole wave lies inside one row
        float v[VEC], old[VEC], d[VEC];
        VecIO<T, VEC>::load(x + e0, v);
        if (accumulate) VecIO<T, VEC>::load(dx + e0, old);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            float p = exp_io<T>(v[k] - lse_a);
            if (rel + k == (uint32_t)lab_a) p = p - 1.0f;
            d[k] = p * gl_a;
            if (accumulate) d[k] = old[k] + d[k];
        }
        VecIO<T, VEC>::store(dx + e0, d);
        return;
    }
    // a row boundary (or the end of the tensor) falls inside this wave
    const uint32_t row1 = row0 + 1 < rows ? row0 + 1 : row0;
    const float lse_b = lse_in[row1];
    const float gl_b = dloss[row1];
    const int32_t lab_b = labels[row1];
    for (uint32_t k = 0; k < (uint32_t)VEC && e0 + k < total; ++k) {
        uint32_t r = rel + k;
        const bool next = r >= V;
        if (next) r -= V;
        const int32_t lab = next ? lab_b : lab_a;
        if (next && r == 0 && (lab < 0 || (uint32_t)lab >= V)) *err_flag = 1;
        float xv[1], d[1];
        VecIO<T, 1>::load(x + e0 + k, xv);
        float p = exp_io<T>(xv[0] - (next ? lse_b : lse_a));
        if (r == (uint32_t)lab) p = p - 1.0f;
        d[0] = p * (next ? gl_b : gl_a);
        if (accumulate) {
            float o1[1];
            VecIO<T, 1>::load(dx + e0 + k, o1);
            d[0] = o1[0] + d[0];
        }
        VecIO<T, 1>::store(dx + e0 + k, d);
    }
}

template <typename T>
int ce_typed(hipStream_t s, bool backward, const T* x, const int32_t* labels, float* loss, float* lse_out,
             const float* dloss, const float* lse_in, T* dx, uint64_t rows, uint32_t V, int acc, int* err_flag) {
    constexpr int WIDE = WideVec<T>::value;
    // the element-wise head realigns every row, which needs the two tensors to
    // share their alignment and the element size to divide 16
    const bool wide = V >= 4 * WIDE && aligned16(x) && (!backward || aligned16(dx));
    const dim3 grid((uint32_t)rows), block(kCeBlock);
    if (!backward) {
        if (wide) hipLaunchKernelGGL((ce_fwd_kernel<T, WIDE>), grid, block, 0, s, x, labels, loss, lse_out, V, err_flag);
        else hipLaunchKernelGGL((ce_fwd_kernel<T, 1>), grid, block, 0, s, x, labels, loss, lse_out, V, err_flag);
    } else if (lse_in != nullptr && aligned16(x) && aligned16(dx) && V >= (uint32_t)(kCeFlatBlock * WIDE)) {
        // slabs of rows keep element indices within 32 bits; a multiple of 16
        // rows keeps every slab 16-byte aligned
        const uint32_t per_wave = (uint32_t)kCeFlatBlock * WIDE;
        uint64_t max_rows = 0xfff00000ull / V;
        max_rows = max_rows >= 16 ? max_rows / 16 * 16 : 1;
        if (max_rows == 1 && rows > 1 && (V * sizeof(T)) % 16 != 0)
            return set_error(AGRAD_EINVAL, "cross-entropy backward: class axis of %u is too long", V);
        for (uint64_t r0 = 0; r0 < rows; r0 += max_rows) {
            const uint64_t nr = rows - r0 < max_rows ? rows - r0 : max_rows;
            const uint32_t total = (uint32_t)(nr * V);
            const uint32_t waves = (total + per_wave - 1) / per_wave;
            hipLaunchKernelGGL((ce_bwd_flat_kernel<T, WIDE>), dim3(waves), dim3(kCeFlatBlock), 0, s,
                               x + r0 * V, labels + r0, dloss + r0, lse_in + r0, dx + r0 * V, V, (uint32_t)nr, total,
                               acc, err_flag);
        }
    } else {
        if (wide) hipLaunchKernelGGL((ce_bwd_kernel<T, WIDE>), grid, block, 0, s, x, labels, dloss, lse_in, dx, V, acc, err_flag);
        else hipLaunchKernelGGL((ce_bwd_kernel<T, 1>), grid, block, 0, s, x, labels, dloss, lse_in, dx, V, acc, err_flag);
    }
    return check_hip(hipGetLastError(), "cross-entropy launch");
}

// ---------------------------------------------------------------------------
// Loss and gradient in ONE launch, in place: the row of logits becomes the row of
// (softmax - onehot) * scale, and row_loss / lse are written on the way -- the form the
// reference uses behind its output projection (fused_linear_ce_logits_to_dlogits and its
// per-row-scaled variant, metal_ops.metal:8808-9152; the chunk's rows are numbered from
// row_base in targets / row_loss / lse / row_scale).  A target outside [0, V) -- an ignored
// position -- or a row with no finite logit gives loss 0, lse 0 and a zero row, as there.
//
// The separate forward and backward kernels above move 3 * V * e bytes per row (the
// logits read twice).  Here a workgroup holds its row IN REGISTERS between the statistics
// and the rewrite -- the sixteen waves a CU gives 128 registers each are a third of a
// megabyte -- so a row is read from memory once and written once: 2 * V * e bytes.  All of a
// thread's loads are issued before the first wait (a thread past the end of the row loads
// the row's first vector and ignores it: no load sits behind a branch).  fp32 rows keep
// exp(x - max) in the registers the logits came in and the rewrite is a multiplication;
// bf16 rows stay packed (half the registers) and take the hardware exp2 a second time.
// Rows too long for the registers (fp32 beyond 81920 classes) take ce_fused_mem_kernel: the
// same arithmetic with the second pass reading memory again.
constexpr int kCeRowBlock = 1024;

template <int BLOCK> __device__ __forceinline__ float block_sum(float v, float* lds);

template <int BLOCK>
__device__ __forceinline__ float block_max(float v, float* lds) {
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) v = fmaxf(v, __shfl_xor(v, off));
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = v;
    __syncthreads();
    float t = lds[0];
#pragma unroll
    for (int w = 1; w < BLOCK / kWave; ++w) t = fmaxf(t, lds[w]);
    __syncthreads();
    return t;
}

// Tells the compiler that a packed vector may have changed: what it unpacked from it before is
// unpacked again where it is next needed, instead of being kept in twice the registers.
__device__ __forceinline__ void forget_unpacked(u32x4& r) {
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
}
__device__ __forceinline__ void forget_unpacked(f32x4&) {}

struct CeFusedArgs {
    const int32_t* targets; float* row_loss; float* lse; const float* row_scale;
    uint32_t V, row_base; float scale; uint32_t write_grad;
};

// exp(x - shift) in the fused kernels.  bf16 rows fold the subtraction into the argument of
// the hardware exp2 (one fma: `bias` = -shift * log2 e); the kernel that holds a long bf16 row
// issues vector instructions for most of its run time, and this is one of its ten an element.
template <typename T> __device__ __forceinline__ float exp_shifted(float x, float shift, float) { return exp_io<T>(x - shift); }
template <> __device__ __forceinline__ float exp_shifted<bf16_t>(float x, float, float bias) {
    return __builtin_amdgcn_exp2f(__builtin_fmaf(x, kLog2eHi, bias));
}

// One vector of the rewrite: v[k] = (e[k] * inv - [first + k == hit]) * mul.  The target is
// looked for once a vector, not once an element (a compare, a select and an add of the
// five instructions an element otherwise costs here).
template <int VEC>
__device__ __forceinline__ void ce_rewrite(float (&v)[VEC], float inv, float mul, uint32_t first, uint32_t hit) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) v[k] = v[k] * inv;
    if (hit - first < (uint32_t)VEC) {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
            if (first + k == hit) v[k] = v[k] - 1.0f;
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) v[k] = v[k] * mul;
}

// A vector of the gradient to memory.  bf16: the hardware's pair conversion alone -- a NaN
// comes out as the hardware's quiet NaN instead of with the payload bits the integer rule
// keeps; a softmax that meets a NaN is NaN throughout, and the two compares a pair cost are
// a tenth of this kernel's instructions.
template <typename T, int VEC>
__device__ __forceinline__ void ce_store_grad(T* p, const float (&v)[VEC]) { VecIO<T, VEC>::store(p, v); }
template <>
__device__ __forceinline__ void ce_store_grad<bf16_t, 8>(bf16_t* p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const f32x2_hw pair = {v[2 * i], v[2 * i + 1]};
        w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_hw));
    }
    u32x4 t; t.x = w[0]; t.y = w[1]; t.z = w[2]; t.w = w[3];
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}

// what thread 0 leaves for the row
__device__ __forceinline__ void ce_fused_row_results(const CeFusedArgs& a, uint32_t grow, bool valid, float lse,
                                                     float target_logit) {
    if (threadIdx.x == 0) {
        if (a.row_loss != nullptr) a.row_loss[grow] = valid ? lse - target_logit : 0.0f;
        if (a.lse != nullptr) a.lse[grow] = valid ? lse : 0.0f;
    }
}

// (Sixteen vectors a thread compile to 86 registers, which is five waves a SIMD and two
// 512-thread workgroups a CU; held to six waves -- 80 registers, 22 of them spilled -- three
// workgroups share a CU and 16384 rows of 32768 fp32 classes take 780 us instead of 810: a
// third workgroup in another phase is worth more than the spills cost.)
template <typename T, int VEC, int NV, int BLOCK>
__global__ void __launch_bounds__(BLOCK, (BLOCK == 512 && NV == 16) ? 6 : 1)
ce_fused_reg_kernel(T* x, const CeFusedArgs a) {
    __shared__ float lds[BLOCK / kWave];
    typedef RawVec<T, VEC> Raw;
    const uint32_t V = a.V;
    // (the thread's number is read anew before the last pass over the registers: what the
    // compiler would otherwise derive from it once and keep -- an index and an address per
    // vector -- costs the longest rows their last registers)
    uint32_t tid = threadIdx.x;
    T* base = x + (uint64_t)blockIdx.x * V;
    const uint32_t grow = a.row_base + blockIdx.x;
    const RowSplit<T, VEC> sp(base, V);
    T* body = base + sp.head;
    // every load of the row, then the few elements before and after the aligned body, then the target's logit
    typename Raw::type raw[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = (uint32_t)i * BLOCK + tid;
        raw[i] = Raw::load(body + (uint64_t)(idx < sp.nvec ? idx : 0u) * VEC);
    }
    const uint32_t extra = sp.head + (V - sp.tail_start);         // fewer than 2 * VEC elements
    const uint32_t e_at = tid < sp.head ? tid : sp.tail_start + (tid - sp.head);
    float xe = -INFINITY;
    {
        float t1[1];
        VecIO<T, 1>::load(base + (tid < extra ? e_at : 0u), t1);
        if (tid < extra) xe = t1[0];
    }
    const int32_t target = a.targets[grow];
    const bool in_range = target >= 0 && (uint32_t)target < V;
    float target_logit;
    {
        float t1[1];
        VecIO<T, 1>::load(base + (in_range ? (uint32_t)target : 0u), t1);
        target_logit = t1[0];
    }

    float m = xe;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = (uint32_t)i * BLOCK + tid;
        float v[VEC];
        Raw::unpack(raw[i], v);
        if (idx < sp.nvec) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) m = fmaxf(m, v[k]);
        }
    }
    m = block_max<BLOCK>(m, lds);
#pragma unroll
    for (int i = 0; i < NV; ++i) forget_unpacked(raw[i]);
    const bool finite = m > -INFINITY;          // (uniform) a row of -inf has no softmax
    const float shift = finite ? m : 0.0f;
    const float bias = -shift * kLog2eHi;

    float sum = tid < extra ? exp_io<T>(xe - shift) : 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = (uint32_t)i * BLOCK + tid;
        float v[VEC];
        Raw::unpack(raw[i], v);
        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            v[k] = exp_shifted<T>(v[k], shift, bias);
            part = part + v[k];
        }
        if (idx < sp.nvec) sum = sum + part;
        if constexpr (sizeof(T) == 4) raw[i] = typename Raw::type{v[0], v[1], v[2], v[3]};      // keeps exp(x - max)
    }
    sum = block_sum<BLOCK>(sum, lds);
#pragma unroll
    for (int i = 0; i < NV; ++i) forget_unpacked(raw[i]);

    const bool valid = in_range && finite && sum > 0.0f;
    const float lse = shift + logf(sum);
    ce_fused_row_results(a, grow, valid, lse, target_logit);
    if ((a.write_grad & 1u) == 0u) return;

    asm volatile("" : "+v"(tid));
    const float scale = a.row_scale != nullptr ? a.row_scale[grow] : a.scale;
    const float inv = valid ? 1.0f / sum : 0.0f;
    const float mul = valid ? scale : 0.0f;
    const float both = inv * mul;
    const uint32_t hit = valid ? (uint32_t)target : 0xffffffffu;          // matches no element when the row is ignored
    if (tid < extra) {
        float d[1];
        d[0] = exp_io<T>(xe - shift) * inv;
        if (e_at == hit) d[0] = d[0] - 1.0f;
        d[0] = d[0] * mul;
        VecIO<T, 1>::store(base + e_at, d);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = (uint32_t)i * BLOCK + tid;
        float v[VEC];
        Raw::unpack(raw[i], v);
        const uint32_t first = sp.head + idx * VEC;
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float p = v[k] * inv;
                if (first + k == hit) p = p - 1.0f;
                v[k] = p * mul;
            }
        } else {
            // bf16 rows: nothing per element but the exponential and one product (the kernel
            // issues vector instructions for most of its run time); the target's element is
            // put right below, by the thread that stores its vector
#pragma unroll
            for (int k = 0; k < VEC; ++k) v[k] = exp_shifted<T>(v[k], shift, bias) * both;
        }
        if (idx < sp.nvec) ce_store_grad<T, VEC>(body + (uint64_t)idx * VEC, v);
    }
    if constexpr (sizeof(T) != 4) {
        // (a later store of the same thread to the same place: in order)
        const uint32_t hv = (hit - sp.head) / VEC;
        if (hit >= sp.head && hit < sp.tail_start && tid == hv % BLOCK) {
            float d[1];
            d[0] = (exp_io<T>(target_logit - shift) * inv - 1.0f) * mul;
            VecIO<T, 1>::store(base + hit, d);
        }
    }
}

// the same for rows of any length and alignment: statistics from one pass over memory, the
// rewrite from a second (VEC == 1: element by element)
template <typename T, int VEC>
__global__ void __launch_bounds__(kCeRowBlock)
ce_fused_mem_kernel(T* x, const CeFusedArgs a) {
    __shared__ MaxSum lds[kCeRowBlock / kWave];
    const uint32_t V = a.V, tid = threadIdx.x;
    T* base = x + (uint64_t)blockIdx.x * V;
    const uint32_t grow = a.row_base + blockIdx.x;
    const int32_t target = a.targets[grow];
    const bool in_range = target >= 0 && (uint32_t)target < V;
    float target_logit;
    {
        float t1[1];
        VecIO<T, 1>::load(base + (in_range ? (uint32_t)target : 0u), t1);
        target_logit = t1[0];
    }
    const MaxSum t = row_max_sum<T, VEC, kCeRowBlock>(base, V, lds);      // (ends with a barrier: the target's logit is in)
    const bool valid = in_range && t.m > -INFINITY && t.s > 0.0f;
    const float lse = t.m + logf(t.s);
    ce_fused_row_results(a, grow, valid, lse, target_logit);
    if ((a.write_grad & 1u) == 0u) return;

    const float scale = a.row_scale != nullptr ? a.row_scale[grow] : a.scale;
    const float inv = valid ? 1.0f / t.s : 0.0f;
    const float mul = valid ? scale : 0.0f;
    const float shift = valid ? t.m : 0.0f;
    const uint32_t hit = valid ? (uint32_t)target : 0xffffffffu;
    const RowSplit<T, VEC> sp(base, V);
    if constexpr (VEC > 1) {
        const uint32_t extra = sp.head + (V - sp.tail_start);
        if (tid < extra) {
            const uint32_t e = tid < sp.head ? tid : sp.tail_start + (tid - sp.head);
            float d[1];
            VecIO<T, 1>::load(base + e, d);
            d[0] = exp_io<T>(d[0] - shift) * inv;
            if (e == hit) d[0] = d[0] - 1.0f;
            d[0] = d[0] * mul;
            VecIO<T, 1>::store(base + e, d);
        }
    }
    T* body = base + sp.head;
    for (uint32_t i0 = tid; i0 < sp.nvec; i0 += kCeRowBlock * kCeBwdUnroll) {
        float v[kCeBwdUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * kCeRowBlock;
            VecIO<T, VEC>::load(body + (uint64_t)(i < sp.nvec ? i : 0u) * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * kCeRowBlock;
            const uint32_t first = sp.head + i * VEC;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float p = exp_io<T>(v[u][k] - shift) * inv;
                if (first + k == hit) p = p - 1.0f;
                v[u][k] = p * mul;
            }
            if (i < sp.nvec) VecIO<T, VEC>::store(body + (uint64_t)i * VEC, v[u]);
        }
    }
}

// ---------------------------------------------------------------------------
// The same, with a row shared by a TEAM of workgroups.  A row that one workgroup holds in
// registers makes that workgroup read, compute and write in turn, and at most two such
// workgroups fit a CU: measured, the pattern alone (load all, barrier, store all) moves
// 0.88 of what a streaming copy moves, and rows beyond 80 K classes do not fit at all.  Here
// G workgroups of 256 threads take a slice of the row each -- a few vectors a thread, so
// many workgroups share a CU and their phases interleave like a stream's -- and exchange
// one (max, sum) pair per slice through memory:
//   slice:  m_j = max x,  s_j = sum exp(x - m_j)        (the slice stays in registers)
//   post:   two 64-bit device-scope stores, {m_j, tag} and {s_j, tag}: each word says by
//           its tag which row of the launch it belongs to, so no store has to wait for
//           another and no counter is needed
//   next:   the loads of the team's next row, into a second set of registers
//   wait:   lane j of the first wave polls member j's two words (device-scope loads)
//           until both carry this row's tag; the other waves sit at the workgroup barrier
//   row:    M = max m_j,  S = sum_j s_j exp(m_j - M), j ascending: the same in every
//           member, which then rewrites its slice as (exp(x - M) / S - onehot) * scale
// The grid is what is resident at once (the occupancy the runtime reports, times the
// CUs), teams are neighbours in it, and a team walks rows team, team + teams, ...: every
// member of a team is on the GPU while the others wait for it.  The wait is bounded all
// the same: a member that is not joined within its budget of polls (kTeamSpinBudget unless the host says otherwise) sets the second
// error word, stops waiting for the rest of the launch and finishes (with wrong numbers;
// the pass boundary reports the error) -- no wave waits for ever.
// Tags are the team's row count + 1; a fill in front of the launch clears the words.  The
// words alternate between two sets by the parity of the row count, so a fast member's next
// post cannot land on a pair that a slow one has yet to read (it posts row r + 2 only after
// everyone has posted r + 1, which each does after reading the pairs of r).
// ---------------------------------------------------------------------------
constexpr int kTeamBlock = 256;
constexpr uint32_t kTeamMaxMembers = 32, kTeamMaxTeams = 2048;
constexpr uint32_t kTeamSpinBudget = 1u << 20;         // polls of ~1 us
constexpr uint64_t kTeamWordsPerTeam = 2ull * kTeamMaxMembers * 2;      // two sets of {m, tag}, {s, tag} per member
constexpr uint64_t kTeamScratchBytes = (uint64_t)kTeamMaxTeams * kTeamWordsPerTeam * 8;

// what a row needs besides its vectors: the element before / after the aligned part that
// this thread owns (member 0), the target and the target's logit
struct CeRowExtras {
    float xe, target_logit;
    int32_t target;
};

template <typename T, int VEC, int NV>
__global__ void __launch_bounds__(kTeamBlock)
ce_fused_team_kernel(T* x, const CeFusedArgs a, uint32_t rows, uint32_t G, uint32_t teams,
                     unsigned long long* words, int* err_words, uint32_t spin_budget) {
    constexpr int BLOCK = kTeamBlock;
    __shared__ float lds[BLOCK / kWave];
    __shared__ float team_m[kTeamMaxMembers], team_s[kTeamMaxMembers];
    __shared__ uint32_t alone;                  // this workgroup has stopped waiting for its team
    typedef RawVec<T, VEC> Raw;
    const uint32_t V = a.V, tid = threadIdx.x;
    const uint32_t team = blockIdx.x / G, member = blockIdx.x - team * G;
    unsigned long long* slots = words + (uint64_t)team * kTeamWordsPerTeam;
    if (tid == 0) alone = 0;
    __syncthreads();

    // the slice of `member` in a row, and the requests for it
    struct Slice { T* base; T* body; uint32_t head, tail_start, lo, hi; };
    auto slice_of = [&](uint32_t row) {
        Slice c;
        c.base = x + (uint64_t)row * V;
        const RowSplit<T, VEC> sp(c.base, V);
        c.body = c.base + sp.head;
        c.head = sp.head;
        c.tail_start = sp.tail_start;
        const uint32_t per = (sp.nvec + G - 1) / G;                     // vectors of a slice (at most NV * BLOCK)
        c.lo = member * per < sp.nvec ? member * per : sp.nvec;
        c.hi = c.lo + per < sp.nvec ? c.lo + per : sp.nvec;
        return c;
    };
    auto ask = [&](const Slice& c, uint32_t grow, typename Raw::type (&raw)[NV], CeRowExtras& ex) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint32_t idx = c.lo + (uint32_t)i * BLOCK + tid;
            raw[i] = Raw::load(c.body + (uint64_t)(idx < c.hi ? idx : 0u) * VEC);   // (past the slice: the row's first vector)
        }
        const uint32_t extra = member == 0 ? c.head + (V - c.tail_start) : 0u;
        const uint32_t e_at = tid < c.head ? tid : c.tail_start + (tid - c.head);
        float t1[1];
        VecIO<T, 1>::load(c.base + (tid < extra ? e_at : 0u), t1);
        ex.xe = t1[0];
        ex.target = a.targets[grow];
        VecIO<T, 1>::load(c.base + (ex.target >= 0 && (uint32_t)ex.target < V ? (uint32_t)ex.target : 0u), t1);
        ex.target_logit = t1[0];
    };

    typename Raw::type raw[NV], ahead[NV];
    CeRowExtras ex, ex_ahead;
    uint32_t row = team;
    if (row >= rows) return;
    Slice c = slice_of(row);
    ask(c, a.row_base + row, raw, ex);
    for (uint32_t it = 0;; ++it) {
        const uint32_t grow = a.row_base + row;
        const uint32_t next = row + teams;
        const bool more = next < rows;                                  // (uniform)
        const uint32_t extra = member == 0 ? c.head + (V - c.tail_start) : 0u;
        const uint32_t e_at = tid < c.head ? tid : c.tail_start + (tid - c.head);
        const float xe = tid < extra ? ex.xe : -INFINITY;
        const int32_t target = ex.target;
        const bool in_range = target >= 0 && (uint32_t)target < V;
        const float target_logit = ex.target_logit;

        float m = xe;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint32_t idx = c.lo + (uint32_t)i * BLOCK + tid;
            float v[VEC];
            Raw::unpack(raw[i], v);
#pragma unroll
            for (int k = 0; k < VEC; ++k) m = fmaxf(m, idx < c.hi ? v[k] : -INFINITY);
        }
        m = block_max<BLOCK>(m, lds);
#pragma unroll
        for (int i = 0; i < NV; ++i) forget_unpacked(raw[i]);
        const float own_shift = m > -INFINITY ? m : 0.0f;
        const float own_bias = -own_shift * kLog2eHi;
        float sum = tid < extra ? exp_io<T>(xe - own_shift) : 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint32_t idx = c.lo + (uint32_t)i * BLOCK + tid;
            float v[VEC];
            Raw::unpack(raw[i], v);
            float part = 0.0f;
#pragma unroll
            for (int k = 0; k < VEC; ++k) part = part + exp_shifted<T>(v[k], own_shift, own_bias);
            sum = sum + (idx < c.hi ? part : 0.0f);
        }
        sum = block_sum<BLOCK>(sum, lds);
#pragma unroll
        for (int i = 0; i < NV; ++i) forget_unpacked(raw[i]);

        // post this slice's pair
        const uint32_t tag = it + 1u;
        unsigned long long* now = slots + (uint64_t)(it & 1u) * kTeamMaxMembers * 2;
        if (tid == 0) {
            const unsigned long long up = (unsigned long long)tag << 32;
            __hip_atomic_store(now + member * 2, up | __float_as_uint(m), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(now + member * 2 + 1, up | __float_as_uint(sum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // the next row is on its way while the team assembles
        const Slice c_next = slice_of(more ? next : row);
        if (more) ask(c_next, a.row_base + next, ahead, ex_ahead);
        // wait for the team's pairs
        if (tid < G) {
            unsigned long long w0 = 0, w1 = 0;
            uint32_t budget = alone == 0 ? spin_budget : 1u;
            for (;;) {
                w0 = __hip_atomic_load(now + tid * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                w1 = __hip_atomic_load(now + tid * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((uint32_t)(w0 >> 32) == tag && (uint32_t)(w1 >> 32) == tag) break;
                if (--budget == 0) {
                    alone = 1;
                    err_words[1] = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            team_m[tid] = __uint_as_float((uint32_t)w0);
            team_s[tid] = __uint_as_float((uint32_t)w1);
        }
        __syncthreads();
        float M = -INFINITY;
        for (uint32_t j = 0; j < G; ++j) M = fmaxf(M, team_m[j]);
        const bool finite = M > -INFINITY;          // (uniform) a row of -inf has no softmax
        const float shift = finite ? M : 0.0f;
        const float bias = -shift * kLog2eHi;
        float total = 0.0f;
        for (uint32_t j = 0; j < G; ++j)
            if (team_m[j] > -INFINITY) total = total + team_s[j] * exp_io<T>(team_m[j] - shift);

        const bool valid = in_range && finite && total > 0.0f;
        const float lse = shift + logf(total);
        if (member == 0) ce_fused_row_results(a, grow, valid, lse, target_logit);
        if ((a.write_grad & 1u) != 0u) {
            const float scale = a.row_scale != nullptr ? a.row_scale[grow] : a.scale;
            const float inv = valid ? 1.0f / total : 0.0f;
            const float mul = valid ? scale : 0.0f;
            const uint32_t hit = valid ? (uint32_t)target : 0xffffffffu;      // matches no element when the row is ignored
            if (tid < extra) {
                float d[1];
                d[0] = exp_io<T>(xe - shift) * inv;
                if (e_at == hit) d[0] = d[0] - 1.0f;
                d[0] = d[0] * mul;
                VecIO<T, 1>::store(c.base + e_at, d);
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const uint32_t idx = c.lo + (uint32_t)i * BLOCK + tid;
                float v[VEC];
                Raw::unpack(raw[i], v);
                const uint32_t first = c.head + idx * VEC;
#pragma unroll
                for (int k = 0; k < VEC; ++k) v[k] = exp_shifted<T>(v[k], shift, bias);
                ce_rewrite<VEC>(v, inv, mul, first, hit);
                if (idx < c.hi) VecIO<T, VEC>::store(c.body + (uint64_t)idx * VEC, v);
            }
        }
        if (!more) break;
        __syncthreads();                             // (team_m / team_s are written again)
#pragma unroll
        for (int i = 0; i < NV; ++i) raw[i] = ahead[i];
        ex = ex_ahead;
        row = next;
        c = c_next;
    }
}

// Geometry of the register-resident kernel.  Two workgroups of 512 threads share a CU when a
// thread's share of the row leaves the kernel within 128 registers (kCeHalfMaxNV vectors: fp32
// rows up to 40960 classes, bf16 up to 81920): one workgroup's exponentials and stores then
// overlap the other's loads, which a lone workgroup per CU cannot do -- it reads, computes and
// writes in turn.  Longer rows take one workgroup of 1024 threads per CU (up to kCeFullMaxNV
// vectors a thread), and beyond that the two-pass kernel.
constexpr int kCeHalfBlock = 512, kCeHalfMaxNV = 20, kCeFullMaxNV = 20;

// workgroups of a kernel that share a CU, times the CUs: what is on the GPU at once
uint32_t resident_workgroups(const void* kernel, int block) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block, 0) != hipSuccess || cus < 1 || per_cu < 1) {
        (void)hipGetLastError();
        return 0;
    }
    return (uint32_t)cus * (uint32_t)per_cu;
}

// the team kernel for a row of `vectors` aligned vectors at most; false if no geometry fits
template <typename T, int NV>
bool ce_fused_team_launch(hipStream_t s, T* x, const CeFusedArgs& a, uint64_t rows, uint32_t vectors, void* scratch,
                          int* err_words, uint32_t polls, int* rc) {
    constexpr int WIDE = WideVec<T>::value;
    const uint32_t G = (vectors + NV * kTeamBlock - 1) / (NV * kTeamBlock);
    if (G < 2 || G > kTeamMaxMembers) return false;
    static const uint32_t resident = resident_workgroups((const void*)ce_fused_team_kernel<T, WIDE, NV>, kTeamBlock);
    uint32_t teams = resident / G;
    if (teams > kTeamMaxTeams) teams = kTeamMaxTeams;
    if (teams > rows) teams = (uint32_t)rows;
    if (teams == 0) return false;                  // (a team would not be on the GPU all at once)
    unsigned long long* words = reinterpret_cast<unsigned long long*>(scratch);
    *rc = launch_fill(s, words, 0u, 4, (uint64_t)teams * kTeamWordsPerTeam * 2);
    if (*rc != AGRAD_OK) return true;
    hipLaunchKernelGGL((ce_fused_team_kernel<T, WIDE, NV>), dim3(teams * G), dim3(kTeamBlock), 0, s, x, a, (uint32_t)rows, G,
                       teams, words, err_words, polls ? polls : kTeamSpinBudget);
    *rc = check_hip(hipGetLastError(), "fused cross-entropy launch");
    return true;
}

template <typename T>
int ce_fused_typed(hipStream_t s, T* x, const CeFusedArgs& a, uint64_t rows, void* team_scratch, int* err_words,
                   uint32_t team_polls) {
    constexpr int WIDE = WideVec<T>::value;
    const dim3 grid((uint32_t)rows);
    // the element-wise head realigns every row to 16 bytes, which needs the element size to divide the misalignment
    const bool wide = a.V >= 4 * WIDE && (reinterpret_cast<uintptr_t>(x) % sizeof(T)) == 0;
    if (!wide) {
        hipLaunchKernelGGL((ce_fused_mem_kernel<T, 1>), grid, dim3(kCeRowBlock), 0, s, x, a);
        return check_hip(hipGetLastError(), "fused cross-entropy launch");
    }
    const uint32_t vectors = a.V / WIDE;                          // aligned vectors of a row, at most
#define AGRAD_CE_REG(N, BLOCK) \
    if (vectors <= (uint32_t)(N) * BLOCK) { hipLaunchKernelGGL((ce_fused_reg_kernel<T, WIDE, N, BLOCK>), grid, dim3(BLOCK), 0, s, x, a); return check_hip(hipGetLastError(), "fused cross-entropy launch"); }
    AGRAD_CE_REG(4, kCeHalfBlock) AGRAD_CE_REG(8, kCeHalfBlock) AGRAD_CE_REG(12, kCeHalfBlock) AGRAD_CE_REG(16, kCeHalfBlock)
    AGRAD_CE_REG(20, kCeHalfBlock)
    AGRAD_CE_REG(12, kCeRowBlock) AGRAD_CE_REG(16, kCeRowBlock) AGRAD_CE_REG(20, kCeRowBlock)
#undef AGRAD_CE_REG
    static_assert(kCeHalfMaxNV == 20 && kCeFullMaxNV == 20, "the instantiations above");
    if (team_scratch != nullptr && err_words != nullptr) {
        // a row that no workgroup can hold: a team of workgroups holds it, a slice each
        int rc = AGRAD_OK;
        if (ce_fused_team_launch<T, 4>(s, x, a, rows, vectors, team_scratch, err_words, team_polls, &rc)) return rc;
        if (ce_fused_team_launch<T, 8>(s, x, a, rows, vectors, team_scratch, err_words, team_polls, &rc)) return rc;
        if (ce_fused_team_launch<T, 16>(s, x, a, rows, vectors, team_scratch, err_words, team_polls, &rc)) return rc;
    }
    hipLaunchKernelGGL((ce_fused_mem_kernel<T, WIDE>), grid, dim3(kCeRowBlock), 0, s, x, a);
    return check_hip(hipGetLastError(), "fused cross-entropy launch");
}

// ---------------------------------------------------------------------------
// Softmax over the last axis (cpu_softmax_forward / backward, backend.py:354-374):
//   forward   y = exp(x - max) / sum(exp(x - max))          (a division, as on the CPU)
//   backward  dx (+)= y * (dy - sum(dy * y))
// One workgroup per row, two passes over the row (the second one is served by the
// caches): statistics first, then the element-wise pass.  Rows of up to 4 KB take
// one-wave workgroups, longer rows 256 threads.
// ---------------------------------------------------------------------------
template <typename T, int VEC, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, uint32_t V) {
    __shared__ MaxSum lds[BLOCK / kWave];
    const uint64_t row = blockIdx.x;
    const T* base = x + row * V;
    T* out = y + row * V;
    const MaxSum t = row_max_sum<T, VEC, BLOCK>(base, V, lds);
    const RowSplit<T, VEC> sp(base, V);
    if constexpr (VEC > 1) {
        const uint32_t extra = sp.head + (V - sp.tail_start);
        if (threadIdx.x < extra) {
            const uint32_t e = threadIdx.x < sp.head ? threadIdx.x : sp.tail_start + (threadIdx.x - sp.head);
            float v[1];
            VecIO<T, 1>::load(base + e, v);
            v[0] = quotient_io<T>(exp_io<T>(v[0] - t.m), row_scale<T>(t.s));
            VecIO<T, 1>::store(out + e, v);
        }
    }
    const T* body = base + sp.head;
    T* obody = out + sp.head;
    const float scale = row_scale<T>(t.s);
    for (uint32_t i0 = threadIdx.x; i0 < sp.nvec; i0 += BLOCK * kCeBwdUnroll) {
        float v[kCeBwdUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) VecIO<T, VEC>::load(body + (uint64_t)i * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) v[u][k] = quotient_io<T>(exp_io<T>(v[u][k] - t.m), scale);
                VecIO<T, VEC>::store(obody + (uint64_t)i * VEC, v[u]);
            }
        }
    }
}

// sum over the workgroup, fixed order: lanes by xor butterflies, waves in index order
template <int BLOCK>
__device__ __forceinline__ float block_sum(float v, float* lds) {
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) v = v + __shfl_xor(v, off);
    if constexpr (BLOCK > kWave) {
        if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = v;
        __syncthreads();
        v = lds[0];
#pragma unroll
        for (int w = 1; w < BLOCK / kWave; ++w) v = v + lds[w];
        __syncthreads();
    }
    return v;
}

template <typename T, int VEC, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
softmax_bwd_kernel(const T* __restrict__ y, const T* __restrict__ dy, T* dx, uint32_t V, int accumulate) {
    __shared__ float lds[BLOCK / kWave];
    const uint64_t row = blockIdx.x;
    const T* yb = y + row * V;
    const T* gb = dy + row * V;
    T* out = dx + row * V;
    const RowSplit<T, VEC> sp(yb, V);      // the launcher checked that the three tensors share their alignment
    const uint32_t extra = VEC > 1 ? sp.head + (V - sp.tail_start) : 0;
    const uint32_t e = threadIdx.x < sp.head ? threadIdx.x : sp.tail_start + (threadIdx.x - sp.head);
    float dot = 0.0f;
    if (threadIdx.x < extra) {
        float a[1], b[1];
        VecIO<T, 1>::load(yb + e, a);
        VecIO<T, 1>::load(gb + e, b);
        dot = b[0] * a[0];
    }
    for (uint32_t i0 = threadIdx.x; i0 < sp.nvec; i0 += BLOCK * kCeBwdUnroll) {
        float a[kCeBwdUnroll][VEC], b[kCeBwdUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) {
                VecIO<T, VEC>::load(yb + sp.head + (uint64_t)i * VEC, a[u]);
                VecIO<T, VEC>::load(gb + sp.head + (uint64_t)i * VEC, b[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) dot = dot + b[u][k] * a[u][k];
            }
        }
    }
    dot = block_sum<BLOCK>(dot, lds);
    if (threadIdx.x < extra) {
        float a[1], b[1];
        VecIO<T, 1>::load(yb + e, a);
        VecIO<T, 1>::load(gb + e, b);
        b[0] = a[0] * (b[0] - dot);
        if (accumulate) {
            float o[1];
            VecIO<T, 1>::load(out + e, o);
            b[0] = o[0] + b[0];
        }
        VecIO<T, 1>::store(out + e, b);
    }
    for (uint32_t i0 = threadIdx.x; i0 < sp.nvec; i0 += BLOCK * kCeBwdUnroll) {
        float a[kCeBwdUnroll][VEC], b[kCeBwdUnroll][VEC], o[kCeBwdUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) {
                VecIO<T, VEC>::load(yb + sp.head + (uint64_t)i * VEC, a[u]);
                VecIO<T, VEC>::load(gb + sp.head + (uint64_t)i * VEC, b[u]);
                if (accumulate) VecIO<T, VEC>::load(out + sp.head + (uint64_t)i * VEC, o[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kCeBwdUnroll; ++u) {
            const uint32_t i = i0 + u * BLOCK;
            if (i < sp.nvec) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float t = a[u][k] * (b[u][k] - dot);
                    if (accumulate) t = o[u][k] + t;
                    b[u][k] = t;
                }
                VecIO<T, VEC>::store(out + sp.head + (uint64_t)i * VEC, b[u]);
            }
        }
    }
}

// Rows of up to 64 * NV vectors whose length is a whole number of vectors: one wave
// holds the row in registers, so it is read once (forward: 2 passes of traffic in
// all, backward 3) and there is no barrier.  Same arithmetic as the two-pass kernels.
template <typename T, int VEC, int NV>
__global__ void __launch_bounds__(kWave)
softmax_fwd_reg_kernel(const T* __restrict__ x, T* __restrict__ y, uint32_t V, uint32_t VV) {
    const uint64_t row = blockIdx.x;
    const T* base = x + row * V;
    T* out = y + row * V;
    float v[NV][VEC];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) VecIO<T, VEC>::load(base + (uint64_t)c * VEC, v[i]);
    }
    // the CPU's order: row maximum, exp(x - max) once per element, their sum, a division
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) m = fmaxf(m, v[i][k]);
        }
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) m = fmaxf(m, __shfl_xor(m, off));
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                v[i][k] = exp_io<T>(v[i][k] - m);      // a row of -inf only: exp(nan) -> nan, as on the CPU
                sum = sum + v[i][k];
            }
        }
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) sum = sum + __shfl_xor(sum, off);
    const float scale = row_scale<T>(sum);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) v[i][k] = quotient_io<T>(v[i][k], scale);
            VecIO<T, VEC>::store(out + (uint64_t)c * VEC, v[i]);
        }
    }
}

template <typename T, int VEC, int NV>
__global__ void __launch_bounds__(kWave)
softmax_bwd_reg_kernel(const T* __restrict__ y, const T* __restrict__ dy, T* dx, uint32_t V, uint32_t VV, int accumulate) {
    const uint64_t row = blockIdx.x;
    const T* yb = y + row * V;
    const T* gb = dy + row * V;
    T* out = dx + row * V;
    float a[NV][VEC], b[NV][VEC];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
            VecIO<T, VEC>::load(yb + (uint64_t)c * VEC, a[i]);
            VecIO<T, VEC>::load(gb + (uint64_t)c * VEC, b[i]);
        }
    }
    float dot = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) dot = dot + b[i][k] * a[i][k];
        }
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) dot = dot + __shfl_xor(dot, off);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t c = i * kWave + threadIdx.x;
        if (c < VV) {
            float o[VEC];
            if (accumulate) VecIO<T, VEC>::load(out + (uint64_t)c * VEC, o);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float t = a[i][k] * (b[i][k] - dot);
                o[k] = accumulate ? (o[k] + t) : t;
            }
            VecIO<T, VEC>::store(out + (uint64_t)c * VEC, o);
        }
    }
}

template <typename T, int VEC, int NV>
void softmax_reg_launch(hipStream_t s, bool backward, const T* a, const T* b, T* out, uint64_t rows, uint32_t V, int acc) {
    const dim3 grid((uint32_t)rows);
    if (!backward) hipLaunchKernelGGL((softmax_fwd_reg_kernel<T, VEC, NV>), grid, dim3(kWave), 0, s, a, out, V, V / VEC);
    else hipLaunchKernelGGL((softmax_bwd_reg_kernel<T, VEC, NV>), grid, dim3(kWave), 0, s, a, b, out, V, V / VEC, acc);
}

template <typename T>
int softmax_typed(hipStream_t s, bool backward, const T* a, const T* b, T* out, uint64_t rows, uint32_t V, int acc) {
    constexpr int WIDE = WideVec<T>::value;
    // rows of any length keep 16-byte accesses through the head / tail split, which
    // needs every tensor to sit at the same offset within 16 bytes
    const uintptr_t mis = reinterpret_cast<uintptr_t>(a) & 15u;
    const bool same = (reinterpret_cast<uintptr_t>(out) & 15u) == mis && (!b || (reinterpret_cast<uintptr_t>(b) & 15u) == mis);
    const bool wide = V >= 4 * WIDE && same && mis % sizeof(T) == 0;
    const bool small = (uint64_t)V * sizeof(T) <= 4096;
    const dim3 grid((uint32_t)rows);
    if (mis == 0 && same && V % WIDE == 0 && V / WIDE <= 8 * kWave) {
        // every row starts 16-byte aligned and fits a wave's registers
        const uint32_t nv = (V / WIDE + kWave - 1) / kWave;
        if (nv <= 1) softmax_reg_launch<T, WIDE, 1>(s, backward, a, b, out, rows, V, acc);
        else if (nv <= 2) softmax_reg_launch<T, WIDE, 2>(s, backward, a, b, out, rows, V, acc);
        else if (nv <= 4) softmax_reg_launch<T, WIDE, 4>(s, backward, a, b, out, rows, V, acc);
        else softmax_reg_launch<T, WIDE, 8>(s, backward, a, b, out, rows, V, acc);
        return check_hip(hipGetLastError(), "softmax launch");
    }
#define AGRAD_SM(VEC, BLOCK)                                                                                     \
    do {                                                                                                         \
        if (!backward) hipLaunchKernelGGL((softmax_fwd_kernel<T, VEC, BLOCK>), grid, dim3(BLOCK), 0, s, a, out, V); \
        else hipLaunchKernelGGL((softmax_bwd_kernel<T, VEC, BLOCK>), grid, dim3(BLOCK), 0, s, a, b, out, V, acc);   \
    } while (0)
    if (wide && small) AGRAD_SM(WIDE, 64);
    else if (wide) AGRAD_SM(WIDE, 256);
    else if (small) AGRAD_SM(1, 64);
    else AGRAD_SM(1, 256);
#undef AGRAD_SM
    return check_hip(hipGetLastError(), "softmax launch");
}

int ce_check(const char* what, int dtype, uint64_t rows, uint32_t V) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "%s: unknown dtype %d", what, dtype);
    if (rows > 0x7fffffffull) return set_error(AGRAD_EINVAL, "%s: too many rows", what);
    if (V >= 0x7fffffffu) return set_error(AGRAD_EINVAL, "%s: vocabulary too large", what);
    return AGRAD_OK;
}

}  // namespace

int launch_ce_fwd(hipStream_t s, int dtype, const void* logits, const int32_t* labels, float* loss,
                  float* lse_out, uint64_t rows, uint32_t V, int* err_flag) {
    if (int rc = ce_check("cross-entropy forward", dtype, rows, V)) return rc;
    if (rows == 0) return AGRAD_OK;
    if (V == 0) return set_error(AGRAD_EINVAL, "cross-entropy forward: empty class axis");
    if (logits == nullptr || labels == nullptr || loss == nullptr)
        return set_error(AGRAD_EINVAL, "cross-entropy forward: null operand");
    if (dtype == AGRAD_F32)
        return ce_typed<float>(s, false, (const float*)logits, labels, loss, lse_out, nullptr, nullptr, nullptr, rows, V, 0, err_flag);
    return ce_typed<bf16_t>(s, false, (const bf16_t*)logits, labels, loss, lse_out, nullptr, nullptr, nullptr, rows, V, 0, err_flag);
}

int launch_ce_bwd(hipStream_t s, int dtype, const void* logits, const int32_t* labels, const float* dloss,
                  const float* lse, void* dlogits, uint64_t rows, uint32_t V, uint32_t flags, int* err_flag) {
    if (int rc = ce_check("cross-entropy backward", dtype, rows, V)) return rc;
    if (rows == 0 || V == 0) return AGRAD_OK;
    if (logits == nullptr || labels == nullptr || dloss == nullptr || dlogits == nullptr)
        return set_error(AGRAD_EINVAL, "cross-entropy backward: null operand");
    const int acc = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    if (dtype == AGRAD_F32)
        return ce_typed<float>(s, true, (const float*)logits, labels, nullptr, nullptr, dloss, lse, (float*)dlogits, rows, V, acc, err_flag);
    return ce_typed<bf16_t>(s, true, (const bf16_t*)logits, labels, nullptr, nullptr, dloss, lse, (bf16_t*)dlogits, rows, V, acc, err_flag);
}

uint64_t ce_fused_scratch_bytes() { return kTeamScratchBytes; }

int launch_ce_fused(hipStream_t s, int dtype, void* logits, const int32_t* targets, float* row_loss, float* lse,
                    const float* row_scale, uint64_t rows, uint32_t V, uint64_t row_base, float scale,
                    uint32_t write_grad, void* team_scratch, int* err_words, uint32_t team_polls) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "fused cross-entropy: unknown dtype %d", dtype);
    if (rows == 0 || V == 0) return AGRAD_OK;
    if (logits == nullptr || targets == nullptr) return set_error(AGRAD_EINVAL, "fused cross-entropy: null logits or targets");
    if (write_grad > 1u) return set_error(AGRAD_EINVAL, "fused cross-entropy: write_grad is 0 or 1 (the fp16 gradient store of the reference is not built)");
    if (rows > 0x7fffffffull || row_base + rows > 0xffffffffull) return set_error(AGRAD_EINVAL, "fused cross-entropy: too many rows");
    const CeFusedArgs a{targets, row_loss, lse, row_scale, V, (uint32_t)row_base, scale, write_grad};
    if (dtype == AGRAD_F32) return ce_fused_typed<float>(s, (float*)logits, a, rows, team_scratch, err_words, team_polls);
    return ce_fused_typed<bf16_t>(s, (bf16_t*)logits, a, rows, team_scratch, err_words, team_polls);
}

int launch_softmax_fwd(hipStream_t s, int dtype, const void* x, void* y, uint64_t rows, uint32_t V) {
    if (int rc = ce_check("softmax forward", dtype, rows, V)) return rc;
    if (rows == 0 || V == 0) return AGRAD_OK;
    if (x == nullptr || y == nullptr) return set_error(AGRAD_EINVAL, "softmax forward: null operand");
    if (dtype == AGRAD_F32) return softmax_typed<float>(s, false, (const float*)x, nullptr, (float*)y, rows, V, 0);
    return softmax_typed<bf16_t>(s, false, (const bf16_t*)x, nullptr, (bf16_t*)y, rows, V, 0);
}

int launch_softmax_bwd(hipStream_t s, int dtype, const void* y, const void* dy, void* dx, uint64_t rows, uint32_t V,
                       uint32_t flags) {
    if (int rc = ce_check("softmax backward", dtype, rows, V)) return rc;
    if (rows == 0 || V == 0) return AGRAD_OK;
    if (y == nullptr || dy == nullptr || dx == nullptr) return set_error(AGRAD_EINVAL, "softmax backward: null operand");
    const int acc = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    if (dtype == AGRAD_F32) return softmax_typed<float>(s, true, (const float*)y, (const float*)dy, (float*)dx, rows, V, acc);
    return softmax_typed<bf16_t>(s, true, (const bf16_t*)y, (const bf16_t*)dy, (bf16_t*)dx, rows, V, acc);
}

}  // namespace agrad
