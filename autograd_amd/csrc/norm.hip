// LayerNorm / RMSNorm forward and backward for gfx950, with the residual add
// fused in (forward: h = x + r is normalised and optionally stored; backward:
// the incoming residual gradient is added to dx in the same pass).
//
// Row mapping.  A row of C elements is owned by TPR threads, the smallest TPR
// that lets a thread hold its share (NV 128-bit vectors) in registers:
//   TPR = 16, 32  four / two rows per wavefront (C = 384 is 16 lanes x 6 vectors);
//                 narrow rows would otherwise leave lanes idle and pay the
//                 per-row reductions once per row instead of once per 2-4 rows
//   TPR = 64      one wavefront per row
//                 (all three: cross-lane sums by DPP / ds_swizzle only, sixteen
//                 to four rows per 256-thread workgroup)
//   TPR = 128, 256, 1024  one workgroup per row, wave totals staged through LDS
// A row is read from HBM exactly once per pass; the two-pass mean / variance of
// the reference (backend.py:416-433) runs on registers.
//
// Backward keeps per-column partial sums of dgamma / dbeta in registers while a
// workgroup walks its rows (grid-stride), writes one partial row per workgroup
// to a workspace, and a second small kernel folds the partial rows in fixed
// order: no atomics, run-to-run deterministic.
//
// Arithmetic order follows the reference CPU kernels: LayerNorm
// backend.py:416-487, RMSNorm backend.py:1097-1108, 1228-1251, 1737-1745,
// 1990-2011.  Rows that are unaligned or have C % vector != 0 take a scalar
// workgroup-per-row kernel with the same arithmetic.
#include "common.hpp"
#include "launch.hpp"

#include <cstdlib>
#include <map>
#include <mutex>
#include <vector>

// Partial dgamma / dbeta rows of the entry point that allocates nothing
// (agrad_norm_backward_noalloc): a fixed array in every GPU's memory, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress;
// the device address it yields (one per GPU) is what kernels are given.
static __device__ __align__(256) unsigned char scratch[AGRAD_NOALLOC_SCRATCH_BYTES];

namespace agrad {

namespace {

constexpr int kMaxEPT = 24;  // most elements of a row a thread may keep in registers

// a * b + c.  fp32 tensors: two roundings, like the CPU kernels (bit-level
// closeness to numpy).  bf16 tensors: one fused instruction -- their results are
// rounded to 8 bits anyway, and at 2 bytes per element the instruction count, not
// HBM, is what the norm kernels run into first.
template <typename T>
__device__ __forceinline__ float mad(float a, float b, float c) {
    if constexpr (sizeof(T) == 2) return __builtin_fmaf(a, b, c);
    else return a * b + c;
}

template <typename T>
struct NormFwdArgs {
    const T* x; const T* res; const float* gamma; const float* beta; T* h; T* y;
    uint64_t rows; uint32_t C; float eps; int kind;
};

template <typename T>
struct NormBwdArgs {
    const T* x; const T* dy; const float* gamma; const T* dres; T* dx; T* dx2;
    float* pgamma; float* pbeta;      // [blocks, C] partial rows, one per workgroup
    uint64_t rows; uint32_t C; float eps; int kind; uint32_t flags;
};

// Second stage of the dgamma / dbeta column sums: out[c] (+)= sum over the P
// partial rows the backward kernel left in the workspace.  One workgroup covers
// 8 column vectors with 128 row lanes; a row lane loads its rows 8 at a time
// (independent loads, one memory latency per 1024 rows) and adds them in row
// order; the 128 lane sums are then added in lane order in two steps.  Fixed
// order, no atomics: the result is the same on every run.
//
// An in-kernel alternative (ticket counters, partial rows exchanged through
// agent-scope atomic stores, a 16-ary tree) was measured 3 to 11 us slower per
// call on MI355X than this second launch, and device-wide fences slower still
// (each one writes back a whole L2), so the second launch stayed.
constexpr int kFinalizeCols = 8;     // column vectors of a finalize workgroup (2, in 256-thread workgroups, was measured 1.5-3.5 us slower)
constexpr int kFinalizeLanes = 128;  // row lanes per column vector

// One finalize workgroup: column block `col_block` of out[c] (+)= sum over the P rows of src.
template <int W>   // W = 4: float4 columns, W = 1: scalar columns
__device__ __forceinline__ void colsum_finalize_block(const float* __restrict__ src, float* __restrict__ dst, uint32_t P,
                                                      uint32_t C, int accumulate, int out_bf16, uint32_t col_block) {
    constexpr int COLS = kFinalizeCols, LANES = kFinalizeLanes, BATCH = 8;
    __shared__ float tile[LANES][COLS * W];
    __shared__ float tile2[LANES / 16][COLS * W];
    const uint32_t cl = threadIdx.x % COLS, rl = threadIdx.x / COLS;
    const uint32_t c = (col_block * COLS + cl) * W;
    float s[W];
#pragma unroll
    for (int k = 0; k < W; ++k) s[k] = 0.0f;
    if (c < C) {
        for (uint32_t r0 = rl; r0 < P; r0 += LANES * BATCH) {
            float v[BATCH][W];
#pragma unroll
            for (uint32_t j = 0; j < BATCH; ++j) {
                const uint32_t r = r0 + j * LANES;
                if (r < P) {
                    if constexpr (W == 4) {
                        const float4 t = *reinterpret_cast<const float4*>(src + (uint64_t)r * C + c);
                        v[j][0] = t.x; v[j][1] = t.y; v[j][2] = t.z; v[j][3] = t.w;
                    } else {
                        v[j][0] = src[(uint64_t)r * C + c];
                    }
                }
            }
#pragma unroll
            for (uint32_t j = 0; j < BATCH; ++j) {
                const uint32_t r = r0 + j * LANES;
                if (r < P) {
#pragma unroll
                    for (int k = 0; k < W; ++k) s[k] = s[k] + v[j][k];
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < W; ++k) tile[rl][cl * W + k] = s[k];
    __syncthreads();
    // 128 lane sums -> 8 (each adds 16 in lane order) -> 1
    if (rl < LANES / 16) {
#pragma unroll
        for (int k = 0; k < W; ++k) {
            float t = tile[rl * 16][cl * W + k];
#pragma unroll
            for (int j = 1; j < 16; ++j) t = t + tile[rl * 16 + j][cl * W + k];
            tile2[rl][cl * W + k] = t;
        }
    }
    __syncthreads();
    if (rl == 0 && c < C) {
#pragma unroll
        for (int k = 0; k < W; ++k) {
            float t = tile2[0][cl * W + k];
#pragma unroll
            for (int j = 1; j < LANES / 16; ++j) t = t + tile2[j][cl * W + k];
            if (out_bf16) {
                // a bf16 destination: the sum is finished in fp32 and rounded once
                bf16_t* d16 = reinterpret_cast<bf16_t*>(dst);
                if (accumulate) t = bf16_bits_to_f32(d16[c + k]) + t;
                d16[c + k] = (bf16_t)f32_to_bf16_bits(t);
            } else {
                dst[c + k] = accumulate ? (dst[c + k] + t) : t;
            }
        }
    }
}

template <int W>
__global__ void __launch_bounds__(kFinalizeCols * kFinalizeLanes)
colsum_finalize_kernel(const float* __restrict__ pg, const float* __restrict__ pb, uint32_t P, uint32_t C,
                       float* __restrict__ dgamma, float* __restrict__ dbeta, int accumulate, int out_bf16) {
    const float* src = blockIdx.y == 0 ? pg : pb;
    float* dst = blockIdx.y == 0 ? dgamma : dbeta;
    if (src == nullptr) return;                      // uniform over the workgroup
    colsum_finalize_block<W>(src, dst, P, C, accumulate, out_bf16, blockIdx.x);
}

// The same fold for up to kFinalizeManyJobs column sums that were left pending, in ONE
// launch: blockIdx.z names the job, and a job runs exactly the workgroups, loads and adds
// that colsum_finalize_kernel would run for it, so the results are the same bits.  What it
// saves is the launches: a finalize is a few microseconds of launch floor around a few
// hundred nanoseconds of work, paid once per norm of a network when every backward call
// folds its own partial rows.
struct ColsumJobs { ColsumJob job[kFinalizeManyJobs]; };

template <int W>
__global__ void __launch_bounds__(kFinalizeCols * kFinalizeLanes)
colsum_finalize_many_kernel(const ColsumJobs jobs) {
    const ColsumJob& j = jobs.job[blockIdx.z];
    const float* src = blockIdx.y == 0 ? j.pa : j.pb;
    float* dst = reinterpret_cast<float*>(blockIdx.y == 0 ? j.out_a : j.out_b);
    if (src == nullptr || dst == nullptr) return;    // uniform over the workgroup
    if (blockIdx.x * (kFinalizeCols * W) >= j.C) return;     // (the grid is as wide as the widest job)
    colsum_finalize_block<W>(src, dst, j.P, j.C, (int)j.accumulate, (int)j.out_bf16, blockIdx.x);
}

// gamma / beta are fp32 whatever the activation type: VEC of them is one or two
// 128-bit loads.
template <int VEC>
__device__ __forceinline__ void load_param(const float* p, float (&v)[VEC]) {
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

// Rotating LDS slot for consecutive row reductions (three slots: a slot is
// rewritten only after two later barriers).
struct SlotRing {
    int cur = 0;
    __device__ __forceinline__ int next() { const int s = cur; cur = cur == 2 ? 0 : cur + 1; return s; }
};

template <typename T> __device__ __forceinline__ float round_through(float v);
template <> __device__ __forceinline__ float round_through<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_through<bf16_t>(float v) {
    return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

// ----------------------------------------------------------------------------
// forward, register-resident row
// ----------------------------------------------------------------------------
// Workgroup size of the forward kernel when a row needs at most one wave: the
// rows of a workgroup never talk to each other, so the smallest workgroup (one
// wave) gives the dispatcher the most freedom.
constexpr int kFwdGroupBlock = 64;

// The flavour (KIND), the fused residual (RES) and which parameters there are (PARAMS: 0 none,
// 1 gamma, 2 gamma and beta) are compile-time: with them as run-time branches the fp32 kernel
// at C = 1536 held more values live and took 36.5 us where the specialised one takes 33.3 us
// (a plain copy: 31.3 us), and a parameter load behind a branch waits for itself alone -- NV
// cache round trips one after the other between the row sums and the stores.  Here the NV
// vectors of gamma (and beta) are requested together: before the row where params_early()
// says so (they arrive while the row is in flight, at the price of NV * VEC registers each),
// else right after the row sums.  A PARAMS == 2 launch may still lack one of the two (a
// LayerNorm without bias): the missing one is read from kNoParam and ignored.
__device__ const float kNoParam[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};

template <typename T>
constexpr bool params_early(int tpr, int kind, int params) {
    return tpr >= 32 && tpr <= 128;
}

template <typename T, int VEC, int NV, int TPR, int KIND, bool RES, int PARAMS>
__global__ void __launch_bounds__(TPR >= 128 ? TPR : kFwdGroupBlock)
norm_fwd_kernel(const NormFwdArgs<T> a) {
    constexpr int BLOCK = TPR >= 128 ? TPR : kFwdGroupBlock;
    constexpr int RPB = BLOCK / TPR;
    constexpr bool EARLY = params_early<T>(TPR, KIND, PARAMS);
    __shared__ float lds[3 * kRowSumSlot * (TPR > kWave ? TPR / kWave : 1)];

    const int sub = threadIdx.x / TPR;
    const int lane = threadIdx.x % TPR;
    const uint64_t row = (uint64_t)blockIdx.x * RPB + sub;
    if (row >= a.rows) return;  // a lane group leaves alone: its sums never read other groups; RPB == 1 never exits
    const uint32_t C = a.C;
    const uint64_t base = row * C;

    // Every load of the row is issued before anything waits for one.  A load behind a
    // branch gets a full wait of its own (its value meets the zeros of the lanes that skip
    // it), which puts the NV vectors of a row one memory latency after the other; so a lane
    // past the end of the row loads the row's first vector instead (a valid address, one
    // cache line for all such lanes) and its values are zeroed afterwards.
    typedef RawVec<T, VEC> Raw;
    float v[NV][VEC];
    float gam[PARAMS >= 1 ? NV : 1][VEC], bet[PARAMS >= 2 ? NV : 1][VEC];
    bool on[NV];
    uint32_t col_ld[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t col = (uint32_t)(i * TPR + lane) * VEC;
        on[i] = col < C;
        col_ld[i] = on[i] ? col : 0u;
    }
    const bool has_gamma = PARAMS == 1 || a.gamma != nullptr, has_beta = a.beta != nullptr;
    auto load_params = [&]() {
        if constexpr (PARAMS >= 1) {
            const float* gp = has_gamma ? a.gamma : kNoParam;
            const uint32_t gmask = has_gamma ? ~0u : 0u;
#pragma unroll
            for (int i = 0; i < NV; ++i) load_param<VEC>(gp + (col_ld[i] & gmask), gam[i]);
        }
        if constexpr (PARAMS >= 2) {
            const float* bp = has_beta ? a.beta : kNoParam;
            const uint32_t bmask = has_beta ? ~0u : 0u;
#pragma unroll
            for (int i = 0; i < NV; ++i) load_param<VEC>(bp + (col_ld[i] & bmask), bet[i]);
        }
    };
    if constexpr (EARLY) load_params();
    typename Raw::type rx[NV], rr[RES ? NV : 1];
#pragma unroll
    for (int i = 0; i < NV; ++i) rx[i] = Raw::load(a.x + base + col_ld[i]);
    if constexpr (RES) {
#pragma unroll
        for (int i = 0; i < NV; ++i) rr[i] = Raw::load(a.res + base + col_ld[i]);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        Raw::unpack(rx[i], v[i]);
#pragma unroll
        for (int k = 0; k < VEC; ++k) v[i][k] = on[i] ? v[i][k] : 0.0f;
    }
    if constexpr (RES) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            float r[VEC];
            Raw::unpack(rr[i], r);
#pragma unroll
            for (int k = 0; k < VEC; ++k) v[i][k] = on[i] ? round_through<T>(v[i][k] + r[k]) : 0.0f;
            if (on[i] && a.h != nullptr) VecIO<T, VEC>::store(a.h + base + col_ld[i], v[i]);
        }
    }

    const float fC = (float)C;
    float scale;  // 1 / sqrt(var + eps)  or  1 / sqrt(mean(x^2) + eps)
    if constexpr (KIND == AGRAD_NORM_LAYER) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) s = s + v[i][k];
        const float mean = row_sum<TPR>(s, lds, 0) / fC;
        float q = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float d = on[i] ? (v[i][k] - mean) : 0.0f;
                v[i][k] = d;
                q = mad<T>(d, d, q);
            }
        const float var = row_sum<TPR>(q, lds, 1) / fC;
        scale = 1.0f / sqrtf(var + a.eps);
    } else {
        float q = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) q = mad<T>(v[i][k], v[i][k], q);
        const float ms = row_sum<TPR>(q, lds, 0) / fC;
        scale = 1.0f / sqrtf(ms + a.eps);
    }

    if constexpr (!EARLY) load_params();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        float o[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) o[k] = v[i][k] * scale;
        if constexpr (PARAMS >= 1) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) o[k] = has_gamma ? o[k] * gam[i][k] : o[k];
        }
        if constexpr (PARAMS >= 2) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) o[k] = has_beta ? o[k] + bet[i][k] : o[k];
        }
        if (on[i]) VecIO<T, VEC>::store(a.y + base + col_ld[i], o);
    }
}

// ----------------------------------------------------------------------------
// backward, register-resident row, dgamma / dbeta partials per workgroup
// ----------------------------------------------------------------------------
// Threads of a backward workgroup whose rows take a wave or less each (512 and 1024, with a
// half and a quarter of the partial rows, were measured: within 1 us either way at 16384 rows).
constexpr int kBwdGroupBlock = 256;
// The residual gradient of a row is requested (all its vectors together) with the next row's
// prefetch, or only once the row's own sums are under way.
constexpr bool kDresEarly = false;

// Compile-time: the flavour (KIND), which column sums are kept (SUMS: 0 none, 1 dgamma, 2 dgamma
// and dbeta -- their accumulators are NV * VEC registers each, and an RMSNorm has no beta) and
// whether a residual gradient comes in (DRES).  As run-time branches these cost registers (the
// bf16 kernel at C = 1536 held 207 and ran two waves per SIMD) and put every load that sat
// behind one of them a memory latency of its own away from the next.
template <typename T, int VEC, int NV, int TPR, int KIND, int SUMS, bool DRES>
__global__ void __launch_bounds__(TPR >= 128 ? TPR : kBwdGroupBlock)
norm_bwd_kernel(const NormBwdArgs<T> a) {
    constexpr int BLOCK = TPR >= 128 ? TPR : kBwdGroupBlock;
    constexpr int RPB = BLOCK / TPR;
    constexpr int NWAVES = BLOCK / kWave;
    constexpr bool is_ln = KIND == AGRAD_NORM_LAYER;
    constexpr bool want_pg = SUMS >= 1, want_pb = SUMS >= 2;
    __shared__ float lds[3 * kRowSumSlot * (TPR > kWave ? TPR / kWave : 1)];
    extern __shared__ float comb[];  // (NWAVES - 1) * C floats when RPB > 1

    const int sub = threadIdx.x / TPR;
    const int lane = threadIdx.x % TPR;
    const uint32_t C = a.C;
    const float fC = (float)C;
    const bool acc = (a.flags & AGRAD_ACC_INPUT_GRAD) != 0;
    const bool acc2 = (a.flags & AGRAD_ACC_INPUT_GRAD2) != 0;

    // A lane with nothing to load (past the end of the row, no next row, no gamma) loads
    // from a valid address that every such lane shares and never uses the value: a load
    // behind a branch gets a wait of its own, which would put a row's vectors one memory
    // latency after the other.
    bool on[NV];
    uint32_t col_ld[NV];
    float gam[NV][VEC], pg[want_pg ? NV : 1][VEC], pb[want_pb ? NV : 1][VEC];
    const bool has_gamma = a.gamma != nullptr;
    {
        const float* gp = has_gamma ? a.gamma : kNoParam;
        const uint32_t gmask = has_gamma ? ~0u : 0u;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint32_t col = (uint32_t)(i * TPR + lane) * VEC;
            on[i] = col < C;
            col_ld[i] = on[i] ? col : 0u;
            load_param<VEC>(gp + (col_ld[i] & gmask), gam[i]);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) gam[i][k] = has_gamma ? gam[i][k] : 1.0f;
    }
#pragma unroll
    for (int i = 0; i < (want_pg ? NV : 1); ++i)
#pragma unroll
        for (int k = 0; k < VEC; ++k) pg[i][k] = 0.0f;
#pragma unroll
    for (int i = 0; i < (want_pb ? NV : 1); ++i)
#pragma unroll
        for (int k = 0; k < VEC; ++k) pb[i][k] = 0.0f;
    SlotRing ring;

    // Rows are software-pipelined: the x and dy vectors of the NEXT row are requested (as
    // raw bits) before the current row is worked on, so a wave always has a row of loads in
    // flight while it computes; the current row's residual gradient is requested with them.
    typedef RawVec<T, VEC> Raw;
    typename Raw::type nx[NV], ng[NV], rd[DRES ? NV : 1];
    const uint64_t stride = (uint64_t)gridDim.x * RPB;
    uint64_t row = (uint64_t)blockIdx.x * RPB + sub;
    {
        const bool live = row < a.rows;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint64_t off = live ? row * C + col_ld[i] : 0ull;
            nx[i] = Raw::load(a.x + off);
            ng[i] = Raw::load(a.dy + off);
        }
    }
    for (; row < a.rows; row += stride) {
        const uint64_t base = row * C;
        float xv[NV][VEC], g[NV][VEC];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            Raw::unpack(nx[i], xv[i]);
            Raw::unpack(ng[i], g[i]);
            if (!on[i]) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) { xv[i][k] = 0.0f; g[i][k] = 0.0f; }
            }
        }
        {
            const bool live = row + stride < a.rows;
            const uint64_t nbase = (row + stride) * C;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const uint64_t off = live ? nbase + col_ld[i] : 0ull;
                nx[i] = Raw::load(a.x + off);
                ng[i] = Raw::load(a.dy + off);
            }
        }
        if constexpr (DRES && kDresEarly) {
#pragma unroll
            for (int i = 0; i < NV; ++i) rd[i] = Raw::load(a.dres + base + col_ld[i]);
        }

        // Row statistics and the two row sums of the dx formula in ONE reduction
        // phase (after the mean, for LayerNorm).  With d = x - mean (or x):
        //   q = sum d^2,   s1 = sum dy*gamma,   s2r = sum dy*gamma*d,
        // and sum dy*gamma*x_hat = s2r * scale.  xv becomes d, then x_hat.
        if constexpr (is_ln) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int k = 0; k < VEC; ++k) s = s + xv[i][k];
            const float mean = row_sum<TPR>(s, lds, ring.next()) / fC;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int k = 0; k < VEC; ++k) xv[i][k] = on[i] ? (xv[i][k] - mean) : 0.0f;
        }
        float q = 0.0f, s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float d = xv[i][k];
                q = mad<T>(d, d, q);
                const float dyg = g[i][k] * gam[i][k];
                s1 = s1 + dyg;
                s2 = mad<T>(dyg, d, s2);
            }
        if constexpr (DRES && !kDresEarly) {
#pragma unroll
            for (int i = 0; i < NV; ++i) rd[i] = Raw::load(a.dres + base + col_ld[i]);
        }
        if (a.dx != nullptr) row_sum3<TPR>(q, s1, s2, lds, ring.next());
        else q = row_sum<TPR>(q, lds, ring.next());
        const float scale = 1.0f / sqrtf(q / fC + a.eps);
        s2 = s2 * scale;

#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float xh = xv[i][k] * scale;
                xv[i][k] = xh;
                if constexpr (want_pg) pg[i][k] = mad<T>(g[i][k], xh, pg[i][k]);
                if constexpr (want_pb) pb[i][k] = pb[i][k] + g[i][k];
                g[i][k] = g[i][k] * gam[i][k];
            }

        if (a.dx != nullptr) {
            float c1 = 0.0f, c2;
            if constexpr (is_ln) {
                c1 = (s1 / fC) * scale;
                c2 = (s2 / fC) * scale;
            } else {
                c2 = s2 / fC;
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                float t[VEC];
                if constexpr (is_ln) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) {
                        const float u = mad<T>(g[i][k], scale, -c1);
                        t[k] = mad<T>(-xv[i][k], c2, u);
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < VEC; ++k)
                        t[k] = mad<T>(-xv[i][k], c2, g[i][k]) * scale;
                }
                if constexpr (DRES) {
                    float r[VEC];
                    Raw::unpack(rd[i], r);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) t[k] = r[k] + t[k];
                }
                if (on[i]) {
                    const uint32_t col = col_ld[i];
                    if (a.dx2 != nullptr) {
                        float t2[VEC];
                        if (acc2) {
                            VecIO<T, VEC>::load(a.dx2 + base + col, t2);
#pragma unroll
                            for (int k = 0; k < VEC; ++k) t2[k] = t2[k] + t[k];
                        } else {
#pragma unroll
                            for (int k = 0; k < VEC; ++k) t2[k] = t[k];
                        }
                        VecIO<T, VEC>::store(a.dx2 + base + col, t2);
                    }
                    if (acc) {
                        float old[VEC];
                        VecIO<T, VEC>::load(a.dx + base + col, old);
#pragma unroll
                        for (int k = 0; k < VEC; ++k) t[k] = old[k] + t[k];
                    }
                    VecIO<T, VEC>::store(a.dx + base + col, t);
                }
            }
        }
    }

    // one partial row per workgroup
    if constexpr (want_pg) {
        if constexpr (RPB > 1) {
            // lane groups of one wave first (fixed order), then the waves through LDS
            if constexpr (TPR < kWave) {
#pragma unroll
                for (int i = 0; i < NV; ++i)
#pragma unroll
                    for (int k = 0; k < VEC; ++k) {
                        if constexpr (TPR == 16) {
                            pg[i][k] = pg[i][k] + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, pg[i][k]), kSwizzleXor16));
                            if constexpr (want_pb) pb[i][k] = pb[i][k] + __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, pb[i][k]), kSwizzleXor16));
                        }
                        pg[i][k] = pg[i][k] + __shfl_xor(pg[i][k], 32);
                        if constexpr (want_pb) pb[i][k] = pb[i][k] + __shfl_xor(pb[i][k], 32);
                    }
            }
            const int wave = threadIdx.x / kWave;
            const bool owner = (threadIdx.x % kWave) < TPR;   // one lane group per wave speaks for it
#pragma unroll
            for (int pass = 0; pass < SUMS; ++pass) {
                float* out = pass == 0 ? a.pgamma : a.pbeta;
                if (wave > 0 && owner) {
#pragma unroll
                    for (int i = 0; i < NV; ++i)
                        if (on[i]) {
#pragma unroll
                            for (int k = 0; k < VEC; ++k)
                                comb[(uint32_t)(wave - 1) * C + col_ld[i] + k] = pass == 0 ? pg[i][k] : pb[want_pb ? i : 0][k];
                        }
                }
                __syncthreads();
                if (wave == 0 && owner) {
#pragma unroll
                    for (int i = 0; i < NV; ++i)
                        if (on[i]) {
                            float t[VEC];
#pragma unroll
                            for (int k = 0; k < VEC; ++k) {
                                t[k] = pass == 0 ? pg[i][k] : pb[want_pb ? i : 0][k];
                                for (int w = 0; w < NWAVES - 1; ++w) t[k] = t[k] + comb[(uint32_t)w * C + col_ld[i] + k];
                            }
#pragma unroll
                            for (int k = 0; k < VEC; k += 2)
                                { out[(uint64_t)blockIdx.x * C + col_ld[i] + k] = t[k]; out[(uint64_t)blockIdx.x * C + col_ld[i] + k + 1] = t[k + 1]; }
                        }
                }
                __syncthreads();
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i)
                if (on[i]) {
#pragma unroll
                    for (int k = 0; k < VEC; k += 2) {
                        { a.pgamma[(uint64_t)blockIdx.x * C + col_ld[i] + k] = pg[i][k]; a.pgamma[(uint64_t)blockIdx.x * C + col_ld[i] + k + 1] = pg[i][k + 1]; }
                        if constexpr (want_pb) { a.pbeta[(uint64_t)blockIdx.x * C + col_ld[i] + k] = pb[i][k]; a.pbeta[(uint64_t)blockIdx.x * C + col_ld[i] + k + 1] = pb[i][k + 1]; }
                    }
                }
        }
    }
}

// ----------------------------------------------------------------------------
// scalar fallbacks: any C, any alignment; one 256-thread workgroup per row,
// the row is re-read from memory for each pass.
// ----------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float ld1(const T* p) { float v[1]; VecIO<T, 1>::load(p, v); return v[0]; }
template <typename T>
__device__ __forceinline__ void st1(T* p, float f) { float v[1] = {f}; VecIO<T, 1>::store(p, v); }

template <typename T>
__device__ __forceinline__ float generic_row_value(const NormFwdArgs<T>& a, uint64_t idx) {
    float v = ld1(a.x + idx);
    if (a.res != nullptr) v = round_through<T>(v + ld1(a.res + idx));
    return v;
}

template <typename T>
__global__ void __launch_bounds__(256) norm_fwd_generic_kernel(const NormFwdArgs<T> a) {
    __shared__ float lds[3 * kRowSumSlot * 4];
    const uint32_t C = a.C;
    const float fC = (float)C;
    const uint64_t base = (uint64_t)blockIdx.x * C;
    float mean = 0.0f, scale;
    if (a.kind == AGRAD_NORM_LAYER) {
        float s = 0.0f;
        for (uint32_t c = threadIdx.x; c < C; c += 256) s = s + generic_row_value(a, base + c);
        mean = row_sum<256>(s, lds, 0) / fC;
        float q = 0.0f;
        for (uint32_t c = threadIdx.x; c < C; c += 256) {
            const float d = generic_row_value(a, base + c) - mean;
            q = q + d * d;
        }
        scale = 1.0f / sqrtf(row_sum<256>(q, lds, 1) / fC + a.eps);
    } else {
        float q = 0.0f;
        for (uint32_t c = threadIdx.x; c < C; c += 256) {
            const float v = generic_row_value(a, base + c);
            q = q + v * v;
        }
        scale = 1.0f / sqrtf(row_sum<256>(q, lds, 0) / fC + a.eps);
    }
    for (uint32_t c = threadIdx.x; c < C; c += 256) {
        const float v = generic_row_value(a, base + c);
        if (a.res != nullptr && a.h != nullptr) st1(a.h + base + c, v);
        float o = (v - mean) * scale;
        if (a.gamma != nullptr) o = o * a.gamma[c];
        if (a.beta != nullptr) o = o + a.beta[c];
        st1(a.y + base + c, o);
    }
}

template <typename T>
__global__ void __launch_bounds__(256) norm_bwd_generic_kernel(const NormBwdArgs<T> a) {
    __shared__ float lds[3 * kRowSumSlot * 4];
    const uint32_t C = a.C;
    const float fC = (float)C;
    const bool is_ln = a.kind == AGRAD_NORM_LAYER;
    const bool acc = (a.flags & AGRAD_ACC_INPUT_GRAD) != 0;
    const bool acc2 = (a.flags & AGRAD_ACC_INPUT_GRAD2) != 0;
    bool first = true;
    SlotRing ring;
    for (uint64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
        const uint64_t base = row * C;
        float mean = 0.0f, scale;
        if (is_ln) {
            float s = 0.0f;
            for (uint32_t c = threadIdx.x; c < C; c += 256) s = s + ld1(a.x + base + c);
            mean = row_sum<256>(s, lds, ring.next()) / fC;
            float q = 0.0f;
            for (uint32_t c = threadIdx.x; c < C; c += 256) {
                const float d = ld1(a.x + base + c) - mean;
                q = q + d * d;
            }
            scale = 1.0f / sqrtf(row_sum<256>(q, lds, ring.next()) / fC + a.eps);
        } else {
            float q = 0.0f;
            for (uint32_t c = threadIdx.x; c < C; c += 256) {
                const float v = ld1(a.x + base + c);
                q = q + v * v;
            }
            scale = 1.0f / sqrtf(row_sum<256>(q, lds, ring.next()) / fC + a.eps);
        }
        float s1 = 0.0f, s2 = 0.0f;
        for (uint32_t c = threadIdx.x; c < C; c += 256) {
            const float xh = (ld1(a.x + base + c) - mean) * scale;
            const float g = ld1(a.dy + base + c);
            // each thread owns its columns of this workgroup's partial row
            if (a.pgamma != nullptr) {
                float* p = a.pgamma + (uint64_t)blockIdx.x * C + c;
                *p = first ? (g * xh) : (*p + g * xh);
            }
            if (a.pbeta != nullptr) {
                float* p = a.pbeta + (uint64_t)blockIdx.x * C + c;
                *p = first ? g : (*p + g);
            }
            const float dyg = g * (a.gamma != nullptr ? a.gamma[c] : 1.0f);
            s1 = s1 + dyg;
            s2 = s2 + dyg * xh;
        }
        first = false;
        if (a.dx != nullptr) {
            row_sum2<256>(s1, s2, lds, ring.next());
            const float c1 = (s1 / fC) * scale;
            const float c2 = is_ln ? (s2 / fC) * scale : (s2 / fC);
            for (uint32_t c = threadIdx.x; c < C; c += 256) {
                const float xh = (ld1(a.x + base + c) - mean) * scale;
                const float dyg = ld1(a.dy + base + c) * (a.gamma != nullptr ? a.gamma[c] : 1.0f);
                float t;
                if (is_ln) {
                    t = dyg * scale;
                    t = t - c1;
                    t = t - xh * c2;
                } else {
                    t = (dyg - xh * c2) * scale;
                }
                if (a.dres != nullptr) t = ld1(a.dres + base + c) + t;
                if (a.dx2 != nullptr) st1(a.dx2 + base + c, acc2 ? (ld1(a.dx2 + base + c) + t) : t);
                st1(a.dx + base + c, acc ? (ld1(a.dx + base + c) + t) : t);
            }
        }
    }
}

// ----------------------------------------------------------------------------
// geometry
// ----------------------------------------------------------------------------
struct NormPlan {
    bool generic;
    int tpr;  // 16, 32, 64, 128, 256, 1024
    int nv;   // vectors per thread
    int rpb;  // rows per workgroup
};

// Elements of a row a thread may hold.  Forward keeps one array; backward keeps
// x, dy, gamma, the two column accumulators and the prefetched next row, so it
// gets fewer -- except bf16, whose prefetched rows stay packed (half the
// registers).  Measured on MI355X over the benchmark shapes.
int norm_max_ept(bool backward, int dtype) {
    if (!backward) return 24;
    return dtype == AGRAD_BF16 ? 24 : 16;
}

NormPlan plan_norm(uint32_t C, int dtype, bool aligned, bool backward) {
    const int vec = dtype == AGRAD_BF16 ? 8 : 4;
    NormPlan p{true, 256, 0, 1};
    if (!aligned || C % vec != 0) return p;
    const uint32_t cv = C / vec;
    const uint32_t max_nv = (uint32_t)(norm_max_ept(backward, dtype) / vec);
    const int tprs[6] = {16, 32, 64, 128, 256, 1024};
    for (int t : tprs) {
        const uint32_t nv = (cv + t - 1) / t;
        if (nv <= max_nv) {
            p.generic = false;
            p.tpr = t;
            p.nv = (int)nv;
            p.rpb = t >= 128 ? 1 : (backward ? kBwdGroupBlock : kFwdGroupBlock) / t;
            return p;
        }
    }
    return p;
}

// The backward kernel is a persistent grid: every workgroup walks rows with a
// stride of the grid and leaves one partial dgamma/dbeta row.  Measured on
// MI355X over the benchmark shapes: a grid larger than what the GPU holds at
// once (`resident`, from the occupancy query -- register use differs a lot
// between instantiations) loses to one round, because the stragglers of the
// second round run on a mostly idle chip; and beyond 768 workgroups (three to a
// CU) more waves only add loads in flight that the memory system does not need
// -- every load of a row is in flight at once here: 65536 x 4096 bf16 without
// column sums 386 us with 1024 workgroups, 376 us with 768; 256 or 512 lose
// 10 to 90 % at every shape.
constexpr uint32_t kMaxBwdBlocks = 768;

uint32_t bwd_blocks(const NormPlan& p, uint64_t rows, uint32_t resident) {
    const uint64_t want = (rows + p.rpb - 1) / p.rpb;
    const uint64_t cap = resident && resident < kMaxBwdBlocks ? resident : kMaxBwdBlocks;
    return (uint32_t)(want < cap ? (want ? want : 1) : cap);
}

uint32_t cu_count() {
    static const uint32_t value = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess) return 0u;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0u;
        return (uint32_t)(n > 0 ? n : 0);
    }();
    return value;
}

template <int TPR>
inline size_t bwd_dyn_lds(const NormPlan& p, uint32_t C) {
    constexpr int BLOCK = TPR >= 128 ? TPR : kBwdGroupBlock;
    return p.rpb > 1 ? (size_t)(BLOCK / kWave - 1) * C * sizeof(float) : 0;
}

template <typename T, int VEC, int NV, int TPR>
void fwd_launch(hipStream_t s, const NormFwdArgs<T>& a, uint32_t grid) {
    constexpr int BLOCK = TPR >= 128 ? TPR : kFwdGroupBlock;
    const bool res = a.res != nullptr;
    // which parameters: none, gamma alone, or the two-parameter kernel (which also takes beta alone)
    const int params = a.gamma == nullptr && a.beta == nullptr ? 0 : a.beta == nullptr ? 1 : 2;
#define AGRAD_FWD(KIND, RES, PARAMS) \
    hipLaunchKernelGGL((norm_fwd_kernel<T, VEC, NV, TPR, KIND, RES, PARAMS>), dim3(grid), dim3(BLOCK), 0, s, a)
#define AGRAD_FWD_KIND(KIND)                                                                          \
    switch (params) {                                                                                 \
        case 0: if (res) AGRAD_FWD(KIND, true, 0); else AGRAD_FWD(KIND, false, 0); break;             \
        case 1: if (res) AGRAD_FWD(KIND, true, 1); else AGRAD_FWD(KIND, false, 1); break;             \
        default: if (res) AGRAD_FWD(KIND, true, 2); else AGRAD_FWD(KIND, false, 2); break;            \
    }
    if (a.kind == AGRAD_NORM_LAYER) { AGRAD_FWD_KIND(AGRAD_NORM_LAYER) } else { AGRAD_FWD_KIND(AGRAD_NORM_RMS) }
#undef AGRAD_FWD_KIND
#undef AGRAD_FWD
}

// Which (lanes per row, vectors per lane) pairs plan_norm can choose: it takes the fewest
// lanes whose share fits, so a wider group is only ever chosen with more than half of the
// largest share (a narrower group would have fitted otherwise) -- except the narrowest and
// the widest group, which take what is left below and above.
constexpr bool norm_shape_reachable(int tpr, int nv, int max_nv) {
    return nv <= max_nv && (tpr == 16 || tpr == 1024 || 2 * nv > max_nv);
}

template <typename T, int VEC, int TPR>
int fwd_pick_nv(hipStream_t s, const NormPlan& p, const NormFwdArgs<T>& a) {
    const uint32_t grid = (uint32_t)((a.rows + p.rpb - 1) / p.rpb);
    switch (p.nv) {
#define AGRAD_CASE(N)                                                                  \
    case N:                                                                            \
        if constexpr (norm_shape_reachable(TPR, N, kMaxEPT / VEC)) {                   \
            fwd_launch<T, VEC, N, TPR>(s, a, grid);                                    \
            return AGRAD_OK;                                                           \
        }                                                                              \
        break;
        AGRAD_CASE(1) AGRAD_CASE(2) AGRAD_CASE(3) AGRAD_CASE(4) AGRAD_CASE(5) AGRAD_CASE(6)
#undef AGRAD_CASE
    }
    return set_error(AGRAD_EINVAL, "norm forward: no kernel for nv=%d", p.nv);
}

// Which backward kernel: the flavour, the column sums it keeps and whether a residual
// gradient comes in.  LayerNorm keeps both sums or none (a frozen gamma or beta gets its
// partial rows written and not folded); RMSNorm keeps dgamma or none.
struct BwdVariant { int kind, sums; bool dres; };

// fn(kernel) for the instantiation that (T, VEC, NV, TPR, v) names
template <typename T, int VEC, int NV, int TPR, typename Fn>
void with_bwd_kernel(const BwdVariant& v, Fn&& fn) {
#define AGRAD_BWD(KIND, SUMS) \
    do { if (v.dres) fn(norm_bwd_kernel<T, VEC, NV, TPR, KIND, SUMS, true>); else fn(norm_bwd_kernel<T, VEC, NV, TPR, KIND, SUMS, false>); } while (0)
    if (v.kind == AGRAD_NORM_LAYER) { if (v.sums) AGRAD_BWD(AGRAD_NORM_LAYER, 2); else AGRAD_BWD(AGRAD_NORM_LAYER, 0); }
    else { if (v.sums) AGRAD_BWD(AGRAD_NORM_RMS, 1); else AGRAD_BWD(AGRAD_NORM_RMS, 0); }
#undef AGRAD_BWD
}

// fn(kernel, workgroup size, dynamic LDS bytes) for the kernel that (T, plan, v) names; false if there is none
template <typename T, typename Fn>
bool with_planned_bwd_kernel(const NormPlan& p, uint32_t C, const BwdVariant& v, Fn&& fn) {
    constexpr int VEC = WideVec<T>::value;
    constexpr int MAXNV = (sizeof(T) == 2 ? 24 : 16) / VEC;      // norm_max_ept(backward) / VEC
    bool found = false;
#define AGRAD_CASE(TPR, N)                                                                              \
    if constexpr (norm_shape_reachable(TPR, N, MAXNV)) {                                                \
        if (p.tpr == TPR && p.nv == N) {                                                                \
            constexpr int BLOCK = TPR >= 128 ? TPR : kBwdGroupBlock;                                    \
            with_bwd_kernel<T, VEC, N, TPR>(v, [&](auto kernel) { fn(kernel, BLOCK, bwd_dyn_lds<TPR>(p, C)); }); \
            found = true;                                                                               \
        }                                                                                               \
    }
#define AGRAD_TPR(TPR) AGRAD_CASE(TPR, 1) AGRAD_CASE(TPR, 2) AGRAD_CASE(TPR, 3) AGRAD_CASE(TPR, 4)
    AGRAD_TPR(16) AGRAD_TPR(32) AGRAD_TPR(64) AGRAD_TPR(128) AGRAD_TPR(256) AGRAD_TPR(1024)
#undef AGRAD_TPR
#undef AGRAD_CASE
    return found;
}

// workgroups of the chosen backward instantiation the GPU holds at once (0: unknown).
// Asked of the runtime once per instantiation and remembered.
uint32_t bwd_resident(const NormPlan& p, uint32_t C, int dtype, const BwdVariant& v) {
    if (p.generic) return 0;
    static std::mutex mu;
    static std::map<uint64_t, uint32_t> known;
    // (the dynamic LDS of the sub-wave geometries grows with C: part of the key)
    const uint64_t key = ((uint64_t)C << 32) | ((uint64_t)dtype << 24) | ((uint64_t)p.tpr << 8) | ((uint64_t)p.nv << 4) |
                         ((uint64_t)v.kind << 3) | ((uint64_t)v.sums << 1) | (v.dres ? 1u : 0u);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = known.find(key);
        if (it != known.end()) return it->second;
    }
    int per_cu = 0;
    auto ask = [&](auto kernel, int block, size_t dyn) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block, dyn) != hipSuccess) per_cu = 0;
    };
    const bool found = dtype == AGRAD_BF16 ? with_planned_bwd_kernel<bf16_t>(p, C, v, ask) : with_planned_bwd_kernel<float>(p, C, v, ask);
    if (!found || per_cu <= 0) { (void)hipGetLastError(); per_cu = 0; }
    const uint32_t resident = (uint32_t)per_cu * cu_count();
    std::lock_guard<std::mutex> lock(mu);
    known[key] = resident;
    return resident;
}

template <typename T>
int norm_fwd_typed(hipStream_t s, const NormPlan& p, const NormFwdArgs<T>& a) {
    constexpr int VEC = WideVec<T>::value;
    if (p.generic) {
        hipLaunchKernelGGL((norm_fwd_generic_kernel<T>), dim3((uint32_t)a.rows), dim3(256), 0, s, a);
        return AGRAD_OK;
    }
    switch (p.tpr) {
        case 16: return fwd_pick_nv<T, VEC, 16>(s, p, a);
        case 32: return fwd_pick_nv<T, VEC, 32>(s, p, a);
        case 64: return fwd_pick_nv<T, VEC, 64>(s, p, a);
        case 128: return fwd_pick_nv<T, VEC, 128>(s, p, a);
        case 256: return fwd_pick_nv<T, VEC, 256>(s, p, a);
        default: return fwd_pick_nv<T, VEC, 1024>(s, p, a);
    }
}

template <typename T>
int norm_bwd_typed(hipStream_t s, const NormPlan& p, const NormBwdArgs<T>& a, uint32_t grid, const BwdVariant& v) {
    if (p.generic) {
        hipLaunchKernelGGL((norm_bwd_generic_kernel<T>), dim3(grid), dim3(256), 0, s, a);
        return AGRAD_OK;
    }
    const bool found = with_planned_bwd_kernel<T>(p, a.C, v, [&](auto kernel, int block, size_t dyn) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), dyn, s, a);
    });
    if (!found) return set_error(AGRAD_EINVAL, "norm backward: no kernel for %d lanes x %d vectors", p.tpr, p.nv);
    return AGRAD_OK;
}

}  // namespace

// Where finalize launches go while a caller collects them (see ColsumDefer in launch.hpp).
static thread_local std::vector<ColsumJob>* g_colsum_sink = nullptr;
ColsumDefer::ColsumDefer(std::vector<ColsumJob>* sink) : prev_(g_colsum_sink) { if (sink) g_colsum_sink = sink; }
ColsumDefer::~ColsumDefer() { g_colsum_sink = prev_; }

static bool colsum_job_vec4(const ColsumJob& j) {
    return j.C % 4 == 0 && (!j.out_a || aligned16(j.out_a)) && (!j.out_b || aligned16(j.out_b)) &&
           (!j.pa || aligned16(j.pa)) && (!j.pb || aligned16(j.pb));
}

int launch_colsum_finalize(hipStream_t s, const float* pa, const float* pb, uint32_t P, uint32_t C,
                           float* out_a, float* out_b, int accumulate, bool out_bf16) {
    if (g_colsum_sink != nullptr) {
        // left pending: the caller folds it later, together with others (launch_colsum_finalize_many)
        g_colsum_sink->push_back(ColsumJob{pa, pb, out_a, out_b, P, C, accumulate ? 1u : 0u, out_bf16 ? 1u : 0u});
        return AGRAD_OK;
    }
    const ColsumJob j{pa, pb, out_a, out_b, P, C, 0, 0};
    if (colsum_job_vec4(j))
        hipLaunchKernelGGL((colsum_finalize_kernel<4>), dim3((C / 4 + kFinalizeCols - 1) / kFinalizeCols, 2), dim3(kFinalizeCols * kFinalizeLanes), 0, s, pa, pb, P, C,
                           out_a, out_b, accumulate, out_bf16 ? 1 : 0);
    else
        hipLaunchKernelGGL((colsum_finalize_kernel<1>), dim3((C + kFinalizeCols - 1) / kFinalizeCols, 2), dim3(kFinalizeCols * kFinalizeLanes), 0, s, pa, pb, P, C,
                           out_a, out_b, accumulate, out_bf16 ? 1 : 0);
    return check_hip(hipGetLastError(), "column-sum finalize launch");
}

// do the destination rows a (of job ja) and b (of job jb) share bytes?
static bool outputs_overlap(const void* a, const ColsumJob& ja, const void* b, const ColsumJob& jb) {
    if (a == nullptr || b == nullptr) return false;
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    const uintptr_t an = (uintptr_t)ja.C * (ja.out_bf16 ? 2u : 4u), bn = (uintptr_t)jb.C * (jb.out_bf16 ? 2u : 4u);
    return a0 < b0 + bn && b0 < a0 + an;
}

int launch_colsum_finalize_many(hipStream_t s, const ColsumJob* jobs, size_t n) {
    // The jobs are taken in order and share a launch while they can: up to kFinalizeManyJobs of
    // one column width (float4 or scalar) whose destinations are all different.  A job that
    // writes where an earlier job of the batch writes (a gamma tied between two norms: one stores,
    // the other adds) starts a new launch, so that the two happen in the callers' order.
    ColsumJobs batch;
    uint32_t count = 0, widest = 0;
    int batch_vec4 = 1;
    auto flush = [&]() -> int {
        if (count == 0) return AGRAD_OK;
        const uint32_t w = batch_vec4 ? 4u : 1u;
        const dim3 grid(((widest + w - 1) / w + kFinalizeCols - 1) / kFinalizeCols, 2, count);
        if (batch_vec4) hipLaunchKernelGGL((colsum_finalize_many_kernel<4>), grid, dim3(kFinalizeCols * kFinalizeLanes), 0, s, batch);
        else hipLaunchKernelGGL((colsum_finalize_many_kernel<1>), grid, dim3(kFinalizeCols * kFinalizeLanes), 0, s, batch);
        count = 0;
        widest = 0;
        return check_hip(hipGetLastError(), "batched column-sum finalize launch");
    };
    for (size_t i = 0; i < n; ++i) {
        const ColsumJob& j = jobs[i];
        if (j.C == 0 || j.P == 0 || (j.pa == nullptr && j.pb == nullptr)) continue;
        const int vec4 = colsum_job_vec4(j) ? 1 : 0;
        bool clash = count == (uint32_t)kFinalizeManyJobs || (count != 0 && vec4 != batch_vec4);
        for (uint32_t k = 0; k < count && !clash; ++k) {
            const ColsumJob& o = batch.job[k];
            clash = outputs_overlap(j.out_a, j, o.out_a, o) || outputs_overlap(j.out_a, j, o.out_b, o) ||
                    outputs_overlap(j.out_b, j, o.out_a, o) || outputs_overlap(j.out_b, j, o.out_b, o);
        }
        if (clash) if (int rc = flush()) return rc;
        batch_vec4 = vec4;
        batch.job[count++] = j;
        widest = j.C > widest ? j.C : widest;
    }
    return flush();
}

uint64_t norm_bwd_workspace_bytes(uint64_t rows, uint32_t C, int dtype) {
    // sized for the largest grid any kernel of this shape runs with: the scalar geometry, and
    // the register-resident one in each of its flavours that keeps column sums
    NormPlan vecp = plan_norm(C, dtype, true, true);
    NormPlan genp{true, 256, 0, 1};
    uint64_t blocks = bwd_blocks(genp, rows, 0);
    if (!vecp.generic) {
        for (int kind : {AGRAD_NORM_LAYER, AGRAD_NORM_RMS})
            for (int dres = 0; dres < 2; ++dres) {
                const BwdVariant v{kind, kind == AGRAD_NORM_LAYER ? 2 : 1, dres != 0};
                const uint64_t b = bwd_blocks(vecp, rows, bwd_resident(vecp, C, dtype, v));
                if (b > blocks) blocks = b;
            }
    }
    return 2ull * blocks * C * sizeof(float);
}

int launch_norm_fwd(hipStream_t s, int kind, int dtype, const void* x, const void* residual,
                    const float* gamma, const float* beta, void* h_out, void* y,
                    uint64_t rows, uint32_t C, float eps) {
    if (kind != AGRAD_NORM_LAYER && kind != AGRAD_NORM_RMS)
        return set_error(AGRAD_EINVAL, "norm forward: unknown kind %d", kind);
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16)
        return set_error(AGRAD_EINVAL, "norm forward: unknown dtype %d", dtype);
    if (rows == 0 || C == 0) return AGRAD_OK;
    if (x == nullptr || y == nullptr) return set_error(AGRAD_EINVAL, "norm forward: null x or y");
    if (rows > 0x7fffffffull) return set_error(AGRAD_EINVAL, "norm forward: too many rows");
    const bool aligned = aligned16(x) && aligned16(y) && (!residual || aligned16(residual)) &&
                         (!h_out || aligned16(h_out)) && (!gamma || aligned16(gamma)) &&
                         (!beta || aligned16(beta));
    const NormPlan p = plan_norm(C, dtype, aligned, false);
    if (dtype == AGRAD_F32) {
        NormFwdArgs<float> a{(const float*)x, (const float*)residual, gamma, beta, (float*)h_out,
                             (float*)y, rows, C, eps, kind};
        return norm_fwd_typed<float>(s, p, a);
    }
    NormFwdArgs<bf16_t> a{(const bf16_t*)x, (const bf16_t*)residual, gamma, beta, (bf16_t*)h_out,
                          (bf16_t*)y, rows, C, eps, kind};
    return norm_fwd_typed<bf16_t>(s, p, a);
}

int launch_norm_bwd(hipStream_t s, int kind, int dtype, const void* x, const void* dy,
                    const float* gamma, const void* dres_in, void* dx, void* dx2,
                    float* dgamma, float* dbeta, void* workspace, uint64_t workspace_bytes,
                    uint64_t rows, uint32_t C, float eps, uint32_t flags) {
    if (kind != AGRAD_NORM_LAYER && kind != AGRAD_NORM_RMS)
        return set_error(AGRAD_EINVAL, "norm backward: unknown kind %d", kind);
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16)
        return set_error(AGRAD_EINVAL, "norm backward: unknown dtype %d", dtype);
    if (C == 0) return AGRAD_OK;
    if (x == nullptr || dy == nullptr) return set_error(AGRAD_EINVAL, "norm backward: null x or dy");
    if (dx == nullptr && dx2 != nullptr) return set_error(AGRAD_EINVAL, "norm backward: dx2 without dx");
    if (dx == nullptr && dgamma == nullptr && dbeta == nullptr) return AGRAD_OK;
    if (rows > 0x7fffffffull) return set_error(AGRAD_EINVAL, "norm backward: too many rows");
    const bool aligned = aligned16(x) && aligned16(dy) && (!dres_in || aligned16(dres_in)) &&
                         (!dx || aligned16(dx)) && (!dx2 || aligned16(dx2)) &&
                         (!gamma || aligned16(gamma));
    NormPlan p = plan_norm(C, dtype, aligned, true);
    const bool want_params = dgamma != nullptr || dbeta != nullptr;
    // an RMSNorm has no beta: a caller that asks for sum(dy) under one takes the scalar kernel
    if (kind == AGRAD_NORM_RMS && dbeta != nullptr) p = NormPlan{true, 256, 0, 1};
    const BwdVariant variant{kind, !want_params ? 0 : kind == AGRAD_NORM_LAYER ? 2 : 1, dres_in != nullptr};
    const uint32_t grid = bwd_blocks(p, rows, bwd_resident(p, C, dtype, variant));
    if (rows == 0) {
        // nothing to add: stored parameter grads become zero, accumulated ones stay
        if (want_params && !(flags & AGRAD_ACC_PARAM_GRAD)) {
            const int gsize = (flags & AGRAD_PARAM_GRAD_BF16) ? 2 : 4;
            if (dgamma) if (int rc = launch_fill(s, dgamma, 0, gsize, C)) return rc;
            if (dbeta) if (int rc = launch_fill(s, dbeta, 0, gsize, C)) return rc;
        }
        return AGRAD_OK;
    }
    float *pg = nullptr, *pb = nullptr;
    if (want_params) {
        const uint64_t need = 2ull * grid * C * sizeof(float);
        if (workspace == nullptr || workspace_bytes < need)
            return set_error(AGRAD_EWORKSPACE, "norm backward: workspace %llu < %llu bytes",
                             (unsigned long long)workspace_bytes, (unsigned long long)need);
        if (!aligned16(workspace)) return set_error(AGRAD_EINVAL, "norm backward: workspace must be 16-byte aligned");
        float* w = (float*)workspace;
        // the register-resident LayerNorm kernel keeps both sums whichever are asked for (the
        // other's partial rows are written and not folded); the scalar kernel keeps what it is given
        if (dgamma || (!p.generic && variant.sums == 2)) pg = w;
        if (dbeta || (!p.generic && variant.sums == 2)) pb = w + (uint64_t)grid * C;
    }
    int rc;
    if (dtype == AGRAD_F32) {
        NormBwdArgs<float> a{(const float*)x, (const float*)dy, gamma, (const float*)dres_in,
                             (float*)dx, (float*)dx2, pg, pb, rows, C, eps, kind, flags};
        rc = norm_bwd_typed<float>(s, p, a, grid, variant);
    } else {
        NormBwdArgs<bf16_t> a{(const bf16_t*)x, (const bf16_t*)dy, gamma, (const bf16_t*)dres_in,
                              (bf16_t*)dx, (bf16_t*)dx2, pg, pb, rows, C, eps, kind, flags};
        rc = norm_bwd_typed<bf16_t>(s, p, a, grid, variant);
    }
    if (rc != AGRAD_OK) return rc;
    if (want_params)
        return launch_colsum_finalize(s, dgamma ? pg : nullptr, dbeta ? pb : nullptr, grid, C, dgamma, dbeta,
                                      (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0, (flags & AGRAD_PARAM_GRAD_BF16) != 0);
    return check_hip(hipGetLastError(), "norm backward launch");
}

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each GPU
hipStream_t g_scratch_stream[kMaxDevices] = {};   // the stream whose call used it last
bool g_scratch_used[kMaxDevices] = {};
}  // namespace

// Called by agrad_ctx_create with `device` current: looks up, once per GPU, where
// that GPU keeps its copy of `scratch`.
int norm_noalloc_setup(int device) {
    if (device < 0 || device >= kMaxDevices)
        return set_error(AGRAD_EINVAL, "device %d beyond the %d the scratch table covers", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[device] != nullptr) return AGRAD_OK;
    void* ptr = nullptr;
    if (int rc = check_hip(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"))
        return rc;
    if (ptr == nullptr) return set_error(AGRAD_EHIP, "hipGetSymbolAddress(scratch) returned no address");
    g_scratch_ptr[device] = ptr;
    return AGRAD_OK;
}

// launch_norm_bwd with the partial rows in this GPU's `scratch`.  Every partial row
// the finalize kernel reads is written by the backward kernel of the same call, so
// nothing has to be cleared between calls; two calls in flight on one GPU (two
// streams, two contexts) would overwrite each other's rows.
int launch_norm_bwd_noalloc(hipStream_t s, int device, int kind, int dtype, const void* x, const void* dy,
                            const float* gamma, const void* dres_in, void* dx, void* dx2,
                            float* dgamma, float* dbeta, uint64_t rows, uint32_t C, float eps, uint32_t flags) {
    void* ptr = nullptr;
    if (device >= 0 && device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        ptr = g_scratch_ptr[device];
        // Calls on one stream follow one another; a call from ANOTHER stream (another context)
        // while the last user's work may still be running would overwrite its partial rows.
        if (ptr != nullptr && (dgamma != nullptr || dbeta != nullptr)) {
            if (g_scratch_used[device] && g_scratch_stream[device] != s && !is_capturing()) {
                const hipError_t busy = hipStreamQuery(g_scratch_stream[device]);
                if (busy == hipErrorNotReady)
                    return set_error(AGRAD_EINVAL, "norm backward (no allocation): the fixed scratch of device %d is still in "
                                     "use by work on another stream; synchronise that stream first", device);
                (void)hipGetLastError();        // (a stream that no longer exists has nothing in flight)
            }
            g_scratch_used[device] = true;
            g_scratch_stream[device] = s;
        }
    }
    if (ptr == nullptr) return set_error(AGRAD_EINVAL, "norm backward (no allocation): device %d was never set up", device);
    if ((dgamma != nullptr || dbeta != nullptr) && rows > 0 && C > 0) {
        if (dtype != AGRAD_F32 && dtype != AGRAD_BF16)
            return set_error(AGRAD_EINVAL, "norm backward: unknown dtype %d", dtype);
        const uint64_t need = norm_bwd_workspace_bytes(rows, C, dtype);
        if (need > AGRAD_NOALLOC_SCRATCH_BYTES)
            return set_error(AGRAD_EINVAL,
                             "norm backward (no allocation): rows=%llu C=%u need %llu bytes of partial rows, the fixed "
                             "scratch holds %llu; use agrad_norm_backward with a workspace",
                             (unsigned long long)rows, C, (unsigned long long)need,
                             (unsigned long long)AGRAD_NOALLOC_SCRATCH_BYTES);
    }
    return launch_norm_bwd(s, kind, dtype, x, dy, gamma, dres_in, dx, dx2, dgamma, dbeta, ptr,
                           AGRAD_NOALLOC_SCRATCH_BYTES, rows, C, eps, flags);
}

}  // namespace agrad
