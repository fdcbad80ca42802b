// Strided gather into a dense tensor: dst[dense index over shape] (+)=
// src[sum_i coord_i * stride_i].  One kernel family serves Contiguous forward
// (a permuted / transposed view made dense) and the Permute / Transpose
// gradients (x.grad += the inverse permutation of out.grad), which the
// reference runs as contiguous_forward_kernel and strided_add_backward_kernel
// (metal_ops.metal:429-449, 1002-1023; cpu_permute_backward, cpu_transpose_backward,
// cpu_contiguous_forward, backend.py:286-313): one thread per element, a div/mod
// chain per dimension, 4-byte accesses.
//
// Here the host first simplifies the index space (drops extent-1 dimensions, merges
// neighbours that walk memory like one dimension) and then picks one of two kernels:
//   * rows:  the source is contiguous along the innermost dense dimension (a
//     [B,T,H,D] <-> [B,H,T,D] layout change): a thread moves one 16-byte vector;
//     the div/mod chain runs once per vector over the remaining dimensions;
//   * tiles: the unit-stride source dimension is another one (a true transpose):
//     256-byte-square tiles (64x64 fp32, 128x128 bf16) go through LDS so that both the reads (along the source's
//     contiguous dimension) and the writes (along the destination's) are
//     coalesced 16-byte accesses; the other dimensions enumerate tiles.  2-byte
//     elements travel through LDS as 32-bit words of two destination neighbours;
// A source with no unit-stride dimension, or extents that do not divide into
// vectors, takes the same kernels with one element per access.
//
// Overwriting moves raw bits (any 2- or 4-byte element type); accumulating adds in
// fp32 and rounds once for bf16 storage.
#include "common.hpp"
#include "launch.hpp"

namespace agrad {

namespace {

constexpr int kMaxDims = AGRAD_MAX_DIMS;
constexpr int kRowsBlock = 64;
constexpr int kTileBlock = 256;
constexpr uint32_t kXcds = 8;           // accelerator dies of the GPU; workgroups are dealt to them round-robin
// tile edge in elements: 256 bytes along either contiguous dimension
template <int ES> struct TileOf { static constexpr int value = 256 / ES; };

struct Dims {
    uint32_t n;
    uint32_t size[kMaxDims];      // outermost first; in the rows kernel the innermost is in vectors
    uint64_t stride[kMaxDims];    // source stride in elements
};

// raw element / vector types by element size
template <int ES> struct Elem;
template <> struct Elem<4> { typedef uint32_t type; };
template <> struct Elem<2> { typedef uint16_t type; };

template <int ES> __device__ __forceinline__ float elem_to_f32(typename Elem<ES>::type b) {
    if constexpr (ES == 4) return __uint_as_float(b);
    else return bf16_bits_to_f32(b);
}
template <int ES> __device__ __forceinline__ typename Elem<ES>::type f32_to_elem(float f) {
    if constexpr (ES == 4) return __float_as_uint(f);
    else return (uint16_t)f32_to_bf16_bits(f);
}
template <int ES> __device__ __forceinline__ typename Elem<ES>::type add_elem(typename Elem<ES>::type a,
                                                                             typename Elem<ES>::type b) {
    return f32_to_elem<ES>(elem_to_f32<ES>(a) + elem_to_f32<ES>(b));
}

// 16-byte vector of ES-byte elements: dst (+)= src
template <int ES>
__device__ __forceinline__ u32x4 add_vec(const u32x4& d, const u32x4& s) {
    const uint32_t dw[4] = {d.x, d.y, d.z, d.w}, sw[4] = {s.x, s.y, s.z, s.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (ES == 4) {
            o[i] = __float_as_uint(__uint_as_float(dw[i]) + __uint_as_float(sw[i]));
        } else {
            const float lo = __uint_as_float(dw[i] << 16) + __uint_as_float(sw[i] << 16);
            const float hi = __uint_as_float(dw[i] & 0xffff0000u) + __uint_as_float(sw[i] & 0xffff0000u);
            o[i] = pack_bf16x2(lo, hi);
        }
    }
    return u32x4{o[0], o[1], o[2], o[3]};
}

// ---- rows: VEC elements per thread along the innermost dimension ----------------
template <int ES, int VEC>
__global__ void __launch_bounds__(kRowsBlock)
strided_rows_kernel(const typename Elem<ES>::type* __restrict__ src, typename Elem<ES>::type* dst, Dims d,
                    uint32_t total, int accumulate) {
    const uint32_t idx = blockIdx.x * kRowsBlock + threadIdx.x;
    if (idx >= total) return;
    uint32_t rem = idx;
    uint64_t off = 0;
#pragma unroll
    for (int i = kMaxDims - 1; i >= 0; --i) {
        if (i < (int)d.n) {
            const uint32_t q = rem / d.size[i];
            off += (uint64_t)(rem - q * d.size[i]) * d.stride[i];
            rem = q;
        }
    }
    if constexpr (VEC == 1) {
        typename Elem<ES>::type v = __builtin_nontemporal_load(src + off);
        if (accumulate) v = add_elem<ES>(dst[idx], v);
        __builtin_nontemporal_store(v, dst + idx);
    } else {
        u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + off));
        u32x4* out = reinterpret_cast<u32x4*>(dst + (uint64_t)idx * VEC);
        if (accumulate) v = add_vec<ES>(__builtin_nontemporal_load(out), v);
        __builtin_nontemporal_store(v, out);
    }
}

// ---- tiles ---------------------------------------------------------------------
// The dense destination has its innermost dimension I (extent ni, source stride
// si != 1); the source is contiguous along dimension J (extent nj, dense
// destination stride dj).  d lists the remaining ("batch") dimensions with their
// source strides; bstride_dst holds their dense destination strides.
struct TileGeom {
    uint32_t ni, nj, tiles_i, tiles_j;
    uint32_t tiles, per_xcd;      // all tiles; tiles per XCD (the grid is 8 * per_xcd workgroups)
    uint64_t si;                  // source stride of I
    uint64_t dj;                  // destination stride of J
    uint64_t bstride_dst[kMaxDims];
};

template <int ES, int VEC>
__global__ void __launch_bounds__(kTileBlock)
strided_tile_kernel(const typename Elem<ES>::type* __restrict__ src, typename Elem<ES>::type* dst, Dims d,
                    TileGeom g, int accumulate) {
    typedef typename Elem<ES>::type E;
    constexpr int kTile = TileOf<ES>::value;
    // one padding word per row keeps the column reads of the second phase off one bank
    constexpr int kPitch = kTile + (ES == 4 ? 1 : 2);
    __shared__ E tile[kTile][kPitch];

    // Workgroups go to the eight XCDs in turn, each with an L2 of its own: workgroup b takes
    // tile (b % 8) * per_xcd + b / 8, so that the tiles one L2 sees one after the other are
    // neighbours in the destination and their 256-byte pieces of a row leave it together.
    uint32_t rem = (blockIdx.x % kXcds) * g.per_xcd + blockIdx.x / kXcds;
    if (rem >= g.tiles) return;
    const uint32_t ti = rem % g.tiles_i; rem /= g.tiles_i;
    const uint32_t tj = rem % g.tiles_j; rem /= g.tiles_j;
    uint64_t src_base = 0, dst_base = 0;
#pragma unroll
    for (int i = kMaxDims - 1; i >= 0; --i) {
        if (i < (int)d.n) {
            const uint32_t q = rem / d.size[i];
            const uint32_t c = rem - q * d.size[i];
            src_base += (uint64_t)c * d.stride[i];
            dst_base += (uint64_t)c * g.bstride_dst[i];
            rem = q;
        }
    }
    const uint32_t i0 = ti * kTile, j0 = tj * kTile;
    constexpr int kLanesPerRow = kTile / VEC;              // lanes that cover one tile row
    constexpr int kRowsPerPass = kTileBlock / kLanesPerRow;
    const uint32_t lane = threadIdx.x % kLanesPerRow;
    const uint32_t row = threadIdx.x / kLanesPerRow;

    // phase 1: read along J (the source's contiguous dimension); tile[i][j]
#pragma unroll
    for (int r0 = 0; r0 < kTile; r0 += kRowsPerPass) {
        const uint32_t i = r0 + row, j = lane * VEC;
        if (i0 + i < g.ni && j0 + j < g.nj) {
            const E* p = src + src_base + (uint64_t)(i0 + i) * g.si + (j0 + j);
            if constexpr (VEC == 1) {
                tile[i][j] = __builtin_nontemporal_load(p);
            } else {
                const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    if constexpr (ES == 4) tile[i][j + k] = w[k];
                    else tile[i][j + k] = (uint16_t)(w[k / 2] >> ((k & 1) * 16));
                }
            }
        }
    }
    __syncthreads();
    // phase 2: write along I (the destination's contiguous dimension)
#pragma unroll
    for (int r0 = 0; r0 < kTile; r0 += kRowsPerPass) {
        const uint32_t j = r0 + row, i = lane * VEC;
        if (j0 + j < g.nj && i0 + i < g.ni) {
            E* p = dst + dst_base + (uint64_t)(j0 + j) * g.dj + (i0 + i);
            if constexpr (VEC == 1) {
                E v = tile[i][j];
                if (accumulate) v = add_elem<ES>(*p, v);
                __builtin_nontemporal_store(v, p);
            } else {
                uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    if constexpr (ES == 4) w[k] = tile[i + k][j];
                    else w[k / 2] |= (uint32_t)tile[i + k][j] << ((k & 1) * 16);
                }
                u32x4 v = {w[0], w[1], w[2], w[3]};
                u32x4* out = reinterpret_cast<u32x4*>(p);
                if (accumulate) v = add_vec<ES>(__builtin_nontemporal_load(out), v);
                __builtin_nontemporal_store(v, out);
            }
        }
    }
}

// 2-byte elements, vector path: the same 128 x 128 tile moved as 32-bit WORDS.  A thread
// reads the same eight columns of two neighbouring source rows i, i + 1 and pairs them up
// column by column (one byte-permute each), so that a word already holds two elements
// that are neighbours in the DESTINATION; the tile is stored transposed, word (j, i/2), and
// phase 2 reads four words (eight elements along I) with one 16-byte LDS access.  Ten LDS
// accesses per pair of vectors where the element-wise tile takes thirty-two.  Groups of
// four words are XOR-swizzled with the tile row (j / 8), which spreads both phases over
// all 64 banks without padding (32 KB a tile).
__global__ void __launch_bounds__(kTileBlock)
transpose_pairs16_kernel(const uint16_t* __restrict__ src, uint16_t* dst, Dims d, TileGeom g, int accumulate) {
    constexpr int kTile = 128, kWords = kTile / 2;          // words along I in a tile row
    __shared__ __attribute__((aligned(16))) uint32_t tile[kTile][kWords];

    // Workgroups go to the eight XCDs in turn, each with an L2 of its own: workgroup b takes
    // tile (b % 8) * per_xcd + b / 8, so that the tiles one L2 sees one after the other are
    // neighbours in the destination and their 256-byte pieces of a row leave it together.
    uint32_t rem = (blockIdx.x % kXcds) * g.per_xcd + blockIdx.x / kXcds;
    if (rem >= g.tiles) return;
    const uint32_t ti = rem % g.tiles_i; rem /= g.tiles_i;
    const uint32_t tj = rem % g.tiles_j; rem /= g.tiles_j;
    uint64_t src_base = 0, dst_base = 0;
#pragma unroll
    for (int i = kMaxDims - 1; i >= 0; --i) {
        if (i < (int)d.n) {
            const uint32_t q = rem / d.size[i];
            const uint32_t c = rem - q * d.size[i];
            src_base += (uint64_t)c * d.stride[i];
            dst_base += (uint64_t)c * g.bstride_dst[i];
            rem = q;
        }
    }
    const uint32_t i0 = ti * kTile, j0 = tj * kTile;
    const uint32_t lane = threadIdx.x % 16;                 // which vector of a 128-element row
    const uint32_t row = threadIdx.x / 16;                  // 16 rows (row pairs) per pass

    // phase 1: rows i, i + 1 of the source, eight columns each
    u32x4 lo[4], hi[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const uint32_t i = (pass * 16 + row) * 2, j = lane * 8;
        lo[pass] = u32x4{0u, 0u, 0u, 0u};
        hi[pass] = u32x4{0u, 0u, 0u, 0u};
        if (i0 + i < g.ni && j0 + j < g.nj) {               // (extents are multiples of 8: row i + 1 exists)
            const uint16_t* p = src + src_base + (uint64_t)(i0 + i) * g.si + (j0 + j);
            lo[pass] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
            hi[pass] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + g.si));
        }
    }
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const uint32_t ip = pass * 16 + row;                // the row pair: word column of the transposed tile
        const uint32_t a[4] = {lo[pass].x, lo[pass].y, lo[pass].z, lo[pass].w};
        const uint32_t b[4] = {hi[pass].x, hi[pass].y, hi[pass].z, hi[pass].w};
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            // element k of row i in the low half, of row i + 1 in the high half
            const uint32_t word = (k & 1) ? __builtin_amdgcn_perm(b[k / 2], a[k / 2], 0x07060302u)
                                          : __builtin_amdgcn_perm(b[k / 2], a[k / 2], 0x05040100u);
            const uint32_t jj = lane * 8 + k;
            tile[jj][(((ip >> 2) ^ (jj >> 3)) & 15u) * 4u + (ip & 3u)] = word;
        }
    }
    __syncthreads();
    // phase 2: a destination row j, eight elements along I per thread
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
        const uint32_t j = pass * 16 + row, i = lane * 8;
        if (j0 + j < g.nj && i0 + i < g.ni) {
            u32x4 v = *reinterpret_cast<const u32x4*>(&tile[j][((lane ^ (j >> 3)) & 15u) * 4u]);
            u32x4* out = reinterpret_cast<u32x4*>(dst + dst_base + (uint64_t)(j0 + j) * g.dj + (i0 + i));
            if (accumulate) v = add_vec<2>(__builtin_nontemporal_load(out), v);
            __builtin_nontemporal_store(v, out);
        }
    }
}

// The dense index space with extent-1 dimensions dropped and neighbours merged
// where the source walks them like one dimension.
struct Simplified {
    int n;
    uint64_t size[AGRAD_MAX_DIMS];
    uint64_t stride[AGRAD_MAX_DIMS];
};

void simplify(int ndim, const uint32_t* shape, const uint64_t* strides, Simplified* s) {
    s->n = 0;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] == 1) continue;
        if (s->n > 0 && s->stride[s->n - 1] == strides[i] * shape[i]) {
            s->size[s->n - 1] *= shape[i];
            s->stride[s->n - 1] = strides[i];
        } else {
            s->size[s->n] = shape[i];
            s->stride[s->n] = strides[i];
            ++s->n;
        }
    }
    if (s->n == 0) {           // a single element
        s->size[0] = 1;
        s->stride[0] = 1;
        s->n = 1;
    }
}

template <int ES>
int strided_typed(hipStream_t st, const void* src_v, void* dst_v, const Simplified& s, uint64_t numel, int acc) {
    typedef typename Elem<ES>::type E;
    const E* src = (const E*)src_v;
    E* dst = (E*)dst_v;
    constexpr int WIDE = 16 / ES;
    const int n = s.n;
    const bool ptrs16 = aligned16(src) && aligned16(dst);

    if (s.stride[n - 1] != 1) {
        // a transpose: is there a source-contiguous dimension to tile against?
        int J = -1;
        for (int i = n - 2; i >= 0; --i)
            if (s.stride[i] == 1) { J = i; break; }
        if (J >= 0) {
            constexpr int kTile = TileOf<ES>::value;
            TileGeom g;
            Dims d;
            uint64_t dense[AGRAD_MAX_DIMS];
            dense[n - 1] = 1;
            for (int i = n - 2; i >= 0; --i) dense[i] = dense[i + 1] * s.size[i + 1];
            g.ni = (uint32_t)s.size[n - 1];
            g.nj = (uint32_t)s.size[J];
            g.si = s.stride[n - 1];
            g.dj = dense[J];
            g.tiles_i = (g.ni + kTile - 1) / kTile;
            g.tiles_j = (g.nj + kTile - 1) / kTile;
            d.n = 0;
            uint64_t blocks = (uint64_t)g.tiles_i * g.tiles_j;
            bool vec = ptrs16 && g.ni % WIDE == 0 && g.nj % WIDE == 0 && g.si % WIDE == 0 && g.dj % WIDE == 0;
            for (int i = 0; i < n - 1; ++i) {
                if (i == J) continue;
                d.size[d.n] = (uint32_t)s.size[i];
                d.stride[d.n] = s.stride[i];
                g.bstride_dst[d.n] = dense[i];
                vec = vec && s.stride[i] % WIDE == 0 && dense[i] % WIDE == 0;
                blocks *= s.size[i];
                ++d.n;
            }
            for (int i = d.n; i < kMaxDims; ++i) { d.size[i] = 1; d.stride[i] = 0; g.bstride_dst[i] = 0; }
            if (blocks > 0x7ffffff0ull) return set_error(AGRAD_EINVAL, "strided copy: too many tiles");
            g.tiles = (uint32_t)blocks;
            g.per_xcd = (uint32_t)((blocks + kXcds - 1) / kXcds);
            blocks = (uint64_t)g.per_xcd * kXcds;
            if constexpr (ES == 2) {
                if (vec) {
                    hipLaunchKernelGGL(transpose_pairs16_kernel, dim3((uint32_t)blocks), dim3(kTileBlock), 0, st,
                                       src, dst, d, g, acc);
                    return check_hip(hipGetLastError(), "strided copy launch");
                }
            }
            if (vec)
                hipLaunchKernelGGL((strided_tile_kernel<ES, WIDE>), dim3((uint32_t)blocks), dim3(kTileBlock), 0, st,
                                   src, dst, d, g, acc);
            else
                hipLaunchKernelGGL((strided_tile_kernel<ES, 1>), dim3((uint32_t)blocks), dim3(kTileBlock), 0, st,
                                   src, dst, d, g, acc);
            return check_hip(hipGetLastError(), "strided copy launch");
        }
    }

    Dims d;
    d.n = (uint32_t)n;
    bool vec = ptrs16 && s.stride[n - 1] == 1 && s.size[n - 1] % WIDE == 0;
    for (int i = 0; i < n - 1; ++i) vec = vec && s.stride[i] % WIDE == 0;
    for (int i = 0; i < n; ++i) { d.size[i] = (uint32_t)s.size[i]; d.stride[i] = s.stride[i]; }
    for (int i = n; i < kMaxDims; ++i) { d.size[i] = 1; d.stride[i] = 0; }
    uint64_t total = numel;
    if (vec) {
        d.size[n - 1] = (uint32_t)(s.size[n - 1] / WIDE);
        d.stride[n - 1] = WIDE;
        total = numel / WIDE;
    }
    if (total > 0xffffff00ull) return set_error(AGRAD_EINVAL, "strided copy: %llu elements exceed one launch", (unsigned long long)numel);
    const uint32_t blocks = (uint32_t)((total + kRowsBlock - 1) / kRowsBlock);
    if (vec)
        hipLaunchKernelGGL((strided_rows_kernel<ES, WIDE>), dim3(blocks), dim3(kRowsBlock), 0, st, src, dst, d,
                           (uint32_t)total, acc);
    else
        hipLaunchKernelGGL((strided_rows_kernel<ES, 1>), dim3(blocks), dim3(kRowsBlock), 0, st, src, dst, d,
                           (uint32_t)total, acc);
    return check_hip(hipGetLastError(), "strided copy launch");
}

}  // namespace

uint64_t strided_extent(int ndim, const uint32_t* shape, const uint64_t* strides) {
    uint64_t last = 0;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] == 0) return 0;
        last += (uint64_t)(shape[i] - 1) * strides[i];
    }
    return last + 1;
}

int launch_strided_copy(hipStream_t s, int dtype, const void* src, void* dst, int ndim, const uint32_t* shape,
                        const uint64_t* strides, uint32_t flags) {
    if (ndim < 0 || ndim > AGRAD_MAX_DIMS) return set_error(AGRAD_EINVAL, "strided copy: %d dimensions (at most %d)", ndim, AGRAD_MAX_DIMS);
    if (ndim > 0 && (shape == nullptr || strides == nullptr)) return set_error(AGRAD_EINVAL, "strided copy: null shape");
    uint64_t numel = 1;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] != 0 && numel > 0xffffffffffffull / shape[i]) return set_error(AGRAD_EINVAL, "strided copy: shape too large");
        numel *= shape[i];
    }
    if (numel == 0) return AGRAD_OK;
    if (src == nullptr || dst == nullptr) return set_error(AGRAD_EINVAL, "strided copy: null operand");
    const uint32_t es = dtype_size(dtype);
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & (es - 1))
        return set_error(AGRAD_EINVAL, "strided copy: operand not aligned to its element size");
    Simplified sp;
    simplify(ndim, shape, strides, &sp);
    if (sp.n > kMaxDims) return set_error(AGRAD_EINVAL, "strided copy: %d independent dimensions (at most %d)", sp.n, kMaxDims);
    for (int i = 0; i < sp.n; ++i)
        if (sp.size[i] > 0xffffffffull) return set_error(AGRAD_EINVAL, "strided copy: a merged dimension exceeds 2^32");
    const int acc = (flags & AGRAD_ACC_INPUT_GRAD) ? 1 : 0;
    return es == 4 ? strided_typed<4>(s, src, dst, sp, numel, acc) : strided_typed<2>(s, src, dst, sp, numel, acc);
}

}  // namespace agrad
