// Token / position embedding: gather forward and the deterministic gradient.
//
// Forward  out[n,:] = W[ids[n],:] (+ wpe[n % T,:]) is a row copy with 128-bit
// accesses (cpu_gather_forward, backend.py:525-529).
//
// Backward dW[ids[n],:] += dY[n,:] (np.add.at, backend.py:531-538) is done
// without float atomics:
//   1. (token, row) pairs are ordered so that each token's rows form one run,
//      in ascending row order, and every row learns its place in that order.
//      Up to 65536 rows this is ONE launch: every workgroup owns a hash group of
//      tokens, scans all ids for its own, and orders its pairs in LDS (runs of
//      distinct tokens then follow hash-group order, which is all the next step
//      needs).  Larger inputs take a stable LSD radix sort by token (rocPRIM);
//   2. one launch reads dY once: a token's only row is moved by a wave of its own; the
//      rows of a run are added in ascending order by one wave per column block (the
//      ordering marks where runs start, and waves at the front of the grid look for
//      the marks); a long run (a frequent token) is cut into chunks of rows whose sums
//      pass through the workspace and are added in chunk order by the wave that an
//      arrival counter names the last of its group.  Every table row is written once.
// Every sum has a fixed order, so the result is run-to-run identical, and runs of
// up to 127 rows are bit-identical to the sequential CPU sum.
#include "common.hpp"
#include "launch.hpp"

#include <cstdlib>
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

namespace agrad {

namespace {

constexpr int kGatherBlock = 256;

inline uint64_t align256(uint64_t v) { return (v + 255) & ~255ull; }

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename T, int VEC, int UNROLL>
__global__ void __launch_bounds__(kGatherBlock)
gather_fwd_kernel(const int32_t* __restrict__ ids, const T* __restrict__ W, const T* __restrict__ wpe,
                  T* __restrict__ out, uint32_t total, uint32_t CV, uint32_t C, uint32_t T_len,
                  uint32_t V, int* err_flag) {
    const uint32_t first = blockIdx.x * (kGatherBlock * UNROLL) + threadIdx.x;
    int32_t tok[UNROLL];
    uint32_t rows[UNROLL], col[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kGatherBlock;
        tok[u] = -1;
        rows[u] = 0;
        col[u] = 0;
        if (idx < total) {
            rows[u] = idx / CV;
            col[u] = (idx - rows[u] * CV) * VEC;
            tok[u] = ids[rows[u]];
        }
    }
    float v[UNROLL][VEC], p[UNROLL][VEC];
    bool ok[UNROLL];
    // (the position rows do not wait for the ids: asked for first, from a valid row whatever the id)
    if (wpe != nullptr) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) VecIO<T, VEC>::load(wpe + (uint64_t)(rows[u] % T_len) * C + col[u], p[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kGatherBlock;
        ok[u] = idx < total && tok[u] >= 0 && (uint32_t)tok[u] < V;
        if (ok[u]) {
            VecIO<T, VEC>::load(W + (uint64_t)tok[u] * C + col[u], v[u]);
        } else if (idx < total && col[u] == 0) {
            *err_flag = 1;
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        if (ok[u]) {
            if (wpe != nullptr) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) v[u][k] = v[u][k] + p[u][k];
            }
            VecIO<T, VEC>::store(out + (uint64_t)rows[u] * C + col[u], v[u]);
        }
    }
}

// Bit-exact variant of the plain gather for bf16 / fp32: moves raw 16-byte
// words, so NaN payloads and -0.0 survive untouched.
template <int UNROLL>
__global__ void __launch_bounds__(kGatherBlock)
gather_rows16_kernel(const int32_t* __restrict__ ids, const u32x4* __restrict__ W,
                     u32x4* __restrict__ out, uint32_t total, uint32_t CV, uint32_t V, int* err_flag) {
    const uint32_t first = blockIdx.x * (kGatherBlock * UNROLL) + threadIdx.x;
    // phase 1: every token id this thread needs (independent loads)
    int32_t tok[UNROLL];
    uint32_t cv[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kGatherBlock;
        tok[u] = -1;
        cv[u] = 1;
        if (idx < total) {
            const uint32_t row = idx / CV;
            cv[u] = idx - row * CV;
            tok[u] = ids[row];
        }
    }
    // phase 2: the table rows, all in flight together
    u32x4 v[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kGatherBlock;
        ok[u] = idx < total && tok[u] >= 0 && (uint32_t)tok[u] < V;
        if (ok[u]) v[u] = __builtin_nontemporal_load(W + (uint64_t)tok[u] * CV + cv[u]);
        else if (idx < total && cv[u] == 0) *err_flag = 1;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint32_t idx = first + u * kGatherBlock;
        if (ok[u]) __builtin_nontemporal_store(v[u], out + idx);
    }
}

// Zeroes the table rows that a list of token ids names, 16 bytes to a thread.  The gradient
// of an embedding table is zero outside the rows its backward pass stored, so clearing the
// rows the last backward pass touched restores an all-zero table for N*C items written
// where the full fill writes V*C.  Ids outside [0, V) name no row (the backward pass stored
// none for them) and are skipped; a row listed twice is cleared twice.
__global__ void __launch_bounds__(kGatherBlock)
zero_rows16_kernel(const int32_t* __restrict__ rows, u32x4* __restrict__ table, uint32_t total,
                   uint32_t CV, uint32_t V) {
    const uint32_t idx = blockIdx.x * kGatherBlock + threadIdx.x;
    if (idx >= total) return;
    const uint32_t row = idx / CV;
    const uint32_t cv = idx - row * CV;
    const int32_t tok = rows[row];
    if (tok < 0 || (uint32_t)tok >= V) return;
    __builtin_nontemporal_store(u32x4{0u, 0u, 0u, 0u}, table + (uint64_t)tok * CV + cv);
}

// any C, any alignment
template <typename U>
__global__ void __launch_bounds__(kGatherBlock)
zero_rows_scalar_kernel(const int32_t* __restrict__ rows, U* __restrict__ table, uint64_t total,
                        uint32_t C, uint32_t V) {
    const uint64_t idx = (uint64_t)blockIdx.x * kGatherBlock + threadIdx.x;
    if (idx >= total) return;
    const uint64_t row = idx / C;
    const uint32_t c = (uint32_t)(idx - row * C);
    const int32_t tok = rows[row];
    if (tok < 0 || (uint32_t)tok >= V) return;
    table[(uint64_t)tok * C + c] = (U)0;
}

// scalar raw-bits gather (any C, any alignment)
template <typename U>
__global__ void __launch_bounds__(kGatherBlock)
gather_scalar_kernel(const int32_t* __restrict__ ids, const U* __restrict__ W, const U* __restrict__ wpe,
                     U* __restrict__ out, uint64_t total, uint32_t C, uint32_t T_len, uint32_t V,
                     int* err_flag) {
    const uint64_t idx = (uint64_t)blockIdx.x * kGatherBlock + threadIdx.x;
    if (idx >= total) return;
    const uint64_t row = idx / C;
    const uint32_t col = (uint32_t)(idx - row * C);
    const int32_t tok = ids[row];
    if (tok < 0 || (uint32_t)tok >= V) {
        if (col == 0) *err_flag = 1;
        return;
    }
    if (wpe == nullptr) {
        out[idx] = W[(uint64_t)tok * C + col];
    } else {
        float a[1], b[1];
        VecIO<U, 1>::load(W + (uint64_t)tok * C + col, a);
        VecIO<U, 1>::load(wpe + (row % T_len) * C + col, b);
        a[0] = a[0] + b[0];
        VecIO<U, 1>::store(out + idx, a);
    }
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
// keys[i] = ids[i] (out-of-range ids become the sentinel V and are skipped
// later), vals[i] = i
__global__ void __launch_bounds__(256)
emb_prepare_kernel(const int32_t* __restrict__ ids, uint32_t* __restrict__ keys,
                   uint32_t* __restrict__ vals, uint32_t N, uint32_t V, int* err_flag) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= N) return;
    const int32_t t = ids[i];
    const bool bad = t < 0 || (uint32_t)t >= V;
    if (bad) *err_flag = 1;
    keys[i] = bad ? V : (uint32_t)t;
    vals[i] = i;
}

// One-launch replacement for the radix sort when N <= kGroupSortMaxN.  What the
// segmented sum needs is not a total order by token, only that each token's
// rows sit next to each other in ascending row order.  Workgroup g owns the
// tokens whose hash falls in group g.  It reads ALL ids (64 KiB at N = 16384,
// served by L2), keeps the (token, row) pairs it owns in LDS, counts how many
// rows belong to lower-numbered groups (that is where its slice of the output
// starts), orders its pairs by (token, row) and writes them out.  No atomics on
// global memory, and the output is the same on every run.
//
// How a group orders its pairs depends on how many it has:
//  * up to one per thread (the usual case: a few dozen): by rank counting;
//  * more: some token is frequent (padding, a newline, "the").  The rows of ONE
//    token need no sorting network: they are distinct integers below N, so the
//    group marks them in an N-bit map and a row's place is the number of set
//    bits below it.  The group picks its most frequent token from a sample,
//    moves that token's rows into the bit map and orders only what is left --
//    by rank when that fits one pair per thread, with a bitonic network in LDS
//    otherwise.  (All rows one token: 640 us with the network over the whole
//    list, against 40 us this way, at N = 16384.)
//  * what is left after taking the frequent token out still exceeds LDS (two
//    tokens of one group holding most rows): gathered into the group's slice of
//    `spill` and sorted there -- slow, correct, and rare.
constexpr int kSortBlock = 512;
constexpr uint32_t kGroupSortMaxN = 65536;
constexpr uint32_t kSortLdsEntries = 3072;   // (token, row) pairs a workgroup keeps in LDS
constexpr uint32_t kRankSortMax = kSortBlock;  // lists up to one key per thread can be placed by rank ...
constexpr uint32_t kRankDirect = kSortBlock / 2;    // ... and are, up to this many (two threads or more share a key's comparisons)
constexpr uint32_t kRowMapWords = kGroupSortMaxN / 32;
constexpr uint32_t kSortWaves = kSortBlock / kWave;
static_assert(kRowMapWords % (2 * kSortWaves) == 0, "the waves share the row map in whole pairs of words");

// Bitonic network in its "flip" form: every comparator puts the smaller key at
// the lower index, so positions >= n behave as +infinity and need no padding.
// THREADS threads cooperate; SYNC() separates the steps.
template <int THREADS, typename SyncFn>
__device__ __forceinline__ void bitonic_sort_u64(unsigned long long* keys, uint32_t n, uint32_t tid, SyncFn sync) {
    uint32_t n2 = 1;
    while (n2 < n) n2 <<= 1;
    for (uint32_t k = 2; k <= n2; k <<= 1) {
        for (uint32_t j = k >> 1; j > 0; j >>= 1) {
            const uint32_t mask = (j == (k >> 1)) ? (k - 1) : j;
            for (uint32_t i = tid; i < n; i += THREADS) {
                const uint32_t partner = i ^ mask;
                if (partner > i && partner < n) {
                    const unsigned long long a = keys[i], b = keys[partner];
                    if (a > b) { keys[i] = b; keys[partner] = a; }
                }
            }
            sync();
        }
    }
}

// What the ordering step tells row n about its token's run, one 16-byte word per row:
//   R == 0               nothing to do for this row: a later row of a short run, or an id
//                        outside the table;
//   1 <= R <= kSoloRun   row n is the FIRST (lowest) row of a run of R rows, which one wave adds
//                        up in ascending order; x = the run's second row, or kNoRow when the
//                        ordering did not have it at hand (then it is row_s[start + 1]);
//   R > kSoloRun         row n is row number x of a long run of R rows.
// `start` is the place in row_s[] where the run begins.
struct __attribute__((aligned(16))) RunInfo { uint32_t tok, start, R, x; };

constexpr uint32_t kChunkRows = 64;      // a long run is cut into chunks of this many rows (the last takes the rest)
constexpr uint32_t kSoloRun = 2 * kChunkRows - 1;   // longest run that one wave adds up alone, in np.add.at's order
constexpr uint32_t kGroupChunks = 16;    // ... whose partial rows are added in groups of this many (the last takes the rest)
constexpr uint32_t kTicketFold = 32;     // arrival counters per chunk group: column block kb counts on kb % kTicketFold
constexpr uint32_t kNoRow = 0xFFFFFFFFu;
// row_s[] holds a row in its low 30 bits.  The top bit marks a TASK of the gradient kernel:
// the first row of a run of 2 .. kSoloRun rows, or the first row of a chunk of a long run.
// (A row that is its token's only row is no task: the row itself moves its vector.)  The
// bit below it marks the tasks of more than kRowRunMax rows: where a row's wave can add up
// a few rows itself (rows of few column blocks), only these are tasks.
constexpr uint32_t kTaskFlag = 0x80000000u;
constexpr uint32_t kBigTaskFlag = 0x40000000u;
constexpr uint32_t kRowMask = 0x3FFFFFFFu;
constexpr uint32_t kRowRunMax = 10;      // (the partner and one batch of rows)
// places of row_s[] that one wave of the gradient kernel searches for tasks: few where every run is a
// task, so that many waves share them; a wave's worth where only the runs of more than kRowRunMax rows are
constexpr uint32_t kTaskSpan = 16, kBigTaskSpan = 64;

// Layout of the order buffer, in 32-bit words: row_s[N] | (pad to 4) RunInfo[N] | group
// tickets | run tickets.  The tickets are arrival counters of the gradient kernel's long
// runs; the ordering step zeroes them and the gradient kernel leaves them zero.
__host__ __device__ inline uint64_t order_info_word(uint64_t N) { return (N + 3) & ~3ull; }
__host__ __device__ inline uint64_t order_ticket_word(uint64_t N) { return order_info_word(N) + 4 * N; }
__host__ __device__ inline uint64_t order_group_tickets(uint64_t N) { return (N / (kChunkRows * 2) + 1) * kTicketFold; }
__host__ __device__ inline uint64_t order_run_tickets(uint64_t N) { return (N / (kChunkRows * kGroupChunks * 2) + 1) * kTicketFold; }
__host__ __device__ inline uint64_t order_words(uint64_t N) { return order_ticket_word(N) + order_group_tickets(N) + order_run_tickets(N); }

// the task marks of row number j of a run of R rows (of a token inside the table)
__host__ __device__ inline uint32_t task_marks(uint32_t j, uint32_t R) {
    if (R <= kSoloRun) return j != 0 || R < 2 ? 0u : R > kRowRunMax ? kTaskFlag | kBigTaskFlag : kTaskFlag;
    return j % kChunkRows == 0 && j / kChunkRows < R / kChunkRows ? kTaskFlag | kBigTaskFlag : 0u;
}

// How the gradient kernel's task workgroups (of `waves` waves) share the work: a wave has a
// span of `span` places of row_s[] and ONE column block, and takes that block of every
// task that starts in the span.  A workgroup holds `spans` spans x `blocks` column blocks
// (blocks: a power of two); rows with more column blocks take `sets` workgroups per span.
struct TaskGrid {
    uint32_t blocks, spans, sets, wgs;
    uint32_t big_wgs;           // workgroups in front of those that take only the tasks of more than kRowRunMax rows, or 0
    uint32_t cg, cg_magic;      // (the row part) column groups of a row; ceil(2^32 / cg) where that divides exactly, or 0
};
// u / g.cg for u below rows x g.cg
__device__ __forceinline__ uint32_t row_of_unit(uint32_t u, const TaskGrid& g) {
    return g.cg == 1 ? u : g.cg_magic != 0 ? __umulhi(u, g.cg_magic) : u / g.cg;
}
inline TaskGrid task_grid(uint32_t N, uint32_t CB, uint32_t waves, uint32_t span, uint32_t cg) {
    TaskGrid g;
    g.cg = cg;
    // floor(u * ceil(2^32 / cg) / 2^32) = u / cg for u < 2^32 / cg, which holds for every u < N * cg then
    g.cg_magic = cg > 1 && (uint64_t)N * cg * cg < (1ull << 32) ? (uint32_t)(((1ull << 32) + cg - 1) / cg) : 0u;
    g.blocks = 1;
    while (g.blocks < CB && g.blocks * 2 <= waves) g.blocks *= 2;
    g.spans = waves / g.blocks;
    g.sets = (CB + g.blocks - 1) / g.blocks;
    const uint32_t places = g.spans * span;
    g.wgs = (((N + places - 1) / places) * g.sets + 7u) & ~7u;
    // Where every run is a task, the big ones (the chunks of long runs above all: their sums
    // have two hand-offs still to go through) get workgroups of their own, in front of all others.
    const uint32_t big_places = g.spans * kBigTaskSpan;
    g.big_wgs = span == kBigTaskSpan ? 0u : (((N + big_places - 1) / big_places) * g.sets + 7u) & ~7u;
    return g;
}
// Workgroups go to the GPU's eight XCDs in turn.  The chunks of a long run start every
// kChunkRows places, so the workgroups with that work would be every 2nd, 4th or 8th one --
// a fraction of the XCDs.  Workgroup b therefore takes piece task_piece(b) of the work: b with
// its low three bits XOR-ed by all its higher three-bit groups, a permutation within every
// eight consecutive numbers under which any such regular subset lands on all XCDs alike.
__host__ __device__ inline uint32_t task_piece(uint32_t b) {
    uint32_t fold = 0;
    for (uint32_t x = b >> 3; x != 0; x >>= 3) fold ^= x;
    return b ^ (fold & 7u);
}

// smallest index in sorted keys[0..n) whose key is not below `bound`
__device__ __forceinline__ uint32_t first_not_below(const unsigned long long* keys, uint32_t n, unsigned long long bound) {
    uint32_t lo = 0, hi = n;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (keys[mid] < bound) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// The hash group of a token: the bits just below bit 24 of a 24-bit Fibonacci product
// (a full-rate multiply; tokens that agree in their low 24 bits share a group, which is
// as good a partition as any).
__device__ __forceinline__ uint32_t token_group(uint32_t tok, uint32_t log2G) {
    return (__umul24(tok, 0x9E3779u) >> (24u - log2G)) & ((1u << log2G) - 1u);
}

// the work of workgroup `g` of the grouping sort (kSortBlock threads)
__device__ __forceinline__ void
emb_group_sort_body(uint32_t g, const int32_t* __restrict__ ids, uint32_t* __restrict__ order,
                    unsigned long long* __restrict__ spill, uint32_t N, uint32_t V, uint32_t log2G, int* err_flag) {
    __shared__ unsigned long long keys[kSortLdsEntries];
    __shared__ unsigned long long few[kRankSortMax + 1];
    __shared__ uint32_t row_map[kRowMapWords];
    // the ranking of a short list uses `few`'s bytes (a long list's rest comes later)
    uint32_t* tally = reinterpret_cast<uint32_t*>(few);     // per key: smaller tokens | same token << 10 | same token, lower row << 20
    uint32_t* placed = tally + kRankSortMax;                // rows by rank, kRankSortMax + 1 of them
    __shared__ uint32_t s_count, s_less, s_rest, s_below, s_wave_rows[kSortWaves];
    uint32_t* __restrict__ row_s = order;
    RunInfo* __restrict__ info = reinterpret_cast<RunInfo*>(order + order_info_word(N));
    // a pair leaves for the order: its row at place `at`, and what the row is told
    auto emit = [&](uint32_t tok, uint32_t row, uint32_t at, uint32_t j, uint32_t R, uint32_t next) {
        RunInfo ri;
        ri.tok = tok;
        ri.start = at - j;
        if (tok >= V) { ri.R = 0; ri.x = 0; }
        else if (R <= kSoloRun) { ri.R = j == 0 ? R : 0u; ri.x = next; }
        else { ri.R = R; ri.x = j; }
        row_s[at] = tok < V ? row | task_marks(j, R) : row;
        info[row] = ri;
    };
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & (kWave - 1);
    auto lanes_below = [&](unsigned long long mask) {     // set bits of `mask` below this lane
        return (uint32_t)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    };
    if (tid == 0) { s_count = 0; s_less = 0; s_rest = 0; s_below = 0; }
    tally[tid] = 0;                     // kRankSortMax == kSortBlock
    {   // this group's share of the gradient kernel's arrival counters
        const uint32_t groups = 1u << log2G;
        const uint32_t words = (uint32_t)(order_group_tickets(N) + order_run_tickets(N));
        uint32_t* tickets = order + order_ticket_word(N);
        for (uint32_t w = g * kSortBlock + tid; w < words; w += groups * kSortBlock) tickets[w] = 0;
    }
    __syncthreads();

    uint32_t less = 0, worst = 0;                   // `worst`: the largest id seen, as unsigned (a negative id is huge)
    // A thread reads four consecutive ids with one 16-byte load and keeps kScanLoads of
    // them in flight: one round covers 8192 rows.
    constexpr int kScanLoads = 4, ROUND = 4 * kScanLoads, AGG = 8;
    const bool wide_ids = (reinterpret_cast<uintptr_t>(ids) & 15u) == 0;
    for (uint32_t base = 0; base < N; base += kSortBlock * ROUND) {
        const bool whole = base + kSortBlock * ROUND <= N;          // no row of this round lies beyond N
        uint32_t t[ROUND];
        auto row_of = [&](int r) { return base + ((uint32_t)(r >> 2) * kSortBlock + tid) * 4u + (uint32_t)(r & 3); };
        if (whole && wide_ids) {
#pragma unroll
            for (int r = 0; r < ROUND; r += 4) {
                const u32x4 q = *reinterpret_cast<const u32x4*>(ids + row_of(r));
                t[r] = q.x; t[r + 1] = q.y; t[r + 2] = q.z; t[r + 3] = q.w;
            }
        } else {
#pragma unroll
            for (int r = 0; r < ROUND; ++r) t[r] = row_of(r) < N ? (uint32_t)ids[row_of(r)] : 0u;
        }
        // The pairs this group owns go into the list.  One LDS atomic per wave and
        // eight ids, not one per pair: a frequent token would otherwise queue
        // thousands of them on one address, and waiting for each one's return
        // value in turn costs the usual case a microsecond.
#pragma unroll
        for (int r0 = 0; r0 < ROUND; r0 += AGG) {
            unsigned long long owners[AGG];
            uint32_t wave_total = 0;
#pragma unroll
            for (int a = 0; a < AGG; ++a) {
                const bool live = whole || row_of(r0 + a) < N;
                worst = t[r0 + a] > worst ? t[r0 + a] : worst;
                const uint32_t tok = t[r0 + a] < V ? t[r0 + a] : V;
                const uint32_t owner = token_group(tok, log2G);
                less += (live && owner < g) ? 1u : 0u;
                owners[a] = __builtin_amdgcn_ballot_w64(live && owner == g);
                wave_total += (uint32_t)__popcll(owners[a]);
            }
            if (wave_total) {
                uint32_t first = 0;
                if (lane == 0) first = atomicAdd(&s_count, wave_total);
                first = (uint32_t)__builtin_amdgcn_readfirstlane((int)first);
#pragma unroll
                for (int a = 0; a < AGG; ++a) {
                    if (owners[a] == 0) continue;
                    const uint32_t slot = first + lanes_below(owners[a]);
                    if (((owners[a] >> lane) & 1ull) && slot < kSortLdsEntries) {
                        const uint32_t tok = t[r0 + a] < V ? t[r0 + a] : V;
                        keys[slot] = ((unsigned long long)tok << 32) | row_of(r0 + a);
                    }
                    first += (uint32_t)__popcll(owners[a]);
                }
            }
        }
    }
    if (g == 0 && worst >= V) *err_flag = 1;
    // rows owned by lower groups: exact integer wave totals, added in LDS
    {
        uint32_t v = less;
        v += __builtin_amdgcn_update_dpp(0, v, kDppQuadXor1, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppQuadXor2, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppRowHalfMirror, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppRowMirror, 0xf, 0xf, true);
        v += __builtin_amdgcn_ds_swizzle(v, kSwizzleXor16);
        const uint32_t total = __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 32);
        if (lane == 0 && total) atomicAdd(&s_less, total);
    }
    __syncthreads();
    const uint32_t count = s_count;
    const uint32_t offset = s_less;

    // The n <= kRankSortMax pairs of keys[], ranked by counting: every key is unique, so its
    // place in the order is the number of smaller keys.  The threads share the counting:
    // `parts` threads per key, each comparing the key with its slice of the list (broadcast
    // LDS reads), their tallies added in LDS.  A pair of token t leaves for place
    // offset + rank + shift(t).  (tally[] is zero on entry.)
    auto rank_and_emit = [&](uint32_t n, auto shift) {
        const uint32_t parts = n ? kSortBlock / n : 1u;             // threads per key
        const uint32_t part = n ? tid / n : 0u, k = part < parts ? tid - part * n : n;
        const uint32_t j_lo = (part * n) / parts, j_hi = k < n ? ((part + 1) * n) / parts : j_lo;
        const unsigned long long mine = k < n ? keys[k] : ~0ull;
        const uint32_t my_tok = (uint32_t)(mine >> 32), my_row = (uint32_t)mine;
        uint32_t smaller_tok = 0, same = 0, same_before = 0;
#pragma unroll 8
        for (uint32_t j = j_lo; j < j_hi; ++j) {
            const unsigned long long other = keys[j];
            const uint32_t tok = (uint32_t)(other >> 32), row = (uint32_t)other;
            smaller_tok += tok < my_tok ? 1u : 0u;
            same += tok == my_tok ? 1u : 0u;
            same_before += (tok == my_tok && row < my_row) ? 1u : 0u;
        }
        if (k < n) atomicAdd(&tally[k], smaller_tok | (same << 10) | (same_before << 20));
        __syncthreads();
        uint32_t rank = 0, run = 0, j = 0;
        if (tid < n) {
            const uint32_t packed = tally[tid];
            j = packed >> 20;
            run = (packed >> 10) & 1023u;
            rank = (packed & 1023u) + j;
            placed[rank] = (uint32_t)keys[tid];
        }
        __syncthreads();
        if (tid < n) {
            const uint32_t next = j + 1 < run ? placed[rank + 1] : kNoRow;
            const uint32_t tok = (uint32_t)(keys[tid] >> 32);
            emit(tok, (uint32_t)keys[tid], offset + rank + shift(tok), j, run, next);
        }
    };
    // (up to kRankDirect pairs: beyond, a thread has hundreds of comparisons to make, and what
    // makes a list that long is a frequent token, which the path below takes out first)
    if (count <= kRankDirect) {
        rank_and_emit(count, [](uint32_t) { return 0u; });
        return;
    }

    // -- a frequent token: of 64 evenly spaced pairs of the list, the token seen
    // most often among 16 candidates.  Every wave works it out for itself from
    // the same samples.  (Which pairs the list holds, and in what order, varies
    // from run to run; a different choice changes the time taken, never the output.)
    const uint32_t listed = count < kSortLdsEntries ? count : kSortLdsEntries;
    const bool reread = count > kSortLdsEntries;
    uint32_t hot = 0;
    {
        const uint32_t sample = (uint32_t)(keys[(lane * listed) / kWave] >> 32);
        uint32_t best_votes = 0;
#pragma nounroll
        for (int k = 0; k < kWave; k += 4) {
            const uint32_t candidate = (uint32_t)__builtin_amdgcn_readlane((int)sample, k);
            const uint32_t votes = (uint32_t)__popcll(__ballot(sample == candidate));
            if (votes > best_votes) { best_votes = votes; hot = candidate; }
        }
    }
    for (uint32_t w = tid; w < kRowMapWords; w += kSortBlock) row_map[w] = 0;
    __syncthreads();         // the map is clear, and `keys` may be overwritten

    // its rows go into the row map, every other pair into `rest`.  A list that
    // fits LDS is split from LDS and stays intact; a longer one is read again
    // from the ids, and `keys` becomes the rest.
    unsigned long long* rest = reread ? keys : few;
    const uint32_t rest_cap = reread ? kSortLdsEntries : kRankSortMax;
    auto split = [&](uint32_t tok, uint32_t row) {
        if (tok == hot) {
            atomicOr(&row_map[row >> 5], 1u << (row & 31));
        } else {
            const uint32_t slot = atomicAdd(&s_rest, 1u);
            if (slot < rest_cap) rest[slot] = ((unsigned long long)tok << 32) | row;
        }
    };
    auto owner_of = [&](int32_t t, uint32_t& tok) {
        tok = (uint32_t)t < V ? (uint32_t)t : V;
        return token_group(tok, log2G);
    };
    if (!reread) {
        for (uint32_t i = tid; i < count; i += kSortBlock) {
            const unsigned long long key = keys[i];
            split((uint32_t)(key >> 32), (uint32_t)key);
        }
    } else {
        // four consecutive ids per 16-byte load, four loads in flight per thread; a thread ORs
        // the marks of its four rows into the map's word (the rows of one load lie in one word)
        constexpr int AGAIN = 4;
        for (uint32_t base = 0; base < N; base += kSortBlock * AGAIN * 4) {
            uint32_t t[AGAIN][4];
#pragma unroll
            for (int r = 0; r < AGAIN; ++r) {
                const uint32_t row0 = base + ((uint32_t)r * kSortBlock + tid) * 4u;
                if (wide_ids && row0 + 4 <= N) {
                    const u32x4 q = *reinterpret_cast<const u32x4*>(ids + row0);
                    t[r][0] = q.x; t[r][1] = q.y; t[r][2] = q.z; t[r][3] = q.w;
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) t[r][c] = row0 + c < N ? (uint32_t)ids[row0 + c] : 0u;
                }
            }
#pragma unroll
            for (int r = 0; r < AGAIN; ++r) {
                const uint32_t row0 = base + ((uint32_t)r * kSortBlock + tid) * 4u;
                uint32_t marks = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    uint32_t tok;
                    const bool own = row0 + c < N && owner_of((int32_t)t[r][c], tok) == g;
                    if (own && tok == hot) marks |= 1u << c;
                    else if (own) split(tok, row0 + c);
                }
                if (marks) atomicOr(&row_map[row0 >> 5], marks << (row0 & 31u));
            }
        }
    }
    __syncthreads();
    const uint32_t rest_n = s_rest;

    // pairs of a sorted list: a pair's run is found by bisection, its successor is its neighbour
    auto emit_sorted = [&](const unsigned long long* sorted, uint32_t n, uint32_t i, uint32_t shift) {
        const unsigned long long key = sorted[i];
        const uint32_t tok = (uint32_t)(key >> 32);
        const uint32_t lo = first_not_below(sorted, n, (unsigned long long)tok << 32);
        const uint32_t hi = first_not_below(sorted, n, (unsigned long long)(tok + 1u) << 32);
        emit(tok, (uint32_t)key, offset + i + shift, i - lo, hi - lo, i + 1 < hi ? (uint32_t)sorted[i + 1] : kNoRow);
    };

    if (rest_n > rest_cap) {
        if (!reread) {
            // no single frequent token: the network over the whole list
            bitonic_sort_u64<kSortBlock>(keys, count, tid, [] { __syncthreads(); });
            for (uint32_t i = tid; i < count; i += kSortBlock) emit_sorted(keys, count, i, 0u);
            return;
        }
        // gather the group's pairs into its slice of `spill` (slices are
        // disjoint: [offset, offset + count)), sort there, then split
        __syncthreads();
        if (tid == 0) s_count = 0;
        __syncthreads();
        unsigned long long* mine = spill + offset;
        for (uint32_t i = tid; i < N; i += kSortBlock) {
            uint32_t tok;
            if (owner_of(ids[i], tok) == g) mine[atomicAdd(&s_count, 1u)] = ((unsigned long long)tok << 32) | i;
        }
        __threadfence_block();
        __syncthreads();
        bitonic_sort_u64<kSortBlock>(mine, count, tid, [] { __threadfence_block(); __syncthreads(); });
        for (uint32_t i = tid; i < count; i += kSortBlock) emit_sorted(mine, count, i, 0u);
        return;
    }

    // -- the rest, in order; pairs above the frequent token leave room for its rows
    const uint32_t hot_rows = count - rest_n;
    uint32_t n_below = 0;                          // pairs of the rest that sort before the frequent token
    if (rest_n <= kRankDirect) {
        // a short rest: ranked by counting, as a short list is.  That wants the rest in keys[]
        // and zero tallies: a rest split off the list in LDS sits in the tallies' bytes and
        // moves over first (the list itself is not needed any more).
        if (!reread) {
            const unsigned long long pair = tid < rest_n ? few[tid] : 0ull;
            __syncthreads();
            if (tid < rest_n) keys[tid] = pair;
            tally[tid] = 0;
            __syncthreads();
        }
        if (tid < rest_n) n_below = (uint32_t)(keys[tid] >> 32) < hot ? 1u : 0u;
        rank_and_emit(rest_n, [&](uint32_t tok) { return tok > hot ? hot_rows : 0u; });
    } else {
        bitonic_sort_u64<kSortBlock>(rest, rest_n, tid, [] { __syncthreads(); });
        for (uint32_t i = tid; i < rest_n; i += kSortBlock) {
            const uint32_t tok = (uint32_t)(rest[i] >> 32);
            n_below += tok < hot ? 1u : 0u;
            emit_sorted(rest, rest_n, i, tok > hot ? hot_rows : 0u);
        }
    }
    if (n_below) atomicAdd(&s_below, n_below);
    __syncthreads();
    const uint32_t below = s_below;

    // -- the frequent token's rows.  Word w of the map holds rows 32 w ... 32 w + 31.
    // The waves share the words that rows below N can mark, an even number each.
    const uint32_t wave = tid / kWave;
    const uint32_t words = (N + 31) / 32;
    const uint32_t per_wave = ((words + kSortWaves - 1) / kSortWaves + 1) & ~1u;     // at most kRowMapWords / kSortWaves
    const uint32_t w_begin = wave * per_wave;
    {
        uint32_t v = 0;
        for (uint32_t j = lane; j < per_wave; j += kWave) v += (uint32_t)__popc(row_map[w_begin + j]);
        v += __builtin_amdgcn_update_dpp(0, v, kDppQuadXor1, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppQuadXor2, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppRowHalfMirror, 0xf, 0xf, true);
        v += __builtin_amdgcn_update_dpp(0, v, kDppRowMirror, 0xf, 0xf, true);
        v += __builtin_amdgcn_ds_swizzle(v, kSwizzleXor16);
        const uint32_t wave_rows = __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 32);   // read with every lane active
        if (lane == 0) s_wave_rows[wave] = wave_rows;
    }
    __syncthreads();
    uint32_t at = offset + below;
    for (uint32_t w = 0; w < wave; ++w) at += s_wave_rows[w];
    const uint32_t mine_rows = s_wave_rows[wave];
    if (mine_rows == 0) return;
    if (mine_rows * 4u >= per_wave * 32u) {
        // Many marks (a quarter of the wave's rows or more): the wave takes its words two at a
        // time, each half-wave gives one word's 32 rows a lane each, and a marked row's place
        // is the count of marks before it, so a store instruction writes up to 64
        // neighbouring entries.
        const uint32_t upper = lane >> 5, bit = lane & 31u;
#pragma nounroll
        for (uint32_t w0 = w_begin; w0 < w_begin + per_wave; w0 += 2) {
            const uint32_t word0 = row_map[w0], word1 = row_map[w0 + 1];
            const uint32_t n0 = (uint32_t)__popc(word0);
            const uint32_t word = upper ? word1 : word0;
            if ((word >> bit) & 1u) {
                const uint32_t to = at + (upper ? n0 : 0u) + (uint32_t)__popc(word & ((1u << bit) - 1u));
                emit(hot, (w0 + upper) * 32u + bit, to, to - (offset + below), hot_rows, kNoRow);
            }
            at += n0 + (uint32_t)__popc(word1);
        }
        return;
    }
    // Few marks: a pass over all the wave's rows would mostly find nothing (two thousand rows
    // of a token among 65536 are four marks a word).  The wave takes 64 words at a time, a
    // lane each; the lanes' mark counts are summed up across the wave (with every lane
    // active), and each lane then walks the marks of its own word.
#pragma nounroll
    for (uint32_t w0 = w_begin; w0 < w_begin + per_wave; w0 += kWave) {
        const uint32_t w = w0 + lane;
        uint32_t word = w < w_begin + per_wave ? row_map[w] : 0u;
        const uint32_t n = (uint32_t)__popc(word);
        uint32_t upto = n;                                  // marks in this lane's word and the lanes' before it
#pragma unroll
        for (int d = 1; d < kWave; d *= 2) {
            const uint32_t other = (uint32_t)__shfl_up((int)upto, d, kWave);
            if (lane >= (uint32_t)d) upto += other;
        }
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)upto, kWave - 1);
        uint32_t to = at + upto - n;
        while (word != 0) {
            const uint32_t bit = (uint32_t)__builtin_ctz(word);
            word &= word - 1u;
            emit(hot, w * 32u + bit, to, to - (offset + below), hot_rows, kNoRow);
            ++to;
        }
        at += total;
    }
}

// log2 of the number of hash groups (= ordering workgroups).  128 up to 16384
// rows: beside the forward gather they take a quarter of the GPU's thread slots
// for a few microseconds (256 took half: forward 13.2 -> 11.8 us at 16384 x 384
// fp32, 38 -> 36.5 us at 16384 x 1536), and 64 make each group's ranking too long.
// Above that the groups double with the rows, which keeps a group at a hundred or
// so pairs; every group still reads all ids (256 KiB at 65536 rows, from L2),
// about 10 us beside a gather of 100 us or more, where the radix sort's launches
// took 37 us before the gather could start (65536 x 1024 fp32: 127 -> 106 us).
// The stand-alone sort uses the same number, so that both ways to the order give
// the same order and the gradient sums associate identically.
inline uint32_t group_sort_log2g(uint32_t n) { return n > 32768 ? 9u : n > 16384 ? 8u : n > 1024 ? 7u : 4u; }

__global__ void __launch_bounds__(kSortBlock)
emb_group_sort_kernel(const int32_t* __restrict__ ids, uint32_t* __restrict__ order,
                      unsigned long long* __restrict__ spill, uint32_t N, uint32_t V, uint32_t log2G, int* err_flag) {
    emb_group_sort_body(blockIdx.x, ids, order, spill, N, V, log2G, err_flag);
}

// Forward gather and the ordering of the ids for the later gradient in ONE
// launch.  The two only share their input, the gather is bound by memory
// bandwidth and the ordering by latency, so the first `groups` workgroups do the
// ordering (they are dispatched first and are done within a few microseconds)
// while all the others stream table rows: the ordering then costs the backward
// pass nothing and the forward pass next to nothing.  (Doing the same with a
// second stream and events was measured three times more expensive than the
// ordering itself.)  One 16-byte vector per thread; with a position table the
// rows are added in fp32.  Held to 80 scalar registers: compiled to 86 or more
// (the ordering code's appetite, the gather needs a dozen) the gather ran 5 %
// slower -- 38.2 against 36.2 us at 16384 x 1536 fp32.
constexpr int kGatherPerThread = 2;

template <typename T, int VEC, bool RAW>
__global__ void __launch_bounds__(kSortBlock) __attribute__((amdgpu_num_sgpr(80)))
gather_sort_kernel(const int32_t* __restrict__ ids, const T* __restrict__ W, const T* __restrict__ wpe,
                   T* __restrict__ out, uint32_t total, uint32_t CV, uint32_t C, uint32_t T_len, uint32_t V,
                   uint32_t* __restrict__ order, unsigned long long* __restrict__ spill,
                   uint32_t N, uint32_t log2G, int* err_flag, int32_t* __restrict__ kept) {
    const uint32_t groups = 1u << log2G;
    if (blockIdx.x < groups) {
        emb_group_sort_body(blockIdx.x, ids, order, spill, N, V, log2G, err_flag);
        return;
    }
    // the gather proper: kGatherPerThread vectors per thread, all in flight together (the
    // ordering code sets this kernel's register and LDS footprint, so fewer waves fit a
    // CU than in a plain copy: each has to keep more bytes in flight)
    const uint32_t first = (blockIdx.x - groups) * (kSortBlock * kGatherPerThread) + threadIdx.x;
    uint32_t row[kGatherPerThread], cv[kGatherPerThread];
    int32_t tok[kGatherPerThread];
#pragma unroll
    for (int u = 0; u < kGatherPerThread; ++u) {
        const uint32_t idx = first + u * kSortBlock;
        row[u] = idx / CV;
        cv[u] = idx - row[u] * CV;
        tok[u] = idx < total ? ids[row[u]] : -1;      // (the ordering workgroups report bad ids)
    }
    if constexpr (RAW) {
        u32x4 v[kGatherPerThread];
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u)
            if ((uint32_t)tok[u] < V) v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W) + (uint64_t)tok[u] * CV + cv[u]);
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u)
            if ((uint32_t)tok[u] < V) __builtin_nontemporal_store(v[u], reinterpret_cast<u32x4*>(out) + first + u * kSortBlock);
    } else {
        // (the position rows do not wait for the ids: asked for first, from a valid row whatever the id)
        float v[kGatherPerThread][VEC], p[kGatherPerThread][VEC];
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u)
            VecIO<T, VEC>::load(wpe + (uint64_t)(row[u] % T_len) * C + cv[u] * VEC, p[u]);
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u) {
            if ((uint32_t)tok[u] < V) VecIO<T, VEC>::load(W + (uint64_t)tok[u] * C + cv[u] * VEC, v[u]);
        }
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u) {
            if ((uint32_t)tok[u] < V) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) v[u][k] = v[u][k] + p[u][k];
                VecIO<T, VEC>::store(out + (uint64_t)row[u] * C + cv[u] * VEC, v[u]);
            }
        }
    }
    // a copy of the ids this pass read, for the caller that later clears exactly the rows
    // of the table's gradient that the backward pass of these ids stores
    if (kept != nullptr) {
#pragma unroll
        for (int u = 0; u < kGatherPerThread; ++u)
            if (cv[u] == 0 && first + u * kSortBlock < total) kept[row[u]] = tok[u];
    }
}

// The ordering of the ids at the front of the zero fill of the table's gradient: one launch for
// a caller that clears dW and orders the ids before its forward pass and then gathers with the
// plain kernel.  Measured on MI355X it is the worse of the two hosts: the fill alone runs best
// with few waves on a CU, this kernel's 512-thread workgroups (the ordering's shape) fill at full
// occupancy (a tenth slower), and the launch takes 3 us (50 MB table) to 25 us (1 GB) longer than
// the plain fill where the same ordering workgroups cost the forward gather 1 to 3 us -- which is
// why the forward call keeps them.  It still beats a fill and an ordering launched one after the
// other (8 us more at 16384 ids, 44 us at 65536).
constexpr uint32_t kFillOrderIdleLds = 0;      // dynamic LDS that nothing touches (an occupancy cap): none pays here

__global__ void __launch_bounds__(kSortBlock) __attribute__((amdgpu_num_sgpr(80)))
fill_order_kernel(const int32_t* __restrict__ ids, uint32_t* __restrict__ order, unsigned long long* __restrict__ spill,
                  uint32_t N, uint32_t V, uint32_t log2G, int* err_flag, u32x4* __restrict__ dst, uint64_t vectors) {
    const uint32_t groups = 1u << log2G;
    if (blockIdx.x < groups) {
        emb_group_sort_body(blockIdx.x, ids, order, spill, N, V, log2G, err_flag);
        return;
    }
    const uint64_t i = (uint64_t)(blockIdx.x - groups) * kSortBlock + threadIdx.x;
    if (i < vectors) __builtin_nontemporal_store(u32x4{0u, 0u, 0u, 0u}, dst + i);
}

template <typename T, int VEC>
__device__ __forceinline__ void store_grad_row(T* dW, uint64_t off, const float (&acc)[VEC], bool accumulate) {
    float o[VEC];
    if (accumulate) {
        VecIO<T, VEC>::load(dW + off, o);
#pragma unroll
        for (int k = 0; k < VEC; ++k) o[k] = o[k] + acc[k];
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) o[k] = acc[k];
    }
    VecIO<T, VEC>::store(dW + off, o);
}

// The gradient sum proper, one launch, no float atomics.  dY is read once and every row of
// dW is written once.  The grid has two parts.
//
// ROWS.  A wave takes one row of dY and KW neighbouring blocks of 64 column vectors (the
// whole row when it has up to KW blocks); one 16-byte scalar load tells it what the row is
// (RunInfo).  A row that is its token's only row moves its vectors to the table -- most rows
// do; where a wave takes one column block (KW = 1), the first row of a run of up to
// kRowRunMax rows also adds that run itself; every other row ends there.  With a position
// table a workgroup takes one position t and column block, its waves the rows b*T + t of
// the batch; besides the above they leave their vectors in LDS, where wave 0 adds them in
// ascending b: dwpe[t, :] (+)= sum_b dY[b, t, :].
//
// TASKS, at the FRONT of the grid so that they are under way while the rest walks the rows.
// A wave searches kTaskSpan or kBigTaskSpan places of row_s[] for marked rows and takes ONE
// column block of every one found (TaskGrid; the tasks of more than kRowRunMax rows carry a
// second mark and, where the rows leave all runs to the tasks, go first):
//   * the first row of a run of 2 .. kSoloRun rows: the wave adds the run's rows in
//     ascending order -- the very sequence of fp32 adds np.add.at makes -- and stores the
//     table row;
//   * the first row of a chunk of a LONGER run (a frequent token: padding, "the"), which is
//     cut into chunks of kChunkRows rows: the wave adds up its chunk's rows (eight in
//     flight) and leaves the partial row in the workspace.  The wave that completes a group
//     of kGroupChunks chunks -- it learns that from an arrival counter -- adds the group's
//     partial rows in chunk order, and the wave that completes the run's last group adds
//     the groups in order and stores the table row.  Which wave does the adding varies from
//     call to call, what it adds in which order does not: the same bits every time.  The
//     counters are zero before and after the call.
// (One wave per row and column block, runs included, started half a million waves at
// 65536 rows of 4096 bf16 columns, most of them with nothing to do, behind the waves that
// had: 30 to 45 us of the call.)
constexpr int kRowBatch = 8;          // rows a wave keeps in flight
                                      // (16 for the chunks of long runs take the kernel from 60 to 90 registers: fewer waves
                                      // per CU, and single rows move 3 to 10 % slower for 4 % on Zipf ids)
constexpr int kPosWaves = 4;          // most waves that share the rows of one position
constexpr int kPosRows = 4;           // rows that each of them has in flight
constexpr int kRowSumBlock = 256;
constexpr uint32_t kRowSumWaves = kRowSumBlock / kWave;
constexpr int kRowBlocksMax = 8;      // most column blocks of a row that one wave moves
constexpr uint64_t kRowWavesEasy = 131072;

// Partial rows travel between waves of one launch, which may sit on different L2 caches:
// they are written and read with device-scope accesses (which go past the L2 to where
// all of the GPU's caches agree), two floats at a time, so that the arrival counters
// need no cache write-back or invalidation.
template <int VEC>
__device__ __forceinline__ void store_partial(float* p, const float (&acc)[VEC]) {
    if constexpr (VEC % 2 == 0) {
#pragma unroll
        for (int k = 0; k < VEC; k += 2) {
            const unsigned long long w = (unsigned long long)__float_as_uint(acc[k]) | ((unsigned long long)__float_as_uint(acc[k + 1]) << 32);
            __hip_atomic_store(reinterpret_cast<unsigned long long*>(p + k), w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) __hip_atomic_store(p + k, acc[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <int VEC>
__device__ __forceinline__ void load_partial(const float* p, float (&v)[VEC]) {
    if constexpr (VEC % 2 == 0) {
#pragma unroll
        for (int k = 0; k < VEC; k += 2) {
            const unsigned long long w = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p + k), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            v[k] = __uint_as_float((uint32_t)w);
            v[k + 1] = __uint_as_float((uint32_t)(w >> 32));
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) v[k] = __hip_atomic_load(p + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// acc += dY[r, col ...] for the rows r that lanes 0 .. cnt-1 hold in `mine`, in lane order
template <typename T, int VEC, int BATCH = kRowBatch>
__device__ __forceinline__ void add_lane_rows(float (&acc)[VEC], uint32_t mine, uint32_t cnt, const T* __restrict__ dY,
                                              uint32_t C, uint32_t col, bool live) {
    typedef RawVec<T, VEC> Raw;
#pragma nounroll
    for (uint32_t q0 = 0; q0 < cnt; q0 += BATCH) {
        typename Raw::type v[BATCH];
#pragma unroll
        for (int q = 0; q < BATCH; ++q) {
            const uint32_t r = (uint32_t)__builtin_amdgcn_readlane((int)mine, (int)(q0 + q));
            v[q] = Raw::zero();
            if (q0 + q < cnt && live) v[q] = Raw::load(dY + (uint64_t)r * C + col);
        }
#pragma unroll
        for (int q = 0; q < BATCH; ++q) {
            if (q0 + q < cnt) {
                float x[VEC];
                Raw::unpack(v[q], x);
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] = acc[k] + x[k];
            }
        }
    }
}

// acc += dY[row_s[p], col ...] for p = from .. to-1, ascending (p is the same in every lane).
// The wave fetches 64 places of row_s[] with one load, a place per lane, and hands the rows
// round from there.
template <typename T, int VEC, int BATCH = kRowBatch>
__device__ __forceinline__ void add_listed_rows(float (&acc)[VEC], const uint32_t* __restrict__ row_s, uint32_t from,
                                                uint32_t to, const T* __restrict__ dY, uint32_t C, uint32_t col, bool live,
                                                uint32_t lane) {
#pragma nounroll
    for (uint32_t base = from; base < to; base += kWave) {
        const uint32_t cnt = to - base < kWave ? to - base : kWave;
        const uint32_t mine = lane < cnt ? row_s[base + lane] & kRowMask : 0u;
        add_lane_rows<T, VEC, BATCH>(acc, mine, cnt, dY, C, col, live);
    }
}

// sum = slots[first], slots[first + 1], ... (n of them), added in that order; the
// partial rows were written by other waves of this launch
template <int VEC>
__device__ __forceinline__ void add_partial_rows(float (&sum)[VEC], const float* slots, uint64_t first,
                                                 uint32_t n, uint32_t C, uint32_t col, bool live) {
    constexpr int BATCH = VEC >= 8 ? 4 : 8;         // partial rows in flight
#pragma unroll
    for (int k = 0; k < VEC; ++k) sum[k] = 0.0f;
#pragma nounroll
    for (uint32_t i0 = 0; i0 < n; i0 += BATCH) {
        float v[BATCH][VEC];
#pragma unroll
        for (int q = 0; q < BATCH; ++q) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) v[q][k] = 0.0f;
            if (i0 + q < n && live) load_partial<VEC>(slots + (first + i0 + q) * C + col, v[q]);
        }
#pragma unroll
        for (int q = 0; q < BATCH; ++q) {
            if (i0 + q < n) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) sum[k] = (i0 + q == 0) ? v[q][k] : sum[k] + v[q][k];
            }
        }
    }
}

// One arrival at a counter; true for the wave whose arrival is number `expected` (it also
// puts the counter back to zero).  A wave arrives after its partial rows have been
// written, so the wave that arrives last finds all of them.  What makes that true: the
// partial rows are device-scope (sc1) stores, which are acknowledged only once they are
// past the L2, and the explicit s_waitcnt vmcnt(0) below holds the wave until every one of
// its stores has been acknowledged -- only then does the counter move.  The workgroup-scope
// release fence beside it is a compiler barrier only: on gfx950 it emits no vmcnt wait
// (a workgroup shares its L1), so the explicit wait is what orders stores and counter
// across workgroups, without the L2 write-back an agent-scope release would cost.
__device__ __forceinline__ bool arrive_last(uint32_t* ticket, uint32_t expected, uint32_t lane) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");          // keeps the compiler from moving stores down
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                // every store of this wave has been acknowledged
    uint32_t old = 0;
    if (lane == 0) old = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    old = (uint32_t)__builtin_amdgcn_readfirstlane((int)old);
    if (old + 1u != expected) return false;
    if (lane == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return true;
}

// What the tasks of the gradient kernel work on.
template <typename T, typename TO>
struct RowSumArgs {
    const uint32_t* __restrict__ row_s;
    uint32_t* group_tickets;
    uint32_t* run_tickets;
    const T* __restrict__ dY;
    TO* dW;
    float* part;            // a partial row per chunk of a long run ...
    float* part2;           // ... and per group of chunks
    uint32_t C, CV, CB;
    bool accumulate;
};

// Column block kb of the run of 1 .. kSoloRun rows that row `n` starts.  The row's own vector,
// its partner's and the list of the rows after those are asked for together: every lane
// loads from a valid place (a lane outside the row from the row's start), with no branch
// between the loads for the compiler to put a wait into.
template <typename T, typename TO, int VEC>
__device__ __forceinline__ void sum_short_run(const RowSumArgs<T, TO>& a, const RunInfo& ri, uint32_t n, uint32_t kb, uint32_t lane) {
    typedef RawVec<T, VEC> Raw;
    const uint32_t cv = kb * kWave + lane, col = cv * VEC;
    const bool live = cv < a.CV;
    const uint32_t col_ld = live ? col : 0u;
    float acc[VEC];
    if (ri.R == 1) {
        const typename Raw::type own = Raw::load(a.dY + (uint64_t)n * a.C + col_ld);
        Raw::unpack(own, acc);
    } else {
        const uint32_t rest = ri.R - 2, cnt = rest < kWave ? rest : kWave;
        uint32_t mine = a.row_s[ri.start + 1 + (lane < cnt ? lane + 1 : 0u)];       // (asked for first: needed first)
        const uint32_t r1 = ri.x != kNoRow ? ri.x : a.row_s[ri.start + 1] & kRowMask;
        const typename Raw::type first = Raw::load(a.dY + (uint64_t)n * a.C + col_ld);
        const typename Raw::type second = Raw::load(a.dY + (uint64_t)r1 * a.C + col_ld);
        mine &= kRowMask;
        float x[VEC];
        Raw::unpack(first, acc);
        Raw::unpack(second, x);
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k] = acc[k] + x[k];
        if (cnt != 0) add_lane_rows<T, VEC>(acc, mine, cnt, a.dY, a.C, col, live);
        if (rest > kWave) add_listed_rows<T, VEC>(acc, a.row_s, ri.start + 2 + kWave, ri.start + ri.R, a.dY, a.C, col, live, lane);
    }
    if (live) store_grad_row<TO, VEC>(a.dW, (uint64_t)ri.tok * a.C + col, acc, a.accumulate);
}

// Column block kb of the chunk of a long run that starts with row number ri.x of the run.
template <typename T, typename TO, int VEC>
__device__ __forceinline__ void sum_chunk(const RowSumArgs<T, TO>& a, const RunInfo& ri, uint32_t kb, uint32_t lane) {
    const uint32_t R = ri.R, start = ri.start, CB = a.CB, C = a.C;
    const uint32_t n1 = R / kChunkRows;                             // chunks (at least 2)
    const uint32_t c = ri.x / kChunkRows;
    const uint32_t lo = start + c * kChunkRows, hi = c + 1 == n1 ? start + R : lo + kChunkRows;
    auto col_of = [&](uint32_t b) { return (b * kWave + lane) * VEC; };
    auto live_in = [&](uint32_t b) { return b * kWave + lane < a.CV; };
    float acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
    add_listed_rows<T, VEC>(acc, a.row_s, lo, hi, a.dY, C, col_of(kb), live_in(kb), lane);
    if (live_in(kb)) store_partial<VEC>(a.part + (uint64_t)(lo / kChunkRows) * C + col_of(kb), acc);
    // the group of chunks this one belongs to, and its counter
    const uint32_t n2 = n1 / kGroupChunks ? n1 / kGroupChunks : 1u;   // groups
    const uint32_t q = c / kGroupChunks < n2 ? c / kGroupChunks : n2 - 1;
    const uint32_t c_lo = q * kGroupChunks, c_hi = q + 1 == n2 ? n1 : c_lo + kGroupChunks;
    const uint32_t g_at = start + c_lo * kChunkRows;                  // where the group starts
    const uint32_t fold = kb % kTicketFold, n_fold = (CB - 1 - fold) / kTicketFold + 1;
    if (!arrive_last(a.group_tickets + (g_at / (kChunkRows * 2)) * kTicketFold + fold, (c_hi - c_lo) * n_fold, lane)) return;
    for (uint32_t b = fold; b < CB; b += kTicketFold) {
        float sum[VEC];
        add_partial_rows<VEC>(sum, a.part, g_at / kChunkRows, c_hi - c_lo, C, col_of(b), live_in(b));
        if (!live_in(b)) continue;
        if (n2 == 1) store_grad_row<TO, VEC>(a.dW, (uint64_t)ri.tok * C + col_of(b), sum, a.accumulate);
        else store_partial<VEC>(a.part2 + (uint64_t)(g_at / (kChunkRows * kGroupChunks)) * C + col_of(b), sum);
    }
    if (n2 == 1) return;
    if (!arrive_last(a.run_tickets + (start / (kChunkRows * kGroupChunks * 2)) * kTicketFold + fold, n2, lane)) return;
    for (uint32_t b = fold; b < CB; b += kTicketFold) {
        float sum[VEC];
        // group q' starts kChunkRows * kGroupChunks places after group q' - 1: its slot is the next
        add_partial_rows<VEC>(sum, a.part2, start / (kChunkRows * kGroupChunks), n2, C, col_of(b), live_in(b));
        if (live_in(b)) store_grad_row<TO, VEC>(a.dW, (uint64_t)ri.tok * C + col_of(b), sum, a.accumulate);
    }
}

// POS: a workgroup takes the B rows of one position (one column block); otherwise a wave
// takes one row and KW neighbouring column blocks.
template <typename T, typename TO, int VEC, int KW, bool POS>
__global__ void __launch_bounds__(POS ? kPosWaves * kWave : kRowSumBlock)
emb_row_sum_kernel(const uint32_t* __restrict__ order, uint32_t* group_tickets, const T* __restrict__ dY, TO* dW,
                   TO* dwpe, float* part, uint32_t N, uint32_t C, uint32_t CV, uint32_t CB, uint32_t V, uint32_t T_len,
                   uint32_t B, int accumulate, int accumulate_pos, TaskGrid tg) {
    static_assert(!POS || KW == 1, "a position's rows go one column block at a time");
    typedef RawVec<T, VEC> Raw;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves = POS ? blockDim.x / kWave : kRowSumWaves;     // waves of a workgroup
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const uint32_t* __restrict__ row_s = order;
    const RunInfo* __restrict__ info = reinterpret_cast<const RunInfo*>(order + order_info_word(N));
    constexpr uint32_t kSpan = KW == 1 ? kBigTaskSpan : kTaskSpan;       // (tg: the host's task_grid() for this span)
    const uint32_t task_wgs = tg.big_wgs + tg.wgs;
    RowSumArgs<T, TO> a;
    a.row_s = row_s;
    a.group_tickets = group_tickets;
    a.run_tickets = group_tickets + order_group_tickets(N);     // (the counters follow the RunInfo words of `order`)
    a.dY = dY;
    a.dW = dW;
    a.part = part;
    a.part2 = part + (uint64_t)(N / kChunkRows + 1) * C;
    a.C = C; a.CV = CV; a.CB = CB;
    a.accumulate = accumulate != 0;
    // runs that a row wave adds up itself when it takes one column block (a task's way to the
    // rows is one round trip to memory longer, and these are most of the runs of ids that
    // rarely repeat); wider row waves leave every run to the tasks
    constexpr uint32_t kRowRun = KW == 1 ? kRowRunMax : 1;
    static_assert(kRowRunMax == kRowBatch + 2, "the partner and one batch of rows");

    if (blockIdx.x < task_wgs) {
        // in front: the workgroups of the big tasks alone (where there are such); then those of
        // every other task -- or, where the rows add short runs themselves, of the big tasks only
        const bool big_pass = blockIdx.x < tg.big_wgs;
        const uint32_t piece = task_piece(big_pass ? blockIdx.x : blockIdx.x - tg.big_wgs);
        const uint32_t group = piece / tg.sets, set = piece - group * tg.sets;
        if (wave >= tg.spans * tg.blocks) return;
        const uint32_t span = group * tg.spans + wave / tg.blocks;
        const uint32_t kb = set * tg.blocks + wave % tg.blocks;                 // this wave's column block
        const uint32_t places = big_pass ? kBigTaskSpan : kSpan;
        if (kb >= CB || span * places >= N) return;
        static_assert(kSpan <= kWave && kBigTaskSpan <= kWave, "a lane per place of the span");
        const uint32_t p = span * places + lane;
        const uint32_t word = lane < places && p < N ? row_s[p] : 0u;
        const uint32_t marks = word & (kTaskFlag | kBigTaskFlag);
        const bool wanted = KW == 1 || big_pass ? (marks & kBigTaskFlag) != 0 : marks == kTaskFlag;
        unsigned long long marked = __builtin_amdgcn_ballot_w64(wanted);
        while (marked != 0) {
            const uint32_t at = (uint32_t)__builtin_ctzll(marked);
            marked &= marked - 1;
            const uint32_t row = (uint32_t)__builtin_amdgcn_readlane((int)word, (int)at) & kRowMask;
            const RunInfo ri = info[row];
            if (ri.R <= kRowRun) continue;                      // (the row itself adds its few partners)
            if (ri.R <= kSoloRun) sum_short_run<T, TO, VEC>(a, ri, row, kb, lane);
            else sum_chunk<T, TO, VEC>(a, ri, kb, lane);
        }
        return;
    }

    if constexpr (!POS) {
        const uint32_t CG = tg.cg;                              // groups of KW column blocks in a row
        const uint32_t unit = (blockIdx.x - task_wgs) * waves + wave;
        if (unit >= N * CG) return;
        const uint32_t n = row_of_unit(unit, tg), kg = unit - n * CG;
        const RunInfo ri = info[n];
        if constexpr (KW == 1) {
            if (ri.R == 0 || ri.R > kRowRun) return;
            sum_short_run<T, TO, VEC>(a, ri, n, kg, lane);
        } else {
            if (ri.R != 1) return;                              // (runs are summed by the tasks)
            typename Raw::type own[KW];
#pragma unroll
            for (int w = 0; w < KW; ++w) {
                const uint32_t cv = (kg * KW + w) * kWave + lane;
                own[w] = Raw::zero();
                if (cv < CV) own[w] = Raw::load(dY + (uint64_t)n * C + cv * VEC);
            }
#pragma unroll
            for (int w = 0; w < KW; ++w) {
                const uint32_t cv = (kg * KW + w) * kWave + lane;
                float x[VEC];
                Raw::unpack(own[w], x);
                if (cv < CV) store_grad_row<TO, VEC>(dW, (uint64_t)ri.tok * C + cv * VEC, x, accumulate != 0);
            }
        }
    } else {
        // The workgroup has position t and one column block.  In a pass its waves read
        // waves x kPosRows rows of the batch -- wave w the rows b0 + w, b0 + waves + w, ..., all in
        // flight, each with what the row is -- and leave the vectors in LDS, where wave 0 adds them
        // in ascending b; the other waves meanwhile add up the short runs that their rows start.
        // (A batch's last rows are read again where B is no multiple of a pass: every load has a
        // valid address and no branch around it.)
        __shared__ typename Raw::type shared_rows[kPosWaves * kPosRows][kWave];
        const uint32_t unit = blockIdx.x - task_wgs;
        if (unit >= T_len * CB) return;
        const uint32_t t = row_of_unit(unit, tg), kb = unit - t * CB;     // (tg.cg == CB here)
        const uint32_t cv = kb * kWave + lane, col = cv * VEC;
        const bool live = cv < CV;
        const uint32_t col_ld = live ? col : 0u;
        const uint32_t pass_rows = waves * kPosRows;
        float pos_acc[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) pos_acc[k] = 0.0f;
#pragma nounroll
        for (uint32_t b0 = 0; b0 < B; b0 += pass_rows) {
            RunInfo ri[kPosRows];
            typename Raw::type v[kPosRows];
#pragma unroll
            for (int j = 0; j < kPosRows; ++j) {
                const uint32_t b = b0 + j * waves + wave;
                const uint32_t n = (b < B ? b : B - 1) * T_len + t;
                ri[j] = info[n];
                v[j] = Raw::load(dY + (uint64_t)n * C + col_ld);
            }
#pragma unroll
            for (int j = 0; j < kPosRows; ++j) {
                const uint32_t b = b0 + j * waves + wave;
                if (b < B) {
                    shared_rows[j * waves + wave][lane] = v[j];
                    if (ri[j].R == 1 && live) {
                        float x[VEC];
                        Raw::unpack(v[j], x);
                        store_grad_row<TO, VEC>(dW, (uint64_t)ri[j].tok * C + col, x, accumulate != 0);
                    }
                }
            }
            __syncthreads();
            if (wave == 0) {
                const uint32_t rows = B - b0 < pass_rows ? B - b0 : pass_rows;
                for (uint32_t r = 0; r < rows; ++r) {           // (row b0 + r sits in slot r = j * waves + w)
                    float x[VEC];
                    Raw::unpack(shared_rows[r][lane], x);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) pos_acc[k] = b0 + r == 0 ? x[k] : pos_acc[k] + x[k];
                }
            }
#pragma unroll
            for (int j = 0; j < kPosRows; ++j) {
                const uint32_t b = b0 + j * waves + wave;
                if (b < B && ri[j].R >= 2 && ri[j].R <= kRowRun) sum_short_run<T, TO, VEC>(a, ri[j], b * T_len + t, kb, lane);
            }
            if (b0 + pass_rows < B) __syncthreads();            // (LDS is written again only if a pass follows)
        }
        if (wave == 0 && live) store_grad_row<TO, VEC>(dwpe, (uint64_t)t * C + col, pos_acc, accumulate_pos != 0);
    }
}

// The radix path's ordering is by token throughout: the run of place p is found by two
// bisections of the sorted tokens.  Also zeroes the gradient kernel's arrival counters.
__global__ void __launch_bounds__(256)
emb_run_info_kernel(const uint32_t* __restrict__ tok_s, uint32_t* order, uint32_t N, uint32_t V) {
    const uint32_t p = blockIdx.x * 256 + threadIdx.x;
    {
        const uint32_t words = (uint32_t)(order_group_tickets(N) + order_run_tickets(N));
        uint32_t* tickets = order + order_ticket_word(N);
        for (uint32_t w = p; w < words; w += gridDim.x * 256) tickets[w] = 0;
    }
    if (p >= N) return;
    const volatile uint32_t* row_s = order;
    RunInfo* info = reinterpret_cast<RunInfo*>(order + order_info_word(N));
    const uint32_t tok = tok_s[p];
    uint32_t lo = 0, hi = p;                    // first place holding tok
    while (lo < hi) { const uint32_t mid = (lo + hi) >> 1; if (tok_s[mid] < tok) lo = mid + 1; else hi = mid; }
    const uint32_t start = lo;
    lo = p + 1; hi = N;                         // first place after the run
    while (lo < hi) { const uint32_t mid = (lo + hi) >> 1; if (tok_s[mid] <= tok) lo = mid + 1; else hi = mid; }
    const uint32_t R = lo - start, j = p - start;
    // (the neighbour's word may already carry its task mark: only the row bits are read)
    const uint32_t row = row_s[p] & kRowMask;
    RunInfo ri;
    ri.tok = tok;
    ri.start = start;
    if (tok >= V) { ri.R = 0; ri.x = 0; }
    else if (R <= kSoloRun) { ri.R = j == 0 ? R : 0u; ri.x = j + 1 < R ? row_s[p + 1] & kRowMask : kNoRow; }
    else { ri.R = R; ri.x = j; }
    if (tok < V && task_marks(j, R) != 0) order[p] = row | task_marks(j, R);
    info[row] = ri;
}

// dwpe[t, c] (+)= sum_b dY[b, t, c], b ascending
template <typename T, typename TO, int VEC>
__global__ void __launch_bounds__(256)
pos_grad_kernel(const T* __restrict__ dY, TO* dwpe, uint32_t B, uint64_t TCV, uint64_t TC, int accumulate) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= TCV) return;
    const uint64_t off = idx * VEC;
    // eight rows of the batch in flight (the adds stay in ascending b); the rows past the last
    // are read from the last one, so that no load sits behind a branch
    typedef RawVec<T, VEC> Raw;
    float acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
#pragma nounroll
    for (uint32_t b0 = 0; b0 < B; b0 += kRowBatch) {
        typename Raw::type v[kRowBatch];
#pragma unroll
        for (int q = 0; q < kRowBatch; ++q) v[q] = Raw::load(dY + (uint64_t)(b0 + q < B ? b0 + q : B - 1) * TC + off);
#pragma unroll
        for (int q = 0; q < kRowBatch; ++q) {
            if (b0 + q < B) {
                float x[VEC];
                Raw::unpack(v[q], x);
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k] = b0 + q == 0 ? x[k] : acc[k] + x[k];
            }
        }
    }
    store_grad_row<TO, VEC>(dwpe, off, acc, accumulate != 0);
}

// Scratch of the ordering step: input key / value arrays of the radix path (the
// grouping sort uses the same bytes as N 64-bit spill slots) and rocPRIM's temp.
struct SortPlan {
    uint64_t off_keys_in, off_vals_in, off_keys_out, off_temp, temp_bytes, total;
};

int plan_sort(uint64_t N, uint32_t V, SortPlan* p) {
    size_t temp = 0;
    uint32_t* nil = nullptr;
    int bits = 1;
    while ((1ull << bits) <= V) ++bits;  // keys run up to the sentinel V
    hipError_t err = rocprim::radix_sort_pairs(nullptr, temp, nil, nil, nil, nil, (size_t)N, 0u,
                                               (unsigned)bits, (hipStream_t)0, false);
    if (err != hipSuccess) return check_hip(err, "radix sort temp-size query");
    uint64_t o = 0;
    // keys_in and vals_in are adjacent: the grouping sort uses the pair as N 64-bit spill slots
    p->off_keys_in = o;  o += align256(N * 4);
    p->off_vals_in = o;  o += align256(N * 4);
    p->off_keys_out = o; o += align256(N * 4);     // the sorted tokens (radix path)
    p->off_temp = o;     o += align256(temp);
    p->temp_bytes = temp;
    p->total = o;
    return AGRAD_OK;
}

// bytes of the order buffer (see order_words)
inline uint64_t order_bytes(uint64_t N) { return align256(order_words(N) * 4); }

// fp32 partial rows of the long runs: one per chunk, one per group of chunks
inline uint64_t partial_rows(uint64_t N) { return N / kChunkRows + 1 + N / (kChunkRows * kGroupChunks) + 1; }

template <typename T, typename TO = T>
int embedding_sum_typed(hipStream_t s, uint32_t* order, const T* dY, TO* dW, float* part, uint32_t N, uint32_t C,
                        uint32_t V, uint32_t flags, TO* dwpe, uint32_t B, uint32_t T_len) {
    const int acc = (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0;
    const int acc_pos = (flags & AGRAD_ACC_PARAM_GRAD2) ? 1 : 0;
    constexpr int WIDE = WideVec<T>::value;
    // (a bf16 row under an fp32 upstream moves 8 bytes per vector: 8-byte alignment is implied by 16)
    const bool wide = C % WIDE == 0 && aligned16(dY) && aligned16(dW) && (!dwpe || aligned16(dwpe));
    const uint32_t CV = wide ? C / WIDE : C;
    const uint32_t CB = (CV + kWave - 1) / kWave;               // column blocks: a wave's worth of vectors each
    // workgroups: the tasks' (a span of row_s[] each); then four rows each -- or, with a position
    // table, one position and column block each, with a wave per row of the batch
    const uint32_t waves = dwpe ? (B < (uint32_t)kPosWaves ? B : (uint32_t)kPosWaves) : kRowSumWaves;
    // Column blocks of a row per wave: one, while that starts no more than kRowWavesEasy waves
    // (a wave that takes a whole wide row alone moves single rows 3 to 10 % slower); beyond, as
    // many as bring the count down to that -- a wave with nothing to do costs about 0.08 ns
    // of the call, and they run after the waves that have.
    int KW = 1;
    if (wide && !dwpe)
        while (KW < kRowBlocksMax && KW < (int)CB && (uint64_t)N * ((CB + KW - 1) / KW) > kRowWavesEasy) KW *= 2;
    const uint32_t CG = (CB + KW - 1) / KW;
    const TaskGrid tg = task_grid(N, CB, waves, KW == 1 ? kBigTaskSpan : kTaskSpan, CG);
    const uint64_t task_wgs = (uint64_t)tg.big_wgs + tg.wgs;
    const uint64_t row_wgs = dwpe ? (uint64_t)T_len * CB : ((uint64_t)N * CG + waves - 1) / waves;
    if (task_wgs + row_wgs >= 0x7fffffffull || (uint64_t)N * CB >= 0xffffff00ull)
        return set_error(AGRAD_EINVAL, "embedding backward: %u rows of %u columns are too many", N, C);
    const uint32_t grid = (uint32_t)(task_wgs + row_wgs);
    const uint32_t block = waves * kWave;
#define AGRAD_ROW_SUM(VEC, KW, POS) \
    hipLaunchKernelGGL((emb_row_sum_kernel<T, TO, VEC, KW, POS>), dim3(grid), dim3(block), 0, s, order, \
                       order + order_ticket_word(N), dY, dW, dwpe, part, N, C, CV, CB, V, T_len, B, \
                       acc, acc_pos, tg)
    if (dwpe) {
        if (wide) AGRAD_ROW_SUM(WIDE, 1, true); else AGRAD_ROW_SUM(1, 1, true);
    } else if (!wide) {
        AGRAD_ROW_SUM(1, 1, false);
    } else {
        switch (KW) {
            case 1: AGRAD_ROW_SUM(WIDE, 1, false); break;
            case 2: AGRAD_ROW_SUM(WIDE, 2, false); break;
            case 4: AGRAD_ROW_SUM(WIDE, 4, false); break;
            default: AGRAD_ROW_SUM(WIDE, kRowBlocksMax, false); break;
        }
    }
#undef AGRAD_ROW_SUM
    return check_hip(hipGetLastError(), "embedding backward launch");
}

int check_embedding_sizes(const char* what, uint64_t N, uint32_t V) {
    if (N >= 0x40000000ull) return set_error(AGRAD_EINVAL, "%s: too many rows", what);
    if (V == 0 || V >= 0x7fffffffu) return set_error(AGRAD_EINVAL, "%s: bad vocabulary size %u", what, V);
    return AGRAD_OK;
}

}  // namespace

uint64_t embedding_order_bytes(uint64_t N) { return N ? order_bytes(N) : 0; }

uint64_t embedding_sort_workspace_bytes(uint64_t N, uint32_t V) {
    if (N == 0) return 0;
    SortPlan p;
    if (plan_sort(N, V, &p) != AGRAD_OK) return 0;
    return p.total;
}

// order[0 .. N) = rows (with the task marks in their top two bits), each token's rows
// adjacent and ascending; then (from the next multiple of four words) a RunInfo per row;
// then the gradient kernel's arrival counters, zeroed
int launch_embedding_sort(hipStream_t s, const int32_t* ids, uint32_t* order, void* workspace,
                          uint64_t workspace_bytes, uint64_t N, uint32_t V, int* err_flag) {
    if (N == 0) return AGRAD_OK;
    if (int rc = check_embedding_sizes("embedding sort", N, V)) return rc;
    if (ids == nullptr || order == nullptr) return set_error(AGRAD_EINVAL, "embedding sort: null operand");
    SortPlan p;
    if (int rc = plan_sort(N, V, &p)) return rc;
    if (workspace == nullptr || workspace_bytes < p.total)
        return set_error(AGRAD_EWORKSPACE, "embedding sort: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)p.total);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
        return set_error(AGRAD_EINVAL, "embedding sort: workspace must be 256-byte aligned");
    if ((reinterpret_cast<uintptr_t>(order) & 15u) != 0)
        return set_error(AGRAD_EINVAL, "embedding sort: the order buffer must be 16-byte aligned");
    uint8_t* ws = (uint8_t*)workspace;
    const uint32_t n = (uint32_t)N;
    if (n <= kGroupSortMaxN) {
        static_assert(sizeof(unsigned long long) == 2 * sizeof(uint32_t), "spill layout");
        unsigned long long* spill = reinterpret_cast<unsigned long long*>(ws + p.off_keys_in);
        const uint32_t log2G = group_sort_log2g(n);
        hipLaunchKernelGGL(emb_group_sort_kernel, dim3(1u << log2G), dim3(kSortBlock), 0, s, ids, order,
                           spill, n, V, log2G, err_flag);
        return check_hip(hipGetLastError(), "embedding sort launch");
    }
    if (is_capturing())
        return set_error(AGRAD_EINVAL, "an embedding gradient over %u rows uses the library radix sort, which is not "
                         "recorded into graphs (up to %u rows are)", n, kGroupSortMaxN);
    uint32_t* keys_in = (uint32_t*)(ws + p.off_keys_in);
    uint32_t* vals_in = (uint32_t*)(ws + p.off_vals_in);
    hipLaunchKernelGGL(emb_prepare_kernel, dim3((n + 255) / 256), dim3(256), 0, s, ids, keys_in, vals_in, n, V, err_flag);
    int bits = 1;
    while ((1ull << bits) <= V) ++bits;
    size_t temp = p.temp_bytes;
    uint32_t* tok_s = (uint32_t*)(ws + p.off_keys_out);
    hipError_t err = rocprim::radix_sort_pairs(ws + p.off_temp, temp, keys_in, tok_s, vals_in, order,
                                               (size_t)N, 0u, (unsigned)bits, s, false);
    if (int rc = check_hip(err, "radix sort")) return rc;
    hipLaunchKernelGGL(emb_run_info_kernel, dim3((n + 255) / 256), dim3(256), 0, s, tok_s, order, n, V);
    return check_hip(hipGetLastError(), "embedding order launch");
}

// order = the ids' ordering for the later gradient and, in the same launch where the shapes
// allow, zero_dst[0 .. zero_bytes) = 0 (the table's gradient, cleared before the backward pass)
int launch_embedding_order(hipStream_t s, const int32_t* ids, uint32_t* order, void* sort_workspace,
                           uint64_t sort_workspace_bytes, uint64_t N, uint32_t V, void* zero_dst, uint64_t zero_bytes,
                           int* err_flag) {
    if (zero_dst == nullptr) zero_bytes = 0;
    const uint64_t vectors = zero_bytes / 16;
    const bool fused = N > 0 && N <= kGroupSortMaxN && zero_bytes > 0 && zero_bytes % 16 == 0 && aligned16(zero_dst) &&
                       vectors / kSortBlock < 0x7ff00000ull;
    if (!fused) {
        if (zero_bytes) if (int rc = launch_fill(s, zero_dst, 0, 1, zero_bytes)) return rc;
        return launch_embedding_sort(s, ids, order, sort_workspace, sort_workspace_bytes, N, V, err_flag);
    }
    if (int rc = check_embedding_sizes("embedding order", N, V)) return rc;
    if (ids == nullptr || order == nullptr) return set_error(AGRAD_EINVAL, "embedding order: null operand");
    SortPlan p;
    if (int rc = plan_sort(N, V, &p)) return rc;
    if (sort_workspace == nullptr || sort_workspace_bytes < p.total)
        return set_error(AGRAD_EWORKSPACE, "embedding order: workspace %llu < %llu bytes",
                         (unsigned long long)sort_workspace_bytes, (unsigned long long)p.total);
    if ((reinterpret_cast<uintptr_t>(sort_workspace) & 255u) != 0)
        return set_error(AGRAD_EINVAL, "embedding order: workspace must be 256-byte aligned");
    if ((reinterpret_cast<uintptr_t>(order) & 15u) != 0)
        return set_error(AGRAD_EINVAL, "embedding order: the order buffer must be 16-byte aligned");
    unsigned long long* spill = reinterpret_cast<unsigned long long*>((uint8_t*)sort_workspace + p.off_keys_in);
    const uint32_t n = (uint32_t)N, log2G = group_sort_log2g(n);
    const uint32_t grid = (1u << log2G) + (uint32_t)((vectors + kSortBlock - 1) / kSortBlock);
    hipLaunchKernelGGL(fill_order_kernel, dim3(grid), dim3(kSortBlock), kFillOrderIdleLds, s, ids, order, spill, n, V, log2G,
                       err_flag, reinterpret_cast<u32x4*>(zero_dst), vectors);
    return check_hip(hipGetLastError(), "embedding order launch");
}

// out = W[ids] (+ wpe) and order = the ids' ordering for the later gradient
int launch_gather_fwd_sorted(hipStream_t s, int dtype, const int32_t* ids, const void* W, const void* wpe,
                             void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V, uint32_t* order,
                             void* sort_workspace, uint64_t sort_workspace_bytes, int* err_flag, int32_t* kept) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "gather: unknown dtype %d", dtype);
    if (N == 0) return AGRAD_OK;
    if (order == nullptr) return set_error(AGRAD_EINVAL, "gather: null order buffer");
    if (kept != nullptr && (const int32_t*)kept == ids) return set_error(AGRAD_EINVAL, "gather: the kept ids may not be the ids");
    const uint32_t esz = dtype_size(dtype);
    const uint32_t per16 = 16 / esz;
    const bool wide = C > 0 && C % per16 == 0 && W != nullptr && out != nullptr && aligned16(W) && aligned16(out) &&
                      (!wpe || aligned16(wpe));
    const uint64_t total_vec = wide ? N * (C / per16) : 0;
    const bool fused = wide && N <= kGroupSortMaxN && total_vec < 0xff000000ull &&
                       ids != nullptr && (wpe == nullptr || T > 0);
    if (!fused) {
        if (int rc = launch_embedding_sort(s, ids, order, sort_workspace, sort_workspace_bytes, N, V, err_flag)) return rc;
        if (kept != nullptr) {
            if (ids == nullptr) return set_error(AGRAD_EINVAL, "gather: null ids");
            if (int rc = launch_copy(s, ids, kept, N * 4)) return rc;
        }
        if (C == 0) return AGRAD_OK;
        return launch_gather_fwd(s, dtype, ids, W, wpe, out, N, T, C, V, err_flag);
    }
    if (int rc = check_embedding_sizes("gather", N, V)) return rc;
    SortPlan p;
    if (int rc = plan_sort(N, V, &p)) return rc;
    if (sort_workspace == nullptr || sort_workspace_bytes < p.total)
        return set_error(AGRAD_EWORKSPACE, "gather: sort workspace %llu < %llu bytes",
                         (unsigned long long)sort_workspace_bytes, (unsigned long long)p.total);
    if ((reinterpret_cast<uintptr_t>(sort_workspace) & 255u) != 0)
        return set_error(AGRAD_EINVAL, "gather: sort workspace must be 256-byte aligned");
    unsigned long long* spill = reinterpret_cast<unsigned long long*>((uint8_t*)sort_workspace + p.off_keys_in);
    const uint32_t n = (uint32_t)N, CV = C / per16, total = (uint32_t)total_vec;
    const uint32_t log2G = group_sort_log2g(n);
    const uint32_t grid = (1u << log2G) + (total + kSortBlock * kGatherPerThread - 1) / (kSortBlock * kGatherPerThread);
    if ((reinterpret_cast<uintptr_t>(order) & 15u) != 0)
        return set_error(AGRAD_EINVAL, "gather: the order buffer must be 16-byte aligned");
    if (wpe == nullptr) {
        hipLaunchKernelGGL((gather_sort_kernel<float, 4, true>), dim3(grid), dim3(kSortBlock), 0, s, ids, (const float*)W,
                           (const float*)nullptr, (float*)out, total, CV, C, T ? T : 1u, V, order, spill, n, log2G, err_flag, kept);
    } else if (dtype == AGRAD_F32) {
        hipLaunchKernelGGL((gather_sort_kernel<float, 4, false>), dim3(grid), dim3(kSortBlock), 0, s, ids, (const float*)W,
                           (const float*)wpe, (float*)out, total, CV, C, T, V, order, spill, n, log2G, err_flag, kept);
    } else {
        hipLaunchKernelGGL((gather_sort_kernel<bf16_t, 8, false>), dim3(grid), dim3(kSortBlock), 0, s, ids, (const bf16_t*)W,
                           (const bf16_t*)wpe, (bf16_t*)out, total, CV, C, T, V, order, spill, n, log2G, err_flag, kept);
    }
    return check_hip(hipGetLastError(), "gather launch");
}

uint64_t embedding_bwd_sorted_workspace_bytes(uint64_t N, uint32_t C) {
    if (N == 0 || C == 0) return 0;
    return align256(partial_rows(N) * C * 4);       // the long runs' partial rows
}

int launch_embedding_bwd_sorted(hipStream_t s, int dtype, uint32_t* order, const void* dY, void* dW,
                                void* dwpe, void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t T,
                                uint32_t C, uint32_t V, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "embedding backward: unknown dtype %d", dtype);
    if (N == 0 || C == 0) return AGRAD_OK;
    if (int rc = check_embedding_sizes("embedding backward", N, V)) return rc;
    if (order == nullptr || dY == nullptr || dW == nullptr) return set_error(AGRAD_EINVAL, "embedding backward: null operand");
    const uint64_t need = embedding_bwd_sorted_workspace_bytes(N, C);
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "embedding backward: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if ((reinterpret_cast<uintptr_t>(workspace) & 15u) != 0)
        return set_error(AGRAD_EINVAL, "embedding backward: workspace must be 16-byte aligned");
    float* part = (float*)workspace;
    if ((reinterpret_cast<uintptr_t>(order) & 15u) != 0)
        return set_error(AGRAD_EINVAL, "embedding backward: the order buffer must be 16-byte aligned");
    uint32_t B = 0;
    if (dwpe != nullptr) {
        if (T == 0 || N % T != 0) return set_error(AGRAD_EINVAL, "embedding backward: %llu rows are not a whole number of sequences of %u", (unsigned long long)N, T);
        B = (uint32_t)(N / T);
    }
    if (flags & AGRAD_PARAM_GRAD_BF16) {
        if (dtype != AGRAD_F32) return set_error(AGRAD_EINVAL, "embedding backward: AGRAD_PARAM_GRAD_BF16 goes with an fp32 upstream gradient");
        return embedding_sum_typed<float, bf16_t>(s, order, (const float*)dY, (bf16_t*)dW, part, (uint32_t)N, C, V, flags, (bf16_t*)dwpe, B, T);
    }
    if (dtype == AGRAD_F32)
        return embedding_sum_typed<float>(s, order, (const float*)dY, (float*)dW, part, (uint32_t)N, C, V, flags, (float*)dwpe, B, T);
    return embedding_sum_typed<bf16_t>(s, order, (const bf16_t*)dY, (bf16_t*)dW, part, (uint32_t)N, C, V, flags, (bf16_t*)dwpe, B, T);
}

int launch_gather_fwd(hipStream_t s, int dtype, const int32_t* ids, const void* W, const void* wpe,
                      void* out, uint64_t N, uint32_t T, uint32_t C, uint32_t V, int* err_flag) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "gather: unknown dtype %d", dtype);
    if (N == 0 || C == 0) return AGRAD_OK;
    if (ids == nullptr || W == nullptr || out == nullptr) return set_error(AGRAD_EINVAL, "gather: null operand");
    if (wpe != nullptr && T == 0) return set_error(AGRAD_EINVAL, "gather: position table needs T > 0");
    if (T == 0) T = 1;
    const uint32_t esz = dtype_size(dtype);
    const uint32_t per16 = 16 / esz;
    const bool wide = C % per16 == 0 && aligned16(W) && aligned16(out) && (!wpe || aligned16(wpe));
    const uint64_t total_vec = wide ? N * (C / per16) : 0;
    if (wide && total_vec < 0xffff0000ull) {
        const uint32_t CV = C / per16;
        const uint32_t total = (uint32_t)total_vec;
        constexpr int UNROLL = 1;
        const uint32_t grid = (total + kGatherBlock * UNROLL - 1) / (kGatherBlock * UNROLL);
        if (wpe == nullptr) {
            hipLaunchKernelGGL((gather_rows16_kernel<UNROLL>), dim3(grid), dim3(kGatherBlock), 0, s, ids,
                               (const u32x4*)W, (u32x4*)out, total, CV, V, err_flag);
        } else if (dtype == AGRAD_F32) {
            hipLaunchKernelGGL((gather_fwd_kernel<float, 4, UNROLL>), dim3(grid), dim3(kGatherBlock), 0, s, ids,
                               (const float*)W, (const float*)wpe, (float*)out, total, CV, C, T, V, err_flag);
        } else {
            hipLaunchKernelGGL((gather_fwd_kernel<bf16_t, 8, UNROLL>), dim3(grid), dim3(kGatherBlock), 0, s, ids,
                               (const bf16_t*)W, (const bf16_t*)wpe, (bf16_t*)out, total, CV, C, T, V, err_flag);
        }
    } else {
        const uint64_t total = N * C;
        const uint64_t grid = (total + kGatherBlock - 1) / kGatherBlock;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "gather: output too large");
        if (dtype == AGRAD_F32)
            hipLaunchKernelGGL((gather_scalar_kernel<float>), dim3((uint32_t)grid), dim3(kGatherBlock), 0, s, ids,
                               (const float*)W, (const float*)wpe, (float*)out, total, C, T, V, err_flag);
        else
            hipLaunchKernelGGL((gather_scalar_kernel<bf16_t>), dim3((uint32_t)grid), dim3(kGatherBlock), 0, s, ids,
                               (const bf16_t*)W, (const bf16_t*)wpe, (bf16_t*)out, total, C, T, V, err_flag);
    }
    return check_hip(hipGetLastError(), "gather launch");
}

int launch_embedding_grad_reset(hipStream_t s, int dtype, const int32_t* rows, uint64_t N, void* dW,
                                uint32_t C, uint32_t V) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "embedding grad reset: unknown dtype %d", dtype);
    if (N == 0 || C == 0 || V == 0) return AGRAD_OK;
    if (rows == nullptr || dW == nullptr) return set_error(AGRAD_EINVAL, "embedding grad reset: null operand");
    const uint32_t esz = dtype_size(dtype);
    const uint32_t per16 = 16 / esz;
    const bool wide = C % per16 == 0 && aligned16(dW);
    const uint64_t total_vec = wide ? N * (C / per16) : 0;
    if (wide && total_vec < 0xffff0000ull) {
        const uint32_t total = (uint32_t)total_vec;
        const uint32_t grid = (total + kGatherBlock - 1) / kGatherBlock;
        hipLaunchKernelGGL(zero_rows16_kernel, dim3(grid), dim3(kGatherBlock), 0, s, rows, (u32x4*)dW, total,
                           C / per16, V);
    } else {
        const uint64_t total = N * C;
        const uint64_t grid = (total + kGatherBlock - 1) / kGatherBlock;
        if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "embedding grad reset: too many items");
        if (dtype == AGRAD_F32)
            hipLaunchKernelGGL((zero_rows_scalar_kernel<uint32_t>), dim3((uint32_t)grid), dim3(kGatherBlock), 0, s,
                               rows, (uint32_t*)dW, total, C, V);
        else
            hipLaunchKernelGGL((zero_rows_scalar_kernel<uint16_t>), dim3((uint32_t)grid), dim3(kGatherBlock), 0, s,
                               rows, (uint16_t*)dW, total, C, V);
    }
    return check_hip(hipGetLastError(), "embedding grad reset launch");
}

// one workspace for the unsorted entry point: [order | sort scratch | partial rows]
uint64_t embedding_bwd_workspace_bytes(uint64_t N, uint32_t C, uint32_t V, int dtype) {
    (void)dtype;
    if (N == 0 || C == 0) return 0;
    return order_bytes(N) + embedding_sort_workspace_bytes(N, V) + embedding_bwd_sorted_workspace_bytes(N, C);
}

int launch_embedding_bwd(hipStream_t s, int dtype, const int32_t* ids, const void* dY, void* dW,
                         void* workspace, uint64_t workspace_bytes, uint64_t N, uint32_t C,
                         uint32_t V, uint32_t flags, int* err_flag) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "embedding backward: unknown dtype %d", dtype);
    if (N == 0 || C == 0) return AGRAD_OK;
    if (ids == nullptr || dY == nullptr || dW == nullptr) return set_error(AGRAD_EINVAL, "embedding backward: null operand");
    if (int rc = check_embedding_sizes("embedding backward", N, V)) return rc;
    const uint64_t sort_bytes = embedding_sort_workspace_bytes(N, V);
    const uint64_t part_bytes = embedding_bwd_sorted_workspace_bytes(N, C);
    const uint64_t need = order_bytes(N) + sort_bytes + part_bytes;
    if (workspace == nullptr || workspace_bytes < need)
        return set_error(AGRAD_EWORKSPACE, "embedding backward: workspace %llu < %llu bytes",
                         (unsigned long long)workspace_bytes, (unsigned long long)need);
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
        return set_error(AGRAD_EINVAL, "embedding backward: workspace must be 256-byte aligned");
    uint8_t* ws = (uint8_t*)workspace;
    uint32_t* order = (uint32_t*)ws;
    if (int rc = launch_embedding_sort(s, ids, order, ws + order_bytes(N), sort_bytes, N, V, err_flag)) return rc;
    return launch_embedding_bwd_sorted(s, dtype, order, dY, dW, nullptr, ws + order_bytes(N) + sort_bytes, part_bytes, N, 0,
                                       C, V, flags);
}

int launch_pos_embedding_bwd(hipStream_t s, int dtype, const void* dY, void* dwpe, uint32_t B,
                             uint32_t T, uint32_t C, uint32_t flags) {
    if (dtype != AGRAD_F32 && dtype != AGRAD_BF16) return set_error(AGRAD_EINVAL, "position grad: unknown dtype %d", dtype);
    if (B == 0 || T == 0 || C == 0) return AGRAD_OK;
    if (dY == nullptr || dwpe == nullptr) return set_error(AGRAD_EINVAL, "position grad: null operand");
    const int acc = (flags & AGRAD_ACC_PARAM_GRAD) ? 1 : 0;
    const uint64_t TC = (uint64_t)T * C;
    const uint32_t per16 = 16 / dtype_size(dtype);
    const bool wide = TC % per16 == 0 && aligned16(dY) && aligned16(dwpe) &&
                      ((TC * dtype_size(dtype)) % 16 == 0);
    const uint64_t n = wide ? TC / per16 : TC;
    const uint64_t grid = (n + 255) / 256;
    if (grid > 0x7fffffffull) return set_error(AGRAD_EINVAL, "position grad: table too large");
    if (flags & AGRAD_PARAM_GRAD_BF16) {        // fp32 rows summed into a bf16 table (bias_grad_reduce_bf16, metal_ops.metal:12101)
        if (dtype != AGRAD_F32) return set_error(AGRAD_EINVAL, "position grad: AGRAD_PARAM_GRAD_BF16 goes with an fp32 upstream gradient");
        if (wide) hipLaunchKernelGGL((pos_grad_kernel<float, bf16_t, 4>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)dY, (bf16_t*)dwpe, B, n, TC, acc);
        else hipLaunchKernelGGL((pos_grad_kernel<float, bf16_t, 1>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)dY, (bf16_t*)dwpe, B, n, TC, acc);
    } else if (dtype == AGRAD_F32) {
        if (wide) hipLaunchKernelGGL((pos_grad_kernel<float, float, 4>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)dY, (float*)dwpe, B, n, TC, acc);
        else hipLaunchKernelGGL((pos_grad_kernel<float, float, 1>), dim3((uint32_t)grid), dim3(256), 0, s, (const float*)dY, (float*)dwpe, B, n, TC, acc);
    } else {
        if (wide) hipLaunchKernelGGL((pos_grad_kernel<bf16_t, bf16_t, 8>), dim3((uint32_t)grid), dim3(256), 0, s, (const bf16_t*)dY, (bf16_t*)dwpe, B, n, TC, acc);
        else hipLaunchKernelGGL((pos_grad_kernel<bf16_t, bf16_t, 1>), dim3((uint32_t)grid), dim3(256), 0, s, (const bf16_t*)dY, (bf16_t*)dwpe, B, n, TC, acc);
    }
    return check_hip(hipGetLastError(), "position grad launch");
}

}  // namespace agrad
