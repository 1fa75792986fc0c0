// NN-Descent step as a local join around the picked neighbour (K = 64).
//
// The reference's step (index.cu:156-376) lets node u meet the forward list N(v) and the reverse list R(v) of
// each neighbour v it picks: one pivot against many rows, every row gathered for one evaluation. Here the same
// pairs are formed the other way round: all pickers of one v are the ROWS of a tile (32 at a time), N(v) and R(v)
// are its COLUMNS (up to 128), every row of the tile is gathered once and meets every column:
//   dense part   32 x 128 x 1024 contraction on the matrix cores (fp32 MFMA 32x32x2; eight waves: the 32-column
//                blocks that exist x equal parts of the dimensions)
//   sparse part  eight picker rows at a time in an LDS rank table that the column rows probe (apoe_ranktab.h); a
//                wave keeps the pairs of its sixteen columns in registers, so a row is read from memory once per tile
//   insertion    a pair closer than the row's last list entry (and not in that list) is offered to the row node
//                with a 64-bit atomicMin on slot hash(id) of its proposal row: (distance, id), the smallest wins;
//                in symmetric mode the pair is offered to the column node as well (both endpoints, as the classic
//                NN-Descent join does; the reference's step updates u only)
// and a second kernel merges every node's proposals into its sorted list (wave-level rank merge, new before old
// on equal distance, index.cu:333-351) and registers the entries that are new in a list with their nodes' reverse
// lists (slot = registrations so far, modulo K; every registration a 64-bit atomicMin, so beyond K the closer entry
// of a slot stays, index.cu:362-372). Lists are read as the step found them and proposals are minima under a total
// order, so the lists a step leaves do not depend on the order in which tiles run. The reverse lists are append-only
// over the steps: a node that later drops v stays in R(v) (a stale column costs one evaluation and can never enter a
// list wrongly: its distance is computed again), and while a list has fewer than K registrations its content does
// not depend on the order either; beyond K, which entries share a slot follows the arrival order of the counter.
#include <hipcub/hipcub.hpp>

#include <algorithm>

#include "apoe_gram.h"
#include "apoe_internal.h"
#include "apoe_ranktab.h"

namespace apoe {

constexpr int JT_ROWS = 32;
constexpr int JT_COLS = 128;
constexpr int JT_THREADS = 512;
constexpr int JT_STRIDE = JT_COLS + 1;
constexpr int JT_SEEN = 512; // slots of the id set that removes repeated columns
// The kernels below are built for lists of KK = 64 and KK = 128 entries (index.cu:6 has K 64; a degree above 32 needs
// 2 * degree <= K there, index.cu:702). A node has 2 * KK proposal slots: two proposals of one step whose ids hash to one
// slot are one proposal, the closer one. With KK = 128 the columns of a picked node (its list and its reverse list, up to
// 256) are two tiles: the list, then what the reverse list adds to it.
constexpr int JOIN_PICKS = 4; // index.cu:157,171-181
constexpr int JOIN_COUNT_PARTS = 256, JOIN_COUNT_AT = 8; // partial insertion counters in the step's work array, one per 64-byte line, from word 8
constexpr int JT_BATCH = 2;   // column rows a wave probes together
constexpr int JT_OWN = JT_COLS / (JT_THREADS / WAVE); // columns of a tile that one wave owns: their pairs stay in its registers

__device__ __forceinline__ uint32_t prop_slot(uint32_t id, uint32_t P) { return (uint32_t)(mix64(id) >> 40) & (P - 1); }

__device__ __forceinline__ float join_key_dist(unsigned long long key) {
    uint32_t u = (uint32_t)(key >> 32);
    u ^= (u >> 31) ? 0x80000000u : 0xFFFFFFFFu;
    return __uint_as_float(u);
}

// One wave per node: the picking rule of the expansion step (group g takes the first unsampled slot >= g; none
// left: slot 0 again), the picked neighbours counted per target.
template <uint32_t KK>
__global__ __launch_bounds__(256) void join_pick_kernel(uint32_t n, uint32_t* ids, uint32_t* picks, uint32_t* pick_cnt) {
    constexpr int KL = KK / WAVE; // list entries per lane: entry e sits in register e / 64 of lane e % 64
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const uint32_t u = blockIdx.x * 4 + wave;
    if (u >= n) return;
    const size_t base = (size_t)u * KK;
    uint32_t own[KL];
    uint64_t m0[KL];
#pragma unroll
    for (int k = 0; k < KL; k++) {
        own[k] = ids[base + k * WAVE + lane];
        m0[k] = __ballot(!(own[k] & FLAG));
    }
    uint32_t slot[JOIN_PICKS], mine = EMPTY; // everything here is wave-uniform except `mine`: lane g keeps the g-th pick
#pragma unroll
    for (int g = 0; g < JOIN_PICKS; g++) {
        uint32_t s = 0;
        bool found = false;
#pragma unroll
        for (int k = 0; k < KL; k++) {
            const uint64_t a = k == 0 ? m0[0] & ~((1ull << g) - 1) : m0[k];
            if (!found && a) {
                s = k * WAVE + __ffsll((unsigned long long)a) - 1;
                m0[k] &= ~(1ull << (s % WAVE));
                if ((uint32_t)lane == s % WAVE) ids[base + s] = own[k] | FLAG;
                found = true;
            }
        }
        slot[g] = s;
        bool dup = false;
#pragma unroll
        for (int t = 0; t < g; t++) dup |= slot[t] == s;
        uint32_t v = 0;
#pragma unroll
        for (int k = 0; k < KL; k++)
            if (s / WAVE == (uint32_t)k) v = (uint32_t)__builtin_amdgcn_readlane((int)own[k], s % WAVE) & ~FLAG;
        if (dup || v >= n) v = EMPTY;
        if (lane == g) mine = v;
    }
    if (lane < JOIN_PICKS) {
        picks[(size_t)u * JOIN_PICKS + lane] = mine;
        if (mine != EMPTY) atomicAdd(&pick_cnt[mine], 1u);
    }
}

__global__ __launch_bounds__(256) void join_tile_count_kernel(uint32_t n, uint32_t halves, const uint32_t* pick_cnt, uint32_t* tile_cnt) {
    const uint32_t v = blockIdx.x * blockDim.x + threadIdx.x;
    if (v < n) tile_cnt[v] = (pick_cnt[v] + JT_ROWS - 1) / JT_ROWS * halves;
    if (v == n) tile_cnt[v] = 0;
}

// The pickers of every v side by side, and the node of every tile.
__global__ __launch_bounds__(256) void join_fill_kernel(uint32_t n, uint32_t halves, const uint32_t* picks, const uint32_t* pick_off, const uint32_t* tile_off,
                                                        uint32_t* pick_fill, uint32_t* pick_src, uint32_t* tile_v) {
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (uint64_t)n * JOIN_PICKS) return;
    const uint32_t v = picks[t];
    if (v == EMPTY) return;
    const uint32_t k = atomicAdd(&pick_fill[v], 1u);
    pick_src[pick_off[v] + k] = (uint32_t)(t / JOIN_PICKS);
    if (k % JT_ROWS == 0)
        for (uint32_t h = 0; h < halves; h++) tile_v[tile_off[v] + k / JT_ROWS * halves + h] = v;
}

struct JoinArgs {
    CorpusView C;
    float dense_mul;
    uint32_t n, P, symmetric;
    const uint32_t* ids;
    const float* dist;
    const unsigned long long* rev;
    const uint32_t *pick_off, *pick_src, *tile_off, *tile_v;
    unsigned long long* prop;
    unsigned long long* work; // [0] next tile, [1] pairs evaluated, [2] rows gathered, [3] a row did not fit the table
    uint32_t index_bits, slot_cap, span;
};

struct JoinLds {
    uint32_t G, tab, row_list, rowptr, rownnz, row_id, col_id, row_worst, col_worst, seen, scan, ctl, total;
    // KK = 64: the picker rows' own lists have an array of their own; KK = 128: they are loaded when the products are done and
    // sit behind the rank table, inside the region that staged the dense rows before
    __host__ __device__ JoinLds(uint32_t index_bits, uint32_t slot_cap, bool narrow, uint32_t KK = 64) {
        uint32_t o = 0;
        G = o; o += JT_ROWS * JT_STRIDE * 4;
        row_list = o; o += KK == 64 ? JT_ROWS * 64 * 4 : 0;
        o = (o + 7) & ~7u;
        rowptr = o; o += (JT_ROWS + JT_COLS) * 8;
        rownnz = o; o += (JT_ROWS + JT_COLS) * 4;
        row_id = o; o += JT_ROWS * 4;
        col_id = o; o += JT_COLS * 4;
        row_worst = o; o += JT_ROWS * 4;
        col_worst = o; o += JT_COLS * 4;
        seen = o; o += JT_SEEN * 4;
        scan = o; o += 20 * 4;
        ctl = o; o += 8 * 4;
        o = (o + 15) & ~15u;
        // the rank table of the sparse part; before it is built, the same bytes hold the dense parts of the picker rows
        uint32_t table = (RankTabLds(index_bits, slot_cap, narrow).total + 15) & ~15u;
        const uint32_t rows = (uint32_t)(JT_ROWS * DENSE_BYTES);
        if (KK != 64) { row_list = o + table; table += JT_ROWS * KK * 4; }
        tab = o; o += table > rows ? table : rows;
        total = o;
    }
};

// Dense part of a tile on v_mfma_f32_16x16x4_f32. A wave owns 16 columns and a range of 16-float blocks of the
// dimensions; the picker rows come from LDS (`A`: row r, float4 c at A[r * 256 + (c ^ (r & 7))] -- the swizzle spreads
// the sixteen rows of a read over the banks without padding), the column rows straight from memory. Lane (j, g), j =
// lane % 16, g = lane / 16, supplies float4 number 4 b + g of block b for row j (A operand) and for column j (B
// operand): the four multiplies of a block take one component each, so k-slot g of multiply c stands for dimension
// 16 b + 4 g + c on both sides. RING column blocks are in flight ahead of the one being multiplied (a ring of
// registers, refilled as it is consumed). Rows 16..31 of the tile take a second accumulator fed from the same column
// registers, and only when the tile has them: a tile of at most 16 rows costs half the matrix time.
// Result: lane (j, g) holds row 4 g + e (+ 16), column j in acc0[e] (acc1[e]).
typedef float floatx4 __attribute__((ext_vector_type(4)));
template <int RING>
__device__ __forceinline__ void join_dense16(const float4* A, uint32_t nr, const float4* pb, int lane, int b_begin, int b_end, floatx4& acc0,
                                             floatx4& acc1) {
    const int j = lane & 15, g = lane >> 4;
    const uint32_t i0 = min((uint32_t)j, nr - 1), i1 = min(16u + (uint32_t)j, nr - 1);
    const float4* a0 = A + i0 * (DIM / 4);
    const float4* a1 = A + i1 * (DIM / 4);
    const uint32_t s0 = i0 & 7, s1 = i1 & 7;
    const bool two = nr > 16; // wave-uniform
    float4 ring[RING];
#pragma unroll
    for (int u = 0; u < RING; u++) ring[u] = pb[4 * (b_begin + u)];
#pragma unroll 1
    for (int b = b_begin; b < b_end; b += RING) {
        const bool more = b + RING < b_end;
#pragma unroll
        for (int u = 0; u < RING; u++) {
            const float4 bv = ring[u];
            if (more) ring[u] = pb[4 * (b + u + RING)];
            const uint32_t c = 4u * (uint32_t)(b + u) + (uint32_t)g;
            const float4 av = a0[c ^ s0];
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, bv.x, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, bv.y, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, bv.z, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, bv.w, acc0, 0, 0, 0);
            if (two) {
                const float4 aw = a1[c ^ s1];
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw.x, bv.x, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw.y, bv.y, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw.z, bv.z, acc1, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(aw.w, bv.w, acc1, 0, 0, 0);
            }
        }
    }
}

// 64 values, one per lane, in ascending order over the lanes (bitonic network, 21 exchanges).
__device__ __forceinline__ uint32_t wave_sort_u32(uint32_t v, int lane) {
#pragma unroll
    for (int k = 2; k <= WAVE; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            const uint32_t o = __shfl_xor(v, j, WAVE);
            const bool take_min = ((lane & j) == 0) == ((lane & k) == 0 || k == WAVE);
            v = take_min ? min(v, o) : max(v, o);
        }
    }
    return v;
}

// The hybrid inner products of a tile, G[r * JT_STRIDE + c] = dense_mul * <row r, column c>_dense + <row r, column c>_sparse for
// the R rows and M columns whose record addresses and shapes `rowptr` / `rownnz` hold (rows at [0, JT_ROWS), columns at
// [JT_ROWS, JT_ROWS + JT_COLS): gram_rows_gather). All JT_THREADS threads call it after a barrier behind those arrays; it
// ends with a barrier. `tabreg` = the table region of JoinLds, `unfit` = counter of rows whose terms did not fit the table.
template <bool NARROW>
__device__ __forceinline__ void tile_hybrid_ips(const CorpusView& C, float dense_mul, char* tabreg, const RankTab& T, uint32_t index_bits, uint32_t slot_cap,
                                                float* G, const unsigned long long* rowptr, const uint32_t* rownnz, uint32_t* scan, uint32_t R,
                                                uint32_t M, unsigned long long* unfit, int tid, int wave, int lane) {
    constexpr int NW = JT_THREADS / WAVE;
    // dense part: the eight waves share the 16-column blocks that exist (8, 4, 2 or 1 by the number of columns) and, for
    // each block, equal parts of the dimensions (1, 2, 4 or 8): no wave idles when a tile has few columns. The picker
    // rows are staged in the table region, which is free until the sparse part. Partial tiles are added into G in a
    // fixed order, a barrier between them.
    {
        const uint32_t nblk = M <= 16 ? 1u : M <= 32 ? 2u : M <= 64 ? 4u : 8u, parts = (uint32_t)NW / nblk;
        const uint32_t blk = (uint32_t)wave % nblk, part = (uint32_t)wave / nblk;
        const bool active = blk * 16 < M;
        const uint32_t per = (DIM / 16) / parts; // 16-float blocks of the dimensions per part: 64, 32, 16 or 8
        float4* A = reinterpret_cast<float4*>(tabreg);
        const uint32_t jcol = min(blk * 16 + (uint32_t)(lane & 15), M - 1);
        const float4* pb = reinterpret_cast<const float4*>(rowptr[JT_ROWS + jcol] - DENSE_BYTES) + (lane >> 4);
#pragma unroll 4
        for (uint32_t i = tid; i < R * (DIM / 4); i += JT_THREADS) {
            const uint32_t r = i / (DIM / 4), c = i % (DIM / 4);
            A[r * (DIM / 4) + (c ^ (r & 7))] = reinterpret_cast<const float4*>(rowptr[r] - DENSE_BYTES)[c];
        }
        __syncthreads();
        floatx4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        if (active) {
            if (per >= 16) join_dense16<16>(A, R, pb, lane, (int)(part * per), (int)((part + 1) * per), acc0, acc1);
            else join_dense16<8>(A, R, pb, lane, (int)(part * per), (int)((part + 1) * per), acc0, acc1);
        }
        auto store = [&](bool add) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float* at = &G[(4 * (lane >> 4) + e) * JT_STRIDE + blk * 16 + (lane & 15)];
                *at = add ? *at + dense_mul * acc0[e] : dense_mul * acc0[e];
                if (R > 16) {
                    float* at1 = at + 16 * JT_STRIDE;
                    *at1 = add ? *at1 + dense_mul * acc1[e] : dense_mul * acc1[e];
                }
            }
        };
        for (uint32_t ph = 0; ph < parts; ph++) {
            if (active && part == ph) store(ph != 0);
            if (ph + 1 < parts) __syncthreads();
        }
    }
    __syncthreads();
    // sparse part: groups of eight rows in the rank table, every column probes it once per group. The pairs of a
    // group's rows are requested while the group before it is probed; the pairs of a wave's columns stay in its
    // registers for the whole tile: a build and the probes find their operands there.
    auto row_pairs = [&](uint32_t i) { Pairs p = gram_row(C, rowptr, rownnz, i); p.narrow = NARROW ? 1u : 0u; return p; };
    auto col_pairs = [&](uint32_t b) { Pairs p = gram_row(C, rowptr + JT_ROWS, rownnz + JT_ROWS, b); p.narrow = NARROW ? 1u : 0u; return p; };
    uint32_t a0 = 0;
    PivotRegs pv;
    ranktab_pivots_load(pv, [&](uint32_t t) { return row_pairs(a0 + t); }, min((uint32_t)RT_T, R - a0), tid, JT_THREADS);
    // the wave's columns wave, wave + NW, ...: read once per tile, probed once per group; their shapes
    // (nnz | ns << 16) are wave-uniform and stay in scalar registers
    RtRow<NARROW> own[JT_OWN];
    uint32_t own_shape[JT_OWN];
#pragma unroll
    for (int k = 0; k < JT_OWN; k++) {
        const uint32_t b = wave + k * NW;
        own_shape[k] = 0;
        if (b < M) {
            own_shape[k] = uniform(rownnz[JT_ROWS + b]);
            rt_row_load(own[k], col_pairs(b), lane);
        }
    }
    while (a0 < R) {
        uint32_t nt = min((uint32_t)RT_T, R - a0);
        uint32_t built;
        while (true) {
            built = ranktab_build<NARROW>(T, [&](uint32_t t) { return row_pairs(a0 + t); }, pv, nt, scan, tid, JT_THREADS);
            if (built != EMPTY || nt == 1) break;
            nt = (nt + 1) / 2; // the registers hold the first pivots of the group whatever nt is
        }
        const uint32_t a1 = a0 + nt;
        if (a1 < R) ranktab_pivots_load(pv, [&](uint32_t t) { return row_pairs(a1 + t); }, min((uint32_t)RT_T, R - a1), tid, JT_THREADS);
        if (built == EMPTY) { // one row alone does not fit: its sparse part is missing, the host is told
            if (tid == 0) atomicAdd(unfit, 1ull);
            a0 = a1;
            continue;
        }
        const uint32_t n_ovf = NARROW ? 0u : uniform(min(scan[16], (uint32_t)RT_OVF));
#pragma unroll
        for (int q = 0; q < JT_OWN / JT_BATCH; q++) {
            const uint32_t b0 = wave + q * JT_BATCH * NW;
            if (b0 < M) { // wave-uniform
                float acc[JT_BATCH][RT_T];
                RtRow<NARROW> rows[JT_BATCH];
                uint32_t shape[JT_BATCH];
#pragma unroll
                for (int k = 0; k < JT_BATCH; k++) {
                    rows[k] = own[q * JT_BATCH + k];
                    rows[k].touch();
                    shape[k] = own_shape[q * JT_BATCH + k];
                    asm volatile("" : "+s"(shape[k])); // as touch(): the lane masks of a row are made where they are used
#pragma unroll
                    for (int t = 0; t < RT_T; t++) acc[k][t] = 0.f;
                }
                ranktab_probe_rows<NARROW, JT_BATCH>(T, rows, shape, [&](int k) { return col_pairs(b0 + k * NW); }, n_ovf, acc, lane);
                uint32_t t, r;
                const float z = wave_sum_2x8(acc, lane, &t, &r);
                const uint32_t b = b0 + r * NW;
                if ((lane & 15) < 4 && t < nt && b < M) G[(a0 + t) * JT_STRIDE + b] += z;
            }
            __builtin_amdgcn_sched_barrier(0); // one batch at a time: the scheduler must not pile up the reads of all of them
        }
        a0 = a1;
        __syncthreads();
    }
}

// 128 values, two per lane (element e = a of lane e for e < 64, b of lane e - 64 beyond), in ascending order of e.
__device__ __forceinline__ void wave_sort_u32x2(uint32_t& a, uint32_t& b, int lane) {
#pragma unroll
    for (int k = 2; k <= 2 * WAVE; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            if (j == WAVE) { // partners sit in the same lane; k = 128: ascending everywhere
                const uint32_t lo = min(a, b), hi = max(a, b);
                a = lo;
                b = hi;
            } else {
                const uint32_t oa = __shfl_xor(a, j, WAVE), ob = __shfl_xor(b, j, WAVE);
                const bool lower = (lane & j) == 0;
                const bool up_a = k >= WAVE ? true : (lane & k) == 0;              // element e = lane: bit 6 clear
                const bool up_b = k == 2 * WAVE ? true : k == WAVE ? false : (lane & k) == 0; // element e = 64 + lane: bit 6 set
                a = (lower == up_a) ? min(a, oa) : max(a, oa);
                b = (lower == up_b) ? min(b, ob) : max(b, ob);
            }
        }
    }
}

template <bool NARROW, uint32_t KK>
__global__ __launch_bounds__(JT_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void join_tile_kernel(JoinArgs a) {
    constexpr uint32_t HALVES = KK / 64; // tiles per block of picker rows
    a.C.narrow = NARROW ? 1u : 0u;
    extern __shared__ __align__(16) char smem[];
    const JoinLds L(a.index_bits, a.slot_cap, NARROW, KK);
    const RankTab T = ranktab_at(smem + L.tab, a.index_bits, a.slot_cap, a.span, NARROW);
    float* G = reinterpret_cast<float*>(smem + L.G);
    uint32_t* row_list = reinterpret_cast<uint32_t*>(smem + L.row_list);
    unsigned long long* rowptr = reinterpret_cast<unsigned long long*>(smem + L.rowptr);
    uint32_t* rownnz = reinterpret_cast<uint32_t*>(smem + L.rownnz);
    uint32_t* row_id = reinterpret_cast<uint32_t*>(smem + L.row_id);
    uint32_t* col_id = reinterpret_cast<uint32_t*>(smem + L.col_id);
    float* row_worst = reinterpret_cast<float*>(smem + L.row_worst);
    float* col_worst = reinterpret_cast<float*>(smem + L.col_worst);
    uint32_t* seen = reinterpret_cast<uint32_t*>(smem + L.seen);
    uint32_t* scan = reinterpret_cast<uint32_t*>(smem + L.scan);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl); // [0] tile, [1] columns

    const int tid = threadIdx.x, wave = (int)uniform(tid / WAVE), lane = lane_id();
    constexpr int NW = JT_THREADS / WAVE;
    const uint32_t n_tiles = a.tile_off[a.n];

    if (tid == 0) { ctl[2] = 0; ctl[3] = 0; } // pairs and rows of this workgroup's tiles
    while (true) {
        __syncthreads();
        if (tid == 0) { ctl[0] = (uint32_t)atomicAdd(a.work, 1ull); ctl[1] = 0; }
        for (uint32_t i = tid; i < JT_SEEN; i += JT_THREADS) seen[i] = EMPTY;
        __syncthreads();
        const uint32_t tile = uniform(ctl[0]);
        if (tile >= n_tiles) break;
        const uint32_t v = uniform(a.tile_v[tile]);
        const uint32_t p0 = uniform(a.pick_off[v]), cnt = uniform(a.pick_off[v + 1]) - p0;
        const uint32_t local = tile - uniform(a.tile_off[v]);
        const uint32_t r0 = local / HALVES * JT_ROWS, half = local % HALVES;
        const uint32_t R = min((uint32_t)JT_ROWS, cnt - r0);

        // rows: pickers of v; columns: N(v) and R(v) without repeats
        if (tid < JT_ROWS) {
            const uint32_t u = (uint32_t)tid < R ? a.pick_src[p0 + r0 + tid] : EMPTY;
            row_id[tid] = u;
            row_worst[tid] = u != EMPTY ? a.dist[(size_t)u * KK + KK - 1] : -INF_DIS;
        }
        if (HALVES == 1) {
            if (tid < 2 * (int)KK) {
                uint32_t c;
                if (tid < (int)KK) c = a.ids[(size_t)v * KK + tid] & ~FLAG;
                else c = (uint32_t)a.rev[(size_t)v * KK + (tid - KK)];
                if (c < a.n && id_set_insert(seen, JT_SEEN - 1, c)) col_id[atomicAdd(const_cast<uint32_t*>(&ctl[1]), 1u)] = c;
            }
        } else {
            // first tile: the list of v without repeats; second tile: what the reverse list adds to it
            uint32_t c = EMPTY, rc = EMPTY;
            if (tid < (int)KK) {
                c = a.ids[(size_t)v * KK + tid] & ~FLAG;
                if (half == 1) rc = (uint32_t)a.rev[(size_t)v * KK + tid];
                const bool fresh = c < a.n && id_set_insert(seen, JT_SEEN - 1, c);
                if (fresh && half == 0) col_id[atomicAdd(const_cast<uint32_t*>(&ctl[1]), 1u)] = c;
            }
            if (half == 1) {
                __syncthreads();
                if (rc < a.n && id_set_insert(seen, JT_SEEN - 1, rc)) col_id[atomicAdd(const_cast<uint32_t*>(&ctl[1]), 1u)] = rc;
            }
        }
        __syncthreads();
        const uint32_t M = uniform(ctl[1]);
        if (M == 0) continue;
        // the rows' own lists (who is already a neighbour), the columns' thresholds, where every row's pairs are
        // each row's list in ascending id order (the proposals look an id up by binary search): wave w reads and sorts rows w, w + 8, ...
        if (KK == 64) {
            uint32_t mine[JT_ROWS / NW];
#pragma unroll
            for (int k = 0; k < JT_ROWS / NW; k++) {
                const uint32_t r = wave + k * NW;
                mine[k] = r < R ? a.ids[(size_t)row_id[r] * KK + lane] & ~FLAG : 0u;
            }
#pragma unroll
            for (int k = 0; k < JT_ROWS / NW; k++) {
                const uint32_t r = wave + k * NW;
                if (r < R) row_list[r * KK + lane] = wave_sort_u32(mine[k], lane);
            }
        }
        if ((uint32_t)tid < M) col_worst[tid] = a.symmetric ? a.dist[(size_t)col_id[tid] * KK + KK - 1] : -INF_DIS;
        gram_rows_gather(a.C, row_id, R, rowptr, rownnz, tid, JT_THREADS);
        gram_rows_gather(a.C, col_id, M, rowptr + JT_ROWS, rownnz + JT_ROWS, tid, JT_THREADS);
        __syncthreads();
        tile_hybrid_ips<NARROW>(a.C, a.dense_mul, smem + L.tab, T, a.index_bits, a.slot_cap, G, rowptr, rownnz, scan, R, M, a.work + 3, tid, wave, lane);
        if (KK == 128) { // the rows' own lists, behind the table (the bytes staged dense rows until now: all waves are past that)
            uint32_t lo[JT_ROWS / NW], hi[JT_ROWS / NW];
#pragma unroll
            for (int k = 0; k < JT_ROWS / NW; k++) {
                const uint32_t r = wave + k * NW;
                lo[k] = r < R ? a.ids[(size_t)row_id[r] * KK + lane] & ~FLAG : 0u;
                hi[k] = r < R ? a.ids[(size_t)row_id[r] * KK + WAVE + lane] & ~FLAG : 0u;
            }
#pragma unroll
            for (int k = 0; k < JT_ROWS / NW; k++) {
                const uint32_t r = wave + k * NW;
                if (r < R) {
                    wave_sort_u32x2(lo[k], hi[k], lane);
                    row_list[r * KK + lane] = lo[k];
                    row_list[r * KK + WAVE + lane] = hi[k];
                }
            }
            __syncthreads();
        }
        // proposals
        for (uint32_t p = tid; p < R * M; p += JT_THREADS) {
            const uint32_t r = p / M, c = p % M;
            const uint32_t uid = row_id[r], cid = col_id[c];
            if (uid == cid) continue;
            const float d = 1.0f - G[r * JT_STRIDE + c];
            if (d < row_worst[r]) {
                const uint32_t* lst = row_list + r * KK;
                uint32_t lo = 0, len = KK;
                while (len > 0) {
                    const uint32_t half = len >> 1;
                    if (lst[lo + half] < cid) { lo += half + 1; len -= half + 1; } else len = half;
                }
                if (lo >= KK || lst[lo] != cid) atomicMin(&a.prop[(size_t)uid * a.P + prop_slot(cid, a.P)], dist_id_key(d, cid));
            }
            if (d < col_worst[c]) atomicMin(&a.prop[(size_t)cid * a.P + prop_slot(uid, a.P)], dist_id_key(d, uid));
        }
        if (tid == 0) { // summed here, sent once when the workgroup leaves: a million atomics on one address per step would queue up
            ctl[2] += R * M;
            ctl[3] += R + M;
            if (ctl[2] >= 0x40000000u) { atomicAdd(a.work + 1, (unsigned long long)ctl[2]); ctl[2] = 0; }
        }
    }
    if (tid == 0) {
        atomicAdd(a.work + 1, (unsigned long long)ctl[2]);
        atomicAdd(a.work + 2, (unsigned long long)ctl[3]);
    }
}

// One wave per node: its proposals (2 * KK slots, PL per lane) merged into its list (KL entries per lane: entry e in register
// e / 64 of lane e % 64); the entries that are new in the list register with their nodes' reverse lists (index.cu:362-372
// registers every entry of a changed list and starts the reverse lists again with every step; the join keeps them over the
// steps, so an entry registers once, when it enters). Proposal slots are left empty.
template <uint32_t KK>
__global__ __launch_bounds__(256) void join_apply_kernel(uint32_t n, uint32_t* ids, float* dist, unsigned long long* prop, unsigned long long* rev,
                                                         uint32_t* rev_cnt, unsigned long long* inserted) {
    constexpr int KL = KK / WAVE, PL = 2 * KL;
    constexpr uint32_t P = 2 * KK;
    const int wave = threadIdx.x / WAVE, lane = lane_id();
    const uint32_t u = blockIdx.x * 4 + wave;
    if (u >= n) return;
    const size_t base = (size_t)u * KK, pbase = (size_t)u * P;
    unsigned long long key[PL];
    bool some = false;
#pragma unroll
    for (int s = 0; s < PL; s++) {
        key[s] = prop[pbase + s * WAVE + lane];
        some |= key[s] != ~0ull;
    }
    if (__ballot(some) == 0) return;
#pragma unroll
    for (int s = 0; s < PL; s++) prop[pbase + s * WAVE + lane] = ~0ull;
    uint32_t own_id[KL];
    float own_d[KL];
#pragma unroll
    for (int k = 0; k < KL; k++) {
        own_id[k] = ids[base + k * WAVE + lane];
        own_d[k] = dist[base + k * WAVE + lane];
    }
    // a proposal counts if it names another node that is not in the list yet (one id always hashes to one slot: no repeats among them)
    bool valid[PL];
    float d[PL];
#pragma unroll
    for (int s = 0; s < PL; s++) {
        const uint32_t c = (uint32_t)key[s];
        valid[s] = key[s] != ~0ull && c != u && c < n;
        d[s] = join_key_dist(key[s]);
    }
#pragma unroll
    for (int k = 0; k < KL; k++) {
        for (uint32_t i = 0; i < WAVE; i++) {
            const uint32_t x = (uint32_t)__builtin_amdgcn_readlane((int)own_id[k], i) & ~FLAG;
#pragma unroll
            for (int s = 0; s < PL; s++) valid[s] = valid[s] && x != (uint32_t)key[s];
        }
    }
    uint64_t nb[PL], any = 0;
#pragma unroll
    for (int s = 0; s < PL; s++) { nb[s] = __ballot(valid[s]); any |= nb[s]; }
    if (any == 0) return;
    // new: rank among the new ones by (distance, id), plus the old entries strictly closer (new first on ties)
    uint32_t rank_new[PL], le_old[KL];
#pragma unroll
    for (int s = 0; s < PL; s++) rank_new[s] = 0;
#pragma unroll
    for (int k = 0; k < KL; k++) le_old[k] = 0;
#pragma unroll
    for (int t = 0; t < PL; t++) {
        for (uint64_t rest = nb[t]; rest; rest &= rest - 1) {
            const unsigned long long ki = readlane64(key[t], (uint32_t)__builtin_ctzll(rest));
#pragma unroll
            for (int s = 0; s < PL; s++) rank_new[s] += ki < key[s];
#pragma unroll
            for (int k = 0; k < KL; k++) le_old[k] += join_key_dist(ki) <= own_d[k]; // old entry: new ones at or below its distance go first
        }
    }
#pragma unroll
    for (int k = 0; k < KL; k++) {
        for (uint32_t i = 0; i < WAVE; i++) {
            const float di = readlane_f32(own_d[k], i);
#pragma unroll
            for (int s = 0; s < PL; s++) rank_new[s] += di < d[s];
        }
    }
    bool new_in[PL];
    uint32_t n_ins = 0;
#pragma unroll
    for (int s = 0; s < PL; s++) {
        new_in[s] = valid[s] && rank_new[s] < KK;
        n_ins += __popcll(__ballot(new_in[s]));
    }
    if (n_ins == 0) return;
#pragma unroll
    for (int k = 0; k < KL; k++) {
        const uint32_t rank_old = (uint32_t)(k * WAVE + lane) + le_old[k];
        if (rank_old < KK) { ids[base + rank_old] = own_id[k]; dist[base + rank_old] = own_d[k]; }
    }
#pragma unroll
    for (int s = 0; s < PL; s++) {
        if (new_in[s]) { ids[base + rank_new[s]] = (uint32_t)key[s]; dist[base + rank_new[s]] = d[s]; }
    }
    if (lane == 0) atomicAdd(inserted + (blockIdx.x % JOIN_COUNT_PARTS) * 8, (unsigned long long)n_ins); // one address for every node would serialise a million atomics
    // reverse registration of the new entries: (distance, u) in one word, slot count % K keeps the closer one beyond K
    auto reg = [&](uint32_t e, float dv) {
        const uint32_t v = e & ~FLAG;
        if (v >= n) return;
        const uint32_t slot = atomicAdd(&rev_cnt[v], 1u);
        const unsigned long long k = dist_id_key(dv, u);
        // every registration is a minimum (the lists start at ~0 and the join never starts them again): a store into a slot
        // that a later registration of the same step has already reached through its wrap-around could undo that one
        atomicMin(rev + (size_t)v * KK + (slot % KK), k);
    };
#pragma unroll
    for (int s = 0; s < PL; s++) {
        if (new_in[s]) reg((uint32_t)key[s], d[s]);
    }
}

__global__ static void join_account_kernel(unsigned long long* work, unsigned long long* counter) {
    counter[2] += work[1]; // pairs evaluated
    counter[3] += work[2]; // rows gathered (each read in full, dense part included)
    unsigned long long inserted = 0; // the partial counts of join_apply_kernel
    for (int p = 0; p < JOIN_COUNT_PARTS; p++) inserted += work[JOIN_COUNT_AT + p * 8];
    counter[0] = inserted;
}

__global__ __launch_bounds__(256) static void fill_u64_kernel(unsigned long long* p, uint64_t count, unsigned long long v) {
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (uint64_t)gridDim.x * blockDim.x) p[t] = v;
}
__global__ __launch_bounds__(256) static void fill_u32_kernel2(uint32_t* p, uint64_t count, uint32_t v) {
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (uint64_t)gridDim.x * blockDim.x) p[t] = v;
}

// ---- hybrid Gram matrices of whole neighbour lists, tile by tile (the prune of lists longer than 64 entries) ----
//
// For node u = node0 + q the valid entries of its list (distance below INF_DIS, a document, not u itself),
// in list order, are the rows and columns of a Gram matrix of at most 128 x 128. Tile t computes rows
// [32 t, 32 t + 32) against the columns [32 t, m): the upper triangle, diagonal blocks whole. The products go to
// gram[q * 128 * 128 + i * 128 + j] for i <= j (entries below the diagonal of a diagonal block are
// written too). Same tile body as the local join: every row of a tile is gathered once, dense part on the matrix cores,
// sparse part through the rank table.
constexpr uint32_t GT_MAX = 128;                 // longest list
struct GramTileArgs {
    CorpusView C;
    float dense_mul;
    uint32_t K, node0, n_nodes;
    const uint32_t* ids;
    const float* dist;
    float* gram;
    unsigned long long* work; // [0] next tile, [3] a row did not fit the table
    uint32_t index_bits, slot_cap, span;
};

template <bool NARROW>
__global__ __launch_bounds__(JT_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void gram_tile_kernel(GramTileArgs a) {
    a.C.narrow = NARROW ? 1u : 0u;
    extern __shared__ __align__(16) char smem[];
    const JoinLds L(a.index_bits, a.slot_cap, NARROW);
    const RankTab T = ranktab_at(smem + L.tab, a.index_bits, a.slot_cap, a.span, NARROW);
    float* G = reinterpret_cast<float*>(smem + L.G);
    unsigned long long* rowptr = reinterpret_cast<unsigned long long*>(smem + L.rowptr);
    uint32_t* rownnz = reinterpret_cast<uint32_t*>(smem + L.rownnz);
    uint32_t* row_id = reinterpret_cast<uint32_t*>(smem + L.row_id);
    uint32_t* col_id = reinterpret_cast<uint32_t*>(smem + L.col_id);
    uint32_t* valid = reinterpret_cast<uint32_t*>(smem + L.seen); // the node's valid list entries, in list order
    uint32_t* scan = reinterpret_cast<uint32_t*>(smem + L.scan);
    volatile uint32_t* ctl = reinterpret_cast<volatile uint32_t*>(smem + L.ctl); // [0] tile, [1] valid entries
    static_assert(JT_SEEN >= (int)GT_MAX, "the id set's words hold a whole list");
    const int tid = threadIdx.x, wave = (int)uniform(tid / WAVE), lane = lane_id();
    const uint64_t lane_lt = (1ull << lane) - 1;
    while (true) { // a workgroup takes a node and runs its tiles one after the other: the columns of a tile are the rows and columns of the next
        __syncthreads();
        if (tid == 0) ctl[0] = (uint32_t)atomicAdd(a.work, 1ull);
        __syncthreads();
        const uint32_t slot = uniform(ctl[0]);
        if (slot >= a.n_nodes) break;
        const uint32_t u = a.node0 + slot;
        if (wave == 0) {
            const size_t base = (size_t)u * a.K;
            uint32_t m = 0;
            for (uint32_t b0 = 0; b0 < a.K; b0 += WAVE) {
                const uint32_t v = (a.ids[base + b0 + lane] & ~FLAG);
                const float dv = a.dist[base + b0 + lane];
                const bool ok = dv < INF_DIS && v < a.C.n && v != u;
                const uint64_t b = __ballot(ok);
                if (ok) valid[m + __popcll(b & lane_lt)] = v;
                m += __popcll(b);
            }
            if (lane == 0) ctl[1] = m;
        }
        __syncthreads();
        const uint32_t m = uniform(ctl[1]);
        float* out = a.gram + (size_t)slot * GT_MAX * GT_MAX;
        for (uint32_t r0 = 0; r0 < m; r0 += JT_ROWS) {
            const uint32_t R = min((uint32_t)JT_ROWS, m - r0), M = m - r0;
            if ((uint32_t)tid < R) row_id[tid] = valid[r0 + tid];
            if ((uint32_t)tid < M) col_id[tid] = valid[r0 + tid];
            __syncthreads();
            gram_rows_gather(a.C, row_id, R, rowptr, rownnz, tid, JT_THREADS);
            gram_rows_gather(a.C, col_id, M, rowptr + JT_ROWS, rownnz + JT_ROWS, tid, JT_THREADS);
            __syncthreads();
            tile_hybrid_ips<NARROW>(a.C, a.dense_mul, smem + L.tab, T, a.index_bits, a.slot_cap, G, rowptr, rownnz, scan, R, M, a.work + 3, tid, wave, lane);
            for (uint32_t p = tid; p < R * M; p += JT_THREADS) {
                const uint32_t r = p / M, c = p % M;
                out[(size_t)(r0 + r) * GT_MAX + r0 + c] = G[r * JT_STRIDE + c];
            }
            __syncthreads(); // G and the id arrays are rewritten by the next tile
        }
    }
}

static void join_table_shape(const apoe_corpus* c, uint32_t* index_bits, uint32_t* slot_cap, uint32_t* span) {
    *span = next_pow2(std::max(c->max_term + 1, 1024u));
    *index_bits = c->narrow ? 2 * *span : 65536u;
    const uint32_t want = RT_T * (c->max_nnz_s + c->max_nnz_b);
    *slot_cap = std::min<uint32_t>(std::max<uint32_t>((want + 63) & ~63u, 256u), (uint32_t)APOE_JOIN_MAX_ROW_TERMS);
}

int join_alloc(apoe_knn* g) {
    const size_t n = g->n;
    APOE_TRY(g->picks.alloc(n * JOIN_PICKS));
    APOE_TRY(g->pick_cnt.alloc(n + 1));
    APOE_TRY(g->pick_off.alloc(n + 1));
    APOE_TRY(g->pick_fill.alloc(n + 1));
    APOE_TRY(g->pick_src.alloc(n * JOIN_PICKS));
    APOE_TRY(g->tile_cnt.alloc(n + 1));
    APOE_TRY(g->tile_off.alloc(n + 1));
    const size_t halves = g->K / 64, P = 2 * (size_t)g->K;
    APOE_TRY(g->tile_v.alloc((n + n * JOIN_PICKS / JT_ROWS + 1) * halves));
    APOE_TRY(g->prop.alloc(n * P));
    APOE_TRY(g->join_work.alloc(JOIN_COUNT_AT + JOIN_COUNT_PARTS * 8));
    size_t temp_bytes = 0;
    APOE_HIP(hipcub::DeviceScan::ExclusiveSum(nullptr, temp_bytes, g->pick_cnt.p, g->pick_off.p, (int)(n + 1), g->ctx->stream));
    APOE_TRY(g->scan_tmp.alloc(temp_bytes));
    fill_u64_kernel<<<1024, 256, 0, g->ctx->stream>>>(g->prop.p, (uint64_t)n * P, ~0ull);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

int launch_nnd_join_iterate(apoe_knn* g) {
    apoe_ctx* ctx = g->ctx;
    hipStream_t st = ctx->stream;
    const uint32_t n = g->n;
    APOE_REQUIRE(g->K == 64 || g->K == 128, "the local-join step is built for K = 64 and K = 128 lists, this handle has K = %u", g->K);
    const bool k128 = g->K == 128;
    const uint32_t halves = g->K / 64;
    if (!g->prop.p) APOE_TRY(join_alloc(g));
    uint32_t index_bits, slot_cap, span;
    join_table_shape(g->corpus, &index_bits, &slot_cap, &span);
    const JoinLds L(index_bits, slot_cap, g->corpus->narrow, g->K);
    APOE_REQUIRE(L.total <= ctx->lds_per_block, "the local-join tile needs %u bytes of LDS, a workgroup may have %zu", L.total, ctx->lds_per_block);

    APOE_HIP(hipMemsetAsync(g->counter.p, 0, sizeof(unsigned long long), st)); // [0] inserted; [2], [3] accumulate over the build
    fill_u32_kernel2<<<1024, 256, 0, st>>>(g->pick_cnt.p, (uint64_t)n + 1, 0u);
    fill_u32_kernel2<<<1024, 256, 0, st>>>(g->pick_fill.p, (uint64_t)n + 1, 0u);
    fill_u64_kernel<<<8, 256, 0, st>>>(g->join_work.p, JOIN_COUNT_AT + JOIN_COUNT_PARTS * 8, 0ull);
    if (k128) join_pick_kernel<128><<<(n + 3) / 4, 256, 0, st>>>(n, g->ids.p, g->picks.p, g->pick_cnt.p);
    else join_pick_kernel<64><<<(n + 3) / 4, 256, 0, st>>>(n, g->ids.p, g->picks.p, g->pick_cnt.p);
    APOE_HIP(hipGetLastError());
    join_tile_count_kernel<<<(n + 256) / 256, 256, 0, st>>>(n, halves, g->pick_cnt.p, g->tile_cnt.p);
    APOE_HIP(hipGetLastError());
    size_t temp_bytes = g->scan_tmp.n;
    APOE_HIP(hipcub::DeviceScan::ExclusiveSum(g->scan_tmp.p, temp_bytes, g->pick_cnt.p, g->pick_off.p, (int)(n + 1), st));
    temp_bytes = g->scan_tmp.n;
    APOE_HIP(hipcub::DeviceScan::ExclusiveSum(g->scan_tmp.p, temp_bytes, g->tile_cnt.p, g->tile_off.p, (int)(n + 1), st));
    const uint64_t total = (uint64_t)n * JOIN_PICKS;
    join_fill_kernel<<<(uint32_t)((total + 255) / 256), 256, 0, st>>>(n, halves, g->picks.p, g->pick_off.p, g->tile_off.p, g->pick_fill.p, g->pick_src.p, g->tile_v.p);
    APOE_HIP(hipGetLastError());

    JoinArgs a{};
    a.C = g->corpus->view();
    a.dense_mul = g->dense_scale * g->dense_scale;
    a.n = n;
    a.P = 2 * g->K;
    a.symmetric = g->join_symmetric ? 1u : 0u;
    a.ids = g->ids.p;
    a.dist = g->dist.p;
    a.rev = g->rev.p;
    a.pick_off = g->pick_off.p;
    a.pick_src = g->pick_src.p;
    a.tile_off = g->tile_off.p;
    a.tile_v = g->tile_v.p;
    a.prop = g->prop.p;
    a.work = g->join_work.p;
    a.index_bits = index_bits;
    a.slot_cap = slot_cap;
    a.span = span;
    auto kernel = k128 ? (g->corpus->narrow ? &join_tile_kernel<true, 128> : &join_tile_kernel<false, 128>)
                       : (g->corpus->narrow ? &join_tile_kernel<true, 64> : &join_tile_kernel<false, 64>);
    APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total));
    int per_cu = 1;
    APOE_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel), JT_THREADS, L.total));
    if (per_cu < 1) per_cu = 1;
    kernel<<<(uint32_t)per_cu * (uint32_t)ctx->num_cus, JT_THREADS, L.total, st>>>(a);
    APOE_HIP(hipGetLastError());
    if (k128) join_apply_kernel<128><<<(n + 3) / 4, 256, 0, st>>>(n, g->ids.p, g->dist.p, g->prop.p, g->rev.p, g->rev_cnt.p, g->join_work.p + JOIN_COUNT_AT);
    else join_apply_kernel<64><<<(n + 3) / 4, 256, 0, st>>>(n, g->ids.p, g->dist.p, g->prop.p, g->rev.p, g->rev_cnt.p, g->join_work.p + JOIN_COUNT_AT);
    APOE_HIP(hipGetLastError());
    join_account_kernel<<<1, 1, 0, st>>>(g->join_work.p, g->counter.p);
    APOE_HIP(hipGetLastError());
    return APOE_OK;
}

// Gram matrices (upper triangles) of the lists of nodes [node0, node0 + n_nodes) into gram[n_nodes][128][128]. *unfit = rows
// whose sparse terms did not fit the tile's table (their products lack the sparse part: the caller must not use the result).
int launch_gram_tiles(apoe_knn* g, uint32_t node0, uint32_t n_nodes, float* gram, unsigned long long* unfit) {
    apoe_ctx* ctx = g->ctx;
    hipStream_t st = ctx->stream;
    APOE_REQUIRE(g->K <= GT_MAX, "Gram tiles are built for lists of at most %u entries", GT_MAX);
    if (!g->join_work.p) APOE_TRY(g->join_work.alloc(JOIN_COUNT_AT + JOIN_COUNT_PARTS * 8));
    uint32_t index_bits, slot_cap, span;
    join_table_shape(g->corpus, &index_bits, &slot_cap, &span);
    const JoinLds L(index_bits, slot_cap, g->corpus->narrow);
    APOE_REQUIRE(L.total <= ctx->lds_per_block, "a Gram tile needs %u bytes of LDS, a workgroup may have %zu", L.total, ctx->lds_per_block);
    fill_u64_kernel<<<1, 64, 0, st>>>(g->join_work.p, 8, 0ull);
    APOE_HIP(hipGetLastError());
    GramTileArgs a{};
    a.C = g->corpus->view();
    a.dense_mul = g->dense_scale * g->dense_scale;
    a.K = g->K;
    a.node0 = node0;
    a.n_nodes = n_nodes;
    a.ids = g->ids.p;
    a.dist = g->dist.p;
    a.gram = gram;
    a.work = g->join_work.p;
    a.index_bits = index_bits;
    a.slot_cap = slot_cap;
    a.span = span;
    auto kernel = g->corpus->narrow ? &gram_tile_kernel<true> : &gram_tile_kernel<false>;
    APOE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)L.total));
    int per_cu = 1;
    APOE_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel), JT_THREADS, L.total));
    if (per_cu < 1) per_cu = 1;
    kernel<<<(uint32_t)per_cu * (uint32_t)ctx->num_cus, JT_THREADS, L.total, st>>>(a);
    APOE_HIP(hipGetLastError());
    if (unfit) {
        unsigned long long h[4] = {0, 0, 0, 0};
        APOE_HIP(hipMemcpyAsync(h, g->join_work.p, sizeof(h), hipMemcpyDeviceToHost, st));
        APOE_HIP(hipStreamSynchronize(st));
        *unfit = h[3];
    }
    return APOE_OK;
}

// Whether launch_gram_tiles can serve this handle: lists of at most 128 entries, rows that fit a tile's table, LDS for a tile.
bool gram_tiles_fit(const apoe_knn* g) {
    if (g->K > GT_MAX || g->corpus->max_nnz_s + g->corpus->max_nnz_b > (uint32_t)APOE_JOIN_MAX_ROW_TERMS) return false;
    uint32_t index_bits, slot_cap, span;
    join_table_shape(g->corpus, &index_bits, &slot_cap, &span);
    return JoinLds(index_bits, slot_cap, g->corpus->narrow).total <= g->ctx->lds_per_block;
}

// Pairs evaluated and rows gathered by the tiles of the last step, and whether a row did not fit the table.
int join_step_counters(apoe_knn* g, unsigned long long* out3) {
    unsigned long long h[4] = {0, 0, 0, 0};
    APOE_HIP(hipMemcpy(h, g->join_work.p, sizeof(h), hipMemcpyDeviceToHost));
    out3[0] = h[1];
    out3[1] = h[2];
    out3[2] = h[3];
    return APOE_OK;
}

} // namespace apoe
