// Sparse inner products of many rows against a small group of pivot rows at once: the pivots' terms go
// into ONE LDS table that is addressed through a bitmap with running counts (a "rank table"), and every
// other row then looks each of its pairs up exactly once for the whole group.
//
//   word[w] = (bits, count of set bits in words before w)      one ds_read_b64 per look-up
//   slot of a term = count + popcount(bits below its bit)      no hashing, no probe loop, no key compare
//   vals[slot], vals[slot_cap + slot] = one value per pivot of the group (zero where the pivot lacks the term), pivots 0-3 and
//   4-7 in two planes: two ds_read_b128 whose 64 lanes spread over all LDS banks (side by side, a read would touch every second
//   16-byte unit only)
//
// A corpus in the narrow pair format (term ids below 65536, the path known from the position in the row)
// maps a term to bit (term | path * span) with span = the power of two above the largest term id: distinct
// terms have distinct bits, the table is a perfect hash and a miss costs one 8-byte read whose 64 lanes
// mostly fall into different banks. Wide corpora hash the 32-bit key to a bit; two terms of a group that
// fall on one bit are told apart by the stored key and the loser goes to a short overflow list.
#pragma once

#include "apoe_device.h"

namespace apoe {

#ifdef __HIPCC__

// Inclusive prefix sum over the wave with DPP adds only (no LDS crossbar): four shifted adds inside each row of 16
// lanes, then the last lane of a row is added to the row after it (row_bcast:15 for rows 1 and 3, row_bcast:31 for
// rows 2 and 3).
__device__ __forceinline__ uint32_t wave_scan_add_dpp(uint32_t v) {
    int x = (int)v;
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false); // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false); // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false); // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false); // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false); // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false); // row_bcast:31 into rows 2 and 3
    return (uint32_t)x;
}

constexpr int RT_T = 8;     // pivots per table: two float4 per term
constexpr int RT_OVF = 32;  // overflow entries (wide corpora only)

struct RankTabLds { // byte offsets inside the table region
    uint32_t word, keys, vals, ovf_key, ovf_val, total;
    __host__ __device__ RankTabLds(uint32_t index_bits, uint32_t slot_cap, bool narrow) {
        uint32_t o = 0;
        vals = o; o += slot_cap * RT_T * 4;
        word = o; o += (index_bits / 32) * 8;
        keys = o; o += narrow ? 0 : slot_cap * 4;
        ovf_key = o; o += narrow ? 0 : RT_OVF * 4;
        o = (o + 15) & ~15u;
        ovf_val = o; o += narrow ? 0 : RT_OVF * RT_T * 4;
        total = o;
    }
};

struct RankTab {
    uint2* word;      // [index_bits / 32]
    uint32_t* keys;   // [slot_cap], wide only
    float4* vals;     // [RT_T / 4][slot_cap]: plane h holds pivots 4h .. 4h + 3 of every slot
    uint32_t* ovf_key;
    float4* ovf_val;
    uint32_t index_bits, slot_cap;
    uint32_t span; // narrow: bit index of a BM25 term = term + span
};

__device__ __forceinline__ RankTab ranktab_at(char* region, uint32_t index_bits, uint32_t slot_cap, uint32_t span, bool narrow) {
    const RankTabLds L(index_bits, slot_cap, narrow);
    RankTab T;
    T.word = reinterpret_cast<uint2*>(region + L.word);
    T.keys = reinterpret_cast<uint32_t*>(region + L.keys);
    T.vals = reinterpret_cast<float4*>(region + L.vals);
    T.ovf_key = reinterpret_cast<uint32_t*>(region + L.ovf_key);
    T.ovf_val = reinterpret_cast<float4*>(region + L.ovf_val);
    T.index_bits = index_bits;
    T.slot_cap = slot_cap;
    T.span = span;
    return T;
}

// Bit index of a pair. key: raw key as the record load delivers it (narrow: the 16-bit term; wide: term | path bit).
template <bool NARROW>
__device__ __forceinline__ uint32_t ranktab_index(const RankTab& T, uint32_t key, bool bm25) {
    if (NARROW) return key + (bm25 ? T.span : 0u);
    const uint32_t k = key ^ (key >> 15);
    return ((k * 0x9E3779B1u) >> 12) & (T.index_bits - 1);
}

// The pairs of the pivots of one group, spread over the threads of the block: thread i holds pair i of every
// pivot (rows with more pairs than the block has threads read the rest when the table is built). Loaded ahead of
// time, while the previous group is still being probed, so that a build does not wait for memory.
constexpr int RT_PV = 1;
struct PivotRegs {
    uint2 kv[RT_T][RT_PV]; // raw pairs
};
template <typename PivotFn>
__device__ __forceinline__ void ranktab_pivots_load(PivotRegs& r, PivotFn pivot, uint32_t nt, int tid, int nthreads) {
#pragma unroll
    for (int t = 0; t < RT_T; t++) {
        if ((uint32_t)t < nt) {
            const Pairs sp = pivot(t);
#pragma unroll
            for (int k = 0; k < RT_PV; k++) {
                const uint32_t j = tid + k * nthreads;
                r.kv[t][k] = j < sp.nnz ? sp.raw(j) : make_uint2(0u, 0u);
            }
        }
    }
}

// Bitmap and running counts of the terms that `each` hands out: each(f) calls f(raw pair, is BM25, pivot index) for
// every pair that this thread is responsible for. All threads of the block call this (the block size is a multiple of
// 64, at most 1024); `scan` is LDS scratch of 20 words. Returns the number of distinct terms. Does NOT end with a
// barrier: the counts of other threads' words are readable after the caller's next one. With `cap` below the number
// of distinct terms the counts are not written (the caller gives the table up).
template <bool NARROW, typename EachFn>
__device__ __forceinline__ uint32_t ranktab_build_bits(const RankTab& T, EachFn each, uint32_t cap, uint32_t* scan, int tid, int nthreads) {
    const uint32_t W = T.index_bits / 32;
    const int lane = tid & (WAVE - 1), wave = tid / WAVE, nwaves = nthreads / WAVE;
    for (uint32_t w = tid; w < W; w += nthreads) T.word[w] = make_uint2(0u, 0u);
    if (tid == 0) scan[16] = 0; // overflow count
    __syncthreads();
    // 1. bits
    each([&](uint2 kv, bool bm25, int) {
        const uint32_t idx = ranktab_index<NARROW>(T, kv.x, bm25);
        atomicOr(&T.word[idx >> 5].x, 1u << (idx & 31));
    });
    __syncthreads();
    // 2. running counts: thread i owns the words [i * per, (i + 1) * per), per even: read and written two words
    // (16 bytes) at a time, which spreads a wave's accesses over half of the LDS banks instead of four of them
    const uint32_t per = ((W + nthreads - 1) / nthreads + 1) & ~1u;
    uint4* word2 = reinterpret_cast<uint4*>(T.word);
    uint32_t mine = 0;
    for (uint32_t k = 0; k < per; k += 2) {
        const uint32_t w = tid * per + k;
        if (w < W) {
            const uint4 two = word2[w >> 1];
            mine += __popc(two.x) + __popc(two.z);
        }
    }
    const uint32_t incl = wave_scan_add_dpp(mine);
    if (lane == WAVE - 1) scan[wave] = incl;
    __syncthreads();
    uint32_t before = incl - mine, total = 0;
    for (int w = 0; w < nwaves; w++) {
        const uint32_t s = scan[w];
        if (w < wave) before += s;
        total += s;
    }
    if (total > cap) return total;
    for (uint32_t k = 0; k < per; k += 2) {
        const uint32_t w = tid * per + k;
        if (w < W) {
            uint4 two = word2[w >> 1];
            two.y = before;
            before += __popc(two.x);
            two.w = before;
            before += __popc(two.z);
            word2[w >> 1] = two;
        }
    }
    return total;
}

// Slot of a term in a table built by ranktab_build_bits, or EMPTY if the term is not in it (w = T.word[idx >> 5]).
__device__ __forceinline__ uint32_t ranktab_slot(uint2 w, uint32_t idx) {
    return ((w.x >> (idx & 31)) & 1u) ? w.y + __popc(w.x & ((1u << (idx & 31)) - 1u)) : EMPTY;
}

// Builds the table from the pairs that `each` hands out (as ranktab_build_bits; it is called twice: bits, then values, and
// must hand out the same pairs both times). Returns the number of distinct terms, or EMPTY if they
// exceed the slot capacity or the overflow list (the table is then unusable: the caller retries with fewer pivots).
// Ends with a barrier: the table is ready on return.
template <bool NARROW, typename EachFn>
__device__ __forceinline__ uint32_t ranktab_build_each(const RankTab& T, EachFn each, uint32_t* scan, int tid, int nthreads) {
    const uint32_t total = ranktab_build_bits<NARROW>(T, each, T.slot_cap, scan, tid, nthreads);
    if (total > T.slot_cap) {
        __syncthreads();
        return EMPTY;
    }
    for (uint32_t s = tid; s < total; s += nthreads) {
        T.vals[s] = make_float4(0.f, 0.f, 0.f, 0.f);
        T.vals[T.slot_cap + s] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (!NARROW) {
        for (uint32_t s = tid; s < total; s += nthreads) T.keys[s] = EMPTY;
        for (uint32_t s = tid; s < RT_OVF; s += nthreads) T.ovf_key[s] = EMPTY;
        for (uint32_t s = tid; s < RT_OVF * (RT_T / 4); s += nthreads) T.ovf_val[s] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();
    // 3. values (and keys)
    each([&](uint2 kv, bool bm25, int t) {
        const uint32_t idx = ranktab_index<NARROW>(T, kv.x, bm25);
        const uint2 w = T.word[idx >> 5];
        const uint32_t slot = w.y + __popc(w.x & ((1u << (idx & 31)) - 1u));
        if (NARROW) {
            reinterpret_cast<uint32_t*>(T.vals)[((t >> 2) * T.slot_cap + slot) * 4 + (t & 3)] = kv.y;
        } else {
            const uint32_t old = atomicCAS(&T.keys[slot], EMPTY, kv.x);
            if (old == EMPTY || old == kv.x) {
                reinterpret_cast<uint32_t*>(T.vals)[((t >> 2) * T.slot_cap + slot) * 4 + (t & 3)] = kv.y;
            } else { // another term of the group sits on this bit
                uint32_t at = EMPTY;
                for (uint32_t s = 0; s < RT_OVF; s++) {
                    const uint32_t o = atomicCAS(&T.ovf_key[s], EMPTY, kv.x);
                    if (o == EMPTY) atomicAdd(&scan[16], 1u);
                    if (o == EMPTY || o == kv.x) { at = s; break; }
                }
                if (at != EMPTY) reinterpret_cast<uint32_t*>(T.ovf_val)[at * RT_T + t] = kv.y;
                else atomicAdd(&scan[16], RT_OVF + 1u);
            }
        }
    });
    __syncthreads();
    if (!NARROW) { // every thread reads the count before any thread can start the next build, which clears it
        const uint32_t ov = scan[16];
        __syncthreads();
        if (ov > RT_OVF) return EMPTY;
    }
    return total;
}

// The table of pivots [0, nt) (nt <= RT_T) whose pairs are spread over the threads of the block: pivot(t) gives the
// Pairs of pivot t, `regs` its first pairs (ranktab_pivots_load).
template <bool NARROW, typename PivotFn>
__device__ __forceinline__ uint32_t ranktab_build(const RankTab& T, PivotFn pivot, const PivotRegs& regs, uint32_t nt, uint32_t* scan, int tid,
                                                  int nthreads) {
    return ranktab_build_each<NARROW>(T, [&](auto f) {
#pragma unroll
        for (int t = 0; t < RT_T; t++) {
            if ((uint32_t)t < nt) {
                const Pairs sp = pivot(t);
#pragma unroll
                for (int k = 0; k < RT_PV; k++) {
                    const uint32_t j = tid + k * nthreads;
                    if (j < sp.nnz) f(regs.kv[t][k], j >= sp.ns, t);
                }
                for (uint32_t j = tid + RT_PV * nthreads; j < sp.nnz; j += nthreads) f(sp.raw(j), j >= sp.ns, t);
            }
        }
    }, scan, tid, nthreads);
}

// One pair against the table: acc[t] += value * (pivot t's value of the term). `in` = the lane holds a pair.
// The value slot is read whatever the bitmap says (a miss reads slot 0 with multiplier zero): the reads of several
// pairs can then be issued together, and the 64 lanes of a miss read one address, which LDS serves as a broadcast.
struct RankProbe {
    uint32_t slot;
    float mul;
};
template <bool NARROW>
__device__ __forceinline__ RankProbe ranktab_locate(const RankTab& T, uint2 w, uint32_t idx, uint32_t val_bits, bool in) {
    const bool hit = in && ((w.x >> (idx & 31)) & 1u);
    RankProbe p;
    p.slot = hit ? w.y + __popc(w.x & ((1u << (idx & 31)) - 1u)) : 0u;
    p.mul = hit ? __uint_as_float(val_bits) : 0.f;
    return p;
}

// Sum of four per-lane accumulators over the wave, all four at once: after two exchange-and-add steps inside
// each quad, lane l holds pivot t(l) = 2 * (l & 1) + ((l >> 1) & 1) summed over its quad; then one sum per lane.
// Returns that pivot's total in every lane whose (l & 3) names it; *t_out = the pivot this lane holds.
__device__ __forceinline__ float wave_sum4_dpp(const float acc[4], int lane, uint32_t* t_out) {
    const bool odd = lane & 1, hi = lane & 2;
    const float keep0 = odd ? acc[2] : acc[0], keep1 = odd ? acc[3] : acc[1];
    const float give0 = odd ? acc[0] : acc[2], give1 = odd ? acc[1] : acc[3];
    const float x0 = keep0 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give0), 0xB1, 0xF, 0xF, false));
    const float x1 = keep1 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give1), 0xB1, 0xF, 0xF, false));
    const float keep = hi ? x1 : x0, give = hi ? x0 : x1;
    float z = keep + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give), 0x4E, 0xF, 0xF, false));
    z += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, z), 0x124, 0xF, 0xF, false)); // row_ror:4
    z += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, z), 0x128, 0xF, 0xF, false)); // row_ror:8
    z += __shfl_xor(z, 16, WAVE);
    z += __shfl_xor(z, 32, WAVE);
    *t_out = 2u * (lane & 1) + ((lane >> 1) & 1);
    return z;
}

constexpr int RT_CHUNKS = 4; // pairs of a streamed row per lane kept in registers (256 pairs a row); longer rows read the rest when they are probed

// Raw pairs of a streamed row in registers: lane l holds the four consecutive pairs 4l .. 4l + 3 (one 16-byte load of
// values and one 8-byte load of terms per lane and narrow row). Narrow keys are 16 bits wide: two share a register.
__device__ __forceinline__ uint32_t rt_pair(int c, int lane) { return (uint32_t)(RT_CHUNKS * lane + c); }
template <bool NARROW>
struct RtRow;
template <>
struct RtRow<true> {
    uint32_t v[RT_CHUNKS], k2[RT_CHUNKS / 2];
    // tells the compiler that the keys may have changed: what is derived from them (bit index, masks) is then computed
    // where it is used instead of once for all rows ahead of a loop, where it would occupy registers for the whole loop
    __device__ __forceinline__ void touch() { asm volatile("" : "+v"(k2[0]), "+v"(k2[1])); }
    __device__ __forceinline__ uint32_t key(int c) const { return (c & 1) ? (k2[c >> 1] >> 16) : (k2[c >> 1] & 0xFFFFu); }
    __device__ __forceinline__ void set(int c, uint2 kv) {
        v[c] = kv.y;
        if (c & 1) k2[c >> 1] |= kv.x << 16;
        else k2[c >> 1] = kv.x;
    }
};
template <>
struct RtRow<false> {
    uint32_t v[RT_CHUNKS], k[RT_CHUNKS];
    __device__ __forceinline__ void touch() { asm volatile("" : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3])); }
    __device__ __forceinline__ uint32_t key(int c) const { return k[c]; }
    __device__ __forceinline__ void set(int c, uint2 kv) { v[c] = kv.y; k[c] = kv.x; }
};
// dst = take ? src : dst, member by member (a wave-uniform choice between rows that stay in registers)
__device__ __forceinline__ void rt_row_select(RtRow<true>& dst, const RtRow<true>& src, bool take) {
#pragma unroll
    for (int c = 0; c < RT_CHUNKS; c++) dst.v[c] = take ? src.v[c] : dst.v[c];
#pragma unroll
    for (int c = 0; c < RT_CHUNKS / 2; c++) dst.k2[c] = take ? src.k2[c] : dst.k2[c];
}
__device__ __forceinline__ void rt_row_select(RtRow<false>& dst, const RtRow<false>& src, bool take) {
#pragma unroll
    for (int c = 0; c < RT_CHUNKS; c++) {
        dst.v[c] = take ? src.v[c] : dst.v[c];
        dst.k[c] = take ? src.k[c] : dst.k[c];
    }
}
__device__ __forceinline__ void rt_row_load(RtRow<true>& r, const Pairs& sp, int lane) {
    static_assert(RT_CHUNKS == 4, "one uint4 of values and one uint2 of terms per lane");
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    uint2 k = make_uint2(0u, 0u);
    if (rt_pair(0, lane) < sp.nnz) { // the arrays start on 128-byte boundaries and are padded to them: the last lane reads inside the record
        v = reinterpret_cast<const uint4*>(sp.base)[lane];
        k = reinterpret_cast<const uint2*>(sp.base + narrow_keys_offset(sp.nnz))[lane];
    }
    r.v[0] = v.x; r.v[1] = v.y; r.v[2] = v.z; r.v[3] = v.w;
    r.k2[0] = k.x; r.k2[1] = k.y;
}
__device__ __forceinline__ void rt_row_load(RtRow<false>& r, const Pairs& sp, int lane) {
#pragma unroll
    for (int c = 0; c < RT_CHUNKS; c += 2) {
        uint4 kv = make_uint4(0u, 0u, 0u, 0u);
        if (rt_pair(c, lane) < sp.nnz) kv = reinterpret_cast<const uint4*>(sp.base)[(RT_CHUNKS * lane + c) / 2]; // an odd count: the second pair is masked by its index
        r.k[c] = kv.x; r.v[c] = kv.y; r.k[c + 1] = kv.z; r.v[c + 1] = kv.w;
    }
}

// The table of a group whose pivots are held one per wave, in registers: this wave's row `pr` (shape = nnz | ns << 16)
// becomes pivot t when `mine` is set (wave-uniform); `tail` = the Pairs of that row, read for the pairs beyond the
// register window only. Everything else as ranktab_build_each.
template <bool NARROW>
__device__ __forceinline__ uint32_t ranktab_build_rows(const RankTab& T, const RtRow<NARROW>& pr, uint32_t shape, bool mine, int t, const Pairs& tail,
                                                       uint32_t* scan, int tid, int nthreads) {
    const int lane = tid & (WAVE - 1);
    const uint32_t nnz = mine ? shape & 0xFFFFu : 0u, ns = shape >> 16;
    return ranktab_build_each<NARROW>(T, [&](auto f) {
#pragma unroll
        for (int c = 0; c < RT_CHUNKS; c++) {
            const uint32_t j = rt_pair(c, lane);
            if (j < nnz) f(make_uint2(pr.key(c), pr.v[c]), NARROW ? j >= ns : false, t);
        }
        for (uint32_t j = RT_CHUNKS * WAVE + lane; j < nnz; j += WAVE) f(tail.raw(j), j >= ns, t);
    }, scan, tid, nthreads);
}

// NB streamed rows against the table at once: acc[r][0..7] += per-pivot sums of this lane's pairs of row r.
// All bitmap reads of the batch are issued before the first value read; the value reads follow in two halves (chunks
// 0-1, then 2-3 of every row), each issued whole before its multiplies: three LDS round trips per batch whatever NB
// is, and at most NB x 2 x 8 value registers in flight. shape[r] = nnz | ns << 16 of row r (wave-uniform;
// 0: the row is not there); tail(r) gives the Pairs of row r for the pairs beyond the register window.
template <bool NARROW, int NB, typename TailFn>
__device__ __forceinline__ void ranktab_probe_rows(const RankTab& T, const RtRow<NARROW> (&rows)[NB], const uint32_t (&shape)[NB], TailFn tail,
                                                   uint32_t n_ovf, float (&acc)[NB][RT_T], int lane) {
    static_assert(RT_CHUNKS % 2 == 0, "the value reads go out in two halves");
    auto add8 = [&](int r, float m, const float4& lo, const float4& hi) {
        acc[r][0] = fmaf(m, lo.x, acc[r][0]);
        acc[r][1] = fmaf(m, lo.y, acc[r][1]);
        acc[r][2] = fmaf(m, lo.z, acc[r][2]);
        acc[r][3] = fmaf(m, lo.w, acc[r][3]);
        acc[r][4] = fmaf(m, hi.x, acc[r][4]);
        acc[r][5] = fmaf(m, hi.y, acc[r][5]);
        acc[r][6] = fmaf(m, hi.z, acc[r][6]);
        acc[r][7] = fmaf(m, hi.w, acc[r][7]);
    };
    auto overflow = [&](int r, uint32_t key, uint32_t val_bits, bool in) {
        for (uint32_t o = 0; o < n_ovf; o++) { // wave-uniform count, zero for narrow corpora
            if (in && T.ovf_key[o] == key) add8(r, __uint_as_float(val_bits), T.ovf_val[2 * o], T.ovf_val[2 * o + 1]);
        }
    };
    auto index_of = [&](int r, int c) {
        const uint32_t key = rows[r].key(c);
        return ranktab_index<NARROW>(T, key, NARROW ? rt_pair(c, lane) >= (shape[r] >> 16) : (int)key < 0);
    };
    uint2 w[NB][RT_CHUNKS];
#pragma unroll
    for (int r = 0; r < NB; r++) {
        const uint32_t nnz = shape[r] & 0xFFFFu;
#pragma unroll
        for (int c = 0; c < RT_CHUNKS; c++) w[r][c] = T.word[rt_pair(c, lane) < nnz ? index_of(r, c) >> 5 : 0u];
    }
#pragma unroll
    for (int r = 0; r < NB; r++) asm volatile("" : "+v"(w[r][0].x), "+v"(w[r][1].x), "+v"(w[r][2].x), "+v"(w[r][3].x));
#pragma unroll
    for (int h = 0; h < RT_CHUNKS; h += 2) {
        RankProbe p[NB][2];
        float4 lo[NB][2], hi[NB][2];
        bool ok[NB][2];
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t nnz = shape[r] & 0xFFFFu;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const bool in = rt_pair(h + c, lane) < nnz;
                p[r][c] = ranktab_locate<NARROW>(T, w[r][h + c], index_of(r, h + c), rows[r].v[h + c], in);
                lo[r][c] = T.vals[p[r][c].slot];
                hi[r][c] = T.vals[T.slot_cap + p[r][c].slot];
                ok[r][c] = true;
                if (!NARROW) ok[r][c] = p[r][c].mul == 0.f || T.keys[p[r][c].slot] == rows[r].key(h + c);
            }
        }
#pragma unroll
        for (int r = 0; r < NB; r++) asm volatile("" : "+v"(lo[r][0].x), "+v"(lo[r][1].x), "+v"(hi[r][0].x), "+v"(hi[r][1].x));
#pragma unroll
        for (int r = 0; r < NB; r++) {
            const uint32_t nnz = shape[r] & 0xFFFFu;
#pragma unroll
            for (int c = 0; c < 2; c++) add8(r, ok[r][c] ? p[r][c].mul : 0.f, lo[r][c], hi[r][c]);
            if (!NARROW && n_ovf) {
#pragma unroll
                for (int c = 0; c < 2; c++) overflow(r, rows[r].key(h + c), rows[r].v[h + c], rt_pair(h + c, lane) < nnz && !ok[r][c]);
            }
        }
    }
    // rows longer than the register window
#pragma unroll
    for (int r = 0; r < NB; r++) {
        const uint32_t nnz = shape[r] & 0xFFFFu, ns = shape[r] >> 16;
        if (nnz > RT_CHUNKS * WAVE) {
            const Pairs sp = tail(r);
            for (uint32_t j0 = RT_CHUNKS * WAVE; j0 < nnz; j0 += WAVE) {
                const uint32_t j = j0 + lane;
                const bool in = j < nnz;
                const uint2 kv = in ? sp.raw(j) : make_uint2(0u, 0u);
                const uint32_t ix = ranktab_index<NARROW>(T, kv.x, NARROW ? j >= ns : (int)kv.x < 0);
                const uint2 ww = T.word[in ? ix >> 5 : 0u];
                const RankProbe q = ranktab_locate<NARROW>(T, ww, ix, kv.y, in);
                const float4 vl = T.vals[q.slot], vh = T.vals[T.slot_cap + q.slot];
                bool good = true;
                if (!NARROW) good = q.mul == 0.f || T.keys[q.slot] == kv.x;
                add8(r, good ? q.mul : 0.f, vl, vh);
                if (!NARROW && n_ovf) overflow(r, kv.x, kv.y, in && !good);
            }
        }
    }
}

// The wave totals of 2 streamed rows x 8 pivots from the per-lane accumulators of ranktab_probe_rows<., 2>. The two
// halves of the pivots (0-3, 4-7) of each row are reduced inside every 16-lane row of the wave like four sums at once
// (two exchange-and-add steps inside each quad leave lane l with pivot t(l) = 2 * (l & 1) + ((l >> 1) & 1) of its half,
// then two rotations inside the 16 lanes); the four 16-lane rows of the wave then share out the four (streamed row,
// half) combinations between them with three cross-row exchanges. Returns the total of streamed row *r_out, pivot *t_out.
__device__ __forceinline__ float wave_sum_2x8(const float (&acc)[2][RT_T], int lane, uint32_t* t_out, uint32_t* r_out) {
    float z[4]; // (row 0, low half), (row 0, high half), (row 1, low), (row 1, high)
    const bool odd = lane & 1, hi = lane & 2;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const float* a = &acc[k >> 1][4 * (k & 1)];
        const float keep0 = odd ? a[2] : a[0], keep1 = odd ? a[3] : a[1];
        const float give0 = odd ? a[0] : a[2], give1 = odd ? a[1] : a[3];
        const float x0 = keep0 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give0), 0xB1, 0xF, 0xF, false));
        const float x1 = keep1 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give1), 0xB1, 0xF, 0xF, false));
        const float keep = hi ? x1 : x0, give = hi ? x0 : x1;
        float y = keep + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give), 0x4E, 0xF, 0xF, false));
        y += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, y), 0x124, 0xF, 0xF, false)); // row_ror:4
        y += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, y), 0x128, 0xF, 0xF, false)); // row_ror:8
        z[k] = y;
    }
    const bool q0 = lane & 16, q1 = lane & 32;
    const float keepA0 = q0 ? z[2] : z[0], giveA0 = q0 ? z[0] : z[2];
    const float keepA1 = q0 ? z[3] : z[1], giveA1 = q0 ? z[1] : z[3];
    const float xa = keepA0 + __shfl_xor(giveA0, 16, WAVE);
    const float xb = keepA1 + __shfl_xor(giveA1, 16, WAVE);
    const float keepB = q1 ? xb : xa, giveB = q1 ? xa : xb;
    // 16-lane row q of the wave now holds combination k(q) = 2 * (q & 1) + (q >> 1): streamed row k >> 1, half k & 1
    const uint32_t k = 2u * ((lane >> 4) & 1) + ((lane >> 5) & 1);
    *r_out = k >> 1;
    *t_out = 4u * (k & 1) + 2u * (lane & 1) + ((lane >> 1) & 1);
    return keepB + __shfl_xor(giveB, 32, WAVE);
}

// The wave totals of one streamed row x 8 pivots from the per-lane accumulators of ranktab_probe_rows<., 1>: as
// wave_sum_2x8 with two (low half, high half) instead of four combinations. Returns the total of pivot *t_out.
__device__ __forceinline__ float wave_sum_1x8(const float (&acc)[RT_T], int lane, uint32_t* t_out) {
    float z[2];
    const bool odd = lane & 1, hi = lane & 2;
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const float* a = &acc[4 * k];
        const float keep0 = odd ? a[2] : a[0], keep1 = odd ? a[3] : a[1];
        const float give0 = odd ? a[0] : a[2], give1 = odd ? a[1] : a[3];
        const float x0 = keep0 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give0), 0xB1, 0xF, 0xF, false));
        const float x1 = keep1 + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give1), 0xB1, 0xF, 0xF, false));
        const float keep = hi ? x1 : x0, give = hi ? x0 : x1;
        float y = keep + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give), 0x4E, 0xF, 0xF, false));
        y += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, y), 0x124, 0xF, 0xF, false)); // row_ror:4
        y += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, y), 0x128, 0xF, 0xF, false)); // row_ror:8
        z[k] = y;
    }
    const bool q0 = lane & 16;
    const float keep = q0 ? z[1] : z[0], give = q0 ? z[0] : z[1];
    float x = keep + __shfl_xor(give, 16, WAVE);
    x += __shfl_xor(x, 32, WAVE);
    *t_out = 4u * ((lane >> 4) & 1) + 2u * (lane & 1) + ((lane >> 1) & 1);
    return x;
}

#endif // __HIPCC__

} // namespace apoe
