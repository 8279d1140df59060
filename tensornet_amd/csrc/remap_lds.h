// Key remap through LDS: the fast path of the per-slot first-occurrence remap
// (core/kernels/sparse_table_ops.cc:119-131) for large batches.
//
// A global hash table costs one or two random 64-byte granules and up to two
// device atomics per lookup.  Here every tile of 2048 consecutive lookups first
// combines its own repeats in an LDS hash table and hands one record per
// distinct sign to a bucket chosen by the slot and a hash of the sign (fixed
// room per bucket; the only global atomics are one per tile and run of
// records for a bucket); then one workgroup per bucket builds the bucket's
// hash table in LDS -- sign, smallest position, number of occurrences -- and
// writes for the first occurrence of every tile the position of the sign's
// first occurrence in the slot.  All records of one (slot, sign) land in one
// bucket, a bucket belongs to one slot, and the positions it writes to lie
// inside that slot's window of the concatenated lookup order, so the scatter
// back stays local.
//
//   k_tile_dedup   per tile of 2048 lookups: LDS hash table -> first position of every sign inside the tile,
//                  one record per distinct sign of the tile handed to its bucket (+ fingerprints of the signs)
//   k_lds_dedup    per bucket: LDS hash table -> first position in the slot, occurrence counts
//   k_lds_flags    first-occurrence flags per tile (coalesced: first_of[gi] == gi)
//   k_lds_assign   ranks, distinct lists, show counts; the tiles' offsets come from a sum over the
//                  counts of the tiles before (k_scan_tiles, shared with the global-table path,
//                  only when there are too many tiles for that)
//   k_lds_mapped   mapped ids and the per-lookup distinct index
//
// With at most 128 slots the groups of equal signs over all slots come out of
// LDS too: k_lds_dedup hands every distinct (slot, sign) record -- sign, first
// position, occurrences, slot -- to a second level of buckets chosen by the sign's
// hash alone (fixed room per bucket, one global atomic per touched bucket), and
// one workgroup per such bucket (k_group_count) finds the signs shared between
// slots with an LDS table of slot masks; k_group_emit numbers the groups from the
// counts of the buckets before its own (summed by itself, or by the scan
// k_group_offsets when there are too many buckets) and writes their member lists.
//
// If an LDS table ever overflows (more distinct signs in a bucket than it has
// room for) DEV_ERR_REMAP_OVERFLOW is raised; every index written stays in
// bounds and the host repeats the call on the global-table path.
#ifndef TN_REMAP_LDS_H_
#define TN_REMAP_LDS_H_

#include "sparse_kernels.h"

namespace tn {

constexpr int LDS_TILE = 2048;          // lookups per tile of the partition kernel
constexpr int TILE_THREADS = 512;
constexpr int TILE_ITEMS = LDS_TILE / TILE_THREADS;
constexpr int TILE_TABLE = 2 * LDS_TILE;  // entries of a tile's LDS hash table: two per lookup
static_assert(LDS_TILE % TILE_THREADS == 0, "whole rounds");
constexpr int L1_ROOM = 1536;           // room of a first-level bucket
constexpr int LDS_MAX_SUB = 4096;       // buckets per slot at most
constexpr int LDS_TABLE = 2048;         // entries of a bucket's LDS hash table (> L1_ROOM: an insert always ends)
constexpr int DEDUP_THREADS = 512;      // a bucket's phases are short and separated by barriers: many wavefronts hide them
constexpr int DEDUP_ITEMS = L1_ROOM / DEDUP_THREADS;  // records a thread of k_lds_dedup holds in registers
static_assert(L1_ROOM % DEDUP_THREADS == 0 && L1_ROOM < LDS_TABLE, "a bucket fits its table and the registers of one workgroup");
constexpr int LDS_SPAN2 = 512;          // second-level buckets whose counts one first-level bucket gathers in LDS
constexpr int GRP_TARGET = 1024;        // records per second-level bucket if every lookup were distinct
constexpr int GRP_CAP = 1536;           // room of a second-level bucket
constexpr int GRP_TABLE = 2048;         // entries of its LDS hash table (> GRP_CAP: an insert always ends)
constexpr int GRP_THREADS = 512;        // threads of k_group_count
constexpr int GRP_RECS = GRP_CAP / GRP_THREADS;  // records per thread of a second-level bucket's workgroup
static_assert(GRP_CAP % GRP_THREADS == 0 && GRP_CAP % 256 == 0 && GRP_CAP < GRP_TABLE, "a bucket fits its table and the registers of one workgroup");
constexpr int EMIT_THREADS = 512;
constexpr int EMIT_RECS = GRP_CAP / EMIT_THREADS;  // records per thread of k_group_emit
constexpr int GRP_ITEMS = (GRP_TABLE + 1 + GRP_THREADS - 1) / GRP_THREADS;
constexpr int GRP_SLOTS = 128;          // slot masks are 128 bits wide
static_assert((uint64_t)LDS_MAX_SUB * L1_ROOM <= 0x7FFFFFull && GRP_SLOTS <= 256,
              "a record's word holds the occurrences of a sign in its slot and the slot");

// Raises DEV_ERR_REMAP_OVERFLOW.  A batch that overflows does so in a million places at once: atomics on the one
// word would queue up for milliseconds, so only those that do not see the flag yet set it.
__device__ __forceinline__ void flag_overflow(DevStatus* status) {
    if (!(ld_relaxed(&status->err) & DEV_ERR_REMAP_OVERFLOW)) atomicOr(&status->err, DEV_ERR_REMAP_OVERFLOW);
}

// A distinct (slot, sign) record on its way to the grouping.
struct GroupRec {
    uint64_t sign;
    uint32_t gi;   // position of its first occurrence
    uint32_t cnt;  // bits 0-22 occurrences in its slot, 23 all of them within one tile, 24-31 the slot (< GRP_SLOTS)
};
constexpr uint32_t REC_CNT_MASK = 0x7FFFFFu;
constexpr uint32_t REC_ONE_TILE = 0x800000u;


// [0, n) from a 32-bit hash without a division; grows with the hash
__device__ __forceinline__ uint32_t scale32(uint32_t h, uint32_t n) { return __umulhi(h, n); }

// First-level bucket of a slot, place in a tile's LDS table, second-level bucket, home slot in the table: all
// grow with the one hash of the sign (the first two with its upper half).  The signs of a first-level bucket
// therefore go to a few neighbouring second-level buckets, whose cursors its workgroup gathers in LDS, and the
// signs of a second-level bucket lie in one stretch of the table, which keeps the probes of a workgroup within
// few pages.
__device__ __forceinline__ uint32_t group_bucket(uint64_t sign, uint32_t nb2) {
    return (uint32_t)__umul64hi(mix64(sign), (uint64_t)nb2);
}

// What a tile hands to a first-level bucket: one record per distinct sign of the tile (per slot, where a tile
// spans several).  y: bits 0-31 the position of the sign's first occurrence in the tile, 32-43 its occurrences in
// the tile (1 .. LDS_TILE), 44-55 the slot.
__device__ __forceinline__ ulonglong2 tile_record(uint64_t sign, uint32_t gi, uint32_t cnt, uint32_t slot) {
    return make_ulonglong2(sign, (uint64_t)gi | ((uint64_t)cnt << 32) | ((uint64_t)slot << 44));
}
static_assert(LDS_TILE < (1 << 12) && MAX_SLOTS < (1 << 12), "a tile record's fields");

// The first pass over the lookups.  A tile of LDS_TILE consecutive lookups first combines its own repeats in an
// LDS hash table -- every lookup learns the first position of its sign inside the tile (first_of, written in
// order) -- and hands ONE record per distinct sign on to the sign's first-level bucket: sign, first position in
// the tile, occurrences in the tile.  However often a sign occurs in a slot, it puts at most one record per tile
// into its bucket, so buckets of fixed room do (bcursor[b] = records handed to bucket b, the records at
// prec[b * L1_ROOM ...]); no histogram of the lookups and no scan of bucket sizes is needed, and the passes that
// follow work on the tiles' distinct signs instead of on the lookups.
//
// The table has two entries per lookup of the tile.  The lookups of a slot own the entries [2 a, 2 b) if they sit
// at the tile's positions [a, b): tiles that span slots (any number of them) keep the slots apart without a pass
// per slot.  The last entry of a slot's range belongs to the sign that equals EMPTY_KEY; the others are filled by
// linear probing.  The lookup that turns out to be its sign's first in the tile hands the record on: it holds the
// sign and its hash in registers already, so the table is never walked (most of its entries are free, and a walk
// pays for every one of them).  Places in the buckets: an LDS counter per bucket the tile can touch gives a
// record its place among the tile's records for the bucket, one global atomic per touched bucket reserves the
// tile's slice of it.
//
// It also leaves the fingerprints of the batch's signs, which a push compares its own with (k_verify_values: one
// per 64 strided lookups of a tile of 256 x 8, which are the lookups of the wavefronts w and w + 4 here), and,
// with exact != nullptr, a copy of the signs.
static_assert(LDS_TILE == VERIFY_TILE && TILE_THREADS == 512, "k_tile_dedup and k_verify_values fingerprint the same runs of lookups");
constexpr int TILE_LDS_SLOTS = 128;  // up to this many slots their value pointers and bucket ranges sit in LDS
constexpr int LDS_SPAN = 4096;       // first-level buckets one tile may touch (its LDS counters)
// dynamic LDS of k_tile_dedup: lb[N + 1], then (few slots) the slots' value pointers and bucket ranges, then a
// counter per bucket the widest tile touches
inline size_t tile_dedup_lds(int N, uint32_t span_cap) {
    const size_t lb = align_up(((size_t)N + 1) * sizeof(uint32_t), 8);
    return (N <= TILE_LDS_SLOTS ? lb + (size_t)N * (sizeof(uint64_t) + sizeof(uint2)) : lb) + (size_t)span_cap * sizeof(uint32_t);
}
__global__ __launch_bounds__(TILE_THREADS) __attribute__((amdgpu_waves_per_eu(6, 8))) void k_tile_dedup(const SlotDesc* __restrict__ descs,
                                                             const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                             uint32_t* bcursor, ulonglong2* __restrict__ prec,
                                                             ulonglong2* __restrict__ prints,
                                                             uint64_t* __restrict__ exact,
                                                             uint32_t* __restrict__ first_of, DevStatus* status,
                                                             uint32_t span_cap) {
    extern __shared__ uint32_t lb[];  // lb[N + 1], sized by the launch; then vals[N], tb[N], hist[span_cap] (see tile_dedup_lds)
    __shared__ unsigned long long keys[TILE_TABLE];
    __shared__ uint32_t word[TILE_TABLE];  // bits 16-31 smallest position in the tile, 0-15 occurrences
    __shared__ ulonglong2 fp[TILE_THREADS / 64];
    // With few slots everything a tile needs of its slots' descriptors comes in with the slots' first lookups, in
    // one round trip, instead of in a second one once the tile knows its slot.
    const bool lds_descs = N <= TILE_LDS_SLOTS;
    const int64_t** vals = reinterpret_cast<const int64_t**>(lb + ((N + 2) & ~1));
    uint2* tb = reinterpret_cast<uint2*>(vals + N);
    uint32_t* hist = lds_descs ? reinterpret_cast<uint32_t*>(tb + N) : lb + ((N + 2) & ~1);
    for (int i = threadIdx.x; i <= N; i += TILE_THREADS) {
        lb[i] = lbase[i];
        if (lds_descs && i < N) {
            vals[i] = descs[i].values;
            tb[i] = make_uint2(descs[i].tbase, descs[i].tcap);
        }
    }
    __syncthreads();
    auto slot_values = [&](int sl) { return lds_descs ? vals[sl] : descs[sl].values; };
    auto slot_buckets = [&](int sl) { return lds_descs ? tb[sl] : make_uint2(descs[sl].tbase, descs[sl].tcap); };
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t ntiles = (L + LDS_TILE - 1) / LDS_TILE;
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const uint32_t g0 = tile * LDS_TILE;
        const uint32_t g1 = min(L, g0 + (uint32_t)LDS_TILE) - 1;
        const uint32_t n_tile = g1 - g0 + 1;
        const int s0 = find_slot(lb, N, g0);
        const bool one_slot = g1 < lb[s0 + 1];  // the usual case: the slot's values and buckets sit in registers
        const int64_t* v0 = slot_values(s0) - lb[s0];
        uint64_t sg[TILE_ITEMS];
        int sl[TILE_ITEMS];
#pragma unroll
        for (int j = 0; j < TILE_ITEMS; j++) {
            const uint32_t gi = g0 + j * TILE_THREADS + threadIdx.x;
            sg[j] = 0;
            sl[j] = s0;
            if (gi <= g1) {
                if (one_slot) {
                    sg[j] = (uint64_t)v0[gi];
                } else {
                    sl[j] = find_slot(lb, N, gi);
                    sg[j] = (uint64_t)slot_values(sl[j])[gi - lb[sl[j]]];
                }
            }
        }
        // buckets the tile can touch: from the first bucket of its first slot to the last bucket of its last slot
        // (span_cap at most: the host sizes the counters for the widest tile of the call, LDS_SPAN at most)
        const uint2 b0 = slot_buckets(s0);
        uint32_t span = b0.y;
        if (!one_slot) {
            const uint2 bl = slot_buckets(find_slot(lb, N, g1));
            span = bl.x + bl.y - b0.x;
        }
        span = min(span, span_cap);
        for (int i = threadIdx.x; i < TILE_TABLE; i += TILE_THREADS) {
            keys[i] = EMPTY_KEY;
            word[i] = 0xFFFF0000u;
        }
        for (uint32_t i = threadIdx.x; i < span; i += TILE_THREADS) hist[i] = 0;
        // the hash of every sign once: fingerprint, place in the table, bucket
        uint32_t hs[TILE_ITEMS];
        {
            Fingerprint print;
#pragma unroll
            for (int j = 0; j < TILE_ITEMS; j++) {
                const uint32_t gi = g0 + j * TILE_THREADS + threadIdx.x;
                const uint64_t m = mix64(sg[j]);
                hs[j] = (uint32_t)(m >> 32);
                if (gi <= g1) {
                    print.add_mixed(gi, m);
                    if (exact) exact[gi] = sg[j];  // a push is to compare the signs themselves
                }
            }
            print.wave_sum();
            if (lane == 0) fp[wave] = make_ulonglong2(print.a, print.b);
        }
        __syncthreads();
        if (threadIdx.x < 4)
            prints[tile * 4 + threadIdx.x] = make_ulonglong2(fp[threadIdx.x].x + fp[threadIdx.x + 4].x,
                                                             fp[threadIdx.x].y + fp[threadIdx.x + 4].y);
        // every lookup finds or claims the entry of its sign and lowers the entry's position to its own
        uint32_t ent[TILE_ITEMS];
#pragma unroll
        for (int j = 0; j < TILE_ITEMS; j++) {
            const uint32_t pos = j * TILE_THREADS + threadIdx.x;
            ent[j] = 0;
            if (pos >= n_tile) continue;
            uint32_t a = 0, m = n_tile;  // the slot's lookups sit at the tile's positions [a, a + m)
            if (!one_slot) {
                a = max(lb[sl[j]], g0) - g0;
                m = min(lb[sl[j] + 1], g1 + 1) - g0 - a;
            }
            const uint32_t lo = 2 * a, size = 2 * m - 1;
            uint32_t e = lo + size;  // the entry of the sign EMPTY_KEY
            if (sg[j] != EMPTY_KEY) {
                e = lo + scale32(hs[j], size);
                for (;;) {  // at most m distinct signs in 2 m - 1 entries: a free one exists
                    const unsigned long long old = atomicCAS(&keys[e], (unsigned long long)EMPTY_KEY, sg[j]);
                    if (old == EMPTY_KEY || old == sg[j]) break;
                    e = (e + 1 == lo + size) ? lo : e + 1;
                }
            }
            atomicMin(&word[e], pos << 16);
            ent[j] = e;
        }
        __syncthreads();
        // ... counts itself there and reads the sign's first position in the tile; the lookup at that position
        // takes a place among the tile's records for its bucket
        uint32_t place[TILE_ITEMS];  // 0xFFFFFFFF: not a first occurrence (or no lookup)
        uint32_t bloc[TILE_ITEMS];   // the bucket, counted from the tile's first
#pragma unroll
        for (int j = 0; j < TILE_ITEMS; j++) {
            const uint32_t pos = j * TILE_THREADS + threadIdx.x;
            place[j] = 0xFFFFFFFFu;
            bloc[j] = 0;
            if (pos >= n_tile) continue;
            const uint32_t old = atomicAdd(&word[ent[j]], 1u);
            const uint32_t f = old >> 16;
            first_of[g0 + pos] = g0 + f;
            if (f == pos) {
                const uint2 bb = one_slot ? b0 : slot_buckets(sl[j]);
                bloc[j] = bb.x + scale32(hs[j], bb.y) - b0.x;
                if (bloc[j] < span)
                    place[j] = atomicAdd(&hist[bloc[j]], 1u);
                else
                    flag_overflow(status);  // (more buckets under one tile than it has counters for)
            }
        }
        __syncthreads();
        // the tile's slice of every bucket it touches; all atomics of a thread are in flight together
        for (uint32_t i0 = 0; i0 < span; i0 += TILE_THREADS * 4) {
            uint32_t got[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t i = i0 + q * TILE_THREADS + threadIdx.x;
                const uint32_t cnt = i < span ? hist[i] : 0;
                got[q] = cnt ? atomicAdd(&bcursor[b0.x + i], cnt) : 0;
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t i = i0 + q * TILE_THREADS + threadIdx.x;
                if (i < span) hist[i] = got[q];
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < TILE_ITEMS; j++) {
            if (place[j] == 0xFFFFFFFFu) continue;
            const uint32_t pos = j * TILE_THREADS + threadIdx.x;
            const uint32_t at = hist[bloc[j]] + place[j];
            if (at < (uint32_t)L1_ROOM)
                prec[(size_t)(b0.x + bloc[j]) * L1_ROOM + at] =
                    tile_record(sg[j], g0 + pos, word[ent[j]] & 0xFFFFu, (uint32_t)sl[j]);
            else
                flag_overflow(status);
        }
        __syncthreads();
    }
}

__device__ __forceinline__ uint32_t lds_slot(uint64_t sign) { return (uint32_t)(mix64(sign) >> 7) & (LDS_TABLE - 1); }

// One workgroup per first-level bucket: the records its tiles handed in, one per distinct sign of a tile, are
// combined in an LDS hash table -- sign, smallest position, occurrences.  first_of[position of a tile's first
// occurrence] = position of the sign's first occurrence in its slot (k_tile_dedup left the tile's own there, and
// left every other lookup pointing at its tile's: two hops from any lookup); cnt_at[first position] =
// occurrences of the sign.  With EMIT every distinct sign of the bucket is also appended to its second-level
// bucket (recs[c * GRP_CAP ...], cursor2[c] = records handed in).
template <bool EMIT>
__global__ __launch_bounds__(DEDUP_THREADS) void k_lds_dedup(const uint32_t* __restrict__ bcursor, uint32_t nbuckets,
                                                   const ulonglong2* __restrict__ prec,
                                                   uint32_t* __restrict__ first_of, uint32_t* __restrict__ cnt_at,
                                                   DevStatus* status, uint32_t nb2, uint32_t* cursor2,
                                                   GroupRec* __restrict__ recs) {
    __shared__ unsigned long long keys[LDS_TABLE + 1];  // entry LDS_TABLE: the sign EMPTY_KEY itself
    __shared__ uint32_t minpos[LDS_TABLE + 1];
    __shared__ uint32_t cnts[LDS_TABLE + 1];
    __shared__ uint32_t hist2[EMIT ? LDS_SPAN2 : 1];
    __shared__ uint32_t c_lo_sh, slot_sh;
    // The buckets of a slot scatter four-byte words over the same stretch of first_of and cnt_at (the slot's
    // positions): on one die they meet in one L2 and leave it as whole lines.
    const DieShare share(nbuckets);
    for (uint32_t b = share.first; b < share.end; b += share.step) {
        const uint32_t n = min(bcursor[b], (uint32_t)L1_ROOM);
        if (n == 0) continue;
        const size_t first = (size_t)b * L1_ROOM;
        // The bucket's records sit in registers, all loads issued together and in flight while the tables
        // are cleared.
        uint64_t sg[DEDUP_ITEMS];
        uint32_t gp[DEDUP_ITEMS], mu[DEDUP_ITEMS];
#pragma unroll
        for (int j = 0; j < DEDUP_ITEMS; j++) {
            const uint32_t i = j * DEDUP_THREADS + threadIdx.x;
            const ulonglong2 r = (i < n) ? prec[first + i] : make_ulonglong2(0, 0xFFFFFFFFull);  // no position: nothing to do
            sg[j] = r.x;
            gp[j] = (uint32_t)r.y;
            mu[j] = (uint32_t)(r.y >> 32) & 0xFFFu;
            if (EMIT && i == 0) slot_sh = (uint32_t)(r.y >> 44);  // every record of a bucket is of one slot
        }
        for (int i = threadIdx.x; i <= LDS_TABLE; i += DEDUP_THREADS) {
            keys[i] = EMPTY_KEY;
            minpos[i] = 0xFFFFFFFFu;
            cnts[i] = 0;
        }
        if (EMIT) {
            for (int i = threadIdx.x; i < LDS_SPAN2; i += DEDUP_THREADS) hist2[i] = 0;
            if (threadIdx.x == 0) c_lo_sh = 0xFFFFFFFFu;
        }
        __syncthreads();
        uint32_t c_min = 0xFFFFFFFFu;
        uint32_t hs[DEDUP_ITEMS];
#pragma unroll
        for (int j = 0; j < DEDUP_ITEMS; j++) {
            const uint64_t sign = sg[j];
            const uint32_t gi = gp[j];
            hs[j] = LDS_TABLE;
            if (gi == 0xFFFFFFFFu) continue;
            if (EMIT) c_min = min(c_min, group_bucket(sign, nb2));
            uint32_t h = LDS_TABLE;
            if (sign != EMPTY_KEY) {
                h = lds_slot(sign);
                for (;;) {  // at most L1_ROOM < LDS_TABLE distinct signs: a free entry exists
                    unsigned long long old = keys[h];
                    if (old == EMPTY_KEY) old = atomicCAS(&keys[h], (unsigned long long)EMPTY_KEY, sign);
                    if (old == EMPTY_KEY || old == sign) break;
                    h = (h + 1) & (LDS_TABLE - 1);
                }
            }
            atomicMin(&minpos[h], gi);
            atomicAdd(&cnts[h], mu[j]);
            hs[j] = h;
        }
        if (EMIT) {
            for (int o = 32; o > 0; o >>= 1) c_min = min(c_min, (uint32_t)__shfl_xor((int)c_min, o));
            if ((threadIdx.x & 63) == 0) atomicMin(&c_lo_sh, c_min);
        }
        __syncthreads();
        const uint32_t c_lo = EMIT ? c_lo_sh : 0;
#pragma unroll
        for (int j = 0; j < DEDUP_ITEMS; j++) {
            const uint32_t gi = gp[j];
            if (gi == 0xFFFFFFFFu) continue;
            const uint32_t h = hs[j];
            const uint32_t f = minpos[h];
            if (f != gi) {
                first_of[gi] = f;  // k_tile_dedup left first_of[gi] = gi
            } else {
                if (!EMIT) cnt_at[gi] = cnts[h];  // with EMIT the record carries the count
                if (EMIT) {  // one record per occupied entry gets here
                    // the sign's only record: all its lookups lie in one tile (what a push makes of it: the tile's
                    // click sum for the sign is the whole sum)
                    if (cnts[h] == mu[j]) cnts[h] |= REC_ONE_TILE;
                    const uint32_t local = group_bucket(sg[j], nb2) - c_lo;
                    if (local < LDS_SPAN2) atomicAdd(&hist2[local], 1u);
                }
            }
        }
        if (EMIT) {
            __syncthreads();
            for (int i = threadIdx.x; i < LDS_SPAN2; i += DEDUP_THREADS)
                if (hist2[i]) hist2[i] = atomicAdd(&cursor2[c_lo + i], hist2[i]);  // this bucket's slice
            __syncthreads();
            for (int e = threadIdx.x; e <= LDS_TABLE; e += DEDUP_THREADS) {
                const uint32_t cnt = cnts[e];  // (with the one-tile mark)
                if (cnt == 0) continue;
                GroupRec r;
                r.sign = (e == LDS_TABLE) ? EMPTY_KEY : (uint64_t)keys[e];
                r.gi = minpos[e];
                r.cnt = cnt | (slot_sh << 24);
                const uint32_t c = group_bucket(r.sign, nb2);
                const uint32_t local = c - c_lo;
                const uint32_t at = (local < LDS_SPAN2) ? atomicAdd(&hist2[local], 1u) : atomicAdd(&cursor2[c], 1u);
                if (at < (uint32_t)GRP_CAP)
                    recs[(size_t)c * GRP_CAP + at] = r;
                else
                    flag_overflow(status);
            }
        }
        __syncthreads();
    }
}

// Rank of the first occurrence at position gi = number of first occurrences before it: the
// count up to its 64-lookup word (wordpre, written by k_lds_assign) plus the flags below it
// in the word.  Both arrays are small enough to stay in L2 (L / 8 and L / 16 bytes), so a
// rank costs two cache hits instead of a random read of a 4-byte-per-lookup array.
__device__ __forceinline__ uint32_t rank_of(const uint8_t* __restrict__ flag8, const uint32_t* __restrict__ wordpre,
                                            uint32_t gi) {
    const uint64_t word = reinterpret_cast<const uint64_t*>(flag8)[gi >> 6];
    return wordpre[gi >> 6] + (uint32_t)__popcll(word & ((1ull << (gi & 63)) - 1ull));
}

// Tile counts of first occurrences; a lookup is one iff first_of[gi] == gi.  The first workgroups also add up
// what the first-level buckets of every slot were handed: status->tile_share_q16 = the largest share
// records / lookups among the slots with more than one bucket's worth of lookups, in 1 / 65536 (the host sizes
// the next call's buckets from it).
__global__ __launch_bounds__(REMAP_THREADS) void k_lds_flags(uint32_t L, const uint32_t* __restrict__ first_of,
                                                             uint8_t* __restrict__ flag8,
                                                             uint32_t* __restrict__ tilesum,
                                                             const SlotDesc* __restrict__ descs, int N,
                                                             const uint32_t* __restrict__ bcursor,
                                                             DevStatus* status) {
    __shared__ uint32_t red[4];
    for (int sl = blockIdx.x; sl < N; sl += gridDim.x) {
        const SlotDesc& d = descs[sl];
        if (d.len <= (uint32_t)L1_ROOM) continue;  // (the same for the whole workgroup)
        uint32_t mine = 0;
        for (uint32_t b = threadIdx.x; b < d.tcap; b += REMAP_THREADS) mine += bcursor[d.tbase + b];
        const uint32_t all = block_sum_256(mine, red);
        if (threadIdx.x == 0) {
            const uint64_t q = ((uint64_t)all << 16) / d.len + 1;
            atomicMax(&status->tile_share_q16, (uint32_t)(q < 65536 ? q : 65536));
        }
        __syncthreads();
    }
    const uint32_t base = blockIdx.x * REMAP_TILE + threadIdx.x * REMAP_ITEMS;
    uint32_t bits = 0;
    static_assert(REMAP_ITEMS == 8, "a thread's lookups are two 16-byte loads");
    if (base + REMAP_ITEMS <= L) {
        const uint4 a = reinterpret_cast<const uint4*>(first_of + base)[0];
        const uint4 b = reinterpret_cast<const uint4*>(first_of + base)[1];
        bits = (a.x == base ? 1u : 0u) | (a.y == base + 1 ? 2u : 0u) | (a.z == base + 2 ? 4u : 0u) |
               (a.w == base + 3 ? 8u : 0u) | (b.x == base + 4 ? 16u : 0u) | (b.y == base + 5 ? 32u : 0u) |
               (b.z == base + 6 ? 64u : 0u) | (b.w == base + 7 ? 128u : 0u);
        flag8[base / REMAP_ITEMS] = (uint8_t)bits;
    } else if (base < L) {
        for (int j = 0; j < REMAP_ITEMS; j++) {
            const uint32_t gi = base + j;
            if (gi >= L) break;
            if (first_of[gi] == gi) bits |= 1u << j;
        }
        flag8[base / REMAP_ITEMS] = (uint8_t)bits;
    }
    uint32_t total = block_sum_256(__popc(bits), red);
    if (threadIdx.x == 0) tilesum[blockIdx.x] = total;
}

// Ranks of the first occurrences (per 64-lookup word: wordpre, see rank_of) and, with LISTS, the distinct
// lists and show counts.  Each thread owns 8 consecutive lookups; all loads are
// issued before any dependent store.
template <bool LISTS>
__global__ __launch_bounds__(REMAP_THREADS) void k_lds_assign(
    const SlotDesc* __restrict__ descs, const uint32_t* __restrict__ lbase, int N, uint32_t L,
    const uint8_t* __restrict__ flag8, const uint32_t* __restrict__ tileoff, const uint32_t* __restrict__ cnt_at,
    uint32_t* __restrict__ wordpre, uint32_t* __restrict__ ubase, uint64_t* __restrict__ uniq_sign,
    uint32_t* __restrict__ uniq_slot, uint32_t* __restrict__ ushow, const uint32_t* __restrict__ tilesum,
    DevStatus* status) {
    // lb[N + 1], sized by the launch: a fixed array for the largest slot count would take 16 KB of LDS per
    // workgroup away from the grouping kernel that runs beside this one
    extern __shared__ uint32_t lb[];
    __shared__ uint32_t red[4];
    load_lbase(lb, lbase, N);
    const uint32_t base = blockIdx.x * REMAP_TILE + threadIdx.x * REMAP_ITEMS;
    uint32_t bits = 0;
    if (base < L) bits = flag8[base / REMAP_ITEMS];
    uint32_t off;
    if (tilesum) {
        // a few thousand tiles: every workgroup adds up the counts of the tiles before its own (they sit in
        // L2), which costs less than a scan kernel of one workgroup between two launches
        uint32_t part = 0;
        for (uint32_t i = threadIdx.x; i < blockIdx.x; i += REMAP_THREADS) part += tilesum[i];
        off = block_sum_256(part, red);
    } else {
        off = tileoff[blockIdx.x];
    }
    uint32_t total;
    uint32_t u = off + block_excl_scan_256<uint32_t>(__popc(bits), red, &total);
    if (tilesum && blockIdx.x == gridDim.x - 1) {  // what k_scan_tiles leaves besides the offsets
        const uint32_t U = off + total;
        if (threadIdx.x == 0) {
            status->n_unique = U;
            const uint32_t g = U + U / 2;
            status->gcap = g < 16 ? 16 : g;
        }
        for (int sl = threadIdx.x; sl <= N; sl += REMAP_THREADS)
            if (lb[sl] >= L) ubase[sl] = U;
    }
    if (base >= L) return;
    if ((base & 63u) == 0) wordpre[base >> 6] = u;  // first occurrences before this 64-lookup word
    int sls[REMAP_ITEMS];
    uint64_t vals[REMAP_ITEMS];
    uint32_t cnts[REMAP_ITEMS];
    int sl = find_slot(lb, N, base);
#pragma unroll
    for (int j = 0; j < REMAP_ITEMS; j++) {
        const uint32_t gi = base + j;
        sls[j] = sl;
        vals[j] = 0;
        cnts[j] = 0;
        if (gi < L) {
            while (gi >= lb[sl + 1]) sl++;
            sls[j] = sl;
            if (LISTS && (bits & (1u << j))) {
                vals[j] = (uint64_t)descs[sl].values[gi - lb[sl]];
                cnts[j] = cnt_at[gi];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < REMAP_ITEMS; j++) {
        const uint32_t gi = base + j;
        if (gi >= L) break;
        sl = sls[j];
        if (gi == lb[sl]) {
            ubase[sl] = u;
            for (int e = sl - 1; e >= 0 && lb[e] == gi; e--) ubase[e] = u;
        }
        if (bits & (1u << j)) {
            if (LISTS) {
                uniq_sign[u] = vals[j];
                uniq_slot[u] = (uint32_t)sl;
                ushow[u] = cnts[j];  // batch_show = occurrences (sparse_table_ops.cc:290-293)
            }
            u++;
        }
    }
}

// mapped id = rank of the sign's first occurrence, relative to the slot.
__global__ __launch_bounds__(256) void k_lds_mapped(const SlotDesc* __restrict__ descs,
                                                    const uint32_t* __restrict__ lbase,
                                                    const uint32_t* __restrict__ ubase, int N, uint32_t L,
                                                    const uint32_t* __restrict__ first_of,
                                                    const uint8_t* __restrict__ flag8,
                                                    const uint32_t* __restrict__ wordpre,
                                                    uint32_t* __restrict__ u_of_gi) {
    extern __shared__ uint32_t lb[];  // lb[N + 1], sized by the launch (see k_lds_assign)
    load_lbase(lb, lbase, N);
    // four consecutive lookups per thread: one 16-byte load and store, one slot search
    const uint32_t stride = gridDim.x * blockDim.x;
    const uint32_t quads = (L + 3) / 4;
    for (uint32_t q = blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += stride) {
        const uint32_t g0 = q * 4;
        uint32_t f[4], u[4];
        if (g0 + 4 <= L) {
            const uint4 v = reinterpret_cast<const uint4*>(first_of)[q];
            f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) f[j] = g0 + j < L ? first_of[g0 + j] : 0u;
        }
        // A lookup points at the first occurrence inside its tile, which points at the first one in the slot
        // (itself, if it is that): the second hop stays inside the lookup's own tile for a repeat within a
        // tile, and is the identity for a first occurrence.
#pragma unroll
        for (int j = 0; j < 4; j++) f[j] = first_of[f[j]];
#pragma unroll
        for (int j = 0; j < 4; j++) u[j] = rank_of(flag8, wordpre, f[j]);
        if (g0 + 4 <= L) {
            reinterpret_cast<uint4*>(u_of_gi)[q] =
                make_uint4(u[0] | (f[0] == g0 ? FIRST_BIT : 0u), u[1] | (f[1] == g0 + 1 ? FIRST_BIT : 0u),
                           u[2] | (f[2] == g0 + 2 ? FIRST_BIT : 0u), u[3] | (f[3] == g0 + 3 ? FIRST_BIT : 0u));
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (g0 + j < L) u_of_gi[g0 + j] = u[j] | (f[j] == g0 + j ? FIRST_BIT : 0u);
        }
        int sl = find_slot(lb, N, g0);
        int64_t* out = descs[sl].mapped - lb[sl];
        uint32_t ub = ubase[sl];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t gi = g0 + j;
            if (gi >= L) break;
            if (gi >= lb[sl + 1]) {
                do sl++; while (gi >= lb[sl + 1]);
                out = descs[sl].mapped - lb[sl];
                ub = ubase[sl];
            }
            out[gi] = (int64_t)(u[j] - ub);
        }
    }
}

// One workgroup per second-level bucket: groups its records by sign (all slots
// of a sign meet here) with an LDS table of slot masks.  The place of a record
// among its group's members (ascending slot order) is the number of lower
// slots in the mask.  Per record it leaves
//   x: bits 0-11 index of its group among the bucket's groups of the same kind
//      (one record / several), 12-23 index among the bucket's big groups, 24-31 records k of the group
//   y: bits 0-15 records of the bucket's earlier several-record groups, 16-23 place, 24-31 slot
// and per bucket the number of groups with one record, with several, the
// records of the latter, and the big groups.  At most GRP_SLOTS slots.
// LDS of a workgroup that groups second-level buckets (group_count_bucket).
struct GroupCountLds {
    unsigned long long keys[GRP_TABLE + 1];  // entry GRP_TABLE: the sign EMPTY_KEY itself
    unsigned long long mlo[GRP_TABLE + 1], mhi[GRP_TABLE + 1];
    uint16_t rech[GRP_CAP];
    unsigned long long sh[GRP_THREADS / 64];
};

// One second-level bucket, by a workgroup of GRP_THREADS threads (the caller puts a barrier between two buckets).
__device__ __forceinline__ void group_count_bucket(uint32_t c, GroupCountLds& lds, const uint32_t* __restrict__ cursor2,
                                                   const GroupRec* __restrict__ recs, uint32_t big_k,
                                                   uint2* __restrict__ aux, uint4* __restrict__ bcounts) {
    unsigned long long* const keys = lds.keys;
    unsigned long long* const mlo = lds.mlo;
    unsigned long long* const mhi = lds.mhi;
    uint16_t* const rech = lds.rech;
    unsigned long long* const sh = lds.sh;
    // Once every record knows its entry (rech) the keys are dead: the entries' group numbers and offsets
    // take their place, which lets three workgroups instead of two share a CU's LDS.
    uint2* const einfo = reinterpret_cast<uint2*>(keys);  // x: info word, y: records before the group
    const uint32_t n = min(cursor2[c], (uint32_t)GRP_CAP);
    if (n == 0) {
        if (threadIdx.x == 0) bcounts[c] = make_uint4(0, 0, 0, 0);
        return;
    }
    const size_t first = (size_t)c * GRP_CAP;
    // all records of the bucket sit in registers (GRP_CAP = GRP_THREADS x GRP_RECS), loaded together
    // and in flight while the table is cleared
    uint64_t sg[GRP_RECS];
    uint32_t sl[GRP_RECS];  // slot of the record, 0xFFFFFFFF = no record
#pragma unroll
    for (int j = 0; j < GRP_RECS; j++) {
        const uint32_t i = j * GRP_THREADS + threadIdx.x;
        sg[j] = 0;
        sl[j] = 0xFFFFFFFFu;
        if (i < n) {
            const GroupRec r = recs[first + i];
            sg[j] = r.sign;
            sl[j] = r.cnt >> 24;
        }
    }
    for (int i = threadIdx.x; i <= GRP_TABLE; i += GRP_THREADS) {
        keys[i] = EMPTY_KEY;
        mlo[i] = 0;
        mhi[i] = 0;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < GRP_RECS; j++) {
        if (sl[j] == 0xFFFFFFFFu) continue;
        const uint64_t sign = sg[j];
        uint32_t h = GRP_TABLE;
        if (sign != EMPTY_KEY) {
            h = (uint32_t)(mix64(sign) >> 9) & (GRP_TABLE - 1);
            for (;;) {  // n <= GRP_CAP < GRP_TABLE: a free entry exists
                unsigned long long old = keys[h];
                if (old == EMPTY_KEY) old = atomicCAS(&keys[h], (unsigned long long)EMPTY_KEY, sign);
                if (old == EMPTY_KEY || old == sign) break;
                h = (h + 1) & (GRP_TABLE - 1);
            }
        }
        atomicOr(sl[j] < 64 ? &mlo[h] : &mhi[h], 1ull << (sl[j] & 63));
        rech[j * GRP_THREADS + threadIdx.x] = (uint16_t)h;
    }
    __syncthreads();
    uint32_t ks[GRP_ITEMS];
    unsigned long long v = 0;  // 16-bit fields: groups of one record, of several, records of those, big groups
    for (int j = 0; j < GRP_ITEMS; j++) {
        const uint32_t e = j * GRP_THREADS + threadIdx.x;
        const uint32_t k = (e <= GRP_TABLE) ? (uint32_t)(__popcll(mlo[e]) + __popcll(mhi[e])) : 0;
        ks[j] = k;
        if (k == 1) v += 1ull;
        if (k > 1) v += (1ull << 16) + ((unsigned long long)k << 32) + (is_big(k, big_k) ? 1ull << 48 : 0ull);
    }
    unsigned long long total;
    unsigned long long ex = block_excl_scan<unsigned long long, GRP_THREADS / 64>(v, sh, &total);
    if (threadIdx.x == 0)
        bcounts[c] = make_uint4((uint32_t)(total & 0xFFFF), (uint32_t)((total >> 16) & 0xFFFF),
                                (uint32_t)((total >> 32) & 0xFFFF), (uint32_t)(total >> 48));
    for (int j = 0; j < GRP_ITEMS; j++) {
        const uint32_t k = ks[j];
        if (k == 0) continue;
        const uint32_t e = j * GRP_THREADS + threadIdx.x;
        if (k == 1) {
            einfo[e] = make_uint2((uint32_t)(ex & 0xFFFF) | (1u << 24), 0u);
            ex += 1ull;
        } else {
            einfo[e] = make_uint2((uint32_t)((ex >> 16) & 0xFFFF) | ((uint32_t)(ex >> 48) << 12) | (k << 24),
                                  (uint32_t)((ex >> 32) & 0xFFFF));
            ex += (1ull << 16) + ((unsigned long long)k << 32) + (is_big(k, big_k) ? 1ull << 48 : 0ull);
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < GRP_RECS; j++) {
        const uint32_t s1 = sl[j];
        if (s1 == 0xFFFFFFFFu) continue;
        const uint32_t i = j * GRP_THREADS + threadIdx.x;
        const uint32_t h = rech[i];
        uint32_t place;
        if (s1 < 64)
            place = (uint32_t)__popcll(mlo[h] & ((1ull << s1) - 1ull));
        else
            place = (uint32_t)__popcll(mlo[h]) + (uint32_t)__popcll(mhi[h] & ((1ull << (s1 - 64)) - 1ull));
        const uint2 ei = einfo[h];
        aux[first + i] = make_uint2(ei.x, ei.y | (place << 16) | (s1 << 24));
    }
}

__global__ __launch_bounds__(GRP_THREADS) void k_group_count(uint32_t nb2, const uint32_t* __restrict__ cursor2,
                                                     const GroupRec* __restrict__ recs, uint32_t big_k,
                                                     uint2* __restrict__ aux, uint4* __restrict__ bcounts) {
    __shared__ GroupCountLds lds;
    for (uint32_t c = blockIdx.x; c < nb2; c += gridDim.x) {
        group_count_bucket(c, lds, cursor2, recs, big_k, aux, bcounts);
        __syncthreads();
    }
}

// Exclusive scan of the per-bucket counts (one workgroup); also the totals.
__global__ __launch_bounds__(1024) void k_group_offsets(const uint4* __restrict__ bcounts, uint4* __restrict__ bbase,
                                                        uint32_t nb2, DevStatus* status) {
    constexpr int ITEMS = 8;
    __shared__ uint4 wsum[16];
    __shared__ uint4 carry_sh;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    auto add = [](uint4 a, uint4 b) { return make_uint4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); };
    if (threadIdx.x == 0) carry_sh = make_uint4(0, 0, 0, 0);
    __syncthreads();
    for (uint32_t start = 0; start < nb2; start += 1024 * ITEMS) {
        const uint32_t i0 = start + threadIdx.x * ITEMS;
        uint4 v[ITEMS];
        uint4 mine = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
            v[j] = (i0 + j < nb2) ? bcounts[i0 + j] : make_uint4(0, 0, 0, 0);
            mine = add(mine, v[j]);
        }
        uint4 inc = mine;
        for (int o = 1; o < 64; o <<= 1) {
            const uint4 t = make_uint4(__shfl_up(inc.x, o), __shfl_up(inc.y, o), __shfl_up(inc.z, o), __shfl_up(inc.w, o));
            if (lane >= o) inc = add(inc, t);
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        uint4 base = carry_sh;
        for (int wv = 0; wv < wave; wv++) base = add(base, wsum[wv]);
        uint4 run = make_uint4(base.x + inc.x - mine.x, base.y + inc.y - mine.y, base.z + inc.z - mine.z,
                               base.w + inc.w - mine.w);
#pragma unroll
        for (int j = 0; j < ITEMS; j++) {
            if (i0 + j < nb2) bbase[i0 + j] = run;
            run = add(run, v[j]);
        }
        __syncthreads();
        if (threadIdx.x == 1023) carry_sh = add(base, inc);
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        status->n_single = carry_sh.x;
        status->n_multi = carry_sh.y;
        status->n_members = carry_sh.z;
        status->n_big = carry_sh.w;
    }
}

// The table row of every distinct record, found or, for an absent sign, inserted and filled
// (SparseKernelBlock::GetWeight, optimizer_kernel.h:299-308): rrow[record] = row, NO_ROW if the
// table is full.  It needs nothing but the records the dedup handed over, so it runs on a
// stream of its own beside the grouping and the ranking (random reads of the table against LDS
// and streaming work).  A sign present in several slots is probed once per slot; whichever
// thread claims a free slot first owns the insertion, the others find the key there.
// A new row is not filled here: one or two lanes of a wavefront drawing sixteen normal deviates would hold up
// the other sixty (with 1 % of the lookups new, most wavefronts have such a lane); the record is listed and
// k_init_new_recs fills the rows with every lane busy.  The list is the bucket's own -- newrec[c * GRP_CAP ...],
// newcnt[c] entries -- not one list of the call: places in one list are handed out by atomics on one counter,
// which take about 11 ns each one after the other (one per wavefront, tens of thousands, took longer than all the
// probes together; one per bucket still kept every workgroup waiting for its turn among a thousand).
__global__ __launch_bounds__(256) void k_probe_recs(uint32_t nb2, const uint32_t* __restrict__ cursor2,
                                                    const GroupRec* __restrict__ recs, uint32_t* __restrict__ rrow,
                                                    uint32_t* __restrict__ newrec, uint32_t* __restrict__ newcnt,
                                                    Store s, DevStatus* status) {
    __shared__ uint32_t s_count;
    for (uint32_t c = blockIdx.x; c < nb2; c += gridDim.x) {
        const uint32_t n = min(cursor2[c], (uint32_t)GRP_CAP);
        const size_t first = (size_t)c * GRP_CAP;
        if (threadIdx.x == 0) s_count = 0;
        __syncthreads();
        for (uint32_t i0 = 0; i0 < n; i0 += 256) {
            const uint32_t i = i0 + threadIdx.x;
            bool is_new = false;
            if (i < n) {
                const uint64_t sign = recs[first + i].sign;
                const uint32_t row = probe_slot<true>(s, sign, is_new);
                rrow[first + i] = row;
                if (row == NO_ROW) atomicOr(&status->err, DEV_ERR_TABLE_FULL);
            }
            if (is_new) newrec[first + atomicAdd(&s_count, 1u)] = i;  // rare: about one record in forty (at most n)
        }
        __syncthreads();
        if (threadIdx.x == 0) newcnt[c] = s_count;
        __syncthreads();
    }
}

// Elements 2 q and 2 q + 1 of a new row (the row initialiser of init_row, spread over lanes); with q == 0 also
// the row's padding columns and optimizer state.
__device__ __forceinline__ void init_row_pair(const Store& s, const OptDev& o, uint64_t seed, uint64_t sign, uint64_t row,
                                              uint32_t q, float stddev) {
    float* w = s.w + row * s.wstride;
    const int c = 2 * (int)q;
    float2 z = make_float2(0.f, 0.f);
    if (!o.zero_init) {
        z = normal_pair(rnd64(seed, sign, (uint64_t)q));
        z.x = (z.x * stddev) * o.initial_scale;
        z.y = (z.y * stddev) * o.initial_scale;
    }
    w[c] = z.x;
    if (c + 1 < s.D) w[c + 1] = z.y;
    if (q == 0) {
        for (int e = s.D; e < s.wlen; e++) w[e] = 0.f;  // cvm columns / padding
        init_state(s, o, s.st + row * s.sstride);
    }
}

// Fills the rows k_probe_recs inserted, `parts` workgroups per bucket's list (a batch of few buckets and many new
// signs still fills the device) and one lane per pair of elements; the first workgroup also adds up the lists'
// lengths: the call's number of new rows.
__global__ __launch_bounds__(256) void k_init_new_recs(Store s, OptDev o, uint64_t seed,
                                                       const GroupRec* __restrict__ recs,
                                                       const uint32_t* __restrict__ rrow, uint32_t nb2,
                                                       const uint32_t* __restrict__ newrec,
                                                       const uint32_t* __restrict__ newcnt, DevStatus* status,
                                                       uint32_t parts) {
    __shared__ uint32_t red[4];
    if (blockIdx.x == 0) {
        uint32_t mine = 0;
        for (uint32_t c = threadIdx.x; c < nb2; c += 256) mine += min(newcnt[c], (uint32_t)GRP_CAP);
        uint32_t total;
        block_excl_scan_256<uint32_t>(mine, red, &total);
        if (threadIdx.x == 0) status->n_new = total;
    }
    const uint32_t pairs = (uint32_t)(s.D + 1) / 2;
    const float stddev = (float)(1.0 / sqrt((double)s.D));
    for (uint32_t w = blockIdx.x; w < nb2 * parts; w += gridDim.x) {
        const uint32_t c = w / parts, part = w - c * parts;
        const uint32_t cnt = min(newcnt[c], (uint32_t)GRP_CAP);
        const size_t first = (size_t)c * GRP_CAP;
        for (uint32_t t = part * 256 + threadIdx.x; t < cnt * pairs; t += parts * 256) {
            const uint32_t j = t / pairs, q = t - j * pairs;
            const size_t i = first + min(newrec[first + j], (uint32_t)GRP_CAP - 1);
            init_row_pair(s, o, seed, recs[i].sign, rrow[i], q, stddev);
        }
    }
}

// Numbers the groups and writes the member lists: groups with one record get
// ids and member places counted up from 0 (place == id), groups with several
// get ids counted down from ids_cap - 1 and slices carved from the top of the
// member array, in bucket order.
//
// A bucket's groups and members occupy contiguous ranges of those arrays, but its records
// arrive in hash order: written record by record, every store is a transaction of its own
// (several million per call, which is what the kernel's time was).  So the bucket's part of
// the arrays is first put together in LDS and then copied out in order; only where_u, indexed
// by the distinct index of the record, stays a scattered store.  where_u[u] = {place in the member
// list (with WHERE_ONE_TILE if all lookups of the record lie in one tile), table row of the record's sign
// (rrow, from k_probe_recs)}; the groups get the rows too.  A group with big_k records or more is listed in
// big_list and, with {row, first member, records, group}, in big_desc.
//
// SLOT_RANKS: a record carries its rank in its slot instead of the position of its first occurrence
// (the pull of a small batch); its distinct index is the slot's base plus that rank.
template <bool SLOT_RANKS>
__global__ __launch_bounds__(EMIT_THREADS) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_group_emit(uint32_t nb2, const uint32_t* __restrict__ cursor2,
                                                    const GroupRec* __restrict__ recs, const uint2* __restrict__ aux,
                                                    const uint4* __restrict__ bbase,
                                                    const uint4* __restrict__ bcounts,
                                                    const uint8_t* __restrict__ flag8,
                                                    const uint32_t* __restrict__ wordpre, uint32_t ids_cap,
                                                    uint32_t big_k, uint64_t* __restrict__ grp_sign,
                                                    uint32_t* __restrict__ grp_off, uint32_t* __restrict__ grp_cnt,
                                                    uint32_t* __restrict__ big_list, uint4* __restrict__ big_desc,
                                                    Member* __restrict__ list, uint2* __restrict__ where_u,
                                                    const uint32_t* __restrict__ rrow,
                                                    uint32_t* __restrict__ grp_row, DevStatus* status,
                                                    const uint32_t* __restrict__ ubase, uint32_t n_slots) {
    // [0, n1): the groups of one record (group = member); from n1 on: in s_mem the members of the other groups,
    // last group first, in s_sign / s_row those groups themselves, whose offsets and sizes have arrays of their
    // own (such a group has two records at least, so there are n / 2 of them at most).  A member entry is packed
    // into eight bytes while it waits here {u | slot << 32 | show << 40}: 35 KB per workgroup, four to a CU.
    __shared__ unsigned long long s_mem[GRP_CAP];
    __shared__ unsigned long long s_sign[GRP_CAP];
    __shared__ uint32_t s_row[GRP_CAP];
    __shared__ uint32_t s_off[GRP_CAP / 2];
    __shared__ uint16_t s_cnt[GRP_CAP / 2];  // at most GRP_SLOTS records per group
    __shared__ uint4 s_part[EMIT_THREADS / 64];
    __shared__ uint32_t s_ub[SLOT_RANKS ? GRP_SLOTS + 1 : 1];  // the slots' bases (a small batch: one round trip less per record)
    if (SLOT_RANKS)
        for (uint32_t i = threadIdx.x; i <= n_slots && i <= (uint32_t)GRP_SLOTS; i += EMIT_THREADS) s_ub[i] = ubase[i];
    for (uint32_t c = blockIdx.x; c < nb2; c += gridDim.x) {
        const uint32_t n = min(cursor2[c], (uint32_t)GRP_CAP);
        const size_t first = (size_t)c * GRP_CAP;
        // the bucket's records first: their loads are in flight while the bucket's offsets are worked out
        GroupRec rs[EMIT_RECS];
        uint2 as[EMIT_RECS];
        uint32_t us[EMIT_RECS], rows[EMIT_RECS];
#pragma unroll
        for (int j = 0; j < EMIT_RECS; j++) {
            const uint32_t i = j * EMIT_THREADS + threadIdx.x;
            // (a small batch reads the bucket's whole room, wanted or not: the loads do not wait for its count then)
            if (SLOT_RANKS || i < n) {
                rs[j] = recs[first + i];
                as[j] = aux[first + i];
                rows[j] = rrow[first + i];
            }
        }
        uint4 bb;
        if (bbase) {
            if (n == 0) continue;
            bb = bbase[c];
        } else {
            // One bucket per workgroup and a few thousand buckets: the counts of the buckets before this one
            // (in L2) are added up here, which saves the launch of a scan kernel between the grouping's two
            // passes; the last workgroup leaves the totals (what k_group_offsets leaves).
            uint4 acc = make_uint4(0, 0, 0, 0);
            for (uint32_t i = threadIdx.x; i < c; i += EMIT_THREADS) {
                const uint4 v = bcounts[i];
                acc = make_uint4(acc.x + v.x, acc.y + v.y, acc.z + v.z, acc.w + v.w);
            }
            for (int o = 32; o > 0; o >>= 1)
                acc = make_uint4(acc.x + __shfl_xor(acc.x, o), acc.y + __shfl_xor(acc.y, o), acc.z + __shfl_xor(acc.z, o),
                                 acc.w + __shfl_xor(acc.w, o));
            if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
            __syncthreads();
            bb = make_uint4(0, 0, 0, 0);
            for (int wv = 0; wv < EMIT_THREADS / 64; wv++) {
                const uint4 v = s_part[wv];
                bb = make_uint4(bb.x + v.x, bb.y + v.y, bb.z + v.z, bb.w + v.w);
            }
            if (c == nb2 - 1 && threadIdx.x == 0) {
                const uint4 v = bcounts[c];
                status->n_single = bb.x + v.x;
                status->n_multi = bb.y + v.y;
                status->n_members = bb.z + v.z;
                status->n_big = bb.w + v.w;
            }
            if (n == 0) continue;  // (own sums: the workgroup has this one bucket, s_part is not written again)
        }
        const uint4 bc = bcounts[c];
        const uint32_t n1 = bc.x, nm = bc.y, nr = bc.z;  // groups of one record, of several, records of the latter
        const uint32_t top = ids_cap - 1 - bb.z;         // member place of local member 0 of the several-record groups
#pragma unroll
        for (int j = 0; j < EMIT_RECS; j++)
            if (j * EMIT_THREADS + threadIdx.x < n)
                us[j] = SLOT_RANKS ? s_ub[(rs[j].cnt >> 24) & (GRP_SLOTS - 1)] + rs[j].gi : rank_of(flag8, wordpre, rs[j].gi);
#pragma unroll
        for (int j = 0; j < EMIT_RECS; j++) {
            if (j * EMIT_THREADS + threadIdx.x >= n) continue;
            const GroupRec r = rs[j];
            const uint2 a = as[j];
            const uint32_t k = a.x >> 24, idx = a.x & 0xFFFu, bigidx = (a.x >> 12) & 0xFFFu;
            const uint32_t place = (a.y >> 16) & 0xFFu, sl = a.y >> 24;
            // batch_show = occurrences (sparse_table_ops.cc:290-293), batch_click starts at zero
            const unsigned long long m = (unsigned long long)us[j] | ((unsigned long long)sl << 32) |
                                         ((unsigned long long)(r.cnt & REC_CNT_MASK) << 40);
            const uint32_t one_tile = (r.cnt & REC_ONE_TILE) ? WHERE_ONE_TILE : 0u;
            if (k == 1) {
                const uint32_t g = bb.x + idx;
                s_mem[idx] = m;
                s_sign[idx] = r.sign;
                s_row[idx] = rows[j];
                where_u[us[j]] = make_uint2(g | one_tile, rows[j]);
            } else {
                const uint32_t g = ids_cap - 1 - (bb.y + idx);
                const uint32_t before = a.y & 0xFFFFu;        // records of the bucket's earlier groups of this kind
                const uint32_t t = before + k - 1 - place;    // local member: the group's last record first
                s_mem[n1 + t] = m;
                where_u[us[j]] = make_uint2((top - t) | one_tile, rows[j]);
                if (place == 0) {
                    s_row[n1 + idx] = rows[j];  // every record of the sign was given the same row
                    s_sign[n1 + idx] = r.sign;
                    s_off[idx] = top - (before + k - 1);
                    s_cnt[idx] = (uint16_t)k;
                    if (is_big(k, big_k)) {
                        big_list[bb.w + bigidx] = g;
                        // (what k_apply_big would otherwise fetch through g: one round trip less per sign)
                        big_desc[bb.w + bigidx] = make_uint4(rows[j], top - (before + k - 1), k, g);
                    }
                }
            }
        }
        __syncthreads();
        auto member = [](unsigned long long m) {
            Member e;
            e.u = (uint32_t)m;
            e.slot = (uint32_t)(m >> 32) & 0xFFu;
            e.show = (int32_t)(m >> 40);
            e.click = 0;
            return e;
        };
        for (uint32_t i = threadIdx.x; i < n1; i += EMIT_THREADS) {
            const uint32_t g = bb.x + i;
            list[g] = member(s_mem[i]);
            grp_sign[g] = s_sign[i];
            grp_off[g] = g;  // (group = member)
            grp_cnt[g] = 1;
            grp_row[g] = s_row[i];
        }
        for (uint32_t i = threadIdx.x; i < nr; i += EMIT_THREADS) list[top - i] = member(s_mem[n1 + i]);
        for (uint32_t i = threadIdx.x; i < nm; i += EMIT_THREADS) {
            const uint32_t g = ids_cap - 1 - (bb.y + i);
            grp_sign[g] = s_sign[n1 + i];
            grp_off[g] = s_off[i];
            grp_cnt[g] = s_cnt[i];
            grp_row[g] = s_row[n1 + i];
        }
        __syncthreads();
    }
}

}  // namespace tn

#endif  // TN_REMAP_LDS_H_
