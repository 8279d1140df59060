// Pull and push of a small batch (every slot fits one workgroup's LDS table): the same plan as the
// path through two levels of buckets leaves, from far fewer launches.  A batch of a few thousand
// lookups spends its time in the dependent launches of that path (about 3 us each, whatever the
// kernel does), not in its kernels, so here
//
//   pull  k_small_slots          one workgroup per slot: per-slot first-occurrence remap in LDS
//                                (sparse_table_ops.cc:115-137), lookup-or-insert of every distinct sign
//                                (sparse_table.cc:52-66), its record handed to its second-level bucket
//         k_small_group_finish   the first pass of the grouping (what k_group_count does) beside: the slots'
//                                counts added up, the call's status published to the host (which returns as
//                                soon as it sees it), rows into the variables (sparse_table_ops.cc:244-265),
//                                distinct indices made global
//         k_group_emit<true>     the groups of equal signs over all slots, as ever
//   push  k_small_verify         slot descriptors in, comparison with the plan's signs, click sums
//         k_small_apply          every group by one launch (tells the host that the comparison is complete); with
//                                more than 12 slots the signs with 5 records or more by wavefronts of their own in it
//
// Workgroups of one launch never wait for each other, and none needs another's results: what needs them runs
// in the next launch.
#ifndef TN_SMALL_BATCH_H_
#define TN_SMALL_BATCH_H_

#include "remap_lds.h"

namespace tn {

constexpr int SMALL_THREADS = 1024;
constexpr int SMALL_ITEMS = 4;                               // lookups per thread of k_small_slots
constexpr int SMALL_SLOT_MAX = SMALL_THREADS * SMALL_ITEMS;  // lookups of a slot at most
constexpr int SMALL_SLOTS = GRP_SLOTS;                       // slots at most (the grouping's slot masks)
constexpr int SMALL_NB2_MAX = 512;                           // second-level buckets at most
constexpr int SMALL_PARTS_MAX = 8;                           // workgroups of k_small_slots per slot at most
constexpr int SMALL_SLOT_WORKGROUPS = 256;                   // ... and for all slots together
constexpr int SMALL_TILE = 1024;                             // lookups per workgroup of k_small_verify

// What a workgroup of k_small_slots leaves for the launch after it: the slot's distinct signs (the same in
// every workgroup of the slot), the rows it inserted and the error flags it raised.
struct SlotOut {
    uint32_t n_unique, n_new, err, pad;
};

// Persistent device state of the small path (zero when allocated).  A call uses one of the two sets of
// bucket cursors and clears the other for the call after it.
struct SmallState {
    uint32_t cursor2[2][SMALL_NB2_MAX];
    SlotOut slot_out[SMALL_SLOT_WORKGROUPS];  // one per workgroup of k_small_slots
};

// Bytes of dynamic LDS of k_small_slots for a table of `entries` entries and nb2 second-level buckets.
inline size_t small_slots_lds(uint32_t entries, uint32_t nb2) {
    return ((size_t)entries + 1) * 16 + (size_t)nb2 * sizeof(uint32_t);
}

__device__ __forceinline__ void host_store(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// First launch of a small pull (see the head of the file).  host_descs: the slot descriptors in the host's pinned
// staging buffer; descs, lbase: where they go in device memory, for the launches after this one.  entries: the
// size of the workgroup's LDS table, a power of two and at least twice the longest slot.  prow[first lookup of
// the slot + r]: table row of the slot's distinct sign of rank r.  cursor2 / recs / rrow: the second-level
// buckets, as k_lds_dedup<true> and k_probe_recs fill them, but a record carries its rank in its slot (gi).
__global__ __launch_bounds__(SMALL_THREADS) void k_small_slots(
    const SlotDesc* host_descs, SlotDesc* descs, uint32_t* lbase, int N, uint32_t L, uint32_t entries,
    Store s, OptDev o, uint64_t seed, uint64_t* __restrict__ vals_copy, uint32_t* __restrict__ u_of_gi,
    uint32_t* __restrict__ prow, uint32_t nb2, uint32_t* cursor2, uint32_t* cursor2_next, GroupRec* __restrict__ recs,
    uint32_t* __restrict__ rrow, SmallState* state, uint32_t parts) {
    extern __shared__ unsigned long long smem64[];
    unsigned long long* keys = smem64;  // entry `entries`: the sign EMPTY_KEY itself
    uint32_t* minpos = reinterpret_cast<uint32_t*>(keys + entries + 1);
    uint32_t* cnts = minpos + entries + 1;
    uint32_t* hist2 = cnts + entries + 1;
    __shared__ SlotDesc sd;
    __shared__ uint32_t wsum[SMALL_THREADS / 64];
    __shared__ uint32_t sh_new, sh_err;
    // `parts` workgroups per slot: each of them works out the whole remap of the slot (in LDS, the same in all),
    // then takes every parts-th distinct sign through the table and every parts-th wavefront's lookups to the
    // outputs.  A CU sustains about 0.2 random 64-byte reads per nanosecond: the 2600 probes of a slot of 4096
    // lookups keep one CU busy for 13 us (measured with the device's clock around the kernel's phases), while
    // most of the device has nothing to do.
    const int sl = blockIdx.x / parts;
    const uint32_t part = blockIdx.x % parts;
    const uint32_t tid = threadIdx.x;
    // the slot's descriptor comes straight out of the host's staging buffer (one round trip over the bus,
    // in flight while the tables are cleared)
    if (tid < sizeof(SlotDesc) / 4)
        reinterpret_cast<uint32_t*>(&sd)[tid] = reinterpret_cast<const uint32_t*>(host_descs + sl)[tid];
    for (uint32_t i = tid; i <= entries; i += SMALL_THREADS) {
        keys[i] = EMPTY_KEY;
        minpos[i] = 0xFFFFFFFFu;
        cnts[i] = 0;
    }
    for (uint32_t i = tid; i < nb2; i += SMALL_THREADS) hist2[i] = 0;
    if (blockIdx.x == 0)
        for (uint32_t i = tid; i < (uint32_t)SMALL_NB2_MAX; i += SMALL_THREADS) cursor2_next[i] = 0;
    if (tid == 0) {
        sh_new = 0;
        sh_err = 0;
    }
    __syncthreads();
    const SlotDesc d = sd;
    if (tid == 0 && part == 0) {
        descs[sl] = d;
        lbase[sl] = d.lbase;
        if (sl == N - 1) lbase[N] = L;
    }
    const uint32_t n = d.len;
    // a thread's lookups are consecutive: the ranks of its first occurrences are, too
    uint64_t sg[SMALL_ITEMS];
    uint32_t h[SMALL_ITEMS];
    const uint32_t p0 = tid * SMALL_ITEMS;
#pragma unroll
    for (int j = 0; j < SMALL_ITEMS; j++) sg[j] = p0 + j < n ? (uint64_t)d.values[p0 + j] : 0;
    const int lane = (int)(tid & 63);
#pragma unroll
    for (int j = 0; j < SMALL_ITEMS; j++) {
        h[j] = entries;
        const bool valid = p0 + j < n;
        const uint64_t sign = sg[j];
        // A frequent sign fills whole wavefronts: the lanes that hold the same sign as the first valid lane let
        // that lane (the lowest position among them) enter it with their number, instead of queueing up on
        // one LDS address, and take its entry from it.
        const unsigned long long vmask = __ballot(valid);
        if (vmask == 0) continue;
        const int leader = __ffsll((long long)vmask) - 1;
        const uint64_t lead_sign = ((uint64_t)(uint32_t)__shfl((int)(sign >> 32), leader) << 32) |
                                   (uint32_t)__shfl((int)(uint32_t)sign, leader);
        const bool same = valid && sign == lead_sign;
        const unsigned long long smask = __ballot(same);
        const bool pooled = __popcll(smask) >= 8;
        const bool follower = pooled && same && lane != leader;
        if (valid && !follower) {
            if (sign != EMPTY_KEY) {
                uint32_t e = (uint32_t)(mix64(sign) >> 7) & (entries - 1);
                for (;;) {  // entries >= 2 n: a free entry exists
                    unsigned long long old = keys[e];
                    if (old == EMPTY_KEY) old = atomicCAS(&keys[e], (unsigned long long)EMPTY_KEY, sign);
                    if (old == EMPTY_KEY || old == sign) break;
                    e = (e + 1) & (entries - 1);
                }
                h[j] = e;
            }
            atomicMin(&minpos[h[j]], p0 + j);
            atomicAdd(&cnts[h[j]], pooled && lane == leader ? (uint32_t)__popcll(smask) : 1u);
        }
        const uint32_t lead_h = (uint32_t)__shfl((int)h[j], leader);
        if (follower) h[j] = lead_h;
    }
    __syncthreads();
    uint32_t firsts = 0;
#pragma unroll
    for (int j = 0; j < SMALL_ITEMS; j++)
        if (p0 + j < n && minpos[h[j]] == p0 + j) firsts |= 1u << j;
    uint32_t total = 0;
    uint32_t rank0 = block_excl_scan<uint32_t, SMALL_THREADS / 64>(__popc(firsts), wsum, &total);  // (barriers inside)
    // the entry of a distinct sign now takes its rank in place of the position (every thread has read the positions)
    uint32_t mine = 0;  // the distinct signs this workgroup takes through the table
    {
        uint32_t r = rank0;
#pragma unroll
        for (int j = 0; j < SMALL_ITEMS; j++)
            if (firsts & (1u << j)) {
                if (r % parts == part) mine |= 1u << j;
                minpos[h[j]] = r++;
            }
    }
    __syncthreads();
    // lookup-or-insert of the distinct signs (optimizer_kernel.h:299-308; the probe sequence of probe_slot).  A
    // thread's signs go through their sequences side by side: the key groups of all of them are read in one round
    // trip, the compare-and-swaps of those that found a free slot go out together, and so on round by round --
    // one after the other, a wavefront would spend a round trip on every sign that needs a second group or
    // claims a slot, in every one of its four places.  A row this workgroup inserts is listed in LDS (the key
    // table is dead) and filled further down by all threads: one lane of a wavefront drawing the normal deviates
    // of a row would hold up the other sixty-three.  The rows are read by the next launch only: another slot's
    // workgroup may be filling the row of a sign that this one finds claimed.
    unsigned long long* new_sign = keys;                                   // [n] at most
    uint32_t* new_row = reinterpret_cast<uint32_t*>(keys + n);            // (the table has 2 n + 1 entries or more)
    uint32_t rows[SMALL_ITEMS], place[SMALL_ITEMS];
    uint32_t err = 0, fresh = 0;
    {
        uint64_t at[SMALL_ITEMS];
        uint32_t live = 0;
#pragma unroll
        for (int j = 0; j < SMALL_ITEMS; j++) {
            rows[j] = NO_ROW;
            at[j] = 0;
            if (!(mine & (1u << j))) continue;
            if (sg[j] == EMPTY_KEY) {
                bool is_new = false;
                rows[j] = probe_slot<true>(s, sg[j], is_new);
                if (is_new) fresh |= 1u << j;
            } else {
                at[j] = home_group(sg[j], s.cap);
                live |= 1u << j;
            }
        }
        const uint64_t groups = s.cap / PROBE_WIDTH;
        for (uint64_t round = 0; live != 0 && round < 2 * groups + 64; round++) {
            ulonglong2 q[SMALL_ITEMS][4];
#pragma unroll
            for (int j = 0; j < SMALL_ITEMS; j++) {
                if (!(live & (1u << j))) continue;
                const ulonglong2* g = reinterpret_cast<const ulonglong2*>(s.keys + at[j]);
                q[j][0] = g[0], q[j][1] = g[1], q[j][2] = g[2], q[j][3] = g[3];
            }
            uint32_t claim = 0, where[SMALL_ITEMS];
#pragma unroll
            for (int j = 0; j < SMALL_ITEMS; j++) {
                where[j] = PROBE_WIDTH;
                if (!(live & (1u << j))) continue;
                const uint64_t k[PROBE_WIDTH] = {q[j][0].x, q[j][0].y, q[j][1].x, q[j][1].y,
                                                 q[j][2].x, q[j][2].y, q[j][3].x, q[j][3].y};
                bool free_slot = false;
#pragma unroll
                for (int e = PROBE_WIDTH - 1; e >= 0; e--)  // the first slot of the group that holds the sign or is free
                    if (k[e] == sg[j] || k[e] == EMPTY_KEY) {
                        where[j] = (uint32_t)e;
                        free_slot = k[e] == EMPTY_KEY;
                    }
                if (where[j] == PROBE_WIDTH) {
                    at[j] = at[j] + PROBE_WIDTH >= s.cap ? 0 : at[j] + PROBE_WIDTH;  // on to the next group
                } else if (free_slot) {
                    claim |= 1u << j;
                } else {
                    rows[j] = (uint32_t)(at[j] + where[j]);
                    live &= ~(1u << j);
                }
            }
            uint64_t old[SMALL_ITEMS];
#pragma unroll
            for (int j = 0; j < SMALL_ITEMS; j++)
                if (claim & (1u << j)) old[j] = atomicCAS(ull(&s.keys[at[j] + where[j]]), EMPTY_KEY, sg[j]);
#pragma unroll
            for (int j = 0; j < SMALL_ITEMS; j++) {
                if (!(claim & (1u << j))) continue;
                if (old[j] == EMPTY_KEY || old[j] == sg[j]) {
                    rows[j] = (uint32_t)(at[j] + where[j]);
                    if (old[j] == EMPTY_KEY) fresh |= 1u << j;
                    live &= ~(1u << j);
                }  // else another sign took the slot: the group is read again
            }
        }
        uint32_t r = rank0;
#pragma unroll
        for (int j = 0; j < SMALL_ITEMS; j++) {
            if (!(firsts & (1u << j))) continue;
            if (!(mine & (1u << j))) {
                r++;
                continue;
            }
            if (rows[j] == NO_ROW) {
                err |= DEV_ERR_TABLE_FULL;
            } else if (fresh & (1u << j)) {
                const uint32_t k = atomicAdd(&sh_new, 1u);
                new_sign[k] = sg[j];
                new_row[k] = rows[j];
            }
            prow[d.lbase + r] = rows[j];
            place[j] = atomicAdd(&hist2[group_bucket(sg[j], nb2)], 1u);
            r++;
        }
    }
    __syncthreads();
    for (uint32_t b = tid; b < nb2; b += SMALL_THREADS) {
        const uint32_t c = hist2[b];
        hist2[b] = c ? atomicAdd(&cursor2[b], c) : 0u;  // this slot's slice of the bucket
    }
    {
        // the new rows (row initialiser of init_row): a thread per pair of elements
        const uint32_t pairs = (uint32_t)(s.D + 1) / 2;
        const uint32_t work = sh_new * pairs;
        const float stddev = (float)(1.0 / sqrt((double)s.D));
        for (uint32_t t = tid; t < work; t += SMALL_THREADS) {
            const uint32_t k = t / pairs;
            init_row_pair(s, o, seed, (uint64_t)new_sign[k], new_row[k], t - k * pairs, stddev);
        }
    }
    __syncthreads();
    {
        uint32_t r = rank0;
#pragma unroll
        for (int j = 0; j < SMALL_ITEMS; j++) {
            if (!(firsts & (1u << j))) continue;
            if (!(mine & (1u << j))) {
                r++;
                continue;
            }
            const uint32_t b = group_bucket(sg[j], nb2);
            const uint32_t at = hist2[b] + place[j];
            if (at < (uint32_t)GRP_CAP) {
                GroupRec rec;
                rec.sign = sg[j];
                rec.gi = r;  // the record's rank in its slot (k_group_emit<true> adds the slot's base)
                rec.cnt = cnts[h[j]] | ((uint32_t)sl << 24);  // batch_show = occurrences (sparse_table_ops.cc:290-293)
                recs[(size_t)b * GRP_CAP + at] = rec;
                rrow[(size_t)b * GRP_CAP + at] = rows[j];
            } else {
                err |= DEV_ERR_REMAP_OVERFLOW;  // the host repeats the call with more buckets
            }
            r++;
        }
    }
    if (err) atomicOr(&sh_err, err);
    __syncthreads();
    // the lookups' outputs last: nothing in this kernel waits for these stores
#pragma unroll
    for (int j = 0; j < SMALL_ITEMS; j++) {
        if (p0 + j >= n || (tid >> 6) % parts != part) continue;
        const uint32_t r = minpos[h[j]];
        d.mapped[p0 + j] = (int64_t)r;
        vals_copy[d.lbase + p0 + j] = sg[j];
        u_of_gi[d.lbase + p0 + j] = r | ((firsts & (1u << j)) ? FIRST_BIT : 0u);  // relative to the slot until the next launch
    }
    if (tid == 0) {  // for the next launch, which adds up the slots' counts and publishes the call's status
        SlotOut out;
        out.n_unique = total;
        out.n_new = sh_new;
        out.err = sh_err;
        out.pad = 0;
        state->slot_out[blockIdx.x] = out;
    }
}

// Second launch of a small pull, two kinds of workgroups.  The first nb2 group the second-level buckets
// (group_count_bucket: what k_group_count does).  The others finish what the slots' workgroups began:
// vars[slot][rank, :] = table row of the slot's distinct sign of that rank (PopulatePulledVariable_,
// sparse_table_ops.cc:244-265), and the distinct indices of the lookups made global (rank in the slot + base
// of the slot; the ranks of a slot occupy the first positions of its window of lookup positions).  Each of them
// adds up the slots' counts itself; the first also leaves the bases and the call's status in device memory and
// publishes them to the host, which returns from the call when it sees them.
template <int VEC>
__global__ __launch_bounds__(GRP_THREADS) void k_small_group_finish(
    uint32_t nb2, const uint32_t* __restrict__ cursor2, const GroupRec* __restrict__ recs, uint32_t big_k,
    uint2* __restrict__ aux, uint4* __restrict__ bcounts, Store s, const SlotDesc* __restrict__ descs,
    const uint32_t* __restrict__ lbase, uint32_t* ubase, int N, uint32_t L, const uint32_t* __restrict__ prow,
    uint32_t* __restrict__ u_of_gi, const SmallState* __restrict__ state, uint32_t parts, DevStatus* status,
    uint32_t* host_dst, uint32_t* host_seq, uint32_t seq) {
    __shared__ GroupCountLds lds;
    if (blockIdx.x < nb2) {
        group_count_bucket(blockIdx.x, lds, cursor2, recs, big_k, aux, bcounts);
        return;
    }
    // (the grouping's LDS is free here)
    uint32_t* lb = reinterpret_cast<uint32_t*>(lds.mlo);  // lb[N + 1]
    uint32_t* ub = reinterpret_cast<uint32_t*>(lds.mhi);  // ub[N + 1]
    uint32_t* wsum = reinterpret_cast<uint32_t*>(lds.sh);
    uint32_t* misc = reinterpret_cast<uint32_t*>(lds.rech);  // [0] new rows, [1] error flags, [2] distinct signs
    SlotDesc* sd = reinterpret_cast<SlotDesc*>(lds.keys);  // the slots' descriptors (N <= SMALL_SLOTS: 8 KB of the 16)
    const uint32_t tid = threadIdx.x;
    const bool publisher = blockIdx.x == nb2;
    static_assert(SMALL_SLOT_WORKGROUPS <= GRP_THREADS && SMALL_SLOTS <= SMALL_SLOT_WORKGROUPS, "a thread per workgroup of k_small_slots");
    // what this thread moves: one 16-byte (or 4-byte) part of the row of one lookup position.  Its row number and
    // the descriptors are read at once, beside the slots' counts: one round trip instead of three in a row.
    const uint32_t chunks = (uint32_t)(s.wdim / VEC);
    const uint64_t t = (uint64_t)(blockIdx.x - nb2) * GRP_THREADS + tid;
    const bool in_range = t < (uint64_t)L * chunks;
    const uint32_t gi = in_range ? (uint32_t)(t / chunks) : 0u;
    const uint32_t c = (uint32_t)(t - (uint64_t)gi * chunks);
    const uint32_t row = in_range ? prow[gi] : NO_ROW;
    for (uint32_t i = tid; i < (uint32_t)N * (uint32_t)(sizeof(SlotDesc) / 4); i += GRP_THREADS)
        reinterpret_cast<uint32_t*>(sd)[i] = reinterpret_cast<const uint32_t*>(descs)[i];
    uint32_t mine = 0, nn = 0, ee = 0;
    if (tid < (uint32_t)N * parts) {  // (every workgroup of a slot leaves the slot's count, and its own share of the rest)
        const SlotOut so = state->slot_out[tid];
        nn = so.n_new;
        ee = so.err;
    }
    if (tid < (uint32_t)N) mine = state->slot_out[tid * parts].n_unique;
    for (uint32_t i = tid; i <= (uint32_t)N; i += GRP_THREADS) lb[i] = lbase[i];
    if (tid < 2) misc[tid] = 0;
    const uint32_t base = block_excl_scan<uint32_t, GRP_THREADS / 64>(mine, wsum, &misc[2]);  // (barriers inside)
    if (tid < (uint32_t)N) ub[tid] = base;
    if (publisher) {
        if (nn) atomicAdd(&misc[0], nn);
        if (ee) atomicOr(&misc[1], ee);
    }
    __syncthreads();
    const uint32_t U = misc[2];
    if (tid == 0) ub[N] = U;
    if (publisher && tid < 64) {  // one wavefront: device copies, then the host's, then the word the host polls
        const uint32_t sw = sizeof(DevStatus) / 4;
        for (uint32_t i = tid; i <= (uint32_t)N; i += 64) {
            const uint32_t v = i < (uint32_t)N ? ub[i] : U;
            ubase[i] = v;
            host_store(host_dst + sw + i, v);
        }
        if (tid == 0) {
            DevStatus st{};
            st.err = misc[1];
            st.n_unique = U;
            st.n_new = misc[0];
            st.gcap = U + U / 2 < 16 ? 16 : U + U / 2;
            *status = st;
            *s.count += misc[0];
            const uint32_t* sp = reinterpret_cast<const uint32_t*>(&st);
            for (uint32_t i = 0; i < sw; i++) host_store(host_dst + i, sp[i]);
        }
        __threadfence_system();
        if (tid == 0) host_store(host_seq, seq);
    }
    __syncthreads();
    // (one thread per position and part of the row: few rows per thread would leave the rows' round trips in a queue)
    if (!in_range) return;
    const int sl = find_slot(lb, N, gi);
    if (c == 0) u_of_gi[gi] += ub[sl];
    const uint32_t r = gi - lb[sl];
    if (r >= ub[sl + 1] - ub[sl]) return;  // beyond the slot's distinct signs
    const SlotDesc& d = sd[sl];
    if ((int64_t)r >= d.rows) return;      // the host reports the variable as too small
    if (row > s.cap) return;  // NO_ROW (table full): never address the table with it
    if (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4*>(s.w + (uint64_t)row * s.wstride + c * 4);
        *reinterpret_cast<float4*>(d.var + (uint64_t)r * s.wdim + c * 4) = v;
    } else {
        d.var[(uint64_t)r * s.wdim + c] = s.w[(uint64_t)row * s.wstride + c];
    }
}

// First launch of a small push on the last pull's plan: the slot descriptors come in from the host's staging
// buffer (a workgroup reads those of its tile's slots into LDS, the first also copies all of them to device
// memory for the update kernels), the signs are compared with the plan's copy, and with CLICKS the non-zero labels are added to
// the click sums of the member lists (sparse_table_ops.cc:283-296; a few thousand lookups do not queue up on
// any entry).  A mismatch also goes to the host (pinned memory); that the comparison is complete, the kernel
// launched next tells it.
template <bool CLICKS>
__global__ __launch_bounds__(256) void k_small_verify(const SlotDesc* host_descs, SlotDesc* push_descs,
                                                      const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                      const uint64_t* __restrict__ vals_copy, DevStatus* status,
                                                      const uint32_t* __restrict__ u_of_gi,
                                                      const uint2* __restrict__ where_u, Member* list,
                                                      uint32_t* host_mismatch) {
    extern __shared__ uint32_t lb[];      // lb[N + 1]
    __shared__ SlotDesc sd[SMALL_SLOTS];  // the descriptors of the slots the tile touches: sd[0] is slot s0's
    for (int i = threadIdx.x; i <= N; i += 256) lb[i] = lbase[i];
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        status->err = 0;  // what the pull reported is on the host; the update kernels start from a clean slate
        status->abort = 0;
    }
    __syncthreads();
    constexpr uint32_t DW = sizeof(SlotDesc) / 4;
    const int s0 = find_slot(lb, N, blockIdx.x * SMALL_TILE);
    const int s1 = find_slot(lb, N, min(L, (blockIdx.x + 1) * (uint32_t)SMALL_TILE) - 1);
    {
        const uint32_t* src = reinterpret_cast<const uint32_t*>(host_descs + s0);
        const uint32_t words = (uint32_t)(s1 - s0 + 1) * DW;
        for (uint32_t i = threadIdx.x; i < words; i += 256) reinterpret_cast<uint32_t*>(sd)[i] = src[i];
    }
    if (blockIdx.x == 0) {  // all of them into device memory, for the update kernels
        const uint32_t words = (uint32_t)N * DW;
        for (uint32_t i = threadIdx.x; i < words; i += 256)
            reinterpret_cast<uint32_t*>(push_descs)[i] = reinterpret_cast<const uint32_t*>(host_descs)[i];
    }
    __syncthreads();
    const uint32_t g0 = blockIdx.x * SMALL_TILE;
    const uint32_t g1 = min(L, g0 + (uint32_t)SMALL_TILE);
    bool bad = false;
    constexpr int PER = SMALL_TILE / 256;
    uint64_t now[PER], then[PER];
    int label[PER];
    uint32_t u[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t gi = g0 + j * 256 + threadIdx.x;
        now[j] = then[j] = 0;
        label[j] = 0;
        u[j] = 0;
        if (gi < g1) {
            const int sl = find_slot(lb, N, gi);
            now[j] = (uint64_t)sd[sl - s0].values[gi - lb[sl]];
            then[j] = vals_copy[gi];
            if (CLICKS) {
                label[j] = (int)sd[sl - s0].labels[gi - lb[sl]];
                u[j] = u_of_gi[gi] & ~FIRST_BIT;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < PER; j++) {
        bad |= now[j] != then[j];
        if (CLICKS && label[j] != 0) atomicAdd(&list[where_u[u[j]].x & WHERE_PLACE].click, label[j]);
    }
    if (bad) {
        atomicOr(&status->mismatch, 1u);
        host_store(host_mismatch, 1u);
    }
}

// Bytes of dynamic LDS of k_small_apply when its launch includes the workgroups for the signs with many records:
// per wavefront the staging and the row of apply_big_groups, then its pointer, count, flag and divisor arrays.
inline size_t small_apply_wave_lds(int D) { return align_up(big_lds_bytes(D), 8) + BIG_CHUNK * (8 + 4 + 4 + 4); }
inline size_t small_apply_big_lds(int D) { return 4 * small_apply_wave_lds(D); }

// The updates of a small push by one launch.  The first big_blocks workgroups (if the plan lists signs with many
// records; they start first, their chains are the longest): each of their wavefronts takes such signs the way
// k_apply_big does -- as a launch of its own that kernel costs a small batch as much again as this one.  The
// workgroups after those: every group with fewer than big_k records, one record or several, by the lane groups
// of k_apply_vec, the records of a sign four at a time.
// Nothing is reported to the host but that this kernel runs, which tells it that the comparison of the signs,
// launched before, is complete: on the plan of the last pull every sign has its row, and the host has compared
// the slots' distinct counts with the rows of the gradient matrices itself.
template <int KIND, int LPG>
__global__ __launch_bounds__(256) void k_small_apply(Store s, OptDev o, PushSrc src, int N, DevStatus* status,
                                                     const uint32_t* __restrict__ grp_row,
                                                     const uint32_t* __restrict__ grp_off,
                                                     const uint32_t* __restrict__ grp_cnt,
                                                     const Member* __restrict__ list, uint32_t big_k,
                                                     uint32_t ids_cap, uint32_t* host_seq, uint32_t seq,
                                                     uint32_t big_blocks, const uint32_t* __restrict__ big_list,
                                                     int gbuf_floats, uint32_t wave_lds, uint32_t wave_arrays) {
    extern __shared__ unsigned long long big_lds[];  // (only the first big_blocks workgroups use it)
    if (blockIdx.x == 0 && threadIdx.x == 0) host_store(host_seq, seq);
    // the slots' gradient matrices and bases from LDS: one round trip less in every record's chain of loads
    __shared__ SlotDesc sd[SMALL_SLOTS];
    __shared__ uint32_t ub[SMALL_SLOTS + 1];
    const uint32_t words = (uint32_t)N * (uint32_t)(sizeof(SlotDesc) / 4);
    for (uint32_t i = threadIdx.x; i < words; i += 256)
        reinterpret_cast<uint32_t*>(sd)[i] = reinterpret_cast<const uint32_t*>(src.descs)[i];
    for (uint32_t i = threadIdx.x; i <= (uint32_t)N; i += 256) ub[i] = src.ubase[i];
    // a plan that turned out not to be this batch's: nothing to do (the host analyses the batch itself)
    const uint32_t stop = status->mismatch | status->abort;
    const uint32_t n_single = status->n_single, n_multi = status->n_multi;
    __syncthreads();
    if (stop) return;
    src.descs = sd;
    src.ubase = ub;
    if (blockIdx.x < big_blocks) {
        const int wave = (int)(threadIdx.x >> 6), lane = (int)(threadIdx.x & 63);
        char* base = reinterpret_cast<char*>(big_lds) + (size_t)wave * wave_lds;  // (wave_arrays: where the arrays start in it)
        float* gbuf = reinterpret_cast<float*>(base);
        const float** gptr = reinterpret_cast<const float**>(base + wave_arrays);
        int* gshow = reinterpret_cast<int*>(gptr + BIG_CHUNK);
        int* gok = gshow + BIG_CHUNK;
        float* den = reinterpret_cast<float*>(gok + BIG_CHUNK);
        apply_big_groups<KIND>(s, o, src, status, big_list, grp_row, grp_off, grp_cnt, list, gbuf_floats, nullptr, gbuf,
                               gptr, gshow, gok, den, lane, blockIdx.x * 4 + (uint32_t)wave, big_blocks * 4,
                               [] { wave_sync(); });
        return;
    }
    const int sub = threadIdx.x % LPG;
    const int lane0 = (int)__lane_id() - sub;
    const uint32_t gstride = (gridDim.x - big_blocks) * (blockDim.x / LPG);
    const float c1 = 1 - o.beta1, c2 = 1 - o.beta2;
    for (uint32_t t = (blockIdx.x - big_blocks) * (blockDim.x / LPG) + threadIdx.x / LPG; t < n_single + n_multi; t += gstride) {
        const uint32_t g = group_id(t, n_single, n_multi, ids_cap);
        const uint32_t row = grp_row[g];
        if (row > s.cap) continue;  // NO_ROW, or no row number at all: never address the table with it
        const uint32_t k = grp_cnt[g];
        if (is_big(k, big_k)) continue;
        apply_group_vec<KIND, LPG, 4>(s, o, src, status, row, k, list + grp_off[g], nullptr, sub, lane0, c1, c2);
    }
}

}  // namespace tn

#endif  // TN_SMALL_BATCH_H_
