// Device code of the sparse pull / push path.  Included by sparse_table.hip only.
//
// HBM layout of one table (structure of arrays, all indexed by the slot number
// of an open-addressing hash table with linear probing):
//     keys[cap + 1]              uint64 sign, EMPTY_KEY where free
//     w   [cap + 1][wstride]     embedding weights (+2 cvm columns)
//     st  [cap + 1][sstride]     optimizer state
// When a weight row and its state fit one 128-byte line together, the two are
// interleaved (st = w + wlen, both strides 32 floats): an update then touches
// one line of the table instead of two.
// Slot `cap` is reserved for the one sign whose value equals EMPTY_KEY.
// A pull touches keys and w only (one 64-byte granule each for dim 16); the
// optimizer state is touched by push alone.
//
// Per-call scratch (all sized by the number of lookups L of the call):
//     dedup table   per slot of the op, open addressing over the slot's signs,
//                   entry {sign, position of first occurrence, rank}
//     group table   open addressing over the distinct signs of all slots,
//                   entry {sign, members - 1, group number}
// Both are filled with 0xFF bytes before use, which is EMPTY_KEY / "no
// position yet" / "count -1" at once.
//
// What a pull works out about its batch -- the distinct signs of every slot,
// the groups of equal signs across slots with their table rows -- is kept as
// the table's "plan"; a push whose signs are verified (on the device) to be
// the same batch reuses it instead of repeating remap, grouping and probing.
#ifndef TN_SPARSE_KERNELS_H_
#define TN_SPARSE_KERNELS_H_

#include "tn_common.h"

namespace tn {

struct Store {
    uint64_t cap;
    uint64_t* keys;
    float* w;
    float* st;
    uint32_t* special;            // 1 when the sign EMPTY_KEY itself is resident
    unsigned long long* count;    // resident keys
    int D, wdim;
    int wlen, slen;        // floats of a weight / state row (incl. padding to a multiple of 4)
    int wstride, sstride;  // distance between consecutive rows, in floats (>= wlen / slen)
};

// One slot (input tensor pair) of a pull / push op.  64 bytes.
struct SlotDesc {
    const int64_t* values;
    int64_t* mapped;        // pull
    const int64_t* labels;  // push
    float* var;             // pull
    const float* grads;     // push
    int64_t rows;           // rows of var (pull) / of grads (push)
    uint32_t len;
    uint32_t lbase;         // first lookup of the slot in the concatenated order
    uint32_t tbase;         // first entry of the slot's dedup table
    uint32_t tcap;          // entries of the slot's dedup table (+1 special)
};

struct DedupEntry {
    uint64_t key;
    uint32_t minpos;  // smallest in-slot position of the sign
    uint32_t rank;    // index of the sign in the compact distinct list of the call
};

struct GroupEntry {
    uint64_t key;
    uint32_t cnt;  // members - 1 (starts at 0xFFFFFFFF)
    uint32_t g;    // number of the group
};

// One record of a push in its group's member list: which distinct sign of which
// slot, and its batch_show / batch_click (SparsePushSignInfo's counts).
// where_u[u].x: the record's place in the member list; the top bit marks a record whose lookups all lie in one
// tile of 2048 consecutive lookups (only the remap through LDS sets it).
constexpr uint32_t WHERE_ONE_TILE = 0x80000000u;
constexpr uint32_t WHERE_PLACE = 0x7FFFFFFFu;

struct __attribute__((aligned(16))) Member {
    uint32_t u;
    uint32_t slot;
    int32_t show;
    int32_t click;
};

constexpr int REMAP_ITEMS = 8;
constexpr int REMAP_THREADS = 256;
constexpr int REMAP_TILE = REMAP_ITEMS * REMAP_THREADS;
constexpr int MAX_SLOTS = 4095;  // lbase[MAX_SLOTS + 1] fills 16 KB of LDS

__device__ __forceinline__ unsigned long long* ull(uint64_t* p) { return reinterpret_cast<unsigned long long*>(p); }

// Hands out consecutive indices from *counter to the lanes whose flag is set,
// with one atomic per wavefront.
__device__ __forceinline__ uint32_t wave_alloc(bool flag, uint32_t* counter) {
    unsigned long long mask = __ballot(flag);
    if (mask == 0) return 0;
    int leader = __ffsll((long long)mask) - 1;
    int lane = (int)__lane_id();
    uint32_t base = 0;
    if (lane == leader) base = atomicAdd(counter, (uint32_t)__popcll(mask));
    base = __shfl(base, leader);
    return base + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
}

// ------------------------------------------------------------------ fills
__global__ __launch_bounds__(256) void k_fill_ff(uint4* p, size_t n16) {
    size_t stride = (size_t)gridDim.x * blockDim.x;
    uint4 v = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) p[i] = v;
}

// fills the first (status->gcap + 1) group entries
__global__ __launch_bounds__(256) void k_fill_groups(GroupEntry* gt, const DevStatus* status) {
    size_t n16 = (size_t)status->gcap + 1;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    uint4 v = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
    uint4* p = reinterpret_cast<uint4*>(gt);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) p[i] = v;
}

__global__ void k_reset_status(DevStatus* status, uint32_t n_unique, uint32_t gcap) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        status->err = 0;
        status->n_unique = n_unique;
        status->n_single = 0;
        status->n_multi = 0;
        status->n_new = 0;
        status->gcap = gcap;
        status->n_members = 0;
        status->mismatch = 0;
        status->abort = 0;
        status->n_big = 0;
        status->tile_share_q16 = 0;
    }
}

// Small host<->device transfers done by kernels on the stream (pinned host
// memory is device-accessible): cheaper than a copy command each.  The same
// launch prepares the call's status block (STATUS_NEW_PLAN: everything cleared;
// STATUS_REUSE_PLAN: a push on the last pull's plan keeps the counts and clears
// the flags), clears `zero[0 .. n_zero)` and copies copy_n words from copy_src to copy_dst.
enum { STATUS_KEEP = 0, STATUS_NEW_PLAN = 1, STATUS_REUSE_PLAN = 2 };

__global__ __launch_bounds__(256) void k_stage_in(const uint32_t* __restrict__ host_src, uint32_t* __restrict__ dst_a,
                                                  uint32_t words_a, uint32_t* __restrict__ dst_b, uint32_t words_b,
                                                  DevStatus* status, int status_mode, uint32_t* __restrict__ zero,
                                                  uint32_t n_zero, const DevStatus* plan_status,
                                                  const uint32_t* __restrict__ copy_src, uint32_t* __restrict__ copy_dst,
                                                  uint32_t copy_n) {
    const uint32_t stride = gridDim.x * blockDim.x;
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    for (uint32_t i = tid; i < words_a + words_b; i += stride) {
        if (i < words_a)
            dst_a[i] = host_src[i];
        else
            dst_b[i - words_a] = host_src[i];
    }
    for (uint32_t i = tid; i < n_zero; i += stride) zero[i] = 0;
    for (uint32_t i = tid; i < copy_n; i += stride) copy_dst[i] = copy_src[i];
    if (tid == 0 && status_mode != STATUS_KEEP) {
        // a push on the last pull's plan has a status block of its own: the plan's counts, fresh flags
        if (status_mode == STATUS_REUSE_PLAN && plan_status != status) *status = *plan_status;
        status->err = 0;
        status->mismatch = 0;
        status->abort = 0;
        if (status_mode == STATUS_NEW_PLAN) {
            status->n_unique = 0;
            status->n_single = 0;
            status->n_multi = 0;
            status->n_new = 0;
            status->gcap = 0;
            status->n_members = 0;
            status->n_big = 0;
            status->tile_share_q16 = 0;
        }
    }
}

// host_dst: a DevStatus followed by n_ubase words.  With count != nullptr the rows the call
// inserted are added to the table's number of resident keys.  With host_seq != nullptr the word seq is written
// there once everything else is on the host: a host that polls that word has the status a few microseconds
// after this kernel, well before a wait on the stream would return.
__global__ __launch_bounds__(256) void k_publish(const DevStatus* __restrict__ status,
                                                 const uint32_t* __restrict__ ubase, uint32_t n_ubase,
                                                 uint32_t* __restrict__ host_dst, unsigned long long* count,
                                                 uint32_t* host_seq, uint32_t seq) {
    if (count && threadIdx.x == 0) *count += status->n_new;
    const uint32_t sw = sizeof(DevStatus) / 4;
    const uint32_t* sp = reinterpret_cast<const uint32_t*>(status);
    for (uint32_t i = threadIdx.x; i < sw + n_ubase; i += blockDim.x)
        host_dst[i] = i < sw ? sp[i] : ubase[i - sw];
    if (host_seq) {
        __threadfence_system();
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_store(host_seq, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

__global__ void k_finish_insert(Store s, const DevStatus* status) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *s.count += status->n_new;
}

// ------------------------------------------------------- table probe/insert
// One thread per sign.  rows[i] = slot of signs[i] (NO_ROW if absent / full).
// With INSERT an absent sign claims the first free slot of its probe sequence
// (SparseKernelBlock::GetWeight's insert, optimizer_kernel.h:299-308) and the
// index i of every claim is appended to newlist (or, without a newlist, the
// claiming thread initialises the row on the spot).
// Groups with one record are numbered upwards from 0, groups with several
// downwards from ids_cap - 1: the i-th group in enumeration order.
__device__ __forceinline__ uint32_t group_id(uint32_t i, uint32_t n_single, uint32_t n_multi, uint32_t ids_cap) {
    return i < n_single ? i : ids_cap - n_multi + (i - n_single);
}

constexpr int PROBE_WIDTH = 8;
static_assert(PROBE_WIDTH == 8, "probe_slot reads a group as four 16-byte loads");

// First slot of the aligned group of PROBE_WIDTH slots that holds the home slot of a sign.
__device__ __forceinline__ uint64_t home_group(uint64_t sign, uint64_t cap) {
    return slot_of(sign, cap) & ~(uint64_t)(PROBE_WIDTH - 1);
}

__device__ __forceinline__ void init_row(const Store& s, const OptDev& o, uint64_t seed, uint64_t sign, uint64_t row);

// The probe sequence of `sign` from the group at idx on, whose eight keys the caller has loaded
// already (q0..q3): several probes of a thread can have their first groups in flight together.
template <bool INSERT>
__device__ __forceinline__ uint32_t probe_from(const Store& s, uint64_t sign, uint64_t idx, ulonglong2 q0, ulonglong2 q1,
                                               ulonglong2 q2, ulonglong2 q3, bool& is_new) {
    // Linear probing in aligned groups of PROBE_WIDTH slots, starting at the group of the home
    // slot (the capacity is a multiple of PROBE_WIDTH): a group is one 64-byte granule, read
    // with four 16-byte loads in one round trip, and at a load of 0.75 few probes need a second
    // group.  Unaligned windows straddle granule boundaries and were measured at half the rate.
    for (uint64_t p = 0; p < s.cap; p += PROBE_WIDTH) {
        if (p != 0) {
            // plain loads: a key never changes once set, and a stale free slot is settled by the compare-and-swap
            const ulonglong2* g = reinterpret_cast<const ulonglong2*>(s.keys + idx);
            q0 = g[0], q1 = g[1], q2 = g[2], q3 = g[3];
        }
        const uint64_t k[PROBE_WIDTH] = {q0.x, q0.y, q1.x, q1.y, q2.x, q2.y, q3.x, q3.y};
#pragma unroll
        for (int j = 0; j < PROBE_WIDTH; j++) {
            if (k[j] == sign) return (uint32_t)(idx + j);
            if (k[j] == EMPTY_KEY) {
                if (!INSERT) return NO_ROW;
                uint64_t old = atomicCAS(ull(&s.keys[idx + j]), EMPTY_KEY, sign);
                if (old == EMPTY_KEY || old == sign) {
                    is_new = old == EMPTY_KEY;
                    return (uint32_t)(idx + j);
                }
            }
        }
        idx = idx + PROBE_WIDTH >= s.cap ? 0 : idx + PROBE_WIDTH;
    }
    return NO_ROW;
}

// Slot of `sign` in the table, NO_ROW if absent (or, with INSERT, if the table
// is full).  With INSERT an absent sign claims the first free slot of its probe
// sequence and is_new tells whether this call made the claim.
template <bool INSERT>
__device__ __forceinline__ uint32_t probe_slot(const Store& s, uint64_t sign, bool& is_new) {
    is_new = false;
    if (sign == EMPTY_KEY) {
        if (INSERT) {
            is_new = atomicCAS(s.special, 0u, 1u) == 0u;
            return (uint32_t)s.cap;
        }
        return ld_relaxed(s.special) ? (uint32_t)s.cap : NO_ROW;
    }
    const uint64_t idx = home_group(sign, s.cap);
    const ulonglong2* g = reinterpret_cast<const ulonglong2*>(s.keys + idx);
    return probe_from<INSERT>(s, sign, idx, g[0], g[1], g[2], g[3], is_new);
}

// With groups_of != nullptr the signs are those of its groups (ids_cap = size of the id space).
template <bool INSERT>
__global__ __launch_bounds__(256) void k_probe(Store s, const uint64_t* __restrict__ signs, int64_t n_host,
                                               const DevStatus* groups_of, uint32_t ids_cap,
                                               uint32_t* __restrict__ rows, uint32_t* __restrict__ newlist,
                                               DevStatus* status, uint32_t miss_err, OptDev o, uint64_t seed) {
    __shared__ uint32_t wcount[4];
    __shared__ uint32_t block_base;
    const uint32_t n_single = groups_of ? groups_of->n_single : 0, n_multi = groups_of ? groups_of->n_multi : 0;
    const int64_t n = groups_of ? (int64_t)n_single + n_multi : n_host;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // every thread of the workgroup takes part in every round: the places of the new rows of a round are handed
    // out with one atomic per workgroup (atomics on the one counter run one after the other, about 11 ns each)
    for (int64_t t0 = (int64_t)blockIdx.x * blockDim.x; t0 < n; t0 += stride) {
        const int64_t t = t0 + threadIdx.x;
        bool is_new = false;
        int64_t i = 0;
        uint64_t sign = 0;
        uint32_t row = NO_ROW;
        if (t < n) {
            i = groups_of ? (int64_t)group_id((uint32_t)t, n_single, n_multi, ids_cap) : t;
            sign = signs[i];
            row = probe_slot<INSERT>(s, sign, is_new);
            rows[i] = row;
            if (row == NO_ROW && miss_err) atomicOr(&status->err, miss_err);
        }
        if (INSERT) {
            const unsigned long long mask = __ballot(is_new);
            const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
            if (lane == 0) wcount[wave] = (uint32_t)__popcll(mask);
            __syncthreads();
            if (threadIdx.x == 0) {
                const uint32_t total = wcount[0] + wcount[1] + wcount[2] + wcount[3];
                block_base = total ? atomicAdd(&status->n_new, total) : 0u;
            }
            __syncthreads();
            if (is_new) {
                uint32_t j = block_base + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
                for (int wv = 0; wv < wave; wv++) j += wcount[wv];
                if (newlist)
                    newlist[j] = (uint32_t)i;  // initialised by k_init_rows
                else
                    init_row(s, o, seed, sign, row);  // the thread that claimed the row fills it
            }
            __syncthreads();
        }
    }
}

// ---------------------------------------------------------- row initialiser
__device__ __forceinline__ uint64_t rnd64(uint64_t seed, uint64_t sign, uint64_t ctr) {
    return mix64(mix64(sign ^ seed) + (ctr + 1) * 0x9E3779B97F4A7C15ull);
}

// Two independent N(0,1) draws from 64 random bits (Box-Muller).
__device__ __forceinline__ float2 normal_pair(uint64_t bits) {
    float u1 = ((float)(uint32_t)(bits >> 32) + 1.0f) * 2.3283064365386963e-10f;  // (0, 1]
    float u2 = (float)(uint32_t)bits * 2.3283064365386963e-10f;                   // [0, 1)
    float r = sqrtf(-2.0f * logf(u1));
    float sn, cs;
    sincosf(6.283185307179586f * u2, &sn, &cs);
    return make_float2(r * cs, r * sn);
}

__device__ __forceinline__ void init_state(const Store& s, const OptDev& o, float* st) {
    if (o.kind == OPT_ADAGRAD) {
        st[0] = o.initial_g2sum;  // ada_grad_kernel.cc:94-98
        st[1] = 0.f;
        st[2] = 0.f;
        st[3] = 0.f;  // no_show_days = 0 (int bits)
    } else {
        for (int i = 0; i < s.slen; i++) st[i] = 0.f;  // m=v=0 / z=n=0, show, delta_show
    }
}

// New rows: w[i] = N(0, 1/sqrt(D)) * initial_scale, or zeros under
// sparse_zero_init; fresh optimizer state (ada_grad_kernel.cc:78-103,
// adam_kernel.cc:89-110, ftrl_kernel.cc:34-55).  The draw is a pure function
// of (seed, sign, element).  One thread per new row.
__device__ __forceinline__ void init_row(const Store& s, const OptDev& o, uint64_t seed, uint64_t sign, uint64_t row) {
    const float stddev = (float)(1.0 / sqrt((double)s.D));
    float* w = s.w + row * s.wstride;
    if (o.zero_init) {
        for (int c = 0; c < s.D; c++) w[c] = 0.f;
    } else {
        for (int c = 0; c < s.D; c += 2) {
            float2 z = normal_pair(rnd64(seed, sign, (uint64_t)(c >> 1)));
            w[c] = (z.x * stddev) * o.initial_scale;
            if (c + 1 < s.D) w[c + 1] = (z.y * stddev) * o.initial_scale;
        }
    }
    for (int c = s.D; c < s.wlen; c++) w[c] = 0.f;  // cvm columns / padding
    init_state(s, o, s.st + row * s.sstride);
}

__global__ __launch_bounds__(256) void k_init_rows(Store s, OptDev o, uint64_t seed, const uint64_t* __restrict__ signs,
                                                   const uint32_t* __restrict__ rows,
                                                   const uint32_t* __restrict__ newlist, const DevStatus* status) {
    const uint32_t n_new = status->n_new;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t j = blockIdx.x * blockDim.x + threadIdx.x; j < n_new; j += stride) {
        const uint32_t i = newlist[j];
        init_row(s, o, seed, signs[i], rows[i]);
    }
}

// ------------------------------------------------- show decay / elimination
struct DecayConf {
    int kind;
    float rate;            // show_decay_rate
    float show_threshold;
    int no_show_days;
    int elimination_logic;
};

// SparseTable::ShowDecay (core/ps/table/sparse_table.cc:139 -> optimizer_kernel.h:422-427,549-553):
// one pass over every slot of the table; resident rows get
//   AdaGrad  show *= rate; click *= rate; no_show_days += delta_days   (ada_grad_kernel.cc:191-195)
//   Ftrl     show *= rate                                              (ftrl_kernel.cc:124)
//   Adam     nothing                                                   (adam_kernel.h:67)
__global__ __launch_bounds__(256) void k_show_decay(Store s, DecayConf c, int delta_days) {
    const uint64_t n = s.cap + 1;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const bool resident = i < s.cap ? s.keys[i] != EMPTY_KEY : *s.special != 0;
        if (!resident) continue;
        float* st = s.st + i * s.sstride;
        if (c.kind == OPT_ADAGRAD) {
            st[1] *= c.rate;
            st[2] *= c.rate;
            st[3] = __int_as_float(__float_as_int(st[3]) + delta_days);
        } else if (c.kind == OPT_FTRL) {
            st[2 * s.D] *= c.rate;
        }
    }
}

// Value::DeleteByShow for the rows of given signs: out[i] = 1 if the row would be left out of a
// saved table (optimizer_kernel.h:332,345; ada_grad_kernel.cc:197-204, ftrl_kernel.cc:126,
// adam_kernel.h:69), 0 otherwise and for absent signs.
__global__ __launch_bounds__(256) void k_delete_by_show(Store s, DecayConf c, const uint32_t* __restrict__ rows,
                                                        int64_t n, uint8_t* __restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t row = rows[i];
        bool del = false;
        if (row != NO_ROW) {
            const float* st = s.st + (uint64_t)row * s.sstride;
            if (c.kind == OPT_ADAGRAD) {
                const bool low = st[1] < c.show_threshold, old = __float_as_int(st[3]) > c.no_show_days;
                del = c.elimination_logic == 1 ? (low && old) : (low || old);
            } else if (c.kind == OPT_FTRL) {
                del = st[2 * s.D] < c.show_threshold;
            }
        }
        out[i] = del ? 1 : 0;
    }
}

// Every resident row among the slots [first, first + n_slots) of the table (slot `cap` is
// the row of the sign 0xFFFF...F), compacted into signs / w / state in no particular order;
// with skip_eliminated rows for which DeleteByShow holds are left out (what a saved table
// holds, optimizer_kernel.h:332,345).  *count = rows written.
__global__ __launch_bounds__(256) void k_export_range(Store s, DecayConf c, uint64_t first, uint64_t n_slots,
                                                      int skip_eliminated, uint64_t* __restrict__ signs,
                                                      float* __restrict__ w, float* __restrict__ state,
                                                      uint32_t* count) {
    const int sf = (c.kind == OPT_ADAGRAD) ? 4 : 2 * s.D + 2;
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t rounds = (n_slots + stride - 1) / stride;  // whole wavefronts take part in every round
    for (uint64_t r = 0; r < rounds; r++) {
        const uint64_t k = r * stride + (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
        const uint64_t i = first + k;
        bool take = false;
        uint64_t sign = EMPTY_KEY;
        if (k < n_slots && i <= s.cap) {
            if (i < s.cap) {
                sign = s.keys[i];
                take = sign != EMPTY_KEY;
            } else {
                take = *s.special != 0;
            }
            if (take && skip_eliminated) {
                const float* st = s.st + i * s.sstride;
                if (c.kind == OPT_ADAGRAD) {
                    const bool low = st[1] < c.show_threshold, old = __float_as_int(st[3]) > c.no_show_days;
                    take = !(c.elimination_logic == 1 ? (low && old) : (low || old));
                } else if (c.kind == OPT_FTRL) {
                    take = !(st[2 * s.D] < c.show_threshold);
                }
            }
        }
        const uint32_t at = wave_alloc(take, count);
        if (take) {
            signs[at] = sign;
            const float* sw = s.w + i * s.wstride;
            const float* ss = s.st + i * s.sstride;
            for (int q = 0; q < s.wdim; q++) w[(uint64_t)at * s.wdim + q] = sw[q];
            for (int q = 0; q < sf; q++) state[(uint64_t)at * sf + q] = ss[q];
        }
    }
}

// ------------------------------------------------------------------ gathers
// out[i, :] = w[rows[i], 0:wdim]   (SparseTable::Pull's append, sparse_table.cc:64)
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_rows(Store s, const uint32_t* __restrict__ rows, int64_t n,
                                                     float* __restrict__ out) {
    const int chunks = s.wdim / VEC;
    const int64_t total = n * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int64_t i = t / chunks;
        const int c = (int)(t - i * chunks);
        const uint32_t row = rows[i];
        if (VEC == 4) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row != NO_ROW) v = *reinterpret_cast<const float4*>(s.w + (uint64_t)row * s.wstride + c * 4);
            *reinterpret_cast<float4*>(out + i * s.wdim + c * 4) = v;
        } else {
            out[i * s.wdim + c] = (row != NO_ROW) ? s.w[(uint64_t)row * s.wstride + c] : 0.f;
        }
    }
}

// Snapshot load: table row <- caller row (+ given or fresh state).
__global__ __launch_bounds__(256) void k_load_rows(Store s, OptDev o, const uint32_t* __restrict__ rows, int64_t n,
                                                   const float* __restrict__ w, const float* __restrict__ state) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t row = rows[i];
        if (row == NO_ROW) continue;
        float* dw = s.w + (uint64_t)row * s.wstride;
        for (int c = 0; c < s.wdim; c++) dw[c] = w[i * s.wdim + c];
        for (int c = s.wdim; c < s.wlen; c++) dw[c] = 0.f;
        float* ds = s.st + (uint64_t)row * s.sstride;
        if (state) {
            const int sf = (o.kind == OPT_ADAGRAD) ? 4 : 2 * s.D + 2;
            for (int c = 0; c < sf; c++) ds[c] = state[i * sf + c];
            for (int c = sf; c < s.slen; c++) ds[c] = 0.f;
        } else {
            init_state(s, o, ds);
        }
    }
}

__global__ __launch_bounds__(256) void k_export_rows(Store s, OptDev o, const uint32_t* __restrict__ rows, int64_t n,
                                                     float* __restrict__ w, float* __restrict__ state,
                                                     uint8_t* __restrict__ found) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int sf = (o.kind == OPT_ADAGRAD) ? 4 : 2 * s.D + 2;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const uint32_t row = rows[i];
        if (found) found[i] = row != NO_ROW;
        const float* sw = s.w + (uint64_t)row * s.wstride;
        const float* ss = s.st + (uint64_t)row * s.sstride;
        if (w)
            for (int c = 0; c < s.wdim; c++) w[i * s.wdim + c] = (row != NO_ROW) ? sw[c] : 0.f;
        if (state)
            for (int c = 0; c < sf; c++) state[i * sf + c] = (row != NO_ROW) ? ss[c] : 0.f;
    }
}

// Re-insertion of every resident row into a larger table.
__global__ __launch_bounds__(256) void k_rehash(Store from, Store to, DevStatus* status) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i <= from.cap; i += stride) {
        uint64_t dst;
        if (i == from.cap) {
            if (*from.special == 0) continue;
            *to.special = 1;
            dst = to.cap;
        } else {
            const uint64_t sign = from.keys[i];
            if (sign == EMPTY_KEY) continue;
            uint64_t idx = home_group(sign, to.cap);  // the probe sequence of probe_slot
            dst = EMPTY_KEY;
            for (uint64_t p = 0; p < to.cap; ++p) {
                uint64_t old = atomicCAS(ull(&to.keys[idx]), EMPTY_KEY, sign);
                if (old == EMPTY_KEY) {
                    dst = idx;
                    break;
                }
                idx = (idx + 1 == to.cap) ? 0 : idx + 1;
            }
            if (dst == EMPTY_KEY) {
                atomicOr(&status->err, DEV_ERR_TABLE_FULL);
                continue;
            }
        }
        const float* sw = from.w + i * from.wstride;
        float* dw = to.w + dst * to.wstride;
        for (int c = 0; c < from.wlen; c++) dw[c] = sw[c];
        const float* ss = from.st + i * from.sstride;
        float* ds = to.st + dst * to.sstride;
        for (int c = 0; c < from.slen; c++) ds[c] = ss[c];
    }
}

// -------------------------------------------------------------------- remap
// Slot of a lookup: last s with lbase[s] <= gi (lbase[N] = L), skipping empty slots.
__device__ __forceinline__ int find_slot(const uint32_t* lb, int N, uint32_t gi) {
    int lo = 0, hi = N;  // invariant: lb[lo] <= gi < lb[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (lb[mid] <= gi)
            lo = mid;
        else
            hi = mid;
    }
    return lo;
}

__device__ __forceinline__ void load_lbase(uint32_t* sh, const uint32_t* lbase, int N) {
    for (int i = threadIdx.x; i <= N; i += blockDim.x) sh[i] = lbase[i];
    __syncthreads();
}

// Step 1: every lookup finds or claims the entry of its sign in its slot's
// dedup table, remembers the entry (tidx) and lowers the entry's minpos to its
// own in-slot position.  After the kernel, minpos is the position of the
// sign's first occurrence: exactly the lookup on which the reference's
// std::map insert succeeds (sparse_table_ops.cc:122-131).
// Entries only ever change from EMPTY_KEY to a sign and minpos only decreases,
// so ordinary (possibly stale) loads are safe: a stale value costs one atomic,
// whose return value is the truth.
__global__ __launch_bounds__(256) void k_remap_insert(const SlotDesc* __restrict__ descs,
                                                      const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                      DedupEntry* dt, uint32_t* __restrict__ tidx,
                                                      uint64_t* __restrict__ vals_copy) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t gi = blockIdx.x * blockDim.x + threadIdx.x; gi < L; gi += stride) {
        const int sl = find_slot(lb, N, gi);
        const SlotDesc& d = descs[sl];
        const uint32_t li = gi - lb[sl];
        const uint64_t sign = (uint64_t)d.values[li];
        vals_copy[gi] = sign;
        const uint32_t tbase = d.tbase, tcap = d.tcap;
        uint32_t e;
        if (sign == EMPTY_KEY) {
            e = tbase + tcap;
        } else {
            uint32_t idx = (uint32_t)slot_of(sign, tcap);
            for (;;) {
                e = tbase + idx;
                uint64_t k = dt[e].key;
                if (k == sign) break;
                if (k == EMPTY_KEY) {
                    uint64_t old = atomicCAS(ull(&dt[e].key), EMPTY_KEY, sign);
                    if (old == EMPTY_KEY || old == sign) break;
                }
                idx = (idx + 1 == tcap) ? 0 : idx + 1;
            }
        }
        tidx[gi] = e;
        if (dt[e].minpos > li) atomicMin(&dt[e].minpos, li);
    }
}

__device__ __forceinline__ uint32_t block_sum_256(uint32_t v, uint32_t* sh /*4*/) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) sh[wave] = v;
    __syncthreads();
    uint32_t t = sh[0] + sh[1] + sh[2] + sh[3];
    __syncthreads();
    return t;
}

// exclusive prefix of v over the 256 threads of the block; *total = block sum
// Exclusive scan over a workgroup of WAVES wavefronts (sh: WAVES entries of LDS).
template <typename T, int WAVES>
__device__ __forceinline__ T block_excl_scan(T v, T* sh, T* total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    T inc = v;
    for (int o = 1; o < 64; o <<= 1) {
        T t = __shfl_up(inc, o);
        if (lane >= o) inc += t;
    }
    if (lane == 63) sh[wave] = inc;
    __syncthreads();
    T base = 0, all = 0;
#pragma unroll
    for (int wv = 0; wv < WAVES; wv++) {
        if (wv < wave) base += sh[wv];
        all += sh[wv];
    }
    if (total) *total = all;
    __syncthreads();
    return base + inc - v;
}

template <typename T>
__device__ __forceinline__ T block_excl_scan_256(T v, T* sh /*4*/, T* total) {
    return block_excl_scan<T, 4>(v, sh, total);
}

// Step 2: a lookup is a first occurrence iff its position equals its entry's
// minpos.  One flag bit per lookup (8 per thread), one count per tile.
__global__ __launch_bounds__(REMAP_THREADS) void k_flag_count(const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                              const DedupEntry* __restrict__ dt,
                                                              const uint32_t* __restrict__ tidx,
                                                              uint8_t* __restrict__ flag8,
                                                              uint32_t* __restrict__ tilesum) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    __shared__ uint32_t red[4];
    load_lbase(lb, lbase, N);
    const uint32_t base = blockIdx.x * REMAP_TILE + threadIdx.x * REMAP_ITEMS;
    uint32_t bits = 0;
    if (base < L) {
        int sl = find_slot(lb, N, base);
        for (int j = 0; j < REMAP_ITEMS; j++) {
            const uint32_t gi = base + j;
            if (gi >= L) break;
            while (gi >= lb[sl + 1]) sl++;
            const uint32_t li = gi - lb[sl];
            if (dt[tidx[gi]].minpos == li) bits |= 1u << j;
        }
        flag8[base / REMAP_ITEMS] = (uint8_t)bits;
    }
    uint32_t total = block_sum_256(__popc(bits), red);
    if (threadIdx.x == 0) tilesum[blockIdx.x] = total;
}

// Exclusive scan of in[0 .. n) by one workgroup of 1024 threads: out[i] = sum of in[0 .. i);
// returns the total.  Every thread takes SCAN_ITEMS consecutive entries, so arrays of a few
// thousand entries need one round of barriers.  wsum: 16 entries of LDS, carry: one.
constexpr int SCAN_ITEMS = 8;

template <typename Out>
__device__ __forceinline__ uint32_t scan_u32_1024(const uint32_t* __restrict__ in, uint32_t n, uint32_t* wsum,
                                                  uint32_t* carry, Out out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) *carry = 0;
    __syncthreads();
    for (uint32_t start = 0; start < n; start += 1024 * SCAN_ITEMS) {
        const uint32_t i0 = start + threadIdx.x * SCAN_ITEMS;
        uint32_t v[SCAN_ITEMS];
        uint32_t mine = 0;
#pragma unroll
        for (int j = 0; j < SCAN_ITEMS; j++) {
            v[j] = (i0 + j < n) ? in[i0 + j] : 0;
            mine += v[j];
        }
        uint32_t inc = mine;
        for (int o = 1; o < 64; o <<= 1) {
            uint32_t t = __shfl_up(inc, o);
            if (lane >= o) inc += t;
        }
        if (lane == 63) wsum[wave] = inc;
        __syncthreads();
        uint32_t base = *carry;
        for (int wv = 0; wv < wave; wv++) base += wsum[wv];
        uint32_t run = base + inc - mine;
#pragma unroll
        for (int j = 0; j < SCAN_ITEMS; j++) {
            if (i0 + j < n) out(i0 + j, run);
            run += v[j];
        }
        __syncthreads();
        if (threadIdx.x == 1023) *carry = base + inc;
        __syncthreads();
    }
    return *carry;
}

// Step 3 (one workgroup): exclusive scan of the tile counts; total distinct
// count U; size of the group table; ubase of trailing empty slots.
__global__ __launch_bounds__(1024) void k_scan_tiles(const uint32_t* __restrict__ tilesum,
                                                     uint32_t* __restrict__ tileoff, uint32_t ntiles,
                                                     const uint32_t* __restrict__ lbase, uint32_t* __restrict__ ubase,
                                                     int N, uint32_t L, DevStatus* status) {
    __shared__ uint32_t wsum[16];
    __shared__ uint32_t carry_sh;
    const uint32_t U = scan_u32_1024(tilesum, ntiles, wsum, &carry_sh, [&](uint32_t i, uint32_t v) { tileoff[i] = v; });
    if (threadIdx.x == 0) {
        status->n_unique = U;
        uint32_t g = U + U / 2;
        status->gcap = g < 16 ? 16 : g;
    }
    for (int sl = threadIdx.x; sl <= N; sl += blockDim.x)
        if (lbase[sl] >= L) ubase[sl] = U;
}

// Step 4: rank of every first occurrence = number of first occurrences before
// it in the concatenated order; the compact lists of distinct signs follow.
__global__ __launch_bounds__(REMAP_THREADS) void k_assign_rank(
    const SlotDesc* __restrict__ descs, const uint32_t* __restrict__ lbase, int N, uint32_t L, DedupEntry* dt,
    const uint32_t* __restrict__ tidx, const uint8_t* __restrict__ flag8, const uint32_t* __restrict__ tileoff,
    uint32_t* __restrict__ ubase, uint64_t* __restrict__ uniq_sign, uint32_t* __restrict__ uniq_slot) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    __shared__ uint32_t red[4];
    load_lbase(lb, lbase, N);
    const uint32_t base = blockIdx.x * REMAP_TILE + threadIdx.x * REMAP_ITEMS;
    uint32_t bits = 0;
    if (base < L) bits = flag8[base / REMAP_ITEMS];
    uint32_t u = tileoff[blockIdx.x] + block_excl_scan_256<uint32_t>(__popc(bits), red, nullptr);
    if (base >= L) return;
    int sl = find_slot(lb, N, base);
    for (int j = 0; j < REMAP_ITEMS; j++) {
        const uint32_t gi = base + j;
        if (gi >= L) break;
        while (gi >= lb[sl + 1]) sl++;
        if (gi == lb[sl]) {
            // first lookup of slot sl: u distinct signs precede it; empty slots just before share the value
            ubase[sl] = u;
            for (int e = sl - 1; e >= 0 && lb[e] == gi; e--) ubase[e] = u;
        }
        if (bits & (1u << j)) {
            dt[tidx[gi]].rank = u;
            uniq_sign[u] = (uint64_t)descs[sl].values[gi - lb[sl]];
            uniq_slot[u] = (uint32_t)sl;
            u++;
        }
    }
}

constexpr uint32_t FIRST_BIT = 0x80000000u;

// Step 5: mapped id = rank within the slot (sparse_table_ops.cc:130).  The
// index of each lookup's distinct sign is kept for the push (u_of_gi, top bit
// set on first occurrences).
__global__ __launch_bounds__(256) void k_write_mapped(const SlotDesc* __restrict__ descs,
                                                      const uint32_t* __restrict__ lbase,
                                                      const uint32_t* __restrict__ ubase, int N, uint32_t L,
                                                      const DedupEntry* __restrict__ dt,
                                                      const uint32_t* __restrict__ tidx,
                                                      const uint8_t* __restrict__ flag8,
                                                      uint32_t* __restrict__ u_of_gi, int write_ids) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t gi = blockIdx.x * blockDim.x + threadIdx.x; gi < L; gi += stride) {
        const uint32_t u = dt[tidx[gi]].rank;
        const uint32_t first = (flag8[gi >> 3] >> (gi & 7)) & 1u;
        u_of_gi[gi] = u | (first ? FIRST_BIT : 0u);
        if (write_ids) {
            const int sl = find_slot(lb, N, gi);
            descs[sl].mapped[gi - lb[sl]] = (int64_t)(u - ubase[sl]);
        }
    }
}

// Push: batch_show = occurrences, batch_click = sum of labels per distinct sign
// (sparse_table_ops.cc:283-296; labels are narrowed to int as there), kept in
// the member lists.  Every sign starts at show 1 / click 0 ...
__global__ __launch_bounds__(256) void k_reset_counts(Member* __restrict__ list, const DevStatus* status,
                                                      uint32_t ids_cap, int keep_show) {
    const uint32_t n_single = status->n_single, n_members = status->n_members;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t t = blockIdx.x * blockDim.x + threadIdx.x; t < n_single + n_members; t += stride) {
        const uint32_t i = group_id(t, n_single, n_members, ids_cap);  // the member array is laid out like the ids
        if (!keep_show) list[i].show = 1;
        list[i].click = 0;
    }
}

constexpr int COUNT_TILE = 2048;
constexpr int COUNT_SLOTS = 4096;  // LDS table entries per tile (load factor <= 0.5)

// ... and the repeated lookups and the non-zero labels are added.  Repeats
// are concentrated on few signs, so each tile of 2048 lookups first adds them
// up in an LDS hash table and issues one global atomic per sign it saw.
__global__ __launch_bounds__(256) void k_count_show(const SlotDesc* __restrict__ descs,
                                                    const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                    const uint32_t* __restrict__ u_of_gi,
                                                    const uint2* __restrict__ where_u, Member* list,
                                                    int with_click) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    __shared__ uint32_t keys[COUNT_SLOTS];
    __shared__ int32_t cnts[COUNT_SLOTS];
    __shared__ int32_t clks[COUNT_SLOTS];
    if (with_click) load_lbase(lb, lbase, N);
    const uint32_t ntiles = (L + COUNT_TILE - 1) / COUNT_TILE;
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        for (int i = threadIdx.x; i < COUNT_SLOTS; i += 256) {
            keys[i] = 0xFFFFFFFFu;
            cnts[i] = 0;
            clks[i] = 0;
        }
        __syncthreads();
        for (int j = 0; j < COUNT_TILE / 256; j++) {
            const uint32_t gi = tile * COUNT_TILE + j * 256 + threadIdx.x;
            if (gi >= L) break;
            const uint32_t v = u_of_gi[gi];
            const uint32_t u = v & ~FIRST_BIT;
            int label = 0;
            if (with_click) {
                const int sl = find_slot(lb, N, gi);
                label = (int)descs[sl].labels[gi - lb[sl]];
            }
            const bool repeat = (v & FIRST_BIT) == 0;
            if (!repeat && label == 0) continue;
            uint32_t h = (u * 2654435761u) >> 20;  // 12 bits
            for (;;) {
                uint32_t old = atomicCAS(&keys[h], 0xFFFFFFFFu, u);
                if (old == 0xFFFFFFFFu || old == u) break;
                h = (h + 1) & (COUNT_SLOTS - 1);
            }
            if (repeat) atomicAdd(&cnts[h], 1);
            if (label != 0) atomicAdd(&clks[h], label);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < COUNT_SLOTS; i += 256) {
            const uint32_t u = keys[i];
            if (u == 0xFFFFFFFFu) continue;
            Member* m = &list[where_u[u].x & WHERE_PLACE];
            if (cnts[i]) atomicAdd(&m->show, cnts[i]);
            if (clks[i]) atomicAdd(&m->click, clks[i]);
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------ push grouping
// Where the sign / gradient / counts of record u of a push come from.
struct PushSrc {
    // table-level push (SparseTable::Push): records in one array
    const tn_sign_info* infos;
    const float* grads;
    // op-level push: compact distinct lists of the remap + per-slot gradient matrices
    const uint64_t* uniq_sign;
    const uint32_t* uniq_slot;
    const uint32_t* ubase;
    const SlotDesc* descs;
    int dim;
    // op-level push of pooled gradients: one reduced gradient row per distinct sign, record order
    const float* flat;
};

__device__ __forceinline__ uint64_t src_sign(const PushSrc& p, uint32_t u) {
    return p.infos ? p.infos[u].sign : p.uniq_sign[u];
}

// Records with the same sign must be applied one after the other in record
// order (sparse_table.cc:72-82).  Every record joins the group of its sign...
__global__ __launch_bounds__(256) void k_group_insert(PushSrc src, int64_t n_host, DevStatus* status, GroupEntry* gt,
                                                      uint32_t* __restrict__ gidx, uint32_t* __restrict__ ord) {
    const int64_t n = src.infos ? n_host : (int64_t)status->n_unique;
    const uint32_t gcap = status->gcap;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < n; u += stride) {
        const uint64_t sign = src_sign(src, (uint32_t)u);
        uint32_t e;
        if (sign == EMPTY_KEY) {
            e = gcap;
        } else {
            uint32_t idx = (uint32_t)slot_of(sign, gcap);
            for (;;) {
                e = idx;
                uint64_t k = gt[e].key;  // a stale EMPTY_KEY only costs a compare-and-swap
                if (k == sign) break;
                if (k == EMPTY_KEY) {
                    uint64_t old = atomicCAS(ull(&gt[e].key), EMPTY_KEY, sign);
                    if (old == EMPTY_KEY || old == sign) break;
                }
                idx = (idx + 1 == gcap) ? 0 : idx + 1;
            }
        }
        gidx[u] = e;
        ord[u] = atomicAdd(&gt[e].cnt, 1u) + 1u;  // arrival number inside the group
    }
}

constexpr int COMPACT_ITEMS = 16;

// Signs with big_k records or more are applied by one wavefront each.
__device__ __forceinline__ bool is_big(uint32_t k, uint32_t big_k) { return k >= big_k; }

// Numbers the groups found in one span of 256 x ITEMS table entries
// (ks[j] = records of the thread's j-th entry, 0 = unused) and gives each a
// slice of the member array.  Groups with one record get ids and member places
// counted up from 0 (place == id); groups with several get ids counted down
// from ids_cap - 1 and slices carved from the top of the member array; groups
// with big_k records or more are also listed in big_list.  Four atomics per span.
// write(j, g, off) stores the result for the thread's j-th entry.
template <int ITEMS, typename W>
__device__ __forceinline__ void compact_span(DevStatus* status, const uint32_t (&ks)[ITEMS], uint32_t ids_cap,
                                             uint32_t big_k, uint32_t* __restrict__ big_list, W write) {
    __shared__ unsigned long long sh[4];
    __shared__ uint32_t bases[4];
    unsigned long long cnt = 0;  // bits 0-31 single groups, 32-63 multi groups
    unsigned long long mem = 0;  // bits 0-39 records of multi groups, 40-63 big groups
    for (int j = 0; j < ITEMS; j++) {
        if (ks[j] == 1) cnt += 1ull;
        if (ks[j] > 1) {
            cnt += 1ull << 32;
            mem += ks[j];
            if (is_big(ks[j], big_k)) mem += 1ull << 40;
        }
    }
    unsigned long long tcnt, tmem;
    const unsigned long long ecnt = block_excl_scan_256<unsigned long long>(cnt, sh, &tcnt);
    const unsigned long long emem = block_excl_scan_256<unsigned long long>(mem, sh, &tmem);
    if (threadIdx.x == 0 && (uint32_t)tcnt) bases[0] = atomicAdd(&status->n_single, (uint32_t)tcnt);
    if (threadIdx.x == 64 && (tcnt >> 32)) bases[1] = atomicAdd(&status->n_multi, (uint32_t)(tcnt >> 32));
    if (threadIdx.x == 128 && tmem) bases[2] = atomicAdd(&status->n_members, (uint32_t)(tmem & 0xFFFFFFFFFFull));
    if (threadIdx.x == 192 && (tmem >> 40)) bases[3] = atomicAdd(&status->n_big, (uint32_t)(tmem >> 40));
    __syncthreads();
    uint32_t gs = bases[0] + (uint32_t)ecnt;                              // next single id
    uint32_t gm = bases[1] + (uint32_t)(ecnt >> 32);                      // multi groups before mine
    uint32_t mm = bases[2] + (uint32_t)(emem & 0xFFFFFFFFFFull);          // multi records before mine
    uint32_t bb = bases[3] + (uint32_t)(emem >> 40);
    for (int j = 0; j < ITEMS; j++) {
        const uint32_t k = ks[j];
        if (k == 0) continue;
        if (k == 1) {
            write(j, gs, gs);
            gs++;
        } else {
            const uint32_t g = ids_cap - 1 - gm;
            mm += k;
            write(j, g, ids_cap - mm);
            if (is_big(k, big_k)) big_list[bb++] = g;
            gm++;
        }
    }
    __syncthreads();
}

// ...every group gets a number and a slice of the member array...
__global__ __launch_bounds__(256) void k_group_compact(DevStatus* status, GroupEntry* gt,
                                                       uint64_t* __restrict__ grp_sign,
                                                       uint32_t* __restrict__ grp_off,
                                                       uint32_t* __restrict__ grp_cnt,
                                                       uint32_t* __restrict__ big_list, uint32_t big_k,
                                                       uint32_t ids_cap) {
    const uint32_t n = status->gcap + 1;
    const uint32_t span = 256 * COMPACT_ITEMS;
    for (uint32_t base = blockIdx.x * span; base < n; base += gridDim.x * span) {
        uint32_t ks[COMPACT_ITEMS];
        for (int j = 0; j < COMPACT_ITEMS; j++) {
            const uint32_t e = base + j * 256 + threadIdx.x;  // neighbouring lanes read neighbouring entries
            const uint32_t c = (e < n) ? gt[e].cnt : 0xFFFFFFFFu;
            ks[j] = (c != 0xFFFFFFFFu) ? c + 1 : 0;
        }
        compact_span(status, ks, ids_cap, big_k, big_list, [&](int j, uint32_t g, uint32_t off) {
            const uint32_t e = base + j * 256 + threadIdx.x;
            gt[e].g = g;
            grp_sign[g] = (e == n - 1) ? EMPTY_KEY : gt[e].key;
            grp_off[g] = off;
            grp_cnt[g] = ks[j];
        });
    }
}

// ...the members are written into it in arrival order...
__global__ __launch_bounds__(256) void k_group_fill(int64_t n_host, const uint32_t* n_dev, const GroupEntry* gt,
                                                    const uint32_t* __restrict__ grp_off,
                                                    const uint32_t* __restrict__ gidx,
                                                    const uint32_t* __restrict__ ord, uint32_t* __restrict__ arrival) {
    const int64_t n = n_dev ? (int64_t)*n_dev : n_host;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < n; u += stride)
        arrival[grp_off[gt[gidx[u]].g] + ord[u]] = (uint32_t)u;
}

// ...and finally put in ascending record order: the place of a record is the
// number of members of its group that precede it.
__global__ __launch_bounds__(256) void k_group_rank(int64_t n_host, const uint32_t* n_dev, const GroupEntry* gt,
                                                    const uint32_t* __restrict__ grp_off,
                                                    const uint32_t* __restrict__ gidx,
                                                    const uint32_t* __restrict__ arrival,
                                                    const uint32_t* __restrict__ uniq_slot,
                                                    const uint32_t* __restrict__ ushow, Member* __restrict__ list,
                                                    uint2* __restrict__ where_u) {
    const int64_t n = n_dev ? (int64_t)*n_dev : n_host;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; u < n; u += stride) {
        const GroupEntry en = gt[gidx[u]];
        const uint32_t k = en.cnt + 1;
        const uint32_t off = grp_off[en.g];
        uint32_t pos = 0;
        if (k > 1) {
            const uint32_t* mem = arrival + off;
            for (uint32_t t = 0; t < k; t++) pos += mem[t] < (uint32_t)u;
        }
        Member m;
        m.u = (uint32_t)u;
        m.slot = uniq_slot ? uniq_slot[u] : 0u;
        m.show = ushow ? (int32_t)ushow[u] : 1;
        m.click = 0;
        list[off + pos] = m;
        where_u[u] = make_uint2(off + pos, en.g);
    }
}

// ------------------------------------------ grouping by slot masks (N <= 128)
// Within one slot all signs are distinct, so a sign has at most one record per
// slot and its records in ascending order are its slots in ascending order.
// With at most 128 slots the set of slots of a sign fits two words: records
// mark their slot with one atomic (no value returned), and the place of a
// record in its group's member list is the number of marked slots below its
// own -- no arrival order, no sorting.  A cleared bit means "slot present"
// (entries are filled with 0xFF bytes).
struct MaskEntry {
    uint64_t key;
    uint32_t g;         // number of the group
    uint32_t off;       // start of its member list
    uint64_t nlo, nhi;  // complemented slot masks (16-byte aligned)
};

__global__ __launch_bounds__(256) void k_fill_masks(MaskEntry* gt, const DevStatus* status) {
    size_t n16 = ((size_t)status->gcap + 1) * 2;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    uint4 v = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
    uint4* p = reinterpret_cast<uint4*>(gt);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) p[i] = v;
}

__global__ __launch_bounds__(256) void k_mask_insert(const uint64_t* __restrict__ uniq_sign,
                                                     const uint32_t* __restrict__ uniq_slot, DevStatus* status,
                                                     MaskEntry* gt, uint32_t* __restrict__ gidx) {
    const uint32_t n = status->n_unique;
    const uint32_t gcap = status->gcap;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t u = blockIdx.x * blockDim.x + threadIdx.x; u < n; u += stride) {
        const uint64_t sign = uniq_sign[u];
        uint32_t e;
        if (sign == EMPTY_KEY) {
            e = gcap;
        } else {
            uint32_t idx = (uint32_t)slot_of(sign, gcap);
            for (;;) {
                e = idx;
                uint64_t k = gt[e].key;  // a stale EMPTY_KEY only costs a compare-and-swap
                if (k == sign) break;
                if (k == EMPTY_KEY) {
                    uint64_t old = atomicCAS(ull(&gt[e].key), EMPTY_KEY, sign);
                    if (old == EMPTY_KEY || old == sign) break;
                }
                idx = (idx + 1 == gcap) ? 0 : idx + 1;
            }
        }
        gidx[u] = e;
        const uint32_t sl = uniq_slot[u];
        atomicAnd(ull(sl < 64 ? &gt[e].nlo : &gt[e].nhi), ~(1ull << (sl & 63)));
    }
}

__global__ __launch_bounds__(256) void k_mask_compact(DevStatus* status, MaskEntry* gt,
                                                      uint64_t* __restrict__ grp_sign,
                                                      uint32_t* __restrict__ grp_off,
                                                      uint32_t* __restrict__ grp_cnt,
                                                      uint32_t* __restrict__ big_list, uint32_t big_k,
                                                      uint32_t ids_cap) {
    const uint32_t n = status->gcap + 1;
    const uint32_t span = 256 * COMPACT_ITEMS;
    for (uint32_t base = blockIdx.x * span; base < n; base += gridDim.x * span) {
        uint32_t ks[COMPACT_ITEMS];
        for (int j = 0; j < COMPACT_ITEMS; j++) {
            const uint32_t e = base + j * 256 + threadIdx.x;  // neighbouring lanes read neighbouring entries
            ks[j] = 0;
            if (e < n) {
                const ulonglong2 m = *reinterpret_cast<const ulonglong2*>(&gt[e].nlo);
                ks[j] = (uint32_t)(__popcll(~m.x) + __popcll(~m.y));
            }
        }
        compact_span(status, ks, ids_cap, big_k, big_list, [&](int j, uint32_t g, uint32_t off) {
            const uint32_t e = base + j * 256 + threadIdx.x;
            *reinterpret_cast<uint2*>(&gt[e].g) = make_uint2(g, off);
            grp_sign[g] = (e == n - 1) ? EMPTY_KEY : gt[e].key;
            grp_off[g] = off;
            grp_cnt[g] = ks[j];
        });
    }
}

__global__ __launch_bounds__(256) void k_mask_fill(const DevStatus* status, const MaskEntry* gt,
                                                   const uint32_t* __restrict__ gidx,
                                                   const uint32_t* __restrict__ uniq_slot,
                                                   const uint32_t* __restrict__ ushow, Member* __restrict__ list,
                                                   uint2* __restrict__ where_u) {
    const uint32_t n = status->n_unique;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t u = blockIdx.x * blockDim.x + threadIdx.x; u < n; u += stride) {
        const MaskEntry* en = &gt[gidx[u]];
        const ulonglong2 masks = *reinterpret_cast<const ulonglong2*>(&en->nlo);
        const uint2 go = *reinterpret_cast<const uint2*>(&en->g);
        const uint32_t sl = uniq_slot[u];
        const uint64_t lo = ~masks.x, hi = ~masks.y;
        uint32_t pos;
        if (sl < 64)
            pos = (uint32_t)__popcll(lo & ((1ull << sl) - 1ull));
        else
            pos = (uint32_t)__popcll(lo) + (uint32_t)__popcll(hi & ((1ull << (sl - 64)) - 1ull));
        Member m;
        m.u = u;
        m.slot = sl;
        m.show = ushow ? (int32_t)ushow[u] : 1;
        m.click = 0;
        list[go.y + pos] = m;
        where_u[u] = make_uint2(go.y + pos, go.x);
    }
}

// vars[slot][rank, :] = table row of the sign, for every distinct sign u of
// every slot (PopulatePulledVariable_, sparse_table_ops.cc:244-265).
// grp_row == nullptr: where_u[u].y is the row itself instead of the group that has it.
template <int VEC>
__global__ __launch_bounds__(256) void k_gather_vars(Store s, DevStatus* status, const uint32_t* __restrict__ grp_row,
                                                     const uint2* __restrict__ where_u,
                                                     const uint32_t* __restrict__ ubase, int N,
                                                     const SlotDesc* __restrict__ descs) {
    __shared__ uint32_t ub[MAX_SLOTS + 1];
    // A remap whose LDS tables overflowed dropped records: their where_u entries were never written (the
    // host repeats the call on the other path).  The flag is final before this kernel starts.
    if (status->err & DEV_ERR_REMAP_OVERFLOW) return;
    load_lbase(ub, ubase, N);
    const int chunks = s.wdim / VEC;
    const int64_t total = (int64_t)status->n_unique * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int64_t u = t / chunks;
        const int c = (int)(t - u * chunks);
        const uint32_t row = grp_row ? grp_row[where_u[u].y] : where_u[u].y;
        const int sl = find_slot(ub, N, (uint32_t)u);  // the slot whose window of distinct indices holds u
        const int64_t r = (int64_t)u - (int64_t)ub[sl];
        const SlotDesc& d = descs[sl];
        if (r >= d.rows) {
            if (c == 0) atomicOr(&status->err, DEV_ERR_VAR_CAPACITY);
            continue;
        }
        if (row > s.cap) continue;  // NO_ROW, or no row number at all: never address the table with it
        if (VEC == 4) {
            float4 v = *reinterpret_cast<const float4*>(s.w + (uint64_t)row * s.wstride + c * 4);
            *reinterpret_cast<float4*>(d.var + r * s.wdim + c * 4) = v;
        } else {
            d.var[r * s.wdim + c] = s.w[(uint64_t)row * s.wstride + c];
        }
    }
}

// -------------------------------------------------------------------- apply
// Resolves a member to its gradient row and counts; false if the op's gradient
// matrix has no such row.
__device__ __forceinline__ bool src_record(const PushSrc& p, Member member, const float*& g, int& show, int& click) {
    const uint32_t u = member.u;
    if (p.infos) {
        g = p.grads + (uint64_t)u * p.dim;
        show = p.infos[u].batch_show;
        click = p.infos[u].batch_click;
        return true;
    }
    show = member.show;
    click = member.click;
    if (p.flat) {
        g = p.flat + (uint64_t)u * p.dim;
        return true;
    }
    const uint32_t sl = member.slot;
    const int64_t r = (int64_t)u - (int64_t)p.ubase[sl];
    const SlotDesc& d = p.descs[sl];
    if (r >= d.rows) return false;
    g = d.grads + (uint64_t)r * p.dim;
    show = member.show;
    click = member.click;
    return true;
}

// The same through the gradient addresses worked out beforehand (k_member_grads): the record's
// member entry and its address are independent loads, the gradient is one round trip away
// instead of two.  ga == nullptr: resolve here.
__device__ __forceinline__ bool record_at(const PushSrc& p, const Member* mem, const float* const* ga, uint32_t j,
                                          const float*& g, int& show, int& click) {
    if (!ga) return src_record(p, mem[j], g, show, click);
    const Member m = mem[j];
    g = ga[j];
    show = m.show;
    click = m.click;
    return g != nullptr;
}

// Gradient row of every record of the groups with several records (their member lists fill the
// top of the member array): gaddr[place], nullptr where the op's gradient matrix has no such row.
// One coalesced pass that takes the slot descriptor out of the per-record chains of the apply
// kernels for those groups.
__global__ __launch_bounds__(256) void k_member_grads(PushSrc src, const DevStatus* status,
                                                      const Member* __restrict__ list,
                                                      const float** __restrict__ gaddr, uint32_t ids_cap) {
    if (status->mismatch | status->abort) return;
    const uint32_t n_members = status->n_members;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t t = blockIdx.x * blockDim.x + threadIdx.x; t < n_members; t += stride) {
        const uint32_t place = ids_cap - n_members + t;
        const float* gp = nullptr;
        int sh, ck;
        gaddr[place] = src_record(src, list[place], gp, sh, ck) ? gp : nullptr;
    }
}

// Push: are the signs of this call the ones the plan was built from?  With CLICKS the same
// pass adds the non-zero labels to the click sums of the plan's member lists, which start
// at zero (sparse_table_ops.cc:283-296; on a mismatch the plan is discarded anyway).  A
// mismatch is also written to host_mismatch (pinned host memory, cleared by the host before the
// launch), which the host reads once the kernel is done.  With gaddr != nullptr the first
// threads also do the work of k_member_grads (one launch less; harmless on a mismatch).
//
// One atomic per non-zero label would queue up on the entries of the frequent signs (a
// sign that takes a few percent of a slot's lookups receives thousands of adds): a workgroup
// first sums the labels of its tile per distinct record in an LDS table and then adds every
// entry to memory once.  A label that finds the table crowded goes to memory directly.
//
// What the signs are compared with: COPY, the plan's copy of them (the pulls that leave one: the small
// batches' and the one through the global table); else the fingerprints that k_tile_dedup left, one per 64 strided
// lookups of a tile (the lookups of one wavefront, here as there): 16 bytes to read instead of 512.  A
// fingerprint is two 64-bit sums over the run, of mix64(sign) and of its halves exchanged, each term times an
// odd weight drawn from the position.  One changed sign always alters the sums (the hash is a bijection, the
// weight odd); signs that changed places, or several changed signs, escape only if both sums come out equal by
// chance, which for hashes that behave as random numbers has odds below 2^-66.  (The reference has no such
// check: every push analyses its batch from scratch, sparse_table_ops.cc:274-297.)
struct Fingerprint {
    uint64_t a = 0, b = 0;
    __device__ __forceinline__ void add(uint32_t gi, uint64_t sign) { add_mixed(gi, mix64(sign)); }
    // m = mix64(sign), for a caller that has it already
    __device__ __forceinline__ void add_mixed(uint32_t gi, uint64_t m) {
        const uint32_t w = (gi * 0x9E3779B1u) | 1u;
        a += m * w;
        b += ((m << 32) | (m >> 32)) * w;
    }
    __device__ __forceinline__ void wave_sum() {
#pragma unroll
        for (int o = 32; o; o >>= 1) {
            a += __shfl_xor((unsigned long long)a, o);
            b += __shfl_xor((unsigned long long)b, o);
        }
    }
};
constexpr int VERIFY_ITEMS = 8;
constexpr int VERIFY_TILE = 256 * VERIFY_ITEMS;  // lookups per tile
constexpr int CLICK_BITS = 11;
constexpr int CLICK_TABLE = 1 << CLICK_BITS;     // entries of the tile's click table
constexpr int CLICK_TRIES = 16;

template <bool CLICKS, bool COPY>
__global__ __launch_bounds__(256) void k_verify_values(const SlotDesc* __restrict__ descs,
                                                       const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                       const uint64_t* __restrict__ vals_copy, DevStatus* status,
                                                       const uint32_t* __restrict__ u_of_gi,
                                                       const uint2* __restrict__ where_u, Member* list,
                                                       uint32_t* host_mismatch, PushSrc src,
                                                       const float** __restrict__ gaddr) {
    extern __shared__ uint32_t lb[];  // lb[N + 1], sized by the launch: more tiles in flight per CU than with a fixed array
    __shared__ uint32_t ckey[CLICKS ? CLICK_TABLE : 1];
    __shared__ int csum[CLICKS ? CLICK_TABLE : 1];
    __shared__ uint32_t crowded;  // a label of the tile went to memory directly: its record's sum in the table is not all of it
    load_lbase(lb, lbase, N);
    bool bad = false;
    const uint32_t n_members = gaddr ? status->n_members : 0;
    const uint32_t ntiles = (L + VERIFY_TILE - 1) / VERIFY_TILE;
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        if (CLICKS) {
            for (int i = threadIdx.x; i < CLICK_TABLE; i += 256) {
                ckey[i] = 0xFFFFFFFFu;  // no distinct index: they stay below FIRST_BIT
                csum[i] = 0;
            }
            if (threadIdx.x == 0) crowded = 0;
            __syncthreads();
        }
        const uint32_t g0 = tile * VERIFY_TILE;
        const uint32_t g1 = min(L, g0 + (uint32_t)VERIFY_TILE) - 1;
        const int s0 = find_slot(lb, N, g0);
        const bool one_slot = g1 < lb[s0 + 1];  // the usual case: the tile lies inside one slot
        uint64_t now[VERIFY_ITEMS], then[VERIFY_ITEMS];
        int label[VERIFY_ITEMS];
        uint32_t u[VERIFY_ITEMS];
#pragma unroll
        for (int j = 0; j < VERIFY_ITEMS; j++) {
            const uint32_t gi = g0 + j * 256 + threadIdx.x;
            now[j] = then[j] = 0;
            label[j] = 0;
            u[j] = 0;
            if (gi <= g1) {
                const int sl = one_slot ? s0 : find_slot(lb, N, gi);
                const SlotDesc& d = descs[sl];
                now[j] = (uint64_t)d.values[gi - lb[sl]];
                if (COPY) then[j] = vals_copy[gi];
                if (CLICKS) {
                    label[j] = (int)d.labels[gi - lb[sl]];
                    u[j] = u_of_gi[gi] & ~FIRST_BIT;
                }
                if (gi < n_members) {  // the member lists of the groups with several records fill the top of the array
                    const uint32_t place = L - n_members + gi;
                    const float* gp = nullptr;
                    int sh, ck;
                    gaddr[place] = src_record(src, list[place], gp, sh, ck) ? gp : nullptr;
                }
            }
        }
        if (!COPY) {
            Fingerprint print;
#pragma unroll
            for (int j = 0; j < VERIFY_ITEMS; j++) {
                const uint32_t gi = g0 + j * 256 + threadIdx.x;
                if (gi <= g1) print.add(gi, now[j]);
            }
            print.wave_sum();
            const ulonglong2 left = reinterpret_cast<const ulonglong2*>(vals_copy)[tile * (256 / 64) + (threadIdx.x >> 6)];
            bad |= print.a != left.x || print.b != left.y;
        }
#pragma unroll
        for (int j = 0; j < VERIFY_ITEMS; j++) {
            if (COPY) bad |= now[j] != then[j];
            if (CLICKS && label[j] != 0) {
                uint32_t h = (u[j] * 2654435761u) >> (32 - CLICK_BITS);
                bool placed = false;
                for (int tries = 0; tries < CLICK_TRIES && !placed; tries++) {
                    uint32_t old = ckey[h];
                    if (old == 0xFFFFFFFFu) old = atomicCAS(&ckey[h], 0xFFFFFFFFu, u[j]);
                    if (old == 0xFFFFFFFFu || old == u[j]) {
                        atomicAdd(&csum[h], label[j]);
                        placed = true;
                    }
                    h = (h + 1) & (CLICK_TABLE - 1);
                }
                if (!placed) {
                    crowded = 1;
                    atomicAdd(&list[where_u[u[j]].x & WHERE_PLACE].click, label[j]);
                }
            }
        }
        if (CLICKS) {
            __syncthreads();
            constexpr int PER = CLICK_TABLE / 256;
            uint32_t place[PER];
            int sum[PER];
#pragma unroll
            for (int j = 0; j < PER; j++) {
                const int e = j * 256 + threadIdx.x;
                sum[j] = csum[e];
                place[j] = sum[j] != 0 ? where_u[ckey[e]].x : 0u;
            }
            // A record whose lookups all lie in this tile gets its whole sum here: a plain store (the sums start at
            // zero), where an atomic would wait for its turn at the memory's atomic unit.
            const bool plain_ok = crowded == 0;
#pragma unroll
            for (int j = 0; j < PER; j++) {
                if (sum[j] == 0) continue;
                if ((place[j] & WHERE_ONE_TILE) && plain_ok)
                    list[place[j] & WHERE_PLACE].click = sum[j];
                else
                    atomicAdd(&list[place[j] & WHERE_PLACE].click, sum[j]);
            }
            __syncthreads();
        }
    }
    if (bad) {
        atomicOr(&status->mismatch, 1u);
        *host_mismatch = 1u;
    }
}

// The three update rules on one element.
//   AdaGrad  ada_grad_kernel.cc:105-129     Adam  adam_kernel.cc:112-125
//   Ftrl     ftrl_kernel.cc:57-80
__device__ __forceinline__ void adam_elem(const OptDev& o, float c1, float c2, float g, float& w, float& m, float& v) {
    m = o.beta1 * m + c1 * g;
    v = o.beta2 * v + c2 * g * g;
    w -= o.lr * m / (o.eps + sqrtf(v));
}

__device__ __forceinline__ void ftrl_elem(const OptDev& o, float g, float& w, float& z, float& n) {
    const float g2 = g * g;
    z += g - o.lr * (sqrtf(n + g2) - sqrtf(n)) * w;
    n += g2;
    if (fabsf(z) <= o.lambda1) {
        w = 0.f;
    } else {
        w = -1 / ((o.beta + sqrtf(n)) * o.lr + o.lambda2);
        if (z > 0)
            w *= z - o.lambda1;
        else
            w *= z + o.lambda1;
    }
}

// Most signs occur in one slot only: one record, no ordering problem, no
// loop.  LPG lanes update the row of one such sign; its member entry sits at
// the place of its group number.
template <int KIND, int LPG>
__global__ __launch_bounds__(256) void k_apply_single(Store s, OptDev o, PushSrc src, DevStatus* status,
                                                      const uint32_t* __restrict__ grp_row,
                                                      const Member* __restrict__ list) {
    // a push launched on a plan that turned out not to be its batch's (the host redoes it), or whose inputs are unusable
    if (status->mismatch | status->abort) return;
    const uint32_t n_single = status->n_single;
    const int D = s.D;
    const int sub = threadIdx.x % LPG;
    const int lane0 = (int)__lane_id() - sub;
    const uint32_t gstride = gridDim.x * (blockDim.x / LPG);
    const float c1 = 1 - o.beta1, c2 = 1 - o.beta2;
    for (uint32_t g = blockIdx.x * (blockDim.x / LPG) + threadIdx.x / LPG; g < n_single; g += gstride) {
        const uint32_t row = grp_row[g];
        if (row > s.cap) continue;  // NO_ROW (unknown sign: flagged by the probe), or no row number at all
        const float* gp;
        int bshow, bclick;
        if (!src_record(src, list[g], gp, bshow, bclick)) {
            if (sub == 0) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            continue;
        }
        float* wp = s.w + (uint64_t)row * s.wstride;
        float* sp = s.st + (uint64_t)row * s.sstride;
        const float4 gr = reinterpret_cast<const float4*>(gp)[sub];
        float4 w = reinterpret_cast<float4*>(wp)[sub];
        if (KIND == OPT_ADAGRAD) {
            const float4 h = *reinterpret_cast<const float4*>(sp);
            const float p0 = gr.x * gr.x, p1 = gr.y * gr.y, p2 = gr.z * gr.z, p3 = gr.w * gr.w;
            double tot = 0.0;  // add_g2sum: double accumulator over the float products, element order 0..D-1
            for (int l = 0; l < LPG; l++) {
                double cand = tot;
                cand += (double)p0;
                cand += (double)p1;
                cand += (double)p2;
                cand += (double)p3;
                tot = __shfl(cand, lane0 + l);
            }
            const float g2sum = (float)((double)h.x + tot / (double)D);
            const float den = o.eps + sqrtf(g2sum);
            w.x -= o.lr * gr.x / den;
            w.y -= o.lr * gr.y / den;
            w.z -= o.lr * gr.z / den;
            w.w -= o.lr * gr.w / den;
            reinterpret_cast<float4*>(wp)[sub] = w;
            if (sub == 0) {
                const float show = h.y + (float)bshow, click = h.z + (float)bclick;
                *reinterpret_cast<float4*>(sp) = make_float4(g2sum, show, click, 0.f);  // no_show_days = 0
                if (o.use_cvm) {
                    wp[D] = show;
                    wp[D + 1] = logf(click + 1) - logf(show + 1);
                }
            }
        } else {
            float4 a = reinterpret_cast<float4*>(sp)[sub];
            float4 b = reinterpret_cast<float4*>(sp + D)[sub];
            if (KIND == OPT_ADAM) {
                adam_elem(o, c1, c2, gr.x, w.x, a.x, b.x);
                adam_elem(o, c1, c2, gr.y, w.y, a.y, b.y);
                adam_elem(o, c1, c2, gr.z, w.z, a.z, b.z);
                adam_elem(o, c1, c2, gr.w, w.w, a.w, b.w);
            } else {
                ftrl_elem(o, gr.x, w.x, a.x, b.x);
                ftrl_elem(o, gr.y, w.y, a.y, b.y);
                ftrl_elem(o, gr.z, w.z, a.z, b.z);
                ftrl_elem(o, gr.w, w.w, a.w, b.w);
            }
            reinterpret_cast<float4*>(wp)[sub] = w;
            reinterpret_cast<float4*>(sp)[sub] = a;
            reinterpret_cast<float4*>(sp + D)[sub] = b;
            if (sub == 0) sp[2 * D + 1] = __int_as_float(__float_as_int(sp[2 * D + 1]) + bshow);
        }
    }
}

// One group of LPG lanes owns one distinct sign: it loads the row once, applies
// the sign's records in ascending record order (slot 0 first; the member list
// is sorted) and stores the row once.  Each lane holds one float4 of every
// per-element array; the next record's gradient is fetched while the current
// one is applied.  Groups with big_k records or more are left to k_apply_big.
// AHEAD = 1: the next record's gradient is fetched while the current one is applied (what keeps the most
// wavefronts on a CU: the kernels of a large batch).  AHEAD > 1: records are taken AHEAD at a time, the gradients
// of the next AHEAD and the member entries of the AHEAD after those in flight meanwhile: a chain of k records
// costs k / AHEAD round trips instead of 2 k, which is what a small batch, whose kernels are as long as their
// longest chain, is after.
template <int KIND, int LPG, int AHEAD = 1>
__device__ __forceinline__ void apply_group_vec(const Store& s, const OptDev& o, const PushSrc& src, DevStatus* status,
                                                uint32_t row, uint32_t k, const Member* mem, const float* const* ga,
                                                int sub, int lane0, float c1, float c2) {
    const int D = s.D;
    float* wp = s.w + (uint64_t)row * s.wstride;
    float* sp = s.st + (uint64_t)row * s.sstride;
    float4 w = reinterpret_cast<float4*>(wp)[sub];
    float4 a, b;          // Adam m,v / Ftrl z,n
    float g2sum = 0.f, show = 0.f, click = 0.f;
    int delta_show = 0;
    if (KIND == OPT_ADAGRAD) {
        float4 h = *reinterpret_cast<const float4*>(sp);
        g2sum = h.x;
        show = h.y;
        click = h.z;
    } else {
        a = reinterpret_cast<float4*>(sp)[sub];
        b = reinterpret_cast<float4*>(sp + D)[sub];
        delta_show = __float_as_int(sp[2 * D + 1]);
    }
    bool any = false;
    // one record applied to the row held in registers
    auto step = [&](const float4 gr, const int bshow, const int bclick) {
        any = true;
        if (KIND == OPT_ADAGRAD) {
            show += (float)bshow;
            click += (float)bclick;
            const float p0 = gr.x * gr.x, p1 = gr.y * gr.y, p2 = gr.z * gr.z, p3 = gr.w * gr.w;
            // add_g2sum: double accumulator over the float products, element order 0..D-1
            double tot = 0.0;
            for (int l = 0; l < LPG; l++) {
                double cand = tot;
                cand += (double)p0;
                cand += (double)p1;
                cand += (double)p2;
                cand += (double)p3;
                tot = __shfl(cand, lane0 + l);
            }
            g2sum = (float)((double)g2sum + tot / (double)D);
            const float den = o.eps + sqrtf(g2sum);
            w.x -= o.lr * gr.x / den;
            w.y -= o.lr * gr.y / den;
            w.z -= o.lr * gr.z / den;
            w.w -= o.lr * gr.w / den;
        } else if (KIND == OPT_ADAM) {
            delta_show += bshow;
            adam_elem(o, c1, c2, gr.x, w.x, a.x, b.x);
            adam_elem(o, c1, c2, gr.y, w.y, a.y, b.y);
            adam_elem(o, c1, c2, gr.z, w.z, a.z, b.z);
            adam_elem(o, c1, c2, gr.w, w.w, a.w, b.w);
        } else {
            delta_show += bshow;
            ftrl_elem(o, gr.x, w.x, a.x, b.x);
            ftrl_elem(o, gr.y, w.y, a.y, b.y);
            ftrl_elem(o, gr.z, w.z, a.z, b.z);
            ftrl_elem(o, gr.w, w.w, a.w, b.w);
        }
    };
    auto no_gradient = [&]() {
        if (sub == 0) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
    };
    if (AHEAD == 1) {
        const float* gp;
        int nshow = 0, nclick = 0;
        bool nok = record_at(src, mem, ga, 0, gp, nshow, nclick);
        float4 gnext = make_float4(0.f, 0.f, 0.f, 0.f);
        if (nok) gnext = reinterpret_cast<const float4*>(gp)[sub];
        for (uint32_t j = 0; j < k; j++) {
            const float4 gr = gnext;
            const int bshow = nshow, bclick = nclick;
            const bool ok = nok;
            if (j + 1 < k) {
                nok = record_at(src, mem, ga, j + 1, gp, nshow, nclick);
                if (nok) gnext = reinterpret_cast<const float4*>(gp)[sub];
            }
            if (!ok) {
                no_gradient();
                continue;
            }
            step(gr, bshow, bclick);
        }
    } else {
        // chunk c: applied; chunk c + 1: gradients in flight; chunk c + 2: member entries in flight.  Every load is
        // issued whether its record exists or not (past the end: the group's last member again, the row in place of
        // a gradient): a load under a condition makes the compiler wait for all loads where the branches join.
        Member m1[AHEAD], m2[AHEAD];
        const float* a1[AHEAD];  // with ga: the records' gradient addresses, worked out beforehand
        const float* a2[AHEAD];
        float4 g0[AHEAD], g1[AHEAD];
        int sh0[AHEAD], ck0[AHEAD], sh1[AHEAD], ck1[AHEAD];
        bool ok0[AHEAD], ok1[AHEAD];
        auto fetch = [&](const Member (&m)[AHEAD], const float* const (&a)[AHEAD], uint32_t first, float4 (&g)[AHEAD],
                         int (&sh)[AHEAD], int (&ck)[AHEAD], bool (&ok)[AHEAD]) {
#pragma unroll
            for (int q = 0; q < AHEAD; q++) {
                const float* gp = nullptr;
                if (ga) {
                    gp = a[q];
                    sh[q] = m[q].show;
                    ck[q] = m[q].click;
                    ok[q] = gp != nullptr && first + q < k;
                } else {
                    ok[q] = src_record(src, m[q], gp, sh[q], ck[q]) && first + q < k;
                }
                g[q] = reinterpret_cast<const float4*>(ok[q] ? gp : wp)[sub];
            }
        };
#pragma unroll
        for (int q = 0; q < AHEAD; q++) {
            m1[q] = mem[min((uint32_t)q, k - 1)];
            m2[q] = mem[min((uint32_t)(AHEAD + q), k - 1)];
            a1[q] = ga ? ga[min((uint32_t)q, k - 1)] : nullptr;
            a2[q] = ga ? ga[min((uint32_t)(AHEAD + q), k - 1)] : nullptr;
        }
        fetch(m1, a1, 0, g0, sh0, ck0, ok0);
#pragma unroll
        for (int q = 0; q < AHEAD; q++) {
            m1[q] = m2[q];
            a1[q] = a2[q];
        }
        for (uint32_t c0 = 0; c0 < k; c0 += AHEAD) {
#pragma unroll
            for (int q = 0; q < AHEAD; q++) {
                m2[q] = mem[min(c0 + 2 * AHEAD + q, k - 1)];
                a2[q] = ga ? ga[min(c0 + 2 * AHEAD + q, k - 1)] : nullptr;
            }
            fetch(m1, a1, c0 + AHEAD, g1, sh1, ck1, ok1);
            if constexpr (KIND == OPT_ADAGRAD) {
                // The records of the window depend on each other through g2sum (one rounded addition per record)
                // and through the row (one subtraction per element and record) only.  Everything else -- the sums of
                // squares with their hand-over from lane to lane, the square roots, the divisions -- is worked
                // out for all records of the window side by side; the two chains then run over the results, in
                // record order.  The same operations on the same operands as record after record.
                double mq[AHEAD];
#pragma unroll
                for (int q = 0; q < AHEAD; q++) mq[q] = 0.0;
                for (int l = 0; l < LPG; l++) {
#pragma unroll
                    for (int q = 0; q < AHEAD; q++) {
                        double cand = mq[q];  // add_g2sum: double accumulator over the float products, element order 0..D-1
                        cand += (double)(g0[q].x * g0[q].x);
                        cand += (double)(g0[q].y * g0[q].y);
                        cand += (double)(g0[q].z * g0[q].z);
                        cand += (double)(g0[q].w * g0[q].w);
                        mq[q] = __shfl(cand, lane0 + l);
                    }
                }
#pragma unroll
                for (int q = 0; q < AHEAD; q++) mq[q] = mq[q] / (double)D;
                float g2[AHEAD];
                bool missing = false;
#pragma unroll
                for (int q = 0; q < AHEAD; q++) {
                    if (ok0[q]) {
                        any = true;
                        show += (float)sh0[q];
                        click += (float)ck0[q];
                        g2sum = (float)((double)g2sum + mq[q]);
                    } else if (c0 + q < k) {
                        missing = true;
                    }
                    g2[q] = g2sum;
                }
                float4 st4[AHEAD];
#pragma unroll
                for (int q = 0; q < AHEAD; q++) {
                    const float den = o.eps + sqrtf(g2[q]);
                    st4[q] = make_float4(o.lr * g0[q].x / den, o.lr * g0[q].y / den, o.lr * g0[q].z / den,
                                         o.lr * g0[q].w / den);
                }
#pragma unroll
                for (int q = 0; q < AHEAD; q++) {
                    if (!ok0[q]) continue;
                    w.x -= st4[q].x;
                    w.y -= st4[q].y;
                    w.z -= st4[q].z;
                    w.w -= st4[q].w;
                }
                if (missing) no_gradient();
            } else {
#pragma unroll
                for (int q = 0; q < AHEAD; q++) {
                    if (c0 + q >= k) break;
                    if (!ok0[q]) {
                        no_gradient();
                        continue;
                    }
                    step(g0[q], sh0[q], ck0[q]);
                }
            }
#pragma unroll
            for (int q = 0; q < AHEAD; q++) {
                g0[q] = g1[q];
                sh0[q] = sh1[q];
                ck0[q] = ck1[q];
                ok0[q] = ok1[q];
                m1[q] = m2[q];
                a1[q] = a2[q];
            }
        }
    }
    if (!any) return;
    reinterpret_cast<float4*>(wp)[sub] = w;
    if (KIND == OPT_ADAGRAD) {
        if (sub == 0) {
            *reinterpret_cast<float4*>(sp) = make_float4(g2sum, show, click, 0.f);  // no_show_days = 0
            if (o.use_cvm) {
                wp[D] = show;
                wp[D + 1] = logf(click + 1) - logf(show + 1);
            }
        }
    } else {
        reinterpret_cast<float4*>(sp)[sub] = a;
        reinterpret_cast<float4*>(sp + D)[sub] = b;
        if (sub == 0) sp[2 * D + 1] = __int_as_float(delta_show);
    }
}

template <int KIND, int LPG>
__global__ __launch_bounds__(256) void k_apply_vec(Store s, OptDev o, PushSrc src, DevStatus* status,
                                                   const uint32_t* __restrict__ grp_row,
                                                   const uint32_t* __restrict__ grp_off,
                                                   const uint32_t* __restrict__ grp_cnt,
                                                   const Member* __restrict__ list, uint32_t big_k,
                                                   uint32_t ids_cap, const float* const* __restrict__ gaddr) {
    // a push launched on a plan that turned out not to be its batch's (the host redoes it), or whose inputs are unusable
    if (status->mismatch | status->abort) return;
    const uint32_t n_multi = status->n_multi;
    const int sub = threadIdx.x % LPG;                       // my float4 inside the row
    const int lane0 = (int)__lane_id() - sub;                // first lane of my group in the wavefront
    const uint32_t gstride = gridDim.x * (blockDim.x / LPG);
    const float c1 = 1 - o.beta1, c2 = 1 - o.beta2;
    for (uint32_t gi = blockIdx.x * (blockDim.x / LPG) + threadIdx.x / LPG; gi < n_multi; gi += gstride) {
        const uint32_t g = ids_cap - n_multi + gi;  // groups with several records sit at the top of the id space
        const uint32_t row = grp_row[g];
        if (row > s.cap) continue;  // NO_ROW (unknown sign: flagged by the probe), or no row number at all
        const uint32_t k = grp_cnt[g];
        if (is_big(k, big_k)) continue;
        apply_group_vec<KIND, LPG>(s, o, src, status, row, k, list + grp_off[g],
                                                 gaddr ? gaddr + grp_off[g] : nullptr, sub, lane0, c1, c2);
    }
}

// Value of v in lane `src` (the same for the whole wavefront), by register read-out.
__device__ __forceinline__ float lane_value(float v, int src) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ __forceinline__ double lane_value(double v, int src) {
    const long long b = __double_as_longlong(v);
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(b & 0xFFFFFFFFll), src);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(b >> 32), src);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

constexpr int BIG_DIM_MAX = 128;    // largest dim k_apply_big stages in LDS
constexpr int BIG_GBUF = 2176;      // floats of gradient staging per wavefront at most (dynamic LDS: big_gbuf_floats)

// Staging for up to BIG_CHUNK records of dim D (rows padded by one float), capped at BIG_GBUF.  The
// kernel is bound by the wavefronts a CU can hold (chains of dependent loads per sign), so the
// LDS of a wavefront is kept small enough not to be what limits them.
constexpr int BIG_CHUNK = 64;
constexpr int BIG_LOADS = 8;  // gradient loads a lane issues before it waits for the first
inline int big_gbuf_floats(int D) { return BIG_CHUNK * (D + 1) < BIG_GBUF ? BIG_CHUNK * (D + 1) : BIG_GBUF; }
// dynamic LDS of k_apply_big: the staging and the row (weights and two state vectors)
inline size_t big_lds_bytes(int D) { return (size_t)(big_gbuf_floats(D) + 3 * D) * sizeof(float); }

// A sign with many records (it occurs in many slots) would make one lane
// group chase a long chain of dependent loads.  Here one wavefront owns the
// sign: the row lives in LDS and the (already ordered) records are taken up
// to BIG_CHUNK at a time: the lanes resolve and fetch the gradients in parallel,
// then the records are applied strictly in order -- for AdaGrad the g2sum
// chain by one lane, the square roots by one lane per record, the element
// updates by one lane per element.
// The groups big_list[first], big_list[first + stride], ... by the wavefront that calls it (lane = the thread's
// lane).  gbuf: gbuf_floats floats of staging followed by the row (rw[D], ra[D], rb[D]); gptr, gshow, gok,
// den: BIG_CHUNK entries each, all in LDS and the wavefront's own.  sync(): makes what the lanes wrote to that
// LDS visible to each other (a workgroup of one wavefront: __syncthreads; a wavefront among others: wave_sync).
template <int KIND, typename Sync>
__device__ __forceinline__ void apply_big_groups(const Store& s, const OptDev& o, const PushSrc& src, DevStatus* status,
                                                 const uint32_t* __restrict__ big_list,
                                                 const uint32_t* __restrict__ grp_row,
                                                 const uint32_t* __restrict__ grp_off,
                                                 const uint32_t* __restrict__ grp_cnt,
                                                 const Member* __restrict__ list, int gbuf_floats,
                                                 const float* const* __restrict__ gaddr, float* gbuf, const float** gptr,
                                                 int* gshow, int* gok, float* den, int lane, uint32_t first,
                                                 uint32_t stride, Sync sync) {
    const int D = s.D;
    float* rw = gbuf + gbuf_floats;
    float* ra = rw + D;
    float* rb = ra + D;
    const int Dp = D + 1;  // padded staging row: lanes walking down a column hit different banks
    // a push launched on a plan that turned out not to be its batch's (the host redoes it), or whose inputs are unusable
    if (status->mismatch | status->abort) return;
    const uint32_t n_big = status->n_big;
    const int per_chunk = (gbuf_floats / Dp) < BIG_CHUNK ? (gbuf_floats / Dp) : BIG_CHUNK;
    const float c1 = 1 - o.beta1, c2 = 1 - o.beta2;
    const bool pow2 = (D & (D - 1)) == 0;
    const double inv_d = 1.0 / (double)D;  // exact when D is a power of two
    // D divides 64: the lanes tile (records, elements) as lane = record * D + element
    const bool tiled = D <= 64 && 64 % D == 0;
    const int li = tiled ? lane % D : 0, lm = tiled ? lane / D : 0, mstep = tiled ? 64 / D : 1;
    for (uint32_t bi = first; bi < n_big; bi += stride) {
        const uint32_t g = big_list[bi];
        const uint32_t row = grp_row[g];
        if (row > s.cap) continue;  // NO_ROW, or no row number at all: never address the table with it
        const uint32_t k = grp_cnt[g];
        const uint32_t off = grp_off[g];
        float* wp = s.w + (uint64_t)row * s.wstride;
        float* sp = s.st + (uint64_t)row * s.sstride;
        for (int i = lane; i < D; i += 64) {
            rw[i] = wp[i];
            if (KIND != OPT_ADAGRAD) {
                ra[i] = sp[i];
                rb[i] = sp[D + i];
            }
        }
        // the scalars of the row, the same in every lane
        float g2sum = 0.f, show = 0.f, click = 0.f;
        int delta_show = 0;
        if (KIND == OPT_ADAGRAD) {
            g2sum = sp[0];
            show = sp[1];
            click = sp[2];
        } else {
            delta_show = __float_as_int(sp[2 * D + 1]);
        }
        bool any = false;
        sync();
        for (uint32_t c0 = 0; c0 < k; c0 += per_chunk) {
            const int cn = (int)((k - c0) < (uint32_t)per_chunk ? (k - c0) : (uint32_t)per_chunk);
            // lane m resolves record m of the chunk and keeps its counts
            bool ok = false;
            int sh = 0, ck = 0;
            if (lane < cn) {
                const float* gp = nullptr;
                ok = record_at(src, list + off + c0, gaddr ? gaddr + off + c0 : nullptr, lane, gp, sh, ck);
                gptr[lane] = gp;
                gshow[lane] = sh;
                gok[lane] = ok ? 1 : 0;
            }
            const unsigned long long okmask = __ballot(ok);  // the usable records, known to every lane
            sync();
            // gradients into the staging, BIG_LOADS loads of a lane in flight at a time
            if (tiled) {  // lane = (record within a round, element): no division per element
                for (int m0 = lm; m0 < cn; m0 += mstep * BIG_LOADS) {
                    float v[BIG_LOADS];
#pragma unroll
                    for (int q = 0; q < BIG_LOADS; q++) {
                        const int m = m0 + q * mstep;
                        v[q] = (m < cn && ((okmask >> m) & 1ull)) ? gptr[m][li] : 0.f;
                    }
#pragma unroll
                    for (int q = 0; q < BIG_LOADS; q++) {
                        const int m = m0 + q * mstep;
                        if (m < cn) gbuf[m * Dp + li] = v[q];
                    }
                }
            } else {
                for (int t0 = lane; t0 < cn * D; t0 += 64 * BIG_LOADS) {
                    float v[BIG_LOADS];
#pragma unroll
                    for (int q = 0; q < BIG_LOADS; q++) {
                        const int t = t0 + q * 64;
                        v[q] = 0.f;
                        if (t < cn * D) {
                            const int m = t / D, i = t - m * D;
                            if ((okmask >> m) & 1ull) v[q] = gptr[m][i];
                        }
                    }
#pragma unroll
                    for (int q = 0; q < BIG_LOADS; q++) {
                        const int t = t0 + q * 64;
                        if (t < cn * D) {
                            const int m = t / D;
                            gbuf[m * Dp + (t - m * D)] = v[q];
                        }
                    }
                }
            }
            sync();
            if (KIND == OPT_ADAGRAD) {
                // add_g2sum / dim of record `lane`: double sum of float products in element order
                double mq = 0.0;
                if (lane < cn) {
                    const float* gr = gbuf + lane * Dp;
                    double tot = 0.0;
                    for (int i = 0; i < D; i++) tot += (double)(gr[i] * gr[i]);
                    mq = pow2 ? tot * inv_d : tot / (double)D;
                }
                // g2sum after every record (float += double, rounded each time), show and click in
                // record order: every lane runs the same chain on values read out of the records'
                // lanes, lane m keeps the g2sum its record meets
                const float fsh = (float)sh, fck = (float)ck;
                float myg2 = 0.f;
                for (int m = 0; m < cn; m++) {
                    if (!((okmask >> m) & 1ull)) continue;
                    show += lane_value(fsh, m);
                    click += lane_value(fck, m);
                    g2sum = (float)((double)g2sum + lane_value(mq, m));
                    if (lane == m) myg2 = g2sum;
                }
                if (lane < cn) den[lane] = o.eps + sqrtf(myg2);
                sync();
                // the steps lr * g / den of all records and elements by all lanes (independent divisions),
                // then per element the subtractions in record order
                if (tiled) {
                    for (int m = lm; m < cn; m += mstep) gbuf[m * Dp + li] = o.lr * gbuf[m * Dp + li] / den[m];
                } else {
                    for (int t = lane; t < cn * D; t += 64) {
                        const int m = t / D, i = t - m * D;
                        gbuf[m * Dp + i] = o.lr * gbuf[m * Dp + i] / den[m];
                    }
                }
                sync();
                for (int i = lane; i < D; i += 64) {
                    float w = rw[i];
                    for (int m = 0; m < cn; m++)
                        if ((okmask >> m) & 1ull) w -= gbuf[m * Dp + i];
                    rw[i] = w;
                }
            } else {
                if (lane == 0)
                    for (int m = 0; m < cn; m++)
                        if (gok[m]) delta_show += gshow[m];
                for (int i = lane; i < D; i += 64) {
                    float w = rw[i], a = ra[i], b = rb[i];
                    for (int m = 0; m < cn; m++) {
                        if (!gok[m]) continue;
                        if (KIND == OPT_ADAM)
                            adam_elem(o, c1, c2, gbuf[m * Dp + i], w, a, b);
                        else
                            ftrl_elem(o, gbuf[m * Dp + i], w, a, b);
                    }
                    rw[i] = w;
                    ra[i] = a;
                    rb[i] = b;
                }
            }
            const unsigned long long chunk_mask = cn == 64 ? ~0ull : (1ull << cn) - 1ull;
            if (okmask) any = true;
            if (lane == 0 && okmask != chunk_mask) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            sync();
        }
        if (any) {
            for (int i = lane; i < D; i += 64) {
                wp[i] = rw[i];
                if (KIND != OPT_ADAGRAD) {
                    sp[i] = ra[i];
                    sp[D + i] = rb[i];
                }
            }
            if (lane == 0) {
                if (KIND == OPT_ADAGRAD) {
                    sp[0] = g2sum;
                    sp[1] = show;
                    sp[2] = click;
                    sp[3] = 0.f;  // no_show_days = 0
                    if (o.use_cvm) {
                        wp[D] = show;
                        wp[D + 1] = logf(click + 1) - logf(show + 1);
                    }
                } else {
                    sp[2 * D + 1] = __int_as_float(delta_show);
                }
            }
        }
        sync();
    }
}

// Fences a wavefront's LDS traffic: what its lanes wrote before is what they read after (the LDS unit takes a
// wavefront's instructions in order; the fence keeps the compiler from moving them across).
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int KIND>
__global__ __launch_bounds__(64) void k_apply_big(Store s, OptDev o, PushSrc src, DevStatus* status,
                                                  const uint32_t* __restrict__ big_list,
                                                  const uint32_t* __restrict__ grp_row,
                                                  const uint32_t* __restrict__ grp_off,
                                                  const uint32_t* __restrict__ grp_cnt,
                                                  const Member* __restrict__ list, int gbuf_floats,
                                                  const float* const* __restrict__ gaddr) {
    extern __shared__ float gbuf[];  // gbuf_floats floats of staging, then the row: rw[D], ra[D], rb[D]
    __shared__ const float* gptr[BIG_CHUNK];
    __shared__ int gshow[BIG_CHUNK], gok[BIG_CHUNK];
    __shared__ float den[BIG_CHUNK];
    apply_big_groups<KIND>(s, o, src, status, big_list, grp_row, grp_off, grp_cnt, list, gbuf_floats, gaddr, gbuf, gptr,
                           gshow, gok, den, (int)threadIdx.x, blockIdx.x, gridDim.x, [] { __syncthreads(); });
}

// k_apply_big for AdaGrad rows of D elements, D a power of two from 4 to 64, on a plan whose big_desc lists
// {row, first member, records, group} of every sign with many records (written by k_group_emit): one wavefront
// per sign, its records up to BigTile<D>::CHUNK at a time.  The lanes tile (record, element) as
// lane = record * D + element, 64 / D records a round, and keep the gradients of their rounds in registers, so
// every gradient load of a chunk is in flight at once; the sign's description is asked for together with the
// status, the row together with the first records.  The staging in LDS only turns the tile round -- a lane per
// record for the sum of squares (double, in element order), a lane per element for the subtractions (in record
// order) -- and every loop over it fetches several entries before it uses the first, so that no step of a chain
// waits for LDS.  Operation for operation the arithmetic of apply_big_groups.
template <int D>
struct BigTile {
    static constexpr int R = 64 / D;                                            // records a round
    static constexpr int MOST = D == 32 ? 8 : 16;                               // (what the register file takes without spilling)
    static constexpr int ROUNDS = BIG_CHUNK / R < MOST ? BIG_CHUNK / R : MOST;  // gradient registers of a lane
    static constexpr int CHUNK = R * ROUNDS;
    static constexpr int DP = D + 1;  // padded staging row: lanes walking down a column hit different banks
};
template <int D>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(6, 8))) void k_apply_big_adagrad(
    Store s, OptDev o, PushSrc src, DevStatus* status, const uint4* __restrict__ big_desc, uint32_t desc_cap,
    const Member* __restrict__ list, const float* const* __restrict__ gaddr) {
    using T = BigTile<D>;
    constexpr int R = T::R, DP = T::DP;
    __shared__ float gbuf[T::CHUNK * DP];
    __shared__ const float* gptr[T::CHUNK];
    __shared__ float den[T::CHUNK];
    const int lane = (int)threadIdx.x;
    const int li = lane & (D - 1), lm = lane / D;
    uint4 head = big_desc[blockIdx.x < desc_cap ? blockIdx.x : desc_cap - 1];  // (before the status is known)
    // a push launched on a plan that turned out not to be its batch's (the host redoes it), or whose inputs are unusable
    if (status->mismatch | status->abort) return;
    const uint32_t n_big = status->n_big;
    constexpr double inv_d = 1.0 / (double)D;  // exact: D is a power of two
    for (uint32_t bi = blockIdx.x; bi < n_big; bi += gridDim.x) {
        if (bi != blockIdx.x) head = big_desc[bi];
        const uint32_t row = head.x, off = head.y, k = head.z;
        if (row > s.cap) continue;  // NO_ROW, or no row number at all: never address the table with it
        float* wp = s.w + (uint64_t)row * s.wstride;
        float* sp = s.st + (uint64_t)row * s.sstride;
        float w = lane < D ? wp[lane] : 0.f;
        float g2sum = sp[0], show = sp[1], click = sp[2];
        bool any = false;
        for (uint32_t c0 = 0; c0 < k; c0 += T::CHUNK) {
            const int cn = (int)((k - c0) < (uint32_t)T::CHUNK ? (k - c0) : (uint32_t)T::CHUNK);
            bool ok = false;
            int sh = 0, ck = 0;
            if (lane < cn) {
                const float* gp = nullptr;
                ok = record_at(src, list + off + c0, gaddr ? gaddr + off + c0 : nullptr, lane, gp, sh, ck);
                gptr[lane] = gp;
            }
            const unsigned long long okmask = __ballot(ok);
            const unsigned long long chunk_mask = cn == 64 ? ~0ull : (1ull << cn) - 1ull;
            __syncthreads();
            {
                float v[T::ROUNDS];
#pragma unroll
                for (int q = 0; q < T::ROUNDS; q++) {
                    const int m = lm + q * R;
                    v[q] = (m < cn && ((okmask >> m) & 1ull)) ? gptr[m][li] : 0.f;
                }
#pragma unroll
                for (int q = 0; q < T::ROUNDS; q++) gbuf[(lm + q * R) * DP + li] = v[q];
            }
            __syncthreads();
            // add_g2sum / dim of record `lane`: double sum of float products in element order
            double mq = 0.0;
            if (lane < cn) {
                const float* gr = gbuf + lane * DP;
                constexpr int AT_ONCE = D < 16 ? D : 16;
                double tot = 0.0;
#pragma unroll
                for (int i0 = 0; i0 < D; i0 += AT_ONCE) {
                    float a[AT_ONCE];
#pragma unroll
                    for (int i = 0; i < AT_ONCE; i++) a[i] = gr[i0 + i];
#pragma unroll
                    for (int i = 0; i < AT_ONCE; i++) tot += (double)(a[i] * a[i]);
                }
                mq = tot * inv_d;
            }
            // g2sum after every record (float += double, rounded each time), show and click in record order:
            // every lane runs the same chain on values read out of the records' lanes, lane m keeps the g2sum
            // its record meets
            const float fsh = (float)sh, fck = (float)ck;
            float myg2 = 0.f;
            if (okmask == chunk_mask) {
                for (int m = 0; m < cn; m++) {
                    show += lane_value(fsh, m);
                    click += lane_value(fck, m);
                    g2sum = (float)((double)g2sum + lane_value(mq, m));
                    if (lane == m) myg2 = g2sum;
                }
            } else {
                for (int m = 0; m < cn; m++) {
                    if (!((okmask >> m) & 1ull)) continue;
                    show += lane_value(fsh, m);
                    click += lane_value(fck, m);
                    g2sum = (float)((double)g2sum + lane_value(mq, m));
                    if (lane == m) myg2 = g2sum;
                }
            }
            if (lane < cn) den[lane] = o.eps + sqrtf(myg2);
            __syncthreads();
            // the steps lr * g / den of all records and elements (independent divisions, the operands of a few
            // rounds fetched together); a record without a gradient row steps by zero, which leaves the weights
            // as they are
#pragma unroll 4
            for (int m = lm; m < cn; m += R) {
                const float gv = gbuf[m * DP + li], dn = den[m];
                gbuf[m * DP + li] = ((okmask >> m) & 1ull) ? o.lr * gv / dn : 0.f;
            }
            __syncthreads();
            // per element the subtractions in record order
            if (lane < D) {
                for (int m0 = 0; m0 < cn; m0 += 8) {
                    float t[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) t[j] = m0 + j < cn ? gbuf[(m0 + j) * DP + lane] : 0.f;
#pragma unroll
                    for (int j = 0; j < 8; j++) w -= t[j];
                }
            }
            if (okmask) any = true;
            if (lane == 0 && okmask != chunk_mask) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            __syncthreads();
        }
        if (any) {
            if (lane < D) wp[lane] = w;
            if (lane == 0) {
                sp[0] = g2sum;
                sp[1] = show;
                sp[2] = click;
                sp[3] = 0.f;  // no_show_days = 0
                if (o.use_cvm) {
                    wp[D] = show;
                    wp[D + 1] = logf(click + 1) - logf(show + 1);
                }
            }
        }
    }
}


// Any dim / alignment: one thread per distinct sign, scalar loops.
template <int KIND>
__global__ __launch_bounds__(256) void k_apply_scalar(Store s, OptDev o, PushSrc src, DevStatus* status,
                                                      const uint32_t* __restrict__ grp_row,
                                                      const uint32_t* __restrict__ grp_off,
                                                      const uint32_t* __restrict__ grp_cnt,
                                                      const Member* __restrict__ list, uint32_t big_k,
                                                      uint32_t ids_cap) {
    // a push launched on a plan that turned out not to be its batch's (the host redoes it), or whose inputs are unusable
    if (status->mismatch | status->abort) return;
    const uint32_t n_single = status->n_single, n_multi = status->n_multi;
    const int D = s.D;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t t = blockIdx.x * blockDim.x + threadIdx.x; t < n_single + n_multi; t += stride) {
        const uint32_t g = group_id(t, n_single, n_multi, ids_cap);
        const uint32_t row = grp_row[g];
        if (row > s.cap) continue;  // NO_ROW, or no row number at all: never address the table with it
        const uint32_t k = grp_cnt[g];
        if (is_big(k, big_k)) continue;
        const Member* mem = list + grp_off[g];
        float* w = s.w + (uint64_t)row * s.wstride;
        float* sp = s.st + (uint64_t)row * s.sstride;
        for (uint32_t j = 0; j < k; j++) {
            const float* gp;
            int bshow, bclick;
            if (!src_record(src, mem[j], gp, bshow, bclick)) {
                atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
                continue;
            }
            if (KIND == OPT_ADAGRAD) {
                float show = sp[1] + (float)bshow;
                float click = sp[2] + (float)bclick;
                double add = 0.0;
                for (int i = 0; i < D; i++) add += (double)(gp[i] * gp[i]);
                float g2sum = (float)((double)sp[0] + add / (double)D);
                const float den = o.eps + sqrtf(g2sum);
                for (int i = 0; i < D; i++) w[i] -= o.lr * gp[i] / den;
                sp[0] = g2sum;
                sp[1] = show;
                sp[2] = click;
                sp[3] = 0.f;
                if (o.use_cvm) {
                    w[D] = show;
                    w[D + 1] = logf(click + 1) - logf(show + 1);
                }
            } else if (KIND == OPT_ADAM) {
                sp[2 * D + 1] = __int_as_float(__float_as_int(sp[2 * D + 1]) + bshow);
                float* m = sp;
                float* v = sp + D;
                const float c1 = 1 - o.beta1, c2 = 1 - o.beta2;
                for (int i = 0; i < D; i++) {
                    const float gi = gp[i];
                    m[i] = o.beta1 * m[i] + c1 * gi;
                    v[i] = o.beta2 * v[i] + c2 * gi * gi;
                    w[i] -= o.lr * m[i] / (o.eps + sqrtf(v[i]));
                }
            } else {
                sp[2 * D + 1] = __int_as_float(__float_as_int(sp[2 * D + 1]) + bshow);
                float* z = sp;
                float* nn = sp + D;
                for (int i = 0; i < D; i++) {
                    const float gi = gp[i];
                    const float g2 = gi * gi;
                    z[i] += gi - o.lr * (sqrtf(nn[i] + g2) - sqrtf(nn[i])) * w[i];
                    nn[i] += g2;
                    if (fabsf(z[i]) <= o.lambda1) {
                        w[i] = 0.f;
                    } else {
                        float nw = -1 / ((o.beta + sqrtf(nn[i])) * o.lr + o.lambda2);
                        if (z[i] > 0)
                            nw *= z[i] - o.lambda1;
                        else
                            nw *= z[i] + o.lambda1;
                        w[i] = nw;
                    }
                }
            }
        }
    }
}

}  // namespace tn

#endif  // TN_SPARSE_KERNELS_H_
