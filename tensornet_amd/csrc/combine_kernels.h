// The step TensorFlow runs around the pull / push ops of a slot: the combiner of
// tf.nn.embedding_lookup_sparse on the pulled rows (forward) and the reduction of
// its gradient to one row per distinct sign (backward), which the reference
// receives ready-made as the `grads` input of SparseTablePush
// (tensornet/layers/embedding_features.py:278-280, core/kernels/sparse_table_ops.cc:336-352).
//
//   forward   out[b, :] = (sum over the lookups i of example b, in order, of var[mapped[i], :]) / d(n_b)
//             d(n) = 1 (sum), n (mean), sqrt(n) (sqrtn); an example without lookups gives zeros
//   backward  g[u, :]   = sum over the lookups i of distinct sign u, in order, of dout[b(i), :] * (1 / d(n_b(i)))
//
// Both are deterministic: sums run in occurrence order.  The backward pass
// gets the lookups of every distinct sign side by side, in position order, from a
// counting sort per slot followed by an ordering of every sign's lookups by example
// (k_place_lookups, k_rank_short, k_rank_mid, k_order_huge).
#ifndef TN_COMBINE_KERNELS_H_
#define TN_COMBINE_KERNELS_H_

#include "sparse_kernels.h"

namespace tn {

enum { COMBINE_SUM = 0, COMBINE_MEAN = 1, COMBINE_SQRTN = 2 };
constexpr int COMBINE_WINDOW = 8;  // lookups of an example / of a distinct sign read ahead with independent loads

// In these kernels a SlotDesc carries: values = mapped ids (forward) / signs (backward),
// mapped = example index of every lookup, grads = rows to read (variable / pooled gradient),
// var = rows to write (forward: out[batch, dim]), rows = rows of `grads`, len = lookups.
__device__ __forceinline__ const int64_t* example_of(const SlotDesc& d) { return d.mapped; }

__device__ __forceinline__ float combine_divisor(uint32_t n, int combiner) {
    if (combiner == COMBINE_SUM || n == 0) return 1.f;
    return combiner == COMBINE_MEAN ? (float)n : sqrtf((float)n);
}

// Forward, step 1: where the lookups of every example start (rowptr[s * (batch + 1) + b], with
// rowptr[.. + batch] = lookups of the slot), from the sorted example ids; also checks them.
__global__ __launch_bounds__(256) void k_example_rowptr(const SlotDesc* __restrict__ descs,
                                                        const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                        int64_t batch, uint32_t* __restrict__ rowptr,
                                                        DevStatus* status) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t gi = blockIdx.x * blockDim.x + threadIdx.x; gi < L; gi += stride) {
        const int sl = find_slot(lb, N, gi);
        const SlotDesc& d = descs[sl];
        const int64_t* ex = example_of(d);
        const uint32_t i = gi - lb[sl];
        const int64_t b = ex[i];
        const int64_t prev = i > 0 ? ex[i - 1] : -1;
        if (b < 0 || b >= batch || prev > b) {
            atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            continue;
        }
        uint32_t* rp = rowptr + (size_t)sl * (batch + 1);
        for (int64_t r = prev + 1; r <= b; r++) rp[r] = i;  // example b starts here; the ones skipped are empty
        if (i == d.len - 1)
            for (int64_t r = b + 1; r <= batch; r++) rp[r] = d.len;
    }
}

// Forward, step 2: one group of `chunks` threads per (slot, example) sums the rows of the example's
// lookups in order, divides, and writes the output row (zeros for an example without lookups).
template <int VEC>
__global__ __launch_bounds__(256) void k_combine_fwd(const SlotDesc* __restrict__ descs, int N, int dim, int64_t batch,
                                                     int combiner, const uint32_t* __restrict__ rowptr,
                                                     DevStatus* status) {
    if (status->err) return;  // bad example ids: the row pointers are not to be trusted
    const int chunks = dim / VEC;
    const int64_t per_slot = batch * chunks;
    const int64_t total = (int64_t)N * per_slot;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const int sl = (int)(t / per_slot);
        const int64_t rest = t - (int64_t)sl * per_slot;
        const int64_t b = rest / chunks;
        const int c = (int)(rest - b * chunks);
        const SlotDesc& d = descs[sl];
        const uint32_t* rp = rowptr + (size_t)sl * (batch + 1);
        const uint32_t lo = d.len ? rp[b] : 0, hi = d.len ? rp[b + 1] : 0;
        const int64_t* ids = d.values;
        const float* rows = d.grads;
        const int64_t nrows = d.rows;
        float acc[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) acc[q] = 0.f;
        bool bad_id = false;
        // windows of COMBINE_WINDOW lookups: ids first, then their rows, all loads independent;
        // the additions run in lookup order
        for (uint32_t j0 = lo; j0 < hi; j0 += COMBINE_WINDOW) {
            int64_t wid[COMBINE_WINDOW];
#pragma unroll
            for (int q = 0; q < COMBINE_WINDOW; q++) wid[q] = (j0 + q < hi) ? ids[j0 + q] : -1;
            float wr[COMBINE_WINDOW][VEC];
#pragma unroll
            for (int q = 0; q < COMBINE_WINDOW; q++) {
                const bool in = j0 + q < hi;
                const bool ok = in && wid[q] >= 0 && wid[q] < nrows;
                if (in && !ok) bad_id = true;
                const float* row = rows + (ok ? wid[q] : 0) * dim + c * VEC;
                if (VEC == 4) {
                    const float4 v = ok ? *reinterpret_cast<const float4*>(row) : make_float4(0.f, 0.f, 0.f, 0.f);
                    wr[q][0] = v.x;
                    wr[q][1 % VEC] = v.y;
                    wr[q][2 % VEC] = v.z;
                    wr[q][3 % VEC] = v.w;
                } else {
                    wr[q][0] = ok ? row[0] : 0.f;
                }
            }
#pragma unroll
            for (int q = 0; q < COMBINE_WINDOW; q++)
                if (j0 + q < hi)
#pragma unroll
                    for (int v = 0; v < VEC; v++) acc[v] += wr[q][v];
        }
        if (bad_id && c == 0) atomicOr(&status->err, DEV_ERR_VAR_CAPACITY);
        const float div = combine_divisor(hi - lo, combiner);
        float* o = d.var + b * dim + c * VEC;
        if (VEC == 4)
            *reinterpret_cast<float4*>(o) = make_float4(acc[0] / div, acc[1 % VEC] / div, acc[2 % VEC] / div, acc[3 % VEC] / div);
        else
            o[0] = acc[0] / div;
    }
}

// Backward, step 1: the value of every lookup: its example in the high word, the number of
// lookups of that example in the low word -- all the reduction needs to know about the lookup, so
// that it reads them in the order of the distinct signs instead of chasing positions.  The first
// lookup of an example writes the values of all its lookups.
__global__ __launch_bounds__(256) void k_lookup_keys(const SlotDesc* __restrict__ descs,
                                                     const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                     int64_t batch, uint64_t* __restrict__ vals, DevStatus* status,
                                                     uint32_t* long_count) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    // [0] list of the frequent signs, filled by k_reduce_pooled; [1], [2] lists of k_place_lookups
    if (blockIdx.x == 0 && threadIdx.x < 3) long_count[threadIdx.x] = 0;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t gi = blockIdx.x * blockDim.x + threadIdx.x; gi < L; gi += stride) {
        const int sl = find_slot(lb, N, gi);
        const SlotDesc& d = descs[sl];
        const int64_t* ex = example_of(d);
        const uint32_t i = gi - lb[sl];
        const int64_t b = ex[i];
        const int64_t prev = i > 0 ? ex[i - 1] : -1;
        if (b < 0 || b >= batch || prev > b) {
            atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            status->abort = 1;  // values of later lookups may never be written: nothing downstream may run
            vals[gi] = ~0ull;
            continue;
        }
        if (prev == b) continue;
        uint32_t j = i;
        while (j < d.len && ex[j] == b) j++;
        const uint64_t v = ((uint64_t)b << 32) | (uint64_t)(j - i);
        for (uint32_t q = i; q < j; q++) vals[lb[sl] + q] = v;
    }
}

// Step 2: the values of the lookups of every distinct index side by side, in position order:
// svals[seg_off[u] .. seg_off[u + 1]).  The example ids of a slot ascend with the position and two lookups of
// one sign in one example carry the same value, so "position order" is "ascending value" and ties do not
// matter: no stable sort is needed.
//   k_place_lookups  a few workgroups per slot (the distinct indices of a slot's lookups fill a window of their
//                    own, ascending with the slots): counts the lookups of every index in an LDS array, scans
//                    the counts into seg_off, and puts every lookup into its index's segment -- in the order the
//                    atomics arrive; indices with ORDER_MID lookups or more are listed for the kernels below
//   k_rank_short     a lookup of a short segment finds its place by counting the values of its segment below it
//   k_rank_mid       a sorting network in LDS, one workgroup per segment of ORDER_MID .. ORDER_HUGE - 1 lookups
//   k_order_huge     the few longer segments: counting sort over the example ids, one workgroup each
// A slot with more distinct signs than the LDS array holds (lds_cap) keeps its counters in `gcur`.
constexpr int PLACE_THREADS = 1024;
constexpr int PLACE_ITEMS = 8;
constexpr uint32_t ORDER_MID = 64;
constexpr uint32_t ORDER_HUGE = 1024;

// `parts` workgroups per slot: each of them streams all lookups of the slot (they come out of L2 after the first)
// and takes those whose distinct index lies in its share of the slot's window of distinct indices -- a workgroup
// per slot leaves most of the device idle, and what bounds it are the LDS atomics and the stores that depend on
// them, which a share divides.  The lookups of the indices below its share, which it counts on the way, come
// before its own in svals.
__global__ __launch_bounds__(PLACE_THREADS) void k_place_lookups(
    const uint32_t* __restrict__ lbase, const uint32_t* __restrict__ ubase, int N, uint32_t L,
    const uint32_t* __restrict__ u_of_gi, const uint64_t* __restrict__ vals, uint32_t* __restrict__ tkey,
    uint64_t* __restrict__ tval, uint32_t* __restrict__ seg_off, uint32_t* __restrict__ gcur, uint32_t lds_cap,
    uint32_t* __restrict__ mid_list, uint32_t* __restrict__ huge_list, uint32_t* counts, const DevStatus* status,
    uint32_t parts) {
    extern __shared__ uint32_t lcur[];
    __shared__ uint32_t red[PLACE_THREADS / 64];
    __shared__ uint32_t carry_sh;
    if (status->abort) return;
    const int sl = blockIdx.x / parts;
    const uint32_t part = blockIdx.x % parts;
    const uint32_t l0 = lbase[sl], len = lbase[sl + 1] - l0;
    const uint32_t ub = ubase[sl], us = ubase[sl + 1] - ub;
    if (sl == N - 1 && part == 0 && threadIdx.x == 0) seg_off[ubase[N]] = L;
    if (len == 0) return;
    // my share of the slot's distinct indices (relative to ub)
    const uint32_t r0 = (uint32_t)((uint64_t)us * part / parts), r1 = (uint32_t)((uint64_t)us * (part + 1) / parts);
    const uint32_t mine = r1 - r0;
    if (mine == 0) return;
    uint32_t* const cur = mine <= lds_cap ? lcur : gcur + ub + r0;
    const uint32_t* const keys = u_of_gi + l0;
    for (uint32_t i = threadIdx.x; i < mine; i += PLACE_THREADS) cur[i] = 0;
    __syncthreads();
    // (eight lookups per thread at a time, their loads in flight together)
    uint32_t below = 0;  // lookups of the indices before my share
    for (uint32_t i0 = threadIdx.x; i0 < len; i0 += PLACE_THREADS * PLACE_ITEMS) {
        uint32_t k[PLACE_ITEMS];
#pragma unroll
        for (int j = 0; j < PLACE_ITEMS; j++) {
            const uint32_t i = i0 + j * PLACE_THREADS;
            k[j] = i < len ? (keys[i] & ~FIRST_BIT) - ub : 0xFFFFFFFFu;
        }
#pragma unroll
        for (int j = 0; j < PLACE_ITEMS; j++) {
            if (k[j] < r0)
                below++;
            else if (k[j] < r1)
                atomicAdd(&cur[k[j] - r0], 1u);
        }
    }
    {
        uint32_t total;
        block_excl_scan<uint32_t, PLACE_THREADS / 64>(below, red, &total);
        if (threadIdx.x == 0) carry_sh = l0 + total;  // the lookups of the slots before, and of the shares before, come first
    }
    __syncthreads();
    for (uint32_t i0 = 0; i0 < mine; i0 += PLACE_THREADS) {
        const uint32_t i = i0 + threadIdx.x;
        const uint32_t cnt = i < mine ? ld_relaxed(cur + i) : 0u;  // (counted by atomics: not through the L1 cache)
        uint32_t total;
        const uint32_t at = carry_sh + block_excl_scan<uint32_t, PLACE_THREADS / 64>(cnt, red, &total);
        if (i < mine) {
            cur[i] = at;
            seg_off[ub + r0 + i] = at;
            if (cnt >= ORDER_HUGE)
                huge_list[atomicAdd(&counts[2], 1u)] = ub + r0 + i;
            else if (cnt >= ORDER_MID)
                mid_list[atomicAdd(&counts[1], 1u)] = ub + r0 + i;
        }
        __syncthreads();
        if (threadIdx.x == 0) carry_sh += total;
        __syncthreads();
    }
    for (uint32_t i0 = threadIdx.x; i0 < len; i0 += PLACE_THREADS * PLACE_ITEMS) {
        uint32_t k[PLACE_ITEMS];
        uint64_t v[PLACE_ITEMS];
#pragma unroll
        for (int j = 0; j < PLACE_ITEMS; j++) {
            const uint32_t i = i0 + j * PLACE_THREADS;
            k[j] = i < len ? (keys[i] & ~FIRST_BIT) - ub : 0xFFFFFFFFu;
            v[j] = (k[j] >= r0 && k[j] < r1) ? vals[l0 + i] : 0ull;
        }
#pragma unroll
        for (int j = 0; j < PLACE_ITEMS; j++) {
            if (k[j] < r0 || k[j] >= r1) continue;
            const uint32_t at = atomicAdd(&cur[k[j] - r0], 1u);
            tkey[at] = ub + k[j];
            tval[at] = v[j];
        }
    }
}

__global__ __launch_bounds__(256) void k_rank_short(uint32_t L, const uint32_t* __restrict__ tkey,
                                                    const uint64_t* __restrict__ tval,
                                                    const uint32_t* __restrict__ seg_off, uint64_t* __restrict__ svals,
                                                    const DevStatus* status) {
    if (status->abort) return;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t t = blockIdx.x * blockDim.x + threadIdx.x; t < L; t += stride) {
        const uint32_t u = tkey[t];
        const uint32_t lo = seg_off[u], hi = seg_off[u + 1];
        if (hi - lo >= ORDER_MID) continue;
        const uint64_t v = tval[t];
        uint32_t rank = 0;
        for (uint32_t j = lo; j < hi; j++) {
            const uint64_t o = tval[j];
            rank += (o < v || (o == v && j < t)) ? 1u : 0u;
        }
        svals[lo + rank] = v;
    }
}

__global__ __launch_bounds__(256) void k_rank_mid(const uint32_t* __restrict__ mid_list, const uint32_t* counts,
                                                  const uint32_t* __restrict__ seg_off,
                                                  const uint64_t* __restrict__ tval, uint64_t* __restrict__ svals,
                                                  const DevStatus* status) {
    __shared__ uint64_t seg[ORDER_HUGE];
    if (status->abort) return;
    const uint32_t n_mid = counts[1];
    for (uint32_t k = blockIdx.x; k < n_mid; k += gridDim.x) {
        const uint32_t u = mid_list[k];
        const uint32_t lo = seg_off[u], n = seg_off[u + 1] - lo;  // ORDER_MID <= n < ORDER_HUGE
        uint32_t p2 = ORDER_MID;
        while (p2 < n) p2 <<= 1;
        // bitonic sorting network over the segment padded with the largest value to a power of two
        for (uint32_t i = threadIdx.x; i < p2; i += 256) seg[i] = i < n ? tval[lo + i] : ~0ull;
        __syncthreads();
        for (uint32_t size = 2; size <= p2; size <<= 1) {
            for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
                for (uint32_t t = threadIdx.x; t < p2 / 2; t += 256) {
                    const uint32_t a = 2 * t - (t & (stride - 1));  // lower element of the t-th pair
                    const uint32_t b = a + stride;
                    const bool up = (a & size) == 0;
                    const uint64_t x = seg[a], y = seg[b];
                    if ((x > y) == up) {
                        seg[a] = y;
                        seg[b] = x;
                    }
                }
                __syncthreads();
            }
        }
        for (uint32_t i = threadIdx.x; i < n; i += 256) svals[lo + i] = seg[i];
        __syncthreads();
    }
}

// cnt: `batch` counters in LDS (in_lds) or in a part of gcnt of the workgroup's own.
__global__ __launch_bounds__(256) void k_order_huge(const uint32_t* __restrict__ huge_list, const uint32_t* counts,
                                                    const uint32_t* __restrict__ seg_off,
                                                    const uint64_t* __restrict__ tval, uint64_t* __restrict__ svals,
                                                    uint32_t batch, int in_lds, uint32_t* __restrict__ gcnt,
                                                    const DevStatus* status) {
    extern __shared__ uint32_t lcnt[];
    __shared__ uint32_t red[4];
    __shared__ uint32_t carry_sh;
    if (status->abort) return;
    uint32_t* const cnt = in_lds ? lcnt : gcnt + (size_t)blockIdx.x * batch;
    const uint32_t n_huge = counts[2];
    for (uint32_t k = blockIdx.x; k < n_huge; k += gridDim.x) {
        const uint32_t u = huge_list[k];
        const uint32_t lo = seg_off[u], hi = seg_off[u + 1];
        for (uint32_t i = threadIdx.x; i < batch; i += 256) cnt[i] = 0;
        if (threadIdx.x == 0) carry_sh = 0;
        __syncthreads();
        for (uint32_t j = lo + threadIdx.x; j < hi; j += 256) atomicAdd(&cnt[(uint32_t)(tval[j] >> 32)], 1u);
        __syncthreads();
        for (uint32_t i0 = 0; i0 < batch; i0 += 256) {
            const uint32_t i = i0 + threadIdx.x;
            const uint32_t c = i < batch ? ld_relaxed(cnt + i) : 0u;
            uint32_t total;
            const uint32_t at = carry_sh + block_excl_scan_256<uint32_t>(c, red, &total);
            if (i < batch) cnt[i] = at;
            __syncthreads();
            if (threadIdx.x == 0) carry_sh += total;
            __syncthreads();
        }
        for (uint32_t j = lo + threadIdx.x; j < hi; j += 256) {
            const uint64_t v = tval[j];
            svals[lo + atomicAdd(&cnt[(uint32_t)(v >> 32)], 1u)] = v;
        }
        __syncthreads();
    }
}

// The share of a lookup in the gradient of its distinct sign: its example's pooled row times
// 1 / d(lookups of the example), chunk c.
template <int VEC>
__device__ __forceinline__ void add_lookup_share(const float* __restrict__ pooled, uint64_t v, int dim, int c,
                                                 int combiner, float (&acc)[VEC]) {
    if (v == ~0ull) return;  // flagged by k_lookup_keys
    const uint32_t b = (uint32_t)(v >> 32);
    const float scale = combiner == COMBINE_SUM ? 1.f : 1.f / combine_divisor((uint32_t)v, combiner);
    const float* row = pooled + (uint64_t)b * dim + c * VEC;
    if (VEC == 4) {
        const float4 g = *reinterpret_cast<const float4*>(row);
        acc[0] += g.x * scale;
        acc[1] += g.y * scale;
        acc[2] += g.z * scale;
        acc[3] += g.w * scale;
    } else {
        acc[0] += row[0] * scale;
    }
}

// Step 3: one group of `chunks` threads per distinct index sums its lookups' shares of the
// pooled gradient rows, in position order.  A distinct index with long_min lookups or more (a
// frequent sign) is left out: k_place_lookups has listed those, one workgroup each sums them (k_reduce_long).
template <int VEC>
__global__ __launch_bounds__(256) void k_reduce_pooled(const SlotDesc* __restrict__ descs,
                                                       const uint32_t* __restrict__ ubase, int N, int dim,
                                                       int combiner, const DevStatus* status,
                                                       const uint32_t* __restrict__ seg_off,
                                                       const uint64_t* __restrict__ svals, float* __restrict__ flat,
                                                       uint32_t long_min) {
    if (status->abort) return;
    __shared__ uint32_t ub[MAX_SLOTS + 1];
    load_lbase(ub, ubase, N);
    const int chunks = dim / VEC;
    const int64_t total = (int64_t)status->n_unique * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const uint32_t u = (uint32_t)(t / chunks);
        const int c = (int)(t - (int64_t)u * chunks);
        const uint32_t lo = seg_off[u], hi = seg_off[u + 1];
        if (hi - lo >= long_min) continue;  // (listed by k_place_lookups: k_reduce_long sums those)
        float acc[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) acc[q] = 0.f;
        const float* pooled = descs[find_slot(ub, N, u)].grads;  // the slot whose window of distinct indices holds u
        for (uint32_t j0 = lo; j0 < hi; j0 += COMBINE_WINDOW) {  // values of a window first, then their rows
            uint64_t wv[COMBINE_WINDOW];
#pragma unroll
            for (int q = 0; q < COMBINE_WINDOW; q++) wv[q] = (j0 + q < hi) ? svals[j0 + q] : ~0ull;
#pragma unroll
            for (int q = 0; q < COMBINE_WINDOW; q++) add_lookup_share<VEC>(pooled, wv[q], dim, c, combiner, acc);
        }
        float* o = flat + (uint64_t)u * dim + c * VEC;
        if (VEC == 4)
            *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        else
            o[0] = acc[0];
    }
}

// One workgroup per frequent distinct index: its 256 / chunks thread groups each sum every
// (256 / chunks)-th lookup in position order, then the partial sums are added in group order.
// The order of the additions is fixed, so the result does not vary from run to run.
constexpr int LONG_PART_FLOATS = 1024;  // 256 threads x 4 floats

template <int VEC>
__global__ __launch_bounds__(256) void k_reduce_long(const SlotDesc* __restrict__ descs,
                                                     const uint32_t* __restrict__ ubase, int N, int dim, int combiner,
                                                     const uint32_t* __restrict__ seg_off,
                                                     const uint64_t* __restrict__ svals, float* __restrict__ flat,
                                                     const uint32_t* __restrict__ mid_list,
                                                     const uint32_t* __restrict__ huge_list,
                                                     const uint32_t* counts, const DevStatus* status) {
    if (status->abort) return;
    __shared__ float part[LONG_PART_FLOATS];
    const int chunks = dim / VEC;
    const int groups = 256 / chunks;
    const int q = threadIdx.x / chunks, c = threadIdx.x - q * chunks;
    // the frequent ones: the two lists k_place_lookups left (ORDER_MID lookups or more)
    const uint32_t n_mid = counts[1], n_long = n_mid + counts[2];
    for (uint32_t k = blockIdx.x; k < n_long; k += gridDim.x) {
        const uint32_t u = k < n_mid ? mid_list[k] : huge_list[k - n_mid];
        const uint32_t lo = seg_off[u], hi = seg_off[u + 1];
        const float* pooled = descs[find_slot(ubase, N, u)].grads;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[v] = 0.f;
        if (q < groups) {
            for (uint32_t j0 = lo + q; j0 < hi; j0 += COMBINE_WINDOW * groups) {  // values of a window first, then their rows
                uint64_t wv[COMBINE_WINDOW];
#pragma unroll
                for (int w = 0; w < COMBINE_WINDOW; w++) wv[w] = (j0 + w * groups < hi) ? svals[j0 + w * groups] : ~0ull;
#pragma unroll
                for (int w = 0; w < COMBINE_WINDOW; w++) add_lookup_share<VEC>(pooled, wv[w], dim, c, combiner, acc);
            }
        }
#pragma unroll
        for (int v = 0; v < VEC; v++) part[threadIdx.x * VEC + v] = acc[v];
        __syncthreads();
        if (q == 0) {
            float sum[VEC];
#pragma unroll
            for (int v = 0; v < VEC; v++) sum[v] = 0.f;
            for (int g = 0; g < groups; g++)
#pragma unroll
                for (int v = 0; v < VEC; v++) sum[v] += part[(g * chunks + c) * VEC + v];
            float* o = flat + (uint64_t)u * dim + c * VEC;
            if (VEC == 4)
                *reinterpret_cast<float4*>(o) = make_float4(sum[0], sum[1], sum[2], sum[3]);
            else
                o[0] = sum[0];
        }
        __syncthreads();
    }
}

}  // namespace tn

#endif  // TN_COMBINE_KERNELS_H_
