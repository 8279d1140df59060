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
// gets the lookups of every distinct sign side by side from a stable sort of
// (distinct index, position) pairs.
#ifndef TN_COMBINE_KERNELS_H_
#define TN_COMBINE_KERNELS_H_

#include "sparse_kernels.h"

namespace tn {

enum { COMBINE_SUM = 0, COMBINE_MEAN = 1, COMBINE_SQRTN = 2 };

// In these kernels a SlotDesc carries: values = mapped ids (forward) / signs (backward),
// mapped = example index of every lookup, grads = rows to read (variable / pooled gradient),
// var = rows to write (forward: out[batch, dim]), rows = rows of `grads`, len = lookups.
__device__ __forceinline__ const int64_t* example_of(const SlotDesc& d) { return d.mapped; }

__device__ __forceinline__ float combine_divisor(uint32_t n, int combiner) {
    if (combiner == COMBINE_SUM || n == 0) return 1.f;
    return combiner == COMBINE_MEAN ? (float)n : sqrtf((float)n);
}

// One group of `chunks` threads per lookup; the group of the first lookup of an example
// sums the example's rows, divides, writes the output row, and clears the rows of the
// examples without lookups before it (after it, for the slot's last example).
template <int VEC>
__global__ __launch_bounds__(256) void k_combine_fwd(const SlotDesc* __restrict__ descs,
                                                     const uint32_t* __restrict__ lbase, int N, uint32_t L, int dim,
                                                     int64_t batch, int combiner, DevStatus* status) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const int chunks = dim / VEC;
    const int64_t total = (int64_t)L * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const uint32_t gi = (uint32_t)(t / chunks);
        const int c = (int)(t - (int64_t)gi * chunks);
        const int sl = find_slot(lb, N, gi);
        const SlotDesc& d = descs[sl];
        const int64_t* ex = example_of(d);
        const uint32_t i = gi - lb[sl];
        const int64_t b = ex[i];
        const int64_t prev = i > 0 ? ex[i - 1] : -1;
        if (b < 0 || b >= batch || prev > b) {
            if (c == 0) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
            continue;
        }
        if (prev == b) continue;  // not the first lookup of its example
        float acc[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) acc[q] = 0.f;
        uint32_t j = i;
        for (; j < d.len && ex[j] == b; j++) {
            const int64_t id = d.values[j];
            if (id < 0 || id >= d.rows) {
                if (c == 0) atomicOr(&status->err, DEV_ERR_VAR_CAPACITY);
                continue;
            }
            const float* row = d.grads + id * dim + c * VEC;
            if (VEC == 4) {
                const float4 v = *reinterpret_cast<const float4*>(row);
                acc[0] += v.x;
                acc[1] += v.y;
                acc[2] += v.z;
                acc[3] += v.w;
            } else {
                acc[0] += row[0];
            }
        }
        const float div = combine_divisor(j - i, combiner);
        float* out = d.var;
        auto put = [&](int64_t r, const float* v) {
            float* o = out + r * dim + c * VEC;
            if (VEC == 4)
                *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
            else
                o[0] = v[0];
        };
        float zero[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) {
            zero[q] = 0.f;
            acc[q] = acc[q] / div;
        }
        put(b, acc);
        for (int64_t r = prev + 1; r < b; r++) put(r, zero);
        if (j == d.len)
            for (int64_t r = b + 1; r < batch; r++) put(r, zero);
    }
}

// out[0 .. n) = 0 (a slot without lookups)
__global__ __launch_bounds__(256) void k_zero_f32(float* __restrict__ out, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = 0.f;
}

// Backward, step 1: sort keys (distinct index of every lookup) and values (its position);
// with a mean / sqrtn combiner also the number of lookups of the lookup's example.
__global__ __launch_bounds__(256) void k_lookup_keys(const SlotDesc* __restrict__ descs,
                                                     const uint32_t* __restrict__ lbase, int N, uint32_t L,
                                                     const uint32_t* __restrict__ u_of_gi, int64_t batch, int combiner,
                                                     uint32_t* __restrict__ keys, uint32_t* __restrict__ vals,
                                                     uint32_t* __restrict__ nlook, DevStatus* status) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t gi = blockIdx.x * blockDim.x + threadIdx.x; gi < L; gi += stride) {
        keys[gi] = u_of_gi[gi] & ~FIRST_BIT;
        vals[gi] = gi;
        const int sl = find_slot(lb, N, gi);
        const SlotDesc& d = descs[sl];
        const int64_t* ex = example_of(d);
        const uint32_t i = gi - lb[sl];
        const int64_t b = ex[i];
        const int64_t prev = i > 0 ? ex[i - 1] : -1;
        if (b < 0 || b >= batch || prev > b) atomicOr(&status->err, DEV_ERR_GRAD_ROWS);
        if (combiner == COMBINE_SUM || prev == b) continue;
        uint32_t j = i;
        while (j < d.len && ex[j] == b) j++;
        for (uint32_t q = i; q < j; q++) nlook[lb[sl] + q] = j - i;  // the example's first lookup tells the others
    }
}

// Step 2 (after the sort): where the lookups of every distinct index start.
__global__ __launch_bounds__(256) void k_segment_starts(const uint32_t* __restrict__ skeys, uint32_t L,
                                                        const DevStatus* status, uint32_t* __restrict__ seg_off) {
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < L; i += stride) {
        const uint32_t k = skeys[i];
        if (i == 0 || skeys[i - 1] != k) seg_off[k] = i;
        if (i == L - 1) seg_off[status->n_unique] = L;
    }
}

// Step 3: one group of `chunks` threads per distinct index sums its lookups' share of the
// pooled gradient rows, in position order.
template <int VEC>
__global__ __launch_bounds__(256) void k_reduce_pooled(const SlotDesc* __restrict__ descs,
                                                       const uint32_t* __restrict__ lbase, int N, int dim,
                                                       int64_t batch, int combiner, const DevStatus* status,
                                                       const uint32_t* __restrict__ seg_off,
                                                       const uint32_t* __restrict__ svals,
                                                       const uint32_t* __restrict__ nlook, float* __restrict__ flat) {
    __shared__ uint32_t lb[MAX_SLOTS + 1];
    load_lbase(lb, lbase, N);
    const int chunks = dim / VEC;
    const int64_t total = (int64_t)status->n_unique * chunks;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        const uint32_t u = (uint32_t)(t / chunks);
        const int c = (int)(t - (int64_t)u * chunks);
        const uint32_t lo = seg_off[u], hi = seg_off[u + 1];
        float acc[VEC];
#pragma unroll
        for (int q = 0; q < VEC; q++) acc[q] = 0.f;
        if (lo < hi) {
            const int sl = find_slot(lb, N, svals[lo]);  // all lookups of a distinct index lie in one slot
            const SlotDesc& d = descs[sl];
            const int64_t* ex = example_of(d);
            for (uint32_t j = lo; j < hi; j++) {
                const uint32_t gi = svals[j];
                const int64_t b = ex[gi - lb[sl]];
                if (b < 0 || b >= batch) continue;  // flagged by k_lookup_keys
                const float scale = combiner == COMBINE_SUM ? 1.f : 1.f / combine_divisor(nlook[gi], combiner);
                const float* row = d.grads + b * dim + c * VEC;
                if (VEC == 4) {
                    const float4 v = *reinterpret_cast<const float4*>(row);
                    acc[0] += v.x * scale;
                    acc[1] += v.y * scale;
                    acc[2] += v.z * scale;
                    acc[3] += v.w * scale;
                } else {
                    acc[0] += row[0] * scale;
                }
            }
        }
        float* o = flat + (uint64_t)u * dim + c * VEC;
        if (VEC == 4)
            *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        else
            o[0] = acc[0];
    }
}

}  // namespace tn

#endif  // TN_COMBINE_KERNELS_H_
