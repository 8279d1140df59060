// DenseTable: flat fp32 parameter array with Adam / AdaGrad state resident in HBM.
// Follows core/ps/table/dense_table.cc:37-101, DenseOptimizerKernel
// (core/ps/optimizer/optimizer_kernel.h:171-246), DenseAdamValue::Apply
// (adam_kernel.cc:46-55) and DenseAdaGradValue::Apply (ada_grad_kernel.cc:42-48).
//
// The update is a pure stream: per parameter it reads g,w,m,v and writes
// w,m,v (28 bytes) plus the 4-byte copy of w into the caller's variable, so it
// is bound by HBM bandwidth.  One thread handles one float4 of each array.
// The reference's 8 blocks all step together on a single worker, so their
// beta powers are identical and one pair is kept on the host.
//
// With shard_num > 1 the table is one worker's share: it holds the contiguous
// range [begin, end) of the concatenated parameters (ceil(total / shard_num)
// per shard), applies that slice of the gradients and writes that slice of
// the variables; the other ranges belong to other workers.
#include "tn_common.h"

#include <algorithm>
#include <cmath>

namespace tn {

namespace {

struct DenseTable {
    std::shared_ptr<OptConf> opt;
    int shard_num = 1, self_shard_id = 0;
    uint32_t handle = 0;
    int device = 0;
    bool initialized = false;
    int64_t total = 0;           // elements of the whole table (all shards)
    int64_t begin = 0, end = 0;  // this shard's range of it (dense_table.cc:46-66); arrays hold end - begin
    float* w = nullptr;
    float* s0 = nullptr;  // Adam m      / AdaGrad d2sum
    float* s1 = nullptr;  // Adam v      / AdaGrad g2sum
    float* s2 = nullptr;  //               AdaGrad m
    float beta1_power = 1.f, beta2_power = 1.f;  // adam_kernel.cc:27-28
    std::mutex mu;
};

std::mutex g_dense_mu;
std::vector<DenseTable*> g_dense_tables;

DenseTable* get_dense(uint32_t h) {
    std::lock_guard<std::mutex> lk(g_dense_mu);
    if (h >= g_dense_tables.size()) return nullptr;
    return g_dense_tables[h];
}

struct AdamArgs {
    float alpha, c1, c2, eps;
};
struct AdaGradArgs {
    float lr, gdr, c, eps;
};

__device__ __forceinline__ void adam_elem(float g, float& w, float& m, float& v, const AdamArgs& a) {
    m += (g - m) * a.c1;
    v += (g * g - v) * a.c2;
    w -= (m * a.alpha) / (sqrtf(v) + a.eps);
}

__device__ __forceinline__ void adagrad_elem(float g, float& w, float& d2, float& g2, float& m, const AdaGradArgs& a) {
    d2 = a.gdr * d2 + 1.0f;
    g2 = a.gdr * g2 + g * g;
    m += (g - m) * a.c;
    w -= a.lr * m / (sqrtf(g2) / sqrtf(d2) + a.eps);
}

// n4 float4 groups starting at the (16-byte aligned) pointers.
__global__ __launch_bounds__(256) void k_dense_adam_v4(const float4* __restrict__ g, float4* __restrict__ w,
                                                       float4* __restrict__ m, float4* __restrict__ v,
                                                       float4* __restrict__ out, int64_t n4, AdamArgs a) {
    // every element is read once and written once per step: the accesses are marked non-temporal
    // so that the stream does not displace the caches' contents
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        float4 gg = stream_load(&g[i]);
        float4 ww = stream_load(&w[i]), mm = stream_load(&m[i]), vv = stream_load(&v[i]);
        adam_elem(gg.x, ww.x, mm.x, vv.x, a);
        adam_elem(gg.y, ww.y, mm.y, vv.y, a);
        adam_elem(gg.z, ww.z, mm.z, vv.z, a);
        adam_elem(gg.w, ww.w, mm.w, vv.w, a);
        stream_store(&w[i], ww);
        stream_store(&m[i], mm);
        stream_store(&v[i], vv);
        if (out) stream_store(&out[i], ww);
    }
}

__global__ __launch_bounds__(256) void k_dense_adam_s(const float* __restrict__ g, float* __restrict__ w,
                                                      float* __restrict__ m, float* __restrict__ v,
                                                      float* __restrict__ out, int64_t n, AdamArgs a) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float ww = w[i], mm = m[i], vv = v[i];
        adam_elem(g[i], ww, mm, vv, a);
        w[i] = ww;
        m[i] = mm;
        v[i] = vv;
        if (out) out[i] = ww;
    }
}

// The same for AdaGrad (ada_grad_kernel.cc:25-48): five arrays in, four (five with the variable) out.
__global__ __launch_bounds__(256) void k_dense_adagrad_v4(const float4* __restrict__ g, float4* __restrict__ w,
                                                          float4* __restrict__ d2, float4* __restrict__ g2,
                                                          float4* __restrict__ m, float4* __restrict__ out, int64_t n4,
                                                          AdaGradArgs a) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        float4 gg = stream_load(&g[i]);
        float4 ww = stream_load(&w[i]), dd = stream_load(&d2[i]), ss = stream_load(&g2[i]), mm = stream_load(&m[i]);
        adagrad_elem(gg.x, ww.x, dd.x, ss.x, mm.x, a);
        adagrad_elem(gg.y, ww.y, dd.y, ss.y, mm.y, a);
        adagrad_elem(gg.z, ww.z, dd.z, ss.z, mm.z, a);
        adagrad_elem(gg.w, ww.w, dd.w, ss.w, mm.w, a);
        stream_store(&w[i], ww);
        stream_store(&d2[i], dd);
        stream_store(&g2[i], ss);
        stream_store(&m[i], mm);
        if (out) stream_store(&out[i], ww);
    }
}

__global__ __launch_bounds__(256) void k_dense_adagrad_s(const float* __restrict__ g, float* __restrict__ w,
                                                         float* __restrict__ d2, float* __restrict__ g2,
                                                         float* __restrict__ m, float* __restrict__ out, int64_t n,
                                                         AdaGradArgs a) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float ww = w[i], dd = d2[i], gg2 = g2[i], mm = m[i];
        adagrad_elem(g[i], ww, dd, gg2, mm, a);
        w[i] = ww;
        d2[i] = dd;
        g2[i] = gg2;
        m[i] = mm;
        if (out) out[i] = ww;
    }
}

__global__ __launch_bounds__(256) void k_fill_f32(float* p, int64_t n, float val) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = val;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

int launch_grid(int64_t work_items, int threads, int max_blocks) {
    int64_t b = (work_items + threads - 1) / threads;
    if (b < 1) b = 1;
    if (b > max_blocks) b = max_blocks;
    return (int)b;
}

int dense_meta(uint32_t handle, DenseMeta& m) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad dense table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    m.kind = t->opt->kind;
    m.shard_num = t->shard_num;
    m.self_shard_id = t->self_shard_id;
    m.initialized = t->initialized;
    m.total = t->total;
    m.length = t->end - t->begin;
    m.beta1_power = t->beta1_power;
    m.beta2_power = t->beta2_power;
    return TN_OK;
}

int dense_set_powers(uint32_t handle, float beta1_power, float beta2_power) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad dense table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    t->beta1_power = beta1_power;
    t->beta2_power = beta2_power;
    return TN_OK;
}

int dense_copy_range(uint32_t handle, int64_t off, int64_t n, float* const arr[4], bool to_host) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad dense table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "dense table not initialised");
    if (off < 0 || n < 0 || off + n > t->end - t->begin) return fail(TN_ERR_INVALID_ARGUMENT, "dense table range out of bounds");
    float* dev[4] = {t->w, t->s0, t->s1, t->s2};
    for (int a = 0; a < 4; a++) {
        if (!dev[a] || !arr[a] || n == 0) continue;
        if (to_host)
            TN_HIP(hipMemcpy(arr[a], dev[a] + off, (size_t)n * sizeof(float), hipMemcpyDeviceToHost));
        else
            TN_HIP(hipMemcpy(dev[a] + off, arr[a], (size_t)n * sizeof(float), hipMemcpyHostToDevice));
    }
    return TN_OK;
}

}  // namespace tn

using namespace tn;

extern "C" {

int tn_dense_table_create(tn_opt_t opt, int shard_num, int self_shard_id, uint32_t* handle) {
    if (!handle) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_create: handle is NULL");
    auto conf = get_opt(opt);
    if (!conf) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_create: unknown optimizer handle");
    if (conf->kind == OPT_FTRL)
        return fail(TN_ERR_UNSUPPORTED, "tn_dense_table_create: dense Ftrl is an empty stub in the reference");
    if (shard_num < 1 || self_shard_id < 0 || self_shard_id >= shard_num)
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_create: shard " + std::to_string(self_shard_id) + " of " +
                                                 std::to_string(shard_num));
    DenseTable* t = new DenseTable();
    t->opt = conf;
    t->shard_num = shard_num;
    t->self_shard_id = self_shard_id;
    if (hipGetDevice(&t->device) != hipSuccess) t->device = 0;
    std::lock_guard<std::mutex> lk(g_dense_mu);
    t->handle = (uint32_t)g_dense_tables.size();
    g_dense_tables.push_back(t);
    *handle = t->handle;
    return TN_OK;
}

static int dense_alloc(DenseTable* t, int64_t total, hipStream_t st) {
    if (t->initialized) {
        if (t->total != total)
            return fail(TN_ERR_ALREADY_INIT, "dense table already init with element size:" + std::to_string(t->total) +
                                                 " but " + std::to_string(total) + " expected");
        return TN_OK;
    }
    if (total <= 0) return fail(TN_ERR_INVALID_ARGUMENT, "dense table init: total elements must be positive");
    if (total > 0x7fffffffLL)
        return fail(TN_ERR_INVALID_ARGUMENT, "dense table init: total elements exceed int (dense_table.cc:37)");
    // DenseTable::Init, dense_table.cc:46-66: ceil(total / shards) elements per shard, the last
    // one shorter; a shard that starts past the end gets no kernel
    const int64_t every = (total + t->shard_num - 1) / t->shard_num;
    t->begin = std::min<int64_t>((int64_t)t->self_shard_id * every, total);
    t->end = std::min<int64_t>(t->begin + every, total);
    const int64_t len = t->end - t->begin;
    if (len > 0) {
        size_t bytes = (size_t)len * sizeof(float);
        TN_HIP(hipMalloc((void**)&t->w, bytes));
        TN_HIP(hipMalloc((void**)&t->s0, bytes));
        TN_HIP(hipMalloc((void**)&t->s1, bytes));
        int blocks = launch_grid(len, 256, 8192);
        TN_LAUNCH(k_fill_f32, dim3(blocks), dim3(256), st, t->w, len, 0.f);
        TN_LAUNCH(k_fill_f32, dim3(blocks), dim3(256), st, t->s0, len, 0.f);
        if (t->opt->kind == OPT_ADAGRAD) {
            TN_HIP(hipMalloc((void**)&t->s2, bytes));
            TN_LAUNCH(k_fill_f32, dim3(blocks), dim3(256), st, t->s1, len, t->opt->initial_g2sum);
            TN_LAUNCH(k_fill_f32, dim3(blocks), dim3(256), st, t->s2, len, 0.f);
        } else {
            TN_LAUNCH(k_fill_f32, dim3(blocks), dim3(256), st, t->s1, len, 0.f);
        }
    }
    TN_HIP(hipGetLastError());
    t->total = total;
    t->initialized = true;
    return TN_OK;
}

}  // extern "C"

int tn::dense_ensure_init(uint32_t handle, int64_t total) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad dense table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    TN_TRY(dense_alloc(t, total, nullptr));
    TN_HIP(hipStreamSynchronize(nullptr));
    return TN_OK;
}

extern "C" {

int tn_dense_table_init(uint32_t handle, int N, const float* const* vars, const int64_t* var_lens, void* stream) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_init: bad dense table handle " + std::to_string(handle));
    if (N <= 0 || !vars || !var_lens) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_init: no variables");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    int64_t total = 0;
    for (int i = 0; i < N; i++) {
        if (var_lens[i] < 0 || (var_lens[i] > 0 && !vars[i]))
            return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_init: bad variable " + std::to_string(i));
        total += var_lens[i];
    }
    TN_TRY(dense_alloc(t, total, st));
    int64_t off = 0;
    for (int i = 0; i < N; i++) {
        const int64_t lo = std::max(off, t->begin), hi = std::min(off + var_lens[i], t->end);
        if (lo < hi)
            TN_HIP(hipMemcpyAsync(t->w + (lo - t->begin), vars[i] + (lo - off), (size_t)(hi - lo) * sizeof(float),
                                  hipMemcpyDeviceToDevice, st));
        off += var_lens[i];
    }
    TN_HIP(hipStreamSynchronize(st));
    return TN_OK;
}

int tn_dense_table_push_pull(uint32_t handle, int N, float* const* vars, const float* const* grads,
                             const int64_t* lens, float learning_rate, void* stream) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_push_pull: bad dense table handle " + std::to_string(handle));
    if (N <= 0 || !grads || !lens) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_push_pull: no gradients");
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "tn_dense_table_push_pull: dense table not initialised");
    int64_t total = 0;
    for (int i = 0; i < N; i++) {
        if (lens[i] < 0 || (lens[i] > 0 && !grads[i]))
            return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_push_pull: bad gradient " + std::to_string(i));
        total += lens[i];
    }
    // CHECK_EQ(total_elements, table->TotalElements()), dense_table_ops.cc:179
    if (total != t->total)
        return fail(TN_ERR_DIM_MISMATCH, "tn_dense_table_push_pull: gradients hold " + std::to_string(total) +
                                             " elements, table " + std::to_string(t->total));
    hipStream_t st = (hipStream_t)stream;
    const OptConf& o = *t->opt;
    AdamArgs aa{};
    AdaGradArgs ga{};
    if (o.kind == OPT_ADAM) {
        // adam_kernel.cc:47-50: float powers, alpha evaluated in double then narrowed
        t->beta1_power *= o.beta1;
        t->beta2_power *= o.beta2;
        aa.alpha = (float)((double)learning_rate * std::sqrt(1.0 - (double)t->beta2_power) /
                           (1.0 - (double)t->beta1_power));
        aa.c1 = (float)(1.0 - (double)o.beta1);
        aa.c2 = (float)(1.0 - (double)o.beta2);
        aa.eps = o.epsilon;
    } else {
        ga.lr = learning_rate;
        ga.gdr = o.grad_decay_rate;
        ga.c = (float)(1.0 - (double)o.mom_decay_rate);
        ga.eps = o.epsilon;
    }
    int64_t var_off = 0;
    for (int i = 0; i < N; i++) {
        // the part of variable i inside this shard's range
        const int64_t lo = std::max(var_off, t->begin), hi = std::min(var_off + lens[i], t->end);
        const int64_t skip = lo - var_off;
        var_off += lens[i];
        if (lo >= hi) continue;
        const int64_t n = hi - lo, off = lo - t->begin;
        float* out = (vars && vars[i]) ? vars[i] + skip : nullptr;
        const float* g = grads[i] + skip;
        if (o.kind == OPT_ADAM) {
            bool vec = (off % 4 == 0) && aligned16(g) && (!out || aligned16(out));
            int64_t n4 = vec ? n / 4 : 0;
            if (n4 > 0) {
                int blocks = launch_grid(n4, 256, 1 << 20);
                TN_LAUNCH(k_dense_adam_v4, dim3(blocks), dim3(256), st, (const float4*)g, (float4*)(t->w + off), (float4*)(t->s0 + off), (float4*)(t->s1 + off), (float4*)out, n4, aa);
            }
            int64_t done = n4 * 4;
            if (done < n) {
                int blocks = launch_grid(n - done, 256, 1 << 20);
                TN_LAUNCH(k_dense_adam_s, dim3(blocks), dim3(256), st, g + done, t->w + off + done, t->s0 + off + done, t->s1 + off + done, out ? out + done : nullptr, n - done, aa);
            }
        } else {
            bool vec = (off % 4 == 0) && aligned16(g) && (!out || aligned16(out));
            int64_t n4 = vec ? n / 4 : 0;
            if (n4 > 0) {
                int blocks = launch_grid(n4, 256, 1 << 20);
                TN_LAUNCH(k_dense_adagrad_v4, dim3(blocks), dim3(256), st, (const float4*)g, (float4*)(t->w + off), (float4*)(t->s0 + off), (float4*)(t->s1 + off), (float4*)(t->s2 + off), (float4*)out, n4, ga);
            }
            int64_t done = n4 * 4;
            if (done < n) {
                int blocks = launch_grid(n - done, 256, 1 << 20);
                TN_LAUNCH(k_dense_adagrad_s, dim3(blocks), dim3(256), st, g + done, t->w + off + done, t->s0 + off + done, t->s1 + off + done, t->s2 + off + done, out ? out + done : nullptr, n - done, ga);
            }
        }
    }
    TN_HIP(hipGetLastError());
    return TN_OK;
}

int tn_dense_table_total_elements(uint32_t handle, int64_t* total) {
    DenseTable* t = get_dense(handle);
    if (!t || !total) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_total_elements: bad handle");
    *total = t->total;
    return TN_OK;
}

int tn_dense_table_range(uint32_t handle, int64_t* begin, int64_t* end) {
    DenseTable* t = get_dense(handle);
    if (!t || !begin || !end) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_range: bad handle");
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "tn_dense_table_range: dense table not initialised");
    *begin = t->begin;
    *end = t->end;
    return TN_OK;
}

int tn_dense_table_get_weight(uint32_t handle, float* w, void* stream) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_get_weight: bad handle");
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "tn_dense_table_get_weight: dense table not initialised");
    if (t->end > t->begin)
        TN_HIP(hipMemcpyAsync(w, t->w, (size_t)(t->end - t->begin) * sizeof(float), hipMemcpyDeviceToDevice,
                              (hipStream_t)stream));
    return TN_OK;
}

int tn_dense_table_set_weight(uint32_t handle, const float* w, void* stream) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_set_weight: bad handle");
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "tn_dense_table_set_weight: dense table not initialised");
    if (t->end > t->begin)
        TN_HIP(hipMemcpyAsync(t->w, w, (size_t)(t->end - t->begin) * sizeof(float), hipMemcpyDeviceToDevice,
                              (hipStream_t)stream));
    return TN_OK;
}

int tn_dense_table_get_state(uint32_t handle, float* s0, float* s1, float* s2, void* stream) {
    DenseTable* t = get_dense(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_dense_table_get_state: bad handle");
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->initialized) return fail(TN_ERR_NOT_INIT, "tn_dense_table_get_state: dense table not initialised");
    size_t bytes = (size_t)(t->end - t->begin) * sizeof(float);
    hipStream_t st = (hipStream_t)stream;
    if (bytes == 0) return TN_OK;
    if (s0) TN_HIP(hipMemcpyAsync(s0, t->s0, bytes, hipMemcpyDeviceToDevice, st));
    if (s1) TN_HIP(hipMemcpyAsync(s1, t->s1, bytes, hipMemcpyDeviceToDevice, st));
    if (s2 && t->s2) TN_HIP(hipMemcpyAsync(s2, t->s2, bytes, hipMemcpyDeviceToDevice, st));
    return TN_OK;
}

}  // extern "C"
