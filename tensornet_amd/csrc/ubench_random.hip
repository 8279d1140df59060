// Random-access ceilings of the device for the access patterns of the sparse table:
// a stand-alone program (no library code) that times, on a table-sized allocation,
//
//   read64    64 bytes of a random 128-byte-pitch row, 4 lanes per row
//   gather    the same rows in random order, each copied to the next 64 bytes of
//             a dense array                                                   (k_gather_vars)
//   rmw80     64 + 16 bytes of a random row read, updated and written back     (an update)
//   apply     the same through an index array, with a 64-byte gradient row
//             gathered from a second array                                     (k_apply_single)
//   probe_*   one random key lookup: an unaligned window of 4 keys read with 4
//             loads, an aligned 64-byte group of 8 keys per thread, and the
//             same group read by 8 lanes                                       (k_probe)
//
// Every pattern issues independent accesses from full occupancy, so the rates are what the
// memory system delivers for that pattern, not what a dependent chain allows.  The kernels of
// the library are compared with these rates next to the 8 TB/s streaming peak.
//
//   ubench_random [table GiB, default 64]      prints one line per pattern and a JSON line
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>

#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));           \
            return 1;                                                              \
        }                                                                          \
    } while (0)

namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}

constexpr int ROW_FLOATS = 32;  // 128-byte pitch: 16 weights, 4 state words, padding

// i-th row of a batch: ascending through the table in windows, as the groups of a plan are
__device__ __forceinline__ uint64_t row_of(uint64_t i, uint64_t n, uint64_t rows) {
    const uint64_t window = rows / n;
    return i * window + __umul64hi(mix64(i + 1), window);
}

template <bool WRITE>
__global__ __launch_bounds__(256) void k_rows(float* tab, uint64_t rows, uint64_t n, float* sink) {
    const int sub = threadIdx.x & 3;
    const uint64_t stride = (uint64_t)gridDim.x * 64;
    float acc = 0.f;
    for (uint64_t i = (uint64_t)blockIdx.x * 64 + (threadIdx.x >> 2); i < n; i += stride) {
        float* p = tab + row_of(i, n, rows) * ROW_FLOATS;
        float4 v = reinterpret_cast<float4*>(p)[sub];
        if (WRITE) {
            float4 h = reinterpret_cast<float4*>(p + 16)[0];
            v.x += h.x;
            v.y += 1.f;
            reinterpret_cast<float4*>(p)[sub] = v;
            if (sub == 0) {
                h.x += 1.f;
                reinterpret_cast<float4*>(p + 16)[0] = h;
            }
        } else {
            acc += v.x + v.y + v.z + v.w;
        }
    }
    if (acc == 1.2345f) sink[0] = acc;
}

// rows in random order (the order of the distinct indices of a batch), dense output
__global__ __launch_bounds__(256) void k_gather(const float* __restrict__ tab, uint64_t rows, uint64_t n,
                                                float* __restrict__ dense) {
    const int sub = threadIdx.x & 3;
    const uint64_t stride = (uint64_t)gridDim.x * 64;
    for (uint64_t i = (uint64_t)blockIdx.x * 64 + (threadIdx.x >> 2); i < n; i += stride) {
        const uint64_t r = __umul64hi(mix64(i + 1), rows);
        reinterpret_cast<float4*>(dense + i * 16)[sub] = reinterpret_cast<const float4*>(tab + r * ROW_FLOATS)[sub];
    }
}

__global__ void k_fill_index(uint32_t* rows_idx, uint32_t* grad_idx, uint64_t n, uint64_t rows) {
    for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
        rows_idx[i] = (uint32_t)row_of(i, n, rows);
        grad_idx[i] = (uint32_t)__umul64hi(mix64(i + 77), 2 * n);
    }
}

__global__ __launch_bounds__(256) void k_apply(float* tab, const uint32_t* __restrict__ rows_idx,
                                               const uint32_t* __restrict__ grad_idx, const float* __restrict__ grads,
                                               uint32_t n) {
    const int sub = threadIdx.x & 3;
    const uint32_t stride = gridDim.x * 64;
    for (uint32_t g = blockIdx.x * 64 + (threadIdx.x >> 2); g < n; g += stride) {
        float* p = tab + (uint64_t)rows_idx[g] * ROW_FLOATS;
        const float4 gr = reinterpret_cast<const float4*>(grads + (uint64_t)grad_idx[g] * 16)[sub];
        float4 v = reinterpret_cast<float4*>(p)[sub];
        float4 h = reinterpret_cast<float4*>(p + 16)[0];
        float sq = gr.x * gr.x + gr.y * gr.y + gr.z * gr.z + gr.w * gr.w;
        sq += __shfl_xor(sq, 1);
        sq += __shfl_xor(sq, 2);
        const float g2 = h.x + sq / 16.f, den = 1e-8f + sqrtf(g2);
        v.x -= 0.01f * gr.x / den;
        v.y -= 0.01f * gr.y / den;
        v.z -= 0.01f * gr.z / den;
        v.w -= 0.01f * gr.w / den;
        reinterpret_cast<float4*>(p)[sub] = v;
        if (sub == 0) {
            h.x = g2;
            h.y += 1.f;
            reinterpret_cast<float4*>(p + 16)[0] = h;
        }
    }
}

// MODE 0: 4 keys from the home slot on, 4 loads, wrapping; 1: aligned group of 8 keys, one thread;
// 2: aligned group of 8 keys, 8 lanes
template <int MODE>
__global__ __launch_bounds__(256) void k_probe(const uint64_t* __restrict__ keys, uint64_t cap, uint64_t n,
                                               uint32_t* __restrict__ out) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t threads = MODE == 2 ? n * 8 : n;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < threads; t += stride) {
        const uint64_t i = MODE == 2 ? t >> 3 : t;
        const uint64_t sign = mix64(i + 12345);
        uint64_t idx = row_of(i, n, cap);  // home slots ascend through the table, as those of a plan's groups do
        uint32_t found = 0xFFFFFFFFu;
        if (MODE == 0) {
            uint64_t k[4], at[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                at[j] = idx + j;
                if (at[j] >= cap) at[j] -= cap;
                k[j] = keys[at[j]];
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (k[j] == sign) found = (uint32_t)at[j];
        } else if (MODE == 1) {
            idx &= ~7ull;
            const ulonglong2* g = reinterpret_cast<const ulonglong2*>(keys + idx);
            const ulonglong2 q0 = g[0], q1 = g[1], q2 = g[2], q3 = g[3];
            const uint64_t k[8] = {q0.x, q0.y, q1.x, q1.y, q2.x, q2.y, q3.x, q3.y};
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (k[j] == sign) found = (uint32_t)idx + j;
        } else {
            idx = (idx & ~7ull) + (t & 7);
            const unsigned long long m = __ballot(keys[idx] == sign);
            const uint32_t hit = (uint32_t)((m >> (__lane_id() & ~7u)) & 0xFFu);
            if (hit) found = (uint32_t)(idx & ~7ull) + (uint32_t)__ffs(hit) - 1;
            if ((t & 7) != 0) continue;
        }
        out[i] = found;
    }
}

struct Timer {
    hipEvent_t a, b;
    Timer() {
        (void)hipEventCreate(&a);
        (void)hipEventCreate(&b);
    }
    template <typename F>
    float best_us(F launch) {
        float best = 1e30f;
        for (int rep = 0; rep < 4; rep++) {
            (void)hipEventRecord(a, 0);
            launch();
            (void)hipEventRecord(b, 0);
            (void)hipEventSynchronize(b);
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, a, b);
            if (ms < best) best = ms;
        }
        return best * 1e3f;
    }
};

}  // namespace

int main(int argc, char** argv) {
    const uint64_t gib = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 64;
    const uint64_t bytes = gib << 30, rows = bytes / (ROW_FLOATS * 4), cap = bytes / 16 / 8 * 8;  // keys: 1/16 of the rows' bytes
    float *tab, *grads, *sink;
    uint64_t* keys;
    uint32_t *rows_idx, *grad_idx, *out;
    const uint64_t n_max = 2000000;
    CK(hipMalloc(&tab, bytes));
    CK(hipMemset(tab, 0, bytes));
    CK(hipMalloc(&keys, cap * 8));
    CK(hipMemset(keys, 0xFF, cap * 8));
    CK(hipMalloc(&grads, 2 * n_max * 64));
    CK(hipMemset(grads, 0, 2 * n_max * 64));
    CK(hipMalloc(&rows_idx, n_max * 4));
    CK(hipMalloc(&grad_idx, n_max * 4));
    CK(hipMalloc(&out, n_max * 4));
    CK(hipMalloc(&sink, 64));
    Timer tm;
    std::string json = "{\"table_gib\": " + std::to_string(gib);
    auto report = [&](const char* name, uint64_t n, float us) {
        std::printf("%-18s n %8llu  %8.1f us  %6.2f G/s\n", name, (unsigned long long)n, us, n / us / 1e3);
        json += ", \"" + std::string(name) + "_" + std::to_string(n / 1000000) + "M_us\": " + std::to_string(us);
    };
    for (uint64_t n : {1000000ull, 2000000ull}) {
        const int cover = (int)((n + 63) / 64);
        report("read64", n, tm.best_us([&] { hipLaunchKernelGGL(k_rows<false>, dim3(cover), dim3(256), 0, 0, tab, rows, n, sink); }));
        report("gather", n, tm.best_us([&] { hipLaunchKernelGGL(k_gather, dim3(cover), dim3(256), 0, 0, tab, rows, n, grads); }));
        report("rmw80", n, tm.best_us([&] { hipLaunchKernelGGL(k_rows<true>, dim3(cover), dim3(256), 0, 0, tab, rows, n, sink); }));
        hipLaunchKernelGGL(k_fill_index, dim3(1024), dim3(256), 0, 0, rows_idx, grad_idx, n, rows);
        CK(hipDeviceSynchronize());
        report("apply", n, tm.best_us([&] { hipLaunchKernelGGL(k_apply, dim3(cover), dim3(256), 0, 0, tab, rows_idx, grad_idx, grads, (uint32_t)n); }));
        const int pb = (int)((n + 255) / 256);
        report("probe_unaligned4", n, tm.best_us([&] { hipLaunchKernelGGL(k_probe<0>, dim3(pb), dim3(256), 0, 0, keys, cap, n, out); }));
        report("probe_group8", n, tm.best_us([&] { hipLaunchKernelGGL(k_probe<1>, dim3(pb), dim3(256), 0, 0, keys, cap, n, out); }));
        report("probe_group8_lanes", n, tm.best_us([&] { hipLaunchKernelGGL(k_probe<2>, dim3(pb * 8), dim3(256), 0, 0, keys, cap, n, out); }));
    }
    CK(hipDeviceSynchronize());
    std::printf("%s}\n", json.c_str());
    return 0;
}
