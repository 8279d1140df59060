// Shared declarations of the HIP library behind include/tensornet_amd.h.
// gfx950 only: 64-wide wavefronts, no portability layers.
#ifndef TN_COMMON_H_
#define TN_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "tensornet_amd.h"

namespace tn {

// ------------------------------------------------------------------ errors
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);

#define TN_HIP(expr)                                                                               \
    do {                                                                                           \
        hipError_t _e = (expr);                                                                    \
        if (_e != hipSuccess) {                                                                    \
            return ::tn::fail(TN_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(_e));      \
        }                                                                                          \
    } while (0)

#define TN_TRY(expr)              \
    do {                          \
        int _rc = (expr);         \
        if (_rc != TN_OK) return _rc; \
    } while (0)

// -------------------------------------------------------------- optimizers
enum OptKind { OPT_ADAGRAD = 0, OPT_ADAM = 1, OPT_FTRL = 2 };

// All hyper-parameters are float, as in core/ps/optimizer/optimizer.h:36-144.
struct OptConf {
    int kind = OPT_ADAGRAD;
    float learning_rate = 0.01f;
    float show_decay_rate = 0.98f;
    int sparse_zero_init = 0;
    // AdaGrad
    float initial_g2sum = 0.f, initial_scale = 1.f, epsilon = 1e-8f;
    float grad_decay_rate = 1.f, mom_decay_rate = 1.f, show_threshold = 0.f;
    int no_show_days = 1000, elimination_logic = 0;
    // Adam
    float beta1 = 0.9f, beta2 = 0.999f;
    // Ftrl
    float beta = 1.f, lambda1 = 0.1f, lambda2 = 1.f;
};

// Snapshot of the optimizer passed by value to kernels.
struct OptDev {
    int kind;
    int zero_init;
    int use_cvm;
    float lr, eps, initial_g2sum, initial_scale;
    float beta1, beta2;           // Adam
    float beta, lambda1, lambda2; // Ftrl
};

std::shared_ptr<OptConf> get_opt(tn_opt_t h);

// ------------------------------------------------------------ device bits
constexpr uint64_t EMPTY_KEY = 0xFFFFFFFFFFFFFFFFull;
constexpr uint32_t NO_ROW = 0xFFFFFFFFu;

// status / error flags latched on the device by kernels
enum : uint32_t {
    DEV_ERR_VAR_CAPACITY = 1u,
    DEV_ERR_UNKNOWN_KEY = 2u,
    DEV_ERR_TABLE_FULL = 4u,
    DEV_ERR_GRAD_ROWS = 8u,
    DEV_ERR_REMAP_OVERFLOW = 16u,  // the LDS remap met a bucket it cannot hold: repeat on the global-table path
};

struct DevStatus {
    uint32_t err;        // DEV_ERR_* bits
    uint32_t n_unique;   // U = sum of per-slot distinct signs
    uint32_t n_single;   // distinct signs (groups) with one record: numbered 0 .. n_single-1
    uint32_t n_multi;    // groups with several records: numbered downwards from the top of the id space
    uint32_t n_new;      // rows inserted by this call
    uint32_t gcap;       // slots of the per-call group table
    uint32_t n_members;  // records in groups with several records (their lists fill the member array from the top)
    uint32_t mismatch;   // a push found other signs than the plan was built from
    uint32_t n_big;      // groups with many records (handled one wavefront each)
    uint32_t abort;      // the call's inputs are unusable (flagged in err): later kernels of the call do nothing
    uint32_t tile_share_q16;  // remap through LDS: records handed to the first-level buckets per lookup, largest share of a slot, in 1 / 65536
    uint32_t pad[1];
};

// The chip is eight dies, each with an L2 of its own, and the workgroups of a launch go to the dies in turn
// (workgroup i to die i % 8).  A kernel whose neighbouring work items touch the same memory gives every die a
// contiguous share of the items, taken up by the die's workgroups in launch order: neighbours then meet in one L2
// instead of eight.  `for (i = share.first; i < share.end; i += share.step)` in place of a grid-stride loop over
// n items; any grid covers every item once.
constexpr uint32_t XCDS = 8;
struct DieShare {
    uint32_t first, end, step;
    __device__ __forceinline__ explicit DieShare(uint32_t n) {
        const uint32_t dies = min(XCDS, (uint32_t)gridDim.x), die = blockIdx.x % dies, per_die = (n + dies - 1) / dies;
        first = min(n, die * per_die) + blockIdx.x / dies;
        end = min(n, (die + 1) * per_die);
        step = (gridDim.x - die + dies - 1) / dies;  // workgroups of the launch on this die
    }
};

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}

// maps a sign to [0, cap) without a division
__device__ __forceinline__ uint64_t slot_of(uint64_t sign, uint64_t cap) { return __umul64hi(mix64(sign), cap); }

__device__ __forceinline__ uint64_t ld_relaxed(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_relaxed(const uint32_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16-byte accesses marked non-temporal, for data that is read once or written once per call and
// should not displace what the caches hold.
typedef float native_float4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 stream_load(const float4* p) {
    const native_float4 v = __builtin_nontemporal_load(reinterpret_cast<const native_float4*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stream_store(float4* p, float4 v) {
    native_float4 n;
    n.x = v.x;
    n.y = v.y;
    n.z = v.z;
    n.w = v.w;
    __builtin_nontemporal_store(n, reinterpret_cast<native_float4*>(p));
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// grow-only device buffer
struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    int ensure(size_t need);
    void release();
};

int launch_grid(int64_t work_items, int threads, int max_blocks);

// Host-side access to a dense table for the checkpoint code (defined beside the table).
struct DenseMeta {
    int kind;  // OPT_ADAM / OPT_ADAGRAD
    int shard_num, self_shard_id;
    bool initialized;
    int64_t total;   // elements of the whole table
    int64_t length;  // elements of this shard's range
    float beta1_power, beta2_power;
};
int dense_meta(uint32_t handle, DenseMeta& m);
// DenseTable::Init(total): allocates on first use, a different size afterwards is an error.
int dense_ensure_init(uint32_t handle, int64_t total);
int dense_set_powers(uint32_t handle, float beta1_power, float beta2_power);
// Copies elements [off, off + n) of the shard's range between the table's arrays and host arrays: arr[0] = w,
// arr[1..3] = the optimizer's state arrays in the order its value prints them (Adam m, v;
// AdaGrad d2sum, g2sum, m); arrays the optimizer lacks are skipped.
int dense_copy_range(uint32_t handle, int64_t off, int64_t n, float* const arr[4], bool to_host);

// ---------------------------------------------------------------- profiling
// When enabled (tn_profile_enable) every kernel launch is bracketed by a pair
// of HIP events on the stream it is launched on; tn_profile_summary adds the
// elapsed times up per kernel name.
extern bool g_profile_on;
void prof_begin(const char* name, hipStream_t st);
void prof_end(hipStream_t st);

#define TN_LAUNCH_LDS(KERNEL, GRID, BLOCK, LDS_BYTES, STREAM, ...)              \
    do {                                                                       \
        if (::tn::g_profile_on) ::tn::prof_begin(#KERNEL, STREAM);             \
        hipLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS_BYTES, STREAM, __VA_ARGS__); \
        if (::tn::g_profile_on) ::tn::prof_end(STREAM);                        \
    } while (0)

#define TN_LAUNCH(KERNEL, GRID, BLOCK, STREAM, ...) TN_LAUNCH_LDS(KERNEL, GRID, BLOCK, 0, STREAM, __VA_ARGS__)

}  // namespace tn

#endif  // TN_COMMON_H_
