// SparseTable host side: registry, HBM storage management and the launch
// sequences of pull / push at table level (core/ps/table/sparse_table.cc:52-83)
// and at operator level (core/kernels/sparse_table_ops.cc:170-265,317-368).
#include "combine_kernels.h"
#include "remap_lds.h"
#include "small_batch.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstring>

// Device memory of tn_sparse_table_pull_static, the one entry point that allocates nothing: the call's
// status block, then the row number and the new-row list of every requested sign.  Every GPU the library
// runs on holds its own copy until the process ends; host code reaches it through the address that
// hipGetSymbolAddress returns for the current device (static_scratch below), never through this name.
constexpr int64_t TN_STATIC_MAX_SIGNS = 1 << 20;
constexpr size_t TN_STATIC_STATUS_BYTES = 256;
constexpr size_t TN_STATIC_SCRATCH_BYTES = TN_STATIC_STATUS_BYTES + 2 * (size_t)TN_STATIC_MAX_SIGNS * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[TN_STATIC_SCRATCH_BYTES];

namespace tn {

namespace {

constexpr double MAX_LOAD = 0.75;                       // optimizer_kernel.h:266
constexpr double RESERVE_LOAD = 0.5;                    // what a reservation is sized for where memory allows
constexpr uint64_t DEFAULT_SLOTS = 8ull * 15485863ull;  // optimizer_kernel.h:43,263
constexpr uint64_t MAX_SLOTS_PER_TABLE = 0xFFFFFFF0ull; // rows are addressed with 32 bits
constexpr int PROBE_RECS_GRID = 1024;  // workgroups of k_probe_recs (measured: 512-1024 are best)
// Below this many lookups a call keeps all its kernels on the caller's stream.  The kernels of a smaller
// batch are too short for the overlap on the side streams to win back what the events that fork and
// join them cost the host (measured: 106 k lookups 0.22 -> 0.17 ms per pull + push, 2.1 M 0.33 -> 0.31 ms,
// 5 M 0.67 -> 0.71 ms).
constexpr size_t ONE_STREAM_LOOKUPS = 3u << 20;
constexpr uint32_t SELF_SCAN_TILES = 8192;  // tiles of the ranking pass up to which no scan kernel runs between its launches
constexpr int GRID_CAP = 256 * 8;                       // 256 CUs x 8 workgroups of 256 threads
constexpr int TILE_GRID = 256 * 3;                      // workgroups of k_tile_dedup: what the chip holds of it at once
constexpr size_t LDS_MIN_LOOKUPS = 1024;  // from here on the remap through LDS wins: it also takes fewer launches (cfg1, 8 k lookups: 0.154 -> 0.136 ms)

// Up to this many lookups a batch whose slots each fit one workgroup (SMALL_SLOT_MAX lookups, SMALL_SLOTS slots)
// takes the path of few launches (small_batch.h).
constexpr size_t SMALL_MAX_LOOKUPS = 1u << 18;

// A small batch of at most this many slots leaves every sign to the lane groups of k_small_apply.  With more slots a
// sign with SMALL_BIG_GROUP records or more is taken by a wavefront of its own (the first workgroups of the same
// launch): a small batch's kernels are as long as their longest chain, and the records of a sign applied one after
// the other by a lane group (four elements per lane) take four times as long as by a wavefront with a lane per
// element (measured, 4096 x 26 slots, Adam: the updates take 0.040 ms with every sign left to the lane groups,
// 0.020 ms with the threshold at 5; 1024 x 8 slots: no difference between 4 and 12 slots here).
constexpr int SMALL_NO_BIG_SLOTS = 12;
constexpr uint32_t SMALL_BIG_GROUP = 5;
constexpr uint32_t BIG_GROUP_DEFAULT = 16;

enum { FLOW_NONE = 0, FLOW_PULL = 1, FLOW_PUSH = 2 };

struct HostStatus {
    DevStatus st;
    uint32_t ubase[MAX_SLOTS + 1];
};

struct SparseTable {
    std::shared_ptr<OptConf> opt;
    std::string name, group;
    int dim = 0, use_cvm = 0, shard_num = 1, self_shard_id = 0;
    uint32_t handle = 0;
    int device = 0;
    uint64_t seed = 0x243F6A8885A308D3ull;
    uint64_t reserve_keys = 0;
    bool allocated = false;
    Store store{};
    uint64_t count_upper = 0;  // upper bound of resident keys known without a device read
    uint64_t booked = 0;       // part of count_upper booked for the inserts of the pending call

    DevBuf ws;                      // per-call scratch
    DevBuf plan_buf;                // what the last pull op worked out about its batch (see Plan)
    bool plan_valid = false;
    bool plan_has_show = false;     // the plan already holds batch_show of every distinct sign
    int plan_N = 0;
    std::vector<int64_t> plan_lens;
    uint64_t epoch = 0;             // bumped whenever rows move (growth)
    uint64_t plan_epoch = 0;
    DevStatus* dstatus = nullptr;   // device: status of table-level calls
    DevStatus* dplan = nullptr;     // device: status / counts of the op-level plan
    DevStatus* dpush = nullptr;     // device: status of a push that reuses the plan (the plan's counts, flags of its own)
    HostStatus* hpull = nullptr;    // pinned
    HostStatus* hpush = nullptr;    // pinned
    unsigned long long* hcount = nullptr;  // pinned: the number of resident keys is read into it
    char* hstage = nullptr;         // pinned staging of slot descriptors
    size_t hstage_bytes = 0;
    hipEvent_t stage_ev = nullptr;  // staging buffer free again
    hipEvent_t verify_ev = nullptr; // a push's comparison of the signs has been published
    DevBuf comb_buf;                // slot descriptors of a combine op
    DevBuf pooled_ws;               // scratch of a push of pooled gradients (ordered lookups, reduced rows)
    size_t place_lds = 0, huge_lds = 0;  // dynamic LDS of k_place_lookups / k_order_huge on this device (0: not asked yet)
    // The path of few launches for small batches: its device state, the words in pinned memory its kernels
    // report through ([0] a pull's status is on the host, [1] a push's signs are compared) with the numbers the
    // host expects there next, the dynamic LDS k_small_slots may have.
    SmallState* small_state = nullptr;
    uint32_t* hseq = nullptr;
    uint32_t seq_pull = 0, seq_verify = 0;
    std::vector<int64_t> plan_counts;  // distinct signs per slot of the small pull that left the plan
    uint32_t small_calls = 0;  // (its parity: which set of bucket cursors the next small pull uses)
    size_t small_lds = 0;
    bool plan_small = false;   // the plan was left by a small pull: a push may take the small path, too
    bool plan_prints = false;  // the plan holds fingerprints of the batch's signs, not a copy of them
    bool exact_verify = false; // pulls that leave fingerprints keep a copy of the signs as well, pushes compare that
    bool plan_exact = false;   // the plan holds such a copy
    uint32_t plan_big_k = BIG_GROUP_DEFAULT;  // records from which the plan lists a sign as one for k_apply_big
    bool plan_big_desc = false;               // the plan's big_desc goes with its big_list (a pull grouped through LDS)
    hipStream_t side = nullptr;     // the signs with many records are applied here, beside the others
    hipStream_t side2 = nullptr;    // a pull probes the table here, beside the grouping of its distinct records
    // The slot descriptors of a call reach the device here while the caller's stream still runs the tail of the
    // call before (a pull's gather, a push's updates): the kernel reads pinned host memory, whose round trips
    // would otherwise stand at the head of every call.
    hipStream_t aux = nullptr;
    hipEvent_t fork_ev = nullptr, join_ev = nullptr, join2_ev = nullptr;
    hipEvent_t apply_ev = nullptr;  // a push's updates are done (its status is published beside what follows)
    // Detached updates (tn_sparse_table_set_detached_updates): the update kernels of a large push run on the
    // table's own streams and the caller's stream does not wait for them, so that whatever the caller queues next
    // -- above all the analysis of the next pull's batch, which touches no table row -- runs beside them.
    // upd_ev marks their end (and that of the push's status); every call on the table orders its stream behind
    // it before it touches a row, the plan's groups or the table's memory (order_after_updates).
    bool detach_updates = false;
    bool detached_now = false;      // the push being queued has its updates detached
    bool upd_pending = false;       // upd_ev has been recorded and no host-side wait has covered it since
    hipEvent_t upd_ev = nullptr;
    // what the detached kernels read of the plan buffer: the slot arrays at its head (laid out by the slot count)
    // and the groups from upd_groups_off on, less the first upd_slack bytes (the groups' signs, which they leave alone)
    int upd_N = 0;
    size_t upd_groups_off = 0, upd_slack = 0;
    // The call before this one on the table, if it left work behind on `flow_stream` that the next call of the
    // training loop may overlap with: FLOW_PULL = a pull that returned before its gather, FLOW_PUSH = a push
    // on that pull's plan.  Every entry point clears it (ensure_allocated); pull and push set it again.
    int flow = 0;
    hipStream_t flow_stream = nullptr;
    bool push_pub_on_side = false;  // the pending push's status is published on the side stream
    // A pull whose status is final before its last kernel (the gather) publishes it on the side stream
    // meanwhile and returns when it is there: ready_ev = the status can be published, pub_ev = it is on
    // the host, tail_ev = the gather is done (what a call on another stream has to wait for).
    hipEvent_t ready_ev = nullptr, pub_ev = nullptr, tail_ev = nullptr;
    bool tail_recorded = false;
    bool one_stream = false;        // the running call is small: its kernels all go to the caller's stream
    bool plan_clicks_dirty = false;  // a push has added clicks to the member lists of the current plan
    // Distinct records per lookup seen by the recent pulls (1 = every lookup distinct, the safe start):
    // sizes the number of second-level buckets, whose room is fixed.  A batch with more distinct
    // records than expected overflows a bucket and takes the fallback path once; the estimate is then reset.
    double distinct_est = 1.0;
    // Records a tile of the remap through LDS hands to the first-level buckets per lookup (1 = no sign repeats
    // inside a tile, the safe start), for the slot where that share is largest: sizes the first-level buckets,
    // whose room is fixed, with the same fallback as above.
    double tile_est = 1.0;
    uint64_t pull_lookups = 0;  // lookups of the pull whose status is pending
    bool stage_pending = false;
    bool push_pending = false;      // hpush holds an unchecked status
    bool pull_pending = false;
    int pull_slots = 0, push_slots = 0;  // N of the pending calls
    std::vector<int64_t> pending_rows;  // var rows of a pending async pull
    int async_pull = 0;
    bool small_path = true;         // small batches take the path of few launches (tn_sparse_table_set_small_batch_path)
    int latched = TN_OK;
    std::string latched_msg;
    std::vector<int64_t> last_counts;
    hipStream_t last_stream = nullptr;
    std::mutex mu;
};

std::mutex g_tables_mu;
std::vector<SparseTable*> g_tables;

SparseTable* get_table(uint32_t h) {
    std::lock_guard<std::mutex> lk(g_tables_mu);
    if (h >= g_tables.size()) return nullptr;
    return g_tables[h];
}

OptDev make_optdev(const SparseTable* t) {
    const OptConf& c = *t->opt;
    OptDev o{};
    o.kind = c.kind;
    o.zero_init = c.sparse_zero_init;
    o.use_cvm = t->use_cvm;
    o.lr = c.learning_rate;
    o.eps = c.epsilon;
    o.initial_g2sum = c.initial_g2sum;
    o.initial_scale = c.initial_scale;
    o.beta1 = c.beta1;
    o.beta2 = c.beta2;
    o.beta = c.beta;
    o.lambda1 = c.lambda1;
    o.lambda2 = c.lambda2;
    return o;
}

int round4(int x) { return (x + 3) & ~3; }
constexpr size_t LINE_BYTES = 128;  // L2 line: what a random access to the table moves

void layout(const SparseTable* t, Store& s) {
    s.D = t->dim;
    s.wdim = t->dim + (t->use_cvm ? 2 : 0);
    bool vec = (t->dim % 4) == 0;
    s.wlen = vec ? round4(s.wdim) : s.wdim;
    int sf = (t->opt->kind == OPT_ADAGRAD) ? 4 : 2 * t->dim + 2;
    s.slen = vec ? round4(sf) : sf;
    s.wstride = s.wlen;
    s.sstride = s.slen;
}

// Weights and state of a row share one 128-byte line (or a power-of-two part of one) when they fit and the table stays
// below half of the device memory that way (dim-16 AdaGrad: 136 instead of 88 bytes per slot);
// an update then touches one line of the table instead of two.
void choose_strides(Store& s, uint64_t cap) {
    if (s.wlen % 4 != 0 || (s.wlen + s.slen) * sizeof(float) > LINE_BYTES) return;
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return;
    size_t pitch = 32;  // a power of two, so that no row straddles a line
    while (pitch < (s.wlen + s.slen) * sizeof(float)) pitch *= 2;
    if ((cap + 1) * (pitch + sizeof(uint64_t)) > total_b / 2) return;
    s.wstride = s.sstride = (int)(pitch / sizeof(float));
}

bool interleaved(const Store& s) { return s.wstride != s.wlen; }

int state_floats(const SparseTable* t) { return (t->opt->kind == OPT_ADAGRAD) ? 4 : 2 * t->dim + 2; }

void free_store(Store& s);

int alloc_store(const SparseTable* t, uint64_t cap, Store& s, hipStream_t st) {
    layout(t, s);
    if (cap < 64) cap = 64;
    cap = (cap + PROBE_WIDTH - 1) / PROBE_WIDTH * PROBE_WIDTH;  // probing goes by aligned groups of slots
    if (cap > MAX_SLOTS_PER_TABLE) return fail(TN_ERR_UNSUPPORTED, "sparse table: more than 2^32 slots");
    s.cap = cap;
    choose_strides(s, cap);
    const size_t rows = (size_t)cap + 1;
    // whatever was allocated before a failure is released again: the caller keeps no half-built store
    auto oom = [&](const char* what, hipError_t e) {
        const std::string msg = std::string("hipMalloc ") + what + ": " + hipGetErrorString(e);
        free_store(s);
        return fail(TN_ERR_OUT_OF_MEMORY, msg);
    };
    hipError_t e;
    e = hipMalloc((void**)&s.keys, rows * sizeof(uint64_t) + 64);
    if (e != hipSuccess) return oom("keys", e);
    e = hipMalloc((void**)&s.w, rows * s.wstride * sizeof(float));
    if (e != hipSuccess) return oom("weights", e);
    if (interleaved(s)) {
        s.st = s.w + s.wlen;
    } else {
        e = hipMalloc((void**)&s.st, rows * s.sstride * sizeof(float));
        if (e != hipSuccess) return oom("state", e);
    }
    void* small = nullptr;
    e = hipMalloc(&small, 64);
    if (e != hipSuccess) return oom("counters", e);
    s.count = (unsigned long long*)small;
    s.special = (uint32_t*)((char*)small + 8);
    e = hipMemsetAsync(small, 0, 64, st);
    if (e == hipSuccess) e = hipMemsetAsync(s.keys, 0xFF, rows * sizeof(uint64_t), st);
    if (e != hipSuccess) {
        const std::string msg = std::string("hipMemsetAsync (new table): ") + hipGetErrorString(e);
        free_store(s);
        return fail(TN_ERR_HIP, msg);
    }
    return TN_OK;
}

void free_store(Store& s) {
    if (s.keys) (void)hipFree(s.keys);
    if (s.w) (void)hipFree(s.w);
    if (s.st && !interleaved(s)) (void)hipFree(s.st);
    if (s.count) (void)hipFree(s.count);
    s = Store{};
}

int ensure_side_buffers(SparseTable* t) {
    if (t->dstatus) return TN_OK;
    TN_HIP(hipMalloc((void**)&t->dstatus, 3 * sizeof(DevStatus)));
    TN_HIP(hipMemset(t->dstatus, 0, 3 * sizeof(DevStatus)));
    t->dplan = t->dstatus + 1;
    t->dpush = t->dstatus + 2;
    TN_HIP(hipHostMalloc((void**)&t->hpull, sizeof(HostStatus), hipHostMallocDefault));
    TN_HIP(hipHostMalloc((void**)&t->hpush, sizeof(HostStatus), hipHostMallocDefault));
    std::memset(t->hpull, 0, sizeof(HostStatus));
    std::memset(t->hpush, 0, sizeof(HostStatus));
    TN_HIP(hipHostMalloc((void**)&t->hcount, 64, hipHostMallocDefault));
    TN_HIP(hipHostMalloc((void**)&t->hseq, 64, hipHostMallocDefault));
    std::memset(t->hseq, 0, 64);
    TN_HIP(hipMalloc((void**)&t->small_state, sizeof(SmallState)));
    TN_HIP(hipMemset(t->small_state, 0, sizeof(SmallState)));
    t->hstage_bytes = (size_t)MAX_SLOTS * sizeof(SlotDesc) + (MAX_SLOTS + 1) * sizeof(uint32_t);
    TN_HIP(hipHostMalloc((void**)&t->hstage, t->hstage_bytes, hipHostMallocDefault));
    TN_HIP(hipEventCreateWithFlags(&t->stage_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->verify_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->fork_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->join_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->join2_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->ready_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->pub_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->tail_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->apply_ev, hipEventDisableTiming));
    TN_HIP(hipEventCreateWithFlags(&t->upd_ev, hipEventDisableTiming));
    TN_HIP(hipStreamCreateWithFlags(&t->side, hipStreamNonBlocking));  // default priority
    TN_HIP(hipStreamCreateWithFlags(&t->side2, hipStreamNonBlocking));
    TN_HIP(hipStreamCreateWithFlags(&t->aux, hipStreamNonBlocking));
    return TN_OK;
}

// Slots for a reservation of `keys` signs.  Growth starts at a load of 0.75 (optimizer_kernel.h:266); a reservation
// is sized for a load of 0.5 where that keeps the table (with its rows interleaved) below half of the device
// memory: probe chains are shorter there (cfg3: the probes of a pull take 0.078 instead of 0.096 ms).
uint64_t reserved_slots(const SparseTable* t, uint64_t keys) {
    const uint64_t tight = (uint64_t)((double)keys / MAX_LOAD) + 64;
    const uint64_t roomy = (uint64_t)((double)keys / RESERVE_LOAD) + 64;
    Store s{};
    layout(t, s);
    size_t pitch = 32;
    while (pitch < (s.wlen + s.slen) * sizeof(float)) pitch *= 2;
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return tight;
    return (roomy + 1) * (pitch + sizeof(uint64_t)) <= total_b / 2 ? roomy : tight;
}

// Orders `st` behind the detached updates of the last push, if any (a wait for an event that has completed
// costs nothing on the device).
int order_after_updates(SparseTable* t, hipStream_t st) {
    if (t->upd_pending) TN_HIP(hipStreamWaitEvent(st, t->upd_ev, 0));
    return TN_OK;
}

// A call on another stream than the table's last one: what that call left running there (a pull's gather, a small
// push's updates: tail_ev) is waited for on the device, and a call whose status is still pending on the host.
int order_after_other_stream(SparseTable* t, hipStream_t st) {
    if (!t->last_stream || t->last_stream == st) return TN_OK;
    if (t->tail_recorded) TN_HIP(hipStreamWaitEvent(st, t->tail_ev, 0));
    if (t->push_pending || t->pull_pending) TN_HIP(hipStreamSynchronize(t->last_stream));
    return TN_OK;
}

// beside_updates: the caller (the pull op) orders its stream behind detached updates itself, as late as it can.
int ensure_allocated(SparseTable* t, hipStream_t st, bool beside_updates = false) {
    TN_TRY(ensure_side_buffers(t));
    if (!beside_updates) TN_TRY(order_after_updates(t, st));
    TN_TRY(order_after_other_stream(t, st));
    t->flow = FLOW_NONE;  // pull and push read it before they get here and set it again
    if (t->allocated) return TN_OK;
    uint64_t cap = DEFAULT_SLOTS;
    if (t->reserve_keys) cap = reserved_slots(t, t->reserve_keys);
    TN_TRY(alloc_store(t, cap, t->store, st));
    t->allocated = true;
    t->count_upper = 0;
    return TN_OK;
}

const char* dev_err_text(uint32_t err) {
    if (err & DEV_ERR_TABLE_FULL) return "sparse table is full";
    if (err & DEV_ERR_UNKNOWN_KEY) return "embedding of a pushed sign not created yet (push before pull)";
    if (err & DEV_ERR_VAR_CAPACITY) return "distinct signs of a slot exceed the rows of its variable";
    if (err & DEV_ERR_GRAD_ROWS) return "gradient matrix of a slot has fewer rows than the slot has distinct signs";
    return "";
}

int dev_err_code(uint32_t err) {
    if (err & DEV_ERR_TABLE_FULL) return TN_ERR_TABLE_FULL;
    if (err & DEV_ERR_UNKNOWN_KEY) return TN_ERR_UNKNOWN_KEY;
    if (err & DEV_ERR_VAR_CAPACITY) return TN_ERR_VAR_CAPACITY;
    if (err & DEV_ERR_GRAD_ROWS) return TN_ERR_INVALID_ARGUMENT;
    return TN_OK;
}

void latch(SparseTable* t, int code, const std::string& msg) {
    if (code != TN_OK && t->latched == TN_OK) {
        t->latched = code;
        t->latched_msg = msg;
    }
}

// Examines the status blocks of finished calls (the stream must have been synchronised).
void harvest(SparseTable* t) {
    // a pending push is older than a pending pull (a push collects everything before it starts)
    if (t->push_pending) {
        t->push_pending = false;
        if (t->push_pub_on_side) {  // its status went out on the side stream, behind its updates
            t->push_pub_on_side = false;
            const hipError_t e = hipStreamSynchronize(t->side);
            if (e != hipSuccess) latch(t, TN_ERR_HIP, std::string("sparse push: ") + hipGetErrorString(e));
            t->upd_pending = false;  // (detached updates end on that stream, ahead of the status)
        }
        const HostStatus& h = *t->hpush;
        int N = t->push_slots;
        if (N > 0) {
            t->last_counts.assign(N, 0);
            for (int s = 0; s < N; s++) t->last_counts[s] = (int64_t)h.ubase[s + 1] - (int64_t)h.ubase[s];
        }
        latch(t, dev_err_code(h.st.err), std::string("sparse push: ") + dev_err_text(h.st.err));
    }
    if (t->pull_pending) {
        t->pull_pending = false;
        const HostStatus& h = *t->hpull;
        int N = t->pull_slots;
        // the call booked room for every sign it could have inserted; keep what it did insert
        if (t->booked >= h.st.n_new) t->count_upper -= t->booked - h.st.n_new;
        t->booked = 0;
        t->last_counts.assign(N, 0);
        for (int s = 0; s < N; s++) t->last_counts[s] = (int64_t)h.ubase[s + 1] - (int64_t)h.ubase[s];
        if (t->pull_lookups > 0) {  // rises at once, falls within about ten pulls
            const double now = (double)h.ubase[N] / (double)t->pull_lookups;
            t->distinct_est = std::min(1.0, std::max(now, 0.75 * t->distinct_est + 0.25 * now));
            if (h.st.tile_share_q16 != 0) {  // (a pull through LDS with a slot of more than one bucket)
                const double share = (double)h.st.tile_share_q16 / 65536.0;
                t->tile_est = std::min(1.0, std::max(share, 0.75 * t->tile_est + 0.25 * share));
            }
        }
        latch(t, dev_err_code(h.st.err), std::string("sparse pull: ") + dev_err_text(h.st.err));
        for (int s = 0; s < N && s < (int)t->pending_rows.size(); s++)
            if (t->last_counts[s] >= t->pending_rows[s])  // CHECK_LT(signs.size(), max_var_count)
                latch(t, TN_ERR_VAR_CAPACITY,
                      "sparse pull: slot " + std::to_string(s) + " has " + std::to_string(t->last_counts[s]) +
                          " distinct signs, its variable only " + std::to_string(t->pending_rows[s]) + " rows");
    }
}

int take_latched(SparseTable* t) {
    int code = t->latched;
    if (code != TN_OK) {
        set_error(t->latched_msg);
        t->latched = TN_OK;
        t->latched_msg.clear();
    }
    return code;
}

int sync_table(SparseTable* t, hipStream_t st) {
    if (t->upd_pending) {
        TN_HIP(hipEventSynchronize(t->upd_ev));
        t->upd_pending = false;
    }
    TN_HIP(hipStreamSynchronize(st));
    if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
    harvest(t);
    return take_latched(t);
}

// Moves every resident row into a freshly allocated table of `cap` slots.
int grow_to(SparseTable* t, uint64_t cap, hipStream_t st) {
    Store& s = t->store;
    if (cap > MAX_SLOTS_PER_TABLE) cap = MAX_SLOTS_PER_TABLE;
    if (cap <= s.cap) return fail(TN_ERR_TABLE_FULL, "sparse table cannot grow beyond 2^32 slots");
    Store bigger{};
    int rc = alloc_store(t, cap, bigger, st);
    if (rc != TN_OK) {
        free_store(bigger);
        return rc;
    }
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, t->dstatus, 0u, 0u);
    TN_LAUNCH(k_rehash, dim3(launch_grid((int64_t)s.cap + 1, 256, GRID_CAP * 4)), dim3(256), st, s, bigger, t->dstatus);
    TN_HIP(hipMemcpyAsync(bigger.count, s.count, sizeof(unsigned long long), hipMemcpyDeviceToDevice, st));
    TN_HIP(hipStreamSynchronize(st));
    free_store(s);
    s = bigger;
    t->epoch++;  // cached row numbers are stale now
    return TN_OK;
}

// The number of resident keys, read on the stream `st` itself (a copy on the null stream would wait for,
// and hold up, every blocking stream of the process: other tables' calls).
int read_count(SparseTable* t, hipStream_t st, uint64_t* out) {
    TN_HIP(hipMemcpyAsync(t->hcount, t->store.count, sizeof(unsigned long long), hipMemcpyDeviceToHost, st));
    TN_HIP(hipStreamSynchronize(st));
    t->count_upper = *t->hcount;
    *out = *t->hcount;
    return TN_OK;
}

// Makes room for up to `incoming` new keys: grows (re-inserts into a larger
// table) when the load factor could pass MAX_LOAD (optimizer_kernel.h:266).
// Callers have collected the status of earlier calls (t->booked == 0).
int ensure_room(SparseTable* t, uint64_t incoming, hipStream_t st) {
    Store& s = t->store;
    if ((double)(t->count_upper + incoming) > MAX_LOAD * (double)s.cap) {
        TN_TRY(order_after_updates(t, st));  // growing moves the rows
        uint64_t cnt = 0;  // the bound may be loose: read the true count
        TN_TRY(read_count(t, st, &cnt));
        if ((double)(cnt + incoming) > MAX_LOAD * (double)s.cap) {
            uint64_t need = (uint64_t)((double)(cnt + incoming) / MAX_LOAD) + 64;
            TN_TRY(grow_to(t, std::max<uint64_t>(need, s.cap * 2), st));
        }
    }
    t->count_upper += incoming;
    t->booked = incoming;
    return TN_OK;
}

// ---------------------------------------------------------------- workspace
struct Carver {
    char* base;
    size_t off = 0;
    template <typename T>
    T* take(size_t n) {
        off = align_up(off, 256);
        T* p = reinterpret_cast<T*>(base + off);
        off += n * sizeof(T);
        return p;
    }
};

// Results of analysing one batch.  For an op-level call they live in the
// table's plan buffer and survive until the next op-level call, so that a push
// of the same batch can reuse them; a table-level push carves the group part
// from the per-call scratch.
struct Plan {
    SlotDesc* descs;
    SlotDesc* push_descs;  // descriptors of the push that reuses the plan (the pull's gather may still read `descs`)
    uint32_t* push_ubase;  // ... and its copy of ubase, which its status is published from (the next pull rewrites ubase)
    uint32_t* lbase;
    uint32_t* ubase;
    uint64_t* vals_copy;   // signs of every lookup, concatenated; after a pull through LDS their fingerprints instead
    uint32_t* u_of_gi;     // lookup -> index of its distinct sign
    uint64_t* uniq_sign;   // per-slot distinct signs, slot-major, first-occurrence order
    uint32_t* uniq_slot;
    uint32_t* ushow;       // batch_show per distinct sign, when the remap already knows it
    uint64_t* grp_sign;    // distinct signs over all slots
    uint32_t* grp_row;     // their table rows
    uint32_t* grp_off;
    uint32_t* grp_cnt;
    Member* list;          // members of every group, ascending (with their show / click counts)
    uint2* where_u;        // record -> {its place in `list`, its group}
    uint32_t* big_list;    // groups with BIG_GROUP records or more
    uint4* big_desc;       // {row, first member, records, group} of those groups (k_group_emit writes it, the other groupings do not)
    uint32_t big_cap;      // entries of big_list / big_desc
    const float** gaddr;   // gradient row of every record of the groups with several records (a push fills it)
    uint64_t* vals_exact;  // copy of the signs beside their fingerprints (tn_sparse_table_set_exact_verify), else nullptr
};

// Per-call scratch of the analysis.
struct Scratch {
    DedupEntry* dt;
    size_t dt_entries;
    uint32_t* tidx;
    uint8_t* flag8;
    uint32_t* tilesum;
    uint32_t* tileoff;
    uint32_t ntiles;
    // LDS remap
    uint32_t nbuckets;
    uint32_t span_cap;   // first-level buckets the widest tile touches (LDS counters of k_tile_dedup)
    uint32_t* bcursor;   // per first-level bucket: records handed in
    ulonglong2* prec;    // the tiles' records by bucket, L1_ROOM each: {sign, position | occurrences | slot}
    uint32_t* first_of;
    uint32_t* cnt_at;
    uint32_t* wordpre;  // first occurrences before every 64-lookup word
    // grouping through LDS (second-level buckets)
    uint32_t nb2;
    uint32_t* cursor2;
    GroupRec* recs;
    uint2* aux;
    uint32_t* rrow;      // per distinct record: table row of its sign
    uint32_t* newrec;    // per second-level bucket: its records whose rows the pull inserted ...
    uint32_t* newcnt;    // ... and how many
    uint4* bcounts;
    uint4* bbase;
    void* gt;  // GroupEntry[] or MaskEntry[]
    uint32_t* gidx;
    uint32_t* ord;
    uint32_t* arrival;
};

size_t group_cap(size_t n) { return std::max<size_t>(16, n + n / 2); }

// Signs with this many records or more are applied by one wavefront each
// (k_apply_big); rows too wide for its LDS staging stay with the lane groups.
constexpr uint32_t BIG_GROUP = BIG_GROUP_DEFAULT;
uint32_t big_threshold(const Store& s) { return s.D <= BIG_DIM_MAX ? BIG_GROUP : 0xFFFFFFFFu; }

void carve_groups(Carver& c, Plan& p, size_t n) {
    p.grp_sign = c.take<uint64_t>(n);
    p.grp_row = c.take<uint32_t>(n);
    p.grp_off = c.take<uint32_t>(n);
    p.grp_cnt = c.take<uint32_t>(n);
    p.list = c.take<Member>(n);
    p.where_u = c.take<uint2>(n);
    p.big_cap = (uint32_t)(n / std::min<uint32_t>(BIG_GROUP, SMALL_BIG_GROUP) + 64);  // (the lowest threshold a plan may use)
    p.big_list = c.take<uint32_t>(p.big_cap);
    p.big_desc = c.take<uint4>(p.big_cap);
    p.gaddr = c.take<const float*>(n);
}

void carve_group_scratch(Carver& c, Scratch& w, size_t n) {
    w.gt = c.take<MaskEntry>(group_cap(n) + 1);  // the larger of the two entry types
    w.gidx = c.take<uint32_t>(n);
    w.ord = c.take<uint32_t>(n);
    w.arrival = c.take<uint32_t>(n);
}

size_t carve_plan(char* base, Plan& p, int N, size_t L, bool exact = false) {
    Carver c{base};
    p.descs = c.take<SlotDesc>(N);
    p.push_descs = c.take<SlotDesc>(N);
    p.lbase = c.take<uint32_t>(N + 1);
    p.ubase = c.take<uint32_t>(N + 1);
    p.push_ubase = c.take<uint32_t>(N + 1);
    p.vals_copy = c.take<uint64_t>(std::max<size_t>(L, 16));  // (the fingerprints of a short batch: 64 bytes a tile)
    p.u_of_gi = c.take<uint32_t>(L);
    p.uniq_sign = c.take<uint64_t>(L);
    p.uniq_slot = c.take<uint32_t>(L);
    p.ushow = c.take<uint32_t>(L);
    carve_groups(c, p, L);
    p.vals_exact = exact ? c.take<uint64_t>(L) : nullptr;  // last: the other arrays keep their places either way
    return align_up(c.off, 256);
}

// Second-level buckets of a batch of L lookups: GRP_TARGET records each on average if the batch has the
// expected share of distinct records plus a quarter (GRP_CAP is the room of a bucket).
uint32_t second_level_buckets(size_t L, double distinct_est) {
    const double expected = std::min(1.0, distinct_est * 1.25) * (double)L;
    return (uint32_t)std::max<size_t>(1, ((size_t)expected + GRP_TARGET - 1) / GRP_TARGET);
}

// dt_entries: entries of the global dedup table, or (use_lds) the number of buckets.
// First-level buckets of a slot of `len` lookups whose tiles hand on `share` records per lookup: L1_FILL records
// each on average (L1_ROOM is the room of a bucket); a slot that fits one bucket whatever its signs has one.
constexpr size_t L1_FILL = 1150;
constexpr double L1_MARGIN = 1.15;
size_t first_level_buckets(size_t len, double share) {
    if (len <= (size_t)L1_ROOM) return 1;
    return ((size_t)((double)len * std::min(1.0, share * L1_MARGIN)) + L1_FILL - 1) / L1_FILL;
}

size_t carve_scratch(char* base, Scratch& w, size_t L, size_t dt_entries, bool use_lds, double distinct_est = 1.0,
                     int N = 0) {
    Carver c{base};
    if (use_lds) {
        w.nbuckets = (uint32_t)dt_entries;
        w.nb2 = second_level_buckets(L, distinct_est);
        // room for the buckets of a batch of distinct signs only: a call that overflows is repeated with that
        // many, and must not pay for a larger buffer then (freeing and allocating waits for the whole device)
        const size_t nb2_room = std::max<size_t>(w.nb2, (L + GRP_TARGET - 1) / GRP_TARGET);
        const size_t nb1_room = std::max<size_t>(dt_entries, L / L1_FILL + (size_t)N + 1);
        w.bcursor = c.take<uint32_t>(nb1_room + 1 + nb2_room);  // (the part in use is zeroed together)
        w.cursor2 = w.bcursor + dt_entries + 1;
        w.recs = c.take<GroupRec>(nb2_room * GRP_CAP);
        w.aux = c.take<uint2>(nb2_room * GRP_CAP);
        w.rrow = c.take<uint32_t>(nb2_room * GRP_CAP);
        w.newrec = c.take<uint32_t>(nb2_room * GRP_CAP);
        w.newcnt = c.take<uint32_t>(nb2_room);
        w.bcounts = c.take<uint4>(nb2_room);
        w.bbase = c.take<uint4>(nb2_room);
        w.prec = c.take<ulonglong2>(nb1_room * (size_t)L1_ROOM);
        w.first_of = c.take<uint32_t>(L);
        w.cnt_at = c.take<uint32_t>(L);
        w.wordpre = c.take<uint32_t>(L / 64 + 2);
        w.dt = nullptr;
        w.dt_entries = 0;
        w.tidx = nullptr;
    } else {
        w.dt = c.take<DedupEntry>(dt_entries);
        w.dt_entries = dt_entries;
        w.tidx = c.take<uint32_t>(L);
    }
    w.flag8 = c.take<uint8_t>(L / REMAP_ITEMS + REMAP_THREADS);
    w.ntiles = (uint32_t)((L + REMAP_TILE - 1) / REMAP_TILE);
    w.tilesum = c.take<uint32_t>(w.ntiles + 1);
    w.tileoff = c.take<uint32_t>(w.ntiles + 1);
    carve_group_scratch(c, w, L);
    return align_up(c.off, 256);
}

// Validates the slot arrays of an op and fills the descriptors; returns L.
// With *use_lds set on entry the slots are laid out for the LDS remap if the batch
// qualifies (tbase/tcap = first bucket / number of buckets of the slot, dt_entries =
// number of buckets); otherwise *use_lds comes back false and tbase/tcap describe the
// slot's region of the global dedup table.
int stage_slots(SparseTable* t, int N, const int64_t* const* values, const int64_t* lens, std::vector<SlotDesc>& descs,
                std::vector<uint32_t>& lbase, size_t& L, size_t& dt_entries, const char* what, bool* use_lds,
                uint32_t* span_cap = nullptr) {
    if (N <= 0 || !values || !lens) return fail(TN_ERR_INVALID_ARGUMENT, std::string(what) + ": no slots");
    if (N > MAX_SLOTS)
        return fail(TN_ERR_UNSUPPORTED, std::string(what) + ": more than " + std::to_string(MAX_SLOTS) + " slots");
    descs.assign(N, SlotDesc{});
    lbase.assign(N + 1, 0);
    size_t l = 0, te = 0;
    for (int s = 0; s < N; s++) {
        if (lens[s] < 0 || (lens[s] > 0 && !values[s]))
            return fail(TN_ERR_INVALID_ARGUMENT, std::string(what) + ": bad values tensor of slot " + std::to_string(s));
        SlotDesc& d = descs[s];
        d.values = values[s];
        d.len = (uint32_t)lens[s];
        d.lbase = (uint32_t)l;
        d.tbase = (uint32_t)te;
        size_t tcap = (size_t)lens[s] + (size_t)lens[s] / 2 + 8;
        d.tcap = (uint32_t)tcap;
        lbase[s] = (uint32_t)l;
        l += (size_t)lens[s];
        te += tcap + 1;
        if (l > 0x7FFFFFF0ull || te > 0xFFFFFFF0ull)
            return fail(TN_ERR_UNSUPPORTED, std::string(what) + ": more than 2^31 lookups in one call");
    }
    lbase[N] = (uint32_t)l;
    L = l;
    dt_entries = te;
    if (use_lds && *use_lds) {
        bool ok = l >= LDS_MIN_LOOKUPS;
        for (int s = 0; s < N && ok; s++) ok = (size_t)lens[s] <= (size_t)LDS_MAX_SUB * L1_FILL;
        *use_lds = ok;
        if (ok) {
            // The buckets have fixed room for the records the tiles hand in (one per distinct sign of a tile):
            // sized from the share of such records the recent pulls had, with a margin; a batch that overflows
            // them is repeated with buckets for a batch without repeats.
            size_t nb = 0;
            for (int s = 0; s < N; s++) {
                const size_t sub = first_level_buckets((size_t)lens[s], t->tile_est);
                descs[s].tbase = (uint32_t)nb;
                descs[s].tcap = (uint32_t)sub;
                nb += sub;
            }
            dt_entries = nb;
            // buckets the widest tile of the partition kernel touches: first bucket of the slot of
            // its first lookup .. last bucket of the slot of its last lookup
            size_t widest = 1;
            int s0 = 0, s1 = 0;
            for (size_t g0 = 0; g0 < l; g0 += LDS_TILE) {
                const size_t g1 = std::min(l, g0 + (size_t)LDS_TILE) - 1;
                while (s0 + 1 < N && lbase[s0 + 1] <= g0) s0++;
                if (s1 < s0) s1 = s0;
                while (s1 + 1 < N && lbase[s1 + 1] <= g1) s1++;
                widest = std::max<size_t>(widest, (size_t)descs[s1].tbase + descs[s1].tcap - descs[s0].tbase);
            }
            if (span_cap) *span_cap = (uint32_t)std::min<size_t>(widest, LDS_SPAN);
        }
    }
    return TN_OK;
}

// Slot descriptors to the device (dst_descs; the slots' first lookups to dst_lbase unless nullptr); the same
// launch prepares the call's status block `ds` (status_mode) and clears `zero[0 .. n_zero)`.  It runs on `run_on`.
int upload_slots(SparseTable* t, SlotDesc* dst_descs, uint32_t* dst_lbase, DevStatus* ds,
                 const std::vector<SlotDesc>& descs, const std::vector<uint32_t>& lbase, hipStream_t run_on,
                 int status_mode, uint32_t* zero = nullptr, uint32_t n_zero = 0, const uint32_t* copy_src = nullptr,
                 uint32_t* copy_dst = nullptr, uint32_t copy_n = 0) {
    if (t->stage_pending) {
        TN_HIP(hipEventSynchronize(t->stage_ev));
        t->stage_pending = false;
    }
    const size_t db = descs.size() * sizeof(SlotDesc);
    const size_t lb = dst_lbase ? lbase.size() * sizeof(uint32_t) : 0;
    std::memcpy(t->hstage, descs.data(), db);
    if (lb) std::memcpy(t->hstage + db, lbase.data(), lb);
    TN_LAUNCH(k_stage_in, dim3(launch_grid((int64_t)std::max<size_t>((db + lb) / 4, n_zero), 256, 64)), dim3(256),
              run_on, reinterpret_cast<const uint32_t*>(t->hstage), reinterpret_cast<uint32_t*>(dst_descs),
              (uint32_t)(db / 4), dst_lbase, (uint32_t)(lb / 4), ds, status_mode, zero, n_zero,
              (const DevStatus*)t->dplan, copy_src, copy_dst, copy_n);
    TN_HIP(hipEventRecord(t->stage_ev, run_on));
    t->stage_pending = true;
    return TN_OK;
}

// own_copies: the source of a push on the last pull's plan, whose kernels may still run (detached updates) or
// be staged (the next pull's descriptors go in beside them) while the next pull rewrites p.descs and p.ubase:
// it reads the push's own descriptors and its own copy of the slots' distinct bases.
PushSrc op_source(const Plan& p, int dim, bool own_copies = false) {
    PushSrc src{};
    src.uniq_sign = p.uniq_sign;
    src.uniq_slot = p.uniq_slot;
    src.ubase = own_copies ? p.push_ubase : p.ubase;
    src.descs = own_copies ? p.push_descs : p.descs;
    src.dim = dim;
    return src;
}

// Groups n records (n_host of them, or status->n_unique) by sign: group arrays
// and member lists in ascending record order.  Works for any records: arrival
// order by atomics, then every record finds its place among its group's members.
void launch_grouping(const Plan& p, const Scratch& w, const PushSrc& src, int64_t n_host, int64_t n_upper,
                     uint32_t big_k, const uint32_t* ushow, DevStatus* ds, hipStream_t st) {
    const uint32_t* n_dev = src.infos ? nullptr : &ds->n_unique;
    GroupEntry* gt = static_cast<GroupEntry*>(w.gt);
    const int gblocks = launch_grid(n_upper, 256, GRID_CAP * 2);
    const int tblocks = launch_grid((int64_t)group_cap(n_upper) + 1, 256, GRID_CAP * 2);
    TN_LAUNCH(k_fill_groups, dim3(tblocks), dim3(256), st, gt, ds);
    TN_LAUNCH(k_group_insert, dim3(gblocks), dim3(256), st, src, n_host, ds, gt, w.gidx, w.ord);
    TN_LAUNCH(k_group_compact, dim3(launch_grid((int64_t)group_cap(n_upper) / COMPACT_ITEMS + 1, 256, GRID_CAP)),
              dim3(256), st, ds, gt, p.grp_sign, p.grp_off, p.grp_cnt, p.big_list, big_k, (uint32_t)n_upper);
    TN_LAUNCH(k_group_fill, dim3(gblocks), dim3(256), st, n_host, n_dev, gt, p.grp_off, w.gidx, w.ord, w.arrival);
    TN_LAUNCH(k_group_rank, dim3(gblocks), dim3(256), st, n_host, n_dev, gt, p.grp_off, w.gidx, w.arrival,
              src.uniq_slot, ushow, p.list, p.where_u);
}

constexpr int MASK_SLOTS = 128;
constexpr uint32_t LONG_SEGMENT = 64;  // lookups of one distinct sign from which a workgroup sums them


// The same result for the distinct signs of an op with at most 128 slots, from slot masks.
void launch_mask_grouping(const Plan& p, const Scratch& w, int64_t n_upper, uint32_t big_k, const uint32_t* ushow,
                          DevStatus* ds, hipStream_t st) {
    MaskEntry* gt = static_cast<MaskEntry*>(w.gt);
    const int gblocks = launch_grid(n_upper, 256, GRID_CAP * 2);
    const int tblocks = launch_grid(2 * (int64_t)group_cap(n_upper) + 2, 256, GRID_CAP * 2);
    TN_LAUNCH(k_fill_masks, dim3(tblocks), dim3(256), st, gt, ds);
    TN_LAUNCH(k_mask_insert, dim3(gblocks), dim3(256), st, p.uniq_sign, p.uniq_slot, ds, gt, w.gidx);
    TN_LAUNCH(k_mask_compact, dim3(launch_grid((int64_t)group_cap(n_upper) / COMPACT_ITEMS + 1, 256, GRID_CAP)),
              dim3(256), st, ds, gt, p.grp_sign, p.grp_off, p.grp_cnt, p.big_list, big_k, (uint32_t)n_upper);
    TN_LAUNCH(k_mask_fill, dim3(gblocks), dim3(256), st, ds, gt, w.gidx, p.uniq_slot, ushow, p.list, p.where_u);
}

// Analyses the batch staged in p.descs: per-slot distinct signs and mapped ids,
// groups of equal signs, and the table row of every group (inserting absent
// signs for a pull).  use_lds picks the remap through LDS (pull only).  The
// upload of the descriptors has cleared the status block and, for the LDS path,
// the bucket counters.
int launch_build_plan(SparseTable* t, const Plan& p, const Scratch& w, int N, uint32_t L, bool for_pull, bool use_lds,
                      hipStream_t st) {
    DevStatus* ds = t->dplan;
    const Store& s = t->store;
    const int lblocks = launch_grid(L, 256, GRID_CAP * 2);
    const bool lds_groups = use_lds && N <= GRP_SLOTS;
    // second-level buckets up to which k_group_emit adds up the bucket counts itself (one bucket per workgroup)
    const bool own_offsets = w.nb2 <= (uint32_t)GRID_CAP * 4;
    if (use_lds) {
        // (as many workgroups as the chip holds of this kernel at once -- three per CU --, each taking its tiles in turn)
        const int tiles = launch_grid((int64_t)(L + LDS_TILE - 1) / LDS_TILE, 1, TILE_GRID);
        const size_t tile_lds = tile_dedup_lds(N, w.span_cap);
        TN_LAUNCH_LDS(k_tile_dedup, dim3(tiles), dim3(TILE_THREADS), tile_lds, st, p.descs, p.lbase, N, L, w.bcursor, w.prec,
                      reinterpret_cast<ulonglong2*>(p.vals_copy), p.vals_exact, w.first_of, ds, w.span_cap);
        if (lds_groups)
            TN_LAUNCH((k_lds_dedup<true>), dim3(launch_grid(w.nbuckets, 1, GRID_CAP * 2)), dim3(DEDUP_THREADS), st, w.bcursor,
                      w.nbuckets, w.prec, w.first_of, w.cnt_at, ds, w.nb2, w.cursor2, w.recs);
        else
            TN_LAUNCH((k_lds_dedup<false>), dim3(launch_grid(w.nbuckets, 1, GRID_CAP * 2)), dim3(DEDUP_THREADS), st, w.bcursor,
                      w.nbuckets, w.prec, w.first_of, w.cnt_at, ds, w.nb2, w.cursor2, w.recs);
        if (lds_groups) {
            // The grouping of the distinct records only needs what the dedup handed over: it runs on
            // the side stream beside the ranking of the first occurrences (LDS / latency bound
            // against streaming kernels) and joins before the member lists are written.
            const int bblocks = launch_grid(w.nb2, 1, GRID_CAP * 4);
            hipStream_t sd = t->one_stream ? st : t->side, sd2 = t->one_stream ? st : t->side2;
            if (!t->one_stream) {
                TN_HIP(hipEventRecord(t->fork_ev, st));
                TN_HIP(hipStreamWaitEvent(t->side, t->fork_ev, 0));
            }
            TN_LAUNCH(k_group_count, dim3(bblocks), dim3(GRP_THREADS), sd, w.nb2, w.cursor2, w.recs,
                      big_threshold(s), w.aux, w.bcounts);
            if (!own_offsets) TN_LAUNCH(k_group_offsets, dim3(1), dim3(1024), sd, w.bcounts, w.bbase, w.nb2, ds);
            if (!t->one_stream) {
                TN_HIP(hipEventRecord(t->join_ev, t->side));
                // ... and so do the rows of the records' signs, on a stream of their own
                TN_HIP(hipStreamWaitEvent(t->side2, t->fork_ev, 0));
            }
            // few workgroups: enough probes in flight for the memory system, most of every CU left to the grouping
            TN_LAUNCH(k_probe_recs, dim3(std::min(bblocks, PROBE_RECS_GRID)), dim3(256), sd2, w.nb2, w.cursor2, w.recs, w.rrow,
                      w.newrec, w.newcnt, s, ds);
            const uint32_t init_parts = std::max<uint32_t>(1, (uint32_t)GRID_CAP / w.nb2);
            TN_LAUNCH(k_init_new_recs, dim3(launch_grid((int64_t)w.nb2 * init_parts, 1, GRID_CAP)), dim3(256), sd2, s,
                      make_optdev(t), t->seed, w.recs, w.rrow, w.nb2, w.newrec, w.newcnt, ds, init_parts);
            if (!t->one_stream) TN_HIP(hipEventRecord(t->join2_ev, t->side2));
        }
        TN_LAUNCH(k_lds_flags, dim3(w.ntiles), dim3(REMAP_THREADS), st, L, w.first_of, w.flag8, w.tilesum, p.descs, N,
                  w.bcursor, ds);
        // up to SELF_SCAN_TILES tiles the ranking pass adds up the tile counts itself
        const uint32_t* own_sums = w.ntiles <= SELF_SCAN_TILES ? w.tilesum : nullptr;
        if (!own_sums)
            TN_LAUNCH(k_scan_tiles, dim3(1), dim3(1024), st, w.tilesum, w.tileoff, w.ntiles, p.lbase, p.ubase, N, L, ds);
        const size_t lb_lds = ((size_t)N + 1) * sizeof(uint32_t);
        if (lds_groups)
            TN_LAUNCH_LDS((k_lds_assign<false>), dim3(w.ntiles), dim3(REMAP_THREADS), lb_lds, st, p.descs, p.lbase, N, L,
                          w.flag8, w.tileoff, w.cnt_at, w.wordpre, p.ubase, p.uniq_sign, p.uniq_slot, p.ushow, own_sums, ds);
        else
            TN_LAUNCH_LDS((k_lds_assign<true>), dim3(w.ntiles), dim3(REMAP_THREADS), lb_lds, st, p.descs, p.lbase, N, L,
                          w.flag8, w.tileoff, w.cnt_at, w.wordpre, p.ubase, p.uniq_sign, p.uniq_slot, p.ushow, own_sums, ds);
        TN_LAUNCH_LDS(k_lds_mapped, dim3(lblocks), dim3(256), lb_lds, st, p.descs, p.lbase, p.ubase, N, L, w.first_of,
                      w.flag8, w.wordpre, p.u_of_gi);
    } else {
        TN_LAUNCH(k_fill_ff, dim3(launch_grid((int64_t)w.dt_entries, 256, GRID_CAP * 2)), dim3(256), st,
                  reinterpret_cast<uint4*>(w.dt), w.dt_entries);
        TN_LAUNCH(k_remap_insert, dim3(lblocks), dim3(256), st, p.descs, p.lbase, N, L, w.dt, w.tidx, p.vals_copy);
        TN_LAUNCH(k_flag_count, dim3(w.ntiles), dim3(REMAP_THREADS), st, p.lbase, N, L, w.dt, w.tidx, w.flag8,
                  w.tilesum);
        TN_LAUNCH(k_scan_tiles, dim3(1), dim3(1024), st, w.tilesum, w.tileoff, w.ntiles, p.lbase, p.ubase, N, L, ds);
        TN_LAUNCH(k_assign_rank, dim3(w.ntiles), dim3(REMAP_THREADS), st, p.descs, p.lbase, N, L, w.dt, w.tidx, w.flag8,
                  w.tileoff, p.ubase, p.uniq_sign, p.uniq_slot);
        TN_LAUNCH(k_write_mapped, dim3(lblocks), dim3(256), st, p.descs, p.lbase, p.ubase, N, L, w.dt, w.tidx, w.flag8,
                  p.u_of_gi, for_pull ? 1 : 0);
    }
    const uint32_t* ushow = use_lds ? p.ushow : nullptr;
    // from here on the groups and member lists are written, which detached updates of the push before still read
    TN_TRY(order_after_updates(t, st));
    if (lds_groups) {
        const int bblocks = launch_grid(w.nb2, 1, GRID_CAP * 4);
        if (!t->one_stream) {
            TN_HIP(hipStreamWaitEvent(st, t->join_ev, 0));
            TN_HIP(hipStreamWaitEvent(st, t->join2_ev, 0));
        }
        TN_LAUNCH((k_group_emit<false>), dim3(bblocks), dim3(EMIT_THREADS), st, w.nb2, w.cursor2, w.recs, w.aux,
                  own_offsets ? nullptr : w.bbase, w.bcounts, w.flag8, w.wordpre, L, big_threshold(s),
                  p.grp_sign, p.grp_off, p.grp_cnt, p.big_list, p.big_desc, p.list, p.where_u, w.rrow, p.grp_row, ds,
                  (const uint32_t*)nullptr, 0u);
        t->plan_big_desc = true;
        return TN_OK;  // the rows were found beside the grouping
    } else if (N <= MASK_SLOTS)
        launch_mask_grouping(p, w, (int64_t)L, big_threshold(s), ushow, ds, st);
    else
        launch_grouping(p, w, op_source(p, 0), 0, (int64_t)L, big_threshold(s), ushow, ds, st);
    if (for_pull)
        TN_LAUNCH((k_probe<true>), dim3(lblocks), dim3(256), st, s, p.grp_sign, (int64_t)0, ds, L, p.grp_row,
                  (uint32_t*)nullptr, ds, (uint32_t)DEV_ERR_TABLE_FULL, make_optdev(t), t->seed);
    else
        TN_LAUNCH((k_probe<false>), dim3(lblocks), dim3(256), st, s, p.grp_sign, (int64_t)0, ds, L, p.grp_row,
                  (uint32_t*)nullptr, ds, (uint32_t)DEV_ERR_UNKNOWN_KEY, make_optdev(t), t->seed);
    return TN_OK;
}

// The three kernels touch disjoint rows.  k_apply_single saturates the memory system (it runs
// at the device's rate for random row updates); k_apply_big and k_apply_vec are bound by
// dependent chains and instruction issue, so they run one after the other beside it.  The pair is
// the longer chain: it stays on the caller's stream and k_apply_single goes to the table's side
// stream, forked from and joined back into the caller's stream by events (a kernel that waits for
// an event of another stream starts 15-30 us late: better the chain that has the time to spare).
//
// detach: none of them on the caller's stream, which does not wait for them either -- k_apply_single on the
// auxiliary stream; the caller of this function records their end (see SparseTable::upd_ev).
template <int KIND>
int launch_apply_kind(SparseTable* t, int lpg, const Store& s, const OptDev& o, const PushSrc& src, DevStatus* ds,
                      const Plan& p, int64_t n_upper, hipStream_t st, bool addr_ready, uint32_t big_k, bool detach,
                      bool big_desc) {
    const uint32_t ids_cap = (uint32_t)n_upper;
    const bool with_big = big_k != 0xFFFFFFFFu;
    const float* const* gaddr = (with_big && !src.infos && !src.flat) ? p.gaddr : nullptr;
    detach = detach && !t->one_stream && lpg != 0;
    t->detached_now = detach;
    const bool forked = (with_big || detach) && !t->one_stream;
    // op-level gradients: their addresses for the records of the groups with several records, once, in a
    // coalesced pass ahead of everything (beside k_apply_single it would take several times as long)
    if (with_big && gaddr && !addr_ready)
        TN_LAUNCH(k_member_grads, dim3(launch_grid(n_upper, 256, GRID_CAP * 2)), dim3(256), st, src, ds, p.list,
                  p.gaddr, ids_cap);
    if (forked) {
        TN_HIP(hipEventRecord(t->fork_ev, st));
        TN_HIP(hipStreamWaitEvent(t->side, t->fork_ev, 0));
        if (detach) TN_HIP(hipStreamWaitEvent(t->aux, t->fork_ev, 0));
    }
    if (with_big) {
        const int gfloats = big_gbuf_floats(s.D);
        const int big_blocks = launch_grid(n_upper / BIG_GROUP + 1, 1, 16384);
        hipStream_t bst = detach ? t->side : st;
#define TN_LAUNCH_BIG_ADAGRAD(DIM)                                                                                  \
    TN_LAUNCH((k_apply_big_adagrad<DIM>), dim3(big_blocks), dim3(64), bst, s, o, src, ds, (const uint4*)p.big_desc, \
              p.big_cap, p.list, gaddr)
        // AdaGrad rows of a power-of-two dim on a plan that describes its frequent signs: the kernel made for them
        const bool tiled = KIND == OPT_ADAGRAD && big_desc;
        if (tiled && s.D == 4) TN_LAUNCH_BIG_ADAGRAD(4);
        else if (tiled && s.D == 8) TN_LAUNCH_BIG_ADAGRAD(8);
        else if (tiled && s.D == 16) TN_LAUNCH_BIG_ADAGRAD(16);
        else if (tiled && s.D == 32) TN_LAUNCH_BIG_ADAGRAD(32);
        else if (tiled && s.D == 64) TN_LAUNCH_BIG_ADAGRAD(64);
        else
            TN_LAUNCH_LDS((k_apply_big<KIND>), dim3(big_blocks), dim3(64), big_lds_bytes(s.D), bst, s, o, src, ds,
                          p.big_list, p.grp_row, p.grp_off, p.grp_cnt, p.list, gfloats, gaddr);
#undef TN_LAUNCH_BIG_ADAGRAD
    }
#define TN_LAUNCH_VEC(LPG)                                                                                        \
    do {                                                                                                          \
        TN_LAUNCH((k_apply_single<KIND, LPG>), dim3(launch_grid(n_upper * LPG, 256, GRID_CAP * 4)), dim3(256),    \
                  detach ? t->aux : (forked ? t->side : st), s, o, src, ds, p.grp_row, p.list);                   \
        TN_LAUNCH((k_apply_vec<KIND, LPG>), dim3(launch_grid(n_upper * LPG / 2, 256, GRID_CAP * 4)), dim3(256),    \
                  detach ? t->side : st, s, o, src, ds, p.grp_row, p.grp_off, p.grp_cnt, p.list, big_k, ids_cap,  \
                  gaddr);                                                                                         \
    } while (0)
    switch (lpg) {
        case 1: TN_LAUNCH_VEC(1); break;
        case 2: TN_LAUNCH_VEC(2); break;
        case 4: TN_LAUNCH_VEC(4); break;
        case 8: TN_LAUNCH_VEC(8); break;
        case 16: TN_LAUNCH_VEC(16); break;
        case 32: TN_LAUNCH_VEC(32); break;
        default:
            TN_LAUNCH((k_apply_scalar<KIND>), dim3(launch_grid(n_upper, 256, GRID_CAP * 2)), dim3(256), st, s, o, src, ds,
                      p.grp_row, p.grp_off, p.grp_cnt, p.list, big_k, ids_cap);
    }
#undef TN_LAUNCH_VEC
    if (forked && !detach) {
        TN_HIP(hipEventRecord(t->join_ev, t->side));
        TN_HIP(hipStreamWaitEvent(st, t->join_ev, 0));
    }
    return TN_OK;
}

// Lanes that share a row in the update kernels (a float4 each), 0 if the rows cannot be handled that way.
int lanes_per_group(const Store& s, bool vec_ok) {
    if (!vec_ok || s.D % 4 != 0) return 0;
    const int q = s.D / 4;
    return (q >= 1 && q <= 32 && (q & (q - 1)) == 0) ? q : 0;
}

// Applies the grouped records; n_upper bounds the number of records.
// addr_ready: p.gaddr already holds the gradient addresses of the multi-record groups' records.
// big_k: the number of records from which the plan's grouping listed a sign for k_apply_big (0: the table's default).
// big_desc: p.big_desc describes the signs of p.big_list (the plan of a pull that grouped through LDS).
int launch_apply(SparseTable* t, const Plan& p, const PushSrc& src, DevStatus* ds, int64_t n_upper, bool vec_ok,
                 hipStream_t st, bool addr_ready = false, uint32_t big_k = 0, bool detach = false, bool big_desc = false) {
    const Store& s = t->store;
    const OptDev o = make_optdev(t);
    const int lpg = lanes_per_group(s, vec_ok);
    if (big_k == 0) big_k = big_threshold(s);
    switch (o.kind) {
        case OPT_ADAGRAD: return launch_apply_kind<OPT_ADAGRAD>(t, lpg, s, o, src, ds, p, n_upper, st, addr_ready, big_k, detach, big_desc);
        case OPT_ADAM: return launch_apply_kind<OPT_ADAM>(t, lpg, s, o, src, ds, p, n_upper, st, addr_ready, big_k, detach, big_desc);
        default: return launch_apply_kind<OPT_FTRL>(t, lpg, s, o, src, ds, p, n_upper, st, addr_ready, big_k, detach, big_desc);
    }
}

// The updates of a small push, one launch: the lane groups' workgroups for every group below the plan's threshold
// and, if the plan lists signs with many records, workgroups whose wavefronts take those (as a kernel of its own
// after this one, k_apply_big made 4096 x 26 slots, Adam, 0.080 ms per pull + push; beside it on the table's side
// stream 0.113 ms: the events that fork and join the streams cost more than the overlap wins).
template <int KIND>
int launch_small_apply_kind(SparseTable* t, int lpg, int N, const OptDev& o, const PushSrc& src, DevStatus* ds,
                            const Plan& p, int64_t n_upper, hipStream_t st, uint32_t* host_seq, uint32_t seq) {
    const Store& s = t->store;
    const uint32_t big_k = t->plan_big_k;
    const bool with_big = big_k != 0xFFFFFFFFu && (uint32_t)N >= big_k;
    // (a wavefront per sign with big_k records or more, four to a workgroup, 512 workgroups at most)
    const int big_blocks = with_big ? launch_grid((n_upper / big_k + 1 + 3) / 4, 1, 512) : 0;
    const size_t lds = with_big ? small_apply_big_lds(s.D) : 0;
#define TN_LAUNCH_SMALL(LPG)                                                                                          \
    do {                                                                                                              \
        const int group_blocks = launch_grid(n_upper * LPG, 256, GRID_CAP * 4);                                       \
        TN_LAUNCH_LDS((k_small_apply<KIND, LPG>), dim3(group_blocks + big_blocks), dim3(256), lds, st, s, o, src, N, ds, \
                      p.grp_row, p.grp_off, p.grp_cnt, p.list, big_k, (uint32_t)n_upper, host_seq, seq,              \
                      (uint32_t)big_blocks, p.big_list, big_gbuf_floats(s.D), (uint32_t)small_apply_wave_lds(s.D),    \
                      (uint32_t)align_up(big_lds_bytes(s.D), 8));                                                    \
    } while (0)
    switch (lpg) {
        case 1: TN_LAUNCH_SMALL(1); break;
        case 2: TN_LAUNCH_SMALL(2); break;
        case 4: TN_LAUNCH_SMALL(4); break;
        case 8: TN_LAUNCH_SMALL(8); break;
        case 16: TN_LAUNCH_SMALL(16); break;
        default: TN_LAUNCH_SMALL(32); break;
    }
#undef TN_LAUNCH_SMALL
    return TN_OK;
}

int launch_small_apply(SparseTable* t, int lpg, int N, const PushSrc& src, DevStatus* ds, const Plan& p, int64_t n_upper,
                       hipStream_t st, uint32_t* host_seq, uint32_t seq) {
    const OptDev o = make_optdev(t);
    switch (o.kind) {
        case OPT_ADAGRAD: return launch_small_apply_kind<OPT_ADAGRAD>(t, lpg, N, o, src, ds, p, n_upper, st, host_seq, seq);
        case OPT_ADAM: return launch_small_apply_kind<OPT_ADAM>(t, lpg, N, o, src, ds, p, n_upper, st, host_seq, seq);
        default: return launch_small_apply_kind<OPT_FTRL>(t, lpg, N, o, src, ds, p, n_upper, st, host_seq, seq);
    }
}

// Bytes of dynamic LDS a workgroup of `kernel` may have on this device (128 KB at most), after telling the
// runtime that the kernel wants them.
size_t big_lds_bytes_for(const void* kernel, size_t cap = 128 * 1024) {
    int dev = 0, most = 0;
    size_t bytes = 48 * 1024;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&most, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && most > 2048)
        bytes = std::min<size_t>((size_t)most - 2048, cap);  // (room for the kernel's static arrays)
    if (bytes > 48 * 1024 &&
        hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        bytes = 48 * 1024;
    }
    return bytes;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Entries of the LDS table of k_small_slots for slots of at most max_len lookups (load <= 0.5).
uint32_t small_entries(size_t max_len) {
    uint32_t e = 64;
    while ((size_t)e < 2 * max_len) e *= 2;
    return e;
}

// Does the batch qualify for the path of few launches?  (nb2: its second-level buckets.)
bool small_batch_fits(SparseTable* t, int N, const int64_t* lens, size_t L, uint32_t nb2) {
    if (!t->small_path || t->async_pull || N > SMALL_SLOTS || L == 0 || L > SMALL_MAX_LOOKUPS || nb2 > (uint32_t)SMALL_NB2_MAX) return false;
    size_t max_len = 0;
    for (int s = 0; s < N; s++) max_len = std::max<size_t>(max_len, (size_t)lens[s]);
    if (max_len > (size_t)SMALL_SLOT_MAX) return false;
    if (!t->small_lds)
        t->small_lds = big_lds_bytes_for(reinterpret_cast<const void*>(k_small_slots),
                                         small_slots_lds(small_entries(SMALL_SLOT_MAX), SMALL_NB2_MAX));
    return small_slots_lds(small_entries(max_len), nb2) <= t->small_lds;
}

// Waits for a kernel of the small path to report through pinned memory: *flag == want.  The word is polled for a
// while (it arrives a few microseconds after the kernel's end, well before a wait on the stream or on an event
// returns), then the stream is waited for, which also brings a failed launch to light.
int wait_reported(const uint32_t* flag, uint32_t want, hipStream_t st, const char* what) {
    const volatile uint32_t* f = flag;
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
        for (int i = 0; i < 256; i++) {
            if (*f == want) {
                // what the device wrote before the word (the status block) is read after it
                std::atomic_thread_fence(std::memory_order_acquire);
                return TN_OK;
            }
            __builtin_ia32_pause();
        }
        if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) break;
    }
    TN_HIP(hipStreamSynchronize(st));
    if (*f != want) return fail(TN_ERR_HIP, std::string(what) + ": the device did not report");
    std::atomic_thread_fence(std::memory_order_acquire);
    return TN_OK;
}

}  // namespace
}  // namespace tn

using namespace tn;

extern "C" {

int tn_sparse_table_create(tn_opt_t opt, const char* name, int dimension, int use_cvm, int shard_num,
                           int self_shard_id, const char* embedding_group, uint32_t* handle) {
    if (!handle) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_create: handle is NULL");
    auto conf = get_opt(opt);
    if (!conf) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_create: unknown optimizer handle");
    if (dimension <= 0 || dimension > 4096)
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_create: dimension must be in [1, 4096]");
    if (shard_num != 1 || self_shard_id != 0)
        return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_create: one worker only (shard_num 1, self_shard_id 0)");
    std::string group = embedding_group ? embedding_group : "";
    std::lock_guard<std::mutex> lk(g_tables_mu);
    if (!group.empty()) {  // sparse_table.cc:175-180
        for (SparseTable* t : g_tables)
            if (t->group == group) {
                *handle = t->handle;
                return TN_OK;
            }
    }
    SparseTable* t = new SparseTable();
    t->opt = conf;
    t->name = name ? name : "";
    t->group = group;
    t->dim = dimension;
    // only the AdaGrad row maintains the cvm columns (ada_grad_kernel.cc:99-102,123-128)
    t->use_cvm = (use_cvm && conf->kind == OPT_ADAGRAD) ? 1 : 0;
    t->shard_num = shard_num;
    t->self_shard_id = self_shard_id;
    if (hipGetDevice(&t->device) != hipSuccess) t->device = 0;
    t->handle = (uint32_t)g_tables.size();
    g_tables.push_back(t);
    *handle = t->handle;
    return TN_OK;
}

int tn_sparse_table_reserve(uint32_t handle, uint64_t max_keys) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_reserve: bad table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->allocated) {
        t->reserve_keys = max_keys;
        return TN_OK;
    }
    hipStream_t st = t->last_stream;
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    uint64_t want = reserved_slots(t, max_keys);
    if (want <= t->store.cap) return TN_OK;
    return grow_to(t, want, st);
}

int tn_sparse_table_clear(uint32_t handle) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_clear: bad table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->allocated) return TN_OK;
    // everything the table has queued, on whichever stream
    if (t->last_stream) TN_HIP(hipStreamSynchronize(t->last_stream));
    TN_HIP(hipStreamSynchronize(t->side));
    TN_HIP(hipStreamSynchronize(t->side2));
    TN_HIP(hipStreamSynchronize(t->aux));
    harvest(t);
    free_store(t->store);
    t->ws.release();
    t->plan_buf.release();
    t->comb_buf.release();
    t->pooled_ws.release();
    t->allocated = false;
    t->plan_valid = false;
    t->tail_recorded = false;
    t->flow = FLOW_NONE;
    t->count_upper = 0;
    t->booked = 0;
    t->epoch++;
    t->latched = TN_OK;
    t->latched_msg.clear();
    return TN_OK;
}

int tn_sparse_table_set_seed(uint32_t handle, uint64_t seed) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_set_seed: bad table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    t->seed = seed;
    return TN_OK;
}

int tn_sparse_table_key_count(uint32_t handle, uint64_t* count) {
    SparseTable* t = get_table(handle);
    if (!t || !count) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_key_count: bad table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    *count = 0;
    if (!t->allocated) return TN_OK;
    // Only this table's own work is waited for: the count is kept by kernels on the stream of the table's last
    // call (a pull that publishes its status on the side stream has waited for that before it returned).
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(t->last_stream));
        harvest(t);
    }
    uint64_t cnt = 0;
    TN_TRY(read_count(t, t->last_stream, &cnt));
    *count = cnt;
    return TN_OK;
}

int tn_sparse_table_capacity(uint32_t handle, uint64_t* slots) {
    SparseTable* t = get_table(handle);
    if (!t || !slots) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_capacity: bad table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    *slots = t->allocated ? t->store.cap : 0;
    return TN_OK;
}

int tn_sparse_table_row_layout(uint32_t handle, int* weight_floats, int* state_floats_out) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_row_layout: bad table handle");
    if (weight_floats) *weight_floats = t->dim + (t->use_cvm ? 2 : 0);
    if (state_floats_out) *state_floats_out = state_floats(t);
    return TN_OK;
}

int tn_sparse_table_set_async(uint32_t handle, int async_pull) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_set_async: bad table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    t->async_pull = async_pull ? 1 : 0;
    return TN_OK;
}

int tn_sparse_table_set_small_batch_path(uint32_t handle, int enable) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad sparse table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    t->small_path = enable != 0;
    return TN_OK;
}

int tn_sparse_table_set_exact_verify(uint32_t handle, int enable) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad sparse table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    t->exact_verify = enable != 0;
    return TN_OK;
}

int tn_sparse_table_set_detached_updates(uint32_t handle, int enable) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "bad sparse table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    t->detach_updates = enable != 0;
    return TN_OK;
}

int tn_sparse_table_sync(uint32_t handle) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_sync: bad table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    if (!t->allocated) return TN_OK;
    return sync_table(t, t->last_stream);
}

int tn_sparse_table_last_unique_counts(uint32_t handle, int N, int64_t* counts) {
    SparseTable* t = get_table(handle);
    if (!t || !counts) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_last_unique_counts: bad table handle");
    std::lock_guard<std::mutex> lk(t->mu);
    if (t->pull_pending || t->push_pending) {
        TN_HIP(hipStreamSynchronize(t->last_stream));
        harvest(t);
    }
    if ((int)t->last_counts.size() != N)
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_last_unique_counts: last op had " +
                                                 std::to_string(t->last_counts.size()) + " slots");
    for (int s = 0; s < N; s++) counts[s] = t->last_counts[s];
    return TN_OK;
}

// ------------------------------------------------------------ table level
int tn_sparse_table_pull(uint32_t handle, const uint64_t* signs, int64_t n, int dim, float* out, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_pull: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && (!signs || !out))) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_pull: NULL buffer");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    const int wdim = t->dim + (t->use_cvm ? 2 : 0);
    if (dim != wdim)
        return fail(TN_ERR_DIM_MISMATCH,
                    "tn_sparse_table_pull: dim " + std::to_string(dim) + " but table rows hold " + std::to_string(wdim));
    if (n > 0x7FFFFFF0LL) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_pull: more than 2^31 signs");
    t->last_stream = st;
    if (n == 0) return sync_table(t, st);
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    TN_TRY(ensure_room(t, (uint64_t)n, st));
    TN_TRY(t->ws.ensure(2 * align_up((size_t)n * sizeof(uint32_t), 256)));
    Carver c{(char*)t->ws.p};
    uint32_t* rows = c.take<uint32_t>(n);
    uint32_t* newlist = c.take<uint32_t>(n);
    const Store& s = t->store;
    const OptDev o = make_optdev(t);
    const int blocks = launch_grid(n, 256, GRID_CAP * 2);
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, t->dstatus, (uint32_t)n, 0u);
    TN_LAUNCH((k_probe<true>), dim3(blocks), dim3(256), st, s, signs, n, (const DevStatus*)nullptr, 0u, rows, newlist, t->dstatus, (uint32_t)DEV_ERR_TABLE_FULL, make_optdev(t), t->seed);
    TN_LAUNCH(k_init_rows, dim3(blocks), dim3(256), st, s, o, t->seed, signs, rows, newlist, t->dstatus);
    TN_LAUNCH(k_finish_insert, dim3(1), dim3(64), st, s, t->dstatus);
    if (wdim % 4 == 0 && s.wstride % 4 == 0 && aligned16(out))
        TN_LAUNCH((k_gather_rows<4>), dim3(launch_grid(n * (wdim / 4), 256, GRID_CAP * 4)), dim3(256), st, s, rows, n, out);
    else
        TN_LAUNCH((k_gather_rows<1>), dim3(launch_grid(n * wdim, 256, GRID_CAP * 4)), dim3(256), st, s, rows, n, out);
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpull->st, t->dstatus, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    t->hpull->ubase[0] = 0;
    t->pull_pending = true;
    t->pull_slots = 0;
    t->pending_rows.clear();
    return sync_table(t, st);
}

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
std::mutex g_static_mu;  // one call at a time uses a GPU's scratch array
unsigned char* g_static_ptr[STATIC_MAX_DEVICES] = {};

// Address of the current device's copy of `scratch`, looked up once per device.
int static_scratch(int* device, unsigned char** out) {
    int dev = 0;
    TN_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= STATIC_MAX_DEVICES)
        return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_pull_static: device number beyond " + std::to_string(STATIC_MAX_DEVICES));
    if (!g_static_ptr[dev]) {
        unsigned char* ptr = nullptr;
        TN_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(TN_ERR_HIP, "tn_sparse_table_pull_static: no address for the scratch array");
        g_static_ptr[dev] = ptr;
    }
    *device = dev;
    *out = g_static_ptr[dev];
    return TN_OK;
}
}  // namespace

int tn_sparse_table_pull_static(uint32_t handle, const uint64_t* signs, int64_t n, int dim, float* out, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_pull_static: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && (!signs || !out)))
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_pull_static: NULL buffer");
    if (n > TN_STATIC_MAX_SIGNS)
        return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_pull_static: " + std::to_string(n) + " signs, at most " +
                                            std::to_string(TN_STATIC_MAX_SIGNS) + " per call (use tn_sparse_table_pull)");
    std::lock_guard<std::mutex> sk(g_static_mu);
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    int dev = 0;
    unsigned char* ptr = nullptr;
    TN_TRY(static_scratch(&dev, &ptr));
    if (!t->allocated)
        return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_pull_static: the table has no storage yet (its first call through "
                                        "another entry point allocates it); this entry point allocates nothing");
    if (dev != t->device)
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_pull_static: the table lives on device " +
                                                 std::to_string(t->device) + ", the current device is " + std::to_string(dev));
    // the prologue every entry point shares (ensure_allocated), less the allocation
    TN_TRY(order_after_updates(t, st));
    TN_TRY(order_after_other_stream(t, st));
    t->flow = FLOW_NONE;
    const int wdim = t->dim + (t->use_cvm ? 2 : 0);
    if (dim != wdim)
        return fail(TN_ERR_DIM_MISMATCH, "tn_sparse_table_pull_static: dim " + std::to_string(dim) +
                                             " but table rows hold " + std::to_string(wdim));
    if (t->push_pending || t->pull_pending) {
        if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    if (n == 0) return sync_table(t, st);
    const Store& s = t->store;
    // every requested sign may be new; a table that would have to grow for them needs a new allocation
    if ((double)(t->count_upper + (uint64_t)n) > MAX_LOAD * (double)s.cap) {
        uint64_t cnt = 0;  // the bound may be loose: read the true count (pinned memory, no allocation)
        TN_TRY(read_count(t, st, &cnt));
        if ((double)(cnt + (uint64_t)n) > MAX_LOAD * (double)s.cap)
            return fail(TN_ERR_TABLE_FULL, "tn_sparse_table_pull_static: the table would have to grow for " +
                                               std::to_string(n) + " more signs, which needs an allocation "
                                               "(tn_sparse_table_reserve beforehand, or tn_sparse_table_pull)");
    }
    t->count_upper += (uint64_t)n;
    t->booked = (uint64_t)n;
    DevStatus* ds = reinterpret_cast<DevStatus*>(ptr);
    uint32_t* rows = reinterpret_cast<uint32_t*>(ptr + TN_STATIC_STATUS_BYTES);
    uint32_t* newlist = rows + TN_STATIC_MAX_SIGNS;
    const OptDev o = make_optdev(t);
    const int blocks = launch_grid(n, 256, GRID_CAP * 2);
    // the array keeps the last call's contents: the status block is cleared here, rows[0 .. n) and
    // newlist[0 .. new rows) are written by this call's probe before anything reads them
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, ds, (uint32_t)n, 0u);
    TN_LAUNCH((k_probe<true>), dim3(blocks), dim3(256), st, s, signs, n, (const DevStatus*)nullptr, 0u, rows, newlist, ds,
              (uint32_t)DEV_ERR_TABLE_FULL, o, t->seed);
    TN_LAUNCH(k_init_rows, dim3(blocks), dim3(256), st, s, o, t->seed, signs, rows, newlist, ds);
    TN_LAUNCH(k_finish_insert, dim3(1), dim3(64), st, s, ds);
    if (wdim % 4 == 0 && s.wstride % 4 == 0 && aligned16(out))
        TN_LAUNCH((k_gather_rows<4>), dim3(launch_grid(n * (wdim / 4), 256, GRID_CAP * 4)), dim3(256), st, s, rows, n, out);
    else
        TN_LAUNCH((k_gather_rows<1>), dim3(launch_grid(n * wdim, 256, GRID_CAP * 4)), dim3(256), st, s, rows, n, out);
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpull->st, ds, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    t->hpull->ubase[0] = 0;
    t->pull_pending = true;
    t->pull_slots = 0;
    t->pending_rows.clear();
    return sync_table(t, st);  // the scratch array is free again when the lock is released
}

int tn_sparse_table_push(uint32_t handle, const tn_sign_info* infos, const float* grads, int64_t n, int dim,
                         void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_push: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && (!infos || !grads))) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_push: NULL buffer");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    const int wdim = t->dim + (t->use_cvm ? 2 : 0);
    if (dim != wdim)
        return fail(TN_ERR_DIM_MISMATCH,
                    "tn_sparse_table_push: dim " + std::to_string(dim) + " but table rows hold " + std::to_string(wdim));
    if (n > 0x7FFFFFF0LL) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_push: more than 2^31 records");
    t->last_stream = st;
    if (n == 0) return TN_OK;
    if (t->push_pending || t->pull_pending) {  // one status block per direction: collect the previous one first
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    Plan p{};
    Scratch w{};
    {
        Carver probe{nullptr};
        carve_groups(probe, p, (size_t)n);
        carve_group_scratch(probe, w, (size_t)n);
        TN_TRY(t->ws.ensure(align_up(probe.off, 256) + 256));
        Carver c{(char*)t->ws.p};
        carve_groups(c, p, (size_t)n);
        carve_group_scratch(c, w, (size_t)n);
    }
    PushSrc src{};
    src.infos = infos;
    src.grads = grads;
    src.dim = dim;
    DevStatus* ds = t->dstatus;
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, ds, (uint32_t)n, (uint32_t)group_cap((size_t)n));
    launch_grouping(p, w, src, n, n, big_threshold(t->store), nullptr, ds, st);
    TN_LAUNCH((k_probe<false>), dim3(launch_grid(n, 256, GRID_CAP * 2)), dim3(256), st, t->store, p.grp_sign,
              (int64_t)0, ds, (uint32_t)n, p.grp_row, (uint32_t*)nullptr, ds, (uint32_t)DEV_ERR_UNKNOWN_KEY, make_optdev(t), t->seed);
    TN_TRY(launch_apply(t, p, src, ds, n, aligned16(grads) && dim % 4 == 0, st));
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpush->st, t->dstatus, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    t->push_pending = true;
    t->push_slots = 0;
    return TN_OK;
}

int tn_sparse_table_load_rows(uint32_t handle, const uint64_t* signs, const float* w, const float* state, int64_t n,
                              void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_load_rows: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && (!signs || !w))) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load_rows: NULL buffer");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    t->last_stream = st;
    if (n == 0) return TN_OK;
    if (n > 0x7FFFFFF0LL) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_load_rows: more than 2^31 rows per call");
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    TN_TRY(ensure_room(t, (uint64_t)n, st));
    TN_TRY(t->ws.ensure(2 * align_up((size_t)n * sizeof(uint32_t), 256)));
    Carver c{(char*)t->ws.p};
    uint32_t* rows = c.take<uint32_t>(n);
    uint32_t* newlist = c.take<uint32_t>(n);
    const Store& s = t->store;
    const int blocks = launch_grid(n, 256, GRID_CAP * 4);
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, t->dstatus, (uint32_t)n, 0u);
    TN_LAUNCH((k_probe<true>), dim3(blocks), dim3(256), st, s, signs, n, (const DevStatus*)nullptr, 0u, rows, newlist, t->dstatus, (uint32_t)DEV_ERR_TABLE_FULL, make_optdev(t), t->seed);
    TN_LAUNCH(k_finish_insert, dim3(1), dim3(64), st, s, t->dstatus);
    TN_LAUNCH(k_load_rows, dim3(blocks), dim3(256), st, s, make_optdev(t), rows, n, w, state);
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpull->st, t->dstatus, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    t->pull_pending = true;
    t->pull_slots = 0;
    t->pending_rows.clear();
    return sync_table(t, st);
}

int tn_sparse_table_export_rows(uint32_t handle, const uint64_t* signs, int64_t n, float* w, float* state,
                                uint8_t* found, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_export_rows: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && !signs)) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_export_rows: NULL buffer");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    t->last_stream = st;
    if (n == 0) return TN_OK;
    if (n > 0x7FFFFFF0LL) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_export_rows: more than 2^31 rows per call");
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    TN_TRY(t->ws.ensure(align_up((size_t)n * sizeof(uint32_t), 256)));
    uint32_t* rows = (uint32_t*)t->ws.p;
    const Store& s = t->store;
    const int blocks = launch_grid(n, 256, GRID_CAP * 4);
    TN_LAUNCH((k_probe<false>), dim3(blocks), dim3(256), st, s, signs, n, (const DevStatus*)nullptr, 0u, rows, (uint32_t*)nullptr, t->dstatus, 0u, make_optdev(t), t->seed);
    TN_LAUNCH(k_export_rows, dim3(blocks), dim3(256), st, s, make_optdev(t), rows, n, w, state, found);
    TN_HIP(hipGetLastError());
    TN_HIP(hipStreamSynchronize(st));
    return TN_OK;
}

namespace {
DecayConf make_decayconf(const SparseTable* t) {
    const OptConf& c = *t->opt;
    DecayConf d{};
    d.kind = c.kind;
    d.rate = c.show_decay_rate;
    d.show_threshold = c.show_threshold;
    d.no_show_days = c.no_show_days;
    d.elimination_logic = c.elimination_logic;
    return d;
}
}  // namespace

int tn_sparse_table_export_range(uint32_t handle, uint64_t first_slot, uint64_t n_slots, int skip_eliminated,
                                 uint64_t* signs, float* w, float* state, uint64_t* count, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_export_range: bad table handle " + std::to_string(handle));
    if (!count || (n_slots > 0 && (!signs || !w || !state)))
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_export_range: NULL buffer");
    if (n_slots > 0x7FFFFFF0ull) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_export_range: more than 2^31 slots per call");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    if (t->push_pending || t->pull_pending) {
        if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    *count = 0;
    const Store& s = t->store;
    if (n_slots == 0 || first_slot > s.cap) return TN_OK;
    TN_LAUNCH(k_reset_status, dim3(1), dim3(64), st, t->dstatus, 0u, 0u);
    TN_LAUNCH(k_export_range, dim3(launch_grid((int64_t)n_slots, 256, GRID_CAP * 4)), dim3(256), st, s, make_decayconf(t),
              first_slot, n_slots, skip_eliminated, signs, w, state, &t->dstatus->n_new);
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpull->st, t->dstatus, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    TN_HIP(hipStreamSynchronize(st));
    *count = t->hpull->st.n_new;
    return TN_OK;
}

int tn_sparse_table_name(uint32_t handle, char* name, int cap) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_name: bad table handle " + std::to_string(handle));
    if (!name || cap <= 0) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_name: NULL buffer");
    std::snprintf(name, (size_t)cap, "%s", t->name.c_str());
    return TN_OK;
}

int tn_sparse_table_optimizer(uint32_t handle, int* kind, int* use_cvm) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_optimizer: bad table handle " + std::to_string(handle));
    if (kind) *kind = t->opt->kind;
    if (use_cvm) *use_cvm = t->use_cvm ? 1 : 0;
    return TN_OK;
}

int tn_sparse_table_show_decay(uint32_t handle, int delta_days, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_show_decay: bad table handle " + std::to_string(handle));
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    if (t->push_pending || t->pull_pending) {
        if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    if (t->opt->kind == OPT_ADAM) return TN_OK;  // adam_kernel.h:67
    const Store& s = t->store;
    TN_LAUNCH(k_show_decay, dim3(launch_grid((int64_t)s.cap + 1, 256, GRID_CAP * 8)), dim3(256), st, s, make_decayconf(t),
              delta_days);
    TN_HIP(hipGetLastError());
    return TN_OK;
}

int tn_sparse_table_delete_by_show(uint32_t handle, const uint64_t* signs, int64_t n, uint8_t* out, void* stream) {
    SparseTable* t = get_table(handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "tn_sparse_table_delete_by_show: bad table handle " + std::to_string(handle));
    if (n < 0 || (n > 0 && (!signs || !out))) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_delete_by_show: NULL buffer");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    t->last_stream = st;
    if (n == 0) return TN_OK;
    if (n > 0x7FFFFFF0LL) return fail(TN_ERR_UNSUPPORTED, "tn_sparse_table_delete_by_show: more than 2^31 rows per call");
    if (t->push_pending || t->pull_pending) {
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    TN_TRY(t->ws.ensure(align_up((size_t)n * sizeof(uint32_t), 256)));
    uint32_t* rows = (uint32_t*)t->ws.p;
    const Store& s = t->store;
    const int blocks = launch_grid(n, 256, GRID_CAP * 4);
    TN_LAUNCH((k_probe<false>), dim3(blocks), dim3(256), st, s, signs, n, (const DevStatus*)nullptr, 0u, rows,
              (uint32_t*)nullptr, t->dstatus, 0u, make_optdev(t), t->seed);
    TN_LAUNCH(k_delete_by_show, dim3(blocks), dim3(256), st, s, make_decayconf(t), rows, n, out);
    TN_HIP(hipGetLastError());
    TN_HIP(hipStreamSynchronize(st));
    return TN_OK;
}

// --------------------------------------------------------------- op level
int tn_sparse_table_pull_op(uint32_t table_handle, int N, const int64_t* const* values, const int64_t* value_lens,
                            float* const* vars, const int64_t* var_rows, int var_dim, int64_t* const* mapped_values,
                            void* stream) {
    SparseTable* t = get_table(table_handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "SparseTablePull: bad table handle " + std::to_string(table_handle));
    if (!vars || !var_rows || !mapped_values) return fail(TN_ERR_INVALID_ARGUMENT, "SparseTablePull: NULL argument");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    // the call before was a push on the last pull's plan, on this stream: its updates may still be running
    bool behind_push = t->flow == FLOW_PUSH && t->flow_stream == st;
    // (detached updates of the push before: the analysis of this call's batch runs beside them; the stream is
    // ordered behind them where the call first touches what they read or write)
    TN_TRY(ensure_allocated(t, st, true));
    const int wdim = t->dim + (t->use_cvm ? 2 : 0);
    if (var_dim != wdim)
        return fail(TN_ERR_DIM_MISMATCH, "SparseTablePull: variable dim " + std::to_string(var_dim) +
                                             " but table rows hold " + std::to_string(wdim));
    // An earlier push on the same stream need not be waited for: this call runs behind it and
    // collects its status when it waits for its own work.
    const bool same_stream = !t->last_stream || t->last_stream == st;
    if (!same_stream || t->async_pull) TN_TRY(order_after_updates(t, st));
    if (t->pull_pending || (t->push_pending && (t->async_pull || !same_stream))) {
        if (!same_stream) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    // The remap through LDS needs the call's status on the host to fall back if a
    // bucket overflowed, so it is only used when the pull waits for its stream anyway.
    bool use_lds = !t->async_pull;
    bool small_allowed = true;
    for (int attempt = 0; attempt < 3; attempt++) {
        const double est_used = std::min(t->distinct_est, t->tile_est);  // what this attempt's buckets are sized from
        std::vector<SlotDesc> descs;
        std::vector<uint32_t> lbase;
        size_t L = 0, dt_entries = 0;
        uint32_t span_cap = 0;
        TN_TRY(stage_slots(t, N, values, value_lens, descs, lbase, L, dt_entries, "SparseTablePull", &use_lds,
                           &span_cap));
        bool vec = (wdim % 4 == 0) && (t->store.wstride % 4 == 0);
        for (int s = 0; s < N; s++) {
            if (var_rows[s] < 0 || !vars[s] || (value_lens[s] > 0 && !mapped_values[s]))
                return fail(TN_ERR_INVALID_ARGUMENT,
                            "sparse pull variable must Matrix(sign_id_cnt, dim), slot " + std::to_string(s));
            descs[s].var = vars[s];
            descs[s].rows = var_rows[s];
            descs[s].mapped = mapped_values[s];
            vec = vec && aligned16(vars[s]);
        }
        if (L == 0) {
            t->last_counts.assign(N, 0);
            return take_latched(t);
        }
        t->one_stream = L < ONE_STREAM_LOOKUPS;
        TN_TRY(ensure_room(t, (uint64_t)L, st));
        // a batch whose slots each fit one workgroup takes the path of few launches (small_batch.h)
        const bool small = small_allowed && small_batch_fits(t, N, value_lens, L, second_level_buckets(L, t->distinct_est));
        const bool lds_scratch = use_lds || small;
        if (small) dt_entries = 1;  // no first-level buckets
        Plan p{};
        Scratch w{};
        const bool exact = t->exact_verify && use_lds && !small;
        // (a plan buffer that has to grow is freed first: not under detached updates that still read it)
        if (t->upd_pending && carve_plan(nullptr, p, N, L, exact) > t->plan_buf.bytes)
            TN_HIP(hipEventSynchronize(t->upd_ev));
        TN_TRY(t->plan_buf.ensure(carve_plan(nullptr, p, N, L, exact)));
        carve_plan((char*)t->plan_buf.p, p, N, L, exact);
        TN_TRY(t->ws.ensure(carve_scratch(nullptr, w, L, dt_entries, lds_scratch, t->distinct_est, N)));
        carve_scratch((char*)t->ws.p, w, L, dt_entries, lds_scratch, t->distinct_est, N);
        w.span_cap = span_cap;
        t->plan_valid = false;
        // Detached updates of the push before read its plan in this same buffer.  A batch of the same slot count
        // and about the same size lays its plan out over it array by array, and what this call writes before it
        // orders itself behind them (the per-lookup arrays) stays clear of what they read; any other batch waits.
        // So does a call that keeps a copy of its signs for the exact comparison: the copy lies behind the group
        // arrays, where a batch of another size puts it on top of the gradient addresses the updates still read,
        // and the call's first kernel writes it.
        if (t->upd_pending && (exact || N != t->upd_N ||
                               (size_t)((const char*)p.grp_sign - (const char*)t->plan_buf.p) >
                                   t->upd_groups_off + t->upd_slack))
            TN_TRY(order_after_updates(t, st));
        if (small) {
            TN_TRY(order_after_updates(t, st));
            if (t->stage_pending) {
                TN_HIP(hipEventSynchronize(t->stage_ev));
                t->stage_pending = false;
            }
            std::memcpy(t->hstage, descs.data(), descs.size() * sizeof(SlotDesc));
            size_t max_len = 0;
            for (int s = 0; s < N; s++) max_len = std::max<size_t>(max_len, (size_t)value_lens[s]);
            const uint32_t entries = small_entries(max_len);
            const uint32_t set = t->small_calls++ & 1u;
            uint32_t* cur = t->small_state->cursor2[set];
            uint32_t* next = t->small_state->cursor2[set ^ 1u];
            const uint32_t seq = ++t->seq_pull;
            const Store& s = t->store;
            DevStatus* ds = t->dplan;
            uint32_t* prow = w.first_of;  // row of the slot's distinct sign of rank r at [first lookup of the slot + r]
            // workgroups per slot: about five hundred lookups' worth of table probes each, within the device's CUs
            uint32_t parts = (uint32_t)std::max<size_t>(1, std::min<size_t>(SMALL_PARTS_MAX, (max_len + 511) / 512));
            while (parts > 1 && (size_t)N * parts > (size_t)SMALL_SLOT_WORKGROUPS) parts--;
            TN_LAUNCH_LDS(k_small_slots, dim3(N * parts), dim3(SMALL_THREADS), small_slots_lds(entries, w.nb2), st,
                          reinterpret_cast<const SlotDesc*>(t->hstage), p.descs, p.lbase, N, (uint32_t)L, entries, s,
                          make_optdev(t), t->seed, p.vals_copy, p.u_of_gi, prow, w.nb2, cur, next, w.recs, w.rrow,
                          t->small_state, parts);
            const uint32_t big_k = N <= SMALL_NO_BIG_SLOTS || big_threshold(s) == 0xFFFFFFFFu ? 0xFFFFFFFFu : SMALL_BIG_GROUP;
            t->plan_big_k = big_k;
            t->plan_big_desc = false;  // (the small push's update kernel goes through big_list)
            // the grouping's first pass (one workgroup per second-level bucket) and, beside it, a thread per
            // (lookup position, part of a row) for the variables
            const int finish_blocks = (int)(((uint64_t)L * (uint64_t)(vec ? wdim / 4 : wdim) + GRP_THREADS - 1) / GRP_THREADS);
            if (vec)
                TN_LAUNCH((k_small_group_finish<4>), dim3(w.nb2 + finish_blocks), dim3(GRP_THREADS), st, w.nb2, cur, w.recs,
                          big_k, w.aux, w.bcounts, s, p.descs, p.lbase, p.ubase, N, (uint32_t)L, prow, p.u_of_gi,
                          t->small_state, parts, ds, reinterpret_cast<uint32_t*>(t->hpull), t->hseq + 0, seq);
            else
                TN_LAUNCH((k_small_group_finish<1>), dim3(w.nb2 + finish_blocks), dim3(GRP_THREADS), st, w.nb2, cur, w.recs,
                          big_k, w.aux, w.bcounts, s, p.descs, p.lbase, p.ubase, N, (uint32_t)L, prow, p.u_of_gi,
                          t->small_state, parts, ds, reinterpret_cast<uint32_t*>(t->hpull), t->hseq + 0, seq);
            TN_LAUNCH((k_group_emit<true>), dim3(w.nb2), dim3(EMIT_THREADS), st, w.nb2, cur, w.recs, w.aux,
                      (const uint4*)nullptr, w.bcounts, (const uint8_t*)nullptr, (const uint32_t*)nullptr, (uint32_t)L,
                      big_k, p.grp_sign, p.grp_off, p.grp_cnt, p.big_list, p.big_desc, p.list, p.where_u, w.rrow,
                      p.grp_row, ds, p.ubase, (uint32_t)N);
            TN_HIP(hipGetLastError());
            // the call returns when the second launch has reported: what follows is complete in stream order
            TN_HIP(hipEventRecord(t->tail_ev, st));
            t->tail_recorded = true;
            t->pull_pending = true;
            t->pull_slots = N;
            t->pull_lookups = (uint64_t)L;
            t->pending_rows.assign(var_rows, var_rows + N);
            t->plan_valid = true;
            t->plan_small = true;
            t->plan_clicks_dirty = false;
            t->plan_has_show = true;
            t->plan_prints = false;
            t->plan_exact = false;
            t->plan_N = N;
            t->plan_lens.assign(value_lens, value_lens + N);
            t->plan_epoch = t->epoch;
            TN_TRY(wait_reported(t->hseq + 0, seq, st, "SparseTablePull"));
            if (t->hpull->st.err & DEV_ERR_REMAP_OVERFLOW) {
                // a second-level bucket overflowed (more distinct records than the recent pulls had): once more
                // with buckets for a batch of distinct signs only, then on the other paths
                t->hpull->st.err &= ~DEV_ERR_REMAP_OVERFLOW;
                harvest(t);
                if (est_used >= 1.0) small_allowed = false;
                t->distinct_est = 1.0;
                t->tile_est = 1.0;
                t->latched = TN_OK;
                t->latched_msg.clear();
                continue;
            }
            harvest(t);
            t->plan_counts = t->last_counts;
            return take_latched(t);
        }
        t->plan_small = false;
        t->plan_big_k = big_threshold(t->store);
        t->plan_big_desc = false;
        // Behind a push of the training loop the descriptors go in on the auxiliary stream, beside that push's
        // updates: those read the push's own descriptors and status block, and nothing of the scratch buffer.
        // (Same slot count: the arrays at the head of the plan buffer keep their places.)
        const bool hoist = behind_push && attempt == 0 && !t->one_stream && N == t->plan_N && !t->upd_pending;
        behind_push = false;
        if (hoist && t->tail_recorded) TN_HIP(hipStreamWaitEvent(t->aux, t->tail_ev, 0));  // the gather that read p.descs
        TN_TRY(upload_slots(t, p.descs, p.lbase, t->dplan, descs, lbase, hoist ? t->aux : st, STATUS_NEW_PLAN,
                            use_lds ? w.bcursor : nullptr, use_lds ? w.nbuckets + 1 + w.nb2 : 0));
        if (hoist) TN_HIP(hipStreamWaitEvent(st, t->stage_ev, 0));

        const Store& s = t->store;
        DevStatus* ds = t->dplan;
        TN_TRY(launch_build_plan(t, p, w, N, (uint32_t)L, true, use_lds, st));
        // The grouping through LDS leaves the row of every distinct record in where_u itself, and the
        // call's status (counts, new rows, errors) is final before the gather starts: it is published
        // on the side stream beside the gather, and the call returns when the host has it.  The
        // variables are complete in stream order, as the outputs of any call that takes a stream.
        const bool final_early = use_lds && N <= GRP_SLOTS && !t->async_pull;
        const bool early = final_early && !t->one_stream;
        // A call that keeps to the caller's stream publishes there, ahead of the gather, and tells the host through
        // a word in pinned memory: the host prepares the push while the gather runs.
        const bool early_inline = final_early && t->one_stream;
        const uint32_t seq = early_inline ? ++t->seq_pull : 0;
        const uint32_t* rows_of_groups = (use_lds && N <= GRP_SLOTS) ? nullptr : p.grp_row;
        if (early) TN_HIP(hipEventRecord(t->ready_ev, st));
        if (early_inline)
            TN_LAUNCH(k_publish, dim3(1), dim3(256), st, ds, p.ubase, (uint32_t)(N + 1),
                      reinterpret_cast<uint32_t*>(t->hpull), s.count, t->hseq + 0, seq);
        if (vec)
            TN_LAUNCH((k_gather_vars<4>), dim3(launch_grid((int64_t)L * (wdim / 4), 256, GRID_CAP * 4)), dim3(256), st, s,
                      ds, rows_of_groups, p.where_u, p.ubase, N, p.descs);
        else
            TN_LAUNCH((k_gather_vars<1>), dim3(launch_grid((int64_t)L * wdim, 256, GRID_CAP * 4)), dim3(256), st, s, ds,
                      rows_of_groups, p.where_u, p.ubase, N, p.descs);
        TN_HIP(hipGetLastError());
        if (early || early_inline) {
            TN_HIP(hipEventRecord(t->tail_ev, st));
            t->tail_recorded = true;
        }
        if (early) TN_HIP(hipStreamWaitEvent(t->side, t->ready_ev, 0));
        if (!early_inline)
            TN_LAUNCH(k_publish, dim3(1), dim3(256), early ? t->side : st, ds, p.ubase, (uint32_t)(N + 1),
                      reinterpret_cast<uint32_t*>(t->hpull), s.count, (uint32_t*)nullptr, 0u);
        if (early) TN_HIP(hipEventRecord(t->pub_ev, t->side));
        t->pull_pending = true;
        t->pull_slots = N;
        t->pull_lookups = (uint64_t)L;
        t->pending_rows.assign(var_rows, var_rows + N);
        // a push of the same batch may reuse the analysis
        t->plan_valid = true;
        t->plan_clicks_dirty = false;  // a new plan's click sums start at zero
        t->plan_has_show = use_lds;
        t->plan_prints = use_lds;
        t->plan_exact = exact;
        t->plan_N = N;
        t->plan_lens.assign(value_lens, value_lens + N);
        t->plan_epoch = t->epoch;
        if (t->async_pull) return TN_OK;
        if (early)
            TN_HIP(hipEventSynchronize(t->pub_ev));
        else if (early_inline)
            TN_TRY(wait_reported(t->hseq + 0, seq, st, "SparseTablePull"));
        else
            TN_HIP(hipStreamSynchronize(st));
        if (use_lds && (t->hpull->st.err & DEV_ERR_REMAP_OVERFLOW)) {
            // rows the failed attempt inserted belong to signs of this batch; keep them counted
            t->hpull->st.err &= ~DEV_ERR_REMAP_OVERFLOW;
            harvest(t);
            // The batch had more distinct records than the buckets were sized for (the share of the recent pulls
            // plus a quarter).  Sized for a batch of distinct signs only, a bucket cannot overflow short of an
            // adversarial hash (first level: 768 lookups for 2048 entries; second level: 1024 records expected
            // in room for 1536), so the call is repeated through LDS once more -- at the cost of a pull, not of
            // the global-table path, which remains for the batch that overflows even then.
            if (est_used >= 1.0) use_lds = false;
            t->distinct_est = 1.0;
            t->tile_est = 1.0;
            t->latched = TN_OK;
            t->latched_msg.clear();
            continue;
        }
        if (early) {
            t->push_pub_on_side = false;  // a push's status went out on the side stream ahead of this call's
            harvest(t);
            t->flow = FLOW_PULL;
            t->flow_stream = st;
            return take_latched(t);
        }
        if (early_inline) {
            harvest(t);
            return take_latched(t);
        }
        return sync_table(t, st);
    }
    return fail(TN_ERR_HIP, "SparseTablePull: remap fell back three times");
}

}  // extern "C"

namespace {

// SparseTablePush.  With example_ids the gradients are pooled ([batch, dim] per slot, one row per
// example): they are first reduced to one row per distinct sign (the gradient of the combiner).
int push_op_impl(uint32_t table_handle, int N, const int64_t* const* values, const int64_t* value_lens,
                 const float* const* grads, const int64_t* grad_rows, int grad_dim,
                 const int64_t* const* feature_labels, const int64_t* const* example_ids, int64_t batch, int combiner,
                 void* stream) {
    SparseTable* t = get_table(table_handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "SparseTablePush: bad table handle " + std::to_string(table_handle));
    if (!grads || (!grad_rows && !example_ids) || !feature_labels)
        return fail(TN_ERR_INVALID_ARGUMENT, "SparseTablePush: NULL argument");
    const bool pooled = example_ids != nullptr;
    if (pooled && (batch <= 0 || combiner < COMBINE_SUM || combiner > COMBINE_SQRTN))
        return fail(TN_ERR_INVALID_ARGUMENT, "SparseTablePush (pooled): bad batch size or combiner");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    // the call before was a pull on this stream that returned before its gather
    const bool behind_pull = t->flow == FLOW_PULL && t->flow_stream == st;
    TN_TRY(ensure_allocated(t, st));
    const int wdim = t->dim + (t->use_cvm ? 2 : 0);
    if (grad_dim != wdim)
        return fail(TN_ERR_DIM_MISMATCH, "SparseTablePush: gradient dim " + std::to_string(grad_dim) +
                                             " but table rows hold " + std::to_string(wdim));
    std::vector<SlotDesc> descs;
    std::vector<uint32_t> lbase;
    size_t L = 0, dt_entries = 0;
    TN_TRY(stage_slots(t, N, values, value_lens, descs, lbase, L, dt_entries, "SparseTablePush", nullptr));
    bool vec = (grad_dim % 4 == 0);
    for (int s = 0; s < N; s++) {
        const int64_t rows = pooled ? batch : grad_rows[s];
        if (rows < 0 || (rows > 0 && !grads[s]) || (value_lens[s] > 0 && !feature_labels[s]) ||
            (pooled && value_lens[s] > 0 && !example_ids[s]))
            return fail(TN_ERR_INVALID_ARGUMENT,
                        "sparse push grad must Matrix(sign_id_cnt, dim), slot " + std::to_string(s));
        descs[s].grads = grads[s];
        descs[s].rows = rows;
        descs[s].labels = feature_labels[s];
        if (pooled) descs[s].mapped = const_cast<int64_t*>(example_ids[s]);  // example index of every lookup
        vec = vec && aligned16(grads[s]);
    }
    if (t->push_pending || t->pull_pending) {
        // a call pending on another stream (an asynchronous pull) builds the plan this push reads
        if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    if (L == 0) return TN_OK;
    t->one_stream = L < ONE_STREAM_LOOKUPS;
    Plan p{};
    Scratch w{};
    // Same batch as the last pull?  Necessary conditions on the host, the signs
    // themselves are compared on the device.
    bool reuse = t->plan_valid && t->plan_epoch == t->epoch && t->plan_N == N &&
                 std::equal(value_lens, value_lens + N, t->plan_lens.begin());
    // A push on the last pull's plan has its own descriptors and status block (the plan's counts, flags of its
    // own): the pull's gather may still be running, and the next pull may stage its slots while this push's
    // updates run.  A push that analyses its batch itself uses the plan's.
    DevStatus* ds = reuse ? t->dpush : t->dplan;
    const SlotDesc* pd = nullptr;  // set with the plan
    const int lblocks = launch_grid(L, 256, GRID_CAP * 2);
    const bool with_click = t->opt->kind == OPT_ADAGRAD;  // the only optimizer that reads batch_click
    // show / click counts of the batch into the member lists of a plan that has none
    auto launch_counts = [&]() -> int {
        TN_LAUNCH(k_reset_counts, dim3(lblocks), dim3(256), st, p.list, ds, (uint32_t)L, 0);
        TN_LAUNCH(k_count_show, dim3(launch_grid((int64_t)(L + COUNT_TILE - 1) / COUNT_TILE, 1, GRID_CAP)), dim3(256),
                  st, pd, p.lbase, N, (uint32_t)L, p.u_of_gi, p.where_u, p.list, with_click ? 1 : 0);
        return TN_OK;
    };
    // Where the apply kernels find the gradient of a record.  Pooled gradients are first reduced
    // to one row per distinct sign: stable sort of (distinct index, position) pairs, then one
    // ordered sum per distinct index.
    PushSrc src{};
    const uint32_t* pub_ubase = nullptr;  // a push on the pull's plan publishes its own copy of the distinct counts
    auto prepare_src = [&]() -> int {
        src = op_source(p, grad_dim, pd == p.push_descs);
        if (!pooled) return TN_OK;
        if (!t->place_lds) {
            t->place_lds = big_lds_bytes_for(reinterpret_cast<const void*>(k_place_lookups));
            t->huge_lds = big_lds_bytes_for(reinterpret_cast<const void*>(k_order_huge));
        }
        const bool huge_in_lds = (size_t)batch * sizeof(uint32_t) <= t->huge_lds;
        const int huge_grid = huge_in_lds ? GRID_CAP : 64;
        Carver c{nullptr};
        uint32_t *long_count, *gcur, *seg_off, *tkey, *mid_list, *huge_list, *gcnt;
        uint64_t *vals, *svals, *tval;
        float* flat;
        auto carve = [&](Carver& cv) {
            long_count = cv.take<uint32_t>(4);  // [1], [2]: entries of the lists of k_place_lookups (mid, huge)
            mid_list = cv.take<uint32_t>(L / ORDER_MID + 1);
            huge_list = cv.take<uint32_t>(L / ORDER_HUGE + 1);
            gcur = cv.take<uint32_t>(L);
            tkey = cv.take<uint32_t>(L);
            vals = cv.take<uint64_t>(L);
            tval = cv.take<uint64_t>(L);
            svals = cv.take<uint64_t>(L);
            seg_off = cv.take<uint32_t>(L + 1);
            flat = cv.take<float>(L * (size_t)grad_dim);
            gcnt = cv.take<uint32_t>(huge_in_lds ? 0 : (size_t)huge_grid * (size_t)batch);
        };
        carve(c);
        TN_TRY(t->pooled_ws.ensure(align_up(c.off, 256)));
        Carver c2{(char*)t->pooled_ws.p};
        carve(c2);
        TN_LAUNCH(k_lookup_keys, dim3(lblocks), dim3(256), st, pd, p.lbase, N, (uint32_t)L, batch, vals, ds, long_count);
        // The lookups of every distinct sign side by side, ascending by example (= by position): into their
        // sign's segment first, then ordered inside it.  A few workgroups per slot, each with an LDS counter per
        // distinct index of its share of the slot (a slot has at most as many as lookups).
        size_t max_len = 0;
        for (int s = 0; s < N; s++) max_len = std::max<size_t>(max_len, (size_t)value_lens[s]);
        // (one workgroup per slot: with several, each streaming the slot for its share of the distinct indices,
        // the kernel took longer -- 0.20 against 0.17 ms with five, 0.16 with two -- as did a split by position,
        // which needs a matrix of counts)
        const uint32_t parts = 1;
        const size_t place_bytes = std::min(t->place_lds, align_up((max_len / parts + 2) * sizeof(uint32_t), 256));
        const uint32_t place_cap = (uint32_t)(place_bytes / sizeof(uint32_t));
        TN_LAUNCH_LDS(k_place_lookups, dim3(N * parts), dim3(PLACE_THREADS), place_bytes, st, p.lbase, p.ubase, N, (uint32_t)L,
                      p.u_of_gi, vals, tkey, tval, seg_off, gcur, place_cap, mid_list, huge_list, long_count, ds, parts);
        // The three kernels that order the segments work on segments of their own (short, middle, huge), the two
        // that sum them likewise (those below LONG_SEGMENT lookups, those from it on): a large batch runs them side
        // by side on the table's streams.
        const bool fork = !t->one_stream;
        hipStream_t s_mid = fork ? t->side : st, s_huge = fork ? t->side2 : st;
        if (fork) {
            TN_HIP(hipEventRecord(t->fork_ev, st));
            TN_HIP(hipStreamWaitEvent(t->side, t->fork_ev, 0));
            TN_HIP(hipStreamWaitEvent(t->side2, t->fork_ev, 0));
        }
        TN_LAUNCH(k_rank_short, dim3(launch_grid(L, 256, GRID_CAP * 4)), dim3(256), st, (uint32_t)L, tkey, tval, seg_off,
                  svals, ds);
        TN_LAUNCH(k_rank_mid, dim3(launch_grid((int64_t)L / ORDER_MID + 1, 1, GRID_CAP * 2)), dim3(256), s_mid, mid_list,
                  long_count, seg_off, tval, svals, ds);
        TN_LAUNCH_LDS(k_order_huge, dim3(launch_grid((int64_t)L / ORDER_HUGE + 1, 1, huge_grid)), dim3(256),
                      huge_in_lds ? (size_t)batch * sizeof(uint32_t) : 0, s_huge, huge_list, long_count, seg_off, tval, svals,
                      (uint32_t)batch, huge_in_lds ? 1 : 0, gcnt, ds);
        // signs with LONG_SEGMENT lookups or more get a workgroup each instead of one thread group
        static_assert(LONG_SEGMENT == ORDER_MID, "the lists of k_place_lookups are the frequent signs of k_reduce_long");
        const int chunks = vec ? grad_dim / 4 : grad_dim;
        const uint32_t long_min = chunks <= 256 ? LONG_SEGMENT : 0xFFFFFFFFu;
        const int long_blocks = launch_grid((int64_t)L / LONG_SEGMENT + 1, 1, GRID_CAP);
        if (fork) {
            // the frequent signs are summed on the side stream, behind the two kernels that ordered their segments
            TN_HIP(hipEventRecord(t->join2_ev, t->side2));
            TN_HIP(hipStreamWaitEvent(t->side, t->join2_ev, 0));
        }
        if (vec) {
            TN_LAUNCH((k_reduce_pooled<4>), dim3(launch_grid((int64_t)L * chunks, 256, GRID_CAP * 4)), dim3(256), st,
                      pd, p.ubase, N, grad_dim, combiner, ds, seg_off, svals, flat, long_min);
            TN_LAUNCH((k_reduce_long<4>), dim3(long_blocks), dim3(256), s_mid, pd, p.ubase, N, grad_dim, combiner,
                      seg_off, svals, flat, mid_list, huge_list, long_count, ds);
        } else {
            TN_LAUNCH((k_reduce_pooled<1>), dim3(launch_grid((int64_t)L * chunks, 256, GRID_CAP * 4)), dim3(256), st,
                      pd, p.ubase, N, grad_dim, combiner, ds, seg_off, svals, flat, long_min);
            if (long_min != 0xFFFFFFFFu)
                TN_LAUNCH((k_reduce_long<1>), dim3(long_blocks), dim3(256), s_mid, pd, p.ubase, N, grad_dim,
                          combiner, seg_off, svals, flat, mid_list, huge_list, long_count, ds);
        }
        if (fork) {
            TN_HIP(hipEventRecord(t->join_ev, t->side));
            TN_HIP(hipStreamWaitEvent(st, t->join_ev, 0));
        }
        src.flat = flat;
        return TN_OK;
    };
    const int small_lpg = lanes_per_group(t->store, vec && t->store.wstride % 4 == 0);
    if (reuse && t->plan_small && t->small_path && !pooled && small_lpg != 0 && N <= SMALL_SLOTS) {
        // A small batch on the plan of its small pull: slot descriptors, comparison of the signs and click sums by
        // one launch, the updates by one or two more (small_batch.h).  The call's status block is the plan's:
        // nothing of the next call runs beside this one.  The device has nothing to report: every sign of the plan
        // has its row, and whether a gradient matrix has a row for every distinct sign of its slot is known here.
        carve_plan((char*)t->plan_buf.p, p, N, L);
        pd = p.push_descs;
        ds = t->dplan;
        if (t->stage_pending) {
            TN_HIP(hipEventSynchronize(t->stage_ev));
            t->stage_pending = false;
        }
        std::memcpy(t->hstage, descs.data(), descs.size() * sizeof(SlotDesc));
        t->hpush->st.mismatch = 0;
        const bool clicks = with_click;  // (a small pull's plan has the show counts)
        if (clicks) {
            if (t->plan_clicks_dirty)
                TN_LAUNCH(k_reset_counts, dim3(lblocks), dim3(256), st, p.list, ds, (uint32_t)L, 1);
            t->plan_clicks_dirty = true;
        }
        const uint32_t seq_v = ++t->seq_verify;
        const int tiles = (int)((L + SMALL_TILE - 1) / SMALL_TILE);
        const size_t vlds = ((size_t)N + 1) * sizeof(uint32_t);
        if (clicks)
            TN_LAUNCH_LDS((k_small_verify<true>), dim3(tiles), dim3(256), vlds, st,
                          reinterpret_cast<const SlotDesc*>(t->hstage), p.push_descs, p.lbase, N, (uint32_t)L, p.vals_copy,
                          ds, p.u_of_gi, p.where_u, p.list, &t->hpush->st.mismatch);
        else
            TN_LAUNCH_LDS((k_small_verify<false>), dim3(tiles), dim3(256), vlds, st,
                          reinterpret_cast<const SlotDesc*>(t->hstage), p.push_descs, p.lbase, N, (uint32_t)L, p.vals_copy,
                          ds, p.u_of_gi, p.where_u, p.list, &t->hpush->st.mismatch);
        // (the small path stages no copy of the slots' bases: its kernels all run on the caller's stream, ahead of
        // whatever rewrites the plan's)
        PushSrc small_src = op_source(p, grad_dim, true);
        small_src.ubase = p.ubase;
        TN_TRY(launch_small_apply(t, small_lpg, N, small_src, ds, p, (int64_t)L, st, t->hseq + 1, seq_v));
        // what a call on another stream has to wait for: the updates are still running when this call returns
        TN_HIP(hipEventRecord(t->tail_ev, st));
        t->tail_recorded = true;
        TN_HIP(hipGetLastError());
        // the outcome of the comparison: the updates are queued behind it and do nothing on a mismatch
        TN_TRY(wait_reported(t->hseq + 1, seq_v, st, "SparseTablePush"));
        if (t->hpush->st.mismatch == 0) {
            t->last_counts = t->plan_counts;
            // (the records without a gradient row were left out by the update kernel, as on the other paths)
            for (int s = 0; s < N; s++)
                if (grad_rows[s] < t->plan_counts[s])
                    return fail(TN_ERR_INVALID_ARGUMENT, std::string("sparse push: ") + dev_err_text(DEV_ERR_GRAD_ROWS) +
                                                             " (slot " + std::to_string(s) + ")");
            return TN_OK;
        }
        reuse = false;  // another batch than the last pull's: analysed below
    } else if (reuse) {
        carve_plan((char*)t->plan_buf.p, p, N, L, t->plan_exact);
        pd = p.push_descs;
        // behind a pull that returned before its gather the descriptors go in on the auxiliary stream, beside
        // that gather (the plan's counts are final from ready_ev on)
        const bool hoist = behind_pull && !t->one_stream;
        if (hoist) TN_HIP(hipStreamWaitEvent(t->aux, t->ready_ev, 0));
        TN_TRY(upload_slots(t, p.push_descs, nullptr, ds, descs, lbase, hoist ? t->aux : st, STATUS_REUSE_PLAN, nullptr, 0,
                            p.ubase, p.push_ubase, (uint32_t)(N + 1)));
        pub_ubase = p.push_ubase;
        if (hoist) TN_HIP(hipStreamWaitEvent(st, t->stage_ev, 0));
        // On a plan with show counts the verify pass also sums the clicks; they start at zero
        // after the pull, a further push on the same plan clears them first.
        const bool clicks = t->plan_has_show && with_click;
        const int vblocks = launch_grid((int64_t)(L + VERIFY_TILE - 1) / VERIFY_TILE, 1, GRID_CAP * 2);
        const size_t vlds = ((size_t)N + 1) * sizeof(uint32_t);
        // the outcome comes back through pinned host memory, written by the verify kernel itself
        t->hpush->st.mismatch = 0;
        uint32_t* host_mismatch = &t->hpush->st.mismatch;
        // op-level gradients (not pooled): the verify pass also works out the gradient addresses of the records
        // of the groups with several records (see k_member_grads)
        const PushSrc vsrc = op_source(p, grad_dim, true);
        const bool addr_in_verify = !pooled && t->plan_big_k != 0xFFFFFFFFu;
        const float** vgaddr = addr_in_verify ? p.gaddr : nullptr;
        // (a macro: the profiler names a kernel by the text of its launch)
#define TN_VERIFY(CLICKS, COPY)                                                                                      \
    TN_LAUNCH_LDS((k_verify_values<CLICKS, COPY>), dim3(vblocks), dim3(256), vlds, st, pd, p.lbase, N, (uint32_t)L, \
                  then_vals, ds, p.u_of_gi, p.where_u, p.list, host_mismatch, vsrc, vgaddr)
        const bool copy = !t->plan_prints || t->plan_exact;
        const uint64_t* then_vals = t->plan_exact ? p.vals_exact : p.vals_copy;
        if (clicks) {
            if (t->plan_clicks_dirty)
                TN_LAUNCH(k_reset_counts, dim3(lblocks), dim3(256), st, p.list, ds, (uint32_t)L, 1);
            t->plan_clicks_dirty = true;
            if (copy)
                TN_VERIFY(true, true);
            else
                TN_VERIFY(true, false);
        } else if (copy) {
            TN_VERIFY(false, true);
        } else {
            TN_VERIFY(false, false);
        }
#undef TN_VERIFY
        TN_HIP(hipEventRecord(t->verify_ev, st));
        // Counts and apply kernels are queued before the host knows the outcome: the counts only
        // touch the plan's member lists, which a mismatch discards anyway, and the apply kernels
        // return at once when the mismatch flag is set.  The device never waits for the host.
        if (!t->plan_has_show) TN_TRY(launch_counts());
        TN_TRY(prepare_src());
        TN_TRY(launch_apply(t, p, src, ds, (int64_t)L, vec, st, addr_in_verify, t->plan_big_k,
                            t->detach_updates && !pooled, t->plan_big_desc));
        if (t->detached_now) {
            // their end, for whoever touches the table next; the status goes out behind them (below)
            TN_HIP(hipEventRecord(t->apply_ev, t->aux));
            TN_HIP(hipStreamWaitEvent(t->side, t->apply_ev, 0));
        }
        TN_HIP(hipEventSynchronize(t->verify_ev));
        reuse = t->hpush->st.mismatch == 0;
        if (t->detached_now && !reuse) {
            // (the update kernels return at once on a mismatch; what follows works on the caller's stream)
            TN_HIP(hipEventRecord(t->upd_ev, t->side));
            t->upd_pending = true;
            t->detached_now = false;
            TN_TRY(order_after_updates(t, st));
        }
    }
    if (!reuse) {
        // another batch than the last pull's: analyse it here, on the global-table path
        // (its status cannot be waited for, a push only enqueues)
        t->plan_valid = false;
        ds = t->dplan;
        pub_ubase = nullptr;
        TN_TRY(t->plan_buf.ensure(carve_plan(nullptr, p, N, L)));
        carve_plan((char*)t->plan_buf.p, p, N, L);
        pd = p.descs;
        TN_TRY(t->ws.ensure(carve_scratch(nullptr, w, L, dt_entries, false)));
        carve_scratch((char*)t->ws.p, w, L, dt_entries, false);
        TN_TRY(upload_slots(t, p.descs, p.lbase, ds, descs, lbase, st, STATUS_NEW_PLAN));
        TN_TRY(launch_build_plan(t, p, w, N, (uint32_t)L, false, false, st));
        TN_TRY(launch_counts());
        TN_TRY(prepare_src());
        TN_TRY(launch_apply(t, p, src, ds, (int64_t)L, vec, st));
    }
    TN_HIP(hipGetLastError());
    // The status of a large push goes out on the side stream, behind the updates and beside whatever the caller's
    // stream runs next (a pull's status follows it on that stream, so whoever has that one has this one too).
    const bool pub_on_side = reuse && !t->one_stream;
    const bool detached = reuse && t->detached_now;  // (the side stream is behind all update kernels already)
    t->detached_now = false;
    if (pub_on_side && !detached) {
        TN_HIP(hipEventRecord(t->apply_ev, st));
        TN_HIP(hipStreamWaitEvent(t->side, t->apply_ev, 0));
    }
    TN_LAUNCH(k_publish, dim3(1), dim3(256), pub_on_side ? t->side : st, ds, pub_ubase ? pub_ubase : p.ubase,
              (uint32_t)(N + 1), reinterpret_cast<uint32_t*>(t->hpush), (unsigned long long*)nullptr, (uint32_t*)nullptr, 0u);
    if (detached) {
        TN_HIP(hipEventRecord(t->upd_ev, t->side));
        t->upd_pending = true;
        t->upd_N = N;
        t->upd_groups_off = (size_t)((const char*)p.grp_sign - (const char*)t->plan_buf.p);
        t->upd_slack = (size_t)((const char*)p.grp_row - (const char*)p.grp_sign);
    }
    t->push_pending = true;
    t->push_pub_on_side = pub_on_side;
    t->push_slots = N;
    // (the reduction of pooled gradients reads the plan's slot layout until the end of the call: nothing of the
    // next pull may run beside it)
    if (reuse && !pooled) {
        t->flow = FLOW_PUSH;
        t->flow_stream = st;
    }
    return TN_OK;
}

}  // namespace

extern "C" {

int tn_sparse_table_push_op(uint32_t table_handle, int N, const int64_t* const* values, const int64_t* value_lens,
                            const float* const* grads, const int64_t* grad_rows, int grad_dim,
                            const int64_t* const* feature_labels, void* stream) {
    return push_op_impl(table_handle, N, values, value_lens, grads, grad_rows, grad_dim, feature_labels, nullptr, 0, 0,
                        stream);
}

int tn_sparse_table_push_pooled_op(uint32_t table_handle, int N, const int64_t* const* values,
                                   const int64_t* value_lens, const int64_t* const* example_ids,
                                   const float* const* pooled_grads, int64_t batch, int grad_dim, int combiner,
                                   const int64_t* const* feature_labels, void* stream) {
    if (!example_ids) return fail(TN_ERR_INVALID_ARGUMENT, "SparseTablePush (pooled): NULL argument");
    return push_op_impl(table_handle, N, values, value_lens, pooled_grads, nullptr, grad_dim, feature_labels, example_ids,
                        batch, combiner, stream);
}

int tn_sparse_table_combine_op(uint32_t table_handle, int N, const int64_t* const* mapped_values,
                               const int64_t* value_lens, const int64_t* const* example_ids, const float* const* vars,
                               const int64_t* var_rows, int dim, int64_t batch, int combiner, float* const* out,
                               void* stream) {
    SparseTable* t = get_table(table_handle);
    if (!t) return fail(TN_ERR_BAD_HANDLE, "embedding combine: bad table handle " + std::to_string(table_handle));
    if (!mapped_values || !value_lens || !example_ids || !vars || !var_rows || !out || N <= 0)
        return fail(TN_ERR_INVALID_ARGUMENT, "embedding combine: NULL argument");
    if (N > MAX_SLOTS) return fail(TN_ERR_UNSUPPORTED, "embedding combine: too many slots");
    if (dim <= 0 || batch <= 0 || combiner < COMBINE_SUM || combiner > COMBINE_SQRTN)
        return fail(TN_ERR_INVALID_ARGUMENT, "embedding combine: bad dim, batch size or combiner");
    std::lock_guard<std::mutex> lk(t->mu);
    hipStream_t st = (hipStream_t)stream;
    TN_TRY(ensure_allocated(t, st));
    std::vector<SlotDesc> descs(N, SlotDesc{});
    std::vector<uint32_t> lbase(N + 1, 0);
    size_t L = 0;
    bool vec = dim % 4 == 0;
    for (int s = 0; s < N; s++) {
        if (value_lens[s] < 0 || var_rows[s] < 0 || !out[s] ||
            (value_lens[s] > 0 && (!mapped_values[s] || !example_ids[s] || !vars[s])))
            return fail(TN_ERR_INVALID_ARGUMENT, "embedding combine: bad tensors of slot " + std::to_string(s));
        SlotDesc& d = descs[s];
        d.values = mapped_values[s];
        d.mapped = const_cast<int64_t*>(example_ids[s]);
        d.grads = vars[s];
        d.var = out[s];
        d.rows = var_rows[s];
        d.len = (uint32_t)value_lens[s];
        d.lbase = (uint32_t)L;
        lbase[s] = (uint32_t)L;
        L += (size_t)value_lens[s];
        if (L > 0x7FFFFFF0ull) return fail(TN_ERR_UNSUPPORTED, "embedding combine: more than 2^31 lookups in one call");
        vec = vec && aligned16(vars[s]) && aligned16(out[s]);
    }
    lbase[N] = (uint32_t)L;
    // an earlier call's status is collected first: this call uses the table's status block
    if (t->push_pending || t->pull_pending) {
        if (t->last_stream && t->last_stream != st) TN_HIP(hipStreamSynchronize(t->last_stream));
        TN_HIP(hipStreamSynchronize(st));
        harvest(t);
    }
    t->last_stream = st;
    {
        const size_t db = (size_t)N * sizeof(SlotDesc), lb = (size_t)(N + 1) * sizeof(uint32_t);
        const size_t rp = (size_t)N * (size_t)(batch + 1) * sizeof(uint32_t);
        TN_TRY(t->comb_buf.ensure(align_up(db, 256) + align_up(lb, 256) + rp));
        SlotDesc* ddescs = (SlotDesc*)t->comb_buf.p;
        uint32_t* dlbase = (uint32_t*)((char*)t->comb_buf.p + align_up(db, 256));
        uint32_t* rowptr = (uint32_t*)((char*)dlbase + align_up(lb, 256));
        if (t->stage_pending) {
            TN_HIP(hipEventSynchronize(t->stage_ev));
            t->stage_pending = false;
        }
        std::memcpy(t->hstage, descs.data(), db);
        std::memcpy(t->hstage + db, lbase.data(), lb);
        TN_LAUNCH(k_stage_in, dim3(launch_grid((int64_t)(db + lb) / 4, 256, 64)), dim3(256), st,
                  reinterpret_cast<const uint32_t*>(t->hstage), reinterpret_cast<uint32_t*>(ddescs), (uint32_t)(db / 4),
                  dlbase, (uint32_t)(lb / 4), t->dstatus, (int)STATUS_NEW_PLAN, (uint32_t*)nullptr, 0u,
                  (const DevStatus*)t->dstatus, (const uint32_t*)nullptr, (uint32_t*)nullptr, 0u);
        TN_HIP(hipEventRecord(t->stage_ev, st));
        t->stage_pending = true;
        // where the lookups of every example start, then one thread group per (slot, example)
        if (L > 0)
            TN_LAUNCH(k_example_rowptr, dim3(launch_grid(L, 256, GRID_CAP * 2)), dim3(256), st, ddescs, dlbase, N,
                      (uint32_t)L, batch, rowptr, t->dstatus);
        if (vec)
            TN_LAUNCH((k_combine_fwd<4>), dim3(launch_grid((int64_t)N * batch * (dim / 4), 256, GRID_CAP * 4)), dim3(256),
                      st, ddescs, N, dim, batch, combiner, rowptr, t->dstatus);
        else
            TN_LAUNCH((k_combine_fwd<1>), dim3(launch_grid((int64_t)N * batch * dim, 256, GRID_CAP * 4)), dim3(256), st,
                      ddescs, N, dim, batch, combiner, rowptr, t->dstatus);
    }
    TN_HIP(hipGetLastError());
    TN_HIP(hipMemcpyAsync(&t->hpull->st, t->dstatus, sizeof(DevStatus), hipMemcpyDeviceToHost, st));
    TN_HIP(hipStreamSynchronize(st));
    const uint32_t err = t->hpull->st.err;
    if (err & DEV_ERR_VAR_CAPACITY) return fail(TN_ERR_VAR_CAPACITY, "embedding combine: a mapped id is not a row of its variable");
    if (err & DEV_ERR_GRAD_ROWS)
        return fail(TN_ERR_INVALID_ARGUMENT, "embedding combine: example ids must be non-decreasing and in [0, batch)");
    return TN_OK;
}

}  // extern "C"
