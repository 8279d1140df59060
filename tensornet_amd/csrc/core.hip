// Error reporting, optimizer registry and small shared host helpers of the
// C ABI (include/tensornet_amd.h).  Optimizer factories follow
// core/main/py_wrapper.cc:82-162; objects are immortal like the reference's
// (py_wrapper.cc:112).
#include "tn_common.h"

#include <cstring>

namespace tn {

namespace {
thread_local std::string t_last_error;
std::mutex g_opt_mu;
std::vector<std::shared_ptr<OptConf>> g_opts;
}  // namespace

void set_error(const std::string& msg) { t_last_error = msg; }

int fail(int code, const std::string& msg) {
    t_last_error = msg;
    return code;
}

std::shared_ptr<OptConf> get_opt(tn_opt_t h) {
    std::lock_guard<std::mutex> lk(g_opt_mu);
    if (h < 0 || (size_t)h >= g_opts.size()) return nullptr;
    return g_opts[h];
}

static tn_opt_t register_opt(std::shared_ptr<OptConf> c) {
    std::lock_guard<std::mutex> lk(g_opt_mu);
    g_opts.push_back(std::move(c));
    return (tn_opt_t)(g_opts.size() - 1);
}

int DevBuf::ensure(size_t need) {
    if (need <= bytes) return TN_OK;
    if (p) {
        hipError_t e = hipFree(p);
        p = nullptr;
        bytes = 0;
        if (e != hipSuccess) return fail(TN_ERR_HIP, std::string("hipFree: ") + hipGetErrorString(e));
    }
    size_t want = align_up(need + need / 4, 1 << 20);
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
        p = nullptr;
        return fail(TN_ERR_OUT_OF_MEMORY, "hipMalloc(" + std::to_string(want) + "): " + hipGetErrorString(e));
    }
    bytes = want;
    return TN_OK;
}

// ---------------------------------------------------------------- profiling
bool g_profile_on = false;
namespace {
struct ProfRec {
    const char* name;
    hipEvent_t a, b;
};
std::mutex g_prof_mu;
std::vector<ProfRec> g_prof_recs;
std::vector<hipEvent_t> g_prof_pool;

hipEvent_t prof_event() {
    if (!g_prof_pool.empty()) {
        hipEvent_t e = g_prof_pool.back();
        g_prof_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}
}  // namespace

void prof_begin(const char* name, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfRec r{name, prof_event(), prof_event()};
    (void)hipEventRecord(r.a, st);
    g_prof_recs.push_back(r);
}

void prof_end(hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    if (!g_prof_recs.empty()) (void)hipEventRecord(g_prof_recs.back().b, st);
}

void DevBuf::release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    bytes = 0;
}

}  // namespace tn

using namespace tn;

extern "C" {

const char* tn_last_error(void) { return t_last_error.c_str(); }

const char* tn_version(void) { return "tensornet_amd 0.1 (gfx950)"; }

int tn_profile_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_profile_on = on != 0;
    return TN_OK;
}

int tn_profile_reset(void) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    for (auto& r : g_prof_recs) {
        (void)hipEventSynchronize(r.b);
        g_prof_pool.push_back(r.a);
        g_prof_pool.push_back(r.b);
    }
    g_prof_recs.clear();
    return TN_OK;
}

int tn_profile_summary(char* buf, size_t cap) {
    if (!buf || cap == 0) return fail(TN_ERR_INVALID_ARGUMENT, "tn_profile_summary: no buffer");
    std::lock_guard<std::mutex> lk(g_prof_mu);
    struct Acc {
        const char* name;
        long count;
        double ms;
    };
    std::vector<Acc> acc;
    for (auto& r : g_prof_recs) {
        TN_HIP(hipEventSynchronize(r.b));
        float ms = 0.f;
        TN_HIP(hipEventElapsedTime(&ms, r.a, r.b));
        bool hit = false;
        for (auto& a : acc)
            if (std::string(a.name) == r.name) {
                a.count++;
                a.ms += ms;
                hit = true;
                break;
            }
        if (!hit) acc.push_back(Acc{r.name, 1, ms});
    }
    std::string out;
    for (auto& a : acc) {
        char line[256];
        snprintf(line, sizeof(line), "%s\t%ld\t%.6f\n", a.name, a.count, a.ms);
        out += line;
    }
    if (out.size() + 1 > cap) return fail(TN_ERR_INVALID_ARGUMENT, "tn_profile_summary: buffer too small");
    memcpy(buf, out.c_str(), out.size() + 1);
    return TN_OK;
}

void tn_adagrad_params_default(tn_adagrad_params* p) {
    if (!p) return;
    p->learning_rate = 0.01f;  // optimizer.h:64
    p->show_decay_rate = 0.98f;
    p->show_threshold = 0.0f;
    p->initial_g2sum = 0.f;
    p->initial_scale = 1.f;
    p->epsilon = 1e-8f;
    p->grad_decay_rate = 1.0f;
    p->mom_decay_rate = 1.0f;
    p->no_show_days = 1000;
    p->elimination_logic = 0;
}

void tn_adam_params_default(tn_adam_params* p) {
    if (!p) return;
    p->learning_rate = 0.01f;
    p->show_decay_rate = 0.98f;
    p->beta1 = 0.9f;
    p->beta2 = 0.999f;
    p->epsilon = 1e-8f;
    p->initial_scale = 1.0f;
}

void tn_ftrl_params_default(tn_ftrl_params* p) {
    if (!p) return;
    p->learning_rate = 0.01f;
    p->show_decay_rate = 0.98f;
    p->show_threshold = 0.0f;
    p->beta = 1.f;
    p->lambda1 = 0.1f;
    p->lambda2 = 1.f;
    p->initial_scale = 1.0f;
}

int tn_opt_create_adagrad(const tn_adagrad_params* p, tn_opt_t* out) {
    if (!p || !out) return fail(TN_ERR_INVALID_ARGUMENT, "tn_opt_create_adagrad: NULL argument");
    if (p->elimination_logic != 0 && p->elimination_logic != 1)
        return fail(TN_ERR_INVALID_ARGUMENT,
                    "elimination_logic must be in the set of valid values {0, 1}, but got: " +
                        std::to_string(p->elimination_logic));
    auto c = std::make_shared<OptConf>();
    c->kind = OPT_ADAGRAD;
    c->learning_rate = p->learning_rate;
    c->show_decay_rate = p->show_decay_rate;
    c->show_threshold = p->show_threshold;
    c->initial_g2sum = p->initial_g2sum;
    c->initial_scale = p->initial_scale;
    c->epsilon = p->epsilon;
    c->grad_decay_rate = p->grad_decay_rate;
    c->mom_decay_rate = p->mom_decay_rate;
    c->no_show_days = p->no_show_days;
    c->elimination_logic = p->elimination_logic;
    *out = register_opt(c);
    return TN_OK;
}

int tn_opt_create_adam(const tn_adam_params* p, tn_opt_t* out) {
    if (!p || !out) return fail(TN_ERR_INVALID_ARGUMENT, "tn_opt_create_adam: NULL argument");
    auto c = std::make_shared<OptConf>();
    c->kind = OPT_ADAM;
    c->learning_rate = p->learning_rate;
    c->show_decay_rate = p->show_decay_rate;
    c->beta1 = p->beta1;
    c->beta2 = p->beta2;
    c->epsilon = p->epsilon;
    c->initial_scale = p->initial_scale;
    *out = register_opt(c);
    return TN_OK;
}

int tn_opt_create_ftrl(const tn_ftrl_params* p, tn_opt_t* out) {
    if (!p || !out) return fail(TN_ERR_INVALID_ARGUMENT, "tn_opt_create_ftrl: NULL argument");
    auto c = std::make_shared<OptConf>();
    c->kind = OPT_FTRL;
    c->learning_rate = p->learning_rate;
    c->show_decay_rate = p->show_decay_rate;
    c->show_threshold = p->show_threshold;
    c->beta = p->beta;
    c->lambda1 = p->lambda1;
    c->lambda2 = p->lambda2;
    c->initial_scale = p->initial_scale;
    *out = register_opt(c);
    return TN_OK;
}

int tn_opt_set_sparse_zero_init(tn_opt_t opt, int zero_init) {
    auto c = get_opt(opt);
    if (!c) return fail(TN_ERR_BAD_HANDLE, "tn_opt_set_sparse_zero_init: unknown optimizer handle");
    c->sparse_zero_init = zero_init ? 1 : 0;
    return TN_OK;
}

int tn_opt_set_learning_rate(tn_opt_t opt, float lr) {
    auto c = get_opt(opt);
    if (!c) return fail(TN_ERR_BAD_HANDLE, "tn_opt_set_learning_rate: unknown optimizer handle");
    c->learning_rate = lr;
    return TN_OK;
}

int tn_opt_get_learning_rate(tn_opt_t opt, float* lr) {
    auto c = get_opt(opt);
    if (!c || !lr) return fail(TN_ERR_BAD_HANDLE, "tn_opt_get_learning_rate: unknown optimizer handle");
    *lr = c->learning_rate;
    return TN_OK;
}

}  // extern "C"
