// Exercises the C++ host-side mirror (include/tensornet_amd.hpp) the way the
// reference's own gtest files use its tables (test/ps/table/sparse_table_test.cc):
// create an optimizer and a table, pull signs, push gradients.  Host-only
// checks always run; with `--gpu` a small pull/push/dense round trip runs on
// the device and is compared with a closed form.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <unistd.h>
#include <cstring>
#include <string>
#include <vector>

#include "tensornet_amd.hpp"

using namespace tensornet;

static int failures = 0;
#define EXPECT(cond)                                                          \
    do {                                                                      \
        if (!(cond)) {                                                        \
            std::printf("FAILED %s:%d: %s [%s]\n", __FILE__, __LINE__, #cond, LastError().c_str()); \
            failures++;                                                       \
        }                                                                     \
    } while (0)

static void host_checks() {
    AdaGrad* opt = new AdaGrad();  // optimizers are immortal, like the reference's
    opt->learning_rate = 0.01f;
    opt->initial_g2sum = 0.1f;
    opt->initial_scale = 0.1f;
    SparseTable* a = CreateSparseTable(opt, "a", 8, 1, 0, "shared-group");
    SparseTable* b = CreateSparseTable(opt, "b", 8, 1, 0, "shared-group");
    SparseTable* c = CreateSparseTable(opt, "c", 8, 1, 0, "");
    EXPECT(a && b && c);
    EXPECT(a == b && a->GetHandle() == b->GetHandle());  // sparse_table.cc:175-180
    EXPECT(c->GetHandle() != a->GetHandle());
    EXPECT(SparseTableRegistry::Instance()->Get((uint32_t)c->GetHandle()) == c);
    EXPECT(SparseTableRegistry::Instance()->Get(123456) == nullptr);
    EXPECT(CreateSparseTable(opt, "bad", 0, 1, 0, "") == nullptr);      // dimension must be positive
    EXPECT(CreateSparseTable(opt, "bad", 8, 2, 1, "") == nullptr);      // one worker only
    EXPECT(CreateDenseTable(new Ftrl(), 1, 0) == nullptr);              // dense Ftrl is a stub in the reference
    DenseTable* d = CreateDenseTable(new Adam(), 1, 0);
    EXPECT(d && DenseTableRegistry::Instance()->Get(d->GetHandle()) == d);
    EXPECT(d->TotalElements() == 0);
    EXPECT(sizeof(SparsePushSignInfo) == 16);
    AdaGrad bad;
    bad.elimination_logic = 7;
    EXPECT(CreateSparseTable(&bad, "x", 8, 1, 0, "") == nullptr);
    EXPECT(LastError().find("elimination_logic") != std::string::npos || LastError().size() > 0);
}

template <typename T>
static T* to_device(const std::vector<T>& v) {
    T* p = nullptr;
    if (hipMalloc((void**)&p, v.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
    (void)hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice);
    return p;
}

static void gpu_checks() {
    const int D = 8;
    AdaGrad* opt = new AdaGrad();
    opt->learning_rate = 0.5f;
    opt->initial_g2sum = 0.f;
    opt->epsilon = 0.f;
    opt->SetSparseZeroInit(true);
    SparseTable* t = CreateSparseTable(opt, "gpu", D, 1, 0, "");
    EXPECT(t && t->Reserve(1000) == TN_OK);
    std::vector<uint64_t> signs = {11, 22, 11, 33};
    uint64_t* dsigns = to_device(signs);
    float* dout = nullptr;
    EXPECT(hipMalloc((void**)&dout, 4 * D * sizeof(float)) == hipSuccess);
    EXPECT(t->Pull(dsigns, 4, D, dout) == TN_OK);
    EXPECT(t->KeyCount() == 3);
    // push g = 2 on sign 11 twice (sequentially) and once on 22: with g2sum0 = 0, eps = 0,
    // AdaGrad gives w = -lr*2/sqrt(4) = -0.5, then g2sum = 8: w -= 0.5*2/sqrt(8)
    std::vector<SparsePushSignInfo> infos = {{11, 1, 0}, {22, 3, 1}, {11, 2, 1}};
    std::vector<float> grads(3 * D, 2.0f);
    SparsePushSignInfo* dinfos = to_device(infos);
    float* dgrads = to_device(grads);
    EXPECT(t->Push(dinfos, dgrads, 3, D) == TN_OK);
    EXPECT(t->Sync() == TN_OK);
    EXPECT(t->Pull(dsigns, 4, D, dout) == TN_OK);
    std::vector<float> out(4 * D);
    (void)hipMemcpy(out.data(), dout, out.size() * sizeof(float), hipMemcpyDeviceToHost);
    const float w11 = -0.5f - 0.5f * 2.0f / std::sqrt(8.0f);
    for (int i = 0; i < D; i++) {
        EXPECT(std::fabs(out[i] - w11) < 1e-6f);
        EXPECT(out[2 * D + i] == out[i]);          // same sign, same row
        EXPECT(std::fabs(out[D + i] + 0.5f) < 1e-6f);
        EXPECT(out[3 * D + i] == 0.0f);            // sign 33 was never pushed
    }
    // an unknown sign in a push is reported, not fatal
    std::vector<SparsePushSignInfo> unknown = {{99, 1, 0}};
    SparsePushSignInfo* dunknown = to_device(unknown);
    EXPECT(t->Push(dunknown, dgrads, 1, D) == TN_OK);
    EXPECT(t->Sync() == TN_ERR_UNKNOWN_KEY);

    // operator level: two slots sharing sign 22
    std::vector<int64_t> v0 = {22, 33, 22}, v1 = {44, 22};
    int64_t *dv0 = to_device(v0), *dv1 = to_device(v1);
    float *var0 = nullptr, *var1 = nullptr;
    int64_t *m0 = nullptr, *m1 = nullptr;
    (void)hipMalloc((void**)&var0, 4 * D * sizeof(float));
    (void)hipMalloc((void**)&var1, 3 * D * sizeof(float));
    (void)hipMalloc((void**)&m0, 3 * sizeof(int64_t));
    (void)hipMalloc((void**)&m1, 2 * sizeof(int64_t));
    std::vector<ops::PullSlot> pull = {{dv0, 3, var0, 4, m0}, {dv1, 2, var1, 3, m1}};
    EXPECT(ops::SparseTablePull((uint32_t)t->GetHandle(), pull, D) == TN_OK);
    int64_t hm0[3], hm1[2];
    (void)hipMemcpy(hm0, m0, sizeof(hm0), hipMemcpyDeviceToHost);
    (void)hipMemcpy(hm1, m1, sizeof(hm1), hipMemcpyDeviceToHost);
    EXPECT(hm0[0] == 0 && hm0[1] == 1 && hm0[2] == 0 && hm1[0] == 0 && hm1[1] == 1);
    // U_s must stay below the rows of the variable (sparse_table_ops.cc:136)
    std::vector<ops::PullSlot> tight = {{dv0, 3, var0, 2, m0}};
    EXPECT(ops::SparseTablePull((uint32_t)t->GetHandle(), tight, D) == TN_ERR_VAR_CAPACITY);

    // SparseTable::ShowDecay / Save / Load: a second table of the same name reads the files back
    EXPECT(t->ShowDecay(1) == TN_OK);
    const char* tmp = std::getenv("TMPDIR");
    std::string pattern = std::string(tmp ? tmp : "/tmp") + "/tn_host_mirror_XXXXXX";  // a fresh directory per run
    const char* made = mkdtemp(&pattern[0]);
    EXPECT(made != nullptr);
    const std::string ckpt = made ? made : pattern;
    EXPECT(t->Save(ckpt, "txt") == TN_OK);
    SparseTable* t2 = CreateSparseTable(opt, "gpu", D, 1, 0, "");
    EXPECT(t2 && t2 != t && t2->Load(ckpt, "txt") == TN_OK);
    EXPECT(t2->KeyCount() == t->KeyCount());
    EXPECT(t2->Pull(dsigns, 4, D, dout) == TN_OK);
    std::vector<float> back(4 * D);
    (void)hipMemcpy(back.data(), dout, back.size() * sizeof(float), hipMemcpyDeviceToHost);
    for (int i = 0; i < D; i++) EXPECT(std::fabs(back[i] - w11) < 1e-5f);  // text keeps six digits

    // dense Adam, first step from zero moments: w -= lr * g / (|g| + eps')
    Adam* adam = new Adam();
    DenseTable* d = CreateDenseTable(adam, 1, 0);
    std::vector<float> w(1000, 1.0f), g(1000, 0.25f);
    float *dw = to_device(w), *dg = to_device(g);
    EXPECT(d->Init(1000, dw) == TN_OK);
    EXPECT(d->Init(999, dw) == TN_ERR_ALREADY_INIT);
    EXPECT(d->PushPull(dg, 0.1f, dw, 1000) == TN_OK);
    (void)hipDeviceSynchronize();
    (void)hipMemcpy(w.data(), dw, w.size() * sizeof(float), hipMemcpyDeviceToHost);
    for (int i = 0; i < 1000; i++) EXPECT(std::fabs(w[i] - 0.9f) < 1e-5f);

    // DenseTable::Save / Load: the file initialises a second table, and a second step on the
    // copy equals a second step on the original (weights, moments and beta powers came along)
    EXPECT(d->Save(ckpt) == TN_OK);
    DenseTable* d2 = CreateDenseTable(adam, 1, 0);
    const std::string from = ckpt + "/dense_table/" + std::to_string(d->GetHandle()) + "/0";
    const std::string to_dir = ckpt + "/dense_table/" + std::to_string(d2->GetHandle());
    EXPECT(d2->Load(ckpt) != TN_OK);  // no file for this handle yet
    EXPECT(std::system(("mkdir -p " + to_dir + " && cp " + from + " " + to_dir + "/0").c_str()) == 0);
    EXPECT(d2->Load(ckpt) == TN_OK);
    EXPECT(d2->TotalElements() == 1000);
    float* dw2 = nullptr;
    (void)hipMalloc((void**)&dw2, 1000 * sizeof(float));
    EXPECT(d->PushPull(dg, 0.1f, dw, 1000) == TN_OK);
    EXPECT(d2->PushPull(dg, 0.1f, dw2, 1000) == TN_OK);
    (void)hipDeviceSynchronize();
    std::vector<float> w2(1000);
    (void)hipMemcpy(w.data(), dw, w.size() * sizeof(float), hipMemcpyDeviceToHost);
    (void)hipMemcpy(w2.data(), dw2, w2.size() * sizeof(float), hipMemcpyDeviceToHost);
    for (int i = 0; i < 1000; i++) EXPECT(std::fabs(w[i] - w2[i]) < 1e-5f);
}

int main(int argc, char** argv) {
    host_checks();
    if (argc > 1 && std::strcmp(argv[1], "--gpu") == 0) gpu_checks();
    if (failures == 0) std::printf("host mirror ok\n");
    return failures ? 1 : 0;
}
