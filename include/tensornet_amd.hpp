// tensornet_amd.hpp -- C++ host-side mirror of the reference's table / optimizer /
// operator interfaces for the sparse pull / push path, as thin inline wrappers
// over the C ABI of tensornet_amd.h.  Names, argument meaning and defaults
// follow the reference (paths relative to its tree):
//
//   tensornet::AdaGrad / Adam / Ftrl      core/ps/optimizer/optimizer.h:71-144
//   tensornet::SparsePushSignInfo         core/ps_interface/ps_raw_interface.h:22-35
//   tensornet::SparseTable, CreateSparseTable, SparseTableRegistry
//                                         core/ps/table/sparse_table.h:32-102
//   tensornet::DenseTable, CreateDenseTable, DenseTableRegistry
//                                         core/ps/table/dense_table.h:30-86
//   tensornet::ops::SparseTablePull / SparseTablePush / DenseTableInit /
//   DenseTablePushPull                    core/ops/*.cc, core/kernels/*_table_ops.cc
//
// Differences a maintainer needs to know:
//   * buffers are device pointers (HIP), not butil::IOBuf / tensorflow::Tensor;
//   * what the reference turns into a fatal CHECK is returned as a status code
//     (TN_OK == 0, see tensornet_amd.h); tensornet::LastError() has the text;
//   * a sparse table lives in HBM and is sized with Reserve().
#ifndef TENSORNET_AMD_HPP_
#define TENSORNET_AMD_HPP_

#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "tensornet_amd.h"

namespace tensornet {

inline std::string LastError() { return tn_last_error(); }

// ------------------------------------------------------------- optimizers
class OptimizerBase {
public:
    virtual ~OptimizerBase() {}
    virtual std::string Name() const = 0;

    void SetSparseZeroInit(bool sparse_zero_init) {
        sparse_zero_init_ = sparse_zero_init;
        if (handle_ >= 0) tn_opt_set_sparse_zero_init(handle_, sparse_zero_init ? 1 : 0);
    }
    void SetUseCvm(bool use_cvm) { use_cvm_ = use_cvm; }
    bool ShouldUseCvm() const { return use_cvm_; }
    void SetSchedule(float const_lr) {
        learning_rate = const_lr;
        if (handle_ >= 0) tn_opt_set_learning_rate(handle_, const_lr);
    }

    // Registers the hyper-parameters with the library on first use (they are
    // read when the optimizer is first attached to a table, as the reference
    // reads them through the shared pointer).
    tn_opt_t Handle() const {
        if (handle_ < 0) {
            handle_ = Register();
            if (handle_ >= 0 && sparse_zero_init_) tn_opt_set_sparse_zero_init(handle_, 1);
        }
        return handle_;
    }

public:
    float learning_rate = 0.01f;
    float show_decay_rate = 0.98f;
    bool sparse_zero_init_ = false;
    bool use_cvm_ = false;

protected:
    virtual tn_opt_t Register() const = 0;
    mutable tn_opt_t handle_ = -1;
};

class Adam : public OptimizerBase {
public:
    std::string Name() const override { return "Adam"; }
    float beta1 = 0.9f;
    float beta2 = 0.999f;
    float epsilon = 1e-08f;
    float initial_scale = 1.0f;

protected:
    tn_opt_t Register() const override {
        tn_adam_params p{learning_rate, show_decay_rate, beta1, beta2, epsilon, initial_scale};
        tn_opt_t h = -1;
        return tn_opt_create_adam(&p, &h) == TN_OK ? h : -1;
    }
};

class AdaGrad : public OptimizerBase {
public:
    std::string Name() const override { return "AdaGrad"; }
    float initial_g2sum = 0;
    float initial_scale = 1.0f;
    float epsilon = 1e-08f;
    float grad_decay_rate = 1.0f;
    float mom_decay_rate = 1.0f;
    float show_threshold = 0.0f;
    int no_show_days = 1000;
    int elimination_logic = 0;

protected:
    tn_opt_t Register() const override {
        tn_adagrad_params p{learning_rate,   show_decay_rate, show_threshold, initial_g2sum, initial_scale,
                            epsilon,         grad_decay_rate, mom_decay_rate, no_show_days,  elimination_logic};
        tn_opt_t h = -1;
        return tn_opt_create_adagrad(&p, &h) == TN_OK ? h : -1;
    }
};

class Ftrl : public OptimizerBase {
public:
    std::string Name() const override { return "Ftrl"; }
    float initial_scale = 0;  // C++ default of the reference (its Python factory passes 1.0)
    float beta = 1;
    float lambda1 = 0.1f;
    float lambda2 = 1;
    float show_threshold = 0.0f;

protected:
    tn_opt_t Register() const override {
        tn_ftrl_params p{learning_rate, show_decay_rate, show_threshold, beta, lambda1, lambda2, initial_scale};
        tn_opt_t h = -1;
        return tn_opt_create_ftrl(&p, &h) == TN_OK ? h : -1;
    }
};

// ------------------------------------------------------------ sparse table
struct SparsePushSignInfo {
    SparsePushSignInfo() : SparsePushSignInfo(0, 0, 0) {}
    SparsePushSignInfo(uint64_t s, int bs, int cs) : sign(s), batch_show(bs), batch_click(cs) {}
    uint64_t sign;
    int batch_show;
    int batch_click;
};
static_assert(sizeof(SparsePushSignInfo) == sizeof(tn_sign_info), "record layout of the push");

class SparseTable {
public:
    // SparseTable::Pull: n device signs -> out[n, dim] (device), absent signs are inserted.
    int Pull(const uint64_t* signs, int64_t n, int dim, float* out_emb, void* stream = nullptr) {
        return tn_sparse_table_pull(handle_, signs, n, dim, out_emb, stream);
    }
    // SparseTable::Push: n records applied in array order.
    int Push(const SparsePushSignInfo* infos, const float* grads, int64_t n, int dim, void* stream = nullptr) {
        return tn_sparse_table_push(handle_, reinterpret_cast<const tn_sign_info*>(infos), grads, n, dim, stream);
    }
    size_t GetHandle() const { return handle_; }
    std::string GetName() const { return name_; }
    std::string GetEmbeddingGroup() const { return embedding_group_; }
    // SparseOptimizerKernelBase::KeyCount
    size_t KeyCount() const {
        uint64_t n = 0;
        tn_sparse_table_key_count(handle_, &n);
        return n;
    }
    // SparseTable::Save / Load (sparse_table.h:55-57): the reference's checkpoint files.
    int Save(const std::string& filepath, const std::string& mode = "txt") {
        return tn_sparse_table_save(handle_, filepath.c_str(), mode.c_str());
    }
    int Load(const std::string& filepath, const std::string& mode = "txt") {
        return tn_sparse_table_load(handle_, filepath.c_str(), mode.c_str());
    }
    // SparseTable::ShowDecay (sparse_table.h:59)
    int ShowDecay(int delta_days, void* stream = nullptr) const {
        return tn_sparse_table_show_decay(handle_, delta_days, stream);
    }
    // HBM sizing (no counterpart in the reference, whose host maps grow by themselves).
    int Reserve(uint64_t max_keys) { return tn_sparse_table_reserve(handle_, max_keys); }
    int Clear() { return tn_sparse_table_clear(handle_); }
    // small batches on the path of few launches (the default) or on the one every other batch takes: same results
    int SetSmallBatchPath(bool enable) { return tn_sparse_table_set_small_batch_path(handle_, enable ? 1 : 0); }
    // the updates of a large push beside what the caller queues next; its gradients then stay untouched until the
    // table's next waiting call has returned (the reference's push is asynchronous in the same way)
    int SetDetachedUpdates(bool enable) { return tn_sparse_table_set_detached_updates(handle_, enable ? 1 : 0); }
    // a large push compares the signs of its batch with a copy the pull kept, instead of with their fingerprints
    int SetExactVerify(bool enable) { return tn_sparse_table_set_exact_verify(handle_, enable ? 1 : 0); }
    int Sync() { return tn_sparse_table_sync(handle_); }

private:
    friend SparseTable* CreateSparseTable(const OptimizerBase*, const std::string&, int, int, int, const std::string&);
    SparseTable(uint32_t handle, const std::string& name, const std::string& group)
        : handle_(handle), name_(name), embedding_group_(group) {}
    uint32_t handle_;
    std::string name_;
    std::string embedding_group_;
};

class SparseTableRegistry {
public:
    static SparseTableRegistry* Instance() {
        static SparseTableRegistry instance;
        return &instance;
    }
    // nullptr for an unknown handle (the reference CHECK-fails).
    SparseTable* Get(uint32_t table_handle) {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = tables_.find(table_handle);
        return it == tables_.end() ? nullptr : it->second.get();
    }

private:
    friend SparseTable* CreateSparseTable(const OptimizerBase*, const std::string&, int, int, int, const std::string&);
    std::mutex mu_;
    std::map<uint32_t, std::unique_ptr<SparseTable>> tables_;
};

// CreateSparseTable(opt, name, dimension, shard_num, self_shard_id, embedding_group):
// a non-empty embedding_group that already exists returns the existing table.
inline SparseTable* CreateSparseTable(const OptimizerBase* opt, const std::string& name, int dimension, int shard_num,
                                      int self_shard_id, const std::string& embedding_group) {
    if (!opt) return nullptr;
    uint32_t h = 0;
    if (tn_sparse_table_create(opt->Handle(), name.c_str(), dimension, opt->ShouldUseCvm() ? 1 : 0, shard_num,
                               self_shard_id, embedding_group.c_str(), &h) != TN_OK)
        return nullptr;
    SparseTableRegistry* reg = SparseTableRegistry::Instance();
    std::lock_guard<std::mutex> lk(reg->mu_);
    auto it = reg->tables_.find(h);
    if (it == reg->tables_.end())
        it = reg->tables_.emplace(h, std::unique_ptr<SparseTable>(new SparseTable(h, name, embedding_group))).first;
    return it->second.get();
}

// ------------------------------------------------------------- dense table
class DenseTable {
public:
    // DenseTable::Init + SetWeight from one flat device array.
    int Init(int total_elements, const float* w, void* stream = nullptr) {
        const float* vars[1] = {w};
        int64_t lens[1] = {total_elements};
        return tn_dense_table_init(handle_, 1, vars, lens, stream);
    }
    int SetWeight(const float* w, void* stream = nullptr) { return tn_dense_table_set_weight(handle_, w, stream); }
    int GetWeight(float* w, void* stream = nullptr) const { return tn_dense_table_get_weight(handle_, w, stream); }
    // DenseOptimizerKernelBase::Apply followed by GetWeight (PsLocalServer::DensePushPullAsync).
    int PushPull(const float* grad, float lr, float* w_out, int64_t total, void* stream = nullptr) {
        float* vars[1] = {w_out};
        const float* grads[1] = {grad};
        int64_t lens[1] = {total};
        return tn_dense_table_push_pull(handle_, 1, vars, grads, lens, lr, stream);
    }
    // DenseTable::Save / Load (dense_table.cc:103-157): text file <filepath>/dense_table/<handle>/0.
    int Save(const std::string& filepath) const { return tn_dense_table_save(handle_, filepath.c_str()); }
    int Load(const std::string& filepath) { return tn_dense_table_load(handle_, filepath.c_str()); }
    uint32_t GetHandle() const { return handle_; }
    int TotalElements() const {
        int64_t t = 0;
        tn_dense_table_total_elements(handle_, &t);
        return (int)t;
    }

private:
    friend DenseTable* CreateDenseTable(const OptimizerBase*, int, int);
    explicit DenseTable(uint32_t handle) : handle_(handle) {}
    uint32_t handle_;
};

class DenseTableRegistry {
public:
    static DenseTableRegistry* Instance() {
        static DenseTableRegistry singleton;
        return &singleton;
    }
    DenseTable* Get(uint32_t table_handle) {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = tables_.find(table_handle);
        return it == tables_.end() ? nullptr : it->second.get();
    }

private:
    friend DenseTable* CreateDenseTable(const OptimizerBase*, int, int);
    std::mutex mu_;
    std::map<uint32_t, std::unique_ptr<DenseTable>> tables_;
};

inline DenseTable* CreateDenseTable(const OptimizerBase* opt, int shard_num, int self_shard_id) {
    if (!opt) return nullptr;
    uint32_t h = 0;
    if (tn_dense_table_create(opt->Handle(), shard_num, self_shard_id, &h) != TN_OK) return nullptr;
    DenseTableRegistry* reg = DenseTableRegistry::Instance();
    std::lock_guard<std::mutex> lk(reg->mu_);
    return reg->tables_.emplace(h, std::unique_ptr<DenseTable>(new DenseTable(h))).first->second.get();
}

// ---------------------------------------------------------------- operators
namespace ops {

// One slot of an op: a values tensor with its variable (pull) or its gradient
// and labels (push).  All pointers are device memory.
struct PullSlot {
    const int64_t* values;
    int64_t len;
    float* var;            // [var_rows, dim]
    int64_t var_rows;
    int64_t* mapped_values;  // [len]
};
struct PushSlot {
    const int64_t* values;
    int64_t len;
    const float* grad;     // [grad_rows, dim], row j = j-th distinct sign
    int64_t grad_rows;
    const int64_t* labels;   // [len]
};

// SparseTablePull(resources: N*resource, values: N*int64) -> mapped_values: N*int64
inline int SparseTablePull(uint32_t table_handle, const std::vector<PullSlot>& slots, int dim, void* stream = nullptr) {
    const int n = (int)slots.size();
    std::vector<const int64_t*> values(n);
    std::vector<int64_t> lens(n), rows(n);
    std::vector<float*> vars(n);
    std::vector<int64_t*> mapped(n);
    for (int i = 0; i < n; i++) {
        values[i] = slots[i].values;
        lens[i] = slots[i].len;
        vars[i] = slots[i].var;
        rows[i] = slots[i].var_rows;
        mapped[i] = slots[i].mapped_values;
    }
    return tn_sparse_table_pull_op(table_handle, n, values.data(), lens.data(), vars.data(), rows.data(), dim,
                                   mapped.data(), stream);
}

// SparseTablePush(values: N*int64, grads: N*float, feature_labels: N*int64)
inline int SparseTablePush(uint32_t table_handle, const std::vector<PushSlot>& slots, int dim, void* stream = nullptr) {
    const int n = (int)slots.size();
    std::vector<const int64_t*> values(n), labels(n);
    std::vector<int64_t> lens(n), rows(n);
    std::vector<const float*> grads(n);
    for (int i = 0; i < n; i++) {
        values[i] = slots[i].values;
        lens[i] = slots[i].len;
        grads[i] = slots[i].grad;
        rows[i] = slots[i].grad_rows;
        labels[i] = slots[i].labels;
    }
    return tn_sparse_table_push_op(table_handle, n, values.data(), lens.data(), grads.data(), rows.data(), dim,
                                   labels.data(), stream);
}

// DenseTableInit(vars: N*resource)
inline int DenseTableInit(uint32_t table_handle, const std::vector<const float*>& vars,
                          const std::vector<int64_t>& lens, void* stream = nullptr) {
    return tn_dense_table_init(table_handle, (int)vars.size(), vars.data(), lens.data(), stream);
}

// DenseTablePushPull(vars, grads: N*float, learning_rate)
inline int DenseTablePushPull(uint32_t table_handle, const std::vector<float*>& vars,
                              const std::vector<const float*>& grads, const std::vector<int64_t>& lens,
                              float learning_rate, void* stream = nullptr) {
    return tn_dense_table_push_pull(table_handle, (int)vars.size(), vars.data(), grads.data(), lens.data(),
                                    learning_rate, stream);
}

}  // namespace ops
}  // namespace tensornet

#endif  // TENSORNET_AMD_HPP_
