// oracle.cc -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A single-thread CPU restatement of the reference algorithm for the sparse
// pull / push path and the dense Adam / AdaGrad update, written from a reading
// of the reference sources (paths relative to the reference tree).  It is the
// checker the HIP path is compared against in tests/, in
// __graft_entry__.smoke() and as bench.py's cpu_baseline; nothing in the
// product library links, imports or calls it.
//
// It keeps the reference's data structures on purpose (so that timing it is a
// fair "port" baseline): std::map first-occurrence remap per slot, 8 hash
// blocks of std::unordered_map<uint64, Value*> with the hi/lo-swapped hasher,
// a free-list pool allocator of 65536 objects per pool, per-record Apply, and
// byte buffers that are appended to and cut from like the reference's IOBuf
// (every pulled row and every pushed record is copied twice).
//
// How each function is pinned (no execution of the reference is possible in
// this build: its translation units need brpc/butil, Boost, Eigen and
// protoc-generated headers that the image lacks):
//   remap / show / click   brute force + numpy.unique identities + hand-made
//                          known-answer vectors        (tests/test_oracle_remap.py)
//   AdaGrad / Adam / Ftrl  numpy closed forms with explicit float32/float64
//                          casts, exactly-representable known answers, both
//                          Ftrl branches, repeated Applies (tests/test_oracle_optim.py)
//   dense Adam / AdaGrad   numpy closed form; beta=0 special case reduces to
//                          w -= lr*g/(|g|+eps)           (tests/test_oracle_dense.py)
//   row initialiser        distribution only (mean/std), as the reference's
//                          own generator is wall-clock seeded.
//   ShowDecay / DeleteByShow  closed forms and hand-made cases for every
//                          optimizer and both elimination logics   (tests/test_oracle_decay.py)
//   checkpoint streams     sparse blocks (text and binary) against hand-written
//                          files and struct layouts, old-format detection,
//                          round trips (tests/test_oracle_checkpoint.py); the dense
//                          table's text file against texts written out by hand
//                          from the reference's stream operators
//                          (tests/test_oracle_dense_checkpoint.py)
// One detail is an assumption, stated in the functions concerned: unqualified
// sqrt/abs/log on floats are taken to resolve to the float overloads (the
// libstdc++ <math.h>/<stdlib.h> wrappers being pulled in by the reference's
// third-party headers).  The double-overload reading differs by <= 1 ulp of
// fp32, far inside the 1e-5 relative tolerance of the update comparison.
//
// Build: see oracle/Makefile (g++ -O2 -ffp-contract=off, no -march: the
// reference's release flags have no FMA target either).

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <memory>
#include <new>
#include <random>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

namespace {

// ------------------------------------------------------------------ buffers
// Append/cut byte queue standing in for butil::IOBuf as the path uses it
// (core/ps/table/sparse_table.cc:64,72-74; core/kernels/sparse_table_ops.cc:88-92,263).
struct ByteQueue {
    std::vector<char> data;
    size_t head = 0;
    void append(const void* p, size_t n) {
        const char* c = static_cast<const char*>(p);
        data.insert(data.end(), c, c + n);
    }
    size_t cutn(void* out, size_t n) {
        size_t avail = data.size() - head;
        if (n > avail) n = avail;
        std::memcpy(out, data.data() + head, n);
        head += n;
        return n;
    }
    size_t size() const { return data.size() - head; }
};

// ---------------------------------------------------------------- allocator
// Fixed-size free-list pool, core/utility/allocator.h:26-129.
class Pool {
public:
    Pool(int type_sizeof, int block_len) : sz_((type_sizeof + 7) & ~7), len_(block_len) { grow(); }
    ~Pool() {
        for (void* p : pools_) free(p);
    }
    void* allocate() {
        if (!free_) grow();
        void* v = free_;
        free_ = *static_cast<void**>(free_);
        return v;
    }

private:
    void grow() {
        void* pool = nullptr;
        if (posix_memalign(&pool, 8, size_t(sz_) * len_) != 0) std::abort();
        pools_.push_back(pool);
        char* base = static_cast<char*>(pool);
        for (int i = 0; i < len_; i++) {
            void** b = reinterpret_cast<void**>(base + size_t(sz_) * i);
            *b = free_;
            free_ = b;
        }
    }
    int sz_, len_;
    void* free_ = nullptr;
    std::vector<void*> pools_;
};

// ------------------------------------------------------------------ configs
enum Kind { K_ADAGRAD = 0, K_ADAM = 1, K_FTRL = 2 };

// Hyper-parameters, all float as in core/ps/optimizer/optimizer.h:36-144.
struct Opt {
    int kind = 0;
    float learning_rate = 0.01f;
    float show_decay_rate = 0.98f;
    bool sparse_zero_init = false;
    bool use_cvm = false;
    // AdaGrad
    float initial_g2sum = 0, initial_scale = 1, epsilon = 1e-8f, grad_decay_rate = 1, mom_decay_rate = 1;
    float show_threshold = 0;
    int no_show_days = 1000, elimination_logic = 0;
    // Adam
    float beta1 = 0.9f, beta2 = 0.999f;
    // Ftrl
    float beta = 1, lambda1 = 0.1f, lambda2 = 1;
};

// Row of the sparse table: a small header followed by the float payload,
// like SparseAdaGradValue / SparseAdamValue / SparseFtrlValue
// (ada_grad_kernel.h:52-84, adam_kernel.h:54-87, ftrl_kernel.h:51-89).
struct Row {
    float g2sum;        // AdaGrad
    float show;         // AdaGrad show_ / Adam+Ftrl serialised show_
    float click;        // AdaGrad
    int no_show_days;   // AdaGrad
    int delta_show;     // Adam, Ftrl (data_struct.h:57)
    float data[1];      // w[wdim] then (Adam) m,v / (Ftrl) z,n
};

struct SignInfo {  // core/ps_interface/ps_raw_interface.h:22-35
    uint64_t sign;
    int batch_show;
    int batch_click;
};

// sparse_key_hasher, core/ps/optimizer/optimizer_kernel.h:248-252
struct KeyHasher {
    size_t operator()(const uint64_t& sign) const { return std::hash<uint64_t>()(sign >> 32 | sign << 32); }
};

class Table {
public:
    static constexpr int kBlocks = 8;  // SPARSE_KERNEL_BLOCK_NUM, optimizer_kernel.h:43

    Table(const Opt& o, int dim, uint64_t seed, size_t buckets) : opt(o), D(dim), rng(seed) {
        // only the AdaGrad row maintains the two cvm columns (ada_grad_kernel.cc:99-102,123-128)
        if (opt.kind != K_ADAGRAD) opt.use_cvm = false;
        wdim = D + (opt.use_cvm ? 2 : 0);
        payload = (opt.kind == K_ADAGRAD) ? wdim : 3 * D;
        int bytes = int(sizeof(Row) - sizeof(float) + sizeof(float) * payload);
        for (int i = 0; i < kBlocks; i++) {
            // optimizer_kernel.h:263-266: 15485863 initial buckets, max load 0.75
            blocks.emplace_back(new Block(buckets, bytes));
        }
    }

    int BlockId(uint64_t sign) const { return int(KeyHasher()(sign) % kBlocks); }  // optimizer_kernel.h:556

    // SparseKernelBlock::GetWeight, optimizer_kernel.h:299-308
    Row* GetOrCreate(uint64_t sign) {
        Block& b = *blocks[BlockId(sign)];
        auto ins = b.values.insert({sign, nullptr});
        if (ins.second) {
            Row* r = static_cast<Row*>(b.pool.allocate());
            Construct(r);
            ins.first->second = r;
        }
        return ins.first->second;
    }

    Row* Find(uint64_t sign) {
        Block& b = *blocks[BlockId(sign)];
        auto it = b.values.find(sign);
        return it == b.values.end() ? nullptr : it->second;
    }

    size_t KeyCount() const {
        size_t n = 0;
        for (auto& b : blocks) n += b->values.size();
        return n;
    }

    // Row constructors: ada_grad_kernel.cc:78-103, adam_kernel.cc:89-110, ftrl_kernel.cc:34-55
    void Construct(Row* r) {
        r->g2sum = opt.initial_g2sum;
        r->show = 0;
        r->click = 0;
        r->no_show_days = 0;
        r->delta_show = 0;
        float* w = r->data;
        if (opt.sparse_zero_init) {
            for (int i = 0; i < D; i++) w[i] = 0.0f;
        } else {
            // std::normal_distribution<float>(0, 1 / sqrt(dim)) on the minstd engine
            // (core/utility/random.h:30-42; there seeded from the wall clock).
            std::normal_distribution<float> dist(0, 1 / std::sqrt(double(D)));
            for (int i = 0; i < D; i++) w[i] = dist(rng) * opt.initial_scale;
        }
        for (int i = D; i < payload; i++) w[i] = 0.0f;  // cvm tail / m,v / z,n
    }

    void Apply(Row* r, const float* g, int batch_show, int batch_click) {
        switch (opt.kind) {
            case K_ADAGRAD: ApplyAdaGrad(r, g, batch_show, batch_click); break;
            case K_ADAM: ApplyAdam(r, g, batch_show); break;
            default: ApplyFtrl(r, g, batch_show); break;
        }
    }

    // SparseAdaGradValue::Apply, ada_grad_kernel.cc:105-129
    void ApplyAdaGrad(Row* r, const float* g, int batch_show, int batch_click) {
        r->show += batch_show;    // float += int
        r->click += batch_click;  // float += int
        r->no_show_days = 0;
        float* w = r->data;
        double add_g2sum = 0;
        for (int i = 0; i < D; ++i) {
            add_g2sum += g[i] * g[i];  // float product widened to double
        }
        r->g2sum += add_g2sum / D;  // float = float(double(g2sum) + add/D)
        for (int i = 0; i < D; ++i) {
            w[i] -= opt.learning_rate * g[i] / (opt.epsilon + sqrtf(r->g2sum));
        }
        if (opt.use_cvm) {
            float log_show = logf(r->show + 1);
            float log_click = logf(r->click + 1);
            w[D] = r->show;
            w[D + 1] = (log_click - log_show);
        }
    }

    // SparseAdamValue::Apply, adam_kernel.cc:112-125 (no bias correction, no step counter)
    void ApplyAdam(Row* r, const float* g, int batch_show) {
        r->delta_show += batch_show;
        float* w = r->data;
        float* m = r->data + D;
        float* v = r->data + 2 * D;
        for (int i = 0; i < D; ++i) {
            m[i] = opt.beta1 * m[i] + (1 - opt.beta1) * g[i];
            v[i] = opt.beta2 * v[i] + (1 - opt.beta2) * g[i] * g[i];
            w[i] -= opt.learning_rate * m[i] / (opt.epsilon + sqrtf(v[i]));
        }
    }

    // SparseFtrlValue::Apply, ftrl_kernel.cc:57-80 (learning_rate multiplies where
    // the textbook divides by alpha: follow the code)
    void ApplyFtrl(Row* r, const float* g, int batch_show) {
        r->delta_show += batch_show;
        float* w = r->data;
        float* z = r->data + D;
        float* n = r->data + 2 * D;
        for (int i = 0; i < D; ++i) {
            float g2 = g[i] * g[i];
            z[i] += g[i] - opt.learning_rate * (sqrtf(n[i] + g2) - sqrtf(n[i])) * w[i];
            n[i] += g2;
            if (fabsf(z[i]) <= opt.lambda1) {
                w[i] = 0;
            } else {
                w[i] = -1 / ((opt.beta + sqrtf(n[i])) * opt.learning_rate + opt.lambda2);
                if (z[i] > 0) {
                    w[i] *= z[i] - opt.lambda1;
                } else {
                    w[i] *= z[i] + opt.lambda1;
                }
            }
        }
    }

    // SparseTable::Pull, core/ps/table/sparse_table.cc:52-66
    void Pull(const uint64_t* signs, int64_t n, int dim, ByteQueue& out) {
        for (int64_t i = 0; i < n; ++i) {
            Row* r = GetOrCreate(signs[i]);
            out.append(r->data, sizeof(float) * dim);
        }
    }

    // SparseTable::Push, core/ps/table/sparse_table.cc:68-83 (+ SparseKernelBlock::Apply :310-320)
    int Push(ByteQueue& buf, int dim) {
        std::vector<float> grad(dim);
        SignInfo info;
        int missing = 0;
        while (sizeof(info) == buf.cutn(&info, sizeof(info))) {
            size_t grad_size = sizeof(float) * dim;
            if (grad_size != buf.cutn(grad.data(), grad_size)) return -1;
            Row* r = Find(info.sign);
            if (!r) {  // the reference aborts here (optimizer_kernel.h:315)
                missing++;
                continue;
            }
            Apply(r, grad.data(), info.batch_show, info.batch_click);
        }
        return missing;
    }

    // SparseOptimizerKernel::ShowDecay -> SparseKernelBlock::ShowDecay (optimizer_kernel.h:422-427,549-553):
    // every resident row; AdaGrad ada_grad_kernel.cc:191-195, Ftrl ftrl_kernel.cc:124, Adam adam_kernel.h:67 (no-op)
    void ShowDecay(int delta_days) {
        for (auto& b : blocks) {
            for (auto& kv : b->values) {
                Row* r = kv.second;
                if (opt.kind == K_ADAGRAD) {
                    r->show *= opt.show_decay_rate;
                    r->click *= opt.show_decay_rate;
                    r->no_show_days += delta_days;
                } else if (opt.kind == K_FTRL) {
                    r->show *= opt.show_decay_rate;
                }
            }
        }
    }

    // Value::DeleteByShow: would the row be left out of a saved table (optimizer_kernel.h:332,345)?
    // AdaGrad ada_grad_kernel.cc:197-204, Ftrl ftrl_kernel.cc:126, Adam adam_kernel.h:69
    bool DeleteByShow(const Row* r) const {
        if (opt.kind == K_ADAGRAD) {
            if (opt.elimination_logic == 1) return r->show < opt.show_threshold && r->no_show_days > opt.no_show_days;
            return r->show < opt.show_threshold || r->no_show_days > opt.no_show_days;
        }
        if (opt.kind == K_FTRL) return r->show < opt.show_threshold;
        return false;
    }

    // ---- checkpoint streams of one hash block: SparseKernelBlock's operator<< / operator>>
    // (optimizer_kernel.h:324-420) with the value formats of ada_grad_kernel.cc:131-189,
    // adam_kernel.cc:127-167, ftrl_kernel.cc:82-122, followed by the std::endl that
    // SparseOptimizerKernel::Serialized appends (optimizer_kernel.h:484).  Rows for which
    // DeleteByShow holds are left out.
    const char* Name() const { return opt.kind == K_ADAGRAD ? "AdaGrad" : opt.kind == K_ADAM ? "Adam" : "Ftrl"; }

    void SerializeRowTxt(std::ostream& os, const Row* r) const {
        const float* w = r->data;
        if (opt.kind == K_ADAGRAD) {
            os << D << "\t";
            for (int i = 0; i < D; i++) os << w[i] << "\t";
            os << r->g2sum << "\t";
            os << r->show << "\t";
            os << r->no_show_days << "\t";
            if (opt.use_cvm) os << r->click;
        } else {
            const float* a = r->data + D;
            const float* b = r->data + 2 * D;
            for (int i = 0; i < D; i++) {
                os << w[i] << "\t";
                os << a[i] << "\t";
                os << b[i] << "\t";
            }
            os << r->show;
        }
    }

    void SerializeRowBin(std::ostream& os, const Row* r) const {
        os.write(reinterpret_cast<const char*>(r->data), D * sizeof(float));
        if (opt.kind == K_ADAGRAD) {
            os.write(reinterpret_cast<const char*>(&r->g2sum), sizeof(float));
            os.write(reinterpret_cast<const char*>(&r->show), sizeof(float));
            os.write(reinterpret_cast<const char*>(&r->no_show_days), sizeof(int));
            if (opt.use_cvm) os.write(reinterpret_cast<const char*>(&r->click), sizeof(float));
        } else {
            os.write(reinterpret_cast<const char*>(r->data + D), D * sizeof(float));
            os.write(reinterpret_cast<const char*>(r->data + 2 * D), D * sizeof(float));
            os.write(reinterpret_cast<const char*>(&r->show), sizeof(float));
        }
    }

    std::string SerializeBlock(int block, bool bin) const {
        std::ostringstream os;
        const Block& b = *blocks[block];
        if (bin) {
            os.write(reinterpret_cast<const char*>(&D), sizeof(D));
            for (const auto& kv : b.values) {
                if (DeleteByShow(kv.second)) continue;
                os.write(reinterpret_cast<const char*>(&kv.first), sizeof(kv.first));
                SerializeRowBin(os, kv.second);
            }
        } else {
            os << "opt_name:" << Name() << std::endl;
            os << "dim:" << D << std::endl;
            for (const auto& kv : b.values) {
                if (DeleteByShow(kv.second)) continue;
                os << kv.first << "\t";
                SerializeRowTxt(os, kv.second);
                os << std::endl;
            }
        }
        os << std::endl;
        return os.str();
    }

    void CvmColumns(Row* r) {
        if (!opt.use_cvm) return;
        float log_show = logf(r->show + 1);
        float log_click = logf(r->click + 1);
        r->data[D] = r->show;
        r->data[D + 1] = (log_click - log_show);
    }

    // a freshly allocated value (the reference allocates a new one per record and lets the
    // stream overwrite what the format holds)
    Row* FreshRow(uint64_t sign) {
        Row* r = GetOrCreate(sign);
        Construct(r);
        return r;
    }

    void DeSerializeRowTxt(std::istream& is, Row* r, bool old_compat) {
        float* w = r->data;
        if (opt.kind == K_ADAGRAD) {
            int dim_in_file;
            is >> dim_in_file;
            for (int i = 0; i < D; i++) is >> w[i];
            is >> r->g2sum;
            is >> r->show;
            if (!old_compat) {
                is >> r->no_show_days;
                if (opt.use_cvm) {
                    is >> r->click;
                    CvmColumns(r);
                }
            }
        } else {
            float* a = r->data + D;
            float* b = r->data + 2 * D;
            for (int i = 0; i < D; i++) {
                is >> w[i];
                is >> a[i];
                is >> b[i];
            }
            is >> r->show;
        }
    }

    // returns the number of rows read, -1 on an optimizer / dim mismatch
    int64_t DeSerializeBlock(const std::string& data, bool bin) {
        std::istringstream is(data);
        int64_t n = 0;
        if (bin) {
            int dim = 0;
            is.read(reinterpret_cast<char*>(&dim), sizeof(dim));
            if (dim != D) return -1;
            uint64_t sign = 0;
            while (is.read(reinterpret_cast<char*>(&sign), sizeof(sign))) {
                Row* r = FreshRow(sign);
                is.read(reinterpret_cast<char*>(r->data), D * sizeof(float));
                if (opt.kind == K_ADAGRAD) {
                    is.read(reinterpret_cast<char*>(&r->g2sum), sizeof(float));
                    is.read(reinterpret_cast<char*>(&r->show), sizeof(float));
                    is.read(reinterpret_cast<char*>(&r->no_show_days), sizeof(int));
                    if (opt.use_cvm) {
                        is.read(reinterpret_cast<char*>(&r->click), sizeof(float));
                        CvmColumns(r);
                    }
                } else {
                    is.read(reinterpret_cast<char*>(r->data + D), D * sizeof(float));
                    is.read(reinterpret_cast<char*>(r->data + 2 * D), D * sizeof(float));
                    is.read(reinterpret_cast<char*>(&r->show), sizeof(float));
                }
                n++;
            }
            return n;
        }
        std::string opt_name;
        is.ignore(std::numeric_limits<std::streamsize>::max(), ':') >> opt_name;
        if (opt_name != Name()) return -1;
        int dim = 0;
        is.ignore(std::numeric_limits<std::streamsize>::max(), ':') >> dim;
        if (dim != D) return -1;
        // AdaGrad::NeedOldCompat (optimizer.h:94-115): the first row decides whether the file predates
        // the no_show_days column; that row is then parsed from the sampled line
        bool old_compat = false;
        std::string sample;
        if (opt.kind == K_ADAGRAD) {
            std::string line, cell;
            std::getline(is, line);
            std::getline(is, line);
            std::istringstream iss(line);
            int columns = 0;
            while (std::getline(iss, cell, '\t')) ++columns;
            old_compat = columns == D + 4;
            sample = line;
        }
        std::istringstream sample_is(sample);
        uint64_t sign = 0;
        while (sample_is >> sign) {
            DeSerializeRowTxt(sample_is, FreshRow(sign), old_compat);
            n++;
        }
        while (is >> sign) {
            DeSerializeRowTxt(is, FreshRow(sign), old_compat);
            n++;
        }
        return n;
    }

    Opt opt;
    int D, wdim, payload;
    std::minstd_rand rng;  // std::default_random_engine in libstdc++

    int StateFloats() const { return opt.kind == K_ADAGRAD ? 4 : 2 * D + 2; }

    void GetState(const Row* r, float* st) const {
        if (opt.kind == K_ADAGRAD) {
            st[0] = r->g2sum;
            st[1] = r->show;
            st[2] = r->click;
            std::memcpy(&st[3], &r->no_show_days, 4);
        } else {
            std::memcpy(st, r->data + D, sizeof(float) * 2 * D);
            st[2 * D] = r->show;
            std::memcpy(&st[2 * D + 1], &r->delta_show, 4);
        }
    }
    void SetState(Row* r, const float* st) {
        if (opt.kind == K_ADAGRAD) {
            r->g2sum = st[0];
            r->show = st[1];
            r->click = st[2];
            std::memcpy(&r->no_show_days, &st[3], 4);
        } else {
            std::memcpy(r->data + D, st, sizeof(float) * 2 * D);
            r->show = st[2 * D];
            std::memcpy(&r->delta_show, &st[2 * D + 1], 4);
        }
    }

private:
    struct Block {
        Block(size_t buckets, int bytes) : values(buckets), pool(bytes, 1 << 16) { values.max_load_factor(0.75f); }
        std::unordered_map<uint64_t, Row*, KeyHasher> values;
        Pool pool;
    };
    std::vector<std::unique_ptr<Block>> blocks;
};

// ------------------------------------------------------------------- remap
// SparsePullVarInfo ctor, core/kernels/sparse_table_ops.cc:119-131
int64_t PullRemap(const int64_t* values, int64_t n, int64_t* out, std::vector<uint64_t>& signs) {
    std::map<uint64_t, size_t> sign_id_mapping;
    for (int64_t i = 0; i < n; ++i) {
        const uint64_t sign = (uint64_t)values[i];
        auto inserted = sign_id_mapping.insert({sign, sign_id_mapping.size()});
        if (inserted.second) signs.push_back(sign);
        out[i] = (int64_t)inserted.first->second;
    }
    return (int64_t)signs.size();
}

// SparsePushVarInfo ctor, core/kernels/sparse_table_ops.cc:280-296
void PushRemap(const int64_t* values, const int64_t* labels, int64_t n, std::vector<SignInfo>& infos) {
    std::map<uint64_t, int> sign_id_mapping;
    for (int64_t i = 0; i < n; ++i) {
        uint64_t sign = (uint64_t)values[i];
        int label = static_cast<int>(labels[i]);
        auto ret = sign_id_mapping.insert({sign, (int)sign_id_mapping.size()});
        if (ret.second) {
            infos.push_back(SignInfo{sign, 1, label});
        } else {
            infos[ret.first->second].batch_show += 1;
            infos[ret.first->second].batch_click += label;
        }
    }
}

// ------------------------------------------------------------------- dense
// DenseOptimizerKernel + DenseAdamValue / DenseAdaGradValue for one worker:
// [0,total) cut into 8 blocks of ceil(total/8) (optimizer_kernel.h:174-188),
// each with its own beta powers (adam_kernel.cc:26-38).
struct DenseBlock {
    float beta1_power = 1, beta2_power = 1;
    std::vector<float> w, a, b, c;  // Adam: w,m,v ; AdaGrad: w,d2sum,g2sum,m
};

struct Dense {
    Opt opt;
    int64_t total = 0;
    std::vector<DenseBlock> blocks;

    void Init(int64_t total_elements) {
        total = total_elements;
        size_t per_block = (size_t)std::ceil(total * 1.0 / 8);  // DENSE_KERNEL_BLOCK_NUM
        for (size_t off = 0; off < (size_t)total; off += per_block) {
            size_t sz = per_block;
            if (off + per_block > (size_t)total) sz = total - off;
            DenseBlock blk;
            blk.w.assign(sz, 0.0f);
            blk.a.assign(sz, 0.0f);
            if (opt.kind == K_ADAGRAD) {
                blk.b.assign(sz, opt.initial_g2sum);  // ada_grad_kernel.cc:31-33
                blk.c.assign(sz, 0.0f);
            } else {
                blk.b.assign(sz, 0.0f);
            }
            blocks.push_back(std::move(blk));
        }
    }

    void SetWeight(const float* w) {  // optimizer_kernel.h:206-214
        size_t off = 0;
        for (auto& b : blocks) {
            std::memcpy(b.w.data(), w + off, b.w.size() * sizeof(float));
            off += b.w.size();
        }
    }

    void GetWeight(float* w) const {  // optimizer_kernel.h:216-221
        size_t off = 0;
        for (auto& b : blocks) {
            std::memcpy(w + off, b.w.data(), b.w.size() * sizeof(float));
            off += b.w.size();
        }
    }

    // DenseOptimizerKernel::Apply, optimizer_kernel.h:192-204: the block's slice of
    // the gradient is first copied into a fresh array, then applied.
    void Apply(const float* grad, float lr) {
        size_t off = 0;
        for (auto& b : blocks) {
            std::vector<float> g(grad + off, grad + off + b.w.size());
            if (opt.kind == K_ADAGRAD)
                ApplyAdaGrad(b, g.data(), lr);
            else
                ApplyAdam(b, g.data(), lr);
            off += b.w.size();
        }
    }

    const char* Name() const { return opt.kind == K_ADAGRAD ? "AdaGrad" : "Adam"; }

    // DenseTable::Save (core/ps/table/dense_table.cc:103-128) down to the value streams:
    // table header, then DenseOptimizerKernel::Serialized (optimizer_kernel.h:224-229) =
    // per block "opt_name:" + value + endl (block stream, :139-146) + endl, the value being
    // DenseAdamValue's (adam_kernel.cc:57-69) or DenseAdaGradValue's (ada_grad_kernel.cc:50-60).
    // `total` here is the length of one shard's kernel; table_total is what the table of
    // all shards holds (equal with one shard).
    std::string Serialize(int rank_num, int table_total) const {
        std::ostringstream os;
        os << "total_elements:" << table_total << std::endl;
        os << "rank_num:" << rank_num << std::endl;
        for (const DenseBlock& b : blocks) {
            os << "opt_name:" << Name() << std::endl;
            int array_size = (int)b.w.size();
            os << "array_size:" << array_size << std::endl;
            if (opt.kind == K_ADAM) {
                os << "beta1_power:" << b.beta1_power << std::endl;
                os << "beta2_power:" << b.beta2_power << std::endl;
                for (int i = 0; i < array_size; i++) os << b.w[i] << "\t" << b.a[i] << "\t" << b.b[i] << std::endl;
            } else {
                for (int i = 0; i < array_size; i++)
                    os << b.w[i] << "\t" << b.a[i] << "\t" << b.b[i] << "\t" << b.c[i] << std::endl;
            }
            os << std::endl;  // block stream: os << value << endl
            os << std::endl;  // Serialized: os << block << endl
        }
        return os.str();
    }

    // DenseTable::Load (dense_table.cc:130-157) on a table created with the file's total;
    // returns 0, or -1 total / -2 rank_num / -3 optimizer / -4 block length mismatch (the
    // reference's CHECKs).  Value streams: adam_kernel.cc:71-87, ada_grad_kernel.cc:62-76.
    int DeSerialize(const std::string& data, int shard_num, int table_total) {
        std::istringstream is(data);
        const auto skip = std::numeric_limits<std::streamsize>::max();
        int total_elements = 0, rank_num = 0;
        is.ignore(skip, ':') >> total_elements;
        is.ignore(skip, ':') >> rank_num;
        if (shard_num != rank_num) return -2;
        if (total_elements != table_total) return -1;
        for (DenseBlock& b : blocks) {
            std::string name;
            is.ignore(skip, ':') >> name;
            if (name != Name()) return -3;
            int array_size = 0;
            is.ignore(skip, ':') >> array_size;
            if (array_size != (int)b.w.size()) return -4;
            if (opt.kind == K_ADAM) {
                is.ignore(skip, ':') >> b.beta1_power;
                is.ignore(skip, ':') >> b.beta2_power;
                for (int i = 0; i < array_size; i++) is >> b.w[i] >> b.a[i] >> b.b[i];
            } else {
                for (int i = 0; i < array_size; i++) is >> b.w[i] >> b.a[i] >> b.b[i] >> b.c[i];
            }
        }
        return 0;
    }

    // DenseAdamValue::Apply, adam_kernel.cc:46-55.  Eigen evaluates each
    // expression elementwise in float; double scalars are narrowed to float first.
    void ApplyAdam(DenseBlock& b, const float* g, float lr) {
        b.beta1_power *= opt.beta1;
        b.beta2_power *= opt.beta2;
        const float alpha = (float)(lr * std::sqrt(1.0 - b.beta2_power) / (1.0 - b.beta1_power));
        const float c1 = (float)(1.0 - opt.beta1);
        const float c2 = (float)(1.0 - opt.beta2);
        const size_t n = b.w.size();
        float* w = b.w.data();
        float* m = b.a.data();
        float* v = b.b.data();
        for (size_t i = 0; i < n; i++) {
            m[i] += (g[i] - m[i]) * c1;
            v[i] += (g[i] * g[i] - v[i]) * c2;
            w[i] -= (m[i] * alpha) / (sqrtf(v[i]) + opt.epsilon);
        }
    }

    // DenseAdaGradValue::Apply, ada_grad_kernel.cc:42-48
    void ApplyAdaGrad(DenseBlock& b, const float* g, float lr) {
        const float c = (float)(1.0 - opt.mom_decay_rate);
        const size_t n = b.w.size();
        float* w = b.w.data();
        float* d2 = b.a.data();
        float* g2 = b.b.data();
        float* m = b.c.data();
        for (size_t i = 0; i < n; i++) {
            d2[i] = opt.grad_decay_rate * d2[i] + 1;
            g2[i] = opt.grad_decay_rate * g2[i] + g[i] * g[i];
            m[i] += (g[i] - m[i]) * c;
            w[i] -= lr * m[i] / (sqrtf(g2[i]) / sqrtf(d2[i]) + opt.epsilon);
        }
    }
};

void FillOpt(Opt& o, int kind, const float* p, int use_cvm, int zero_init) {
    o.kind = kind;
    o.use_cvm = use_cvm != 0;
    o.sparse_zero_init = zero_init != 0;
    o.learning_rate = p[0];
    if (kind == K_ADAGRAD) {
        o.initial_g2sum = p[1];
        o.initial_scale = p[2];
        o.epsilon = p[3];
        o.grad_decay_rate = p[4];
        o.mom_decay_rate = p[5];
    } else if (kind == K_ADAM) {
        o.beta1 = p[1];
        o.beta2 = p[2];
        o.epsilon = p[3];
        o.initial_scale = p[4];
    } else {
        o.beta = p[1];
        o.lambda1 = p[2];
        o.lambda2 = p[3];
        o.initial_scale = p[4];
    }
    // common tail of the parameter array
    o.show_decay_rate = p[8];
    o.show_threshold = p[9];
    o.no_show_days = (int)p[10];
    o.elimination_logic = (int)p[11];
}

}  // namespace

// ------------------------------------------------------------------- C ABI
extern "C" {

// params: AdaGrad {lr, initial_g2sum, initial_scale, epsilon, grad_decay_rate, mom_decay_rate}
//         Adam    {lr, beta1, beta2, epsilon, initial_scale}
//         Ftrl    {lr, beta, lambda1, lambda2, initial_scale}
//         all kinds, at [8..11]: {show_decay_rate, show_threshold, no_show_days, elimination_logic}
// buckets: initial bucket count per hash block (the reference uses 15485863).
void* orc_table_create(int kind, const float* params, int dim, int use_cvm, int zero_init, uint64_t seed,
                       uint64_t buckets) {
    Opt o;
    FillOpt(o, kind, params, use_cvm, zero_init);
    return new Table(o, dim, seed, (size_t)buckets);
}
void orc_table_destroy(void* t) { delete static_cast<Table*>(t); }
int orc_table_weight_floats(void* t) { return static_cast<Table*>(t)->wdim; }
int orc_table_state_floats(void* t) { return static_cast<Table*>(t)->StateFloats(); }
uint64_t orc_table_key_count(void* t) { return static_cast<Table*>(t)->KeyCount(); }
void orc_table_show_decay(void* t, int delta_days) { static_cast<Table*>(t)->ShowDecay(delta_days); }
// Checkpoint stream of hash block `block` (uncompressed).  Returns its size; copies it if cap suffices.
int64_t orc_table_serialize_block(void* tp, int block, int bin, uint8_t* out, int64_t cap) {
    const std::string s = static_cast<Table*>(tp)->SerializeBlock(block, bin != 0);
    if ((int64_t)s.size() <= cap && out) std::memcpy(out, s.data(), s.size());
    return (int64_t)s.size();
}
// Reads such a stream back; returns the rows read, -1 on a mismatch of optimizer or dim.
int64_t orc_table_deserialize_block(void* tp, int bin, const uint8_t* data, int64_t n) {
    return static_cast<Table*>(tp)->DeSerializeBlock(std::string(reinterpret_cast<const char*>(data), (size_t)n), bin != 0);
}
// out[i] = 1 if signs[i] is resident and Value::DeleteByShow holds for its row
void orc_table_delete_by_show(void* tp, const uint64_t* signs, int64_t n, uint8_t* out) {
    Table* t = static_cast<Table*>(tp);
    for (int64_t i = 0; i < n; ++i) {
        Row* r = t->Find(signs[i]);
        out[i] = (r && t->DeleteByShow(r)) ? 1 : 0;
    }
}

// Snapshot injection through the row pointer (what the reference allows via
// the mutable float* of SparseOptimizerKernelBase::GetWeight, optimizer_kernel.h:84).
void orc_table_set_rows(void* tp, const uint64_t* signs, const float* w, const float* state, int64_t n) {
    Table* t = static_cast<Table*>(tp);
    int sf = t->StateFloats();
    for (int64_t i = 0; i < n; i++) {
        Row* r = t->GetOrCreate(signs[i]);
        std::memcpy(r->data, w + i * t->wdim, sizeof(float) * t->wdim);
        if (state) t->SetState(r, state + i * sf);
    }
}
// found[i] = 0 for absent signs (rows left untouched).
void orc_table_get_rows(void* tp, const uint64_t* signs, int64_t n, float* w, float* state, uint8_t* found) {
    Table* t = static_cast<Table*>(tp);
    int sf = t->StateFloats();
    for (int64_t i = 0; i < n; i++) {
        Row* r = t->Find(signs[i]);
        found[i] = r ? 1 : 0;
        if (!r) continue;
        std::memcpy(w + i * t->wdim, r->data, sizeof(float) * t->wdim);
        if (state) t->GetState(r, state + i * sf);
    }
}

void orc_table_pull(void* tp, const uint64_t* signs, int64_t n, int dim, float* out) {
    ByteQueue q;
    static_cast<Table*>(tp)->Pull(signs, n, dim, q);
    q.cutn(out, sizeof(float) * dim * n);
}

// returns the number of records whose sign was absent (the reference aborts on the first)
int orc_table_push(void* tp, const SignInfo* infos, const float* grads, int64_t n, int dim) {
    ByteQueue q;
    for (int64_t i = 0; i < n; i++) {
        q.append(&infos[i], sizeof(SignInfo));
        q.append(grads + i * dim, sizeof(float) * dim);
    }
    return static_cast<Table*>(tp)->Push(q, dim);
}

int64_t orc_pull_remap(const int64_t* values, int64_t n, int64_t* mapped, uint64_t* signs_out) {
    std::vector<uint64_t> signs;
    int64_t u = PullRemap(values, n, mapped, signs);
    if (signs_out) std::memcpy(signs_out, signs.data(), sizeof(uint64_t) * signs.size());
    return u;
}

int64_t orc_push_remap(const int64_t* values, const int64_t* labels, int64_t n, SignInfo* infos_out) {
    std::vector<SignInfo> infos;
    PushRemap(values, labels, n, infos);
    std::memcpy(infos_out, infos.data(), sizeof(SignInfo) * infos.size());
    return (int64_t)infos.size();
}

// SparseTablePullKernel::ComputeAsync with one shard, core/kernels/sparse_table_ops.cc:170-265.
// Returns 0, or 4 when a slot has U_s >= var_rows[s] (CHECK_LT :136), or 3 on dim mismatch.
int orc_pull_op(void* tp, int N, const int64_t* const* values, const int64_t* lens, float* const* vars,
                const int64_t* var_rows, int var_dim, int64_t* const* mapped, int64_t* uniq_counts) {
    Table* t = static_cast<Table*>(tp);
    std::vector<std::vector<uint64_t>> slot_signs(N);
    for (int s = 0; s < N; s++) {
        int64_t u = PullRemap(values[s], lens[s], mapped[s], slot_signs[s]);
        if (uniq_counts) uniq_counts[s] = u;
        if (!(u < var_rows[s])) return 4;
    }
    // request: signs of all slots in slot order with (var_index, sign_index) (:217-224)
    std::vector<uint64_t> req;
    std::vector<std::pair<size_t, size_t>> call_sign_infos;
    for (int s = 0; s < N; s++)
        for (size_t j = 0; j < slot_signs[s].size(); j++) {
            req.push_back(slot_signs[s][j]);
            call_sign_infos.emplace_back((size_t)s, j);
        }
    ByteQueue emb;
    t->Pull(req.data(), (int64_t)req.size(), var_dim, emb);
    // PopulatePulledVariable_ (:244-265)
    size_t emb_size = sizeof(float) * var_dim;
    for (size_t i = 0; i < call_sign_infos.size(); i++) {
        float* w_matrix = vars[call_sign_infos[i].first];
        emb.cutn(w_matrix + call_sign_infos[i].second * var_dim, emb_size);
    }
    return 0;
}

// SparseTablePushKernel::ComputeAsync with one shard, core/kernels/sparse_table_ops.cc:317-368.
// Returns the number of records with an unknown sign.
int orc_push_op(void* tp, int N, const int64_t* const* values, const int64_t* lens, const float* const* grads,
                int grad_dim, const int64_t* const* labels, int64_t* uniq_counts) {
    Table* t = static_cast<Table*>(tp);
    ByteQueue buf;
    for (int s = 0; s < N; s++) {
        std::vector<SignInfo> infos;
        PushRemap(values[s], labels[s], lens[s], infos);
        if (uniq_counts) uniq_counts[s] = (int64_t)infos.size();
        const float* grad_matrix = grads[s];
        for (size_t j = 0; j < infos.size(); j++) {
            buf.append(&infos[j], sizeof(SignInfo));
            buf.append(grad_matrix + (size_t)grad_dim * j, sizeof(float) * grad_dim);
        }
    }
    return t->Push(buf, grad_dim);
}

// Dense: params as for orc_table_create.
void* orc_dense_create(int kind, const float* params, int64_t total) {
    Dense* d = new Dense();
    FillOpt(d->opt, kind, params, 0, 0);
    d->Init(total);
    return d;
}
void orc_dense_destroy(void* d) { delete static_cast<Dense*>(d); }
void orc_dense_set_weight(void* d, const float* w) { static_cast<Dense*>(d)->SetWeight(w); }
void orc_dense_get_weight(void* d, float* w) { static_cast<Dense*>(d)->GetWeight(w); }
void orc_dense_apply(void* d, const float* grad, float lr) { static_cast<Dense*>(d)->Apply(grad, lr); }
// The text of the table's checkpoint file.  Returns its size; copies it if cap suffices.
int64_t orc_dense_serialize(void* dp, int rank_num, int table_total, uint8_t* out, int64_t cap) {
    const std::string s = static_cast<Dense*>(dp)->Serialize(rank_num, table_total);
    if ((int64_t)s.size() <= cap && out) std::memcpy(out, s.data(), s.size());
    return (int64_t)s.size();
}
int orc_dense_deserialize(void* dp, int shard_num, int table_total, const uint8_t* data, int64_t n) {
    return static_cast<Dense*>(dp)->DeSerialize(std::string(reinterpret_cast<const char*>(data), (size_t)n), shard_num,
                                                table_total);
}
void orc_dense_get_powers(void* dp, int block, float* out) {
    const DenseBlock& b = static_cast<Dense*>(dp)->blocks[(size_t)block];
    out[0] = b.beta1_power;
    out[1] = b.beta2_power;
}
int orc_dense_num_blocks(void* d) { return (int)static_cast<Dense*>(d)->blocks.size(); }
// which: 0 = first state array (Adam m / AdaGrad d2sum), 1 = second (v / g2sum), 2 = third (AdaGrad m)
void orc_dense_get_state(void* dp, int which, float* out) {
    Dense* d = static_cast<Dense*>(dp);
    size_t off = 0;
    for (auto& b : d->blocks) {
        const std::vector<float>& src = which == 0 ? b.a : (which == 1 ? b.b : b.c);
        if (!src.empty()) std::memcpy(out + off, src.data(), src.size() * sizeof(float));
        off += b.w.size();
    }
}

}  // extern "C"
