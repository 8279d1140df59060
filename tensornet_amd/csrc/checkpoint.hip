// SparseTable::Save / Load in the reference's on-disk formats
// (core/ps/table/sparse_table.cc:84-137, SparseOptimizerKernel::Serialized / DeSerialized,
// core/ps/optimizer/optimizer_kernel.h:462-538, block streams :324-420, value formats
// ada_grad_kernel.cc:131-189, adam_kernel.cc:127-167, ftrl_kernel.cc:82-122):
//
//   <filepath>/sparse_table/<name or handle>/rank_0/block_<i>.gz      i = 0..7, gzip
//   row of sign s goes to file (s >> 32 | s << 32) % 8                (optimizer_kernel.h:248-252,556)
//   bin:  int32 dim, then per row {u64 sign, value}, then '\n'
//         AdaGrad value  w[dim] g2sum show no_show_days(i32) [click if cvm]
//         Adam / Ftrl    w[dim] m|z[dim] v|n[dim] show
//   txt:  "opt_name:<Name>\n" "dim:<dim>\n", one row per line, tab separated, floats as
//         operator<< prints them (%g, 6 significant digits), then '\n'
//         AdaGrad  sign dim w.. g2sum show no_show_days [click]      Adam / Ftrl  sign (w m v).. show
//   rows for which DeleteByShow holds are left out of a saved table.
//
// Host code over the library's own C ABI: the table is read out of HBM range by range
// (tn_sparse_table_export_range) and filled through tn_sparse_table_load_rows.
#include <dirent.h>
#include <sys/stat.h>
#include <zlib.h>

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <regex>
#include <string>
#include <thread>
#include <vector>

#include "tensornet_amd.h"
#include "tn_common.h"

namespace tn {
namespace {

constexpr int kBlocks = 8;                       // SPARSE_KERNEL_BLOCK_NUM
constexpr uint64_t kChunkSlots = 1ull << 20;     // table slots read out per round
constexpr size_t kLoadBatch = 1u << 20;          // rows handed to the table per round

int block_of(uint64_t sign) { return (int)(((sign >> 32) | (sign << 32)) % kBlocks); }

const char* opt_name(int kind) { return kind == OPT_ADAGRAD ? "AdaGrad" : kind == OPT_ADAM ? "Adam" : "Ftrl"; }

int make_dirs(const std::string& path) {
    std::string cur;
    for (size_t i = 0; i <= path.size(); i++) {
        if (i == path.size() || path[i] == '/') {
            if (!cur.empty() && ::mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST)
                return fail(TN_ERR_INVALID_ARGUMENT, "cannot create directory " + cur);
        }
        if (i < path.size()) cur.push_back(path[i]);
    }
    return TN_OK;
}

bool dir_exists(const std::string& path) {
    struct stat sb;
    return ::stat(path.c_str(), &sb) == 0 && S_ISDIR(sb.st_mode);
}

// what operator<< prints for a float / an int with default stream flags
void put_float(std::string& out, float v) {
    char buf[48];
    std::snprintf(buf, sizeof(buf), "%g", (double)v);
    out += buf;
}

struct TableInfo {
    uint32_t handle;
    int kind, use_cvm, wf, sf, dim;
    std::string dir;  // .../rank_0
};

int table_info(uint32_t handle, const char* filepath, bool for_load, TableInfo& ti) {
    ti.handle = handle;
    TN_TRY(tn_sparse_table_optimizer(handle, &ti.kind, &ti.use_cvm));
    TN_TRY(tn_sparse_table_row_layout(handle, &ti.wf, &ti.sf));
    ti.dim = ti.wf - (ti.use_cvm ? 2 : 0);
    char name[512];
    TN_TRY(tn_sparse_table_name(handle, name, (int)sizeof(name)));
    std::string base = std::string(filepath) + "/sparse_table/";
    std::string ident = std::to_string(handle);
    // sparse_table.cc:89-93,115-121: the table's name if it has one (on load: if that directory exists)
    if (name[0] && (!for_load || dir_exists(base + name))) ident = name;
    ti.dir = base + ident + "/rank_0";
    return TN_OK;
}

// ------------------------------------------------------------------ save
void append_row(const TableInfo& ti, bool bin, uint64_t sign, const float* w, const float* st, std::string& out) {
    const int D = ti.dim;
    if (bin) {
        out.append(reinterpret_cast<const char*>(&sign), 8);
        out.append(reinterpret_cast<const char*>(w), (size_t)D * 4);
        if (ti.kind == OPT_ADAGRAD) {
            out.append(reinterpret_cast<const char*>(&st[0]), 4);  // g2sum
            out.append(reinterpret_cast<const char*>(&st[1]), 4);  // show
            out.append(reinterpret_cast<const char*>(&st[3]), 4);  // no_show_days (int bits)
            if (ti.use_cvm) out.append(reinterpret_cast<const char*>(&st[2]), 4);  // click
        } else {
            out.append(reinterpret_cast<const char*>(st), (size_t)2 * D * 4);  // m, v / z, n
            out.append(reinterpret_cast<const char*>(&st[2 * D]), 4);          // show
        }
        return;
    }
    out += std::to_string(sign);
    out += '\t';
    if (ti.kind == OPT_ADAGRAD) {
        out += std::to_string(D);
        out += '\t';
        for (int i = 0; i < D; i++) {
            put_float(out, w[i]);
            out += '\t';
        }
        put_float(out, st[0]);
        out += '\t';
        put_float(out, st[1]);
        out += '\t';
        int days;
        std::memcpy(&days, &st[3], 4);
        out += std::to_string(days);
        out += '\t';
        if (ti.use_cvm) put_float(out, st[2]);
    } else {
        for (int i = 0; i < D; i++) {
            put_float(out, w[i]);
            out += '\t';
            put_float(out, st[i]);
            out += '\t';
            put_float(out, st[D + i]);
            out += '\t';
        }
        put_float(out, st[2 * D]);
    }
    out += '\n';
}

struct DeviceBufs {
    uint64_t* signs = nullptr;
    float* w = nullptr;
    float* st = nullptr;
    ~DeviceBufs() {
        if (signs) (void)hipFree(signs);
        if (w) (void)hipFree(w);
        if (st) (void)hipFree(st);
    }
    int alloc(size_t rows, int wf, int sf) {
        if (hipMalloc((void**)&signs, rows * 8) != hipSuccess || hipMalloc((void**)&w, rows * wf * 4) != hipSuccess ||
            hipMalloc((void**)&st, rows * sf * 4) != hipSuccess)
            return fail(TN_ERR_OUT_OF_MEMORY, "checkpoint: device staging buffers");
        return TN_OK;
    }
};

int save_table(uint32_t handle, const char* filepath, const char* mode) {
    if (!filepath || !mode) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: NULL argument");
    const bool bin = std::string(mode) == "bin";  // anything else is text, as in optimizer_kernel.h:475-479
    TableInfo ti;
    TN_TRY(table_info(handle, filepath, false, ti));
    TN_TRY(make_dirs(ti.dir));
    gzFile files[kBlocks] = {};
    auto close_all = [&]() {
        for (gzFile& f : files)
            if (f) {
                gzclose(f);
                f = nullptr;
            }
    };
    for (int b = 0; b < kBlocks; b++) {
        const std::string path = ti.dir + "/block_" + std::to_string(b) + ".gz";
        files[b] = gzopen(path.c_str(), "wb");
        if (!files[b]) {
            close_all();
            return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: cannot write " + path);
        }
        std::string head;
        if (bin) {
            head.append(reinterpret_cast<const char*>(&ti.dim), 4);
        } else {
            head = std::string("opt_name:") + opt_name(ti.kind) + "\ndim:" + std::to_string(ti.dim) + "\n";
        }
        if (gzwrite(files[b], head.data(), (unsigned)head.size()) != (int)head.size()) {
            close_all();
            return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: write failed in " + path);
        }
    }
    uint64_t cap = 0;
    int rc = tn_sparse_table_capacity(handle, &cap);
    DeviceBufs dev;
    if (rc == TN_OK) rc = dev.alloc(kChunkSlots, ti.wf, ti.sf);
    std::vector<uint64_t> hs(kChunkSlots);
    std::vector<float> hw(kChunkSlots * ti.wf), hst(kChunkSlots * ti.sf);
    for (uint64_t first = 0; rc == TN_OK && first <= cap; first += kChunkSlots) {
        uint64_t n = 0;
        rc = tn_sparse_table_export_range(handle, first, kChunkSlots, 1, dev.signs, dev.w, dev.st, &n, nullptr);
        if (rc != TN_OK || n == 0) continue;
        if (hipMemcpy(hs.data(), dev.signs, n * 8, hipMemcpyDeviceToHost) != hipSuccess ||
            hipMemcpy(hw.data(), dev.w, n * ti.wf * 4, hipMemcpyDeviceToHost) != hipSuccess ||
            hipMemcpy(hst.data(), dev.st, n * ti.sf * 4, hipMemcpyDeviceToHost) != hipSuccess) {
            rc = fail(TN_ERR_HIP, "tn_sparse_table_save: copy to the host failed");
            break;
        }
        // one thread per file: format and compress the block's share of the chunk
        std::vector<std::thread> threads;
        std::vector<int> ok(kBlocks, 1);
        for (int b = 0; b < kBlocks; b++) {
            threads.emplace_back([&, b]() {
                std::string out;
                for (uint64_t i = 0; i < n; i++)
                    if (block_of(hs[i]) == b) append_row(ti, bin, hs[i], &hw[i * ti.wf], &hst[i * ti.sf], out);
                for (size_t off = 0; off < out.size();) {
                    const unsigned part = (unsigned)std::min<size_t>(out.size() - off, 1u << 30);
                    if (gzwrite(files[b], out.data() + off, part) != (int)part) {
                        ok[b] = 0;
                        return;
                    }
                    off += part;
                }
            });
        }
        for (auto& th : threads) th.join();
        for (int b = 0; b < kBlocks; b++)
            if (!ok[b]) rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: write failed in " + ti.dir);
    }
    for (int b = 0; b < kBlocks && rc == TN_OK; b++)  // the std::endl after the block
        if (gzwrite(files[b], "\n", 1) != 1) rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: write failed in " + ti.dir);
    // closing flushes what zlib still holds: a full disk shows here at the latest
    for (gzFile& f : files)
        if (f) {
            if (gzclose(f) != Z_OK && rc == TN_OK)
                rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_save: closing a block file failed in " + ti.dir);
            f = nullptr;
        }
    return rc;
}

// ------------------------------------------------------------------ load
int read_gz(const std::string& path, std::string& out) {
    gzFile f = gzopen(path.c_str(), "rb");
    if (!f) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: cannot read " + path);
    std::vector<char> buf(1 << 20);
    int got;
    while ((got = gzread(f, buf.data(), (unsigned)buf.size())) > 0) out.append(buf.data(), (size_t)got);
    gzclose(f);
    if (got < 0) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: corrupt file " + path);
    return TN_OK;
}

struct RowBatch {
    std::vector<uint64_t> signs;
    std::vector<float> w, st;
};

// Rows waiting to go to the table, in the layout tn_sparse_table_load_rows takes.
struct Loader {
    const TableInfo& ti;
    DeviceBufs dev;
    RowBatch batch;
    explicit Loader(const TableInfo& t) : ti(t) {}

    int init() { return dev.alloc(kLoadBatch, ti.wf, ti.sf); }

    // value fields in file order; fields the format lacks keep what a fresh value holds
    void add(uint64_t sign, const float* w, float g2sum_or_show, const float* a, const float* b, float show, int days,
             float click, bool cvm_columns) {
        const int D = ti.dim;
        batch.signs.push_back(sign);
        const size_t w0 = batch.w.size(), s0 = batch.st.size();
        batch.w.resize(w0 + ti.wf, 0.f);
        batch.st.resize(s0 + ti.sf, 0.f);
        std::memcpy(&batch.w[w0], w, (size_t)D * 4);
        if (ti.kind == OPT_ADAGRAD) {
            float* st = &batch.st[s0];
            st[0] = g2sum_or_show;
            st[1] = show;
            st[2] = click;
            std::memcpy(&st[3], &days, 4);
            if (ti.use_cvm && cvm_columns) {  // ada_grad_kernel.cc:158-163,181-186
                const float log_show = logf(show + 1);
                const float log_click = logf(click + 1);
                batch.w[w0 + D] = show;
                batch.w[w0 + D + 1] = (log_click - log_show);
            }
        } else {
            std::memcpy(&batch.st[s0], a, (size_t)D * 4);
            std::memcpy(&batch.st[s0 + D], b, (size_t)D * 4);
            batch.st[s0 + 2 * D] = show;  // delta_show stays 0
        }
    }

    int flush() {
        const size_t n = batch.signs.size();
        if (n == 0) return TN_OK;
        if (hipMemcpy(dev.signs, batch.signs.data(), n * 8, hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(dev.w, batch.w.data(), n * ti.wf * 4, hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(dev.st, batch.st.data(), n * ti.sf * 4, hipMemcpyHostToDevice) != hipSuccess)
            return fail(TN_ERR_HIP, "tn_sparse_table_load: copy to the device failed");
        TN_TRY(tn_sparse_table_load_rows(ti.handle, dev.signs, dev.w, dev.st, (int64_t)n, nullptr));
        batch.signs.clear();
        batch.w.clear();
        batch.st.clear();
        return TN_OK;
    }

    int maybe_flush() { return batch.signs.size() >= kLoadBatch ? flush() : TN_OK; }
};

int parse_bin(const TableInfo& ti, const std::string& data, Loader& ld) {
    const int D = ti.dim;
    if (data.size() < 4) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: truncated block file");
    int dim;
    std::memcpy(&dim, data.data(), 4);
    if (dim != D)
        return fail(TN_ERR_DIM_MISMATCH, "tn_sparse_table_load: file holds dim " + std::to_string(dim) + ", table " +
                                             std::to_string(D));
    const size_t value = ti.kind == OPT_ADAGRAD ? (size_t)D * 4 + 12 + (ti.use_cvm ? 4 : 0) : (size_t)3 * D * 4 + 4;
    size_t off = 4;
    while (off + 8 + value <= data.size()) {  // a short tail (the final '\n') ends the stream, as is.read does
        uint64_t sign;
        std::memcpy(&sign, &data[off], 8);
        const float* p = reinterpret_cast<const float*>(&data[off + 8]);
        std::vector<float> v(value / 4);
        std::memcpy(v.data(), p, value);
        if (ti.kind == OPT_ADAGRAD) {
            int days;
            std::memcpy(&days, &v[D + 2], 4);
            ld.add(sign, v.data(), v[D], nullptr, nullptr, v[D + 1], days, ti.use_cvm ? v[D + 3] : 0.f, true);
        } else {
            ld.add(sign, v.data(), 0.f, &v[D], &v[2 * D], v[3 * D], 0, 0.f, false);
        }
        TN_TRY(ld.maybe_flush());
        off += 8 + value;
    }
    return TN_OK;
}

// whitespace-separated tokens, as operator>> reads them
struct Tokens {
    const char* p;
    const char* end;
    bool next(const char*& b, const char*& e) {
        while (p < end && (*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) p++;
        if (p >= end) return false;
        b = p;
        while (p < end && !(*p == ' ' || *p == '\t' || *p == '\n' || *p == '\r')) p++;
        e = p;
        return true;
    }
    bool u64(uint64_t& v) {
        const char *b, *e;
        if (!next(b, e)) return false;
        v = std::strtoull(std::string(b, e).c_str(), nullptr, 10);
        return true;
    }
    bool f32(float& v) {
        const char *b, *e;
        if (!next(b, e)) return false;
        v = std::strtof(std::string(b, e).c_str(), nullptr);
        return true;
    }
    bool i32(int& v) {
        const char *b, *e;
        if (!next(b, e)) return false;
        v = (int)std::strtol(std::string(b, e).c_str(), nullptr, 10);
        return true;
    }
};

int parse_txt(const TableInfo& ti, const std::string& data, Loader& ld) {
    const int D = ti.dim;
    // "opt_name:<Name>\n" "dim:<dim>\n"
    size_t c1 = data.find(':');
    if (c1 == std::string::npos) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: no header in block file");
    size_t e1 = data.find('\n', c1);
    const std::string name = data.substr(c1 + 1, e1 == std::string::npos ? std::string::npos : e1 - c1 - 1);
    if (name != opt_name(ti.kind))  // optimizer_kernel.h:370-373
        return fail(TN_ERR_INVALID_ARGUMENT, "last trained model with optimizer is:" + name + " but current model use:" +
                                                 opt_name(ti.kind) + " instead");
    size_t c2 = data.find(':', e1);
    if (c2 == std::string::npos) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: no dim in block file");
    size_t e2 = data.find('\n', c2);
    if (e2 == std::string::npos) e2 = data.size();
    const int dim = std::atoi(data.substr(c2 + 1, e2 - c2 - 1).c_str());
    if (dim != D)
        return fail(TN_ERR_DIM_MISMATCH, "tn_sparse_table_load: file holds dim " + std::to_string(dim) + ", table " +
                                             std::to_string(D));
    size_t body = std::min(e2 + 1, data.size());
    // AdaGrad::NeedOldCompat (optimizer.h:94-115): dim + 4 columns in the first row = a file without no_show_days
    bool old_compat = false;
    if (ti.kind == OPT_ADAGRAD) {
        size_t le = data.find('\n', body);
        if (le == std::string::npos) le = data.size();
        int columns = 0;
        size_t s = body;
        while (s < le) {  // std::getline(.., '\t'): a trailing tab opens no further cell
            size_t t = data.find('\t', s);
            if (t == std::string::npos || t > le) t = le;
            columns++;
            s = t + 1;
        }
        old_compat = columns == D + 4;
    }
    Tokens tk{data.data() + body, data.data() + data.size()};
    std::vector<float> w(D), a(D), b(D);
    uint64_t sign;
    while (tk.u64(sign)) {
        if (ti.kind == OPT_ADAGRAD) {
            int dim_in_row = 0, days = 0;
            float g2sum = 0.f, show = 0.f, click = 0.f;
            tk.i32(dim_in_row);
            for (int i = 0; i < D; i++) tk.f32(w[i]);
            tk.f32(g2sum);
            tk.f32(show);
            if (!old_compat) {
                tk.i32(days);
                if (ti.use_cvm) tk.f32(click);
            }
            ld.add(sign, w.data(), g2sum, nullptr, nullptr, show, days, click, !old_compat);
        } else {
            float show = 0.f;
            for (int i = 0; i < D; i++) {
                tk.f32(w[i]);
                tk.f32(a[i]);
                tk.f32(b[i]);
            }
            tk.f32(show);
            ld.add(sign, w.data(), 0.f, a.data(), b.data(), show, 0, 0.f, false);
        }
        TN_TRY(ld.maybe_flush());
    }
    return TN_OK;
}

int load_table(uint32_t handle, const char* filepath, const char* mode) {
    if (!filepath || !mode) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: NULL argument");
    TableInfo ti;
    TN_TRY(table_info(handle, filepath, true, ti));
    // file pattern: sparse_block_0.gz | block_0.gz | block_0_bin.gz ...; a suffix names the mode,
    // no suffix means text (optimizer_kernel.h:496-520)
    std::string actual_mode = mode, prefix = "sparse_block_", suffix;
    std::vector<std::string> children;
    if (DIR* d = ::opendir(ti.dir.c_str())) {
        while (dirent* e = ::readdir(d))
            if (e->d_name[0] != '.') children.push_back(e->d_name);
        ::closedir(d);
    }
    if (children.empty()) return fail(TN_ERR_INVALID_ARGUMENT, "tn_sparse_table_load: no files in " + ti.dir);
    std::sort(children.begin(), children.end());
    std::smatch match;
    static const std::regex pattern(R"((.*?)(\d+)(.*)\.gz)");
    if (std::regex_match(children.front(), match, pattern)) {
        prefix = match[1];
        if (match[3].matched && match[3].length() > 0) {
            suffix = match[3];
            actual_mode = suffix.substr(1);
        } else {
            actual_mode = "txt";
        }
    }
    const bool bin = actual_mode == "bin";
    Loader ld(ti);
    TN_TRY(ld.init());
    for (int b = 0; b < kBlocks; b++) {
        std::string data;
        TN_TRY(read_gz(ti.dir + "/" + prefix + std::to_string(b) + suffix + ".gz", data));
        TN_TRY(bin ? parse_bin(ti, data, ld) : parse_txt(ti, data, ld));
    }
    return ld.flush();
}

// ------------------------------------------------------------------ dense table
// DenseTable::Save / Load (core/ps/table/dense_table.cc:103-157): one plain text file
//   <filepath>/dense_table/<handle>/<self_shard_id>     (the shard's own range of the table)
//   "total_elements:<n>\n" "rank_num:<shards>\n", then per block of ceil(range / 8) elements
//   (DenseOptimizerKernel, optimizer_kernel.h:174-188,224-235; block stream :139-160)
//   "opt_name:<Name>\n" "array_size:<len>\n" [Adam: "beta1_power:<f>\n" "beta2_power:<f>\n"]
//   one element per line, tab separated: Adam w m v (adam_kernel.cc:57-87), AdaGrad
//   w d2sum g2sum m (ada_grad_kernel.cc:50-76), then two empty lines.
constexpr int kDenseBlocks = 8;                 // DENSE_KERNEL_BLOCK_NUM
constexpr int64_t kDenseChunk = 1 << 20;        // elements formatted / parsed per round

std::string dense_file(uint32_t handle, const char* filepath, const DenseMeta& m) {
    return std::string(filepath) + "/dense_table/" + std::to_string(handle) + "/" + std::to_string(m.self_shard_id);
}

int save_dense(uint32_t handle, const char* filepath) {
    if (!filepath) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_save: NULL path");
    DenseMeta m;
    TN_TRY(dense_meta(handle, m));
    if (!m.initialized || m.length == 0) return TN_OK;  // no kernel for this shard: nothing is written (dense_table.cc:106-109)
    const std::string file = dense_file(handle, filepath, m);
    TN_TRY(make_dirs(file.substr(0, file.rfind('/'))));
    FILE* f = std::fopen(file.c_str(), "wb");
    if (!f) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_save: cannot write " + file);
    const int arrays = m.kind == OPT_ADAM ? 3 : 4;
    std::vector<float> host[4];
    for (int a = 0; a < arrays; a++) host[a].resize((size_t)std::min<int64_t>(kDenseChunk, m.length));
    float* arr[4] = {host[0].data(), host[1].data(), host[2].data(), arrays == 4 ? host[3].data() : nullptr};
    std::string out = "total_elements:" + std::to_string(m.total) + "\nrank_num:" + std::to_string(m.shard_num) + "\n";
    const int64_t per_block = (m.length + kDenseBlocks - 1) / kDenseBlocks;
    int rc = TN_OK;
    for (int64_t b0 = 0; b0 < m.length && rc == TN_OK; b0 += per_block) {
        const int64_t len = std::min(per_block, m.length - b0);
        out += std::string("opt_name:") + opt_name(m.kind) + "\narray_size:" + std::to_string(len) + "\n";
        if (m.kind == OPT_ADAM) {
            out += "beta1_power:";
            put_float(out, m.beta1_power);
            out += "\nbeta2_power:";
            put_float(out, m.beta2_power);
            out += '\n';
        }
        for (int64_t c0 = 0; c0 < len && rc == TN_OK; c0 += kDenseChunk) {
            const int64_t n = std::min(kDenseChunk, len - c0);
            rc = dense_copy_range(handle, b0 + c0, n, arr, true);
            for (int64_t i = 0; i < n && rc == TN_OK; i++) {
                for (int a = 0; a < arrays; a++) {
                    put_float(out, host[a][(size_t)i]);
                    out += a + 1 < arrays ? '\t' : '\n';
                }
            }
            if (std::fwrite(out.data(), 1, out.size(), f) != out.size())
                rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_save: write failed on " + file);
            out.clear();
        }
        out += "\n\n";
    }
    if (rc == TN_OK && std::fwrite(out.data(), 1, out.size(), f) != out.size())
        rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_save: write failed on " + file);
    if (std::fclose(f) != 0 && rc == TN_OK) rc = fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_save: close failed on " + file);
    return rc;
}

// "<anything>:<token>" as `is.ignore(max, ':') >> x` reads it
bool after_colon(Tokens& tk, std::string& token) {
    while (tk.p < tk.end && *tk.p != ':') tk.p++;
    if (tk.p >= tk.end) return false;
    tk.p++;
    const char *b, *e;
    if (!tk.next(b, e)) return false;
    token.assign(b, e);
    return true;
}

int load_dense(uint32_t handle, const char* filepath) {
    if (!filepath) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_load: NULL path");
    DenseMeta m;
    TN_TRY(dense_meta(handle, m));
    const std::string file = dense_file(handle, filepath, m);
    FILE* f = std::fopen(file.c_str(), "rb");
    if (!f) return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_load: cannot read " + file);
    std::string data;
    {
        std::vector<char> buf(1 << 22);
        size_t got;
        while ((got = std::fread(buf.data(), 1, buf.size(), f)) > 0) data.append(buf.data(), got);
        std::fclose(f);
    }
    const std::string bad = "tn_dense_table_load: malformed file " + file;
    Tokens tk{data.data(), data.data() + data.size()};
    std::string tok;
    if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
    const int64_t total = std::strtoll(tok.c_str(), nullptr, 10);
    if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
    const int rank_num = std::atoi(tok.c_str());
    if (rank_num != m.shard_num)  // CHECK_EQ(shard_num_, rank_num), dense_table.cc:140
        return fail(TN_ERR_INVALID_ARGUMENT, "tn_dense_table_load: file written by " + std::to_string(rank_num) +
                                                 " shards, table has " + std::to_string(m.shard_num));
    TN_TRY(dense_ensure_init(handle, total));  // CHECK_EQ(0, Init(total_elements_)), :142
    TN_TRY(dense_meta(handle, m));
    const int64_t length = m.length;  // this shard's range; without a kernel nothing more is read (:144-147)
    const int arrays = m.kind == OPT_ADAM ? 3 : 4;
    std::vector<float> host[4];
    for (int a = 0; a < arrays; a++) host[a].resize((size_t)std::min<int64_t>(kDenseChunk, std::max<int64_t>(length, 1)));
    float* arr[4] = {host[0].data(), host[1].data(), host[2].data(), arrays == 4 ? host[3].data() : nullptr};
    const int64_t per_block = (length + kDenseBlocks - 1) / kDenseBlocks;
    bool have_powers = false;
    float b1p = 1.f, b2p = 1.f;
    for (int64_t b0 = 0; b0 < length; b0 += per_block) {
        const int64_t len = std::min(per_block, length - b0);
        if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
        if (tok != opt_name(m.kind))  // optimizer_kernel.h:153-155
            return fail(TN_ERR_INVALID_ARGUMENT, "last trained model with optimizer is:" + tok +
                                                     " but current model use:" + opt_name(m.kind) + " instead");
        if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
        if (std::strtoll(tok.c_str(), nullptr, 10) != len)  // CHECK_EQ(array_size, w_.size())
            return fail(TN_ERR_DIM_MISMATCH, "tn_dense_table_load: block of " + tok + " elements, table expects " +
                                                 std::to_string(len));
        if (m.kind == OPT_ADAM) {
            float p1, p2;
            if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
            p1 = std::strtof(tok.c_str(), nullptr);
            if (!after_colon(tk, tok)) return fail(TN_ERR_INVALID_ARGUMENT, bad);
            p2 = std::strtof(tok.c_str(), nullptr);
            // every block steps on every push, so all blocks of one file hold the same powers
            if (have_powers && (p1 != b1p || p2 != b2p))
                return fail(TN_ERR_UNSUPPORTED, "tn_dense_table_load: blocks with different beta powers in " + file);
            b1p = p1;
            b2p = p2;
            have_powers = true;
        }
        for (int64_t c0 = 0; c0 < len; c0 += kDenseChunk) {
            const int64_t n = std::min(kDenseChunk, len - c0);
            for (int64_t i = 0; i < n; i++)
                for (int a = 0; a < arrays; a++)
                    if (!tk.f32(host[a][(size_t)i])) return fail(TN_ERR_INVALID_ARGUMENT, bad);
            TN_TRY(dense_copy_range(handle, b0 + c0, n, arr, false));
        }
    }
    if (have_powers) TN_TRY(dense_set_powers(handle, b1p, b2p));
    return TN_OK;
}

}  // namespace
}  // namespace tn

extern "C" {

int tn_dense_table_save(uint32_t handle, const char* filepath) { return tn::save_dense(handle, filepath); }

int tn_dense_table_load(uint32_t handle, const char* filepath) { return tn::load_dense(handle, filepath); }

int tn_sparse_table_save(uint32_t handle, const char* filepath, const char* mode) {
    return tn::save_table(handle, filepath, mode);
}

int tn_sparse_table_load(uint32_t handle, const char* filepath, const char* mode) {
    return tn::load_table(handle, filepath, mode);
}

}  // extern "C"
