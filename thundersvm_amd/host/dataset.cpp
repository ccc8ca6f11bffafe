#include "dataset.h"

#include "text_parse.h"

#include <fcntl.h>
#include <omp.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <memory>
#include <stdexcept>

DataSet::DataSet(const node2d &instances, int n_features, const std::vector<float_type> &y)
    : y_(y), instances_(instances), n_features_(n_features) {}

// ------------------------------------------------------------------------------------------------
// LibSVM text loader.  The reference reads 16 MB at a time and lets every OpenMP thread parse a run of whole lines
// of the buffer (src/thundersvm/dataset.cpp:20-100); here the whole file is mapped, cut into
// runs of whole lines, four per thread, parsed side by side and joined in file order.  Each token "i:v" gives what
// the reference's sscanf("%d:%f") gives: v is the correctly rounded float of the decimal text.
// Unlike the reference, a last line without a newline is kept (the reference's buffer walk stops at the last newline
// it has seen and loses that line) and blank lines are skipped (the reference turns one into an instance without
// features and with label 0).
// ------------------------------------------------------------------------------------------------
namespace {

using tsvm::is_blank;
using tsvm::parse_double;
using tsvm::parse_float;

struct LoadedRun {
    std::vector<float_type> y;
    DataSet::node2d rows;
    size_t max_index = 0;
    bool zero_based = false;
    bool bad = false;
};

void parse_run(const char *p, const char *end, LoadedRun &out) {
    std::vector<DataSet::node> row;   // assembled here, copied out at its final size: one allocation per instance
    while (p < end) {
        const char *eol = (const char *) memchr(p, '\n', end - p);
        if (!eol) eol = end;
        while (p < eol && is_blank(*p)) ++p;
        if (p < eol) {
            const char *q;
            out.y.push_back(parse_double(p, eol, &q));
            if (q == p) { out.bad = true; return; }
            p = q;
            row.clear();
            while (p < eol) {
                while (p < eol && is_blank(*p)) ++p;
                if (p >= eol) break;
                long idx = 0;
                bool neg = false;
                const char *s = p;
                if (*s == '-' || *s == '+') neg = *s++ == '-';
                const char *digits = s;
                for (; s < eol && *s >= '0' && *s <= '9'; ++s) idx = idx * 10 + (*s - '0');
                if (s == digits || s >= eol || *s != ':') { out.bad = true; return; }
                if (neg) idx = -idx;
                p = s + 1;
                if (p >= eol || is_blank(*p)) { out.bad = true; return; }   // "index:" without a value
                const float v = parse_float(p, eol, &q);
                if (q == p) { out.bad = true; return; }
                p = q;
                row.emplace_back((int) idx, (kernel_type) v);
                if (idx == 0) out.zero_based = true;
                if (idx > 0 && (size_t) idx > out.max_index) out.max_index = (size_t) idx;
            }
            out.rows.emplace_back(row.begin(), row.end());
        }
        p = eol + 1;
    }
}

}  // namespace

void DataSet::load_from_file(std::string file_name, int n_threads) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.clear();
    n_features_ = 0;
    zero_based_ = false;
    const int fd = open(file_name.c_str(), O_RDONLY);
    if (fd < 0) throw std::runtime_error("file " + file_name + " not found");
    struct stat st;
    if (fstat(fd, &st) != 0) { close(fd); throw std::runtime_error("file " + file_name + " cannot be read"); }
    const size_t size = (size_t) st.st_size;
    if (n_threads <= 0) n_threads = omp_get_max_threads();
    // The file's pages are parsed where the page cache holds them (a private read-only mapping: no copy, every thread
    // faults in the part it parses).  The library calls behind parse_float / parse_double need text that ends in a
    // character no number contains: inside the mapping that is the line's newline, so the mapping is parsed up to
    // the last newline, and a last line without one is parsed from a NUL-terminated copy.
    struct Mapping {
        void *p = MAP_FAILED;
        size_t n = 0;
        ~Mapping() { if (p != MAP_FAILED) munmap(p, n); }
    } map;
    std::unique_ptr<char[]> copy;
    const char *text = nullptr;
    if (size > 0) {
        map.p = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
        map.n = size;
    }
    if (map.p != MAP_FAILED) {
        text = (const char *) map.p;
    } else if (size > 0) {   // a file that cannot be mapped (a pipe, a special file system): read it, every thread its share
        copy.reset(new char[size + 1]);
        copy[size] = 0;
        bool read_ok = true;
        const size_t piece = (size + n_threads - 1) / std::max(n_threads, 1);
#pragma omp parallel for num_threads(n_threads) schedule(static, 1)
        for (int t = 0; t < n_threads; ++t) {
            size_t off = std::min(size, (size_t) t * piece);
            const size_t stop = std::min(size, off + piece);
            while (off < stop) {
                const ssize_t got = pread(fd, copy.get() + off, stop - off, (off_t) off);
                if (got <= 0) {
#pragma omp atomic write
                    read_ok = false;
                    break;
                }
                off += (size_t) got;
            }
        }
        if (!read_ok) { close(fd); throw std::runtime_error("file " + file_name + " cannot be read"); }
        text = copy.get();
    }
    close(fd);
    size_t body = size;   // the part that ends in a newline
    if (map.p != MAP_FAILED) {
        const void *last_nl = memrchr(text, '\n', size);
        body = last_nl ? (size_t) ((const char *) last_nl - text) + 1 : 0;
    }
    const std::string tail = body < size ? std::string(text + body, size - body) : std::string();
    // runs of whole lines: run r starts behind the first newline at or after byte r * body / n_runs
    const int n_body_runs = n_threads == 1 ? 1 : n_threads * 4;
    const int n_runs = n_body_runs + 1;                     // the last run is the line without a newline, if any
    std::vector<size_t> cut(n_body_runs + 1, body);
    cut[0] = 0;
    for (int r = 1; r < n_body_runs; ++r) {
        const size_t from = std::max(cut[r - 1], body / n_body_runs * r);
        const char *nl = from < body ? (const char *) memchr(text + from, '\n', body - from) : nullptr;
        cut[r] = nl ? (size_t) (nl - text) + 1 : body;
    }
    std::vector<LoadedRun> runs(n_runs);
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (int r = 0; r < n_runs; ++r) {
        if (r < n_body_runs) parse_run(text + cut[r], text + cut[r + 1], runs[r]);
        else parse_run(tail.c_str(), tail.c_str() + tail.size(), runs[r]);
    }
    std::vector<size_t> first(n_runs + 1, 0);
    for (int r = 0; r < n_runs; ++r) {
        if (runs[r].bad) throw std::runtime_error("read error, using [index]:[value] format");
        first[r + 1] = first[r] + runs[r].rows.size();
        if (runs[r].max_index > n_features_) n_features_ = runs[r].max_index;
        zero_based_ = zero_based_ || runs[r].zero_based;
    }
    y_.resize(first[n_runs]);
    instances_.resize(first[n_runs]);
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (int r = 0; r < n_runs; ++r) {
        LoadedRun &run = runs[r];
        std::copy(run.y.begin(), run.y.end(), y_.begin() + first[r]);
        std::move(run.rows.begin(), run.rows.end(), instances_.begin() + first[r]);
        run = LoadedRun();      // the run's own arrays are released by the thread that moved it
    }
    TSVM_LOG << "#instances = " << n_instances() << ", #features = " << n_features();
}

void DataSet::load_from_python(float *y, char **x, int len) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.clear();
    n_features_ = 0;
    for (int i = 0; i < len; ++i) {
        y_.push_back(y[i]);
        instances_.emplace_back();
        std::stringstream ss(x[i]);
        std::string tuple;
        while (ss >> tuple) {
            int ind;
            float v;
            if (sscanf(tuple.c_str(), "%d:%f", &ind, &v) != 2) throw std::runtime_error("read error, using [index]:[value] format");
            instances_.back().emplace_back(ind, v);
            if ((size_t) ind > n_features_) n_features_ = ind;
        }
    }
}

void DataSet::load_from_sparse(int row_size, float *val, int *row_ptr, int *col_ptr, float *label) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.assign(row_size, {});
    n_features_ = 0;
    for (int r = 0; r < row_size; ++r) {
        if (label) y_.push_back(label[r]);
        for (int e = row_ptr[r]; e < row_ptr[r + 1]; ++e) {
            int ind = col_ptr[e] + 1;  // to one-based
            instances_[r].emplace_back(ind, val[e]);
            if ((size_t) ind > n_features_) n_features_ = ind;
        }
    }
}

void DataSet::load_from_dense(int row_size, int features, float *data, float *label) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.assign(row_size, {});
    for (int r = 0; r < row_size; ++r) {
        if (label) y_.push_back(label[r]);
        instances_[r].reserve(features);
        for (int j = 1; j <= features; ++j) instances_[r].emplace_back(j, data[(size_t) r * features + j - 1]);
    }
    n_features_ = features;
}

void DataSet::load_from_csr(int64_t n, const int64_t *row_ptr, const int *col, const double *val, const double *y) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.assign(n, {});
    n_features_ = 0;
    zero_based_ = false;
    for (int64_t r = 0; r < n; ++r) {
        if (y) y_.push_back(y[r]);
        instances_[r].reserve(row_ptr[r + 1] - row_ptr[r]);
        for (int64_t e = row_ptr[r]; e < row_ptr[r + 1]; ++e) {
            instances_[r].emplace_back(col[e], val[e]);
            if (col[e] == 0) zero_based_ = true;
            if ((size_t) col[e] > n_features_) n_features_ = col[e];
        }
    }
}

// Classes are numbered in order of first appearance; perm_ lists the instance ids class by class
// (src/thundersvm/dataset.cpp:190-234).
void DataSet::group_classes(bool classification) {
    start_.clear();
    count_.clear();
    label_.clear();
    perm_.clear();
    const size_t n = instances().size();
    if (!classification) {
        perm_.resize(n);
        for (size_t i = 0; i < n; ++i) perm_[i] = (int) i;
        start_.push_back(0);
        count_.push_back((int) n);
        return;
    }
    std::vector<int> cls(n);
    for (size_t i = 0; i < n; ++i) {
        size_t c = 0;
        while (c < label_.size() && y_[i] != label_[c]) ++c;
        if (c == label_.size()) {
            label_.push_back(int(y_[i]));
            count_.push_back(0);
        }
        count_[c]++;
        cls[i] = (int) c;
    }
    start_.assign(label_.size(), 0);
    for (size_t c = 1; c < label_.size(); ++c) start_[c] = start_[c - 1] + count_[c - 1];
    std::vector<int> cursor(start_);
    perm_.resize(n);
    for (size_t i = 0; i < n; ++i) perm_[cursor[cls[i]]++] = (int) i;
}

DataSet DataSet::grouped_view() const {
    DataSet v;
    v.y_ = y_;
    v.n_features_ = n_features_;
    v.zero_based_ = zero_based_;
    v.base_ = base_ ? base_ : &instances_;
    v.device_slot_ = device_slot_;   // same instances, same device copy
    v.group_classes(true);
    return v;
}

const DataSet::node2d DataSet::instances(int y_i) const {
    node2d out;
    out.reserve(count_[y_i]);
    for (int i = start_[y_i]; i < start_[y_i] + count_[y_i]; ++i) out.push_back(instances()[perm_[i]]);
    return out;
}

const DataSet::node2d DataSet::instances(int y_i, int y_j) const {
    node2d out = instances(y_i);
    node2d other = instances(y_j);
    out.insert(out.end(), other.begin(), other.end());
    return out;
}

const std::vector<int> DataSet::original_index(int y_i) const {
    return std::vector<int>(perm_.begin() + start_[y_i], perm_.begin() + start_[y_i] + count_[y_i]);
}

const std::vector<int> DataSet::original_index(int y_i, int y_j) const {
    std::vector<int> out = original_index(y_i);
    std::vector<int> other = original_index(y_j);
    out.insert(out.end(), other.begin(), other.end());
    return out;
}
