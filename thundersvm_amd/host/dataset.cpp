#include "dataset.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <stdexcept>

DataSet::DataSet(const node2d &instances, int n_features, const std::vector<float_type> &y)
    : y_(y), instances_(instances), n_features_(n_features) {}

// One pass over the file text.  Each token "i:v" is parsed the way the reference's sscanf("%d:%f")
// does: v goes through float (src/thundersvm/dataset.cpp:72-80).  Row order is file order.
void DataSet::load_from_file(std::string file_name) {
    device_slot_ = std::make_shared<std::shared_ptr<void>>();   // new instances: any device copy is stale
    y_.clear();
    instances_.clear();
    n_features_ = 0;
    zero_based_ = false;
    std::ifstream in(file_name, std::ios::binary);
    if (!in.is_open()) throw std::runtime_error("file " + file_name + " not found");
    std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    const char *p = text.c_str();
    const char *end = p + text.size();
    while (p < end) {
        const char *eol = (const char *) memchr(p, '\n', end - p);
        if (!eol) eol = end;
        while (p < eol && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
        if (p < eol) {
            char *q;
            y_.push_back(strtod(p, &q));
            instances_.emplace_back();
            auto &row = instances_.back();
            p = q;
            while (p < eol) {
                while (p < eol && (*p == ' ' || *p == '\t' || *p == '\r')) ++p;
                if (p >= eol) break;
                long idx = strtol(p, &q, 10);
                if (q == p || *q != ':') throw std::runtime_error("read error, using [index]:[value] format");
                p = q + 1;
                float v = strtof(p, &q);
                if (q == p) throw std::runtime_error("read error, using [index]:[value] format");
                p = q;
                row.emplace_back((int) idx, (kernel_type) v);
                if (idx == 0) zero_based_ = true;
                if ((size_t) idx > n_features_) n_features_ = idx;
            }
        }
        p = eol + 1;
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
