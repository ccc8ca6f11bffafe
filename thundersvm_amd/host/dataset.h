// DataSet: LibSVM-format instances, labels and the class grouping used by one-vs-one training.
// Same public surface as include/thundersvm/dataset.h; values are float32-rounded on load
// (src/thundersvm/dataset.cpp:76-79) and held as kernel_type.
#pragma once
#include <memory>

#include "thundersvm.h"

class DataSet {
public:
    struct node {
        node(int index, kernel_type value) : index(index), value(value) {}
        int index;
        kernel_type value;
    };
    typedef std::vector<std::vector<node>> node2d;

    DataSet() = default;
    DataSet(const node2d &instances, int n_features, const std::vector<float_type> &y);

    // n_threads: threads that read and parse (0: as many as OpenMP would start, which the `-o` option sets, as in
    // the reference)
    void load_from_file(std::string file_name, int n_threads = 0);
    void load_from_python(float *y, char **x, int len);
    void load_from_sparse(int row_size, float *val, int *row_ptr, int *col_ptr, float *label);
    void load_from_dense(int row_size, int features, float *data, float *label);
    // CSR with the caller's (1-based) feature ids and double values (already float32-exact)
    void load_from_csr(int64_t n, const int64_t *row_ptr, const int *col, const double *val, const double *y);

    void group_classes(bool classification = true);
    // A grouped DataSet that refers to this one's instances instead of copying them.
    DataSet grouped_view() const;
    size_t n_instances() const { return instances().size(); }
    size_t n_features() const { return n_features_; }
    size_t n_classes() const { return start_.size(); }
    const std::vector<int> &count() const { return count_; }
    const std::vector<int> &start() const { return start_; }
    const std::vector<int> &label() const { return label_; }
    const std::vector<float_type> &y() const { return y_; }
    const node2d &instances() const { return base_ ? *base_ : instances_; }
    const node2d instances(int y_i) const;
    const node2d instances(int y_i, int y_j) const;
    const std::vector<int> original_index() const { return perm_; }
    const std::vector<int> original_index(int y_i) const;
    const std::vector<int> original_index(int y_i, int y_j) const;
    bool is_zero_based() const { return zero_based_; }
    // Slot for a device-resident copy of instances(), filled by the first KernelMatrix built from this
    // DataSet (or by whoever wants the upload to happen early) and shared with its grouped views.  It is
    // dropped when the instances are reloaded.
    std::shared_ptr<void> &device_cache() const { return *device_slot_; }

private:
    std::vector<float_type> y_;
    node2d instances_;
    const node2d *base_ = nullptr;   // set by grouped_view(): instances live in another DataSet
    size_t n_features_ = 0;
    std::vector<int> start_, count_, label_, perm_;
    bool zero_based_ = false;
    mutable std::shared_ptr<std::shared_ptr<void>> device_slot_ = std::make_shared<std::shared_ptr<void>>();
};
