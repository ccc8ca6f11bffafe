// SvmModel::predict_dec_values (src/thundersvm/model/svmmodel.cpp:74-117): decision values of a set of rows against
// the model's support vectors.  With dense support vectors the kernel values are reduced where they are computed
// (tsvm_predict_dec_values_dense) and never written out; otherwise kernel rows per batch, then
// tsvm_sum_kernel_values, as the reference does.
#include <algorithm>
#include <cstdlib>

#include "models.h"

using tsvm::abi_check;
using tsvm::DeviceBuffer;

struct SvmModel::PredictPlan {
    // for both paths
    DeviceBuffer<float_type> rho;
    // unfused path: the reference's arrays as they are
    DeviceBuffer<int> sv_start, sv_count;
    DeviceBuffer<float_type> coef;
    // fused path: every class's support vectors start on a multiple of 128 columns
    int stride = 0;                 // coefficients stored per padded column (0: the fused kernels do not take this model)
    int64_t n_pad = 0;
    std::vector<int> class_tile;    // [n_classes + 1]: first 128-column tile of every class
    DeviceBuffer<int> col_map;      // padded column -> support vector
    DeviceBuffer<float_type> coef_t;   // [n_pad][stride]
    bool many_features = false;     // the 128 x 128 tile kernel (d > 128, no indicator columns)
    // chunk table of the last call, rebuilt when the batch size changes
    mutable size_t chunks_for_m = 0;
    mutable int n_chunks = 0;
    mutable DeviceBuffer<int> chunks, class_chunk_start;
    // the batch rows' indicator masks (grown as needed, kept between calls)
    mutable DeviceBuffer<uint64_t> mask_a;
    mutable DeviceBuffer<int> mask_max;
};

const SvmModel::PredictPlan &SvmModel::predict_plan() const {
    if (predict_plan_) return *predict_plan_;
    // the support vectors' device copy is built by the first predict call and kept for the next ones (the
    // reference rebuilds it per call, svmmodel.cpp:84)
    if (!sv_k_mat) sv_k_mat.reset(new KernelMatrix(sv, param));
    auto plan = std::make_shared<PredictPlan>();
    PredictPlan &P = *plan;
    const DeviceRows &R = sv_k_mat->rows();
    const size_t T = sv.size();
    std::vector<int> sv_start(n_classes, 0);
    for (int c = 1; c < n_classes; ++c) sv_start[c] = sv_start[c - 1] + n_sv[c - 1];
    P.rho.upload(rho);
    P.sv_start.upload(sv_start);
    P.sv_count.upload(n_sv);
    P.coef.upload(coef);
    const bool masks = R.dense && R.ind_first >= 0;
    const int d = masks ? R.ind_first : (int) R.n_features;
    P.stride = R.dense ? tsvm_predict_nc_stride(n_classes, d, masks) : 0;
    if (P.stride > 0) {
        P.many_features = d > 128 && !masks;
        P.class_tile.assign(n_classes + 1, 0);
        for (int c = 0; c < n_classes; ++c) P.class_tile[c + 1] = P.class_tile[c] + (n_sv[c] + 127) / 128;
        P.n_pad = (int64_t) P.class_tile[n_classes] * 128;
        std::vector<int> col_map((size_t) P.n_pad, 0);
        std::vector<float_type> coef_t((size_t) P.n_pad * P.stride, 0.0);
        const int km1 = n_classes - 1;
        for (int c = 0; c < n_classes; ++c) {
            const int64_t p0 = (int64_t) P.class_tile[c] * 128, p1 = (int64_t) P.class_tile[c + 1] * 128;
            for (int64_t p = p0; p < p1; ++p) {
                const int t = (int) (p - p0);
                if (t < n_sv[c]) {
                    const int l = sv_start[c] + t;
                    col_map[p] = l;
                    for (int r = 0; r < km1; ++r) coef_t[(size_t) p * P.stride + r] = coef[(size_t) r * T + l];
                } else {
                    col_map[p] = sv_start[c];   // a valid row; its coefficients stay zero
                }
            }
        }
        P.col_map.upload(col_map);
        P.coef_t.upload(coef_t);
    }
    predict_plan_ = plan;
    return *predict_plan_;
}

// Chunks: runs of column tiles inside one class, short enough that the workgroups walking the same chunk side by
// side keep its support vectors in their XCD's L2, and numerous enough to fill the chip when the batch is small.
static void build_chunks(const std::vector<int> &class_tile, size_t row_blocks, int max_tiles, std::vector<int> &chunks,
                         std::vector<int> &class_chunk_start) {
    const int n_classes = (int) class_tile.size() - 1;
    const int64_t total = class_tile[n_classes];
    const int64_t per = std::max<int64_t>(1, std::min<int64_t>(max_tiles, total * (int64_t) row_blocks / 2048));
    chunks.clear();
    class_chunk_start.assign(n_classes + 1, 0);
    for (int c = 0; c < n_classes; ++c) {
        const int t0 = class_tile[c], nt = class_tile[c + 1] - t0;
        const int pieces = (int) ((nt + per - 1) / per);
        for (int q = 0; q < pieces; ++q) {   // as even as possible
            chunks.push_back(t0 + (int) ((int64_t) nt * q / pieces));
            chunks.push_back(t0 + (int) ((int64_t) nt * (q + 1) / pieces));
        }
        class_chunk_start[c + 1] = class_chunk_start[c] + pieces;
    }
}

bool SvmModel::predict_batch_fused(const PredictPlan &P, const kernel_type *a, int64_t lda, const kernel_type *sd_a, size_t m,
                                   bool indicator_values, float_type *dec_out) const {
    const DeviceRows &R = sv_k_mat->rows();
    // (TSVM_PREDICT_UNFUSED: the two-call form for every batch, to compare the two)
    if (P.stride == 0 || getenv("TSVM_PREDICT_UNFUSED")) return false;
    const bool plan_masks = R.ind_first >= 0;
    if (plan_masks && !indicator_values) return false;   // (the coefficient layout was made for the kernel with masks)
    const int d = plan_masks ? R.ind_first : (int) R.n_features;
    if (lda < (int64_t) ((R.n_features + 7) / 8 * 8)) return false;
    if (P.chunks_for_m != m) {
        std::vector<int> chunks, ccs;
        build_chunks(P.class_tile, P.many_features ? (m + 127) / 128 : (m + 63) / 64, P.many_features ? 8 : 32, chunks, ccs);
        P.n_chunks = (int) chunks.size() / 2;
        P.chunks.upload(chunks);
        P.class_chunk_start.upload(ccs);
        P.chunks_for_m = m;
    }
    if (plan_masks) {
        if (P.mask_a.size() < m) P.mask_a.resize(m);
        if (P.mask_max.size() < 1) P.mask_max.resize(1);
        abi_check(tsvm_indicator_masks(a, lda, (int64_t) m, R.ind_first, (int) R.n_features - R.ind_first, P.mask_a.data(),
                                       P.mask_max.data(), nullptr));
    }
    const int km1 = n_classes - 1;
    // partial sums and decision values: from the persistent row arena (no allocation per call)
    const size_t part_doubles = (size_t) std::max(P.n_chunks, 1) * m * km1, dec_doubles = m * (size_t) n_binary_models;
    float_type *d_part = (float_type *) tsvm::RowArena::instance().acquire((part_doubles + dec_doubles) * sizeof(float_type), false);
    float_type *d_dec = d_part + part_doubles;
    // (a batch row may set more indicator columns than any support vector does: its matches are bounded by the
    // support vectors' count all the same)
    abi_check(tsvm_predict_dec_values_dense(R.x.data(), R.ld, d, R.self_dot.data(), plan_masks ? R.ind_mask.data() : nullptr,
                                            P.col_map.data(), P.n_pad, P.coef_t.data(), P.chunks.data(), P.n_chunks,
                                            P.class_chunk_start.data(), P.rho.data(), n_classes, a, lda, (int64_t) m, sd_a,
                                            plan_masks ? P.mask_a.data() : nullptr, R.ind_max_ones, (int) param.kernel_type,
                                            param.gamma, param.coef0, param.degree, d_part, d_dec, nullptr));
    TSVM_HIP_CHECK(hipMemcpy(dec_out, d_dec, dec_doubles * sizeof(float_type), hipMemcpyDeviceToHost));
    return true;
}

void SvmModel::predict_dec_values(const DataSet::node2d &instances, std::vector<float_type> &dec, int batch_size) const {
    dec.assign(instances.size() * (size_t) n_binary_models, 0);
    if (instances.empty()) return;
    const size_t T = sv.size();
    if (T == 0) {
        for (size_t r = 0; r < instances.size(); ++r)
            for (int p = 0; p < n_binary_models; ++p) dec[r * n_binary_models + p] = -rho[p];
        return;
    }
    const PredictPlan &P = predict_plan();
    const KernelMatrix &k_mat = *sv_k_mat;
    const bool fused = P.stride > 0 && !getenv("TSVM_PREDICT_UNFUSED");
    if (batch_size == -1) {
        if (fused) {
            // no batch x support-vector matrix exists: a batch only needs its own rows on the device
            batch_size = 65536;
        } else {
            const size_t used = tsvm::device_bytes_in_use();
            const size_t free_mem = param.max_mem_size > used ? param.max_mem_size - used : 0;
            batch_size = (int) std::min(free_mem / sizeof(float_type) / (T + k_mat.n_features()), size_t(10000));
        }
        if (batch_size < 1) batch_size = 1;
    }
    const size_t bmax = std::min((size_t) batch_size, instances.size());
    void *d_k = nullptr;
    const int64_t ldk = ((int64_t) T + 15) / 16 * 16;   // (rows padded to 16 elements: get_rows writes whole aligned vectors)
    DeviceBuffer<float_type> d_dec;
    for (size_t b0 = 0; b0 < instances.size(); b0 += batch_size) {
        const size_t bm = std::min((size_t) batch_size, instances.size() - b0);
        if (fused) {
            const KernelMatrix::StagedBatch b = k_mat.stage_batch(instances.data() + b0, bm);
            if (predict_batch_fused(P, b.a, b.lda, b.sd, bm, b.indicator_values, dec.data() + b0 * n_binary_models)) continue;
        }
        // kernel values of one batch (taken from the persistent row arena), then the reduction
        if (!d_k) {
            d_k = tsvm::RowArena::instance().acquire(bmax * (size_t) ldk * k_mat.row_elem_size(), false);
            d_dec.resize(bmax * n_binary_models);
        }
        k_mat.get_rows(instances.data() + b0, bm, d_k, ldk);
        abi_check(tsvm_sum_kernel_values(P.coef.data(), (int) T, P.sv_start.data(), P.sv_count.data(), P.rho.data(), d_k,
                                         k_mat.row_type(), ldk, d_dec.data(), n_classes, (int64_t) bm, nullptr));
        d_dec.download(dec.data() + b0 * n_binary_models, bm * n_binary_models);
    }
}

void SvmModel::predict_dec_values(const DataSet &dataset, std::vector<float_type> &dec, int batch_size) const {
    const std::shared_ptr<void> &slot = dataset.device_cache();
    if (slot && !sv.empty() && dataset.n_instances() > 0) {
        const DeviceRows &A = *std::static_pointer_cast<DeviceRows>(slot);
        const PredictPlan &P = predict_plan();
        const DeviceRows &R = sv_k_mat->rows();
        if (A.dense && P.stride > 0 && A.n == dataset.n_instances()) {
            // do the batch's values in the support vectors' indicator columns qualify?  (counted once per DataSet)
            bool indicator_values = false;
            if (R.ind_first >= 0) {
                const std::vector<int> &st = A.column_stats();
                indicator_values = true;
                for (size_t c = (size_t) R.ind_first; c < std::min(R.n_features, A.n_features); ++c)
                    if (st[A.n_features + c] != 0) indicator_values = false;
            }
            dec.assign(dataset.n_instances() * (size_t) n_binary_models, 0);
            const size_t step = batch_size > 0 ? (size_t) batch_size : A.n;
            bool ok = true;
            for (size_t b0 = 0; b0 < A.n && ok; b0 += step) {
                const size_t bm = std::min(step, A.n - b0);
                ok = predict_batch_fused(P, A.x.data() + b0 * (size_t) A.ld, A.ld, A.self_dot.data() + b0, bm, indicator_values,
                                         dec.data() + b0 * n_binary_models);
            }
            if (ok) return;
        }
    }
    predict_dec_values(dataset.instances(), dec, batch_size);
}

std::vector<float_type> SvmModel::predict(const DataSet::node2d &instances, int batch_size) {   // svmmodel.cpp:157-171
    predict_dec_values(instances, dec_values, batch_size);
    return finish_predict((int) instances.size());
}

std::vector<float_type> SvmModel::predict(const DataSet &dataset, int batch_size) {
    predict_dec_values(dataset, dec_values, batch_size);
    return finish_predict((int) dataset.n_instances());
}
