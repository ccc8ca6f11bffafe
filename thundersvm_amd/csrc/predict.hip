// SvmModel::predict_dec_values as one pass: kernel values of a batch against the support vectors, multiplied by the
// coefficients and summed per class while they are still in registers.  The batch x support-vector matrix of kernel
// values, which the reference writes out and reads back (src/thundersvm/model/svmmodel.cpp:74-117: get_rows, then
// sum_kernel_values, src/thundersvm/kernel/kernelmatrix_kernel.cpp:110-147), never reaches memory.
//
// Layout the host prepares once per model.  The support vectors of class s are columns
// [first tile of s * 128, ...) of a padded column range in which every class starts on a multiple of 128, so that a
// 128-column tile never holds two classes; col_map[p] is the support vector (row of x) behind padded column p, and
// padding columns point at a valid row and have all-zero coefficients.  coef_t[p * nc + c] is coefficient row c
// (0 .. k-2, the layout of svmmodel.h:154-164) of padded column p.  A chunk is a run of column tiles inside one
// class; a workgroup owns one chunk and one block of batch rows and leaves partial[(chunk * m + row) * nc + c], the
// sum over the chunk's columns of coef * K.  A second, small kernel adds the chunks of the two classes of every
// pair in chunk order and subtracts rho.  Every sum has a fixed order: results do not depend on scheduling.
#include "../../include/thundersvm_amd.h"
#include "tsvm_device.h"
#include "tsvm_internal.h"

#include <algorithm>

#include "get_rows_tile.h"

typedef double v2d __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------------------------
// Few features (d <= 128, or indicator columns left to the epilogue): the tile walk of the few-feature get_rows
// kernel (64 batch rows x 128 columns, the next tile's first loads requested ahead of the epilogue), with NC
// running sums per batch row and lane in registers for the whole chunk.
// ------------------------------------------------------------------------------------------------
template <int KT, int NC, int IND, int K_TILES>   // K_TILES: 1 = a single K tile (d <= 16), 2 = any number
__global__ __launch_bounds__(256, 2) void predict_dense_stream_kernel(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ col_map, int d, const double *__restrict__ sd_x,
    const uint64_t *__restrict__ mask_x, const double *__restrict__ a, int64_t lda, int m, const double *__restrict__ sd_a,
    const uint64_t *__restrict__ mask_a, int max_ones, KernelParam kp_in, const double *__restrict__ coef_t,
    const int *__restrict__ chunks, unsigned m_blocks, double *__restrict__ partial, int nc_out) {
    constexpr int TI = 2;
    constexpr int BM = GrShape<TI>::BM;
    constexpr int KTILE = GrShape<TI>::KTILE;
    constexpr int LS = GrShape<TI>::LS;
    constexpr int A_TPR = 256 / BM;
    constexpr int A_VEC = KTILE / 4 / A_TPR;
    constexpr int B_VEC = KTILE / 8;
    __shared__ double As[GrShape<TI>::LDS_DOUBLES];
    __shared__ double Bs[GrShape<TI>::LDS_DOUBLES];
    __shared__ uint64_t exp_tab[32];
    __shared__ double s_sdi[BM];
    __shared__ uint64_t s_mi[BM];
    // per column of the current tile, two generations (a wavefront may stage the next tile's while another still
    // reads this tile's)
    __shared__ double s_sdj[2][GR_BN];
    __shared__ uint64_t s_mj[2][GR_BN];
    __shared__ __attribute__((aligned(16))) double s_coef[2][NC][GR_BN];
    KernelParam kp = kp_in;
    kp.kernel_type = KT;
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int i0 = (int) (logical % m_blocks) * BM;
    const unsigned chunk = logical / m_blocks;
    const unsigned jt0 = (unsigned) chunks[2 * chunk], jt1 = (unsigned) chunks[2 * chunk + 1];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int m_last = m - 1;
    const int a_row = tid / A_TPR, a_k = (tid % A_TPR) * (4 * A_VEC);
    const int b_row = tid >> 1, b_k = (tid & 1) * (4 * B_VEC);
    const int lrow = lane & 15;
    const int lk = lane >> 4;
    // slot (tj, l) of a wavefront's 64 columns holds column 4*l + tj: a lane's four accumulator tiles are four
    // consecutive columns, whose coefficients come out of LDS as two 16-byte reads per coefficient row
    const int b_col = (b_row & 64) + ((b_row & 15) << 2) + ((b_row >> 4) & 3);

    if (tid < 32) exp_tab[tid] = TSVM_EXP2F_TAB[tid];
    if (tid < BM) {
        const int r = min(i0 + tid, m_last);
        s_sdi[tid] = sd_a ? sd_a[r] : 0.0;
        s_mi[tid] = IND ? mask_a[r] : 0;
    }
    const double *a_ptr = a + (uint64_t) (uint32_t) min(i0 + a_row, m_last) * (uint32_t) lda;

    const int n_kt = K_TILES == 1 ? (d > 0 ? 1 : 0) : (d + KTILE - 1) / KTILE;
    const int n_ks_last = (d - (n_kt - 1) * KTILE + 3) / 4;
    v4d ra[A_VEC], rb[B_VEC];
    double pre_sd = 0.0;
    uint64_t pre_m = 0;
    double pre_c[(NC + 1) / 2];
    const double *x_ptr = x;
    const int c_first = tid >> 7;   // this thread brings coefficient rows c_first, c_first + 2, ... of column tid & 127
    auto request_tile = [&](unsigned jt) {
        x_ptr = x + (uint64_t) (uint32_t) col_map[(int) jt * GR_BN + b_col] * (uint32_t) ldx;
        const int p = (int) jt * GR_BN + (tid & 127);
        if (tid < GR_BN) {
            const int jc = col_map[p];
            pre_sd = sd_x ? sd_x[jc] : 0.0;
            pre_m = IND ? mask_x[jc] : 0;
        }
#pragma unroll
        for (int q = 0; q < (NC + 1) / 2; ++q) {
            const int c = c_first + 2 * q;
            pre_c[q] = c < NC ? coef_t[(int64_t) p * NC + c] : 0.0;
        }
    };
    auto load_tile = [&](int kt, bool last) {
        const int k0 = kt * KTILE;
        if (!last) {
#pragma unroll
            for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (a_ptr + (k0 + a_k + 4 * q));
#pragma unroll
            for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (x_ptr + (k0 + b_k + 4 * q));
        } else {
#pragma unroll
            for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (a_ptr + min(k0 + a_k + 4 * q, (int) lda - 4));
#pragma unroll
            for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (x_ptr + min(k0 + b_k + 4 * q, (int) ldx - 4));
        }
    };
    // (IND: the columns from d on are live data, not padding: the batch rows' values there are staged as zeros)
    const int k_live = d - (n_kt - 1) * KTILE;
    auto stage_tile = [&](bool last) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int q = 0; q < A_VEC; ++q)
                As[(a_k + 4 * q + e) * LS + a_row] = (IND && last && a_k + 4 * q + e >= k_live) ? 0.0 : ra[q][e];
#pragma unroll
            for (int q = 0; q < B_VEC; ++q) Bs[(b_k + 4 * q + e) * LS + b_row] = rb[q][e];
        }
    };
    double part[TI * 4][NC];
#pragma unroll
    for (int u = 0; u < TI * 4; ++u)
#pragma unroll
        for (int c = 0; c < NC; ++c) part[u][c] = 0.0;

    request_tile(jt0);
    if (n_kt > 0) load_tile(0, n_kt == 1);
    for (unsigned jt = jt0; jt < jt1; ++jt) {
        const int gen = (int) (jt & 1u);
        if (tid < GR_BN) {
            s_sdj[gen][tid] = pre_sd;
            s_mj[gen][tid] = pre_m;
        }
#pragma unroll
        for (int q = 0; q < (NC + 1) / 2; ++q)
            if (c_first + 2 * q < NC) s_coef[gen][c_first + 2 * q][tid & 127] = pre_c[q];
        v4d acc[TI][4];
#pragma unroll
        for (int ti = 0; ti < TI; ++ti)
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) acc[ti][tj] = (v4d){0.0, 0.0, 0.0, 0.0};
        auto mma_step = [&](int ks) {
            double af[TI], bf[4];
            const int kk = (ks * 4 + lk) * LS;
#pragma unroll
            for (int t = 0; t < TI; ++t) af[t] = As[kk + wi * (16 * TI) + t * 16 + lrow];
#pragma unroll
            for (int t = 0; t < 4; ++t) bf[t] = Bs[kk + wj * 64 + t * 16 + lrow];
#pragma unroll
            for (int ti = 0; ti < TI; ++ti)
#pragma unroll
                for (int tj = 0; tj < 4; ++tj)
                    acc[ti][tj] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[ti], bf[tj], acc[ti][tj], 0, 0, 0);
        };
        if (n_kt > 0) {
            const double *pa = a_ptr + a_k, *pb = x_ptr + b_k;
            if constexpr (K_TILES != 1) {
                for (int kt = 0; kt + 1 < n_kt; ++kt) {
                    stage_tile(false);
                    __syncthreads();
                    if (kt + 2 < n_kt) {
                        pa += KTILE;
                        pb += KTILE;
#pragma unroll
                        for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (pa + 4 * q);
#pragma unroll
                        for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (pb + 4 * q);
                    } else {
                        load_tile(n_kt - 1, true);
                    }
#pragma unroll
                    for (int ks = 0; ks < KTILE / 4; ++ks) mma_step(ks);
                    __syncthreads();
                }
            }
            stage_tile(true);
        }
        __syncthreads();   // the staged tile, this tile's column data and (first tile) the row data are in LDS
        if (jt + 1 < jt1) {   // the next column tile's requests go out now, ahead of this tile's epilogue
            request_tile(jt + 1);
            if (n_kt > 0) load_tile(0, n_kt == 1);
        }
        if (n_kt > 0) {
#pragma unroll
            for (int ks = 0; ks < KTILE / 4; ++ks)
                if (ks < n_ks_last) mma_step(ks);
            __syncthreads();   // every wavefront is done with the staged tile before the next one is written
        }
        double sdj[4];
        uint64_t mj[4];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
            sdj[tj] = s_sdj[gen][wj * 64 + lrow * 4 + tj];
            mj[tj] = IND ? s_mj[gen][wj * 64 + lrow * 4 + tj] : 0;
        }
        // the indicator columns' share of a dot product: 1.0 once per column both rows have set, one addition at a
        // time (the serial chain over those columns, bit for bit)
        auto with_indicators = [&](double dot, uint64_t mi, int tj) -> double {
            if (IND) {
                const int cnt = __popcll(mi & mj[tj]);
                for (int t = 0; t < max_ones; ++t) dot += cnt > t ? 1.0 : 0.0;
            }
            return dot;
        };
        // one batch row's four kernel values, widened to double as the reference widens them before its sums
        auto row_values = [&](int ti, int v, double *kv) {
            const int r = wi * (16 * TI) + ti * 16 + 4 * v + lk;
            const double sdi = s_sdi[r];
            const uint64_t mi = IND ? s_mi[r] : 0;
            if constexpr (KT == TSVM_RBF) {
                // expf's two out-of-range cases only where some argument of the wavefront needs them
                float xs[4];
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) xs[tj] = tsvm_rbf_arg(with_indicators(acc[ti][tj][v], mi, tj), sdi, sdj[tj], kp);
                const float mx = fmaxf(fmaxf(fabsf(xs[0]), fabsf(xs[1])), fmaxf(fabsf(xs[2]), fabsf(xs[3])));
                if (__builtin_amdgcn_ballot_w64(mx > 88.0f) == 0) {
#pragma unroll
                    for (int tj = 0; tj < 4; ++tj) kv[tj] = (double) tsvm_expf_in_range(xs[tj], exp_tab);
                } else {
#pragma unroll
                    for (int tj = 0; tj < 4; ++tj) kv[tj] = (double) tsvm_expf(xs[tj], exp_tab);
                }
            } else {
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) kv[tj] = tsvm_epilogue(with_indicators(acc[ti][tj][v], mi, tj), sdi, sdj[tj], kp, exp_tab);
            }
        };
        auto coef_of = [&](int c, double *cj) {   // coefficient row c of this lane's four columns
            const v2d c01 = *(const v2d *) &s_coef[gen][c][wj * 64 + lrow * 4];
            const v2d c23 = *(const v2d *) &s_coef[gen][c][wj * 64 + lrow * 4 + 2];
            cj[0] = c01[0]; cj[1] = c01[1]; cj[2] = c23[0]; cj[3] = c23[1];
        };
        if constexpr (NC <= 2) {
            // few coefficient rows: they wait in registers and every batch row is finished as soon as its values exist
            double cj[NC][4];
#pragma unroll
            for (int c = 0; c < NC; ++c) coef_of(c, cj[c]);
#pragma unroll
            for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    double kv[4];
                    row_values(ti, v, kv);
#pragma unroll
                    for (int c = 0; c < NC; ++c)
#pragma unroll
                        for (int tj = 0; tj < 4; ++tj) part[ti * 4 + v][c] = __builtin_fma(cj[c][tj], kv[tj], part[ti * 4 + v][c]);
                }
            }
        } else {
            // many coefficient rows: the kernel values take the accumulators' place, then one coefficient row at a time
#pragma unroll
            for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    double kv[4];
                    row_values(ti, v, kv);
#pragma unroll
                    for (int tj = 0; tj < 4; ++tj) acc[ti][tj][v] = kv[tj];
                }
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                double cj[4];
                coef_of(c, cj);
#pragma unroll
                for (int ti = 0; ti < TI; ++ti)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
#pragma unroll
                        for (int tj = 0; tj < 4; ++tj)
                            part[ti * 4 + v][c] = __builtin_fma(cj[tj], acc[ti][tj][v], part[ti * 4 + v][c]);
            }
        }
    }
    // the chunk's sums: over the sixteen lanes that hold the same rows, then over the two wavefront columns (As is
    // free: the last tile's final barrier lies behind every read of it)
    double *red = As;   // [2][BM][NC]
#pragma unroll
    for (int u = 0; u < TI * 4; ++u) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const double s = dpp_row_sum_f64(part[u][c]);
            if (lrow == 0) red[(wj * BM + wi * (16 * TI) + (u >> 2) * 16 + 4 * (u & 3) + lk) * NC + c] = s;
        }
    }
    __syncthreads();
    for (int e = tid; e < BM * nc_out; e += 256) {
        const int r = e / nc_out, c = e % nc_out;
        if (i0 + r < m) partial[((int64_t) chunk * m + i0 + r) * nc_out + c] = red[r * NC + c] + red[(BM + r) * NC + c];
    }
}

// ------------------------------------------------------------------------------------------------
// Many features: 128 x 128 tiles whose K loop is nearly all of the work; each tile's values are reduced as soon as
// they exist (get_rows_tile's FUSE mode) into sums that stay in LDS for the workgroup's chunk of tiles.  Any number
// of coefficient rows up to PD_MAX_NC.
// ------------------------------------------------------------------------------------------------
#define PD_MAX_NC 24

template <int KT>
__global__ __launch_bounds__(256, 2) void predict_dense_tile_kernel(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ col_map, int64_t n_pad, int d,
    const double *__restrict__ sd_x, const double *__restrict__ a, int64_t lda, int m, const double *__restrict__ sd_a,
    KernelParam kp, const double *__restrict__ coef_t, int nc, const int *__restrict__ chunks, unsigned m_blocks,
    double *__restrict__ partial) {
    constexpr int BM = GrShape<4>::BM;
    __shared__ double As[GrShape<4>::LDS_DOUBLES];
    __shared__ double Bs[GrShape<4>::LDS_DOUBLES];
    __shared__ uint64_t exp_tab[32];
    extern __shared__ double red[];   // [2][BM][nc]
    const int tid = threadIdx.x;
    if (tid < 32) exp_tab[tid] = TSVM_EXP2F_TAB[tid];
    for (int e = tid; e < 2 * BM * nc; e += 256) red[e] = 0.0;
    __syncthreads();
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int i0 = (int) (logical % m_blocks) * BM;
    const unsigned chunk = logical / m_blocks;
    const int jt0 = chunks[2 * chunk], jt1 = chunks[2 * chunk + 1];
    for (int jt = jt0; jt < jt1; ++jt) {
        get_rows_tile<KT, 4, double, false, true>(x, ldx, col_map, n_pad, d, sd_x, a, lda, nullptr, m, sd_a, kp, nullptr, nullptr,
                                                  0, i0, jt * GR_BN, As, Bs, exp_tab, coef_t, nc, red);
        __syncthreads();   // the tile's staging memory is free for the next tile; the sums are complete at the end
    }
    for (int e = tid; e < BM * nc; e += 256) {
        const int r = e / nc;
        if (i0 + r < m) partial[((int64_t) chunk * m + i0 + r) * nc + (e % nc)] = red[e] + red[BM * nc + e];
    }
}

// dec[r * P + p] for pair p = (i < j): the chunks of class i under coefficient row j - 1, then the chunks of class j
// under coefficient row i, each in chunk order, minus rho[p] (the order of kernelmatrix_kernel.cpp:129-143).
__global__ __launch_bounds__(256) void predict_combine_kernel(const double *__restrict__ partial, int64_t m, int nc,
                                                              const int *__restrict__ class_chunk_start,
                                                              const double *__restrict__ rho, int n_classes,
                                                              double *__restrict__ dec) {
    const int64_t P = (int64_t) n_classes * (n_classes - 1) / 2;
    const int64_t idx = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= m * P) return;
    const int64_t r = idx / P;
    int p = (int) (idx % P), i = 0;
    while (p >= n_classes - 1 - i) {
        p -= n_classes - 1 - i;
        ++i;
    }
    const int j = i + 1 + p;
    double s = 0.0;
    for (int ch = class_chunk_start[i]; ch < class_chunk_start[i + 1]; ++ch) s += partial[((int64_t) ch * m + r) * nc + (j - 1)];
    double t = 0.0;
    for (int ch = class_chunk_start[j]; ch < class_chunk_start[j + 1]; ++ch) t += partial[((int64_t) ch * m + r) * nc + i];
    dec[idx] = (s + t) - rho[idx % P];
}

static int nc_template(int nc) { return nc <= 4 ? nc : nc <= 6 ? 6 : 8; }

extern "C" {

int tsvm_predict_nc_stride(int n_classes, int d, int has_masks) {
    const int nc = n_classes - 1;
    if (nc < 1) return 0;
    if (d <= 128 || has_masks) return nc <= 8 ? nc_template(nc) : 0;
    return nc <= PD_MAX_NC ? nc : 0;
}

int tsvm_predict_dec_values_dense(const double *sv_x, int64_t ldx, int d, const double *sd_sv, const uint64_t *mask_sv,
                                  const int *col_map, int64_t n_pad, const double *coef_t, const int *chunks,
                                  int n_chunks, const int *class_chunk_start, const double *rho, int n_classes,
                                  const double *a, int64_t lda, int64_t m, const double *sd_a, const uint64_t *mask_a,
                                  int max_ones, int kernel_type, double gamma, double coef0, int degree, double *partial,
                                  double *dec_values, tsvm_stream stream) {
    TSVM_REQUIRE(sv_x && col_map && coef_t && chunks && class_chunk_start && rho && a && partial && dec_values,
                 "tsvm_predict_dec_values_dense: null pointer");
    TSVM_REQUIRE(n_classes >= 2 && m >= 0 && m <= 0x7fff0000 && n_pad >= 0 && n_pad % GR_BN == 0 && n_pad <= 0x7fff0000 &&
                     n_chunks >= 0 && d >= 0,
                 "tsvm_predict_dec_values_dense: bad size");
    TSVM_REQUIRE(ldx % 8 == 0 && lda % 8 == 0 && d <= ldx && d <= lda && ldx <= 0x7fffffff && lda <= 0x7fffffff,
                 "tsvm_predict_dec_values_dense: leading dimensions must be multiples of 8 and at least d (%d): ldx %lld, lda %lld", d,
                 (long long) ldx, (long long) lda);
    TSVM_REQUIRE(((uintptr_t) sv_x % 32 == 0) && ((uintptr_t) a % 32 == 0), "tsvm_predict_dec_values_dense: sv_x and a must be 32-byte aligned");
    TSVM_REQUIRE(kernel_type >= 0 && kernel_type <= 4, "tsvm_predict_dec_values_dense: unknown kernel type %d", kernel_type);
    TSVM_REQUIRE((kernel_type != TSVM_RBF && kernel_type != TSVM_PRECOMPUTED) || (sd_sv && sd_a),
                 "tsvm_predict_dec_values_dense: RBF needs self dot products");
    TSVM_REQUIRE((mask_sv == nullptr) == (mask_a == nullptr) && max_ones >= 0 && max_ones <= 64,
                 "tsvm_predict_dec_values_dense: masks come in pairs, max_ones in [0, 64]");
    const int nc = n_classes - 1;
    const int stride = tsvm_predict_nc_stride(n_classes, d, mask_sv != nullptr);
    TSVM_REQUIRE(stride > 0, "tsvm_predict_dec_values_dense: %d classes are more than this shape (d = %d) takes", n_classes, d);
    if (m == 0) return 0;
    KernelParam kp{kernel_type, degree, gamma, coef0};
    const dim3 block(256);
    if (n_chunks > 0) {
        if (d <= 128 || mask_sv) {
            const unsigned m_blocks = (unsigned) ((m + 63) / 64);
            TSVM_REQUIRE((int64_t) m_blocks * n_chunks < (int64_t) 0x7fffffff, "tsvm_predict_dec_values_dense: grid too large");
            const dim3 grid(m_blocks * (unsigned) n_chunks);
#define PD_STREAM(KTYPE, NC_, IND_, KT_)                                                                                        \
    hipLaunchKernelGGL((predict_dense_stream_kernel<KTYPE, NC_, IND_, KT_>), grid, block, 0, tsvm_s(stream), sv_x, ldx, col_map, d, \
                       sd_sv, mask_sv, a, lda, (int) m, sd_a, mask_a, max_ones, kp, coef_t, chunks, m_blocks, partial, nc)
#define PD_NC(KTYPE, IND_, KT_)                         \
    switch (stride) {                                   \
        case 1: PD_STREAM(KTYPE, 1, IND_, KT_); break;  \
        case 2: PD_STREAM(KTYPE, 2, IND_, KT_); break;  \
        case 3: PD_STREAM(KTYPE, 3, IND_, KT_); break;  \
        case 4: PD_STREAM(KTYPE, 4, IND_, KT_); break;  \
        case 6: PD_STREAM(KTYPE, 6, IND_, KT_); break;  \
        default: PD_STREAM(KTYPE, 8, IND_, KT_); break; \
    }
#define PD_KIND(KTYPE)                            \
    do {                                          \
        if (mask_sv) {                            \
            if (d <= 16) PD_NC(KTYPE, 1, 1)       \
            else PD_NC(KTYPE, 1, 2)               \
        } else {                                  \
            if (d <= 16) PD_NC(KTYPE, 0, 1)       \
            else PD_NC(KTYPE, 0, 2)               \
        }                                         \
    } while (0)
            switch (kernel_type) {
                case TSVM_LINEAR: PD_KIND(TSVM_LINEAR); break;
                case TSVM_POLY: PD_KIND(TSVM_POLY); break;
                case TSVM_SIGMOID: PD_KIND(TSVM_SIGMOID); break;
                default: PD_KIND(TSVM_RBF); break;
            }
#undef PD_KIND
#undef PD_NC
#undef PD_STREAM
        } else {
            const unsigned m_blocks = (unsigned) ((m + 127) / 128);
            TSVM_REQUIRE((int64_t) m_blocks * n_chunks < (int64_t) 0x7fffffff, "tsvm_predict_dec_values_dense: grid too large");
            const dim3 grid(m_blocks * (unsigned) n_chunks);
            const size_t shm = (size_t) 2 * 128 * nc * sizeof(double);
#define PD_TILE(KTYPE)                                                                                                       \
    hipLaunchKernelGGL((predict_dense_tile_kernel<KTYPE>), grid, block, shm, tsvm_s(stream), sv_x, ldx, col_map, n_pad, d, sd_sv, a, \
                       lda, (int) m, sd_a, kp, coef_t, nc, chunks, m_blocks, partial)
            switch (kernel_type) {
                case TSVM_LINEAR: PD_TILE(TSVM_LINEAR); break;
                case TSVM_POLY: PD_TILE(TSVM_POLY); break;
                case TSVM_SIGMOID: PD_TILE(TSVM_SIGMOID); break;
                default: PD_TILE(TSVM_RBF); break;
            }
#undef PD_TILE
        }
        TSVM_LAUNCH_CHECK();
    }
    const int64_t P = (int64_t) n_classes * nc / 2;
    hipLaunchKernelGGL(predict_combine_kernel, dim3((unsigned) ((m * P + 255) / 256)), block, 0, tsvm_s(stream), partial, m, nc,
                       class_chunk_start, rho, n_classes, dec_values);
    TSVM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
