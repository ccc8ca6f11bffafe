// KernelMatrix::get_rows / diag and the predict reduction as gfx950 kernels.
//
// Reference behaviour restated here: src/thundersvm/kernelmatrix.cpp:183-316 and
// src/thundersvm/kernel/kernelmatrix_kernel.cpp:9-160 (the USE_CUDA=OFF, USE_DOUBLE=ON build).
#include "../../include/thundersvm_amd.h"
#include "tsvm_device.h"
#include "tsvm_internal.h"

#include <algorithm>
#include <cstdlib>

#include "get_rows_tile.h"


template <int KT, int TI, typename TO>
__global__ __launch_bounds__(256, (TI == 2 ? 3 : 2)) void get_rows_dense_kernel(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ x_idx, int64_t n, int d,
    const double *__restrict__ sd_x, const double *__restrict__ a, int64_t lda, const int *__restrict__ a_idx, int m,
    const double *__restrict__ sd_a, KernelParam kp, TO *__restrict__ out, const int *__restrict__ out_slots,
    int64_t ldo, unsigned m_blocks, const int *__restrict__ m_dev) {
    __shared__ double As[GrShape<TI>::LDS_DOUBLES];
    __shared__ double Bs[GrShape<TI>::LDS_DOUBLES];
    __shared__ uint64_t exp_tab[32];
    if (threadIdx.x < 32) exp_tab[threadIdx.x] = TSVM_EXP2F_TAB[threadIdx.x];
    __syncthreads();
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int j0 = (int) (logical / m_blocks) * GR_BN;   // n fits 31 bits (checked by the host)
    const int i0 = (int) (logical % m_blocks) * GrShape<TI>::BM;
    if (m_dev) {
        // the number of working rows is only known on the device (m sized the grid): workgroups beyond it leave
        m = *m_dev;
        if (i0 >= m) return;
    }
    get_rows_tile<KT, TI, TO>(x, ldx, x_idx, n, d, sd_x, a, lda, a_idx, m, sd_a, kp, out, out_slots, ldo, i0, j0, As, Bs, exp_tab);
}

// ------------------------------------------------------------------------------------------------
// Dense get_rows for few features (d <= 128), the shape of the multi-class and regression workloads:
// hundreds of thousands of columns, a K loop of only one to eight 16-column tiles, and an epilogue that
// costs as much as the matrix work.  A workgroup keeps its 64 working rows and walks a run of consecutive
// 128-column tiles.  What is fixed per working row (index, slot, self dot product, output offset) is set up
// once, and the first K tile of the next column tile is requested from memory before the current tile's
// epilogue starts, so that the load latency is spent under the epilogue's arithmetic instead of in front of
// the next tile's first MFMA.
//
// IND: the last columns of the data are indicator columns (every value 0 or 1).  The matrix cores then only
// walk the columns before them (d), and the epilogue adds 1.0 once per indicator column that both rows have
// set, one addition at a time: fma(1, 1, acc) = fl(acc + 1) and a product with a zero adds nothing, so this
// is the serial chain over the indicator columns, bit for bit (a pre-summed count would round differently).
// mask_x / mask_a hold one bit per indicator column and row; max_ones bounds the set bits of a row.
// ------------------------------------------------------------------------------------------------
// K_TILES = 3: the K loop for three and more K tiles keeps the tile before the last in a block of its own, so that the
// tiles before it need no test of which kind of load comes next; shapes with fewer K tiles get the shorter code
// (measured in training runs: the larger kernel costs a short K loop more than the test costs a long one).
template <int KT, typename TO, int IND, int K_TILES = 2>   // K_TILES: 1 = a single K tile (d <= 16), 2 = any number, 3 = three and more (LONG_K)
__global__ __launch_bounds__(256, 3) void get_rows_dense_stream_kernel(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ x_idx, int64_t n, int d,
    const double *__restrict__ sd_x, const double *__restrict__ a, int64_t lda, const int *__restrict__ a_idx, int m,
    const double *__restrict__ sd_a, KernelParam kp_in, TO *__restrict__ out, const int *__restrict__ out_slots,
    int64_t ldo, unsigned m_blocks, unsigned j_tiles, unsigned tiles_per_wg, const int *__restrict__ m_dev,
    const uint64_t *__restrict__ mask_x, const uint64_t *__restrict__ mask_a, int max_ones, int vec_ok) {
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
    // per working row of the tile (fixed for the workgroup) and per column of the current tile (two generations: a
    // wavefront may stage the next tile's while another still reads this tile's in its epilogue)
    __shared__ double s_sdi[BM];
    __shared__ uint64_t s_mi[BM];
    __shared__ int s_slot[BM];
    __shared__ double s_sdj[2][GR_BN];
    __shared__ uint64_t s_mj[2][GR_BN];
    KernelParam kp = kp_in;
    kp.kernel_type = KT;
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int i0 = (int) (logical % m_blocks) * BM;
    const unsigned jt0 = (logical / m_blocks) * tiles_per_wg;
    const unsigned jt1 = jt0 + tiles_per_wg < j_tiles ? jt0 + tiles_per_wg : j_tiles;
    if (m_dev) {
        m = *m_dev;
        if (i0 >= m) return;
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int n_last = (int) n - 1, m_last = m - 1;
    const int a_row = tid / A_TPR, a_k = (tid % A_TPR) * (4 * A_VEC);
    const int b_row = tid >> 1, b_k = (tid & 1) * (4 * B_VEC);
    const int lrow = lane & 15;
    const int lk = lane >> 4;
    // Which column of the tile sits in which column slot of the B operand is free to choose.  Slot (tj, l) of a
    // wavefront's 64 columns holds column 4*l + tj, so the four accumulator tiles of a lane are four consecutive
    // columns and a lane's results for one working row leave as one 16- or 32-byte store (16 lanes: one run of 256
    // or 512 bytes of the output row) instead of four stores 64 columns apart.
    const int b_col = (b_row & 64) + ((b_row & 15) << 2) + ((b_row >> 4) & 3);   // column (in the tile) staged by this thread

    if (tid < 32) exp_tab[tid] = TSVM_EXP2F_TAB[tid];
    if (tid < BM) {
        const int r = min(i0 + tid, m_last);
        const int id = a_idx ? a_idx[r] : r;
        s_slot[tid] = out_slots ? out_slots[r] : r;
        s_sdi[tid] = sd_a ? sd_a[id] : 0.0;
        s_mi[tid] = IND ? mask_a[id] : 0;
    }
    int a_r = min(i0 + a_row, m_last);
    if (a_idx) a_r = a_idx[a_r];
    const double *a_ptr = a + (uint64_t) (uint32_t) a_r * (uint32_t) lda;

    const int n_kt = K_TILES == 1 ? (d > 0 ? 1 : 0) : (d + KTILE - 1) / KTILE;   // (K_TILES == 1: the host has checked d <= KTILE)
    const int n_ks_last = (d - (n_kt - 1) * KTILE + 3) / 4;   // groups of four columns in the last K tile, 1 .. KTILE / 4
    v4d ra[A_VEC], rb[B_VEC];
    double pre_sd = 0.0;      // the next tile's column data for column tid (threads below 128)
    uint64_t pre_m = 0;
    const double *x_ptr = x;
    // requests everything of column tile jt that comes from memory: the first K tile and the columns' self dot
    // products and masks
    auto request_tile = [&](unsigned jt) {
        int x_r = min((int) jt * GR_BN + b_col, n_last);
        if (x_idx) x_r = x_idx[x_r];
        x_ptr = x + (uint64_t) (uint32_t) x_r * (uint32_t) ldx;
        if (tid < GR_BN) {
            int jc = min((int) jt * GR_BN + tid, n_last);
            if (x_idx) jc = x_idx[jc];
            pre_sd = sd_x ? sd_x[jc] : 0.0;
            pre_m = IND ? mask_x[jc] : 0;
        }
    };
    // Rows are zero-padded up to ldx / lda (multiples of 8); the last 16-column tile may reach past that: vectors
    // that would start beyond the row re-read its last four columns instead (staged, never multiplied).
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
    // (IND: the columns from d on are live data, not padding, and the last group of four columns may reach into
    // them: the working rows' values there are staged as zeros, which makes every such product an exact zero)
    const int k_live = d - (n_kt - 1) * KTILE;   // columns of the last K tile that belong to the product
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
    if (jt0 < jt1) {
        request_tile(jt0);
        if (n_kt > 0) load_tile(0, n_kt == 1);
    }
    for (unsigned jt = jt0; jt < jt1; ++jt) {
        const int gen = (int) (jt & 1u);
        const int j0 = (int) jt * GR_BN;
        const int jb = j0 + wj * 64 + lrow * 4;   // first of this lane's four columns
        const bool full = (i0 + BM <= m) && (j0 + GR_BN <= (int) n);
        if (tid < GR_BN) {
            s_sdj[gen][tid] = pre_sd;
            s_mj[gen][tid] = pre_m;
        }
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
            // While the successor of a K tile is a whole tile, this thread's loads walk along its two rows with one
            // running pointer each and constant offsets: an address computed per load costs the matrix cores an issue
            // slot per instruction (24 of them per 32 MFMAs before the loop was written this way).  The last tile may
            // reach past the row and is loaded with care.
            const double *pa = a_ptr + a_k, *pb = x_ptr + b_k;
            if constexpr (K_TILES == 1) {
                // (nothing in front of the only tile)
            } else if constexpr (K_TILES == 3) {
                for (int kt = 0; kt + 2 < n_kt; ++kt) {
                    stage_tile(false);
                    __syncthreads();
                    pa += KTILE;
                    pb += KTILE;
#pragma unroll
                    for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (pa + 4 * q);
#pragma unroll
                    for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (pb + 4 * q);
#pragma unroll
                    for (int ks = 0; ks < KTILE / 4; ++ks) mma_step(ks);
                    __syncthreads();
                }
                if (n_kt >= 2) {   // the tile before the last
                    stage_tile(false);
                    __syncthreads();
                    load_tile(n_kt - 1, true);
#pragma unroll
                    for (int ks = 0; ks < KTILE / 4; ++ks) mma_step(ks);
                    __syncthreads();
                }
            } else {
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
        // one value: the indicator columns' share, then the kernel function.  IND = 1..4: that many additions,
        // unrolled (the addend is 1.0 or 0.0: no branch); IND = 5: max_ones of them in a loop
        auto with_indicators = [&](double dot, uint64_t mi, int tj) -> double {
            if (IND) {
                const int cnt = __popcll(mi & mj[tj]);
                if (IND <= 4) {
#pragma unroll
                    for (int t = 0; t < IND; ++t) dot += cnt > t ? 1.0 : 0.0;
                } else {
                    for (int t = 0; t < max_ones; ++t) dot += cnt > t ? 1.0 : 0.0;
                }
            }
            return dot;
        };
        auto finish = [&](double dot, double sdi, uint64_t mi, int tj) -> TO {
            return tsvm_epilogue_as<TO>(with_indicators(dot, mi, tj), sdi, sdj[tj], kp, exp_tab);
        };
        // interior tiles store without a test, four columns at a time; edge tiles (and outputs whose rows are not
        // 16-byte aligned) test and store every element
        typedef TO vec4_t __attribute__((ext_vector_type(4)));
        if (full && vec_ok) {
#pragma unroll
            for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int r = wi * (16 * TI) + ti * 16 + 4 * v + lk;   // row of the tile
                    const double sdi = s_sdi[r];
                    const uint64_t mi = IND ? s_mi[r] : 0;
                    TO *orow = out + (int64_t) ((uint64_t) (uint32_t) s_slot[r] * (uint32_t) ldo) + jb;
                    vec4_t res;
                    if constexpr (KT == TSVM_RBF && sizeof(TO) == 4) {
                        // expf's two out-of-range cases cost four instructions per value; one look at the largest
                        // magnitude among the wavefront's arguments (a NaN passes: it needs neither case) tells whether
                        // any value of this store needs them.  Every instruction saved is an issue slot for the MFMAs.
                        float xs[4];
#pragma unroll
                        for (int tj = 0; tj < 4; ++tj) xs[tj] = tsvm_rbf_arg(with_indicators(acc[ti][tj][v], mi, tj), sdi, sdj[tj], kp);
                        const float mx = fmaxf(fmaxf(fabsf(xs[0]), fabsf(xs[1])), fmaxf(fabsf(xs[2]), fabsf(xs[3])));
                        if (__builtin_amdgcn_ballot_w64(mx > 88.0f) == 0) {
#pragma unroll
                            for (int tj = 0; tj < 4; ++tj) res[tj] = tsvm_expf_in_range(xs[tj], exp_tab);
                        } else {
#pragma unroll
                            for (int tj = 0; tj < 4; ++tj) res[tj] = tsvm_expf(xs[tj], exp_tab);
                        }
                    } else {
#pragma unroll
                        for (int tj = 0; tj < 4; ++tj) res[tj] = finish(acc[ti][tj][v], sdi, mi, tj);
                    }
                    store_streaming((vec4_t *) orow, res);
                }
            }
        } else {
#pragma unroll
            for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int r = wi * (16 * TI) + ti * 16 + 4 * v + lk;
                    if (i0 + r >= m) continue;
                    const double sdi = s_sdi[r];
                    const uint64_t mi = IND ? s_mi[r] : 0;
                    TO *orow = out + (int64_t) ((uint64_t) (uint32_t) s_slot[r] * (uint32_t) ldo) + jb;
#pragma unroll
                    for (int tj = 0; tj < 4; ++tj)
                        if (jb + tj < n) orow[tj] = finish(acc[ti][tj][v], sdi, mi, tj);   // (single values: left to the L2 to merge)
                }
            }
        }
    }
}

// mask[r] = bit b set where x[r][first + b] != 0, b < count <= 64; *max_ones = largest number of set bits of a row
// (raised with atomicMax: the caller clears it)
__global__ void indicator_masks_kernel(const double *__restrict__ x, int64_t ld, int64_t n, int first, int count,
                                       uint64_t *__restrict__ mask, int *__restrict__ max_ones) {
    const int64_t r = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    int ones = 0;
    if (r < n) {
        uint64_t mk = 0;
        const double *row = x + r * ld + first;
        for (int b = 0; b < count; ++b) mk |= (uint64_t) (row[b] != 0.0) << b;
        mask[r] = mk;
        ones = __popcll(mk);
    }
#pragma unroll
    for (int msk = 32; msk >= 1; msk >>= 1) ones = max(ones, __shfl_xor(ones, msk, 64));
    if ((threadIdx.x & 63) == 0 && ones > 0) atomicMax(max_ones, ones);
}

// The m x m block K(x_idx[r], x_idx[t]) (a == x, a_idx == x_idx, rows written in place): tiles that lie below the
// diagonal are filled by the mirror writes of the others and get no workgroup.  Column tile j (128 wide) needs the
// 64-row tiles 0 .. 2j+1, so workgroup c works on column tile j = the largest j with j(j+1) <= c, row tile
// c - j(j+1); dealt out in this order, every XCD gets the same share of the work.
template <int KT, typename TO>
__global__ __launch_bounds__(256, 3) void get_rows_dense_sym_kernel(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ idx, int m, int d, const double *__restrict__ sd_x,
    KernelParam kp, TO *__restrict__ out, int64_t ldo, unsigned m_blocks) {
    __shared__ double As[GrShape<2>::LDS_DOUBLES];
    __shared__ double Bs[GrShape<2>::LDS_DOUBLES];
    __shared__ uint64_t exp_tab[32];
    const int c = (int) blockIdx.x;
    int jt = (int) ((sqrtf(4.0f * (float) c + 1.0f) - 1.0f) * 0.5f);
    while (jt > 0 && jt * (jt + 1) > c) --jt;
    while ((jt + 1) * (jt + 2) <= c) ++jt;
    const int j0 = jt * GR_BN;
    const int i0 = (c - jt * (jt + 1)) * GrShape<2>::BM;
    if (i0 >= m) return;               // (the last column tile has fewer row tiles when m is not a multiple of 128)
    if (threadIdx.x < 32) exp_tab[threadIdx.x] = TSVM_EXP2F_TAB[threadIdx.x];
    __syncthreads();
    get_rows_tile<KT, 2, TO, true>(x, ldx, idx, m, d, sd_x, x, ldx, idx, m, sd_x, kp, out, nullptr, ldo, i0, j0, As, Bs, exp_tab);
}

// ------------------------------------------------------------------------------------------------
// CSR get_rows: out[i][j] = epilogue( sum over row j's non-zeros, in stored order, of v * w[col][i] )
// One workgroup = 256 working rows i (one per thread) x 16 consecutive rows j; the 16 dot products
// live in registers and each thread stores its 16 results as one 64- or 128-byte run of output row i.
// ------------------------------------------------------------------------------------------------
// (JB = 16 stored rows per workgroup; 4 when there are only a few thousand of them, as for the solver's ws x ws
// block, so that the grid still covers the chip and a workgroup's chain of dependent loads is a quarter as long)
// TW: element type of the staged working rows.  Values that are float-exact (everything a LibSVM file or the
// reference's float interfaces can deliver) are staged as float: the products are formed in double either way,
// and these reads, m x 8 bytes per stored non-zero, are what the kernel's time goes into.
template <typename TO, int CS_JB, typename TW>
__global__ __launch_bounds__(256) void get_rows_csr_kernel(
    const double *__restrict__ val, const int *__restrict__ col, const int64_t *__restrict__ row_ptr,
    const int *__restrict__ x_idx, int64_t n, const double *__restrict__ sd_x, const TW *__restrict__ w, int m,
    const double *__restrict__ sd_w, KernelParam kp, TO *__restrict__ out, const int *__restrict__ out_slots,
    int64_t ldo, unsigned i_blocks, int vec_ok) {
    __shared__ uint64_t exp_tab[32];
    const int tid = threadIdx.x;
    if (tid < 32) exp_tab[tid] = TSVM_EXP2F_TAB[tid];
    __syncthreads();
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int64_t j0 = (int64_t) (logical / i_blocks) * CS_JB;
    const int i = (int) (logical % i_blocks) * 256 + tid;
    const bool active = i < m;
    const int ic = active ? i : 0;
    double acc[CS_JB];
#pragma unroll
    for (int jj = 0; jj < CS_JB; ++jj) {
        acc[jj] = 0.0;
        const int64_t j = j0 + jj;
        if (j < n) {
            const int64_t rj = x_idx ? (int64_t) x_idx[j] : j;
            const int64_t e0 = row_ptr[rj], e1 = row_ptr[rj + 1];
            double s = 0.0;
            // eight non-zeros at a time: their loads are all issued before the first product is needed; the
            // products are still added in stored order
            int64_t e = e0;
            for (; e + 8 <= e1; e += 8) {
                double v[8];
                TW x[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    v[u] = val[e + u];
                    x[u] = w[(int64_t) col[e + u] * m + ic];
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) s = __builtin_fma(v[u], (double) x[u], s);
            }
            for (; e < e1; ++e) s = __builtin_fma(val[e], (double) w[(int64_t) col[e] * m + ic], s);
            acc[jj] = s;
        }
    }
    if (!active) return;
    const double sdi = sd_w ? sd_w[i] : 0.0;
    TO *orow = out + (int64_t) (out_slots ? out_slots[i] : i) * ldo;
    TO res[CS_JB];
#pragma unroll
    for (int jj = 0; jj < CS_JB; ++jj) {
        const int64_t j = j0 + jj < n ? j0 + jj : n - 1;
        res[jj] = tsvm_epilogue_as<TO>(acc[jj], sdi, sd_x ? sd_x[x_idx ? (int64_t) x_idx[j] : j] : 0.0, kp, exp_tab);
    }
    // The thread's CS_JB results are consecutive elements of output row i: they leave as 16-byte pieces when the
    // row allows it (every lane of a wavefront writes into another row, so a store instruction touches 64 lines
    // either way; one value at a time the L2 had four times as many partial writes to gather).  Plain stores:
    // marked non-temporal, partial lines go to memory as they are, and the launch took 2.3 ms instead of 0.6.
    constexpr int PER = 16 / (int) sizeof(TO);
    typedef TO piece_t __attribute__((ext_vector_type(PER)));
    if (vec_ok && j0 + CS_JB <= n) {
#pragma unroll
        for (int jj = 0; jj < CS_JB; jj += PER) {
            piece_t pc;
#pragma unroll
            for (int u = 0; u < PER; ++u) pc[u] = res[jj + u];
            *(piece_t *) (orow + j0 + jj) = pc;
        }
    } else {
#pragma unroll
        for (int jj = 0; jj < CS_JB; ++jj)
            if (j0 + jj < n) orow[j0 + jj] = res[jj];
    }
}

// ------------------------------------------------------------------------------------------------
// CSR get_rows on a sliced copy of the stored rows.
//
// The kernel above reads the staged working rows once per stored non-zero: m values for every entry of the matrix,
// gigabytes through the L2 per call.  Here the roles are turned round.  The stored rows are kept a second time in
// slices of 64 rows (sliced ELL): entry k of row 64 s + l lies at slice_ptr[s] + 64 k + l, rows shorter than their
// slice's longest are padded with the column n_features and the value 0, so a wavefront reads 64 rows' k-th entries
// as one contiguous run.  One thread owns one stored row j and sixteen accumulators, one per working row of the
// workgroup's block of sixteen; the block's working rows live in LDS as a dense tile over the features that occur
// in them (a 16-bit table maps a feature to its tile row, or to "absent").  Every stored entry is read once per
// block of sixteen working rows (from the L2: all blocks walk the same rows at the same time), looked up in LDS, and
// if present multiplied into the sixteen sums.  Products with absent features are zero and are left out; the others
// are added in stored order, so every sum is the serial chain of the reference, bit for bit.
// ------------------------------------------------------------------------------------------------
#define SL_T 1024   // threads = stored rows per step of a workgroup (sixteen slices)
#define SL_IB 16    // working rows per workgroup

template <typename TV>
__global__ void csr_slice_fill_kernel(const double *__restrict__ val, const int *__restrict__ col,
                                      const int64_t *__restrict__ row_ptr, int64_t n, const int64_t *__restrict__ slice_ptr,
                                      int pad_col, int *__restrict__ ell_col, TV *__restrict__ ell_val) {
    const int64_t s = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int64_t base = slice_ptr[s];
    const int width = (int) ((slice_ptr[s + 1] - base) >> 6);
    const int64_t j = s * 64 + lane;
    const int64_t e0 = j < n ? row_ptr[j] : 0, len = j < n ? row_ptr[j + 1] - e0 : 0;
    for (int k = threadIdx.x >> 6; k < width; k += blockDim.x >> 6) {
        const bool live = k < len;
        ell_col[base + (int64_t) k * 64 + lane] = live ? col[e0 + k] : pad_col;
        ell_val[base + (int64_t) k * 64 + lane] = live ? (TV) val[e0 + k] : (TV) 0;
    }
}

__global__ void csr_slice_widths_kernel(const int64_t *__restrict__ row_ptr, int64_t n, int *__restrict__ widths) {
    const int64_t j = (int64_t) blockIdx.x * 64 + (threadIdx.x & 63);
    int len = j < n ? (int) (row_ptr[j + 1] - row_ptr[j]) : 0;
#pragma unroll
    for (int msk = 32; msk >= 1; msk >>= 1) len = max(len, __shfl_xor(len, msk, 64));
    if ((threadIdx.x & 63) == 0) widths[blockIdx.x] = len;
}

// LDS layout of the kernel below: tile double[4][slot_cap][4] | remap u16[d + 2] | bits u32[words] | base u32[words].
// The tile takes what the other tables leave of SL_LDS_BUDGET.
#define SL_LDS_BUDGET (156 * 1024)
struct SlicedLds {
    size_t remap, bits, base, total;
    int slot_cap;
};
static SlicedLds sliced_lds(int d) {
    SlicedLds l;
    const size_t words = ((size_t) d + 1 + 31) / 32;
    const size_t tables = (((size_t) d + 2) * 2 + 15) / 16 * 16 + 2 * words * 4 + 16;
    const size_t room = SL_LDS_BUDGET > tables ? SL_LDS_BUDGET - tables : 0;
    l.slot_cap = (int) std::min<size_t>(room / (SL_IB * sizeof(double)), 0xfffe);
    l.remap = (size_t) l.slot_cap * SL_IB * sizeof(double);
    l.bits = l.remap + (((size_t) d + 2) * 2 + 15) / 16 * 16;
    l.base = l.bits + words * 4;
    l.total = l.base + words * 4 + 16;
    return l;
}

// The working rows' tile holds doubles: a float there would have to be widened once per use, and on this part the
// conversion instruction runs at a quarter of the rate of a double-precision multiply-add (with a float tile the
// kernel took 0.36 ms at 512 x 72,000 rows of ~50 entries, the conversions two thirds of it).
// A block of sixteen working rows whose features outnumber the tile's rows is done in two halves (the host has
// checked that eight of the longest rows fit).
template <int KT, typename TO, typename TV>
__global__ __launch_bounds__(SL_T) void get_rows_csr_sliced_kernel(
    const int *__restrict__ ell_col, const TV *__restrict__ ell_val, const int64_t *__restrict__ slice_ptr, int64_t n,
    const double *__restrict__ sd_x, const double *__restrict__ a_val, const int *__restrict__ a_col,
    const int64_t *__restrict__ a_ptr, const int *__restrict__ a_idx, int m, const double *__restrict__ sd_a, int d,
    int slot_cap, KernelParam kp_in, TO *__restrict__ out, const int *__restrict__ out_slots, int64_t ldo, unsigned n_ib,
    int steps, size_t off_remap, size_t off_bits, size_t off_base) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ uint64_t exp_tab[32];
    __shared__ double s_sdi[SL_IB];
    KernelParam kp = kp_in;
    kp.kernel_type = KT;
    __shared__ int64_t s_orow[SL_IB];
    __shared__ int64_t s_arow[SL_IB];
    __shared__ unsigned s_wave_total[SL_T / 64];
    double *tile = (double *) lds;
    uint16_t *remap = (uint16_t *) (lds + off_remap);
    unsigned *bits = (unsigned *) (lds + off_bits);
    unsigned *wbase = (unsigned *) (lds + off_base);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned logical = xcd_remap(blockIdx.x, gridDim.x);
    const int i0 = (int) (logical % n_ib) * SL_IB;
    const int64_t chunk = logical / n_ib;
    const int n_words = (d + 1 + 31) / 32;
    const int wpt = (n_words + SL_T - 1) / SL_T;
    const int64_t n_slices = (n + 63) / 64;
    typedef double tile4 __attribute__((ext_vector_type(4)));
    if (tid < 32) exp_tab[tid] = TSVM_EXP2F_TAB[tid];
    if (tid < SL_IB) {
        const int i = i0 + tid < m ? i0 + tid : m - 1;
        const int64_t row = a_idx ? (int64_t) a_idx[i] : (int64_t) i;
        s_arow[tid] = row;
        s_sdi[tid] = sd_a ? sd_a[row] : 0.0;
        s_orow[tid] = (int64_t) (out_slots ? out_slots[i] : i) * ldo;
    }
    __syncthreads();
    int r0 = 0, nr = SL_IB;   // the working rows of this pass: r0 .. r0 + nr - 1 of the block, at tile positions 0 .. nr - 1
    while (r0 < SL_IB) {
        // which features occur in the pass's rows (wavefront p walks row r0 + p)
        const bool row_live = wave < nr && i0 + r0 + wave < m;
        const int64_t ae0 = row_live ? a_ptr[s_arow[r0 + wave]] : 0, ae1 = row_live ? a_ptr[s_arow[r0 + wave] + 1] : 0;
        for (int w = tid; w < n_words; w += SL_T) bits[w] = 0;
        __syncthreads();
        for (int64_t e = ae0 + lane; e < ae1; e += 64) {
            const int c = a_col[e];
            if (c >= 0 && c < d) atomicOr(&bits[c >> 5], 1u << (c & 31));
        }
        __syncthreads();
        // tile rows in feature order: exclusive prefix sums of the words' bit counts
        unsigned mine = 0;
        for (int q = 0; q < wpt; ++q) {
            const int w = tid * wpt + q;
            mine += w < n_words ? __popc(bits[w]) : 0;
        }
        unsigned incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const unsigned t = __shfl_up(incl, off, 64);
            if (lane >= off) incl += t;
        }
        if (lane == 63) s_wave_total[wave] = incl;
        __syncthreads();
        unsigned before = 0, n_slots = 0;
        for (int w = 0; w < SL_T / 64; ++w) {
            before += w < wave ? s_wave_total[w] : 0;
            n_slots += s_wave_total[w];
        }
        if (n_slots > (unsigned) slot_cap && nr > SL_IB / 2) {   // (uniform) too many features: this half first, then the other
            nr = SL_IB / 2;
            __syncthreads();
            continue;
        }
        unsigned run = before + incl - mine;
        for (int q = 0; q < wpt; ++q) {
            const int w = tid * wpt + q;
            if (w < n_words) {
                wbase[w] = run;
                run += __popc(bits[w]);
            }
        }
        __syncthreads();
        for (int c = tid; c <= d; c += SL_T) {
            const unsigned word = bits[c >> 5], bit = 1u << (c & 31);
            remap[c] = (word & bit) ? (uint16_t) (wbase[c >> 5] + __popc(word & (bit - 1u))) : (uint16_t) 0xffff;
        }
        // The tile in four parts, one per group of four working rows: part g holds 4 values per tile row, [slot_cap][4],
        // so that the 64 lanes of a read, each at another tile row, spread over the LDS banks.
        for (unsigned e = tid; e < (unsigned) slot_cap * SL_IB; e += SL_T) tile[e] = 0.0;
        __syncthreads();
        for (int64_t e = ae0 + lane; e < ae1; e += 64) {
            const int c = a_col[e];
            if (c >= 0 && c < d) {
                const unsigned slot = remap[c];
                if (slot < (unsigned) slot_cap) tile[((unsigned) (wave >> 2) * slot_cap + slot) * 4 + (wave & 3)] = a_val[e];
            }
        }
        __syncthreads();

        for (int step = 0; step < steps; ++step) {
            const int64_t slice = (chunk * steps + step) * (SL_T / 64) + wave;
            if (slice >= n_slices) break;   // (wavefront-uniform; no barrier inside this loop)
            const int64_t base = slice_ptr[slice];
            const int width = (int) ((slice_ptr[slice + 1] - base) >> 6);
            const int64_t j = slice * 64 + lane;
            double acc[SL_IB];
#pragma unroll
            for (int r = 0; r < SL_IB; ++r) acc[r] = 0.0;
            const int *pc = ell_col + base + lane;
            const TV *pv = ell_val + base + lane;
            auto take = [&](int c, double v) {
                const unsigned slot = remap[c];
                if (slot != 0xffffu) {
                    const tile4 *t = (const tile4 *) tile + slot;
#pragma unroll
                    for (int g = 0; g < SL_IB / 4; ++g) {
                        const tile4 a4 = t[(size_t) g * slot_cap];
#pragma unroll
                        for (int u = 0; u < 4; ++u) acc[g * 4 + u] = __builtin_fma(v, a4[u], acc[g * 4 + u]);
                    }
                }
            };
            int k = 0;
            for (; k + 4 <= width; k += 4) {   // four entries' loads go out together; the products keep stored order
                int c[4];
                TV v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    c[u] = pc[(int64_t) (k + u) * 64];
                    v[u] = pv[(int64_t) (k + u) * 64];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) take(c[u], (double) v[u]);
            }
            for (; k < width; ++k) take(pc[(int64_t) k * 64], (double) pv[(int64_t) k * 64]);
            if (j < n) {
                const double sdj = sd_x ? sd_x[j] : 0.0;
#pragma unroll
                for (int p = 0; p < SL_IB; ++p)
                    if (p < nr && i0 + r0 + p < m) out[s_orow[r0 + p] + j] = tsvm_epilogue_as<TO>(acc[p], s_sdi[r0 + p], sdj, kp, exp_tab);
            }
        }
        r0 += nr;
        __syncthreads();   // every wavefront is done with the tile before the next pass rebuilds it
    }
}

// out row r = x row idx[r]; rows are ld doubles long, ld a multiple of 4, moved as 32-byte vectors
__global__ void gather_rows_f64_kernel(const v4d *__restrict__ x, int64_t ld4, const int *__restrict__ idx, int64_t m,
                                       v4d *__restrict__ out) {
    const int64_t total = m * ld4;
    for (int64_t e = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (int64_t) gridDim.x * blockDim.x) {
        const int64_t r = e / ld4, c = e % ld4;
        out[e] = x[(int64_t) idx[r] * ld4 + c];
    }
}

// CSR rows idx[0..m) copied to a new CSR whose row offsets out_ptr are already known; one wavefront per row
__global__ void csr_gather_rows_kernel(const double *__restrict__ val, const int *__restrict__ col,
                                       const int64_t *__restrict__ row_ptr, const int *__restrict__ idx, int64_t m,
                                       const int64_t *__restrict__ out_ptr, double *__restrict__ out_val,
                                       int *__restrict__ out_col) {
    const int64_t r = ((int64_t) blockIdx.x * blockDim.x + threadIdx.x) / 64;
    const int lane = threadIdx.x & 63;
    if (r >= m) return;
    const int64_t src = row_ptr[idx[r]], dst = out_ptr[r], len = out_ptr[r + 1] - dst;
    for (int64_t e = lane; e < len; e += 64) {
        out_val[dst + e] = val[src + e];
        out_col[dst + e] = col[src + e];
    }
}

__global__ void fold_ids_kernel(const int *__restrict__ ids, int count, int period, int *__restrict__ out) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t < count) out[t] = ids[t] % period;
}

__global__ void fill_f64_kernel(double *p, int64_t count, double v) {
    for (int64_t e = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; e < count; e += (int64_t) gridDim.x * blockDim.x)
        p[e] = v;
}

// w[c*m + i] = value of feature c in CSR row idx[i] (clear: 0.0 instead, which takes the rows out of a staging
// matrix again); one wavefront per staged row.
template <typename TW>
__global__ void csr_stage_rows_kernel(const double *__restrict__ val, const int *__restrict__ col,
                                      const int64_t *__restrict__ row_ptr, const int *__restrict__ idx, int m,
                                      int n_features, TW *__restrict__ w, int clear) {
    const int i = (int) ((blockIdx.x * (int64_t) blockDim.x + threadIdx.x) >> 6);
    const int lane = threadIdx.x & 63;
    if (i >= m) return;
    const int64_t r = idx ? (int64_t) idx[i] : (int64_t) i;
    for (int64_t e = row_ptr[r] + lane; e < row_ptr[r + 1]; e += 64) {
        const int c = col[e];
        if (c < n_features) w[(int64_t) c * m + i] = clear ? (TW) 0 : (TW) val[e];
    }
}

// x[r*ld + c] = value of feature c in row r; one wavefront per row.
__global__ void csr_to_dense_kernel(const double *__restrict__ val, const int *__restrict__ col,
                                    const int64_t *__restrict__ row_ptr, int64_t n, double *__restrict__ x, int64_t ld) {
    const int64_t r = (blockIdx.x * (int64_t) blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (r >= n) return;
    for (int64_t e = row_ptr[r] + lane; e < row_ptr[r + 1]; e += 64) {
        const int c = col[e];
        if (c < ld) x[r * ld + c] = val[e];
    }
}

// self_dot[i] = serial fma chain over the row's values (kernelmatrix.cpp:195-205).
__global__ void csr_self_dot_kernel(const double *__restrict__ val, const int64_t *__restrict__ row_ptr, int64_t n,
                                    double *__restrict__ self_dot) {
    const int64_t i = blockIdx.x * (int64_t) blockDim.x + threadIdx.x;
    if (i >= n) return;
    double s = 0.0;
    for (int64_t e = row_ptr[i]; e < row_ptr[i + 1]; ++e) s = __builtin_fma(val[e], val[e], s);
    self_dot[i] = s;
}

__global__ void dense_self_dot_kernel(const double *__restrict__ x, int64_t ld, int64_t n, int d,
                                      double *__restrict__ self_dot) {
    const int64_t i = blockIdx.x * (int64_t) blockDim.x + threadIdx.x;
    if (i >= n) return;
    double s = 0.0;
    const double *r = x + i * ld;
    for (int k = 0; k < d; ++k) s = __builtin_fma(r[k], r[k], s);
    self_dot[i] = s;
}

__global__ void kernel_diag_kernel(const double *__restrict__ self_dot, int64_t n, KernelParam kp,
                                   double *__restrict__ diag) {
    const int64_t i = blockIdx.x * (int64_t) blockDim.x + threadIdx.x;
    if (i >= n) return;
    double v;
    switch (kp.kernel_type) {
        case TSVM_RBF:
        case TSVM_PRECOMPUTED: v = 1.0; break;
        case TSVM_LINEAR: v = self_dot[i]; break;
        default: v = tsvm_epilogue(self_dot[i], 0.0, 0.0, kp, TSVM_EXP2F_TAB); break;
    }
    diag[i] = v;
}

// Column statistics of the data rows: counts[c] = number of entries in column c (dense layout: non-zero values; CSR:
// stored entries), counts[d + c] = how many values are neither 0 nor 1 (none: an indicator column).  The reference's
// KernelMatrix constructor counts the stored entries per column to split the matrix into a dense and a sparse
// part (CSR_DenseCSR, kernelmatrix.cpp:16-74).
__global__ __launch_bounds__(256) void column_stats_dense_kernel(const double *__restrict__ x, int64_t ld, int64_t n, int d,
                                                                 int *__restrict__ counts) {
    const int64_t rows_per = (n + gridDim.x - 1) / gridDim.x;
    const int64_t r0 = (int64_t) blockIdx.x * rows_per, r1 = r0 + rows_per < n ? r0 + rows_per : n;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        int nz = 0, nu = 0;
        for (int64_t r = r0; r < r1; ++r) {
            const double v = x[r * ld + c];
            nz += v != 0.0;
            nu += v != 0.0 && v != 1.0;
        }
        if (nz) atomicAdd(&counts[c], nz);
        if (nu) atomicAdd(&counts[d + c], nu);
    }
}

__global__ __launch_bounds__(256) void column_stats_csr_kernel(const double *__restrict__ val, const int *__restrict__ col,
                                                               int64_t nnz, int d, int *__restrict__ counts) {
    for (int64_t e = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t) gridDim.x * blockDim.x) {
        const double v = val[e];
        const int c = col[e];
        if (c < 0 || c >= d) continue;
        atomicAdd(&counts[c], 1);   // stored entries, as the reference counts them (a stored 0.0 included)
        if (v != 1.0 && v != 0.0) atomicAdd(&counts[d + c], 1);
    }
}

__global__ void fill_i32_kernel(int *p, int64_t count, int v) {
    for (int64_t e = (int64_t) blockIdx.x * blockDim.x + threadIdx.x; e < count; e += (int64_t) gridDim.x * blockDim.x)
        p[e] = v;
}

__global__ void gather_f64_kernel(const double *__restrict__ in, const int *__restrict__ idx, int m,
                                  double *__restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < m) out[i] = in[idx[i]];
}

// ------------------------------------------------------------------------------------------------
// sum_kernel_values (kernelmatrix_kernel.cpp:110-147).
// One workgroup handles SK_R test rows.  For coefficient row c (0..k-2) and SV class s the segment
// sum S[c][s] = sum_{l in SV_s} coef[c*T + l] * K[r][l] is accumulated by 256 threads striding over
// the segment and tree-reduced through LDS; dec(i,j) = S[j-1][i] + S[i][j] - rho.  Every (c, s) belongs to
// exactly one pair, and with s as the outer loop a pair's first term S[j-1][i] (s = i) is always ready before
// its second S[i][j] (s = j): the first is parked in dec itself and the thread that parked it completes the
// value when the second arrives, so no table grows with the number of classes.  The summation
// order differs from the reference's serial loop (results agree to ~1e-13 relative, inside the
// 1e-6 absolute tolerance on decision values).
// ------------------------------------------------------------------------------------------------
#define SK_R 4
#define SK_T 256

template <typename TK>
__global__ __launch_bounds__(SK_T) void sum_kernel_values_kernel(
    const double *__restrict__ coef, int total_sv, const int *__restrict__ sv_start, const int *__restrict__ sv_count,
    const double *__restrict__ rho, const TK *__restrict__ k_mat, int64_t ldk, double *__restrict__ dec,
    int n_classes, int64_t n_instances) {
    __shared__ double red[(SK_T / 64) * SK_R];   // per-wavefront partial sums
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t r0 = (int64_t) blockIdx.x * SK_R;
    const int km1 = n_classes - 1;
    const int64_t P = (int64_t) n_classes * km1 / 2;
    for (int s = 0; s < n_classes; ++s) {
        const int st = sv_start[s], cnt = sv_count[s];
        for (int c = 0; c < km1; ++c) {
            // every (c, s) is used by exactly one pair: (i=s, j=c+1) when c >= s (its first term), (i=c, j=s) when
            // c < s (its second term)
            const double *cf = coef + (int64_t) c * total_sv + st;
            double part[SK_R];
#pragma unroll
            for (int rr = 0; rr < SK_R; ++rr) part[rr] = 0.0;
            // four support vectors per thread at a time: their loads go out together, the sums keep their order
            int l = tid;
            for (; l + 3 * SK_T < cnt; l += 4 * SK_T) {
                double cv[4];
                TK kv[4][SK_R];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    cv[u] = cf[l + u * SK_T];
#pragma unroll
                    for (int rr = 0; rr < SK_R; ++rr) {
                        const int64_t r = r0 + rr < n_instances ? r0 + rr : n_instances - 1;   // a valid row; not added below
                        kv[u][rr] = k_mat[r * ldk + st + l + u * SK_T];   // (read once per class: the L2 serves the repeats)
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int rr = 0; rr < SK_R; ++rr)
                        if (r0 + rr < n_instances) part[rr] = __builtin_fma(cv[u], (double) kv[u][rr], part[rr]);
            }
            for (; l < cnt; l += SK_T) {
                const double cv = cf[l];
#pragma unroll
                for (int rr = 0; rr < SK_R; ++rr) {
                    const int64_t r = r0 + rr;
                    if (r < n_instances) part[rr] = __builtin_fma(cv, (double) k_mat[r * ldk + st + l], part[rr]);
                }
            }
#pragma unroll
            for (int rr = 0; rr < SK_R; ++rr) {
                double v = part[rr];
#pragma unroll
                for (int msk = 32; msk >= 1; msk >>= 1) v += shfl_xor_f64(v, msk);
                if (lane == 0) red[wave * SK_R + rr] = v;
            }
            __syncthreads();
            if (tid < SK_R && r0 + tid < n_instances) {
                double t = 0.0;
                for (int wv = 0; wv < SK_T / 64; ++wv) t += red[wv * SK_R + tid];
                const bool first = c >= s;
                const int i = first ? s : c, j = first ? c + 1 : s;
                const int64_t p = (int64_t) i * (2 * n_classes - i - 1) / 2 + (j - i - 1);
                double *out = dec + (r0 + tid) * P + p;
                *out = first ? t : (*out + t) - rho[p];
            }
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------------
static inline unsigned grid_for(int64_t n, int block) { return (unsigned) ((n + block - 1) / block); }

extern "C" {

int tsvm_csr_self_dot(const double *val, const int64_t *row_ptr, int64_t n, double *self_dot, tsvm_stream stream) {
    TSVM_REQUIRE(n >= 0 && row_ptr && self_dot, "tsvm_csr_self_dot: bad argument");
    if (n == 0) return 0;
    hipLaunchKernelGGL(csr_self_dot_kernel, dim3(grid_for(n, 256)), dim3(256), 0, tsvm_s(stream), val, row_ptr, n, self_dot);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_dense_self_dot(const double *x, int64_t ld, int64_t n, int d, double *self_dot, tsvm_stream stream) {
    TSVM_REQUIRE(n >= 0 && x && self_dot && d >= 0 && d <= ld, "tsvm_dense_self_dot: bad argument");
    if (n == 0) return 0;
    hipLaunchKernelGGL(dense_self_dot_kernel, dim3(grid_for(n, 256)), dim3(256), 0, tsvm_s(stream), x, ld, n, d, self_dot);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_kernel_diag(const double *self_dot, int64_t n, int kernel_type, double gamma, double coef0, int degree,
                     double *diag, tsvm_stream stream) {
    TSVM_REQUIRE(n >= 0 && self_dot && diag, "tsvm_kernel_diag: bad argument");
    TSVM_REQUIRE(kernel_type >= 0 && kernel_type <= 4, "tsvm_kernel_diag: unknown kernel type %d", kernel_type);
    if (n == 0) return 0;
    KernelParam kp{kernel_type, degree, gamma, coef0};
    hipLaunchKernelGGL(kernel_diag_kernel, dim3(grid_for(n, 256)), dim3(256), 0, tsvm_s(stream), self_dot, n, kp, diag);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_csr_to_dense(const double *val, const int *col, const int64_t *row_ptr, int64_t n, double *x, int64_t ld,
                      tsvm_stream stream) {
    TSVM_REQUIRE(n >= 0 && row_ptr && x && ld > 0, "tsvm_csr_to_dense: bad argument");
    if (n == 0) return 0;
    hipLaunchKernelGGL(fill_f64_kernel, dim3(2048), dim3(256), 0, tsvm_s(stream), x, n * ld, 0.0);
    TSVM_LAUNCH_CHECK();
    hipLaunchKernelGGL(csr_to_dense_kernel, dim3(grid_for(n * 64, 256)), dim3(256), 0, tsvm_s(stream), val, col, row_ptr,
                       n, x, ld);
    TSVM_LAUNCH_CHECK();
    return 0;
}

static bool row_type_ok(int row_type, int kernel_type) {
    // float rows are exact only where the reference's value is a float to begin with
    return row_type == TSVM_ROW_F64 || (row_type == TSVM_ROW_F32 && kernel_type != TSVM_LINEAR);
}

// Column tiles a workgroup of the few-feature kernel walks (TSVM_GR_TILES overrides the default of 4).
static int stream_tiles_per_wg() {
    static const int v = [] {
        const char *e = getenv("TSVM_GR_TILES");
        const int t = e ? atoi(e) : 0;
        return t >= 1 && t <= 64 ? t : 4;
    }();
    return v;
}

static int get_rows_dense(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d, const double *sd_x, const double *a,
                          int64_t lda, const int *a_idx, int m, const int *m_dev, const double *sd_a, int kernel_type, double gamma,
                          double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                          tsvm_stream stream, const uint64_t *mask_x = nullptr, const uint64_t *mask_a = nullptr,
                          int max_ones = 0) {
    TSVM_REQUIRE(x && a && out, "tsvm_get_rows_dense: null pointer");
    TSVM_REQUIRE(n >= 0 && m >= 0 && d >= 0, "tsvm_get_rows_dense: negative size");
    TSVM_REQUIRE(n <= 0x7fff0000 && ldx <= 0x7fffffff && lda <= 0x7fffffff && ldo <= 0x7fffffff,
                 "tsvm_get_rows_dense: row counts and leading dimensions must fit 31 bits");
    TSVM_REQUIRE(ldx % 8 == 0 && lda % 8 == 0, "tsvm_get_rows_dense: ldx (%lld) and lda (%lld) must be multiples of 8",
                 (long long) ldx, (long long) lda);
    TSVM_REQUIRE(d <= ldx && d <= lda, "tsvm_get_rows_dense: d (%d) exceeds a leading dimension", d);
    TSVM_REQUIRE(ldo >= n, "tsvm_get_rows_dense: ldo (%lld) < n (%lld)", (long long) ldo, (long long) n);
    TSVM_REQUIRE(((uintptr_t) x % 32 == 0) && ((uintptr_t) a % 32 == 0), "tsvm_get_rows_dense: x and a must be 32-byte aligned");
    TSVM_REQUIRE(kernel_type >= 0 && kernel_type <= 4, "tsvm_get_rows_dense: unknown kernel type %d", kernel_type);
    TSVM_REQUIRE(row_type_ok(row_type, kernel_type), "tsvm_get_rows_dense: row type %d not valid for kernel type %d", row_type,
                 kernel_type);
    TSVM_REQUIRE((kernel_type != TSVM_RBF && kernel_type != TSVM_PRECOMPUTED) || (sd_x && sd_a),
                 "tsvm_get_rows_dense: RBF needs self dot products");
    if (n == 0 || m == 0) return 0;
    KernelParam kp{kernel_type, degree, gamma, coef0};
    // few features: the epilogue weighs as much as the MFMAs, run the 64-row tile at higher occupancy
    // (also when the 128-row tile would leave most of the chip without a workgroup, as for the solver's
    // ws x ws block, whose latency is that of one workgroup walking the whole feature range)
    const int64_t wg4 = ((n + GR_BN - 1) / GR_BN) * ((m + 127) / 128);
    const int ti = (d <= 128 || wg4 < 512 || mask_x) ? 2 : 4;
    const unsigned m_blocks = (unsigned) ((m + 32 * ti - 1) / (32 * ti));
    const int64_t n_blocks = (n + GR_BN - 1) / GR_BN;
    TSVM_REQUIRE(n_blocks * m_blocks < (int64_t) 0x7fffffff, "tsvm_get_rows_dense: grid too large");
    dim3 grid((unsigned) (n_blocks * m_blocks)), block(256);
    // the solver's ws x ws block: symmetric, computed from the tiles on and above the diagonal
    const bool sym = x == a && ldx == lda && x_idx && x_idx == a_idx && n == m && sd_x == sd_a && !out_slots && !m_dev &&
                     ti == 2 && ldo >= n;
    if (sym) {
        grid = dim3((unsigned) (n_blocks * (n_blocks + 1)));   // column tile j: row tiles 0 .. 2j+1
#define GR_SYM(KTYPE, TO)                                                                                                      \
    hipLaunchKernelGGL((get_rows_dense_sym_kernel<KTYPE, TO>), grid, block, 0, tsvm_s(stream), x, ldx, x_idx, m, d, sd_x, kp, (TO *) out, \
                       ldo, m_blocks)
        if (row_type == TSVM_ROW_F32) {
            switch (kernel_type) {
                case TSVM_POLY: GR_SYM(TSVM_POLY, float); break;
                case TSVM_SIGMOID: GR_SYM(TSVM_SIGMOID, float); break;
                default: GR_SYM(TSVM_RBF, float); break;
            }
        } else {
            switch (kernel_type) {
                case TSVM_LINEAR: GR_SYM(TSVM_LINEAR, double); break;
                case TSVM_POLY: GR_SYM(TSVM_POLY, double); break;
                case TSVM_SIGMOID: GR_SYM(TSVM_SIGMOID, double); break;
                default: GR_SYM(TSVM_RBF, double); break;
            }
        }
#undef GR_SYM
        TSVM_LAUNCH_CHECK();
        return 0;
    }
    // few features: workgroups walk runs of column tiles (one tile each while the launch is too small to fill the chip
    // several times over)
    const int64_t total_tiles = n_blocks * m_blocks;
    const unsigned tpw = (unsigned) std::max<int64_t>(1, std::min<int64_t>(stream_tiles_per_wg(), total_tiles / 3072));
    const dim3 sgrid((unsigned) (((n_blocks + tpw - 1) / tpw) * m_blocks));
    // four results per store need every group of four columns of every output row 16-byte aligned
    const int vec_ok = ((uintptr_t) out % 16 == 0) && (ldo % 4 == 0);
    const int ind_mode = !mask_x ? 0 : (max_ones >= 1 && max_ones <= 4) ? max_ones : 5;   // additions unrolled up to four
#define GR_STREAM_K(KTYPE, TO, IND, KT_)                                                                               \
    hipLaunchKernelGGL((get_rows_dense_stream_kernel<KTYPE, TO, IND, KT_>), sgrid, block, 0, tsvm_s(stream), x, ldx, x_idx, n, d, \
                       sd_x, a, lda, a_idx, m, sd_a, kp, (TO *) out, out_slots, ldo, m_blocks, (unsigned) n_blocks, tpw, m_dev, \
                       mask_x, mask_a, max_ones, vec_ok)
#define GR_STREAM(KTYPE, TO, IND)                                                                                     \
    do {                                                                                                              \
        if (d <= 16) GR_STREAM_K(KTYPE, TO, IND, 1);                                                                  \
        else GR_STREAM_K(KTYPE, TO, IND, 2);                                                                          \
    } while (0)
#define GR_LAUNCH_T(KTYPE, TO)                                                                                        \
    do {                                                                                                              \
        if (ti == 2) {                                                                                                \
            switch (ind_mode) {                                                                                       \
                case 0:                                                                                               \
                    if (d > 32)                                                                                       \
                        hipLaunchKernelGGL((get_rows_dense_stream_kernel<KTYPE, TO, 0, 3>), sgrid, block, 0, tsvm_s(stream), x, ldx, \
                                           x_idx, n, d, sd_x, a, lda, a_idx, m, sd_a, kp, (TO *) out, out_slots, ldo, m_blocks, \
                                           (unsigned) n_blocks, tpw, m_dev, mask_x, mask_a, max_ones, vec_ok);        \
                    else GR_STREAM(KTYPE, TO, 0);                                                                     \
                    break;                                                                                            \
                case 1: GR_STREAM(KTYPE, TO, 1); break;                                                               \
                case 2: GR_STREAM(KTYPE, TO, 2); break;                                                               \
                case 3: GR_STREAM(KTYPE, TO, 3); break;                                                               \
                case 4: GR_STREAM(KTYPE, TO, 4); break;                                                               \
                default: GR_STREAM(KTYPE, TO, 5); break;                                                              \
            }                                                                                                         \
        } else                                                                                                        \
            hipLaunchKernelGGL((get_rows_dense_kernel<KTYPE, 4, TO>), grid, block, 0, tsvm_s(stream), x, ldx, x_idx, n, d, sd_x, \
                               a, lda, a_idx, m, sd_a, kp, (TO *) out, out_slots, ldo, m_blocks, m_dev);              \
    } while (0)
#define GR_LAUNCH(KTYPE)                                        \
    do {                                                        \
        if (row_type == TSVM_ROW_F32) GR_LAUNCH_T(KTYPE, float); \
        else GR_LAUNCH_T(KTYPE, double);                        \
    } while (0)
    switch (kernel_type) {
        case TSVM_LINEAR: GR_LAUNCH_T(TSVM_LINEAR, double); break;
        case TSVM_POLY: GR_LAUNCH(TSVM_POLY); break;
        case TSVM_SIGMOID: GR_LAUNCH(TSVM_SIGMOID); break;
        default: GR_LAUNCH(TSVM_RBF); break;
    }
#undef GR_LAUNCH
#undef GR_LAUNCH_T
#undef GR_STREAM
#undef GR_STREAM_K
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_get_rows_dense(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d, const double *sd_x, const double *a,
                        int64_t lda, const int *a_idx, int m, const double *sd_a, int kernel_type, double gamma,
                        double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                        tsvm_stream stream) {
    return get_rows_dense(x, ldx, x_idx, n, d, sd_x, a, lda, a_idx, m, nullptr, sd_a, kernel_type, gamma, coef0, degree, out,
                          row_type, out_slots, ldo, stream);
}

int tsvm_get_rows_dense_counted(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d, const double *sd_x,
                                const double *a, int64_t lda, const int *a_idx, int m_max, const int *m_dev,
                                const double *sd_a, int kernel_type, double gamma, double coef0, int degree, void *out,
                                int row_type, const int *out_slots, int64_t ldo, tsvm_stream stream) {
    TSVM_REQUIRE(m_dev, "tsvm_get_rows_dense_counted: null pointer");
    return get_rows_dense(x, ldx, x_idx, n, d, sd_x, a, lda, a_idx, m_max, m_dev, sd_a, kernel_type, gamma, coef0, degree, out,
                          row_type, out_slots, ldo, stream);
}

int tsvm_indicator_masks(const double *x, int64_t ld, int64_t n, int first_col, int n_cols, uint64_t *masks, int *max_ones,
                         tsvm_stream stream) {
    TSVM_REQUIRE(x && masks && max_ones && n >= 0, "tsvm_indicator_masks: bad argument");
    TSVM_REQUIRE(first_col >= 0 && n_cols >= 1 && n_cols <= 64 && first_col + n_cols <= ld,
                 "tsvm_indicator_masks: columns %d..%d outside the row (ld %lld) or more than 64", first_col, first_col + n_cols,
                 (long long) ld);
    hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(64), 0, tsvm_s(stream), max_ones, (int64_t) 1, 0);
    TSVM_LAUNCH_CHECK();
    if (n == 0) return 0;
    hipLaunchKernelGGL(indicator_masks_kernel, dim3(grid_for(n, 256)), dim3(256), 0, tsvm_s(stream), x, ld, n, first_col, n_cols,
                       masks, max_ones);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_get_rows_dense_indicator(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d_dense, const double *sd_x,
                                  const uint64_t *mask_x, const double *a, int64_t lda, const int *a_idx, int m, const int *m_dev,
                                  const double *sd_a, const uint64_t *mask_a, int max_ones, int kernel_type, double gamma,
                                  double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                                  tsvm_stream stream) {
    TSVM_REQUIRE(mask_x && mask_a, "tsvm_get_rows_dense_indicator: null mask");
    TSVM_REQUIRE(max_ones >= 0 && max_ones <= 64, "tsvm_get_rows_dense_indicator: max_ones %d outside [0, 64]", max_ones);
    return get_rows_dense(x, ldx, x_idx, n, d_dense, sd_x, a, lda, a_idx, m, m_dev, sd_a, kernel_type, gamma, coef0, degree, out,
                          row_type, out_slots, ldo, stream, mask_x, mask_a, max_ones);
}

int tsvm_csr_stage_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int m,
                        int n_features, double *w, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && w && m >= 0 && n_features >= 0, "tsvm_csr_stage_rows: bad argument");
    if (m == 0 || n_features == 0) return 0;
    hipLaunchKernelGGL(fill_f64_kernel, dim3(2048), dim3(256), 0, tsvm_s(stream), w, (int64_t) m * n_features, 0.0);
    TSVM_LAUNCH_CHECK();
    hipLaunchKernelGGL(csr_stage_rows_kernel<double>, dim3(grid_for((int64_t) m * 64, 256)), dim3(256), 0, tsvm_s(stream), val, col,
                       row_ptr, idx, m, n_features, w, 0);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_csr_scatter_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int m,
                          int n_features, void *w, int w_type, int clear, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && w && m >= 0 && n_features >= 0, "tsvm_csr_scatter_rows: bad argument");
    TSVM_REQUIRE(w_type == TSVM_ROW_F64 || w_type == TSVM_ROW_F32, "tsvm_csr_scatter_rows: unknown element type %d", w_type);
    if (m == 0 || n_features == 0) return 0;
    if (w_type == TSVM_ROW_F32)
        hipLaunchKernelGGL(csr_stage_rows_kernel<float>, dim3(grid_for((int64_t) m * 64, 256)), dim3(256), 0, tsvm_s(stream), val,
                           col, row_ptr, idx, m, n_features, (float *) w, clear);
    else
        hipLaunchKernelGGL(csr_stage_rows_kernel<double>, dim3(grid_for((int64_t) m * 64, 256)), dim3(256), 0, tsvm_s(stream), val,
                           col, row_ptr, idx, m, n_features, (double *) w, clear);
    TSVM_LAUNCH_CHECK();
    return 0;
}

static int get_rows_csr(const double *val, const int *col, const int64_t *row_ptr, const int *x_idx, int64_t n, const double *sd_x,
                        const void *w, int w_type, int m, const double *sd_w, int kernel_type, double gamma, double coef0,
                        int degree, void *out, int row_type, const int *out_slots, int64_t ldo, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && w && out, "tsvm_get_rows_csr: null pointer");
    TSVM_REQUIRE(w_type == TSVM_ROW_F64 || w_type == TSVM_ROW_F32, "tsvm_get_rows_csr: unknown staging type %d", w_type);
    TSVM_REQUIRE(n >= 0 && m >= 0 && ldo >= n, "tsvm_get_rows_csr: bad size");
    TSVM_REQUIRE(kernel_type >= 0 && kernel_type <= 4, "tsvm_get_rows_csr: unknown kernel type %d", kernel_type);
    TSVM_REQUIRE(row_type_ok(row_type, kernel_type), "tsvm_get_rows_csr: row type %d not valid for kernel type %d", row_type,
                 kernel_type);
    TSVM_REQUIRE((kernel_type != TSVM_RBF && kernel_type != TSVM_PRECOMPUTED) || (sd_x && sd_w),
                 "tsvm_get_rows_csr: RBF needs self dot products");
    if (n == 0 || m == 0) return 0;
    KernelParam kp{kernel_type, degree, gamma, coef0};
    const unsigned i_blocks = (unsigned) ((m + 255) / 256);
    const int jb = n <= 4096 ? 4 : 16;   // (32, whole 128-byte lines of float rows: 0.78 ms against 0.55 at 72,000 x 20,958)
    const int64_t j_blocks = (n + jb - 1) / jb;
    TSVM_REQUIRE(j_blocks * i_blocks < (int64_t) 0x7fffffff, "tsvm_get_rows_csr: grid too large");
    const dim3 grid((unsigned) (j_blocks * i_blocks));
    // 16-byte pieces of an output row: every row start and every group of jb columns 16-byte aligned
    const int vec_ok = (uintptr_t) out % 16 == 0 && (ldo * (row_type == TSVM_ROW_F32 ? 4 : 8)) % 16 == 0;
#define CSR_LAUNCH_W(TO, JB, TW)                                                                                             \
    hipLaunchKernelGGL((get_rows_csr_kernel<TO, JB, TW>), grid, dim3(256), 0, tsvm_s(stream), val, col, row_ptr, x_idx, n, sd_x, \
                       (const TW *) w, m, sd_w, kp, (TO *) out, out_slots, ldo, i_blocks, vec_ok)
#define CSR_LAUNCH(TO, JB)                                                   \
    do {                                                                     \
        if (w_type == TSVM_ROW_F32) CSR_LAUNCH_W(TO, JB, float);             \
        else CSR_LAUNCH_W(TO, JB, double);                                   \
    } while (0)
    if (row_type == TSVM_ROW_F32) {
        if (jb == 4) CSR_LAUNCH(float, 4); else CSR_LAUNCH(float, 16);
    } else {
        if (jb == 4) CSR_LAUNCH(double, 4); else CSR_LAUNCH(double, 16);
    }
#undef CSR_LAUNCH
#undef CSR_LAUNCH_W
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_get_rows_csr(const double *val, const int *col, const int64_t *row_ptr, const int *x_idx, int64_t n, const double *sd_x,
                      const double *w, int m, const double *sd_w, int kernel_type, double gamma, double coef0,
                      int degree, void *out, int row_type, const int *out_slots, int64_t ldo, tsvm_stream stream) {
    return get_rows_csr(val, col, row_ptr, x_idx, n, sd_x, w, TSVM_ROW_F64, m, sd_w, kernel_type, gamma, coef0, degree, out, row_type,
                        out_slots, ldo, stream);
}

int tsvm_get_rows_csr_staged(const double *val, const int *col, const int64_t *row_ptr, const int *x_idx, int64_t n,
                             const double *sd_x, const void *w, int w_type, int m, const double *sd_w, int kernel_type,
                             double gamma, double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                             tsvm_stream stream) {
    return get_rows_csr(val, col, row_ptr, x_idx, n, sd_x, w, w_type, m, sd_w, kernel_type, gamma, coef0, degree, out, row_type,
                        out_slots, ldo, stream);
}

int tsvm_csr_slice_widths(const int64_t *row_ptr, int64_t n, int *widths, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && widths && n >= 0, "tsvm_csr_slice_widths: bad argument");
    if (n == 0) return 0;
    hipLaunchKernelGGL(csr_slice_widths_kernel, dim3(grid_for(n, 64)), dim3(64), 0, tsvm_s(stream), row_ptr, n, widths);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_csr_to_sliced(const double *val, const int *col, const int64_t *row_ptr, int64_t n, const int64_t *slice_ptr, int pad_col,
                       int *ell_col, void *ell_val, int val_type, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && slice_ptr && ell_col && ell_val && n >= 0, "tsvm_csr_to_sliced: bad argument");
    TSVM_REQUIRE(val_type == TSVM_ROW_F64 || val_type == TSVM_ROW_F32, "tsvm_csr_to_sliced: unknown value type %d", val_type);
    if (n == 0) return 0;
    const dim3 grid(grid_for(n, 64)), block(256);
    if (val_type == TSVM_ROW_F32)
        hipLaunchKernelGGL(csr_slice_fill_kernel<float>, grid, block, 0, tsvm_s(stream), val, col, row_ptr, n, slice_ptr, pad_col, ell_col,
                           (float *) ell_val);
    else
        hipLaunchKernelGGL(csr_slice_fill_kernel<double>, grid, block, 0, tsvm_s(stream), val, col, row_ptr, n, slice_ptr, pad_col, ell_col,
                           (double *) ell_val);
    TSVM_LAUNCH_CHECK();
    return 0;
}

size_t tsvm_get_rows_csr_sliced_lds(int n_features, int max_row_nnz, int val_type) {
    (void) val_type;
    if (n_features < 1 || max_row_nnz < 0) return 0;
    const SlicedLds l = sliced_lds(n_features);
    // half a block of the longest rows has to fit the tile (whole blocks that do not are done in two halves)
    if ((int64_t) l.slot_cap < std::min<int64_t>((int64_t) (SL_IB / 2) * std::max(max_row_nnz, 1), (int64_t) n_features)) return 0;
    return l.total;
}

int tsvm_get_rows_csr_sliced(const int *ell_col, const void *ell_val, int val_type, const int64_t *slice_ptr, int64_t n,
                             const double *sd_x, const double *a_val, const int *a_col, const int64_t *a_ptr, const int *a_idx,
                             int m, const double *sd_a, int n_features, int max_row_nnz, int kernel_type, double gamma,
                             double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                             tsvm_stream stream) {
    TSVM_REQUIRE(ell_col && ell_val && slice_ptr && a_col && a_val && a_ptr && out, "tsvm_get_rows_csr_sliced: null pointer");
    TSVM_REQUIRE(val_type == TSVM_ROW_F64 || val_type == TSVM_ROW_F32, "tsvm_get_rows_csr_sliced: unknown value type %d", val_type);
    TSVM_REQUIRE(n >= 0 && m >= 0 && ldo >= n && n_features >= 1, "tsvm_get_rows_csr_sliced: bad size");
    TSVM_REQUIRE(kernel_type >= 0 && kernel_type <= 4, "tsvm_get_rows_csr_sliced: unknown kernel type %d", kernel_type);
    TSVM_REQUIRE(row_type_ok(row_type, kernel_type), "tsvm_get_rows_csr_sliced: row type %d not valid for kernel type %d", row_type,
                 kernel_type);
    TSVM_REQUIRE((kernel_type != TSVM_RBF && kernel_type != TSVM_PRECOMPUTED) || (sd_x && sd_a),
                 "tsvm_get_rows_csr_sliced: RBF needs self dot products");
    const size_t lds_bytes = tsvm_get_rows_csr_sliced_lds(n_features, max_row_nnz, val_type);
    TSVM_REQUIRE(lds_bytes > 0, "tsvm_get_rows_csr_sliced: %d features with rows of up to %d entries do not fit the LDS", n_features,
                 max_row_nnz);
    if (n == 0 || m == 0) return 0;
    KernelParam kp{kernel_type, degree, gamma, coef0};
    const SlicedLds l = sliced_lds(n_features);
    const unsigned n_ib = (unsigned) ((m + SL_IB - 1) / SL_IB);
    // a workgroup takes `steps` runs of 1024 stored rows: enough workgroups for three rounds of the chip, few enough
    // that building the tile (once per workgroup) stays a small part
    const int64_t runs = (n + SL_T - 1) / SL_T;
    const int steps = (int) std::max<int64_t>(1, std::min<int64_t>(8, runs * n_ib / 768));
    const int64_t chunks = (runs + steps - 1) / steps;
    TSVM_REQUIRE(chunks * n_ib < (int64_t) 0x7fffffff, "tsvm_get_rows_csr_sliced: grid too large");
    const dim3 grid((unsigned) (chunks * n_ib)), block(SL_T);
#define SL_LAUNCH_K(KTYPE, TO, TV)                                                                                           \
    do {                                                                                                                     \
        static bool opted_ = false;                                                                                          \
        if (!opted_) {                                                                                                       \
            TSVM_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(get_rows_csr_sliced_kernel<KTYPE, TO, TV>),          \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, SL_LDS_BUDGET));                        \
            opted_ = true;                                                                                                   \
        }                                                                                                                    \
        hipLaunchKernelGGL((get_rows_csr_sliced_kernel<KTYPE, TO, TV>), grid, block, l.total, tsvm_s(stream), ell_col,       \
                           (const TV *) ell_val, slice_ptr, n, sd_x, a_val, a_col, a_ptr, a_idx, m, sd_a, n_features, l.slot_cap, kp, \
                           (TO *) out, out_slots, ldo, n_ib, steps, l.remap, l.bits, l.base);                                \
    } while (0)
#define SL_LAUNCH(TO, TV)                                              \
    do {                                                               \
        switch (kernel_type) {                                         \
            case TSVM_LINEAR: SL_LAUNCH_K(TSVM_LINEAR, double, TV); break; \
            case TSVM_POLY: SL_LAUNCH_K(TSVM_POLY, TO, TV); break;     \
            case TSVM_SIGMOID: SL_LAUNCH_K(TSVM_SIGMOID, TO, TV); break; \
            default: SL_LAUNCH_K(TSVM_RBF, TO, TV); break;             \
        }                                                              \
    } while (0)
    if (row_type == TSVM_ROW_F32) {
        if (val_type == TSVM_ROW_F32) SL_LAUNCH(float, float); else SL_LAUNCH(float, double);
    } else {
        if (val_type == TSVM_ROW_F32) SL_LAUNCH(double, float); else SL_LAUNCH(double, double);
    }
#undef SL_LAUNCH_K
#undef SL_LAUNCH
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_gather_rows_f64(const double *x, int64_t ld, const int *idx, int64_t m, double *out, tsvm_stream stream) {
    TSVM_REQUIRE(x && idx && out && m >= 0 && ld > 0 && ld % 4 == 0, "tsvm_gather_rows_f64: bad argument");
    TSVM_REQUIRE(((uintptr_t) x % 32 == 0) && ((uintptr_t) out % 32 == 0), "tsvm_gather_rows_f64: x and out must be 32-byte aligned");
    if (m == 0) return 0;
    const int64_t total = m * (ld / 4);
    const unsigned grid = (unsigned) std::min<int64_t>((total + 255) / 256, 65536);
    hipLaunchKernelGGL(gather_rows_f64_kernel, dim3(grid), dim3(256), 0, tsvm_s(stream), (const v4d *) x, ld / 4, idx, m, (v4d *) out);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_csr_gather_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int64_t m,
                         const int64_t *out_ptr, double *out_val, int *out_col, tsvm_stream stream) {
    TSVM_REQUIRE(row_ptr && idx && out_ptr && m >= 0, "tsvm_csr_gather_rows: bad argument");
    if (m == 0) return 0;
    hipLaunchKernelGGL(csr_gather_rows_kernel, dim3(grid_for(m * 64, 256)), dim3(256), 0, tsvm_s(stream), val, col, row_ptr, idx,
                       m, out_ptr, out_val, out_col);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_fold_ids(const int *ids, int count, int period, int *out, tsvm_stream stream) {
    TSVM_REQUIRE(ids && out && count >= 0 && period > 0, "tsvm_fold_ids: bad argument");
    if (count == 0) return 0;
    hipLaunchKernelGGL(fold_ids_kernel, dim3(grid_for(count, 256)), dim3(256), 0, tsvm_s(stream), ids, count, period, out);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_column_stats_dense(const double *x, int64_t ld, int64_t n, int d, int *counts, tsvm_stream stream) {
    TSVM_REQUIRE(x && counts && n >= 0 && d >= 0 && d <= ld, "tsvm_column_stats_dense: bad argument");
    if (d == 0) return 0;
    hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(2 * (int64_t) d, 256)), dim3(256), 0, tsvm_s(stream), counts, 2 * (int64_t) d, 0);
    TSVM_LAUNCH_CHECK();
    if (n == 0) return 0;
    const unsigned grid = (unsigned) std::min<int64_t>((n + 63) / 64, 2048);
    hipLaunchKernelGGL(column_stats_dense_kernel, dim3(grid), dim3(256), 0, tsvm_s(stream), x, ld, n, d, counts);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_column_stats_csr(const double *val, const int *col, int64_t nnz, int d, int *counts, tsvm_stream stream) {
    TSVM_REQUIRE(counts && nnz >= 0 && d >= 0 && (nnz == 0 || (val && col)), "tsvm_column_stats_csr: bad argument");
    if (d == 0) return 0;
    hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(2 * (int64_t) d, 256)), dim3(256), 0, tsvm_s(stream), counts, 2 * (int64_t) d, 0);
    TSVM_LAUNCH_CHECK();
    if (nnz == 0) return 0;
    const unsigned grid = (unsigned) std::min<int64_t>((nnz + 255) / 256, 4096);
    hipLaunchKernelGGL(column_stats_csr_kernel, dim3(grid), dim3(256), 0, tsvm_s(stream), val, col, nnz, d, counts);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_gather_f64(const double *in, const int *idx, int m, double *out, tsvm_stream stream) {
    TSVM_REQUIRE(in && idx && out && m >= 0, "tsvm_gather_f64: bad argument");
    if (m == 0) return 0;
    hipLaunchKernelGGL(gather_f64_kernel, dim3(grid_for(m, 256)), dim3(256), 0, tsvm_s(stream), in, idx, m, out);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_sum_kernel_values(const double *coef, int total_sv, const int *sv_start, const int *sv_count,
                           const double *rho, const void *k_mat, int row_type, int64_t ldk, double *dec_values,
                           int n_classes, int64_t n_instances, tsvm_stream stream) {
    TSVM_REQUIRE(sv_start && sv_count && rho && dec_values, "tsvm_sum_kernel_values: null pointer");
    TSVM_REQUIRE(n_classes >= 2 && n_classes <= 32768, "tsvm_sum_kernel_values: n_classes %d outside [2, 32768]", n_classes);
    TSVM_REQUIRE(total_sv >= 0 && ldk >= total_sv && n_instances >= 0, "tsvm_sum_kernel_values: bad size");
    TSVM_REQUIRE(row_type == TSVM_ROW_F64 || row_type == TSVM_ROW_F32, "tsvm_sum_kernel_values: unknown row type %d", row_type);
    if (n_instances == 0) return 0;
    const size_t shm = 0;
    if (row_type == TSVM_ROW_F32)
        hipLaunchKernelGGL(sum_kernel_values_kernel<float>, dim3(grid_for(n_instances, SK_R)), dim3(SK_T), shm, tsvm_s(stream),
                           coef, total_sv, sv_start, sv_count, rho, (const float *) k_mat, ldk, dec_values, n_classes,
                           n_instances);
    else
        hipLaunchKernelGGL(sum_kernel_values_kernel<double>, dim3(grid_for(n_instances, SK_R)), dim3(SK_T), shm, tsvm_s(stream),
                           coef, total_sv, sv_start, sv_count, rho, (const double *) k_mat, ldk, dec_values, n_classes,
                           n_instances);
    TSVM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
