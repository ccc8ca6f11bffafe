// The dense kernel-row tile: one (32*TI) x 128 block of epilogue(A . X^T) on the fp64 matrix cores, shared by the
// get_rows kernels and the fused prediction kernel.
#pragma once
#include "tsvm_device.h"

typedef double v4d __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------------------------
// Dense get_rows: fp64 MFMA tiled GEMM  out = epilogue(A_ws . X^T)
//
// v_mfma_f64_16x16x4f64 accumulates its four k-slots as a chain of fused multiply-adds in
// ascending slot order, so feeding k-slots in ascending column order reproduces, bit for bit, the
// serial  acc = fma(a[k], x[k], acc), k = 0..d-1  dot product.
//
// Operand layout of the instruction (64 lanes): A lane l holds A[row l%16][k l/16], B lane l
// holds B[k l/16][col l%16], D register v of lane l holds D[row 4v + l/16][col l%16].
// Working-set rows are the A operand (D rows), all-rows X is the B operand (D columns), so the 16
// lanes l%16 of one store cover 16 consecutive j: a 128-byte run of an output row.
//
// Workgroup = 256 threads = 4 wavefronts in a 2x2 grid; each wavefront owns a (16*TI)x64 block of the
// (32*TI)x128 output tile as TIx4 MFMA tiles (16*TI accumulator doubles per lane).  K is walked in tiles
// of 8 or 16 columns staged through LDS in k-major order, with the next tile's global loads in flight
// in registers while the current one is multiplied.
// ------------------------------------------------------------------------------------------------
#define GR_BN 128

// KT: kernel type (compile-time so that only one epilogue is instantiated); TI: 16-row MFMA tiles
// per wavefront in the working-row direction.  Two shapes are used:
//   TI = 4, K tile 8:  128x128 workgroup tile, 2 wavefronts per SIMD (large d, MFMA-bound);
//   TI = 2, K tile 16: 64x128 workgroup tile, half the accumulators, 3 wavefronts per SIMD (small d,
//                      where the epilogue and the stores weigh as much as the MFMAs).
// Either way a wavefront issues 32 MFMAs between two barriers.  LDS tiles are k-major [KTILE][LS];
// LS (130 / 129 doubles) makes the staging writes and the operand reads bank-conflict free.
// TO: element type of the output rows.  The RBF / polynomial / sigmoid values are float-rounded by
// definition (kernelmatrix_kernel.cpp:77-108 calls expf / powf / tanhf), so storing them as float
// loses nothing and halves the bytes written here and read back by update_f.
template <int TI> struct GrShape {
    static constexpr int BM = 32 * TI;
    static constexpr int KTILE = TI == 2 ? 16 : 8;
    static constexpr int LS = TI == 2 ? 129 : 130;
    static constexpr int LDS_DOUBLES = KTILE * LS;   // per operand
};

// One (32*TI) x 128 output tile at rows i0.., columns j0..; As / Bs hold GrShape<TI>::LDS_DOUBLES doubles each.
// SYM: the output is a symmetric matrix (same rows on both sides, out[i][j] at i*ldo + j): every value is also
// written to its mirror position, so that tiles below the diagonal need no workgroup.  kappa(a, b) and kappa(b, a)
// are the same bits: the products of the dot product commute, their order does not change, and the self dot
// products enter as a commutative sum.
//
// FUSE: prediction.  The tile's values are not stored: each is multiplied by its column's fz_nc coefficients
// (fz_coef[column * fz_nc + c], columns counted before x_idx maps them to rows of x) and the products are summed
// over the tile's columns into fz_red[(wj * BM + row) * fz_nc + c] in LDS, wj = 0, 1 being the two wavefront
// columns of the workgroup (each location has exactly one writer, so tiles called one after the other accumulate
// without atomics).  n must be a multiple of 128 and x_idx given; rows beyond m produce sums nobody reads.
template <int KT, int TI, typename TO, bool SYM = false, bool FUSE = false>
__device__ __forceinline__ void get_rows_tile(
    const double *__restrict__ x, int64_t ldx, const int *__restrict__ x_idx, int64_t n, int d,
    const double *__restrict__ sd_x, const double *__restrict__ a, int64_t lda, const int *__restrict__ a_idx, int m,
    const double *__restrict__ sd_a, KernelParam kp_in, TO *__restrict__ out, const int *__restrict__ out_slots,
    int64_t ldo, int i0, int j0, double *__restrict__ As, double *__restrict__ Bs, const uint64_t *__restrict__ exp_tab,
    const double *__restrict__ fz_coef = nullptr, int fz_nc = 0, double *__restrict__ fz_red = nullptr) {
    constexpr int BM = GrShape<TI>::BM;
    constexpr int KTILE = GrShape<TI>::KTILE;
    constexpr int LS = GrShape<TI>::LS;
    constexpr int A_TPR = 256 / BM;           // threads per A row
    constexpr int A_VEC = KTILE / 4 / A_TPR;  // 4-double vectors per thread for the A tile
    constexpr int B_VEC = KTILE / 8;          // 4-double vectors per thread for the B tile (2 threads per row)
    KernelParam kp = kp_in;
    kp.kernel_type = KT;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wi = wave >> 1, wj = wave & 1;
    const int n_last = (int) n - 1, m_last = m - 1;

    // Staging assignment.  Rows beyond the tile's valid range are clamped to the last valid row: what they
    // stage only reaches outputs that are never stored, and every load stays unconditional.  (Any VALU
    // instruction, a zero fill included, is issued at the expense of another wavefront's fp64 MFMA.)
    const int a_row = tid / A_TPR, a_k = (tid % A_TPR) * (4 * A_VEC);
    const int b_row = tid >> 1, b_k = (tid & 1) * (4 * B_VEC);
    // Per-row / per-column data of the epilogue (self dot products, output row offsets).  Everything that goes
    // through an index array is fetched in two batches of independent loads (all indices, then all values),
    // ahead of the K loop, instead of one dependent pair after the other.
    const int lrow = lane & 15;
    const int lk = lane >> 4;
    const int jb = j0 + wj * 64 + lrow;
    const bool full = (i0 + BM <= m) && (j0 + GR_BN <= (int) n);
    int a_r = min(i0 + a_row, m_last), x_r = min(j0 + b_row, n_last);   // staged rows
    int jr[4], ir[TI * 4], slot[TI * 4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) jr[tj] = min(jb + tj * 16, n_last);
#pragma unroll
    for (int u = 0; u < TI * 4; ++u) ir[u] = slot[u] = min(i0 + wi * (16 * TI) + (u >> 2) * 16 + 4 * (u & 3) + lk, m_last);
    if (out_slots) {
#pragma unroll
        for (int u = 0; u < TI * 4; ++u) slot[u] = out_slots[slot[u]];
    }
    if (a_idx) {
        a_r = a_idx[a_r];
#pragma unroll
        for (int u = 0; u < TI * 4; ++u) ir[u] = a_idx[ir[u]];
    }
    if (x_idx) {
        x_r = x_idx[x_r];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) jr[tj] = x_idx[jr[tj]];
    }
    const double *a_ptr = a + (uint64_t) (uint32_t) a_r * (uint32_t) lda;   // first column of this thread's rows
    const double *x_ptr = x + (uint64_t) (uint32_t) x_r * (uint32_t) ldx;
    double sdj[4], sdi[TI * 4];
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) sdj[tj] = 0.0;
#pragma unroll
    for (int u = 0; u < TI * 4; ++u) sdi[u] = 0.0;
    if (sd_x) {
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) sdj[tj] = sd_x[jr[tj]];
    }
    if (sd_a) {
#pragma unroll
        for (int u = 0; u < TI * 4; ++u) sdi[u] = sd_a[ir[u]];
    }
    int64_t orow_off[TI * 4];
#pragma unroll
    for (int u = 0; u < TI * 4; ++u) orow_off[u] = (int64_t) ((uint64_t) (uint32_t) slot[u] * (uint32_t) ldo);

    v4d acc[TI][4];
#pragma unroll
    for (int ti = 0; ti < TI; ++ti)
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) acc[ti][tj] = (v4d){0.0, 0.0, 0.0, 0.0};

    // Rows are padded with zeros up to ldx / lda (multiples of 8).  An 8-column tile therefore always lies
    // inside the padded row.  The last 16-column tile may reach past it: its vectors that would start beyond
    // the row re-read the row's last four columns instead; they are staged but never multiplied (n_ks below).
    const int n_kt = (d + KTILE - 1) / KTILE;
    v4d ra[A_VEC], rb[B_VEC];
    auto load_tile = [&](int kt) {
        const int k0 = kt * KTILE;
#pragma unroll
        for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (a_ptr + (k0 + a_k + 4 * q));
#pragma unroll
        for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (x_ptr + (k0 + b_k + 4 * q));
    };
    auto load_last_tile = [&](int kt) {
        const int k0 = kt * KTILE;
#pragma unroll
        for (int q = 0; q < A_VEC; ++q) ra[q] = *(const v4d *) (a_ptr + min(k0 + a_k + 4 * q, (int) lda - 4));
#pragma unroll
        for (int q = 0; q < B_VEC; ++q) rb[q] = *(const v4d *) (x_ptr + min(k0 + b_k + 4 * q, (int) ldx - 4));
    };
    auto stage_tile = [&]() {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
            for (int q = 0; q < A_VEC; ++q) As[(a_k + 4 * q + e) * LS + a_row] = ra[q][e];
#pragma unroll
            for (int q = 0; q < B_VEC; ++q) Bs[(b_k + 4 * q + e) * LS + b_row] = rb[q][e];
        }
    };
    auto mma_step = [&](int ks) {   // four columns of the staged tile
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
        if (KTILE == 8 || n_kt > 1) load_tile(0);
        else load_last_tile(0);
        // every tile but the last is whole
        for (int kt = 0; kt + 1 < n_kt; ++kt) {
            stage_tile();
            __syncthreads();
            if (KTILE == 8 || kt + 2 < n_kt) load_tile(kt + 1);
            else load_last_tile(kt + 1);
#pragma unroll
            for (int ks = 0; ks < KTILE / 4; ++ks) mma_step(ks);
            __syncthreads();
        }
        stage_tile();
        __syncthreads();
        const int n_ks = (d - (n_kt - 1) * KTILE + 3) / 4;   // groups of four columns left, 1 .. KTILE / 4
#pragma unroll
        for (int ks = 0; ks < KTILE / 4; ++ks)
            if (KTILE == 8 || ks < n_ks) mma_step(ks);       // 8-column tiles are always whole (rows are padded to 8)
    }

    if constexpr (FUSE) {
        // the kernel values take the accumulators' place (widened to double, as the reference widens them before
        // its sums, kernelmatrix_kernel.cpp:110-147) ...
#pragma unroll
        for (int ti = 0; ti < TI; ++ti)
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int tj = 0; tj < 4; ++tj)
                    acc[ti][tj][v] = tsvm_epilogue(acc[ti][tj][v], sdi[ti * 4 + v], sdj[tj], kp, exp_tab);
        // ... and every coefficient row takes its share: four columns per lane, then the sixteen lanes that hold
        // the same rows (a DPP row)
        for (int c = 0; c < fz_nc; ++c) {
            double cj[4];
#pragma unroll
            for (int tj = 0; tj < 4; ++tj) cj[tj] = fz_coef[(int64_t) (jb + tj * 16) * fz_nc + c];
#pragma unroll
            for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    double p = cj[0] * acc[ti][0][v];
#pragma unroll
                    for (int tj = 1; tj < 4; ++tj) p = __builtin_fma(cj[tj], acc[ti][tj][v], p);
                    p = dpp_row_sum_f64(p);
                    if (lrow == 0) {
                        double *r = fz_red + ((wj * BM + wi * (16 * TI) + ti * 16 + 4 * v + lk) * fz_nc + c);
                        *r += p;
                    }
                }
            }
        }
        return;
    }
    // epilogue + store.  Interior tiles take the unguarded path; edge tiles test every element.
    // (Sixteen lanes write 64 or 128 consecutive bytes of an output row: streamed past the L2 when those runs are
    // whole 64-byte pieces of memory, which depends on where the rows start; partial pieces the L2 has to merge.)
    const bool stream_out = !SYM && ((ldo * (int64_t) sizeof(TO)) % 64 == 0) && ((uintptr_t) out % 64 == 0);
    if (full) {
#pragma unroll
        for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                TO *orow = out + orow_off[ti * 4 + v] + jb;
#pragma unroll
                for (int tj = 0; tj < 4; ++tj) {
                    const TO val = tsvm_epilogue_as<TO>(acc[ti][tj][v], sdi[ti * 4 + v], sdj[tj], kp, exp_tab);
                    if (SYM) {   // the solver's block: read again at once
                        orow[tj * 16] = val;
                        out[(int64_t) (jb + tj * 16) * ldo + (i0 + wi * (16 * TI) + ti * 16 + 4 * v + lk)] = val;
                    } else if (stream_out) {
                        store_streaming(orow + tj * 16, val);
                    } else {
                        orow[tj * 16] = val;
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int ti = 0; ti < TI; ++ti) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int i = i0 + wi * (16 * TI) + ti * 16 + 4 * v + lk;
                if (i >= m) continue;
                TO *orow = out + orow_off[ti * 4 + v] + jb;
#pragma unroll
                for (int tj = 0; tj < 4; ++tj)
                    if (jb + tj * 16 < n) {
                        const TO val = tsvm_epilogue_as<TO>(acc[ti][tj][v], sdi[ti * 4 + v], sdj[tj], kp, exp_tab);
                        if (SYM) {
                            orow[tj * 16] = val;
                            out[(int64_t) (jb + tj * 16) * ldo + i] = val;
                        } else {
                            orow[tj * 16] = val;
                        }
                    }
            }
        }
    }
}
