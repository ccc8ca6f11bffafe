// The local SMO solvers: c_smo_solve / nu_smo_solve (src/thundersvm/kernel/smo_kernel.cpp:12-287,
// USE_CUDA=OFF semantics) as one LDS-resident workgroup on gfx950.
//
// Shape of the kernel.  One workgroup of 256 threads (one wavefront per SIMD of the CU) holds the
// whole working set: element t = tid*E + e lives in register slot e of thread tid (E = ws/256
// slots, up to 4: a thread's elements are neighbours, so its share of a block row is one load) with its f and diagonal; alpha lives in LDS (only two entries change per
// iteration) and the I_up / I_low membership of a thread's elements is a bit field in one register.
// One inner iteration is
//   1. (i, up) = first argmin of f over I_up and low = max of f over I_low: a per-thread scan of
//      its E slots, a DPP reduction inside each wavefront, four partial results through LDS;
//   2. row K[i, .] of the gathered ws x ws block (coalesced);
//   3. j2 = first argmin of -b^2/a over I_low with f > up: same reduction shape;
//   4. the two-variable step, row K[j2, .], f -= l * (K[j2, .] - K[i, .]).
// Two workgroup barriers per iteration.  With one wavefront per SIMD nothing hides an instruction's
// issue slot or a taken branch, so the loop body is bound by its instruction count: it is written
// with selects instead of branches (the same loop with if-blocks measured about 1.3x slower), with
// v_min_f64 / v_max_f64 for the value reductions, and with everything that concerns only the two
// chosen elements (their alpha, their set membership) computed once per thread from LDS rather than
// per element.  Reductions are lexicographic (value, element index) minima, so ties go to the lowest
// index exactly as the reference's serial loops resolve them, and all arithmetic is the reference's
// expression order in IEEE double (the library is compiled with -ffp-contract=off; the one fused
// operation, f -= l*(kJ - kI), is an explicit fma as gcc -O3 contracts it on an FMA host, and
// kd_i + kd_t - 2*K_it is written as fma(-2, K_it, kd_i + kd_t), which rounds identically because
// the product by 2 is exact).
#include "../../include/thundersvm_amd.h"
#include "tsvm_device.h"
#include "tsvm_internal.h"

#include <map>
#include <mutex>
#include <utility>

#define TSVM_INF __builtin_inf()
#define MAX_WS 1024
#define SV_T 256           // threads of the solver workgroup
#define SV_W (SV_T / 64)   // wavefronts

// kws[r*ldk + t] = K_r[working_set[t]] for t < ws, 0 for ws <= t < ldk: the ws x ws block the solver
// reads, gathered once per call so that the two row reads per inner iteration
// (smo_kernel.cpp:50-52,107-110) are contiguous; rows are padded to the solver's thread x slot grid
// so every thread can load without a bounds test.
// TB: element type of the block.  Float kernel rows give a float block: the same values in half the bytes, widened
// again when the solver loads them.
template <typename TK, typename TB>
__global__ void gather_ws_block_kernel(const TK *__restrict__ k_rows, const int *__restrict__ slots, int64_t ld,
                                       const int *__restrict__ working_set, int ws, int ldk, TB *__restrict__ kws) {
    const int r = blockIdx.x;
    const TK *row = k_rows + (int64_t) (slots ? slots[r] : r) * ld;
    for (int t = threadIdx.x; t < ldk; t += blockDim.x) kws[(int64_t) r * ldk + t] = t < ws ? (TB) row[working_set[t]] : (TB) 0;
}

// The same block when a table names the slot of every instance's row (a row cache that holds them all): row r
// is the one of instance ids[r]; its slot is also written to slots_out[r], for update_f.
template <typename TK, typename TB>
__global__ void gather_ws_block_by_id_kernel(const TK *__restrict__ k_rows, const int *__restrict__ slot_of_id, int64_t ld,
                                             const int *__restrict__ ids, int ws, int ldk, TB *__restrict__ kws,
                                             int *__restrict__ slots_out) {
    const int r = blockIdx.x;
    const int slot = slot_of_id[ids[r]];
    if (threadIdx.x == 0) slots_out[r] = slot;
    const TK *row = k_rows + (int64_t) slot * ld;
    for (int t = threadIdx.x; t < ldk; t += blockDim.x) kws[(int64_t) r * ldk + t] = t < ws ? (TB) row[ids[t]] : (TB) 0;
}

// Slots for a working set's new rows when the row store has a slot for every instance (nothing is ever
// evicted, so the bookkeeping needs no host): instances seen for the first time take the next free slots in the
// order of the list.  One workgroup; ids_new are distinct.
//   slot_of_id[i]  slot of instance i's row, -1 while it has none           (updated)
//   state[0]       slots in use                                              (updated)
//   state[1]       number of rows to compute for this working set            (written)
//   miss_ids / miss_slots [0 .. state[1])  the instances to compute and where their rows go
//   slots_ws[t]    slot of ids_ws[t], t < ws
//   info[0..1]     state[1], state[0] for the host (pinned host memory or device memory)
#define RA_T 1024
__global__ __launch_bounds__(RA_T) void row_slots_assign_kernel(const int *__restrict__ ids_new, int n_new,
                                                                int *__restrict__ slot_of_id, int *__restrict__ state,
                                                                int *__restrict__ miss_ids, int *__restrict__ miss_slots,
                                                                const int *__restrict__ ids_ws, int ws, int *__restrict__ slots_ws,
                                                                int *__restrict__ info) {
    __shared__ int wave_total[RA_T / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int id = tid < n_new ? ids_new[tid] : 0;
    const bool miss = tid < n_new && slot_of_id[id] < 0;
    const unsigned long long b = __ballot(miss);
    const int before = __popcll(b & ((1ull << lane) - 1ull));
    if (lane == 0) wave_total[wave] = __popcll(b);
    __syncthreads();
    int rank = before, total = 0;
    for (int w = 0; w < RA_T / 64; ++w) {
        const int c = wave_total[w];
        if (w < wave) rank += c;
        total += c;
    }
    const int base = state[0];
    if (miss) {
        slot_of_id[id] = base + rank;
        miss_ids[rank] = id;
        miss_slots[rank] = base + rank;
    }
    __syncthreads();   // the table's new entries are read back below by other threads of this workgroup
    if (tid == 0) {
        state[0] = base + total;
        state[1] = total;
        info[0] = total;
        info[1] = base + total;
    }
    if (tid < ws) slots_ws[tid] = slot_of_id[ids_ws[tid]];
}

// Cross-wavefront combination of the per-wavefront (value, index) minima held in LDS.
__device__ __forceinline__ void block_argmin(const double *s_v, const int *s_i, double &v, int &i, int none) {
    double m = s_v[0];
#pragma unroll
    for (int w = 1; w < SV_W; ++w) m = fmin_f64(m, s_v[w]);
    int r = none;
#pragma unroll
    for (int w = 0; w < SV_W; ++w) r = imin_sel(r, s_v[w] == m ? s_i[w] : none);
    v = m;
    i = r;
}
__device__ __forceinline__ double block_max(const double *s_v) {
    double v = s_v[0];
#pragma unroll
    for (int w = 1; w < SV_W; ++w) v = fmax_f64(v, s_v[w]);
    return v;
}

// The wavefront's lexicographic minimum of the candidates x[e] (element index e*256 + tid):
// value pass, then the smallest element index among those equal to the minimum.  (Taking the index
// from ballots of x[e] == minimum on the scalar unit instead measured slightly slower.)
template <int E>
__device__ __forceinline__ void wave_first_argmin(const double (&x)[E], int tid, double &v, int &idx) {
    double m = x[0];
#pragma unroll
    for (int e = 1; e < E; ++e) m = fmin_f64(m, x[e]);
    m = wave_min_f64(m);
    int r = MAX_WS;
#pragma unroll
    for (int e = E - 1; e >= 0; --e) r = x[e] == m ? tid * E + e : r;
    idx = wave_min_i32(r);
    v = m;
}

// Replaces the `width` membership bits of element t in the bit field of the thread that owns it.
template <int E>
__device__ __forceinline__ unsigned set_member_bits(unsigned m, int tid, int t, unsigned bits, int width) {
    const int sh = (t % E) * width;
    const unsigned field = ((1u << width) - 1u) << sh;
    return tid == t / E ? ((m & ~field) | (bits << sh)) : m;
}

// A thread's E consecutive elements of a block row: one 4E- or 8E-byte load, widened to double.
template <int E, typename TB>
__device__ __forceinline__ void load_row_elems(const TB *__restrict__ row, int tid, double (&out)[E]) {
    if constexpr (E == 1) {
        out[0] = (double) row[tid];
    } else {
        typedef TB vec_t __attribute__((ext_vector_type(E)));
        const vec_t v = *(const vec_t *) (row + tid * E);
#pragma unroll
        for (int e = 0; e < E; ++e) out[e] = (double) v[e];
    }
}

// Each wavefront knows its own best candidate a barrier and an LDS round trip before the workgroup
// knows the winner, and the winner is always one of the four.  One load per lane, 128 bytes apart,
// touches every cache line of a candidate's row, so the row the workgroup then reads is already
// on its way into the CU's L1 / the XCD's L2 (the four candidates' rows of a float block, 4 KB each, fit the L1 together).
// A wavefront without a candidate reports an index
// that may lie beyond the block's ws rows (an inactive element or MAX_WS): it touches row 0 instead.
#define TSVM_TOUCH_ROW(kws, t, ws, ldk, lane) \
    (((const unsigned *) ((kws) + (int64_t) ((t) < (ws) ? (t) : 0) * (ldk)))[(lane) * 32 < (int) ((ldk) * sizeof(*(kws)) / 4) ? (lane) * 32 : 0])

// One solver on a chosen XCD.  A kernel of one workgroup runs on whichever XCD its stream's hardware queue starts
// dealing at; launched as eight workgroups under a CU mask with one CU per XCD, one workgroup lands on every XCD, and
// the one that finds itself on target_xcd does the work while the others leave at once.  Exactly one workgroup is
// elected whatever the dealing: the workgroup on the target claims the launch (gate[0]: the number of the last launch
// claimed, epoch = that number + 1 for this launch), and the last of the eight to arrive (gate[1] counts arrivals,
// eight per launch) claims it if nobody has.  gate[2] tells the host where the solver ran.  Launches that share a gate
// must be ordered (one stream); gate starts as zeros, epoch at 1.
#define TSVM_SOLVER_GRID_ON_XCD 8
__device__ __forceinline__ bool solver_elected(int *gate, int epoch, int target_xcd) {
    __shared__ int s_elected;
    if (threadIdx.x == 0) {
        const int xcd = (int) __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11));   // XCC_ID
        bool won = false;
        if (xcd == target_xcd) won = atomicCAS(&gate[0], epoch - 1, epoch) == epoch - 1;
        __threadfence();
        const int arrived = atomicAdd(&gate[1], 1);
        if (!won && (arrived % TSVM_SOLVER_GRID_ON_XCD) == TSVM_SOLVER_GRID_ON_XCD - 1) {
            __threadfence();
            won = atomicCAS(&gate[0], epoch - 1, epoch) == epoch - 1;
        }
        if (won) gate[2] = xcd;
        s_elected = won;
    }
    __syncthreads();
    return s_elected != 0;
}

// Elements beyond ws are given y = 0, which puts them in neither I_up nor I_low.
template <int E, typename TB>
__global__ __launch_bounds__(SV_T) void c_smo_solve_kernel(
    const int *__restrict__ label, const double *__restrict__ f_val, double *__restrict__ alpha,
    double *__restrict__ alpha_diff, const int *__restrict__ working_set, int ws, double Cp, double Cn,
    const TB *__restrict__ kws, const double *__restrict__ k_diag, double eps, double *__restrict__ diff,
    int max_iter, int *__restrict__ gate, int epoch, int target_xcd) {
    if (gate && !solver_elected(gate, epoch, target_xcd)) return;
    constexpr int LDK = E * SV_T;
    __shared__ double s_kd[LDK];
    __shared__ float s_y[LDK];
    __shared__ double s_a[LDK];
    __shared__ double s_f[2][LDK];
    __shared__ double sA_v[SV_W], sA_l[SV_W], sB_v[SV_W];
    __shared__ int sA_i[SV_W], sB_i[SV_W], sB_go[SV_W];

    // This workgroup is a chain of dependent operations; when a chip-wide kernel runs next to it on
    // another stream its wavefronts must not wait behind that kernel's for issue slots.
    __builtin_amdgcn_s_setprio(3);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    double f[E], a_old[E], kd[E];
    unsigned member = 0;   // bit 2e: element e is in I_up; bit 2e+1: in I_low
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int t = tid * E + e;
        const bool active = t < ws;
        const int w = active ? working_set[t] : 0;
        f[e] = active ? f_val[w] : 0.0;
        a_old[e] = active ? alpha[w] : 0.0;
        const double y = active ? (double) label[w] : 0.0;
        kd[e] = active ? k_diag[w] : 1.0;
        s_kd[t] = kd[e];
        s_y[t] = (float) y;
        s_a[t] = a_old[e];
        member |= ((is_I_up(a_old[e], y, Cp, Cn) ? 1u : 0u) | (is_I_low(a_old[e], y, Cp, Cn) ? 2u : 0u)) << (2 * e);
    }
    // The alpha of the two elements changed by an iteration is written to LDS by thread 0 after the
    // next iteration's first barrier, when no wavefront can still be reading the old values.
    int pend_i = 0, pend_j = 0;
    double pend_ai = a_old[0], pend_aj = a_old[0];   // for thread 0 this is s_a[0]: the first write changes nothing
    // The initial gap fixes the local stopping threshold (smo_kernel.cpp:61-66).  It is the only place
    // where the value of low = max of f over I_low is needed: inside the loop the stopping test
    // low - up < local_eps is evaluated per element, as "no I_low element has f - up >= local_eps"
    // (the same decision, since rounding the subtraction is monotone), which costs a ballot instead of
    // a second cross-lane reduction per iteration.
    double local_eps;
    {
        double mn = TSVM_INF, mx = -TSVM_INF;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            mn = fmin_f64(mn, (member >> (2 * e)) & 1u ? f[e] : TSVM_INF);
            mx = fmax_f64(mx, (member >> (2 * e + 1)) & 1u ? f[e] : -TSVM_INF);
        }
        mn = wave_min_f64(mn);
        mx = wave_max_f64(mx);
        if (lane == 0) { sA_v[wave] = mn; sA_l[wave] = mx; }
        __syncthreads();
        double up0 = sA_v[0];
#pragma unroll
        for (int w = 1; w < SV_W; ++w) up0 = fmin_f64(up0, sA_v[w]);
        const double local_diff = block_max(sA_l) - up0;
        const double t = 0.1f * local_diff;   // float literal, as in the reference (smo_kernel.cpp:64)
        local_eps = eps > t ? eps : t;
        if (tid == 0) diff[0] = local_diff;
        __syncthreads();   // sA_* are written again below
    }
    int numOfIter = 0;
    unsigned touched = 0;
    while (true) {
        const int par = numOfIter & 1;
        // i = first argmin of f over I_up (smo_kernel.cpp:41-59)
        double fu[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            s_f[par][tid * E + e] = f[e];
            fu[e] = (member >> (2 * e)) & 1u ? f[e] : TSVM_INF;
        }
        double v;
        int vi;
        wave_first_argmin<E>(fu, tid, v, vi);
        const unsigned pre_i = TSVM_TOUCH_ROW(kws, vi, ws, LDK, lane);
        if (lane == 0) { sA_v[wave] = v; sA_i[wave] = vi; }
        __syncthreads();
        if (tid == 0) {
            s_a[pend_i] = pend_ai;
            s_a[pend_j] = pend_aj;   // after pend_i: if both name one element the second value is the final one
        }
        double up_value;
        int i;
        block_argmin(sA_v, sA_i, up_value, i, MAX_WS);
        i = up_value < TSVM_INF ? i : 0;
        const TB *row_i = kws + (int64_t) i * LDK;
        double kI[E];
        load_row_elems<E, TB>(row_i, tid, kI);
        const double kd_i = s_kd[i];
        // j2 = first argmin of -b^2/a over I_low with f > up (smo_kernel.cpp:77-90)
        double qs[E];
        bool go = false;   // some I_low element still violates: low - up >= local_eps (smo_kernel.cpp:68)
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const bool low = (member >> (2 * e + 1)) & 1u;
            const double aIJ = __builtin_fma(-2.0, kI[e], kd_i + kd[e]);
            const double bIJ = -up_value + f[e];
            const double q = -bIJ * bIJ / aIJ;
            qs[e] = low && (-up_value > -f[e]) ? q : TSVM_INF;
            go |= low && !(f[e] - up_value < local_eps);
        }
        double ft;
        int fi;
        wave_first_argmin<E>(qs, tid, ft, fi);
        const unsigned pre_j = TSVM_TOUCH_ROW(kws, fi, ws, LDK, lane);
        const bool wave_go = __builtin_amdgcn_ballot_w64(go) != 0;
        if (lane == 0) { sB_v[wave] = ft; sB_i[wave] = fi; sB_go[wave] = wave_go; }
        __syncthreads();
        bool any_go = false;
#pragma unroll
        for (int w = 0; w < SV_W; ++w) any_go |= sB_go[w] != 0;
        if (numOfIter > max_iter || !any_go) break;
        double min_t;
        int j2;
        block_argmin(sB_v, sB_i, min_t, j2, MAX_WS);
        j2 = min_t < TSVM_INF ? j2 : 0;
        const TB *row_j = kws + (int64_t) j2 * LDK;
        double kJ[E];
        load_row_elems<E, TB>(row_j, tid, kJ);
        const double kIj = (double) row_i[j2];
        // two-variable step (smo_kernel.cpp:92-103)
        const double a_i = s_a[i], y_i = (double) s_y[i];
        const double a_j0 = s_a[j2], y_j = (double) s_y[j2];
        const double alpha_i_diff = y_i > 0 ? Cp - a_i : a_i;
        const double q1 = y_j > 0 ? a_j0 : Cn - a_j0;
        const double q2 = (-up_value + s_f[par][j2]) / (kd_i + s_kd[j2] - 2 * kIj);
        const double alpha_j_diff = q1 < q2 ? q1 : q2;
        const double l = alpha_i_diff < alpha_j_diff ? alpha_i_diff : alpha_j_diff;
        const double na_i = a_i + l * y_i;
        const double na_j = (j2 == i ? na_i : a_j0) - l * y_j;
        member = set_member_bits<E>(member, tid, i, (is_I_up(na_i, y_i, Cp, Cn) ? 1u : 0u) | (is_I_low(na_i, y_i, Cp, Cn) ? 2u : 0u), 2);
        member = set_member_bits<E>(member, tid, j2, (is_I_up(na_j, y_j, Cp, Cn) ? 1u : 0u) | (is_I_low(na_j, y_j, Cp, Cn) ? 2u : 0u), 2);
        pend_i = i;
        pend_j = j2;
        pend_ai = na_i;
        pend_aj = na_j;
#pragma unroll
        for (int e = 0; e < E; ++e) f[e] = __builtin_fma(-l, kJ[e] - kI[e], f[e]);
        touched ^= pre_i ^ pre_j;
        ++numOfIter;
    }
    __syncthreads();   // the pending alpha writes of the last step were made before the loop's exit test
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int t = tid * E + e;
        if (t < ws) {
            const double a = s_a[t];
            alpha_diff[t] = -(a - a_old[e]) * (double) s_y[t];
            alpha[working_set[t]] = a;
        }
    }
    // diff may be host memory that a waiting host thread polls: diff[1] is the kernel's last word, and everything
    // written before it (diff[0] in particular) has to be visible system-wide first
    if (tid == 0) {
        __threadfence_system();
        diff[1] = (double) numOfIter;
    }
    if (touched == 0x7ff00001u && numOfIter < 0) diff[0] = 0.0;   // keeps the row-touching loads alive; never true
}

// nu variant (smo_kernel.cpp:127-287): four extrema, two second-order candidates.  Keeps the CPU
// code's j2n score, which uses kd[ip] and K[ip, .] (smo_kernel.cpp:239), and leaves diff[1] alone.
// Membership bits per element: 0 = y>0 & a<C (I_up, positive), 1 = y<0 & a>0 (I_up, negative),
// 2 = y>0 & a>0 (I_low, positive), 3 = y<0 & a<C (I_low, negative).
__device__ __forceinline__ unsigned nu_member_bits(double a, double y, double C) {
    return (y > 0 && a < C ? 1u : 0u) | (y < 0 && a > 0 ? 2u : 0u) | (y > 0 && a > 0 ? 4u : 0u) | (y < 0 && a < C ? 8u : 0u);
}

template <int E, typename TB>
__global__ __launch_bounds__(SV_T) void nu_smo_solve_kernel(
    const int *__restrict__ label, const double *__restrict__ f_val, double *__restrict__ alpha,
    double *__restrict__ alpha_diff, const int *__restrict__ working_set, int ws, double C,
    const TB *__restrict__ kws, const double *__restrict__ k_diag, double eps, double *__restrict__ diff,
    int max_iter, int *__restrict__ gate, int epoch, int target_xcd) {
    if (gate && !solver_elected(gate, epoch, target_xcd)) return;
    constexpr int LDK = E * SV_T;
    __shared__ double s_kd[LDK];
    __shared__ float s_y[LDK];
    __shared__ double s_a[LDK];
    __shared__ double s_f[2][LDK];
    __shared__ double sA_vp[SV_W], sA_vn[SV_W], sA_lp[SV_W], sA_ln[SV_W], sB_vp[SV_W], sB_vn[SV_W];
    __shared__ int sA_ip[SV_W], sA_in[SV_W], sB_ip[SV_W], sB_in[SV_W], sB_go[SV_W];

    __builtin_amdgcn_s_setprio(3);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    double f[E], a_old[E], kd[E];
    unsigned member = 0;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int t = tid * E + e;
        const bool active = t < ws;
        const int w = active ? working_set[t] : 0;
        f[e] = active ? f_val[w] : 0.0;
        a_old[e] = active ? alpha[w] : 0.0;
        const double y = active ? (double) label[w] : 0.0;
        kd[e] = active ? k_diag[w] : 1.0;
        s_kd[t] = kd[e];
        s_y[t] = (float) y;
        s_a[t] = a_old[e];
        member |= nu_member_bits(a_old[e], y, C) << (4 * e);
    }
    int pend_i = 0, pend_j = 0;
    double pend_ai = a_old[0], pend_aj = a_old[0];
    // initial gap -> local stopping threshold (smo_kernel.cpp:176-183); inside the loop the stopping
    // test is evaluated per element, as in the C variant
    double local_eps, first_diff;
    {
        double mnp = TSVM_INF, mnn = TSVM_INF, mxp = -TSVM_INF, mxn = -TSVM_INF;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const unsigned b = member >> (4 * e);
            mnp = fmin_f64(mnp, b & 1u ? f[e] : TSVM_INF);
            mnn = fmin_f64(mnn, b & 2u ? f[e] : TSVM_INF);
            mxp = fmax_f64(mxp, b & 4u ? f[e] : -TSVM_INF);
            mxn = fmax_f64(mxn, b & 8u ? f[e] : -TSVM_INF);
        }
        mnp = wave_min_f64(mnp);
        mnn = wave_min_f64(mnn);
        mxp = wave_max_f64(mxp);
        mxn = wave_max_f64(mxn);
        if (lane == 0) { sA_vp[wave] = mnp; sA_vn[wave] = mnn; sA_lp[wave] = mxp; sA_ln[wave] = mxn; }
        __syncthreads();
        double up_p0 = sA_vp[0], up_n0 = sA_vn[0];
#pragma unroll
        for (int w = 1; w < SV_W; ++w) { up_p0 = fmin_f64(up_p0, sA_vp[w]); up_n0 = fmin_f64(up_n0, sA_vn[w]); }
        const double dp = block_max(sA_lp) - up_p0, dn = block_max(sA_ln) - up_n0;
        const double local_diff = dp > dn ? dp : dn;
        const double t = 0.1 * local_diff;
        local_eps = eps > t ? eps : t;
        first_diff = local_diff;
        __syncthreads();
    }
    int numOfIter = 0;
    unsigned touched = 0;
    while (true) {
        const int par = numOfIter & 1;
        double fup[E], fun[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            s_f[par][tid * E + e] = f[e];
            const unsigned b = member >> (4 * e);
            fup[e] = b & 1u ? f[e] : TSVM_INF;
            fun[e] = b & 2u ? f[e] : TSVM_INF;
        }
        double vp, vn;
        int ipi, ini;
        wave_first_argmin<E>(fup, tid, vp, ipi);
        wave_first_argmin<E>(fun, tid, vn, ini);
        const unsigned pre_i = TSVM_TOUCH_ROW(kws, ipi, ws, LDK, lane) ^ TSVM_TOUCH_ROW(kws, ini, ws, LDK, lane);
        if (lane == 0) { sA_vp[wave] = vp; sA_ip[wave] = ipi; sA_vn[wave] = vn; sA_in[wave] = ini; }
        __syncthreads();
        if (tid == 0) {
            s_a[pend_i] = pend_ai;
            s_a[pend_j] = pend_aj;
        }
        double up_value_p, up_value_n;
        int ip, in;
        block_argmin(sA_vp, sA_ip, up_value_p, ip, MAX_WS);
        block_argmin(sA_vn, sA_in, up_value_n, in, MAX_WS);
        ip = up_value_p < TSVM_INF ? ip : 0;
        in = up_value_n < TSVM_INF ? in : 0;
        const TB *row_p = kws + (int64_t) ip * LDK;
        const TB *row_n = kws + (int64_t) in * LDK;
        double kIp[E], kIn[E];
        load_row_elems<E, TB>(row_p, tid, kIp);
        load_row_elems<E, TB>(row_n, tid, kIn);
        const double kd_ip = s_kd[ip];
        double qp[E], qn[E];
        bool go = false;   // max(low_p - up_p, low_n - up_n) >= local_eps (smo_kernel.cpp:185)
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const unsigned b = member >> (4 * e);
            const double aIJ = __builtin_fma(-2.0, kIp[e], kd_ip + kd[e]);
            const double bp = -up_value_p + f[e], bn = -up_value_n + f[e];
            qp[e] = (b & 4u) && (-up_value_p > -f[e]) ? -bp * bp / aIJ : TSVM_INF;
            qn[e] = (b & 8u) && (-up_value_n > -f[e]) ? -bn * bn / aIJ : TSVM_INF;
            go |= ((b & 4u) && !(f[e] - up_value_p < local_eps)) || ((b & 8u) && !(f[e] - up_value_n < local_eps));
        }
        double ftp, ftn;
        int jpi, jni;
        wave_first_argmin<E>(qp, tid, ftp, jpi);
        wave_first_argmin<E>(qn, tid, ftn, jni);
        const unsigned pre_j = TSVM_TOUCH_ROW(kws, jpi, ws, LDK, lane) ^ TSVM_TOUCH_ROW(kws, jni, ws, LDK, lane);
        const bool wave_go = __builtin_amdgcn_ballot_w64(go) != 0;
        if (lane == 0) { sB_vp[wave] = ftp; sB_ip[wave] = jpi; sB_vn[wave] = ftn; sB_in[wave] = jni; sB_go[wave] = wave_go; }
        __syncthreads();
        bool any_go = false;
#pragma unroll
        for (int w = 0; w < SV_W; ++w) any_go |= sB_go[w] != 0;
        if (numOfIter > max_iter || !any_go) break;
        double f_val_j2p, f_val_j2n;
        int j2p, j2n;
        block_argmin(sB_vp, sB_ip, f_val_j2p, j2p, MAX_WS);
        block_argmin(sB_vn, sB_in, f_val_j2n, j2n, MAX_WS);
        j2p = f_val_j2p < TSVM_INF ? j2p : 0;
        j2n = f_val_j2n < TSVM_INF ? j2n : 0;
        const bool take_p = f_val_j2p < f_val_j2n;
        const int i = take_p ? ip : in;
        const int j2 = take_p ? j2p : j2n;
        const double up_value = take_p ? up_value_p : up_value_n;
        const TB *row_i = take_p ? row_p : row_n;
        const TB *row_j = kws + (int64_t) j2 * LDK;
        double kJ[E];
        load_row_elems<E, TB>(row_j, tid, kJ);
        const double kIj = (double) row_i[j2];
        const double a_i = s_a[i], y_i = (double) s_y[i];
        const double a_j0 = s_a[j2], y_j = (double) s_y[j2];
        const double alpha_i_diff = y_i > 0 ? C - a_i : a_i;
        const double q1 = y_j > 0 ? a_j0 : C - a_j0;
        const double q2 = (-up_value + s_f[par][j2]) / (s_kd[i] + s_kd[j2] - 2 * kIj);
        const double alpha_j_diff = q1 < q2 ? q1 : q2;
        const double l = alpha_i_diff < alpha_j_diff ? alpha_i_diff : alpha_j_diff;
        const double na_i = a_i + l * y_i;
        const double na_j = (j2 == i ? na_i : a_j0) - l * y_j;
        member = set_member_bits<E>(member, tid, i, nu_member_bits(na_i, y_i, C), 4);
        member = set_member_bits<E>(member, tid, j2, nu_member_bits(na_j, y_j, C), 4);
        pend_i = i;
        pend_j = j2;
        pend_ai = na_i;
        pend_aj = na_j;
#pragma unroll
        for (int e = 0; e < E; ++e) f[e] = __builtin_fma(-l, kJ[e] - (take_p ? kIp[e] : kIn[e]), f[e]);
        touched ^= pre_i ^ pre_j;
        ++numOfIter;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int t = tid * E + e;
        if (t < ws) {
            const double a = s_a[t];
            alpha_diff[t] = -(a - a_old[e]) * (double) s_y[t];
            alpha[working_set[t]] = a;
        }
    }
    // diff[0] is the only word this variant reports (smo_kernel.cpp:283 leaves diff[1] alone).  It is written last,
    // behind a system-wide fence, so that a host thread polling it in host memory sees the kernel's end.
    if (tid == 0) {
        __threadfence_system();
        diff[0] = first_diff;
    }
    if (touched == 0x7ff00001u && numOfIter < 0) diff[0] = 0.0;   // keeps the row-touching loads alive; never true
}

// The solver workgroup asks for the rest of the CU's 160 KB of LDS as (unused) dynamic shared memory:
// no other workgroup can then be placed on its CU, so a kernel running concurrently on another
// stream cannot take issue slots, LDS bandwidth or L1 space away from the latency-bound solver.
static hipError_t reserve_cu(const void *kernel, size_t static_lds, size_t *dyn) {
    const size_t cu_lds = 160 * 1024;
    *dyn = cu_lds > static_lds + 1024 ? cu_lds - static_lds - 1024 : 0;
    return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) *dyn);
}

// The dynamic LDS a solver kernel is launched with on the current device.  The attribute query and the opt-in are made
// once per kernel and device (whichever host thread comes first), not per launch.
static int solver_dyn_lds(const void *kernel, size_t *dyn) {
    static std::mutex mu;
    static std::map<std::pair<const void *, int>, size_t> table;
    int dev = 0;
    TSVM_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mu);
    auto it = table.find(std::make_pair(kernel, dev));
    if (it == table.end()) {
        hipFuncAttributes fa;
        TSVM_HIP(hipFuncGetAttributes(&fa, kernel));
        size_t d = 0;
        TSVM_HIP(reserve_cu(kernel, fa.sharedSizeBytes, &d));
        it = table.emplace(std::make_pair(kernel, dev), d).first;
    }
    *dyn = it->second;
    return 0;
}

extern "C" {

static int solver_ldk(int ws_size) { return ws_size <= SV_T ? SV_T : (ws_size <= 2 * SV_T ? 2 * SV_T : 4 * SV_T); }

size_t tsvm_smo_solve_workspace(int ws_size) {
    if (ws_size < 0) return 0;
    return sizeof(double) * (size_t) ws_size * (size_t) solver_ldk(ws_size) + 256;
}

// A float block needs float rows (a double row's values would be rounded).
static bool block_type_ok(int block_type, int row_type) {
    return block_type == TSVM_ROW_F64 || (block_type == TSVM_ROW_F32 && row_type == TSVM_ROW_F32);
}

static int launch_gather(const void *k_rows, int row_type, const int *slots, int64_t ld, const int *working_set, int ws,
                         void *workspace, int block_type, hipStream_t s) {
    TSVM_REQUIRE(row_type == TSVM_ROW_F64 || row_type == TSVM_ROW_F32, "smo_solve: unknown row type %d", row_type);
    TSVM_REQUIRE(block_type_ok(block_type, row_type), "smo_solve: block type %d not valid for row type %d", block_type, row_type);
    if (row_type == TSVM_ROW_F32 && block_type == TSVM_ROW_F32)
        hipLaunchKernelGGL((gather_ws_block_kernel<float, float>), dim3(ws), dim3(256), 0, s, (const float *) k_rows, slots, ld,
                           working_set, ws, solver_ldk(ws), (float *) workspace);
    else if (row_type == TSVM_ROW_F32)
        hipLaunchKernelGGL((gather_ws_block_kernel<float, double>), dim3(ws), dim3(256), 0, s, (const float *) k_rows, slots, ld,
                           working_set, ws, solver_ldk(ws), (double *) workspace);
    else
        hipLaunchKernelGGL((gather_ws_block_kernel<double, double>), dim3(ws), dim3(256), 0, s, (const double *) k_rows, slots, ld,
                           working_set, ws, solver_ldk(ws), (double *) workspace);
    TSVM_LAUNCH_CHECK();
    return 0;
}

#define TSVM_LAUNCH_SOLVER(KERNEL, EVAL, TB, ...)                                                   \
    do {                                                                                            \
        size_t dyn_ = 0;                                                                            \
        if (solver_grid_ == 1) {                                                                    \
            const int rc_ = solver_dyn_lds(reinterpret_cast<const void *>(KERNEL<EVAL, TB>), &dyn_); \
            if (rc_) return rc_;                                                                    \
        }                                                                                           \
        hipLaunchKernelGGL((KERNEL<EVAL, TB>), dim3(solver_grid_), dim3(SV_T), dyn_, s, __VA_ARGS__); \
    } while (0)

#define TSVM_DISPATCH_E_T(KERNEL, TB, ...)                                                      \
    do {                                                                                        \
        if (ws_size <= SV_T) TSVM_LAUNCH_SOLVER(KERNEL, 1, TB, __VA_ARGS__);                    \
        else if (ws_size <= 2 * SV_T) TSVM_LAUNCH_SOLVER(KERNEL, 2, TB, __VA_ARGS__);           \
        else TSVM_LAUNCH_SOLVER(KERNEL, 4, TB, __VA_ARGS__);                                    \
    } while (0)

// (kws_: the block; block_type_: its element type)
#define TSVM_DISPATCH_E(KERNEL, PRE, POST)                                                                           \
    do {                                                                                                             \
        if (block_type_ == TSVM_ROW_F32) {                                                                           \
            const float *kws = (const float *) kws_;                                                                 \
            TSVM_DISPATCH_E_T(KERNEL, float, TSVM_UNPACK PRE, kws, TSVM_UNPACK POST);                                \
        } else {                                                                                                     \
            const double *kws = (const double *) kws_;                                                               \
            TSVM_DISPATCH_E_T(KERNEL, double, TSVM_UNPACK PRE, kws, TSVM_UNPACK POST);                               \
        }                                                                                                            \
    } while (0)
#define TSVM_UNPACK(...) __VA_ARGS__

int tsvm_c_smo_solve(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                     int ws_size, double Cp, double Cn, const void *k_rows, int row_type, const int *slots, int64_t ld,
                     const double *k_diag, double eps, double *diff, int max_iter, void *workspace,
                     tsvm_stream stream) {
    TSVM_REQUIRE(y && f_val && alpha && alpha_diff && working_set && k_rows && k_diag && diff && workspace,
                 "tsvm_c_smo_solve: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_c_smo_solve: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    hipStream_t s = tsvm_s(stream);
    int *gate_ = nullptr;
    const int epoch_ = 0, target_xcd_ = 0, solver_grid_ = 1;
    const int block_type_ = row_type;   // the block keeps the rows' element type
    int rc = launch_gather(k_rows, row_type, slots, ld, working_set, ws_size, workspace, block_type_, s);
    if (rc) return rc;
    const void *kws_ = workspace;
    TSVM_DISPATCH_E(c_smo_solve_kernel, (y, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn),
                    (k_diag, eps, diff, max_iter, gate_, epoch_, target_xcd_));
    TSVM_LAUNCH_CHECK();
    return 0;
}

// c_smo_solve for callers that cannot allocate: the ws x ws block that tsvm_c_smo_solve gathers into the caller's
// workspace goes into a file-scope device array instead (8 MiB, held by every device the library runs on until the
// process ends).  Its device address is looked up once per device; host code never uses the array's name otherwise.
static __device__ __align__(256) double g_solver_block[(size_t) MAX_WS * MAX_WS];
#define TSVM_MAX_DEVICES 64
static double *g_solver_block_ptr[TSVM_MAX_DEVICES];
static std::mutex g_solver_block_mutex;

static int solver_block_address(double **out) {
    int dev = 0;
    TSVM_HIP(hipGetDevice(&dev));
    TSVM_REQUIRE(dev >= 0 && dev < TSVM_MAX_DEVICES, "tsvm_c_smo_solve_static: device ordinal %d outside [0, %d)", dev,
                 TSVM_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_solver_block_mutex);
    if (!g_solver_block_ptr[dev]) {
        double *p = nullptr;
        TSVM_HIP(hipGetSymbolAddress((void **) &p, HIP_SYMBOL(g_solver_block)));
        TSVM_REQUIRE(p != nullptr, "tsvm_c_smo_solve_static: no device address for the static block");
        g_solver_block_ptr[dev] = p;
    }
    *out = g_solver_block_ptr[dev];
    return 0;
}

int tsvm_c_smo_solve_static_init(void) {
    double *block = nullptr;
    int rc = solver_block_address(&block);
    if (rc) return rc;
    size_t dyn = 0;
    const void *kernels[] = {reinterpret_cast<const void *>(c_smo_solve_kernel<1, float>), reinterpret_cast<const void *>(c_smo_solve_kernel<2, float>),
                             reinterpret_cast<const void *>(c_smo_solve_kernel<4, float>), reinterpret_cast<const void *>(c_smo_solve_kernel<1, double>),
                             reinterpret_cast<const void *>(c_smo_solve_kernel<2, double>), reinterpret_cast<const void *>(c_smo_solve_kernel<4, double>)};
    for (const void *k : kernels) {
        rc = solver_dyn_lds(k, &dyn);
        if (rc) return rc;
    }
    return 0;
}

int tsvm_c_smo_solve_static(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                            int ws_size, double Cp, double Cn, const void *k_rows, int row_type, const int *slots, int64_t ld,
                            const double *k_diag, double eps, double *diff, int max_iter, tsvm_stream stream) {
    TSVM_REQUIRE(y && f_val && alpha && alpha_diff && working_set && k_rows && k_diag && diff,
                 "tsvm_c_smo_solve_static: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_c_smo_solve_static: ws_size %d outside [1, %d] (the static block holds %d x %d values)",
                 ws_size, MAX_WS, MAX_WS, MAX_WS);
    double *block = nullptr;
    int rc = solver_block_address(&block);
    if (rc) return rc;
    hipStream_t s = tsvm_s(stream);
    int *gate_ = nullptr;
    const int epoch_ = 0, target_xcd_ = 0, solver_grid_ = 1;
    // the gather writes every element of the ws x ldk block the solver reads (columns beyond ws as zeros), so
    // nothing of the previous call's content is read
    const int block_type_ = row_type;
    rc = launch_gather(k_rows, row_type, slots, ld, working_set, ws_size, block, block_type_, s);
    if (rc) return rc;
    const void *kws_ = block;
    TSVM_DISPATCH_E(c_smo_solve_kernel, (y, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn),
                    (k_diag, eps, diff, max_iter, gate_, epoch_, target_xcd_));
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_smo_solve_block_ld(int ws_size) { return ws_size < 1 ? 0 : solver_ldk(ws_size); }

int tsvm_smo_gather_block(const void *k_rows, int row_type, const int *slots, int64_t ld, const int *cols, int ws_size,
                          void *kws, int block_type, tsvm_stream stream) {
    TSVM_REQUIRE(k_rows && cols && kws, "tsvm_smo_gather_block: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_smo_gather_block: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    return launch_gather(k_rows, row_type, slots, ld, cols, ws_size, kws, block_type, tsvm_s(stream));
}

int tsvm_smo_gather_block_by_id(const void *k_rows, int row_type, const int *slot_of_id, int64_t ld, const int *ids,
                                int ws_size, void *kws, int block_type, int *slots_out, tsvm_stream stream) {
    TSVM_REQUIRE(k_rows && slot_of_id && ids && kws && slots_out, "tsvm_smo_gather_block_by_id: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_smo_gather_block_by_id: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    TSVM_REQUIRE(row_type == TSVM_ROW_F64 || row_type == TSVM_ROW_F32, "tsvm_smo_gather_block_by_id: unknown row type %d", row_type);
    TSVM_REQUIRE(block_type_ok(block_type, row_type), "tsvm_smo_gather_block_by_id: block type %d not valid for row type %d", block_type,
                 row_type);
    if (row_type == TSVM_ROW_F32 && block_type == TSVM_ROW_F32)
        hipLaunchKernelGGL((gather_ws_block_by_id_kernel<float, float>), dim3(ws_size), dim3(256), 0, tsvm_s(stream),
                           (const float *) k_rows, slot_of_id, ld, ids, ws_size, solver_ldk(ws_size), (float *) kws, slots_out);
    else if (row_type == TSVM_ROW_F32)
        hipLaunchKernelGGL((gather_ws_block_by_id_kernel<float, double>), dim3(ws_size), dim3(256), 0, tsvm_s(stream),
                           (const float *) k_rows, slot_of_id, ld, ids, ws_size, solver_ldk(ws_size), (double *) kws, slots_out);
    else
        hipLaunchKernelGGL((gather_ws_block_by_id_kernel<double, double>), dim3(ws_size), dim3(256), 0, tsvm_s(stream),
                           (const double *) k_rows, slot_of_id, ld, ids, ws_size, solver_ldk(ws_size), (double *) kws, slots_out);
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_row_slots_assign(const int *ids_new, int n_new, int *slot_of_id, int *state, int *miss_ids, int *miss_slots,
                          const int *ids_ws, int ws_size, int *slots_ws, int *info, tsvm_stream stream) {
    TSVM_REQUIRE(ids_new && slot_of_id && state && miss_ids && miss_slots && ids_ws && slots_ws && info,
                 "tsvm_row_slots_assign: null pointer");
    TSVM_REQUIRE(n_new >= 0 && n_new <= MAX_WS && ws_size >= 0 && ws_size <= MAX_WS, "tsvm_row_slots_assign: sizes %d, %d outside [0, %d]",
                 n_new, ws_size, MAX_WS);
    hipLaunchKernelGGL(row_slots_assign_kernel, dim3(1), dim3(RA_T), 0, tsvm_s(stream), ids_new, n_new, slot_of_id, state, miss_ids,
                       miss_slots, ids_ws, ws_size, slots_ws, info);
    TSVM_LAUNCH_CHECK();
    return 0;
}

static int c_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set, int ws_size,
                   double Cp, double Cn, const void *kws_, int block_type_, const double *k_diag, double eps, double *diff,
                   int max_iter, int *gate_, int epoch_, int target_xcd_, tsvm_stream stream) {
    TSVM_REQUIRE(y && f_val && alpha && alpha_diff && working_set && kws_ && k_diag && diff, "tsvm_c_smo_solve_block: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_c_smo_solve_block: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    TSVM_REQUIRE(block_type_ == TSVM_ROW_F64 || block_type_ == TSVM_ROW_F32, "tsvm_c_smo_solve_block: unknown block type %d", block_type_);
    hipStream_t s = tsvm_s(stream);
    const int solver_grid_ = gate_ ? TSVM_SOLVER_GRID_ON_XCD : 1;
    TSVM_DISPATCH_E(c_smo_solve_kernel, (y, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn),
                    (k_diag, eps, diff, max_iter, gate_, epoch_, target_xcd_));
    TSVM_LAUNCH_CHECK();
    return 0;
}

static int nu_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set, int ws_size,
                    double C, const void *kws_, int block_type_, const double *k_diag, double eps, double *diff, int max_iter,
                    int *gate_, int epoch_, int target_xcd_, tsvm_stream stream) {
    TSVM_REQUIRE(y && f_val && alpha && alpha_diff && working_set && kws_ && k_diag && diff, "tsvm_nu_smo_solve_block: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_nu_smo_solve_block: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    TSVM_REQUIRE(block_type_ == TSVM_ROW_F64 || block_type_ == TSVM_ROW_F32, "tsvm_nu_smo_solve_block: unknown block type %d", block_type_);
    hipStream_t s = tsvm_s(stream);
    const int solver_grid_ = gate_ ? TSVM_SOLVER_GRID_ON_XCD : 1;
    TSVM_DISPATCH_E(nu_smo_solve_kernel, (y, f_val, alpha, alpha_diff, working_set, ws_size, C),
                    (k_diag, eps, diff, max_iter, gate_, epoch_, target_xcd_));
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_c_smo_solve_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                           int ws_size, double Cp, double Cn, const void *kws, int block_type, const double *k_diag, double eps,
                           double *diff, int max_iter, tsvm_stream stream) {
    return c_block(y, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn, kws, block_type, k_diag, eps, diff, max_iter, nullptr, 0,
                   0, stream);
}

int tsvm_nu_smo_solve_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                            int ws_size, double C, const void *kws, int block_type, const double *k_diag, double eps, double *diff,
                            int max_iter, tsvm_stream stream) {
    return nu_block(y, f_val, alpha, alpha_diff, working_set, ws_size, C, kws, block_type, k_diag, eps, diff, max_iter, nullptr, 0, 0,
                    stream);
}

int tsvm_c_smo_solve_block_on_xcd(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                                  int ws_size, double Cp, double Cn, const void *kws, int block_type, const double *k_diag, double eps,
                                  double *diff, int max_iter, int *gate, int epoch, int xcd, tsvm_stream stream) {
    TSVM_REQUIRE(gate && epoch >= 1 && xcd >= 0 && xcd < TSVM_SOLVER_GRID_ON_XCD, "tsvm_c_smo_solve_block_on_xcd: bad gate, epoch or xcd");
    return c_block(y, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn, kws, block_type, k_diag, eps, diff, max_iter, gate, epoch,
                   xcd, stream);
}

int tsvm_nu_smo_solve_block_on_xcd(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                                   int ws_size, double C, const void *kws, int block_type, const double *k_diag, double eps,
                                   double *diff, int max_iter, int *gate, int epoch, int xcd, tsvm_stream stream) {
    TSVM_REQUIRE(gate && epoch >= 1 && xcd >= 0 && xcd < TSVM_SOLVER_GRID_ON_XCD, "tsvm_nu_smo_solve_block_on_xcd: bad gate, epoch or xcd");
    return nu_block(y, f_val, alpha, alpha_diff, working_set, ws_size, C, kws, block_type, k_diag, eps, diff, max_iter, gate, epoch, xcd,
                    stream);
}

int tsvm_nu_smo_solve(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                      int ws_size, double C, const void *k_rows, int row_type, const int *slots, int64_t ld,
                      const double *k_diag, double eps, double *diff, int max_iter, void *workspace,
                      tsvm_stream stream) {
    TSVM_REQUIRE(y && f_val && alpha && alpha_diff && working_set && k_rows && k_diag && diff && workspace,
                 "tsvm_nu_smo_solve: null pointer");
    TSVM_REQUIRE(ws_size >= 1 && ws_size <= MAX_WS, "tsvm_nu_smo_solve: ws_size %d outside [1, %d]", ws_size, MAX_WS);
    hipStream_t s = tsvm_s(stream);
    int *gate_ = nullptr;
    const int epoch_ = 0, target_xcd_ = 0, solver_grid_ = 1;
    const int block_type_ = row_type;
    int rc = launch_gather(k_rows, row_type, slots, ld, working_set, ws_size, workspace, block_type_, s);
    if (rc) return rc;
    const void *kws_ = workspace;
    TSVM_DISPATCH_E(nu_smo_solve_kernel, (y, f_val, alpha, alpha_diff, working_set, ws_size, C),
                    (k_diag, eps, diff, max_iter, gate_, epoch_, target_xcd_));
    TSVM_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
