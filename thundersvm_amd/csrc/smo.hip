// SMO device kernels for gfx950: update_f, the single-workgroup local solvers and the fused
// sort_f + select_working_set.
//
// Reference behaviour restated here: src/thundersvm/kernel/smo_kernel.cpp:12-332,
// src/thundersvm/solver/csmosolver.cpp:123-165, src/thundersvm/solver/nusmosolver.cpp:48-118
// (the USE_CUDA=OFF, USE_DOUBLE=ON build: first-index tie breaks, serial summation order).
#include "../../include/thundersvm_amd.h"
#include "tsvm_device.h"
#include "tsvm_internal.h"

#define TSVM_INF __builtin_inf()
#define MAX_WS 1024

// ------------------------------------------------------------------------------------------------
// Fused sort_f + select_working_set.
//
// The reference sorts (f, index) pairs ascending (smo_kernel.cpp:321-332) and then walks the
// sorted order from both ends, alternately taking the next unmarked I_up element from the low end
// and the next unmarked I_low element from the high end (csmosolver.cpp:123-165).  Only the first
// n_select candidates from each end can ever be taken, so instead of sorting n pairs this selects,
// per side, the n_select smallest composite keys (f-bits, index) among that side's candidates with
// an MSB-first radix select (11-bit digits, one pass over the keys per digit, early exit once the
// boundary bucket is exactly consumed), sorts those <= 1024 entries in LDS with a bitonic network
// and replays the alternating scan on them.  The high end is handled by complementing key and
// index, so every side is an ascending selection.  Composite keys are unique, which makes the
// result independent of any thread ordering.
//
// Sides: C-SMO 0 = I_up (ascending), 1 = I_low (descending);
//        nu-SMO 0 = I_up&y>0, 1 = I_up&y<0 (ascending), 2 = I_low&y>0, 3 = I_low&y<0 (descending).
// ------------------------------------------------------------------------------------------------
#define SEL_BINS 2048
#define SEL_DIGIT 11
#define SEL_MAX_PASS 9
#define SEL_MAX_SIDES 4
#define SEL_T 256

struct SelState {
    uint64_t pk;      // resolved high bits of the key part
    uint32_t pi;      // resolved high bits of the index part
    uint32_t k_rem;   // entries still to take from inside the boundary bucket
    uint32_t done;    // 1: selection decided; entries matching the prefix are all taken
    uint32_t pad;     // number of digits held by the prefix
};

struct SelWorkspace {   // device-side layout, carved from the caller's workspace
    uint64_t *keys;     // [n] order-preserving transform of f
    uint8_t *flags;     // [n] side membership bits
    uint32_t *hist;     // [SEL_MAX_PASS][SEL_MAX_SIDES][SEL_BINS]
    SelState *state;    // [SEL_MAX_PASS + 1][SEL_MAX_SIDES]
    uint32_t *count;    // [SEL_MAX_SIDES]
    uint64_t *list_key; // [SEL_MAX_SIDES][MAX_WS]
    uint32_t *list_idx; // [SEL_MAX_SIDES][MAX_WS]
};

static size_t sel_align(size_t v) { return (v + 255) & ~(size_t) 255; }

static size_t sel_carve(void *base, int64_t n, SelWorkspace *w) {
    size_t off = 0;
    char *b = (char *) base;
    auto take = [&](size_t bytes) { size_t o = off; off += sel_align(bytes); return b ? b + o : nullptr; };
    void *keys = take(sizeof(uint64_t) * (size_t) n);
    void *flags = take((size_t) n);
    void *hist = take(sizeof(uint32_t) * SEL_MAX_PASS * SEL_MAX_SIDES * SEL_BINS);
    void *state = take(sizeof(SelState) * (SEL_MAX_PASS + 1) * SEL_MAX_SIDES);
    void *count = take(sizeof(uint32_t) * SEL_MAX_SIDES);
    void *lk = take(sizeof(uint64_t) * SEL_MAX_SIDES * MAX_WS);
    void *li = take(sizeof(uint32_t) * SEL_MAX_SIDES * MAX_WS);
    if (w) {
        w->keys = (uint64_t *) keys; w->flags = (uint8_t *) flags;
        w->hist = (uint32_t *) hist; w->state = (SelState *) state; w->count = (uint32_t *) count;
        w->list_key = (uint64_t *) lk; w->list_idx = (uint32_t *) li;
    }
    return off;
}

struct SelGeom {
    int n_sides;
    int n_pass;
    int idx_bits;
    uint32_t idx_mask;
    uint32_t k;   // n_select
};

// digit p of the composite (key: 6 digits of 11,11,11,11,11,9 bits; then the index digits)
__device__ __forceinline__ void sel_digit_geom(int p, int idx_bits, bool &is_key, int &shift, int &width) {
    if (p < 6) {
        is_key = true;
        width = p < 5 ? SEL_DIGIT : 9;
        shift = p < 5 ? 64 - SEL_DIGIT * (p + 1) : 0;
    } else {
        is_key = false;
        const int rb = idx_bits - SEL_DIGIT * (p - 6);
        width = rb < SEL_DIGIT ? rb : SEL_DIGIT;
        shift = rb - width;
    }
}
__device__ __forceinline__ int sel_resolved_key_bits(int p) { return p >= 6 ? 64 : SEL_DIGIT * p; }
__device__ __forceinline__ int sel_resolved_idx_bits(int p, int idx_bits) {
    if (p <= 6) return 0;
    const int r = SEL_DIGIT * (p - 6);
    return r < idx_bits ? r : idx_bits;
}

// -1 / 0 / +1: composite (k, i) versus the prefix on the bits resolved before pass p
__device__ __forceinline__ int sel_cmp_prefix(uint64_t k, uint32_t i, const SelState &st, int p, int idx_bits) {
    const int rk = sel_resolved_key_bits(p);
    if (rk > 0) {
        const uint64_t a = rk == 64 ? k : (k >> (64 - rk));
        const uint64_t b = rk == 64 ? st.pk : (st.pk >> (64 - rk));
        if (a < b) return -1;
        if (a > b) return 1;
    }
    const int ri = sel_resolved_idx_bits(p, idx_bits);
    if (ri > 0) {
        const uint32_t a = i >> (idx_bits - ri);
        const uint32_t b = st.pi >> (idx_bits - ri);
        if (a < b) return -1;
        if (a > b) return 1;
    }
    return 0;
}

__device__ __forceinline__ uint64_t f_to_key(double f) {
    if (f == 0.0) f = 0.0;  // -0.0 and +0.0 compare equal in the reference's sort
    uint64_t u = (uint64_t) __double_as_longlong(f);
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}

__device__ __forceinline__ bool sel_side_descending(int side, int n_sides) { return n_sides == 2 ? side == 1 : side >= 2; }

// What a call needs to find in the workspace: zeroed histograms for the digits that are counted with atomics
// by the whole grid and zeroed list lengths.  Written by sel_init_kernel, and again
// by sel_final_kernel once it has read what it needs, so that the next call on the same workspace (same n,
// same sides) can start counting straight away.
__device__ __forceinline__ void sel_arm(const SelWorkspace &w, const SelGeom &g, int p_full, int64_t gid, int64_t stride) {
    for (int64_t e = gid; e < (int64_t) p_full * SEL_MAX_SIDES * SEL_BINS; e += stride) w.hist[e] = 0;
    if (gid < SEL_MAX_SIDES) w.count[gid] = 0;
}

__global__ void sel_init_kernel(SelWorkspace w, SelGeom g, int p_full) {
    sel_arm(w, g, p_full, (int64_t) blockIdx.x * blockDim.x + threadIdx.x, (int64_t) gridDim.x * blockDim.x);
}

// Computes, in LDS, the state after pass p-1's histogram has been consumed (st_out), from the
// state before it (global state[p-1]) and hist[p-1].  Every workgroup does this redundantly; the first
// SEL_T threads of the workgroup do the work, any others only join the barriers.
//
// A side is decided as soon as the boundary bucket can be taken whole: when everything up to and including
// it fits the side's list (MAX_WS entries), the list is a superset of the k smallest candidates, in which
// every extra entry is larger than all of them, and sel_final_kernel sorts the list and reads it from the
// front.  With 11-bit digits that is the normal case after the second or third pass.
__device__ void sel_advance_state(const SelWorkspace &w, const SelGeom &g, int p, SelState *st_out /* LDS [sides] */,
                                  uint32_t *scratch /* LDS [SEL_T + 8] */) {
    const int tid = threadIdx.x;
    const bool worker = tid < SEL_T;
    const int lane = tid & 63, wave = tid >> 6;
    for (int s = 0; s < g.n_sides; ++s) {
        SelState st = w.state[(p - 1) * SEL_MAX_SIDES + s];
        if (!st.done) {
            const uint32_t *h = w.hist + ((size_t) (p - 1) * SEL_MAX_SIDES + s) * SEL_BINS;
            uint32_t c[SEL_BINS / SEL_T];
            uint32_t sum = 0, incl = 0;
            if (worker) {
#pragma unroll
                for (int e = 0; e < SEL_BINS / SEL_T; ++e) { c[e] = h[tid * (SEL_BINS / SEL_T) + e]; sum += c[e]; }
                incl = sum;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) {
                    uint32_t o = __shfl_up(incl, d, 64);
                    if (lane >= d) incl += o;
                }
                if (lane == 63) scratch[wave] = incl;
            }
            __syncthreads();
            if (worker) {
                uint32_t wave_base = 0, total = 0;
                for (int wv = 0; wv < SEL_T / 64; ++wv) {
                    if (wv < wave) wave_base += scratch[wv];
                    total += scratch[wv];
                }
                const uint32_t excl = wave_base + incl - sum;
                if (total < st.k_rem) {
                    // fewer candidates than requested (only possible on the first digit): take them all
                    if (tid == 0) { st.done = 1; st.k_rem = total; st_out[s] = st; }
                } else if (excl < st.k_rem && st.k_rem <= excl + sum) {
                    uint32_t below = excl;
                    int b = 0;
                    for (int e = 0; e < SEL_BINS / SEL_T; ++e) {
                        if (below + c[e] >= st.k_rem) { b = tid * (SEL_BINS / SEL_T) + e; break; }
                        below += c[e];
                    }
                    const uint32_t cb = h[b];
                    const uint32_t taken = g.k - st.k_rem;   // entries of the buckets decided by earlier digits
                    bool is_key; int shift, width;
                    sel_digit_geom(p - 1, g.idx_bits, is_key, shift, width);
                    if (is_key) st.pk |= (uint64_t) b << shift; else st.pi |= (uint32_t) b << shift;
                    st.k_rem -= below;
                    st.pad = (uint32_t) p;
                    if (cb == st.k_rem || p == g.n_pass || taken + below + cb <= (uint32_t) MAX_WS) st.done = 1;
                    st_out[s] = st;
                }
            }
            __syncthreads();
        } else {
            if (tid == 0) st_out[s] = st;
            __syncthreads();
        }
    }
    __syncthreads();
}

// One count for `bin` from every lane with `valid` set, added to the LDS histogram h with one atomic per distinct
// bin of the wavefront instead of one per lane: the first digit of f (sign and exponent) is the same for most
// instances, and atomics of 64 lanes on one LDS word are carried out one after the other.  May be called in
// divergent code: only the lanes that call take part.
__device__ __forceinline__ void sel_hist_add_wave(uint32_t *h, bool valid, uint32_t bin) {
    uint64_t todo = __ballot(valid);
    while (todo) {
        const int leader = __builtin_ctzll(todo);
        const uint32_t b = (uint32_t) __builtin_amdgcn_readlane((int) bin, leader);
        const uint64_t same = __ballot(valid && bin == b);
        if ((int) (threadIdx.x & 63) == leader) atomicAdd(&h[b], (uint32_t) __popcll(same));
        todo &= ~same;
    }
}

// One candidate's contribution to the histograms of digit p: on every undecided side it belongs to, if it
// matches that side's prefix.
__device__ __forceinline__ void sel_count(const SelGeom &g, const SelState *st, uint32_t (*lhist)[SEL_BINS], int p,
                                          bool is_key, int shift, uint32_t dmask, uint64_t key, uint32_t fl, int64_t j) {
    for (int s = 0; s < g.n_sides; ++s) {
        if (!(fl & (1u << s)) || st[s].done) continue;
        const bool desc = sel_side_descending(s, g.n_sides);
        const uint64_t k2 = desc ? ~key : key;
        const uint32_t i2 = desc ? g.idx_mask - (uint32_t) j : (uint32_t) j;
        if (sel_cmp_prefix(k2, i2, st[s], p, g.idx_bits) != 0) continue;
        const uint32_t dg = is_key ? (uint32_t) (k2 >> shift) & dmask : (i2 >> shift) & dmask;
        atomicAdd(&lhist[s][dg], 1u);
    }
}

// Side membership of an unmarked instance (csmosolver.cpp:133-159, nusmosolver.cpp:60-115).
__device__ __forceinline__ uint32_t sel_flags(double a, double yy, double Cp, double Cn, int n_sides) {
    const bool up = is_I_up(a, yy, Cp, Cn), low = is_I_low(a, yy, Cp, Cn);
    if (n_sides == 2) return (up ? 1u : 0u) | (low ? 2u : 0u);
    return ((up && yy > 0) ? 1u : 0u) | ((up && yy < 0) ? 2u : 0u) | ((low && yy > 0) ? 4u : 0u) | ((low && yy < 0) ? 8u : 0u);
}

// What the selection's first pass needs besides f when update_f makes it (NS sides; see update_f_kernel).
struct SelFuse {
    SelWorkspace w;
    SelGeom g;
    const int *y;
    const double *alpha;
    double Cp, Cn;
    const int *marked;
    int n_marked;
};

// ------------------------------------------------------------------------------------------------
// update_f: f[j] -= sum_t alpha_diff[t] * K_t[j]  (smo_kernel.cpp:300-319)
// Bandwidth-bound stream over the ws x n kernel rows.  The non-zero alpha_diff entries are
// compacted (in order) into LDS once per workgroup; rows with alpha_diff == 0 are never read.
// Each thread owns one to four adjacent columns and keeps 8 to 32 row loads in flight.  On the vector-load
// path the columns are dealt evenly to a number of workgroups that is a multiple of 248 (every CU, or every
// CU left to a stream that leaves one CU per XCD to the local solver, gets the same number of workgroups):
// with a grid of full 256-thread workgroups some CUs stream 2 and others 1, and the launch lasts as long as
// the busiest one.
// ------------------------------------------------------------------------------------------------
#define UF_T 256
#define UF_CHUNK 1024

// TK: element type of the kernel rows; COLS columns per thread (consecutive, loaded as one vector of
// COLS elements); UNROLL rows in flight.  Rows are n columns wide and f holds `repeat` stacked copies
// of the n columns, each of which receives the same sum.
//
// NS > 0: the kernel also makes the first pass of the working-set selection that follows on the updated f, over
// the n * repeat stacked instances and NS sides (what sel_pass_kernel does for digit 0: keys, side flags, the
// first digit's histogram, the state before it), while each new f value is still in a register.  The instances
// of the kept half of the working set (sf.marked) that fall among a workgroup's columns are a bit field in LDS.
#define UF_MAX_REPEAT 4
template <typename TK, int COLS, int UNROLL, int NS>
__global__ __launch_bounds__(UF_T) void update_f_kernel(double *__restrict__ f, const double *__restrict__ alpha_diff,
                                                        int ws, const TK *__restrict__ k_rows,
                                                        const int *__restrict__ slots, int64_t ld, int64_t n, int repeat,
                                                        int vec_per_wg, SelFuse sf) {
    typedef TK vec_t __attribute__((ext_vector_type(COLS)));
    __shared__ uint32_t lhist[NS > 0 ? NS : 1][NS > 0 ? SEL_BINS : 1];
    __shared__ uint32_t mark_bits[NS > 0 ? UF_MAX_REPEAT : 1][NS > 0 ? UF_T * 4 / 32 : 1];   // a workgroup owns at most UF_T * COLS <= 1024 columns
    __shared__ double s_ad[UF_CHUNK];
    __shared__ int64_t s_off[UF_CHUNK];
    __shared__ int s_wave_cnt[UF_T / 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t j = ((int64_t) blockIdx.x * vec_per_wg + tid) * COLS;
    const bool act = tid < vec_per_wg && j < n;   // a vector may reach past n, but never past the padded row (checked by the launcher)
    double sum[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) sum[c] = 0.0;
    const int64_t col_lo = (int64_t) blockIdx.x * vec_per_wg * COLS;
    if (NS > 0) {
        for (int e = tid; e < NS * SEL_BINS; e += UF_T) (&lhist[0][0])[e] = 0;
        for (int e = tid; e < UF_MAX_REPEAT * (UF_T * 4 / 32); e += UF_T) (&mark_bits[0][0])[e] = 0;
        if (blockIdx.x == 0 && tid < NS) {
            SelState s0;
            s0.pk = 0; s0.pi = 0; s0.k_rem = sf.g.k; s0.done = 0; s0.pad = 0;
            sf.w.state[tid] = s0;   // the state before digit 0, for the next pass
        }
        __syncthreads();
        const int64_t col_hi = col_lo + (int64_t) vec_per_wg * COLS;
        for (int i = tid; i < sf.n_marked; i += UF_T) {
            const int64_t id = sf.marked[i];
            for (int r = 0; r < repeat; ++r) {
                const int64_t c = id - r * n;   // column, if the id lies in copy r
                if (c >= col_lo && c < col_hi && c < n) atomicOr(&mark_bits[r][(c - col_lo) >> 5], 1u << ((c - col_lo) & 31));
            }
        }
        // (the barriers of the loop below, or the one before the epilogue, order these writes before their readers)
    }
    for (int base = 0; base < ws; base += UF_CHUNK) {
        // ordered compaction of this chunk's non-zero entries: thread t owns entries 4t..4t+3
        double v[4];
        int cnt = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int t = base + tid * 4 + e;
            v[e] = t < ws ? alpha_diff[t] : 0.0;
            cnt += (v[e] != 0.0);
        }
        int incl = cnt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int o = __shfl_up(incl, d, 64);
            if (lane >= d) incl += o;
        }
        if (lane == 63) s_wave_cnt[wave] = incl;
        __syncthreads();
        int wave_base = 0, total = 0;
#pragma unroll
        for (int w = 0; w < UF_T / 64; ++w) {
            if (w < wave) wave_base += s_wave_cnt[w];
            total += s_wave_cnt[w];
        }
        int pos = wave_base + incl - cnt;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (v[e] != 0.0) {
                const int t = base + tid * 4 + e;
                s_ad[pos] = v[e];
                s_off[pos] = (int64_t) (slots ? slots[t] : t) * ld;
                ++pos;
            }
        }
        __syncthreads();
        if (act) {
            int u = 0;
            for (; u + UNROLL <= total; u += UNROLL) {
                vec_t k[UNROLL];
#pragma unroll
                for (int e = 0; e < UNROLL; ++e) k[e] = load_streaming((const vec_t *) (k_rows + s_off[u + e] + j));
#pragma unroll
                for (int e = 0; e < UNROLL; ++e) {
                    const double ad = s_ad[u + e];
#pragma unroll
                    for (int c = 0; c < COLS; ++c) sum[c] = __builtin_fma(ad, (double) k[e][c], sum[c]);
                }
            }
            for (; u < total; ++u) {
                const vec_t k = load_streaming((const vec_t *) (k_rows + s_off[u] + j));
                const double ad = s_ad[u];
#pragma unroll
                for (int c = 0; c < COLS; ++c) sum[c] = __builtin_fma(ad, (double) k[c], sum[c]);
            }
        }
        __syncthreads();
    }
    if (NS == 0) {
        if (act) {
            for (int r = 0; r < repeat; ++r) {
#pragma unroll
                for (int c = 0; c < COLS; ++c)
                    if (j + c < n) f[(int64_t) r * n + j + c] -= sum[c];
            }
        }
        return;
    }
    __syncthreads();
    if (act) {
        for (int r = 0; r < repeat; ++r) {
            const int64_t j0 = (int64_t) r * n + j;   // the first of this thread's stacked instances in copy r
            // every load first, then the arithmetic: one memory latency for the lot
            double fo[COLS], al[COLS];
            int yv[COLS];
#pragma unroll
            for (int c = 0; c < COLS; ++c) {
                const bool in = j + c < n;
                fo[c] = in ? f[j0 + c] : 0.0;
                al[c] = in ? sf.alpha[j0 + c] : 0.0;
                yv[c] = in ? sf.y[j0 + c] : 1;
            }
            uint32_t fl_all = 0;
#pragma unroll
            for (int c = 0; c < COLS; ++c) {
                const bool in = j + c < n;
                const double fn = fo[c] - sum[c];
                const uint64_t key = f_to_key(fn);
                const int bit = (int) (j + c - col_lo);
                uint32_t fl = 0;
                if (in && !((mark_bits[r][bit >> 5] >> (bit & 31)) & 1u)) fl = sel_flags(al[c], (double) yv[c], sf.Cp, sf.Cn, NS);
                if (in) {
                    f[j0 + c] = fn;
                    sf.w.keys[j0 + c] = key;
                }
                fl_all |= fl << (8 * c);
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const uint64_t k2 = sel_side_descending(s, NS) ? ~key : key;
                    sel_hist_add_wave(lhist[s], (fl >> s) & 1u, (uint32_t) (k2 >> (64 - SEL_DIGIT)));   // digit 0: the key's top bits
                }
            }
            if (COLS == 4 && (j0 & 3) == 0 && j + COLS <= n) {
                *(uint32_t *) (sf.w.flags + j0) = fl_all;   // four flag bytes at once
            } else {
#pragma unroll
                for (int c = 0; c < COLS; ++c)
                    if (j + c < n) sf.w.flags[j0 + c] = (uint8_t) (fl_all >> (8 * c));
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < NS * SEL_BINS; e += UF_T) {
        const uint32_t c = (&lhist[0][0])[e];
        if (c) atomicAdd(&sf.w.hist[e], c);   // hist[0][s][bin], s < NS
    }
}

// Pass p: histogram of digit p of the not-yet-decided candidates.  Pass 0 also builds keys and flags; there a
// workgroup walks one contiguous chunk of the instances and keeps the chunk's marked instances (the half of the
// previous working set that stays, csmosolver.cpp:65-71: never candidates) as a bit field in LDS.
#define SEL_CHUNK_MAX 65536
template <int NS>   // NS = g.n_sides: two sides need half the LDS of four, and a workgroup finds room on a busy CU sooner
__global__ __launch_bounds__(SEL_T) void sel_pass_kernel(SelWorkspace w, const double *__restrict__ f,
                                                         const int *__restrict__ y, const double *__restrict__ alpha,
                                                         int64_t n, double Cp, double Cn, SelGeom g, int p,
                                                         const int *__restrict__ marked, int n_marked) {
    __shared__ uint32_t lhist[NS][SEL_BINS];
    __shared__ SelState st[SEL_MAX_SIDES];
    __shared__ uint32_t scratch[SEL_T + 16];
    __shared__ uint32_t mark_bits[SEL_CHUNK_MAX / 32];
    const int tid = threadIdx.x;
    if (p == 0) {
        if (tid < g.n_sides) {
            SelState s0;
            s0.pk = 0; s0.pi = 0; s0.k_rem = g.k; s0.done = 0; s0.pad = 0;
            st[tid] = s0;
            if (blockIdx.x == 0) w.state[tid] = s0;   // the state before digit 0, for the next pass
        }
        __syncthreads();
    } else {
        sel_advance_state(w, g, p, st, scratch);
        if (blockIdx.x == 0 && tid < g.n_sides) w.state[p * SEL_MAX_SIDES + tid] = st[tid];
    }
    bool any = false;
    for (int s = 0; s < g.n_sides; ++s) any |= !st[s].done;
    if (!any) return;
    for (int e = tid; e < NS * SEL_BINS; e += SEL_T) (&lhist[0][0])[e] = 0;
    bool is_key; int shift, width;
    sel_digit_geom(p, g.idx_bits, is_key, shift, width);
    const uint32_t dmask = (1u << width) - 1;
    if (p == 0) {
        const int64_t chunk = (n + gridDim.x - 1) / gridDim.x;   // <= SEL_CHUNK_MAX (the host sizes the grid)
        const int64_t lo = (int64_t) blockIdx.x * chunk;
        const int64_t hi = lo + chunk < n ? lo + chunk : n;
        for (int e = tid; e < (int) ((chunk + 31) >> 5); e += SEL_T) mark_bits[e] = 0;
        __syncthreads();
        for (int i = tid; i < n_marked; i += SEL_T) {
            const int64_t id = marked[i];
            if (id >= lo && id < hi) atomicOr(&mark_bits[(id - lo) >> 5], 1u << ((id - lo) & 31));
        }
        __syncthreads();
        for (int64_t j = lo + tid; j < hi; j += SEL_T) {
            const double a = alpha[j];
            const double yy = (double) y[j];
            const uint64_t key = f_to_key(f[j]);
            uint32_t fl = 0;
            if (!((mark_bits[(j - lo) >> 5] >> ((j - lo) & 31)) & 1u)) fl = sel_flags(a, yy, Cp, Cn, g.n_sides);
            w.keys[j] = key;
            w.flags[j] = (uint8_t) fl;
            sel_count(g, st, lhist, p, is_key, shift, dmask, key, fl, j);
        }
    } else {
        __syncthreads();
        const int64_t stride = (int64_t) gridDim.x * SEL_T;
        for (int64_t j = (int64_t) blockIdx.x * SEL_T + tid; j < n; j += stride) {
            const uint32_t fl = w.flags[j];
            if (!fl) continue;
            sel_count(g, st, lhist, p, is_key, shift, dmask, w.keys[j], fl, j);
        }
    }
    __syncthreads();
    uint32_t *gh = w.hist + (size_t) p * SEL_MAX_SIDES * SEL_BINS;
    for (int e = tid; e < g.n_sides * SEL_BINS; e += SEL_T) {
        const uint32_t c = (&lhist[0][0])[e];
        if (c) atomicAdd(&gh[e], c);
    }
}

// Appends the selected candidates among instances first, first + stride, ... to their sides' lists; st is the
// final state of every side.
__device__ __forceinline__ void sel_collect(const SelWorkspace &w, int64_t n, const SelGeom &g, const SelState *st,
                                            int64_t first, int64_t stride) {
    for (int64_t j = first; j < n; j += stride) {
        const uint32_t fl = w.flags[j];
        if (!fl) continue;
        const uint64_t key = w.keys[j];
        for (int s = 0; s < g.n_sides; ++s) {
            if (!(fl & (1u << s))) continue;
            const bool desc = sel_side_descending(s, g.n_sides);
            const uint64_t k2 = desc ? ~key : key;
            const uint32_t i2 = desc ? g.idx_mask - (uint32_t) j : (uint32_t) j;
            int cmp;
            if (st[s].k_rem == 0 && st[s].done) {
                cmp = 1;  // nothing to take on this side
            } else {
                // compare on the digits this side consumed before it was decided
                cmp = sel_cmp_prefix(k2, i2, st[s], (int) st[s].pad, g.idx_bits);
            }
            if (cmp <= 0) {
                const uint32_t pos = atomicAdd(&w.count[s], 1u);
                if (pos < MAX_WS) {
                    w.list_key[s * MAX_WS + pos] = k2;
                    w.list_idx[s * MAX_WS + pos] = i2;
                }
            }
        }
    }
}

__device__ __forceinline__ bool sel_undecided(const SelGeom &g, const SelState *st) {
    bool any = false;
    for (int s = 0; s < g.n_sides; ++s) any |= !st[s].done;
    return any;
}

// After the grid-wide passes every side is normally decided: then this kernel appends every selected candidate
// to its side's list.  If a boundary bucket is still too large it does nothing, and sel_final_kernel goes on.
__global__ __launch_bounds__(SEL_T) void sel_compact_kernel(SelWorkspace w, int64_t n, SelGeom g, int p_full) {
    __shared__ SelState st[SEL_MAX_SIDES];
    __shared__ uint32_t scratch[SEL_T + 16];
    sel_advance_state(w, g, p_full, st, scratch);
    if (sel_undecided(g, st)) return;
    sel_collect(w, n, g, st, (int64_t) blockIdx.x * SEL_T + threadIdx.x, (int64_t) gridDim.x * SEL_T);
}

// Digits p_full .. n_pass-1 and the lists, by one workgroup: only when the grid-wide digits left a boundary
// bucket too large to take whole (many equal f values, e.g. the first iteration of a training run, where the
// instance index has to break the ties).  The workgroup walks the candidates once per remaining digit: slow but
// rare, and it keeps a launch per digit out of every call.  st holds the state before digit p_full.
__device__ void sel_tail(const SelWorkspace &w, int64_t n, const SelGeom &g, int p_full, SelState *st,
                         uint32_t (*lhist)[SEL_BINS], uint32_t *scratch) {
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int p = p_full; p < g.n_pass && sel_undecided(g, st); ++p) {
        if (tid < g.n_sides) w.state[p * SEL_MAX_SIDES + tid] = st[tid];
        for (int e = tid; e < g.n_sides * SEL_BINS; e += nt) (&lhist[0][0])[e] = 0;
        __syncthreads();
        bool is_key; int shift, width;
        sel_digit_geom(p, g.idx_bits, is_key, shift, width);
        const uint32_t dmask = (1u << width) - 1;
        for (int64_t j = tid; j < n; j += nt) {
            const uint32_t fl = w.flags[j];
            if (fl) sel_count(g, st, lhist, p, is_key, shift, dmask, w.keys[j], fl, j);
        }
        __syncthreads();
        uint32_t *gh = w.hist + (size_t) p * SEL_MAX_SIDES * SEL_BINS;
        for (int e = tid; e < g.n_sides * SEL_BINS; e += nt) gh[e] = (&lhist[0][0])[e];
        __syncthreads();   // sel_advance_state reads state[p] and hist[p] back from memory
        sel_advance_state(w, g, p + 1, st, scratch);
    }
    sel_collect(w, n, g, st, tid, nt);
    __syncthreads();
}

// Final step: sort each side's list, replay the alternating scan, write the selection.
__device__ __forceinline__ bool comp_less(uint64_t ka, uint32_t ia, uint64_t kb, uint32_t ib) {
    return ka < kb || (ka == kb && ia < ib);
}

// (fold_n > 0: the ids are also written modulo fold_n to out_folded, for problems whose instances are stacked
// copies of fold_n stored rows)
template <int NS>   // NS = g.n_sides (32 KB of LDS with two sides, 64 KB with four)
__global__ __launch_bounds__(MAX_WS) void sel_final_kernel(SelWorkspace w, int64_t n, SelGeom g, int p_full,
                                                           int *__restrict__ out, int fold_n, int *__restrict__ out_folded) {
    __shared__ uint64_t sk[NS][MAX_WS];
    __shared__ uint32_t si[NS][MAX_WS];
    __shared__ int pos_other[NS][MAX_WS];  // position of the same instance in the paired side's list, or -1
    __shared__ int cnt[SEL_MAX_SIDES];
    __shared__ int conflict;
    __shared__ SelState st[SEL_MAX_SIDES];
    __shared__ uint32_t scratch[SEL_T + 16];
    const int tid = threadIdx.x;
    // the test sel_compact_kernel made: if it left the lists empty, the remaining digits and the lists are made here
    sel_advance_state(w, g, p_full, st, scratch);
    if (sel_undecided(g, st)) sel_tail(w, n, g, p_full, st, (uint32_t (*)[SEL_BINS]) &sk[0][0], scratch);
    if (tid < SEL_MAX_SIDES) {
        // (an atomic read: the lengths were counted with atomics, by this workgroup itself on the slow path)
        int c = tid < g.n_sides ? (int) __hip_atomic_load(&w.count[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
        cnt[tid] = c > MAX_WS ? MAX_WS : c;
    }
    if (tid == 0) conflict = 0;
    __syncthreads();
    for (int s = 0; s < g.n_sides; ++s) {
        if (tid < cnt[s]) {
            sk[s][tid] = w.list_key[s * MAX_WS + tid];
            si[s][tid] = w.list_idx[s * MAX_WS + tid];
        } else {
            sk[s][tid] = ~0ull;
            si[s][tid] = ~0u;
        }
    }
    __syncthreads();
    sel_arm(w, g, p_full, tid, MAX_WS);   // everything this call needed from the workspace is in LDS now
    // Bitonic sort, ascending composite, all sides at once.  Thread t owns compare-exchange pair t & 511 of
    // side t >> 9 (and of side 2 + (t >> 9) when there are four), so every thread works in every stage.  With
    // strides up to 64 a wavefront's 64 pairs cover one closed block of 128 entries, stage after stage: such
    // stages only need the wavefront's own LDS accesses kept in order, not a workgroup barrier.
    int m_sort = 2;
    for (int s = 0; s < g.n_sides; ++s)
        while (m_sort < cnt[s]) m_sort <<= 1;   // padding entries are already in place behind the longest list
    const int pr = tid & (MAX_WS / 2 - 1);
    for (int size = 2; size <= m_sort; size <<= 1) {
        for (int strd = size >> 1; strd > 0; strd >>= 1) {
            const int lo = ((pr & ~(strd - 1)) << 1) | (pr & (strd - 1));
            const int hi = lo | strd;
            const bool asc = (lo & size) == 0;
            if (hi < m_sort) {
                for (int s = tid >> 9; s < g.n_sides; s += 2) {
                    const uint64_t ka = sk[s][lo], kb = sk[s][hi];
                    const uint32_t ia = si[s][lo], ib = si[s][hi];
                    const bool sw = asc ? comp_less(kb, ib, ka, ia) : comp_less(ka, ia, kb, ib);
                    if (sw) { sk[s][lo] = kb; sk[s][hi] = ka; si[s][lo] = ib; si[s][hi] = ia; }
                }
            }
            const int next_strd = strd > 1 ? strd >> 1 : (2 * size <= m_sort ? size : 0);
            if (strd > 64 || next_strd > 64) {
                __syncthreads();
            } else {
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");   // LDS accesses of a wavefront complete in order
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
    __syncthreads();
    // real instance ids; descending sides stored idx_mask - id
    for (int s = 0; s < g.n_sides; ++s)
        if (tid < cnt[s] && sel_side_descending(s, g.n_sides)) si[s][tid] = g.idx_mask - si[s][tid];
    __syncthreads();
    // position of each entry in the paired side's list (binary search on the paired side's order)
    const int half = g.n_sides / 2;
    for (int s = 0; s < g.n_sides; ++s) {
        const int o = s < half ? s + half : s - half;
        int res = -1;
        if (tid < cnt[s]) {
            // key of this instance as the paired side stores it: complement of ours (or of the complement)
            const uint64_t k_here = sk[s][tid];
            const uint64_t k_o = ~k_here;
            const uint32_t id = si[s][tid];
            const uint32_t i_o = sel_side_descending(o, g.n_sides) ? g.idx_mask - id : id;
            int lo = 0, hi = cnt[o];
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                const uint32_t im = sel_side_descending(o, g.n_sides) ? g.idx_mask - si[o][mid] : si[o][mid];
                if (comp_less(sk[o][mid], im, k_o, i_o)) lo = mid + 1; else hi = mid;
            }
            if (lo < cnt[o] && sk[o][lo] == k_o && si[o][lo] == id) res = lo;
        }
        pos_other[s][tid] = res;
    }
    __syncthreads();
    const int k = (int) g.k;
    // fast path: round r takes entry r of every side, provided no entry is already consumed by its pair
    const int per = k / g.n_sides;
    bool ok = (k % g.n_sides) == 0;
    for (int s = 0; s < g.n_sides; ++s) ok = ok && cnt[s] >= per;
    if (ok && tid < per) {
        for (int s = 0; s < g.n_sides; ++s) {
            const int po = pos_other[s][tid];
            if (po < 0) continue;
            // the paired side has consumed `tid` entries before this pick if it runs later in the round,
            // `tid + 1` if it runs earlier
            const int o = s < half ? s + half : s - half;
            const int consumed = o < s ? tid + 1 : tid;
            if (po < consumed) atomicOr(&conflict, 1);
        }
    }
    __syncthreads();
    if (ok && !conflict) {
        if (tid < per)
            for (int s = 0; s < g.n_sides; ++s) {
                const int id = (int) si[s][tid];
                out[tid * g.n_sides + s] = id;
                if (fold_n > 0) out_folded[tid * g.n_sides + s] = id % fold_n;
            }
        return;
    }
    // general path: replay the scan serially (small problems, or sides that run dry)
    if (tid == 0) {
        int ptr[SEL_MAX_SIDES] = {0, 0, 0, 0};
        int n_sel = 0;
        while (n_sel < k) {
            bool progressed = false;
            for (int s = 0; s < g.n_sides; ++s) {
                const int o = s < half ? s + half : s - half;
                while (ptr[s] < cnt[s] && pos_other[s][ptr[s]] >= 0 && pos_other[s][ptr[s]] < ptr[o]) ++ptr[s];
                if (ptr[s] < cnt[s] && n_sel < k) {
                    if (fold_n > 0) out_folded[n_sel] = (int) si[s][ptr[s]] % fold_n;
                    out[n_sel++] = (int) si[s][ptr[s]];
                    ++ptr[s];
                    progressed = true;
                }
            }
            if (!progressed) break;
        }
        for (; n_sel < k; ++n_sel) {
            out[n_sel] = -1;
            if (fold_n > 0) out_folded[n_sel] = -1;
        }
    }
}

// The ids a selection has just written, sent to the host by the device itself: host_ids is host memory the device
// can write (pinned, mapped); the ids go there (modulo fold_n when fold_n > 0) and then, behind a system-wide fence,
// `word` goes to host_ids[word_at], which the host polls.  One small kernel in stream order behind the selection,
// in place of a copy, an event and the wake-up of a thread that sleeps on it.
__global__ __launch_bounds__(256) void report_ids_kernel(const int *__restrict__ ids, int n_ids, int fold_n,
                                                         int *__restrict__ host_ids, int word_at, int word) {
    for (int t = threadIdx.x; t < n_ids; t += 256) {
        const int id = ids[t];
        host_ids[t] = fold_n > 0 && id >= 0 ? id % fold_n : id;
    }
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_store(&host_ids[word_at], word, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// ------------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------------
template <typename TK, int COLS, int UNROLL, int NS>
static void launch_update_f(double *f, const double *alpha_diff, int ws_size, const void *k_rows, const int *slots,
                            int64_t ld, int64_t n, int repeat, const SelFuse &sf, hipStream_t s) {
    const int64_t vecs = (n + COLS - 1) / COLS;                        // column vectors, one per thread
    int64_t grid = (vecs + UF_T - 1) / UF_T;
    int vec_per_wg = UF_T;
    if (COLS > 1) {
        // (with one column per thread a workgroup's share has to start on a cache line, or every wavefront's
        // 256-byte read touches three lines instead of two: measured slower than the uneven grid)
        const int64_t per_cu = (vecs + 248 * UF_T - 1) / (248 * UF_T);   // workgroups per CU
        grid = 248 * per_cu;
        vec_per_wg = (int) ((vecs + grid - 1) / grid);
    }
    hipLaunchKernelGGL((update_f_kernel<TK, COLS, UNROLL, NS>), dim3((unsigned) grid), dim3(UF_T), 0, s, f, alpha_diff, ws_size,
                       (const TK *) k_rows, slots, ld, n, repeat, vec_per_wg, sf);
}

// The variant of the kernel for the row type, alignment and size at hand.
template <int NS>
static void dispatch_update_f(double *f, const double *alpha_diff, int ws_size, const void *k_rows, int row_type, const int *slots,
                              int64_t ld, int64_t n, int repeat, const SelFuse &sf, hipStream_t s) {
    // 16-byte loads need every row start 16-byte aligned and the last vector inside the padded row; with few
    // columns one column per thread and more rows in flight keeps more of the chip busy
    const bool big = n >= (int64_t) UF_T * 1024;
    const bool aligned = (uintptr_t) k_rows % 16 == 0;
    if (row_type == TSVM_ROW_F32) {
        if (big && aligned && ld % 4 == 0 && ld >= (n + 3) / 4 * 4) launch_update_f<float, 4, 8, NS>(f, alpha_diff, ws_size, k_rows, slots, ld, n, repeat, sf, s);
        else launch_update_f<float, 1, 32, NS>(f, alpha_diff, ws_size, k_rows, slots, ld, n, repeat, sf, s);
    } else {
        if (big && aligned && ld % 2 == 0 && ld >= (n + 1) / 2 * 2) launch_update_f<double, 2, 8, NS>(f, alpha_diff, ws_size, k_rows, slots, ld, n, repeat, sf, s);
        else launch_update_f<double, 1, 16, NS>(f, alpha_diff, ws_size, k_rows, slots, ld, n, repeat, sf, s);
    }
}

static SelGeom sel_geom(int64_t n, int n_select, int nu) {
    SelGeom g;
    g.n_sides = nu ? 4 : 2;
    int bits = 1;
    while (((int64_t) 1 << bits) < n) ++bits;
    g.idx_bits = bits;
    g.idx_mask = (uint32_t) (((uint64_t) 1 << bits) - 1);
    g.n_pass = 6 + (bits + SEL_DIGIT - 1) / SEL_DIGIT;
    g.k = (uint32_t) n_select;
    return g;
}

static SelWorkspace sel_workspace(void *workspace, int64_t n) {
    SelWorkspace w;
    sel_carve((void *) (((uintptr_t) workspace + 255) & ~(uintptr_t) 255), n, &w);
    return w;
}

// first_pass 1: digit 0 has been counted already, by update_f_kernel, on a workspace left by an earlier selection
static int select_working_set(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                              const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                              bool armed, int fold_n, int *out_folded, int first_pass, tsvm_stream stream) {
    TSVM_REQUIRE(f && y && alpha && out && workspace, "tsvm_select_working_set: null pointer");
    TSVM_REQUIRE(n >= 1 && n <= 0x7fffffffLL, "tsvm_select_working_set: n %lld outside [1, 2^31)", (long long) n);
    TSVM_REQUIRE(n_select >= 0 && n_select <= MAX_WS, "tsvm_select_working_set: n_select %d outside [0, %d]", n_select,
                 MAX_WS);
    TSVM_REQUIRE(n_marked >= 0 && (n_marked == 0 || marked), "tsvm_select_working_set: bad marked list");
    TSVM_REQUIRE(fold_n >= 0 && (fold_n == 0 || out_folded), "tsvm_select_working_set: bad fold arguments");
    if (n_select == 0) return 0;
    hipStream_t s = tsvm_s(stream);
    const SelWorkspace w = sel_workspace(workspace, n);
    const SelGeom g = sel_geom(n, n_select, nu);
    // The first three digits (33 bits of f) are counted by the whole chip, the rest (rarely needed) by one
    // workgroup.  Near convergence the free support vectors crowd within epsilon of the threshold, so the third
    // digit is usually the one that separates them.
    const int p_full = n > ((int64_t) 1 << 26) ? 4 : 3;   // < n_pass, which is at least 7
    // two workgroups per CU: every workgroup adds its histogram to the global one with atomics, and with more
    // workgroups those take longer than the counting they spread (n = 800k: 92 us per call with 1024, 80 with 496)
    unsigned grid = (unsigned) std::min<int64_t>((n + SEL_T - 1) / SEL_T, 496);
    if ((n + grid - 1) / grid > SEL_CHUNK_MAX) grid = (unsigned) ((n + SEL_CHUNK_MAX - 1) / SEL_CHUNK_MAX);
    if (!armed) {
        hipLaunchKernelGGL(sel_init_kernel, dim3(p_full * SEL_MAX_SIDES * SEL_BINS / 1024), dim3(256), 0, s, w, g, p_full);
        TSVM_LAUNCH_CHECK();
    }
    for (int p = first_pass; p < p_full; ++p) {
        if (nu) hipLaunchKernelGGL(sel_pass_kernel<4>, dim3(grid), dim3(SEL_T), 0, s, w, f, y, alpha, n, Cp, Cn, g, p, marked, n_marked);
        else hipLaunchKernelGGL(sel_pass_kernel<2>, dim3(grid), dim3(SEL_T), 0, s, w, f, y, alpha, n, Cp, Cn, g, p, marked, n_marked);
        TSVM_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(sel_compact_kernel, dim3(grid), dim3(SEL_T), 0, s, w, n, g, p_full);
    TSVM_LAUNCH_CHECK();
    if (nu) hipLaunchKernelGGL(sel_final_kernel<4>, dim3(1), dim3(MAX_WS), 0, s, w, n, g, p_full, out, fold_n, out_folded);
    else hipLaunchKernelGGL(sel_final_kernel<2>, dim3(1), dim3(MAX_WS), 0, s, w, n, g, p_full, out, fold_n, out_folded);
    TSVM_LAUNCH_CHECK();
    return 0;
}

extern "C" {

int tsvm_update_f(double *f, const double *alpha_diff, int ws_size, const void *k_rows, int row_type, const int *slots,
                  int64_t ld, int64_t n_cols, int repeat, tsvm_stream stream) {
    TSVM_REQUIRE(f && alpha_diff && k_rows, "tsvm_update_f: null pointer");
    TSVM_REQUIRE(ws_size >= 0 && n_cols >= 0 && ld >= n_cols && repeat >= 1, "tsvm_update_f: bad size (ws=%d n=%lld ld=%lld)",
                 ws_size, (long long) n_cols, (long long) ld);
    TSVM_REQUIRE(row_type == TSVM_ROW_F64 || row_type == TSVM_ROW_F32, "tsvm_update_f: unknown row type %d", row_type);
    if (n_cols == 0 || ws_size == 0) return 0;
    dispatch_update_f<0>(f, alpha_diff, ws_size, k_rows, row_type, slots, ld, n_cols, repeat, SelFuse(), tsvm_s(stream));
    TSVM_LAUNCH_CHECK();
    return 0;
}

int tsvm_update_f_select(double *f, const double *alpha_diff, int ws_size, const void *k_rows, int row_type, const int *slots,
                         int64_t ld, int64_t n_cols, int repeat, const int *y, const double *alpha, double Cp, double Cn,
                         const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace, int *out_folded,
                         tsvm_stream stream) {
    TSVM_REQUIRE(f && alpha_diff && k_rows, "tsvm_update_f_select: null pointer");
    TSVM_REQUIRE(ws_size >= 0 && n_cols >= 1 && ld >= n_cols && repeat >= 1 && repeat <= UF_MAX_REPEAT,
                 "tsvm_update_f_select: bad size (ws=%d n=%lld ld=%lld repeat=%d)", ws_size, (long long) n_cols, (long long) ld, repeat);
    TSVM_REQUIRE(row_type == TSVM_ROW_F64 || row_type == TSVM_ROW_F32, "tsvm_update_f_select: unknown row type %d", row_type);
    TSVM_REQUIRE(y && alpha && out && workspace, "tsvm_update_f_select: null pointer");
    TSVM_REQUIRE(n_select >= 1 && n_select <= MAX_WS, "tsvm_update_f_select: n_select %d outside [1, %d]", n_select, MAX_WS);
    TSVM_REQUIRE(n_marked >= 0 && (n_marked == 0 || marked), "tsvm_update_f_select: bad marked list");
    const int64_t n = n_cols * repeat;
    TSVM_REQUIRE(n <= 0x7fffffffLL, "tsvm_update_f_select: %lld instances, at most 2^31 - 1", (long long) n);
    SelFuse sf;
    sf.w = sel_workspace(workspace, n);
    sf.g = sel_geom(n, n_select, nu);
    sf.y = y; sf.alpha = alpha; sf.Cp = Cp; sf.Cn = Cn; sf.marked = marked; sf.n_marked = n_marked;
    hipStream_t s = tsvm_s(stream);
    if (nu) dispatch_update_f<4>(f, alpha_diff, ws_size, k_rows, row_type, slots, ld, n_cols, repeat, sf, s);
    else dispatch_update_f<2>(f, alpha_diff, ws_size, k_rows, row_type, slots, ld, n_cols, repeat, sf, s);
    TSVM_LAUNCH_CHECK();
    return select_working_set(f, y, alpha, n, Cp, Cn, marked, n_marked, out, n_select, nu, workspace, true,
                              out_folded ? (int) n_cols : 0, out_folded, 1, stream);
}

int tsvm_report_ids(const int *ids, int n_ids, int fold_n, int *host_ids, int word_at, int word, tsvm_stream stream) {
    TSVM_REQUIRE(ids && host_ids, "tsvm_report_ids: null pointer");
    TSVM_REQUIRE(n_ids >= 0 && n_ids <= MAX_WS && word_at >= n_ids && fold_n >= 0, "tsvm_report_ids: bad size (n_ids=%d word_at=%d fold_n=%d)",
                 n_ids, word_at, fold_n);
    hipLaunchKernelGGL(report_ids_kernel, dim3(1), dim3(256), 0, tsvm_s(stream), ids, n_ids, fold_n, host_ids, word_at, word);
    TSVM_LAUNCH_CHECK();
    return 0;
}

size_t tsvm_select_workspace(int64_t n) {
    if (n < 0) return 0;
    return sel_carve(nullptr, n, nullptr) + 256;
}

int tsvm_select_working_set(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                            const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                            tsvm_stream stream) {
    return select_working_set(f, y, alpha, n, Cp, Cn, marked, n_marked, out, n_select, nu, workspace, false, 0, nullptr, 0, stream);
}

int tsvm_select_working_set_again(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                                  const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                                  tsvm_stream stream) {
    return select_working_set(f, y, alpha, n, Cp, Cn, marked, n_marked, out, n_select, nu, workspace, true, 0, nullptr, 0, stream);
}

int tsvm_select_working_set_folded(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                                   const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                                   int again, int fold_n, int *out_folded, tsvm_stream stream) {
    TSVM_REQUIRE(fold_n >= 1, "tsvm_select_working_set_folded: fold_n %d < 1", fold_n);
    return select_working_set(f, y, alpha, n, Cp, Cn, marked, n_marked, out, n_select, nu, workspace, again != 0, fold_n, out_folded,
                              0, stream);
}

}  // extern "C"
