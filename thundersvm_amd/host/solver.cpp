#include "solver.h"
#include "row_cache.h"

#include <chrono>
#include <map>
#include <mutex>
#include <climits>
#include <cmath>
#include <algorithm>

using tsvm::abi_check;
using tsvm::DeviceBuffer;
using tsvm::RowCache;

namespace {

inline bool up_set(float_type a, float_type y, float_type Cp, float_type Cn) { return (y > 0 && a < Cp) || (y < 0 && a > 0); }
inline bool low_set(float_type a, float_type y, float_type Cp, float_type Cn) { return (y > 0 && a > 0) || (y < 0 && a < Cn); }
inline bool free_sv(float_type a, float_type y, float_type Cp, float_type Cn) { return a > 0 && (y > 0 ? a < Cp : a < Cn); }

struct PhaseTimer {
    bool on;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    explicit PhaseTimer(bool on) : on(on) {
        if (on) { TSVM_HIP_CHECK(hipEventCreate(&e0)); TSVM_HIP_CHECK(hipEventCreate(&e1)); }
    }
    ~PhaseTimer() { if (on) { (void) hipEventDestroy(e0); (void) hipEventDestroy(e1); } }
    hipStream_t stream = nullptr;
    void begin() { if (on) TSVM_HIP_CHECK(hipEventRecord(e0, stream)); }
    void end(double &acc) {
        if (!on) return;
        TSVM_HIP_CHECK(hipEventRecord(e1, stream));
        TSVM_HIP_CHECK(hipEventSynchronize(e1));
        float ms = 0;
        TSVM_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        acc += ms;
    }
};

// CU-masked streams are kept for the life of the process and handed from one solve to the next: creating one
// makes a hardware queue, which costs far more than a solve's other set-up (and every few creations the runtime
// spends tens of milliseconds on queue housekeeping).  Keyed by device, lane and lane count (which fix the masks).
struct LaneStreams {
    hipStream_t chip = nullptr, solver = nullptr;
    bool in_use = false;
};
// the streams of all lanes of one lane count on one device: made together, because the chip-wide mask leaves out
// exactly the CUs on which the lanes' solvers land
struct LaneGroup {
    std::vector<LaneStreams> lanes;
};
std::mutex g_masked_mutex;
std::map<long long, std::vector<LaneGroup>> g_masked;   // keyed by device and lane count

// the clock reading of the process's first solve: solves report their start and end relative to it
std::chrono::steady_clock::time_point process_epoch() {
    static const std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
    return t0;
}

// The pooled streams are destroyed by an atexit handler, registered when the first one is made and therefore run
// before the HIP runtime's own tear-down (which, under a profiler, crashed on queues still alive at that point).
void destroy_masked_streams() {
    std::lock_guard<std::mutex> lock(g_masked_mutex);
    for (auto &kv : g_masked)
        for (LaneGroup &g : kv.second)
            for (LaneStreams &m : g.lanes) {
                if (m.solver) (void) hipStreamDestroy(m.solver);
                if (m.chip) (void) hipStreamDestroy(m.chip);
            }
    g_masked.clear();
}

// Makes the 2 * n_lanes streams of a group.  Bit i of a CU mask names CU i/8 of XCD i%8 on the 8-XCD, 256-CU part (a
// mask has to leave every XCD at least one CU: workgroups are dealt to the XCDs in turn).  Every solver stream gets
// CU 0 of every XCD, and lane l's solver is launched so that it runs on XCD l (tsvm_c_smo_solve_block_on_xcd: eight
// workgroups, one per XCD, the one on XCD l solves, the others leave at once).  The lanes thus share the eight CUs
// without sharing a CU, each solver behind another L2.  The chip-wide streams get every CU but those the solvers
// really run on, CU 0 of XCDs 0 .. n_lanes-1: 255 CUs for one lane, 248 for eight.  (On the CUs the two masks share,
// a solver launch's seven idle workgroups wait for room like any workgroup; the solver's result is behind them only in
// stream order, and they are gone long before it is done.)
bool make_lane_group(int n_lanes, LaneGroup &g) {
    g.lanes.assign(n_lanes, LaneStreams());
    uint32_t small[8] = {0xffu, 0, 0, 0, 0, 0, 0, 0};
    uint32_t big[8] = {~((1u << n_lanes) - 1u), ~0u, ~0u, ~0u, ~0u, ~0u, ~0u, ~0u};   // all but CU 0 of XCDs 0 .. n_lanes-1
    bool ok = true;
    for (int l = 0; l < n_lanes && ok; ++l) {
        ok = hipExtStreamCreateWithCUMask(&g.lanes[l].solver, 8, small) == hipSuccess;
        if (!ok) { g.lanes[l].solver = nullptr; break; }
        ok = hipExtStreamCreateWithCUMask(&g.lanes[l].chip, 8, big) == hipSuccess;
        if (!ok) g.lanes[l].chip = nullptr;
    }
    if (!ok) {
        (void) hipGetLastError();
        for (LaneStreams &m : g.lanes) {
            if (m.solver) (void) hipStreamDestroy(m.solver);
            if (m.chip) (void) hipStreamDestroy(m.chip);
        }
        g.lanes.clear();
    }
    return ok;
}

}  // namespace

namespace tsvm {

long long solver_timeout_ms() {
    const char *e = getenv("TSVM_SOLVER_TIMEOUT_MS");
    const long long v = e ? atoll(e) : 0;
    return v > 0 ? v : 300000;
}

void wait_while_pending(const volatile uint64_t *word, uint64_t pending, long long timeout_ms, hipError_t (*stream_state)(void *),
                        void *stream) {
    using clock = std::chrono::steady_clock;
    const auto start = clock::now();
    // (asking the runtime about the stream puts a marker into it: only done when the wait is suspiciously long)
    auto next_check = start + std::chrono::milliseconds(200);
    for (unsigned long long spins = 1; *word == pending; ++spins) {
        if (spins % 4096 != 0) continue;
        const auto now = clock::now();
        if (now < next_check) continue;
        next_check = now + std::chrono::milliseconds(200);
        const hipError_t e = stream_state(stream);
        if (e == hipSuccess) {   // everything enqueued has run: the write is on its way or was never made
            if (*word == pending) throw std::runtime_error("SolveTask: the local solver finished without reporting");
        } else if (e != hipErrorNotReady) {
            TSVM_HIP_CHECK(e);
        }
        if (now - start > std::chrono::milliseconds(timeout_ms))
            throw std::runtime_error("SolveTask: no word from the local solver after " + std::to_string(timeout_ms) +
                                     " ms (TSVM_SOLVER_TIMEOUT_MS); the device may be hung");
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);
}

}  // namespace tsvm

struct SolveTask::Impl {
    const CSMOSolver &solver;
    const KernelMatrix &k_mat;
    const std::vector<int> &y;
    std::vector<float_type> &alpha;
    float_type &rho;
    std::vector<float_type> &f_val;
    const float_type eps, Cp, Cn;
    const int ws_size, out_max_iter;

    // Kernel rows are stored once per distinct data row: n_u columns wide, addressed by the folded id
    // (id % n_u); f, alpha and y keep the reference's n = rep * n_u entries.
    const int n, n_u, rep, row_type;
    const size_t row_esz;
    const int q;
    const int64_t ld;   // row stride in elements: rows stay 32-byte aligned
    const bool nu;
    const int ldk;
    SolverStats stats;
    std::chrono::steady_clock::time_point wall0;

    // d_slots_a holds three tables of ws entries back to back: the slot of every working-set row, then the ids and
    // the slots of the rows to compute; the host fills the same layout in h_slots and sends it with one copy.
    DeviceBuffer<int> d_y, d_ws, d_slots_a, d_slots_b, d_ws_folded;
    DeviceBuffer<float_type> d_alpha, d_f, d_alpha_diff;
    DeviceBuffer<unsigned char> d_sel_ws;
    DeviceBuffer<kernel_type> d_kws;
    // The working set of iteration t is the window d_ws[ws_off .. ws_off + ws_size): the ids kept from the previous
    // set (its second half) are the first half of the next window, so the window just moves on by q per iteration
    // and nothing is copied (csmosolver.cpp:65-71 copies q ids per iteration); at the end of the buffer the last
    // half is moved back to the start.
    static constexpr int WS_HALVES = 64;
    int ws_off = 0, sel_off = 0;   // window of the current iteration / of the latest selection launched
    const int *ws_ids() const { return d_ws.data() + ws_off; }
    // working set as folded ids: a second window, at the same offsets, that the selection fills along with the first
    const int *ws_u() const { return rep > 1 ? d_ws_folded.data() + ws_off : d_ws.data() + ws_off; }

    // The chip-wide work of a task is enqueued on stream `sa` (`ids` is the stream the newly selected ids are read
    // back on for the host-side cache bookkeeping: the same one).
    hipStream_t sa = nullptr, ids = nullptr;
    hipEvent_t selected = nullptr, diff_ready = nullptr;
    // A task that runs alone splits the chip: the local solver (one workgroup, a chain of dependent steps) gets a
    // stream `ss` restricted to one CU of every XCD, everything else runs on `sa`, restricted to the other CUs.
    // The solver then runs next to this iteration's get_rows at nearly its stand-alone speed; sharing CUs with a
    // chip-wide kernel it runs two to three times slower, which is why tasks in lockstep keep the phases apart.
    hipStream_t ss = nullptr;
    hipEvent_t block_done = nullptr, solved = nullptr;
    bool split = false;
    // Once the cache holds every row there is no get_rows left to run next to the solver; the iteration then
    // stays on `sa` from start to end and saves the two hand-overs between the streams.
    bool on_one_stream = false, alone = true;   // alone: no other task's kernels on the chip
    // When the previous iteration computed many rows this one probably will too, and its get_rows will outlast the
    // solver by far.  The block is then computed on the solver's few CUs (several times slower, still well inside
    // the time get_rows takes), so that get_rows need not wait for it on the chip-wide stream.
    int last_rows_computed = 0;
    bool block_on_solver_cus = false;
    long long masked_key = 0;
    int masked_lane = 0;
    int solver_xcd = -1, solver_epoch = 0;   // masked streams: the XCD this lane's solver is launched onto, launches so far
    tsvm::DeviceBuffer<int> d_gate;

    void *k_rows = nullptr;
    bool caching = false;
    RowCache cache;
    std::vector<int> cur_slots, cur_ids, miss_ids, miss_slots;
    // Once the cache holds every row the host's bookkeeping has nothing left to decide: the device gets the
    // table id -> slot, and from then on an iteration takes its slots from it (no ids to the host, no slot
    // table back) and gathers the solver's block from the stored rows.
    bool all_cached = false;
    DeviceBuffer<int> d_slot_of;
    // A store with a slot for every instance never evicts, so which slot a new row gets can be decided on the
    // device (next free one, tsvm_row_slots_assign) and the host hears of it afterwards, with the diff: no ids to
    // the host and no slot table back between the selection and get_rows.  (Dense rows, unfolded problems.)
    bool device_cache = false;
    DeviceBuffer<int> d_cache_state;                  // slots in use, rows to compute
    int *h_cache_info = nullptr, *d_cache_info = nullptr;   // the same two numbers in pinned host memory
    int *h_ids = nullptr, *h_slots = nullptr;
    int *d_ids_host = nullptr;   // h_ids as the device addresses it
    // diff (the solver's 16 bytes for the host, smo_kernel.cpp:87,120) lives in pinned host memory that the device
    // writes directly: no copy in the stream between update_f and the next selection
    double *h_diff = nullptr, *d_diff = nullptr;
    // The host does not wait for an event behind update_f (a marker in the stream costs the device about 6 us
    // before the next kernel starts): it marks the word the solver writes last as pending before it enqueues the
    // solver (diff[1] for c_smo_solve; nu_smo_solve reports diff[0] only, smo_kernel.cpp:283, and writes it at its
    // end), and waits for that word to change.  Both kernels put a system-wide fence before that last write.
    // Everything the host enqueues meanwhile is ordered by the streams.
    static constexpr uint64_t DIFF_PENDING = 0x7ff8dead00000001ull;   // a NaN no computation produces
    bool wait_by_event = false;
    hipStream_t solver_stream = nullptr;
    volatile uint64_t *diff_word() const { return reinterpret_cast<volatile uint64_t *>(h_diff + (nu ? 0 : 1)); }
    // Set when a wait for the solver gave up: the device is taken to be hung, and the destructor then touches neither
    // the streams nor the device memory (synchronising, destroying or freeing would block for good); the task's streams
    // stay marked as in use, its memory stays allocated, and the error reaches the caller.
    bool abandoned = false;
    void wait_for_diff() {
        try {
            tsvm::wait_while_pending(diff_word(), DIFF_PENDING, tsvm::solver_timeout_ms(),
                                     [](void *st) { return hipStreamQuery((hipStream_t) st); }, solver_stream);
        } catch (...) {
            abandoned = true;
            throw;
        }
    }
    // the same wait as a poll (one look per call; the stream is asked, and the time-out checked, every 200 ms)
    std::chrono::steady_clock::time_point solver_enqueued, next_stream_check;
    bool diff_arrived() {
        if (wait_by_event) {
            const hipError_t e = hipEventQuery(diff_ready);
            if (e == hipSuccess) return true;
            if (e != hipErrorNotReady) TSVM_HIP_CHECK(e);
            return false;
        }
        if (*diff_word() != DIFF_PENDING) {
            __atomic_thread_fence(__ATOMIC_ACQUIRE);
            return true;
        }
        const auto now = std::chrono::steady_clock::now();
        if (now < next_stream_check) return false;
        next_stream_check = now + std::chrono::milliseconds(200);
        const hipError_t e = hipStreamQuery(solver_stream);
        if (e == hipSuccess) {
            if (*diff_word() == DIFF_PENDING) {
                abandoned = true;
                throw std::runtime_error("SolveTask: the local solver finished without reporting");
            }
        } else if (e != hipErrorNotReady) {
            abandoned = true;
            TSVM_HIP_CHECK(e);
        }
        if (now - solver_enqueued > std::chrono::milliseconds(tsvm::solver_timeout_ms())) {
            abandoned = true;
            throw std::runtime_error("SolveTask: no word from the local solver (TSVM_SOLVER_TIMEOUT_MS); the device may be hung");
        }
        return false;
    }
    // The new ids come to the host from the device itself (tsvm_report_ids, in stream order behind the selection):
    // h_ids[ws_size] takes the number of the report once its ids are in h_ids.
    int ids_seq = 0;
    bool ids_arrived() const {
        if (!(caching && !all_cached && !device_cache)) return true;
        if (*(volatile int *) (h_ids + ws_size) != ids_seq) return false;
        __atomic_thread_fence(__ATOMIC_ACQUIRE);
        return true;
    }
    void wait_for_ids() {
        using clock = std::chrono::steady_clock;
        const auto start = clock::now();
        auto next_check = start + std::chrono::milliseconds(200);
        for (unsigned long long spins = 1; !ids_arrived(); ++spins) {
            if (spins % 4096 != 0) continue;
            const auto now = clock::now();
            if (now < next_check) continue;
            next_check = now + std::chrono::milliseconds(200);
            const hipError_t e = hipStreamQuery(ids);
            if (e == hipSuccess) {
                if (!ids_arrived()) {
                    abandoned = true;
                    throw std::runtime_error("SolveTask: the selection finished without reporting its ids");
                }
            } else if (e != hipErrorNotReady) {
                abandoned = true;
                TSVM_HIP_CHECK(e);
            }
            if (now - start > std::chrono::milliseconds(tsvm::solver_timeout_ms())) {
                abandoned = true;
                throw std::runtime_error("SolveTask: no ids from the selection (TSVM_SOLVER_TIMEOUT_MS); the device may be hung");
            }
        }
    }
    int rotation_base = 0;   // iteration at which d_slots_a was valid
    long long window_lookups = 0, window_hits = 0, window_first = 0, first_touches = 0;
    std::vector<char> seen;        // instances whose row has been asked for at least once
    int off_below_percent = 5;     // a full cache is switched off when fewer of a window's repeated lookups hit (TSVM_CACHE_OFF_BELOW)
    const int *slots = nullptr;

    int max_iter = 0;
    long long local_iter = 0;
    int same_local_diff_cnt = 0, swap_local_diff_cnt = 0;
    float_type previous_local_diff = INFINITY, last_local_diff = INFINITY, second_last_local_diff = INFINITY;
    PhaseTimer timer;
    bool select_ahead = false, block_first = false, select_enqueued = false;
    bool fuse_select = false;   // update_f also makes the first pass of the selection that follows
    int iter = 0;

    Impl(const CSMOSolver &solver, const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha,
         float_type &rho, std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn, int ws_size,
         int out_max_iter, void *pool, size_t pool_bytes, int lane, int n_lanes)
        : solver(solver), k_mat(k_mat), y(y), alpha(alpha), rho(rho), f_val(f_val), eps(eps), Cp(Cp), Cn(Cn), ws_size(ws_size),
          out_max_iter(out_max_iter), n((int) k_mat.n_instances()), n_u((int) k_mat.n_columns()), rep(k_mat.repeat()),
          row_type(k_mat.row_type()), row_esz(k_mat.row_elem_size()), q(ws_size / 2), ld(((int64_t) n_u + 7) / 8 * 8),
          nu(solver.is_nu()), ldk(tsvm_smo_solve_block_ld(ws_size)), timer(solver.profile) {
        if (ws_size < 1 || ws_size > n || ws_size > 1024)
            throw std::invalid_argument("SolveTask: working-set size " + std::to_string(ws_size) + " for " + std::to_string(n) +
                                        " instances (1 .. min(instances, 1024))");
        wall0 = std::chrono::steady_clock::now();
        (void) process_epoch();
        stats.ws_size = ws_size;
        d_y.resize(n); d_ws.resize((size_t) WS_HALVES * q + ws_size); d_slots_a.resize(3 * (size_t) ws_size); d_slots_b.resize(ws_size);
        if (rep > 1) d_ws_folded.resize(d_ws.size());
        d_alpha.resize(n); d_f.resize(n); d_alpha_diff.resize(ws_size);
        d_sel_ws.resize(tsvm_select_workspace(n));
        d_kws.resize((size_t) ws_size * ldk);
        d_y.upload(y.data(), n);
        d_alpha.upload(alpha.data(), n);
        d_f.upload(f_val.data(), n);
        d_alpha_diff.zero();
        d_kws.zero();
        alone = n_lanes == 1;
        split = !solver.profile && create_split_streams(lane, n_lanes);
        if (split) {
            solver_xcd = lane;
            d_gate.resize(4);
            d_gate.zero();
        }
        if (!split) {
            TSVM_HIP_CHECK(hipStreamCreateWithFlags(&sa, hipStreamNonBlocking));
            ss = sa;
        }
        // The read-back of the newly selected ids follows the selection on the same stream: it is enqueued before
        // anything else of the iteration, so it waits for nothing but the selection.
        ids = sa;
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&selected, hipEventDisableTiming));
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&diff_ready, hipEventDisableTiming));
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&block_done, hipEventDisableTiming));
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&solved, hipEventDisableTiming));

        // Kernel rows live in slots of one pool.  With a cache the pool holds up to pool_rows rows and the
        // host tracks which instance sits in which slot; without one it holds exactly ws rows.
        long long pool_rows = ws_size;
        const long long cache_bytes = solver.cache_bytes;
        tsvm::RowArena &arena = tsvm::RowArena::instance();
        if (cache_bytes != 0 && n_u > ws_size) {
            const long long budget = pool ? (long long) pool_bytes : cache_bytes > 0 ? cache_bytes : (long long) arena.auto_budget();
            const long long fit = budget / (long long) (ld * row_esz);
            // a cache worth having holds a few working sets; one that turns out not to hit is switched off below
            if (fit >= 4LL * ws_size) pool_rows = std::min<long long>(n_u, fit);
        }
        caching = pool_rows > ws_size;
        const size_t need = (size_t) pool_rows * ld * row_esz;
        if (pool) {
            if (need > pool_bytes) throw std::runtime_error("SolveTask: kernel-row pool too small");
            k_rows = pool;
        } else {
            k_rows = arena.acquire(need, cache_bytes < 0);
        }
        if (caching) {
            cache.init(n_u, (int) pool_rows);
            seen.assign(n_u, 0);
            if (const char *e = getenv("TSVM_CACHE_OFF_BELOW")) off_below_percent = atoi(e);
            stats.cache_rows = pool_rows;
            if ((size_t) n_u <= pool_rows) d_slot_of.resize(n_u);
            device_cache = d_slot_of.size() == (size_t) n_u && rep == 1 && k_mat.dense_layout();
        }
        if (device_cache) {
            TSVM_HIP_CHECK(hipMemset(d_slot_of.data(), 0xff, sizeof(int) * (size_t) n_u));
            d_cache_state.resize(2);
            d_cache_state.zero();
            TSVM_HIP_CHECK(hipHostMalloc((void **) &h_cache_info, 2 * sizeof(int), hipHostMallocMapped | hipHostMallocCoherent));
            TSVM_HIP_CHECK(hipHostGetDevicePointer((void **) &d_cache_info, h_cache_info, 0));
            h_cache_info[0] = h_cache_info[1] = 0;
        }
        cur_slots.resize(ws_size);
        cur_ids.resize(ws_size);
        TSVM_HIP_CHECK(hipHostMalloc((void **) &h_diff, 2 * sizeof(double), hipHostMallocMapped | hipHostMallocCoherent));
        TSVM_HIP_CHECK(hipHostGetDevicePointer((void **) &d_diff, h_diff, 0));
        TSVM_HIP_CHECK(hipHostMalloc((void **) &h_ids, (ws_size + 16) * sizeof(int), hipHostMallocMapped | hipHostMallocCoherent));
        TSVM_HIP_CHECK(hipHostGetDevicePointer((void **) &d_ids_host, h_ids, 0));
        h_ids[ws_size] = 0;
        TSVM_HIP_CHECK(hipHostMalloc((void **) &h_slots, 3 * ws_size * sizeof(int)));
        h_diff[0] = h_diff[1] = 0;
        if (!caching) {
            for (int t = 0; t < ws_size; ++t) cur_slots[t] = t;
            upload_rotation(cur_slots);
        }
        solver.init_f(alpha, y, k_mat, d_f.data());
        TSVM_HIP_CHECK(hipDeviceSynchronize());   // uploads, fills and init_f ran on the default stream

        max_iter = std::max(100000, ws_size > INT_MAX / 100 ? INT_MAX : 100 * ws_size);
        timer.stream = sa;
        wait_by_event = timer.on;   // phase timing reads its own events after every phase anyway
        if (solver.trace) {
            solver.trace->ws_size = ws_size;
            solver.trace->diff.clear();
            solver.trace->ws.clear();
        }
        // The next selection is enqueued before the host has seen this iteration's diff, so the device goes
        // straight from update_f into it; if the diff then says stop, that selection was simply not needed.
        // (Not when tracing, which reads the working set back after each iteration, nor when profiling.)
        select_ahead = !solver.trace && !solver.profile;
        // With stacked copies (SVR) a thread of update_f has twice the instances to classify after its rows have
        // streamed by, each behind memory reads that wait on a saturated HBM: measured slower than the separate pass.
        fuse_select = rep == 1 && q > 0;
        // The solver reads the ws x ws block of the kernel matrix.  With few features the block is cheap to
        // compute on its own, without the stored rows, so it and the solver can be enqueued before the host
        // does the cache bookkeeping.  With many features that small launch (64 workgroups walking the whole
        // feature range) costs more than it hides, and the block is gathered from the stored rows instead.
        // (When the solver has CUs of its own the block always comes first: the solver then runs while the rows
        // are computed.)
        block_first = split || k_mat.n_features() < 256;
        stats.ms_setup = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count();
    }

    ~Impl() {
        if (abandoned) {   // nothing that could wait for the device
            for (DeviceBuffer<int> *b : {&d_y, &d_ws, &d_slots_a, &d_slots_b, &d_ws_folded, &d_gate, &d_slot_of, &d_cache_state}) b->abandon();
            for (DeviceBuffer<float_type> *b : {&d_alpha, &d_f, &d_alpha_diff, &d_kws}) b->abandon();
            d_sel_ws.abandon();
            return;
        }
        if (sa) (void) hipStreamSynchronize(sa);   // a selection enqueued ahead may still be running
        if (ss && ss != sa) (void) hipStreamSynchronize(ss);
        if (ids && ids != sa) { (void) hipStreamSynchronize(ids); (void) hipStreamDestroy(ids); }
        if (split) release_split_streams();         // masked streams go back to the pool
        else if (sa) (void) hipStreamDestroy(sa);
        if (block_done) (void) hipEventDestroy(block_done);
        if (solved) (void) hipEventDestroy(solved);
        if (selected) (void) hipEventDestroy(selected);
        if (diff_ready) (void) hipEventDestroy(diff_ready);
        if (h_diff) (void) hipHostFree(h_diff);
        if (h_cache_info) (void) hipHostFree(h_cache_info);
        if (h_ids) (void) hipHostFree(h_ids);
        if (h_slots) (void) hipHostFree(h_slots);
    }

    // Two streams with disjoint CU masks from the pool (make_lane_group above).  Anything unexpected (another CU
    // count, a call failing, TSVM_NO_CU_SPLIT set) leaves the task on one plain stream.
    bool create_split_streams(int lane, int n_lanes) {
        if (!SolveTask::cu_split_available() || n_lanes < 1 || n_lanes > 8 || lane < 0 || lane >= n_lanes) return false;
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return false;
        masked_key = (long long) dev * 16 + n_lanes;
        masked_lane = lane;
        std::lock_guard<std::mutex> lock(g_masked_mutex);
        std::vector<LaneGroup> &groups = g_masked[masked_key];
        LaneStreams *mine = nullptr;
        for (LaneGroup &g : groups)
            if (!g.lanes[lane].in_use) { mine = &g.lanes[lane]; break; }
        if (!mine) {
            LaneGroup g;
            if (!make_lane_group(n_lanes, g)) return false;
            static bool registered = false;
            if (!registered) {
                registered = true;
                atexit(destroy_masked_streams);
            }
            groups.push_back(std::move(g));
            mine = &groups.back().lanes[lane];
        }
        mine->in_use = true;
        sa = mine->chip;
        ss = mine->solver;
        return true;
    }

    void release_split_streams() {
        std::lock_guard<std::mutex> lock(g_masked_mutex);
        for (LaneGroup &g : g_masked[masked_key])
            if (g.lanes[masked_lane].chip == sa) g.lanes[masked_lane].in_use = false;
    }

    // without a cache the slot tables just alternate: the two halves of the working set swap places
    // every iteration, so the rows kept from the previous iteration are re-addressed, never copied
    // (the reference copies q*n values per iteration, csmosolver.cpp:75)
    void upload_rotation(const std::vector<int> &slots_now) {
        std::vector<int> other(ws_size);
        for (int t = 0; t < ws_size; ++t) other[t] = slots_now[(t + q) % ws_size];
        d_slots_a.upload(slots_now.data(), ws_size);
        d_slots_b.upload(other.data(), ws_size);
    }

    // Working-set selection of iteration `it`: the first one picks ws_size ids, later ones keep the last
    // half of the previous set and pick q new ids (csmosolver.cpp:63-77).
    // Moves the window to where the selection of iteration `it` > 0 writes: q ids further, or back to the start of
    // the buffer with the half that stays copied in front.
    void advance_window() {
        int next = sel_off + q;
        if (next + ws_size > (int) d_ws.size()) {
            TSVM_HIP_CHECK(hipMemcpyAsync(d_ws.data(), d_ws.data() + next, sizeof(int) * q, hipMemcpyDeviceToDevice, sa));
            if (rep > 1)
                TSVM_HIP_CHECK(hipMemcpyAsync(d_ws_folded.data(), d_ws_folded.data() + next, sizeof(int) * q,
                                              hipMemcpyDeviceToDevice, sa));
            next = 0;
        }
        sel_off = next;
    }

    void launch_select(int it) {
        const int n_sel = it == 0 ? ws_size : q;
        hipStream_t sel = sa;
        if (it == 0) sel_off = 0;
        else advance_window();
        const int *kept = it == 0 ? nullptr : d_ws.data() + sel_off;            // the half that stays: no candidates
        int *out = d_ws.data() + sel_off + (it == 0 ? 0 : q);
        if (rep > 1) {
            abi_check(tsvm_select_working_set_folded(d_f.data(), d_y.data(), d_alpha.data(), n, Cp, Cn, kept, it == 0 ? 0 : q, out,
                                                     n_sel, nu, d_sel_ws.data(), it > 0, n_u,
                                                     d_ws_folded.data() + sel_off + (it == 0 ? 0 : q), sel));
        } else if (it == 0) {
            abi_check(tsvm_select_working_set(d_f.data(), d_y.data(), d_alpha.data(), n, Cp, Cn, kept, 0, out, n_sel, nu,
                                              d_sel_ws.data(), sel));
        } else {
            abi_check(tsvm_select_working_set_again(d_f.data(), d_y.data(), d_alpha.data(), n, Cp, Cn, kept, q, out, n_sel, nu,
                                                    d_sel_ws.data(), sel));
        }
    }

    void enqueue_select() {
        const int n_new = iter == 0 ? ws_size : q;
        const int first_new = iter == 0 ? 0 : q;
        timer.begin();
        if (!select_enqueued) launch_select(iter);
        select_enqueued = false;
        ws_off = sel_off;
        timer.end(stats.ms_select);
        if (caching && !all_cached && !device_cache) {
            // the new ids travel to the host: written there by a small kernel behind the selection
            abi_check(tsvm_report_ids(ws_ids() + first_new, n_new, 0, d_ids_host, ws_size, ++ids_seq, ids));
        }
    }

    void enqueue_rows() {
        const int n_new = iter == 0 ? ws_size : q;
        const int first_new = iter == 0 ? 0 : q;
        if (caching && all_cached) {
            stats.cache_lookups += n_new;
            stats.cache_hits += n_new;
            last_rows_computed = 0;
            return;
        }
        timer.begin();
        if (device_cache) {
            int *miss_ids = d_slots_a.data() + ws_size, *miss_slots = d_slots_a.data() + 2 * ws_size;
            abi_check(tsvm_row_slots_assign(ws_u() + first_new, n_new, d_slot_of.data(), d_cache_state.data(), miss_ids, miss_slots,
                                            ws_u(), ws_size, d_slots_a.data(), d_cache_info, sa));
            k_mat.get_rows_counted(miss_ids, n_new, d_cache_state.data() + 1, k_rows, ld, miss_slots, sa);
            slots = d_slots_a.data();
        } else if (caching) {
            // look the new ids up and compute only the rows that are not cached
            if (iter > 0) {
                // the first half of the previous working set leaves; the second half moves up and stays pinned
                // (known without the new ids: done while they are still on their way)
                for (int t = 0; t < q; ++t) cache.release(cur_slots[t]);
                for (int t = 0; t < q; ++t) {
                    cur_ids[t] = cur_ids[t + q];
                    cur_slots[t] = cur_slots[t + q];
                }
            }
            miss_ids.clear();
            miss_slots.clear();
            wait_for_ids();
            for (int t = 0; t < n_new; ++t) {
                const int id = h_ids[t] % n_u;   // a second member with the same folded id hits the slot just assigned
                int s = cache.lookup(id);
                stats.cache_lookups++;
                if (!seen[id]) { seen[id] = 1; ++first_touches; }
                if (s >= 0) {
                    stats.cache_hits++;
                } else {
                    s = cache.insert(id);
                    if (s < 0) throw std::runtime_error("SolveTask: kernel-row cache smaller than a working set");
                    miss_ids.push_back(id);
                    miss_slots.push_back(s);
                }
                cur_ids[first_new + t] = id;
                cur_slots[first_new + t] = s;
            }
            int *h_miss_ids = h_slots + ws_size, *h_miss_slots = h_slots + 2 * ws_size;
            std::copy(cur_slots.begin(), cur_slots.end(), h_slots);
            std::copy(miss_ids.begin(), miss_ids.end(), h_miss_ids);
            std::copy(miss_slots.begin(), miss_slots.end(), h_miss_slots);
            const int n_miss = (int) miss_ids.size();
            last_rows_computed = n_miss;
            stats.rows_computed += n_miss;
            TSVM_HIP_CHECK(hipMemcpyAsync(d_slots_a.data(), h_slots, sizeof(int) * (n_miss ? 3 * (size_t) ws_size : (size_t) ws_size),
                                          hipMemcpyHostToDevice, sa));
            if (n_miss) {
                k_mat.get_rows(d_slots_a.data() + ws_size, n_miss, k_rows, ld, d_slots_a.data() + 2 * ws_size, sa);
            }
            slots = d_slots_a.data();
            if (cache.used == n_u && d_slot_of.size() == (size_t) n_u) {
                TSVM_HIP_CHECK(hipMemcpyAsync(d_slot_of.data(), cache.slot_of.data(), sizeof(int) * (size_t) n_u,
                                              hipMemcpyHostToDevice, sa));
                all_cached = true;
            }
            // A cache that has started evicting and still does not hit only costs the id read-back:
            // every 64 iterations, if fewer than 5 % of the window's lookups hit, fall back to rotation.
            // (A cache that can hold every row is never switched off: its misses are first touches.)
            if (cache.cap < n_u && cache.used == cache.cap && iter % 64 == 63) {
                // (lookups of rows never asked for before cannot hit and say nothing about the cache: only the
                // others count, once they are at least a quarter of the window's lookups)
                const long long dl = stats.cache_lookups - window_lookups, dh = stats.cache_hits - window_hits;
                const long long again = dl - (first_touches - window_first);
                if (again * 4 >= dl && dh * 100 < again * off_below_percent) {
                    TSVM_HIP_CHECK(hipStreamSynchronize(sa));
                    caching = false;
                    stats.cache_disabled = true;
                    if (rep > 1) {
                        // Stacked problems may hold one slot at two positions of the working set (instance i and
                        // its copy i + n_u share a stored row).  Rotation needs a slot of its own at every position:
                        // the positions take slots 0 .. ws-1 and all ws rows are computed into them once, as the
                        // path without a cache does at its first iteration.
                        for (int t = 0; t < ws_size; ++t) cur_slots[t] = t;
                        upload_rotation(cur_slots);
                        k_mat.get_rows(ws_u(), ws_size, k_rows, ld, d_slots_a.data(), sa);
                        last_rows_computed = ws_size;
                    } else {
                        upload_rotation(cur_slots);
                    }
                    rotation_base = iter;
                }
            }
            if (iter % 64 == 63) { window_lookups = stats.cache_lookups; window_hits = stats.cache_hits; window_first = first_touches; }
        } else {
            const bool on_a = ((iter - rotation_base) % 2) == 0;
            slots = on_a ? d_slots_a.data() : d_slots_b.data();
            // new rows go to the slots the dropped rows occupied
            last_rows_computed = n_new;
            stats.rows_computed += n_new;
            k_mat.get_rows(ws_u() + first_new, n_new, k_rows, ld, slots + first_new, sa);
        }
        timer.end(stats.ms_get_rows);
    }

    void enqueue_block() {
        timer.begin();
        on_one_stream = !split || (alone && all_cached);
        // (Dense rows only: the CSR block takes too long on eight CUs.  Both launches are matrix-core work with the
        // same cost per value; the block plus the solver's ~0.4 ms has to fit into the time of the rows.)
        block_on_solver_cus = false;
        if (!on_one_stream && alone && block_first && k_mat.dense_layout() && !all_cached) {
            const double per_value = 2.0 * ((k_mat.n_features() + 15) / 16 * 16) / 6.6e13;   // seconds on the whole chip
            const double t_block = per_value * 32.0 * 0.56 * ws_size * (double) ws_size;   // on 8 of 256 CUs; 72 of its 128 tiles
            const double t_rows = per_value * (double) last_rows_computed * n_u;
            block_on_solver_cus = t_block + 0.4e-3 <= t_rows;
        }
        if (caching && all_cached) {
            abi_check(tsvm_smo_gather_block_by_id(k_rows, row_type, d_slot_of.data(), ld, ws_u(), ws_size, d_kws.data(), row_type,
                                                  d_slots_a.data(), sa));
            slots = d_slots_a.data();
        } else if (block_on_solver_cus) {
            TSVM_HIP_CHECK(hipEventRecord(selected, sa));   // the selection is the last thing enqueued on sa
            TSVM_HIP_CHECK(hipStreamWaitEvent(ss, selected, 0));
            k_mat.get_block(ws_u(), ws_size, d_kws.data(), ldk, ss);
        } else if (block_first) {
            k_mat.get_block(ws_u(), ws_size, d_kws.data(), ldk, sa);
        } else {
            abi_check(tsvm_smo_gather_block(k_rows, row_type, slots, ld, ws_u(), ws_size, d_kws.data(), row_type, sa));
        }
        timer.end(stats.ms_local);
        if (!on_one_stream && !block_on_solver_cus) TSVM_HIP_CHECK(hipEventRecord(block_done, sa));
    }

    void enqueue_solver() {
        timer.begin();
        hipStream_t st = on_one_stream ? sa : ss;
        solver_stream = st;
        if (!wait_by_event) {
            *diff_word() = DIFF_PENDING;
            __atomic_thread_fence(__ATOMIC_RELEASE);
        }
        solver_enqueued = std::chrono::steady_clock::now();
        next_stream_check = solver_enqueued + std::chrono::milliseconds(200);
        if (!on_one_stream && !block_on_solver_cus) TSVM_HIP_CHECK(hipStreamWaitEvent(ss, block_done, 0));
        if (solver_xcd >= 0 && st == ss) {   // on the masked solver stream: elected onto this lane's XCD
            ++solver_epoch;
            if (nu)
                abi_check(tsvm_nu_smo_solve_block_on_xcd(d_y.data(), d_f.data(), d_alpha.data(), d_alpha_diff.data(), ws_ids(), ws_size, Cp,
                                                         d_kws.data(), row_type, k_mat.diag(), eps, d_diff, max_iter, d_gate.data(),
                                                         solver_epoch, solver_xcd, st));
            else
                abi_check(tsvm_c_smo_solve_block_on_xcd(d_y.data(), d_f.data(), d_alpha.data(), d_alpha_diff.data(), ws_ids(), ws_size, Cp,
                                                        Cn, d_kws.data(), row_type, k_mat.diag(), eps, d_diff, max_iter, d_gate.data(),
                                                        solver_epoch, solver_xcd, st));
        } else if (nu) {
            abi_check(tsvm_nu_smo_solve_block(d_y.data(), d_f.data(), d_alpha.data(), d_alpha_diff.data(), ws_ids(), ws_size,
                                              Cp, d_kws.data(), row_type, k_mat.diag(), eps, d_diff, max_iter, st));
        } else {
            abi_check(tsvm_c_smo_solve_block(d_y.data(), d_f.data(), d_alpha.data(), d_alpha_diff.data(), ws_ids(), ws_size,
                                             Cp, Cn, d_kws.data(), row_type, k_mat.diag(), eps, d_diff, max_iter, st));
        }
        timer.end(stats.ms_local);
        if (!on_one_stream) TSVM_HIP_CHECK(hipEventRecord(solved, ss));
    }

    void enqueue_update() {
        if (!on_one_stream) TSVM_HIP_CHECK(hipStreamWaitEvent(sa, solved, 0));   // alpha_diff, alpha and diff come from the solver
        if (select_ahead && fuse_select) {
            // the next selection's first pass over the instances rides on update_f's last one
            advance_window();
            abi_check(tsvm_update_f_select(d_f.data(), d_alpha_diff.data(), ws_size, k_rows, row_type, slots, ld, n_u, rep,
                                           d_y.data(), d_alpha.data(), Cp, Cn, d_ws.data() + sel_off, q, d_ws.data() + sel_off + q, q,
                                           nu, d_sel_ws.data(), rep > 1 ? d_ws_folded.data() + sel_off + q : nullptr, sa));
            select_enqueued = true;
            return;
        }
        timer.begin();
        abi_check(tsvm_update_f(d_f.data(), d_alpha_diff.data(), ws_size, k_rows, row_type, slots, ld, n_u, rep, sa));
        timer.end(stats.ms_update_f);
        if (timer.on) {   // (profiling runs every step to completion anyway) how many rows did update_f have to read?
            std::vector<float_type> ad = d_alpha_diff.to_host();
            for (float_type v : ad) stats.update_rows += v != 0;
        }
        if (wait_by_event) TSVM_HIP_CHECK(hipEventRecord(diff_ready, sa));
        if (select_ahead) {
            launch_select(iter + 1);
            select_enqueued = true;
        }
    }

    bool finish_iteration() {
        if (wait_by_event) TSVM_HIP_CHECK(hipEventSynchronize(diff_ready));
        else wait_for_diff();
        const double diff0 = h_diff[0], diff1 = h_diff[1];
        local_iter += (long long) diff1;
        if (device_cache && !all_cached) {
            // (the two numbers may still be the previous iteration's: the slots are assigned after the solver was
            // enqueued; they only steer the schedule, and the hit count is made exact at the end)
            stats.cache_lookups += iter == 0 ? ws_size : q;
            last_rows_computed = h_cache_info[0];
            all_cached = h_cache_info[1] == n_u;
        }
        SolverTrace *trace = solver.trace;
        if (trace && iter < trace->cap_iters) {
            trace->diff.push_back(diff0);
            trace->diff.push_back(diff1);
            std::vector<int> w = d_ws.to_host();
            trace->ws.insert(trace->ws.end(), w.begin() + ws_off, w.begin() + ws_off + ws_size);
        }
        // stall guards and stopping rule (csmosolver.cpp:86-111)
        if (fabs(diff0 - previous_local_diff) < eps * 0.001) {
            same_local_diff_cnt++;
        } else {
            same_local_diff_cnt = 0;
            previous_local_diff = diff0;
        }
        if (fabs(diff0 - second_last_local_diff) < eps * 0.001) swap_local_diff_cnt++;
        else swap_local_diff_cnt = 0;
        second_last_local_diff = last_local_diff;
        last_local_diff = diff0;
        if (iter % 100 == 0)
            TSVM_LOG << "global iter = " << iter << ", total local iter = " << local_iter << ", diff = " << diff0;
        const bool stalled = (same_local_diff_cnt >= 10 || swap_local_diff_cnt >= 10) && fabs(diff0 - 2.0) > eps;
        if (stalled || diff0 < eps || (out_max_iter != -1 && iter == out_max_iter)) {
            TSVM_HIP_CHECK(hipStreamSynchronize(sa));   // a selection enqueued ahead may still be running
            if (device_cache) {   // every slot in use was one miss
                stats.cache_hits = stats.cache_lookups - h_cache_info[1];
                stats.rows_computed = h_cache_info[1];
            }
            d_alpha.download(alpha.data(), n);
            d_f.download(f_val.data(), n);
            rho = solver.calculate_rho(f_val, y, alpha, Cp, Cn);
            stats.n_iter = iter + 1;
            stats.local_iter = local_iter;
            stats.obj = solver.calculate_obj(f_val, alpha, y);
            TSVM_LOG << "global iter = " << iter << ", total local iter = " << local_iter << ", diff = " << diff0
                     << ", obj = " << stats.obj << ", cache hits " << stats.cache_hits << "/" << stats.cache_lookups;
            if (solver_xcd >= 0 && solver_epoch > 0) stats.solver_xcd = d_gate.to_host()[2];   // where the last solver launch ran
            stats.ms_wall = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - wall0).count();
            stats.ms_start = std::chrono::duration<double, std::milli>(wall0 - process_epoch()).count();
            stats.ms_end = stats.ms_start + stats.ms_wall;
            return true;
        }
        ++iter;
        return false;
    }
};

SolveTask::SolveTask(const CSMOSolver &solver, const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha,
                     float_type &rho, std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn, int ws_size,
                     int out_max_iter, void *pool, size_t pool_bytes, int lane, int n_lanes)
    : impl_(new Impl(solver, k_mat, y, alpha, rho, f_val, eps, Cp, Cn, ws_size, out_max_iter, pool, pool_bytes, lane, n_lanes)) {}
SolveTask::~SolveTask() { delete impl_; }
void SolveTask::enqueue_select() { impl_->enqueue_select(); }
void SolveTask::enqueue_rows() { impl_->enqueue_rows(); }
void SolveTask::enqueue_block() { impl_->enqueue_block(); }
void SolveTask::enqueue_solver() { impl_->enqueue_solver(); }
void SolveTask::enqueue_update() { impl_->enqueue_update(); }
bool SolveTask::finish_iteration() { return impl_->finish_iteration(); }
bool SolveTask::rows_ready() const { return impl_->ids_arrived(); }
bool SolveTask::iteration_done() { return impl_->diff_arrived(); }
bool SolveTask::block_needs_rows() const { return !impl_->block_first; }
bool SolveTask::split_streams() const { return impl_->split; }
bool SolveTask::cu_split_available() {
    if (getenv("TSVM_NO_CU_SPLIT")) return false;
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    return hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n_cu == 256;
}
hipStream_t SolveTask::stream() const { return impl_->sa; }
const SolverStats &SolveTask::stats() const { return impl_->stats; }
size_t SolveTask::min_pool_bytes(const KernelMatrix &k_mat, int ws_size) {
    const size_t ld = (k_mat.n_columns() + 7) / 8 * 8;
    return (size_t) ws_size * ld * k_mat.row_elem_size();
}

void CSMOSolver::solve(const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha,
                       float_type &rho, std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn,
                       int ws_size, int out_max_iter) const {
    SolveTask task(*this, k_mat, y, alpha, rho, f_val, eps, Cp, Cn, ws_size, out_max_iter);
    const bool rows_first = task.block_needs_rows();
    do {
        task.enqueue_select();
        if (rows_first) task.enqueue_rows();
        task.enqueue_block();
        task.enqueue_solver();
        if (!rows_first) task.enqueue_rows();   // the host's cache bookkeeping runs while the solver does
        task.enqueue_update();
    } while (!task.finish_iteration());
    stats = task.stats();
}

// csmosolver.cpp:189-214: f starts from a non-zero alpha in batches of 101 rows.
void CSMOSolver::init_f(const std::vector<float_type> &alpha, const std::vector<int> &y, const KernelMatrix &k_mat,
                        float_type *d_f) const {
    const size_t batch_size = 100;
    const int n_u = (int) k_mat.n_columns();
    const int64_t ld = ((int64_t) n_u + 7) / 8 * 8;
    std::vector<int> idx_vec;
    std::vector<float_type> alpha_diff_vec;
    DeviceBuffer<int> d_idx;
    DeviceBuffer<float_type> d_ad;
    DeviceBuffer<unsigned char> d_rows;
    for (size_t i = 0; i < alpha.size(); ++i) {
        if (alpha[i] != 0) {
            idx_vec.push_back((int) (i % (size_t) n_u));
            alpha_diff_vec.push_back(-alpha[i] * y[i]);
        }
        if (idx_vec.size() > batch_size || (i == alpha.size() - 1 && !idx_vec.empty())) {
            const int m = (int) idx_vec.size();
            if (d_rows.size() == 0) {
                d_idx.resize(batch_size + 1);
                d_ad.resize(batch_size + 1);
                d_rows.resize((batch_size + 1) * (size_t) ld * k_mat.row_elem_size());
            }
            d_idx.upload(idx_vec.data(), m);
            d_ad.upload(alpha_diff_vec.data(), m);
            k_mat.get_rows(d_idx.data(), m, d_rows.data(), ld);
            abi_check(tsvm_update_f(d_f, d_ad.data(), m, d_rows.data(), k_mat.row_type(), nullptr, ld, n_u, k_mat.repeat(), nullptr));
            TSVM_HIP_CHECK(hipStreamSynchronize(nullptr));
            idx_vec.clear();
            alpha_diff_vec.clear();
        }
    }
}

// csmosolver.cpp:167-187
float_type CSMOSolver::calculate_rho(const std::vector<float_type> &f_val, const std::vector<int> &y,
                                     std::vector<float_type> &alpha, float_type Cp, float_type Cn) const {
    int n_free = 0;
    double sum_free = 0;
    float_type up_value = INFINITY, low_value = -INFINITY;
    for (size_t i = 0; i < alpha.size(); ++i) {
        if (free_sv(alpha[i], y[i], Cp, Cn)) { n_free++; sum_free += f_val[i]; }
        if (up_set(alpha[i], y[i], Cp, Cn)) up_value = std::min(up_value, f_val[i]);
        if (low_set(alpha[i], y[i], Cp, Cn)) low_value = std::max(low_value, f_val[i]);
    }
    return n_free != 0 ? sum_free / n_free : -(up_value + low_value) / 2;
}

// csmosolver.cpp:227-239
float_type CSMOSolver::calculate_obj(const std::vector<float_type> &f_val, const std::vector<float_type> &alpha,
                                     const std::vector<int> &y) const {
    float_type obj = 0;
    for (size_t i = 0; i < f_val.size(); ++i) obj += alpha[i] - (f_val[i] + y[i]) * alpha[i] * y[i] / 2;
    return -obj;
}

// nusmosolver.cpp:9-46,120-126
float_type NuSMOSolver::calculate_rho(const std::vector<float_type> &f_val, const std::vector<int> &y,
                                      std::vector<float_type> &alpha, float_type Cp, float_type Cn) const {
    int n_free_p = 0, n_free_n = 0;
    float_type sum_free_p = 0, sum_free_n = 0;
    float_type up_p = INFINITY, up_n = INFINITY, low_p = -INFINITY, low_n = -INFINITY;
    for (size_t i = 0; i < alpha.size(); ++i) {
        const float_type a = alpha[i], nf = -f_val[i];
        if (y[i] > 0) {
            if (a > 0 && a < Cp) { n_free_p++; sum_free_p += f_val[i]; }
            if (up_set(a, y[i], Cp, Cn)) up_p = std::min(up_p, nf);
            if (low_set(a, y[i], Cp, Cn)) low_p = std::max(low_p, nf);
        } else {
            if (a > 0 && a < Cn) { n_free_n++; sum_free_n += nf; }
            if (up_set(a, y[i], Cp, Cn)) up_n = std::min(up_n, nf);
            if (low_set(a, y[i], Cp, Cn)) low_n = std::max(low_n, nf);
        }
    }
    const float_type r1 = n_free_p != 0 ? sum_free_p / n_free_p : -(up_p + low_p) / 2;
    const float_type r2 = n_free_n != 0 ? sum_free_n / n_free_n : -(up_n + low_n) / 2;
    float_type rho = (r1 - r2) / 2;
    if (!for_svr) {   // scale_alpha_rho: nu-SVC rescales, nu-SVR does not
        const float_type r = (r1 + r2) / 2;
        for (auto &a : alpha) a /= r;
        rho /= r;
    }
    return rho;
}
