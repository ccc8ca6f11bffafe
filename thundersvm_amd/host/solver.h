// CSMOSolver / NuSMOSolver: the outer SMO loop (src/thundersvm/solver/csmosolver.cpp:10-121,
// nusmosolver.cpp) driving the gfx950 kernels.  f, alpha, y, the working set and the ws x n kernel
// rows stay in HBM for the whole solve; per outer iteration the host reads back 16 bytes (diff).
#pragma once
#include <string>
#include "kernelmatrix.h"

struct SolverTrace {          // optional per-iteration record (parity debugging and tests)
    int cap_iters = 0;
    std::vector<double> diff;   // [iters][2]
    std::vector<int> ws;        // [iters][ws_size]
    int ws_size = 0;
};

struct SolverStats {
    long long n_iter = 0;       // outer iterations
    long long local_iter = 0;   // inner iterations summed
    double obj = 0;
    // accumulated device time per phase in ms (only filled when profile == true)
    double ms_select = 0, ms_get_rows = 0, ms_local = 0, ms_update_f = 0;
    double ms_wall = 0, ms_setup = 0;   // host wall-clock of the whole solve / of everything before the first iteration
    // kernel-row cache
    long long cache_lookups = 0, cache_hits = 0;
    long long cache_rows = 0;     // capacity in rows (0: cache not used)
    bool cache_disabled = false;  // switched off after the warm-up because it was not hitting
    int ws_size = 0;              // working-set size of the solve
    long long rows_computed = 0;  // kernel rows get_rows produced (cache misses), summed over the outer iterations
    long long update_rows = 0;    // kernel rows update_f read (non-zero alpha_diff entries), counted only when profiling
    int solver_xcd = -1;          // several class pairs in flight: the die this pair's local solver ran on (-1: not known)
    double ms_start = 0, ms_end = 0;   // host clock at the solve's start and end, in ms since the process's first solve
};

class SolveTask;

namespace tsvm {
// Spins until *word no longer holds `pending`.  Every 200 ms `stream_state()` is asked for the state of the stream
// that is to write the word (hipSuccess: everything enqueued has run; hipErrorNotReady: still running; anything else
// is thrown as that error).  Throws std::runtime_error when the stream has drained without the word changing, or
// when timeout_ms have passed: a solver kernel that never finishes must not hang its caller for good (the
// reference's blocking copies surface such failures through CUDA_CHECK, include/thundersvm/util/common.h:33-42).
void wait_while_pending(const volatile uint64_t *word, uint64_t pending, long long timeout_ms, hipError_t (*stream_state)(void *),
                        void *stream);
long long solver_timeout_ms();   // TSVM_SOLVER_TIMEOUT_MS, default 300,000
}  // namespace tsvm

class CSMOSolver {
public:
    virtual ~CSMOSolver() = default;
    void solve(const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha, float_type &rho,
               std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn, int ws_size,
               int out_max_iter) const;

    mutable SolverStats stats;
    SolverTrace *trace = nullptr;
    bool profile = false;
    // Budget of the HBM kernel-row cache in bytes: -1 = nine tenths of the free device memory, 0 = no cache.
    long long cache_bytes = -1;

protected:
    friend class SolveTask;
    virtual bool is_nu() const { return false; }
    virtual float_type calculate_rho(const std::vector<float_type> &f_val, const std::vector<int> &y,
                                     std::vector<float_type> &alpha, float_type Cp, float_type Cn) const;
    void init_f(const std::vector<float_type> &alpha, const std::vector<int> &y, const KernelMatrix &k_mat,
                float_type *d_f) const;
    float_type calculate_obj(const std::vector<float_type> &f_val, const std::vector<float_type> &alpha,
                             const std::vector<int> &y) const;
};

class NuSMOSolver : public CSMOSolver {
public:
    explicit NuSMOSolver(bool for_svr) : for_svr(for_svr) {}

protected:
    bool is_nu() const override { return true; }
    float_type calculate_rho(const std::vector<float_type> &f_val, const std::vector<int> &y,
                             std::vector<float_type> &alpha, float_type Cp, float_type Cn) const override;

private:
    bool for_svr;
};

// One SMO solve as a resumable sequence of enqueue steps.  CSMOSolver::solve runs one task to completion; a
// one-vs-one run keeps several tasks (class pairs) in flight and enqueues their steps in turn.  The local
// solver is a single workgroup bound by latency; it runs on a stream restricted to compute units of its own
// (one per XCD and lane), everything else of the task on a stream restricted to the remaining ones, so the
// solver of an iteration runs next to that iteration's get_rows.  Where such streams cannot be had the task
// uses one ordinary stream, and the driver of several tasks keeps their solver phases apart from their
// chip-wide phases with events.  The steps of one outer iteration:
//   enqueue_select, enqueue_block, enqueue_solver, enqueue_rows, enqueue_update, finish_iteration
// (enqueue_rows before enqueue_block when the block is gathered from the stored rows: block_needs_rows()).
class SolveTask {
public:
    // pool / pool_bytes: device memory for the kernel rows (nullptr: taken from the process-wide arena
    // according to solver.cache_bytes).  lane / n_lanes: which of the tasks advanced side by side this one is;
    // every lane's local solver gets CUs of its own.
    SolveTask(const CSMOSolver &solver, const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha,
              float_type &rho, std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn, int ws_size,
              int out_max_iter, void *pool = nullptr, size_t pool_bytes = 0, int lane = 0, int n_lanes = 1);
    ~SolveTask();
    SolveTask(const SolveTask &) = delete;
    SolveTask &operator=(const SolveTask &) = delete;

    void enqueue_select();
    void enqueue_rows();
    void enqueue_block();
    void enqueue_solver();
    void enqueue_update();
    bool finish_iteration();   // waits for this iteration's diff; true once the solve is complete and its results are written
    // For a caller that advances several tasks from one thread without blocking on any of them:
    // rows_ready(): enqueue_rows would not wait (the newly selected ids the host-side row cache needs have arrived, or
    // are not needed); iteration_done(): finish_iteration would not wait.  iteration_done() throws like the blocking
    // wait when the solver's stream has drained without a report or nothing has been heard for the time-out.
    bool rows_ready() const;
    bool iteration_done();
    bool block_needs_rows() const;
    bool split_streams() const;   // the local solver runs on CUs of its own, next to this task's (and other tasks') chip-wide kernels
    hipStream_t stream() const;
    const SolverStats &stats() const;
    static size_t min_pool_bytes(const KernelMatrix &k_mat, int ws_size);
    static bool cu_split_available();   // the device is one whose CUs this code knows how to divide

private:
    struct Impl;
    Impl *impl_;
};
