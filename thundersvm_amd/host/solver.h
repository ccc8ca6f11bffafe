// CSMOSolver / NuSMOSolver: the outer SMO loop (src/thundersvm/solver/csmosolver.cpp:10-121,
// nusmosolver.cpp) driving the gfx950 kernels.  f, alpha, y, the working set and the ws x n kernel
// rows stay in HBM for the whole solve; per outer iteration the host reads back 16 bytes (diff).
#pragma once
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
};

class CSMOSolver {
public:
    virtual ~CSMOSolver() = default;
    void solve(const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha, float_type &rho,
               std::vector<float_type> &f_val, float_type eps, float_type Cp, float_type Cn, int ws_size,
               int out_max_iter) const;

    mutable SolverStats stats;
    SolverTrace *trace = nullptr;
    bool profile = false;
    // Budget of the HBM kernel-row cache in bytes: -1 = half of the free device memory, 0 = no cache.
    long long cache_bytes = -1;
    // Run the local solver and the chip-wide get_rows concurrently on two streams.  Off by default: the
    // solver is a chain of dependent loads, and measured next to get_rows each of its iterations takes
    // 3.6x longer (2.4 ms instead of 0.66 ms per call at n = 800,000), which cancels the overlap.
    bool overlap_streams = false;

protected:
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
