// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// CPU restatement of ThunderSVM's SMO-training / kernel-evaluation path (the
// reference's USE_CUDA=OFF, USE_DOUBLE=ON semantics), written statement by
// statement from the reference sources cited at each function.  It exists only
// as the checker for the HIP path: nothing in the product library may include,
// link or call this file.  Only the tests, the smoke entry and the bench's CPU
// baseline leg load it.
//
// Arithmetic conventions (chosen where the reference leaves them to the
// compiler, and restated independently by the HIP kernels):
//   * a*b+c patterns that gcc -O3 -march=native contracts are written as
//     explicit fma(); everything else is plain IEEE double.  Build with
//     -ffp-contract=off so nothing else is fused.
//   * Feature values are float32-exact (dataset.cpp:76-79 parses "%f" into a
//     float), so every product x_ik*x_jk is exact in double and a dot product
//     is fully defined by its summation order: ascending stored order of the
//     all-rows matrix' non-zeros (Eigen row-major sparse * dense,
//     kernelmatrix_kernel.cpp:149-160).
//   * expf(): the reference calls libm's expf on a double argument
//     (kernelmatrix_kernel.cpp:71-72,87-89).  expf_mode 0 calls libm here;
//     expf_mode 1 uses orc_expf_det, a restatement of the table-driven
//     algorithm glibc >= 2.27 publishes for expf (32-entry 2^(i/32) table,
//     cubic polynomial, all in double), which the HIP epilogue restates too.
//     tests/test_oracle_expf.py counts how often the two differ on this host.
//   * powf() / tanhf() of the polynomial and sigmoid kernels (kernelmatrix_kernel.cpp:94-108): the same two
//     modes, with orc_powf_det / orc_tanhf_det.
//
// Pinning: tests/test_oracle_golden.py (the reference's fixture, row sets and accuracy / MSE / SV-count goldens),
// tests/test_oracle_expf.py, tests/test_oracle_smo.py, tests/test_oracle_probability.py and tests/test_oracle_pins.py
// (closed forms, brute force, invariants, independent minimisers) check every part on its own: both working-set
// selections against list restatements, both calculate_rho variants against closed forms, the SyncMem counter of
// get_working_set_size against a second restatement.  The composite solver (solve + sort_f + select_working_set +
// c_smo_solve / nu_smo_solve + update_f + rho) is pinned at the optimum: run to a gap of 1e-8 on a strictly convex
// problem it reproduces LibSVM's unique solution for all five SVM types.  What stays "parity unpinned" is only the
// trajectory at the default gap of 1e-3 against a run of the reference itself (no fixture of the reference holds alpha
// or rho, and its CPU build cannot be made here: Eigen is absent).  The poly / sigmoid epilogues use restatements of
// libm's powf / tanhf that give libm's bits on every float argument (tests/test_oracle_expf.py samples the sweeps).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <climits>
#include <string>
#include <utility>
#include <vector>
#include <omp.h>

using std::vector;

extern "C" {

// ---------------------------------------------------------------------------
// parameters (include/thundersvm/svmparam.h:14-29 defaults are set by callers)
// ---------------------------------------------------------------------------
enum { ORC_C_SVC = 0, ORC_NU_SVC = 1, ORC_ONE_CLASS = 2, ORC_EPSILON_SVR = 3, ORC_NU_SVR = 4 };
enum { ORC_LINEAR = 0, ORC_POLY = 1, ORC_RBF = 2, ORC_SIGMOID = 3, ORC_PRECOMPUTED = 4 };

struct orc_param {
    int svm_type;
    int kernel_type;
    int degree;
    int expf_mode;       // 0 = libm expf/powf/tanhf, 1 = the restatements orc_expf_det / orc_powf_det / orc_tanhf_det
    double gamma;
    double coef0;
    double C;
    double nu;
    double p;
    double epsilon;
    long long max_mem_size;  // bytes; reference default 8192 MiB
    int max_iter;            // outer-iteration cap, -1 = none (svmmodel.cpp:417-419)
    int nr_weight;
    const int *weight_label;
    const double *weight;
};

// ---------------------------------------------------------------------------
// deterministic expf
// ---------------------------------------------------------------------------
static const uint64_t ORC_EXP2F_TAB[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

static inline double u64_as_double(uint64_t u) { double d; memcpy(&d, &u, 8); return d; }
static inline uint64_t double_as_u64(double d) { uint64_t u; memcpy(&u, &d, 8); return u; }

// exp(x) = 2^(k/32) * 2^(r/32), k = round(x*32/ln2); 2^(r/32) by a cubic in r;
// 2^(k/32) from the table with the integer part added into the exponent field.
// Every a*b+c below is one fma (the form the FMA build of the published routine takes): libm's bits on all 2^32
// arguments on the hosts this was checked on.
float orc_expf_det(float x) {
    if (x != x) return x;
    if (x > 0x1.62e42ep6f) return INFINITY;   // > log(2^128)
    if (x < -0x1.9fe368p6f) return 0.0f;      // < log(2^-150)
    const double InvLn2N = 0x1.71547652b82fep+0 * 32;
    const double SHIFT = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32;
    double xd = (double) x;
    // (the product x * 32/ln2 is fused into both of its uses, as the compiler does in the library's FMA build)
    double kd = fma(InvLn2N, xd, SHIFT);
    uint64_t ki = double_as_u64(kd);
    kd -= SHIFT;
    double r = fma(InvLn2N, xd, -kd);
    uint64_t t = ORC_EXP2F_TAB[ki % 32];
    t += ki << (52 - 5);
    double s = u64_as_double(t);
    double zz = fma(C0, r, C1);
    double r2 = r * r;
    double y = fma(C2, r, 1.0);
    y = fma(zz, r2, y);
    y = y * s;
    return (float) y;
}

float orc_expf_libm(float x) { return expf(x); }

static inline float orc_expf(float x, int mode) { return mode ? orc_expf_det(x) : expf(x); }

// Counts inputs in the bit range [lo_bits, hi_bits] (as uint32 patterns of float) where
// orc_expf_det and libm expf differ; used by the oracle's own pinning test.
long long orc_expf_count_mismatch(uint32_t lo_bits, uint32_t hi_bits, uint32_t stride, uint32_t *first_bad) {
    long long bad = 0;
    uint32_t fb = 0;
    long long nsteps = ((long long) hi_bits - (long long) lo_bits) / stride + 1;
#pragma omp parallel for reduction(+:bad) schedule(static)
    for (long long sidx = 0; sidx < nsteps; ++sidx) {
        uint32_t b = lo_bits + (uint32_t) (sidx * stride);
        float x; memcpy(&x, &b, 4);
        float a = orc_expf_det(x), c = expf(x);
        uint32_t ua, uc; memcpy(&ua, &a, 4); memcpy(&uc, &c, 4);
        if (ua != uc && !(a != a && c != c)) {
            bad++;
#pragma omp critical
            if (fb == 0) fb = b;
        }
    }
    if (first_bad) *first_bad = fb;
    return bad;
}

// ---------------------------------------------------------------------------
// powf and tanhf, restated (expf_mode 1) as the HIP epilogues restate them: the published routines of the libm these
// hosts run (powf: 16-entry log2 table, quartic, y*log2(x) in double, then the expf table and cubic, FMA form;
// tanhf / expm1f: the fdlibm float versions).  orc_powf_count_mismatch / orc_tanhf_count_mismatch compare them with
// libm; run over all 2^32 arguments (for powf: for each of fourteen exponents) they found no difference.
// ---------------------------------------------------------------------------
static const double ORC_POWF_LOG2_TAB[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2 * 32}, {0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2 * 32},
    {0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2 * 32},  {0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2 * 32},
    {0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2 * 32}, {0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3 * 32},
    {0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3 * 32}, {0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4 * 32},
    {0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5 * 32}, {0x1p+0, 0x0p+0 * 32},
    {0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4 * 32},  {0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3 * 32},
    {0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3 * 32},  {0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2 * 32},
    {0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2 * 32},  {0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2 * 32}};
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline int powf_checkint(uint32_t iy) {   // 0: not an integer, 1: odd, 2: even
    int e = iy >> 23 & 0xff;
    if (e < 0x7f) return 0;
    if (e > 0x7f + 23) return 2;
    if (iy & ((1u << (0x7f + 23 - e)) - 1)) return 0;
    if (iy & (1u << (0x7f + 23 - e))) return 1;
    return 2;
}
static inline bool powf_zeroinfnan(uint32_t ix) { return 2 * ix - 1 >= 2u * 0x7f800000 - 1; }

float orc_powf_det(float x, float y) {
    const double A0 = 0x1.27616c9496e0bp-2 * 32, A1 = -0x1.71969a075c67ap-2 * 32, A2 = 0x1.ec70a6ca7baddp-2 * 32,
                 A3 = -0x1.7154748bef6c8p-1 * 32, A4 = 0x1.71547652ab82bp0 * 32;
    uint32_t sign_bias = 0;
    uint32_t ix = f32_bits(x), iy = f32_bits(y);
    if (ix - 0x00800000 >= 0x7f800000 - 0x00800000 || powf_zeroinfnan(iy)) {
        if (powf_zeroinfnan(iy)) {
            if (2 * iy == 0) return 2 * (ix ^ 0x00400000) > 2u * 0x7fc00000 ? x + y : 1.0f;   // (a signalling NaN stays a NaN)
            if (ix == 0x3f800000) return 2 * (iy ^ 0x00400000) > 2u * 0x7fc00000 ? x + y : 1.0f;
            if (2 * ix > 2u * 0x7f800000 || 2 * iy > 2u * 0x7f800000) return x + y;
            if (2 * ix == 2 * 0x3f800000) return 1.0f;
            if ((2 * ix < 2 * 0x3f800000) == !(iy & 0x80000000)) return 0.0f;
            return y * y;
        }
        if (powf_zeroinfnan(ix)) {
            float x2 = x * x;
            if ((ix & 0x80000000) && powf_checkint(iy) == 1) x2 = -x2;
            return (iy & 0x80000000) ? 1 / x2 : x2;
        }
        if (ix & 0x80000000) {
            int yint = powf_checkint(iy);
            if (yint == 0) return NAN;
            if (yint == 1) sign_bias = 1u << (5 + 11);
            ix &= 0x7fffffff;
        }
        if (ix < 0x00800000) {
            ix = f32_bits(x * 0x1p23f);
            ix &= 0x7fffffff;
            ix -= 23 << 23;
        }
    }
    uint32_t tmp = ix - 0x3f330000;
    int i = (tmp >> (23 - 4)) % 16;
    uint32_t top = tmp & 0xff800000;
    uint32_t iz = ix - top;
    int k = (int32_t) top >> (23 - 5);
    double invc = ORC_POWF_LOG2_TAB[i][0], logc = ORC_POWF_LOG2_TAB[i][1];
    double z = (double) bits_f32(iz);
    double r = fma(z, invc, -1.0);
    double y0 = logc + (double) k;
    double r2 = r * r;
    double yy = fma(A0, r, A1);
    double pp = fma(A2, r, A3);
    double r4 = r2 * r2;
    double q = fma(A4, r, y0);
    q = fma(pp, r2, q);
    double logx = fma(yy, r4, q);
    double ylogx = (double) y * logx;
    if ((double_as_u64(ylogx) >> 47 & 0xffff) >= double_as_u64(126.0 * 32) >> 47) {
        if (ylogx > 0x1.fffffffd1d571p+6 * 32) return sign_bias ? -INFINITY : INFINITY;
        if (ylogx <= -150.0 * 32) return sign_bias ? -0.0f : 0.0f;
    }
    const double SHIFT = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32, C2 = 0x1.62e42ff0c52d6p-1 / 32;
    double kd = ylogx + SHIFT;
    uint64_t ki = double_as_u64(kd);
    kd -= SHIFT;
    double rr = ylogx - kd;
    uint64_t t = ORC_EXP2F_TAB[ki % 32];
    t += (ki + sign_bias) << (52 - 5);
    double s = u64_as_double(t);
    double zz = fma(C0, rr, C1);
    double rr2 = rr * rr;
    double e = fma(C2, rr, 1.0);
    e = fma(zz, rr2, e);
    return (float) (e * s);
}

float orc_expm1f_det(float x) {
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f, o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f,
                ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f, Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f,
                Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = f32_bits(x);
    uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffff;
    if (hx >= 0x4195b844) {
        if (hx >= 0x42b17218) {
            if (hx > 0x7f800000) return x + x;
            if (hx == 0x7f800000) return (xsb == 0) ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3eb17218) {
        if (hx < 0x3F851592) {
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t) (invln2 * x + ((xsb == 0) ? 0.5f : -0.5f));
            t = (float) k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000) {
        t = huge + x;
        return x - (t - (huge + x));
    } else k = 0;
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = bits_f32(f32_bits(y) + ((uint32_t) k << 23));
        return y - one;
    }
    if (k < 23) {
        t = bits_f32(0x3f800000 - (0x1000000 >> k));
        y = t - (e - x);
        y = bits_f32(f32_bits(y) + ((uint32_t) k << 23));
    } else {
        t = bits_f32((uint32_t) (0x7f - k) << 23);
        y = x - (e + t);
        y += one;
        y = bits_f32(f32_bits(y) + ((uint32_t) k << 23));
    }
    return y;
}

float orc_tanhf_det(float x) {
    const float one = 1.0f, tiny = 1.0e-30f;
    float t, z;
    int32_t jx = (int32_t) f32_bits(x), ix = jx & 0x7fffffff;
    if (ix >= 0x7f800000) { if (jx >= 0) return one / x + one; else return one / x - one; }
    if (ix < 0x41b00000) {
        if (ix == 0) return x;
        if (ix < 0x24000000) return x * (one + x);
        if (ix >= 0x3f800000) {
            t = orc_expm1f_det(2.0f * fabsf(x));
            z = one - 2.0f / (t + 2.0f);
        } else {
            t = orc_expm1f_det(-2.0f * fabsf(x));
            z = -t / (t + 2.0f);
        }
    } else z = one - tiny;
    return (jx >= 0) ? z : -z;
}

// Arguments with bit patterns lo_bits, lo_bits + stride, ... <= hi_bits on which the restatement and libm differ (two
// NaNs count as equal).
long long orc_powf_count_mismatch(uint32_t lo_bits, uint32_t hi_bits, uint32_t stride, float y, uint32_t *first_bad) {
    long long bad = 0;
    uint32_t fb = 0;
    long long nsteps = ((long long) hi_bits - (long long) lo_bits) / stride + 1;
#pragma omp parallel for reduction(+:bad) schedule(static)
    for (long long sidx = 0; sidx < nsteps; ++sidx) {
        uint32_t b = lo_bits + (uint32_t) (sidx * stride);
        float x = bits_f32(b);
        float a = orc_powf_det(x, y), c = powf(x, y);
        if (f32_bits(a) != f32_bits(c) && !(a != a && c != c)) {
            bad++;
#pragma omp critical
            if (fb == 0) fb = b;
        }
    }
    if (first_bad) *first_bad = fb;
    return bad;
}

long long orc_tanhf_count_mismatch(uint32_t lo_bits, uint32_t hi_bits, uint32_t stride, uint32_t *first_bad) {
    long long bad = 0;
    uint32_t fb = 0;
    long long nsteps = ((long long) hi_bits - (long long) lo_bits) / stride + 1;
#pragma omp parallel for reduction(+:bad) schedule(static)
    for (long long sidx = 0; sidx < nsteps; ++sidx) {
        uint32_t b = lo_bits + (uint32_t) (sidx * stride);
        float x = bits_f32(b);
        float a = orc_tanhf_det(x), c = tanhf(x);
        if (f32_bits(a) != f32_bits(c) && !(a != a && c != c)) {
            bad++;
#pragma omp critical
            if (fb == 0) fb = b;
        }
    }
    if (first_bad) *first_bad = fb;
    return bad;
}

// ---------------------------------------------------------------------------
// index-set predicates (include/thundersvm/kernel/smo_kernel.h:13-23)
// ---------------------------------------------------------------------------
static inline bool is_I_up(double a, double y, double Cp, double Cn) { return (y > 0 && a < Cp) || (y < 0 && a > 0); }
static inline bool is_I_low(double a, double y, double Cp, double Cn) { return (y > 0 && a > 0) || (y < 0 && a < Cn); }
static inline bool is_free(double a, double y, double Cp, double Cn) { return a > 0 && (y > 0 ? a < Cp : a < Cn); }

int orc_is_I_up(double a, double y, double Cp, double Cn) { return is_I_up(a, y, Cp, Cn); }
int orc_is_I_low(double a, double y, double Cp, double Cn) { return is_I_low(a, y, Cp, Cn); }
int orc_is_free(double a, double y, double Cp, double Cn) { return is_free(a, y, Cp, Cn); }

// include/thundersvm/util/common.h:20-23
int orc_max2power(long long n) { return (int) pow(2, floor(log2f((float) n))); }

}  // extern "C"

// ---------------------------------------------------------------------------
// KernelMatrix (src/thundersvm/kernelmatrix.cpp:183-316,378-406)
// ---------------------------------------------------------------------------
struct OrcKernelMatrix {
    int n = 0;          // n_instances_
    int n_features = 0; // max feature index + 1 (kernelmatrix.cpp:200-206)
    long long nnz = 0;
    vector<double> val;
    vector<int> col;
    vector<long long> ptr;
    vector<double> self_dot;
    vector<double> diag;
    orc_param param;
};

static double epilogue_poly(double dot, const orc_param &p) {
    // kernelmatrix_kernel.cpp:94-100: powf(gamma * dot + coef0, degree), float-rounded argument.
    // expf_mode 1: the restated powf (what the HIP epilogue computes).
    float arg = (float) fma(p.gamma, dot, p.coef0);
    if (p.expf_mode) return (double) orc_powf_det(arg, (float) p.degree);
    return (double) powf(arg, (float) p.degree);
}

static double epilogue_sigmoid(double dot, const orc_param &p) {
    // kernelmatrix_kernel.cpp:102-108; expf_mode 1: the restated tanhf.
    float arg = (float) fma(p.gamma, dot, p.coef0);
    if (p.expf_mode) return (double) orc_tanhf_det(arg);
    return (double) tanhf(arg);
}

static inline double epilogue_rbf(double sd0, double sd1, double dot, const orc_param &p) {
    // kernelmatrix_kernel.cpp:71-72,87-89: expf(-(sd0 + sd1 - dot * 2) * gamma)
    double arg = -(sd0 + sd1 - dot * 2) * p.gamma;
    return (double) orc_expf((float) arg, p.expf_mode);
}

// kernelmatrix.cpp:183-249.  Rows are given as CSR with the caller's feature indices unchanged.
static OrcKernelMatrix *km_build(int n, const long long *ptr, const int *col, const double *val, const orc_param &param) {
    OrcKernelMatrix *k = new OrcKernelMatrix();
    k->n = n;
    k->param = param;
    k->nnz = ptr[n];
    k->ptr.assign(ptr, ptr + n + 1);
    k->col.assign(col, col + k->nnz);
    k->val.assign(val, val + k->nnz);
    k->self_dot.resize(n);
    int nf = 0;
    for (int i = 0; i < n; ++i) {
        double sd = 0;
        for (long long j = ptr[i]; j < ptr[i + 1]; ++j) {
            sd = fma(val[j], val[j], sd);
            if (col[j] > nf) nf = col[j];
        }
        k->self_dot[i] = sd;
    }
    k->n_features = nf + 1;
    k->diag.resize(n);
    for (int i = 0; i < n; ++i) {
        switch (param.kernel_type) {
            case ORC_RBF:
            case ORC_PRECOMPUTED: k->diag[i] = 1; break;
            case ORC_LINEAR: k->diag[i] = k->self_dot[i]; break;
            case ORC_POLY: k->diag[i] = epilogue_poly(k->self_dot[i], param); break;
            case ORC_SIGMOID: k->diag[i] = epilogue_sigmoid(k->self_dot[i], param); break;
        }
    }
    return k;
}

// dns_csr_mul (kernelmatrix_kernel.cpp:149-160): result[i][j] = sum over the non-zeros of stored
// row j, in stored order, of val * dense_i[col].  `dense_t` is the working-set rows transposed
// (n_features x m) so that the inner loop runs over i.
static void dot_rows(const OrcKernelMatrix &k, const vector<double> &dense_t, int m, double *out) {
    const int n = k.n;
#pragma omp parallel
    {
        vector<double> acc(m);
#pragma omp for schedule(dynamic, 64)
        for (int j = 0; j < n; ++j) {
            std::fill(acc.begin(), acc.end(), 0.0);
            for (long long e = k.ptr[j]; e < k.ptr[j + 1]; ++e) {
                const double v = k.val[e];
                const double *d = &dense_t[(size_t) k.col[e] * m];
                for (int i = 0; i < m; ++i) acc[i] = __builtin_fma(v, d[i], acc[i]);
            }
            for (int i = 0; i < m; ++i) out[(size_t) i * n + j] = acc[i];
        }
    }
}

static void apply_epilogue(const OrcKernelMatrix &k, const double *sd0, int m, double *out) {
    const int n = k.n;
    const orc_param &p = k.param;
#pragma omp parallel for schedule(static)
    for (long long e = 0; e < (long long) m * n; ++e) {
        int i = (int) (e / n), j = (int) (e % n);
        switch (p.kernel_type) {
            case ORC_RBF:
            case ORC_PRECOMPUTED: out[e] = epilogue_rbf(sd0[i], k.self_dot[j], out[e], p); break;
            case ORC_LINEAR: break;
            case ORC_POLY: out[e] = epilogue_poly(out[e], p); break;
            case ORC_SIGMOID: out[e] = epilogue_sigmoid(out[e], p); break;
        }
    }
}

// KernelMatrix::get_rows(idx) (kernelmatrix.cpp:251-279 -> :378-383 -> kernelmatrix_kernel.cpp:9-25)
static void km_get_rows_idx(const OrcKernelMatrix &k, const int *idx, int m, double *out) {
    vector<double> dense_t((size_t) k.n_features * m, 0.0);
    vector<double> sd0(m);
    for (int i = 0; i < m; ++i) {
        int row = idx[i];
        for (long long e = k.ptr[row]; e < k.ptr[row + 1]; ++e) dense_t[(size_t) k.col[e] * m + i] = k.val[e];
        sd0[i] = k.self_dot[row];
    }
    dot_rows(k, dense_t, m, out);
    apply_epilogue(k, sd0.data(), m, out);
}

// KernelMatrix::get_rows(instances) (kernelmatrix.cpp:281-312 -> :385-406): features with index
// >= n_features_ are dropped from the dot product but still counted in the row's self-dot.
static void km_get_rows_ins(const OrcKernelMatrix &k, int m, const long long *bptr, const int *bcol, const double *bval,
                            double *out) {
    vector<double> dense_t((size_t) k.n_features * m, 0.0);
    vector<double> sd0(m);
    for (int i = 0; i < m; ++i) {
        double sum = 0;
        for (long long e = bptr[i]; e < bptr[i + 1]; ++e) {
            if (bcol[e] < k.n_features) dense_t[(size_t) bcol[e] * m + i] = bval[e];
            sum = fma(bval[e], bval[e], sum);
        }
        sd0[i] = sum;
    }
    dot_rows(k, dense_t, m, out);
    apply_epilogue(k, sd0.data(), m, out);
}

// ---------------------------------------------------------------------------
// svm_kernel:: functions of smo_kernel.cpp
// ---------------------------------------------------------------------------
// sort_f (smo_kernel.cpp:321-332): std::sort of (f, idx) pairs.
static void sort_f(const double *f, int *idx, int n) {
    vector<std::pair<double, int>> pairs;
    pairs.reserve(n);
    for (int i = 0; i < n; ++i) pairs.emplace_back(f[i], idx[i]);
    std::sort(pairs.begin(), pairs.end());
    for (int i = 0; i < n; ++i) idx[i] = pairs[i].second;
}

// CSMOSolver::select_working_set (csmosolver.cpp:123-165)
static void select_working_set_c(vector<int> &ws_indicator, const int *index, const int *y, const double *alpha,
                                 double Cp, double Cn, int *working_set, int ws_size) {
    int n_instances = (int) ws_indicator.size();
    int p_left = 0;
    int p_right = n_instances - 1;
    int n_selected = 0;
    while (n_selected < ws_size) {
        int i;
        if (p_left < n_instances) {
            i = index[p_left];
            while (ws_indicator[i] == 1 || !is_I_up(alpha[i], y[i], Cp, Cn)) {
                p_left++;
                if (p_left == n_instances) break;
                i = index[p_left];
            }
            if (p_left < n_instances) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_right >= 0) {
            i = index[p_right];
            while (ws_indicator[i] == 1 || !is_I_low(alpha[i], y[i], Cp, Cn)) {
                p_right--;
                if (p_right == -1) break;
                i = index[p_right];
            }
            if (p_right >= 0) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_left >= n_instances && p_right < 0) break;  // guard: the reference would spin forever here
    }
}

// NuSMOSolver::select_working_set (nusmosolver.cpp:48-118)
static void select_working_set_nu(vector<int> &ws_indicator, const int *index, const int *y, const double *alpha,
                                  double Cp, double Cn, int *working_set, int ws_size) {
    int n_instances = (int) ws_indicator.size();
    int p_left_p = 0, p_left_n = 0;
    int p_right_p = n_instances - 1, p_right_n = n_instances - 1;
    int n_selected = 0;
    while (n_selected < ws_size) {
        int i;
        if (p_left_p < n_instances) {
            i = index[p_left_p];
            while (ws_indicator[i] == 1 || !(y[i] > 0 && is_I_up(alpha[i], y[i], Cp, Cn))) {
                p_left_p++;
                if (p_left_p == n_instances) break;
                i = index[p_left_p];
            }
            if (p_left_p < n_instances) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_left_n < n_instances) {
            i = index[p_left_n];
            while (ws_indicator[i] == 1 || !(y[i] < 0 && is_I_up(alpha[i], y[i], Cp, Cn))) {
                p_left_n++;
                if (p_left_n == n_instances) break;
                i = index[p_left_n];
            }
            if (p_left_n < n_instances && n_selected < ws_size) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_right_p >= 0) {
            i = index[p_right_p];
            while (ws_indicator[i] == 1 || !(y[i] > 0 && is_I_low(alpha[i], y[i], Cp, Cn))) {
                p_right_p--;
                if (p_right_p == -1) break;
                i = index[p_right_p];
            }
            if (p_right_p >= 0 && n_selected < ws_size) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_right_n >= 0) {
            i = index[p_right_n];
            while (ws_indicator[i] == 1 || !(y[i] < 0 && is_I_low(alpha[i], y[i], Cp, Cn))) {
                p_right_n--;
                if (p_right_n == -1) break;
                i = index[p_right_n];
            }
            if (p_right_n >= 0 && n_selected < ws_size) {
                working_set[n_selected++] = i;
                ws_indicator[i] = 1;
            }
        }
        if (p_left_p >= n_instances && p_left_n >= n_instances && p_right_p < 0 && p_right_n < 0) break;  // guard
    }
}

// c_smo_solve_kernel (smo_kernel.cpp:12-114)
static void c_smo_solve(const int *label, double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                        int ws_size, double Cp, double Cn, const double *k_mat_rows, const double *k_mat_diag,
                        long long row_len, double eps, double *diff, int max_iter) {
    double alpha_i_diff, alpha_j_diff;
    vector<double> kd(ws_size), a_old(ws_size), kIwsI(ws_size), f(ws_size), y(ws_size), a(ws_size);
    for (int tid = 0; tid < ws_size; ++tid) {
        int wsi = working_set[tid];
        f[tid] = f_val[wsi];
        a_old[tid] = a[tid] = alpha[wsi];
        y[tid] = label[wsi];
        kd[tid] = k_mat_diag[wsi];
    }
    double local_eps = 0;
    int numOfIter = 0;
    while (1) {
        int i = 0;
        double up_value = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid)
            if (is_I_up(a[tid], y[tid], Cp, Cn))
                if (f[tid] < up_value) { up_value = f[tid]; i = tid; }
        for (int tid = 0; tid < ws_size; ++tid) kIwsI[tid] = k_mat_rows[row_len * i + working_set[tid]];
        double low_value = -INFINITY;
        for (int tid = 0; tid < ws_size; ++tid)
            if (is_I_low(a[tid], y[tid], Cp, Cn))
                if (f[tid] > low_value) low_value = f[tid];
        double local_diff = low_value - up_value;
        if (numOfIter == 0) {
            local_eps = std::max(eps, 0.1f * local_diff);  // 0.1f: float literal widened to double
            diff[0] = local_diff;
        }
        if (numOfIter > max_iter || local_diff < local_eps) {
            for (int tid = 0; tid < ws_size; ++tid) {
                int wsi = working_set[tid];
                alpha_diff[tid] = -(a[tid] - a_old[tid]) * y[tid];
                alpha[wsi] = a[tid];
            }
            diff[1] = numOfIter;
            break;
        }
        int j2 = 0;
        double min_t = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            if (-up_value > -f[tid] && is_I_low(a[tid], y[tid], Cp, Cn)) {
                double aIJ = kd[i] + kd[tid] - 2 * kIwsI[tid];
                double bIJ = -up_value + f[tid];
                double ft = -bIJ * bIJ / aIJ;
                if (ft < min_t) { min_t = ft; j2 = tid; }
            }
        }
        alpha_i_diff = y[i] > 0 ? Cp - a[i] : a[i];
        alpha_j_diff = std::min(y[j2] > 0 ? a[j2] : Cn - a[j2],
                                (-up_value + f[j2]) / (kd[i] + kd[j2] - 2 * kIwsI[j2]));
        double l = std::min(alpha_i_diff, alpha_j_diff);
        a[i] += l * y[i];
        a[j2] -= l * y[j2];
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            double kJ2wsI = k_mat_rows[row_len * j2 + wsi];
            f[tid] = fma(-l, kJ2wsI - kIwsI[tid], f[tid]);  // f -= l * (kJ2 - kI)
        }
        numOfIter++;
    }
}

// nu_smo_solve_kernel (smo_kernel.cpp:127-287); keeps the j2n score's use of kd[ip]/kIpwsI (:239)
// and leaves diff[1] untouched, as the reference does.
static void nu_smo_solve(const int *y, double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                         int ws_size, double C, const double *k_mat_rows, const double *k_mat_diag, long long row_len,
                         double eps, double *diff, int max_iter) {
    double alpha_i_diff, alpha_j_diff;
    vector<double> kd(ws_size), a_old(ws_size), kIpwsI(ws_size), kInwsI(ws_size), f(ws_size);
    for (int tid = 0; tid < ws_size; ++tid) {
        int wsi = working_set[tid];
        f[tid] = f_val[wsi];
        a_old[tid] = alpha[wsi];
        kd[tid] = k_mat_diag[wsi];
    }
    double local_eps = 0;
    int numOfIter = 0;
    while (1) {
        int ip = 0;
        double up_value_p = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (y[wsi] > 0 && alpha[wsi] < C)
                if (f[tid] < up_value_p) { ip = tid; up_value_p = f[tid]; }
        }
        for (int tid = 0; tid < ws_size; ++tid) kIpwsI[tid] = k_mat_rows[row_len * ip + working_set[tid]];
        int in = 0;
        double up_value_n = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (y[wsi] < 0 && alpha[wsi] > 0)
                if (f[tid] < up_value_n) { in = tid; up_value_n = f[tid]; }
        }
        for (int tid = 0; tid < ws_size; ++tid) kInwsI[tid] = k_mat_rows[row_len * in + working_set[tid]];
        double low_value_p = -INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (y[wsi] > 0 && alpha[wsi] > 0)
                if (f[tid] > low_value_p) low_value_p = f[tid];
        }
        double low_value_n = -INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (y[wsi] < 0 && alpha[wsi] < C)
                if (f[tid] > low_value_n) low_value_n = f[tid];
        }
        double local_diff = std::max(low_value_p - up_value_p, low_value_n - up_value_n);
        if (numOfIter == 0) {
            local_eps = std::max(eps, 0.1 * local_diff);
            diff[0] = local_diff;
        }
        if (numOfIter > max_iter || local_diff < local_eps) {
            for (int tid = 0; tid < ws_size; ++tid) {
                int wsi = working_set[tid];
                alpha_diff[tid] = -(alpha[wsi] - a_old[tid]) * y[wsi];
            }
            break;
        }
        int j2p = 0;
        double f_val_j2p = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (-up_value_p > -f[tid] && y[wsi] > 0 && alpha[wsi] > 0) {
                double aIJ = kd[ip] + kd[tid] - 2 * kIpwsI[tid];
                double bIJ = -up_value_p + f[tid];
                double f_t1 = -bIJ * bIJ / aIJ;
                if (f_t1 < f_val_j2p) { j2p = tid; f_val_j2p = f_t1; }
            }
        }
        int j2n = 0;
        double f_val_j2n = INFINITY;
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            if (-up_value_n > -f[tid] && y[wsi] < 0 && alpha[wsi] < C) {
                double aIJ = kd[ip] + kd[tid] - 2 * kIpwsI[tid];
                double bIJ = -up_value_n + f[tid];
                double f_t2 = -bIJ * bIJ / aIJ;
                if (f_t2 < f_val_j2n) { j2n = tid; f_val_j2n = f_t2; }
            }
        }
        int i, j2;
        double up_value;
        const double *kIwsI;
        if (f_val_j2p < f_val_j2n) {
            i = ip; j2 = j2p; up_value = up_value_p; kIwsI = kIpwsI.data();
        } else {
            i = in; j2 = j2n; kIwsI = kInwsI.data(); up_value = up_value_n;
        }
        alpha_i_diff = y[working_set[i]] > 0 ? C - alpha[working_set[i]] : alpha[working_set[i]];
        alpha_j_diff = std::min(y[working_set[j2]] > 0 ? alpha[working_set[j2]] : C - alpha[working_set[j2]],
                                (-up_value + f[j2]) / (kd[i] + kd[j2] - 2 * kIwsI[j2]));
        double l = std::min(alpha_i_diff, alpha_j_diff);
        alpha[working_set[i]] += l * y[working_set[i]];
        alpha[working_set[j2]] -= l * y[working_set[j2]];
        for (int tid = 0; tid < ws_size; ++tid) {
            int wsi = working_set[tid];
            double kJ2wsI = k_mat_rows[row_len * j2 + wsi];
            f[tid] = fma(-l, kJ2wsI - kIwsI[tid], f[tid]);
        }
        numOfIter++;
    }
}

// update_f (smo_kernel.cpp:300-319)
static void update_f(double *f, const double *alpha_diff, int ws_size, const double *k_mat_rows, long long n) {
#pragma omp parallel for schedule(static)
    for (long long idx = 0; idx < n; ++idx) {
        double sum_diff = 0;
        for (int i = 0; i < ws_size; ++i) {
            double d = alpha_diff[i];
            if (d != 0) sum_diff = fma(d, k_mat_rows[i * n + idx], sum_diff);
        }
        f[idx] -= sum_diff;
    }
}

// ---------------------------------------------------------------------------
// solvers (csmosolver.cpp, nusmosolver.cpp)
// ---------------------------------------------------------------------------
struct OrcTrace {        // optional per-outer-iteration record for parity debugging
    int cap_iters = 0;   // capacity in outer iterations
    double *diff = nullptr;   // [cap][2]: diff[0], diff[1]
    int *ws = nullptr;        // [cap][ws_size]
    long long n_iter = 0;     // outer iterations executed
    long long local_iter = 0; // sum of diff[1]
    double obj = 0;
};

// CSMOSolver::calculate_rho (csmosolver.cpp:167-187)
static double calculate_rho_c(const double *f, const int *y, const double *alpha, int n, double Cp, double Cn) {
    int n_free = 0;
    double sum_free = 0;
    double up_value = INFINITY, low_value = -INFINITY;
    for (int i = 0; i < n; ++i) {
        if (is_free(alpha[i], y[i], Cp, Cn)) { n_free++; sum_free += f[i]; }
        if (is_I_up(alpha[i], y[i], Cp, Cn)) up_value = std::min(up_value, f[i]);
        if (is_I_low(alpha[i], y[i], Cp, Cn)) low_value = std::max(low_value, f[i]);
    }
    return 0 != n_free ? (sum_free / n_free) : (-(up_value + low_value) / 2);
}

// NuSMOSolver::calculate_rho + scale_alpha_rho (nusmosolver.cpp:9-46,120-126)
static double calculate_rho_nu(const double *f, const int *y, double *alpha, int n, double Cp, double Cn, bool for_svr) {
    int n_free_p = 0, n_free_n = 0;
    double sum_free_p = 0, sum_free_n = 0;
    double up_value_p = INFINITY, up_value_n = INFINITY;
    double low_value_p = -INFINITY, low_value_n = -INFINITY;
    for (int i = 0; i < n; ++i) {
        if (y[i] > 0) {
            if (alpha[i] > 0 && alpha[i] < Cp) { n_free_p++; sum_free_p += f[i]; }
            if (is_I_up(alpha[i], y[i], Cp, Cn)) up_value_p = std::min(up_value_p, -f[i]);
            if (is_I_low(alpha[i], y[i], Cp, Cn)) low_value_p = std::max(low_value_p, -f[i]);
        } else {
            if (alpha[i] > 0 && alpha[i] < Cn) { n_free_n++; sum_free_n += -f[i]; }
            if (is_I_up(alpha[i], y[i], Cp, Cn)) up_value_n = std::min(up_value_n, -f[i]);
            if (is_I_low(alpha[i], y[i], Cp, Cn)) low_value_n = std::max(low_value_n, -f[i]);
        }
    }
    double r1 = n_free_p != 0 ? sum_free_p / n_free_p : (-(up_value_p + low_value_p) / 2);
    double r2 = n_free_n != 0 ? sum_free_n / n_free_n : (-(up_value_n + low_value_n) / 2);
    double rho = (r1 - r2) / 2;
    if (!for_svr) {
        double r = (r1 + r2) / 2;
        for (int i = 0; i < n; ++i) alpha[i] /= r;
        rho /= r;
    }
    return rho;
}

// CSMOSolver::calculate_obj (csmosolver.cpp:227-239)
static double calculate_obj(const double *f, const double *alpha, const int *y, int n) {
    double obj = 0;
    for (int i = 0; i < n; ++i) obj += alpha[i] - (f[i] + y[i]) * alpha[i] * y[i] / 2;
    return -obj;
}

// CSMOSolver::init_f (csmosolver.cpp:189-214)
static void init_f(const OrcKernelMatrix &k, const double *alpha, const int *y, double *f) {
    const int n = k.n;
    size_t batch_size = 100;
    vector<int> idx_vec;
    vector<double> alpha_diff_vec;
    for (int i = 0; i < n; ++i) {
        if (alpha[i] != 0) {
            idx_vec.push_back(i);
            alpha_diff_vec.push_back(-alpha[i] * y[i]);
        }
        if (idx_vec.size() > batch_size || (i == n - 1 && !idx_vec.empty())) {
            vector<double> rows(idx_vec.size() * (size_t) n);
            km_get_rows_idx(k, idx_vec.data(), (int) idx_vec.size(), rows.data());
            update_f(f, alpha_diff_vec.data(), (int) idx_vec.size(), rows.data(), n);
            idx_vec.clear();
            alpha_diff_vec.clear();
        }
    }
}

// CSMOSolver::solve (csmosolver.cpp:10-121); nu=true swaps in NuSMOSolver's virtuals.
static void smo_solve(const OrcKernelMatrix &k, const int *y, double *alpha, double *rho, double *f_val, double eps,
                      double Cp, double Cn, int ws_size, int out_max_iter, bool nu, bool for_svr, OrcTrace *trace) {
    const int n = k.n;
    const int q = ws_size / 2;
    vector<int> working_set(ws_size);
    vector<int> f_idx2sort(n);
    vector<double> alpha_diff(ws_size);
    double diff[2] = {0, 0};
    vector<double> k_mat_rows((size_t) ws_size * n);
    init_f(k, alpha, y, f_val);
    int max_iter = std::max(100000, ws_size > INT_MAX / 100 ? INT_MAX : 100 * ws_size);
    long long local_iter = 0;
    int same_local_diff_cnt = 0;
    double previous_local_diff = INFINITY;
    int swap_local_diff_cnt = 0;
    double last_local_diff = INFINITY;
    double second_last_local_diff = INFINITY;
    for (int iter = 0;; ++iter) {
        for (int i = 0; i < n; ++i) f_idx2sort[i] = i;
        sort_f(f_val, f_idx2sort.data(), n);
        vector<int> ws_indicator(n, 0);
        if (0 == iter) {
            if (nu) select_working_set_nu(ws_indicator, f_idx2sort.data(), y, alpha, Cp, Cn, working_set.data(), ws_size);
            else select_working_set_c(ws_indicator, f_idx2sort.data(), y, alpha, Cp, Cn, working_set.data(), ws_size);
            km_get_rows_idx(k, working_set.data(), ws_size, k_mat_rows.data());
        } else {
            for (int i = 0; i < q; ++i) working_set[i] = working_set[q + i];
            for (int i = 0; i < q; ++i) ws_indicator[working_set[i]] = 1;
            if (nu) select_working_set_nu(ws_indicator, f_idx2sort.data(), y, alpha, Cp, Cn, working_set.data() + q, q);
            else select_working_set_c(ws_indicator, f_idx2sort.data(), y, alpha, Cp, Cn, working_set.data() + q, q);
            memcpy(k_mat_rows.data(), k_mat_rows.data() + (size_t) q * n, sizeof(double) * (size_t) q * n);
            km_get_rows_idx(k, working_set.data() + q, q, k_mat_rows.data() + (size_t) q * n);
        }
        if (nu) nu_smo_solve(y, f_val, alpha, alpha_diff.data(), working_set.data(), ws_size, Cp, k_mat_rows.data(),
                             k.diag.data(), n, eps, diff, max_iter);
        else c_smo_solve(y, f_val, alpha, alpha_diff.data(), working_set.data(), ws_size, Cp, Cn, k_mat_rows.data(),
                         k.diag.data(), n, eps, diff, max_iter);
        update_f(f_val, alpha_diff.data(), ws_size, k_mat_rows.data(), n);
        local_iter += (long long) diff[1];
        if (trace && iter < trace->cap_iters) {
            if (trace->diff) { trace->diff[2 * iter] = diff[0]; trace->diff[2 * iter + 1] = diff[1]; }
            if (trace->ws) memcpy(trace->ws + (size_t) iter * ws_size, working_set.data(), sizeof(int) * ws_size);
        }
        if (fabs(diff[0] - previous_local_diff) < eps * 0.001) {
            same_local_diff_cnt++;
        } else {
            same_local_diff_cnt = 0;
            previous_local_diff = diff[0];
        }
        if (fabs(diff[0] - second_last_local_diff) < eps * 0.001) {
            swap_local_diff_cnt++;
        } else {
            swap_local_diff_cnt = 0;
        }
        second_last_local_diff = last_local_diff;
        last_local_diff = diff[0];
        if ((same_local_diff_cnt >= 10 && fabs(diff[0] - 2.0) > eps) || diff[0] < eps ||
            ((out_max_iter != -1) && (iter == out_max_iter)) ||
            (swap_local_diff_cnt >= 10 && fabs(diff[0] - 2.0) > eps)) {
            if (nu) *rho = calculate_rho_nu(f_val, y, alpha, n, Cp, Cn, for_svr);
            else *rho = calculate_rho_c(f_val, y, alpha, n, Cp, Cn);
            double obj = calculate_obj(f_val, alpha, y, n);
            if (trace) { trace->n_iter = iter + 1; trace->local_iter = local_iter; trace->obj = obj; }
            break;
        }
    }
}

// SvmModel::get_working_set_size (svmmodel.cpp:437-451).  `allocated` stands for the reference's
// SyncMem byte counter at the time of the call.
static int working_set_size(long long n_instances, long long n_features, long long max_mem_size, long long allocated) {
    size_t free_mem = (size_t) (max_mem_size - allocated);
    int a = orc_max2power(n_instances);
    size_t b = (size_t) orc_max2power((long long) (free_mem / sizeof(double) / (size_t) (n_instances + n_features)));
    return std::min(a, (int) std::min(b, (size_t) 1024));
}

// ---------------------------------------------------------------------------
// models (svc.cpp, svr.cpp, nusvc.cpp, nusvr.cpp, oneclass_svc.cpp, svmmodel.cpp)
// ---------------------------------------------------------------------------
struct OrcModel {
    orc_param param;
    int n_classes = 2;
    int n_binary_models = 1;
    int n_total_sv = 0;
    vector<int> label;
    vector<int> n_sv;
    vector<double> rho;
    vector<double> coef;        // (n_classes-1) x n_total_sv, LibSVM layout (svmmodel.h:154-164)
    vector<int> sv_indices;     // row ids in the training set
    // support vectors as CSR
    vector<long long> sv_ptr;
    vector<int> sv_col;
    vector<double> sv_val;
    // per binary problem diagnostics
    vector<long long> n_iter, local_iter;
    vector<int> ws_size;        // working-set size of every binary problem
    vector<double> obj;
    vector<vector<double>> alpha_bin;  // signed alpha of every binary problem (alpha*y), training order
    vector<vector<double>> f_bin;
    // trace of the first binary problem (optional)
    OrcTrace trace;
    vector<double> trace_diff;
    vector<int> trace_ws;
    int trace_ws_size = 0;
};

struct Csr {
    vector<long long> ptr{0};
    vector<int> col;
    vector<double> val;
    int rows() const { return (int) ptr.size() - 1; }
    void push_row(const long long *p, const int *c, const double *v, int r) {
        for (long long e = p[r]; e < p[r + 1]; ++e) { col.push_back(c[e]); val.push_back(v[e]); }
        ptr.push_back((long long) col.size());
    }
};

// Bytes the reference's SyncMem counter (syncmem.cpp:58-108: every array counts once, when its host side is first
// touched) holds when get_working_set_size runs in train_binary of a CPU build (svc.cpp:147-166):
//   * the KernelMatrix arrays val_, col_ind_, row_ptr_, self_dot_, diag_ (kernelmatrix.cpp:211-226);
//   * the two parts CSR_DenseCSR splits the columns into (kernelmatrix.cpp:16-181): columns are ordered by entry
//     count (ties by index) and moved to the sparse part one by one until the part would be more than 5 % full,
//     the column more than 50 % full, or four times the part's entries exceed the cells left to the dense part;
//     the dense part is an m x densecol array, the sparse part a CSR (built only if some value lies outside the
//     dense part);
//   * y (int), alpha and f (double) of the problem;
//   * `held`: what the model keeps from earlier problems (the alpha arrays of earlier class pairs, svc.cpp:50-61).
// Small model members (rho, n_sv, label) are left out.
static long long partition_bytes(long long m, long long n_features, const long long *ptr, const int *col, const double *val) {
    vector<long long> col_num((size_t) n_features, 0);
    for (long long e = 0; e < ptr[m]; ++e) col_num[col[e]]++;
    vector<int> col_indices((size_t) n_features);
    for (long long i = 0; i < n_features; ++i) col_indices[i] = (int) i;
    std::sort(col_indices.begin(), col_indices.end(), [&](int a, int b) {
        return col_num[a] != col_num[b] ? col_num[a] < col_num[b] : a < b;
    });
    vector<char> densefg((size_t) n_features, 1);
    long long densecolnum = n_features, total_csr = 0, total_dense = m * n_features, row_sum_num = 0;
    for (long long i = 0; i < n_features; ++i) {
        total_csr += col_num[col_indices[i]];
        total_dense -= m;
        row_sum_num += m;
        long double ratio = 1.0l * total_csr / row_sum_num;
        if (ratio > 0.05 || 1.0l * col_num[col_indices[i]] / m > 0.5 || total_csr * 4 > total_dense) break;
        densecolnum--;
        densefg[col_indices[i]] = 0;
    }
    long long bytes = 0, dense_data_count = 0, sparse_entries = 0;
    for (long long e = 0; e < ptr[m]; ++e) {
        if (densefg[col[e]]) dense_data_count += val[e] != 0;
        else sparse_entries++;
    }
    if (densecolnum > 0) bytes += m * densecolnum * 8;
    if (densecolnum < n_features && dense_data_count != ptr[m]) bytes += sparse_entries * 12 + (m + 1) * 4;
    return bytes;
}

static long long tally_bytes(const Csr &ins, long long n_features, long long held) {
    const long long n = ins.rows(), nnz = (long long) ins.col.size();
    return nnz * 12 + (n + 1) * 4 + n * 8 * 2 + partition_bytes(n, n_features, ins.ptr.data(), ins.col.data(), ins.val.data()) +
           n * (4 + 8 + 8) + held;
}

static void train_binary_generic(OrcModel &m, const Csr &ins, vector<int> &y, vector<double> &alpha,
                                 vector<double> &f, double Cp, double Cn, bool nu, bool for_svr, double *rho,
                                 int ws_override, bool want_trace, long long held = 0) {
    OrcKernelMatrix *k = km_build(ins.rows(), ins.ptr.data(), ins.col.data(), ins.val.data(), m.param);
    int ws = ws_override > 0 ? ws_override
                             : working_set_size(k->n, k->n_features, m.param.max_mem_size, tally_bytes(ins, k->n_features, held));
    m.ws_size.push_back(ws);
    OrcTrace tr;
    if (want_trace) {
        tr.cap_iters = 4096;
        m.trace_diff.assign((size_t) tr.cap_iters * 2, 0.0);
        m.trace_ws.assign((size_t) tr.cap_iters * ws, -1);
        m.trace_ws_size = ws;
        tr.diff = m.trace_diff.data();
        tr.ws = m.trace_ws.data();
    }
    smo_solve(*k, y.data(), alpha.data(), rho, f.data(), m.param.epsilon, Cp, Cn, ws, m.param.max_iter, nu, for_svr, &tr);
    m.n_iter.push_back(tr.n_iter);
    m.local_iter.push_back(tr.local_iter);
    m.obj.push_back(tr.obj);
    if (want_trace) m.trace = tr;
    delete k;
}

extern "C" {

// ---- kernel-matrix level API ------------------------------------------------
void *orc_km_create(int n, const long long *ptr, const int *col, const double *val, const orc_param *param) {
    return km_build(n, ptr, col, val, *param);
}
void orc_km_free(void *k) { delete (OrcKernelMatrix *) k; }
int orc_km_n_features(void *k) { return ((OrcKernelMatrix *) k)->n_features; }
void orc_km_self_dot(void *k, double *out) {
    OrcKernelMatrix *km = (OrcKernelMatrix *) k;
    memcpy(out, km->self_dot.data(), sizeof(double) * km->n);
}
void orc_km_diag(void *k, double *out) {
    OrcKernelMatrix *km = (OrcKernelMatrix *) k;
    memcpy(out, km->diag.data(), sizeof(double) * km->n);
}
void orc_km_get_rows(void *k, const int *idx, int m, double *out) { km_get_rows_idx(*(OrcKernelMatrix *) k, idx, m, out); }
void orc_km_get_rows_instances(void *k, int m, const long long *bptr, const int *bcol, const double *bval, double *out) {
    km_get_rows_ins(*(OrcKernelMatrix *) k, m, bptr, bcol, bval, out);
}

// ---- smo-kernel level API ---------------------------------------------------
void orc_sort_f(const double *f, int *idx, int n) { sort_f(f, idx, n); }

// Returns the selection the reference makes given f (unsorted), y, alpha and the ids already in the
// working set (`marked`, n_marked of them).
void orc_select_working_set(const double *f, const int *y, const double *alpha, int n, double Cp, double Cn,
                            const int *marked, int n_marked, int *out, int n_select, int nu) {
    vector<int> idx(n);
    for (int i = 0; i < n; ++i) idx[i] = i;
    sort_f(f, idx.data(), n);
    vector<int> ind(n, 0);
    for (int i = 0; i < n_marked; ++i) ind[marked[i]] = 1;
    if (nu) select_working_set_nu(ind, idx.data(), y, alpha, Cp, Cn, out, n_select);
    else select_working_set_c(ind, idx.data(), y, alpha, Cp, Cn, out, n_select);
}

void orc_c_smo_solve(const int *label, double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                     int ws_size, double Cp, double Cn, const double *k_mat_rows, const double *k_mat_diag,
                     long long row_len, double eps, double *diff, int max_iter) {
    c_smo_solve(label, f_val, alpha, alpha_diff, working_set, ws_size, Cp, Cn, k_mat_rows, k_mat_diag, row_len, eps,
                diff, max_iter);
}

void orc_nu_smo_solve(const int *y, double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                      int ws_size, double C, const double *k_mat_rows, const double *k_mat_diag, long long row_len,
                      double eps, double *diff, int max_iter) {
    nu_smo_solve(y, f_val, alpha, alpha_diff, working_set, ws_size, C, k_mat_rows, k_mat_diag, row_len, eps, diff,
                 max_iter);
}

void orc_update_f(double *f, const double *alpha_diff, int ws_size, const double *k_mat_rows, long long n) {
    update_f(f, alpha_diff, ws_size, k_mat_rows, n);
}

double orc_calculate_rho(const double *f, const int *y, double *alpha, int n, double Cp, double Cn, int nu, int for_svr) {
    return nu ? calculate_rho_nu(f, y, alpha, n, Cp, Cn, for_svr) : calculate_rho_c(f, y, alpha, n, Cp, Cn);
}
double orc_calculate_obj(const double *f, const double *alpha, const int *y, int n) { return calculate_obj(f, alpha, y, n); }

int orc_working_set_size(long long n_instances, long long n_features, long long max_mem_size, long long allocated) {
    return working_set_size(n_instances, n_features, max_mem_size, allocated);
}

// Full binary solve on a caller-built problem (CSMOSolver::solve / NuSMOSolver::solve).
// trace_diff: [trace_cap][2], trace_ws: [trace_cap][ws_size] (either may be null).
void orc_smo_solve(void *km, const int *y, double *alpha, double *rho, double *f_val, double eps, double Cp, double Cn,
                   int ws_size, int out_max_iter, int nu, int for_svr, int trace_cap, double *trace_diff, int *trace_ws,
                   long long *stats /* n_iter, local_iter */, double *obj) {
    OrcTrace tr;
    tr.cap_iters = trace_cap;
    tr.diff = trace_diff;
    tr.ws = trace_ws;
    smo_solve(*(OrcKernelMatrix *) km, y, alpha, rho, f_val, eps, Cp, Cn, ws_size, out_max_iter, nu != 0, for_svr != 0, &tr);
    if (stats) { stats[0] = tr.n_iter; stats[1] = tr.local_iter; }
    if (obj) *obj = tr.obj;
}

// sum_kernel_values (kernelmatrix_kernel.cpp:110-147)
void orc_sum_kernel_values(const double *coef, int total_sv, const int *sv_start, const int *sv_count, const double *rho,
                           const double *k_mat, double *dec_values, int n_classes, int n_instances) {
#pragma omp parallel for schedule(static)
    for (int idx = 0; idx < n_instances; idx++) {
        int k = 0;
        int n_binary_models = n_classes * (n_classes - 1) / 2;
        for (int i = 0; i < n_classes; ++i) {
            for (int j = i + 1; j < n_classes; ++j) {
                int si = sv_start[i], sj = sv_start[j], ci = sv_count[i], cj = sv_count[j];
                const double *coef1 = &coef[(size_t) (j - 1) * total_sv];
                const double *coef2 = &coef[(size_t) i * total_sv];
                const double *k_values = &k_mat[(size_t) idx * total_sv];
                double sum = 0;
                for (int l = 0; l < ci; ++l) sum = fma(coef1[si + l], k_values[si + l], sum);
                for (int l = 0; l < cj; ++l) sum = fma(coef2[sj + l], k_values[sj + l], sum);
                dec_values[(size_t) idx * n_binary_models + k] = sum - rho[k];
                k++;
            }
        }
    }
}

// ---- model level API --------------------------------------------------------
// Training data: CSR (ptr/col/val, val float32-exact) + y (labels or targets).
// ws_override > 0 forces the working-set size; want_trace records the first binary problem.
void *orc_train(int n, const long long *ptr, const int *col, const double *val, const double *y_in,
                const orc_param *param_in, int ws_override, int want_trace) {
    OrcModel *m = new OrcModel();
    m->param = *param_in;
    const orc_param &param = m->param;
    const int st = param.svm_type;
    if (st == ORC_C_SVC || st == ORC_NU_SVC) {
        // DataSet::group_classes (dataset.cpp:190-234): classes in first-appearance order.
        vector<int> label, count, data_label(n);
        for (int i = 0; i < n; ++i) {
            size_t j;
            for (j = 0; j < label.size(); ++j)
                if (y_in[i] == label[j]) { count[j]++; break; }
            data_label[i] = (int) j;
            if (j == label.size()) { label.push_back((int) y_in[i]); count.push_back(1); }
        }
        int nc = (int) label.size();
        vector<int> start(1, 0);
        for (int i = 1; i < nc; ++i) start.push_back(start[i - 1] + count[i - 1]);
        vector<int> start_copy(start), perm(n);
        for (int i = 0; i < n; ++i) perm[start_copy[data_label[i]]++] = i;
        // SVC::model_setup (svc.cpp:16-39)
        m->n_classes = nc;
        m->n_binary_models = nc * (nc - 1) / 2;
        m->label = label;
        m->rho.assign(m->n_binary_models, 0.0);
        m->n_sv.assign(nc, 0);
        vector<double> c_weight(nc, 1.0);
        for (int i = 0; i < param.nr_weight; ++i)
            for (int j = 0; j < nc; ++j)
                if (param.weight_label[i] == label[j]) { c_weight[j] *= param.weight[i]; break; }
        // SVC::train (svc.cpp:41-108)
        vector<vector<double>> alpha(m->n_binary_models);
        vector<char> is_sv(n, 0);
        int k = 0;
        long long held = 0;
        for (int i = 0; i < nc; ++i) {
            for (int j = i + 1; j < nc; ++j) {
                Csr ins;
                vector<int> original_index;
                for (int l = 0; l < count[i]; ++l) { ins.push_row(ptr, col, val, perm[start[i] + l]); original_index.push_back(perm[start[i] + l]); }
                for (int l = 0; l < count[j]; ++l) { ins.push_row(ptr, col, val, perm[start[j] + l]); original_index.push_back(perm[start[j] + l]); }
                int nn = ins.rows();
                vector<int> y(nn);
                vector<double> f(nn, 0.0);
                alpha[k].assign(nn, 0.0);
                if (st == ORC_C_SVC) {
                    // SVC::train_binary (svc.cpp:147-177)
                    for (int l = 0; l < count[i]; ++l) { y[l] = +1; f[l] = -1; }
                    for (int l = 0; l < count[j]; ++l) { y[count[i] + l] = -1; f[count[i] + l] = +1; }
                    train_binary_generic(*m, ins, y, alpha[k], f, param.C * c_weight[i], param.C * c_weight[j], false,
                                         false, &m->rho[k], ws_override, want_trace && k == 0, held);
                } else {
                    // NuSVC::train_binary (nusvc.cpp:7-45)
                    double sum_pos = param.nu * nn / 2;
                    double sum_neg = sum_pos;
                    for (int l = 0; l < count[i]; ++l) { y[l] = +1; alpha[k][l] = std::min(1., sum_pos); sum_pos -= alpha[k][l]; }
                    for (int l = 0; l < count[j]; ++l) { y[count[i] + l] = -1; alpha[k][count[i] + l] = std::min(1., sum_neg); sum_neg -= alpha[k][count[i] + l]; }
                    train_binary_generic(*m, ins, y, alpha[k], f, 1, 1, true, false, &m->rho[k], ws_override,
                                         want_trace && k == 0, held);
                }
                held += 8LL * nn;   // alpha[k] stays allocated until the coefficients are assembled (svc.cpp:50-61)
                for (int l = 0; l < nn; ++l) alpha[k][l] *= y[l];
                for (int l = 0; l < nn; ++l) is_sv[original_index[l]] = is_sv[original_index[l]] || (alpha[k][l] != 0);
                m->alpha_bin.push_back(alpha[k]);
                m->f_bin.push_back(f);
                k++;
            }
        }
        Csr sv;
        for (int i = 0; i < nc; ++i)
            for (int j = 0; j < count[i]; ++j) {
                int oi = perm[start[i] + j];
                if (is_sv[oi]) { m->n_sv[i]++; sv.push_row(ptr, col, val, oi); m->sv_indices.push_back(oi); }
            }
        m->n_total_sv = sv.rows();
        m->coef.assign((size_t) (nc - 1) * m->n_total_sv, 0.0);
        vector<int> sv_start(1, 0);
        for (int i = 1; i < nc; ++i) sv_start.push_back(sv_start[i - 1] + m->n_sv[i - 1]);
        k = 0;
        for (int i = 0; i < nc; ++i) {
            for (int j = i + 1; j < nc; ++j) {
                int ci = count[i], cj = count[j];
                int mm = sv_start[i];
                for (int l = 0; l < ci; ++l)
                    if (is_sv[perm[start[i] + l]]) m->coef[(size_t) (j - 1) * m->n_total_sv + mm++] = alpha[k][l];
                mm = sv_start[j];
                for (int l = ci; l < ci + cj; ++l)
                    if (is_sv[perm[start[j] + l - ci]]) m->coef[(size_t) i * m->n_total_sv + mm++] = alpha[k][l];
                k++;
            }
        }
        m->sv_ptr = sv.ptr; m->sv_col = sv.col; m->sv_val = sv.val;
    } else {
        // SvmModel::model_setup with n_classes = 2 (svmmodel.cpp:22-29)
        m->n_classes = 2;
        m->n_binary_models = 1;
        m->rho.assign(1, 0.0);
        m->n_sv.assign(2, 0);
        vector<double> coef_vec;
        Csr sv;
        if (st == ORC_EPSILON_SVR || st == ORC_NU_SVR) {
            // SVR::train (svr.cpp:9-41), NuSVR::train (nusvr.cpp:7-41): instances duplicated to 2n rows
            Csr ins2;
            for (int r = 0; r < 2; ++r) for (int i = 0; i < n; ++i) ins2.push_row(ptr, col, val, i);
            vector<double> f(2 * (size_t) n), alpha2(2 * (size_t) n, 0.0);
            vector<int> y(2 * (size_t) n);
            if (st == ORC_EPSILON_SVR) {
                for (int i = 0; i < n; ++i) {
                    f[i] = param.p - y_in[i]; y[i] = +1;
                    f[i + n] = -param.p - y_in[i]; y[i + n] = -1;
                }
                train_binary_generic(*m, ins2, y, alpha2, f, param.C, param.C, false, false, &m->rho[0], ws_override, want_trace);
            } else {
                double sum = param.C * param.nu * n / 2;
                for (int i = 0; i < n; ++i) {
                    alpha2[i] = alpha2[i + n] = std::min(sum, param.C);
                    sum -= alpha2[i];
                    f[i] = f[i + n] = -y_in[i];
                    y[i] = +1; y[i + n] = -1;
                }
                train_binary_generic(*m, ins2, y, alpha2, f, param.C, param.C, true, true, &m->rho[0], ws_override, want_trace);
            }
            // SVR::save_svr_coef (svr.cpp:43-62)
            for (int i = 0; i < n; ++i) {
                double alpha_i = alpha2[i] - alpha2[i + n];
                if (alpha_i != 0) { sv.push_row(ptr, col, val, i); m->sv_indices.push_back(i); coef_vec.push_back(alpha_i); }
            }
            m->alpha_bin.push_back(alpha2);
            m->f_bin.push_back(f);
        } else {
            // OneClassSVC::train (oneclass_svc.cpp:9-57)
            Csr ins;
            for (int i = 0; i < n; ++i) ins.push_row(ptr, col, val, i);
            vector<double> alpha(n, 0.0), f(n, 0.0);
            vector<int> y(n, 1);
            int nn = (int) (param.nu * n);
            for (int i = 0; i < nn; ++i) alpha[i] = 1;
            if (nn < n) alpha[nn] = param.nu * n - nn;
            train_binary_generic(*m, ins, y, alpha, f, 1, 1, false, false, &m->rho[0], ws_override, want_trace);
            for (int i = 0; i < n; ++i)
                if (alpha[i] != 0) { sv.push_row(ptr, col, val, i); m->sv_indices.push_back(i); coef_vec.push_back(alpha[i]); }
            m->alpha_bin.push_back(alpha);
            m->f_bin.push_back(f);
        }
        m->n_sv[0] = sv.rows();
        m->n_sv[1] = 0;
        m->n_total_sv = sv.rows();
        m->coef = coef_vec;
        m->sv_ptr = sv.ptr; m->sv_col = sv.col; m->sv_val = sv.val;
    }
    return m;
}

void orc_model_free(void *m) { delete (OrcModel *) m; }
int orc_model_n_classes(void *m) { return ((OrcModel *) m)->n_classes; }
int orc_model_n_binary(void *m) { return ((OrcModel *) m)->n_binary_models; }
int orc_model_total_sv(void *m) { return ((OrcModel *) m)->n_total_sv; }
long long orc_model_sv_nnz(void *m) { return (long long) ((OrcModel *) m)->sv_val.size(); }
void orc_model_get(void *mp, int *label, int *n_sv, double *rho, double *coef, int *sv_indices, long long *sv_ptr,
                   int *sv_col, double *sv_val, long long *n_iter, long long *local_iter, double *obj) {
    OrcModel *m = (OrcModel *) mp;
    if (label && !m->label.empty()) memcpy(label, m->label.data(), sizeof(int) * m->label.size());
    if (n_sv) memcpy(n_sv, m->n_sv.data(), sizeof(int) * m->n_sv.size());
    if (rho) memcpy(rho, m->rho.data(), sizeof(double) * m->rho.size());
    if (coef && !m->coef.empty()) memcpy(coef, m->coef.data(), sizeof(double) * m->coef.size());
    if (sv_indices && !m->sv_indices.empty()) memcpy(sv_indices, m->sv_indices.data(), sizeof(int) * m->sv_indices.size());
    if (sv_ptr) memcpy(sv_ptr, m->sv_ptr.data(), sizeof(long long) * m->sv_ptr.size());
    if (sv_col && !m->sv_col.empty()) memcpy(sv_col, m->sv_col.data(), sizeof(int) * m->sv_col.size());
    if (sv_val && !m->sv_val.empty()) memcpy(sv_val, m->sv_val.data(), sizeof(double) * m->sv_val.size());
    if (n_iter) memcpy(n_iter, m->n_iter.data(), sizeof(long long) * m->n_iter.size());
    if (local_iter) memcpy(local_iter, m->local_iter.data(), sizeof(long long) * m->local_iter.size());
    if (obj) memcpy(obj, m->obj.data(), sizeof(double) * m->obj.size());
}
long long orc_model_binary_size(void *m, int k) { return (long long) ((OrcModel *) m)->alpha_bin[k].size(); }
void orc_model_binary_get(void *mp, int k, double *alpha_signed, double *f) {
    OrcModel *m = (OrcModel *) mp;
    if (alpha_signed) memcpy(alpha_signed, m->alpha_bin[k].data(), sizeof(double) * m->alpha_bin[k].size());
    if (f) memcpy(f, m->f_bin[k].data(), sizeof(double) * m->f_bin[k].size());
}
int orc_model_ws_size(void *mp, int k) { return ((OrcModel *) mp)->ws_size.at(k); }
// the restated SyncMem counter for one problem given as CSR (n rows, feature ids < n_features)
long long orc_reference_bytes(int n, const long long *ptr, const int *col, const double *val, int n_features, long long held) {
    Csr ins;
    for (int r = 0; r < n; ++r) ins.push_row(ptr, col, val, r);
    return tally_bytes(ins, n_features, held);
}
int orc_model_trace(void *mp, int *ws_size, const double **diff, const int **ws) {
    OrcModel *m = (OrcModel *) mp;
    *ws_size = m->trace_ws_size;
    *diff = m->trace_diff.data();
    *ws = m->trace_ws.data();
    return (int) std::min<long long>(m->trace.n_iter, m->trace.cap_iters);
}

// SvmModel::predict_dec_values (svmmodel.cpp:74-117) on a CSR batch; dec_values is [m][n_binary_models].
void orc_predict_dec_values(void *mp, int nrows, const long long *bptr, const int *bcol, const double *bval,
                            double *dec_values, int batch_size) {
    OrcModel *m = (OrcModel *) mp;
    vector<int> sv_start(m->n_classes, 0);
    for (int i = 1; i < m->n_classes; ++i) sv_start[i] = sv_start[i - 1] + m->n_sv[i - 1];
    OrcKernelMatrix *k = km_build(m->n_total_sv, m->sv_ptr.data(), m->sv_col.data(), m->sv_val.data(), m->param);
    if (batch_size <= 0) batch_size = 10000;
    for (int b0 = 0; b0 < nrows; b0 += batch_size) {
        int bm = std::min(batch_size, nrows - b0);
        vector<long long> p(bm + 1);
        for (int i = 0; i <= bm; ++i) p[i] = bptr[b0 + i] - bptr[b0];
        vector<double> kv((size_t) bm * m->n_total_sv);
        km_get_rows_ins(*k, bm, p.data(), bcol + bptr[b0], bval + bptr[b0], kv.data());
        orc_sum_kernel_values(m->coef.data(), m->n_total_sv, sv_start.data(), m->n_sv.data(), m->rho.data(), kv.data(),
                              dec_values + (size_t) b0 * m->n_binary_models, m->n_classes, bm);
    }
    delete k;
}

// SVC::predict_label voting (svc.cpp:265-288), SvmModel::predict for regression (svmmodel.cpp:157-171),
// OneClassSVC::predict sign (oneclass_svc.cpp:59-66).
void orc_predict_label(void *mp, const double *dec_values, int nrows, double *out) {
    OrcModel *m = (OrcModel *) mp;
    int st = m->param.svm_type;
    if (st == ORC_C_SVC || st == ORC_NU_SVC) {
        for (int l = 0; l < nrows; ++l) {
            vector<int> votes(m->n_classes, 0);
            int k = 0;
            for (int i = 0; i < m->n_classes; ++i)
                for (int j = i + 1; j < m->n_classes; ++j) {
                    if (dec_values[(size_t) l * m->n_binary_models + k] > 0) votes[i]++; else votes[j]++;
                    k++;
                }
            int best = 0;
            for (int i = 1; i < m->n_classes; ++i) if (votes[i] > votes[best]) best = i;
            out[l] = (float) m->label[best];
        }
    } else if (st == ORC_ONE_CLASS) {
        for (int l = 0; l < nrows; ++l) out[l] = dec_values[l] > 0 ? 1 : -1;
    } else {
        for (int l = 0; l < nrows; ++l) out[l] = dec_values[l];
    }
}

// ---------------------------------------------------------------------------
// Probability estimates (svc.cpp:197-430).  The fold loop of SVC::probability_train
// (svc.cpp:432-491) is driven from tests/oracle_lib.py with the model functions above.
// ---------------------------------------------------------------------------

// sigmoidPredict (svc.cpp:197-204)
double orc_sigmoid_predict(double dec_value, double A, double B) {
    double fApB = dec_value * A + B;
    if (fApB >= 0) return exp(-fApB) / (1.0 + exp(-fApB));
    return 1.0 / (1 + exp(fApB));
}

// sigmoidTrain (svc.cpp:318-430): regularised targets, Newton direction on (A, B) with H + sigma*I,
// backtracking line search with the 1e-4 sufficient-decrease rule.
void orc_sigmoid_train(const double *dec, int l, const int *labels, double *A_out, double *B_out) {
    double prior1 = 0, prior0 = 0;
    for (int i = 0; i < l; i++) { if (labels[i] > 0) prior1 += 1; else prior0 += 1; }
    const int max_iter = 100;
    const double min_step = 1e-10, sigma = 1e-12, eps = 1e-5;
    const double hiTarget = (prior1 + 1.0) / (prior1 + 2.0), loTarget = 1 / (prior0 + 2.0);
    vector<double> t(l);
    double A = 0.0, B = log((prior0 + 1.0) / (prior1 + 1.0)), fval = 0.0;
    for (int i = 0; i < l; i++) {
        t[i] = labels[i] > 0 ? hiTarget : loTarget;
        double fApB = dec[i] * A + B;
        if (fApB >= 0) fval += t[i] * fApB + log(1 + exp(-fApB));
        else fval += (t[i] - 1) * fApB + log(1 + exp(fApB));
    }
    int iter;
    for (iter = 0; iter < max_iter; iter++) {
        double h11 = sigma, h22 = sigma, h21 = 0.0, g1 = 0.0, g2 = 0.0;
        for (int i = 0; i < l; i++) {
            double fApB = dec[i] * A + B, p, q;
            if (fApB >= 0) { p = exp(-fApB) / (1.0 + exp(-fApB)); q = 1.0 / (1.0 + exp(-fApB)); }
            else { p = 1.0 / (1.0 + exp(fApB)); q = exp(fApB) / (1.0 + exp(fApB)); }
            double d2 = p * q;
            h11 += dec[i] * dec[i] * d2;
            h22 += d2;
            h21 += dec[i] * d2;
            double d1 = t[i] - p;
            g1 += dec[i] * d1;
            g2 += d1;
        }
        if (fabs(g1) < eps && fabs(g2) < eps) break;
        double det = h11 * h22 - h21 * h21;
        double dA = -(h22 * g1 - h21 * g2) / det;
        double dB = -(-h21 * g1 + h11 * g2) / det;
        double gd = g1 * dA + g2 * dB;
        double stepsize = 1;
        while (stepsize >= min_step) {
            double newA = A + stepsize * dA, newB = B + stepsize * dB, newf = 0.0;
            for (int i = 0; i < l; i++) {
                double fApB = dec[i] * newA + newB;
                if (fApB >= 0) newf += t[i] * fApB + log(1 + exp(-fApB));
                else newf += (t[i] - 1) * fApB + log(1 + exp(fApB));
            }
            if (newf < fval + 0.0001 * stepsize * gd) { A = newA; B = newB; fval = newf; break; }
            stepsize = stepsize / 2.0;
        }
        if (stepsize < min_step) break;
    }
    *A_out = A;
    *B_out = B;
}

// SVC::multiclass_probability (svc.cpp:206-263); r is k x k row-major, p has k entries.
void orc_multiclass_probability(const double *r, int k, double *p) {
    int max_iter = std::max(100, k);
    vector<double> Q((size_t) k * k, 0.0), Qp(k);
    double eps = 0.005 / k;
    for (int t = 0; t < k; t++) {
        p[t] = 1.0 / k;
        Q[t * k + t] = 0;
        for (int j = 0; j < t; j++) {
            Q[t * k + t] += r[j * k + t] * r[j * k + t];
            Q[t * k + j] = Q[j * k + t];
        }
        for (int j = t + 1; j < k; j++) {
            Q[t * k + t] += r[j * k + t] * r[j * k + t];
            Q[t * k + j] = -r[j * k + t] * r[t * k + j];
        }
    }
    for (int iter = 0; iter < max_iter; iter++) {
        double pQp = 0;
        for (int t = 0; t < k; t++) {
            Qp[t] = 0;
            for (int j = 0; j < k; j++) Qp[t] += Q[t * k + j] * p[j];
            pQp += p[t] * Qp[t];
        }
        double max_error = 0;
        for (int t = 0; t < k; t++) max_error = std::max(max_error, fabs(Qp[t] - pQp));
        if (max_error < eps) break;
        for (int t = 0; t < k; t++) {
            double diff = (-Qp[t] + pQp) / Q[t * k + t];
            p[t] += diff;
            pQp = (pQp + diff * (diff * Q[t * k + t] + 2 * Qp[t])) / (1 + diff) / (1 + diff);
            for (int j = 0; j < k; j++) {
                Qp[j] = (Qp[j] + diff * Q[t * k + j]) / (1 + diff);
                p[j] /= (1 + diff);
            }
        }
    }
}

}  // extern "C"
