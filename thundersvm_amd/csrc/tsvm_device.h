// Device-side helpers shared by the gfx950 kernels: the float-rounded kernel epilogues, the
// index-set predicates and wavefront reductions.  Everything here is plain IEEE arithmetic with
// explicit fma(); the library is built with -ffp-contract=off so nothing else fuses.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TSVM_WAVE 64

enum { TSVM_LINEAR = 0, TSVM_POLY = 1, TSVM_RBF = 2, TSVM_SIGMOID = 3, TSVM_PRECOMPUTED = 4 };

struct KernelParam {
    int kernel_type;
    int degree;
    double gamma;
    double coef0;
};

// 2^(i/32) table with i << 47 subtracted (so the integer part of k can be added into the exponent field).
__constant__ const uint64_t TSVM_EXP2F_TAB[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// expf of a float argument, evaluated in double and rounded once to float: the table-driven
// algorithm glibc (>= 2.27) uses for expf.  `tab` points at the 32-entry table (LDS or constant).
// The reference's kernels call libm expf on the host (kernelmatrix_kernel.cpp:71-72,87-89).
__device__ __forceinline__ float tsvm_expf(float x, const uint64_t *tab) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32;
    const double SHIFT = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32;
    // The main path runs unconditionally and the out-of-range cases are selected afterwards (no
    // branches in the epilogue); a NaN argument comes out as NaN through the arithmetic itself.
    double xd = (double) x;
    double z = InvLn2N * xd;
    double kd = z + SHIFT;
    const uint32_t ki = (uint32_t) __double2loint(kd);
    kd -= SHIFT;
    double r = z - kd;
    // s = 2^(k/32): table entry with k/32 added into the exponent field.  The published routine adds
    // ki << 47 to the 64-bit entry; the low word of that term is zero, so only the high word changes.
    const uint64_t t = tab[ki & 31];
    double s = __hiloint2double((int) ((uint32_t) (t >> 32) + (ki << 15)), (int) (uint32_t) t);
    double zz = __builtin_fma(C0, r, C1);
    double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(zz, r2, y);
    y = y * s;
    float res = (float) y;
    res = x > 0x1.62e42ep6f ? __builtin_inff() : res;   // > log(2^128)
    res = x < -0x1.9fe368p6f ? 0.0f : res;              // < log(2^-150)
    return res;
}

// Kernel epilogues (kernelmatrix_kernel.cpp:61-108).  sd0/sd1 are the two rows' self dot products.
// The RBF / polynomial / sigmoid values are floats by definition (expf / powf / tanhf); this returns that
// float, so that a caller storing float rows pays for no round trip through double.
__device__ __forceinline__ float tsvm_epilogue_f32(double dot, double sd0, double sd1, const KernelParam &p,
                                                   const uint64_t *tab) {
    switch (p.kernel_type) {
        case TSVM_POLY: {
            // powf / tanhf of a float-rounded argument: evaluated in double and rounded once to float
            const float arg = (float) __builtin_fma(p.gamma, dot, p.coef0);
            return (float) pow((double) arg, (double) p.degree);
        }
        case TSVM_SIGMOID: {
            const float arg = (float) __builtin_fma(p.gamma, dot, p.coef0);
            return (float) tanh((double) arg);
        }
        default: {
            // -(sd0 + sd1 - 2*dot) * gamma; 2*dot is exact, so the fma rounds exactly where the subtraction would
            const double arg = -__builtin_fma(-2.0, dot, sd0 + sd1) * p.gamma;
            return tsvm_expf((float) arg, tab);
        }
    }
}

__device__ __forceinline__ double tsvm_epilogue(double dot, double sd0, double sd1, const KernelParam &p,
                                                const uint64_t *tab) {
    return p.kernel_type == TSVM_LINEAR ? dot : (double) tsvm_epilogue_f32(dot, sd0, sd1, p, tab);
}

// the value as an element of a kernel row (float rows are never used with the linear kernel)
template <typename TO>
__device__ __forceinline__ TO tsvm_epilogue_as(double dot, double sd0, double sd1, const KernelParam &p,
                                               const uint64_t *tab) {
    if constexpr (sizeof(TO) == 4) return tsvm_epilogue_f32(dot, sd0, sd1, p, tab);
    else return tsvm_epilogue(dot, sd0, sd1, p, tab);
}

// Kernel rows are written once by get_rows and read once by update_f (or by the predict reduction), gigabytes per
// launch: marked non-temporal, they pass through the L2 without pushing out what is read again and again (the data
// rows, f, the solver's block).  Measured on 512 x 426,315 rows: get_rows 0.47 -> 0.40 ms, update_f 6.4 -> 6.8 TB/s.
template <typename T>
__device__ __forceinline__ void store_streaming(T *p, T v) { __builtin_nontemporal_store(v, p); }
template <typename T>
__device__ __forceinline__ T load_streaming(const T *p) { return __builtin_nontemporal_load(p); }

// include/thundersvm/kernel/smo_kernel.h:13-23
__device__ __forceinline__ bool is_I_up(double a, double y, double Cp, double Cn) {
    return (y > 0 && a < Cp) || (y < 0 && a > 0);
}
__device__ __forceinline__ bool is_I_low(double a, double y, double Cp, double Cn) {
    return (y > 0 && a > 0) || (y < 0 && a < Cn);
}

__device__ __forceinline__ double shfl_xor_f64(double v, int mask) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __shfl_xor(lo, mask, TSVM_WAVE);
    hi = __shfl_xor(hi, mask, TSVM_WAVE);
    return __hiloint2double(hi, lo);
}

// Cross-lane moves on the VALU (DPP) instead of the LDS crossbar.  Inside a 16-lane row, quad_perm
// xor-1 / xor-2, row_half_mirror and row_mirror make every lane see the row's result in four steps;
// row_bcast:15 into rows 1 and 3, then row_bcast:31 into rows 2 and 3, carry the row results across,
// so that lane 63 ends up with the wavefront's result, which v_readlane makes uniform.  The full-mask
// moves name no previous value (old = 0 with bound_ctrl), which lets the compiler fold them into the
// consuming 32-bit instruction (v_min_i32 ... quad_perm) instead of copying the source first.
#define TSVM_DPP_XOR1 0xB1          /* quad_perm [1,0,3,2] */
#define TSVM_DPP_XOR2 0x4E          /* quad_perm [2,3,0,1] */
#define TSVM_DPP_HALF_MIRROR 0x141
#define TSVM_DPP_MIRROR 0x140
#define TSVM_DPP_BCAST15 0x142
#define TSVM_DPP_BCAST31 0x143

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_i32(int x) {
    if (ROW_MASK == 0xf) return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xf, 0xf, true);
    return __builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xf, false);   // rows outside the mask keep x
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_f64(double v) {
    int lo = dpp_i32<CTRL, ROW_MASK>(__double2loint(v)), hi = dpp_i32<CTRL, ROW_MASK>(__double2hiint(v));
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double readlane_f64(double v, int lane) {
    int lo = __builtin_amdgcn_readlane(__double2loint(v), lane), hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}

// Wavefront reductions used by the local solvers.  A (value, index) lexicographic minimum -- the
// smallest value wins and, among equal values, the smallest index: the serial loops' "first strict
// improvement" rule (smo_kernel.cpp:43-49,80-89) -- is taken in two branch-free passes: the minimum
// value, then the minimum index among the elements that hold that value.  Every lane returns the
// wavefront's result.  Callers never pass NaN.
//
// v_min_f64 / v_max_f64 are written out because the compiler turns `b < a ? b : a` into a compare
// and two 32-bit selects, three issue slots instead of one, and the solvers are bound by issue slots.
// The instructions may return either zero for min(+0, -0); the solvers only compare and subtract
// these values, where the sign of a zero changes nothing.
__device__ __forceinline__ double fmin_f64(double a, double b) {
    double r;
    asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ double fmax_f64(double a, double b) {
    double r;
    asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ int imin_sel(int a, int b) { return b < a ? b : a; }

__device__ __forceinline__ double wave_min_f64(double v) {
    v = fmin_f64(v, dpp_f64<TSVM_DPP_XOR1>(v));
    v = fmin_f64(v, dpp_f64<TSVM_DPP_XOR2>(v));
    v = fmin_f64(v, dpp_f64<TSVM_DPP_HALF_MIRROR>(v));
    v = fmin_f64(v, dpp_f64<TSVM_DPP_MIRROR>(v));
    v = fmin_f64(v, dpp_f64<TSVM_DPP_BCAST15, 0xa>(v));
    v = fmin_f64(v, dpp_f64<TSVM_DPP_BCAST31, 0xc>(v));
    return readlane_f64(v, 63);
}
__device__ __forceinline__ double wave_max_f64(double v) {
    v = fmax_f64(v, dpp_f64<TSVM_DPP_XOR1>(v));
    v = fmax_f64(v, dpp_f64<TSVM_DPP_XOR2>(v));
    v = fmax_f64(v, dpp_f64<TSVM_DPP_HALF_MIRROR>(v));
    v = fmax_f64(v, dpp_f64<TSVM_DPP_MIRROR>(v));
    v = fmax_f64(v, dpp_f64<TSVM_DPP_BCAST15, 0xa>(v));
    v = fmax_f64(v, dpp_f64<TSVM_DPP_BCAST31, 0xc>(v));
    return readlane_f64(v, 63);
}
__device__ __forceinline__ int wave_min_i32(int v) {
    v = imin_sel(v, dpp_i32<TSVM_DPP_XOR1>(v));
    v = imin_sel(v, dpp_i32<TSVM_DPP_XOR2>(v));
    v = imin_sel(v, dpp_i32<TSVM_DPP_HALF_MIRROR>(v));
    v = imin_sel(v, dpp_i32<TSVM_DPP_MIRROR>(v));
    v = imin_sel(v, dpp_i32<TSVM_DPP_BCAST15, 0xa>(v));
    v = imin_sel(v, dpp_i32<TSVM_DPP_BCAST31, 0xc>(v));
    return __builtin_amdgcn_readlane(v, 63);
}

// Maps the launch's linear workgroup id to a logical one so that logical neighbours run on the
// same XCD (the hardware deals consecutive workgroup ids round-robin over the 8 XCDs, each with
// its own L2).
__device__ __forceinline__ unsigned xcd_remap(unsigned pid, unsigned nwg) {
    const unsigned NX = 8;
    unsigned per = nwg / NX, rem = nwg % NX;
    unsigned xcd = pid % NX, local = pid / NX;
    unsigned base = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
    return base + local;
}
