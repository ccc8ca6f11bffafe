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
// algorithm glibc (>= 2.27) uses for expf, in the form its FMA build takes (libm's bits on all 2^32 arguments).  `tab` points at the 32-entry table (LDS or constant).
// The reference's kernels call libm expf on the host (kernelmatrix_kernel.cpp:71-72,87-89).
// The routine without its two out-of-range cases: the right result for -0x1.9fe368p6 <= x <= 0x1.62e42ep6 and for NaN.
__device__ __forceinline__ float tsvm_expf_in_range(float x, const uint64_t *tab) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32;
    const double SHIFT = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32;
    // (the out-of-range cases are selected afterwards, in tsvm_expf: no branches in the epilogue; a NaN argument
    // comes out as NaN through the arithmetic itself)
    // (k and r both come straight from the exact product x * 32/ln2, as in the library's FMA build, where the
    // compiler fuses the product into the addition of SHIFT and into the subtraction of k: with a rounded product
    // two of the 2^32 arguments gave a neighbouring float)
    double xd = (double) x;
    double kd = __builtin_fma(InvLn2N, xd, SHIFT);
    const uint32_t ki = (uint32_t) __double2loint(kd);
    kd -= SHIFT;
    double r = __builtin_fma(InvLn2N, xd, -kd);
    // s = 2^(k/32): table entry with k/32 added into the exponent field.  The published routine adds
    // ki << 47 to the 64-bit entry; the low word of that term is zero, so only the high word changes.
    const uint64_t t = tab[ki & 31];
    double s = __hiloint2double((int) ((uint32_t) (t >> 32) + (ki << 15)), (int) (uint32_t) t);
    double zz = __builtin_fma(C0, r, C1);
    double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(zz, r2, y);
    y = y * s;
    return (float) y;
}
__device__ __forceinline__ float tsvm_expf(float x, const uint64_t *tab) {
    float res = tsvm_expf_in_range(x, tab);
    res = x > 0x1.62e42ep6f ? __builtin_inff() : res;   // > log(2^128)
    res = x < -0x1.9fe368p6f ? 0.0f : res;              // < log(2^-150)
    return res;
}

// powf, the routine glibc (>= 2.28) uses: log2(x) from a 16-entry table and a quartic, in double, times y, then
// 2^that through the expf table and cubic; every a*b+c is one fma (the form the library's FMA build takes on the
// hosts this was checked on: all 2^32 arguments x for each of fourteen exponents give libm's bits).  Entries are
// {1/c, log2(c) * 32}; the polynomial and the product y*log2(x) carry the same factor 32 (the exp table's size).
__constant__ const double TSVM_POWF_LOG2_TAB[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2 * 32}, {0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2 * 32},
    {0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2 * 32},  {0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2 * 32},
    {0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2 * 32}, {0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3 * 32},
    {0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3 * 32}, {0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4 * 32},
    {0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5 * 32}, {0x1p+0, 0x0p+0 * 32},
    {0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4 * 32},  {0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3 * 32},
    {0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3 * 32},  {0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2 * 32},
    {0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2 * 32},  {0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2 * 32}};

// 0: not an integer, 1: odd integer, 2: even integer (the float with bit pattern iy)
__device__ __forceinline__ int tsvm_powf_checkint(uint32_t iy) {
    const int e = iy >> 23 & 0xff;
    if (e < 0x7f) return 0;
    if (e > 0x7f + 23) return 2;
    if (iy & ((1u << (0x7f + 23 - e)) - 1)) return 0;
    if (iy & (1u << (0x7f + 23 - e))) return 1;
    return 2;
}
__device__ __forceinline__ bool tsvm_powf_zeroinfnan(uint32_t ix) { return 2 * ix - 1 >= 2u * 0x7f800000 - 1; }

// `tab`: the 32-entry table of tsvm_expf (LDS or constant).  The reference calls libm powf on float arguments
// (kernelmatrix_kernel.cpp:94-100).
// (Not inlined, nor tanhf below: the routines are long, their callers' epilogues are instantiated dozens of times, and
// neither kernel is on a path where a call matters.)
__device__ __noinline__ float tsvm_powf(float x, float y, const uint64_t *tab) {
    const double A0 = 0x1.27616c9496e0bp-2 * 32, A1 = -0x1.71969a075c67ap-2 * 32, A2 = 0x1.ec70a6ca7baddp-2 * 32,
                 A3 = -0x1.7154748bef6c8p-1 * 32, A4 = 0x1.71547652ab82bp0 * 32;
    uint32_t sign_bias = 0;
    uint32_t ix = __float_as_uint(x);
    const uint32_t iy = __float_as_uint(y);
    if (ix - 0x00800000 >= 0x7f800000 - 0x00800000 || tsvm_powf_zeroinfnan(iy)) {
        // x is subnormal, zero, negative, infinite or NaN, or y is zero, infinite or NaN
        if (tsvm_powf_zeroinfnan(iy)) {
            if (2 * iy == 0) return 2 * (ix ^ 0x00400000) > 2u * 0x7fc00000 ? x + y : 1.0f;   // (a signalling NaN stays a NaN)
            if (ix == 0x3f800000) return 2 * (iy ^ 0x00400000) > 2u * 0x7fc00000 ? x + y : 1.0f;
            if (2 * ix > 2u * 0x7f800000 || 2 * iy > 2u * 0x7f800000) return x + y;
            if (2 * ix == 2 * 0x3f800000) return 1.0f;
            if ((2 * ix < 2 * 0x3f800000) == !(iy & 0x80000000)) return 0.0f;   // |x| < 1 and y = inf, or |x| > 1 and y = -inf
            return y * y;
        }
        if (tsvm_powf_zeroinfnan(ix)) {
            float x2 = x * x;
            if ((ix & 0x80000000) && tsvm_powf_checkint(iy) == 1) x2 = -x2;
            return (iy & 0x80000000) ? 1 / x2 : x2;
        }
        if (ix & 0x80000000) {   // finite x < 0
            const int yint = tsvm_powf_checkint(iy);
            if (yint == 0) return __uint_as_float(0x7fc00000u);   // a quiet NaN (libm returns one of either sign)
            if (yint == 1) sign_bias = 1u << (5 + 11);
            ix &= 0x7fffffff;
        }
        if (ix < 0x00800000) {   // subnormal x: normalised
            ix = __float_as_uint(x * 0x1p23f);
            ix &= 0x7fffffff;
            ix -= 23 << 23;
        }
    }
    // x = 2^k z, z in [0x1.66p-1, 0x1.66p0): log2(x) * 32 = k * 32 + log2(c) * 32 + log2(z/c) * 32
    const uint32_t tmp = ix - 0x3f330000;
    const int i = (tmp >> (23 - 4)) % 16;
    const uint32_t top = tmp & 0xff800000;
    const uint32_t iz = ix - top;
    const int k = (int32_t) top >> (23 - 5);
    const double invc = TSVM_POWF_LOG2_TAB[i][0], logc = TSVM_POWF_LOG2_TAB[i][1];
    const double z = (double) __uint_as_float(iz);
    const double r = __builtin_fma(z, invc, -1.0);
    const double y0 = logc + (double) k;
    const double r2 = r * r;
    const double yy = __builtin_fma(A0, r, A1);
    const double pp = __builtin_fma(A2, r, A3);
    const double r4 = r2 * r2;
    double q = __builtin_fma(A4, r, y0);
    q = __builtin_fma(pp, r2, q);
    const double logx = __builtin_fma(yy, r4, q);
    const double ylogx = (double) y * logx;
    if (((uint64_t) __double_as_longlong(ylogx) >> 47 & 0xffff) >= ((uint64_t) __double_as_longlong(126.0 * 32) >> 47)) {
        if (ylogx > 0x1.fffffffd1d571p+6 * 32) return sign_bias ? -__builtin_inff() : __builtin_inff();
        if (ylogx <= -150.0 * 32) return sign_bias ? -0.0f : 0.0f;
    }
    // 2^(ylogx / 32): as in tsvm_expf, with the sign of the result carried into the table entry's top bit
    const double SHIFT = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32;
    double kd = ylogx + SHIFT;
    const uint64_t ki = (uint64_t) __double_as_longlong(kd);
    kd -= SHIFT;
    const double rr = ylogx - kd;
    uint64_t t = tab[ki % 32];
    t += (ki + sign_bias) << (52 - 5);
    const double s = __longlong_as_double((long long) t);
    const double zz = __builtin_fma(C0, rr, C1);
    const double rr2 = rr * rr;
    double e = __builtin_fma(C2, rr, 1.0);
    e = __builtin_fma(zz, rr2, e);
    return (float) (e * s);
}

// expm1f and tanhf in float arithmetic, statement by statement the routines glibc's libm uses (the fdlibm float
// versions): all 2^32 arguments give libm's bits.  No operation here may be fused or reassociated (the library is
// built with -ffp-contract=off; float division is correctly rounded).  The reference calls libm tanhf
// (kernelmatrix_kernel.cpp:102-108).
__device__ __forceinline__ float tsvm_expm1f(float x) {
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f, o_threshold = 8.8721679688e+01f, ln2_hi = 6.9313812256e-01f,
                ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f, Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f,
                Q3 = -7.9365076090e-05f, Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
    float y, hi, lo, c = 0.0f, t, e;
    int k;
    uint32_t hx = __float_as_uint(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;
    if (hx >= 0x4195b844u) {   // |x| >= 27 ln 2
        if (hx >= 0x42b17218u) {
            if (hx > 0x7f800000u) return x + x;
            if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;
    }
    if (hx > 0x3eb17218u) {   // |x| > 0.5 ln 2: x = k ln 2 + (hi - lo)
        if (hx < 0x3F851592u) {
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int) (invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
            t = (float) k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {   // |x| < 2^-25
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }
    const float hfx = 0.5f * x;
    const float hxs = x * hfx;
    const float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
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
        y = __uint_as_float(__float_as_uint(y) + ((uint32_t) k << 23));   // k added to the exponent
        return y - one;
    }
    if (k < 23) {
        t = __uint_as_float(0x3f800000u - (0x1000000u >> k));   // 1 - 2^-k
        y = t - (e - x);
        y = __uint_as_float(__float_as_uint(y) + ((uint32_t) k << 23));
    } else {
        t = __uint_as_float((uint32_t) (0x7f - k) << 23);       // 2^-k
        y = x - (e + t);
        y += one;
        y = __uint_as_float(__float_as_uint(y) + ((uint32_t) k << 23));
    }
    return y;
}

__device__ __noinline__ float tsvm_tanhf(float x) {
    const float one = 1.0f, tiny = 1.0e-30f;
    const int jx = (int) __float_as_uint(x), ix = jx & 0x7fffffff;
    if (ix >= 0x7f800000) return jx >= 0 ? one / x + one : one / x - one;
    float z;
    if (ix < 0x41b00000) {   // |x| < 22
        if (ix == 0) return x;
        if (ix < 0x24000000) return x * (one + x);   // |x| < 2^-55
        if (ix >= 0x3f800000) {
            const float t = tsvm_expm1f(2.0f * __builtin_fabsf(x));
            z = one - 2.0f / (t + 2.0f);
        } else {
            const float t = tsvm_expm1f(-2.0f * __builtin_fabsf(x));
            z = -t / (t + 2.0f);
        }
    } else {
        z = one - tiny;
    }
    return jx >= 0 ? z : -z;
}

// The argument of the RBF kernel's expf (kernelmatrix_kernel.cpp:87-89): -(sd0 + sd1 - 2*dot) * gamma, as a float;
// 2*dot is exact, so the fma rounds exactly where the subtraction would.
__device__ __forceinline__ float tsvm_rbf_arg(double dot, double sd0, double sd1, const KernelParam &p) {
    return (float) (-__builtin_fma(-2.0, dot, sd0 + sd1) * p.gamma);
}

// Kernel epilogues (kernelmatrix_kernel.cpp:61-108).  sd0/sd1 are the two rows' self dot products.
// The RBF / polynomial / sigmoid values are floats by definition (expf / powf / tanhf); this returns that
// float, so that a caller storing float rows pays for no round trip through double.
__device__ __forceinline__ float tsvm_epilogue_f32(double dot, double sd0, double sd1, const KernelParam &p,
                                                   const uint64_t *tab) {
    switch (p.kernel_type) {
        case TSVM_POLY: {
            const float arg = (float) __builtin_fma(p.gamma, dot, p.coef0);
            return tsvm_powf(arg, (float) p.degree, tab);
        }
        case TSVM_SIGMOID: {
            const float arg = (float) __builtin_fma(p.gamma, dot, p.coef0);
            return tsvm_tanhf(arg);
        }
        default: return tsvm_expf(tsvm_rbf_arg(dot, sd0, sd1, p), tab);
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

// Kernel rows are written once by get_rows and read once by update_f, gigabytes per
// launch: marked non-temporal, they pass through the L2 without pushing out what is read again and again (the data
// rows, f, the solver's block).  Measured on 512 x 426,315 rows: get_rows 0.47 -> 0.40 ms, update_f 6.4 -> 6.8 TB/s.
// Only for stores that fill whole 64-byte runs: single values written this way reach memory as partial writes (a
// prediction batch whose rows have an odd length: 2.1 times slower; the CSR kernel: 3.7 times).
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

// Sum over the sixteen lanes of a DPP row (lanes 16r .. 16r+15); every lane of the row returns it.
__device__ __forceinline__ double dpp_row_sum_f64(double v) {
    v += dpp_f64<TSVM_DPP_XOR1>(v);
    v += dpp_f64<TSVM_DPP_XOR2>(v);
    v += dpp_f64<TSVM_DPP_HALF_MIRROR>(v);
    v += dpp_f64<TSVM_DPP_MIRROR>(v);
    return v;
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
