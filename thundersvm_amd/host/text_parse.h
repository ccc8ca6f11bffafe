// Decimal text to float / double, shared by the LibSVM text loader and the model-file reader.
#pragma once
#include <cstdint>
#include <cstdlib>
#include <cstring>

namespace tsvm {

static const double kPow10[23] = {1e0,  1e1,  1e2,  1e3,  1e4,  1e5,  1e6,  1e7,  1e8,  1e9,  1e10, 1e11,
                           1e12, 1e13, 1e14, 1e15, 1e16, 1e17, 1e18, 1e19, 1e20, 1e21, 1e22};

inline bool is_blank(char c) { return c == ' ' || c == '\t' || c == '\r'; }

// A decimal number without the library call where that is provably the same.  Up to 19 significant digits fit a
// 64-bit integer w; when w < 2^53 and the decimal exponent is within +-22, w and 10^|e| are exact doubles and their
// product or quotient is the correctly rounded double of the text (one rounding).  Returns false when the text is
// anything else (more digits, a large exponent, "inf", "nan", a hexadecimal float): the caller asks strtod / strtof.
inline bool fast_decimal(const char *p, const char *lim, const char **end, double *out) {
    const char *s = p;
    bool neg = false;
    if (s < lim && (*s == '-' || *s == '+')) neg = *s++ == '-';
    uint64_t w = 0;
    int sig = 0, e10 = 0;
    bool any = false;
    for (; s < lim && *s >= '0' && *s <= '9'; ++s) {
        any = true;
        if (sig >= 19) return false;
        w = w * 10 + (uint64_t) (*s - '0');
        if (w) ++sig;
    }
    if (s < lim && *s == '.') {
        for (++s; s < lim && *s >= '0' && *s <= '9'; ++s) {
            any = true;
            if (sig >= 19) return false;
            w = w * 10 + (uint64_t) (*s - '0');
            if (w) ++sig;
            --e10;
        }
    }
    if (!any) return false;
    if (s < lim && (*s == 'e' || *s == 'E')) {
        const char *t = s + 1;
        bool eneg = false;
        if (t < lim && (*t == '-' || *t == '+')) eneg = *t++ == '-';
        if (t < lim && *t >= '0' && *t <= '9') {
            int ex = 0;
            for (; t < lim && *t >= '0' && *t <= '9'; ++t)
                if (ex < 10000) ex = ex * 10 + (*t - '0');
            e10 += eneg ? -ex : ex;
            s = t;
        }
    }
    if (s < lim && !is_blank(*s) && *s != '\n' && *s != ':') return false;   // something the simple grammar does not cover
    if (w >> 53 || e10 < -22 || e10 > 22) return false;
    double d = (double) w;
    d = e10 < 0 ? d / kPow10[-e10] : d * kPow10[e10];
    *out = neg ? -d : d;
    *end = s;
    return true;
}

// the float of sscanf("%f"): the decimal text rounded once, to float
inline float parse_float(const char *p, const char *lim, const char **end) {
    double d;
    if (fast_decimal(p, lim, end, &d)) {
        // Rounding the correctly rounded double to float gives the correctly rounded float unless the double lies
        // exactly half way between two floats (rounding is monotonic, so the double can only be on the wrong side of
        // that point by being that point).  Zero and float-normal magnitudes only.
        uint64_t bits;
        memcpy(&bits, &d, sizeof bits);
        const double ad = d < 0 ? -d : d;
        if (ad == 0.0 || (ad >= 0x1p-126 && ad < 0x1p127 && (bits & 0x1fffffffull) != 0x10000000ull)) return (float) d;
    }
    char *q;
    const float v = strtof(p, &q);   // (the text is NUL-terminated)
    *end = q;
    return v;
}

inline double parse_double(const char *p, const char *lim, const char **end) {
    double d;
    if (fast_decimal(p, lim, end, &d)) return d;
    char *q;
    d = strtod(p, &q);
    *end = q;
    return d;
}

}  // namespace tsvm
