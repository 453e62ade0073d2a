// Host-side weight initialisation: Tensor.random(rows, cols, java.util.Random) of the
// reference (CpuBackend.java:148-152: data[i] = (float)(rand.nextGaussian() * 0.1), row
// major) reproduced bit for bit, so that a model built here has exactly the weights the
// Java model builds from the same seed.
//
// java.util.Random is specified by the JDK: 48-bit LCG, nextDouble from 26+27 bits,
// nextGaussian by the Marsaglia polar method with StrictMath.log/sqrt (fdlibm log).
//
// The stream is inherently sequential, but every polar-method attempt consumes exactly
// four LCG steps, so attempt i always starts at LCG offset 4*i.  Large tensors are
// therefore filled in parallel: the LCG is jumped ahead to each chunk's first attempt,
// chunks run independently, and their accepted pairs are concatenated in order.
#pragma clang fp contract(off)   // Java never fuses a*b+c; applies to the whole file
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

namespace {

constexpr uint64_t kMult = 0x5DEECE66DULL, kAdd = 0xBULL, kMask = (1ULL << 48) - 1;

struct JavaRandom {
    uint64_t seed;
    bool have_next = false;
    double next_next = 0.0;
};

inline int32_t next_bits(uint64_t &seed, int bits) {
    seed = (seed * kMult + kAdd) & kMask;
    return (int32_t)(uint32_t)(seed >> (48 - bits));
}
inline double next_double(uint64_t &seed) {
    int64_t hi = next_bits(seed, 26), lo = next_bits(seed, 27);
    return (double)((hi << 27) + lo) * 0x1.0p-53;
}

// seed after n LCG steps (affine map composition by repeated squaring)
uint64_t lcg_skip(uint64_t seed, uint64_t n) {
    uint64_t a = kMult, c = kAdd, acc_a = 1, acc_c = 0;
    while (n) {
        if (n & 1) { acc_a = (acc_a * a) & kMask; acc_c = (acc_c * a + c) & kMask; }
        c = ((a + 1) * c) & kMask;
        a = (a * a) & kMask;
        n >>= 1;
    }
    return (acc_a * seed + acc_c) & kMask;
}

// fdlibm __ieee754_log (what StrictMath.log is defined as).
double strict_log(double x) {
    static const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10,
                        two54 = 1.80143985094819840000e+16, Lg1 = 6.666666666666735130e-01,
                        Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01,
                        Lg4 = 2.222219843214978396e-01, Lg5 = 1.818357216161805012e-01,
                        Lg6 = 1.531383769920937332e-01, Lg7 = 1.479819860511658591e-01;
    uint64_t u;
    std::memcpy(&u, &x, 8);
    int32_t hx = (int32_t)(u >> 32);
    uint32_t lx = (uint32_t)u;
    int32_t k = 0;
    if (hx < 0x00100000) {
        if (((hx & 0x7fffffff) | lx) == 0) return -INFINITY;
        if (hx < 0) return NAN;
        k -= 54;
        x *= two54;
        std::memcpy(&u, &x, 8);
        hx = (int32_t)(u >> 32);
    }
    if (hx >= 0x7ff00000) return x + x;
    k += (hx >> 20) - 1023;
    hx &= 0x000fffff;
    int32_t i = (hx + 0x95f64) & 0x100000;
    u = (u & 0xffffffffULL) | ((uint64_t)(uint32_t)(hx | (i ^ 0x3ff00000)) << 32);
    std::memcpy(&x, &u, 8);
    k += (i >> 20);
    double f = x - 1.0;
    if ((0x000fffff & (2 + hx)) < 3) {
        if (f == 0.0) return k == 0 ? 0.0 : (double)k * ln2_hi + (double)k * ln2_lo;
        double R = f * f * (0.5 - 0.33333333333333333 * f);
        if (k == 0) return f - R;
        double dk = (double)k;
        return dk * ln2_hi - ((R - dk * ln2_lo) - f);
    }
    double s = f / (2.0 + f), dk = (double)k, z = s * s, w = z * z;
    i = hx - 0x6147a;
    int32_t j = 0x6b851 - hx;
    double t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
    double t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
    i |= j;
    double R = t2 + t1;
    if (i > 0) {
        double hfsq = 0.5 * f * f;
        if (k == 0) return f - (hfsq - s * (hfsq + R));
        return dk * ln2_hi - ((hfsq - (s * (hfsq + R) + dk * ln2_lo)) - f);
    }
    if (k == 0) return f - s * (f - R);
    return dk * ln2_hi - ((s * (f - R) - dk * ln2_lo) - f);
}

// One polar attempt from `seed` (advances it by four LCG steps).  Returns false if rejected.
inline bool polar_attempt(uint64_t &seed, double &g0, double &g1) {
    double v1 = 2 * next_double(seed) - 1;
    double v2 = 2 * next_double(seed) - 1;
    double s = v1 * v1 + v2 * v2;
    if (s >= 1 || s == 0) return false;
    double mul = std::sqrt(-2 * strict_log(s) / s);
    g0 = v1 * mul;
    g1 = v2 * mul;
    return true;
}

double next_gaussian(JavaRandom &r) {
    if (r.have_next) { r.have_next = false; return r.next_next; }
    double g0, g1;
    while (!polar_attempt(r.seed, g0, g1)) {}
    r.next_next = g1;
    r.have_next = true;
    return g0;
}

// out[i] = (float)(nextGaussian() * scale) for i < n, continuing r's stream.
void fill_gaussian(JavaRandom &r, float *out, int64_t n, double scale, int threads) {
    int64_t i = 0;
    if (n > 0 && r.have_next) { out[i++] = (float)(next_gaussian(r) * scale); }
    int64_t remaining = n - i;
    if (remaining < (1 << 16) || threads <= 1) {
        for (; i < n; i++) out[i] = (float)(next_gaussian(r) * scale);
        return;
    }
    // Parallel part: pairs_needed accepted attempts, acceptance probability pi/4.
    int64_t pairs_needed = (remaining + 1) / 2;
    while (pairs_needed > 0) {
        int64_t attempts = (int64_t)((double)pairs_needed / 0.78539816339 * 1.01) + 4096;
        int64_t per = (attempts + threads - 1) / threads;
        std::vector<std::vector<double>> acc(threads);
        std::vector<std::thread> pool;
        const uint64_t seed0 = r.seed;
        for (int t = 0; t < threads; t++) {
            pool.emplace_back([&, t] {
                int64_t a0 = (int64_t)t * per, a1 = std::min(attempts, a0 + per);
                if (a0 >= a1) return;
                uint64_t s = lcg_skip(seed0, (uint64_t)a0 * 4);
                auto &v = acc[t];
                v.reserve((size_t)((a1 - a0) * 0.8 * 2) + 16);
                double g0, g1;
                for (int64_t a = a0; a < a1; a++)
                    if (polar_attempt(s, g0, g1)) { v.push_back(g0); v.push_back(g1); }
            });
        }
        for (auto &th : pool) th.join();
        // consume chunks in order until pairs_needed is met
        int64_t consumed_attempts = attempts;
        bool done = false;
        for (int t = 0; t < threads && !done; t++) {
            auto &v = acc[t];
            int64_t have = (int64_t)v.size() / 2;
            int64_t take = std::min(have, pairs_needed);
            for (int64_t p = 0; p < take; p++) {
                out[i++] = (float)(v[2 * p] * scale);
                if (i < n) out[i++] = (float)(v[2 * p + 1] * scale);
                else { r.next_next = v[2 * p + 1]; r.have_next = true; }
            }
            pairs_needed -= take;
            if (pairs_needed == 0) {
                // replay this chunk to find the attempt index of its take-th acceptance
                int64_t a0 = (int64_t)t * per;
                uint64_t s = lcg_skip(seed0, (uint64_t)a0 * 4);
                int64_t seen = 0, a = a0;
                double g0, g1;
                while (seen < take) { if (polar_attempt(s, g0, g1)) seen++; a++; }
                consumed_attempts = a;
                done = true;
            }
        }
        r.seed = lcg_skip(seed0, (uint64_t)consumed_attempts * 4);
    }
}

}  // namespace

extern "C" {

void *deepj_host_random_create(int64_t seed) {
    auto *r = new JavaRandom;
    r->seed = ((uint64_t)seed ^ kMult) & kMask;
    return r;
}

void deepj_host_random_destroy(void *h) { delete static_cast<JavaRandom *>(h); }

// Tensor.random: n = rows*cols values (float)(nextGaussian()*scale); threads <= 0 picks the hardware count.
void deepj_host_random_fill(void *h, float *out, int64_t n, double scale, int32_t threads) {
    if (threads <= 0) threads = (int32_t)std::max(1u, std::thread::hardware_concurrency());
    if (threads > 64) threads = 64;
    fill_gaussian(*static_cast<JavaRandom *>(h), out, n, scale, threads);
}

double deepj_host_random_next_gaussian(void *h) { return next_gaussian(*static_cast<JavaRandom *>(h)); }

int32_t deepj_host_random_next_int(void *h, int32_t bound) {
    auto &r = *static_cast<JavaRandom *>(h);
    if (bound <= 0) return next_bits(r.seed, 32);
    int32_t v = next_bits(r.seed, 31), m = bound - 1;
    if ((bound & m) == 0) return (int32_t)(((int64_t)bound * (int64_t)v) >> 31);
    for (;;) {
        int32_t u = v;
        v = u % bound;
        if ((int32_t)((uint32_t)u - (uint32_t)v + (uint32_t)m) >= 0) return v;
        v = next_bits(r.seed, 31);
    }
}

float deepj_host_random_next_float(void *h) {
    auto &r = *static_cast<JavaRandom *>(h);
    return (float)next_bits(r.seed, 24) / (float)(1 << 24);
}

}  // extern "C"
