// Deterministic inputs of the driver: splitmix64-seeded xoshiro256** (public
// domain algorithms by Blackman and Vigna), uniform floats and Box-Muller
// normals computed in double.  The reference seeds rand() from the clock
// (ConvTest.cpp:25,40,334); a fixed generator makes every run and every machine
// see the same layer.
#pragma once

#include <math.h>
#include <stddef.h>
#include <stdint.h>

namespace fastconv {

class Xoshiro256 {
   public:
    explicit Xoshiro256(uint64_t seed) {
        uint64_t sm = seed;
        for (int i = 0; i < 4; i++) {
            uint64_t z = (sm += 0x9e3779b97f4a7c15ULL);
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
            s_[i] = z ^ (z >> 31);
        }
    }
    uint64_t Next() {
        const uint64_t result = Rotl(s_[1] * 5, 7) * 9;
        const uint64_t t = s_[1] << 17;
        s_[2] ^= s_[0];
        s_[3] ^= s_[1];
        s_[1] ^= s_[2];
        s_[0] ^= s_[3];
        s_[2] ^= t;
        s_[3] = Rotl(s_[3], 45);
        return result;
    }
    // uniform in [0, 1) with 53 random bits
    double Unit() { return (double)(Next() >> 11) * (1.0 / 9007199254740992.0); }

   private:
    static uint64_t Rotl(uint64_t v, int k) { return (v << k) | (v >> (64 - k)); }
    uint64_t s_[4];
};

inline void FillUniform(uint64_t seed, float lo, float hi, float *out, size_t n) {
    Xoshiro256 g(seed);
    for (size_t i = 0; i < n; i++) out[i] = (float)((double)lo + ((double)hi - (double)lo) * g.Unit());
}

inline void FillNormal(uint64_t seed, float sigma, float *out, size_t n) {
    Xoshiro256 g(seed);
    const double two_pi = 6.283185307179586476925286766559;
    for (size_t i = 0; i < n; i += 2) {
        double u1 = g.Unit();
        const double u2 = g.Unit();
        if (u1 < 1e-300) u1 = 1e-300;
        const double r = sqrt(-2.0 * log(u1));
        out[i] = (float)((double)sigma * r * cos(two_pi * u2));
        if (i + 1 < n) out[i + 1] = (float)((double)sigma * r * sin(two_pi * u2));
    }
}

}  // namespace fastconv
