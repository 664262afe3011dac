// Test-data generators of the harness.
// The reference's generators (/root/reference/bfAintBGemm/random_gen.hpp:5-66) fill float matrices
// with a leading dimension from libc rand() seeded by the wall clock, so no two runs agree.
// Here every generator takes a seed and uses a fixed, documented generator (splitmix64 for seeding,
// xoshiro256** for the stream, Box-Muller for normals) so the same bits come out on every machine:
//   rand_vector_2d            uniform floats in [min_v, max_v)                (random_gen.hpp:5-16)
//   rand_vector_2d_int_a/_b/_scale   integers in {-2,-1,0,1}, the reference's test regime (:18-54)
//   rand_vector_2d_normal     N(0,1) activations
//   rand_vector_2d_int_range  uniform integers in [lo, hi]  (int8: -128..127, int4: -8..7)
#pragma once
#include <cmath>
#include <cstdint>

namespace bfaintb_host {

struct Rng {
    std::uint64_t s[4];
    explicit Rng(std::uint64_t seed)
    {
        for (auto& w : s) {  // splitmix64
            seed += 0x9e3779b97f4a7c15ull;
            std::uint64_t z = seed;
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
            w = z ^ (z >> 31);
        }
    }
    static std::uint64_t rotl(std::uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    std::uint64_t next()  // xoshiro256**
    {
        const std::uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]; s[2] ^= t; s[3] = rotl(s[3], 45);
        return r;
    }
    double uniform() { return double(next() >> 11) * (1.0 / 9007199254740992.0); }  // [0,1)
    std::int64_t range(std::int64_t lo, std::int64_t hi) { return lo + std::int64_t(next() % std::uint64_t(hi - lo + 1)); }
    double normal()
    {
        double u1 = uniform(), u2 = uniform();
        if (u1 < 1e-300) u1 = 1e-300;
        return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2);
    }
};

}  // namespace bfaintb_host

inline void rand_vector_2d(float* v, int row, int col, int ld, float min_v = 0, float max_v = 1, std::uint64_t seed = 0)
{
    bfaintb_host::Rng g(seed);
    for (int r = 0; r < row; r++)
        for (int c = 0; c < col; c++) v[r * (std::size_t)ld + c] = static_cast<float>(min_v + g.uniform() * (max_v - min_v));
}

inline void rand_vector_2d_int_range(float* v, int row, int col, int ld, int lo, int hi, std::uint64_t seed)
{
    bfaintb_host::Rng g(seed);
    for (int r = 0; r < row; r++)
        for (int c = 0; c < col; c++) v[r * (std::size_t)ld + c] = static_cast<float>(g.range(lo, hi));
}

// The reference regime: rand() % 4 - 2.
inline void rand_vector_2d_int_a(float* v, int row, int col, int ld, std::uint64_t seed = 1) { rand_vector_2d_int_range(v, row, col, ld, -2, 1, seed); }
inline void rand_vector_2d_int_b(float* v, int row, int col, int ld, std::uint64_t seed = 2) { rand_vector_2d_int_range(v, row, col, ld, -2, 1, seed); }
inline void rand_vector_2d_int_scale(float* v, int row, int col, int ld, std::uint64_t seed = 3) { rand_vector_2d_int_range(v, row, col, ld, -2, 1, seed); }

inline void rand_vector_2d_normal(float* v, int row, int col, int ld, std::uint64_t seed)
{
    bfaintb_host::Rng g(seed);
    for (int r = 0; r < row; r++)
        for (int c = 0; c < col; c++) v[r * (std::size_t)ld + c] = static_cast<float>(g.normal());
}
