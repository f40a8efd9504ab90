// Jump-ahead for MT19937 (host side): the polynomials that move the generator forward by a fixed
// number of words in one step, so that one long draw can be cut into segments that are generated
// in parallel and still give exactly the sequential stream.
//
// View the generator as the linear stream of raw 32-bit words w[0], w[1], ... (w[0..623] is the
// current key block; every later word follows from w[n] = w[n-227] ^ T(w[n-624], w[n-623])). Moving
// the 624-word window one word forward is a linear map A over GF(2) on the 19968 window bits. The
// lower 31 bits of the window's oldest word never influence anything, so A's minimal polynomial is
// x * phi(x) with phi the degree-19937 characteristic polynomial of MT19937. For
//     g(x) = x^d mod (x * phi(x))          (at most 19938 coefficients)
// A^d = g(A), that is
//     w[d + j] = XOR over { i : g_i = 1 } of w[i + j]        for every j >= 0,
// so the window d words ahead is a combination of windows 0 ... 19937 words ahead of the current
// one -- a fixed pattern for a fixed distance d. (Haramoto, Matsumoto, Nishimura, Panneton,
// L'Ecuyer: "Efficient jump ahead for F2-linear random number generators", 2008, evaluate g(A)
// by Horner's rule, one word at a time; summing windows of the already generated stream instead
// is the data-parallel form of the same identity.)
//
// phi is not tabulated anywhere in closed form: it is computed once per process by the
// Berlekamp-Massey algorithm from 2 * 19937 + 64 bits of one output bit of the stream.
// Pure C++ (no device code): also compiled and checked on the CPU.
#pragma once

#include <stdint.h>

#include <vector>

namespace bship {
namespace mtjump {

constexpr int kN = 624;
constexpr int kM = 397;
constexpr int kDegree = 19937;             // degree of phi
constexpr int kModDegree = kDegree + 1;    // degree of x * phi(x)
constexpr int kPolyBits = kModDegree;      // coefficients of a residue: x^0 ... x^19937
constexpr int kPolyWords32 = kN;           // 19968 bits hold them
constexpr int kWords64 = 2 * kN;           // room for a product of two residues (39936 bits)

typedef std::vector<uint64_t> Poly;        // bit i of word i/64 = coefficient of x^i

inline bool poly_bit(const Poly& p, int i) { return (p[i >> 6] >> (i & 63)) & 1u; }
inline void poly_flip(Poly& p, int i) { p[i >> 6] ^= uint64_t(1) << (i & 63); }

// p ^= q << shift (q has `qwords` significant words)
inline void poly_xor_shifted(Poly& p, const Poly& q, int qwords, int shift) {
    const int ws = shift >> 6, bs = shift & 63;
    if (bs == 0) {
        for (int i = 0; i < qwords; ++i) p[i + ws] ^= q[i];
    } else {
        for (int i = 0; i < qwords; ++i) {
            p[i + ws] ^= q[i] << bs;
            p[i + ws + 1] ^= q[i] >> (64 - bs);
        }
    }
}

// The next word of the linear stream from the 624 words before it (oldest first).
inline uint32_t next_word(const uint32_t* w) {
    const uint32_t y = (w[0] & 0x80000000u) | (w[1] & 0x7fffffffu);
    return w[kM] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
}

// x * phi(x): Berlekamp-Massey on bit 0 of w[1], w[2], ... of an arbitrary non-zero stream (the
// stream from w[1] on lives where A is invertible, so its minimal polynomial is phi itself).
inline Poly modulus() {
    const int len = 2 * kDegree + 64;
    std::vector<uint32_t> w(len + kN + 1);
    uint32_t s = 19650218u;
    for (int i = 0; i < kN; ++i) { s = 1812433253u * (s ^ (s >> 30)) + uint32_t(i); w[i] = s; }
    for (int n = kN; n < len + kN + 1; ++n) w[n] = next_word(&w[n - kN]);
    const int words = (len + 64) / 64 + 1;
    Poly c(words, 0), b(words, 0), t(words, 0);
    Poly rev(words, 0);                      // bit i = s[n - i]: the sequence so far, newest first
    c[0] = b[0] = 1;
    int l = 0, m = 1;
    for (int n = 0; n < len; ++n) {
        // rev <<= 1, then bit 0 = s[n]
        for (int i = words - 1; i > 0; --i) rev[i] = (rev[i] << 1) | (rev[i - 1] >> 63);
        rev[0] = (rev[0] << 1) | (w[n + 1] & 1u);
        uint64_t acc = 0;
        for (int i = 0; i <= (l >> 6); ++i) acc ^= c[i] & rev[i];
        const bool d = __builtin_parityll(acc);
        if (!d) {
            ++m;
        } else if (2 * l <= n) {
            t = c;
            poly_xor_shifted(c, b, words - (m >> 6) - 1, m);
            l = n + 1 - l;
            b = t;
            m = 1;
        } else {
            poly_xor_shifted(c, b, words - (m >> 6) - 1, m);
            ++m;
        }
    }
    Poly mod(kWords64, 0);
    if (l != kDegree) return mod;            // all zero: the caller refuses to jump
    // connection polynomial c (s[n] = XOR c_i s[n-i]) -> phi_j = c_(l-j); times x
    for (int j = 0; j <= l; ++j)
        if (poly_bit(c, l - j)) poly_flip(mod, j + 1);
    return mod;
}

// p (degree < 2 * kModDegree) mod `mod` (degree kModDegree), in place.
inline void reduce(Poly& p, const Poly& mod) {
    const int mod_words = kModDegree / 64 + 1;
    for (int bit = 2 * kModDegree - 1; bit >= kModDegree; --bit)
        if (poly_bit(p, bit)) poly_xor_shifted(p, mod, mod_words, bit - kModDegree);
}

inline Poly multiply(const Poly& a, const Poly& b, const Poly& mod) {
    const int res_words = kModDegree / 64 + 1;
    Poly p(kWords64 + 1, 0);
    for (int i = 0; i < kModDegree; ++i)
        if (poly_bit(a, i)) poly_xor_shifted(p, b, res_words, i);
    reduce(p, mod);
    return p;
}

// x^e mod `mod` by square and multiply (multiplying by x is a shift).
inline Poly power_of_x(uint64_t e, const Poly& mod) {
    Poly r(kWords64 + 1, 0);
    r[0] = 1;
    int top = 63;
    while (top > 0 && !((e >> top) & 1u)) --top;
    for (int bit = top; bit >= 0; --bit) {
        if (bit != top) r = multiply(r, r, mod);
        if ((e >> bit) & 1u) {
            for (int i = kWords64; i > 0; --i) r[i] = (r[i] << 1) | (r[i - 1] >> 63);
            r[0] <<= 1;
            reduce(r, mod);
        }
    }
    return r;
}

// out[(k-1) * kPolyWords32 ...] = coefficients of x^(k * distance) mod x*phi(x) for k = 1 .. count,
// as 32-bit words (bit i of word i/32). Returns false if phi could not be established.
inline bool jump_polynomials(uint64_t distance, int count, std::vector<uint32_t>& out) {
    static const Poly mod = modulus();
    if (!poly_bit(mod, kModDegree)) return false;
    out.assign(static_cast<size_t>(count) * kPolyWords32, 0u);
    const Poly g1 = power_of_x(distance, mod);
    Poly g = g1;
    for (int k = 1; k <= count; ++k) {
        if (k > 1) g = multiply(g, g1, mod);
        uint32_t* dst = &out[static_cast<size_t>(k - 1) * kPolyWords32];
        for (int i = 0; i < kPolyBits; ++i)
            if (poly_bit(g, i)) dst[i >> 5] |= uint32_t(1) << (i & 31);
    }
    return true;
}

}  // namespace mtjump
}  // namespace bship
