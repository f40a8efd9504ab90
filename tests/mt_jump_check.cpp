// Host-side check of brainstorm_amd/csrc/mt_jump.h, built and run by test_mt_jump.py.
//   mt_jump_check DISTANCE COUNT < 624 key words (decimal)
// prints, for k = 1 .. COUNT, the 624-word block k*DISTANCE words ahead of the given one, formed the
// way the device forms it: as the XOR combination of the stream that the polynomial selects.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../brainstorm_amd/csrc/mt_jump.h"

using namespace bship::mtjump;

int main(int argc, char** argv) {
    if (argc != 3) return 2;
    const unsigned long long distance = strtoull(argv[1], nullptr, 10);
    const int count = atoi(argv[2]);
    std::vector<uint32_t> w(kPolyBits + kN);
    for (int i = 0; i < kN; ++i) {
        unsigned long long v;
        if (scanf("%llu", &v) != 1) return 3;
        w[i] = static_cast<uint32_t>(v);
    }
    for (int n = kN; n < kPolyBits + kN; ++n) w[n] = next_word(&w[n - kN]);
    std::vector<uint32_t> polys;
    if (!jump_polynomials(distance, count, polys)) return 4;
    for (int k = 0; k < count; ++k) {
        const uint32_t* g = &polys[static_cast<size_t>(k) * kPolyWords32];
        for (int j = 0; j < kN; ++j) {
            uint32_t acc = 0;
            for (int i = 0; i < kPolyBits; ++i)
                if ((g[i >> 5] >> (i & 31)) & 1u) acc ^= w[i + j];
            printf("%u\n", acc);
        }
    }
    return 0;
}
