// Writes the known-answer vector for the operand generator: the draws that the C++ standard
// library's own std::default_random_engine (default-constructed) feeds through
// std::uniform_real_distribution<float>(-1, 1).  Uses nothing but the standard library.
//   g++ -O1 make_rng_fixture.cpp -o /tmp/make_rng_fixture && /tmp/make_rng_fixture > minstd_uniform.json
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>

static uint32_t bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }

int main() {
    std::default_random_engine generator;
    std::uniform_real_distribution<float> distribution(-1.0, 1.0);
    const int head = 256;
    const long total = 1000000;
    uint32_t xor_all = 0;
    uint64_t sum_all = 0;
    std::printf("{\n  \"engine_min\": %lu, \"engine_max\": %lu,\n  \"head_f32_bits\": [",
                (unsigned long)generator.min(), (unsigned long)generator.max());
    float last = 0.f;
    for (long i = 0; i < total; ++i) {
        float t = distribution(generator);
        uint32_t b = bits(t);
        xor_all ^= b;
        sum_all += b;
        if (i < head) std::printf("%s%u", i ? ", " : "", b);
        last = t;
    }
    std::printf("],\n  \"total\": %ld, \"xor_f32_bits\": %u, \"sum_f32_bits_mod_2_64\": %llu, \"last_f32_bits\": %u\n}\n",
                total, xor_all, (unsigned long long)sum_all, bits(last));
    return 0;
}
