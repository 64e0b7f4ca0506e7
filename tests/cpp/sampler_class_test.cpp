// Drives mako::gen::Sampler (include/gen/sampler.hpp) through a scripted decode session and prints what it
// returned, one line per step, for tests/test_gpu_cpp_class.py to compare with the oracle.
//   sampler_class_test <logits.f32> <n_vocab> <steps> <seed> <mode> T top_k top_p min_p presence frequency repetition
// mode 0: tok = sample(row); accept(tok)                      (src/gen/session.cpp:441-445, 419-421)
// mode 1: tok = verify(row, draft = first max of the row, acc); accept(tok)   (src/gen/session.cpp:481-496)
// Also checks the constructor's std::invalid_argument on an empty vocabulary (src/gen/sampler.cpp:11-12).
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "gen/sampler.hpp"

int main(int argc, char** argv)
{
    using mako::gen::Sampler;
    using mako::gen::SamplingParams;
    bool threw = false;
    try {
        Sampler bad(SamplingParams{}, 0, 1);
    } catch (const std::invalid_argument&) {
        threw = true;
    }
    std::printf("empty_vocab_throws %d\n", threw ? 1 : 0);
    if (argc < 13)
        return threw ? 0 : 1;
    const uint32_t v = uint32_t(std::atoi(argv[2])), steps = uint32_t(std::atoi(argv[3]));
    const uint64_t seed = std::strtoull(argv[4], nullptr, 10);
    const int mode = std::atoi(argv[5]);
    SamplingParams p;
    p.temperature = float(std::atof(argv[6]));
    p.top_k = uint32_t(std::atoi(argv[7]));
    p.top_p = float(std::atof(argv[8]));
    p.min_p = float(std::atof(argv[9]));
    p.presence_penalty = float(std::atof(argv[10]));
    p.frequency_penalty = float(std::atof(argv[11]));
    p.repetition_penalty = float(std::atof(argv[12]));
    std::vector<float> logits(size_t(v) * steps);
    FILE* f = std::fopen(argv[1], "rb");
    if (!f || std::fread(logits.data(), sizeof(float), logits.size(), f) != logits.size())
        return 2;
    std::fclose(f);
    Sampler s(p, v, seed);
    for (uint32_t i = 0; i < steps; ++i) {
        const float* row = logits.data() + size_t(i) * v;
        int32_t tok;
        bool acc = false;
        if (mode == 0) {
            tok = s.sample(row);
        } else {
            const int32_t draft = int32_t(std::max_element(row, row + v) - row);
            tok = s.verify(row, draft, acc);
        }
        s.accept(tok);
        std::printf("%d %d\n", tok, acc ? 1 : 0);
    }
    return 0;
}
