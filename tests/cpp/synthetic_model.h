// The stand-in model of the generation-loop tests and of the test worker.
#ifndef NCNN_MOE_TESTS_SYNTHETIC_MODEL_H
#define NCNN_MOE_TESTS_SYNTHETIC_MODEL_H

#include <cstdint>
#include <vector>

// A stand-in for the model: the logits after a Session's position p depend on (session, p, token fed)
// through an integer hash, every value a multiple of 2^-20 in [-8, 14), so a checker in another
// language reproduces them exactly.  It writes device rows, as a decode step on the GPU would.
inline std::vector<float> synthetic_logits(uint32_t vocab, uint32_t session, uint32_t position, int32_t fed_token)
{
    const uint32_t seed = (session * 0x9E3779B1u) ^ (position * 0x85EBCA77u) ^ (static_cast<uint32_t>(fed_token) * 0xC2B2AE3Du) ^ 0x27D4EB2Fu;
    std::vector<float> row(vocab);
    for (uint32_t v = 0; v < vocab; ++v)
    {
        uint32_t h = v * 2654435761u + seed;
        h ^= h >> 15;
        h *= 2246822519u;
        h ^= h >> 13;
        h *= 3266489917u;
        h ^= h >> 16;
        float value = static_cast<float>(h >> 8) * (1.0f / 1048576.0f) - 8.0f;
        if ((h & 1023u) == 0u)
            value += 6.0f;
        row[v] = value;
    }
    return row;
}

#endif // NCNN_MOE_TESTS_SYNTHETIC_MODEL_H
