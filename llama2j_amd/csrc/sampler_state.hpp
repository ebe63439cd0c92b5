// What the host keeps of the device sampler between calls (the kernels are in sampler_kernels.hpp).
#pragma once

namespace l2j {

constexpr int kSampleMaxVocab = 36864;  // the most probabilities of one call that fit in LDS: 144 KB
constexpr unsigned long long kJavaRandMult = 0x5DEECE66DULL, kJavaRandMask = (1ULL << 48) - 1;

struct SamplerState {        // the reference's Sampler object, device resident
    unsigned long long rng;  // java.util.Random's 48-bit state
    int n0;                  // candidates of the current sample_topp call
    int nan;                 // bit 0: a NaN among the probabilities (J/Sampler.java:88-90 throws); bit 1: no top-p candidate; bit 2: a grid barrier of the step ran out
    int result;              // the token of the last call
    int pad;
};

}  // namespace l2j
