// The C handle of a host sampler, shared by the entry points that make one and those that borrow it.
#pragma once

#include "sample.hpp"

struct shvsampler {
    llm::Sampler s;
    llm::Dist last;  // the distribution of the last propose
    bool has_last = false;
    shvsampler(float t, int k, float p, int64_t seed) : s(t, k, p, seed) {}
};
