// sample.hpp — one row of logits to one token on the host: the reference's sampler chain
// `penalties -> top_k -> top_p -> min_p -> temp -> dist` (llm/sample.go:23-356), temperature zero
// short-circuiting everything after the penalties into an argmax, and speculative sampling's
// Verify.  The reference keeps this on the host on purpose (a row is 1 MB of arithmetic against a
// token's gigabytes of weights); the greedy arg-max of the token loop itself runs on the device.
//
// Random draws come from this file's own generator: Go's math/rand stream is not reproduced, so a
// seed names a different (still deterministic) sequence than the reference's does.
#pragma once

#include <cstdint>
#include <memory>
#include <vector>

namespace llm {

// A sampler's distribution over the ids that survive its cuts, most likely first (llm/sample.go:151-167).
struct Dist {
    std::vector<int32_t> IDs;
    std::vector<float> P;
    float Of(int32_t id) const;  // zero for an id the cuts removed
};

constexpr int kPenaltyWindow = 64;  // llm/sample.go:89
constexpr int kTopKScan = 256;      // llm/sample.go:53

int32_t Argmax(const float *logits, int n);                       // ties to the lowest id (llm/sample.go:359-367)
std::vector<int32_t> TopN(const float *logits, int n, int k);     // the k highest, descending (llm/sample.go:372-384)
// the k largest logits' ids, descending, ties to the lower id, in one pass (llm/sample.go:59-84)
void TopKOf(const float *logits, int n, int k, std::vector<int32_t> *dst);

class Sampler {
public:
    Sampler(float temp, int topK, float topP, int64_t seed);
    float Temp;
    int TopK;
    float TopP;
    float MinP = 0.f;
    float RepeatPenalty = 1.f, PresencePenalty = 0.f;

    bool Greedy() const { return Temp <= 0.f; }
    // Records tokens for the penalties' window: the prompt before the first Sample, each sampled token after.
    void Accept(const int32_t *ids, int n);
    // Picks a token from one row; the row is returned as it was given (penalties are undone).
    int32_t Sample(float *logits, int n);
    // The distribution Sample draws from (penalties applied and undone).
    Dist DistOf(float *logits, int n);
    // A draft's pick: a draw and the distribution it came from; greedy proposes the arg-max and leaves q empty.
    int32_t Propose(float *logits, int n, Dist *q);
    // Sample at a row where the draft proposed `draft`, drawn from q (llm/sample.go:183-250): kept with
    // probability min(1, p/q), else drawn from max(0, p - q) renormalised.  q == nullptr is Sample.
    int32_t Verify(float *logits, int n, int32_t draft, const Dist *q);
    // The sampler a round's draft proposes with: these cuts and temperature, no penalties, its own generator.
    std::unique_ptr<Sampler> DraftSampler(int64_t seed) const;

private:
    bool penalised() const { return (RepeatPenalty != 1.f && RepeatPenalty > 0.f) || PresencePenalty != 0.f; }
    struct Saved {
        int32_t id;
        float v;
    };
    void penalise(float *logits, int n, std::vector<Saved> *saved) const;
    static void restore(float *logits, const std::vector<Saved> &saved);
    Dist dist(const float *logits, int n);
    int32_t draw(const Dist &d);
    float uniform();  // [0, 1) in steps of 2^-24, as Go's Float32 is
    std::vector<int32_t> history_;
    uint64_t rng_;
    std::vector<int32_t> topk_;
};

}  // namespace llm
