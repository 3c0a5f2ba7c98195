// Flat C entry points over llm::Sampler for ctypes callers: see shv_llm.h.
#include <algorithm>
#include <cstring>

#include "sampler_handle.hpp"
#include "shv_llm.h"

static int copy_dist(const llm::Dist &d, int32_t *ids, float *p, int max) {
    const int n = static_cast<int>(std::min<size_t>(d.IDs.size(), max < 0 ? 0 : max));
    if (ids) std::copy(d.IDs.begin(), d.IDs.begin() + n, ids);
    if (p) std::copy(d.P.begin(), d.P.begin() + n, p);
    return static_cast<int>(d.IDs.size());
}

extern "C" {

shvsampler *shvsampler_new(float temp, int top_k, float top_p, int64_t seed) { return new shvsampler(temp, top_k, top_p, seed); }
void shvsampler_free(shvsampler *h) { delete h; }
void shvsampler_set(shvsampler *h, float min_p, float repeat_penalty, float presence_penalty) {
    h->s.MinP = min_p;
    h->s.RepeatPenalty = repeat_penalty;
    h->s.PresencePenalty = presence_penalty;
}
int shvsampler_greedy(shvsampler *h) { return h->s.Greedy(); }
void shvsampler_accept(shvsampler *h, const int32_t *ids, int n) { h->s.Accept(ids, n); }
int32_t shvsampler_sample(shvsampler *h, float *logits, int n) { return h->s.Sample(logits, n); }
int shvsampler_dist(shvsampler *h, float *logits, int n, int32_t *ids, float *p, int max) { return copy_dist(h->s.DistOf(logits, n), ids, p, max); }
shvsampler *shvsampler_draft(shvsampler *h, int64_t seed) {
    if (h->s.Greedy()) return nullptr;
    shvsampler *d = new shvsampler(h->s.Temp, h->s.TopK, h->s.TopP, seed);
    d->s.MinP = h->s.MinP;
    return d;
}
int32_t shvsampler_propose(shvsampler *h, float *logits, int n) {
    const int32_t id = h->s.Propose(logits, n, &h->last);
    h->has_last = !h->s.Greedy();
    return id;
}
int shvsampler_last_dist(shvsampler *h, int32_t *ids, float *p, int max) { return h->has_last ? copy_dist(h->last, ids, p, max) : 0; }
int32_t shvsampler_verify(shvsampler *h, float *logits, int n, int32_t draft, shvsampler *proposer) {
    return h->s.Verify(logits, n, draft, proposer && proposer->has_last ? &proposer->last : nullptr);
}
void shvsampler_sample_many(shvsampler *h, float *logits, int n, int draws, int32_t *counts) {
    for (int i = 0; i < draws; i++) counts[h->s.Sample(logits, n)]++;
}
int64_t shvsampler_speculate_many(shvsampler *h, shvsampler *ds, float *pl, float *ql, int n, int draws, int32_t *counts) {
    int64_t kept = 0;
    for (int i = 0; i < draws; i++) {
        const int32_t d = shvsampler_propose(ds, ql, n);
        const int32_t g = shvsampler_verify(h, pl, n, d, ds);
        counts[g]++;
        kept += g == d;
    }
    return kept;
}
int32_t shvsampler_argmax(const float *logits, int n) { return llm::Argmax(logits, n); }
int shvsampler_top_n(const float *logits, int n, int k, int32_t *dst) {
    const std::vector<int32_t> v = llm::TopN(logits, n, k);
    std::copy(v.begin(), v.end(), dst);
    return static_cast<int>(v.size());
}
int shvsampler_top_k_of(const float *logits, int n, int k, int32_t *dst) {
    std::vector<int32_t> v;
    llm::TopKOf(logits, n, k, &v);
    std::copy(v.begin(), v.end(), dst);
    return static_cast<int>(v.size());
}

}  // extern "C"
