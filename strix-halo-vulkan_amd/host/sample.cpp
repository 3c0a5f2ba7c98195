// The sampler ladder and speculative sampling's Verify: see sample.hpp.
#include "sample.hpp"

#include <algorithm>
#include <cmath>
#include <limits>
#include <numeric>
#include <unordered_map>

namespace llm {

float Dist::Of(int32_t id) const {
    for (size_t i = 0; i < IDs.size(); i++)
        if (IDs[i] == id) return P[i];
    return 0.f;
}

int32_t Argmax(const float *logits, int n) {
    int32_t best = 0;
    float best_v = -std::numeric_limits<float>::infinity();
    for (int i = 0; i < n; i++)
        if (logits[i] > best_v) {
            best = i;
            best_v = logits[i];
        }
    return best;
}

void TopKOf(const float *logits, int n, int k, std::vector<int32_t> *dst) {
    dst->clear();
    if (k <= 0) return;
    float thr = -std::numeric_limits<float>::infinity();
    for (int i = 0; i < n; i++) {
        const float v = logits[i];
        if (static_cast<int>(dst->size()) == k && !(v > thr)) continue;
        // after every kept logit >= v: an equal logit stays behind the lower id that came first
        const auto at = std::partition_point(dst->begin(), dst->end(), [&](int32_t id) { return !(logits[id] < v); });
        const size_t j = static_cast<size_t>(at - dst->begin());
        if (static_cast<int>(dst->size()) < k) dst->push_back(0);
        else if (static_cast<int>(j) == k) continue;
        std::copy_backward(dst->begin() + j, dst->end() - 1, dst->end());
        (*dst)[j] = i;
        thr = logits[dst->back()];
    }
}

std::vector<int32_t> TopN(const float *logits, int n, int k) {
    if (n <= 0 || k <= 0) return {};
    std::vector<int32_t> idx(n);
    std::iota(idx.begin(), idx.end(), 0);
    if (k > n) k = n;
    // the k largest first, in no particular order, then ordered: a row is too wide to sort whole
    std::nth_element(idx.begin(), idx.begin() + (k > 0 ? k - 1 : 0), idx.end(), [&](int32_t a, int32_t b) { return logits[a] > logits[b]; });
    idx.resize(k);
    std::sort(idx.begin(), idx.end(), [&](int32_t a, int32_t b) { return logits[a] > logits[b]; });
    return idx;
}

Sampler::Sampler(float temp, int topK, float topP, int64_t seed) : Temp(temp), TopK(topK), TopP(topP), rng_(static_cast<uint64_t>(seed)) {}

float Sampler::uniform() {
    // splitmix64; the top 24 bits make the float
    rng_ += 0x9E3779B97F4A7C15ull;
    uint64_t z = rng_;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return static_cast<float>(z >> 40) * (1.0f / 16777216.0f);
}

void Sampler::Accept(const int32_t *ids, int n) {
    if (!penalised()) return;
    history_.insert(history_.end(), ids, ids + n);
    if (history_.size() > static_cast<size_t>(kPenaltyWindow)) history_.erase(history_.begin(), history_.end() - kPenaltyWindow);
}

// llm/sample.go:119-147: a token in the window has a positive logit divided by RepeatPenalty (a
// negative one multiplied), then PresencePenalty subtracted; once per id.
void Sampler::penalise(float *logits, int n, std::vector<Saved> *saved) const {
    saved->clear();
    if (!penalised() || history_.empty()) return;
    for (int32_t id : history_) {
        if (id < 0 || id >= n) continue;
        if (std::any_of(saved->begin(), saved->end(), [&](const Saved &s) { return s.id == id; })) continue;
        float v = logits[id];
        saved->push_back({id, v});
        if (RepeatPenalty > 0.f && RepeatPenalty != 1.f) v = v > 0.f ? v / RepeatPenalty : v * RepeatPenalty;
        logits[id] = v - PresencePenalty;
    }
}

void Sampler::restore(float *logits, const std::vector<Saved> &saved) {
    for (const Saved &s : saved) logits[s.id] = s.v;
}

int32_t Sampler::Sample(float *logits, int n) {
    if (n <= 0) return -1;  // no row, no token
    std::vector<Saved> saved;
    penalise(logits, n, &saved);
    const int32_t id = Greedy() ? Argmax(logits, n) : draw(dist(logits, n));
    restore(logits, saved);
    return id;
}

Dist Sampler::DistOf(float *logits, int n) {
    if (n <= 0) return Dist{};
    std::vector<Saved> saved;
    penalise(logits, n, &saved);
    Dist d = dist(logits, n);
    restore(logits, saved);
    return d;
}

int32_t Sampler::Propose(float *logits, int n, Dist *q) {
    if (n <= 0) {
        if (q) *q = Dist{};
        return -1;
    }
    if (Greedy()) {
        if (q) *q = Dist{};
        return Argmax(logits, n);
    }
    Dist d = dist(logits, n);
    const int32_t id = draw(d);
    if (q) *q = std::move(d);
    return id;
}

int32_t Sampler::Verify(float *logits, int n, int32_t draft, const Dist *q) {
    if (n <= 0) return -1;
    if (!q || Greedy()) return Sample(logits, n);
    std::vector<Saved> saved;
    penalise(logits, n, &saved);
    Dist p = dist(logits, n);
    restore(logits, saved);
    const float pd = p.Of(draft), qd = q->Of(draft);
    if (qd <= 0.f) return draw(p);  // not a draw from q: no proposal to weigh
    if (uniform() * qd < pd) return draft;
    std::unordered_map<int32_t, float> qmap;
    const bool mapped = q->IDs.size() > 64;  // no top-k cut: a map, or the residual is |p| x |q|
    if (mapped)
        for (size_t i = 0; i < q->IDs.size(); i++) qmap[q->IDs[i]] = q->P[i];
    float sum = 0.f;
    for (size_t i = 0; i < p.IDs.size(); i++) {
        float qv;
        if (mapped) {
            auto it = qmap.find(p.IDs[i]);
            qv = it == qmap.end() ? 0.f : it->second;
        } else {
            qv = q->Of(p.IDs[i]);
        }
        float r = p.P[i] - qv;
        if (r < 0.f) r = 0.f;
        p.P[i] = r;
        sum += r;
    }
    if (sum <= 0.f) {
        // p <= q everywhere and yet rejected: rounding.  The most likely id that is not the draft.
        for (int32_t id : p.IDs)
            if (id != draft) return id;
        return draft;
    }
    const float r = uniform() * sum;
    float acc = 0.f;
    int32_t last = -1;
    for (size_t i = 0; i < p.P.size(); i++) {
        if (p.P[i] <= 0.f) continue;
        acc += p.P[i];
        last = p.IDs[i];
        if (r < acc) return last;
    }
    return last;
}

int32_t Sampler::draw(const Dist &d) {
    const float r = uniform();
    float acc = 0.f;
    for (size_t i = 0; i < d.P.size(); i++) {
        acc += d.P[i];
        if (r < acc) return d.IDs[i];
    }
    return d.IDs.back();
}

// The distribution after the cuts and the temperature (llm/sample.go:266-343); penalties are the caller's.
Dist Sampler::dist(const float *logits, int n) {
    int k = TopK;
    if (k <= 0 || k > n) k = n;
    std::vector<int32_t> idx;
    if (k <= kTopKScan) {
        TopKOf(logits, n, k, &topk_);
        idx = topk_;
    } else {
        idx = TopN(logits, n, k);
    }
    // softmax over the survivors, at temperature (exp in double, as the reference forms it)
    const float max_l = logits[idx[0]];
    std::vector<float> probs(idx.size());
    float sum = 0.f;
    for (size_t i = 0; i < idx.size(); i++) {
        const float p = static_cast<float>(std::exp(static_cast<double>((logits[idx[i]] - max_l) / Temp)));
        probs[i] = p;
        sum += p;
    }
    for (float &p : probs) p /= sum;
    auto renormalise = [&](size_t keep) {
        probs.resize(keep);
        idx.resize(keep);
        float re = 0.f;
        for (float p : probs) re += p;
        for (float &p : probs) p /= re;
    };
    if (TopP > 0.f && TopP < 1.f) {
        float acc = 0.f;
        size_t keep = probs.size();
        for (size_t i = 0; i < probs.size(); i++) {
            acc += probs[i];
            if (acc >= TopP) {
                keep = i + 1;
                break;
            }
        }
        renormalise(keep);
    }
    if (MinP > 0.f && MinP < 1.f) {
        // sorted descending, so the survivors are a prefix
        const float cut = MinP * probs[0];
        size_t keep = 1;
        while (keep < probs.size() && probs[keep] >= cut) keep++;
        renormalise(keep);
    }
    return Dist{std::move(idx), std::move(probs)};
}

std::unique_ptr<Sampler> Sampler::DraftSampler(int64_t seed) const {
    if (Greedy()) return nullptr;
    auto d = std::make_unique<Sampler>(Temp, TopK, TopP, seed);
    d->MinP = MinP;
    return d;
}

}  // namespace llm
