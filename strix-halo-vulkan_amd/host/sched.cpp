// The scheduler's policy and its pump: see sched.hpp.
#include "sched.hpp"

#include <algorithm>
#include <chrono>

#include "llm.hpp"

namespace llm {

static int common_prefix(const std::vector<int32_t> &a, const std::vector<int32_t> &b) {
    const size_t n = std::min(a.size(), b.size());
    size_t i = 0;
    while (i < n && a[i] == b[i]) i++;
    return static_cast<int>(i);
}

int Sched::UsablePrefix(const std::vector<int32_t> &held, const std::vector<int32_t> &prompt) {
    // A DeltaNet state has no inverse, so the held sequence counts in full or not at all, and the
    // prompt must be longer because a finished pass's logits are not kept (backend/llm_sched.go:374-383).
    const int n = common_prefix(held, prompt);
    if (n > 0 && n == static_cast<int>(held.size()) && n < static_cast<int>(prompt.size())) return n;
    return 0;
}

Sched::Sched(Graph *g, int slots, const SchedOpts &o, MTPHead *draft) : g_(g), o_(o) {
    if (g) slots = g->Slots();
    if (slots < 1) throw Error("llm: a scheduler needs at least one slot");
    if (o_.Batch < 1) throw Error("llm: scheduler batch " + std::to_string(o_.Batch));
    if (g && o_.Batch > g->MaxRows()) o_.Batch = g->MaxRows();
    if (o_.PreemptChunk < 0 || o_.Reserve < 0) throw Error("llm: scheduler: negative preempt chunk or reserve");
    slots_.resize(slots);
    ckpts_.resize(slots);
    // a batched decode pass carries as many rows as the graph's head was staged for
    step_rows_ = g ? g->StepRows() : slots;
    if (step_rows_ < 1) throw Error("llm: the scheduler needs a graph staged with its head");
    if (o_.SpecDepth < 0) throw Error("llm: scheduler: negative draft depth");
    if (o_.SpecDepth > 0 && g) {
        if (!draft) throw Error("llm: speculative rounds need the draft head staged");
        if (g->DeltaNet().Planes() < o_.SpecDepth + 2)
            throw Error("llm: rounds of " + std::to_string(o_.SpecDepth + 1) + " rows need a graph staged for them (GraphOpts.Speculative, SpecRows)");
        for (int i = 0; i < slots; i++) specs_.push_back(std::make_unique<Speculator>(*g, *draft, o_.SpecDepth, i));
    }
    // without a graph the policy alone says when a round would run
    spec_on_ = o_.SpecDepth > 0;
}

Sched::~Sched() = default;

double Sched::clock_ms() const {
    using namespace std::chrono;
    return duration<double, std::milli>(steady_clock::now().time_since_epoch()).count();
}

// reuse: how much of a prompt the slot saves, and whether by restoring its checkpoint rather than
// continuing what it holds (backend/llm_sched.go:127-138).
int Sched::reuse(const Slot &sl, const std::vector<int32_t> &prompt, bool *restore) const {
    const int n = UsablePrefix(sl.held, prompt);
    *restore = false;
    if (sl.ckpt_len > 0) {
        const int b = sl.ckpt_len;
        if (b > n && b < static_cast<int>(prompt.size()) && common_prefix(sl.held, sl.ckpt_keys) == b &&
            common_prefix(prompt, sl.ckpt_keys) == b) {
            *restore = true;
            return b;
        }
    }
    return n;
}

int Sched::Acquire(int cls, const std::vector<int32_t> &prompt, int mark, double now_ms) {
    (void)now_ms;
    if (cls != kInteractive && cls != kBackground) throw Error("llm: scheduler class " + std::to_string(cls));
    if (mark < 0 || mark > static_cast<int>(prompt.size())) throw Error("llm: checkpoint mark " + std::to_string(mark) + " outside the prompt");
    const int id = next_job_++;
    JobRec &j = jobs_[id];
    j.cls = cls;
    j.arrival = ++arrival_;
    j.prompt = prompt;
    j.mark = mark;
    waiting_.push_back(id);
    grant();
    return id;
}

// grant hands free slots to waiting jobs, best first; it stops at the first waiter that cannot
// be served, so a later arrival never overtakes it (backend/llm_sched.go:294-307).
void Sched::grant() {
    for (;;) {
        const int w = best_waiter();
        if (w < 0) return;
        const JobRec &j = jobs_.at(w);
        const int slot = free_slot(j.cls, j.prompt);
        if (slot < 0) return;
        claim(w, slot);
    }
}

int Sched::best_waiter() const {
    int best = -1;
    for (int w : waiting_) {
        if (best < 0) {
            best = w;
            continue;
        }
        const JobRec &a = jobs_.at(w), &b = jobs_.at(best);
        if (a.cls < b.cls || (a.cls == b.cls && a.arrival < b.arrival)) best = w;
    }
    return best;
}

// free_slot: the free slot that saves the most of the prompt, else the cheapest to overwrite; -1
// when the class may take none (backend/llm_sched.go:321-353).
int Sched::free_slot(int cls, const std::vector<int32_t> &prompt) const {
    int free = 0, bg_busy = 0;
    const int n = static_cast<int>(slots_.size());
    for (const Slot &sl : slots_) {
        if (sl.job < 0)
            free++;
        else if (jobs_.at(sl.job).cls == kBackground)
            bg_busy++;
    }
    if (free == 0) return -1;
    if (cls == kBackground && n > o_.Reserve && bg_busy >= n - o_.Reserve) return -1;
    int best = -1, best_reuse = -1;
    for (int i = 0; i < n; i++) {
        const Slot &sl = slots_[i];
        if (sl.job >= 0) continue;
        bool restore;
        const int r = reuse(sl, prompt, &restore);
        if (best < 0 || r > best_reuse || (r == best_reuse && cheaper(sl, slots_[best]))) best = i, best_reuse = r;
    }
    return best;
}

// cheaper: the better slot to overwrite when neither saves anything: less checkpointed first, so
// that background arrivals do not take a voice command's system prompt by age alone, then the
// least recently used (backend/llm_sched.go:355-365).
bool Sched::cheaper(const Slot &a, const Slot &b) const {
    if (a.ckpt_len != b.ckpt_len) return a.ckpt_len < b.ckpt_len;
    if (a.used_ms != b.used_ms) return a.used_ms < b.used_ms;
    return a.used_seq < b.used_seq;
}

void Sched::claim(int job, int slot) {
    waiting_.erase(std::find(waiting_.begin(), waiting_.end(), job));
    JobRec &j = jobs_.at(job);
    j.slot = slot;
    j.reused = reuse(slots_[slot], j.prompt, &j.restore);
    j.restored = j.restore;
    // A newcomer starts level with the least-served job of its class rather than at zero, or it
    // would hold the device until it had caught up (backend/llm_sched.go:389-396).
    bool first = true;
    for (const Slot &sl : slots_) {
        if (sl.job < 0) continue;
        const JobRec &o = jobs_.at(sl.job);
        if (o.cls == j.cls && (first || o.served_ms < j.served_ms)) j.served_ms = o.served_ms, first = false;
    }
    slots_[slot].job = job;
}

void Sched::Release(int job, double now_ms) {
    auto it = jobs_.find(job);
    if (it == jobs_.end()) return;
    for (const auto &u : units_)
        if (u.second.job == job && u.second.on_device) throw Error("llm: a job with a unit on the device cannot be released");
    std::vector<int> mine;
    for (int u : pending_)
        if (units_.at(u).job == job) mine.push_back(u);
    for (int u : mine) fail(u, "the request was released");
    JobRec &j = it->second;
    if (j.slot >= 0 && slots_[j.slot].job == job) {
        Slot &sl = slots_[j.slot];
        sl.job = -1;
        sl.used_ms = now_ms;
        sl.used_seq = ++used_seq_;
    } else {
        auto w = std::find(waiting_.begin(), waiting_.end(), job);
        if (w != waiting_.end()) waiting_.erase(w);
    }
    jobs_.erase(it);
    grant();
}

SchedJobInfo Sched::Job(int job) const {
    const JobRec &j = jobs_.at(job);
    SchedJobInfo o;
    o.cls = j.cls, o.slot = j.slot, o.reused = j.reused, o.restore = j.restore, o.restored = j.restored, o.stepping = j.stepping;
    o.served_ms = j.served_ms, o.arrival = j.arrival;
    return o;
}

int Sched::Run(int job, const std::vector<int32_t> &ids, bool fresh) {
    JobRec &j = jobs_.at(job);
    if (j.slot < 0) throw Error("llm: the job holds no slot yet");
    if (ids.empty()) throw Error("llm: an empty unit");
    const int id = next_unit_++;
    UnitRec &u = units_[id];
    u.job = job, u.ids = ids, u.fresh = fresh;
    u.restore = j.restore, j.restore = false;  // the job's first unit undoes the detour (backend/llm_sched.go:472)
    u.st.known = true, u.st.left = static_cast<int>(ids.size());
    pending_.push_back(id);
    return id;
}

int Sched::Step(int job, int32_t tok) {
    JobRec &j = jobs_.at(job);
    if (j.slot < 0) throw Error("llm: the job holds no slot yet");
    const int id = next_unit_++;
    UnitRec &u = units_[id];
    u.job = job, u.ids.assign(1, tok), u.step = true;
    u.restore = j.restore, j.restore = false;
    j.stepping = true;  // from here a moment with nothing queued is a moment it is sampling (:161-164)
    u.st.known = true, u.st.left = 1;
    pending_.push_back(id);
    return id;
}

int Sched::Decode(int job, int32_t tok, int room, Sampler *sampler, bool exact, int64_t draft_seed) {
    const int id = Step(job, tok);
    UnitRec &u = units_.at(id);
    u.round = spec_on_;
    u.room = room;
    u.sampler = sampler, u.exact = exact, u.draft_seed = draft_seed;
    return id;
}

// speculates: whether a picked decode unit runs as a speculative round: it asked to, its slot's
// draft is caught up, the round's rows fit the cache and the request's budget, and no other
// conversation of its class is decoding (backend/llm_sched.go:936-953).
bool Sched::speculates(int unit) const {
    const UnitRec &u = units_.at(unit);
    if (!u.round || u.room < 2 || !spec_on_) return false;
    const JobRec &j = jobs_.at(u.job);
    const Slot &sl = slots_[j.slot];
    if (!sl.track) return false;
    if (g_ && static_cast<int>(sl.held.size()) + o_.SpecDepth + 1 > g_->NKV()) return false;
    for (const Slot &o : slots_)
        if (o.job >= 0 && o.job != u.job && jobs_.at(o.job).cls == j.cls && jobs_.at(o.job).stepping) return false;
    return true;
}

void Sched::wipe(Slot &sl, int slot) {
    sl.held.clear(), sl.ckpt_len = 0, sl.ckpt_keys.clear(), ckpts_[slot].reset();
    sl.track = false, sl.ckpt_primed = false, sl.ckpt_res.clear();
}

void Sched::drop_pending(int unit) {
    auto it = std::find(pending_.begin(), pending_.end(), unit);
    if (it != pending_.end()) pending_.erase(it);
}

void Sched::fail(int unit, const std::string &why) {
    UnitRec &u = units_.at(unit);
    drop_pending(unit);
    u.st.done = true, u.st.failed = true, u.st.err = why;
}

void Sched::Withdraw(int unit) {
    auto it = units_.find(unit);
    if (it == units_.end() || it->second.st.done) return;
    if (it->second.on_device) throw Error("llm: the unit is on the device");
    fail(unit, "withdrawn");
}

Sched::UnitState Sched::Unit(int unit) const {
    auto it = units_.find(unit);
    if (it == units_.end()) return UnitState();
    return it->second.st;
}

void Sched::Forget(int unit) {
    auto it = units_.find(unit);
    if (it != units_.end() && it->second.st.done) units_.erase(it);
}

// pick is the policy: the next unit to run, or -1 to wait (backend/llm_sched.go:873-898).
int Sched::pick() const {
    bool interactive = false;
    for (const Slot &sl : slots_)
        if (sl.job >= 0 && jobs_.at(sl.job).cls == kInteractive) interactive = true;
    int best = -1;
    for (int id : pending_) {
        const JobRec &j = jobs_.at(units_.at(id).job);
        if (interactive && j.cls == kBackground) continue;
        if (best < 0) {
            best = id;
            continue;
        }
        const JobRec &b = jobs_.at(units_.at(best).job);
        if (j.served_ms < b.served_ms || (j.served_ms == b.served_ms && j.arrival < b.arrival)) best = id;
    }
    // With nothing of theirs queued the interactive slot-holders still keep the device: only
    // when every one of them is gone does background work run (rule 1).
    return best;
}

// steps: the batch a picked decode step runs in, it and every other pending decode step of its
// class (backend/llm_sched.go:757-770).  A job has at most one step queued, so that is a row a slot.
std::vector<int> Sched::steps(int unit) const {
    std::vector<int> b{unit};
    if (o_.NoBatchDecode) return b;
    const int cls = jobs_.at(units_.at(unit).job).cls;
    std::vector<bool> taken(slots_.size(), false);
    taken[jobs_.at(units_.at(unit).job).slot] = true;
    for (int p : pending_) {
        const UnitRec &u = units_.at(p);
        if (p == unit || !u.step) continue;
        const JobRec &j = jobs_.at(u.job);
        if (j.cls != cls || taken[j.slot]) continue;
        if (static_cast<int>(b.size()) == step_rows_) break;
        taken[j.slot] = true;
        b.push_back(p);
    }
    return b;
}

// coalesce_wait: how much longer a batch of n steps should wait for the conversations of its
// class that are decoding but sampling right now, measured from the end of the last step
// (backend/llm_sched.go:772-789).
double Sched::coalesce_wait(int unit, int n, double now_ms) const {
    if (o_.NoBatchDecode) return 0;
    const int cls = jobs_.at(units_.at(unit).job).cls;
    int peers = 0;
    for (const Slot &sl : slots_)
        if (sl.job >= 0 && jobs_.at(sl.job).cls == cls && jobs_.at(sl.job).stepping) peers++;
    if (n >= peers) return 0;
    return last_step_ms_ + o_.CoalesceMs - now_ms;
}

SchedPass Sched::Next(double now_ms) {
    SchedPass p;
    const int id = pick();
    if (id < 0) return p;
    UnitRec &u = units_.at(id);
    const JobRec &j = jobs_.at(u.job);
    if (u.step && speculates(id)) {
        p.kind = SchedPass::kRound;
        p.unit = id, p.slot = j.slot, p.pos = static_cast<int>(slots_[j.slot].held.size()), p.n = 1, p.step = true;
        p.ids.assign(1, u.ids[u.at]);
        p.room = u.room;
        u.on_device = true;
        return p;
    }
    if (u.step) {
        const std::vector<int> b = steps(id);
        const double wait = coalesce_wait(id, static_cast<int>(b.size()), now_ms);
        if (wait > 0) {
            p.wait_ms = wait;
            return p;
        }
        if (b.size() > 1) {
            p.kind = SchedPass::kSteps;
            p.units = b;
            for (int x : b) {
                UnitRec &r = units_.at(x);
                r.on_device = true;
                p.slots.push_back(jobs_.at(r.job).slot);
                p.ids.push_back(r.ids[r.at]);
            }
            counts_.batches++;
            counts_.batch_rows += static_cast<int>(b.size());
            return p;
        }
    }
    // one chunk of one unit (backend/llm_sched.go:557-607)
    const int left = static_cast<int>(u.ids.size() - u.at);
    int n = std::min(left, o_.Batch);
    if (j.cls == kBackground && o_.PreemptChunk > 0 && left > 1) n = std::min(n, o_.PreemptChunk);
    const Slot &sl = slots_[j.slot];
    int pos = static_cast<int>(sl.held.size());
    if (u.fresh)
        pos = 0;
    else if (u.restore)
        pos = sl.ckpt_len;
    // the chunk that reaches the checkpoint's boundary ends there
    if (j.mark > pos && j.mark < pos + n) n = j.mark - pos;
    p.kind = SchedPass::kChunk;
    p.unit = id, p.slot = j.slot, p.pos = pos, p.n = n;
    p.fresh = u.fresh, p.restore = u.restore && !u.fresh, p.step = u.step;
    p.take = j.mark > 0 && pos + n == j.mark;
    // the draft's cells below a restored checkpoint are still its tokens' if the draft covered what
    // the slot held and the checkpoint kept the residual to resume from (backend/llm_sched.go:625-637)
    p.tracked = sl.track && (!p.restore || sl.ckpt_primed);
    p.prime = spec_on_ && !u.step && (p.fresh || p.tracked);
    p.ids.assign(u.ids.begin() + u.at, u.ids.begin() + u.at + n);
    u.on_device = true;
    return p;
}

void Sched::Finish(const SchedPass &p, double took_ms, bool ok, double now_ms, const std::vector<float> *logits, const std::string &err,
                   const std::vector<int32_t> *toks) {
    if (p.kind == SchedPass::kNone) return;
    counts_.passes++;
    if (p.kind == SchedPass::kRound) {
        // the rows the round kept: its input and every token it drew but the last, which is pending
        // like a sampled token (backend/llm_sched.go:994-1003)
        UnitRec &u = units_.at(p.unit);
        JobRec &j = jobs_.at(u.job);
        Slot &sl = slots_[p.slot];
        u.on_device = false;
        if (ok && (!toks || toks->empty())) throw Error("llm: a finished round names its tokens");
        if (!ok) {
            wipe(sl, p.slot);
        } else {
            sl.held.push_back(p.ids[0]);
            sl.held.insert(sl.held.end(), toks->begin(), toks->end() - 1);
            counts_.rounds++;
            counts_.round_tokens += static_cast<int>(toks->size());
            u.st.toks = *toks;
        }
        last_step_ms_ = now_ms;
        u.st.busy_ms += took_ms;
        j.served_ms += took_ms;
        u.at = u.ids.size(), u.st.left = 0;
        u.st.done = true, u.st.failed = !ok, u.st.err = ok ? std::string() : err;
        drop_pending(p.unit);
        return;
    }
    if (p.kind == SchedPass::kSteps) {
        // each row had the whole pass's latency and a share of its cost (backend/llm_sched.go:845-870)
        const size_t rows = p.units.size();
        const size_t vocab = ok && logits ? logits->size() / rows : 0;
        for (size_t i = 0; i < rows; i++) {
            UnitRec &u = units_.at(p.units[i]);
            JobRec &j = jobs_.at(u.job);
            Slot &sl = slots_[j.slot];
            if (!ok) {
                // which rows' states moved is not something this can say
                wipe(sl, j.slot);
            } else {
                sl.held.push_back(u.ids[u.at]);
                if (vocab) u.st.logits.assign(logits->begin() + i * vocab, logits->begin() + (i + 1) * vocab);
            }
            u.st.busy_ms += took_ms;
            j.served_ms += took_ms / static_cast<double>(rows);
            u.at = u.ids.size(), u.st.left = 0, u.on_device = false;
            u.st.done = true, u.st.failed = !ok, u.st.err = ok ? std::string() : err;
            drop_pending(p.units[i]);
        }
        last_step_ms_ = now_ms;
        return;
    }
    UnitRec &u = units_.at(p.unit);
    JobRec &j = jobs_.at(u.job);
    Slot &sl = slots_[p.slot];
    u.on_device = false;
    if (!ok) {
        // whatever the slot held is no longer something this can describe (backend/llm_sched.go:714-717)
        wipe(sl, p.slot);
    } else if (p.fresh) {
        sl.held = p.ids;
    } else if (p.restore) {
        // pos, not the checkpoint's length: a chunk that ends at the mark re-takes the checkpoint
        sl.held.resize(p.pos);
        sl.held.insert(sl.held.end(), p.ids.begin(), p.ids.end());
        counts_.restores++;
    } else {
        sl.held.insert(sl.held.end(), p.ids.begin(), p.ids.end());
    }
    if (ok) {
        // a priming chunk leaves the draft caught up; a plain step is owed to a draft that was; any
        // other pass leaves the draft behind for good (backend/llm_sched.go:664-690,707-709)
        sl.track = p.prime || (p.step && p.tracked);
    }
    if (ok && p.take) {
        sl.ckpt_len = static_cast<int>(sl.held.size());
        sl.ckpt_keys = sl.held;
        sl.ckpt_primed = p.prime;
        if (!p.prime) sl.ckpt_res.clear();
    }
    if (p.step) last_step_ms_ = now_ms;
    u.st.busy_ms += took_ms;
    j.served_ms += took_ms;
    u.at += p.n, u.fresh = false, u.restore = false;
    u.st.left = static_cast<int>(u.ids.size() - u.at);
    if (!ok || u.at == u.ids.size()) {
        if (ok && logits) u.st.logits = *logits;
        u.st.done = true, u.st.failed = !ok, u.st.err = ok ? std::string() : err;
        drop_pending(p.unit);
    }
}

SchedPass Sched::Pump() {
    if (!g_) throw Error("llm: this scheduler has no graph to run passes on");
    SchedPass p = Next(clock_ms());
    if (p.kind == SchedPass::kNone) return p;
    std::vector<float> logits;
    std::vector<int32_t> toks;
    std::string err;
    bool ok = true;
    const size_t E = g_->GetModel().config().NEmbd;
    const double t0 = clock_ms();
    try {
        if (p.kind == SchedPass::kRound) {
            // backend/llm_sched.go:957-992
            Speculator &sp = *specs_.at(p.slot);
            g_->UseSlot(p.slot);
            if (!g_->Speculating()) g_->Speculate(true);
            g_->SpeculateFirst(true);
            try {
                const UnitRec &u = units_.at(p.unit);
                sp.SetSampler(u.sampler, u.exact, u.draft_seed);
                toks = sp.RoundFrom(p.ids[0], {}, p.room);
            } catch (const std::exception &) {
                // a pass may be left in flight, which would refuse every later UseSlot; the slot's
                // sequence is lost either way
                try {
                    if (g_->InFlight()) g_->Commit();
                    g_->Reset();
                } catch (const std::exception &) {
                }
                throw;
            }
        } else if (p.kind == SchedPass::kSteps) {
            if (g_->Speculating()) g_->Speculate(false);
            g_->DecodeRows(p.slots, p.ids, &logits);
            // each row a slot's draft did not see: owed to it (backend/llm_sched.go:834-840)
            for (size_t i = 0; i < p.slots.size(); i++)
                if (!specs_.empty() && slots_[p.slots[i]].track) specs_[p.slots[i]]->Owe(p.ids[i], g_->ResPort() + i * E);
        } else {
            Speculator *sp = specs_.empty() ? nullptr : specs_[p.slot].get();
            if (g_->Speculating()) g_->Speculate(false);
            g_->UseSlot(p.slot);
            if (p.restore) {
                if (!ckpts_[p.slot]) throw Error("llm: slot " + std::to_string(p.slot) + " has no checkpoint to restore");
                g_->Restore(*ckpts_[p.slot]);
                if (sp && p.tracked) sp->Rewind(ckpts_[p.slot]->past, slots_[p.slot].ckpt_res);
            }
            // only the unit's last chunk's logits are anyone's: the ones between are not read back
            const UnitRec &u = units_.at(p.unit);
            const bool last = u.at + p.n == u.ids.size();
            const bool prime = sp && p.prime;
            if (prime && !p.fresh) sp->Settle();  // a continuation primes from where the draft is, once its owed rows are written
            if (p.fresh) g_->Reset();
            if (prime) {
                const float *res = g_->ExtendResidual(p.ids, last ? &logits : nullptr);
                sp->Prime(p.ids, p.pos, res);
            } else {
                g_->Extend(p.ids, last ? &logits : nullptr, nullptr);
                // a plain step the draft did not see: owed to it
                if (sp && p.step && p.tracked) sp->Owe(p.ids[0], g_->ResPort());
            }
            if (p.take && prime) slots_[p.slot].ckpt_res = sp->Residual();
            if (p.take) {
                // a checkpoint that cannot be taken costs the next request its prefix, not this one its answer
                try {
                    if (!ckpts_[p.slot]) ckpts_[p.slot] = std::make_unique<Checkpoint>();
                    g_->Checkpoint(*ckpts_[p.slot]);
                } catch (const std::exception &) {
                    ckpts_[p.slot].reset();
                    slots_[p.slot].ckpt_len = 0, slots_[p.slot].ckpt_keys.clear();
                    slots_[p.slot].ckpt_primed = false, slots_[p.slot].ckpt_res.clear();
                    p.take = false;
                }
            }
        }
    } catch (const std::exception &e) {
        ok = false;
        err = e.what();
    }
    const double t1 = clock_ms();
    Finish(p, t1 - t0, ok, t1, &logits, err, &toks);
    return p;
}

}  // namespace llm
