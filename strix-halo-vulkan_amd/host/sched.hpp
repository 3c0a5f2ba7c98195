// The language model's scheduler: several conversations interleaved on one graph
// (backend/llm_sched.go:1-59 states the policy; :201-247 the state).
//
// A request holds one of the graph's sequence slots for its whole life and its work reaches the
// device as units, one prefill chunk or one decode step at a time.  Which unit runs next is the
// whole policy:
//   1. interactive before background, strictly: while an interactive request holds a slot no
//      background unit starts, not even in the gap between two of its decode steps;
//   2. within a class, the job that has had the least device time, oldest arrival on a tie;
//   3. a background prefill runs in chunks of PreemptChunk, because a pass cannot be interrupted.
// Pending decode steps of one class share a pass, a row each; a prefill chunk ends at the job's
// checkpoint mark so that the slot's checkpoint can be taken there.
//
// With a draft head every slot has a speculator (backend/llm_sched.go:926-1015): a decode step that
// asked for it runs as a speculative round while no other conversation of its class is decoding
// (two decoding together batch as plain rows instead), a text prefill chunk primes the slot's draft,
// plain and batched steps are owed to it, and a checkpoint keeps the residual the draft resumes from.
// A round names its tokens by arg-max or, handed the request's sampler, by that sampler.
//
// The reference runs this as a goroutine that blocks on a condition variable.  Here the policy
// is a plain state machine with no thread and no clock of its own: Next() says what the device
// should run now, Finish() books what it took.  Pump() is the two around the graph call, for a
// caller that owns the one thread allowed to touch the graph; with no graph the same object is
// the policy alone, which is how it is tested without a device.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace llm {

class Graph;
class MTPHead;
class Speculator;
class Sampler;
struct Checkpoint;

enum SchedClass { kInteractive = 0, kBackground = 1 };  // backend/llm_sched.go:77-80

struct SchedOpts {
    int Batch = 2048;            // rows of the longest prefill chunk (the served -llm-batch)
    int PreemptChunk = 0;        // rows of a background prefill chunk, 0: Batch (rule 3)
    int Reserve = 1;             // slots only the interactive class may take, when there are more slots than that
    bool NoBatchDecode = false;  // every decode step in a pass of its own
    double CoalesceMs = 5;       // how long a batched step waits for the conversations still sampling
    int SpecDepth = 0;           // tokens a speculative round drafts; 0: decode by plain steps only
};

// What the device should run next: nothing, one chunk of one job, or one batched decode pass.
struct SchedPass {
    enum Kind { kNone = 0, kChunk = 1, kSteps = 2, kRound = 3 };
    int kind = kNone;
    double wait_ms = 0;  // kNone: > 0 while a batch waits for sampling peers, call again then
    // kChunk: rows [0, n) of unit's remaining ids on `slot`, whose sequence stands at `pos`
    int unit = -1, slot = -1, pos = 0, n = 0;
    bool fresh = false, restore = false, take = false, step = false;
    // kChunk with a draft head: the chunk primes the slot's draft (a text prefill chunk, fresh or on a
    // slot whose draft is caught up); tracked: the draft was caught up when the pass was handed out
    bool prime = false, tracked = false;
    // kRound: one speculative round of `unit` on `slot` from ids[0], keeping at most `room` tokens
    int room = 0;
    std::vector<int32_t> ids;
    // kSteps: one row per unit
    std::vector<int> units, slots;
};

struct SchedJobInfo {
    int cls = 0, slot = -1, reused = 0;
    bool restore = false;   // the job's first unit will restore the slot's checkpoint
    bool restored = false;  // the reused tokens came from the slot's checkpoint
    bool stepping = false;
    double served_ms = 0;
    uint64_t arrival = 0;
};

struct SchedCounts {
    int restores = 0, batches = 0, batch_rows = 0, passes = 0;  // backend/llm_sched.go:234-237
    int rounds = 0, round_tokens = 0;                           // :238-239
};

class Sched {
public:
    // g may be null: then Pump() is refused and Next()/Finish() are the policy alone over `slots` slots.
    // draft: the staged draft head, one cache slot per sequence slot; with it and SpecDepth > 0 the
    // decode steps queued by Decode() may run as speculative rounds.
    Sched(Graph *g, int slots, const SchedOpts &o, MTPHead *draft = nullptr);
    ~Sched();
    int Slots() const { return static_cast<int>(slots_.size()); }
    const SchedOpts &Opts() const { return o_; }

    // Acquire queues a request for a slot and hands out what is free (backend/llm_sched.go:265-307);
    // the job holds a slot once Job(id).slot >= 0.  mark is the prompt position at which the slot's
    // checkpoint is to be taken, 0 for nowhere.
    int Acquire(int cls, const std::vector<int32_t> &prompt, int mark, double now_ms);
    // Release gives the slot back; what it holds stays for the conversation's next turn (:414-430).
    // A job still waiting is withdrawn; its queued units fail.
    void Release(int job, double now_ms);
    SchedJobInfo Job(int job) const;

    // Run queues a whole prefill on the job's slot, fresh starting the slot's sequence over (:435);
    // Step queues one decode token (:441).  Both return a unit id.
    int Run(int job, const std::vector<int32_t> &ids, bool fresh);
    int Step(int job, int32_t id);
    // Decode is Step for a conversation that may speculate (backend/llm_sched.go:455-464): the unit
    // ends either with the tokens a round drew (Unit().toks, the last of them pending like a
    // sampled one) or, when it ran as a plain step, with that step's logits.  room: how many
    // tokens the request may still take.
    // sampler: the request's own (borrowed until the unit is done), which then names the round's
    // tokens; exact as Speculator::SetSampler has it (a seeded request).
    int Decode(int job, int32_t id, int room, Sampler *sampler = nullptr, bool exact = false, int64_t draft_seed = 1);
    // Withdraw takes a unit that is not on the device out of the queue (:483-495).
    void Withdraw(int unit);

    SchedPass Next(double now_ms);
    // Finish books a pass that Next() handed out: took_ms of device time, ok false when the
    // graph refused it.  logits: the pass's last row for a chunk, [rows][vocab] for a batch.
    void Finish(const SchedPass &p, double took_ms, bool ok, double now_ms, const std::vector<float> *logits = nullptr,
                const std::string &err = std::string(), const std::vector<int32_t> *toks = nullptr);
    // Pump runs one pass on the graph: Next(), the graph calls, Finish(), on the steady clock.
    // It returns the pass it ran; kind kNone when there was nothing to run.
    SchedPass Pump();

    struct UnitState {
        bool known = false, done = false, failed = false;
        double busy_ms = 0;
        int left = 0;  // ids not yet run
        std::string err;
        std::vector<float> logits;
        std::vector<int32_t> toks;  // a speculative round's tokens
    };
    UnitState Unit(int unit) const;
    void Forget(int unit);  // drops a finished unit's result
    SchedCounts Counts() const { return counts_; }
    // what a slot's state is for, and how long its checkpoint is (0: none)
    const std::vector<int32_t> &Held(int slot) const { return slots_.at(slot).held; }
    int CheckpointLen(int slot) const { return slots_.at(slot).ckpt_len; }
    bool Tracked(int slot) const { return slots_.at(slot).track; }  // the slot's draft covers what the slot holds (but for owed rows)
    int Waiting() const { return static_cast<int>(waiting_.size()); }
    int Pending() const { return static_cast<int>(pending_.size()); }

    // how much of prompt a held sequence saves: all of held or nothing, and the prompt must be longer (:378-383)
    static int UsablePrefix(const std::vector<int32_t> &held, const std::vector<int32_t> &prompt);

private:
    struct Slot {
        std::vector<int32_t> held;
        int job = -1;
        double used_ms = -1;
        uint64_t used_seq = 0;
        int ckpt_len = 0;
        std::vector<int32_t> ckpt_keys;
        bool track = false;         // backend/llm_sched.go:216-222
        bool ckpt_primed = false;   // the checkpoint was taken at the end of a priming chunk: ckpt_res goes with it
        std::vector<float> ckpt_res;
    };
    struct JobRec {
        int cls = 0, slot = -1, reused = 0, mark = 0;
        bool restore = false, restored = false, stepping = false;
        uint64_t arrival = 0;
        double served_ms = 0;
        std::vector<int32_t> prompt;
    };
    struct UnitRec {
        int job = -1;
        std::vector<int32_t> ids;
        size_t at = 0;  // ids[at..] are still to run
        bool fresh = false, restore = false, step = false, on_device = false;
        bool round = false, exact = false;
        int room = 0;
        Sampler *sampler = nullptr;
        int64_t draft_seed = 1;
        UnitState st;
    };
    int reuse(const Slot &sl, const std::vector<int32_t> &prompt, bool *restore) const;
    void grant();
    int best_waiter() const;
    int free_slot(int cls, const std::vector<int32_t> &prompt) const;
    bool cheaper(const Slot &a, const Slot &b) const;
    void claim(int job, int slot);
    int pick() const;
    std::vector<int> steps(int unit) const;
    double coalesce_wait(int unit, int n, double now_ms) const;
    bool speculates(int unit) const;
    void wipe(Slot &sl, int slot);
    void drop_pending(int unit);
    void fail(int unit, const std::string &why);
    double clock_ms() const;

    Graph *g_;
    SchedOpts o_;
    std::vector<Slot> slots_;
    std::vector<std::unique_ptr<Checkpoint>> ckpts_;  // the graph-side checkpoint of each slot
    std::vector<std::unique_ptr<Speculator>> specs_;  // one a slot, with a draft head
    bool spec_on_ = false;
    std::map<int, JobRec> jobs_;
    std::map<int, UnitRec> units_;
    std::vector<int> waiting_, pending_;
    uint64_t arrival_ = 0, used_seq_ = 0;
    int next_job_ = 1, next_unit_ = 1, step_rows_ = 1;
    double last_step_ms_ = -1e300;
    SchedCounts counts_;
};

}  // namespace llm
