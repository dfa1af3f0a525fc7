// Continuous batching above the step function: which requests run in the next
// step and with how many tokens.
//
// As the reference's scheduler (src/serve/scheduler.rs:34-76): running requests
// come first, in the order they were admitted, each with what it still has to
// compute (one token when it decodes, the rest of its prompt otherwise), cut to
// the step's token budget; then waiting requests are admitted first-in first-out
// while budget is left; a request that cannot get its pages is skipped for the
// step, and the first waiting request that does not fit stops admission.
//
// Added to that: a cap on one request's portion; finishing at exactly max_new
// tokens without the reference's extra step (src/serve/engine.rs:214-229); and a
// decision for the case the reference spins on (engine.rs:190): when no request
// can advance because pages ran out, the request admitted last gives its pages
// back and goes to the front of the waiting queue, to be computed again from its
// prompt and what it has generated.  Its generator state stays, so its output
// does not change.
//
// One step ahead.  A caller that has started a step on the device may say so
// (launch()) and plan the next one before the first one's sampled tokens are
// back: a request whose next token is being sampled gets an entry of one token
// that names the row of the step in flight where that token will stand, and the
// device hands it over without the host.  What cannot be known yet is left to
// turn out: a request that ends on a stop token has run one token for nothing,
// its entry in the step ahead is marked dead and its sample dropped.  Nothing is
// preempted while a step is in flight; a plan that finds no pages comes back
// empty and the caller commits the step in flight first.  Which tokens run in
// which order, and each request's random draws, are the same as without.  The
// logits are the same up to what the kernels make of a step's row count: a dead
// row makes the step one row larger than the step taken in turn, and where that
// crosses a boundary between kernels (16 to 17 rows, say) the live rows are
// rounded in another order, so that in bfloat16 a greedy near-tie can fall the
// other way.
#pragma once
#include <cstdint>
#include <deque>
#include <vector>

#include "batch.h"
#include "cache_manager.h"
#include "sampler_rng.h"

namespace llmrs {

struct SamplingParams {
    float temperature = 0.0f;  // 0: greedy
    int top_k = 0;             // 0 or >= vocabulary: off
    float top_p = 1.0f;        // >= 1: off
    uint64_t seed = 42;
};

enum class Phase { Free, Waiting, Running, Finished };
enum class Finish { None = 0, Stop = 1, Length = 2 };

struct Request {
    std::vector<int32_t> tokens;  // prompt, then what was generated
    int prompt_len = 0;
    int computed = 0;             // tokens whose keys and values are in the cache
    int max_new = 0;
    std::vector<int32_t> stop;
    SamplingParams sampling;
    Xorshift64 rng;
    Phase phase = Phase::Free;
    Finish finish = Finish::None;
    int preemptions = 0;
    int pending_row = -1;         // >= 0: the step in flight samples its next token, in that row of its samples
    int generated() const { return (int)tokens.size() - prompt_len; }
};

struct PlannedEntry {
    BatchEntry entry;
    bool samples;          // the portion ends at the request's last known token
    int pending_src = -1;  // >= 0: the entry's one token is the sample in that row of the step in flight
    bool dead = false;     // its request ended after the step was started: nothing of it counts
};

class Scheduler {
public:
    Scheduler(CacheManager& cache, int token_budget, int max_chunk, int max_positions);

    // Slot of the new request; -1 when no slot is free (ask again later).
    // Throws when the request could never run: longer than the positions allow,
    // or needing more pages at once than a pool has.
    int add(const int32_t* prompt, int n_prompt, int max_new, const SamplingParams& sp,
            const int32_t* stop, int n_stop);
    // Throws what add() would throw for a request of these lengths; changes nothing.
    void check(int n_prompt, int max_new) const;
    bool idle() const { return running_.empty() && waiting_.empty(); }

    // The next step's entries; empty when idle.
    const std::vector<PlannedEntry>& plan();
    const std::vector<PlannedEntry>& planned() const { return plan_; }
    // Tokens, wanted rows (the last row of each entry that samples) and sampling
    // words (a uniform drawn from each such request's generator) of the plan.
    void plan_tokens(std::vector<int32_t>& tokens, std::vector<int32_t>& want_rows,
                     std::vector<int32_t>& sampling_words);
    // Takes the sampled token of each entry that samples, in plan order; returns
    // the slots that finished (their pages are back; the slot stays until drop()).
    // (With a step in flight: that step's.)
    std::vector<int> commit(const int32_t* sampled, int n_sampled);
    // The planned step has been started on the device: plan() may be called for the step after it.
    // One step can be in flight; commit() lands it.
    void launch();
    bool in_flight() const { return !flight_.empty(); }
    // The most tokens of one request in a step from now on (0 or less: the step's whole budget).
    void set_max_chunk(int max_chunk) { max_chunk_ = max_chunk > 0 ? max_chunk : budget_; }

    const Request& request(int slot) const { return requests_[slot]; }
    void drop(int slot);  // forget a finished request, free its slot
    void abort(int slot); // end a request wherever it stands: pages and slot go back
    int num_running() const { return (int)running_.size(); }
    int num_waiting() const { return (int)waiting_.size(); }
    int64_t preemptions() const { return preemptions_; }

private:
    int portion(const Request& r, int budget) const;
    void preempt_last();

    CacheManager& cache_;
    int budget_, max_chunk_, max_positions_;
    std::vector<Request> requests_;  // by slot
    std::vector<int> running_;       // admission order
    std::deque<int> waiting_;
    std::vector<PlannedEntry> plan_;
    std::vector<PlannedEntry> flight_;   // the step that was started and has not been committed
    int64_t preemptions_ = 0;
};

}  // namespace llmrs
