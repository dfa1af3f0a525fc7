#include "scheduler.h"

#include <algorithm>
#include <cstring>
#include <stdexcept>
#include <string>

namespace llmrs {

Scheduler::Scheduler(CacheManager& cache, int token_budget, int max_chunk, int max_positions)
    : cache_(cache), budget_(token_budget), max_chunk_(max_chunk > 0 ? max_chunk : token_budget),
      max_positions_(max_positions), requests_(cache.max_requests()) {
    if (token_budget <= 0) throw std::invalid_argument("token budget must be positive");
}

void Scheduler::check(int n_prompt, int max_new) const {
    if (n_prompt <= 0) throw std::invalid_argument("a request needs at least one prompt token");
    if (max_new <= 0) throw std::invalid_argument("max_new_tokens must be positive");
    long long total = (long long)n_prompt + max_new;
    if (total > max_positions_)
        throw std::invalid_argument("request needs " + std::to_string(total) + " positions, the model has " +
                                    std::to_string(max_positions_));
    // The most pages a request alone in the pool has to hold at once.  If even
    // that exceeds a pool, no schedule can ever finish it.  Without a window: all
    // it computes (its last token is sampled, never run).  With a window w: the
    // keys a portion's first query still sees and the portion itself, w + n - 1
    // positions in a row for a portion of n; where a portion starts depends on
    // what else shared the budget, so the bound is for the worst start, where
    // that many positions touch one page more than they fill.
    int computed = (int)total - 1;
    for (int g = 0; g < cache_.num_groups(); ++g) {
        int ps = cache_.group(g).page_size, w = cache_.group(g).window;
        int worst = cache_.pages_needed(g, 0, computed);
        if (w > 0) {
            int n = std::min({max_chunk_, budget_, computed});
            long long span = std::min<long long>((long long)w + n - 1, computed);
            worst = std::min<long long>(worst, span <= 1 ? 1 : (span - 1 + ps - 1) / ps + 1);
        }
        if (worst > cache_.pages_total(g))
            throw std::invalid_argument("request needs " + std::to_string(worst) + " pages of cache group " +
                                        std::to_string(g) + ", the pool has " + std::to_string(cache_.pages_total(g)));
    }
}

int Scheduler::add(const int32_t* prompt, int n_prompt, int max_new, const SamplingParams& sp,
                   const int32_t* stop, int n_stop) {
    check(n_prompt, max_new);
    int slot = cache_.acquire_slot();
    if (slot < 0) return -1;
    Request& r = requests_[slot];
    r = Request();
    r.tokens.assign(prompt, prompt + n_prompt);
    r.prompt_len = n_prompt;
    r.max_new = max_new;
    r.stop.assign(stop, stop + n_stop);
    r.sampling = sp;
    r.rng = Xorshift64(sp.seed);
    r.phase = Phase::Waiting;
    waiting_.push_back(slot);
    return slot;
}

int Scheduler::portion(const Request& r, int budget) const {
    int needed = (int)r.tokens.size() - r.computed;
    return std::min({needed, budget, max_chunk_});
}

void Scheduler::preempt_last() {
    int slot = running_.back();
    running_.pop_back();
    Request& r = requests_[slot];
    cache_.release_pages(slot);
    r.computed = 0;
    r.phase = Phase::Waiting;
    ++r.preemptions;
    ++preemptions_;
    waiting_.push_front(slot);
}

const std::vector<PlannedEntry>& Scheduler::plan() {
    const bool ahead = in_flight();
    for (;;) {
        plan_.clear();
        int budget = budget_;
        bool starved = false;
        // 1. running requests, in admission order (scheduler.rs:42-54)
        for (int slot : running_) {
            if (budget == 0) break;
            Request& r = requests_[slot];
            int n = portion(r, budget), src = -1;
            if (r.pending_row >= 0) {
                // its next token is being sampled: one token, unless that one is its last
                if (r.generated() + 1 >= r.max_new) continue;
                n = 1;
                src = r.pending_row;
            }
            if (n <= 0) continue;
            if (!cache_.ensure(slot, r.computed, n)) {
                starved = true;
                continue;  // no pages now; it tries again in the next step
            }
            plan_.push_back({{slot, r.computed, n}, src >= 0 || r.computed + n == (int)r.tokens.size(), src});
            budget -= n;
        }
        // 2. waiting requests, first in first out (scheduler.rs:56-73)
        while (budget > 0 && !waiting_.empty()) {
            int slot = waiting_.front();
            Request& r = requests_[slot];
            int n = portion(r, budget);
            if (!cache_.ensure(slot, r.computed, n)) {
                starved = true;
                break;  // head of the line waits, and so do those behind it
            }
            waiting_.pop_front();
            r.phase = Phase::Running;
            running_.push_back(slot);
            plan_.push_back({{slot, r.computed, n}, r.computed + n == (int)r.tokens.size()});
            budget -= n;
        }
        if (!plan_.empty() || !starved || ahead) return plan_;   // (ahead of a step in flight nobody is preempted)
        // Nothing can advance and pages are the reason.  With nobody running, the
        // head of the queue found an empty pool too small: add() rules that out.
        if (running_.empty())
            throw std::logic_error("a waiting request does not fit an empty cache pool");
        preempt_last();
    }
}

void Scheduler::plan_tokens(std::vector<int32_t>& tokens, std::vector<int32_t>& want_rows,
                            std::vector<int32_t>& sampling_words) {
    tokens.clear();
    want_rows.clear();
    sampling_words.clear();
    for (const auto& p : plan_) {
        Request& r = requests_[p.entry.slot];
        if (p.pending_src >= 0) tokens.push_back(0);     // the device puts the step in flight's sample here
        else tokens.insert(tokens.end(), r.tokens.begin() + p.entry.start, r.tokens.begin() + p.entry.start + p.entry.count);
        if (!p.samples) continue;
        want_rows.push_back((int32_t)tokens.size() - 1);
        float u = r.sampling.temperature > 0.0f ? r.rng.next_f32() : 0.0f;
        int32_t w[4];
        std::memcpy(&w[0], &u, 4);
        std::memcpy(&w[1], &r.sampling.temperature, 4);
        w[2] = r.sampling.top_k;
        std::memcpy(&w[3], &r.sampling.top_p, 4);
        sampling_words.insert(sampling_words.end(), w, w + 4);
    }
}

void Scheduler::launch() {
    if (in_flight()) throw std::logic_error("a step is in flight already: commit it first");
    int row = 0;
    for (const auto& p : plan_) {
        if (p.samples) ++row;
        if (p.dead) continue;
        Request& r = requests_[p.entry.slot];
        r.computed += p.entry.count;
        if (p.samples) r.pending_row = row - 1;
    }
    flight_.swap(plan_);
    plan_.clear();
}

std::vector<int> Scheduler::commit(const int32_t* sampled, int n_sampled) {
    std::vector<int> finished;
    const bool launched = in_flight();
    std::vector<PlannedEntry> step;
    step.swap(launched ? flight_ : plan_);
    int i = 0;
    for (const auto& p : step) {
        if (p.dead) {
            if (p.samples) ++i;
            continue;
        }
        Request& r = requests_[p.entry.slot];
        if (!launched) r.computed += p.entry.count;
        if (!p.samples) continue;  // a portion of a prompt: nothing to sample yet (engine.rs:209)
        if (i >= n_sampled) throw std::invalid_argument("fewer sampled tokens than entries that sample");
        int32_t token = sampled[i++];
        r.pending_row = -1;
        if (std::find(r.stop.begin(), r.stop.end(), token) != r.stop.end()) {
            r.finish = Finish::Stop;  // the stop token itself is not part of the output (engine.rs:214-216)
        } else {
            r.tokens.push_back(token);
            if (r.generated() >= r.max_new) r.finish = Finish::Length;
        }
        if (r.finish != Finish::None) {
            r.phase = Phase::Finished;
            cache_.release_pages(p.entry.slot);
            running_.erase(std::remove(running_.begin(), running_.end(), p.entry.slot), running_.end());
            finished.push_back(p.entry.slot);
            // what the step ahead runs for it (one token past a stop token) is for nothing
            if (launched)
                for (auto& q : plan_)
                    if (q.entry.slot == p.entry.slot) q.dead = true;
        }
    }
    if (i != n_sampled) throw std::invalid_argument("more sampled tokens than entries that sample");
    if (!launched) plan_.clear();
    return finished;
}

void Scheduler::abort(int slot) {
    if (slot < 0 || slot >= (int)requests_.size() || requests_[slot].phase == Phase::Free)
        throw std::logic_error("slot " + std::to_string(slot) + " holds no request");
    running_.erase(std::remove(running_.begin(), running_.end(), slot), running_.end());
    waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), slot), waiting_.end());
    plan_.erase(std::remove_if(plan_.begin(), plan_.end(), [&](const PlannedEntry& p) { return p.entry.slot == slot; }),
                plan_.end());
    for (auto& p : flight_)             // the step in flight keeps its rows: the entry's sample is dropped
        if (p.entry.slot == slot) p.dead = true;
    requests_[slot] = Request();
    cache_.release_slot(slot);
}

void Scheduler::drop(int slot) {
    if (slot < 0 || slot >= (int)requests_.size()) throw std::logic_error("no such slot");
    Request& r = requests_[slot];
    if (r.phase != Phase::Finished) throw std::logic_error("slot " + std::to_string(slot) + " holds no finished request");
    r = Request();
    cache_.release_slot(slot);
}

}  // namespace llmrs
