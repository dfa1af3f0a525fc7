// The C interface of the host core: cache manager, batch builder and scheduler
// behind one handle.  Every function returns a negative number on error and
// leaves the message for llmrs_core_error().
#include <cstring>
#include <exception>
#include <memory>
#include <string>
#include <vector>

#include "batch.h"
#include "cache_manager.h"
#include "scheduler.h"

using namespace llmrs;

namespace {

struct Core {
    std::unique_ptr<CacheManager> cache;
    std::unique_ptr<Scheduler> scheduler;
    std::string error;
    // scratch of the last scheduler plan
    std::vector<int32_t> tokens, want_rows, sampling;
};

thread_local std::string g_create_error;

template <class F>
int guarded(Core* core, F&& f) {
    try {
        return f();
    } catch (const std::exception& e) {
        core->error = e.what();
        return -1;
    }
}

int write_batch(Core* c, const std::vector<BatchEntry>& entries, const int32_t* tokens,
                const int32_t* want_rows, int n_want, const int32_t* sampling, const int32_t* fixed_widths,
                int32_t* words, int cap_words, int32_t* offsets_out) {
    int T = 0;
    for (const auto& e : entries) {
        if (!c->cache->slot_in_use(e.slot)) throw std::logic_error("slot " + std::to_string(e.slot) + " is not in use");
        T += e.count;
    }
    int R = (int)entries.size();
    std::vector<int> widths = table_widths(*c->cache, entries);
    if (fixed_widths)
        for (size_t g = 0; g < widths.size(); ++g) {
            if (fixed_widths[g] < widths[g]) throw std::invalid_argument("block table wider than the fixed width");
            widths[g] = fixed_widths[g];
        }
    BatchLayout l = batch_layout(T, R, n_want, widths);
    if (l.words > cap_words)
        throw std::invalid_argument("batch needs " + std::to_string(l.words) + " words, the buffer has " + std::to_string(cap_words));
    fill_batch(*c->cache, entries, tokens, want_rows, n_want, widths, l, words);
    if (sampling) std::memcpy(words + l.sampling, sampling, sizeof(int32_t) * 4 * n_want);
    // offsets: 9 fixed arrays, then per group (slot_map, table, width)
    int32_t fixed[9] = {l.header, l.tokens, l.positions, l.token_entry, l.q_starts, l.seq_lens, l.slots, l.want_rows, l.sampling};
    std::memcpy(offsets_out, fixed, sizeof(fixed));
    for (int g = 0; g < c->cache->num_groups(); ++g) {
        offsets_out[9 + 3 * g + 0] = group_slot_map_offset(l, g, T, R, widths);
        offsets_out[9 + 3 * g + 1] = group_table_offset(l, g, T, R, widths);
        offsets_out[9 + 3 * g + 2] = widths[g];
    }
    return l.words;
}

}  // namespace

extern "C" {

const char* llmrs_create_error() { return g_create_error.c_str(); }

void* llmrs_core_create(int n_groups, const int* page_size, const int* num_pages, const int* window,
                        int max_requests, int token_budget, int max_chunk, int max_positions) {
    try {
        std::vector<GroupSpec> groups;
        for (int g = 0; g < n_groups; ++g) groups.push_back({page_size[g], num_pages[g], window[g]});
        auto core = std::make_unique<Core>();
        core->cache = std::make_unique<CacheManager>(groups, max_requests);
        core->scheduler = std::make_unique<Scheduler>(*core->cache, token_budget, max_chunk, max_positions);
        return core.release();
    } catch (const std::exception& e) {
        g_create_error = e.what();
        return nullptr;
    }
}

void llmrs_core_destroy(void* h) { delete (Core*)h; }
const char* llmrs_core_error(void* h) { return ((Core*)h)->error.c_str(); }

// ---- cache manager -------------------------------------------------------
int llmrs_slot_acquire(void* h) { auto c = (Core*)h; return guarded(c, [&] { int s = c->cache->acquire_slot(); if (s < 0) { c->error = "no free request slot"; } return s; }); }
int llmrs_slot_release(void* h, int slot) { auto c = (Core*)h; return guarded(c, [&] { c->cache->release_slot(slot); return 0; }); }
int llmrs_slots_in_use(void* h) { return ((Core*)h)->cache->slots_in_use(); }
int llmrs_pages_free(void* h, int g) { return ((Core*)h)->cache->pages_free(g); }
int llmrs_pages_total(void* h, int g) { return ((Core*)h)->cache->pages_total(g); }
int llmrs_pages_held(void* h, int slot, int g) { auto c = (Core*)h; return guarded(c, [&] { return c->cache->pages_held(slot, g); }); }
// 1: pages are there; 0: not enough free pages, nothing taken
int llmrs_ensure(void* h, int slot, int start, int count) { auto c = (Core*)h; return guarded(c, [&] { return c->cache->ensure(slot, start, count) ? 1 : 0; }); }
int llmrs_release_pages(void* h, int slot) { auto c = (Core*)h; return guarded(c, [&] { c->cache->release_pages(slot); return 0; }); }
int llmrs_table(void* h, int slot, int g, int32_t* out, int cap) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        if (!c->cache->slot_in_use(slot)) throw std::logic_error("slot " + std::to_string(slot) + " is not in use");
        const auto& t = c->cache->table(slot, g);
        for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
        return (int)t.size();
    });
}

// ---- batch ---------------------------------------------------------------
// Number of offsets write_batch reports.
int llmrs_batch_num_offsets(void* h) { return 9 + 3 * ((Core*)h)->cache->num_groups(); }

int llmrs_build_batch(void* h, int R, const int32_t* slots, const int32_t* starts, const int32_t* counts,
                      const int32_t* tokens, const int32_t* want_rows, int n_want, const int32_t* fixed_widths,
                      int32_t* words, int cap_words, int32_t* offsets_out) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        std::vector<BatchEntry> entries;
        for (int r = 0; r < R; ++r) entries.push_back({slots[r], starts[r], counts[r]});
        return write_batch(c, entries, tokens, want_rows, n_want, nullptr, fixed_widths, words, cap_words, offsets_out);
    });
}

// ---- scheduler -----------------------------------------------------------
// slot >= 0; -2: no slot free now; -1: the request can never run (see error)
int llmrs_sched_add(void* h, const int32_t* prompt, int n_prompt, int max_new, float temperature, int top_k,
                    float top_p, uint64_t seed, const int32_t* stop, int n_stop) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        SamplingParams sp{temperature, top_k, top_p, seed};
        int slot = c->scheduler->add(prompt, n_prompt, max_new, sp, stop, n_stop);
        return slot < 0 ? -2 : slot;
    });
}
// 0 when a request of these lengths could run, -1 when llmrs_sched_add would refuse it for good (see error)
int llmrs_sched_check(void* h, int n_prompt, int max_new) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        c->scheduler->check(n_prompt, max_new);
        return 0;
    });
}
int llmrs_sched_idle(void* h) { return ((Core*)h)->scheduler->idle() ? 1 : 0; }
int llmrs_sched_running(void* h) { return ((Core*)h)->scheduler->num_running(); }
int llmrs_sched_waiting(void* h) { return ((Core*)h)->scheduler->num_waiting(); }
long long llmrs_sched_preemptions(void* h) { return ((Core*)h)->scheduler->preemptions(); }

// Plans the next step.  Returns R and fills slots/starts/counts/samples (cap each).
int llmrs_sched_plan(void* h, int32_t* slots, int32_t* starts, int32_t* counts, int32_t* samples, int cap) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        const auto& plan = c->scheduler->plan();
        if ((int)plan.size() > cap) throw std::invalid_argument("plan larger than the caller's buffers");
        for (size_t i = 0; i < plan.size(); ++i) {
            slots[i] = plan[i].entry.slot;
            starts[i] = plan[i].entry.start;
            counts[i] = plan[i].entry.count;
            samples[i] = plan[i].samples;
        }
        return (int)plan.size();
    });
}

// For each entry of the plan the row of the step in flight whose sample is its one token, or -1.  Returns R.
int llmrs_sched_plan_sources(void* h, int32_t* sources, int cap) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        const auto& plan = c->scheduler->planned();
        if ((int)plan.size() > cap) throw std::invalid_argument("plan larger than the caller's buffer");
        for (size_t i = 0; i < plan.size(); ++i) sources[i] = plan[i].pending_src;
        return (int)plan.size();
    });
}

// The planned step has been started on the device; the next one may be planned before it is committed.
int llmrs_sched_launch(void* h) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        c->scheduler->launch();
        return 0;
    });
}

int llmrs_sched_in_flight(void* h) { return ((Core*)h)->scheduler->in_flight() ? 1 : 0; }
int llmrs_sched_set_max_chunk(void* h, int max_chunk) { auto c = (Core*)h; return guarded(c, [&] { c->scheduler->set_max_chunk(max_chunk); return 0; }); }

// Writes the planned step's batch.  Returns the words used; n_tokens_out and
// n_want_out get the step's tokens and the number of rows that sample.
int llmrs_sched_build(void* h, const int32_t* fixed_widths, int32_t* words, int cap_words, int32_t* offsets_out,
                      int32_t* n_tokens_out, int32_t* n_want_out) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        c->scheduler->plan_tokens(c->tokens, c->want_rows, c->sampling);
        std::vector<BatchEntry> entries;
        for (const auto& p : c->scheduler->planned()) entries.push_back(p.entry);
        *n_tokens_out = (int32_t)c->tokens.size();
        *n_want_out = (int32_t)c->want_rows.size();
        return write_batch(c, entries, c->tokens.data(), c->want_rows.data(), (int)c->want_rows.size(),
                           c->sampling.data(), fixed_widths, words, cap_words, offsets_out);
    });
}

// Takes one sampled token for each row that sampled; returns the number of
// requests that finished and their slots.
int llmrs_sched_commit(void* h, const int32_t* sampled, int n_sampled, int32_t* finished, int cap) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        std::vector<int> done = c->scheduler->commit(sampled, n_sampled);
        if ((int)done.size() > cap) throw std::invalid_argument("more finished requests than the caller's buffer holds");
        for (size_t i = 0; i < done.size(); ++i) finished[i] = done[i];
        return (int)done.size();
    });
}

// info: prompt_len, generated, computed, phase (0 free, 1 waiting, 2 running, 3 finished),
// finish reason (0 none, 1 stop, 2 length), preemptions
int llmrs_request_info(void* h, int slot, int32_t* info) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        if (slot < 0 || slot >= c->cache->max_requests()) throw std::invalid_argument("no such slot");
        const Request& r = c->scheduler->request(slot);
        info[0] = r.prompt_len;
        info[1] = r.generated();
        info[2] = r.computed;
        info[3] = (int)r.phase;
        info[4] = (int)r.finish;
        info[5] = r.preemptions;
        return 0;
    });
}

// Copies what the request generated so far; returns its length.
int llmrs_request_output(void* h, int slot, int32_t* out, int cap) {
    auto c = (Core*)h;
    return guarded(c, [&] {
        if (slot < 0 || slot >= c->cache->max_requests()) throw std::invalid_argument("no such slot");
        const Request& r = c->scheduler->request(slot);
        int n = r.generated();
        for (int i = 0; i < n && i < cap; ++i) out[i] = r.tokens[r.prompt_len + i];
        return n;
    });
}

int llmrs_request_abort(void* h, int slot) { auto c = (Core*)h; return guarded(c, [&] { c->scheduler->abort(slot); return 0; }); }
int llmrs_request_drop(void* h, int slot) { auto c = (Core*)h; return guarded(c, [&] { c->scheduler->drop(slot); return 0; }); }

// The reference's generator, for callers that sample outside the scheduler.
uint64_t llmrs_xorshift_next(uint64_t* state) {
    Xorshift64 g(1);
    g.state = *state;
    uint64_t x = g.next_u64();
    *state = g.state;
    return x;
}

}  // extern "C"
