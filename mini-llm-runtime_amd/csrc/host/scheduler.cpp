// Which request brings how many tokens to the next step: a pure function of the running requests.
//
// The decision is the reference's (src/scheduler.cpp:11-49, vectors in tests/core_tests.cpp:123-146):
// a request that still has prompt tokens to run is a prompt, the others decode; rank = aged priority
// (priority + whole aging intervals waited), higher first, earlier arrival first among equals.  Policy
// 0 (mixed): every decoding request gets one token, in rank order, while the budget lasts; what is
// left goes to prompts in rank order, each min(budget left, prompt left, chunk).  Policy 1
// (prefill_first): as long as any prompt runs, decoding requests get nothing.
//
// How it is done here: every request gets one rank in one sorted index array, which is swept twice
// (single tokens, then portions), so that the slices come out in the order the step function wants
// them: single tokens in front, portions behind.
//
// portion_step > 1 is this engine's own: a portion that does not end its prompt is cut down to a
// multiple of portion_step, so that step shapes come again and can be replayed as captured graphs; a
// portion shorter than portion_step stays as it is, so that nothing starves.
#include <algorithm>
#include <cstdint>
#include <numeric>
#include <vector>

extern "C" {

struct MlrScheduleItem {
    int64_t key;
    int64_t prefill_remaining;
    int32_t priority;
    int64_t wait_ms;
    uint64_t order;
};

struct MlrSlice {
    int64_t key;
    int64_t tokens;
    int32_t prefill;
};

int64_t mlr_effective_priority(int priority, int64_t wait_ms, int aging_ms) {
    const int64_t waited = wait_ms > 0 ? wait_ms : 0;
    return (int64_t)priority + waited / aging_ms;
}

// Writes at most n slices; returns their number, or -1 on bad arguments.
int mlr_schedule_batch(const MlrScheduleItem* items, int n, int64_t batch_tokens, int64_t prefill_chunk,
                       int policy, int aging_ms, int64_t portion_step, MlrSlice* out) {
    const bool arguments_ok = n >= 0 && batch_tokens > 0 && prefill_chunk > 0 && aging_ms > 0 &&
                              (policy == 0 || policy == 1) && portion_step >= 0;
    if (!arguments_ok) return -1;

    std::vector<int64_t> rank(n);
    bool prompts_run = false;
    for (int i = 0; i < n; ++i) {
        rank[i] = mlr_effective_priority(items[i].priority, items[i].wait_ms, aging_ms);
        prompts_run = prompts_run || items[i].prefill_remaining > 0;
    }
    std::vector<int> by_rank(n);
    std::iota(by_rank.begin(), by_rank.end(), 0);
    std::sort(by_rank.begin(), by_rank.end(), [&](int a, int b) {
        if (rank[a] != rank[b]) return rank[a] > rank[b];
        if (items[a].order != items[b].order) return items[a].order < items[b].order;
        return a < b;
    });

    int written = 0;
    int64_t budget = batch_tokens;
    const bool decoding_runs = policy == 0 || !prompts_run;
    if (decoding_runs) {
        for (int i : by_rank) {
            if (budget == 0) break;
            if (items[i].prefill_remaining > 0) continue;
            out[written++] = MlrSlice{items[i].key, 1, 0};
            budget -= 1;
        }
    }
    for (int i : by_rank) {
        const int64_t left = items[i].prefill_remaining;
        if (left <= 0) continue;
        if (budget == 0) break;
        int64_t take = std::min(std::min(budget, prefill_chunk), left);
        if (portion_step > 1 && take < left && take >= portion_step) take -= take % portion_step;
        out[written++] = MlrSlice{items[i].key, take, 1};
        budget -= take;
    }
    return written;
}

// Which waiting requests start now: a pure function of the queue, the pages that are not set aside and the
// free request slots (the reference's admission, src/engine.cpp:295-355).  The queue is walked by aged
// priority, higher first, earlier arrival first among equals; a request starts when the pages of its whole
// life (prompt and every token it may generate) are free and a slot is; one that does not fit is passed over,
// unless it has waited `reserve_ms` or longer: then nothing behind it starts, so that what is given back goes
// to it.  `sorted` receives the queue's order of the walk (all n indices), `admitted` the indices that start,
// in that order; `waits` counts the requests that did not fit.  Returns the number admitted, -1 on bad arguments.
struct MlrWaiting {
    int64_t pages;
    int32_t priority;
    int64_t waited_ms;
    uint64_t order;
};

int mlr_admit(const MlrWaiting* items, int n, int64_t free_pages, int free_slots, int aging_ms, int64_t reserve_ms,
              int32_t* sorted, int32_t* admitted, int64_t* waits) {
    if (n < 0 || aging_ms <= 0 || reserve_ms < 0 || free_pages < 0) return -1;
    std::vector<int64_t> rank(n);
    for (int i = 0; i < n; ++i) rank[i] = mlr_effective_priority(items[i].priority, items[i].waited_ms, aging_ms);
    std::vector<int32_t> walk(n);
    std::iota(walk.begin(), walk.end(), 0);
    std::sort(walk.begin(), walk.end(), [&](int a, int b) {
        if (rank[a] != rank[b]) return rank[a] > rank[b];
        if (items[a].order != items[b].order) return items[a].order < items[b].order;
        return a < b;
    });
    int started = 0;
    *waits = 0;
    for (int at = 0; at < n; ++at) {
        const int i = walk[at];
        sorted[at] = i;
        if (free_slots <= 0) continue;                   // (the rest of the walk only writes the order down)
        if (items[i].pages <= free_pages) {
            admitted[started++] = i;
            free_pages -= items[i].pages;
            free_slots -= 1;
        } else {
            *waits += 1;
            if (items[i].waited_ms >= reserve_ms) free_slots = 0;      // the pool is kept for this one
        }
    }
    return started;
}

}  // extern "C"
