// The batch-forming decision as a pure function, after the reference's `schedule_batch`
// (src/scheduler.cpp:11-49): requests that still have prompt tokens to run are "prefill",
// the others "decode".  Both lists are ordered by aged priority (priority + wait / aging),
// then by arrival.  Policy mixed: every decoding request first gets one token, then prefilling
// requests in order get min(budget left, prompt left, chunk) until the budget is spent.
// Policy prefill_first: decodes run only when nothing is prefilling.
// portion_step > 1 (ours, not the reference's): a portion that does not end its prompt is cut down to a
// multiple of portion_step, so that the steps' shapes come again and the step function can replay them
// as captured graphs; a portion shorter than portion_step stays as it is.
#include <algorithm>
#include <cstdint>
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
    return priority + std::max<int64_t>(0, wait_ms) / aging_ms;
}

// policy: 0 mixed, 1 prefill_first.  Writes at most n slices; returns their number, or -1 on
// bad arguments.
int mlr_schedule_batch(const MlrScheduleItem* items, int n, int64_t batch_tokens, int64_t prefill_chunk,
                       int policy, int aging_ms, int64_t portion_step, MlrSlice* out) {
    if (n < 0 || batch_tokens <= 0 || prefill_chunk <= 0 || aging_ms <= 0 || (policy != 0 && policy != 1) ||
        portion_step < 0)
        return -1;
    std::vector<MlrScheduleItem> prefill, decode;
    for (int i = 0; i < n; ++i) (items[i].prefill_remaining > 0 ? prefill : decode).push_back(items[i]);
    const auto before = [&](const MlrScheduleItem& l, const MlrScheduleItem& r) {
        const auto lp = mlr_effective_priority(l.priority, l.wait_ms, aging_ms);
        const auto rp = mlr_effective_priority(r.priority, r.wait_ms, aging_ms);
        return lp != rp ? lp > rp : l.order < r.order;
    };
    std::stable_sort(prefill.begin(), prefill.end(), before);
    std::stable_sort(decode.begin(), decode.end(), before);
    int count = 0;
    int64_t remaining = batch_tokens;
    if (policy == 0 || prefill.empty()) {
        for (const auto& item : decode) {
            if (remaining == 0) break;
            out[count++] = {item.key, 1, 0};
            --remaining;
        }
    }
    for (const auto& item : prefill) {
        int64_t tokens = std::min({remaining, item.prefill_remaining, prefill_chunk});
        if (tokens == 0) break;
        if (portion_step > 1 && tokens < item.prefill_remaining) {
            const int64_t whole = tokens - tokens % portion_step;
            if (whole > 0) tokens = whole;                  // (a shorter portion stays: nothing may starve)
        }
        out[count++] = {item.key, tokens, 1};
        remaining -= tokens;
    }
    return count;
}

}  // extern "C"
