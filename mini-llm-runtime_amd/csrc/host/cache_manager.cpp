// Page and slot bookkeeping of the cache, host side only (no device calls).
//
// A request lives in a slot (a small integer) from its admission to its end.  The layers of a
// model fall into groups with equal cache needs; each group has a pool of pages of its own, a
// LIFO free list and a dense block table [slots][max_blocks] (-1 = no page).  A page id of a
// group is valid in every layer of that group.  A step is two-phase, as in the reference's
// page transactions (src/minillm/cuda/page_table.cpp:32-96): `prepare` checks a whole batch
// (slots live, lengths within bounds, enough free pages in every group) and changes nothing;
// `commit` takes the pages and advances the lengths; `retire` (after the step ran) gives
// back the pages that a window has passed.  `release_slot` gives back everything the
// request holds.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

struct Group {
    int page_size = 0, num_pages = 0, window = 0, max_blocks = 0;
    std::vector<int32_t> free_list;          // LIFO: the page freed last is taken first
    std::vector<int32_t> table;              // [slots][max_blocks]
    std::vector<int32_t> owner;              // [num_pages]: slot or -1
    std::vector<int32_t> first_block;        // [slots]: blocks below it were retired
    std::vector<uint8_t> dirty;              // [slots]
};

struct Cache {
    int max_slots = 0, max_length = 0;
    std::vector<uint8_t> live;
    std::vector<int32_t> length;
    std::vector<int32_t> free_slots;         // LIFO
    std::vector<Group> groups;
    std::vector<int32_t> scratch_len;        // per slot, for prepare
};

int blocks_for(int tokens, int page) { return (tokens + page - 1) / page; }

// New total length per slot after the batch; -1 bad slot, -2 too long, -4 bad count.
int new_lengths(Cache& c, const int32_t* slots, const int32_t* counts, int n) {
    c.scratch_len = c.length;
    for (int i = 0; i < n; ++i) {
        const int s = slots[i];
        if (s < 0 || s >= c.max_slots || !c.live[s]) return -1;
        if (counts[i] <= 0) return -4;
        if ((int64_t)c.scratch_len[s] + counts[i] > c.max_length) return -2;
        c.scratch_len[s] += counts[i];
    }
    return 0;
}

}  // namespace

extern "C" {

void* mlr_cache_create(int max_slots, int max_length) {
    if (max_slots <= 0 || max_length <= 0) return nullptr;
    auto* c = new Cache;
    c->max_slots = max_slots;
    c->max_length = max_length;
    c->live.assign(max_slots, 0);
    c->length.assign(max_slots, 0);
    for (int s = max_slots - 1; s >= 0; --s) c->free_slots.push_back(s);
    return c;
}

void mlr_cache_destroy(void* h) { delete static_cast<Cache*>(h); }

// window <= 0: every key is kept.  Returns the group's index or -1.
int mlr_cache_add_group(void* h, int page_size, int num_pages, int window) {
    auto* c = static_cast<Cache*>(h);
    if (page_size <= 0 || num_pages <= 0) return -1;
    Group g;
    g.page_size = page_size;
    g.num_pages = num_pages;
    g.window = window > 0 ? window : 0;
    g.max_blocks = blocks_for(c->max_length, page_size);
    // A fresh pool hands its pages out in a fixed shuffled order.  In ascending order, requests of equal
    // length that start together lie a power of two apart, and the workgroups that read block i of each of
    // them at the same moment meet in the same memory channels (measured: decoding attention over 64 such
    // requests streams at 4.7 TB/s, over pages that lie anywhere at 5.7).
    for (int p = num_pages - 1; p >= 0; --p) g.free_list.push_back(p);
    uint64_t state = 0x9E3779B97F4A7C15ull;
    for (int i = num_pages - 1; i > 0; --i) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        const int j = (int)((state >> 33) % (uint64_t)(i + 1));
        std::swap(g.free_list[i], g.free_list[j]);
    }
    g.table.assign((size_t)c->max_slots * g.max_blocks, -1);
    g.owner.assign(num_pages, -1);
    g.first_block.assign(c->max_slots, 0);
    g.dirty.assign(c->max_slots, 1);
    c->groups.push_back(std::move(g));
    return (int)c->groups.size() - 1;
}

int mlr_cache_max_blocks(void* h, int group) { return static_cast<Cache*>(h)->groups[group].max_blocks; }
int mlr_cache_free_pages(void* h, int group) { return (int)static_cast<Cache*>(h)->groups[group].free_list.size(); }
int mlr_cache_free_slots(void* h) { return (int)static_cast<Cache*>(h)->free_slots.size(); }
const int32_t* mlr_cache_table(void* h, int group) { return static_cast<Cache*>(h)->groups[group].table.data(); }

int mlr_cache_length(void* h, int slot) {
    auto* c = static_cast<Cache*>(h);
    return (slot < 0 || slot >= c->max_slots || !c->live[slot]) ? -1 : c->length[slot];
}

int mlr_cache_acquire_slot(void* h) {
    auto* c = static_cast<Cache*>(h);
    if (c->free_slots.empty()) return -1;
    const int s = c->free_slots.back();
    c->free_slots.pop_back();
    c->live[s] = 1;
    c->length[s] = 0;
    for (auto& g : c->groups) g.first_block[s] = 0;
    return s;
}

// Gives back the slot and every page it holds.  -1: the slot is not live (freed twice).
int mlr_cache_release_slot(void* h, int slot) {
    auto* c = static_cast<Cache*>(h);
    if (slot < 0 || slot >= c->max_slots || !c->live[slot]) return -1;
    for (auto& g : c->groups) {
        int32_t* row = g.table.data() + (size_t)slot * g.max_blocks;
        const int used = blocks_for(c->length[slot], g.page_size);
        for (int b = 0; b < used; ++b) {
            if (row[b] >= 0) {
                g.owner[row[b]] = -1;
                g.free_list.push_back(row[b]);
                row[b] = -1;
            }
        }
        g.dirty[slot] = 1;
        g.first_block[slot] = 0;
    }
    c->live[slot] = 0;
    c->length[slot] = 0;
    c->free_slots.push_back(slot);
    return 0;
}

// Checks the batch {slot, number of new tokens}; a slot may appear once.  Changes nothing.
// 0 ok; -1 slot not live; -2 longer than max_length; -3 not enough free pages (group index in
// *short_group, pages needed and free in need_free[0..1]); -4 bad count; -5 slot twice.
int mlr_cache_prepare(void* h, const int32_t* slots, const int32_t* counts, int n, int* short_group,
                      int* need_free) {
    auto* c = static_cast<Cache*>(h);
    for (int i = 0; i < n; ++i)
        for (int j = 0; j < i; ++j)
            if (slots[i] == slots[j]) return -5;
    const int rc = new_lengths(*c, slots, counts, n);
    if (rc != 0) return rc;
    for (size_t gi = 0; gi < c->groups.size(); ++gi) {
        const Group& g = c->groups[gi];
        int64_t need = 0;
        for (int i = 0; i < n; ++i) {
            const int s = slots[i];
            need += blocks_for(c->scratch_len[s], g.page_size) - blocks_for(c->length[s], g.page_size);
        }
        if (need > (int64_t)g.free_list.size()) {
            if (short_group) *short_group = (int)gi;
            if (need_free) { need_free[0] = (int)need; need_free[1] = (int)g.free_list.size(); }
            return -3;
        }
    }
    return 0;
}

// Takes the pages for the batch and advances the lengths.  Runs `prepare` first and fails the
// same way, without side effects.
int mlr_cache_commit(void* h, const int32_t* slots, const int32_t* counts, int n) {
    auto* c = static_cast<Cache*>(h);
    const int rc = mlr_cache_prepare(h, slots, counts, n, nullptr, nullptr);
    if (rc != 0) return rc;
    for (auto& g : c->groups) {
        for (int i = 0; i < n; ++i) {
            const int s = slots[i];
            const int from = blocks_for(c->length[s], g.page_size);
            const int to = blocks_for(c->length[s] + counts[i], g.page_size);
            int32_t* row = g.table.data() + (size_t)s * g.max_blocks;
            for (int b = from; b < to; ++b) {
                const int page = g.free_list.back();
                g.free_list.pop_back();
                g.owner[page] = s;
                row[b] = page;
            }
            if (to > from) g.dirty[s] = 1;
        }
    }
    for (int i = 0; i < n; ++i) c->length[slots[i]] += counts[i];
    return 0;
}

// `commit` that also reports where each entry's tokens start (the slot's length before the batch).
int mlr_cache_commit_first(void* h, const int32_t* slots, const int32_t* counts, int n, int32_t* first) {
    auto* c = static_cast<Cache*>(h);
    for (int i = 0; i < n; ++i) {
        const int s = slots[i];
        first[i] = (s >= 0 && s < c->max_slots && c->live[s]) ? c->length[s] : -1;
    }
    return mlr_cache_commit(h, slots, counts, n);
}

// After the step ran: in groups with a window, pages whose keys no later query can see go
// back to the pool.  A query at position >= length sees keys > position - window.
int mlr_cache_retire(void* h, const int32_t* slots, int n) {
    auto* c = static_cast<Cache*>(h);
    int freed = 0;
    for (auto& g : c->groups) {
        if (g.window <= 0) continue;
        for (int i = 0; i < n; ++i) {
            const int s = slots[i];
            if (s < 0 || s >= c->max_slots || !c->live[s]) return -1;
            const int first_needed = std::max(0, c->length[s] - g.window + 1);   // lowest key still seen
            const int keep_from = first_needed / g.page_size;
            int32_t* row = g.table.data() + (size_t)s * g.max_blocks;
            for (int b = g.first_block[s]; b < keep_from; ++b) {
                if (row[b] >= 0) {
                    g.owner[row[b]] = -1;
                    g.free_list.push_back(row[b]);
                    row[b] = -1;
                    g.dirty[s] = 1;
                    ++freed;
                }
            }
            g.first_block[s] = std::max(g.first_block[s], keep_from);
        }
    }
    return freed;
}

// Writes the slots whose table row changed since the last call into out (room for every slot)
// and clears the marks.
int mlr_cache_take_dirty(void* h, int group, int32_t* out) {
    auto* c = static_cast<Cache*>(h);
    Group& g = c->groups[group];
    int n = 0;
    for (int s = 0; s < c->max_slots; ++s) {
        if (g.dirty[s]) {
            out[n++] = s;
            g.dirty[s] = 0;
        }
    }
    return n;
}

// Invariants: every page is either free or held by exactly one live slot's table, exactly
// once; free list and owner array agree; rows of dead slots are empty.  0 when they hold.
int mlr_cache_check(void* h) {
    auto* c = static_cast<Cache*>(h);
    for (const auto& g : c->groups) {
        std::vector<int> seen(g.num_pages, 0);
        for (int p : g.free_list) {
            if (p < 0 || p >= g.num_pages || seen[p]++ || g.owner[p] != -1) return 1;
        }
        for (int s = 0; s < c->max_slots; ++s) {
            const int32_t* row = g.table.data() + (size_t)s * g.max_blocks;
            const int used = c->live[s] ? blocks_for(c->length[s], g.page_size) : 0;
            for (int b = 0; b < g.max_blocks; ++b) {
                const int p = row[b];
                if (p < 0) {
                    if (b < used && b >= g.first_block[s]) return 2;       // a needed page is missing
                    continue;
                }
                if (b >= used || p >= g.num_pages || seen[p]++ || g.owner[p] != s) return 3;
            }
        }
        for (int p = 0; p < g.num_pages; ++p)
            if (seen[p] != 1) return 4;                                     // lost or held twice
    }
    int live = 0;
    for (int s = 0; s < c->max_slots; ++s) live += c->live[s];
    if (live + (int)c->free_slots.size() != c->max_slots) return 5;
    return 0;
}

}  // extern "C"
