// Host side of the cache and of a step: slots, page lists and lengths of every sequence, and the
// layout of a step's integer arrays.  Plain C++ with a C ABI (no GPU call in this file): the Python
// classes PagedCache and plan_step are thin faces of it, and it is built and tested without a GPU.
//
// A cache handle owns
//   - a free list of slots, handed out lowest first,
//   - per paged group a free list of pages (lowest first) and a page list per slot,
//   - the length of every slot,
//   - the buffer the last planned step was laid out in.
// Nothing here touches device memory; the pools live in tensors that the Python side allocates.
//
// The reference keeps one padded [batch, T] matrix and derives positions from its mask
// (src/transformers/generation/utils.py:349-481); here tokens lie end to end and a token's position is
// its sequence's cached length plus its index in the step.
#include <algorithm>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

enum { OK = 0, ERR_STEP = 1, ERR_CACHE = 2, ERR_FULL = 3 };

// integers 0..n-1, handed out lowest first; the free ones are kept as a min-heap
struct FreeList {
    std::vector<int> heap;
    std::vector<char> held;
    void init(int n) {
        heap.resize(n);
        for (int i = 0; i < n; ++i) heap[i] = i;
        std::make_heap(heap.begin(), heap.end(), std::greater<int>());
        held.assign(n, 0);
    }
    int size() const { return (int)held.size(); }
    int free_count() const { return (int)heap.size(); }
    int take() {
        if (heap.empty()) return -1;
        std::pop_heap(heap.begin(), heap.end(), std::greater<int>());
        const int i = heap.back();
        heap.pop_back();
        held[i] = 1;
        return i;
    }
    bool is_held(int i) const { return i >= 0 && i < size() && held[i]; }
    bool give(int i) {
        if (!is_held(i)) return false;
        held[i] = 0;
        heap.push_back(i);
        std::push_heap(heap.begin(), heap.end(), std::greater<int>());
        return true;
    }
};

struct Group {
    FreeList pages;
    std::vector<std::vector<int>> lists;  // per slot: page of every 64 positions, -1 where a window has moved on
    int window = 0;                        // 0: all keys are kept; w: a token sees the last w positions only
};

struct Cache {
    int page_size = 64;
    FreeList slots;
    std::vector<int> length;
    std::vector<Group> groups;  // paged groups only
    std::vector<int32_t> plan;  // the last planned step
    std::vector<int> plan_sizes;

    int pages_for(int len) const { return (len + page_size - 1) / page_size; }
    // the first page a sequence of this length still reads: its next token, at position len, sees keys from
    // len - window + 1 on
    int first_needed(const Group& g, int len) const {
        return g.window > 0 ? std::max(0, len - g.window + 1) / page_size : 0;
    }
};

}  // namespace

extern "C" {

const char* ptah_last_error() { return g_error.c_str(); }

int ptah_abi_version() { return 4; }

void* ptah_cache_new(int max_slots, int page_size, int n_groups, const int* group_pages, const int* group_windows) {
    if (max_slots <= 0 || page_size <= 0 || n_groups < 0) {
        fail(ERR_CACHE, "cache: max_slots=%d page_size=%d groups=%d", max_slots, page_size, n_groups);
        return nullptr;
    }
    Cache* c = new Cache;
    c->page_size = page_size;
    c->slots.init(max_slots);
    c->length.assign(max_slots, 0);
    c->groups.resize(n_groups);
    for (int g = 0; g < n_groups; ++g) {
        c->groups[g].pages.init(group_pages[g]);
        c->groups[g].lists.assign(max_slots, {});
        c->groups[g].window = group_windows ? std::max(0, group_windows[g]) : 0;
    }
    return c;
}

void ptah_cache_delete(void* h) { delete static_cast<Cache*>(h); }

int ptah_alloc(void* h) {
    Cache* c = static_cast<Cache*>(h);
    const int s = c->slots.take();
    if (s < 0) {
        fail(ERR_FULL, "no free slot (all %d are held)", c->slots.size());
        return -1;
    }
    c->length[s] = 0;
    return s;
}

int ptah_is_live(void* h, int slot) { return static_cast<Cache*>(h)->slots.is_held(slot) ? 1 : 0; }

int ptah_free(void* h, int slot) {
    Cache* c = static_cast<Cache*>(h);
    if (!c->slots.is_held(slot)) return fail(ERR_CACHE, "slot %d is not allocated", slot);
    for (size_t g = 0; g < c->groups.size(); ++g) {
        for (int p : c->groups[g].lists[slot])
            if (p >= 0 && !c->groups[g].pages.give(p)) return fail(ERR_CACHE, "page %d of group %zu is freed twice", p, g);
        c->groups[g].lists[slot].clear();
    }
    c->length[slot] = 0;
    c->slots.give(slot);
    return OK;
}

int ptah_length(void* h, int slot) {
    Cache* c = static_cast<Cache*>(h);
    if (!c->slots.is_held(slot)) {
        fail(ERR_CACHE, "slot %d is not allocated", slot);
        return -1;
    }
    return c->length[slot];
}

int ptah_free_slots(void* h) { return static_cast<Cache*>(h)->slots.free_count(); }

int ptah_free_pages(void* h, int group) { return static_cast<Cache*>(h)->groups[group].pages.free_count(); }

int ptah_held_pages(void* h, int group) {
    Cache* c = static_cast<Cache*>(h);
    return c->groups[group].pages.size() - c->groups[group].pages.free_count();
}

// Give every slot the pages that new_tokens more tokens need; all or nothing.
int ptah_reserve(void* h, int n, const int* slots, const int* new_tokens) {
    Cache* c = static_cast<Cache*>(h);
    for (int i = 0; i < n; ++i) {
        if (!c->slots.is_held(slots[i])) return fail(ERR_CACHE, "slot %d is not allocated", slots[i]);
        for (int j = 0; j < i; ++j)
            if (slots[j] == slots[i]) return fail(ERR_CACHE, "a slot appears twice in one step: %d", slots[i]);
    }
    // pages that a window has left behind go back to the pool first: no later step reads them, whether
    // this one is accepted or not
    for (Group& gr : c->groups) {
        if (gr.window <= 0) continue;
        for (int i = 0; i < n; ++i) {
            std::vector<int>& l = gr.lists[slots[i]];
            const int keep_from = std::min((int)l.size(), c->first_needed(gr, c->length[slots[i]]));
            for (int k = 0; k < keep_from; ++k)
                if (l[k] >= 0) {
                    gr.pages.give(l[k]);
                    l[k] = -1;
                }
        }
    }
    for (size_t g = 0; g < c->groups.size(); ++g) {
        Group& gr = c->groups[g];
        long need = 0;
        for (int i = 0; i < n; ++i)
            need += std::max(0, c->pages_for(c->length[slots[i]] + new_tokens[i]) - (int)gr.lists[slots[i]].size());
        if (need > gr.pages.free_count())
            return fail(ERR_FULL, "cache group %zu needs %ld more pages of %d tokens for this step, %d of %d are free", g,
                        need, c->page_size, gr.pages.free_count(), gr.pages.size());
    }
    for (Group& gr : c->groups)
        for (int i = 0; i < n; ++i) {
            std::vector<int>& l = gr.lists[slots[i]];
            const int want = c->pages_for(c->length[slots[i]] + new_tokens[i]);
            while ((int)l.size() < want) l.push_back(gr.pages.take());
        }
    return OK;
}

int ptah_commit(void* h, int n, const int* slots, const int* new_tokens) {
    Cache* c = static_cast<Cache*>(h);
    for (int i = 0; i < n; ++i)
        if (!c->slots.is_held(slots[i])) return fail(ERR_CACHE, "slot %d is not allocated", slots[i]);
    for (int i = 0; i < n; ++i) c->length[slots[i]] += new_tokens[i];
    return OK;
}

int ptah_page_count(void* h, int group, int slot) {
    Cache* c = static_cast<Cache*>(h);
    if (!c->slots.is_held(slot)) {
        fail(ERR_CACHE, "slot %d is not allocated", slot);
        return -1;
    }
    return (int)c->groups[group].lists[slot].size();
}

int ptah_pages(void* h, int group, int slot, int* out) {
    Cache* c = static_cast<Cache*>(h);
    const std::vector<int>& l = c->groups[group].lists[slot];
    std::copy(l.begin(), l.end(), out);
    return (int)l.size();
}

// Every page is either free or in exactly one live slot's list, and every live slot has the pages its
// length needs.
int ptah_check(void* h) {
    Cache* c = static_cast<Cache*>(h);
    for (size_t g = 0; g < c->groups.size(); ++g) {
        const Group& gr = c->groups[g];
        std::vector<int> owner(gr.pages.size(), -1);
        int seen = 0;
        for (int s = 0; s < c->slots.size(); ++s) {
            const std::vector<int>& l = gr.lists[s];
            const bool live = c->slots.is_held(s);
            if (!l.empty() && !live) return fail(ERR_CACHE, "freed slot %d still lists %zu pages in group %zu", s, l.size(), g);
            if (live && (int)l.size() < c->pages_for(c->length[s]))
                return fail(ERR_CACHE, "slot %d has length %d but only %zu pages", s, c->length[s], l.size());
            for (size_t k = 0; k < l.size(); ++k) {
                const int p = l[k];
                if (p == -1 && live && (int)k < c->first_needed(gr, c->length[s])) continue;  // behind the window
                if (p < 0 || p >= gr.pages.size()) return fail(ERR_CACHE, "slot %d lists page %d, which does not exist", s, p);
                if (owner[p] >= 0) return fail(ERR_CACHE, "page %d of group %zu is held by slots %d and %d", p, g, owner[p], s);
                if (!gr.pages.is_held(p))
                    return fail(ERR_CACHE, "page %d of group %zu is in slot %d's list and in the free list", p, g, s);
                owner[p] = s;
                ++seen;
            }
        }
        const int held = gr.pages.size() - gr.pages.free_count();
        if (seen != held) return fail(ERR_CACHE, "group %zu: %d pages are marked held, %d are in slot lists", g, held, seen);
    }
    return OK;
}

// Check a step, reserve its pages and lay its arrays out in one int32 buffer:
//   token_ids [M] | token_seq [M] | token_pos [M] | cu_tokens [n+1] | seq_start [n] | seq_slot [n] |
//   logit_rows [R] | one page table [n, width_g] per paged group (width_g = most pages of any sequence)
// want_mode: 0 none, 1 the last token of each sequence, 2 all, 3 the places listed (want_counts per
// sequence, want_places flat).  sizes_out receives the 7 + groups piece sizes; the buffer is read with
// ptah_plan_data.  Returns 0, or 1 (bad step), 2 (cache misuse), 3 (pool full).
int ptah_plan_step(void* h, int n, const int* slots, const int* new_tokens, const long long* token_ids, int vocab,
                   int want_mode, const int* want_counts, const int* want_places, int* sizes_out) {
    Cache* c = static_cast<Cache*>(h);
    if (n <= 0) return fail(ERR_STEP, "a step needs at least one sequence");
    long M = 0;
    for (int i = 0; i < n; ++i) {
        if (new_tokens[i] <= 0) return fail(ERR_STEP, "sequence %d (slot %d) brings no tokens", i, slots[i]);
        M += new_tokens[i];
    }
    for (long t = 0; t < M; ++t)
        if (token_ids[t] < 0 || token_ids[t] >= vocab)
            return fail(ERR_STEP, "token id %lld is outside the vocabulary [0, %d)", token_ids[t], vocab);
    long R = 0;
    if (want_mode == 1) R = n;
    else if (want_mode == 2) R = M;
    else if (want_mode == 3) {
        long at = 0;
        for (int i = 0; i < n; ++i) {
            for (int k = 0; k < want_counts[i]; ++k, ++at)
                if (want_places[at] < 0 || want_places[at] >= new_tokens[i])
                    return fail(ERR_STEP, "sequence %d wants the logits at place %d, but brings %d tokens", i,
                                want_places[at], new_tokens[i]);
            R += want_counts[i];
        }
    } else if (want_mode != 0) {
        return fail(ERR_STEP, "unknown want mode %d", want_mode);
    }
    const int rc = ptah_reserve(h, n, slots, new_tokens);
    if (rc) return rc;

    const int G = (int)c->groups.size();
    std::vector<int> width(G, 1);
    for (int g = 0; g < G; ++g)
        for (int i = 0; i < n; ++i) width[g] = std::max(width[g], (int)c->groups[g].lists[slots[i]].size());
    c->plan_sizes = {(int)M, (int)M, (int)M, n + 1, n, n, (int)R};
    long total = 3 * M + (n + 1) + 2L * n + R;
    for (int g = 0; g < G; ++g) {
        c->plan_sizes.push_back(n * width[g]);
        total += (long)n * width[g];
    }
    c->plan.assign(total, 0);
    int32_t* ids = c->plan.data();
    int32_t *seq = ids + M, *pos = seq + M, *cu = pos + M, *start = cu + n + 1, *slot = start + n, *rows = slot + n;
    int32_t* table = rows + R;
    long at = 0, want_at = 0, row_at = 0;
    for (int i = 0; i < n; ++i) {
        const int len = c->length[slots[i]];
        cu[i] = (int32_t)at;
        start[i] = len;
        slot[i] = slots[i];
        for (int k = 0; k < new_tokens[i]; ++k) {
            ids[at + k] = (int32_t)token_ids[at + k];
            seq[at + k] = i;
            pos[at + k] = len + k;
        }
        if (want_mode == 1) rows[row_at++] = (int32_t)(at + new_tokens[i] - 1);
        else if (want_mode == 2)
            for (int k = 0; k < new_tokens[i]; ++k) rows[row_at++] = (int32_t)(at + k);
        else if (want_mode == 3)
            for (int k = 0; k < want_counts[i]; ++k) rows[row_at++] = (int32_t)(at + want_places[want_at++]);
        at += new_tokens[i];
    }
    cu[n] = (int32_t)at;
    for (int g = 0; g < G; ++g) {
        for (int i = 0; i < n; ++i) {
            const std::vector<int>& l = c->groups[g].lists[slots[i]];
            for (size_t k = 0; k < l.size(); ++k) table[(long)i * width[g] + k] = std::max(0, l[k]);  // a hole is never read
        }
        table += (long)n * width[g];
    }
    std::copy(c->plan_sizes.begin(), c->plan_sizes.end(), sizes_out);
    return OK;
}

const int* ptah_plan_data(void* h) { return static_cast<Cache*>(h)->plan.data(); }

// The common step of decoding, without the general planner's detours: every sequence brings one token and
// wants its logits.  Checks the step, reserves its pages and reports the longest context after it and the
// sum of all of them.
int ptah_decode_prepare(void* h, int n, const int* slots, const long long* tokens, int vocab, int* max_len_out,
                        long long* total_len_out) {
    Cache* c = static_cast<Cache*>(h);
    if (n <= 0) return fail(ERR_STEP, "a step needs at least one sequence");
    for (int i = 0; i < n; ++i)
        if (tokens[i] < 0 || tokens[i] >= vocab)
            return fail(ERR_STEP, "token id %lld is outside the vocabulary [0, %d)", tokens[i], vocab);
    std::vector<int> ones(n, 1);
    const int rc = ptah_reserve(h, n, slots, ones.data());
    if (rc) return rc;
    int longest = 0;
    long long total = 0;
    for (int i = 0; i < n; ++i) {
        longest = std::max(longest, c->length[slots[i]] + 1);
        total += c->length[slots[i]] + 1;
    }
    *max_len_out = longest;
    *total_len_out = total;
    return OK;
}

// ... and lays it out for a captured decode step of n_rows >= n sequences whose page tables are `width` pages
// wide, straight into the buffer that is copied to the device:
//   token_ids | token_seq | token_pos [n_rows each] | cu_tokens [n_rows + 1] | seq_start | seq_slot |
//   logit_rows [n_rows each] | one page table [n_rows, width] per paged group
// Rows past n are padding: token 0 as the first token of a sequence of its own, which lives in pad_slot (a row of
// the state tables that no sequence owns) and on pad_page (a page of every pool that no sequence owns), so that
// padding touches no sequence's keys, values or state, whatever the layers keep there.
int ptah_decode_fill(void* h, int n, const int* slots, const long long* tokens, int n_rows, int width, int pad_slot,
                     int pad_page, int32_t* out) {
    Cache* c = static_cast<Cache*>(h);
    if (n <= 0 || n_rows < n) return fail(ERR_STEP, "decode layout for %d rows cannot hold %d sequences", n_rows, n);
    int32_t *ids = out, *seq = ids + n_rows, *pos = seq + n_rows, *cu = pos + n_rows, *start = cu + n_rows + 1;
    int32_t *slot = start + n_rows, *rows = slot + n_rows, *table = rows + n_rows;
    for (int r = 0; r < n_rows; ++r) {
        const int len = r < n ? c->length[slots[r]] : 0;
        ids[r] = r < n ? (int32_t)tokens[r] : 0;
        seq[r] = r;
        pos[r] = len;
        cu[r] = r;
        start[r] = len;
        slot[r] = r < n ? slots[r] : pad_slot;
        rows[r] = r;
    }
    cu[n_rows] = n_rows;
    for (const Group& gr : c->groups) {
        for (int r = 0; r < n_rows; ++r) {
            int32_t* row = table + (long)r * width;
            if (r >= n) {
                for (int k = 0; k < width; ++k) row[k] = pad_page;
                continue;
            }
            const std::vector<int>& l = gr.lists[slots[r]];
            if ((int)l.size() > width) return fail(ERR_STEP, "a sequence holds %zu pages, the layout has room for %d", l.size(), width);
            for (size_t k = 0; k < l.size(); ++k) row[k] = std::max(0, l[k]);
            for (int k = (int)l.size(); k < width; ++k) row[k] = 0;
        }
        table += (long)n_rows * width;
    }
    return OK;
}

// every listed slot grew by one token
int ptah_commit_ones(void* h, int n, const int* slots) {
    Cache* c = static_cast<Cache*>(h);
    for (int i = 0; i < n; ++i)
        if (!c->slots.is_held(slots[i])) return fail(ERR_CACHE, "slot %d is not allocated", slots[i]);
    for (int i = 0; i < n; ++i) c->length[slots[i]] += 1;
    return OK;
}

}  // extern "C"
