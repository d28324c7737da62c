// The host side of the cache and of a step, in C++ (no GPU code; compiled with the host compiler).
//
//  * PageTables: the pages of one cache group.  The free list and the block tables of the
//    request slots, as the reference's BlockTableManager keeps them
//    (src/engine/block_table_manager.cpp:17-274): the first pages handed out are 0, 1, 2, ...;
//    pages given back are stacked in the order given, so the last one given back is the first
//    one used again (:213-253); growing takes all the pages it needs or none (:60-89);
//    token slot = table[pos / P] * P + pos % P (:91-122).  Beyond the reference: a window
//    gives pages back as soon as no later query can see them, and new table entries are
//    remembered until they have been sent to the device table.
//  * lle_layout_step: the integer arrays of one step (token ids, positions, the request of
//    each token, slots, lengths, wanted rows, and every token's page slot in every group),
//    written into one buffer that travels to the device in one copy.
//
// Functions return 0 or one of the LLE_HOST_* codes; they change nothing when they fail.
#include <algorithm>
#include <cstdint>
#include <vector>

#define LLE_HOST_OK 0
#define LLE_HOST_OUT_OF_PAGES 1
#define LLE_HOST_NO_SUCH_PAGE 2
#define LLE_HOST_FREED_TWICE 3
#define LLE_HOST_TOO_MANY_PAGES 4
#define LLE_HOST_BAD_TOKEN 5
#define LLE_HOST_NO_PAGE_AT_POSITION 6
#define LLE_HOST_BAD_ARGUMENT 7

namespace {

struct PageTables {
    int num_pages = 0, page_size = 1, max_requests = 0, max_pages_per_request = 0;
    int window = -1;                    // < 0: every key stays needed
    std::vector<int32_t> free_list;     // a stack: back() is handed out next
    std::vector<uint8_t> held;
    std::vector<std::vector<int32_t>> tables;  // per request slot: logical page -> physical page, -1 once given back
    std::vector<int32_t> first_live;
    std::vector<int32_t> pending_index, pending_page;  // entries of the device table not yet sent

    int pages_for(int length) const { return (length + page_size - 1) / page_size; }
    int new_pages_needed(int slot, int new_len) const {
        return std::max(0, pages_for(new_len) - (int)tables[slot].size());
    }
    void give_back(int32_t page) {
        held[page] = 0;
        free_list.push_back(page);
    }
};

inline PageTables* pt(void* h) { return static_cast<PageTables*>(h); }

}  // namespace

extern "C" {

const char* lle_error_string(int code) {
    switch (code) {
        case LLE_HOST_OK: return "ok";
        case LLE_HOST_OUT_OF_PAGES: return "not enough free physical blocks";
        case LLE_HOST_NO_SUCH_PAGE: return "page does not exist";
        case LLE_HOST_FREED_TWICE: return "page is given back twice";
        case LLE_HOST_TOO_MANY_PAGES: return "more pages than a request may hold";
        case LLE_HOST_BAD_TOKEN: return "token id outside the vocabulary";
        case LLE_HOST_NO_PAGE_AT_POSITION: return "position without a page";
        case LLE_HOST_BAD_ARGUMENT: return "bad argument";
    }
    return "unknown";
}

void* lle_pt_create(int num_pages, int page_size, int max_requests, int max_pages_per_request, int window) {
    if (num_pages <= 0 || page_size <= 0 || max_requests < 0 || max_pages_per_request < 0) return nullptr;
    PageTables* t = new PageTables;
    t->num_pages = num_pages;
    t->page_size = page_size;
    t->max_requests = max_requests;
    t->max_pages_per_request = max_pages_per_request;
    t->window = window;
    t->free_list.resize(num_pages);
    for (int i = 0; i < num_pages; ++i) t->free_list[i] = num_pages - 1 - i;  // page 0 on top
    t->held.assign(num_pages, 0);
    t->tables.resize(max_requests);
    t->first_live.assign(max_requests, 0);
    return t;
}

void lle_pt_destroy(void* h) { delete pt(h); }

int lle_pt_num_pages(void* h) { return pt(h)->num_pages; }
int lle_pt_num_free(void* h) { return (int)pt(h)->free_list.size(); }
int lle_pt_is_held(void* h, int page) {
    PageTables* t = pt(h);
    return page >= 0 && page < t->num_pages && t->held[page];
}

// n pages from the top of the stack into out[0..n)
int lle_pt_allocate(void* h, int n, int32_t* out) {
    PageTables* t = pt(h);
    if (n < 0) return LLE_HOST_BAD_ARGUMENT;
    if (n > (int)t->free_list.size()) return LLE_HOST_OUT_OF_PAGES;
    for (int i = 0; i < n; ++i) {
        const int32_t page = t->free_list.back();
        t->free_list.pop_back();
        t->held[page] = 1;
        out[i] = page;
    }
    return LLE_HOST_OK;
}

// pages[0..n) back onto the stack, in this order; *bad names the page that is refused
int lle_pt_release(void* h, const int32_t* pages, int n, int32_t* bad) {
    PageTables* t = pt(h);
    std::vector<uint8_t> seen(t->num_pages, 0);
    for (int i = 0; i < n; ++i) {
        const int32_t p = pages[i];
        if (p < 0 || p >= t->num_pages) {
            *bad = p;
            return LLE_HOST_NO_SUCH_PAGE;
        }
        if (!t->held[p] || seen[p]) {
            *bad = p;
            return LLE_HOST_FREED_TWICE;
        }
        seen[p] = 1;
    }
    for (int i = 0; i < n; ++i) t->give_back(pages[i]);
    return LLE_HOST_OK;
}

int lle_pt_table_len(void* h, int slot) { return (int)pt(h)->tables[slot].size(); }
void lle_pt_table_copy(void* h, int slot, int32_t* out) {
    const std::vector<int32_t>& table = pt(h)->tables[slot];
    std::copy(table.begin(), table.end(), out);
}
int lle_pt_first_live(void* h, int slot) { return pt(h)->first_live[slot]; }
int lle_pt_new_pages_needed(void* h, int slot, int new_len) { return pt(h)->new_pages_needed(slot, new_len); }

// pages for positions < new_len of the slot's request: all of them or none
int lle_pt_grow(void* h, int slot, int new_len) {
    PageTables* t = pt(h);
    const int need = t->new_pages_needed(slot, new_len);
    if (need == 0) return LLE_HOST_OK;
    std::vector<int32_t>& table = t->tables[slot];
    if ((int)table.size() + need > t->max_pages_per_request) return LLE_HOST_TOO_MANY_PAGES;
    if (need > (int)t->free_list.size()) return LLE_HOST_OUT_OF_PAGES;
    for (int i = 0; i < need; ++i) {
        const int32_t page = t->free_list.back();
        t->free_list.pop_back();
        t->held[page] = 1;
        t->pending_index.push_back(slot * t->max_pages_per_request + (int)table.size());
        t->pending_page.push_back(page);
        table.push_back(page);
    }
    return LLE_HOST_OK;
}

// The same for n requests at once.  lle_pt_pages_needed_many: the pages that growing all of them
// takes, or -1 if one of them would hold more than a request may.  lle_pt_grow_many: all of
// them grow or none does.
int lle_pt_pages_needed_many(void* h, int n, const int32_t* slots, const int32_t* new_lens) {
    PageTables* t = pt(h);
    int total = 0;
    for (int i = 0; i < n; ++i) {
        const int need = t->new_pages_needed(slots[i], new_lens[i]);
        if ((int)t->tables[slots[i]].size() + need > t->max_pages_per_request) return -1;
        total += need;
    }
    return total;
}

int lle_pt_grow_many(void* h, int n, const int32_t* slots, const int32_t* new_lens) {
    PageTables* t = pt(h);
    const int total = lle_pt_pages_needed_many(h, n, slots, new_lens);
    if (total < 0) return LLE_HOST_TOO_MANY_PAGES;
    if (total > (int)t->free_list.size()) return LLE_HOST_OUT_OF_PAGES;
    for (int i = 0; i < n; ++i) lle_pt_grow(h, slots[i], new_lens[i]);
    return LLE_HOST_OK;
}

// A step that did not happen after all: the pages beyond those of `length` positions go back, last
// taken first (after lle_pt_grow_many and lle_pt_shrink_many with the lengths of before, the stack
// is what it was), and what was noted for the device table about them is dropped.
void lle_pt_shrink(void* h, int slot, int length) {
    PageTables* t = pt(h);
    std::vector<int32_t>& table = t->tables[slot];
    const int keep = std::max(t->pages_for(std::max(length, 0)), t->first_live[slot]);
    if ((int)table.size() <= keep) return;
    while ((int)table.size() > keep) {
        if (table.back() >= 0) t->give_back(table.back());
        table.pop_back();
    }
    const int row = slot * t->max_pages_per_request;
    size_t out = 0;
    for (size_t i = 0; i < t->pending_index.size(); ++i) {
        const int32_t at = t->pending_index[i];
        if (at >= row + keep && at < row + t->max_pages_per_request) continue;
        t->pending_index[out] = at;
        t->pending_page[out] = t->pending_page[i];
        ++out;
    }
    t->pending_index.resize(out);
    t->pending_page.resize(out);
}

void lle_pt_shrink_many(void* h, int n, const int32_t* slots, const int32_t* lengths) {
    for (int i = n - 1; i >= 0; --i) lle_pt_shrink(h, slots[i], lengths[i]);
}

// With a window w the next query (position `length`) sees keys >= length - w + 1: the pages
// before that one's are given back.
void lle_pt_trim(void* h, int slot, int length) {
    PageTables* t = pt(h);
    if (t->window < 0) return;
    const int first_needed = std::max(0, length - t->window + 1) / t->page_size;
    std::vector<int32_t>& table = t->tables[slot];
    const int first = t->first_live[slot];
    if (first_needed > first) {
        const int last = std::min(first_needed, (int)table.size());
        for (int i = first; i < last; ++i) {
            t->give_back(table[i]);
            table[i] = -1;
        }
        t->first_live[slot] = last;
    }
}

void lle_pt_trim_many(void* h, int n, const int32_t* slots, const int32_t* lengths) {
    if (pt(h)->window < 0) return;
    for (int i = 0; i < n; ++i) lle_pt_trim(h, slots[i], lengths[i]);
}

// everything the slot's request holds, in table order (the last page is used again first)
void lle_pt_release_slot(void* h, int slot) {
    PageTables* t = pt(h);
    std::vector<int32_t>& table = t->tables[slot];
    for (size_t i = (size_t)t->first_live[slot]; i < table.size(); ++i) t->give_back(table[i]);
    table.clear();
    t->first_live[slot] = 0;
}

// page * P + offset of position `pos`; -1: no page there, -2: its page was given back
int64_t lle_pt_token_slot(void* h, int slot, int pos) {
    PageTables* t = pt(h);
    const std::vector<int32_t>& table = t->tables[slot];
    const int lp = pos / t->page_size;
    if (pos < 0 || lp >= (int)table.size()) return -1;
    if (table[lp] < 0) return -2;
    return (int64_t)table[lp] * t->page_size + pos % t->page_size;
}

int lle_pt_num_pending(void* h) { return (int)pt(h)->pending_index.size(); }
void lle_pt_take_pending(void* h, int32_t* index, int32_t* pages) {
    PageTables* t = pt(h);
    std::copy(t->pending_index.begin(), t->pending_index.end(), index);
    std::copy(t->pending_page.begin(), t->pending_page.end(), pages);
    t->pending_index.clear();
    t->pending_page.clear();
}

// The integer arrays of a step.  S requests: cache slot, tokens already cached (past) and
// tokens in this step (q_len) of each; `tokens` the N = sum(q_len) token ids in order;
// `logit_rows` the R rows (indices into the N) whose logits are wanted; G cache groups.
// out: token ids [N], positions [N], request of each token [N], slots [S], first row of each
// request and N [S + 1], cached length after the step [S], wanted rows [R], then for every group
// the page slot of every token [N].  *info: the offending index when a code is returned.
//
// `pad` > 0 appends that many requests that stand for nobody (a batch padded to a size for which a
// graph exists): one token each (id 0, position 0, cached length 1), block-table row `pad_slot`
// (a row that points at a page nobody writes), page slot -1 (nothing is written).  The sizes above
// then count them: N + pad tokens, S + pad requests; `logit_rows` may name their rows.
int lle_layout_step(int S, const int32_t* slots, const int32_t* past, const int32_t* q_len, const int32_t* tokens,
                    int vocab_size, int allow_deferred, int R, const int32_t* logit_rows, int G, void* const* groups,
                    int pad, int pad_slot, int32_t* out, int64_t* info) {
    // (no request at all is allowed when the batch is padding only: the warm-up of a graph's kernels)
    if (S < 0 || (S == 0 && pad <= 0) || R < 0 || G < 0 || pad < 0 || (pad > 0 && pad_slot < 0)) return LLE_HOST_BAD_ARGUMENT;
    int64_t N = 0;
    for (int s = 0; s < S; ++s) {
        if (q_len[s] <= 0 || past[s] < 0) {
            *info = s;
            return LLE_HOST_BAD_ARGUMENT;
        }
        N += q_len[s];
    }
    // (with `allow_deferred` an id of -1 stands for a token that is still on the device: the one the
    // step before picked for this request)
    for (int64_t i = 0; i < N; ++i)
        if ((tokens[i] < 0 && !(allow_deferred && tokens[i] == -1)) || (vocab_size > 0 && tokens[i] >= vocab_size)) {
            *info = i;
            return LLE_HOST_BAD_TOKEN;
        }
    for (int r = 0; r < R; ++r)
        if (logit_rows[r] < 0 || logit_rows[r] >= N + pad) {
            *info = r;
            return LLE_HOST_BAD_ARGUMENT;
        }
    // every position of the step has a page in every group (checked before anything is written)
    for (int g = 0; g < G; ++g) {
        const PageTables* t = pt(groups[g]);
        for (int s = 0; s < S; ++s) {
            const std::vector<int32_t>& table = t->tables[slots[s]];
            const int first = past[s] / t->page_size, last = (past[s] + q_len[s] - 1) / t->page_size;
            for (int lp = first; lp <= last; ++lp)
                if (lp >= (int)table.size() || table[lp] < 0) {
                    *info = (int64_t)lp * t->page_size;
                    return LLE_HOST_NO_PAGE_AT_POSITION;
                }
        }
    }
    const int64_t NP = N + pad;
    const int SP = S + pad;
    int32_t* token_ids = out;
    int32_t* positions = token_ids + NP;
    int32_t* token_seq = positions + NP;
    int32_t* seq_slots = token_seq + NP;
    int32_t* cu_tokens = seq_slots + SP;
    int32_t* kv_lens = cu_tokens + SP + 1;
    int32_t* rows = kv_lens + SP;
    int32_t* mapping = rows + R;
    std::copy(tokens, tokens + N, token_ids);
    int64_t at = 0;
    for (int s = 0; s < S; ++s) {
        seq_slots[s] = slots[s];
        cu_tokens[s] = (int32_t)at;
        kv_lens[s] = past[s] + q_len[s];
        for (int i = 0; i < q_len[s]; ++i) {
            positions[at + i] = past[s] + i;
            token_seq[at + i] = s;
        }
        at += q_len[s];
    }
    for (int i = 0; i < pad; ++i) {
        token_ids[N + i] = 0;
        positions[N + i] = 0;
        token_seq[N + i] = S + i;
        seq_slots[S + i] = pad_slot;
        cu_tokens[S + i] = (int32_t)(N + i);
        kv_lens[S + i] = 1;
    }
    cu_tokens[SP] = (int32_t)NP;
    std::copy(logit_rows, logit_rows + R, rows);
    for (int g = 0; g < G; ++g) {
        const PageTables* t = pt(groups[g]);
        const int P = t->page_size;
        int32_t* m = mapping + (int64_t)g * NP;
        at = 0;
        for (int s = 0; s < S; ++s) {
            const std::vector<int32_t>& table = t->tables[slots[s]];
            for (int i = 0; i < q_len[s]; ++i) {
                const int pos = past[s] + i;
                m[at + i] = table[pos / P] * P + pos % P;
            }
            at += q_len[s];
        }
        for (int i = 0; i < pad; ++i) m[N + i] = -1;
    }
    return LLE_HOST_OK;
}

}  // extern "C"
