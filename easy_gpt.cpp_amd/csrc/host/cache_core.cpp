// See cache_core.h.  Plain C++17, no GPU code: it is compiled with the host compiler and tested on the CPU.
#include "cache_core.h"

#include <algorithm>
#include <cstdio>
#include <vector>

namespace {

struct Pool {
    int num_pages = 0;
    int high_water = 0;
    int in_use = 0;
    std::vector<int32_t> free;      // a stack: pages freed last go out first, so that reuse happens early
    std::vector<uint8_t> held;      // per page: taken and not given back

    void init(int n) {
        num_pages = n;
        free.resize(n);
        for (int i = 0; i < n; ++i) free[i] = n - 1 - i;      // page 0 goes out first
        held.assign(n, 0);
    }
    int32_t take() {
        const int32_t p = free.back();
        free.pop_back();
        held[p] = 1;
        ++in_use;
        high_water = std::max(high_water, in_use);
        return p;
    }
    bool give_back(int32_t p) {
        if (p < 0 || p >= num_pages || !held[p]) return false;
        held[p] = 0;
        --in_use;
        free.push_back(p);
        return true;
    }
};

struct Request {
    bool live = false;
    int slot = -1;
    int num_tokens = 0;
    int version = 0;
    std::vector<std::vector<int32_t>> tables;    // per group: page ids in token order, -1 = given back
};

}  // namespace

struct EghCore {
    int page_size = 1;
    std::vector<int> windows;
    std::vector<Pool> pools;
    std::vector<int32_t> free_slots;
    std::vector<uint8_t> slot_held;
    std::vector<Request> requests;
    std::vector<int> free_handles;

    const Request* get(int h) const {
        return (h >= 0 && h < static_cast<int>(requests.size()) && requests[h].live) ? &requests[h] : nullptr;
    }
    Request* get(int h) { return const_cast<Request*>(static_cast<const EghCore*>(this)->get(h)); }
    int n_groups() const { return static_cast<int>(pools.size()); }
    int pages_for(int tokens) const { return (tokens + page_size - 1) / page_size; }
};

extern "C" {

int egh_abi_version(void) { return 3; }

EghCore* egh_create(int n_groups, const int32_t* windows, const int32_t* num_pages, int page_size, int max_requests) {
    if (n_groups < 0 || page_size < 1 || max_requests < 0 || (n_groups > 0 && (!windows || !num_pages))) return nullptr;
    for (int g = 0; g < n_groups; ++g)
        if (num_pages[g] < 0 || windows[g] < 0) return nullptr;
    EghCore* c = new EghCore();
    c->page_size = page_size;
    c->windows.assign(windows, windows + n_groups);
    c->pools.resize(n_groups);
    for (int g = 0; g < n_groups; ++g) c->pools[g].init(num_pages[g]);
    c->free_slots.resize(max_requests);
    for (int i = 0; i < max_requests; ++i) c->free_slots[i] = max_requests - 1 - i;
    c->slot_held.assign(max_requests, 0);
    return c;
}

void egh_destroy(EghCore* c) { delete c; }

int egh_admit(EghCore* c) {
    if (!c) return EGH_BAD_ARGUMENT;
    if (c->free_slots.empty()) return EGH_NO_SLOT;
    int h;
    if (!c->free_handles.empty()) {
        h = c->free_handles.back();
        c->free_handles.pop_back();
    } else {
        h = static_cast<int>(c->requests.size());
        c->requests.emplace_back();
    }
    Request& r = c->requests[h];
    r.live = true;
    r.slot = c->free_slots.back();
    c->free_slots.pop_back();
    c->slot_held[r.slot] = 1;
    r.num_tokens = 0;
    r.version += 1;            // a handle that is used again is another request: cached rows must not match
    r.tables.assign(c->n_groups(), {});
    return h;
}

int egh_release(EghCore* c, int h) {
    Request* r = c ? c->get(h) : nullptr;
    if (!r) return EGH_BAD_HANDLE;
    for (int g = 0; g < c->n_groups(); ++g) {
        for (int32_t p : r->tables[g])
            if (p >= 0 && !c->pools[g].give_back(p)) return EGH_INVARIANT;
        r->tables[g].clear();
    }
    c->slot_held[r->slot] = 0;
    c->free_slots.push_back(r->slot);
    r->live = false;
    r->version += 1;
    c->free_handles.push_back(h);
    return EGH_OK;
}

int egh_slot(const EghCore* c, int h) { const Request* r = c ? c->get(h) : nullptr; return r ? r->slot : EGH_BAD_HANDLE; }
int egh_num_tokens(const EghCore* c, int h) { const Request* r = c ? c->get(h) : nullptr; return r ? r->num_tokens : EGH_BAD_HANDLE; }
int egh_version(const EghCore* c, int h) { const Request* r = c ? c->get(h) : nullptr; return r ? r->version : EGH_BAD_HANDLE; }

int egh_table_len(const EghCore* c, int h, int g) {
    const Request* r = c ? c->get(h) : nullptr;
    if (!r) return EGH_BAD_HANDLE;
    if (g < 0 || g >= c->n_groups()) return EGH_BAD_ARGUMENT;
    return static_cast<int>(r->tables[g].size());
}

int egh_table(const EghCore* c, int h, int g, int32_t* out, int cap) {
    const Request* r = c ? c->get(h) : nullptr;
    if (!r) return EGH_BAD_HANDLE;
    if (g < 0 || g >= c->n_groups() || !out) return EGH_BAD_ARGUMENT;
    const int n = std::min<int>(cap, static_cast<int>(r->tables[g].size()));
    std::copy(r->tables[g].begin(), r->tables[g].begin() + n, out);
    return n;
}

int egh_pages_needed(const EghCore* c, int h, int n_new, int32_t* out) {
    const Request* r = c ? c->get(h) : nullptr;
    if (!r) return EGH_BAD_HANDLE;
    if (n_new < 0 || !out) return EGH_BAD_ARGUMENT;
    const int want = c->pages_for(r->num_tokens + n_new);
    for (int g = 0; g < c->n_groups(); ++g) out[g] = std::max(0, want - static_cast<int>(r->tables[g].size()));
    return EGH_OK;
}

int egh_free_pages(const EghCore* c, int g) { return (c && g >= 0 && g < c->n_groups()) ? static_cast<int>(c->pools[g].free.size()) : EGH_BAD_ARGUMENT; }
int egh_used_pages(const EghCore* c, int g) { return (c && g >= 0 && g < c->n_groups()) ? c->pools[g].in_use : EGH_BAD_ARGUMENT; }
int egh_num_pages(const EghCore* c, int g) { return (c && g >= 0 && g < c->n_groups()) ? c->pools[g].num_pages : EGH_BAD_ARGUMENT; }
int egh_high_water(const EghCore* c, int g) { return (c && g >= 0 && g < c->n_groups()) ? c->pools[g].high_water : EGH_BAD_ARGUMENT; }
int egh_free_slots(const EghCore* c) { return c ? static_cast<int>(c->free_slots.size()) : EGH_BAD_ARGUMENT; }

int egh_reserve(EghCore* c, int n, const int32_t* handles, const int32_t* counts, int32_t* detail) {
    if (!c || n < 0 || (n > 0 && (!handles || !counts))) return EGH_BAD_ARGUMENT;
    const int ng = c->n_groups();
    // first count, then take: nothing is taken unless everything fits
    std::vector<int> promised(ng, 0);
    for (int i = 0; i < n; ++i) {
        const Request* r = c->get(handles[i]);
        if (!r) return EGH_BAD_HANDLE;
        if (counts[i] < 0) return EGH_BAD_ARGUMENT;
        const int want = c->pages_for(r->num_tokens + counts[i]);
        for (int g = 0; g < ng; ++g) {
            const int need = std::max(0, want - static_cast<int>(r->tables[g].size()));
            const int free_now = static_cast<int>(c->pools[g].free.size()) - promised[g];
            if (need > free_now) {
                if (detail) {
                    detail[0] = i; detail[1] = g; detail[2] = need; detail[3] = free_now;
                }
                return EGH_OUT_OF_PAGES;
            }
            promised[g] += need;
        }
    }
    for (int i = 0; i < n; ++i) {
        Request* r = c->get(handles[i]);
        const int want = c->pages_for(r->num_tokens + counts[i]);
        for (int g = 0; g < ng; ++g) {
            const int need = std::max(0, want - static_cast<int>(r->tables[g].size()));
            for (int j = 0; j < need; ++j) r->tables[g].push_back(c->pools[g].take());
            if (need) r->version += 1;
        }
    }
    return EGH_OK;
}

int egh_unreserve(EghCore* c, int n, const int32_t* handles) {
    if (!c || n < 0 || (n > 0 && !handles)) return EGH_BAD_ARGUMENT;
    for (int i = 0; i < n; ++i)
        if (!c->get(handles[i])) return EGH_BAD_HANDLE;
    // in the reverse of the order in which egh_reserve took them, so that the free lists are as before it
    for (int i = n - 1; i >= 0; --i) {
        Request* r = c->get(handles[i]);
        const int keep = c->pages_for(r->num_tokens);
        for (int g = c->n_groups() - 1; g >= 0; --g) {
            std::vector<int32_t>& table = r->tables[g];
            bool changed = false;
            while (static_cast<int>(table.size()) > keep) {
                const int32_t p = table.back();
                if (p >= 0 && !c->pools[g].give_back(p)) return EGH_INVARIANT;
                table.pop_back();
                changed = true;
            }
            if (changed) r->version += 1;
        }
    }
    return EGH_OK;
}

int egh_commit(EghCore* c, int n, const int32_t* handles, const int32_t* counts) {
    if (!c || n < 0 || (n > 0 && (!handles || !counts))) return EGH_BAD_ARGUMENT;
    const int ng = c->n_groups();
    for (int i = 0; i < n; ++i) {
        Request* r = c->get(handles[i]);
        if (!r) return EGH_BAD_HANDLE;
        if (counts[i] < 0) return EGH_BAD_ARGUMENT;
        const int total = r->num_tokens + counts[i];
        for (int g = 0; g < ng; ++g)
            if (c->pages_for(total) > static_cast<int>(r->tables[g].size())) return EGH_NO_PAGE;   // commit without reserve
        r->num_tokens = total;
        for (int g = 0; g < ng; ++g) {
            const int window = c->windows[g];
            if (window <= 0) continue;
            // the next token (position num_tokens) reads keys j > num_tokens - window
            const int first_needed = r->num_tokens - window + 1;
            const int dead = std::max(0, first_needed) / c->page_size;        // pages wholly below first_needed
            bool changed = false;
            for (int j = 0; j < dead; ++j) {
                int32_t& p = r->tables[g][j];
                if (p >= 0) {
                    if (!c->pools[g].give_back(p)) return EGH_INVARIANT;
                    p = -1;
                    changed = true;
                }
            }
            if (changed) r->version += 1;
        }
    }
    return EGH_OK;
}

int egh_slot_index(const EghCore* c, int h, int g, int position) {
    const Request* r = c ? c->get(h) : nullptr;
    if (!r) return EGH_BAD_HANDLE;
    if (g < 0 || g >= c->n_groups() || position < 0) return EGH_BAD_ARGUMENT;
    const int idx = position / c->page_size;
    if (idx >= static_cast<int>(r->tables[g].size()) || r->tables[g][idx] < 0) return EGH_NO_PAGE;
    return r->tables[g][idx] * c->page_size + position % c->page_size;
}

int egh_check(const EghCore* c, char* message, int cap) {
    if (!c) return EGH_BAD_ARGUMENT;
    auto fail = [&](const char* what, int g) {
        if (message && cap > 0) std::snprintf(message, cap, "group %d: %s", g, what);
        return EGH_INVARIANT;
    };
    for (int g = 0; g < c->n_groups(); ++g) {
        const Pool& pool = c->pools[g];
        if (static_cast<int>(pool.free.size()) + pool.in_use != pool.num_pages) return fail("a page was lost", g);
        std::vector<uint8_t> seen(pool.num_pages, 0);
        for (int32_t p : pool.free) {
            if (p < 0 || p >= pool.num_pages) return fail("a free page id is out of range", g);
            if (seen[p]) return fail("a page is on the free list twice", g);
            if (pool.held[p]) return fail("a page is both free and in use", g);
            seen[p] = 1;
        }
        std::vector<uint8_t> in_table(pool.num_pages, 0);
        int held = 0;
        for (const Request& r : c->requests) {
            if (!r.live) continue;
            for (int32_t p : r.tables[g]) {
                if (p < 0) continue;
                if (p >= pool.num_pages) return fail("a table holds a page id out of range", g);
                if (in_table[p]) return fail("a page is in two block tables", g);
                if (!pool.held[p]) return fail("block tables and pool disagree", g);
                in_table[p] = 1;
                ++held;
            }
        }
        if (held != pool.in_use) return fail("block tables and pool disagree", g);
    }
    const int n_slots = static_cast<int>(c->slot_held.size());
    std::vector<uint8_t> slot_seen(n_slots, 0);
    int live = 0;
    for (const Request& r : c->requests) {
        if (!r.live) continue;
        ++live;
        if (r.slot < 0 || r.slot >= n_slots || slot_seen[r.slot] || !c->slot_held[r.slot])
            return fail("a slot is held by two requests or by none", -1);
        slot_seen[r.slot] = 1;
    }
    if (live + static_cast<int>(c->free_slots.size()) != n_slots) return fail("a slot was lost", -1);
    return EGH_OK;
}

int egh_fill_decode_rows(const EghCore* c, int b, int rows, const int32_t* handles, const int32_t* widths,
                         int32_t* small, int32_t* tab, int64_t* row_state) {
    if (!c || b <= 0 || rows < b || !handles || !small || !row_state || (c->n_groups() > 0 && (!widths || !tab)))
        return EGH_BAD_ARGUMENT;
    const int ng = c->n_groups(), ps = c->page_size;
    int changed = 0;
    size_t tab_off = 0;
    for (int i = 0; i < b; ++i) {
        const Request* r = c->get(handles[i]);
        if (!r) return EGH_BAD_HANDLE;
        const int pos = r->num_tokens;
        small[1 * rows + i] = pos;
        small[2 * rows + i] = i;
        small[3 * rows + i] = 1;
        small[4 * rows + i] = pos + 1;
        small[5 * rows + i] = r->slot;
        small[6 * rows + i] = i;
        for (int g = 0; g < ng; ++g) {
            const std::vector<int32_t>& t = r->tables[g];
            const int idx = pos / ps;
            if (idx >= static_cast<int>(t.size()) || t[idx] < 0) return EGH_NO_PAGE;
            if (static_cast<int>(t.size()) > widths[g]) return EGH_BAD_ARGUMENT;
            small[(7 + g) * rows + i] = t[idx] * ps + pos % ps;
        }
    }
    for (int g = 0; g < ng; ++g) {
        for (int i = 0; i < b; ++i) {
            const Request* r = c->get(handles[i]);
            if (row_state[2 * i] != handles[i] || row_state[2 * i + 1] != r->version) {
                const std::vector<int32_t>& t = r->tables[g];
                int32_t* row = tab + tab_off + static_cast<size_t>(i) * widths[g];
                std::copy(t.begin(), t.end(), row);
                std::fill(row + t.size(), row + widths[g], -1);
                changed = 1;
            }
        }
        tab_off += static_cast<size_t>(rows) * widths[g];
    }
    for (int i = 0; i < b; ++i) {
        row_state[2 * i] = handles[i];
        row_state[2 * i + 1] = c->get(handles[i])->version;
    }
    return changed;
}

int egh_fill_decode(const EghCore* c, int b, const int32_t* handles, const int32_t* widths, int32_t* small,
                    int32_t* tab, int64_t* row_state) {
    return egh_fill_decode_rows(c, b, b, handles, widths, small, tab, row_state);
}

int egh_fill_step(const EghCore* c, int b, const int32_t* handles, const int32_t* counts, const int32_t* widths,
                  int32_t* positions, int32_t* q_start, int32_t* q_len, int32_t* kv_len, int32_t* state_slots,
                  int32_t* slots, int32_t* tables) {
    if (!c || b <= 0 || !handles || !counts || !positions || !q_start || !q_len || !kv_len || !state_slots ||
        (c->n_groups() > 0 && (!widths || !slots || !tables)))
        return EGH_BAD_ARGUMENT;
    const int ng = c->n_groups(), ps = c->page_size;
    long total = 0;
    for (int i = 0; i < b; ++i) {
        if (counts[i] < 1) return EGH_BAD_ARGUMENT;
        total += counts[i];
    }
    int start = 0;
    size_t tab_off = 0;
    for (int i = 0; i < b; ++i) {
        const Request* r = c->get(handles[i]);
        if (!r) return EGH_BAD_HANDLE;
        q_start[i] = start;
        q_len[i] = counts[i];
        kv_len[i] = r->num_tokens + counts[i];
        state_slots[i] = r->slot;
        for (int j = 0; j < counts[i]; ++j) positions[start + j] = r->num_tokens + j;
        start += counts[i];
    }
    for (int g = 0; g < ng; ++g) {
        for (int i = 0; i < b; ++i) {
            const Request* r = c->get(handles[i]);
            const std::vector<int32_t>& t = r->tables[g];
            if (static_cast<int>(t.size()) > widths[g]) return EGH_BAD_ARGUMENT;
            int32_t* row = tables + tab_off + static_cast<size_t>(i) * widths[g];
            std::copy(t.begin(), t.end(), row);
            std::fill(row + t.size(), row + widths[g], -1);
            for (int j = 0; j < counts[i]; ++j) {
                const int pos = r->num_tokens + j, idx = pos / ps;
                if (idx >= static_cast<int>(t.size()) || t[idx] < 0) return EGH_NO_PAGE;   // a page that was given back
                slots[static_cast<size_t>(g) * total + q_start[i] + j] = t[idx] * ps + pos % ps;
            }
        }
        tab_off += static_cast<size_t>(b) * widths[g];
    }
    return EGH_OK;
}

}  // extern "C"
