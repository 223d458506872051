// Random sequences of operations on the cache manager's C++ core, with the invariants checked after every one and
// the metadata functions run on exact-size buffers: built with the host compiler's address and undefined-behaviour
// sanitizers by tests/test_host_core_sanitized.py, so that a write past a buffer or a stale index stops the run.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "cache_core.h"

#define REQUIRE(cond)                                                                  \
    do {                                                                               \
        if (!(cond)) {                                                                 \
            std::printf("FAILED %s:%d: %s (seed %u, op %d)\n", __FILE__, __LINE__, #cond, seed, op); \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

struct Live {
    int handle;
    int tokens;
};

int main(int argc, char** argv) {
    const unsigned n_seeds = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 20;
    long total_ops = 0;
    for (unsigned seed = 0; seed < n_seeds; ++seed) {
        int op = -1;
        std::mt19937 rng(seed);
        auto pick = [&](int lo, int hi) { return lo + static_cast<int>(rng() % static_cast<unsigned>(hi - lo + 1)); };
        const int n_groups = pick(1, 3), page_size = (const int[]){1, 3, 4, 16, 64}[pick(0, 4)], max_requests = pick(1, 6);
        std::vector<int32_t> windows(n_groups), num_pages(n_groups);
        for (int g = 0; g < n_groups; ++g) {
            windows[g] = pick(0, 1) ? pick(1, 90) : 0;
            num_pages[g] = pick(4, 60);
        }
        EghCore* c = egh_create(n_groups, windows.data(), num_pages.data(), page_size, max_requests);
        REQUIRE(c != nullptr);
        std::vector<Live> live;
        char message[256];
        for (op = 0; op < 600; ++op, ++total_ops) {
            const int what = pick(0, 99);
            if (what < 15) {
                const int h = egh_admit(c);
                if (static_cast<int>(live.size()) < max_requests) {
                    REQUIRE(h >= 0);
                    live.push_back({h, 0});
                } else {
                    REQUIRE(h == EGH_NO_SLOT);
                }
            } else if (what < 80 && !live.empty()) {
                // a step of some of the live requests: reserve all or nothing, fill the metadata, commit
                std::vector<int> chosen;
                for (int i = 0; i < static_cast<int>(live.size()); ++i)
                    if (pick(0, 1)) chosen.push_back(i);
                if (chosen.empty()) chosen.push_back(pick(0, static_cast<int>(live.size()) - 1));
                const int b = static_cast<int>(chosen.size());
                std::vector<int32_t> handles(b), counts(b);
                const bool single = pick(0, 2) == 0;
                int total = 0;
                for (int i = 0; i < b; ++i) {
                    handles[i] = live[chosen[i]].handle;
                    counts[i] = single ? 1 : (const int[]){1, 1, 2, 5, 17, 40}[pick(0, 5)];
                    total += counts[i];
                }
                std::vector<int32_t> free_before(n_groups);
                for (int g = 0; g < n_groups; ++g) free_before[g] = egh_free_pages(c, g);
                int32_t detail[4] = {-1, -1, -1, -1};
                const int r = egh_reserve(c, b, handles.data(), counts.data(), detail);
                if (r == EGH_OUT_OF_PAGES) {
                    for (int g = 0; g < n_groups; ++g) REQUIRE(egh_free_pages(c, g) == free_before[g]);   // nothing taken
                    REQUIRE(detail[0] >= 0 && detail[0] < b && detail[1] >= 0 && detail[1] < n_groups);
                } else {
                    REQUIRE(r == EGH_OK);
                    std::vector<int32_t> widths(n_groups);
                    int tab_size = 0;
                    for (int g = 0; g < n_groups; ++g) {
                        int w = 1;
                        for (int i = 0; i < b; ++i) w = std::max(w, egh_table_len(c, handles[i], g));
                        widths[g] = w;
                        tab_size += b * w;
                    }
                    std::vector<int32_t> positions(total), q_start(b), q_len(b), kv_len(b), state_slots(b),
                        slots(static_cast<size_t>(n_groups) * total), tables(tab_size);
                    REQUIRE(egh_fill_step(c, b, handles.data(), counts.data(), widths.data(), positions.data(), q_start.data(),
                                          q_len.data(), kv_len.data(), state_slots.data(), slots.data(), tables.data()) == EGH_OK);
                    int t = 0;
                    for (int i = 0; i < b; ++i) {
                        REQUIRE(q_start[i] == t && q_len[i] == counts[i] && kv_len[i] == live[chosen[i]].tokens + counts[i]);
                        for (int j = 0; j < counts[i]; ++j, ++t) {
                            REQUIRE(positions[t] == live[chosen[i]].tokens + j);
                            for (int g = 0; g < n_groups; ++g) {
                                const int s = slots[static_cast<size_t>(g) * total + t];
                                REQUIRE(s == egh_slot_index(c, handles[i], g, positions[t]));
                                REQUIRE(s >= 0 && s < num_pages[g] * page_size);
                            }
                        }
                    }
                    if (single) {
                        std::vector<int32_t> small(static_cast<size_t>(7 + n_groups) * b, -7), tab(tab_size, -7);
                        std::vector<int64_t> row_state(2 * static_cast<size_t>(b), -1);
                        REQUIRE(egh_fill_decode(c, b, handles.data(), widths.data(), small.data(), tab.data(), row_state.data()) == 1);
                        REQUIRE(egh_fill_decode(c, b, handles.data(), widths.data(), small.data(), tab.data(), row_state.data()) == 0);
                        for (int i = 0; i < b; ++i) REQUIRE(small[1 * b + i] == positions[i] && small[4 * b + i] == kv_len[i]);
                        for (int i = 0; i < tab_size; ++i) REQUIRE(tab[i] == tables[i]);
                    }
                    if (pick(0, 6) == 0) {
                        // the step fails: what it reserved goes back and the pools are as before
                        REQUIRE(egh_unreserve(c, b, handles.data()) == EGH_OK);
                        for (int g = 0; g < n_groups; ++g) REQUIRE(egh_free_pages(c, g) == free_before[g]);
                        for (int i = 0; i < b; ++i) REQUIRE(egh_num_tokens(c, handles[i]) == live[chosen[i]].tokens);
                    } else {
                        REQUIRE(egh_commit(c, b, handles.data(), counts.data()) == EGH_OK);
                        for (int i = 0; i < b; ++i) {
                            live[chosen[i]].tokens += counts[i];
                            REQUIRE(egh_num_tokens(c, handles[i]) == live[chosen[i]].tokens);
                        }
                    }
                }
            } else if (!live.empty()) {
                const int i = pick(0, static_cast<int>(live.size()) - 1);
                REQUIRE(egh_release(c, live[i].handle) == EGH_OK);
                REQUIRE(egh_release(c, live[i].handle) != EGH_OK);            // twice is refused
                live.erase(live.begin() + i);
            }
            if (egh_check(c, message, sizeof(message)) != EGH_OK) {
                std::printf("FAILED invariant: %s (seed %u, op %d)\n", message, seed, op);
                return 1;
            }
            // handles that are not live are refused everywhere
            REQUIRE(egh_num_tokens(c, 1000 + op) < 0 && egh_slot(c, -1) < 0);
        }
        for (const Live& l : live) REQUIRE(egh_release(c, l.handle) == EGH_OK);
        for (int g = 0; g < n_groups; ++g) REQUIRE(egh_free_pages(c, g) == num_pages[g] && egh_used_pages(c, g) == 0);
        REQUIRE(egh_free_slots(c) == max_requests);
        egh_destroy(c);
    }
    std::printf("ok: %u seeds, %ld operations\n", n_seeds, total_ops);
    return 0;
}
