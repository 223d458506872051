// The cache manager's bookkeeping and the packing of a step's metadata, in C++ behind a C ABI.
//
// Pages of keys and values with a block table per request and group; groups with a window give pages
// back as a request advances; request slots for per-request state of fixed size.  No device memory is
// touched here: the caller hands in host buffers (pinned, for the engine) that these functions fill.
// The reference keeps per-sample contiguous caches and a stack of free slots
// (/root/reference/src/continuous_batch_server.cpp:44-47,243-248); this is what replaces them.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct EghCore EghCore;

enum { EGH_OK = 0, EGH_NO_SLOT = -1, EGH_BAD_HANDLE = -2, EGH_OUT_OF_PAGES = -3, EGH_BAD_ARGUMENT = -4,
       EGH_NO_PAGE = -5, EGH_INVARIANT = -6 };

int egh_abi_version(void);
// windows[g] == 0: the group keeps every key.  num_pages[g] pages of page_size tokens; max_requests slots.
EghCore* egh_create(int n_groups, const int32_t* windows, const int32_t* num_pages, int page_size, int max_requests);
void egh_destroy(EghCore* c);

int egh_admit(EghCore* c);                                  // a handle >= 0, or EGH_NO_SLOT
int egh_release(EghCore* c, int h);                         // pages and slot go back
int egh_slot(const EghCore* c, int h);
int egh_num_tokens(const EghCore* c, int h);
int egh_version(const EghCore* c, int h);                   // changes whenever a table of the request changes
int egh_table_len(const EghCore* c, int h, int g);
int egh_table(const EghCore* c, int h, int g, int32_t* out, int cap);   // entries written; -1 = page given back
int egh_pages_needed(const EghCore* c, int h, int n_new, int32_t* out);  // per group
int egh_free_pages(const EghCore* c, int g);
int egh_used_pages(const EghCore* c, int g);
int egh_num_pages(const EghCore* c, int g);
int egh_high_water(const EghCore* c, int g);
int egh_free_slots(const EghCore* c);

// Gives back the pages that egh_reserve took for tokens that were never committed (a step that failed between the
// two): every request keeps the pages of its committed tokens.
int egh_unreserve(EghCore* c, int n, const int32_t* handles);

// Pages for the next counts[i] tokens of each request, in every group: all of them or none.
// On EGH_OUT_OF_PAGES detail = {index of the request, group, pages it needs there, free pages there}.
int egh_reserve(EghCore* c, int n, const int32_t* handles, const int32_t* counts, int32_t* detail);
// The tokens are now part of the requests; pages wholly behind a window go back.
int egh_commit(EghCore* c, int n, const int32_t* handles, const int32_t* counts);
// page * page_size + offset of the token at `position`, or EGH_NO_PAGE
int egh_slot_index(const EghCore* c, int h, int g, int position);

// Invariants: no page lost, free twice or in two tables; tables and pools agree; slots likewise.
int egh_check(const EghCore* c, char* message, int cap);

// ---- metadata of a step, written where the caller says (int32 everywhere)
// One token per request (request i's token is token i).  small = 7 + n_groups rows of b entries:
//   0 token ids (left alone)   1 positions   2 q_start = i   3 q_len = 1   4 kv_len   5 state slots
//   6 wanted rows = i   7 + g: the new token's slot in group g
// tab: per group [b][widths[g]] block tables, rows rewritten only when row_state (2 per row: handle, version)
// says they changed.  Returns 1 if a table row was rewritten, 0 if not, < 0 on error.
int egh_fill_decode(const EghCore* c, int b, const int32_t* handles, const int32_t* widths, int32_t* small,
                    int32_t* tab, int64_t* row_state);
// The same into buffers laid out for `rows` >= b requests (a batch padded to a size that a graph exists for): the
// first b entries of every row of `small` and the first b table rows of every group are written, the rest is the
// caller's.
int egh_fill_decode_rows(const EghCore* c, int b, int rows, const int32_t* handles, const int32_t* widths,
                         int32_t* small, int32_t* tab, int64_t* row_state);
// Any mix: counts[i] tokens per request, token-major outputs of T = sum counts entries (positions, slots per
// group [n_groups][T]), per-request outputs of b entries, tables per group [b][widths[g]] concatenated.
int egh_fill_step(const EghCore* c, int b, const int32_t* handles, const int32_t* counts, const int32_t* widths,
                  int32_t* positions, int32_t* q_start, int32_t* q_len, int32_t* kv_len, int32_t* state_slots,
                  int32_t* slots, int32_t* tables);

#ifdef __cplusplus
}
#endif
