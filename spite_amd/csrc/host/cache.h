// Cache manager: pages of keys and values with a block table for each request and each
// group of layers, and slots for per-request state of fixed size.
//
// A group is a set of layers with the same need: every key (full), the keys of the chunk
// that the query lies in (chunk, size C), or the last W keys (window).  Each group has a
// pool of pages of its own.  A page holds `page_size` consecutive positions of one request
// for all layers of the group.  The free list is a stack, as in the reference's BlockPool
// (crates/spite-kvcache/src/paged.rs:55,89-93), so a page that is given back is the next one
// handed out.
//
// Life of a request: admit() -> slot; then for every step reserve(slot, n) (pages for the
// next n positions; fails without changing anything when a pool is short), the kernels run,
// commit(slot, n) (the positions are now cached; pages that no later query can read are
// given back and their table entries become -1); finally release(slot).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#define SP_VIS_FN inline
#include "../visibility.h"

namespace spite {


struct GroupSpec {
    int kind;      // Visibility
    int span;      // chunk size or window; unused for full
    int n_pages;   // pool size
};

// First position that a query at position p may read: the rule shared with the attention kernels.
inline int64_t first_visible(int64_t p, int kind, int span) { return sp_first_visible<int64_t>(p, kind, span); }

class CacheManager {
public:
    CacheManager(int page_size, int max_requests, const std::vector<GroupSpec>& groups);

    int page_size() const { return page_size_; }
    int n_groups() const { return (int)groups_.size(); }
    int max_requests() const { return (int)slots_.size(); }
    int free_pages(int g) const { return (int)free_[g].size(); }
    int total_pages(int g) const { return groups_[g].n_pages; }
    int free_slots() const { return (int)free_slots_.size(); }

    int admit();                               // slot id, or -1 when every slot is taken
    // Slots handed out since the last call, in ascending order, each once however often it was
    // admitted and released meanwhile (never more than max_requests): whoever keeps per-request
    // state on the GPU clears the rows of these slots before the next step runs, whichever
    // caller admitted them.  Returns how many there were; at most `cap` are written.
    int take_fresh(int* out, int cap);
    bool live(int slot) const;
    int64_t cached(int slot) const;            // positions committed
    // Pages that reserve(slot, n) would take from group g's pool.
    int pages_needed(int slot, int64_t n, int g) const;
    bool can_reserve(int slot, int64_t n) const;
    // As can_reserve for a request that is not admitted yet and holds nothing.
    bool can_reserve_new(int64_t n) const;
    int reserve(int slot, int64_t n);          // 0; -1 out of pages (nothing changed); -2 bad slot
    // reserve() for several slots at once: every one of them gets its pages, or nothing changes
    // (-1 out of pages, -2 a slot that is not live or named twice).
    int reserve_all(int n, const int* slots, const int64_t* counts);
    int commit(int slot, int64_t n);           // 0; -2 bad slot; -3 more than was reserved
    int release(int slot);                     // 0; -2 bad slot
    // Pages that a request of `total` positions holds at most at one time in group g, when
    // it is fed in portions of at most `portion` positions.
    int64_t peak_pages(int64_t total, int64_t portion, int g) const;

    const std::vector<int>& table(int slot, int g) const { return slots_[slot].table[g]; }
    // Cache rows (page * page_size + offset) of positions [start, start+n); -1 where no page.
    void slot_mapping(int slot, int g, int64_t start, int64_t n, int32_t* out) const;
    // For the n entries (slot, first position, count) of a step: the cache rows of all their
    // tokens in a row in `slot_map`, and one block-table row of `width` entries each in `table`
    // (-1 past a table's end).  -2: a slot is not live; -4: a table is wider than `width`.
    int fill_step(int n, const int32_t* slots, const int32_t* starts, const int32_t* counts, int g, int width,
                  int32_t* slot_map, int32_t* table) const;
    // 0 when every page is either free or in exactly one table, once; else a message.
    std::string check() const;

private:
    struct Slot {
        bool live = false;
        int64_t cached = 0;
        int64_t reserved = 0;                  // positions with pages, >= cached
        std::vector<std::vector<int>> table;   // [group][logical block] -> page or -1
        std::vector<int64_t> freed_below;      // [group] logical blocks below this are given back
    };
    int page_size_;
    std::vector<GroupSpec> groups_;
    std::vector<std::vector<int>> free_;       // [group] stack of free pages
    std::vector<Slot> slots_;
    std::vector<int> free_slots_;              // stack, lowest id on top at the start
    std::vector<char> fresh_;                  // [slot] admitted and not yet reported by take_fresh
};

}  // namespace spite
