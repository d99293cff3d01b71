#include "cache.h"

#include <algorithm>
#include <stdexcept>

namespace spite {

CacheManager::CacheManager(int page_size, int max_requests, const std::vector<GroupSpec>& groups)
    : page_size_(page_size), groups_(groups) {
    if (page_size < 1) throw std::invalid_argument("page_size must be >= 1");
    if (max_requests < 1) throw std::invalid_argument("max_requests must be >= 1");
    for (const auto& g : groups_) {
        if (g.n_pages < 1) throw std::invalid_argument("every group needs at least one page");
        if (g.kind < 0 || g.kind >= SP_VIS_COUNT) throw std::invalid_argument("unknown visibility");
        if (sp_vis_has_span(g.kind) && g.span < 1) throw std::invalid_argument("chunk or window must be >= 1");
    }
    free_.resize(groups_.size());
    for (size_t g = 0; g < groups_.size(); ++g) {
        // page 0 on top of the stack
        for (int p = groups_[g].n_pages - 1; p >= 0; --p) free_[g].push_back(p);
    }
    slots_.resize(max_requests);
    for (auto& s : slots_) {
        s.table.resize(groups_.size());
        s.freed_below.assign(groups_.size(), 0);
    }
    for (int i = max_requests - 1; i >= 0; --i) free_slots_.push_back(i);
    fresh_.assign(max_requests, 0);
}

int CacheManager::admit() {
    if (free_slots_.empty()) return -1;
    int s = free_slots_.back();
    free_slots_.pop_back();
    Slot& sl = slots_[s];
    sl.live = true;
    sl.cached = sl.reserved = 0;
    for (size_t g = 0; g < groups_.size(); ++g) {
        sl.table[g].clear();
        sl.freed_below[g] = 0;
    }
    fresh_[s] = 1;
    return s;
}

int CacheManager::take_fresh(int* out, int cap) {
    int n = 0;
    for (int s = 0; s < (int)fresh_.size(); ++s) {
        if (!fresh_[s]) continue;
        if (n < cap) out[n] = s;
        ++n;
        fresh_[s] = 0;
    }
    return n;
}

bool CacheManager::live(int slot) const {
    return slot >= 0 && slot < (int)slots_.size() && slots_[slot].live;
}

int64_t CacheManager::cached(int slot) const { return live(slot) ? slots_[slot].cached : -1; }

int CacheManager::pages_needed(int slot, int64_t n, int g) const {
    const Slot& sl = slots_[slot];
    const int64_t end = sl.cached + n;
    const int64_t blocks = (end + page_size_ - 1) / page_size_;
    const int64_t have = (int64_t)sl.table[g].size();
    return blocks > have ? (int)(blocks - have) : 0;
}

bool CacheManager::can_reserve(int slot, int64_t n) const {
    if (!live(slot) || n < 0) return false;
    for (int g = 0; g < n_groups(); ++g)
        if (pages_needed(slot, n, g) > free_pages(g)) return false;
    return true;
}

bool CacheManager::can_reserve_new(int64_t n) const {
    const int64_t blocks = (n + page_size_ - 1) / page_size_;
    for (int g = 0; g < n_groups(); ++g)
        if (blocks > free_pages(g)) return false;
    return true;
}

int CacheManager::reserve(int slot, int64_t n) {
    if (!live(slot) || n < 0) return -2;
    if (!can_reserve(slot, n)) return -1;
    Slot& sl = slots_[slot];
    for (int g = 0; g < n_groups(); ++g) {
        int need = pages_needed(slot, n, g);
        for (int i = 0; i < need; ++i) {
            sl.table[g].push_back(free_[g].back());
            free_[g].pop_back();
        }
    }
    sl.reserved = std::max(sl.reserved, sl.cached + n);
    return 0;
}

int CacheManager::reserve_all(int n, const int* slots, const int64_t* counts) {
    std::vector<int64_t> need(groups_.size(), 0);
    for (int i = 0; i < n; ++i) {
        if (!live(slots[i]) || counts[i] < 0) return -2;
        for (int j = 0; j < i; ++j)
            if (slots[j] == slots[i]) return -2;           // a slot twice: the sums below would be wrong
        for (int g = 0; g < n_groups(); ++g) need[g] += pages_needed(slots[i], counts[i], g);
    }
    for (int g = 0; g < n_groups(); ++g)
        if (need[g] > free_pages(g)) return -1;
    for (int i = 0; i < n; ++i) reserve(slots[i], counts[i]);
    return 0;
}

int CacheManager::commit(int slot, int64_t n) {
    if (!live(slot) || n < 0) return -2;
    Slot& sl = slots_[slot];
    if (sl.cached + n > sl.reserved) return -3;
    sl.cached += n;
    // The next query sits at position `cached`; no later one reads below its first key.
    for (int g = 0; g < n_groups(); ++g) {
        const int64_t frontier = first_visible(sl.cached, groups_[g].kind, groups_[g].span);
        const int64_t upto = std::min<int64_t>(frontier / page_size_, (int64_t)sl.table[g].size());
        for (int64_t b = sl.freed_below[g]; b < upto; ++b) {
            int& page = sl.table[g][b];
            if (page >= 0) { free_[g].push_back(page); page = -1; }
        }
        sl.freed_below[g] = std::max(sl.freed_below[g], upto);
    }
    return 0;
}

int CacheManager::release(int slot) {
    if (!live(slot)) return -2;
    Slot& sl = slots_[slot];
    for (int g = 0; g < n_groups(); ++g) {
        // highest block first, so that the request's first page is handed out first again
        for (auto it = sl.table[g].rbegin(); it != sl.table[g].rend(); ++it)
            if (*it >= 0) free_[g].push_back(*it);
        sl.table[g].clear();
        sl.freed_below[g] = 0;
    }
    sl.live = false;
    sl.cached = sl.reserved = 0;
    free_slots_.push_back(slot);
    return 0;
}

int64_t CacheManager::peak_pages(int64_t total, int64_t portion, int g) const {
    const int64_t ps = page_size_;
    const int64_t back = sp_vis_lookback(groups_[g].kind, groups_[g].span);
    if (back < 0 || portion < 1) return (total + ps - 1) / ps;
    // A portion of n positions that starts at c reads from first_visible(c), at most `back`
    // positions before c.  Portions start anywhere (the budget cuts them), so take the worst
    // alignment; chunks that are whole pages start on a page.
    const int64_t all = (total + ps - 1) / ps;
    const int64_t n = std::min(portion, total);
    int64_t worst;
    if (groups_[g].kind == SP_VIS_CHUNK && groups_[g].span % ps == 0) worst = (back + n + ps - 1) / ps;
    else worst = (back + n - 1) / ps + 2;
    return std::min(all, worst);
}

void CacheManager::slot_mapping(int slot, int g, int64_t start, int64_t n, int32_t* out) const {
    const auto& tab = slots_[slot].table[g];
    for (int64_t i = 0; i < n; ++i) {
        const int64_t pos = start + i, b = pos / page_size_;
        const int page = b < (int64_t)tab.size() ? tab[b] : -1;
        out[i] = page < 0 ? -1 : (int32_t)((int64_t)page * page_size_ + pos % page_size_);
    }
}

int CacheManager::fill_step(int n, const int32_t* slots, const int32_t* starts, const int32_t* counts, int g,
                            int width, int32_t* slot_map, int32_t* table) const {
    int64_t off = 0;
    for (int i = 0; i < n; ++i) {
        if (!live(slots[i])) return -2;
        const auto& tab = slots_[slots[i]].table[g];
        if ((int)tab.size() > width) return -4;
        slot_mapping(slots[i], g, starts[i], counts[i], slot_map + off);
        off += counts[i];
        int32_t* row = table + (int64_t)i * width;
        for (int b = 0; b < width; ++b) row[b] = b < (int)tab.size() ? tab[b] : -1;
    }
    return 0;
}

std::string CacheManager::check() const {
    for (int g = 0; g < n_groups(); ++g) {
        std::vector<int> seen(groups_[g].n_pages, 0);
        for (int p : free_[g]) {
            if (p < 0 || p >= groups_[g].n_pages) return "free list holds a page out of range";
            if (seen[p]++) return "page " + std::to_string(p) + " of group " + std::to_string(g) + " is free twice";
        }
        for (size_t s = 0; s < slots_.size(); ++s) {
            if (!slots_[s].live) {
                if (!slots_[s].table[g].empty()) return "a slot that is not live holds pages";
                continue;
            }
            for (int p : slots_[s].table[g]) {
                if (p < 0) continue;
                if (p >= groups_[g].n_pages) return "table holds a page out of range";
                if (seen[p]++) return "page " + std::to_string(p) + " of group " + std::to_string(g) + " is held twice";
            }
        }
        for (int p = 0; p < groups_[g].n_pages; ++p)
            if (!seen[p]) return "page " + std::to_string(p) + " of group " + std::to_string(g) + " is lost";
    }
    std::vector<int> sl(slots_.size(), 0);
    for (int s : free_slots_) if (sl[s]++) return "slot free twice";
    for (size_t s = 0; s < slots_.size(); ++s)
        if (slots_[s].live == (sl[s] != 0)) return "slot " + std::to_string(s) + " is both live and free, or neither";
    return "";
}

}  // namespace spite
