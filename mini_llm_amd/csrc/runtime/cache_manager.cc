#include "cache_manager.h"

#include <algorithm>
#include <sstream>

namespace minillm {

PagePool::PagePool(int n_pages) : is_free_(n_pages, 1) {
    free_.reserve(n_pages);
    // Highest id at the bottom so that page 0 is handed out first.
    for (int p = n_pages - 1; p >= 0; --p) free_.push_back(p);
}

int PagePool::take() {
    if (free_.empty()) return -1;
    int p = free_.back();
    free_.pop_back();
    is_free_[p] = 0;
    return p;
}

bool PagePool::give_back(int page) {
    if (page < 0 || page >= n_pages() || is_free_[page]) return false;
    is_free_[page] = 1;
    free_.push_back(page);
    return true;
}

CacheManager::CacheManager(const std::vector<GroupSpec>& groups, int n_state_slots)
    : groups_(groups), slot_free_(n_state_slots, 1) {
    for (const auto& g : groups_) pools_.emplace_back(g.n_pages);
    for (int s = n_state_slots - 1; s >= 0; --s) free_slots_.push_back(s);
}

int CacheManager::add_request(int64_t id) {
    if (requests_.count(id)) return -2;
    if (free_slots_.empty()) return -1;
    int slot = free_slots_.back();
    free_slots_.pop_back();
    slot_free_[slot] = 0;
    RequestCache rc;
    rc.id = id;
    rc.state_slot = slot;
    rc.tables.resize(groups_.size());
    rc.first_live.assign(groups_.size(), 0);
    requests_.emplace(id, std::move(rc));
    return slot;
}

int CacheManager::first_needed_block(int g, int from_pos) const {
    const GroupSpec& gs = groups_[g];
    if (gs.window <= 0) return 0;
    int first_key = std::max(0, from_pos - gs.window + 1);
    return first_key / gs.page_size;
}

int CacheManager::pages_needed_fresh(int g, int new_len) const {
    const GroupSpec& gs = groups_[g];
    return (new_len + gs.page_size - 1) / gs.page_size;
}

int CacheManager::pages_needed(int64_t id, int g, int new_len) const {
    auto it = requests_.find(id);
    if (it == requests_.end()) return pages_needed_fresh(g, new_len);
    const RequestCache& rc = it->second;
    const GroupSpec& gs = groups_[g];
    int last = (new_len + gs.page_size - 1) / gs.page_size;   // one past the last block
    int first = first_needed_block(g, rc.length);
    const auto& tab = rc.tables[g];
    int need = 0;
    for (int b = first; b < last; ++b) {
        if (b >= static_cast<int>(tab.size()) || tab[b] < 0) ++need;
    }
    return need;
}

bool CacheManager::can_reserve(int64_t id, int new_len) const {
    for (int g = 0; g < n_groups(); ++g) {
        if (pages_needed(id, g, new_len) > pools_[g].n_free()) return false;
    }
    return true;
}

int CacheManager::reserve(int64_t id, int new_len) {
    auto it = requests_.find(id);
    if (it == requests_.end()) return -2;
    RequestCache& rc = it->second;
    if (new_len < rc.length) return -2;
    if (!can_reserve(id, new_len)) return -1;
    for (int g = 0; g < n_groups(); ++g) {
        const GroupSpec& gs = groups_[g];
        int last = (new_len + gs.page_size - 1) / gs.page_size;
        int first = first_needed_block(g, rc.length);
        auto& tab = rc.tables[g];
        if (static_cast<int>(tab.size()) < last) tab.resize(last, -1);
        for (int b = first; b < last; ++b) {
            if (tab[b] < 0) tab[b] = pools_[g].take();
        }
    }
    rc.reserved = std::max(rc.reserved, new_len);
    return 0;
}

int CacheManager::commit(int64_t id, int new_len) {
    auto it = requests_.find(id);
    if (it == requests_.end()) return -2;
    RequestCache& rc = it->second;
    if (new_len < rc.length || new_len > rc.reserved) return -2;
    rc.length = new_len;
    for (int g = 0; g < n_groups(); ++g) {
        const GroupSpec& gs = groups_[g];
        if (gs.window <= 0) continue;
        // The next query stands at position new_len and needs keys >= new_len - window + 1.
        int first_key = std::max(0, new_len - gs.window + 1);
        int keep_from = first_key / gs.page_size;
        auto& tab = rc.tables[g];
        int upto = std::min(keep_from, static_cast<int>(tab.size()));
        for (int b = rc.first_live[g]; b < upto; ++b) {
            if (tab[b] >= 0) {
                pools_[g].give_back(tab[b]);
                tab[b] = -1;
            }
        }
        rc.first_live[g] = std::max(rc.first_live[g], upto);
    }
    return 0;
}

int CacheManager::free_request(int64_t id) {
    auto it = requests_.find(id);
    if (it == requests_.end()) return -2;
    RequestCache& rc = it->second;
    int freed = 0;
    for (int g = 0; g < n_groups(); ++g) {
        for (int p : rc.tables[g]) {
            if (p >= 0 && pools_[g].give_back(p)) ++freed;
        }
    }
    slot_free_[rc.state_slot] = 1;
    free_slots_.push_back(rc.state_slot);
    requests_.erase(it);
    return freed;
}

int CacheManager::length(int64_t id) const {
    auto it = requests_.find(id);
    return it == requests_.end() ? -2 : it->second.length;
}

int CacheManager::state_slot(int64_t id) const {
    auto it = requests_.find(id);
    return it == requests_.end() ? -2 : it->second.state_slot;
}

int CacheManager::block_table(int64_t id, int g, int* out, int cap) const {
    auto it = requests_.find(id);
    if (it == requests_.end() || g < 0 || g >= n_groups()) return -2;
    const auto& tab = it->second.tables[g];
    int n = static_cast<int>(tab.size());
    for (int b = 0; b < n && b < cap; ++b) out[b] = tab[b];
    return n;
}

int CacheManager::fill_step_common(const int64_t* ids, const int* n_tokens, int n, int* positions,
                                   int* token_seq, int* cu_q, int* starts, int* ctx_len, int* state_slots) const {
    int t = 0;
    cu_q[0] = 0;
    for (int i = 0; i < n; ++i) {
        auto it = requests_.find(ids[i]);
        if (it == requests_.end()) return -(i + 1);
        const RequestCache& rc = it->second;
        starts[i] = rc.length;
        ctx_len[i] = rc.length + n_tokens[i];
        state_slots[i] = rc.state_slot;
        for (int k = 0; k < n_tokens[i]; ++k, ++t) {
            positions[t] = rc.length + k;
            token_seq[t] = i;
        }
        cu_q[i + 1] = t;
    }
    return 0;
}

int CacheManager::fill_step_group(const int64_t* ids, const int* n_tokens, int n, int g, int max_blocks,
                                  int* tables, int* slots) const {
    if (g < 0 || g >= n_groups()) return -1;
    const int ps = groups_[g].page_size;
    int t = 0;
    for (int i = 0; i < n; ++i) {
        auto it = requests_.find(ids[i]);
        if (it == requests_.end()) return -(i + 1);
        const RequestCache& rc = it->second;
        const auto& tab = rc.tables[g];
        const int nb = static_cast<int>(tab.size());
        if (nb > max_blocks) return -(i + 1);
        int* row = tables + static_cast<size_t>(i) * max_blocks;
        for (int b = 0; b < nb; ++b) row[b] = tab[b];
        for (int b = nb; b < max_blocks; ++b) row[b] = 0;
        for (int k = 0; k < n_tokens[i]; ++k, ++t) {
            const int pos = rc.length + k;
            const int blk = pos / ps;
            if (blk >= nb || tab[blk] < 0) return -(i + 1);
            slots[t] = tab[blk] * ps + pos % ps;
        }
    }
    return 0;
}

std::string CacheManager::check() const {
    std::ostringstream err;
    for (int g = 0; g < n_groups(); ++g) {
        std::vector<int> held(pools_[g].n_pages(), 0);
        for (const auto& kv : requests_) {
            for (int p : kv.second.tables[g]) {
                if (p < 0) continue;
                if (p >= pools_[g].n_pages()) {
                    err << "group " << g << ": request " << kv.first << " holds bad page " << p << "; ";
                    continue;
                }
                ++held[p];
            }
        }
        int n_free = 0;
        for (int p = 0; p < pools_[g].n_pages(); ++p) {
            bool f = pools_[g].is_free(p);
            n_free += f;
            if (held[p] > 1) err << "group " << g << ": page " << p << " held " << held[p] << " times; ";
            if (held[p] >= 1 && f) err << "group " << g << ": page " << p << " is held and free; ";
            if (held[p] == 0 && !f) err << "group " << g << ": page " << p << " is lost; ";
        }
        if (n_free != pools_[g].n_free())
            err << "group " << g << ": free list has " << pools_[g].n_free() << " entries, bitmap " << n_free << "; ";
    }
    std::vector<int> slot_held(slot_free_.size(), 0);
    for (const auto& kv : requests_) {
        int s = kv.second.state_slot;
        if (s < 0 || s >= static_cast<int>(slot_free_.size())) {
            err << "request " << kv.first << " has bad slot " << s << "; ";
            continue;
        }
        ++slot_held[s];
    }
    for (size_t s = 0; s < slot_free_.size(); ++s) {
        if (slot_held[s] > 1) err << "slot " << s << " held twice; ";
        if (slot_held[s] == 1 && slot_free_[s]) err << "slot " << s << " held and free; ";
        if (slot_held[s] == 0 && !slot_free_[s]) err << "slot " << s << " lost; ";
    }
    return err.str();
}

}  // namespace minillm
