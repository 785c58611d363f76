// Cache manager: pages of keys/values with one block table per request and
// group of layers, and slots of fixed-size per-request state.
//
// The reference keeps one table per request PER LAYER and a single pool
// (/root/reference/include/runtime/pagekvcache.h:10-45,
//  /root/reference/src/runtime/block_manager.cu:39-99,
//  /root/reference/src/runtime/real_kv_allocator.cu:112-177).
// Here a page id is shared by all layers of a group, groups with different needs
// (all keys, or a window of them) own separate pools, and a window group gives
// pages back as soon as the window has passed them.
#pragma once

#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace minillm {

struct GroupSpec {
    int page_size = 16;   // tokens per page
    int n_pages = 0;      // pages in this group's pool
    int window = 0;       // 0: every earlier key is kept; W>0: only the last W keys are needed
};

class PagePool {
public:
    PagePool() = default;
    explicit PagePool(int n_pages);
    int n_pages() const { return static_cast<int>(is_free_.size()); }
    int n_free() const { return static_cast<int>(free_.size()); }
    // Returns a page id, or -1 when none is free.
    int take();
    // Returns false (and changes nothing) for a bad id or a page that is already free.
    bool give_back(int page);
    bool is_free(int page) const { return page >= 0 && page < n_pages() && is_free_[page]; }

private:
    std::vector<int> free_;        // LIFO: a page given back is the next one handed out
    std::vector<uint8_t> is_free_;
};

struct RequestCache {
    int64_t id = -1;
    int length = 0;                          // tokens whose keys/values (or state) are committed
    int reserved = 0;                        // tokens that pages have been taken for (>= length)
    int state_slot = -1;
    std::vector<std::vector<int>> tables;    // [group][logical block] -> page id, -1 if released/not yet held
    std::vector<int> first_live;             // [group] first logical block that may still be held
};

class CacheManager {
public:
    CacheManager(const std::vector<GroupSpec>& groups, int n_state_slots);

    int n_groups() const { return static_cast<int>(groups_.size()); }
    const GroupSpec& group(int g) const { return groups_[g]; }
    int free_pages(int g) const { return pools_[g].n_free(); }
    int total_pages(int g) const { return pools_[g].n_pages(); }
    int free_state_slots() const { return static_cast<int>(free_slots_.size()); }
    int n_requests() const { return static_cast<int>(requests_.size()); }

    // Registers a request and assigns its state slot. Returns the slot (>= 0),
    // -1 if no slot is free, -2 if the id is already known.
    int add_request(int64_t id);
    bool has_request(int64_t id) const { return requests_.count(id) != 0; }

    // Pages that a request holding `length` committed tokens must newly take in
    // group g so that positions [length, new_len) can be written and attended from.
    int pages_needed(int64_t id, int g, int new_len) const;
    // Same for a request that is not registered yet (length 0).
    int pages_needed_fresh(int g, int new_len) const;
    bool can_reserve(int64_t id, int new_len) const;

    // Takes the pages for positions [length, new_len) in every group; all or nothing.
    // Returns 0, -1 if some group has too few free pages, -2 for an unknown id or a
    // new_len below the committed length.
    int reserve(int64_t id, int new_len);

    // Marks positions below new_len as written (new_len <= reserved) and gives back
    // the pages that every later query's window has passed. Returns 0 or -2.
    int commit(int64_t id, int new_len);

    // Gives back everything the request holds. Returns the number of pages freed, -2 if unknown.
    int free_request(int64_t id);

    int length(int64_t id) const;
    int state_slot(int64_t id) const;
    // Copies the block table of group g (released entries are -1). Returns the number
    // of logical blocks, or -2 for an unknown id. At most `cap` entries are written.
    int block_table(int64_t id, int g, int* out, int cap) const;

    // Index arrays of a step in which request ids[i] feeds n_tokens[i] tokens from its committed
    // length on. Tokens are laid out request after request. Returns 0, or -(i+1) if request i is
    // unknown.
    int fill_step_common(const int64_t* ids, const int* n_tokens, int n, int* positions, int* token_seq,
                         int* cu_q, int* starts, int* ctx_len, int* state_slots) const;
    // For one group: tables[i*max_blocks ..] = block table of request i (entries beyond it 0), and
    // slots[t] = page*page_size + offset of every token. Returns 0, or -(i+1) if request i is unknown,
    // holds no page for one of its tokens, or has more than max_blocks blocks.
    int fill_step_group(const int64_t* ids, const int* n_tokens, int n, int g, int max_blocks, int* tables,
                        int* slots) const;

    // Consistency check: every page is either free or held by exactly one
    // (request, group, block); every slot likewise. Empty string when consistent.
    std::string check() const;

private:
    int first_needed_block(int g, int from_pos) const;

    std::vector<GroupSpec> groups_;
    std::vector<PagePool> pools_;
    std::vector<int> free_slots_;
    std::vector<uint8_t> slot_free_;
    std::unordered_map<int64_t, RequestCache> requests_;
};

}  // namespace minillm
