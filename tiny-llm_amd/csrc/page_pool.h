// Host-side bookkeeping of a fixed pool of KV pages and of the sequence slots that hold them: free list, per-slot page lists,
// transactional reservation, reuse counters.  No device memory is touched here: the owner mirrors `table` to the device.
#pragma once
#include <algorithm>
#include <cstdint>
#include <vector>

namespace tl {

struct PagePoolStats {
    int pages_in_use = 0, peak_pages_in_use = 0;
    long page_allocations = 0, reused_page_allocations = 0;
    long slot_begins = 0, reused_slot_begins = 0;
};

class PagePool {
public:
    PagePool(int num_pages, int page_size, int max_slots, int max_pages_per_seq)
        : page_size_(page_size), max_pages_per_seq_(max_pages_per_seq), free_(num_pages), was_used_(num_pages, 0), pages_(max_slots),
          ctx_(max_slots, 0), live_(max_slots, 0), slot_used_(max_slots, 0), table_((size_t)max_slots * max_pages_per_seq, -1) {
        for (int i = 0; i < num_pages; ++i) free_[i] = num_pages - 1 - i;  // pop_back hands out 0, 1, 2, ...
    }
    int slots() const { return (int)live_.size(); }
    int page_size() const { return page_size_; }
    int max_pages_per_seq() const { return max_pages_per_seq_; }
    bool live(int slot) const { return live_[slot] != 0; }
    int context(int slot) const { return ctx_[slot]; }
    void advance(int slot, int n) { ctx_[slot] += n; }
    int free_pages() const { return (int)free_.size(); }
    const std::vector<int32_t> &table() const { return table_; }
    const PagePoolStats &stats() const { return stats_; }

    void begin(int slot) {
        live_[slot] = 1;
        ctx_[slot] = 0;
        stats_.slot_begins++;
        if (slot_used_[slot]) stats_.reused_slot_begins++;
        slot_used_[slot] = 1;
    }
    // pages needed beyond what the slot holds to reach total_tokens; -1 if the block-table row is too short
    int missing(int slot, int total_tokens) const {
        const int need = (total_tokens + page_size_ - 1) / page_size_;
        if (need > max_pages_per_seq_) return -1;
        return std::max(0, need - (int)pages_[slot].size());
    }
    // call only after the sum of missing() over a step's slots has been checked against free_pages(); returns true if the table changed
    bool reserve(int slot, int total_tokens) {
        const int need = (total_tokens + page_size_ - 1) / page_size_;
        bool changed = false;
        while ((int)pages_[slot].size() < need) {
            const int id = free_.back();
            free_.pop_back();
            stats_.page_allocations++;
            if (was_used_[id]) stats_.reused_page_allocations++;
            was_used_[id] = 1;
            stats_.pages_in_use++;
            stats_.peak_pages_in_use = std::max(stats_.peak_pages_in_use, stats_.pages_in_use);
            table_[(size_t)slot * max_pages_per_seq_ + pages_[slot].size()] = id;
            pages_[slot].push_back(id);
            changed = true;
        }
        return changed;
    }
    // the sequence of `src` changes hands to the free slot `dst`: page list, context; no page moves
    void move(int src, int dst) {
        pages_[dst].swap(pages_[src]);
        pages_[src].clear();
        for (int j = 0; j < max_pages_per_seq_; ++j) {
            table_[(size_t)dst * max_pages_per_seq_ + j] = table_[(size_t)src * max_pages_per_seq_ + j];
            table_[(size_t)src * max_pages_per_seq_ + j] = -1;
        }
        ctx_[dst] = ctx_[src];
        ctx_[src] = 0;
        live_[dst] = 1;
        live_[src] = 0;
        slot_used_[dst] = 1;
    }
    void release(int slot) {
        for (int id : pages_[slot]) {
            free_.push_back(id);
            stats_.pages_in_use--;
        }
        for (size_t j = 0; j < pages_[slot].size(); ++j) table_[(size_t)slot * max_pages_per_seq_ + j] = -1;
        pages_[slot].clear();
        live_[slot] = 0;
        ctx_[slot] = 0;
    }

private:
    int page_size_, max_pages_per_seq_;
    std::vector<int> free_;
    std::vector<char> was_used_;
    std::vector<std::vector<int>> pages_;
    std::vector<int> ctx_;
    std::vector<char> live_, slot_used_;
    std::vector<int32_t> table_;
    PagePoolStats stats_;
};

}  // namespace tl
