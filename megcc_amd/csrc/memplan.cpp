// Static memory plan for a fixed operator sequence: every intermediate tensor is an interval
// (first operator that writes it, one past the last operator that reads it, bytes), and the plan
// gives each interval an offset into one arena so that intervals alive at the same time never
// share bytes.
//
// The result is the one MegCC's compiler computes with its PUSHDOWN allocator
// (compiler/lib/Dialect/Kernel/Transforms/migrate/static_mem_alloc.h:26 selected at
// Transforms/StaticMemoryPlanning.cpp:35; algorithm in static_mem_alloc/pushdown.cpp and the
// event order of static_mem_alloc/best_fit_helper.cpp:7-38), so a model planned here has the same
// arena size and the same offsets as the same model compiled by the reference. Two steps:
//
//   1. ORDER. Walk the time steps in ascending order; at each step first release the intervals
//      that end there, then place the ones that begin there (both in the order they were added).
//      Placement is a best fit over a row of blocks (each either one live interval or a hole):
//      the smallest hole that is large enough, the oldest one among equals. When no hole is large
//      enough the LARGEST hole (the youngest among equals) is stretched to the size asked for -
//      everything above it simply moves up - and only when there is no hole at all a new block is
//      appended at the top. What is kept from this step is not an address but, for every
//      interval, which live interval sat directly under it and which directly above it at the
//      moment it was placed.
//   2. PUSH DOWN. Those "sits on top of" relations form a DAG. The offset of an interval is the
//      largest end offset of the intervals under it, rounded up to the alignment; the arena size
//      is the largest aligned end offset.
//
// The reference's "overwrite" requests (an interval that may reuse the bytes of one that dies in
// the same step) are not part of this plan: its memory-planning pass never issues them
// (StaticMemoryPlanning.cpp:95 only calls add()).
#include <cstddef>
#include <cstdint>
#include <map>
#include <utility>
#include <vector>

#include "memplan.h"

namespace mg {
namespace {

// Row of blocks kept as an index-linked list so that handles stay valid across edits.
class BlockRow {
public:
    static constexpr int NIL = -1;

    struct Neighbours {
        int under = NIL, above = NIL;  // interval ids
    };

    // places `interval` (of `size` bytes) and reports the live intervals around it
    Neighbours place(int interval, size_t size) {
        int blk;
        if (holes_.empty()) {
            blk = new_block();
            link_before(NIL, blk);
        } else {
            auto it = holes_.lower_bound(HoleKey{size, 0});
            if (it == holes_.end()) {
                --it;  // largest, youngest: stretch it
                blocks_[it->second].size = size;
            }
            blk = it->second;
            holes_.erase(it);
            const size_t rest = blocks_[blk].size - size;
            blocks_[blk].interval = interval;
            add_hole_before(blocks_[blk].next, rest);
        }
        blocks_[blk].interval = interval;
        blocks_[blk].size = size;
        where_[interval] = blk;

        Neighbours r;
        int p = blocks_[blk].prev;
        if (p != NIL && blocks_[p].interval == NIL)
            p = blocks_[p].prev;
        if (p != NIL)
            r.under = blocks_[p].interval;
        int q = blocks_[blk].next;
        if (q != NIL && blocks_[q].interval == NIL)
            q = blocks_[q].next;
        if (q != NIL)
            r.above = blocks_[q].interval;
        return r;
    }

    void release(int interval) {
        const int blk = where_.at(interval);
        where_.erase(interval);
        const int after = blocks_[blk].next;
        const size_t size = blocks_[blk].size;
        unlink(blk);
        add_hole_before(after, size);
    }

private:
    struct Block {
        int prev = NIL, next = NIL;
        int interval = NIL;  // NIL: hole
        size_t size = 0;
        uint64_t serial = 0;  // holes only: creation order
    };
    using HoleKey = std::pair<size_t, uint64_t>;  // (size, serial)

    std::vector<Block> blocks_;
    std::vector<int> spare_;
    int head_ = NIL, tail_ = NIL;
    uint64_t next_serial_ = 1;  // 0 is reserved for "before every hole of this size"
    std::map<HoleKey, int> holes_;
    std::map<int, int> where_;  // live interval -> block

    int new_block() {
        if (!spare_.empty()) {
            const int b = spare_.back();
            spare_.pop_back();
            blocks_[b] = Block();
            return b;
        }
        blocks_.emplace_back();
        return (int)blocks_.size() - 1;
    }

    // pos == NIL: append at the top
    void link_before(int pos, int blk) {
        Block& b = blocks_[blk];
        b.next = pos;
        b.prev = pos == NIL ? tail_ : blocks_[pos].prev;
        if (b.prev == NIL)
            head_ = blk;
        else
            blocks_[b.prev].next = blk;
        if (pos == NIL)
            tail_ = blk;
        else
            blocks_[pos].prev = blk;
    }

    void unlink(int blk) {
        Block& b = blocks_[blk];
        if (b.prev == NIL)
            head_ = b.next;
        else
            blocks_[b.prev].next = b.next;
        if (b.next == NIL)
            tail_ = b.prev;
        else
            blocks_[b.next].prev = b.prev;
        spare_.push_back(blk);
    }

    void drop_hole(int blk) {
        holes_.erase(HoleKey{blocks_[blk].size, blocks_[blk].serial});
        unlink(blk);
    }

    // A hole of `size` bytes in front of block `pos` (NIL: at the top); holes that would touch
    // it are swallowed, so two holes are never adjacent. The result is always a NEW hole (it
    // takes the youngest serial), and no hole at all when there is nothing to hold.
    void add_hole_before(int pos, size_t size) {
        if (pos != NIL && blocks_[pos].interval == NIL) {
            const int swallowed = pos;
            pos = blocks_[pos].next;
            size += blocks_[swallowed].size;
            drop_hole(swallowed);
        }
        const int before = pos == NIL ? tail_ : blocks_[pos].prev;
        if (before != NIL && blocks_[before].interval == NIL) {
            size += blocks_[before].size;
            drop_hole(before);
        }
        if (size == 0)
            return;
        const int blk = new_block();
        blocks_[blk].size = size;
        blocks_[blk].serial = next_serial_++;
        link_before(pos, blk);
        holes_.emplace(HoleKey{size, blocks_[blk].serial}, blk);
    }
};

size_t round_up(size_t v, size_t a) {
    return (v + a - 1) & ~(a - 1);
}

}  // namespace

bool plan_memory_pushdown(
        const std::vector<MemInterval>& intervals, size_t alignment, std::vector<size_t>* offsets,
        size_t* arena_bytes, size_t* lower_bound) {
    const size_t n = intervals.size();
    if (alignment == 0 || (alignment & (alignment - 1)))
        return false;
    for (const MemInterval& iv : intervals)
        if (iv.begin >= iv.end)
            return false;

    // time step -> (intervals that begin, intervals that end), each in the order added
    std::map<size_t, std::pair<std::vector<int>, std::vector<int>>> events;
    for (size_t i = 0; i < n; ++i) {
        events[intervals[i].begin].first.push_back((int)i);
        events[intervals[i].end].second.push_back((int)i);
    }

    // step 1
    std::vector<std::vector<int>> under(n);
    {
        BlockRow row;
        std::vector<BlockRow::Neighbours> nb(n);
        for (auto& ev : events) {
            for (int i : ev.second.second)
                row.release(i);
            for (int i : ev.second.first)
                nb[i] = row.place(i, intervals[i].size);
        }
        for (size_t i = 0; i < n; ++i) {
            if (nb[i].above != BlockRow::NIL)
                under[nb[i].above].push_back((int)i);
            if (nb[i].under != BlockRow::NIL)
                under[i].push_back(nb[i].under);
        }
    }

    // step 2: depth-first over the DAG with an explicit stack
    constexpr size_t UNSET = (size_t)-1;
    offsets->assign(n, UNSET);
    size_t peak = 0;
    std::vector<std::pair<int, size_t>> stack;  // (interval, next child to look at)
    std::vector<char> open(n, 0);
    for (size_t root = 0; root < n; ++root) {
        if ((*offsets)[root] != UNSET)
            continue;
        stack.emplace_back((int)root, 0);
        open[root] = 1;
        while (!stack.empty()) {
            const int i = stack.back().first;
            size_t& k = stack.back().second;
            bool descended = false;
            while (k < under[i].size()) {
                const int j = under[i][k++];
                if ((*offsets)[j] == UNSET) {
                    if (open[j])
                        return false;  // a cycle cannot come out of step 1
                    open[j] = 1;
                    stack.emplace_back(j, 0);
                    descended = true;
                    break;
                }
            }
            if (descended)
                continue;
            size_t addr = 0;
            for (int j : under[i]) {
                const size_t e = (*offsets)[j] + intervals[j].size;
                if (e > addr)
                    addr = e;
            }
            addr = round_up(addr, alignment);
            (*offsets)[i] = addr;
            const size_t e = round_up(addr + intervals[i].size, alignment);
            if (e > peak)
                peak = e;
            open[i] = 0;
            stack.pop_back();
        }
    }
    *arena_bytes = peak;

    if (lower_bound) {
        // most bytes alive at one time step, every interval rounded up to the alignment
        // (static_mem_alloc/impl.cpp:100-143)
        size_t live = 0, most = 0;
        for (auto& ev : events) {
            for (int i : ev.second.first)
                live += round_up(intervals[i].size, alignment);
            for (int i : ev.second.second)
                live -= round_up(intervals[i].size, alignment);
            if (live > most)
                most = live;
        }
        *lower_bound = most;
    }
    return true;
}

}  // namespace mg
