// Static memory plan (offsets into one arena) for tensors with known lifetimes.
#pragma once
#include <cstddef>
#include <vector>

namespace mg {

struct MemInterval {
    size_t begin, end;  // alive during time steps [begin, end)
    size_t size;        // bytes
};

// Same plan as MegCC's PUSHDOWN static allocator (compiler/lib/Dialect/Kernel/Transforms/
// migrate/static_mem_alloc.h:26): offsets[i] for every interval, the arena size, and (optional)
// the most bytes alive at one time step, which no plan can beat. `alignment` must be a power of
// two. Returns false for a bad argument (alignment, or an interval with begin >= end).
bool plan_memory_pushdown(
        const std::vector<MemInterval>& intervals, size_t alignment, std::vector<size_t>* offsets,
        size_t* arena_bytes, size_t* lower_bound);

}  // namespace mg
