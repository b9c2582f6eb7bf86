// TEST INFRASTRUCTURE ONLY. C entry point around the reference's own static memory allocator
// (compiler/lib/Dialect/Kernel/Transforms/migrate/static_mem_alloc.h), linked against the
// reference's sources compiled where they lie (see the Makefile): it plans the same intervals
// the product's planner gets, so tests can compare offsets and arena size one to one.
#include <cstddef>
#include <vector>

#include "static_mem_alloc.h"

using mlir::Kernel::migrate::StaticMemAlloc;

extern "C" int ref_plan_memory(
        size_t n, const size_t* begin, const size_t* end, const size_t* size, size_t alignment,
        size_t* offset, size_t* arena_bytes, size_t* lower_bound) {
    // the call sequence of Transforms/StaticMemoryPlanning.cpp:34-96,117-127
    auto solver = StaticMemAlloc::make(StaticMemAlloc::AllocatorAlgo::PUSHDOWN);
    solver->alignment(alignment);
    std::vector<char> keys(n ? n : 1);
    for (size_t i = 0; i < n; ++i)
        solver->add(begin[i], end[i], size[i], &keys[i]);
    solver->solve();
    for (size_t i = 0; i < n; ++i)
        offset[i] = solver->get_start_addr(&keys[i]);
    *arena_bytes = solver->tot_alloc();
    if (lower_bound)
        *lower_bound = solver->tot_alloc_lower_bound();
    return 0;
}
