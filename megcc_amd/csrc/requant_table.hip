// Host-side cache of requantisation threshold tables (see epilogue.h): one table per
// (activation, src scale, filter scale, dst scale), built on first use with the reference's
// literal float sequence evaluated by the host CPU - the same IEEE single-precision multiply,
// multiply, divide, roundf the generated C kernels execute - and kept for the life of the process.
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>

#include "epilogue.h"

namespace mg {

const RequantTable& requant_table_for(int act, float s_src, float s_flt, float s_dst) {
    static std::mutex lock;
    static std::map<std::tuple<int, uint32_t, uint32_t, uint32_t>, std::unique_ptr<RequantTable>> cache;
    auto bits = [](float f) {
        uint32_t u;
        memcpy(&u, &f, 4);
        return u;
    };
    const auto key = std::make_tuple(act, bits(s_src), bits(s_flt), bits(s_dst));
    std::lock_guard<std::mutex> guard(lock);
    auto it = cache.find(key);
    if (it != cache.end())
        return *it->second;
    std::unique_ptr<RequantTable> t(new RequantTable);
    const float c = make_requant_fast(s_src, s_flt, s_dst).c;
    for (int i = 0; i < REQUANT_TABLE_ENTRIES; ++i) {
        if (i == REQUANT_TABLE_ENTRIES - 1)
            t->t[i] = 0;
        else if (act == MEGCC_NONLINE_RELU)
            t->t[i] = requant_threshold<MEGCC_NONLINE_RELU>(i, s_src, s_flt, s_dst, c);
        else if (act == MEGCC_NONLINE_H_SWISH)
            t->t[i] = requant_threshold<MEGCC_NONLINE_H_SWISH>(i, s_src, s_flt, s_dst, c);
        else
            t->t[i] = requant_threshold<MEGCC_NONLINE_IDENTITY>(i, s_src, s_flt, s_dst, c);
    }
    return *(cache[key] = std::move(t));
}

}  // namespace mg
