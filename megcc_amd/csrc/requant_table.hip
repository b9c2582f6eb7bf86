// Host-side cache of requantisation threshold tables (see epilogue.h): one table per
// (activation, src scale, filter scale, dst scale), built on first use with the reference's
// literal float sequence evaluated by the host CPU - the same IEEE single-precision multiply,
// multiply, divide, roundf the generated C kernels execute - and kept for the life of the process.
#include <math.h>

#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"
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

// host evaluation of requant_conv_affine (fmaf is the correctly rounded single fused multiply-add,
// floorf + saturation what v_cvt_flr_i32_f32 does)
static int affine_eval(int a, float c, float d, int lo) {
    const float g = floorf(fmaf((float)a, c, d));
    const float r = g < (float)lo ? (float)lo : (g > 127.f ? 127.f : g);
    return (int)r;
}

RequantAffine requant_affine_for(int act, float s_src, float s_flt, float s_dst) {
    static std::mutex lock;
    static std::map<std::tuple<int, uint32_t, uint32_t, uint32_t>, RequantAffine> cache;
    const RequantAffine none = {0.f, 0.f};
    if ((act != MEGCC_NONLINE_IDENTITY && act != MEGCC_NONLINE_RELU) || !requant_table_ok(s_src, s_flt, s_dst))
        return none;
    auto bits = [](float f) {
        uint32_t u;
        memcpy(&u, &f, 4);
        return u;
    };
    const auto key = std::make_tuple(act, bits(s_src), bits(s_flt), bits(s_dst));
    {
        std::lock_guard<std::mutex> guard(lock);
        auto it = cache.find(key);
        if (it != cache.end())
            return it->second;
    }
    const RequantTable& T = requant_table_for(act, s_src, s_flt, s_dst);
    const int lo = act == MEGCC_NONLINE_RELU ? 0 : -128;
    auto literal = [&](int a) {
        return act == MEGCC_NONLINE_RELU ? requant_conv<MEGCC_NONLINE_RELU>(a, s_src, s_flt, s_dst)
                                         : requant_conv<MEGCC_NONLINE_IDENTITY>(a, s_src, s_flt, s_dst);
    };
    // both sides of every step of F, and the ends of the accumulator range
    struct Point {
        int a, y;
    };
    std::vector<Point> pts;
    pts.push_back({INT32_MIN, literal(INT32_MIN)});
    pts.push_back({INT32_MAX, literal(INT32_MAX)});
    for (int i = 0; i < REQUANT_TABLE_ENTRIES - 1; ++i) {
        const int t = T.t[i];
        if (t == INT32_MIN)
            continue;  // F never drops below this level
        pts.push_back({t, literal(t)});
        if (t < INT32_MAX)
            pts.push_back({t + 1, literal(t + 1)});
    }
    const float c0 = make_requant_fast(s_src, s_flt, s_dst).c;
    RequantAffine found = none;
    for (int k = 0; k <= 16 && found.d == 0.f; ++k) {
        // c' = c0 moved (k + 1) / 2 ulps up (k odd) or down (k even)
        float c = c0;
        for (int s = 0; s < (k + 1) / 2; ++s)
            c = nextafterf(c, (k & 1) ? INFINITY : 0.f);
        double dlo = -1e30, dhi = 1e30;  // floor(a c + d) == y  <=>  y <= a c + d < y + 1
        for (const Point& p : pts) {
            const double prod = (double)(float)p.a * (double)c;
            if (p.y > lo && (double)p.y - prod > dlo)
                dlo = (double)p.y - prod;
            if (p.y < 127 && (double)p.y + 1 - prod < dhi)
                dhi = (double)p.y + 1 - prod;
        }
        if (!(dlo < dhi))
            continue;
        // the middle of the interval first (the most room for the rounding of the fused multiply-add),
        // then points nearer its ends
        static const double kPos[] = {0.5, 0.375, 0.625, 0.25, 0.75};
        for (double pos : kPos) {
            const float d = (float)(dlo + (dhi - dlo) * pos);
            if (!(d > 0.f && d < 1.f))
                continue;
            bool ok = true;
            for (const Point& p : pts)
                if (affine_eval(p.a, c, d, lo) != p.y) {
                    ok = false;
                    break;
                }
            if (ok) {
                found = {c, d};
                break;
            }
        }
    }
    std::lock_guard<std::mutex> guard(lock);
    return cache[key] = found;
}

RequantAffine requant_affine_pick(bool table, int act, float s_src, float s_flt, float s_dst) {
    RequantAffine a = {0.f, 0.f};
    if (table && !options().no_affine)
        a = requant_affine_for(act, s_src, s_flt, s_dst);
    note_requant_affine(a.d != 0.f);
    return a;
}

}  // namespace mg
