// Host-side state of the packet filter (rule table, flow table).
#pragma once

#include "ctx.hpp"

namespace bnk {

struct FilterState {
    bool enforce = false;
};

inline FilterState *filter_create() { return new (std::nothrow) FilterState; }
inline void filter_destroy(FilterState *f) { delete f; }

} // namespace bnk
