#pragma once

#include "coherent_allocator.hpp"

#include "polar_rt_support.hpp"

namespace polar_harness_detail {
extern uint64_t g_deferredReleases;
extern uint64_t g_eventsWaited;
} // namespace polar_harness_detail
