// launch.hpp -- kernel launch that hands the dispatch the profiling events of the current call, if any.
#pragma once
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include "internal.hpp"

#define TFH_LAUNCH_TIMED(kernel, grid, block, lds, st, ...)                                                          \
    do {                                                                                                             \
        tfh::note_kernel(#kernel);                                                                                   \
        const tfh::ProfEvents pe_ = tfh::prof_take();                                                                \
        if (pe_.start)                                                                                               \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, st, (hipEvent_t)pe_.start, (hipEvent_t)pe_.stop, 0, __VA_ARGS__); \
        else                                                                                                         \
            hipLaunchKernelGGL(kernel, grid, block, lds, st, __VA_ARGS__);                                           \
    } while (0)
