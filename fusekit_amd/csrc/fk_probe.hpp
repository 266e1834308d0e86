// Timing probes, in ONE place.  A probe build (-DFK_PROBE_STAMPS, made outside the library's Makefile) records a
// clock per workgroup at phase boundaries of a kernel and exports a reader for them; the library build compiles
// every macro here to nothing and exports no probe symbol.
//
//   FK_PROBE_DEFINE(name, BLOCKS, SLOTS)                 once per source file: the stamp array of BLOCKS x SLOTS
//                                                        clocks and `int fk_probe_read_<name>_stamps(out)`, which
//                                                        copies the array to the host and clears it
//   FK_PROBE_STAMP(name, BLOCKS, SLOTS, block, cond, i)  in a kernel: slot i of workgroup `block`, by the threads
//                                                        for which `cond` holds
#pragma once
#ifdef FK_PROBE_STAMPS
#define FK_PROBE_DEFINE(name, BLOCKS, SLOTS)                                                                       \
    __device__ unsigned long long g_fk_##name##_stamp[(BLOCKS) * (SLOTS)];                                         \
    extern "C" __attribute__((visibility("default"))) int fk_probe_read_##name##_stamps(unsigned long long* out) { \
        const size_t bytes = sizeof(unsigned long long) * (BLOCKS) * (SLOTS);                                      \
        hipError_t e = hipMemcpyFromSymbol(out, HIP_SYMBOL(g_fk_##name##_stamp), bytes);                           \
        if (e != hipSuccess) return (int)e;                                                                        \
        void* p = nullptr;                                                                                         \
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_fk_##name##_stamp));                                              \
        return (int)(e != hipSuccess ? e : hipMemset(p, 0, bytes));                                                \
    }
#define FK_PROBE_STAMP(name, BLOCKS, SLOTS, block, cond, i)                                                    \
    do {                                                                                                       \
        const uint32_t fk_probe_b_ = (block);                                                                  \
        if ((cond) && fk_probe_b_ < (uint32_t)(BLOCKS)) g_fk_##name##_stamp[fk_probe_b_ * (SLOTS) + (i)] = wall_clock64(); \
    } while (0)
#else
#define FK_PROBE_DEFINE(name, BLOCKS, SLOTS)
#define FK_PROBE_STAMP(name, BLOCKS, SLOTS, block, cond, i) \
    do {                                                    \
    } while (0)
#endif
