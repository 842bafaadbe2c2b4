// Wall-clock stamps at numbered points of a kernel, for the measurement build only
// (-DSL_PHASE_STAMPS: `python -m spotlight_amd.build --stamps` links libspotlight_hip_stamps.so;
// the product library is built without it and SL_TS() expands to nothing).
//
// Lane 0 of the first SL_STAMP_WGS workgroups of a launch (by linear workgroup number) stores the
// 100 MHz wall clock into slot i of the translation unit's own table; sl_phase_stamps() copies the
// table of the unit registered under a name to the host.  A translation unit names itself with
// SL_TS_NAME before including this file.
#pragma once
#include "common.h"

#ifdef SL_PHASE_STAMPS
#ifndef SL_TS_NAME
#error "define SL_TS_NAME before including phase_stamps.h"
#endif

typedef int (*sl_ts_reader)(unsigned long long *host, int clear);
void sl_ts_register(const char *name, sl_ts_reader fn);   // decode.hip keeps the list

namespace {
__device__ unsigned long long g_ts[SL_STAMP_WGS * SL_STAMP_SLOTS];

int sl_ts_read_here(unsigned long long *host, int clear) {
    if (hipMemcpyFromSymbol(host, HIP_SYMBOL(g_ts), sizeof(unsigned long long) * SL_STAMP_WGS * SL_STAMP_SLOTS, 0,
                            hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    if (clear) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_ts)) != hipSuccess ||
            hipMemset(p, 0, sizeof(unsigned long long) * SL_STAMP_WGS * SL_STAMP_SLOTS) != hipSuccess) {
            (void)hipGetLastError();
            return -1;
        }
    }
    return 0;
}

struct sl_ts_registrar {
    sl_ts_registrar() { sl_ts_register(SL_TS_NAME, sl_ts_read_here); }
} g_ts_registrar;
}  // namespace

#define SL_TS(i)                                                                                                  \
    do {                                                                                                          \
        const unsigned wg_ = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;                      \
        if (threadIdx.x == 0 && wg_ < SL_STAMP_WGS) g_ts[wg_ * SL_STAMP_SLOTS + (i)] = wall_clock64();            \
    } while (0)
#else
#define SL_TS(i) do { } while (0)
#endif
