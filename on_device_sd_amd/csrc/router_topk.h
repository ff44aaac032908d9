// Pieces of the top-k selection shared by the router kernels: the order-preserving integer key of a
// logit and the wavefront arg-max on (key, id).
#pragma once
#include "common.h"

// total order on doubles as unsigned keys: larger value <=> larger key
__device__ __forceinline__ uint64_t order_key(double v) {
    if (v == 0.0) v = 0.0;   // -0 and +0 compare equal, so they must share a key
    const uint64_t b = (uint64_t)__double_as_longlong(v);
    return (b >> 63) ? ~b : (b | 0x8000000000000000ull);
}

// Wavefront arg-max on (key, -id) with DPP moves: every lane offers one candidate (a lane with nothing
// to offer passes key 0 -- no finite value maps to it -- and the largest id); the largest key wins,
// among equal keys the lowest id.  Returns the winner's id in every lane.
__device__ __forceinline__ int wave_argmax(const uint64_t key, int id) {
    uint32_t klo = (uint32_t)key, khi = (uint32_t)(key >> 32);
#define ODSD_ARGMAX_STEP(CTRL, ROWMASK)                                                                          \
    {                                                                                                            \
        const uint32_t olo = (uint32_t)__builtin_amdgcn_update_dpp((int)klo, (int)klo, CTRL, ROWMASK, 0xF, false); \
        const uint32_t ohi = (uint32_t)__builtin_amdgcn_update_dpp((int)khi, (int)khi, CTRL, ROWMASK, 0xF, false); \
        const int oe = __builtin_amdgcn_update_dpp(id, id, CTRL, ROWMASK, 0xF, false);                          \
        const uint64_t ok = ((uint64_t)ohi << 32) | olo, mk = ((uint64_t)khi << 32) | klo;                       \
        const bool better = ok > mk || (ok == mk && oe < id);                                                    \
        klo = better ? olo : klo;                                                                                \
        khi = better ? ohi : khi;                                                                                \
        id = better ? oe : id;                                                                                   \
    }
    ODSD_ARGMAX_STEP(0x111, 0xF)   // row_shr:1
    ODSD_ARGMAX_STEP(0x112, 0xF)   // row_shr:2
    ODSD_ARGMAX_STEP(0x114, 0xF)   // row_shr:4
    ODSD_ARGMAX_STEP(0x118, 0xF)   // row_shr:8   -> lane 15 of every row holds the row's best
    ODSD_ARGMAX_STEP(0x142, 0xA)   // row_bcast:15 into rows 1 and 3
    ODSD_ARGMAX_STEP(0x143, 0xC)   // row_bcast:31 into rows 2 and 3 -> lane 63 holds the best
#undef ODSD_ARGMAX_STEP
    return __builtin_amdgcn_readlane(id, 63);
}
