// Shared device helpers for the gfx950 MoE kernels (64-wide wavefronts throughout).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/odsd_moe.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef double double4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

#define ODSD_WAVE 64
#define ODSD_GROUP 128     // quantisation group (columns of the reduction dimension)
#define ODSD_FP16_MAX 65504.0f

// ---- bf16 <-> f32 (bf16 is carried as its 16-bit pattern) ------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}
// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T> struct ActIO;
template <> struct ActIO<float> {
    static constexpr int dtype = ODSD_DT_F32;
    __device__ static __forceinline__ float load(const float *p, size_t i) { return p[i]; }
    __device__ static __forceinline__ void store(float *p, size_t i, float v) { p[i] = v; }
    // value after a round trip through the activation dtype
    __device__ static __forceinline__ float round(float v) { return v; }
};
template <> struct ActIO<uint16_t> {
    static constexpr int dtype = ODSD_DT_BF16;
    __device__ static __forceinline__ float load(const uint16_t *p, size_t i) { return bf16_to_f32(p[i]); }
    __device__ static __forceinline__ void store(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16(v); }
    __device__ static __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

// saturating f32 -> fp16 (round to nearest even)
__device__ __forceinline__ half_t f32_to_f16_sat(float v) {
    v = fminf(fmaxf(v, -ODSD_FP16_MAX), ODSD_FP16_MAX);
    return (half_t)v;
}

// ---- wavefront helpers -------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (ODSD_WAVE - 1)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, ODSD_WAVE);
    return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, ODSD_WAVE);
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, ODSD_WAVE));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, ODSD_WAVE));
    return v;
}
// number of set bits of `mask` below this lane
__device__ __forceinline__ int mask_rank(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
}

// ---- host-side launch plumbing shared by the entry points ----------------------------------
// Kernel timing for odsd_moe_forward_events: while a call of that entry point is running on a host
// thread, `odsd_prof` points at its context and every kernel launch of the library on that thread
// passes the start / stop events of its kernel slot to the runtime, which stamps them with the
// kernel's own begin and end times (no marker packets between the kernels).
struct OdsdProf {
    void *const *events;    // [2 * ODSD_N_KERNELS]: start, stop per kernel slot
    uint32_t launched;      // bit k: slot k was launched
};
extern thread_local OdsdProf *odsd_prof;
static inline void odsd_prof_events(int slot, hipEvent_t *start, hipEvent_t *stop) {
    if (odsd_prof) {
        *start = (hipEvent_t)odsd_prof->events[2 * slot];
        *stop = (hipEvent_t)odsd_prof->events[2 * slot + 1];
        odsd_prof->launched |= 1u << slot;
    }
}
// KERNEL goes in parentheses when its template arguments contain commas
#define ODSD_LAUNCH(SLOT, KERNEL, GRID, BLOCK, STREAM, ...)                                         \
    do {                                                                                            \
        if (odsd_prof) {                                                                            \
            hipEvent_t ev0_ = nullptr, ev1_ = nullptr;                                              \
            odsd_prof_events(SLOT, &ev0_, &ev1_);                                                   \
            hipExtLaunchKernelGGL(KERNEL, dim3(GRID), dim3(BLOCK), 0, STREAM, ev0_, ev1_, 0, __VA_ARGS__); \
        } else {                                                                                    \
            hipLaunchKernelGGL(KERNEL, dim3(GRID), dim3(BLOCK), 0, STREAM, __VA_ARGS__);            \
        }                                                                                           \
    } while (0)

#define ODSD_CHECK_LAUNCH()                                   \
    do {                                                      \
        if (hipGetLastError() != hipSuccess) return ODSD_ERR_LAUNCH; \
    } while (0)

static inline bool odsd_aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
static inline size_t odsd_round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// kernels implemented in the other translation units (host launchers)
// norm_ss/norm_w/eps: when norm_ss is given, x is RMS-normalised on the fly from the per-row sums
// of squares (the router and the fp16 copy then see RMSNorm(x))
// dispatch arrays a router launch may fill as well (all five or none)
struct OdsdDispatchOut {
    int32_t *counts, *offsets, *perm, *inv, *slot_token;
    // optional second copy of counts for the host (memory the device can write), or null: entry e is
    // (mirror_tag << 32) | counts[e], so a reader that knows the tag can tell when entry e has arrived
    int64_t *counts_mirror;
    uint32_t mirror_tag;
};
// What the combine of a block leaves for the block after it when it is told that block's RMSNorm
// (calls that run a stack of blocks): the normalised rows in the activation dtype and their fp16 copy.
struct OdsdNextNorm {
    const void *norm_w;
    float eps;
    void *xn, *x16;
};
// router (+ dispatch when `disp` is given)
int odsd_launch_router(const odsd_moe_shape *s, const void *x, const void *gate_w, int32_t *idx,
                       float *w, int64_t *idx64, void *x16, void *ws, size_t ws_bytes,
                       hipStream_t st, const double *norm_ss, const void *norm_w, float eps,
                       double *logits = nullptr, const OdsdDispatchOut *disp = nullptr);
int odsd_launch_dispatch(const odsd_moe_shape *s, const int32_t *idx, int32_t *counts,
                         int32_t *offsets, int32_t *perm, int32_t *inv, int32_t *slot_token,
                         hipStream_t st, int64_t *counts_mirror = nullptr, uint32_t mirror_tag = 0u);
// dispatch_out: the dispatch arrays have NOT been filled; the expert kernel dispatches for itself and
// leaves counts / offsets / perm there (only when odsd_experts_dispatch_inside(s) says it can)
int odsd_launch_experts(const odsd_moe_shape *s, const void *x16, const uint64_t *table,
                        const int32_t *idx, const float *w, const int32_t *counts,
                        const int32_t *offsets, const int32_t *perm, const int32_t *slot_token,
                        const void *residual, float *out_f32, void *out_act, void *ws,
                        size_t ws_bytes, hipStream_t st, double *row_ss,
                        const OdsdDispatchOut *dispatch_out = nullptr, const OdsdNextNorm *next_norm = nullptr);
int odsd_combine_norm_supported(const odsd_moe_shape *s);
int odsd_experts_dispatch_inside(const odsd_moe_shape *s);
