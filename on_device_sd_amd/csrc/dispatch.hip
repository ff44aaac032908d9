// Dispatch: stable counting sort of the P = T*K (token, k) pairs by expert id.
//
// One workgroup per expert e.  Every wavefront owns a contiguous segment of the pair list.
// Pass 1 counts, per segment, the pairs that go to e and the pairs that go to a lower
// expert (ballot + popcount, no atomics).  A prefix over the wavefront totals in LDS gives
// each segment its base; the number of pairs of lower experts is offsets[e], so no
// workgroup waits for another.  Pass 2 walks the segment again and gives the i-th matching
// pair slot offsets[e] + i.  Within an expert the pairs therefore keep (token, k) order --
// the order torch.where yields on the [T,K] mask in the reference
// (demo/src/model/qwen3_runner.py:305-308) -- and the result is the same on every run.
#include "common.h"

#define DISPATCH_MAX_WAVES 16

// ITERS > 0: a wavefront's segment is at most 64 * ITERS pairs long and the ids are kept in
// registers between the two passes; ITERS == 0: any length, the ids are read twice.
template <int ITERS>
__global__ void dispatch_kernel(const int32_t *__restrict__ idx, int P, int K, int E,
                                int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
                                int32_t *__restrict__ perm, int32_t *__restrict__ inv,
                                int32_t *__restrict__ slot_token) {
    __shared__ int s_eq[DISPATCH_MAX_WAVES];
    __shared__ int s_lt[DISPATCH_MAX_WAVES];
    const int e = blockIdx.x;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    // segment length, a multiple of 64
    const int seg = ((P + nwaves - 1) / nwaves + 63) & ~63;
    const int p_begin = wave * seg;
    const int p_end = min(P, p_begin + seg);

    int c_eq = 0, c_lt = 0;
    int vals[ITERS > 0 ? ITERS : 1];
    if (ITERS > 0) {
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            const int p = p_begin + i * 64 + lane;
            vals[i] = p < p_end ? idx[p] : -1;
        }
#pragma unroll
        for (int i = 0; i < ITERS; ++i) {
            c_eq += __popcll(__ballot(vals[i] == e));
            c_lt += __popcll(__ballot(vals[i] >= 0 && vals[i] < e));
        }
    } else {
        for (int p0 = p_begin; p0 < p_end; p0 += 64) {
            const int p = p0 + lane;
            const int v = p < p_end ? idx[p] : -1;
            c_eq += __popcll(__ballot(v == e));
            c_lt += __popcll(__ballot(v >= 0 && v < e));
        }
    }
    if (lane == 0) { s_eq[wave] = c_eq; s_lt[wave] = c_lt; }
    __syncthreads();
    int base = 0, total_eq = 0, total_lt = 0;
    for (int i = 0; i < nwaves; ++i) {
        if (i < wave) base += s_eq[i];
        total_eq += s_eq[i];
        total_lt += s_lt[i];
    }
    if (threadIdx.x == 0) {
        counts[e] = total_eq;
        offsets[e] = total_lt;
        if (e == E - 1) offsets[E] = total_lt + total_eq;
    }
    int run = total_lt + base;
    auto place = [&](int p, int v) {
        const uint64_t m = __ballot(v == e);
        if (v == e) {
            const int slot = run + mask_rank(m);
            perm[p] = slot;
            inv[slot] = p;
            slot_token[slot] = p / K;
        }
        // expert 0's workgroup also marks pairs whose id no expert will claim
        if (e == 0 && p < p_end && (v < 0 || v >= E)) perm[p] = -1;
        run += __popcll(m);
    };
    if (ITERS > 0) {
#pragma unroll
        for (int i = 0; i < ITERS; ++i) place(p_begin + i * 64 + lane, vals[i]);
    } else {
        for (int p0 = p_begin; p0 < p_end; p0 += 64) {
            const int p = p0 + lane;
            place(p, p < p_end ? idx[p] : -1);
        }
    }
    // slots past the last valid pair (only when some ids are out of range) are marked unused
    if (e == E - 1) {
        __syncthreads();
        for (int s = total_lt + total_eq + (int)threadIdx.x; s < P; s += (int)blockDim.x) {
            inv[s] = -1;
            slot_token[s] = -1;
        }
    }
}

int odsd_launch_dispatch(const odsd_moe_shape *s, const int32_t *idx, int32_t *counts, int32_t *offsets,
                         int32_t *perm, int32_t *inv, int32_t *slot_token, hipStream_t st) {
    if (!s) return ODSD_ERR_NULL;
    if (s->T < 0 || s->E <= 0 || s->K <= 0) return ODSD_ERR_SHAPE;
    if ((int64_t)s->T * s->K > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    if (!idx || !counts || !offsets || !perm || !inv || !slot_token) return ODSD_ERR_NULL;
    if (s->T == 0) return ODSD_OK;
    const int P = s->T * s->K;
    // wavefronts per workgroup: enough that a wavefront keeps at most 4 x 64 ids where the pair list
    // allows it (the register-resident forms unroll ITERS loads and 4 ITERS ballots per wavefront)
    const int threads = P <= 1024 ? 256 : (P <= 2048 ? 512 : 1024);
    const int nwaves = threads / 64;
    const int iters = (((P + nwaves - 1) / nwaves + 63) & ~63) / 64;   // 64-pair chunks per wavefront
#define DISPATCH_GO(IT)                                                                            \
    ODSD_LAUNCH(ODSD_KERNEL_DISPATCH, dispatch_kernel<IT>, s->E, threads, st, idx, P, s->K, s->E, counts, \
                offsets, perm, inv, slot_token)
    if (iters <= 2) DISPATCH_GO(2);
    else if (iters <= 4) DISPATCH_GO(4);
    else if (iters <= 8) DISPATCH_GO(8);
    else if (iters <= 32) DISPATCH_GO(32);
    else DISPATCH_GO(0);
#undef DISPATCH_GO
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_dispatch(const odsd_moe_shape *s, const int32_t *idx, int32_t *counts,
                             int32_t *offsets, int32_t *perm, int32_t *inv, int32_t *slot_token,
                             void *stream) {
    return odsd_launch_dispatch(s, idx, counts, offsets, perm, inv, slot_token, (hipStream_t)stream);
}
