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
#ifndef DISPATCH_V4_MIN_PAIRS
#define DISPATCH_V4_MIN_PAIRS 8193
#endif

// ITERS > 0: a wavefront's segment is at most 64 * ITERS pairs long and the ids are kept in
// registers between the two passes; ITERS == 0: any length, the ids are read twice.
template <int ITERS>
__global__ void dispatch_kernel(const int32_t *__restrict__ idx, int P, int K, int E,
                                int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
                                int32_t *__restrict__ perm, int32_t *__restrict__ inv,
                                int32_t *__restrict__ slot_token, int64_t *__restrict__ counts_mirror,
                                uint32_t mirror_tag) {
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
        // a tagged second copy, e.g. in host memory the device can write: one 8-byte store per expert
        if (counts_mirror) counts_mirror[e] = (int64_t)(((uint64_t)mirror_tag << 32) | (uint32_t)total_eq);
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

// Long pair lists (P a multiple of 4): the same scheme with four consecutive ids per lane and load.
// A wavefront's segment is CH chunks of 256 pairs, all fetched by CH 16-byte loads before the first
// is looked at.  A lane counts its own matches (0..4), three ballots (one per bit of that count) give
// the matches in lower lanes and in the chunk, and inside a lane the ids are in pair order -- so the
// slots are those of the one-id-per-lane form.  (At P = 32768, E = 128 the workgroups read 16 MB of
// ids from L2 between them: 32 four-byte loads per lane took 14 us.)
template <int CH>
__global__ __launch_bounds__(1024) void dispatch_v4_kernel(const int32_t *__restrict__ idx, int P, int K, int E,
                                                           int32_t *__restrict__ counts,
                                                           int32_t *__restrict__ offsets,
                                                           int32_t *__restrict__ perm, int32_t *__restrict__ inv,
                                                           int32_t *__restrict__ slot_token, uint32_t magic,
                                                           int64_t *__restrict__ counts_mirror, uint32_t mirror_tag) {
    __shared__ int s_eq[DISPATCH_MAX_WAVES];
    __shared__ int s_lt[DISPATCH_MAX_WAVES];
    typedef int int4_t __attribute__((ext_vector_type(4)));
    const int e = blockIdx.x;
    const int lane = lane_id();
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int p_begin = wave * (CH * 256);
    // (the kernel is bound by its instruction count -- 16 wavefronts on one CU per expert, P * E
    // comparisons in all -- so the first pass only adds up per lane and reduces once per wavefront,
    // and the match masks it builds are what the second pass works from)
    int4_t v[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int p = p_begin + i * 256 + lane * 4;
        v[i] = p < P ? *(const int4_t *)(idx + p) : int4_t{-1, -1, -1, -1};     // P % 4 == 0: all four or none
    }
    uint32_t match[CH];        // bit j: id j of the lane's four belongs to this expert
    int l_eq = 0, l_lt = 0;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        match[i] = (v[i][0] == e ? 1u : 0u) | (v[i][1] == e ? 2u : 0u) | (v[i][2] == e ? 4u : 0u) |
                   (v[i][3] == e ? 8u : 0u);
        l_eq += __popc(match[i]);
#pragma unroll
        for (int j = 0; j < 4; ++j) l_lt += (uint32_t)v[i][j] < (uint32_t)e;     // negative ids compare as huge
    }
    const int c_eq = (int)wave_sum((float)l_eq), c_lt = (int)wave_sum((float)l_lt);   // <= 64 * 4 * CH: exact
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
        // a tagged second copy, e.g. in host memory the device can write: one 8-byte store per expert
        if (counts_mirror) counts_mirror[e] = (int64_t)(((uint64_t)mirror_tag << 32) | (uint32_t)total_eq);
        offsets[e] = total_lt;
        if (e == E - 1) offsets[E] = total_lt + total_eq;
    }
    int run = total_lt + base;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int p = p_begin + i * 256 + lane * 4;
        const int me = __popc(match[i]);
        int below = 0, chunk = 0;
#pragma unroll
        for (int bit = 0; bit < 3; ++bit) {
            const uint64_t m = __ballot(me & (1 << bit));
            below += mask_rank(m) << bit;
            chunk += __popcll(m) << bit;
        }
        int slot = run + below;
        // Most lanes hold no pair of this expert and few hold two: instead of four predicated rounds
        // (one per position), the lanes with matches left take their next one, for as many rounds as
        // the fullest lane needs.
        uint32_t left = match[i];
        while (__any(left != 0)) {
            if (left) {
                const int j = __builtin_ctz(left);
                left &= left - 1;
                const int pj = p + j;
                perm[pj] = slot;
                inv[slot] = pj;
                // pj / K by a multiplication when the host could prove it exact (magic != 0)
                slot_token[slot] = magic ? (int)__umulhi((uint32_t)pj, magic) : pj / K;
                ++slot;
            }
        }
        if (e == 0 && p < P) {     // expert 0's workgroup also marks pairs whose id no expert will claim
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (v[i][j] < 0 || v[i][j] >= E) perm[p + j] = -1;
        }
        run += chunk;
    }
    if (e == E - 1) {
        for (int s = total_lt + total_eq + (int)threadIdx.x; s < P; s += (int)blockDim.x) {
            inv[s] = -1;
            slot_token[s] = -1;
        }
    }
}

int odsd_launch_dispatch(const odsd_moe_shape *s, const int32_t *idx, int32_t *counts, int32_t *offsets,
                         int32_t *perm, int32_t *inv, int32_t *slot_token, hipStream_t st, int64_t *counts_mirror,
                         uint32_t mirror_tag) {
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
                offsets, perm, inv, slot_token, counts_mirror, mirror_tag)
    // four ids per lane and load: wavefronts of CH chunks of 256 pairs, up to 16 of them
    if (P >= DISPATCH_V4_MIN_PAIRS && P % 4 == 0 && odsd_aligned16(idx) && P <= 16 * 8 * 256) {
        const int ch = P <= 4096 ? 1 : (P <= 8192 ? 2 : (P <= 16384 ? 4 : 8));
        const int nw = (P + ch * 256 - 1) / (ch * 256);
        // floor(p / K) == mulhi(p, floor(2^32 / K) + 1) for every p with p * K < 2^32
        const uint32_t magic = (uint64_t)P * (uint64_t)s->K < (1ull << 32) && s->K > 1
                                   ? (uint32_t)((1ull << 32) / (uint32_t)s->K) + 1u : 0u;
#define DISPATCH_V4(CHV)                                                                                   \
    ODSD_LAUNCH(ODSD_KERNEL_DISPATCH, dispatch_v4_kernel<CHV>, s->E, 64 * nw, st, idx, P, s->K, s->E, counts, \
                offsets, perm, inv, slot_token, magic, counts_mirror, mirror_tag)
        if (ch == 1) DISPATCH_V4(1);
        else if (ch == 2) DISPATCH_V4(2);
        else if (ch == 4) DISPATCH_V4(4);
        else DISPATCH_V4(8);
#undef DISPATCH_V4
        ODSD_CHECK_LAUNCH();
        return ODSD_OK;
    }
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
    return odsd_launch_dispatch(s, idx, counts, offsets, perm, inv, slot_token, (hipStream_t)stream, nullptr, 0u);
}
