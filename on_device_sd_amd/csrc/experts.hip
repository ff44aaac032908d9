// Grouped W4A16 expert products and the weighted combine.
//
// w4_gemm_kernel is a weight-streaming kernel: every packed weight byte is read from HBM
// once per pass, 16 bytes per lane (one wavefront reads one [16 rows x 128 columns] tile as
// a contiguous 1 KiB), int4 codes are turned into fp16 in registers, and the products with
// the expert's token rows run on v_mfma_f32_16x16x32_f16 with the WEIGHTS as the A operand
// (16 output features) and up to MB blocks of 16 token rows as the B operand, so a verify
// step's handful of rows per expert costs one skinny MFMA per tile instead of a VALU loop.
// fp32 accumulation throughout.
//
//   MODE 0  gate_up: rows of the fused [2I, H] matrix alternate 16 gate rows / 16 up rows,
//           so one lane holds gate and up of the same feature; epilogue h = silu(g)*u -> fp16
//   MODE 1  down:    y[ks][slot][H] fp32 partials over KS slices of the reduction dimension
//                    (summed in a fixed order by the combine, so split-K stays deterministic)
//
// Token rows of one expert are shared by the 4 wavefronts of a workgroup through LDS
// (double buffered, one 128-column group per stage, loads for the next stage in flight
// while the current one is multiplied).
//
// Replaces: expert_forward_with_weights (demo/src/layers/mlp.py:227-230) inside the
// per-expert loop of _execute_moe_with_placement (demo/src/model/qwen3_runner.py:303-380),
// and the indexed "+=" combine (:363, :376).
#include "w4_gemm.h"

#include <type_traits>

// NB    16-row weight blocks per wavefront          MB  16-row token blocks per pass
// DEPTH groups of weight loads kept in flight       NA  blocks expanded to fp16 at a time
// WK    wavefronts of a workgroup that split the reduction dimension among themselves
//       (their partial sums are added through LDS in a fixed order at the end)
// DIRECT == true  (MB == 1): token rows are never staged; each wavefront reads its B
//       fragments straight from L1/L2 as part of the ring slot -- no barrier in the loop.
// DIRECT == false (WK == 1): token rows go global -> LDS by asynchronous DMA loads
//       (global_load_lds, no registers), double buffered, 16-byte segments XOR-swizzled
//       by the row so that the B-fragment reads are bank-conflict free; one raw s_barrier
//       per group, preceded by a vmcnt wait that leaves the newest loads in flight.
// DISP  (gate_up only) the workgroup dispatches for itself: it scans the [P] expert ids (P <= 4
//       per thread), counts the pairs of its expert and of lower experts (ballot / popcount; the
//       order of the pair list is kept: stable), keeps the tokens of a pass's rows in LDS, and the
//       first workgroup of each expert writes counts[e], offsets[e] and the slots of its pairs
template <int NB, int MB, int MODE, int DEPTH, int NA, int WK, bool DIRECT, int OCC, int WAVES, bool DISP>
__global__ __launch_bounds__(64 * WAVES, OCC) void w4_gemm_kernel(const GemmParams p) {
    static_assert(!DISP || MODE == 0, "only gate_up dispatches");
    static_assert(MODE == 1 || NB % 2 == 0, "gate_up needs gate/up block pairs");
    static_assert(NB % NA == 0, "NA must divide NB");
    static_assert(!DIRECT || MB == 1, "the direct path holds one token block");
    static_assert(DIRECT || WK == 1, "K is split across wavefronts on the direct path only");
    static_assert(!DIRECT || WAVES == 4, "the direct path uses 4 wavefronts");
    static_assert((4 * MB) % WAVES == 0 || DIRECT, "token-row pieces must divide among the threads");
    constexpr int RSUB = WAVES / WK;              // wavefronts along the rows
    // trips round the weight ring per loop iteration (the deeper rings serve short reductions,
    // where a long unrolled body only costs instruction fetches)
    constexpr int RING_TRIPS = DEPTH == 2 ? 4 : 1;
    constexpr int XPT = DIRECT ? 1 : 4 * MB / WAVES;   // 16-byte pieces of a token-row chunk per thread
    constexpr int ROWS_PER_PIECE = 4 * WAVES;     // rows covered by one piece index (16 threads per row)
    constexpr int XS_BYTES = 2 * 16 * MB * 256;
    constexpr int RED_FLOATS = WK > 1 ? (WK - 1) * RSUB * 64 * NB * 4 : 1;
    // one LDS object: token-row buffers (LDS path) or the K-part reduction area (direct path)
    constexpr int LDS_BYTES = DIRECT ? (WK > 1 ? RED_FLOATS * 4 : 16) : XS_BYTES;
    __shared__ __attribute__((aligned(16))) char xs_raw[LDS_BYTES];
    float *red = (float *)xs_raw;
    __shared__ int32_t rows_lds[DISP ? 16 * MB : 1];    // DISP: tokens of the pass's rows
    __shared__ int32_t wsum[2][DISP ? WAVES : 1];        // DISP: per-wavefront totals (pairs of e, pairs below e)

    // workgroup -> (expert, row chunk, k split).  Hardware deals workgroups round-robin over
    // the 8 XCDs.  With many token rows per expert (MB >= 6) consecutive logical ids are kept
    // on one XCD so that an expert's rows stay in one L2; with few rows that locality is worth
    // nothing and would leave an XCD idle for every expert without tokens, so the chunks of
    // one expert are spread over all XCDs instead.
    const int b = blockIdx.x;
    const int L = MB >= 6 ? (b & 7) * p.wg_per_xcd + (b >> 3) : b;
    if (L >= p.n_wg) return;
    const int ks = L % p.KS;
    const int chunk = (L / p.KS) % p.nchunks;
    const int e = L / (p.KS * p.nchunks);

    // the row count, the table row and the first slot are requested together: one round trip to
    // memory before the first weight load instead of three dependent ones
    const uint64_t *trow = p.table + (size_t)e * ODSD_TABLE_COLS;
    const uint64_t t_present = trow[0];
    const uint64_t t_q = MODE == 0 ? trow[0] : trow[2], t_sz = MODE == 0 ? trow[1] : trow[3];
    int M_e, base;
    // DISP: one scan of the id list gives the expert's row count, its first slot and -- for the rows
    // m0 .. m0 + 16 MB - 1 of the expert -- their tokens (in LDS).  Nothing of it is kept in registers:
    // a further pass scans again.
    auto scan_rows = [&](const int m0, const bool first) {
        const int tid_ = threadIdx.x, lane_ = tid_ & 63, wave_ = tid_ >> 6;
        const int pair0 = 4 * tid_;
        int id[4] = {-1, -1, -1, -1};
        if (pair0 + 3 < p.P) {
            const uint4_t v = *(const uint4_t *)(p.idx + pair0);
            id[0] = (int)v.x; id[1] = (int)v.y; id[2] = (int)v.z; id[3] = (int)v.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (pair0 + j < p.P) id[j] = p.idx[pair0 + j];   // the list's ragged end
        }
        int cm = 0, cl = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            cm += id[j] == e;
            cl += (uint32_t)id[j] < (uint32_t)e; // ids outside [0, E) belong to nobody
        }
        // counts of at most 4 per lane: three ballots give the prefix over the lower lanes and the total
        const uint64_t m0b = __ballot(cm & 1), m1b = __ballot(cm & 2), m2b = __ballot(cm & 4);
        const uint64_t l0b = __ballot(cl & 1), l1b = __ballot(cl & 2), l2b = __ballot(cl & 4);
        const int pre = mask_rank(m0b) + 2 * mask_rank(m1b) + 4 * mask_rank(m2b);
        __syncthreads();                          // the previous scan's totals and row list have been read
        if (lane_ == 0) {
            wsum[0][wave_] = __popcll(m0b) + 2 * __popcll(m1b) + 4 * __popcll(m2b);
            wsum[1][wave_] = __popcll(l0b) + 2 * __popcll(l1b) + 4 * __popcll(l2b);
        }
        __syncthreads();
        int before = 0, tot_m = 0, tot_l = 0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const int a = wsum[0][w];
            if (w < wave_) before += a;
            tot_m += a;
            tot_l += wsum[1][w];
        }
        M_e = tot_m;
        base = tot_l;
        int rank = before + pre;
        const bool writer = first && chunk == 0 && ks == 0;
        if (writer && tid_ == 0) {
            p.out_counts[e] = tot_m;
            p.out_offsets[e] = tot_l;
            if (e == p.E - 1) p.out_offsets[p.E] = tot_l + tot_m;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (id[j] == e) {
                const int rel = rank - m0;
                if (rel >= 0 && rel < 16 * MB) rows_lds[rel] = (pair0 + j) / p.K;
                // (the ids come from this library's router, so every pair belongs to some expert's workgroup)
                if (writer) p.out_perm[pair0 + j] = tot_l + rank;
                ++rank;
            }
        }
        __syncthreads();                          // the row list is complete
    };
    if (DISP) {
        scan_rows(0, true);
    } else {
        M_e = p.counts[e];
        base = p.offsets[e];
    }
    if (M_e == 0 || t_present == 0) return;
    // addresses from the table are global memory: say so, or the loads become flat loads
    // whose LDS-side counter forces every wait to drain
    const global_char *qp_c = (const global_char *)t_q;
    const global_char *szp_c = (const global_char *)t_sz;
    const global_char *src_c = (const global_char *)p.src;
    // the expert's packed matrix and its (scale, zero) pairs as buffer resources (reads past the
    // end return zero)
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_q, 0, p.NBLK * p.G * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_sz = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_sz, 0, p.NBLK * p.G * 64, 0x00020000);

    const DequantConsts dc = dequant_consts();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // LDS path: the wavefront index as a scalar (the LDS targets of the copies are per wavefront)
    const int wave = DIRECT ? (tid >> 6) : __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kq = lane >> 4;
    const int kpart = wave % WK, rsub = wave / WK;
    // K range of the workgroup, then of this wavefront
    const int G_begin = ks * p.gper;
    const int G_end = min(p.G, G_begin + p.gper);
    const int gw = (G_end - G_begin + WK - 1) / WK;
    const int g_begin = G_begin + kpart * gw;
    const int g_end = min(G_end, g_begin + gw);
    const int g_last = max(g_end - 1, G_begin);

    // Every load in the main loop is unconditional (out-of-range blocks and groups are
    // clamped to a valid tile and their results never stored): straight-line code lets the
    // hardware counters keep several groups of loads in flight instead of draining them.
    // Addresses are a uniform base plus a 32-bit per-lane byte offset (one VGPR per load).
    const int blk0 = (chunk * RSUB + rsub) * NB;   // first 16-row block of this wavefront
    bool blk_ok[NB];
    uint32_t wq_off[NB], sz_off[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        blk_ok[i] = blk0 + i < p.NBLK;
        const uint32_t blk = blk_ok[i] ? blk0 + i : 0;
        wq_off[i] = (blk * p.G * 64 + lane) * 16u;
        sz_off[i] = (blk * p.G * 16 + r) * 4u;
    }

    // x staging (DMA path): piece = tid + 64*WAVES*i -> row = piece / 16, segment = piece % 16
    const int st_seg = tid & 15;
    const int st_row0 = tid >> 4;
    // LDS byte offset of this lane's B fragment of 32-column step j inside a token block:
    // row r, logical segment 4j + kq, stored at segment ^ (row & 15)
    uint32_t lds_frag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_frag[j] = (uint32_t)((r * 16 + ((4 * j + kq) ^ r)) * 16);

    for (int m0 = 0; m0 < M_e; m0 += 16 * MB) {
        const int mcnt = min(M_e - m0, 16 * MB);
        const int nmb = (mcnt + 15) >> 4;
        const int mcnt_s = DIRECT ? mcnt : scalar_int(mcnt);
        if (DISP && m0 > 0) scan_rows(m0, false);   // the tokens of this pass's rows

        // byte offsets of the token rows this thread fetches
        //   DMA path:    piece i -> row st_row0 + 16 i, source segment st_seg ^ (row & 15)
        //   DIRECT path: row r of the block, columns 8*kq.. of each 32-column step
        // rows past the expert's last one are clamped to its first row: the MFMA columns they
        // feed are never stored
        uint32_t st_off[XPT];
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int row = DIRECT ? r : st_row0 + ROWS_PER_PIECE * i;
            const int slot = base + m0 + (row < mcnt ? row : 0);
            const int srow = DISP ? rows_lds[row < mcnt ? row : 0] : (p.rowmap ? p.rowmap[slot] : slot);
            const int seg = DIRECT ? kq : (st_seg ^ (row & 15));
            st_off[i] = ((uint32_t)srow * (uint32_t)p.src_ld + seg * 8) * 2u;
        }

        float4_t acc[NB][MB];
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int m = 0; m < MB; ++m) acc[i][m] = float4_t{0.f, 0.f, 0.f, 0.f};

        uint4_t wq[DEPTH][NB];
        uint32_t wsz[DEPTH][NB];
        uint4_t xd[DIRECT ? DEPTH : 1][4];   // DIRECT: B fragments travel with the ring slot

        // LDS path: buffer loads -- the expert's matrix is a buffer resource in scalar registers, the
        // per-lane byte offset never changes and the group is the scalar offset operand, so a load
        // costs no vector instruction for its address (the direct path measured faster with plain
        // global loads and the group folded into the per-lane offset)
        auto load_w = [&](int buf, int g) {
            const uint32_t gc = (uint32_t)min(g, g_last);
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                if (DIRECT) {
                    wq[buf][i] = __builtin_nontemporal_load((const global_u4 *)(qp_c + (wq_off[i] + gc * 1024u)));
                    wsz[buf][i] = *(const global_u32 *)(szp_c + (sz_off[i] + gc * 64u));
                } else {
                    wq[buf][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, (int)wq_off[i], (int)(gc * 1024u), 2 /* nt */);
                    wsz[buf][i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sz, (int)sz_off[i], (int)(gc * 64u), 0);
                }
            }
        };
        // DIRECT: the B fragments of group g (refilled only after the products that read them)
        auto load_xd = [&](int buf, int g) {
            const uint32_t gc = (uint32_t)min(g, g_last);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                xd[DIRECT ? buf : 0][j] =
                    *(const global_u4 *)(src_c + (st_off[0] + gc * (ODSD_GROUP * 2u) + j * 64u));
        };
        // XPT asynchronous 16-byte loads per thread: global -> xs[buf] (no registers)
        auto dma_x = [&](int buf, int g) {
            const uint32_t gc = (uint32_t)min(g, g_last);
            const global_char *xg = src_c + (size_t)gc * (ODSD_GROUP * 2u);
#pragma unroll
            for (int i = 0; i < XPT; ++i) {
                // piece i covers ROWS_PER_PIECE rows from row ROWS_PER_PIECE * i on: nothing to
                // fetch for a token block without rows
                if (i * ROWS_PER_PIECE < mcnt_s) {
                    lds_void *dst = (lds_void *)(xs_raw + buf * (16 * MB * 256) + (i * 64 * WAVES + wave * 64) * 16);
                    dma16_to_lds(xg, st_off[i], dst);
                }
            }
        };

        if (!DIRECT) {
            __builtin_amdgcn_s_barrier();   // the previous pass is done with xs
            dma_x(0, g_begin);
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            load_w(d, g_begin + d);
            if (DIRECT) load_xd(d, g_begin + d);
        }
        if (!DIRECT) {
            // x(g_begin) has landed once at most the loads issued after it are outstanding
            ODSD_WAIT_VMCNT(DEPTH * 2 * NB);
            __builtin_amdgcn_s_barrier();
        }

        // One step = one group: expand ring slot d, refill it with group g + DEPTH, multiply.
        // REFILL is a compile-time flag: the last DEPTH groups of the reduction have nothing left
        // to fetch, and their steps are compiled without the refill (a refill clamped to the
        // last group would read that tile again: DEPTH of G tiles per block, 12 % of the stream
        // at G = 16, a third at G = 6).
        auto step = [&](auto refill_c, const int d, const int xb, const int g) {
            constexpr bool REFILL = decltype(refill_c)::value;
            // issue order is pinned: as soon as this slot's codes have been expanded, the DMA
            // of the next group's token rows (into the buffer the previous step read; every
            // wavefront has passed that step's barrier) and the slot's refill, then the products.
            // (The compiler cannot see the DMA loads.  Issued after the expansion, the vmcnt
            // wait it derives for the slot retires exactly the slot and the previous DMA.)
            half8_t bdir[4];
            if (DIRECT) {
#pragma unroll
                for (int j = 0; j < 4; ++j) bdir[j] = __builtin_bit_cast(half8_t, xd[DIRECT ? d : 0][j]);
            }
            // this step's token buffer: one add per 32-column step, the block is an immediate
            const char *xfrag[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) xfrag[j] = xs_raw + (uint32_t)(xb * (16 * MB * 256)) + lds_frag[j];
            const int nmb_s = DIRECT ? nmb : scalar_int(nmb);
#pragma unroll
            for (int h = 0; h < NB; h += NA) {
                half8_t a[NA][4];
#pragma unroll
                for (int i = 0; i < NA; ++i) dequant_tile(dc, wq[d][h + i], wsz[d][h + i], a[i]);
                if (h + NA >= NB) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (!DIRECT && (REFILL || g + 1 < g_end)) dma_x(xb ^ 1, g + 1);
                    if (REFILL) load_w(d, g + DEPTH);      // ring slot d is free again
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    if (m < nmb_s) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            half8_t bx;
                            if (DIRECT) bx = bdir[j];
                            else bx = *(const half8_t *)(xfrag[j] + m * 4096);
#pragma unroll
                            for (int i = 0; i < NA; ++i)
                                acc[h + i][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i][j], bx, acc[h + i][m], 0, 0, 0);
                        }
                    }
                }
            }
            if (DIRECT) {
                __builtin_amdgcn_sched_barrier(0);
                if (REFILL) load_xd(d, g + DEPTH);
            } else {
                __builtin_amdgcn_sched_barrier(0);
                // x(g+1) was issued in this step, before this step's refill: once only the
                // refill is outstanding it has landed (and so has the previous step's refill,
                // which the next step starts with anyway)
                if (REFILL) ODSD_WAIT_VMCNT(2 * NB);
                else ODSD_WAIT_VMCNT(0);
                __builtin_amdgcn_s_barrier();
            }
        };
        // with an even number of steps per trip the token buffer of a step is known at compile
        // time (every trip starts on an even step) and becomes an immediate offset
        constexpr bool XB_STATIC = DEPTH % 2 == 0;
        int it = 0, g = g_begin;
        // Main part: whole trips round the ring while more than DEPTH groups remain (a trip whose
        // later refills run past the last group clamps them: at most DEPTH - 1 tiles per block).
        // Several trips per loop iteration: at a loop header the compiler's wait-count
        // bookkeeping falls back to draining every outstanding load before the first use of ring
        // data, so the fewer headers the stream crosses, the less often the pipeline runs empty.
        while (g + DEPTH < g_end) {
#pragma unroll
            for (int t = 0; t < RING_TRIPS; ++t) {
#pragma unroll
                for (int d = 0; d < DEPTH; ++d) {
                    step(std::true_type{}, d, XB_STATIC ? (d & 1) : (it & 1), g);
                    ++g;
                    ++it;
                }
                if (!(g + DEPTH < g_end)) break;
            }
        }
        // Tail: the groups that are already in the ring.
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (g < g_end) {
                step(std::false_type{}, d, XB_STATIC ? (d & 1) : (it & 1), g);
                ++g;
                ++it;
            }
        }

        if (WK > 1) {
            // partial sums of the K parts: parts 1.. go through LDS, part 0 adds them in order
            __syncthreads();
            if (kpart > 0) {
#pragma unroll
                for (int i = 0; i < NB; ++i)
                    *(float4_t *)&red[(((kpart - 1) * RSUB + rsub) * NB + i) * 256 + lane * 4] = acc[i][0];
            }
            __syncthreads();
            if (kpart == 0) {
#pragma unroll
                for (int k = 1; k < WK; ++k)
#pragma unroll
                    for (int i = 0; i < NB; ++i)
                        acc[i][0] += *(const float4_t *)&red[(((k - 1) * RSUB + rsub) * NB + i) * 256 + lane * 4];
            }
        }

        // epilogue: lane holds rows 4*kq..4*kq+3 of each 16-row block, token column r
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const int row = m * 16 + r;
            if (m < nmb && row < mcnt && kpart == 0) {
                const size_t slot = (size_t)(base + m0 + row);
                if (MODE == 0) {
#pragma unroll
                    for (int i = 0; i < NB; i += 2) {
                        if (blk_ok[i]) {
                            const float4_t gt = acc[i][m], up = acc[(i + 1) % NB][m];
                            half4_t h;
                            h.x = f32_to_f16_sat(silu_f32(gt.x) * up.x);
                            h.y = f32_to_f16_sat(silu_f32(gt.y) * up.y);
                            h.z = f32_to_f16_sat(silu_f32(gt.z) * up.z);
                            h.w = f32_to_f16_sat(silu_f32(gt.w) * up.w);
                            const int feat = ((blk0 + i) >> 1) * 16 + kq * 4;
                            *(half4_t *)(p.h16 + slot * p.ldo + feat) = h;
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NB; ++i) {
                        if (blk_ok[i]) {
                            const int n = (blk0 + i) * 16 + kq * 4;
                            if (p.y_f16) {
                                const float4_t v = acc[i][m];
                                *(half4_t *)((half_t *)p.y + ((size_t)ks * p.P + slot) * p.ldo + n) =
                                    half4_t{f32_to_f16_sat(v.x), f32_to_f16_sat(v.y), f32_to_f16_sat(v.z), f32_to_f16_sat(v.w)};
                            } else {
                                *(float4_t *)(p.y + ((size_t)ks * p.P + slot) * p.ldo + n) = acc[i][m];
                            }
                        }
                    }
                }
            }
        }
        if (WK > 1) __syncthreads();   // red is reused by the next pass
    }
}

// ---------------------------------------------------------------------------------------------
// Combine: out[t] = sum_k w[t,k] * (sum_ks y[ks][perm[t*K+k]]) in k order, fp32, one rounding.
// A pair whose expert has no weights (table row 0) or whose id is out of range adds nothing.
// out_act = cast(residual + cast(moe)): the reference rounds the MoE output to the
// activation dtype before the residual add (qwen3_runner.py:295, :226).
// ---------------------------------------------------------------------------------------------
// KB > 0 (K a multiple of KB, KS == 1): the rows of KB pairs are fetched together -- slot, expert
// and weight first, then KB independent row loads -- and added in k order; with the generic loop
// every row load waits for the one before it (its address hangs on a branch), which is what the
// kernel's time consists of at K = 8.
// YH: 0 = y holds fp32 partial sums of KS slices; 1 = complete sums as fp16; 2 = KS fp16 slices (the
// batched form, KB > 0, takes exactly two)
// Gather-sum of one token's columns c .. c+3: sum over k of w[t,k] * (sum over slices of y[slice][slot(t,k)]).
template <int YH, int KB>
__device__ __forceinline__ float4_t combine_gather(const float *__restrict__ y, const int32_t *__restrict__ idx,
                                                   const float *__restrict__ w, const int32_t *__restrict__ perm,
                                                   const uint64_t *__restrict__ table, const int t, const int c,
                                                   const int H, const int K, const int E, const int KS, const int P) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
        if (KB > 0) {
            for (int k0 = 0; k0 < K; k0 += KB) {
                int slot[KB > 0 ? KB : 1];
                float wk[KB > 0 ? KB : 1];
                bool ok[KB > 0 ? KB : 1];
                uint64_t tq[KB > 0 ? KB : 1];      // first table entry of the pair's expert: 0 = no weights
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    const int pr = t * K + k0 + u;
                    const int sl = perm[pr];
                    const int e = idx[pr];
                    wk[u] = w[pr];
                    // (the row's address must not wait for the table entry: that would be a third
                    // dependent round trip to memory -- slot, then table, then row -- in a kernel that
                    // consists of little else; a pair in range always has a row that exists)
                    const bool in_range = sl >= 0 && e >= 0 && e < E;
                    tq[u] = table[(size_t)(in_range ? e : 0) * ODSD_TABLE_COLS];
                    ok[u] = in_range;
                    slot[u] = in_range ? sl : 0;   // a row that exists; its values are discarded below
                }
                float4_t v[KB > 0 ? KB : 1];
                if (YH == 2) {
                    // two fp16 slices: all 2 KB row loads are issued before the first is used
                    half4_t h0[KB > 0 ? KB : 1], h1[KB > 0 ? KB : 1];
#pragma unroll
                    for (int u = 0; u < KB; ++u) {
                        h0[u] = *(const half4_t *)((const half_t *)y + (size_t)slot[u] * H + c);
                        h1[u] = *(const half4_t *)((const half_t *)y + ((size_t)P + slot[u]) * H + c);
                    }
#pragma unroll
                    for (int u = 0; u < KB; ++u) {
                        v[u] = float4_t{(float)h0[u].x, (float)h0[u].y, (float)h0[u].z, (float)h0[u].w};
                        v[u] += float4_t{(float)h1[u].x, (float)h1[u].y, (float)h1[u].z, (float)h1[u].w};
                    }
                } else {
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    if (YH) {
                        const half4_t hv = *(const half4_t *)((const half_t *)y + (size_t)slot[u] * H + c);
                        v[u] = float4_t{(float)hv.x, (float)hv.y, (float)hv.z, (float)hv.w};
                    } else {
                        v[u] = *(const float4_t *)(y + (size_t)slot[u] * H + c);
                    }
                }
                }
#pragma unroll
                for (int u = 0; u < KB; ++u) {
                    if (ok[u] && tq[u] != 0) {
                        acc.x = fmaf(wk[u], v[u].x, acc.x);
                        acc.y = fmaf(wk[u], v[u].y, acc.y);
                        acc.z = fmaf(wk[u], v[u].z, acc.z);
                        acc.w = fmaf(wk[u], v[u].w, acc.w);
                    }
                }
            }
        } else {
        for (int k = 0; k < K; ++k) {
            const int pr = t * K + k;
            const int slot = perm[pr];
            const int e = idx[pr];
            if (slot < 0 || e < 0 || e >= E || table[(size_t)e * ODSD_TABLE_COLS] == 0) continue;
            float4_t v;
            if (YH) {
                // fp16 values: complete sums (YH == 1) or the partial sums of KS slices (YH == 2)
                const half4_t hv = *(const half4_t *)((const half_t *)y + (size_t)slot * H + c);
                v = float4_t{(float)hv.x, (float)hv.y, (float)hv.z, (float)hv.w};
                if (YH == 2) {
                    for (int sl = 1; sl < KS; ++sl) {      // further slices, in slice order
                        const half4_t hs = *(const half4_t *)((const half_t *)y + ((size_t)sl * P + slot) * H + c);
                        v += float4_t{(float)hs.x, (float)hs.y, (float)hs.z, (float)hs.w};
                    }
                }
            } else {
                v = *(const float4_t *)(y + (size_t)slot * H + c);
                for (int s = 1; s < KS; ++s) v += *(const float4_t *)(y + ((size_t)s * P + slot) * H + c);
            }
            const float wk = w[pr];
            acc.x = fmaf(wk, v.x, acc.x);
            acc.y = fmaf(wk, v.y, acc.y);
            acc.z = fmaf(wk, v.z, acc.z);
            acc.w = fmaf(wk, v.w, acc.w);
        }
        }
        return acc;
}

// What a token's 4 columns become once the sum is there: residual add and the roundings of the
// reference (out_act = cast(residual + cast(moe))), stores, and the values as stored in out_act.
template <typename XT>
__device__ __forceinline__ void combine_finish(const float4_t acc, const XT *__restrict__ residual,
                                               float *__restrict__ out_f32, XT *__restrict__ out_act,
                                               const size_t o, float (&stored)[4]) {
    float res[4] = {0.f, 0.f, 0.f, 0.f};
    if (residual) {
#pragma unroll
        for (int i = 0; i < 4; ++i) res[i] = ActIO<XT>::load(residual, o + i);
    }
    const float a[4] = {acc.x, acc.y, acc.z, acc.w};
    if (out_f32) *(float4_t *)(out_f32 + o) = float4_t{a[0] + res[0], a[1] + res[1], a[2] + res[2], a[3] + res[3]};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float m = ActIO<XT>::round(a[i]);
        stored[i] = ActIO<XT>::round(residual ? __fadd_rn(res[i], m) : m);
        if (out_act) ActIO<XT>::store(out_act, o + i, stored[i]);
    }
}

template <typename XT, int YH, bool STATS, int KB>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y, const int32_t *__restrict__ idx,
                                                      const float *__restrict__ w,
                                                      const int32_t *__restrict__ perm,
                                                      const uint64_t *__restrict__ table,
                                                      const XT *__restrict__ residual,
                                                      float *__restrict__ out_f32, XT *__restrict__ out_act,
                                                      double *__restrict__ row_ss,
                                                      int T, int H, int K, int E, int KS, int P, int nchunk) {
    // One workgroup per (token, 1024-column chunk).  STATS: it also leaves the sum of squares of
    // what it stored in out_act, row_ss[t][chunk] -- the statistic the next block's RMSNorm
    // starts from (chunk sums are added in ascending order by whoever consumes them).
    // (token and chunk share the x dimension of the grid: the y dimension ends at 65535)
    const int t = blockIdx.x / nchunk;
    const int chunk = blockIdx.x - t * nchunk;
    double ss = 0.0;
    const int c = (chunk * 256 + threadIdx.x) * 4;
    if (c < H) {
        const float4_t acc = combine_gather<YH, KB>(y, idx, w, perm, table, t, c, H, K, E, KS, P);
        float stored[4];
        combine_finish<XT>(acc, residual, out_f32, out_act, (size_t)t * H + c, stored);
        if (STATS) {
#pragma unroll
            for (int i = 0; i < 4; ++i) ss += (double)stored[i] * (double)stored[i];
        }
    }
    if (STATS) {
        __shared__ double red[4];
        ss = wave_sum(ss);
        if (lane_id() == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        if (threadIdx.x == 0) row_ss[(size_t)t * nchunk + chunk] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}

// The combine of a block whose successor is known (a stack of blocks): one workgroup per token owns
// the whole row -- 256 threads per 1024-column chunk, each chunk handled exactly as combine_kernel
// handles it, so the row statistic has the same bits -- and once the statistic is complete it also
// applies the next block's RMSNorm (demo/src/layers/layernorm.py:21-27, the arithmetic of
// rmsnorm_kernel and of the router kernel's fold) and leaves what that block starts from: xn, the
// normalised row in the activation dtype (the next router's input), and x16, its fp16 copy (the
// expert kernels' operand).  Otherwise every workgroup of the next router kernel that touches the
// row normalises its columns again (8.2 against 6.0 us per layer at T = 256, H = 2048, E = 128).
template <typename XT, int YH, int KB>
__global__ __launch_bounds__(1024) void combine_norm_kernel(const float *__restrict__ y, const int32_t *__restrict__ idx,
                                                            const float *__restrict__ w,
                                                            const int32_t *__restrict__ perm,
                                                            const uint64_t *__restrict__ table,
                                                            const XT *__restrict__ residual, XT *__restrict__ out_act,
                                                            int T, int H, int K, int E, int KS, int P,
                                                            const XT *__restrict__ next_w, double eps,
                                                            XT *__restrict__ xn_out, half_t *__restrict__ x16_out) {
    __shared__ double red[16];
    const int t = blockIdx.x;
    const int nchunk = (H + 1023) / 1024;              // = blockDim.x / 256
    const int c = (int)threadIdx.x * 4;                // chunk threadIdx.x / 256, its thread threadIdx.x % 256
    const bool in = c < H;
    const size_t o = (size_t)t * H + c;
    float st[4] = {0.f, 0.f, 0.f, 0.f};
    float nw[4] = {0.f, 0.f, 0.f, 0.f};
    double ss = 0.0;
    if (in) {
#pragma unroll
        for (int i = 0; i < 4; ++i) nw[i] = ActIO<XT>::load(next_w, c + i);
        const float4_t acc = combine_gather<YH, KB>(y, idx, w, perm, table, t, c, H, K, E, KS, P);
        combine_finish<XT>(acc, residual, nullptr, out_act, o, st);
#pragma unroll
        for (int i = 0; i < 4; ++i) ss += (double)st[i] * (double)st[i];
    }
    ss = wave_sum(ss);
    if (lane_id() == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    double tot = 0.0;
    for (int n = 0; n < nchunk; ++n) tot += (red[4 * n] + red[4 * n + 1]) + (red[4 * n + 2] + red[4 * n + 3]);
    const double rstd = 1.0 / sqrt(tot / (double)H + eps);
    if (in) {
        half4_t h;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float xn = ActIO<XT>::round((float)((double)st[i] * rstd));
            const float xo = ActIO<XT>::round(__fmul_rn(xn, nw[i]));
            ActIO<XT>::store(xn_out, o + i, xo);
            h[i] = f32_to_f16_sat(xo);
        }
        *(half4_t *)(x16_out + o) = h;
    }
}

// ---- host side ---------------------------------------------------------------------------------
struct ExpertsPlan {
    int MB;          // 16-row token blocks held per pass
    int NB;          // 16-row weight blocks per wavefront
    int WK_gu, WK_dn;  // wavefronts splitting K inside a workgroup (MB == 1 path)
    int KS;          // split of the down projection's reduction dimension across workgroups
    int PS_gu, PS_dn;  // prefill tile kernel: workgroups sharing the row passes of one tile
    int tile;        // MB == 8: the 256 x 256 tile kernel instead of the streaming kernel
    int y_f16;       // down-projection outputs kept as fp16 (unsplit reduction) instead of fp32 partials
    int fused;       // whole-block calls run gate_up and down as one launch (experts_fused.hip)
    int S;           // fused: workgroups per expert = fp16 partial-sum slices of the down projection
    size_t h_bytes, y_bytes;
};

// one-launch expert kernel (experts_fused.hip)
void odsd_launch_experts_fused(FusedParams &fp, int E, hipStream_t st);
int odsd_fused_supported(int H, int I, int S, int E);
int odsd_fused_dispatch_supported(int P);

// Choices are functions of the shape only (the per-expert counts live on the device).
static ExpertsPlan experts_plan(const odsd_moe_shape *s) {
    ExpertsPlan p;
    const long P = (long)s->T * s->K;
    const long mean_rows = (P + s->E - 1) / s->E;
    // token blocks per pass follow the mean number of rows per expert; an expert with more
    // rows than one pass holds takes further passes over its weights.  Measured crossovers
    // (uniform routing, Mixtral and Qwen3-235B expert shapes): 64-row passes win up to ~60 rows
    // per expert, 128-row streaming passes up to ~130, the 256-row tile kernel beyond.
    p.tile = 0;
    if (s->T <= 16) p.MB = 1;
    else if (s->T <= 32) p.MB = 2;
    else if (s->T <= 64) p.MB = 4;      // no expert can have more rows than a 64-row pass holds
    else if (mean_rows <= 16) p.MB = 2;
    else if (mean_rows <= 52) p.MB = 4;
    else { p.MB = 8; p.tile = mean_rows > 136; }
    const long active = s->E < P ? s->E : P;       // upper bound of experts with rows
    const long slots = 512;                        // 256 CUs x 2 workgroups
    const int G_gu = s->H / ODSD_GROUP, G_dn = s->I / ODSD_GROUP;
    p.NB = 4;
    p.WK_gu = p.WK_dn = 1;
    p.KS = 1;
    p.PS_gu = p.PS_dn = 1;
    if (p.MB == 1) {
        // many small work items: 4 wavefronts split K when each still gets >= 2 groups
        p.WK_gu = G_gu >= 8 ? 4 : (G_gu >= 4 ? 2 : 1);
        const long chunks_dn = (s->H / 16 + 4 - 1) / 4;   // with WK = 4: 64 rows per workgroup
        int KS = 1;
        while (KS * 2 <= G_dn / 8 && active * chunks_dn * KS < 4 * slots && KS < 16) KS *= 2;
        p.KS = KS;
        const int gper = (G_dn + KS - 1) / KS;
        p.WK_dn = gper >= 8 ? 4 : (gper >= 4 ? 2 : 1);
    } else if (p.tile) {
        // 256 x 256 tiles: with few experts the tiles alone do not fill 256 CUs.  First hand the
        // row passes of one tile (it re-reads its weights per pass anyway) to several workgroups,
        // then split the down projection's reduction.
        const long mean_passes = (mean_rows + 255) / 256;
        const long tiles_gu = active * ((2 * s->I / 16 + 15) / 16), tiles_dn = active * ((s->H / 16 + 15) / 16);
        while (tiles_gu * p.PS_gu < slots && p.PS_gu * 2 <= mean_passes) p.PS_gu *= 2;
        while (tiles_dn * p.PS_dn < slots && p.PS_dn * 2 <= mean_passes) p.PS_dn *= 2;
        int KS = 1;
        while (tiles_dn * p.PS_dn * KS < slots && KS * 2 <= G_dn / 4 && KS < 16) KS *= 2;
        p.KS = KS;
    } else {
        if (p.MB <= 4) {
            const long wg_gu = active * ((2 * s->I / 16 + 15) / 16);
            if (wg_gu < 4 * slots) p.NB = 2;
        } else {
            p.NB = 2;
        }
        const int nchunks_dn = (s->H / 16 + 4 * p.NB - 1) / (4 * p.NB);
        // up to 4 workgroups per CU with at most 4 token blocks, 2 with 8
        const long want = p.MB <= 4 ? 2 * slots : slots;
        int KS = 1;
        while (KS * 2 <= G_dn / 2 && active * nchunks_dn * KS < want && KS < 16) KS *= 2;
        p.KS = KS;
    }
    // every split must own at least one group
    while (p.KS > 1 && ((G_dn + p.KS - 1) / p.KS) * (p.KS - 1) >= G_dn) p.KS--;
    // The down projection's outputs are stored as fp16 (3 more bits than the bf16 the reference keeps
    // its expert outputs in): half the bytes to write and to read back in the combine (at prefill
    // shapes fp32 would be 0.5 GB per layer each way) -- complete sums without a split of the
    // reduction, one fp16 partial sum per slice with one (added in slice order by the combine; at the
    // Mixtral T = 160 shape the fp32 form wrote and re-read 21 MB per layer).  Calls with at most 16
    // tokens keep fp32 partial sums: they split deepest (up to 16 slices) and move next to nothing.
    p.y_f16 = p.KS == 1 || p.MB >= 2;
    p.h_bytes = odsd_round_up((size_t)(P > 0 ? P : 1) * s->I * sizeof(half_t), 256);
    p.y_bytes = odsd_round_up((size_t)p.KS * (size_t)(P > 0 ? P : 1) * s->H * (p.y_f16 ? sizeof(half_t) : sizeof(float)), 256);
    // The one-launch expert kernel serves calls where nearly every expert has rows and a pass holds
    // them all (8 to 20 rows per expert on average, at most 32 per pass; measured against the
    // two-launch plan on uniform routing it wins up to 20 and loses from 24 on, where many experts
    // need a second pass over their weights): one workgroup per
    // (expert, slice of the intermediate dimension), E * S workgroups for 256 CUs.  The stage entry
    // points keep the two-launch plan above; only the whole-block calls take this path.
    // An expert with more rows than a pass holds streams its slice a second time while the other
    // CUs have nothing left to do (110 against 84 us for the layer with one expert at 33 rows; the
    // two-launch plan stays at 85): a caller that knows the largest count says so in max_rows, and
    // the plan then takes the one-launch kernel only when one pass covers every expert.
    p.fused = 0;
    p.S = 1;
    if (s->T > 16 && mean_rows >= 8 && mean_rows <= 20) {
        int S = 256 / s->E;
        if (S >= 1 && S <= 2 && s->E * S >= 192 && odsd_fused_supported(s->H, s->I, S, s->E)) {
            // (the buffer serves either plan: its size does not depend on the caller's statement)
            const size_t need = odsd_round_up((size_t)S * (size_t)P * s->H * sizeof(half_t), 256);
            if (need > p.y_bytes) p.y_bytes = need;
            if (s->max_rows <= 0 || s->max_rows <= ODSD_ONE_LAUNCH_ROWS) {
                p.fused = 1;
                p.S = S;
            }
        }
    }
    return p;
}

static int experts_check(const odsd_moe_shape *s) {
    if (!s) return ODSD_ERR_NULL;
    if (s->T < 0 || s->H <= 0 || s->E <= 0 || s->K <= 0 || s->I <= 0) return ODSD_ERR_SHAPE;
    if (s->H % ODSD_GROUP || s->I % ODSD_GROUP) return ODSD_ERR_SHAPE;
    if ((int64_t)s->T * s->K > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    if (s->act_dtype != ODSD_DT_F32 && s->act_dtype != ODSD_DT_BF16) return ODSD_ERR_DTYPE;
    // the kernels address token rows and weight tiles with 32-bit byte offsets: a row of x is
    // found at token * H * 2, a row of h at slot * I * 2, a tile inside one expert's matrix
    const int64_t P = (int64_t)s->T * s->K;
    const int64_t hi = s->H > s->I ? s->H : s->I;
    if ((int64_t)s->T * s->H * 2 >= (1LL << 32) || P * s->I * 2 >= (1LL << 32) || P * hi * 2 >= (1LL << 32))
        return ODSD_ERR_UNSUPPORTED;
    if ((int64_t)s->H * s->I >= (1LL << 31)) return ODSD_ERR_UNSUPPORTED;   // 2 I x H / 2 bytes of codes
    return ODSD_OK;
}

extern "C" size_t odsd_experts_workspace_bytes(const odsd_moe_shape *s) {
    if (experts_check(s) != ODSD_OK) return 0;
    const ExpertsPlan p = experts_plan(s);
    return p.h_bytes + p.y_bytes;
}

template <int NB, int MB, int MODE, int DEPTH, int NA, int WK, bool DIRECT, int OCC, int WAVES = 4>
static void launch_gemm(GemmParams &gp, hipStream_t st) {
    gp.nchunks = (gp.NBLK + (WAVES / WK) * NB - 1) / ((WAVES / WK) * NB);
    gp.n_wg = gp.E * gp.nchunks * gp.KS;
    gp.wg_per_xcd = (gp.n_wg + 7) / 8;
    if constexpr (MODE == 0 && !DIRECT && MB <= 4) {
        if (gp.idx) {
            ODSD_LAUNCH(ODSD_KERNEL_GATE_UP, (w4_gemm_kernel<NB, MB, MODE, DEPTH, NA, WK, DIRECT, OCC, WAVES, true>),
                        gp.wg_per_xcd * 8, 64 * WAVES, st, gp);
            return;
        }
    }
    ODSD_LAUNCH(MODE == 0 ? ODSD_KERNEL_GATE_UP : ODSD_KERNEL_DOWN,
                (w4_gemm_kernel<NB, MB, MODE, DEPTH, NA, WK, DIRECT, OCC, WAVES, false>), gp.wg_per_xcd * 8, 64 * WAVES, st, gp);
}

// prefill-shaped tile kernel (experts_prefill.hip)
template <int MODE> void odsd_launch_gemm_prefill(GemmParams &gp, hipStream_t st);

template <int MODE>
static void launch_gemm_plan(const ExpertsPlan &pl, GemmParams &gp, hipStream_t st) {
    const int wk = MODE == 0 ? pl.WK_gu : pl.WK_dn;
    gp.y_f16 = pl.y_f16;
    if (pl.MB == 1) {
        if (wk == 4) launch_gemm<4, 1, MODE, 2, 2, 4, true, 2>(gp, st);
        else if (wk == 2) launch_gemm<4, 1, MODE, 3, 2, 2, true, 2>(gp, st);
        else launch_gemm<4, 1, MODE, 3, 2, 1, true, 2>(gp, st);
    } else if (pl.MB == 2) {
        if (pl.NB == 2) launch_gemm<2, 2, MODE, 2, 2, 1, false, 4>(gp, st);
        else launch_gemm<4, 2, MODE, 3, 4, 1, false, 2>(gp, st);
    } else if (pl.MB == 4) {
        if (pl.NB == 2) launch_gemm<2, 4, MODE, 2, 2, 1, false, 4>(gp, st);
        else launch_gemm<4, 4, MODE, 2, 2, 1, false, 2>(gp, st);
    } else if (pl.tile) {
        odsd_launch_gemm_prefill<MODE>(gp, st);
    } else {
        launch_gemm<2, 8, MODE, 2, 2, 1, false, 2>(gp, st);
    }
}

static int experts_args_ok(const odsd_moe_shape *s) {
    const int rc = experts_check(s);
    return rc;
}

// gate_up + SiLU*mul: x_f16 [T,H] gathered by slot_token -> h_f16 [P,I] in slot order
// the streaming gate_up kernels scan up to 4 ids per thread of their 256
// (measured: with a dozen workgroups per expert the scan costs the gate_up kernel nothing and saves
// the dispatch launch, 4 us of the Zipf-skewed T = 64 layer's 81; with hundreds of workgroups per
// expert it costs gate_up more than the launch it saves: +7 us at the Mixtral T = 160 shape, +6 us
// at T = 5, so those plans keep the dispatch kernel)
static bool stream_dispatch_supported(const ExpertsPlan &pl, const odsd_moe_shape *s) {
    const int chunks = (2 * s->I / 16 + 4 * pl.NB - 1) / (4 * pl.NB);     // gate_up workgroups per expert
    return !pl.tile && (pl.MB == 2 || pl.MB == 4) && chunks <= 32 && s->T * s->K <= 4 * 256;
}

// idx + dispatch_out: the dispatch arrays have not been filled; the kernel dispatches for itself
// and leaves counts / offsets / perm in dispatch_out
static int launch_gate_up(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                          const int32_t *counts, const int32_t *offsets, const int32_t *slot_token,
                          void *h_f16, hipStream_t st, const int32_t *idx, const OdsdDispatchOut *dispatch_out) {
    const int rc = experts_args_ok(s);
    if (rc != ODSD_OK) return rc;
    if (s->T == 0) return ODSD_OK;
    if (!x_f16 || !table || !h_f16) return ODSD_ERR_NULL;
    if (!dispatch_out && (!counts || !offsets || !slot_token)) return ODSD_ERR_NULL;
    if (!odsd_aligned16(x_f16) || !odsd_aligned16(h_f16)) return ODSD_ERR_ALIGN;
    const ExpertsPlan pl = experts_plan(s);
    GemmParams gu{};
    gu.table = table; gu.src = (const half_t *)x_f16; gu.rowmap = slot_token;
    gu.counts = counts; gu.offsets = offsets; gu.h16 = (half_t *)h_f16; gu.y = nullptr;
    gu.src_ld = s->H; gu.G = s->H / ODSD_GROUP; gu.NBLK = 2 * s->I / 16;
    gu.KS = 1; gu.gper = gu.G; gu.PS = pl.PS_gu; gu.ldo = s->I; gu.P = s->T * s->K; gu.E = s->E;
    gu.K = s->K;
    if (dispatch_out) {
        if (!stream_dispatch_supported(pl, s)) return ODSD_ERR_UNSUPPORTED;
        if (!idx || !dispatch_out->counts || !dispatch_out->offsets || !dispatch_out->perm) return ODSD_ERR_NULL;
        if (!odsd_aligned16(idx)) return ODSD_ERR_ALIGN;
        gu.idx = idx;
        gu.out_counts = dispatch_out->counts; gu.out_offsets = dispatch_out->offsets; gu.out_perm = dispatch_out->perm;
    }
    launch_gemm_plan<0>(pl, gu, st);
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_w4_gate_up_silu(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                                    const int32_t *counts, const int32_t *offsets,
                                    const int32_t *slot_token, void *h_f16, void *stream) {
    return launch_gate_up(s, x_f16, table, counts, offsets, slot_token, h_f16, (hipStream_t)stream, nullptr, nullptr);
}

extern "C" int32_t odsd_w4_down_splits(const odsd_moe_shape *s) {
    if (experts_check(s) != ODSD_OK) return 0;
    return experts_plan(s).KS;
}

extern "C" int32_t odsd_experts_one_launch(const odsd_moe_shape *s) {
    const int rc = experts_check(s);
    if (rc != ODSD_OK) return -rc;
    return experts_plan(s).fused;
}

// down: h_f16 [P,I] -> y [KS][P][H] fp32 partial sums over KS slices of I
extern "C" int odsd_w4_down(const odsd_moe_shape *s, const void *h_f16, const uint64_t *table,
                            const int32_t *counts, const int32_t *offsets, void *y, void *stream) {
    const int rc = experts_args_ok(s);
    if (rc != ODSD_OK) return rc;
    if (s->T == 0) return ODSD_OK;
    if (!h_f16 || !table || !counts || !offsets || !y) return ODSD_ERR_NULL;
    if (!odsd_aligned16(h_f16) || !odsd_aligned16(y)) return ODSD_ERR_ALIGN;
    const ExpertsPlan pl = experts_plan(s);
    GemmParams dn{};
    dn.table = table; dn.src = (const half_t *)h_f16; dn.rowmap = nullptr;
    dn.counts = counts; dn.offsets = offsets; dn.h16 = nullptr; dn.y = (float *)y;
    dn.src_ld = s->I; dn.G = s->I / ODSD_GROUP; dn.NBLK = s->H / 16;
    dn.KS = pl.KS; dn.gper = (dn.G + pl.KS - 1) / pl.KS; dn.PS = pl.PS_dn; dn.ldo = s->H; dn.P = s->T * s->K; dn.E = s->E;
    launch_gemm_plan<1>(pl, dn, (hipStream_t)stream);
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

// the whole-row combine is one workgroup per token, 256 threads per 1024 columns
int odsd_combine_norm_supported(const odsd_moe_shape *s) { return s && s->H <= 4096 && s->H % 4 == 0; }

// combine: y partials + routing weights (+ residual) -> out (+ per-row sum of squares of out_act)
// y_slices > 0: y holds that many fp16 partial-sum slices [slice][P][H] (the one-launch expert kernel);
// 0: the layout of the two-launch plan
static int launch_combine(const odsd_moe_shape *s, const void *y_, const int32_t *idx, const float *w,
                          const int32_t *perm, const uint64_t *table, const void *residual,
                          float *out_f32, void *out_act, double *row_ss, hipStream_t st, int y_slices = 0,
                          const OdsdNextNorm *nn = nullptr) {
    const int rc = experts_args_ok(s);
    if (rc != ODSD_OK) return rc;
    if (s->T == 0) return ODSD_OK;
    const float *y = (const float *)y_;
    if (!y || !idx || !w || !perm || !table) return ODSD_ERR_NULL;
    if (!out_f32 && !out_act) return ODSD_ERR_NULL;
    if (row_ss && !out_act) return ODSD_ERR_NULL;
    if (!odsd_aligned16(y) || (out_f32 && !odsd_aligned16(out_f32))) return ODSD_ERR_ALIGN;
    ExpertsPlan pl = experts_plan(s);
    if (y_slices > 0) { pl.KS = y_slices; pl.y_f16 = 1; }
    const int P = s->T * s->K;
    const int nchunk = (s->H / 4 + 255) / 256;
    if ((int64_t)nchunk * s->T > 0x7fffffffLL) return ODSD_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)(nchunk * s->T));
    // rows of 4 pairs fetched together (8: no faster): complete sums, or two fp16 slices
    const bool batched = (pl.KS == 1 || (pl.y_f16 && pl.KS == 2)) && s->K % 4 == 0;
    if (nn) {
        // the whole-row form: the next block's normalised input instead of the row statistic
        if (!odsd_combine_norm_supported(s)) return ODSD_ERR_UNSUPPORTED;
        if (!out_act || out_f32 || row_ss || !nn->norm_w || !nn->xn || !nn->x16) return ODSD_ERR_NULL;
        if (!odsd_aligned16(nn->x16) || !odsd_aligned16(nn->xn)) return ODSD_ERR_ALIGN;
    }
#define COMBINE_GO(XT, YH, ST)                                                                          \
    do {                                                                                                \
        if (batched)                                                                                    \
            ODSD_LAUNCH(ODSD_KERNEL_COMBINE, (combine_kernel<XT, YH, ST, 4>), grid, 256, st, y, idx, w, perm, \
                        table, (const XT *)residual, out_f32, (XT *)out_act, row_ss, s->T, s->H, s->K,  \
                        s->E, pl.KS, P, nchunk);                                                        \
        else                                                                                            \
            ODSD_LAUNCH(ODSD_KERNEL_COMBINE, (combine_kernel<XT, YH, ST, 0>), grid, 256, st, y, idx, w, perm, \
                        table, (const XT *)residual, out_f32, (XT *)out_act, row_ss, s->T, s->H, s->K,  \
                        s->E, pl.KS, P, nchunk);                                                        \
    } while (0)
#define COMBINE_NORM_N(XT, YH, KB)                                                                      \
    ODSD_LAUNCH(ODSD_KERNEL_COMBINE, (combine_norm_kernel<XT, YH, KB>), dim3((unsigned)s->T), 256 * nchunk, st, y, idx, w, \
                perm, table, (const XT *)residual, (XT *)out_act, s->T, s->H, s->K, s->E, pl.KS, P,     \
                (const XT *)nn->norm_w, (double)nn->eps, (XT *)nn->xn, (half_t *)nn->x16)
#define COMBINE_Y(XT, ST)                                    \
    do {                                                     \
        if (nn) {                                            \
            if (pl.y_f16 && pl.KS >= 2) { if (batched) COMBINE_NORM_N(XT, 2, 4); else COMBINE_NORM_N(XT, 2, 0); } \
            else if (pl.y_f16) { if (batched) COMBINE_NORM_N(XT, 1, 4); else COMBINE_NORM_N(XT, 1, 0); }          \
            else { if (batched) COMBINE_NORM_N(XT, 0, 4); else COMBINE_NORM_N(XT, 0, 0); }                        \
        }                                                    \
        else if (pl.y_f16 && pl.KS >= 2) COMBINE_GO(XT, 2, ST);   \
        else if (pl.y_f16) COMBINE_GO(XT, 1, ST);            \
        else COMBINE_GO(XT, 0, ST);                          \
    } while (0)
    if (s->act_dtype == ODSD_DT_BF16) {
        if (row_ss) COMBINE_Y(uint16_t, true);
        else COMBINE_Y(uint16_t, false);
    } else {
        if (row_ss) COMBINE_Y(float, true);
        else COMBINE_Y(float, false);
    }
#undef COMBINE_Y
#undef COMBINE_NORM_N
#undef COMBINE_GO
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_combine(const odsd_moe_shape *s, const void *y, const int32_t *idx, const float *w,
                            const int32_t *perm, const uint64_t *table, const void *residual,
                            float *out_f32, void *out_act, void *stream) {
    return launch_combine(s, y, idx, w, perm, table, residual, out_f32, out_act, nullptr, (hipStream_t)stream);
}

int odsd_launch_experts(const odsd_moe_shape *s, const void *x16, const uint64_t *table, const int32_t *idx,
                        const float *w, const int32_t *counts, const int32_t *offsets, const int32_t *perm,
                        const int32_t *slot_token, const void *residual, float *out_f32, void *out_act,
                        void *ws, size_t ws_bytes, hipStream_t st, double *row_ss,
                        const OdsdDispatchOut *dispatch_out, const OdsdNextNorm *nn) {
    int rc = experts_check(s);
    if (rc != ODSD_OK) return rc;
    if (s->T == 0) return ODSD_OK;
    if (!ws) return ODSD_ERR_NULL;
    if (!odsd_aligned16(ws)) return ODSD_ERR_ALIGN;
    const ExpertsPlan pl = experts_plan(s);
    if (ws_bytes < pl.h_bytes + pl.y_bytes) return ODSD_ERR_WORKSPACE;
    void *h16 = ws;
    float *y = (float *)((char *)ws + pl.h_bytes);
    if (dispatch_out && !(pl.fused ? odsd_fused_dispatch_supported(s->T * s->K) : stream_dispatch_supported(pl, s)))
        return ODSD_ERR_UNSUPPORTED;
    if (pl.fused) {
        if (!x16 || !table || !counts || !offsets || (!slot_token && !dispatch_out)) return ODSD_ERR_NULL;
        if (!odsd_aligned16(x16)) return ODSD_ERR_ALIGN;
        FusedParams fp{};
        fp.table = table; fp.x16 = (const half_t *)x16; fp.rowmap = slot_token;
        fp.counts = counts; fp.offsets = offsets; fp.y = (half_t *)y;
        fp.H = s->H; fp.I = s->I; fp.S = pl.S; fp.P = s->T * s->K;
        fp.G_up = s->H / ODSD_GROUP; fp.G_dn = s->I / ODSD_GROUP;
        fp.K = s->K; fp.E = s->E;
        if (dispatch_out) {
            if (!idx || !dispatch_out->counts || !dispatch_out->offsets || !dispatch_out->perm) return ODSD_ERR_NULL;
            if (!odsd_aligned16(idx)) return ODSD_ERR_ALIGN;
            fp.idx = idx;
            fp.out_counts = dispatch_out->counts; fp.out_offsets = dispatch_out->offsets; fp.out_perm = dispatch_out->perm;
        }
        odsd_launch_experts_fused(fp, s->E, st);
        ODSD_CHECK_LAUNCH();
        return launch_combine(s, y, idx, w, perm, table, residual, out_f32, out_act, row_ss, st, pl.S, nn);
    }
    rc = launch_gate_up(s, x16, table, counts, offsets, slot_token, h16, st, idx, dispatch_out);
    if (rc != ODSD_OK) return rc;
    rc = odsd_w4_down(s, h16, table, counts, offsets, y, st);
    if (rc != ODSD_OK) return rc;
    return launch_combine(s, y, idx, w, perm, table, residual, out_f32, out_act, row_ss, st, 0, nn);
}

// 1: a whole-block call may skip the dispatch kernel for this shape (the expert kernel scans the
// expert ids itself)
int odsd_experts_dispatch_inside(const odsd_moe_shape *s) {
    if (experts_check(s) != ODSD_OK) return 0;
    const ExpertsPlan pl = experts_plan(s);
    return pl.fused ? odsd_fused_dispatch_supported(s->T * s->K) : stream_dispatch_supported(pl, s);
}

extern "C" int odsd_experts_w4(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                               const int32_t *idx, const float *w, const int32_t *counts,
                               const int32_t *offsets, const int32_t *perm, const int32_t *slot_token,
                               const void *residual, float *out_f32, void *out_act, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return odsd_launch_experts(s, x_f16, table, idx, w, counts, offsets, perm, slot_token, residual,
                               out_f32, out_act, workspace, workspace_bytes, (hipStream_t)stream, nullptr,
                               nullptr, nullptr);
}
