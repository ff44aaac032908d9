// Grouped W4A16 expert product for prefill-shaped calls (hundreds of token rows per expert).
//
// With many rows per expert the product is bound by the matrix cores, and what matters is that
// every packed weight is expanded to fp16 exactly once per expert and then shared.  One
// workgroup of 8 wavefronts (two per SIMD, so that one's expansion and LDS traffic hide under
// the other's MFMAs) owns a tile of 256 weight rows x BM token rows and walks the reduction
// dimension in stages of 64 columns:
//   * each wavefront expands 2 of the 16 weight tiles of the stage (int4 -> fp16 in registers,
//     the same bit trick as the streaming kernel) and writes them to LDS in MFMA A-fragment
//     order, [tile][32-column step][lane] x 16 bytes, which every wavefront reads back without
//     bank conflicts;
//   * the token rows of the stage arrive by asynchronous global -> LDS DMA (128 bytes per row,
//     16-byte segments XOR-swizzled by (row >> 1) & 7, conflict-free for the B-fragment reads);
//   * wavefront (wn, wm) multiplies weight tiles 4*wn..4*wn+3 (64 rows) with token blocks
//     MBW*wm..MBW*wm+MBW-1 (16 rows each) on v_mfma_f32_16x16x32_f16: per 32-column step
//     4 A fragments and MBW B fragments feed 4*MBW MFMAs (0.375 KiB of LDS reads per MFMA);
//   * both LDS areas are double buffered; stage s+1 is produced while stage s is multiplied,
//     one raw s_barrier per stage.
// Epilogues are those of the streaming kernel (SiLU(gate)*up -> fp16 h, or fp32 y).
//
// Replaces the same reference code as the streaming kernel: the three F.linear calls of
// expert_forward_with_weights (demo/src/layers/mlp.py:227-230) inside the per-expert loop of
// demo/src/model/qwen3_runner.py:303-380.
#include "w4_gemm.h"

template <int MODE, int MBW>
__global__ __launch_bounds__(512, 2) void w4_gemm_prefill_kernel(const GemmParams p) {
    constexpr int BM = 2 * 16 * MBW;           // token rows per pass
    constexpr int XPT = BM * 8 / 512;          // 16-byte pieces of one token-row stage per thread
    static_assert((BM * 8) % 512 == 0, "token-row pieces must divide among the threads");
    constexpr int XS_STAGE = BM * 128;         // bytes: BM rows x 64 fp16
    constexpr int WS_STAGE = 16 * 2 * 1024;    // bytes: 16 tiles x 2 steps x 64 lanes x 16 B
    // one object per buffer: the compiler must see that the DMA into one buffer cannot alias
    // the reads of the other, or it drains every outstanding load before each LDS read
    __shared__ __attribute__((aligned(16))) char xs0[XS_STAGE];
    __shared__ __attribute__((aligned(16))) char xs1[XS_STAGE];
    __shared__ __attribute__((aligned(16))) char ws0[WS_STAGE];
    __shared__ __attribute__((aligned(16))) char ws1[WS_STAGE];

    // consecutive logical ids stay on one XCD: the row tiles of one expert share its token rows
    const int b = blockIdx.x;
    const int L = (b & 7) * p.wg_per_xcd + (b >> 3);
    if (L >= p.n_wg) return;
    // row chunks innermost: neighbours share the token rows of one (expert, pass, K slice)
    const int chunk = L % p.nchunks;
    const int ks = (L / p.nchunks) % p.KS;
    const int ps = (L / (p.nchunks * p.KS)) % p.PS;
    const int e = L / (p.nchunks * p.KS * p.PS);

    // requested together: one round trip to memory instead of three dependent ones
    const uint64_t *trow = p.table + (size_t)e * ODSD_TABLE_COLS;
    const int M_e = p.counts[e];
    const int base = p.offsets[e];
    const uint64_t t_present = trow[0];
    const uint64_t t_q = MODE == 0 ? trow[0] : trow[2], t_sz = MODE == 0 ? trow[1] : trow[3];
    if (M_e == 0 || t_present == 0) return;
    const global_char *qp_c = (const global_char *)t_q;
    const global_char *szp_c = (const global_char *)t_sz;
    const global_char *src_c = (const global_char *)p.src;
    // gate_up reads its weights through buffer loads: resource in scalar registers, constant
    // per-lane offset, the group as the scalar offset -- no vector instruction per address
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)qp_c, 0, p.NBLK * p.G * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_sz = __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)szp_c, 0, p.NBLK * p.G * 64, 0x00020000);

    const DequantConsts dc = dequant_consts();
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    const int wn = wave & 3, wm = wave >> 2;
    const int G = p.G;
    const int NST = 2 * G;                     // stages of 64 columns
    const int g_begin = ks * p.gper, g_end = min(G, g_begin + p.gper);   // this K slice (never empty)

    // expansion duty: tiles 2*wave and 2*wave+1 of this row chunk (clamped, never out of range)
    uint32_t wq_off[2], sz_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        uint32_t blk = chunk * 16 + 2 * wave + i;
        if (blk >= (uint32_t)p.NBLK) blk = 0;
        wq_off[i] = (blk * G * 64 + lane) * 16u;
        sz_off[i] = (blk * G * 16 + r) * 4u;
    }
    // product duty: tiles 4*wn .. 4*wn+3
    const int cblk0 = chunk * 16 + 4 * wn;
    bool blk_ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) blk_ok[i] = cblk0 + i < p.NBLK;

    for (int m0 = ps * BM; m0 < M_e; m0 += p.PS * BM) {
        const int mcnt = min(M_e - m0, BM);
        const int mrows_w = max(0, min(mcnt - wm * 16 * MBW, 16 * MBW));   // rows of this M half
        const int nmb = (mrows_w + 15) >> 4;

        // token-row pieces of this thread: piece = i*512 + tid -> row = piece/8, segment = piece%8,
        // fetched from source segment  segment ^ ((row >> 1) & 7)
        uint32_t st_off[XPT];
#pragma unroll
        for (int i = 0; i < XPT; ++i) {
            const int piece = i * 512 + tid;
            const int row = piece >> 3, seg = piece & 7;
            const int slot = base + m0 + (row < mcnt ? row : 0);
            const int srow = p.rowmap ? p.rowmap[slot] : slot;
            st_off[i] = ((uint32_t)srow * (uint32_t)p.src_ld + (seg ^ ((row >> 1) & 7)) * 8) * 2u;
        }

        float4_t acc[4][MBW];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int m = 0; m < MBW; ++m) acc[i][m] = float4_t{0.f, 0.f, 0.f, 0.f};

        uint4_t wq[2][2];      // [ring slot = group parity][duty tile]
        uint32_t wsz[2][2];

        auto load_w = [&](int slot, int g) {
            const uint32_t gc = (uint32_t)min(g, G - 1);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                if (MODE == 0) {
                    wq[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, (int)wq_off[i], (int)(gc * 1024u), 2 /* nt */);
                    wsz[slot][i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_sz, (int)sz_off[i], (int)(gc * 64u), 0);
                } else {
                    // (the down projection measured 14 % slower with buffer loads)
                    wq[slot][i] = __builtin_nontemporal_load((const global_u4 *)(qp_c + (wq_off[i] + gc * 1024u)));
                    wsz[slot][i] = *(const global_u32 *)(szp_c + (sz_off[i] + gc * 64u));
                }
            }
        };
        auto dma_x = [&](char *xs, int st) {
            const uint32_t sc = (uint32_t)min(st, NST - 1);
#pragma unroll
            for (int i = 0; i < XPT; ++i) {
                // piece i covers rows 64 i .. 64 i + 63 of the pass: nothing to fetch past its last row
                if (i * 64 < mcnt) {
                    lds_void *dst = (lds_void *)(xs + (i * 512 + wave * 64) * 16);
                    dma16_to_lds(src_c, st_off[i] + sc * 128u, dst);
                }
            }
        };
        // expand the two 32-column steps `half` (0: words x,y  1: words z,w) of ring slot `slot`
        // into weight buffer `buf`
        auto expand = [&](int slot, int half, char *ws) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const DequantPrep pr = dequant_prep(wsz[slot][i]);
                const uint32_t w0 = half ? wq[slot][i].z : wq[slot][i].x;
                const uint32_t w1 = half ? wq[slot][i].w : wq[slot][i].y;
                char *dst = ws + (((2 * wave + i) * 2) * 64 + lane) * 16;
                *(half8_t *)dst = dequant_word(dc, pr, w0);
                *(half8_t *)(dst + 1024) = dequant_word(dc, pr, w1);
            }
        };
        // one quarter of expand(): duty tile i, word w of the half
        auto expand_piece = [&](int slot, int half, char *ws, int i, int w) {
            const DequantPrep pr = dequant_prep(wsz[slot][i]);
            const uint32_t word = half ? (w ? wq[slot][i].w : wq[slot][i].z) : (w ? wq[slot][i].y : wq[slot][i].x);
            char *dst = ws + (((2 * wave + i) * 2) * 64 + lane) * 16 + w * 1024;
            *(half8_t *)dst = dequant_word(dc, pr, word);
        };
        // multiply stage (xs, ws) and, in the same scheduling region, expand the next stage's
        // weights (ring slot eslot, half ehalf) into ews, so that the vector work and the LDS
        // writes of the expansion sit between the MFMAs instead of in front of them
        auto mma_stage = [&](const char *xs, const char *ws, int eslot, int ehalf, char *ews) {
            if (nmb == MBW) {
                // Every token block of this wavefront is in use: branch-free and software
                // pipelined.  The stage is cut into units of 2 token blocks x one 32-column
                // step.  The LDS reads of unit u+1 are issued, then (behind a scheduling fence
                // that keeps them there) the 8 MFMAs of unit u, so the read latency hides under
                // the matrix work of the same wavefront.  The expansion of the next stage's
                // weights is cut into 4 pieces that ride along with the first 4 units.
                static_assert(MBW % 2 == 0, "token blocks are processed in pairs");
                constexpr int UPJ = MBW / 2;           // units per 32-column step
                auto read_a = [&](int jj, half8_t (&a)[4]) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        a[i] = *(const half8_t *)(ws + ((((4 * wn + i) * 2) + jj) * 64 + lane) * 16);
                };
                auto read_b = [&](int jj, int m, half8_t &bx) {
                    const int row = wm * 16 * MBW + m * 16 + r;
                    const int seg = (4 * jj + kq) ^ ((row >> 1) & 7);
                    bx = *(const half8_t *)(xs + row * 128 + seg * 16);
                };
                half8_t a_cur[4], a_nxt[4], b_cur[2], b_nxt[2];
                read_a(0, a_cur);
                read_b(0, 0, b_cur[0]);
                read_b(0, 1, b_cur[1]);
#define PF_UNIT(U)                                                                                      \
    {                                                                                                   \
        constexpr int mp = (U) % UPJ;                                                                   \
        if ((U) + 1 < 2 * UPJ) {                                                                        \
            constexpr int jn = ((U) + 1) / UPJ, mn = ((U) + 1) % UPJ;                                   \
            if (mn == 0) read_a(jn, a_nxt);                                                             \
            read_b(jn, 2 * mn, b_nxt[0]);                                                               \
            read_b(jn, 2 * mn + 1, b_nxt[1]);                                                           \
        }                                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        if ((U) < 4) expand_piece(eslot, ehalf, ews, (U) >> 1, (U) & 1);                                \
        _Pragma("unroll") for (int q = 0; q < 2; ++q)                                                   \
        _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                   \
            acc[i][2 * mp + q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur[i], b_cur[q], acc[i][2 * mp + q], 0, 0, 0);                       \
        __builtin_amdgcn_sched_barrier(0);                                                              \
        if ((U) + 1 < 2 * UPJ) {                                                                        \
            if (((U) + 1) % UPJ == 0) {                                                                 \
                _Pragma("unroll") for (int i = 0; i < 4; ++i) a_cur[i] = a_nxt[i];                      \
            }                                                                                           \
            b_cur[0] = b_nxt[0];                                                                        \
            b_cur[1] = b_nxt[1];                                                                        \
        }                                                                                               \
    }
                static_assert(MBW == 8, "the unit list below is written out for 8 token blocks");
                PF_UNIT(0) PF_UNIT(1) PF_UNIT(2) PF_UNIT(3)
                PF_UNIT(4) PF_UNIT(5) PF_UNIT(6) PF_UNIT(7)
#undef PF_UNIT
            } else {
                expand(eslot, ehalf, ews);
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    half8_t a[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        a[i] = *(const half8_t *)(ws + ((((4 * wn + i) * 2) + jj) * 64 + lane) * 16);
#pragma unroll
                    for (int m = 0; m < MBW; ++m) {
                        if (m < nmb) {
                            const int row = wm * 16 * MBW + m * 16 + r;
                            const int seg = (4 * jj + kq) ^ ((row >> 1) & 7);
                            const half8_t bx = *(const half8_t *)(xs + row * 128 + seg * 16);
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                acc[i][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], bx, acc[i][m], 0, 0, 0);
                        }
                    }
                }
            }
        };

        // prologue: stage 0 in place
        __builtin_amdgcn_s_barrier();          // the previous pass is done with both LDS areas
        dma_x(xs0, 2 * g_begin);
        load_w(0, g_begin);
        load_w(1, g_begin + 1);
        __builtin_amdgcn_sched_barrier(0);
        expand(0, 0, ws0);
        __builtin_amdgcn_sched_barrier(0);
        ODSD_WAIT_VMCNT_LGKM0(4);              // all but the second group's 4 loads have landed
        __builtin_amdgcn_s_barrier();

        // two groups (four stages) per trip: ring slots and buffers are compile-time constants
        for (int g = g_begin; g < g_end; g += 2) {
            // stage 4k   : group g, first half.   produce (g, second half) -> x buf 1, w buf 1
            dma_x(xs1, 2 * g + 1);
            __builtin_amdgcn_sched_barrier(0);
            mma_stage(xs0, ws0, 0, 1, ws1);
            __builtin_amdgcn_sched_barrier(0);
            load_w(0, g + 2);                  // slot 0 is fully expanded
            __builtin_amdgcn_sched_barrier(0);
            ODSD_WAIT_VMCNT_LGKM0(4);          // the DMA is older than the 4 refill loads
            __builtin_amdgcn_s_barrier();
            // stage 4k+1 : group g, second half.  produce (g+1, first half) -> x buf 0, w buf 0
            dma_x(xs0, 2 * g + 2);
            __builtin_amdgcn_sched_barrier(0);
            mma_stage(xs1, ws1, 1, 0, ws0);
            __builtin_amdgcn_sched_barrier(0);
            ODSD_WAIT_VMCNT_LGKM0(0);
            __builtin_amdgcn_s_barrier();
            if (g + 1 >= g_end) break;
            // stage 4k+2 : group g+1, first half.  produce (g+1, second half) -> buffers 1
            dma_x(xs1, 2 * g + 3);
            __builtin_amdgcn_sched_barrier(0);
            mma_stage(xs0, ws0, 1, 1, ws1);
            __builtin_amdgcn_sched_barrier(0);
            load_w(1, g + 3);
            __builtin_amdgcn_sched_barrier(0);
            ODSD_WAIT_VMCNT_LGKM0(4);
            __builtin_amdgcn_s_barrier();
            // stage 4k+3 : group g+1, second half.  produce (g+2, first half) -> buffers 0
            dma_x(xs0, 2 * g + 4);
            __builtin_amdgcn_sched_barrier(0);
            mma_stage(xs1, ws1, 0, 0, ws0);
            __builtin_amdgcn_sched_barrier(0);
            ODSD_WAIT_VMCNT_LGKM0(0);
            __builtin_amdgcn_s_barrier();
        }

        // epilogue: lane holds rows 4*kq..4*kq+3 of each 16-row tile, token column r
#pragma unroll
        for (int m = 0; m < MBW; ++m) {
            const int row = wm * 16 * MBW + m * 16 + r;
            if (m < nmb && row < mcnt) {
                const size_t slot = (size_t)(base + m0 + row);
                if (MODE == 0) {
#pragma unroll
                    for (int i = 0; i < 4; i += 2) {
                        if (blk_ok[i]) {
                            const float4_t gt = acc[i][m], up = acc[i + 1][m];
                            half4_t h;
                            h.x = f32_to_f16_sat(silu_f32(gt.x) * up.x);
                            h.y = f32_to_f16_sat(silu_f32(gt.y) * up.y);
                            h.z = f32_to_f16_sat(silu_f32(gt.z) * up.z);
                            h.w = f32_to_f16_sat(silu_f32(gt.w) * up.w);
                            const int feat = ((cblk0 + i) >> 1) * 16 + kq * 4;
                            *(half4_t *)(p.h16 + slot * p.ldo + feat) = h;
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (blk_ok[i]) {
                            const int n = (cblk0 + i) * 16 + kq * 4;
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
    }
}

template <int MODE>
void odsd_launch_gemm_prefill(GemmParams &gp, hipStream_t st) {
    gp.nchunks = (gp.NBLK + 15) / 16;
    if (gp.PS < 1) gp.PS = 1;
    gp.n_wg = gp.E * gp.nchunks * gp.KS * gp.PS;
    gp.wg_per_xcd = (gp.n_wg + 7) / 8;
    ODSD_LAUNCH(MODE == 0 ? ODSD_KERNEL_GATE_UP : ODSD_KERNEL_DOWN, (w4_gemm_prefill_kernel<MODE, 8>),
                gp.wg_per_xcd * 8, 512, st, gp);
}

template void odsd_launch_gemm_prefill<0>(GemmParams &, hipStream_t);
template void odsd_launch_gemm_prefill<1>(GemmParams &, hipStream_t);
