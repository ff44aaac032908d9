// One launch per MoE block for the experts of verify-shaped calls on models with many small
// experts (Qwen3-30B-A3B: hidden 2048, 128 experts of intermediate 768, 8-32 rows per expert).
//
// The two-launch form (w4_gemm_kernel, MODE 0 then MODE 1) moves as many token-row bytes
// L2 -> LDS as it streams weight bytes from HBM -- every workgroup copies its expert's rows for
// every 128-column group, with a barrier per group -- and pays a launch ramp twice.  Here one
// workgroup of 8 wavefronts owns (expert, slice s of S of the intermediate features) for the
// whole block:
//   * the expert's token rows (at most 16*MB rows x H fp16 = 128 KB) are copied into LDS ONCE,
//     by asynchronous global -> LDS loads, in the B-fragment order of v_mfma_f32_16x16x32_f16
//     ([group][token block][16 rows x 256 B], 16-byte segments XOR-swizzled by the row);
//   * gate_up: each wavefront owns whole (gate block, up block) pairs of the slice and walks them
//     pair after pair, group after group: one step = the two 1 KiB tiles of one group, fetched by
//     buffer loads through a register ring 4 steps deep (two ascending 16 KiB runs per pair) and
//     multiplied with the group's fragments read from LDS; no barrier in the stream;
//   * the codes go to the matrix cores as they are (offset + q as fp16, two logic instructions per
//     4 weights); the offsets leave through the accumulator's start value, and scale and zero point
//     are applied to each group's sum, acc += scale * (sum q x - zero * sum x), in fp32 -- the
//     per-weight (q - zero) * scale in fp16 is what the two-launch kernels spend most of their
//     vector instructions on, and with one workgroup per CU this kernel is bound by those;
//   * h = SiLU(gate) * up of a pair (16*MB rows x 16 features, fp16) goes to LDS in the same
//     fragment order when the pair's last group is done; one barrier after the last pair;
//   * down: the same stream over pairs of output row blocks, the slice's GS groups of each (the
//     ring runs on from gate_up into down without draining), against h from LDS; fp16 partial sums
//     y[s][slot][H] are stored per pair; the combine adds the S slices in order.
// Workgroups hold 157 KB of LDS, so exactly one is resident per CU: E*S is chosen near the CU
// count and every workgroup streams the same number of bytes.
//
// Skewed routing.  A pass holds 16*MB rows.  The rows of an expert beyond its first pass form further
// units of work (expert, slice, pass), and these are NOT left to the expert's own two workgroups
// (which would stream their slices again and again while the rest of the chip has finished): every
// workgroup knows the row count of every expert, so all of them derive the same list of overflow
// units and the same order of helpers -- the workgroups with the fewest rows of their own first --
// and helper r takes units r, r + grid, ...  No queue, no atomics, no waiting between workgroups;
// with no expert beyond one pass (the usual case) nothing of this runs.
//
// Replaces the same reference code as the streaming kernels: the three F.linear calls of
// expert_forward_with_weights (demo/src/layers/mlp.py:227-230) inside the per-expert loop of
// demo/src/model/qwen3_runner.py:303-380.
#include "w4_gemm.h"

#include <type_traits>

// Codes as fp16 without the per-weight scale and zero point.  (x & mask) | magic turns a nibble pair
// into fp16 values offset + q: the low nibbles of the two halves of a word with magic 0x6400
// (1024 + q, one unit in the last place = 1), the high nibbles with 0x5400 (64 + q, one unit in the
// last place = 1/16, so the nibble's 16 q is q).  Element order of the result is that of the MFMA A
// operand: (k0,k1) and (k4,k5) carry 1024 + q, (k2,k3) and (k6,k7) carry 64 + q.  The offsets are
// taken out again through the accumulator's start value (see group_sums), and scale and zero point
// are applied to the group's sum instead of to every weight: 5 vector instructions per 8 weights
// instead of 13.
struct RawConsts {
    uint32_t m_lo, m_hi, magic_lo, magic_hi;
};
__device__ __forceinline__ RawConsts raw_consts() {
    RawConsts c{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.m_lo), "+s"(c.m_hi), "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}
__device__ __forceinline__ half8_t raw_word(const RawConsts &c, const uint32_t x) {
    const uint32_t xs = x >> 8;
    const uint4_t t = {(x & c.m_lo) | c.magic_lo, (x & c.m_hi) | c.magic_hi, (xs & c.m_lo) | c.magic_lo,
                       (xs & c.m_hi) | c.magic_hi};
    return __builtin_bit_cast(half8_t, t);
}
#define ODSD_RAW_OFFSET_LO 1024.0f
#define ODSD_RAW_OFFSET_HI 64.0f

typedef float float2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint64_t uniform_u64(const uint64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// Nothing moves across this point: the scheduling fence binds the machine scheduler, the empty
// statement with a memory clobber binds the instruction selector's ordering of a long straight-line
// block (without it the loads of many later steps are hoisted to the top of the unrolled stream and
// their results spilled).
#define ODSD_FENCE()                         \
    do {                                     \
        __builtin_amdgcn_sched_barrier(0);   \
        asm volatile("" ::: "memory");       \
        __builtin_amdgcn_sched_barrier(0);   \
    } while (0)

// MB    16-row token blocks held per pass (an expert with more rows takes further passes)
// GS    128-column groups of the intermediate dimension per slice (slice = 128*GS features)
// WAVES wavefronts per workgroup
// G_UP  H / 128, G_DN  I / 128: groups of the two reductions (compile time: every tile offset of
//       a wavefront's stream is a constant)
// DISP  0, or the number of 4-id vectors per thread (1 or 2) with which the workgroup dispatches
//       for itself: it scans the [P] expert ids (P <= 4 * DISP * 64 * WAVES, consecutive ids per
//       thread), counts the pairs of its expert and of lower experts (ballot /
//       popcount, the order of the pair list is kept: stable), keeps its expert's token rows in LDS
//       and, as slice 0, writes counts[e], offsets[e] and the slots of its pairs -- what the
//       separate dispatch kernel and two dependent loads per workgroup did before
// Timing-only build (-DODSD_TIMELINE, `make timeline`): every wavefront stamps the 100 MHz real-time
// counter at eight points and leaves the stamps in a buffer the caller registered, 8 values per
// (workgroup, wavefront).  The product build compiles none of it.
#ifdef ODSD_TIMELINE
__device__ unsigned long long *odsd_tl_buf;
extern "C" int odsd_debug_timeline(void *buf) {
    unsigned long long *b = (unsigned long long *)buf;
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(odsd_tl_buf), &b, sizeof(b));
}
#define ODSD_TL(k) tl[k] = __builtin_amdgcn_s_memrealtime()
#else
#define ODSD_TL(k)
#endif

template <int MB, int GS, int WAVES, int G_UP, int G_DN, int DISP>
__global__ __launch_bounds__(64 * WAVES, WAVES / 4) void w4_expert_fused_kernel(const FusedParams p) {
    static_assert(WAVES % 4 == 0 && (8 * GS) % WAVES == 0, "whole gate/up block pairs per wavefront");
    static_assert(G_UP * MB <= ODSD_FUSED_X_BLOCKS, "token rows of a pass must fit the LDS area");
    static_assert(MB == 1 || MB == 2, "one or two token blocks");
    constexpr int PPW = 8 * GS / WAVES;          // gate/up block pairs per wavefront
    constexpr int NT = PPW * G_UP;               // gate_up steps of a wavefront: pair after pair, group after group
    constexpr int DPAIRS = G_UP * 4;             // pairs of down row blocks: H / 32
    constexpr int DP_MIN = DPAIRS / WAVES, DP_EXTRA = DPAIRS % WAVES;   // the first DP_EXTRA wavefronts take one more
    constexpr int NTD = (DP_MIN + (DP_EXTRA ? 1 : 0)) * GS;             // most down steps any wavefront runs
    constexpr int DEPTH = 4;                     // ring: steps (two tiles each) in flight
    constexpr int XBLK = 4096;                   // bytes of one (group, token block): 16 rows x 256 B
    static_assert(NT >= DEPTH && DP_MIN * GS >= DEPTH, "ring deeper than a stream");
    __shared__ __attribute__((aligned(16))) char xs_raw[ODSD_FUSED_X_BLOCKS * XBLK];
    __shared__ __attribute__((aligned(16))) char hs_raw[GS * MB * XBLK];
    // per (group, token block) and token row: (sum of offset_k * x_k, sum of x_k) over the group's 128
    // columns -- the token rows' blocks first, the blocks of h after them
    __shared__ float2_t cx[(G_UP + GS) * MB * 16];
    __shared__ int32_t rows_lds[16 * MB];        // DISP: tokens of the pass's rows
    __shared__ int32_t wsum[2][WAVES];           // DISP: per-wavefront totals (pairs of e, pairs below e)
    __shared__ int32_t cnt_all[ODSD_FUSED_MAX_E];   // DISP: rows of every expert (histogram of the id list)
    __shared__ int32_t helper_lds[WAVES];        // overflow units: per-wavefront counts of the helper order

    constexpr int ROWS = 16 * MB;                // rows of one pass
#ifdef ODSD_TIMELINE
    unsigned long long tl[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
    ODSD_TL(0);
    constexpr int NID = DISP ? 4 * DISP : 1;     // ids per thread
    const int b = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, kq = lane >> 4;
    const int pair0 = NID * tid;

    // The expert ids of this thread's pairs (DISP): 4 or 8 consecutive ones, one or two 16-byte loads.
    auto load_ids = [&](int (&id)[NID]) {
#pragma unroll
        for (int v = 0; v < NID / 4; ++v) {
            uint4_t w = {~0u, ~0u, ~0u, ~0u};
            if (pair0 + 4 * v < p.P) w = *(const uint4_t *)(p.idx + pair0 + 4 * v);   // P is a multiple of 4
            id[4 * v] = (int)w.x; id[4 * v + 1] = (int)w.y; id[4 * v + 2] = (int)w.z; id[4 * v + 3] = (int)w.w;
        }
    };
    // DISP: one scan of the id list for expert e_: its row count, its first slot, and the tokens of its
    // rows m0_ .. m0_ + ROWS - 1 (into rows_lds); the order of the pair list is kept (stable).  `first`
    // (the workgroup's own unit): the histogram of all experts is made on the way, and slice 0 writes
    // counts[e], offsets[e] and the slots of the expert's pairs -- what a separate dispatch kernel and
    // two dependent loads per workgroup did before.  Ends with a barrier.
    auto scan_for = [&](const int (&id)[NID], const int e_, const int m0_, const bool first, const bool writer,
                        int &M_out, int &base_out) {
        int cm = 0, cl = 0;
#pragma unroll
        for (int j = 0; j < NID; ++j) {
            cm += id[j] == e_;
            cl += (uint32_t)id[j] < (uint32_t)e_;   // ids outside [0, E) belong to nobody
        }
        if (first) {
#pragma unroll
            for (int j = 0; j < NID; ++j)
                if ((uint32_t)id[j] < (uint32_t)p.E) atomicAdd(&cnt_all[id[j]], 1);
        }
        // counts of at most NID per lane: one ballot per bit gives the prefix over the lower lanes and the total
        constexpr int NBITS = DISP == 1 ? 3 : 4;
        int pre = 0, tot_eq = 0, tot_lt = 0;
#pragma unroll
        for (int bit = 0; bit < NBITS; ++bit) {
            const uint64_t mb = __ballot(cm & (1 << bit)), lb = __ballot(cl & (1 << bit));
            pre += mask_rank(mb) << bit;
            tot_eq += __popcll(mb) << bit;
            tot_lt += __popcll(lb) << bit;
        }
        if (!first) __syncthreads();              // the previous unit is done with wsum and rows_lds
        if (lane == 0) {
            wsum[0][wave] = tot_eq;
            wsum[1][wave] = tot_lt;
        }
        __syncthreads();
        int before = 0, tot_m = 0, tot_l = 0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const int a = wsum[0][w];
            if (w < wave) before += a;
            tot_m += a;
            tot_l += wsum[1][w];
        }
        M_out = __builtin_amdgcn_readfirstlane(tot_m);
        base_out = __builtin_amdgcn_readfirstlane(tot_l);
        int rank = before + pre;
        if (writer && tid == 0) {
            p.out_counts[e_] = tot_m;
            p.out_offsets[e_] = tot_l;
            if (e_ == p.E - 1) p.out_offsets[p.E] = tot_l + tot_m;
        }
#pragma unroll
        for (int j = 0; j < NID; ++j) {
            if (id[j] == e_) {
                const int rel = rank - m0_;
                if (rel >= 0 && rel < ROWS) rows_lds[rel] = (pair0 + j) / p.K;
                // (the ids come from this library's router, so every pair belongs to some expert's workgroup)
                if (writer) p.out_perm[pair0 + j] = tot_l + rank;
                ++rank;
            }
        }
        __syncthreads();                          // the row list is complete
    };
    // rows of expert x as every workgroup sees them
    auto rows_of = [&](const int x) -> int { return DISP ? cnt_all[x] : p.counts[x]; };

    // ---- the workgroup's own unit: (expert b / S, slice b % S), the expert's first ROWS rows ----------
    int e = b / p.S, s = b - e * p.S;
    // everything the prologue depends on is requested at once (one round trip, not three)
    const uint64_t *trow = p.table + (size_t)e * ODSD_TABLE_COLS;
    uint64_t t_gu_q = trow[0], t_gu_sz = trow[1], t_dn_q = trow[2], t_dn_sz = trow[3];
    int M_e, base, m0 = 0;
    if (DISP) {
        int id[NID];
        load_ids(id);                             // on its way together with the table row
        for (int x = tid; x < p.E; x += 64 * WAVES) cnt_all[x] = 0;
        __syncthreads();
        scan_for(id, e, 0, true, s == 0, M_e, base);
    } else {
        M_e = p.counts[e];
        base = p.offsets[e];
    }
    // After its own unit: does any expert have more rows than one pass holds?  (every wavefront looks
    // at all counts)  If so -- rare -- the overflow units: unit u = (expert, pass >= 1, slice), experts
    // ascending, passes ascending, slices ascending; helper order = workgroups by (rows of their own
    // expert, workgroup id) ascending; this workgroup, helper number `helper`, takes units helper,
    // helper + grid, ...
    int n_units = 0, helper = 0;
    auto overflow_plan = [&]() -> bool {
        bool any_over = false;
        for (int x = lane; x < p.E; x += 64) any_over |= rows_of(x) > ROWS;
        if (!__any(any_over)) return false;
        for (int x = 0; x < p.E; ++x) n_units += ((rows_of(x) + ROWS - 1) / ROWS > 1 ? (rows_of(x) + ROWS - 1) / ROWS - 1 : 0) * p.S;
        const int mine = rows_of(b / p.S);
        int below = 0;
        for (int o = tid; o < (int)gridDim.x; o += 64 * WAVES) {
            const int oc = rows_of(o / p.S);
            below += (oc < mine || (oc == mine && o < b)) ? 1 : 0;
        }
        below = (int)wave_sum((float)below);      // at most 64 * ceil(grid / 512) per wavefront: exact in fp32
        __syncthreads();                          // (the own unit's readers of helper_lds's neighbours are done)
        if (lane == 0) helper_lds[wave] = below;
        __syncthreads();
        for (int w = 0; w < WAVES; ++w) helper += helper_lds[w];
        helper = __builtin_amdgcn_readfirstlane(helper);
        n_units = __builtin_amdgcn_readfirstlane(n_units);
        return true;
    };

    ODSD_TL(1);                                  // own id scan done
    for (int it = 0;; ++it) {
    if (it > 0) {
        if (it == 1 && !overflow_plan()) break;
        const int u = helper + (it - 1) * (int)gridDim.x;
        if (u >= n_units) break;
        // decode unit u
        int acc_u = 0, ue = 0, upass = 0, us = 0;
        for (int x = 0; x < p.E; ++x) {
            const int np = (rows_of(x) + ROWS - 1) / ROWS;
            const int nu = (np > 1 ? np - 1 : 0) * p.S;
            if (u < acc_u + nu) {
                ue = x;
                upass = 1 + (u - acc_u) / p.S;
                us = (u - acc_u) % p.S;
                break;
            }
            acc_u += nu;
        }
        // (wavefront-uniform values that came through LDS: back into scalar registers, so that the table
        // row is a scalar load and the buffer resources are built on the scalar unit)
        e = __builtin_amdgcn_readfirstlane(ue);
        s = __builtin_amdgcn_readfirstlane(us);
        m0 = __builtin_amdgcn_readfirstlane(upass) * ROWS;
        trow = p.table + (size_t)e * ODSD_TABLE_COLS;
        t_gu_q = trow[0]; t_gu_sz = trow[1]; t_dn_q = trow[2]; t_dn_sz = trow[3];
        if (DISP) {
            int id[NID];
            load_ids(id);
            scan_for(id, e, m0, false, false, M_e, base);
        } else {
            M_e = p.counts[e];
            base = p.offsets[e];
        }
    }
    if (M_e <= m0 || t_gu_q == 0) continue;
    // the table row is the same in every lane: say so (the buffer resources built from it must live in
    // scalar registers, or every load is wrapped in a loop over the distinct values)
    t_gu_q = uniform_u64(t_gu_q); t_gu_sz = uniform_u64(t_gu_sz);
    t_dn_q = uniform_u64(t_dn_q); t_dn_sz = uniform_u64(t_dn_sz);
    const global_char *src_c = (const global_char *)p.x16;
    // the expert's packed matrices and their (scale, zero) pairs as buffer resources (reads past
    // the end return zero)
    const __amdgpu_buffer_rsrc_t rsrc_qu = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_gu_q, 0, (2 * p.I / 16) * G_UP * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_szu = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_gu_sz, 0, (2 * p.I / 16) * G_UP * 64, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_qd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_dn_q, 0, (p.H / 16) * G_DN * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_szd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(uintptr_t)t_dn_sz, 0, (p.H / 16) * G_DN * 64, 0x00020000);

    const RawConsts rc = raw_consts();

    // gate_up duty: block pairs of the slice (the slice owns the fused matrix's blocks
    // s*16*GS .. (s+1)*16*GS - 1).  A pair is 2 * G_UP KiB of contiguous tiles -- [gate block][group],
    // then [up block][group] -- and the wavefront walks it group by group, so it reads two ascending
    // runs of G_UP KiB; tile (pair i, block j, group g) sits at the compile-time offset
    // ((2 i + j) * G_UP + g) KiB from the wavefront's first tile.
    const int ublk0 = s * (16 * GS) + wave * (2 * PPW);
    const uint32_t uq_off = ((uint32_t)ublk0 * G_UP * 64 + lane) * 16u;
    // (scale, zero) pairs are fetched in accumulator order: the lane's 4 output rows 4*kq .. 4*kq+3 are
    // 16 contiguous bytes of a tile's 64
    const uint32_t usz_off = ((uint32_t)ublk0 * G_UP * 16 + 4 * kq) * 4u;
    // down duty: pairs of output row blocks; of each block's G_DN tiles the slice reads the GS
    // contiguous ones from s*GS on
    const int npairs_w = DP_MIN + (wave < DP_EXTRA ? 1 : 0);
    const int ntd_w = npairs_w * GS;
    const int dblk0 = 2 * (wave * DP_MIN + min(wave, DP_EXTRA));
    const uint32_t dq_off = (((uint32_t)dblk0 * G_DN + s * GS) * 64 + lane) * 16u;
    const uint32_t dsz_off = (((uint32_t)dblk0 * G_DN + s * GS) * 16 + 4 * kq) * 4u;

    // LDS byte offset of this lane's B fragment of 32-column step j inside a (group, token block):
    // row r, logical segment 4j + kq, stored at segment ^ r
    uint32_t lds_frag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) lds_frag[j] = (uint32_t)((r * 16 + ((4 * j + kq) ^ r)) * 16);

    // token-row copies: one copy instruction moves 4 rows x 256 B (lane -> row lane / 16, stored
    // segment lane % 16).  A wavefront always copies the same quarter of the same token block, for
    // one group per instruction, so it needs one source row per lane.
    // (the first 8 wavefronts copy; the others have none)
    const int quarter = wave & 3;
    const int dm = MB == 2 ? ((wave >> 2) & 1) : 0;           // token block this wavefront copies
    const int row_in_blk = 4 * quarter + kq;
    constexpr int N_PIECES = G_UP * MB / 2;                   // copies per wavefront

    {
        const int mcnt = min(M_e - m0, ROWS);
        // the previous unit is done with both LDS areas (DISP: its scan has passed barriers since)
        if (!DISP && it > 0) __syncthreads();
        // The pass is compiled once per number of token blocks that hold rows: with a run-time count
        // the values that exist on one path only (fragments, group sums, the second block's partial
        // sums) stay live across the whole unrolled stream.
        auto run_pass = [&](auto nmb_c) {
        constexpr int nmb = decltype(nmb_c)::value;

        // One ring for both phases: slot = step % DEPTH holds the two tiles of a step.
        uint4_t wq[DEPTH][2];
        uint4_t wsz[DEPTH][2];
        auto load_u = [&](const int slot, const int t) {      // gate_up step t
            const int tile = 2 * (t / G_UP) * G_UP + t % G_UP;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                wq[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_qu, (int)uq_off, (tile + i * G_UP) * 1024, 2 /* nt */);
                wsz[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_szu, (int)usz_off, (tile + i * G_UP) * 64, 0);
            }
        };
        auto load_d = [&](const int slot, const int u) {      // down step u
            const int tile = 2 * (u / GS) * G_DN + u % GS;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                wq[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_qd, (int)dq_off, (tile + i * G_DN) * 1024, 2 /* nt */);
                wsz[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_szd, (int)dsz_off, (tile + i * G_DN) * 64, 0);
            }
        };
        // rows past the expert's last one are clamped to the first row of the pass: the MFMA
        // columns they feed are never stored
        {
            const int row = dm * 16 + row_in_blk;
            const int slot = base + m0 + (row < mcnt ? row : 0);
            const int srow = DISP ? rows_lds[row < mcnt ? row : 0] : p.rowmap[slot];
            const uint32_t st_off = ((uint32_t)srow * (uint32_t)p.H + (uint32_t)((r ^ row_in_blk) * 8)) * 2u;
            if (dm < nmb && wave < 8) {
                for (int i = 0; i < N_PIECES; ++i) {
                    const int g = MB == 2 ? i : 2 * i + ((wave >> 2) & 1);
                    lds_void *dst = (lds_void *)(xs_raw + (g * MB + dm) * XBLK + quarter * 1024);
                    dma16_to_lds(src_c + (size_t)g * (ODSD_GROUP * 2u), st_off, dst);
                }
            }
        }
        // The ring's first loads go out behind the copies and are not waited for: the group sums
        // below run while they travel (issued in front of the copies they would have to land
        // first -- the counter is in order -- and memory would idle during the sums: 1.3 us).
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) load_u(d, d);
        ODSD_WAIT_VMCNT(4 * DEPTH);                           // the copies have landed; 4 loads per ring step are younger
        __builtin_amdgcn_s_barrier();
        ODSD_TL(2);                                           // token rows in LDS

        // Sums of one (group, token block): the lane reads its four B fragments (token row r, columns
        // 32 j + 8 kq ..), adds the values at the 1024-offset positions and at the 64-offset positions
        // in fp32, the four kq parts are added across the lanes (same order in every lane), and the
        // lanes of kq = 0 store (1024 * lo + 64 * hi, lo + hi) for their row.
        auto group_sums = [&](const char *blk, float2_t *dst) {
            float lo = 0.f, hi = 0.f;
            const half2_t one = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half8_t f = *(const half8_t *)(blk + lds_frag[j]);
                lo = __builtin_amdgcn_fdot2(half2_t{f[0], f[1]}, one, lo, false);
                hi = __builtin_amdgcn_fdot2(half2_t{f[2], f[3]}, one, hi, false);
                lo = __builtin_amdgcn_fdot2(half2_t{f[4], f[5]}, one, lo, false);
                hi = __builtin_amdgcn_fdot2(half2_t{f[6], f[7]}, one, hi, false);
            }
            lo += __shfl_xor(lo, 16, 64);
            hi += __shfl_xor(hi, 16, 64);
            lo += __shfl_xor(lo, 32, 64);
            hi += __shfl_xor(hi, 32, 64);
            if (kq == 0) dst[r] = float2_t{ODSD_RAW_OFFSET_LO * lo + ODSD_RAW_OFFSET_HI * hi, lo + hi};
        };
        for (int bi = wave; bi < G_UP * MB; bi += WAVES) {
            if (bi % MB < nmb) group_sums(xs_raw + bi * XBLK, cx + bi * 16);
        }
        __syncthreads();
        ODSD_TL(3);                                           // group sums of the token rows

        // One step = one group of one block pair: B fragments of the group from LDS, the slot's two
        // tiles expanded to fp16, the slot refilled with the step DEPTH ahead, 2 x MB x 4 MFMAs.
        // Both streams of a wavefront are unrolled: ring slots, tile offsets and LDS addresses are
        // constants, and the wait the compiler derives for a slot leaves the younger slots in flight.
        float4_t acc[2][MB];
        auto step = [&](const int slot, const char *frag_base, const float2_t *sums, auto refill) {
            ODSD_FENCE();
            half8_t bx[MB][4];
            float2_t cxv[MB];
#pragma unroll
            for (int m = 0; m < nmb; ++m) {
#pragma unroll
                for (int j = 0; j < 4; ++j) bx[m][j] = *(const half8_t *)(frag_base + m * XBLK + lds_frag[j]);
                cxv[m] = sums[m * 16 + r];
            }
            half8_t a[2][4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i][0] = raw_word(rc, wq[slot][i].x);
                a[i][1] = raw_word(rc, wq[slot][i].y);
                a[i][2] = raw_word(rc, wq[slot][i].z);
                a[i][3] = raw_word(rc, wq[slot][i].w);
            }
            const uint4_t sz0 = wsz[slot][0], sz1 = wsz[slot][1];
            ODSD_FENCE();
            refill();                                         // the slot is free again
            ODSD_FENCE();
            // The matrix and scaling part of a step runs at raised priority: of the SIMD's two wavefronts
            // the one that already holds its operands goes first, and reaches its next refill sooner
            // (62.4 -> 61.9 us at T = 256, 60.3 -> 59.2 at T = 128; raising the first half of the step
            // instead changes nothing).
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int m = 0; m < nmb; ++m) {
                {
                    // the group's sum of q_k x_k: the accumulator starts at minus the offsets' share
                    const float nc = -cxv[m].x, xsum = cxv[m].y;
                    float4_t t[2];
                    t[0] = t[1] = float4_t{nc, nc, nc, nc};
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            t[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i][j], bx[m][j], t[i], 0, 0, 0);
                    // w = (q - zero) * scale per output row: acc += scale * (sum q x - zero * sum x)
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const uint4_t sz = i ? sz1 : sz0;
                        const half2_t p0 = as_half2(sz.x), p1 = as_half2(sz.y), p2 = as_half2(sz.z), p3 = as_half2(sz.w);
                        acc[i][m].x = __builtin_fmaf((float)p0.x, __builtin_fmaf(-(float)p0.y, xsum, t[i].x), acc[i][m].x);
                        acc[i][m].y = __builtin_fmaf((float)p1.x, __builtin_fmaf(-(float)p1.y, xsum, t[i].y), acc[i][m].y);
                        acc[i][m].z = __builtin_fmaf((float)p2.x, __builtin_fmaf(-(float)p2.y, xsum, t[i].z), acc[i][m].z);
                        acc[i][m].w = __builtin_fmaf((float)p3.x, __builtin_fmaf(-(float)p3.y, xsum, t[i].w), acc[i][m].w);
                    }
                }
            }
            // the step's arithmetic has no memory side: tie its results to the fence, or the whole
            // chain of a step may be ordered behind the loads of the steps after it
#pragma unroll
            for (int m = 0; m < nmb; ++m)
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    asm volatile("" : "+v"(acc[i][m].x), "+v"(acc[i][m].y), "+v"(acc[i][m].z), "+v"(acc[i][m].w));
            __builtin_amdgcn_s_setprio(0);
            ODSD_FENCE();
        };
        auto zero_acc = [&]() {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int m = 0; m < MB; ++m) acc[i][m] = float4_t{0.f, 0.f, 0.f, 0.f};
        };
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int pi = t / G_UP, g = t % G_UP;
            if (g == 0) zero_acc();
            step(t % DEPTH, xs_raw + (g * MB) * XBLK, cx + (g * MB) * 16, [&]() {
                // past the end of gate_up the ring goes on with the first steps of the down stream
                if (t + DEPTH < NT) load_u(t % DEPTH, t + DEPTH);
                else if (t + DEPTH - NT < ntd_w) load_d(t % DEPTH, t + DEPTH - NT);
            });
            if (g == G_UP - 1 || t == NT - 1) {
                // h = SiLU(gate) * up of this pair's 16 features -> LDS, in fragment order: the lane
                // holds features 4*kq .. 4*kq+3 of token column r
                const int fbl = wave * PPW + pi;             // 16-feature block inside the slice
                const int gl = fbl >> 3, seg = (fbl & 7) * 2 + (kq >> 1);
#pragma unroll
                for (int m = 0; m < nmb; ++m) {
                    {
                        const float4_t gt = acc[0][m], up = acc[1][m];
                        half4_t h;
                        h.x = f32_to_f16_sat(silu_f32(gt.x) * up.x);
                        h.y = f32_to_f16_sat(silu_f32(gt.y) * up.y);
                        h.z = f32_to_f16_sat(silu_f32(gt.z) * up.z);
                        h.w = f32_to_f16_sat(silu_f32(gt.w) * up.w);
                        char *dst = hs_raw + (gl * MB + m) * XBLK + r * 256 + ((seg ^ r) * 16) + (kq & 1) * 8;
                        *(half4_t *)dst = h;
                    }
                }
            }
        }
        ODSD_TL(4);                                           // this wavefront's gate_up stream done
        __syncthreads();                                      // h is complete
        ODSD_TL(5);
        for (int bi = wave; bi < GS * MB; bi += WAVES) {
            if (bi % MB < nmb) group_sums(hs_raw + bi * XBLK, cx + (G_UP * MB + bi) * 16);
        }
        __syncthreads();
        ODSD_TL(6);                                           // group sums of h

        // down: step u = group u % GS of output block pair u / GS, against h from LDS; the slice's
        // partial sums are stored as fp16 when a pair's last group is done
#pragma unroll
        for (int u = 0; u < NTD; ++u) {
            if (u >= DP_MIN * GS && u >= ntd_w) break;
            const int pi = u / GS, gl = u % GS;
            if (gl == 0) zero_acc();
            step((NT + u) % DEPTH, hs_raw + (gl * MB) * XBLK, cx + ((G_UP + gl) * MB) * 16, [&]() {
                if (u + DEPTH < NTD && u + DEPTH < ntd_w) load_d((NT + u) % DEPTH, u + DEPTH);
            });
            if (gl == GS - 1) {
                // lane holds outputs 4*kq .. 4*kq+3 of each block, token column r
#pragma unroll
                for (int m = 0; m < nmb; ++m) {
                    const int row = m * 16 + r;
                    if (row < mcnt) {
                        const size_t slot = (size_t)(base + m0 + row);
                        half_t *yrow = p.y + ((size_t)s * p.P + slot) * p.H;
#pragma unroll
                        for (int i = 0; i < 2; ++i) {
                            const int n = (dblk0 + 2 * pi + i) * 16 + kq * 4;
                            const float4_t v = acc[i][m];
                            *(half4_t *)(yrow + n) =
                                half4_t{f32_to_f16_sat(v.x), f32_to_f16_sat(v.y), f32_to_f16_sat(v.z), f32_to_f16_sat(v.w)};
                        }
                    }
                }
            }
        }
        };   // run_pass
        if (MB == 1 || mcnt <= 16) run_pass(std::integral_constant<int, 1>{});
        else run_pass(std::integral_constant<int, MB>{});
    }
    }   // units
#ifdef ODSD_TIMELINE
    ODSD_TL(7);
    if (odsd_tl_buf && (threadIdx.x & 63) == 0) {
        unsigned long long *o = odsd_tl_buf + ((size_t)blockIdx.x * WAVES + (threadIdx.x >> 6)) * 8;
        for (int k = 0; k < 8; ++k) o[k] = tl[k];
    }
#endif
}

// Shapes the fused kernel is built for; the caller has checked them with odsd_fused_supported().
void odsd_launch_experts_fused(FusedParams &fp, int E, hipStream_t st) {
    // (MB = 2: up to 32 rows per pass; experts with at most 16 rows skip the second token block)
    static_assert(ODSD_ONE_LAUNCH_ROWS == 16 * 2, "rows of one pass as the header states them");
    if (fp.idx && fp.P <= 4 * 512)
        ODSD_LAUNCH(ODSD_KERNEL_EXPERTS, (w4_expert_fused_kernel<2, 3, 8, 16, 6, 1>), E * fp.S, 512, st, fp);
    else if (fp.idx)
        ODSD_LAUNCH(ODSD_KERNEL_EXPERTS, (w4_expert_fused_kernel<2, 3, 8, 16, 6, 2>), E * fp.S, 512, st, fp);
    else
        ODSD_LAUNCH(ODSD_KERNEL_EXPERTS, (w4_expert_fused_kernel<2, 3, 8, 16, 6, 0>), E * fp.S, 512, st, fp);
}

// the in-kernel dispatch holds the whole id list in one or two vectors of 4 ids per thread
int odsd_fused_dispatch_supported(int P) { return P % 4 == 0 && P <= 8 * 512; }

// H = 2048 (4 sub-passes of 8 wavefronts x 4 blocks), slices of 384 features, token rows of one
// pass within the 128 KB row area
int odsd_fused_supported(int H, int I, int S, int E) {
    if (S < 1 || I % (ODSD_GROUP * S) || E > ODSD_FUSED_MAX_E) return 0;
    if (I / (ODSD_GROUP * S) != 3 || I / ODSD_GROUP != 6) return 0;
    if (H != 2048) return 0;
    if ((H / ODSD_GROUP) * 2 > ODSD_FUSED_X_BLOCKS) return 0;
    return 1;
}
