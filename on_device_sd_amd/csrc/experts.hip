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
#include "common.h"

#define XS_STRIDE 136   // halfs per LDS row: 128 + 8 (16-byte skew between rows)

struct GemmParams {
    const uint64_t *table;   // [E][4]
    const half_t *src;       // activations, fp16
    const int32_t *rowmap;   // slot -> source row (gate_up: token), or null: row = slot
    const int32_t *counts;
    const int32_t *offsets;
    half_t *h16;             // MODE 0 output [P][I]
    float *y;                // MODE 1 output [KS][P][ldo]
    int src_ld;              // elements per source row (= reduction length Kd)
    int G;                   // groups of 128 in the reduction dimension
    int NBLK;                // 16-row blocks of the (fused) weight matrix
    int nchunks;             // workgroup tiles along the rows
    int KS;                  // splits of the reduction dimension
    int gper;                // groups per split
    int ldo;                 // I (MODE 0) or H (MODE 1)
    int P;
    int n_wg;                // E * nchunks * KS
    int wg_per_xcd;          // ceil(n_wg / 8)
};

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// 4 words (32 codes) of one lane -> 4 x 8 fp16 weights  (w = (code - zero) * scale).
// The integer part of the zero point is folded into the exact integer step that removes the
// 1024 (low nibbles) / 64 (high nibbles, pre-scaled by 16) offset of the fp16 bit trick, so
// only the fractional part of the zero point is rounded.
__device__ __forceinline__ void dequant_tile(const uint4_t raw, const uint32_t szbits, half8_t (&a)[4]) {
    const half2_t sz = as_half2(szbits);
    const half_t s = sz.x, z = sz.y;
    const half_t zi = __builtin_rintf16(z);
    const half_t zf = z - zi;                      // exact
    const half_t c_lo = (half_t)(-1024.0f) - zi;   // exact for |zi| <= 1024
    const half_t c_hi = (half_t)(-64.0f) - zi;
    const half_t nz = -(zf * s);
    const half2_t S = {s, s}, CLO = {c_lo, c_lo}, CHI = {c_hi, c_hi}, NZ = {nz, nz};
    const half2_t R16 = {(half_t)0.0625f, (half_t)0.0625f};
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t x = w[j], xs = x >> 8;
        const half2_t t0 = as_half2((x & 0x000F000Fu) | 0x64006400u);
        const half2_t t1 = as_half2((x & 0x00F000F0u) | 0x64006400u);
        const half2_t t2 = as_half2((xs & 0x000F000Fu) | 0x64006400u);
        const half2_t t3 = as_half2((xs & 0x00F000F0u) | 0x64006400u);
        const half2_t q0 = t0 + CLO;
        const half2_t q1 = __builtin_elementwise_fma(t1, R16, CHI);
        const half2_t q2 = t2 + CLO;
        const half2_t q3 = __builtin_elementwise_fma(t3, R16, CHI);
        const half2_t v0 = __builtin_elementwise_fma(q0, S, NZ);
        const half2_t v1 = __builtin_elementwise_fma(q1, S, NZ);
        const half2_t v2 = __builtin_elementwise_fma(q2, S, NZ);
        const half2_t v3 = __builtin_elementwise_fma(q3, S, NZ);
        a[j] = half8_t{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
    }
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

template <int NB, int MB, int MODE>
__global__ __launch_bounds__(256) void w4_gemm_kernel(const GemmParams p) {
    static_assert(MODE == 1 || NB % 2 == 0, "gate_up needs gate/up block pairs");
    __shared__ __attribute__((aligned(16))) half_t xs[2][16 * MB][XS_STRIDE];

    // workgroup -> (expert, row chunk, k split); consecutive logical ids share an XCD so
    // that one expert's token rows stay in one L2
    const int b = blockIdx.x;
    const int L = (b & 7) * p.wg_per_xcd + (b >> 3);
    if (L >= p.n_wg) return;
    const int ks = L % p.KS;
    const int chunk = (L / p.KS) % p.nchunks;
    const int e = L / (p.KS * p.nchunks);

    const int M_e = p.counts[e];
    if (M_e == 0) return;
    const uint64_t *trow = p.table + (size_t)e * ODSD_TABLE_COLS;
    if (trow[0] == 0) return;
    const uint4_t *qp = (const uint4_t *)(MODE == 0 ? trow[0] : trow[2]);
    const uint32_t *szp = (const uint32_t *)(MODE == 0 ? trow[1] : trow[3]);
    const int base = p.offsets[e];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    const int g_begin = ks * p.gper;
    const int g_end = min(p.G, g_begin + p.gper);

    const int blk0 = (chunk * 4 + wave) * NB;   // first 16-row block of this wavefront
    bool blk_ok[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) blk_ok[i] = blk0 + i < p.NBLK;

    // x staging: row = piece / 16, 16-byte segment = piece % 16, piece = tid + 256 i
    const int st_seg = tid & 15;
    const int st_row0 = tid >> 4;

    for (int m0 = 0; m0 < M_e; m0 += 16 * MB) {
        const int mcnt = min(M_e - m0, 16 * MB);
        const int nmb = (mcnt + 15) >> 4;

        const half_t *st_src[MB];
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int row = st_row0 + 16 * i;
            st_src[i] = nullptr;
            if (row < mcnt) {
                const int slot = base + m0 + row;
                const int srow = p.rowmap ? p.rowmap[slot] : slot;
                st_src[i] = p.src + (size_t)srow * p.src_ld + st_seg * 8;
            }
        }

        float4_t acc[NB][MB];
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int m = 0; m < MB; ++m) acc[i][m] = float4_t{0.f, 0.f, 0.f, 0.f};

        uint4_t wq[2][NB];
        uint32_t wsz[2][NB];
        uint4_t xr[MB];

        auto load_w = [&](int buf, int g) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                if (blk_ok[i] && g < g_end) {
                    const size_t tile = (size_t)(blk0 + i) * p.G + g;
                    wq[buf][i] = __builtin_nontemporal_load(qp + tile * 64 + lane);
                    wsz[buf][i] = szp[tile * 16 + r];
                } else {
                    wq[buf][i] = uint4_t{0, 0, 0, 0};
                    wsz[buf][i] = 0;
                }
            }
        };
        auto load_x = [&](int g) {
#pragma unroll
            for (int i = 0; i < MB; ++i) {
                if (st_src[i] != nullptr && i < nmb)
                    xr[i] = *(const uint4_t *)(st_src[i] + (size_t)g * ODSD_GROUP);
                else
                    xr[i] = uint4_t{0, 0, 0, 0};
            }
        };
        auto store_x = [&](int buf) {
#pragma unroll
            for (int i = 0; i < MB; ++i)
                if (i < nmb) *(uint4_t *)&xs[buf][st_row0 + 16 * i][st_seg * 8] = xr[i];
        };
        auto compute = [&](int buf, int xbuf) {
            half8_t a[NB][4];
#pragma unroll
            for (int i = 0; i < NB; ++i) dequant_tile(wq[buf][i], wsz[buf][i], a[i]);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < nmb) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const half8_t bx = *(const half8_t *)&xs[xbuf][m * 16 + r][j * 32 + kq * 8];
#pragma unroll
                        for (int i = 0; i < NB; ++i)
                            acc[i][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i][j], bx, acc[i][m], 0, 0, 0);
                    }
                }
            }
        };

        // software pipeline: weights two groups ahead in registers, x one group ahead
        __syncthreads();   // previous pass is done with xs
        load_x(g_begin);
        load_w(0, g_begin);
        load_w(1, g_begin + 1);
        store_x(0);
        __syncthreads();
        for (int g = g_begin; g < g_end; g += 2) {
            // even step: weights in buffer 0, x in xs[0]
            if (g + 1 < g_end) load_x(g + 1);
            compute(0, 0);
            load_w(0, g + 2);
            if (g + 1 < g_end) store_x(1);
            __syncthreads();
            if (g + 1 >= g_end) break;
            // odd step: weights in buffer 1, x in xs[1]
            if (g + 2 < g_end) load_x(g + 2);
            compute(1, 1);
            load_w(1, g + 3);
            if (g + 2 < g_end) store_x(0);
            __syncthreads();
        }

        // epilogue: lane holds rows 4*kq..4*kq+3 of each 16-row block, token column r
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const int row = m * 16 + r;
            if (m < nmb && row < mcnt) {
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
                            *(float4_t *)(p.y + ((size_t)ks * p.P + slot) * p.ldo + n) = acc[i][m];
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Combine: out[t] = sum_k w[t,k] * (sum_ks y[ks][perm[t*K+k]]) in k order, fp32, one rounding.
// A pair whose expert has no weights (table row 0) or whose id is out of range adds nothing.
// out_act = cast(residual + cast(moe)): the reference rounds the MoE output to the
// activation dtype before the residual add (qwen3_runner.py:295, :226).
// ---------------------------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void combine_kernel(const float *__restrict__ y, const int32_t *__restrict__ idx,
                                                      const float *__restrict__ w,
                                                      const int32_t *__restrict__ perm,
                                                      const uint64_t *__restrict__ table,
                                                      const XT *__restrict__ residual,
                                                      float *__restrict__ out_f32, XT *__restrict__ out_act,
                                                      int T, int H, int K, int E, int KS, int P) {
    const int t = blockIdx.y;
    const int c = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (c >= H) return;
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < K; ++k) {
        const int pr = t * K + k;
        const int slot = perm[pr];
        const int e = idx[pr];
        if (slot < 0 || e < 0 || e >= E || table[(size_t)e * ODSD_TABLE_COLS] == 0) continue;
        float4_t v = *(const float4_t *)(y + (size_t)slot * H + c);
        for (int s = 1; s < KS; ++s) v += *(const float4_t *)(y + ((size_t)s * P + slot) * H + c);
        const float wk = w[pr];
        acc.x = fmaf(wk, v.x, acc.x);
        acc.y = fmaf(wk, v.y, acc.y);
        acc.z = fmaf(wk, v.z, acc.z);
        acc.w = fmaf(wk, v.w, acc.w);
    }
    const size_t o = (size_t)t * H + c;
    float res[4] = {0.f, 0.f, 0.f, 0.f};
    if (residual) {
#pragma unroll
        for (int i = 0; i < 4; ++i) res[i] = ActIO<XT>::load(residual, o + i);
    }
    const float a[4] = {acc.x, acc.y, acc.z, acc.w};
    if (out_f32) *(float4_t *)(out_f32 + o) = float4_t{a[0] + res[0], a[1] + res[1], a[2] + res[2], a[3] + res[3]};
    if (out_act) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float m = ActIO<XT>::round(a[i]);
            ActIO<XT>::store(out_act, o + i, residual ? __fadd_rn(res[i], m) : m);
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------
struct ExpertsPlan {
    int MB;          // 16-row token blocks held per pass
    int NB;          // 16-row weight blocks per wavefront
    int KS;          // split of the down projection's reduction dimension
    size_t h_bytes, y_bytes;
};

static ExpertsPlan experts_plan(const odsd_moe_shape *s) {
    ExpertsPlan p;
    // rows one expert can receive is at most T (distinct ids per token); size the register
    // tile for the common case and let rarer, larger experts take extra passes
    const long P = (long)s->T * s->K;
    const long mean_rows = (P + s->E - 1) / s->E;
    if (s->T <= 16) p.MB = 1;
    else if (s->T <= 32) p.MB = 2;
    else p.MB = (mean_rows * 3 / 2 <= 64) ? 4 : 8;
    p.NB = 4;
    // down projection: enough workgroups to cover the machine (~4 per CU)
    const int nchunks_dn = (s->H / 16 + 4 * p.NB - 1) / (4 * p.NB);
    const long active = s->E < P ? s->E : P;
    const int G = s->I / ODSD_GROUP;
    int KS = 1;
    while (KS * 2 <= G && active * nchunks_dn * KS < 1024 && KS < 16) KS *= 2;
    // every split must own at least one group
    while (KS > 1 && ((G + KS - 1) / KS) * (KS - 1) >= G) KS--;
    p.KS = KS;
    p.h_bytes = odsd_round_up((size_t)(P > 0 ? P : 1) * s->I * sizeof(half_t), 256);
    p.y_bytes = odsd_round_up((size_t)KS * (size_t)(P > 0 ? P : 1) * s->H * sizeof(float), 256);
    return p;
}

static int experts_check(const odsd_moe_shape *s) {
    if (!s) return ODSD_ERR_NULL;
    if (s->T < 0 || s->H <= 0 || s->E <= 0 || s->K <= 0 || s->I <= 0) return ODSD_ERR_SHAPE;
    if (s->H % ODSD_GROUP || s->I % ODSD_GROUP) return ODSD_ERR_SHAPE;
    if ((int64_t)s->T * s->K > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    if (s->act_dtype != ODSD_DT_F32 && s->act_dtype != ODSD_DT_BF16) return ODSD_ERR_DTYPE;
    return ODSD_OK;
}

extern "C" size_t odsd_experts_workspace_bytes(const odsd_moe_shape *s) {
    if (experts_check(s) != ODSD_OK) return 0;
    const ExpertsPlan p = experts_plan(s);
    return p.h_bytes + p.y_bytes;
}

template <int NB, int MB, int MODE>
static void launch_gemm(GemmParams &gp, hipStream_t st) {
    gp.wg_per_xcd = (gp.n_wg + 7) / 8;
    w4_gemm_kernel<NB, MB, MODE><<<gp.wg_per_xcd * 8, 256, 0, st>>>(gp);
}

template <int MODE>
static void launch_gemm_mb(int MB, GemmParams &gp, hipStream_t st) {
    switch (MB) {
        case 1: launch_gemm<4, 1, MODE>(gp, st); break;
        case 2: launch_gemm<4, 2, MODE>(gp, st); break;
        case 4: launch_gemm<4, 4, MODE>(gp, st); break;
        default: launch_gemm<4, 8, MODE>(gp, st); break;
    }
}

int odsd_launch_experts(const odsd_moe_shape *s, const void *x16, const uint64_t *table, const int32_t *idx,
                        const float *w, const int32_t *counts, const int32_t *offsets, const int32_t *perm,
                        const int32_t *slot_token, const void *residual, float *out_f32, void *out_act,
                        void *ws, size_t ws_bytes, hipStream_t st) {
    const int rc = experts_check(s);
    if (rc != ODSD_OK) return rc;
    if (s->T == 0) return ODSD_OK;
    if (!x16 || !table || !idx || !w || !counts || !offsets || !perm || !slot_token || !ws)
        return ODSD_ERR_NULL;
    if (!out_f32 && !out_act) return ODSD_ERR_NULL;
    if (!odsd_aligned16(x16) || !odsd_aligned16(ws) || (out_f32 && !odsd_aligned16(out_f32)))
        return ODSD_ERR_ALIGN;
    const ExpertsPlan pl = experts_plan(s);
    if (ws_bytes < pl.h_bytes + pl.y_bytes) return ODSD_ERR_WORKSPACE;
    half_t *h16 = (half_t *)ws;
    float *y = (float *)((char *)ws + pl.h_bytes);
    const int P = s->T * s->K;

    GemmParams gu{};
    gu.table = table; gu.src = (const half_t *)x16; gu.rowmap = slot_token;
    gu.counts = counts; gu.offsets = offsets; gu.h16 = h16; gu.y = nullptr;
    gu.src_ld = s->H; gu.G = s->H / ODSD_GROUP; gu.NBLK = 2 * s->I / 16;
    gu.nchunks = (gu.NBLK + 4 * pl.NB - 1) / (4 * pl.NB);
    gu.KS = 1; gu.gper = gu.G; gu.ldo = s->I; gu.P = P;
    gu.n_wg = s->E * gu.nchunks;
    launch_gemm_mb<0>(pl.MB, gu, st);
    ODSD_CHECK_LAUNCH();

    GemmParams dn{};
    dn.table = table; dn.src = h16; dn.rowmap = nullptr;
    dn.counts = counts; dn.offsets = offsets; dn.h16 = nullptr; dn.y = y;
    dn.src_ld = s->I; dn.G = s->I / ODSD_GROUP; dn.NBLK = s->H / 16;
    dn.nchunks = (dn.NBLK + 4 * pl.NB - 1) / (4 * pl.NB);
    dn.KS = pl.KS; dn.gper = (dn.G + pl.KS - 1) / pl.KS; dn.ldo = s->H; dn.P = P;
    dn.n_wg = s->E * dn.nchunks * dn.KS;
    launch_gemm_mb<1>(pl.MB, dn, st);
    ODSD_CHECK_LAUNCH();

    const dim3 grid((s->H / 4 + 255) / 256, s->T);
    if (s->act_dtype == ODSD_DT_BF16)
        combine_kernel<uint16_t><<<grid, 256, 0, st>>>(y, idx, w, perm, table, (const uint16_t *)residual,
                                                       out_f32, (uint16_t *)out_act, s->T, s->H, s->K,
                                                       s->E, pl.KS, P);
    else
        combine_kernel<float><<<grid, 256, 0, st>>>(y, idx, w, perm, table, (const float *)residual,
                                                    out_f32, (float *)out_act, s->T, s->H, s->K, s->E,
                                                    pl.KS, P);
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_experts_w4(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                               const int32_t *idx, const float *w, const int32_t *counts,
                               const int32_t *offsets, const int32_t *perm, const int32_t *slot_token,
                               const void *residual, float *out_f32, void *out_act, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return odsd_launch_experts(s, x_f16, table, idx, w, counts, offsets, perm, slot_token, residual,
                               out_f32, out_act, workspace, workspace_bytes, (hipStream_t)stream);
}
