// Router: logits = x . Wg^T accumulated in fp64, then softmax / top-k per token.
//
// Two kernels.
//  1. router_partial_kernel: a split-K [T,H]x[H,E] product on the fp64 matrix cores
//     (v_mfma_f64_16x16x4_f64).  One wavefront owns a tile of 16 tokens x (16*NE) experts
//     over one K slice and writes fp64 partial logits.  fp64 accumulation makes the logits
//     the exact dot product to ~1e-16, so the top-k choice does not depend on the
//     summation order -- which is what lets the expert indices be bit-exact against a CPU
//     restatement.  The tile with expert group 0 also writes the fp16 copy of x that the
//     expert kernels consume.
//  2. router_topk_kernel: one wavefront per token sums the partials in a fixed order,
//     selects the K largest logits (ties to the lower index) by K rounds of a wavefront
//     arg-max and computes the weights in fp32.
//
// Replaces: Qwen3MoEGate.forward (demo/src/layers/moe_layer.py:41-58), the stateless form
// (:210-216) and GPUOperators.router (demo/src/operators/gpu_operators.py:48-69).
#include "common.h"
#include "router_topk.h"

#define ROUTER_MAX_NE 4    // expert tiles (of 16) per wavefront
#define ROUTER_MAX_V 8     // most logits per lane in the top-k kernel -> E <= 512

// 8 consecutive activations of one row: the raw load and the conversion are separate so that
// the loads of the next chunk can be in flight while the current one is multiplied
template <typename XT> struct Row8;
template <> struct Row8<uint16_t> {  // 8 bf16 = 16 bytes
    typedef uint4_t Raw;
    __device__ static __forceinline__ Raw raw(const uint16_t *p) { return *(const uint4_t *)p; }
    __device__ static __forceinline__ void cvt(const Raw &u, float (&v)[8]) {
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <> struct Row8<float> {
    struct Raw { float4_t a, b; };
    __device__ static __forceinline__ Raw raw(const float *p) {
        return Raw{*(const float4_t *)p, *(const float4_t *)(p + 4)};
    }
    __device__ static __forceinline__ void cvt(const Raw &u, float (&v)[8]) {
        v[0] = u.a.x; v[1] = u.a.y; v[2] = u.a.z; v[3] = u.a.w;
        v[4] = u.b.x; v[5] = u.b.y; v[6] = u.b.z; v[7] = u.b.w;
    }
};

// unit = (token tile, expert group, k split); 4 units (wavefronts) per workgroup.
template <typename XT, int NE, bool REDUCE4>
__global__ __launch_bounds__(256) void router_partial_kernel(const XT *__restrict__ x,
                                                             const XT *__restrict__ wg,
                                                             double *__restrict__ partial,
                                                             half_t *__restrict__ x16, int T, int H,
                                                             int E, int S, int EG, int n_units,
                                                             const double *__restrict__ norm_ss,
                                                             const XT *__restrict__ norm_w, double eps) {
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n_units) return;
    const int lane = lane_id();
    const int r = lane & 15, kg = lane >> 4;
    const int s = unit % S;
    const int eg = (unit / S) % EG;
    const int tt = unit / (S * EG);
    const int Hs = H / S;
    const int k0 = s * Hs;
    const int t = tt * 16 + r;
    const bool t_ok = t < T;

    // Which (row, column) of the 16x16 result each of this lane's 4 accumulators holds is
    // read back from the matrix core itself: D = A.B with A[i][0]=i, B[0][j]=1 gives D=i,
    // and A[i][0]=1, B[0][j]=j gives D=j.
    int di[4], dj[4];
    {
        const double4_t z = {0.0, 0.0, 0.0, 0.0};
        const double a_i = kg == 0 ? (double)r : 0.0, one = kg == 0 ? 1.0 : 0.0;
        const double4_t pi = __builtin_amdgcn_mfma_f64_16x16x4f64(a_i, one, z, 0, 0, 0);
        const double4_t pj = __builtin_amdgcn_mfma_f64_16x16x4f64(one, a_i, z, 0, 0, 0);
        di[0] = (int)pi.x; di[1] = (int)pi.y; di[2] = (int)pi.z; di[3] = (int)pi.w;
        dj[0] = (int)pj.x; dj[1] = (int)pj.y; dj[2] = (int)pj.z; dj[3] = (int)pj.w;
    }

    double4_t acc[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) acc[i] = double4_t{0.0, 0.0, 0.0, 0.0};

    // fused RMSNorm (demo/src/layers/layernorm.py:21-27): the row statistic comes from the kernel
    // that produced x; the arithmetic per element is that of the stand-alone RMSNorm kernel
    const bool normed = norm_ss != nullptr;
    double rstd = 1.0;
    if (normed) {
        const int nchunk = (H + 1023) / 1024;   // the statistic arrives as per-chunk sums
        double tot = 0.0;
        for (int c = 0; c < nchunk; ++c) tot += norm_ss[(size_t)(t_ok ? t : 0) * nchunk + c];
        rstd = 1.0 / sqrt(tot / (double)H + eps);
    }
    const XT *xrow = x + (size_t)(t_ok ? t : 0) * H;
    const XT *wrow[NE];
    bool e_ok[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int e = (eg * NE + i) * 16 + r;
        e_ok[i] = e < E;
        wrow[i] = wg + (size_t)(e_ok[i] ? e : 0) * H;
    }

    // One chunk = 32 columns.  The raw loads of chunk c+1 are issued before chunk c is
    // converted and multiplied (two register sets used in turn), so that their latency hides
    // under the 8*NE fp64 MFMAs of the current chunk.
    typedef typename Row8<XT>::Raw Raw;
    struct Chunk {
        Raw x, n, w[NE];
    };
    auto fetch = [&](Chunk &ck, int c) {
        const int h = k0 + min(c, Hs - 32) + kg * 8;    // past the end: reload the last chunk
        ck.x = Row8<XT>::raw(xrow + h);
        if (normed) ck.n = Row8<XT>::raw(norm_w + h);
#pragma unroll
        for (int i = 0; i < NE; ++i) ck.w[i] = Row8<XT>::raw(wrow[i] + h);
    };
    auto consume = [&](const Chunk &ck, int c) {
        const int h = k0 + c + kg * 8;
        float xa[8];
        Row8<XT>::cvt(ck.x, xa);
        if (normed) {
            float nw[8];
            Row8<XT>::cvt(ck.n, nw);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float xn = ActIO<XT>::round((float)((double)xa[j] * rstd));
                xa[j] = ActIO<XT>::round(__fmul_rn(xn, nw[j]));
            }
        }
        if (!t_ok) {
#pragma unroll
            for (int j = 0; j < 8; ++j) xa[j] = 0.0f;
        }
        if (x16 != nullptr && eg == 0 && t_ok) {
            half8_t o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = f32_to_f16_sat(xa[j]);
            *(half8_t *)(x16 + (size_t)t * H + h) = o;
        }
        double xd[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) xd[j] = (double)xa[j];
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            float wa[8];
            Row8<XT>::cvt(ck.w[i], wa);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const double wd = e_ok[i] ? (double)wa[j] : 0.0;
                acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(xd[j], wd, acc[i], 0, 0, 0);
            }
        }
    };
    Chunk ca, cb;
    fetch(ca, 0);
    for (int c = 0; c < Hs; c += 64) {
        fetch(cb, c + 32);
        consume(ca, c);
        if (c + 32 >= Hs) break;
        fetch(ca, c + 64);
        consume(cb, c + 32);
    }

    // When the K slices come in fours, the 4 wavefronts of this workgroup hold 4 consecutive
    // slices of the same tile: add them through LDS in slice order and write one partial.
    int s_out = s, S_out = S;
    if (REDUCE4) {
        __shared__ double red[3][NE][4][64];
        const int wave = threadIdx.x >> 6;
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < NE; ++i) {
                red[wave - 1][i][0][lane] = acc[i].x;
                red[wave - 1][i][1][lane] = acc[i].y;
                red[wave - 1][i][2][lane] = acc[i].z;
                red[wave - 1][i][3][lane] = acc[i].w;
            }
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int i = 0; i < NE; ++i) {
                acc[i].x += red[w][i][0][lane];
                acc[i].y += red[w][i][1][lane];
                acc[i].z += red[w][i][2][lane];
                acc[i].w += red[w][i][3][lane];
            }
        s_out = s >> 2;
        S_out = S >> 2;
    }
    (void)S_out;
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const double v[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int tq = tt * 16 + di[q];
            const int eq = (eg * NE + i) * 16 + dj[q];
            if (tq < T && eq < E) partial[((size_t)s_out * T + tq) * E + eq] = v[q];
        }
    }
}

// V = logits per lane (experts lane, lane + 64, ...): 1, 2, 4 or 8 for E <= 64, 128, 256, 512
// the selection for token t by one wavefront; lane k < K returns the k-th winner's expert id
template <int V>
__device__ __forceinline__ int topk_token(const double *__restrict__ partial, const int t, int T, int E,
                                          int K, int S, int renorm, int32_t *__restrict__ idx,
                                          float *__restrict__ w, int64_t *__restrict__ idx64,
                                          double *__restrict__ logits) {
    const int lane = lane_id();

    double lg[V];
    uint64_t key[V];
    uint32_t taken = 0;   // bit v set: expert lane + 64 v already selected
    // partial sums in slice order; the loads of one slice batch are independent of each other
#pragma unroll
    for (int v = 0; v < V; ++v) lg[v] = 0.0;
    constexpr int SB = V <= 2 ? 8 : 4;   // slices loaded together
    for (int s0 = 0; s0 < S; s0 += SB) {
        double part[SB][V];
#pragma unroll
        for (int u = 0; u < SB; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const int e = lane + 64 * v;
                part[u][v] = (e < E && s0 + u < S) ? partial[((size_t)(s0 + u) * T + t) * E + e] : 0.0;
            }
#pragma unroll
        for (int u = 0; u < SB; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) lg[v] += part[u][v];
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        key[v] = order_key(lg[v]);
        if (lane + 64 * v >= E) taken |= 1u << v;
        else if (logits) logits[(size_t)t * E + lane + 64 * v] = lg[v];
    }

    int my_e = 0;          // lane k keeps the k-th winner
    double my_l = 0.0;
    double l_max = 0.0;
    for (int k = 0; k < K; ++k) {
        // best remaining candidate of this lane: largest key, then lowest expert.  A lane with
        // nothing left offers key 0 (no finite logit maps to it) and the largest expert id.
        uint64_t bk = 0;
        int be = 0x7fffffff;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (!((taken >> v) & 1u)) {
                if (be == 0x7fffffff || key[v] > bk) {
                    bk = key[v];
                    be = lane + 64 * v;
                }
            }
        }
        const int we = wave_argmax(bk, be);   // the same in every lane
        // the winner's logit sits in lane (we & 63), slot (we >> 6)
        double cand = lg[0];
#pragma unroll
        for (int v = 1; v < V; ++v) cand = (we >> 6) == v ? lg[v] : cand;
        const uint64_t cb = (uint64_t)__double_as_longlong(cand);
        const uint32_t wlo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)cb, we & 63);
        const uint32_t whi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(cb >> 32), we & 63);
        const double wl = __longlong_as_double((long long)(((uint64_t)whi << 32) | wlo));
        if ((we & 63) == lane) taken |= 1u << (we >> 6);
        if (lane == k) { my_e = we; my_l = wl; }
        if (k == 0) l_max = wl;
    }

    // weights in fp32; differences are taken in fp64 before the cast
    float num = 0.0f;
    if (lane < K) num = expf((float)(my_l - l_max));
    float den;
    if (renorm) {
        den = wave_sum(num);
    } else {
        float part = 0.0f;
#pragma unroll
        for (int v = 0; v < V; ++v)
            if (lane + 64 * v < E) part += expf((float)(lg[v] - l_max));
        den = wave_sum(part);
    }
    if (lane < K) {
        const size_t o = (size_t)t * K + lane;
        idx[o] = my_e;
        w[o] = num / den;
        if (idx64) idx64[o] = (int64_t)my_e;
    }
    return my_e;
}

template <int V>
__global__ __launch_bounds__(256) void router_topk_kernel(const double *__restrict__ partial, int T, int E,
                                                          int K, int S, int renorm,
                                                          int32_t *__restrict__ idx,
                                                          float *__restrict__ w,
                                                          int64_t *__restrict__ idx64,
                                                          double *__restrict__ logits) {
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= T) return;
    topk_token<V>(partial, t, T, E, K, S, renorm, idx, w, idx64, logits);
}

// Few tokens (T <= 16, P = T * K <= ROUTER_SMALL_PAIRS): one workgroup, one wavefront per token, and
// behind a barrier the same workgroup sorts the pairs by expert -- the dispatch of dispatch.hip on a
// list that fits LDS, without its launch (decode and short verify steps: 4 us of a 107 us layer at
// T = 5).  A pair's slot is the number of pairs of lower experts plus the number of earlier pairs of
// its own expert, which is the stable order of the dispatch kernel.
#define ROUTER_SMALL_PAIRS 128
template <int V>
__global__ __launch_bounds__(1024) void router_topk_dispatch_small_kernel(
    const double *__restrict__ partial, int T, int E, int K, int S, int renorm, int32_t *__restrict__ idx,
    float *__restrict__ w, int64_t *__restrict__ idx64, double *__restrict__ logits,
    int32_t *__restrict__ counts, int32_t *__restrict__ offsets, int32_t *__restrict__ perm,
    int32_t *__restrict__ inv, int32_t *__restrict__ slot_token, int64_t *__restrict__ counts_mirror,
    uint32_t mirror_tag) {
    __shared__ int32_t ids[ROUTER_SMALL_PAIRS];
    const int t = threadIdx.x >> 6, lane = lane_id();
    if (t < T) {
        const int my_e = topk_token<V>(partial, t, T, E, K, S, renorm, idx, w, idx64, logits);
        if (lane < K) ids[t * K + lane] = my_e;
    }
    __syncthreads();
    // wavefront w sorts out experts w, w + nw, ...: the pair list sits in two registers per lane (pairs
    // lane and lane + 64), ballots count the pairs of the expert and of lower experts, and the lanes
    // that hold a pair of the expert take consecutive slots in pair order
    const int P = T * K, nw = blockDim.x >> 6;
    const int id0 = lane < P ? ids[lane] : -1, id1 = lane + 64 < P ? ids[lane + 64] : -1;
    for (int e = t; e < E; e += nw) {
        const uint64_t m0 = __ballot(id0 == e), m1 = __ballot(id1 == e);
        const int c0 = __popcll(m0), c = c0 + __popcll(m1);
        const int lt = __popcll(__ballot(id0 >= 0 && id0 < e)) + __popcll(__ballot(id1 >= 0 && id1 < e));
        if (lane == 0) {
            counts[e] = c;
            if (counts_mirror) counts_mirror[e] = (int64_t)(((uint64_t)mirror_tag << 32) | (uint32_t)c);
            offsets[e] = lt;
            if (e == E - 1) offsets[E] = lt + c;
        }
        if (id0 == e) {
            const int slot = lt + mask_rank(m0);
            perm[lane] = slot;
            inv[slot] = lane;
            slot_token[slot] = lane / K;
        }
        if (id1 == e) {
            const int slot = lt + c0 + mask_rank(m1);
            perm[lane + 64] = slot;
            inv[slot] = lane + 64;
            slot_token[slot] = (lane + 64) / K;
        }
    }
}

// ---- host side -----------------------------------------------------------------------------
struct RouterPlan {
    int NE, EG, TT, S;
    size_t partial_bytes;
};

static RouterPlan router_plan(const odsd_moe_shape *s, bool normed) {
    RouterPlan p;
    const int ET = (s->E + 15) / 16;
    p.TT = (s->T + 15) / 16;
    // Expert tiles per wavefront: more of them re-use a token chunk more often, fewer give more and
    // shorter wavefront units.  With few 16 x 16 output tiles the kernel is a latency chain and short
    // units win (E = 128: 4.6 against 6.9 us at T = 128, 6.5 against 7.1 at 256, 8.4 against 10.6 at
    // 320); from ~512 tiles on the re-use wins (T = 4096, H = 4096: 94 against 117 us).  With the
    // RMSNorm folded in, every expert group also repeats the normalisation of its token chunk (two
    // fp64 conversions per element): two tiles per wavefront are then the least (T = 256 in the
    // 48-layer stack: 8.2 us against 9.3 with one, 8.3 with four).
    const long tiles = (long)p.TT * ET;
    const int ne = tiles <= 192 ? (normed ? 2 : 1) : (tiles <= 512 ? 2 : 4);
    p.NE = ET >= ne ? ne : (ET >= 2 ? 2 : 1);
    p.EG = (ET + p.NE - 1) / p.NE;
    // split K until there are ~2048 wavefront units or the slices get down to 64 columns
    int S = 1;
    const int maxS = s->H / 64;
    while (S * 2 <= maxS && (s->H / (S * 2)) % 32 == 0 && s->H % (S * 2) == 0 &&
           (long)p.TT * p.EG * S < 2048)
        S *= 2;
    p.S = S;
    p.partial_bytes = odsd_round_up((size_t)S * (size_t)(s->T > 0 ? s->T : 1) * s->E * sizeof(double), 256);
    return p;
}

static int router_check(const odsd_moe_shape *s) {
    if (!s) return ODSD_ERR_NULL;
    if (s->T < 0 || s->H <= 0 || s->E <= 0 || s->K <= 0) return ODSD_ERR_SHAPE;
    if (s->H % 128) return ODSD_ERR_SHAPE;
    if (s->K > s->E) return ODSD_ERR_SHAPE;
    if (s->E > 64 * ROUTER_MAX_V || s->K > 64) return ODSD_ERR_UNSUPPORTED;
    if (s->act_dtype != ODSD_DT_F32 && s->act_dtype != ODSD_DT_BF16) return ODSD_ERR_DTYPE;
    return ODSD_OK;
}

extern "C" size_t odsd_router_workspace_bytes(const odsd_moe_shape *s) {
    if (router_check(s) != ODSD_OK) return 0;
    // (the split of K, and with it the partial sums, depends on whether the RMSNorm is folded in)
    const size_t a = router_plan(s, false).partial_bytes, b = router_plan(s, true).partial_bytes;
    return a > b ? a : b;
}

template <typename XT, int NE>
static void launch_partial(const RouterPlan &p, const odsd_moe_shape *s, const void *x, const void *gw,
                           double *partial, void *x16, hipStream_t st, const double *norm_ss,
                           const void *norm_w, float eps) {
    const int n_units = p.TT * p.EG * p.S;
    if (p.S % 4 == 0)
        ODSD_LAUNCH(ODSD_KERNEL_ROUTER_LOGITS, (router_partial_kernel<XT, NE, true>), n_units / 4, 256, st,
                    (const XT *)x, (const XT *)gw, partial, (half_t *)x16, s->T, s->H, s->E, p.S, p.EG,
                    n_units, norm_ss, (const XT *)norm_w, (double)eps);
    else
        ODSD_LAUNCH(ODSD_KERNEL_ROUTER_LOGITS, (router_partial_kernel<XT, NE, false>), (n_units + 3) / 4, 256,
                    st, (const XT *)x, (const XT *)gw, partial, (half_t *)x16, s->T, s->H, s->E, p.S, p.EG,
                    n_units, norm_ss, (const XT *)norm_w, (double)eps);
}

int odsd_launch_router(const odsd_moe_shape *s, const void *x, const void *gate_w, int32_t *idx, float *w,
                       int64_t *idx64, void *x16, void *ws, size_t ws_bytes, hipStream_t st,
                       const double *norm_ss, const void *norm_w, float eps, double *logits,
                       const OdsdDispatchOut *disp) {
    const int rc = router_check(s);
    if (rc != ODSD_OK) return rc;
    if (disp && (!disp->counts || !disp->offsets || !disp->perm || !disp->inv || !disp->slot_token))
        return ODSD_ERR_NULL;
    if (s->T == 0) return ODSD_OK;
    if (!x || !gate_w || !idx || !w || !ws) return ODSD_ERR_NULL;
    if (norm_ss && (!norm_w || !odsd_aligned16(norm_w))) return norm_w ? ODSD_ERR_ALIGN : ODSD_ERR_NULL;
    if (!odsd_aligned16(x) || !odsd_aligned16(gate_w) || !odsd_aligned16(ws) ||
        (x16 && !odsd_aligned16(x16)))
        return ODSD_ERR_ALIGN;
    const RouterPlan p = router_plan(s, norm_ss != nullptr);
    if (ws_bytes < p.partial_bytes) return ODSD_ERR_WORKSPACE;
    double *partial = (double *)ws;
    const bool bf = s->act_dtype == ODSD_DT_BF16;
#define ROUTER_GO(NEV)                                                                   \
    do {                                                                                 \
        if (bf) launch_partial<uint16_t, NEV>(p, s, x, gate_w, partial, x16, st, norm_ss, norm_w, eps); \
        else launch_partial<float, NEV>(p, s, x, gate_w, partial, x16, st, norm_ss, norm_w, eps);       \
    } while (0)
    if (p.NE == 4) ROUTER_GO(4);
    else if (p.NE == 2) ROUTER_GO(2);
    else ROUTER_GO(1);
#undef ROUTER_GO
    ODSD_CHECK_LAUNCH();
    const int S_out = p.S % 4 == 0 ? p.S / 4 : p.S;
    // one wavefront per token; with few tokens each gets a workgroup of its own (a CU to itself:
    // 4.4 against 4.9 us at T = 256), with many, four share one (8.6 against 9.8 us at T = 4096)
    // (one CU then runs every token's selection: with 2 logits per lane 16 tokens take 10.2 us against
    // 8.6 for the two kernels, 5 tokens 7.2 against 8.4; with one logit per lane 16 tokens 5.4 against 8.1)
    const int topk_v = s->E <= 64 ? 1 : (s->E <= 128 ? 2 : (s->E <= 256 ? 4 : 8));
    if (disp && s->T * topk_v <= 16 && s->K <= 64 && s->T * s->K <= ROUTER_SMALL_PAIRS) {
        // a wavefront per token, and enough of them that the sort has at most 8 experts each
        const int small_waves = max(s->T, min(16, (s->E + 7) / 8));
#define TOPK_SMALL_GO(VV)                                                                                      \
    ODSD_LAUNCH(ODSD_KERNEL_ROUTER_TOPK, router_topk_dispatch_small_kernel<VV>, 1, 64 * small_waves, st,        \
                (const double *)partial, s->T, s->E, s->K, S_out, s->renorm, idx, w, idx64, logits, disp->counts, \
                disp->offsets, disp->perm, disp->inv, disp->slot_token, disp->counts_mirror, disp->mirror_tag)
        if (s->E <= 64) TOPK_SMALL_GO(1);
        else if (s->E <= 128) TOPK_SMALL_GO(2);
        else if (s->E <= 256) TOPK_SMALL_GO(4);
        else TOPK_SMALL_GO(8);
#undef TOPK_SMALL_GO
        ODSD_CHECK_LAUNCH();
        return ODSD_OK;
    }
    const int tk_waves = s->T <= 512 ? 1 : 4;
#define TOPK_GO(VV)                                                                                   \
    ODSD_LAUNCH(ODSD_KERNEL_ROUTER_TOPK, router_topk_kernel<VV>, (s->T + tk_waves - 1) / tk_waves, 64 * tk_waves, st, \
                (const double *)partial, s->T, s->E, s->K, S_out, s->renorm, idx, w, idx64, logits)
    if (s->E <= 64) TOPK_GO(1);
    else if (s->E <= 128) TOPK_GO(2);
    else if (s->E <= 256) TOPK_GO(4);
    else TOPK_GO(8);
#undef TOPK_GO
    ODSD_CHECK_LAUNCH();
    if (disp)
        return odsd_launch_dispatch(s, idx, disp->counts, disp->offsets, disp->perm, disp->inv, disp->slot_token, st,
                                    disp->counts_mirror, disp->mirror_tag);
    return ODSD_OK;
}

extern "C" int odsd_router_topk(const odsd_moe_shape *s, const void *x, const void *gate_w,
                                int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                                void *workspace, size_t workspace_bytes, void *stream) {
    return odsd_launch_router(s, x, gate_w, out_idx, out_w, out_idx64, x_f16, workspace, workspace_bytes,
                              (hipStream_t)stream, nullptr, nullptr, 0.0f, nullptr, nullptr);
}

extern "C" int odsd_route_dispatch(const odsd_moe_shape *s, const void *x, const void *gate_w,
                                   int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                                   int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv,
                                   int32_t *slot_token, void *workspace, size_t workspace_bytes, void *stream) {
    const OdsdDispatchOut d{counts, offsets, perm, inv, slot_token};
    return odsd_launch_router(s, x, gate_w, out_idx, out_w, out_idx64, x_f16, workspace, workspace_bytes,
                              (hipStream_t)stream, nullptr, nullptr, 0.0f, nullptr, &d);
}

extern "C" int odsd_route_dispatch_host_counts(const odsd_moe_shape *s, const void *x, const void *gate_w,
                                               int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                                               int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv,
                                               int32_t *slot_token, int64_t *counts_host, uint32_t tag,
                                               void *workspace, size_t workspace_bytes, void *stream) {
    const OdsdDispatchOut d{counts, offsets, perm, inv, slot_token, counts_host, tag};
    return odsd_launch_router(s, x, gate_w, out_idx, out_w, out_idx64, x_f16, workspace, workspace_bytes,
                              (hipStream_t)stream, nullptr, nullptr, 0.0f, nullptr, &d);
}

extern "C" int odsd_router_topk_logits(const odsd_moe_shape *s, const void *x, const void *gate_w,
                                       int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                                       double *out_logits, void *workspace, size_t workspace_bytes,
                                       void *stream) {
    if (!out_logits) return ODSD_ERR_NULL;
    return odsd_launch_router(s, x, gate_w, out_idx, out_w, out_idx64, x_f16, workspace, workspace_bytes,
                              (hipStream_t)stream, nullptr, nullptr, 0.0f, out_logits, nullptr);
}
