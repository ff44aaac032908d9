// Causal attention of a decode / verify step over the paged KV cache (gfx950).
//
// One workgroup per (sequence, KV head, group of 64 query rows); a query row is one (token, query
// head) pair of the KV head's group, so with grouped-query attention a verify step of 8 tokens and
// 8 query heads per KV head fills the 64 rows.  Each of the 4 wavefronts owns 16 rows and walks
// the sequence's cached keys 32 at a time:
//   * S^T = K Q^T on the matrix cores (v_mfma_f32_16x16x32, keys as the A operand straight from
//     the cache rows, the wavefront's Q rows as the B operand held in registers), which leaves
//     the scores of one query row in the 4 lanes that share lane % 16 -- the layout the P operand
//     of the second product needs, so the probabilities never move between lanes;
//   * online softmax in fp32 (running maximum and sum per row, exp2 with the scale folded in);
//   * O += P V with V^T as the B operand: the 32 x head_dim tile of V is transposed through LDS
//     once per workgroup (double buffered, one barrier per tile) and shared by the wavefronts.
// The cache is addressed through the sequence's block table exactly as the reference gathers it:
// position p lives in slot block_table[p / block_size] * block_size + p % block_size.
//
// Replaces Qwen3Attention._fallback_decode_attention (demo/src/layers/attention.py:290-352: gather
// of the cached K/V by slot, repeat_interleave for GQA, causal mask with offset k_len - q_len,
// scaled_dot_product_attention) and the flash_attn_with_kvcache call it stands in for (:252-272).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

struct AttnParams {
    const void *q;             // [n_tokens, H, HD]
    const void *k_cache;       // [num_slots, KVH * HD]
    const void *v_cache;
    void *out;                 // [n_tokens, H, HD]
    const int32_t *q_lens;     // [n_seqs] or null (1 each)
    const int32_t *context_lens;
    const int32_t *block_tables;   // [n_seqs, max_blocks]
    int n_seqs, H, KVH, max_blocks, block_size;
    int64_t num_slots;
    float scale_log2e;         // softmax scale * log2(e)
};

template <typename T> struct AttnT;
template <> struct AttnT<half_t> {
    typedef half8_t V8;
    __device__ static __forceinline__ float4_t mfma(V8 a, V8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (half_t)v); }
};
template <> struct AttnT<__bf16> {
    typedef bf16x8_t V8;
    __device__ static __forceinline__ float4_t mfma(V8 a, V8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint16_t from_f32(float v) { return f32_to_bf16(v); }
};

// position of key `key` (0..31) of a tile inside a row of the transposed V tile: the 8 keys a
// lane group kq feeds to one product step (4 of each 16-key half) sit next to each other
__device__ __forceinline__ int vt_pos(int key) { return 8 * ((key & 15) >> 2) + 4 * (key >> 4) + (key & 3); }

template <typename T, int HD>
__global__ __launch_bounds__(256) void paged_attn_kernel(const AttnParams p) {
    typedef typename AttnT<T>::V8 V8;
    constexpr int NJ = HD / 32;          // 32-dim steps of the score product
    constexpr int NDB = HD / 16;         // 16-dim column blocks of the output
    constexpr int VT_LD = 40;            // halfs per row of the transposed V tile (32 keys + pad)
    constexpr int PIECES = 32 * (HD / 8) / 256;   // 16-byte pieces of a V tile per thread
    __shared__ __attribute__((aligned(16))) uint16_t vt[2][HD * VT_LD];

    const int seq = blockIdx.x / p.KVH, kvh = blockIdx.x % p.KVH;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, kq = lane >> 4;
    const int Gq = p.H / p.KVH;
    const int L = p.context_lens[seq];
    int ql = 1, q0 = 0;
    if (p.q_lens) {
        ql = p.q_lens[seq];
        for (int i = 0; i < seq; ++i) q0 += p.q_lens[i];
    } else {
        q0 = seq;
    }
    const int rows_total = ql * Gq;
    if (L <= 0 || ql <= 0 || (int)blockIdx.y * 64 >= rows_total) return;
    const int row0 = ((int)blockIdx.y * 4 + wave) * 16;
    const bool wave_active = row0 < rows_total;
    const int D = p.KVH * HD;
    const uint16_t *kc = (const uint16_t *)p.k_cache, *vc = (const uint16_t *)p.v_cache;
    const int32_t *bt = p.block_tables + (size_t)seq * p.max_blocks;

    // slot of position pos (clamped into the sequence; a broken table entry reads slot 0, masked below)
    auto slot_of = [&](int pos) -> int64_t {
        const int pc = min(pos, L - 1);
        const int blk = pc / p.block_size;
        const int64_t b = blk < p.max_blocks ? bt[blk] : -1;
        const int64_t s = b * p.block_size + (pc - blk * p.block_size);
        return (s >= 0 && s < p.num_slots) ? s : 0;
    };

    // this lane's query row (B operand of S^T = K Q^T: lane (c, kq) holds Q[row c][32 j + 8 kq ..])
    const int row = row0 + c;
    const bool row_ok = wave_active && row < rows_total;
    const int tok = row_ok ? row / Gq : 0, hq = row_ok ? row % Gq : 0;
    V8 qf[NJ];
    {
        const uint16_t *qp = (const uint16_t *)p.q + ((size_t)(q0 + tok) * p.H + kvh * Gq + hq) * HD + 8 * kq;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint4_t raw = {0u, 0u, 0u, 0u};
            if (row_ok) raw = *(const uint4_t *)(qp + 32 * j);
            qf[j] = __builtin_bit_cast(V8, raw);
        }
    }
    const int kmax = row_ok ? L - ql + tok : -1;      // last position this row attends

    float m_run = -INFINITY, l_run = 0.0f;             // per query row c (replicated over kq)
    float4_t o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Software pipeline over the 32-key tiles: the cache slots of a tile are looked up two tiles
    // ahead (block table -> slot is a dependent load), its K fragments and V pieces are fetched one
    // tile ahead, so that a tile's products never wait for a chain of two loads.
    //   K: lane (c, kq) reads 16 bytes of key row 16 t + c for each 32-dim step (the A operand)
    //   V: piece = tid + 256 u -> key = piece / (HD / 8), dims 8 * (piece % (HD / 8)) ..
    int64_t kslot[2], vslot[PIECES];
    auto lookup = [&](int k0) {
#pragma unroll
        for (int t = 0; t < 2; ++t) kslot[t] = slot_of(k0 + 16 * t + c);
#pragma unroll
        for (int u = 0; u < PIECES; ++u) vslot[u] = slot_of(k0 + (tid + 256 * u) / (HD / 8));
    };
    uint4_t kreg[2][NJ], vreg[PIECES];
    auto fetch = [&]() {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint16_t *kp = kc + kslot[t] * D + kvh * HD + 8 * kq;
#pragma unroll
            for (int j = 0; j < NJ; ++j) kreg[t][j] = *(const uint4_t *)(kp + 32 * j);
        }
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int ch = (tid + 256 * u) % (HD / 8);
            vreg[u] = *(const uint4_t *)(vc + vslot[u] * D + kvh * HD + 8 * ch);
        }
    };
    auto store_v = [&](int buf) {
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int piece = tid + 256 * u;
            const int key = piece / (HD / 8), ch = piece % (HD / 8);
            const int pos = vt_pos(key);
            const uint32_t w[4] = {vreg[u].x, vreg[u].y, vreg[u].z, vreg[u].w};
#pragma unroll
            for (int i = 0; i < 8; ++i)
                vt[buf][(8 * ch + i) * VT_LD + pos] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
        }
    };

    const int n_tiles = (L + 31) / 32;
    lookup(0);
    fetch();                                            // tile 0
    lookup(32);                                         // slots of tile 1 (clamped past the end)
    store_v(0);
    V8 kf[2][NJ];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < NJ; ++j) kf[t][j] = __builtin_bit_cast(V8, kreg[t][j]);
    __syncthreads();
    for (int it = 0; it < n_tiles; ++it) {
        const int k0 = it * 32, buf = it & 1;
        const bool more = it + 1 < n_tiles;
        if (more) {
            fetch();                                    // tile it + 1, in flight while this one is computed
            lookup(k0 + 64);                            // slots of tile it + 2
        }
        if (wave_active) {
            // scores S^T[key][row] for the two 16-key halves
            float4_t st[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NJ; ++j) acc = AttnT<T>::mfma(kf[t][j], qf[j], acc);
                st[t] = acc;
            }
            // lane (c, kq) holds keys k0 + 16 t + 4 kq + i of query row c: mask, running max and sum
            float sv[8];
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const float a[4] = {st[t].x, st[t].y, st[t].z, st[t].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int pos = k0 + 16 * t + 4 * kq + i;
                    const float v = pos <= kmax ? a[i] * p.scale_log2e : -INFINITY;
                    sv[4 * t + i] = v;
                    mx = fmaxf(mx, v);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, ODSD_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, ODSD_WAVE));
            const float m_new = fmaxf(m_run, mx);
            // a row with nothing to attend yet keeps m = -inf: use 0 as the reference point then
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = exp2f(m_run - m_ref);        // m_run = -inf -> 0
            float ps = 0.0f;
            uint16_t pb[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float e = exp2f(sv[i] - m_ref);         // masked -> 0
                pb[i] = AttnT<T>::from_f32(e);
                ps += e;
            }
            ps += __shfl_xor(ps, 16, ODSD_WAVE);
            ps += __shfl_xor(ps, 32, ODSD_WAVE);
            l_run = l_run * alpha + ps;
            m_run = m_new;
            const V8 pf = __builtin_bit_cast(V8, uint4_t{(uint32_t)pb[0] | ((uint32_t)pb[1] << 16),
                                                          (uint32_t)pb[2] | ((uint32_t)pb[3] << 16),
                                                          (uint32_t)pb[4] | ((uint32_t)pb[5] << 16),
                                                          (uint32_t)pb[6] | ((uint32_t)pb[7] << 16)});
            // the output tile holds rows 4 kq + i in lane (dim, kq): fetch those rows' alpha
            float al[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, 4 * kq + i, ODSD_WAVE);
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                const V8 vf = __builtin_bit_cast(V8, *(const uint4_t *)&vt[buf][(16 * db + c) * VT_LD + 8 * kq]);
                float4_t acc = o[db];
                acc.x *= al[0]; acc.y *= al[1]; acc.z *= al[2]; acc.w *= al[3];
                o[db] = AttnT<T>::mfma(pf, vf, acc);
            }
        }
        if (more) {
            store_v(buf ^ 1);
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < NJ; ++j) kf[t][j] = __builtin_bit_cast(V8, kreg[t][j]);
        }
        __syncthreads();
    }

    if (wave_active) {
        float inv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float l = __shfl(l_run, 4 * kq + i, ODSD_WAVE);
            inv[i] = l > 0.0f ? 1.0f / l : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = row0 + 4 * kq + i;
            if (r < rows_total) {
                const int t2 = r / Gq, h2 = r % Gq;
                uint16_t *op = (uint16_t *)p.out + ((size_t)(q0 + t2) * p.H + kvh * Gq + h2) * HD + c;
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    const float v = (i == 0 ? o[db].x : i == 1 ? o[db].y : i == 2 ? o[db].z : o[db].w) * inv[i];
                    op[16 * db] = AttnT<T>::from_f32(v);
                }
            }
        }
    }
}

extern "C" int odsd_paged_attention(const void *q, const void *k_cache, const void *v_cache,
                                    const int32_t *block_tables, const int32_t *context_lens,
                                    const int32_t *q_lens, int32_t n_seqs, int32_t max_q_len,
                                    int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                                    int32_t block_size, int32_t max_blocks, int64_t num_slots,
                                    float softmax_scale, int32_t dtype, void *out, void *stream) {
    if (n_seqs < 0 || max_q_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads ||
        block_size <= 0 || max_blocks <= 0 || num_slots <= 0)
        return ODSD_ERR_SHAPE;
    if (head_dim != 64 && head_dim != 128) return ODSD_ERR_UNSUPPORTED;
    if (dtype != ODSD_DT_BF16 && dtype != ODSD_DT_F16) return ODSD_ERR_DTYPE;
    if (n_seqs == 0) return ODSD_OK;
    if (!q || !k_cache || !v_cache || !block_tables || !context_lens || !out) return ODSD_ERR_NULL;
    if (!odsd_aligned16(q) || !odsd_aligned16(k_cache) || !odsd_aligned16(v_cache)) return ODSD_ERR_ALIGN;
    if ((int64_t)n_seqs * num_kv_heads > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    AttnParams p{};
    p.q = q; p.k_cache = k_cache; p.v_cache = v_cache; p.out = out;
    p.q_lens = q_lens; p.context_lens = context_lens; p.block_tables = block_tables;
    p.n_seqs = n_seqs; p.H = num_heads; p.KVH = num_kv_heads; p.max_blocks = max_blocks;
    p.block_size = block_size; p.num_slots = num_slots;
    p.scale_log2e = softmax_scale * 1.4426950408889634f;
    const int rows_max = max_q_len * (num_heads / num_kv_heads);
    const dim3 grid((unsigned)(n_seqs * num_kv_heads), (unsigned)((rows_max + 63) / 64));
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODSD_DT_F16) {
        if (head_dim == 128) paged_attn_kernel<half_t, 128><<<grid, 256, 0, st>>>(p);
        else paged_attn_kernel<half_t, 64><<<grid, 256, 0, st>>>(p);
    } else {
        if (head_dim == 128) paged_attn_kernel<__bf16, 128><<<grid, 256, 0, st>>>(p);
        else paged_attn_kernel<__bf16, 64><<<grid, 256, 0, st>>>(p);
    }
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}
