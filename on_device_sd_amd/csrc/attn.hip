// Causal attention over cached or packed keys (gfx950): the decode / verify step over the paged KV
// cache, and the prefill step over the step's own variable-length sequences.
//
// One workgroup per (sequence, KV head, group of 64 query rows, slice of the keys); a query row is
// one (token, query head) pair of the KV head's group, so with grouped-query attention a verify
// step of 8 tokens and 8 query heads per KV head fills the 64 rows.  Each of the 4 wavefronts owns
// 16 rows; the workgroup walks its keys 32 at a time:
//   * the tile's K and V rows are fetched once per workgroup (two tiles ahead, into registers) and
//     put into LDS one tile ahead, both as stored ([key][head_dim], 16- and 32-byte segments of a
//     row XORed with the key against bank conflicts); all wavefronts read their operands from
//     there (double buffered, one barrier per tile);
//   * S^T = K Q^T on the matrix cores (v_mfma_f32_16x16x32, keys as the A operand, the
//     wavefront's Q rows as the B operand held in registers), which leaves the scores of one
//     query row in the 4 lanes that share lane % 16 -- the layout the P operand of the second
//     product needs, so the probabilities never move between lanes;
//   * softmax in fp32 in the exp2 domain with the scale folded in; a row's reference point (the
//     value subtracted before exp2) follows its running maximum lazily, and the sum of the
//     probabilities stays a per-lane partial sum until the end, so most tiles exchange nothing
//     between lanes;
//   * O += P V with V^T as the B operand: a lane needs one head dimension of 8 keys, which
//     ds_read_b64_tr_b16 delivers from the row-major tile (the 16 lanes of a group read 4 keys x
//     16 dimensions and each gets one dimension's column of 4), so V is never transposed in memory.
// A verify step has few (sequence, KV head) pairs and long key lists, so the keys of one sequence
// are cut into `splits` slices handled by different workgroups; each leaves its reference point,
// sum and unnormalised output, and a small second kernel merges the slices of a row (the usual
// rescaling by exp2(m_slice - m_all)), in slice order.
// Paged form: the cache is addressed through the sequence's block table exactly as the reference
// gathers it: position p lives in slot block_table[p / block_size] * block_size + p % block_size.
// Packed form: the keys of sequence s are rows cu_seqlens_k[s] .. of k / v.
//
// Replaces Qwen3Attention._fallback_decode_attention (demo/src/layers/attention.py:290-352: gather
// of the cached K/V by slot, repeat_interleave for GQA, causal mask with offset k_len - q_len,
// scaled_dot_product_attention), the flash_attn_with_kvcache call it stands in for (:252-272) and
// the flash_attn_varlen_func call of the prefill branch (:229-240).
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));

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
    // variable-length mode (prefill): q / k / v rows of sequence s are q[cu_q[s] ..], k[cu_k[s] ..]
    // (contiguous, no block table); both null in paged mode
    const int32_t *cu_q, *cu_k;
    int splits;                // workgroups sharing one sequence's keys (blockIdx.z)
    float *part;               // splits > 1: partial results [seq, kvh, row group][split][64][HD + 4]
};

template <typename T> struct AttnT;
template <> struct AttnT<half_t> {
    typedef half8_t V8;
    __device__ static __forceinline__ float4_t mfma(V8 a, V8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint16_t from_f32(float v) { return __builtin_bit_cast(uint16_t, (half_t)v); }
    // two values, round to nearest even, as one 32-bit word (a in the low half)
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, h2));
    }
};
template <> struct AttnT<__bf16> {
    typedef bf16x8_t V8;
    __device__ static __forceinline__ float4_t mfma(V8 a, V8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint16_t from_f32(float v) { return f32_to_bf16(v); }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) {   // v_cvt_pk_bf16_f32
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        typedef float f2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, b2));
    }
};

// first query token of sequence seq: the sum of the query lengths before it, one wavefront-wide pass
__device__ __forceinline__ int attn_first_token(const int32_t *q_lens, int seq) {
    int part = 0;
    for (int i = threadIdx.x & 63; i < seq; i += 64) part += q_lens[i];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) part += __shfl_xor(part, d, ODSD_WAVE);
    return part;
}

template <typename T, int HD, bool ALIGNED>
__global__ __launch_bounds__(256, 2) void paged_attn_kernel(const AttnParams p) {
    typedef typename AttnT<T>::V8 V8;
    constexpr int NJ = HD / 32;          // 32-dim steps of the score product
    constexpr int NDB = HD / 16;         // 16-dim column blocks of the output
    constexpr int PIECES = 32 * (HD / 8) / 256;   // 16-byte pieces of a V tile per thread
    // V tile as stored ([key][HD]); the 32-byte segment (16 dims) of a row is XORed with vswz(key):
    // a transposing read touches 8 consecutive keys' segments of one column block per half wavefront
    __shared__ __attribute__((aligned(16))) uint16_t vs[2][32 * HD];
    auto vswz = [](int key) { return HD == 128 ? (key & 7) : ((key >> 1) & 3); };
    // K tile as stored ([key][HD]), 16-byte pieces of a row XORed with the key so that the 16 lanes
    // reading the same piece of 16 different keys hit different banks
    __shared__ __attribute__((aligned(16))) uint16_t kt[2][32 * HD];

    const int seq = blockIdx.x / p.KVH, kvh = blockIdx.x % p.KVH;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, kq = lane >> 4;
    const int Gq = p.H / p.KVH;
    const bool varlen = p.cu_k != nullptr;
    const int k_start = varlen ? p.cu_k[seq] : 0;
    const int L = varlen ? p.cu_k[seq + 1] - k_start : p.context_lens[seq];
    const int ql = varlen ? p.cu_q[seq + 1] - p.cu_q[seq] : (p.q_lens ? p.q_lens[seq] : 1);
    const int rows_total = ql * Gq;
    // (a sequence without cached keys still owns output rows: they are written as zeros below)
    if (ql <= 0 || (int)blockIdx.y * 64 >= rows_total) return;
    const int row0 = ((int)blockIdx.y * 4 + wave) * 16;
    const bool wave_active = row0 < rows_total;
    const int D = p.KVH * HD;
    const uint16_t *kc = (const uint16_t *)p.k_cache, *vc = (const uint16_t *)p.v_cache;
    const int32_t *bt = p.block_tables + (size_t)seq * p.max_blocks;

    // this lane's query row (B operand of S^T = K Q^T: lane (c, kq) holds Q[row c][32 j + 8 kq ..]);
    // fetched after the first K / V tiles are on their way (the first token of the sequence is a
    // prefix sum over the query lengths: a dependent chain that nothing else waits for)
    const int row = row0 + c;
    const bool row_ok = wave_active && row < rows_total;
    const int tok = row_ok ? row / Gq : 0, hq = row_ok ? row % Gq : 0;
    V8 qf[NJ];
    int q0 = seq;
    auto first_token = [&]() {
        if (varlen) q0 = p.cu_q[seq];
        else if (p.q_lens) q0 = attn_first_token(p.q_lens, seq);
    };
    auto load_q = [&]() {
        first_token();
        const uint16_t *qp = (const uint16_t *)p.q + ((size_t)(q0 + tok) * p.H + kvh * Gq + hq) * HD + 8 * kq;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            uint4_t raw = {0u, 0u, 0u, 0u};
            if (row_ok) raw = *(const uint4_t *)(qp + 32 * j);
            qf[j] = __builtin_bit_cast(V8, raw);
        }
    };
    const int kmax = row_ok ? L - ql + tok : -1;      // last position this row attends
    int kmin_wave = row_ok ? kmax : 0x7fffffff;        // tiles ending at or before it need no mask
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) kmin_wave = min(kmin_wave, __shfl_xor(kmin_wave, d, ODSD_WAVE));
    const float sc = p.scale_log2e;

    // per query row c: the reference point of its exponentials (the same in its 4 kq lanes) and
    // this lane's share of the sum of its probabilities
    float m_run = -INFINITY, l_run = 0.0f;
    float4_t o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Software pipeline over the 32-key tiles, two tiles deep.  A tile's K and V rows are fetched
    // once per workgroup, 16 bytes per thread and piece (piece = tid + 256 u -> key = piece /
    // (HD / 8), dims 8 * (piece % (HD / 8)) ..), two tiles ahead into one of two register sets;
    // one tile ahead they go to LDS, as stored, and every wavefront reads its
    // MFMA operands from there (K fetched per wavefront instead costs four times the L2 traffic
    // and was what bounded the kernel).  During tile `it`: the set that held tile `it` is refilled
    // with tile it + 2, the other set (tile it + 1) goes to the other LDS buffers, and the
    // block-table entries of tile it + 3 are requested BEFORE the fetches (the load counter retires
    // in order: a younger table read awaited by the next tile would otherwise drain the big
    // fetches issued before it).  The steady-state tiles fetch unconditionally and the last two
    // tiles are compiled without the fetch, so that no wait is placed after a join of "fetched"
    // and "did not fetch".
    // ALIGNED (block_size a multiple of 32): a tile lies in one cache block, so its table entry is
    // one wavefront-uniform read; otherwise every lane reads the entries of its own keys.
    constexpr int NE = ALIGNED ? 1 : PIECES;            // table entries a tile needs per lane
    const int k_last = L - 1;
    const int bs = p.block_size;
    auto entry_at = [&](int pos) -> int32_t { return varlen ? 0 : bt[min(min(pos, k_last) / bs, p.max_blocks - 1)]; };
    auto request = [&](int k0, int32_t (&e)[NE]) {
        if constexpr (ALIGNED) {
            e[0] = entry_at(k0);
        } else {
#pragma unroll
            for (int u = 0; u < PIECES; ++u) e[u] = entry_at(k0 + (tid + 256 * u) / (HD / 8));
        }
    };
    // slot of position pos (clamped into the sequence) in the block whose table entry is b; an
    // entry that is negative, beyond the table or beyond the cache reads slot 0
    auto slot_in = [&](int32_t b, int pos) -> int64_t {
        const int pc = min(pos, k_last);
        const int blk = pc / bs;
        const int64_t sl = (int64_t)b * bs + (pc - blk * bs);
        return (b >= 0 && blk < p.max_blocks && sl < p.num_slots) ? sl : 0;
    };
    uint4_t kreg[2][PIECES], vreg[2][PIECES];
    // fetch of the tile at k0, whose table entries are e
    auto fetch = [&](auto set, int k0, const int32_t (&e)[NE]) {
        constexpr int S = decltype(set)::value;
        if constexpr (ALIGNED) {
            // everything about the block is wavefront-uniform: one 64-bit base per tile, and a lane
            // adds the 32-bit offset of its row (clamped to the sequence's last key in the tile)
            const int k0c = min(k0, k_last & ~31);
            const int blk = k0c / bs;
            const int32_t b = e[0];
            const bool ok = varlen || (b >= 0 && blk < p.max_blocks && ((int64_t)b + 1) * bs <= p.num_slots);
            const int64_t slot0 = varlen ? (int64_t)k_start + k0c : (ok ? (int64_t)b * bs + (k0c - blk * bs) : 0);
            const int lim = ok ? k_last - k0c : 0;
            const size_t base = (size_t)slot0 * D + kvh * HD;
            const uint16_t *kb = kc + base, *vb = vc + base;
#pragma unroll
            for (int u = 0; u < PIECES; ++u) {
                const int piece = tid + 256 * u;
                const uint32_t off = (uint32_t)min(piece / (HD / 8), lim) * (uint32_t)D + 8 * (piece % (HD / 8));
                kreg[S][u] = *(const uint4_t *)(kb + off);
                vreg[S][u] = *(const uint4_t *)(vb + off);
            }
        } else {
#pragma unroll
            for (int u = 0; u < PIECES; ++u) {
                const int piece = tid + 256 * u;
                const int64_t sl = slot_in(e[u], k0 + piece / (HD / 8));
                const size_t off = (size_t)sl * D + kvh * HD + 8 * (piece % (HD / 8));
                kreg[S][u] = *(const uint4_t *)(kc + off);
                vreg[S][u] = *(const uint4_t *)(vc + off);
            }
        }
    };
    // a tile's K and V rows into the LDS buffers `buf`, 16 bytes per thread and piece, as stored
    auto store_kv = [&](auto set, int buf) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int piece = tid + 256 * u;
            const int key = piece / (HD / 8), ch = piece % (HD / 8);
            *(uint4_t *)&vs[buf][key * HD + 16 * ((ch >> 1) ^ vswz(key)) + 8 * (ch & 1)] = vreg[S][u];
            *(uint4_t *)&kt[buf][key * HD + 8 * (ch ^ (key & (HD / 8 - 1)))] = kreg[S][u];
        }
    };

    // this workgroup's slice of the 32-key tiles
    // (keys past the last one that any row of this workgroup attends are never visited: in a
    // prefill the early row groups stop long before the end of the sequence)
    const int last_tok = min(ql - 1, ((int)blockIdx.y * 64 + 63) / Gq);
    const int k_end = max(0, min(L, L - ql + last_tok + 1));   // no visible key at all: no tiles, zeros out
    const int all_tiles = (k_end + 31) / 32;
    const int per_split = (all_tiles + p.splits - 1) / p.splits;
    const int t_begin = min(all_tiles, (int)blockIdx.z * per_split);
    const int n_tiles = min(all_tiles, t_begin + per_split) - t_begin;
    const int kbase = t_begin * 32;
    int32_t pend[NE];                                   // entries of the tile after the newest fetched one

    // one tile; S: the register set that held it (free now). FETCH: tile it + 2 exists and is fetched (and
    // the entries of tile it + 3 requested); STORE: tile it + 1 exists and its V goes to LDS
    auto tile = [&](auto set, auto fetch_c, auto store_c, int it) {
        constexpr int S = decltype(set)::value;
        constexpr bool FETCH = decltype(fetch_c)::value, STORE = decltype(store_c)::value;
        const int k0 = kbase + it * 32, buf = it & 1;
        float4_t st[2];
        if (wave_active) {
            // scores S^T[key][row] for the two 16-key halves
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int key = 16 * t + c;
                    const uint4_t kraw = *(const uint4_t *)&kt[buf][key * HD + 8 * ((4 * j + kq) ^ (key & (HD / 8 - 1)))];
                    acc = AttnT<T>::mfma(__builtin_bit_cast(V8, kraw), qf[j], acc);
                }
                st[t] = acc;
            }
        }
        if constexpr (FETCH) {
            int32_t now[NE];
#pragma unroll
            for (int i = 0; i < NE; ++i) now[i] = pend[i];
            request(k0 + 96, pend);
            fetch(set, k0 + 64, now);
        }
        if (wave_active) {
            // lane (c, kq) holds keys k0 + 16 t + 4 kq + i of query row c (raw scores, before the
            // softmax scale).  Only tiles that reach past the first row's last key need the mask.
            float a[8] = {st[0].x, st[0].y, st[0].z, st[0].w, st[1].x, st[1].y, st[1].z, st[1].w};
            if (k0 + 31 > kmin_wave) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    a[i] = k0 + 16 * (i >> 2) + 4 * kq + (i & 3) <= kmax ? a[i] : -INFINITY;
            }
            float mx = fmaxf(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), fmaxf(fmaxf(a[4], a[5]), fmaxf(a[6], a[7])));
            // The reference point m_run of a row moves only when some score of the wavefront
            // exceeds it by more than 2^8 (probabilities up to 256 are as exact in fp16 / bf16 as
            // those below 1, and the sums are fp32): most tiles then need no exchange between
            // lanes at all -- no maximum, no rescaling of the output, no sum (l_run stays a
            // per-lane partial sum until the end).
            if (__any(mx * sc > m_run + 8.0f)) {
                mx = fmaxf(mx, __shfl_xor(mx, 16, ODSD_WAVE));
                mx = fmaxf(mx, __shfl_xor(mx, 32, ODSD_WAVE));
                const float m_new = fmaxf(m_run, mx * sc);
                // a row with nothing to attend yet keeps m = -inf: use 0 as the reference point then
                const float alpha = __builtin_amdgcn_exp2f(m_run - (m_new == -INFINITY ? 0.0f : m_new));   // m_run = -inf -> 0
                l_run *= alpha;
                m_run = m_new;
                // the output tile holds rows 4 kq + i in lane (dim, kq): fetch those rows' alpha
                float al[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) al[i] = __shfl(alpha, 4 * kq + i, ODSD_WAVE);
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    o[db].x *= al[0]; o[db].y *= al[1]; o[db].z *= al[2]; o[db].w *= al[3];
                }
            }
            const float neg_ref = m_run == -INFINITY ? 0.0f : -m_run;
            float pe[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) pe[i] = __builtin_amdgcn_exp2f(fmaf(a[i], sc, neg_ref));   // masked -> 0
            l_run += ((pe[0] + pe[1]) + (pe[2] + pe[3])) + ((pe[4] + pe[5]) + (pe[6] + pe[7]));
            const V8 pf = __builtin_bit_cast(V8, uint4_t{AttnT<T>::pack2(pe[0], pe[1]), AttnT<T>::pack2(pe[2], pe[3]),
                                                          AttnT<T>::pack2(pe[4], pe[5]), AttnT<T>::pack2(pe[6], pe[7])});
            // B operand of column block db: dimension 16 db + c of keys 4 kq .. + 3 and 16 + 4 kq .. + 3
            // (the keys of pf's 8 probabilities).  Lane c of a group addresses key 4 kq + c / 4,
            // dimensions 16 db + 4 (c % 4) .. + 3; the read hands it column c of the group's 4 x 16 block.
            const int key_a = 4 * kq + (c >> 2), key_b = key_a + 16;
            const uint16_t *va = &vs[buf][key_a * HD + 4 * (c & 3)], *vb = &vs[buf][key_b * HD + 4 * (c & 3)];
            const int swa = vswz(key_a), swb = vswz(key_b);
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                typedef short s4_t __attribute__((ext_vector_type(4)));
                typedef __attribute__((address_space(3))) s4_t lds_s4;
                const s4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)(va + 16 * (db ^ swa)));
                const s4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4 *)(vb + 16 * (db ^ swb)));
                typedef short s8_t __attribute__((ext_vector_type(8)));
                const V8 vf = __builtin_bit_cast(V8, s8_t{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w});
                o[db] = AttnT<T>::mfma(pf, vf, o[db]);
            }
        }
        // K and V of tile it + 1 (other set, fetched during tile it - 1) into the other LDS buffers
        if constexpr (STORE) store_kv(std::integral_constant<int, S ^ 1>{}, buf ^ 1);
        __syncthreads();
    };

    if (n_tiles > 0) {
        const std::integral_constant<int, 0> s0;
        const std::integral_constant<int, 1> s1;
        const std::true_type yes;
        const std::false_type no;
        // prologue: tiles 0 and 1 fetched, tile 0 in LDS, the entries of tile 2 requested
        request(kbase, pend);
        fetch(s0, kbase, pend);
        if (n_tiles > 1) {
            request(kbase + 32, pend);
            fetch(s1, kbase + 32, pend);
        }
        request(kbase + 64, pend);
        load_q();
        store_kv(s0, 0);
        __syncthreads();
        int it = 0;
        for (; it + 3 < n_tiles; it += 2) {
            tile(s0, yes, yes, it);
            tile(s1, yes, yes, it + 1);
        }
        // one to three tiles are left, `it` is even
        const int left = n_tiles - it;
        if (left == 3) {
            tile(s0, yes, yes, it);
            tile(s1, no, yes, it + 1);
            tile(s0, no, no, it + 2);
        } else if (left == 2) {
            tile(s0, no, yes, it);
            tile(s1, no, no, it + 1);
        } else {
            tile(s0, no, no, it);
        }
    } else {
        first_token();     // the rows are still written (zeros): they need the sequence's first row
    }

    l_run += __shfl_xor(l_run, 16, ODSD_WAVE);
    l_run += __shfl_xor(l_run, 32, ODSD_WAVE);
    if (wave_active && p.splits > 1) {
        // partial result of this slice: rows of the workgroup's 64, [HD] unnormalised output, m, l
        float *base = p.part + ((((size_t)blockIdx.x * gridDim.y + blockIdx.y) * p.splits + blockIdx.z) * 64) * (HD + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float *rowp = base + (size_t)(wave * 16 + 4 * kq + i) * (HD + 4);
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                rowp[16 * db + c] = i == 0 ? o[db].x : i == 1 ? o[db].y : i == 2 ? o[db].z : o[db].w;
        }
        if (kq == 0) {
            float *rowp = base + (size_t)(wave * 16 + c) * (HD + 4);
            rowp[HD] = m_run;
            rowp[HD + 1] = l_run;
        }
        return;
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

// Merge of the key slices: out[row] = sum_s exp2(m_s - m) O_s / sum_s exp2(m_s - m) l_s, slices in
// order. One workgroup per (sequence, KV head, row group, 256 VEC / HD rows): a thread owns VEC
// neighbouring output elements of a row and walks the slices.  VEC = 4 (one 16-byte load per slice;
// rows of the partial results are HD + 4 floats apart so that they stay 16-byte aligned) when there
// are at most 4 slices: a quarter of the workgroups and of the exponentials; with more slices there
// are few rows, and one element per thread keeps more of the chip busy.  (More rows per workgroup,
// taken in turn, measured slower: each turn is one more exposed load latency.)
template <typename T, int HD, int SB, int VEC>
__global__ __launch_bounds__(256) void paged_attn_merge_kernel(const AttnParams p) {
    static_assert(VEC == 1 || VEC == 4, "one element or one 16-byte vector per thread");
    constexpr int TPR = HD / VEC;                       // threads per row
    constexpr int RPW = 256 / TPR;                      // rows per workgroup
    const int seq = blockIdx.x / p.KVH, kvh = blockIdx.x % p.KVH;
    const int Gq = p.H / p.KVH;
    const bool varlen = p.cu_k != nullptr;
    const int ql = varlen ? p.cu_q[seq + 1] - p.cu_q[seq] : (p.q_lens ? p.q_lens[seq] : 1);
    const int rows_total = ql * Gq;
    // the sequence's first token: a chain of its own (a wavefront-wide sum over the query lengths),
    // started before the partial results are requested and by every lane of the wavefront
    int q0 = seq;
    if (varlen) q0 = p.cu_q[seq];
    else if (p.q_lens) q0 = attn_first_token(p.q_lens, seq);
    const int d = VEC * ((int)threadIdx.x % TPR);
    const int r = (int)blockIdx.z * RPW + (int)threadIdx.x / TPR;
    const int row = (int)blockIdx.y * 64 + r;
    if (row >= rows_total) return;
    const float *base = p.part + ((((size_t)blockIdx.x * gridDim.y + blockIdx.y) * p.splits) * 64 + r) * (HD + 4);
    const size_t stride = (size_t)64 * (HD + 4);
    // one pass, SB slices at a time (all their loads in flight together; SB = 4 when there are no
    // more than 4 slices, so that none is fetched twice), rescaling the running
    // sums whenever a batch raises the reference point
    float m = -INFINITY, l = 0.0f;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
    for (int s0 = 0; s0 < p.splits; s0 += SB) {
        float ms[SB], ls[SB];
        float os[SB][VEC];
#pragma unroll
        for (int u = 0; u < SB; ++u) {
            // (every load unconditional, on a clamped slice: loads under a branch serialise)
            const float *rp = base + (size_t)min(s0 + u, p.splits - 1) * stride;
            const float2_t ml = *(const float2_t *)(rp + HD);
            ms[u] = ml.x;
            ls[u] = ml.y;
            if constexpr (VEC == 4) {
                const float4_t v = *(const float4_t *)(rp + d);
                os[u][0] = v.x; os[u][1] = v.y; os[u][2] = v.z; os[u][3] = v.w;
            } else {
                os[u][0] = rp[d];
            }
        }
#pragma unroll
        for (int u = 0; u < SB; ++u) {
            if (s0 + u >= p.splits) {
                ms[u] = -INFINITY;
                ls[u] = 0.0f;
#pragma unroll
                for (int i = 0; i < VEC; ++i) os[u][i] = 0.0f;
            }
        }
        float mb = m;
#pragma unroll
        for (int u = 0; u < SB; ++u) mb = fmaxf(mb, ms[u]);
        const float ref = mb == -INFINITY ? 0.0f : mb;
        const float keep = exp2f(m - ref);            // m = -inf -> 0
        l *= keep;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] *= keep;
#pragma unroll
        for (int u = 0; u < SB; ++u) {
            const float f = exp2f(ms[u] - ref);
            l += f * ls[u];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += f * os[u][i];
        }
        m = mb;
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    const int tok = row / Gq, hq = row % Gq;
    uint16_t *op = (uint16_t *)p.out + ((size_t)(q0 + tok) * p.H + kvh * Gq + hq) * HD + d;
    if constexpr (VEC == 4) {
        typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
        *(u16x4 *)op = u16x4{AttnT<T>::from_f32(acc[0] * inv), AttnT<T>::from_f32(acc[1] * inv),
                             AttnT<T>::from_f32(acc[2] * inv), AttnT<T>::from_f32(acc[3] * inv)};
    } else {
        op[0] = AttnT<T>::from_f32(acc[0] * inv);
    }
}

#ifndef ATTN_TARGET_WGS
#define ATTN_TARGET_WGS 512
#endif
// key slices per sequence: enough workgroups to fill the chip, at least 8 tiles of keys each
static int attn_splits(int n_seqs, int kvh, int row_groups, int max_blocks, int block_size) {
    const long base = (long)n_seqs * kvh * row_groups;
    const long max_tiles = ((long)max_blocks * block_size + 31) / 32;
    long s = (ATTN_TARGET_WGS + base - 1) / base;
    if (s > max_tiles / 8) s = max_tiles / 8;
    if (s > 64) s = 64;
    return s < 1 ? 1 : (int)s;
}

extern "C" size_t odsd_paged_attention_workspace_bytes(int32_t n_seqs, int32_t max_q_len, int32_t num_heads,
                                                       int32_t num_kv_heads, int32_t head_dim,
                                                       int32_t block_size, int32_t max_blocks) {
    if (n_seqs <= 0 || max_q_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads ||
        block_size <= 0 || max_blocks <= 0 || (head_dim != 64 && head_dim != 128))
        return 0;
    const int64_t rows = (int64_t)max_q_len * (num_heads / num_kv_heads);
    if ((rows + 63) / 64 > 65535) return 0;
    const int rg = (int)((rows + 63) / 64);
    const int splits = attn_splits(n_seqs, num_kv_heads, rg, max_blocks, block_size);
    if (splits == 1) return 256;
    return odsd_round_up((size_t)n_seqs * num_kv_heads * rg * splits * 64 * (head_dim + 4) * sizeof(float), 256);
}

extern "C" int odsd_paged_attention(const void *q, const void *k_cache, const void *v_cache,
                                    const int32_t *block_tables, const int32_t *context_lens,
                                    const int32_t *q_lens, int32_t n_seqs, int32_t max_q_len,
                                    int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                                    int32_t block_size, int32_t max_blocks, int64_t num_slots,
                                    float softmax_scale, int32_t dtype, void *out, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    if (n_seqs < 0 || max_q_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads ||
        block_size <= 0 || max_blocks <= 0 || num_slots <= 0 || !(softmax_scale > 0.0f))
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
    const int64_t rows = (int64_t)max_q_len * (num_heads / num_kv_heads);
    if ((rows + 63) / 64 > 65535) return ODSD_ERR_UNSUPPORTED;     // grid.y
    const int rg = (int)((rows + 63) / 64);
    p.splits = attn_splits(n_seqs, num_kv_heads, rg, max_blocks, block_size);
    if (p.splits > 1) {
        const size_t need = odsd_paged_attention_workspace_bytes(n_seqs, max_q_len, num_heads, num_kv_heads,
                                                                 head_dim, block_size, max_blocks);
        if (!workspace) return ODSD_ERR_NULL;
        if (!odsd_aligned16(workspace)) return ODSD_ERR_ALIGN;
        if (workspace_bytes < need) return ODSD_ERR_WORKSPACE;
        p.part = (float *)workspace;
    }
    const dim3 grid((unsigned)(n_seqs * num_kv_heads), (unsigned)rg, (unsigned)p.splits);
    const int mvec = p.splits > 4 ? 1 : 4;
    const dim3 mgrid((unsigned)(n_seqs * num_kv_heads), (unsigned)rg, (unsigned)(64 / (256 * mvec / head_dim)));
    hipStream_t st = (hipStream_t)stream;
#define ATTN_GO(T, HDV)                                                              \
    do {                                                                             \
        if (block_size % 32 == 0) paged_attn_kernel<T, HDV, true><<<grid, 256, 0, st>>>(p);  \
        else paged_attn_kernel<T, HDV, false><<<grid, 256, 0, st>>>(p);              \
        if (p.splits > 4) paged_attn_merge_kernel<T, HDV, 8, 1><<<mgrid, 256, 0, st>>>(p);      \
        else if (p.splits > 1) paged_attn_merge_kernel<T, HDV, 4, 4><<<mgrid, 256, 0, st>>>(p); \
    } while (0)
    if (dtype == ODSD_DT_F16) {
        if (head_dim == 128) ATTN_GO(half_t, 128);
        else ATTN_GO(half_t, 64);
    } else {
        if (head_dim == 128) ATTN_GO(__bf16, 128);
        else ATTN_GO(__bf16, 64);
    }
#undef ATTN_GO
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

// ---- variable-length (prefill) form ----------------------------------------------------------------
extern "C" size_t odsd_varlen_attention_workspace_bytes(int32_t n_seqs, int32_t max_seqlen_q, int32_t max_seqlen_k,
                                                        int32_t num_heads, int32_t num_kv_heads, int32_t head_dim) {
    if (max_seqlen_k <= 0) return 0;
    return odsd_paged_attention_workspace_bytes(n_seqs, max_seqlen_q, num_heads, num_kv_heads, head_dim, 32,
                                                (max_seqlen_k + 31) / 32);
}

extern "C" int odsd_varlen_attention(const void *q, const void *k, const void *v, const int32_t *cu_seqlens_q,
                                     const int32_t *cu_seqlens_k, int32_t n_seqs, int32_t max_seqlen_q,
                                     int32_t max_seqlen_k, int32_t num_heads, int32_t num_kv_heads,
                                     int32_t head_dim, float softmax_scale, int32_t dtype, void *out,
                                     void *workspace, size_t workspace_bytes, void *stream) {
    if (n_seqs < 0 || max_seqlen_q <= 0 || max_seqlen_k <= 0 || num_heads <= 0 || num_kv_heads <= 0 ||
        num_heads % num_kv_heads || !(softmax_scale > 0.0f))
        return ODSD_ERR_SHAPE;
    if (head_dim != 64 && head_dim != 128) return ODSD_ERR_UNSUPPORTED;
    if (dtype != ODSD_DT_BF16 && dtype != ODSD_DT_F16) return ODSD_ERR_DTYPE;
    if (n_seqs == 0) return ODSD_OK;
    if (!q || !k || !v || !cu_seqlens_q || !cu_seqlens_k || !out) return ODSD_ERR_NULL;
    if (!odsd_aligned16(q) || !odsd_aligned16(k) || !odsd_aligned16(v)) return ODSD_ERR_ALIGN;
    if ((int64_t)n_seqs * num_kv_heads > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    AttnParams p{};
    p.q = q; p.k_cache = k; p.v_cache = v; p.out = out;
    p.cu_q = cu_seqlens_q; p.cu_k = cu_seqlens_k;
    p.n_seqs = n_seqs; p.H = num_heads; p.KVH = num_kv_heads;
    p.block_size = 32; p.max_blocks = (max_seqlen_k + 31) / 32; p.num_slots = 0;
    p.scale_log2e = softmax_scale * 1.4426950408889634f;
    const int64_t rows = (int64_t)max_seqlen_q * (num_heads / num_kv_heads);
    if ((rows + 63) / 64 > 65535) return ODSD_ERR_UNSUPPORTED;     // grid.y
    const int rg = (int)((rows + 63) / 64);
    p.splits = attn_splits(n_seqs, num_kv_heads, rg, p.max_blocks, 32);
    if (p.splits > 1) {
        const size_t need = odsd_varlen_attention_workspace_bytes(n_seqs, max_seqlen_q, max_seqlen_k, num_heads,
                                                                  num_kv_heads, head_dim);
        if (!workspace) return ODSD_ERR_NULL;
        if (!odsd_aligned16(workspace)) return ODSD_ERR_ALIGN;
        if (workspace_bytes < need) return ODSD_ERR_WORKSPACE;
        p.part = (float *)workspace;
    }
    const dim3 grid((unsigned)(n_seqs * num_kv_heads), (unsigned)rg, (unsigned)p.splits);
    const int mvec = p.splits > 4 ? 1 : 4;
    const dim3 mgrid((unsigned)(n_seqs * num_kv_heads), (unsigned)rg, (unsigned)(64 / (256 * mvec / head_dim)));
    hipStream_t st = (hipStream_t)stream;
#define ATTN_GO(T, HDV)                                                              \
    do {                                                                             \
        paged_attn_kernel<T, HDV, true><<<grid, 256, 0, st>>>(p);                    \
        if (p.splits > 4) paged_attn_merge_kernel<T, HDV, 8, 1><<<mgrid, 256, 0, st>>>(p);      \
        else if (p.splits > 1) paged_attn_merge_kernel<T, HDV, 4, 4><<<mgrid, 256, 0, st>>>(p); \
    } while (0)
    if (dtype == ODSD_DT_F16) {
        if (head_dim == 128) ATTN_GO(half_t, 128);
        else ATTN_GO(half_t, 64);
    } else {
        if (head_dim == 128) ATTN_GO(__bf16, 128);
        else ATTN_GO(__bf16, 64);
    }
#undef ATTN_GO
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}
