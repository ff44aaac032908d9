// Shared pieces of the W4 GEMM kernels: launch parameters, the int4 -> fp16 expansion and the
// wait-count helper.
#pragma once
#include "common.h"


typedef __attribute__((address_space(1))) uint4_t global_u4;
typedef __attribute__((address_space(1))) uint32_t global_u32;
typedef __attribute__((address_space(1))) char global_char;

struct GemmParams {
    const uint64_t *table;   // [E][4]
    const half_t *src;       // activations, fp16
    const int32_t *rowmap;   // slot -> source row (gate_up: token), or null: row = slot
    const int32_t *counts;
    const int32_t *offsets;
    half_t *h16;             // MODE 0 output [P][I]
    float *y;                // MODE 1 output [KS][P][ldo]: fp32 partial sums, or fp16 ones when y_f16
    int y_f16;               // the partial (KS == 1: complete) sums are stored as fp16
    int src_ld;              // elements per source row (= reduction length Kd)
    int G;                   // groups of 128 in the reduction dimension
    int NBLK;                // 16-row blocks of the (fused) weight matrix
    int nchunks;             // workgroup tiles along the rows
    int KS;                  // splits of the reduction dimension
    int gper;                // groups per split
    int PS;                  // prefill tile kernel: workgroups sharing the row passes of one tile
    int ldo;                 // I (MODE 0) or H (MODE 1)
    int P;
    int E;
    int n_wg;                // E * nchunks * KS (* PS)
    int wg_per_xcd;          // ceil(n_wg / 8)
    // gate_up with the dispatch inside (idx given; counts / offsets / rowmap are then NOT inputs):
    // every workgroup finds its expert's pairs in the id list itself, and the first workgroup of
    // each expert leaves counts / offsets / perm for the down projection and the combine
    const int32_t *idx;      // [P] expert id per (token, k) pair, or null
    int32_t *out_counts, *out_offsets, *out_perm;
    int K;
};

// Launch parameters of the one-launch expert kernel (experts_fused.hip)
#define ODSD_FUSED_X_BLOCKS 32   // (group, token block) areas of 4 KiB in its token-row LDS area
#define ODSD_FUSED_MAX_E 256     // experts it keeps row counts of (one workgroup per expert slice: E * S ~ 256)
struct FusedParams {
    const uint64_t *table;   // [E][4]
    const half_t *x16;       // activations, fp16 [T][H]
    const int32_t *rowmap;   // slot -> token
    const int32_t *counts;
    const int32_t *offsets;
    half_t *y;               // [S][P][H] fp16 partial sums of the down projection
    int H, I;
    int S;                   // slices of the intermediate dimension (workgroups per expert)
    int P;
    int G_up, G_dn;          // H / 128, I / 128
    // dispatch inside the kernel (idx given): every workgroup finds its expert's pairs in the id
    // list itself, and slice 0 of each expert leaves counts / offsets / perm for the combine
    const int32_t *idx;      // [P] expert id per (token, k) pair, or null: counts / offsets / rowmap are inputs
    int32_t *out_counts, *out_offsets, *out_perm;
    int K, E;
};

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// Constants of the code -> fp16 bit trick.  (x & mask) | magic is one VOP3 instruction
// (v_and_or_b32), but gfx9 VOP3 takes no literal and a single scalar operand, so with
// compile-time constants the compiler emits v_and + v_or.  Passing the constants through an
// empty asm once per kernel makes them opaque register values (masks in SGPRs, the magic
// number in a VGPR), and the fused form is selected.
struct DequantConsts {
    uint32_t m_lo, m_hi, magic;
};
__device__ __forceinline__ DequantConsts dequant_consts() {
    DequantConsts c{0x000F000Fu, 0x00F000F0u, 0x64006400u};
    asm volatile("" : "+s"(c.m_lo), "+s"(c.m_hi), "+v"(c.magic));
    return c;
}

// Per-(row, group) constants of w = (code - zero) * scale.  The integer part of the zero point
// is folded into the exact integer step that removes the 1024 (low nibbles) / 64 (high nibbles,
// pre-scaled by 16) offset of the fp16 bit trick, so only the fractional part of the zero
// point is rounded.
struct DequantPrep {
    half2_t S, CLO, CHI, NZ;
};
__device__ __forceinline__ DequantPrep dequant_prep(const uint32_t szbits) {
    const half2_t sz = as_half2(szbits);
    const half_t s = sz.x, z = sz.y;
    const half_t zi = __builtin_rintf16(z);
    const half_t zf = z - zi;                      // exact
    const half_t c_lo = (half_t)(-1024.0f) - zi;   // exact for |zi| <= 1024
    const half_t c_hi = (half_t)(-64.0f) - zi;
    const half_t nz = -(zf * s);
    return DequantPrep{half2_t{s, s}, half2_t{c_lo, c_lo}, half2_t{c_hi, c_hi}, half2_t{nz, nz}};
}

// one word (8 codes of one lane) -> 8 fp16 weights, the A operand of one 32-column MFMA step
__device__ __forceinline__ half8_t dequant_word(const DequantConsts &c, const DequantPrep &p, const uint32_t x) {
    const half2_t R16 = {(half_t)0.0625f, (half_t)0.0625f};
    const uint32_t xs = x >> 8;
    const half2_t t0 = as_half2((x & c.m_lo) | c.magic);
    const half2_t t1 = as_half2((x & c.m_hi) | c.magic);
    const half2_t t2 = as_half2((xs & c.m_lo) | c.magic);
    const half2_t t3 = as_half2((xs & c.m_hi) | c.magic);
    const half2_t q0 = t0 + p.CLO;
    const half2_t q1 = __builtin_elementwise_fma(t1, R16, p.CHI);
    const half2_t q2 = t2 + p.CLO;
    const half2_t q3 = __builtin_elementwise_fma(t3, R16, p.CHI);
    const half2_t v0 = __builtin_elementwise_fma(q0, p.S, p.NZ);
    const half2_t v1 = __builtin_elementwise_fma(q1, p.S, p.NZ);
    const half2_t v2 = __builtin_elementwise_fma(q2, p.S, p.NZ);
    const half2_t v3 = __builtin_elementwise_fma(q3, p.S, p.NZ);
    return half8_t{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
}

// 4 words (32 codes) of one lane -> 4 x 8 fp16 weights
__device__ __forceinline__ void dequant_tile(const DequantConsts &c, const uint4_t raw, const uint32_t szbits,
                                             half8_t (&a)[4]) {
    const DequantPrep p = dequant_prep(szbits);
    a[0] = dequant_word(c, p, raw.x);
    a[1] = dequant_word(c, p, raw.y);
    a[2] = dequant_word(c, p, raw.z);
    a[3] = dequant_word(c, p, raw.w);
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt = bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8)
#define ODSD_WAIT_VMCNT_LGKM0(N) \
    __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (((N) >> 4) << 14) | (7 << 4) | (0x0 << 8))
#define ODSD_WAIT_VMCNT(N) \
    __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (((N) >> 4) << 14) | (7 << 4) | (0xF << 8))

typedef __attribute__((address_space(3))) void lds_void;

// A wavefront-uniform global address as an opaque scalar: the compiler keeps it in an SGPR pair
// and uses it as the scalar base of a global load (saddr form) instead of folding the uniform
// part into the per-lane offset with a vector add per load.
__device__ __forceinline__ const global_char *scalar_base(const global_char *p) {
    asm volatile("" : "+s"(p));
    return p;
}
// The same for a loop-invariant integer that should be compared on the scalar unit inside a loop
// (hoisted out of the loop, such a comparison comes back as a lane mask that is moved through a
// vector register on every trip).
__device__ __forceinline__ int scalar_int(int v) {
    asm volatile("" : "+s"(v));
    return v;
}

// Asynchronous 16-byte-per-lane copy global -> LDS (no registers): lane l of the wavefront
// writes dst + 16*l.  `dst` must be the same for all lanes.  Written as inline assembly on
// purpose: the compiler models the builtin form as an access that may touch both memories,
// and while one is outstanding it turns every later wait -- including the lgkmcnt waits of
// ordinary LDS reads -- into a full drain, which serialises LDS reads and MFMAs.  Issued
// this way the copy is invisible to the compiler's counters, so
//   * the caller must order it against LDS reads of the same bytes itself
//     (s_waitcnt vmcnt + s_barrier), and
//   * vmcnt waits the compiler derives for other loads are at worst stricter than needed.
__device__ __forceinline__ void dma16_to_lds(const global_char *base, uint32_t byte_off, lds_void *dst) {
    const uint32_t m0v = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(byte_off), "s"(base)
                 : "memory");   // m0 is a reserved register: the compiler sets it itself before every use
}

