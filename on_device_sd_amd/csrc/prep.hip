// W4 quantiser, streaming-layout packer, RMSNorm and activation conversion for gfx950.
// All of these are HBM-bound byte movers; none of them is shaped as a GEMM.
#include "common.h"

// -----------------------------------------------------------------------------------------
// Quantiser: one wavefront per (row, group of 128 columns); lane l owns columns 2l, 2l+1.
// Arithmetic follows quantize_tensor (pre_exp/expert_skip_prediction/quant.py:99-106) per
// group with 4 bits: scale=(max-min)/15, zero=0-min/scale (a float, never rounded to an
// integer), q=clamp(round(w/scale+zero),0,15).  scale and zero are rounded to fp16 before
// the codes are computed.  Every fp32 step is a single correctly rounded operation
// (__f*_rn) so that a CPU restatement gets the same bits.
// -----------------------------------------------------------------------------------------
template <typename WT>
__global__ __launch_bounds__(256) void w4_quantize_kernel(const WT *__restrict__ w, int64_t n_units,
                                                          int64_t G, uint8_t *__restrict__ q,
                                                          uint16_t *__restrict__ scale,
                                                          uint16_t *__restrict__ zero) {
    const int lane = lane_id();
    const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // row * G + g
    if (unit >= n_units) return;
    const size_t base = (size_t)unit * ODSD_GROUP + 2 * lane;
    const float w0 = ActIO<WT>::load(w, base);
    const float w1 = ActIO<WT>::load(w, base + 1);
    const float mn = wave_min(fminf(w0, w1));
    const float mx = wave_max(fmaxf(w0, w1));
    const float s32 = __fdiv_rn(__fsub_rn(mx, mn), 15.0f);
    half_t s16 = (half_t)s32;
    if (!(s16 > (half_t)0.0f)) s16 = (half_t)1.0f;
    if (__builtin_isinf((float)s16)) s16 = (half_t)ODSD_FP16_MAX;
    const float sf = (float)s16;
    float z32 = __fsub_rn(0.0f, __fdiv_rn(mn, sf));
    z32 = fminf(fmaxf(z32, -ODSD_FP16_MAX), ODSD_FP16_MAX);
    const half_t z16 = (half_t)z32;
    const float zf = (float)z16;
    const float t0 = rintf(__fadd_rn(__fdiv_rn(w0, sf), zf));
    const float t1 = rintf(__fadd_rn(__fdiv_rn(w1, sf), zf));
    const uint32_t c0 = (uint32_t)fminf(fmaxf(t0, 0.0f), 15.0f);
    const uint32_t c1 = (uint32_t)fminf(fmaxf(t1, 0.0f), 15.0f);
    q[(size_t)unit * (ODSD_GROUP / 2) + lane] = (uint8_t)(c0 | (c1 << 4));
    if (lane == 0) {
        scale[unit] = __builtin_bit_cast(uint16_t, s16);
        zero[unit] = __builtin_bit_cast(uint16_t, z16);
    }
}

// -----------------------------------------------------------------------------------------
// Packer.  One thread per (destination block, group, lane): gathers its 4 words of 8 codes
// and writes them as one 16-byte store, so a wavefront later streams one [16 rows x 128
// columns] tile as a single contiguous 1 KiB read.
//   word j of lane l (r = l%16, kq = l/16): row 16*b+r, columns 128*g + 32*j + 8*kq + i,
//   code i in nibble {0,4,1,5,2,6,3,7}[i]  (pairs (0,1),(2,3),(4,5),(6,7) then fall out of
//   the masks 0x000F000F / 0x00F000F0 of the word and of the word >> 8).
// -----------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t permute_nibbles(uint32_t c) {
    // input nibble i (LSB first) = code i; output nibble pos(i)
    uint32_t o = 0;
    o |= ((c >> 0) & 0xFu) << 0;    // i=0 -> 0
    o |= ((c >> 4) & 0xFu) << 16;   // i=1 -> 4
    o |= ((c >> 8) & 0xFu) << 4;    // i=2 -> 1
    o |= ((c >> 12) & 0xFu) << 20;  // i=3 -> 5
    o |= ((c >> 16) & 0xFu) << 8;   // i=4 -> 2
    o |= ((c >> 20) & 0xFu) << 24;  // i=5 -> 6
    o |= ((c >> 24) & 0xFu) << 12;  // i=6 -> 3
    o |= ((c >> 28) & 0xFu) << 28;  // i=7 -> 7
    return o;
}

__global__ __launch_bounds__(256) void w4_pack_kernel(const uint8_t *__restrict__ q,
                                                      const uint16_t *__restrict__ scale,
                                                      const uint16_t *__restrict__ zero, int64_t nb_src,
                                                      int64_t G, int block_stride, int block_offset,
                                                      uint4_t *__restrict__ qp,
                                                      uint32_t *__restrict__ sz) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t total = nb_src * G * 64;
    if (gid >= total) return;
    const int lane = (int)(gid & 63);
    const int64_t bg = gid >> 6;
    const int64_t g = bg % G;
    const int64_t b = bg / G;
    const int r = lane & 15, kq = lane >> 4;
    const int64_t row = b * 16 + r;
    const int64_t kbytes = G * (ODSD_GROUP / 2);
    const uint32_t *src = (const uint32_t *)(q + row * kbytes + g * 64 + kq * 4);
    uint4_t out;
    out.x = permute_nibbles(src[0]);
    out.y = permute_nibbles(src[4]);   // +16 bytes
    out.z = permute_nibbles(src[8]);
    out.w = permute_nibbles(src[12]);
    const int64_t bd = b * block_stride + block_offset;
    qp[(bd * G + g) * 64 + lane] = out;
    if (kq == 0) {
        const uint32_t s = scale[row * G + g], z = zero[row * G + g];
        sz[(bd * G + g) * 16 + r] = s | (z << 16);
    }
}

// -----------------------------------------------------------------------------------------
// RMSNorm (demo/src/layers/layernorm.py:21-27): statistics in fp64, the normalised value is
// rounded to the activation dtype BEFORE the weight multiply, the product is rounded again.
// One workgroup per token.
// -----------------------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const XT *__restrict__ x, const XT *__restrict__ wt,
                                                      int H, double eps, XT *__restrict__ out) {
    __shared__ double red[2][4];
    const size_t row = (size_t)blockIdx.x * H;
    // The sum of squares is built exactly as the combine kernel builds the row statistic it
    // leaves for the next block (per 1024-column chunk: 4 consecutive columns per thread, a
    // wavefront sum, the 4 wavefront sums pairwise; chunks added in ascending order), so that
    // the stand-alone and the folded RMSNorm give the same bits.
    double tot = 0.0;
    for (int c0 = 0, n = 0; c0 < H; c0 += 1024, ++n) {
        const int c = c0 + (int)threadIdx.x * 4;
        double ss = 0.0;
        if (c < H) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const double v = (double)ActIO<XT>::load(x, row + c + i);
                ss += v * v;
            }
        }
        ss = wave_sum(ss);
        if (lane_id() == 0) red[n & 1][threadIdx.x >> 6] = ss;
        __syncthreads();
        tot += (red[n & 1][0] + red[n & 1][1]) + (red[n & 1][2] + red[n & 1][3]);
    }
    const double r = 1.0 / sqrt(tot / (double)H + eps);
    for (int h = threadIdx.x; h < H; h += 256) {
        const float xn = ActIO<XT>::round((float)((double)ActIO<XT>::load(x, row + h) * r));
        ActIO<XT>::store(out, row + h, __fmul_rn(xn, ActIO<XT>::load(wt, h)));
    }
}

// Fused residual add + RMSNorm (RMSNorm.add_rms_forward, demo/src/layers/layernorm.py:29-36):
//   s = float(x) + float(residual); residual_out = cast(s);
//   normed = cast(s * rsqrt(mean(s^2) + eps)) * weight   -- statistics over the UNROUNDED sum s.
// One workgroup per token; the sum is recomputed in the second sweep instead of being kept.
template <typename XT>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(const XT *__restrict__ x, const XT *__restrict__ res,
                                                          const XT *__restrict__ wt, int H, double eps,
                                                          XT *__restrict__ out, XT *__restrict__ res_out) {
    __shared__ double red[4];
    const size_t row = (size_t)blockIdx.x * H;
    double ss = 0.0;
    for (int h = threadIdx.x; h < H; h += 256) {
        const float s = __fadd_rn(ActIO<XT>::load(x, row + h), ActIO<XT>::load(res, row + h));
        ss += (double)s * (double)s;
    }
    ss = wave_sum(ss);
    if (lane_id() == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const double tot = (red[0] + red[1]) + (red[2] + red[3]);
    const double r = 1.0 / sqrt(tot / (double)H + eps);
    for (int h = threadIdx.x; h < H; h += 256) {
        const float s = __fadd_rn(ActIO<XT>::load(x, row + h), ActIO<XT>::load(res, row + h));
        ActIO<XT>::store(res_out, row + h, s);
        const float xn = ActIO<XT>::round((float)((double)s * r));
        ActIO<XT>::store(out, row + h, __fmul_rn(xn, ActIO<XT>::load(wt, h)));
    }
}

template <typename XT>
__global__ __launch_bounds__(256) void convert_f16_kernel(const XT *__restrict__ x, int64_t n,
                                                          half_t *__restrict__ o) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * 256;
    for (; i < n; i += step) o[i] = f32_to_f16_sat(ActIO<XT>::load(x, i));
}

// -----------------------------------------------------------------------------------------
// entry points
// -----------------------------------------------------------------------------------------
extern "C" int odsd_w4_quantize(const void *w, int32_t w_dtype, int64_t N, int64_t Kd, uint8_t *q,
                                uint16_t *scale, uint16_t *zero, void *stream) {
    if (!w || !q || !scale || !zero) return ODSD_ERR_NULL;
    if (N <= 0 || Kd <= 0 || Kd % ODSD_GROUP) return ODSD_ERR_SHAPE;
    const int64_t G = Kd / ODSD_GROUP, units = N * G;
    if ((units + 3) / 4 > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    const dim3 grid((unsigned)((units + 3) / 4));
    hipStream_t st = (hipStream_t)stream;
    if (w_dtype == ODSD_DT_F32)
        w4_quantize_kernel<float><<<grid, 256, 0, st>>>((const float *)w, units, G, q, scale, zero);
    else if (w_dtype == ODSD_DT_BF16)
        w4_quantize_kernel<uint16_t><<<grid, 256, 0, st>>>((const uint16_t *)w, units, G, q, scale, zero);
    else
        return ODSD_ERR_DTYPE;
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" size_t odsd_w4_packed_q_bytes(int64_t N, int64_t Kd) {
    if (N <= 0 || Kd <= 0 || N % 16 || Kd % ODSD_GROUP) return 0;
    return (size_t)N * (size_t)Kd / 2;
}
extern "C" size_t odsd_w4_packed_sz_bytes(int64_t N, int64_t Kd) {
    if (N <= 0 || Kd <= 0 || N % 16 || Kd % ODSD_GROUP) return 0;
    return (size_t)N * (size_t)(Kd / ODSD_GROUP) * 4;
}

extern "C" int odsd_w4_pack(const uint8_t *q, const uint16_t *scale, const uint16_t *zero, int64_t N,
                            int64_t Kd, int32_t block_stride, int32_t block_offset, uint32_t *qp,
                            uint16_t *sz, void *stream) {
    if (!q || !scale || !zero || !qp || !sz) return ODSD_ERR_NULL;
    if (N <= 0 || Kd <= 0 || N % 16 || Kd % ODSD_GROUP) return ODSD_ERR_SHAPE;
    if (block_stride < 1 || block_offset < 0 || block_offset >= block_stride) return ODSD_ERR_SHAPE;
    if (!odsd_aligned16(qp) || (((uintptr_t)q) & 3u) || (((uintptr_t)sz) & 3u)) return ODSD_ERR_ALIGN;
    const int64_t G = Kd / ODSD_GROUP, nb = N / 16, total = nb * G * 64;
    if ((total + 255) / 256 > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    w4_pack_kernel<<<dim3((unsigned)((total + 255) / 256)), 256, 0, (hipStream_t)stream>>>(
        q, scale, zero, nb, G, block_stride, block_offset, (uint4_t *)qp, (uint32_t *)sz);
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_rmsnorm(const void *x, const void *weight, int32_t dtype, int32_t T, int32_t H,
                            float eps, void *out, void *stream) {
    if (!x || !weight || !out) return ODSD_ERR_NULL;
    if (T < 0 || H <= 0) return ODSD_ERR_SHAPE;
    if (T == 0) return ODSD_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODSD_DT_F32)
        ODSD_LAUNCH(ODSD_KERNEL_NORM, rmsnorm_kernel<float>, T, 256, st, (const float *)x, (const float *)weight,
                    H, (double)eps, (float *)out);
    else if (dtype == ODSD_DT_BF16)
        ODSD_LAUNCH(ODSD_KERNEL_NORM, rmsnorm_kernel<uint16_t>, T, 256, st, (const uint16_t *)x,
                    (const uint16_t *)weight, H, (double)eps, (uint16_t *)out);
    else
        return ODSD_ERR_DTYPE;
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_add_rmsnorm(const void *x, const void *residual, const void *weight, int32_t dtype,
                                int32_t T, int32_t H, float eps, void *out, void *residual_out, void *stream) {
    if (!x || !residual || !weight || !out || !residual_out) return ODSD_ERR_NULL;
    if (T < 0 || H <= 0) return ODSD_ERR_SHAPE;
    if (T == 0) return ODSD_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODSD_DT_F32)
        add_rmsnorm_kernel<float><<<T, 256, 0, st>>>((const float *)x, (const float *)residual,
                                                     (const float *)weight, H, (double)eps, (float *)out,
                                                     (float *)residual_out);
    else if (dtype == ODSD_DT_BF16)
        add_rmsnorm_kernel<uint16_t><<<T, 256, 0, st>>>((const uint16_t *)x, (const uint16_t *)residual,
                                                        (const uint16_t *)weight, H, (double)eps,
                                                        (uint16_t *)out, (uint16_t *)residual_out);
    else
        return ODSD_ERR_DTYPE;
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}

extern "C" int odsd_convert_act_f16(const void *x, int32_t dtype, int64_t n, void *x_f16, void *stream) {
    if (!x || !x_f16) return ODSD_ERR_NULL;
    if (n < 0) return ODSD_ERR_SHAPE;
    if (n == 0) return ODSD_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ODSD_DT_F32)
        convert_f16_kernel<float><<<(unsigned)blocks, 256, 0, st>>>((const float *)x, n, (half_t *)x_f16);
    else if (dtype == ODSD_DT_BF16)
        convert_f16_kernel<uint16_t><<<(unsigned)blocks, 256, 0, st>>>((const uint16_t *)x, n,
                                                                      (half_t *)x_f16);
    else
        return ODSD_ERR_DTYPE;
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}
