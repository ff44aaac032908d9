/*
 * odsd_moe.h -- C ABI of the MI355X (gfx950) MoE-block library, libodsd_moe.so.
 *
 * One hot path: router logits -> softmax -> top-k (optional renormalisation) ->
 * stable dispatch by expert -> grouped W4A16 (group-128 asymmetric, fp16 scale/zero)
 * SwiGLU experts -> deterministic weighted combine (+ residual), plus the RMSNorm that
 * precedes it in a decoder layer.
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless stated otherwise; all tensors are dense
 *    row-major; `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *  - every call is asynchronous on `stream`, performs no host synchronisation, allocates
 *    and frees nothing, and keeps no pointer after it returns;
 *  - every call returns an odsd_status (0 = ok); nothing aborts or throws across the ABI;
 *  - T tokens, H hidden size, E experts, K experts per token, I expert intermediate size,
 *    P = T*K (token, k) pairs; pair p = t*K + k;
 *  - activation dtype codes: ODSD_DT_F32 (float) or ODSD_DT_BF16 (bfloat16 bit patterns).
 *
 * Reference interfaces each entry point stands in for (paths relative to the
 * potatoZhx/on_device_sd tree):
 *   odsd_router_topk   Qwen3MoEGate.forward                    demo/src/layers/moe_layer.py:25-60
 *   odsd_router_topk_logits  + GPUOperators.router            demo/src/operators/gpu_operators.py:48-69
 *   odsd_route_dispatch      Qwen3ModelRunner.route_experts    demo/src/model/qwen3_runner.py:86-119
 *                      Qwen3ModelRunner.route_experts          demo/src/model/qwen3_runner.py:86-119
 *                      GPUOperators.router                     demo/src/operators/gpu_operators.py:48-69
 *   odsd_dispatch      mask / torch.where per expert           demo/src/model/qwen3_runner.py:303-314
 *   odsd_experts_w4    expert_forward_with_weights             demo/src/layers/mlp.py:209-231
 *                      _execute_moe_with_placement             demo/src/model/qwen3_runner.py:269-385
 *                      ExpertOperator.expert_forward           demo/src/operators/base_operator.py:19-34
 *   odsd_moe_forward   Qwen3MoELayerWithWeights.forward        demo/src/layers/moe_layer.py:193-254
 *                      ModelRunner.forward_moe                 demo/src/core/model_runner.py:175-193
 *   odsd_moe_stack_forward  Qwen3DecoderLayer.forward (MoE half), layer after layer
 *                                                              demo/src/layers/decoder_layer.py:126-140
 *   odsd_rmsnorm       RMSNorm.rms_forward                     demo/src/layers/layernorm.py:21-27
 *   odsd_w4_quantize   quantize_tensor (form, per group)       pre_exp/expert_skip_prediction/quant.py:85-108
 *   odsd_w4_pack       (no counterpart: the reference holds fp16/bf16 weights only;
 *                       parameter_loader.py:424-539 is where a loader would call it)
 *   odsd_kv_store      store_kvcache                           demo/src/layers/attention.py:32-79
 *   odsd_paged_attention  _fallback_decode_attention / flash_attn_with_kvcache   attention.py:252-352
 */
#ifndef ODSD_MOE_H
#define ODSD_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 110: events / static forms of the whole block, KV store, paged and packed attention added (100: the MoE block)
 * 112: odsd_moe_shape.max_rows (was reserved, 0 keeps the old meaning), odsd_experts_one_launch
 * 113: odsd_moe_static_init
 * 114: odsd_moe_stack_forward, odsd_moe_stack_forward_events
 * 115: odsd_route_dispatch_host_counts */
#define ODSD_VERSION 115

typedef enum odsd_status {
    ODSD_OK = 0,
    ODSD_ERR_NULL = 1,        /* a required pointer is NULL                              */
    ODSD_ERR_SHAPE = 2,       /* a size is non-positive or violates a divisibility rule  */
    ODSD_ERR_UNSUPPORTED = 3, /* valid but outside what the kernels cover (E, K limits)  */
    ODSD_ERR_ALIGN = 4,       /* a pointer is not 16-byte aligned                        */
    ODSD_ERR_WORKSPACE = 5,   /* workspace smaller than the *_workspace_bytes() answer   */
    ODSD_ERR_LAUNCH = 6,      /* the HIP runtime refused a launch                        */
    ODSD_ERR_DTYPE = 7,       /* unknown dtype code                                      */
    ODSD_ERR_SCRATCH = 8      /* odsd_moe_forward_static: the shape needs more than
                                 ODSD_STATIC_SCRATCH_BYTES of scratch memory             */
} odsd_status;

enum { ODSD_DT_F32 = 0, ODSD_DT_BF16 = 1, ODSD_DT_F16 = 2 /* attention entry point only */ };

/* Shape of one MoE layer call.  Rules: H % 128 == 0, I % 128 == 0, 1 <= K <= E <= 512,
 * K <= 64, T >= 0 (T == 0 is a no-op). */
typedef struct odsd_moe_shape {
    int32_t T, H, E, K, I;
    int32_t renorm;     /* 0: weights = softmax over all E gathered at the top-k
                           1: those weights divided by their sum (== softmax over the K
                              selected logits, the demo engine's top-k -> softmax)        */
    int32_t act_dtype;  /* dtype of x, gate weight, residual and out_act                 */
    int32_t max_rows;   /* 0: not known.  > 0: the caller states that no expert has more (token, k)
                           pairs than this in the call -- it has read the per-expert counts, as
                           the reference engine does between route_experts and forward_moe
                           (qwen3_runner.py:110-112).  The experts calls then stay away from a
                           plan that would stream an expert's weights a second time for a few
                           rows.  A wrong value costs time, never correctness.              */
} odsd_moe_shape;

/* Per-expert weight table: E rows of 4 device addresses (as uint64):
 *   [0] packed gate_up codes   [1] gate_up (scale, zero) pairs
 *   [2] packed down codes      [3] down (scale, zero) pairs
 * in the layout odsd_w4_pack writes.  A row whose first entry is 0 marks an expert whose
 * weights are not available: its pairs contribute nothing (qwen3_runner.py:330-333).
 * Substitution (qwen3_runner.py:322-329) is a row that points at another expert's arrays. */
#define ODSD_TABLE_COLS 4

int         odsd_version(void);
const char *odsd_status_string(int status);

/* ---- W4 storage ------------------------------------------------------------------- */
/* Canonical form of one [N, Kd] matrix (nn.Linear layout, Kd = input size, Kd % 128 == 0):
 *   q     uint8  [N, Kd/2]    code(2j) low nibble, code(2j+1) high nibble of byte j
 *   scale fp16   [N, Kd/128]  zero fp16 [N, Kd/128];  w ~= (code - zero) * scale          */
int odsd_w4_quantize(const void *w, int32_t w_dtype, int64_t N, int64_t Kd,
                     uint8_t *q, uint16_t *scale, uint16_t *zero, void *stream);

/* Bytes of the streaming layout of an [N, Kd] matrix (N % 16 == 0). */
size_t odsd_w4_packed_q_bytes(int64_t N, int64_t Kd);
size_t odsd_w4_packed_sz_bytes(int64_t N, int64_t Kd);

/* Canonical -> streaming layout.  Source 16-row block b goes to destination block
 * b*block_stride + block_offset, so gate_proj (stride 2, offset 0) and up_proj (stride 2,
 * offset 1) interleave into one [2I, H] gate_up matrix; down_proj uses (1, 0). */
int odsd_w4_pack(const uint8_t *q, const uint16_t *scale, const uint16_t *zero,
                 int64_t N, int64_t Kd, int32_t block_stride, int32_t block_offset,
                 uint32_t *qp, uint16_t *sz, void *stream);

/* ---- RMSNorm ------------------------------------------------------------------------ */
/* out = cast(x * rsqrt(mean(x^2) + eps)) * weight, cast BEFORE the weight multiply. */
int odsd_rmsnorm(const void *x, const void *weight, int32_t dtype, int32_t T, int32_t H,
                 float eps, void *out, void *stream);
/* Fused residual add + RMSNorm, RMSNorm.add_rms_forward of demo/src/layers/layernorm.py:29-36
 * (the post-attention norm of a real decoder layer, qwen3_runner.py:201-204):
 *   s = float(x) + float(residual); residual_out = cast(s);
 *   out = cast(s * rsqrt(mean(s^2) + eps)) * weight   (statistics over the unrounded sum).
 * out / residual_out may alias x / residual. */
int odsd_add_rmsnorm(const void *x, const void *residual, const void *weight, int32_t dtype,
                     int32_t T, int32_t H, float eps, void *out, void *residual_out, void *stream);

/* ---- Router ------------------------------------------------------------------------- */
size_t odsd_router_workspace_bytes(const odsd_moe_shape *s);
/* x [T,H], gate_w [E,H] in act_dtype.  Logits are accumulated in fp64.
 * out_idx  int32 [T,K] experts in descending logit order, ties to the lower index
 * out_w    float [T,K]
 * out_idx64 (optional) the same indices as int64, the dtype torch.topk returns
 * x_f16    (optional) fp16 copy of x [T,H], the operand format of odsd_experts_w4 */
int odsd_router_topk(const odsd_moe_shape *s, const void *x, const void *gate_w,
                     int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                     void *workspace, size_t workspace_bytes, void *stream);
/* The same, and the summed fp64 logits out_logits [T,E] (row-major) besides: the
 * `scores = F.linear(flat_hidden, router_weight)` that GPUOperators.router returns
 * (demo/src/operators/gpu_operators.py:48-69) and Qwen3MoEGate.forward computes first
 * (demo/src/layers/moe_layer.py:44). */
int odsd_router_topk_logits(const odsd_moe_shape *s, const void *x, const void *gate_w,
                            int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                            double *out_logits, void *workspace, size_t workspace_bytes, void *stream);

/* act_dtype [n] -> fp16 [n] (saturating); for callers that route elsewhere. */
int odsd_convert_act_f16(const void *x, int32_t dtype, int64_t n, void *x_f16, void *stream);

/* Router and dispatch in one call: what route_experts does before the host reads the activated
 * set (demo/src/model/qwen3_runner.py:86-119 followed by the per-expert masks of :303-314).
 * Outputs as odsd_router_topk and odsd_dispatch below. */
int odsd_route_dispatch(const odsd_moe_shape *s, const void *x, const void *gate_w,
                        int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                        int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv,
                        int32_t *slot_token, void *workspace, size_t workspace_bytes, void *stream);

/* The same call with a second copy of the counts written by the kernel itself to counts_host: [E] int64
 * in pinned host memory that the device can address (hipHostMalloc), entry e = (tag << 32) | counts[e],
 * one 8-byte store each.  The engine reads the activated set on the host between routing and
 * execution (qwen3_runner.py:110-112).  A device-to-host copy on the stream in front of the experts
 * cost 4 to 11 us per layer, an event record 3 to 5; with the tag (a number the caller changes from
 * call to call) the host can tell from the buffer alone when every entry has arrived, and nothing
 * but the kernels sits on the stream.  counts_host may be null (then this is odsd_route_dispatch). */
int odsd_route_dispatch_host_counts(const odsd_moe_shape *s, const void *x, const void *gate_w,
                                    int32_t *out_idx, float *out_w, int64_t *out_idx64, void *x_f16,
                                    int32_t *counts, int32_t *offsets, int32_t *perm, int32_t *inv,
                                    int32_t *slot_token, int64_t *counts_host, uint32_t tag, void *workspace,
                                    size_t workspace_bytes, void *stream);

/* ---- Dispatch ----------------------------------------------------------------------- */
/* Stable counting sort of the P pairs by expert id.
 * counts [E], offsets [E+1], perm [P] pair -> slot (-1 if the id is outside [0,E)),
 * inv [P] slot -> pair, slot_token [P] slot -> token (= inv / K). */
int odsd_dispatch(const odsd_moe_shape *s, const int32_t *idx, int32_t *counts,
                  int32_t *offsets, int32_t *perm, int32_t *inv, int32_t *slot_token,
                  void *stream);

/* ---- Experts + combine -------------------------------------------------------------- */
size_t odsd_experts_workspace_bytes(const odsd_moe_shape *s);
/* Grouped W4 gate_up -> SiLU*mul -> down over the dispatched pairs, then
 *   moe[t] = sum_k w[t,k] * y[perm[t*K+k]]   (fp32, k order, one rounding)
 * out_f32 (optional) float [T,H]  = moe (+ residual if given)
 * out_act (optional) act_dtype [T,H] = cast(residual + cast(moe)) as the reference rounds it
 * residual (optional) act_dtype [T,H]. */
int odsd_experts_w4(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                    const int32_t *idx, const float *w, const int32_t *counts,
                    const int32_t *offsets, const int32_t *perm, const int32_t *slot_token,
                    const void *residual, float *out_f32, void *out_act,
                    void *workspace, size_t workspace_bytes, void *stream);

/* The three kernels of odsd_experts_w4 one by one (same arguments, same results), for
 * callers that keep h / y themselves or time the stages:
 *   h_f16 fp16 [P, I] in slot order; y: a buffer of odsd_w4_down_splits(s)*P*H*4 bytes that
 *   odsd_w4_down fills and odsd_combine reads -- [splits][P][H] partial sums over slices of I,
 *   which odsd_combine adds in slice order: fp16 values (a value beyond +-65504 saturates), except
 *   for calls with T <= 16, which keep float partial sums when the reduction is split.
 * They stand in for the three F.linear calls of mlp.py:227-230 (gate/up fused with
 * SiLU*mul, then down) and the indexed "+=" of qwen3_runner.py:363. */
int     odsd_w4_gate_up_silu(const odsd_moe_shape *s, const void *x_f16, const uint64_t *table,
                             const int32_t *counts, const int32_t *offsets,
                             const int32_t *slot_token, void *h_f16, void *stream);
int32_t odsd_w4_down_splits(const odsd_moe_shape *s);
/* 1 if odsd_experts_w4 / odsd_moe_forward run gate_up, SiLU*mul and down of this shape in one
 * launch (one workgroup per expert slice, token rows resident in LDS, at most
 * ODSD_ONE_LAUNCH_ROWS rows of an expert per pass over its weights), 0 if they run the two
 * launches of the stage calls, negative status for a bad shape.  (A planning query: no
 * counterpart in the reference, whose per-expert loop has no such choice.) */
#define ODSD_ONE_LAUNCH_ROWS 32
int32_t odsd_experts_one_launch(const odsd_moe_shape *s);
int     odsd_w4_down(const odsd_moe_shape *s, const void *h_f16, const uint64_t *table,
                     const int32_t *counts, const int32_t *offsets, void *y, void *stream);
int     odsd_combine(const odsd_moe_shape *s, const void *y, const int32_t *idx, const float *w,
                     const int32_t *perm, const uint64_t *table, const void *residual,
                     float *out_f32, void *out_act, void *stream);

/* ---- Whole block -------------------------------------------------------------------- */
size_t odsd_moe_workspace_bytes(const odsd_moe_shape *s);
/* router -> dispatch -> experts -> combine in one call, no host round trip.
 * norm_weight (optional): apply RMSNorm(x) first (x is then the residual stream and is
 * also used as `residual` when add_residual != 0).
 * Routing outputs out_idx/out_w/out_counts/out_offsets/out_perm are optional.
 * row_sumsq_out (optional, needs out_act): double [T][ceil(H/1024)], sums of squares of every
 *   row of out_act, one per 1024-column chunk.
 * row_sumsq_in  (optional): the same statistic of x, e.g. the previous block's row_sumsq_out;
 *   with it and norm_weight the RMSNorm is folded into the router kernel (one launch fewer). */
int odsd_moe_forward(const odsd_moe_shape *s, const void *x, const void *norm_weight,
                     float eps, const void *gate_w, const uint64_t *table,
                     int32_t add_residual, float *out_f32, void *out_act,
                     int32_t *out_idx, float *out_w, int32_t *out_counts,
                     int32_t *out_offsets, int32_t *out_perm,
                     const double *row_sumsq_in, double *row_sumsq_out,
                     void *workspace, size_t workspace_bytes, void *stream);

/* ---- A stack of blocks ------------------------------------------------------------------------ */
/* n_layers blocks in a row on one hidden state:  h <- h + MoE_l(RMSNorm_l(h)),  l = 0 .. n_layers-1
 * (Qwen3DecoderLayer.forward without its attention half, demo/src/layers/decoder_layer.py:126-140,
 * looped over the layers as the model's forward does), with no host round trip between the blocks.
 *   x [T,H] act_dtype (not written); out [T,H] act_dtype: the hidden state after the last block
 *   norm_w, gate_w, tables: HOST arrays of n_layers device pointers -- per layer the RMSNorm weight
 *   [H], the router weight [E,H] (both act_dtype) and the expert table (as for odsd_moe_forward)
 * Every layer has the shape *s.  Results are those of n_layers odsd_moe_forward calls with
 * norm_weight and add_residual set, bit for bit (between two blocks the combine of the first owns
 * whole rows and applies the RMSNorm of the second; with H > 4096 it hands over the row statistic
 * and the second block's router kernel normalises on the fly -- the same bits either way). */
size_t odsd_moe_stack_workspace_bytes(const odsd_moe_shape *s);
int    odsd_moe_stack_forward(const odsd_moe_shape *s, int32_t n_layers, const void *x,
                              const void *const *norm_w, const void *const *gate_w,
                              const uint64_t *const *tables, float eps, void *out,
                              void *workspace, size_t workspace_bytes, void *stream);

/* ---- KV-cache store (the attention step next to the block) --------------------------------- */
/* Rows of this step's keys and values to their slots of the paged cache: for i in [0, N)
 *   row = src_index ? src_index[i] : i;  slot = slot_mapping[i];
 *   if slot != -1:  k_cache[slot, :] = key[row, :];  v_cache[slot, :] = value[row, :]
 * key / value: [n_src, D] with row strides key_stride / value_stride (in elements, >= D);
 * k_cache / v_cache: [num_slots, D] dense; elt_bytes 2 (fp16 / bf16) or 4; bytes are copied as
 * they are.  Slots must be distinct (two rows with one slot race, as in the reference's kernel);
 * a slot outside [0, num_slots) or a row outside [0, n_src) is skipped like slot -1.
 * Stands in for store_kvcache (demo/src/layers/attention.py:32-79) and, with src_index, for the
 * index_select of the draft tokens in front of it on the verify path (:222-228). */
int odsd_kv_store(const void *key, const void *value, int64_t key_stride, int64_t value_stride,
                  void *k_cache, void *v_cache, const int32_t *slot_mapping, const int32_t *src_index,
                  int32_t N, int32_t n_src, int32_t D, int32_t elt_bytes, int64_t num_slots, void *stream);

/* Causal attention of a decode / verify step over the paged KV cache.
 *   q            [n_tokens, num_heads, head_dim]: the sequences' query tokens one after the other,
 *                q_lens[s] of them for sequence s (q_lens == NULL: one each, a decode step)
 *   k_cache, v_cache  [num_slots, num_kv_heads * head_dim]; position p of sequence s lives in slot
 *                block_tables[s][p / block_size] * block_size + p % block_size
 *   context_lens [n_seqs]: cached tokens of the sequence INCLUDING this step's (stored before)
 *   query j of sequence s attends positions 0 .. context_lens[s] - q_lens[s] + j; query head h
 *   reads KV head h / (num_heads / num_kv_heads); scores scaled by softmax_scale (> 0); fp32 softmax
 *   out          [n_tokens, num_heads, head_dim] in the dtype of q (ODSD_DT_BF16 or ODSD_DT_F16)
 * max_q_len: an upper bound of q_lens (sizes the launch); head_dim 64 or 128.
 * workspace: odsd_paged_attention_workspace_bytes(...) bytes (with few sequences the keys of one
 * sequence are shared out between workgroups, whose partial results land there).
 * Stands in for Qwen3Attention._fallback_decode_attention and the flash_attn_with_kvcache call
 * it replaces (demo/src/layers/attention.py:252-352), on the context of
 * PagedKVCache.get_verify_context / get_attention_context (demo/src/memory/paged_kv_cache.py:500-580). */
int odsd_paged_attention(const void *q, const void *k_cache, const void *v_cache,
                         const int32_t *block_tables, const int32_t *context_lens,
                         const int32_t *q_lens, int32_t n_seqs, int32_t max_q_len,
                         int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                         int32_t block_size, int32_t max_blocks, int64_t num_slots,
                         float softmax_scale, int32_t dtype, void *out, void *workspace,
                         size_t workspace_bytes, void *stream);
size_t odsd_paged_attention_workspace_bytes(int32_t n_seqs, int32_t max_q_len, int32_t num_heads,
                                            int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                                            int32_t max_blocks);

/* Causal attention of a prefill step: variable-length sequences packed one after the other, keys
 * and values taken from the step's own k / v (no cache read).
 *   q [total_q, num_heads, head_dim], k / v [total_k, num_kv_heads, head_dim], contiguous
 *   cu_seqlens_q / cu_seqlens_k  int32 [n_seqs + 1]: row ranges of the sequences
 *   query i of a sequence attends keys 0 .. i + (k_len - q_len) of it (the mask is aligned to
 *   the bottom right corner when the lengths differ, as in flash-attn >= 2.1)
 * max_seqlen_q / max_seqlen_k: upper bounds of the lengths; softmax_scale > 0; head_dim 64 or 128;
 * workspace: odsd_varlen_attention_workspace_bytes(...) bytes.
 * Stands in for the flash_attn_varlen_func call of Qwen3Attention.forward
 * (demo/src/layers/attention.py:229-240; flash_attn itself is not part of the reference tree). */
int     odsd_varlen_attention(const void *q, const void *k, const void *v, const int32_t *cu_seqlens_q,
                              const int32_t *cu_seqlens_k, int32_t n_seqs, int32_t max_seqlen_q,
                              int32_t max_seqlen_k, int32_t num_heads, int32_t num_kv_heads,
                              int32_t head_dim, float softmax_scale, int32_t dtype, void *out,
                              void *workspace, size_t workspace_bytes, void *stream);
size_t odsd_varlen_attention_workspace_bytes(int32_t n_seqs, int32_t max_seqlen_q, int32_t max_seqlen_k,
                                             int32_t num_heads, int32_t num_kv_heads, int32_t head_dim);

/* The same call with every kernel timed, for measurement (no counterpart in the reference):
 * events = 2 * ODSD_N_KERNELS hipEvent_t handles created by the caller; the launch of kernel slot k
 * carries events[2k] and events[2k+1] as its start and stop events (hipExtLaunchKernel), so after
 * the stream has been synchronised hipEventElapsedTime(events[2k], events[2k+1]) is that kernel's
 * own duration; nothing is inserted between the kernels.  *launched_mask gets bit k set for every
 * slot that was launched (a block without a stand-alone RMSNorm leaves slot 0 out); the events of
 * the other slots are not touched.  Results are those of odsd_moe_forward. */
enum {
    ODSD_KERNEL_NORM = 0,           /* stand-alone RMSNorm                          */
    ODSD_KERNEL_ROUTER_LOGITS = 1,  /* fp64 logit partials (+ fp16 copy of x)       */
    ODSD_KERNEL_ROUTER_TOPK = 2,
    ODSD_KERNEL_DISPATCH = 3,
    ODSD_KERNEL_GATE_UP = 4,
    ODSD_KERNEL_DOWN = 5,
    ODSD_KERNEL_COMBINE = 6,
    ODSD_KERNEL_EXPERTS = 7,        /* gate_up + SiLU*mul + down as one launch (shapes with many
                                       small experts; slots 4 and 5 are then left out)          */
    ODSD_N_KERNELS = 8
};
int odsd_moe_forward_events(const odsd_moe_shape *s, const void *x, const void *norm_weight,
                            float eps, const void *gate_w, const uint64_t *table,
                            int32_t add_residual, float *out_f32, void *out_act,
                            const double *row_sumsq_in, double *row_sumsq_out,
                            void *workspace, size_t workspace_bytes, void *stream,
                            void *const *events, uint32_t *launched_mask);

/* The stack call with every kernel timed (measurement only, as odsd_moe_forward_events): events =
 * n_layers * 2 * ODSD_N_KERNELS handles, layer l using events[l * 2 * ODSD_N_KERNELS ..];
 * launched_masks [n_layers] (host) gets the slots each layer launched. */
int odsd_moe_stack_forward_events(const odsd_moe_shape *s, int32_t n_layers, const void *x,
                                  const void *const *norm_w, const void *const *gate_w,
                                  const uint64_t *const *tables, float eps, void *out,
                                  void *workspace, size_t workspace_bytes, void *stream,
                                  void *const *events, uint32_t *launched_masks);

/* odsd_moe_forward without a workspace argument and without any allocation, for callers that
 * cannot call hipMalloc: code under HIP graph capture, tight serving loops, harnesses that
 * forbid it.  It has no counterpart in the reference.  The workspace is a device array inside
 * the library (ODSD_STATIC_SCRATCH_BYTES per GPU the library runs on, held until the process
 * ends).  A shape whose odsd_moe_workspace_bytes() exceeds that size is refused with
 * ODSD_ERR_SCRATCH.  All calls on one GPU share the one array: calls that overlap on a GPU
 * (two streams, two threads) race; run them one after the other.  Arguments and results are
 * those of odsd_moe_forward. */
#define ODSD_STATIC_SCRATCH_BYTES (64u << 20)
/* Set-up of the call below for the current device (no counterpart in the reference either): looks the
 * array's device address up once and keeps it.  Call it once per device before the first
 * odsd_moe_forward_static -- always before one that runs while a stream is being captured into a HIP
 * graph, where the look-up must not happen.  (Without it the first odsd_moe_forward_static on a
 * device does the look-up itself, which is fine outside capture.)  Allocates nothing. */
int odsd_moe_static_init(void);
int odsd_moe_forward_static(const odsd_moe_shape *s, const void *x, const void *norm_weight,
                            float eps, const void *gate_w, const uint64_t *table,
                            int32_t add_residual, float *out_f32, void *out_act,
                            int32_t *out_idx, float *out_w, int32_t *out_counts,
                            int32_t *out_offsets, int32_t *out_perm,
                            const double *row_sumsq_in, double *row_sumsq_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ODSD_MOE_H */
