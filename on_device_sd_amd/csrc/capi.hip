// Entry points that tie the stages together: version/status strings and the whole-block
// call (RMSNorm -> router -> dispatch -> experts -> combine) that never returns to the host
// between stages.  Stands in for Qwen3MoELayerWithWeights.forward
// (demo/src/layers/moe_layer.py:193-254) and for route_experts + forward_moe called back to
// back (demo/src/model/qwen3_runner.py:86-119, :212-226) when the engine needs no decision
// in between.
#include "common.h"

#include <mutex>

extern "C" int odsd_version(void) { return ODSD_VERSION; }

extern "C" const char *odsd_status_string(int status) {
    switch (status) {
        case ODSD_OK: return "ok";
        case ODSD_ERR_NULL: return "a required pointer is NULL";
        case ODSD_ERR_SHAPE: return "bad shape (non-positive size or divisibility rule violated)";
        case ODSD_ERR_UNSUPPORTED: return "shape outside the supported range (E <= 512, K <= 64)";
        case ODSD_ERR_ALIGN: return "pointer not 16-byte aligned";
        case ODSD_ERR_WORKSPACE: return "workspace too small";
        case ODSD_ERR_LAUNCH: return "HIP launch failed";
        case ODSD_ERR_DTYPE: return "unknown dtype code";
        case ODSD_ERR_SCRATCH: return "the call needs more scratch memory than the library's static array holds";
        default: return "unknown status";
    }
}

struct MoeLayout {
    size_t router, xn, x16, idx, w, counts, offsets, perm, inv, slot_token, experts, total;
};

static MoeLayout moe_layout(const odsd_moe_shape *s) {
    MoeLayout l;
    const size_t T = s->T > 0 ? s->T : 1, P = T * s->K;
    const size_t act = s->act_dtype == ODSD_DT_F32 ? 4 : 2;
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o += odsd_round_up(bytes, 256); return at; };
    l.router = take(odsd_router_workspace_bytes(s));
    l.xn = take(T * s->H * act);
    l.x16 = take(T * s->H * 2);
    l.idx = take(P * 4);
    l.w = take(P * 4);
    l.counts = take((size_t)s->E * 4);
    l.offsets = take((size_t)(s->E + 1) * 4);
    l.perm = take(P * 4);
    l.inv = take(P * 4);
    l.slot_token = take(P * 4);
    l.experts = take(odsd_experts_workspace_bytes(s));
    l.total = o;
    return l;
}

extern "C" size_t odsd_moe_workspace_bytes(const odsd_moe_shape *s) {
    if (!s) return 0;
    if (odsd_router_workspace_bytes(s) == 0 || odsd_experts_workspace_bytes(s) == 0) return 0;
    return moe_layout(s).total;
}

thread_local OdsdProf *odsd_prof = nullptr;

// One whole block.
static int moe_forward_impl(const odsd_moe_shape *s, const void *x, const void *norm_weight, float eps,
                            const void *gate_w, const uint64_t *table, int32_t add_residual,
                            float *out_f32, void *out_act, int32_t *out_idx, float *out_w,
                            int32_t *out_counts, int32_t *out_offsets, int32_t *out_perm,
                            const double *row_sumsq_in, double *row_sumsq_out,
                            void *workspace, size_t workspace_bytes, void *stream,
                            bool prepared = false, const void *next_norm_w = nullptr) {
    // prepared: the previous block's combine has already applied this block's RMSNorm and left the
    // normalised rows and their fp16 copy in this workspace; next_norm_w: this block's combine does
    // the same for the block after it
    if (!s) return ODSD_ERR_NULL;
    const size_t need = odsd_moe_workspace_bytes(s);
    if (need == 0) return ODSD_ERR_SHAPE;
    if (s->T == 0) return ODSD_OK;
    if (!x || !gate_w || !table || !workspace) return ODSD_ERR_NULL;
    if (!odsd_aligned16(workspace)) return ODSD_ERR_ALIGN;
    if (workspace_bytes < need) return ODSD_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    const MoeLayout l = moe_layout(s);
    char *ws = (char *)workspace;
    int32_t *idx = out_idx ? out_idx : (int32_t *)(ws + l.idx);
    float *w = out_w ? out_w : (float *)(ws + l.w);
    int32_t *counts = out_counts ? out_counts : (int32_t *)(ws + l.counts);
    int32_t *offsets = out_offsets ? out_offsets : (int32_t *)(ws + l.offsets);
    int32_t *perm = out_perm ? out_perm : (int32_t *)(ws + l.perm);
    int32_t *inv = (int32_t *)(ws + l.inv);
    int32_t *slot_token = (int32_t *)(ws + l.slot_token);
    void *x16 = ws + l.x16;

    // RMSNorm: with the row statistics at hand (left by the previous block's combine) the router
    // kernel normalises on the fly; otherwise the stand-alone kernel runs first
    const void *xin = x;
    const bool fold = norm_weight && row_sumsq_in && !prepared;
    if (row_sumsq_out && !out_act) return ODSD_ERR_NULL;
    if (prepared) {
        xin = ws + l.xn;
    } else if (norm_weight && !fold) {
        const int rc = odsd_rmsnorm(x, norm_weight, s->act_dtype, s->T, s->H, eps, ws + l.xn, stream);
        if (rc != ODSD_OK) return rc;
        xin = ws + l.xn;
    }
    // shapes served by the one-launch expert kernel need no dispatch kernel: its workgroups scan the
    // expert ids themselves and leave counts / offsets / perm (inv and slot_token are not produced:
    // nothing after the experts reads them); otherwise the router launch dispatches as well (with few
    // tokens inside its top-k kernel, else by the dispatch kernel)
    const OdsdDispatchOut inside{counts, offsets, perm, nullptr, nullptr};
    const OdsdDispatchOut outside{counts, offsets, perm, inv, slot_token};
    const bool dispatch_inside = odsd_experts_dispatch_inside(s) && odsd_aligned16(idx);
    int rc = odsd_launch_router(s, xin, gate_w, idx, w, nullptr, prepared ? nullptr : x16, ws + l.router,
                                l.xn - l.router, st, fold ? row_sumsq_in : nullptr, norm_weight, eps,
                                nullptr, dispatch_inside ? nullptr : &outside);
    if (rc != ODSD_OK) return rc;
    // (the combine runs after this block's last reader of xn and x16, so it may overwrite them in place)
    const OdsdNextNorm nn{next_norm_w, eps, ws + l.xn, x16};
    return odsd_launch_experts(s, x16, table, idx, w, counts, offsets, perm, slot_token,
                               add_residual ? x : nullptr, out_f32, out_act, ws + l.experts,
                               l.total - l.experts, st, row_sumsq_out, dispatch_inside ? &inside : nullptr,
                               next_norm_w ? &nn : nullptr);
}

extern "C" int odsd_moe_forward(const odsd_moe_shape *s, const void *x, const void *norm_weight, float eps,
                                const void *gate_w, const uint64_t *table, int32_t add_residual,
                                float *out_f32, void *out_act, int32_t *out_idx, float *out_w,
                                int32_t *out_counts, int32_t *out_offsets, int32_t *out_perm,
                                const double *row_sumsq_in, double *row_sumsq_out,
                                void *workspace, size_t workspace_bytes, void *stream) {
    return moe_forward_impl(s, x, norm_weight, eps, gate_w, table, add_residual, out_f32, out_act, out_idx,
                            out_w, out_counts, out_offsets, out_perm, row_sumsq_in, row_sumsq_out,
                            workspace, workspace_bytes, stream);
}

extern "C" int odsd_moe_forward_events(const odsd_moe_shape *s, const void *x, const void *norm_weight,
                                       float eps, const void *gate_w, const uint64_t *table,
                                       int32_t add_residual, float *out_f32, void *out_act,
                                       const double *row_sumsq_in, double *row_sumsq_out,
                                       void *workspace, size_t workspace_bytes, void *stream,
                                       void *const *events, uint32_t *launched_mask) {
    if (!events || !launched_mask) return ODSD_ERR_NULL;
    for (int i = 0; i < 2 * ODSD_N_KERNELS; ++i)
        if (!events[i]) return ODSD_ERR_NULL;
    OdsdProf prof{events, 0u};
    odsd_prof = &prof;
    const int rc = moe_forward_impl(s, x, norm_weight, eps, gate_w, table, add_residual, out_f32, out_act,
                                    nullptr, nullptr, nullptr, nullptr, nullptr, row_sumsq_in, row_sumsq_out,
                                    workspace, workspace_bytes, stream);
    odsd_prof = nullptr;
    *launched_mask = prof.launched;
    return rc;
}

// ---- a stack of blocks ------------------------------------------------------------------------------
// L layers of  h = h + MoE_l(RMSNorm_l(h))  (Qwen3DecoderLayer.forward without attention,
// demo/src/layers/decoder_layer.py:126-140, looped over the layers) in one call: the blocks run as
// odsd_moe_forward would, every block after the first with its RMSNorm folded into the router kernel
// through the row statistic that the previous block's combine leaves.
struct StackLayout {
    size_t moe, hbuf[2], rowss[2], total;
};

static StackLayout stack_layout(const odsd_moe_shape *s) {
    StackLayout l;
    const size_t T = s->T > 0 ? s->T : 1;
    const size_t act = s->act_dtype == ODSD_DT_F32 ? 4 : 2;
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o += odsd_round_up(bytes, 256); return at; };
    l.moe = take(moe_layout(s).total);
    l.hbuf[0] = take(T * s->H * act);
    l.hbuf[1] = take(T * s->H * act);
    const size_t nchunk = ((size_t)s->H + 1023) / 1024;
    l.rowss[0] = take(T * nchunk * sizeof(double));
    l.rowss[1] = take(T * nchunk * sizeof(double));
    l.total = o;
    return l;
}

extern "C" size_t odsd_moe_stack_workspace_bytes(const odsd_moe_shape *s) {
    if (!s || odsd_moe_workspace_bytes(s) == 0) return 0;
    return stack_layout(s).total;
}

static int moe_stack_impl(const odsd_moe_shape *s, int32_t n_layers, const void *x, const void *const *norm_w,
                          const void *const *gate_w, const uint64_t *const *tables, float eps, void *out,
                          void *workspace, size_t workspace_bytes, void *stream, void *const *events,
                          uint32_t *masks) {
    if (!s) return ODSD_ERR_NULL;
    if (n_layers < 0) return ODSD_ERR_SHAPE;
    const size_t need = odsd_moe_stack_workspace_bytes(s);
    if (need == 0) return ODSD_ERR_SHAPE;
    if (s->T == 0 || n_layers == 0) return ODSD_OK;
    if (!x || !norm_w || !gate_w || !tables || !out || !workspace) return ODSD_ERR_NULL;
    for (int l = 0; l < n_layers; ++l)
        if (!norm_w[l] || !gate_w[l] || !tables[l]) return ODSD_ERR_NULL;
    if (x == out) return ODSD_ERR_SHAPE;                       // the first block reads x while it writes out
    if (!odsd_aligned16(workspace) || !odsd_aligned16(out)) return ODSD_ERR_ALIGN;
    if (workspace_bytes < need) return ODSD_ERR_WORKSPACE;
    const StackLayout sl = stack_layout(s);
    const MoeLayout ml = moe_layout(s);
    char *ws = (char *)workspace;
    char *mws = ws + sl.moe;
    void *hbuf[2] = {ws + sl.hbuf[0], ws + sl.hbuf[1]};
    double *rowss[2] = {(double *)(ws + sl.rowss[0]), (double *)(ws + sl.rowss[1])};
    OdsdProf prof{nullptr, 0u};
    auto begin_layer = [&](int l) {
        if (events) {
            prof.events = events + (size_t)l * 2 * ODSD_N_KERNELS;
            prof.launched = 0u;
            odsd_prof = &prof;
        }
    };
    auto end_layer = [&](int l) {
        if (events) {
            masks[l] = prof.launched;
            odsd_prof = nullptr;
        }
    };
    auto in_of = [&](int l) -> const void * { return l == 0 ? x : hbuf[(l - 1) & 1]; };
    auto out_of = [&](int l) -> void * { return l == n_layers - 1 ? out : hbuf[l & 1]; };

    // Between two blocks the combine of the first applies the RMSNorm of the second (it owns whole
    // rows and has the row statistic): the second block's router then reads normalised rows and its
    // expert kernel the fp16 copy, instead of every router workgroup normalising its columns again.  Rows longer than the combine keeps in registers fall back to handing over
    // the row statistic (the router kernel normalises on the fly).  Same bits either way.
    const bool hand_rows = odsd_combine_norm_supported(s);
    for (int l = 0; l < n_layers; ++l) {
        begin_layer(l);
        const bool last = l + 1 == n_layers;
        int rc;
        if (hand_rows)
            rc = moe_forward_impl(s, in_of(l), norm_w[l], eps, gate_w[l], tables[l], 1, nullptr, out_of(l),
                                  nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, mws, ml.total, stream,
                                  l > 0, last ? nullptr : norm_w[l + 1]);
        else
            rc = moe_forward_impl(s, in_of(l), norm_w[l], eps, gate_w[l], tables[l], 1, nullptr, out_of(l),
                                  nullptr, nullptr, nullptr, nullptr, nullptr, l > 0 ? rowss[(l - 1) & 1] : nullptr,
                                  last ? nullptr : rowss[l & 1], mws, ml.total, stream);
        end_layer(l);
        if (rc != ODSD_OK) return rc;
    }
    return ODSD_OK;
}

extern "C" int odsd_moe_stack_forward(const odsd_moe_shape *s, int32_t n_layers, const void *x,
                                      const void *const *norm_w, const void *const *gate_w,
                                      const uint64_t *const *tables, float eps, void *out, void *workspace,
                                      size_t workspace_bytes, void *stream) {
    return moe_stack_impl(s, n_layers, x, norm_w, gate_w, tables, eps, out, workspace, workspace_bytes, stream,
                          nullptr, nullptr);
}

extern "C" int odsd_moe_stack_forward_events(const odsd_moe_shape *s, int32_t n_layers, const void *x,
                                             const void *const *norm_w, const void *const *gate_w,
                                             const uint64_t *const *tables, float eps, void *out, void *workspace,
                                             size_t workspace_bytes, void *stream, void *const *events,
                                             uint32_t *launched_masks) {
    if (!events || !launched_masks) return ODSD_ERR_NULL;
    for (size_t i = 0; i < (size_t)(n_layers > 0 ? n_layers : 0) * 2 * ODSD_N_KERNELS; ++i)
        if (!events[i]) return ODSD_ERR_NULL;
    const int rc = moe_stack_impl(s, n_layers, x, norm_w, gate_w, tables, eps, out, workspace, workspace_bytes, stream,
                                  events, launched_masks);
    odsd_prof = nullptr;
    return rc;
}

// ---- the whole block for callers that cannot allocate -------------------------------------------
// The workspace of odsd_moe_forward lives in a device array of this library instead of coming from
// the caller.  Each GPU holds its own copy of the array at its own address; the address is looked
// up once per device (with that device current) and used from then on -- the array's name itself
// means nothing to host code.
static __device__ __align__(256) unsigned char scratch[ODSD_STATIC_SCRATCH_BYTES];

#define ODSD_MAX_DEVICES 64
static std::mutex scratch_mutex;
static void *scratch_ptr[ODSD_MAX_DEVICES];   // per device, filled on the first call on that device

static int scratch_for_current_device(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= ODSD_MAX_DEVICES) return ODSD_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
            (void)hipGetLastError();
            return ODSD_ERR_LAUNCH;
        }
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return ODSD_OK;
}

// Looks the array up for the current device.  Meant to be called once per device at set-up, so that
// the call below does no runtime query at all on its hot path -- in particular none while a stream
// is being captured into a HIP graph.
extern "C" int odsd_moe_static_init(void) {
    void *ws = nullptr;
    return scratch_for_current_device(&ws);
}

extern "C" int odsd_moe_forward_static(const odsd_moe_shape *s, const void *x, const void *norm_weight,
                                       float eps, const void *gate_w, const uint64_t *table,
                                       int32_t add_residual, float *out_f32, void *out_act,
                                       int32_t *out_idx, float *out_w, int32_t *out_counts,
                                       int32_t *out_offsets, int32_t *out_perm,
                                       const double *row_sumsq_in, double *row_sumsq_out, void *stream) {
    if (!s) return ODSD_ERR_NULL;
    const size_t need = odsd_moe_workspace_bytes(s);
    if (need == 0) return ODSD_ERR_SHAPE;
    if (need > (size_t)ODSD_STATIC_SCRATCH_BYTES) return ODSD_ERR_SCRATCH;
    if (s->T == 0) return ODSD_OK;
    void *ws = nullptr;
    const int rc = scratch_for_current_device(&ws);
    if (rc != ODSD_OK) return rc;
    // every kernel of the block writes what it later reads, so nothing in the array has to start at
    // zero and the previous call's contents are simply overwritten
    return moe_forward_impl(s, x, norm_weight, eps, gate_w, table, add_residual, out_f32, out_act, out_idx,
                            out_w, out_counts, out_offsets, out_perm, row_sumsq_in, row_sumsq_out, ws,
                            (size_t)ODSD_STATIC_SCRATCH_BYTES, stream);
}
