// KV-cache store for the attention step next to the MoE block: the rows of this step's keys and
// values go to their slots of the paged cache.  A byte mover: one wavefront copies one row of K and
// the matching row of V with 16-byte loads and stores, nothing is computed.
//
// Replaces store_kvcache_kernel / store_kvcache (demo/src/layers/attention.py:32-79) and the
// index_select of the draft tokens in front of it on the verify path (:222-228); the slot list is
// PagedKVCache.get_verify_context / get_attention_context's slot_mapping
// (demo/src/memory/paged_kv_cache.py:542-580).
#include "common.h"

template <typename V>
__global__ __launch_bounds__(256) void kv_store_kernel(const char *__restrict__ key, const char *__restrict__ value,
                                                       int64_t key_stride_b, int64_t value_stride_b,
                                                       char *__restrict__ k_cache, char *__restrict__ v_cache,
                                                       const int32_t *__restrict__ slot_mapping,
                                                       const int32_t *__restrict__ src_index, int N, int n_src,
                                                       int row_bytes, int64_t num_slots) {
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6);      // one wavefront per row
    if (i >= N) return;
    const int64_t slot = slot_mapping[i];
    if (slot < 0 || slot >= num_slots) return;               // -1: the row has no slot (attention.py:45-46)
    int64_t src = i;
    if (src_index) {
        src = src_index[i];
        if (src < 0 || src >= n_src) return;
    }
    const char *ks = key + src * key_stride_b, *vs = value + src * value_stride_b;
    char *kd = k_cache + slot * (int64_t)row_bytes, *vd = v_cache + slot * (int64_t)row_bytes;
    for (int b = lane_id() * (int)sizeof(V); b < row_bytes; b += 64 * (int)sizeof(V)) {
        const V kv = *(const V *)(ks + b);
        const V vv = *(const V *)(vs + b);
        *(V *)(kd + b) = kv;
        *(V *)(vd + b) = vv;
    }
}

extern "C" int odsd_kv_store(const void *key, const void *value, int64_t key_stride, int64_t value_stride,
                             void *k_cache, void *v_cache, const int32_t *slot_mapping,
                             const int32_t *src_index, int32_t N, int32_t n_src, int32_t D, int32_t elt_bytes,
                             int64_t num_slots, void *stream) {
    if (N < 0 || n_src < 0 || D <= 0 || num_slots < 0 || key_stride < D || value_stride < D) return ODSD_ERR_SHAPE;
    if (elt_bytes != 2 && elt_bytes != 4) return ODSD_ERR_DTYPE;
    if (N == 0) return ODSD_OK;
    if (!key || !value || !k_cache || !v_cache || !slot_mapping) return ODSD_ERR_NULL;
    if ((int64_t)D * elt_bytes > 0x7fffffffLL) return ODSD_ERR_SHAPE;
    const int row_bytes = D * elt_bytes;
    const int64_t ksb = key_stride * elt_bytes, vsb = value_stride * elt_bytes;
    const unsigned grid = (unsigned)((N + 3) / 4);
    hipStream_t st = (hipStream_t)stream;
    // widest access that every row start and the row length allow
    const uintptr_t all = (uintptr_t)key | (uintptr_t)value | (uintptr_t)k_cache | (uintptr_t)v_cache |
                          (uintptr_t)ksb | (uintptr_t)vsb | (uintptr_t)row_bytes;
#define KV_GO(V)                                                                                              \
    kv_store_kernel<V><<<grid, 256, 0, st>>>((const char *)key, (const char *)value, ksb, vsb, (char *)k_cache, \
                                             (char *)v_cache, slot_mapping, src_index, N, n_src, row_bytes, num_slots)
    if ((all & 15u) == 0) KV_GO(uint4_t);
    else if ((all & 3u) == 0) KV_GO(uint32_t);
    else KV_GO(uint16_t);
#undef KV_GO
    ODSD_CHECK_LAUNCH();
    return ODSD_OK;
}
