// Host-side argument checking shared by the attention entry points.
#include "attn_common.h"

int mi_attn_validate(const mi_attn_args* a, const char* who) {
    if (!a) return mi_fail(MI_E_NULL, "%s: args is null", who);
    if (!a->q || !a->k || !a->v || !a->cu_seqlens_q) return mi_fail(MI_E_NULL, "%s: q, k, v and cu_seqlens_q are required", who);
    if (a->dtype != MI_BF16) return mi_fail(MI_E_DTYPE, "%s: only bf16 is supported (dtype code %d)", who, a->dtype);
    if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 96 && a->head_dim != 128)
        return mi_fail(MI_E_SHAPE, "%s: head_dim %d unsupported (32, 64, 96, 128)", who, a->head_dim);
    if (a->n_q_heads <= 0 || a->n_kv_heads <= 0 || a->n_q_heads % a->n_kv_heads != 0)
        return mi_fail(MI_E_SHAPE, "%s: n_q_heads=%d must be a positive multiple of n_kv_heads=%d", who, a->n_q_heads, a->n_kv_heads);
    if (a->total_q < 0 || a->total_k < 0 || a->total_q > 0x7fffffffLL || a->total_k > 0x7fffffffLL || a->n_docs < 0)
        return mi_fail(MI_E_SHAPE, "%s: bad token counts q=%lld k=%lld docs=%d", who, (long long)a->total_q, (long long)a->total_k, a->n_docs);
    if (a->total_q > 0 && (a->n_docs < 1 || a->total_k < 1))
        return mi_fail(MI_E_SHAPE, "%s: non-empty query needs at least one document and one key", who);
    if (!mi_aligned16(a->q) || !mi_aligned16(a->k) || !mi_aligned16(a->v))
        return mi_fail(MI_E_ALIGN, "%s: q, k, v must be 16-byte aligned", who);
    if (a->q_stride_token % 8 || a->q_stride_head % 8 || a->k_stride_token % 8 || a->k_stride_head % 8 ||
        a->v_stride_token % 8 || a->v_stride_head % 8)
        return mi_fail(MI_E_ALIGN, "%s: strides must be multiples of 8 elements", who);
    if (!(a->softmax_scale > 0.f)) return mi_fail(MI_E_SHAPE, "%s: softmax_scale must be positive", who);
    if (a->rotary_cos || a->rotary_sin) {
        if (!a->rotary_cos || !a->rotary_sin || !a->position_ids_q)
            return mi_fail(MI_E_NULL, "%s: fused rotary needs cos, sin and the query position ids", who);
        if (a->head_dim != 64 && a->head_dim != 128) return mi_fail(MI_E_SHAPE, "%s: fused rotary needs head_dim 64 or 128", who);
        if (a->rotary_table_rows <= 0 || a->rotary_table_rows > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "%s: bad rotary table size", who);
        if (!mi_aligned16(a->rotary_cos) || !mi_aligned16(a->rotary_sin)) return mi_fail(MI_E_ALIGN, "%s: rotary tables must be 16-byte aligned", who);
    }
    if (!(a->dropout_p >= 0.f) || a->dropout_p >= 1.f) return mi_fail(MI_E_SHAPE, "%s: dropout_p must be in [0, 1)", who);
    return MI_OK;
}

void mi_attn_fill_params(const mi_attn_args* a, AttnParams* p) {
    *p = AttnParams{};
    p->q = (const __bf16*)a->q; p->k = (const __bf16*)a->k; p->v = (const __bf16*)a->v;
    p->o = (__bf16*)a->o; p->lse = a->lse;
    p->cu_q = a->cu_seqlens_q; p->cu_k = a->cu_seqlens_k ? a->cu_seqlens_k : a->cu_seqlens_q;
    p->n_docs = a->n_docs; p->causal = a->causal;
    p->total_q = (int)a->total_q; p->total_k = (int)a->total_k;
    p->nq = a->n_q_heads; p->nkv = a->n_kv_heads; p->n_rep = a->n_q_heads / a->n_kv_heads;
    p->q_st = a->q_stride_token; p->q_sh = a->q_stride_head;
    p->k_st = a->k_stride_token; p->k_sh = a->k_stride_head;
    p->v_st = a->v_stride_token; p->v_sh = a->v_stride_head;
    p->o_st = a->o_stride_token; p->o_sh = a->o_stride_head;
    p->scale = a->softmax_scale;
    p->scale_log2 = a->softmax_scale * 1.4426950408889634f;
    if (a->rotary_interleaved) {
        p->cos32 = (const float*)a->rotary_cos; p->sin32 = (const float*)a->rotary_sin;
    } else {
        p->cos = (const __bf16*)a->rotary_cos; p->sin = (const __bf16*)a->rotary_sin;
    }
    p->pos_q = a->position_ids_q; p->pos_k = a->position_ids_k; p->table_rows = (int)a->rotary_table_rows;
    if (a->dropout_p > 0.f) {
        int t = (int)(a->dropout_p * 256.0f + 0.5f);
        t = t < 1 ? 1 : (t > 255 ? 255 : t);
        p->drop_thr = (uint32_t)t;
        p->drop_rscale = 256.0f / (float)(256 - t);
        p->drop_seed = (uint32_t)(a->dropout_seed & 0xffffffffu) ^ (uint32_t)(a->dropout_seed >> 32);
    }
}

// Compute units of the current device (256 on an MI355X), asked once per device.
int mi_compute_units() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}
