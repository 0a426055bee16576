// Launch parameters shared by the attention kernels and their callers.
#pragma once
#include "mynn_common.h"

namespace mynn {

struct AttnParams {
    void *out;
    const void *q, *k, *v, *k_scale, *v_scale;
    float scale;
    int is_causal;
    int B, Sq, Hq, Hkv, cache_len;
    int active;               // host value, used when d_active == nullptr
    const int32_t *d_active;  // device value (graph replay)
    int q_pos_offset;         // host value, used when d_active == nullptr
    int nsplit;
    int slice;                // key rows per slice (gridDim.y slices cover the cache)
    int heads_per_wg;         // query heads one workgroup serves (divides Hq/Hkv)
    // fused decode form: raw qkv projection row(s) [B, (Hq+2*Hkv)*D], RoPE tables, device position;
    // K and V then are the caches the new row is appended to
    const void *qkv, *cos_t, *sin_t;
    const int64_t *d_pos;
    // additive mask (operator slot 3), storage type: element (b * Hq + h) * mask_os + sq * mask_rs + key
    const void *mask;
    long mask_os, mask_rs;
    int rope_q;               // prefill kernel: Q is un-rotated; rotate row sq by table row d_pos[sq] (cos_t, sin_t, d_pos above)
    const int32_t *d_past;    // fused decode form: cache row the new token is appended to (KVCacheUpdate's offset)
    // paged K/V (page_table != nullptr; streaming decode and prefill kernels): k and v are pools [n_pages, Hkv, P, D] with
    // P = 1 << page_shift rows per page (an int8 cache: scale pools [n_pages, Hkv, P]); row r of sequence b lives in pool
    // page page_table[b * pages_per_seq + (r >> page_shift)], row r % P of it; cache_len is pages_per_seq * P.  Entries of
    // pages no row below the active length falls into are never read.
    const int32_t *page_table;
    int page_shift, pages_per_seq;
    float *part_o;            // [B*Hq*Sq, nsplit, D]
    float *part_ml;           // [B*Hq*Sq, nsplit, 2]
    // element strides of Q and out: batch, head, row.  Reference layout [B,Hq,Sq,D] is
    // (Hq*Sq*D, Sq*D, D); token-major [B,Sq,Hq*D] is (Sq*Hq*D, D, Hq*D).
    long q_bs, q_hs, q_rs, o_bs, o_hs, o_rs;
};

inline void attn_reference_layout(AttnParams &p, int D) {
    p.q_bs = p.o_bs = (long)p.Hq * p.Sq * D;
    p.q_hs = p.o_hs = (long)p.Sq * D;
    p.q_rs = p.o_rs = D;
}
inline void attn_token_major_layout(AttnParams &p, int D) {
    p.q_bs = p.o_bs = (long)p.Sq * p.Hq * D;
    p.q_hs = p.o_hs = D;
    p.q_rs = p.o_rs = (long)p.Hq * D;
}

void attn_plan(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int kv_len, int cache_len, bool fused,
               int *slice, int *nsplit, int *heads_per_wg);
bool attention_fused_supported(int D, int G);
bool attention_fused_kv8_supported(int D, int cache_len);
size_t attn_scratch_bytes(int B, int Hq, int Sq, int D, int nsplit);
int attention_decode_launch(AttnParams p, int D, int dtype, int kv_int8, void *scratch, hipStream_t s);
int attention_prefill_launch(const AttnParams &p, int D, int dtype, hipStream_t s);
bool attention_prefill_supported(const AttnParams &p, int D, int dtype, int kv_int8);
// streaming decode kernel (attention_stream.hip): taken when eligible; attn_plan then returns its plan
bool attn_stream_eligible(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int kv_len, int cache_len);
void attn_stream_plan(int B, int Hkv, int kv_len, int *slice, int *nsplit);
int attn_stream_max_ranges(int B, int Hkv, int kv_len_max);  // most key ranges any length <= kv_len_max is planned with
void attn_stream_plan_paged(int B, int Hkv, int kv_len, int page_shift, int *slice, int *nsplit);
int attn_stream_max_ranges_paged(int B, int Hkv, int kv_len_max, int page_shift);
bool attn_stream_possible(int B, int Sq, int Hq, int Hkv, int D, int dtype, int cache_len);
// bytes of partial results that hold for EVERY call with this shape and an active length / cache length up to cache_len
size_t attn_max_scratch_bytes(int B, int Sq, int Hq, int Hkv, int D, int dtype, int kv_int8, int cache_len);
int attention_stream_launch(const AttnParams &p, int D, int dtype, int kv_int8, hipStream_t s);
// paged K/V: the streaming kernel takes every decode shape it has a form for, whatever the sizes
bool attn_stream_paged_supported(int Sq, int Hq, int Hkv, int D, int dtype, int page_rows);
// out = merge of the nsplit partial results in p.part_o / p.part_ml (its own launch)
int attention_merge_launch(const AttnParams &p, int D, int dtype, hipStream_t s);

}  // namespace mynn
