// Internal launchers shared between translation units (the C ABI wraps some of them; the decoder
// executor calls them directly).
#pragma once
#include "mynn_common.h"

namespace mynn {

// gemv.hip -- one activation row, T in == T out
template <typename T>
int gemv_norm(void *out, const void *x, const void *norm_w, float eps, const int8_t *wq, const void *scale,
              int N, int K, hipStream_t s);
template <typename T>
int gemv_residual(void *out, const void *act, const int8_t *wq, const void *scale, const void *residual,
                  int N, int K, hipStream_t s);
template <typename T>
int gemv_norm_swiglu(void *out, const void *x, const void *norm_w, float eps, const int8_t *wq,
                     const void *scale, int N, int K, hipStream_t s, uint64_t *fill = nullptr, int fill_words = 0);
int dequant_gemv_dispatch(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K,
                          int act_dtype, int out_dtype, hipStream_t s);

// gemm.hip -- matrix-core DequantMatMul, M >= 16, 16-bit types
// skinny.hip -- 16 <= M <= 64 rows against int8 weights streamed once (scale after the sum); `scratch` holds
// skinny_scratch_bytes(M, N, K) of f32 partial sums; epi is one of GEMM_* (SWIGLU: interleaved gate/up rows)
bool skinny_gemm_supported(int M, int N, int K);
size_t skinny_scratch_bytes(int M, int N, int K);
// `packed`: wq is a tiled copy (skinny_packed_bytes, made by skinny_pack_weight) that a wave reads sequentially
size_t skinny_packed_bytes(int N, int K);
int skinny_pack_weight(void *dst, const int8_t *wq, int N, int K, hipStream_t s);
// x[r, n] = T(x[r, n] + bias[n]) in place, x [rows, N] (elementwise.hip)
int add_bias_rows(void *x, const void *bias, int rows, int N, int dtype, hipStream_t s);
// paging: the caches are pools [n_pages, Hkv, 1 << shift, D]; row r of sequence b goes to pool page
// table[b * pages_per_seq + (r >> shift)] (a device array), row r % (1 << shift) of it.  table == nullptr: contiguous caches.
struct KvPaging {
    const int32_t *table = nullptr;
    int shift = 0, pages_per_seq = 0;
};
// row index (in rows of D elements) of cache row `r` of kv head `hk` of sequence `b`
__device__ inline size_t kv_cache_row(const KvPaging &pg, int b, int hk, int r, int Hkv, int max_seq) {
    if (!pg.table) return ((size_t)b * Hkv + hk) * max_seq + r;
    const int page = pg.table[(size_t)b * pg.pages_per_seq + (r >> pg.shift)];
    return (((size_t)page * Hkv + hk) << pg.shift) + (size_t)(r & ((1 << pg.shift) - 1));
}
// rope (optional, plain store of a q|k|v projection): instead of storing the projection, rotate q and k by the
// rows' positions and write q to q_out and k, v into the caches -- what rope_kv_append would do next
struct SkinnyRope {
    void *q_out, *k_cache, *v_cache;
    const void *cos_t, *sin_t;
    const int64_t *position;
    const int32_t *d_past;
    int S, Hq, Hkv, D, max_seq;
    KvPaging paging;
    void *k_scale = nullptr, *v_scale = nullptr;  // int8 caches: the per-row scale buffers (head_dim 64 or 128)
};
int dequant_gemm_skinny(void *out, const void *act, const int8_t *wq, bool packed, const void *scale, const void *res, int M,
                        int N, int K, int dtype, int epi, float *scratch, hipStream_t s, const void *norm_w = nullptr,
                        float eps = 0.f, void *nrm_out = nullptr, bool *normed = nullptr, const SkinnyRope *rope = nullptr,
                        bool *roped = nullptr);

// matrix-core GEMM pieces.  A dequantised weight is [N, Kp] of the 16-bit type, Kp = K rounded up to 64,
// zero padded (gemm_weight_bytes); dequant_weight_rows writes one (group/which: see gemm.hip), and
// gemm_nt_mfma multiplies by it: out = store(act . wt^T) with the store one of GEMM_*.
enum { GEMM_PLAIN = 0, GEMM_RESIDUAL = 1, GEMM_SWIGLU = 2 };
size_t gemm_weight_bytes(int N, int K);
int dequant_weight_rows(void *dst, const int8_t *wq, const void *scale, int N, int K, int dtype, int group, int which,
                        hipStream_t s);
// RMSNormalization -> DynamicQuantizeLinear (symmetric, per row) in one launch; scratch_norm ([rows, dim] of
// the storage type) is used only when the rows do not fit the vector kernel
int rms_norm_dynquant(int8_t *y, void *y_scale, void *scratch_norm, const void *x, const void *w, int rows, int dim, float eps,
                      int dtype, hipStream_t s);
// row interleave of the two halves of a fused gate/up operand (groups of `group` rows)
int interleave_row_groups(void *dst, const void *src, size_t rows, size_t row_bytes, int group, int which, hipStream_t s);
// QuantizedMatMul (int8 x int8 -> exact int32 -> two scales) with the large direct-to-LDS tiles of the
// matrix-core GEMM; res (optional) is added to the rounded result and rounded again
bool qgemm_dma_supported(int M, int N, int K);
int qgemm_dma(void *out, int32_t *acc_out, const int8_t *lhs, const void *lhs_scale, const int8_t *rhs, const void *rhs_scale,
              const void *res, int M, int N, int K, int dtype, int epi, hipStream_t s);
// tile: 0 heuristic; 1 = 256x128, 2 = 256x256 (register staged); 3 = 256x256, 4 = 256x320 (direct to LDS)
int gemm_nt_mfma(void *out, const void *act, const void *wt, const void *res, int M, int N, int K, int dtype, int epi,
                 hipStream_t s, int tile = 0);
// W_T = T(wq * scale) into `ws` (gemm_weight_bytes), then out = act . W_T^T
int dequant_gemm_mfma(void *out, const void *act, const int8_t *wq, const void *scale, int M, int N, int K, int dtype, void *ws,
                      int tile, hipStream_t s);

// elementwise.hip
// device-side loop state of a batch-1 decode model; a null `ids` means "no bookkeeping"
// q|k|v projection + decode attention in one launch (qkv_attention.hip), batch 1
struct QkvAttnParams {
    const void *x, *norm_w;  // the residual stream row [K] and the RMSNorm weights
    float eps;
    const int8_t *wq;        // [N, K] int8, rows of q, k, v
    const void *scale;       // [N]
    int N, K;
    uint64_t *qkv;           // hand-over vector of N 16-bit elements: all 0xFFFF ("empty") on entry
    int gemv_blocks, groups; // filled in by the launcher
    void *out;               // [Hq * D]
    void *k_cache, *v_cache; // [Hkv, max_seq, D]; paging.table set: page pools [n_pages, Hkv, page rows, D]
    void *k_scale, *v_scale; // int8 cache (BuildOptions::quant_kv_cache): [Hkv, max_seq] row scales; null: 16-bit cache
    KvPaging paging;         // paged cache: the sequence's page table (at most 64 pages)
    const void *cos_t, *sin_t;
    const int64_t *d_pos;
    const int32_t *d_active;
    const int32_t *d_past;   // the cache row the new token is appended to (KVCacheUpdate's offset)
    int Hq, Hkv, max_seq;
    float softmax_scale;
    int *err;                // set to 1 by a wait that ran out
    int spin_limit;
    // optional third stage, the o projection + residual: x2 = T(T(o_wq . attn * o_scale) + x).  The attention
    // output then travels through attn_words (Hq * D 16-bit elements, all 0xFFFF on entry) instead of `out`.
    const int8_t *o_wq;      // [K, Hq * D] int8 (null: the launch ends with the attention)
    const void *o_scale;     // [K]
    void *o_out;             // [K]
    uint64_t *attn_words;
    int o_blocks;            // filled in by the launcher
    // optional: the input row is not `x` but row *d_ids of the int8 embedding table times its scale, rounded to
    // the storage type (the first layer of a step; x is then not read)
    const int8_t *embed_w;   // [vocab, K]
    const void *embed_s;     // [vocab]
    const int64_t *d_ids;
    int vocab;
};
bool qkv_attention_supported(int H, int Hq, int Hkv, int D, int max_seq, int dtype);

// Batch-1 W8A8 linear in one launch (qgemv_fused.hip): (RMSNorm ->) per-row quantisation -> int8 x int8 GEMV ->
// plain / residual / SwiGLU store.  norm_w null: no normalisation; epi: GEMM_PLAIN / GEMM_RESIDUAL / GEMM_SWIGLU
bool qgemv_fused_supported(const void *act, const void *norm_w, const int8_t *wq, int N, int K);
int qgemv_fused(void *out, const void *act, const void *norm_w, float eps, const int8_t *wq, const void *scale, const void *residual,
                int N, int K, int dtype, int epi, hipStream_t s);
int qkv_attention_launch(QkvAttnParams p, int D, int dtype, hipStream_t s);

struct AdvanceState {
    int64_t *ids, *pos;
    int32_t *past, *active, *tokens, *step;
    int cap;
};

// gemv.hip -- the decode step's lm_head with the greedy token and the loop state in the same launch
bool gemv_norm_argmax_supported(const void *x, const void *norm_w, const int8_t *wq, int N, int K);
constexpr int kGemvArgmaxWords = 4096 / 4 + 1;  // candidate words a launch may use
template <typename T>
int gemv_norm_argmax(void *out, const void *x, const void *norm_w, float eps, const int8_t *wq, const void *scale, int N, int K,
                     uint64_t *cand, int32_t *next, AdvanceState adv, int *err, int spin_limit, hipStream_t s);

// out[r] = index of the LAST maximum of logits row r; when adv.ids != nullptr the launch also
// records the token and moves the decode loop on by one position
template <typename T>
int argmax_rows(int32_t *out, const void *logits, int rows, int n, AdvanceState adv, hipStream_t s);
template <typename T>
int embed_dequant(void *out, const int8_t *table, const void *scale, const int64_t *ids, int n_ids, int vocab,
                  int hidden, hipStream_t s);

// rope_kv.hip -- RoPE of q and k plus the KV-cache append, from the fused qkv projection output.
// qkv [B*S, (Hq+2*Hkv)*D] token-major; q_out [B*S, Hq*D]; caches [B,Hkv,max_seq,D];
// position[S] selects the table row; rows land at cache positions past+s where past is *d_past
// when d_past != nullptr, else past_host.
template <typename T>
int rope_kv_append(void *q_out, void *k_cache, void *v_cache, const void *qkv, const void *cos_t, const void *sin_t,
                   const int64_t *position, const int32_t *d_past, int past_host, int B, int S, int Hq, int Hkv, int D,
                   int max_seq, hipStream_t s, KvPaging paging = KvPaging());
// the same for an int8 KV cache: k (after RoPE, rounded to T) and v are quantised per token row into
// the caches and their scale rows [B,Hkv,max_seq] (QuantizingKVCacheUpdate, CPU backend rounding)
template <typename T>
int rope_quant_kv_append(void *q_out, int8_t *k_cache, int8_t *v_cache, void *k_scale, void *v_scale, const void *qkv,
                         const void *cos_t, const void *sin_t, const int64_t *position, const int32_t *d_past, int B,
                         int S, int Hq, int Hkv, int D, int max_seq, hipStream_t s, KvPaging paging = KvPaging());

}  // namespace mynn
