// Static Llama decoder executor behind the reference's per-session model ABI
// (model_init / model / model_destroy, src/codegen/cuda.rs:2727-2825).
//
// The reference generates one libmodel.so per graph whose model() launches ~30 kernels per layer
// over up to 16 streams, reading `past_len` / `active_seq_kv` on the host at launch time.  Here the
// op sequence of crates/llm/src/decoder.rs:222-391,780-865 is fixed code:
//   decode (seq_q == 1, int8 weights): 6 launches per layer, all scalars (token, position,
//     past_len, active length) live in device memory, the whole step is captured once into a
//     hipGraph and replayed; a decode loop can run many steps without a host round trip.
//   everything else (prefill rows, un-quantised checkpoints): op-by-op launches in the
//     reference's order, with the reference's kernel choice per op.
// One stream, one arena allocated at init; weights and KV buffers stay caller-owned.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "attention.h"
#include "kernels.h"
#include "kv_pages.h"

namespace mynn {

// ---- plain (un-quantised) linear: out[m,n] = T(sum_k act[m,k] * w[n,k]), one wave per element.
// Serves the reference's float checkpoints (its cuBLAS Gemm path); not a tuned kernel.
template <typename T>
__global__ __launch_bounds__(64) void dense_linear_kernel(T *out, const T *act, const T *w, int N, int K,
                                                         int out_stride) {
    const int n = blockIdx.x, m = blockIdx.y, lane = threadIdx.x;
    float acc = 0.f;
    for (int k = lane; k < K; k += 64) acc = fmaf(Elem<T>::ld(act, (size_t)m * K + k), Elem<T>::ld(w, (size_t)n * K + k), acc);
    acc = wave_sum(acc);
    if (lane == 0) Elem<T>::st(out, (size_t)m * out_stride + n, acc);
}

template <typename T>
__global__ void swiglu_rows_kernel(T *out, const T *gate, const T *up, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float g = Elem<T>::ld(gate, i);
    float sig = 1.0f / (1.0f + expf(-g));
    Elem<T>::st(out, i, (g * sig) * Elem<T>::ld(up, i));
}

// Streaming-KV graph (crates/llm/src/decoder.rs:281-347): q is rotated by the token's position, k and v leave
// un-rotated, all three in the operators' [heads, S, D] layout.  qkv [S, (Hq + 2 Hkv) D] token-major.
template <typename T>
__global__ __launch_bounds__(64) void stream_split_kernel(T *q_ref, T *k_new, T *v_new, const T *qkv, const T *cos_t, const T *sin_t,
                                                         const int64_t *position, int S, int Hq, int Hkv, int D) {
    const int s = blockIdx.x, head = blockIdx.y, half = D / 2;
    const T *src = qkv + ((size_t)s * (Hq + 2 * Hkv) + head) * D;
    if (head < Hq) {
        T *dst = q_ref + ((size_t)head * S + s) * D;
        const size_t tab = (size_t)position[s] * D;
        for (int j = threadIdx.x; j < half; j += blockDim.x) {
            const float xl = Elem<T>::ld(src, j), xh = Elem<T>::ld(src, j + half);
            Elem<T>::st(dst, j, xl * Elem<T>::ld(cos_t, tab + j) - xh * Elem<T>::ld(sin_t, tab + j));
            Elem<T>::st(dst, j + half, xh * Elem<T>::ld(cos_t, tab + j + half) + xl * Elem<T>::ld(sin_t, tab + j + half));
        }
        return;
    }
    const bool is_k = head < Hq + Hkv;
    T *dst = (is_k ? k_new : v_new) + ((size_t)(is_k ? head - Hq : head - Hq - Hkv) * S + s) * D;
    for (int j = threadIdx.x; j < D; j += blockDim.x) dst[j] = src[j];
}
// [H, S, D] -> [S, H * D]
template <typename T>
__global__ void heads_to_tokens_kernel(T *out, const T *in, int H, int S, int D) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)H * S * D) return;
    const int d = (int)(i % D), h = (int)((i / D) % H), s = (int)(i / ((size_t)D * H));
    out[i] = in[((size_t)h * S + s) * D + d];
}

struct Lin {
    const void *w = nullptr;      // int8 [N,K] when scale != nullptr, else T [N,K]
    const void *scale = nullptr;  // T [N]
    int N = 0, K = 0;
};

struct Layer {
    const void *norm1 = nullptr, *norm2 = nullptr;
    Lin qkv, o, gate, up, gu, down;  // qkv = rows of q,k,v concatenated; gu = gate/up rows interleaved
    void *k_cache = nullptr, *v_cache = nullptr;
    void *k_scale = nullptr, *v_scale = nullptr;  // int8 KV cache: per-token scales [B,Hkv,max_seq]
    // (everything below points into the model's WeightSet)
    void *qkv_b = nullptr;  // qkv_bias: the q, k, v projection biases concatenated [QD + 2 KD], T
    // prefill executors: weights dequantised once to the 16-bit type, [N, Kp] (wt_gu: gate/up in groups of 32)
    void *wt_qkv = nullptr, *wt_o = nullptr, *wt_gu = nullptr, *wt_down = nullptr;
    // few-row executors: int8 weights re-tiled so that a wave streams them sequentially
    void *pk_qkv = nullptr, *pk_o = nullptr, *pk_gu = nullptr, *pk_down = nullptr;
    // W8A8 prefill executors: int8 gate/up rows and their scales interleaved in groups of 32 (SwiGLU store)
    void *q8_gu = nullptr, *q8_gu_scale = nullptr;
};

// Every copy the library derives from a checkpoint's weights, made at most once and shared by the executors of a
// session (prefill, decode, few-row): the q|k|v and gate/up repacks, the 16-bit resident copy of the matrix-core path,
// the tiled int8 copy of the few-row path, the W8A8 gate/up interleave.  A copy is made by the first executor that
// needs it (under the set's mutex) and lives until the last holder -- the caller's handle or a model -- lets go.
struct WeightLayer {
    void *qkv_w = nullptr, *qkv_s = nullptr, *gu_w = nullptr, *gu_s = nullptr, *qkv_b = nullptr;
    void *wt_qkv = nullptr, *wt_o = nullptr, *wt_gu = nullptr, *wt_down = nullptr;
    void *pk_qkv = nullptr, *pk_o = nullptr, *pk_gu = nullptr, *pk_down = nullptr;
    void *q8_gu = nullptr, *q8_gu_scale = nullptr;
};
struct WeightSet {
    std::mutex mu;
    int refs = 1;
    // what the copies depend on: the shapes, the storage type, the caller's buffers
    int n_layers = 0, hidden = 0, n_heads = 0, n_kv_heads = 0, head_dim = 0, ffn = 0, vocab = 0, dtype = 0, int8_weights = 0, qkv_bias = 0;
    std::vector<void *> initializer;
    std::vector<WeightLayer> layers;
    void *wt_lm_head = nullptr, *pk_lm_head = nullptr;
    bool repacked = false, resident16 = false, packed8 = false, q8 = false;
    size_t bytes_repack = 0, bytes_resident16 = 0, bytes_packed8 = 0, bytes_q8 = 0;
};
static size_t initializer_count(const mynn_model_config &c) {
    return 2 + (size_t)c.n_layers * (2 + 14 + (c.qkv_bias ? 3 : 0)) + 1 + 2;
}
static WeightSet *weight_set_new(const mynn_model_config &c, void **init) {
    WeightSet *w = new WeightSet;
    w->n_layers = c.n_layers; w->hidden = c.hidden; w->n_heads = c.n_heads; w->n_kv_heads = c.n_kv_heads; w->head_dim = c.head_dim;
    w->ffn = c.ffn; w->vocab = c.vocab; w->dtype = c.dtype; w->int8_weights = c.weights_int8; w->qkv_bias = c.qkv_bias;
    w->initializer.assign(init, init + initializer_count(c));
    w->layers.resize(c.n_layers);
    return w;
}
static bool weight_set_fits(const WeightSet &w, const mynn_model_config &c) {
    return w.n_layers == c.n_layers && w.hidden == c.hidden && w.n_heads == c.n_heads && w.n_kv_heads == c.n_kv_heads &&
           w.head_dim == c.head_dim && w.ffn == c.ffn && w.vocab == c.vocab && w.dtype == c.dtype && w.int8_weights == c.weights_int8 &&
           w.qkv_bias == c.qkv_bias;
}
static void weight_set_release(WeightSet *w) {
    if (!w) return;
    {
        std::lock_guard<std::mutex> lk(w->mu);
        if (--w->refs > 0) return;
    }
    for (WeightLayer &L : w->layers)
        for (void *p : {L.qkv_w, L.qkv_s, L.gu_w, L.gu_s, L.qkv_b, L.wt_qkv, L.wt_o, L.wt_gu, L.wt_down, L.pk_qkv, L.pk_o, L.pk_gu, L.pk_down,
                        L.q8_gu, L.q8_gu_scale})
            if (p) (void)hipFree(p);
    if (w->wt_lm_head) (void)hipFree(w->wt_lm_head);
    if (w->pk_lm_head) (void)hipFree(w->pk_lm_head);
    delete w;
}

struct Launch {
    const char *name;
    double bytes;
    double flops;
};

struct Model {
    mynn_model_config cfg{};
    bool quant = true;
    Lin embed, lm_head;
    const void *final_norm = nullptr;
    std::vector<Layer> layers;
    void *wt_lm_head = nullptr, *pk_lm_head = nullptr;
    WeightSet *wset = nullptr;  // the derived weight copies (shared with the session's other executors)
    bool w8a8_fused = false;  // W8A8 with the large int8 tiles: norm+quantise, residual and SwiGLU ride on the launches
    bool qgemv1 = false;      // W8A8 at batch 1: norm, quantiser, int8 GEMV and residual / SwiGLU of a linear in one launch
    bool resident16 = false;  // the wt_* copies exist and the matrix-core path with fused stores is used
    bool skinny = false;      // 16..64 rows: int8 weights streamed once through the few-row matrix-core kernel
    float *skinny_scratch = nullptr;
    void *cos_t = nullptr, *sin_t = nullptr;
    // arena
    char *arena = nullptr;
    size_t arena_bytes = 0;
    void *x = nullptr, *x2 = nullptr, *nrm = nullptr, *qkv = nullptr, *q = nullptr, *attn = nullptr, *g = nullptr,
         *u = nullptr, *hmid = nullptr, *proj = nullptr, *logits = nullptr;
    int8_t *a8 = nullptr;    // W8A8: the current linear's activation rows as int8 [rows, max(H, QD, F)]
    void *a8_scale = nullptr;  // and their per-row scales [rows]
    int64_t *d_ids = nullptr, *d_pos = nullptr;
    int32_t *d_past = nullptr, *d_active = nullptr, *d_next = nullptr, *d_tokens = nullptr, *d_step = nullptr;
    void *attn_scratch = nullptr;
    int nsplit = 1, slice = 0, heads_per_wg = 1;
    int token_cap = 0;
    // host staging (pinned)
    char *h_stage = nullptr;
    size_t stage_bytes = 0, next_stage = 256;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    bool use_graph = false;
    int launches = 0;
    // batch-1 decode: projection and attention share a launch; m.qkv is then the hand-over vector between them
    // (all 0xFFFF between uses) and d_past[3] the error word of its bounded waits
    // the device-resident loop replays kLoopSteps steps per graph launch where it can (a graph launch costs the device a
    // few microseconds of its own, a tenth of a batch-1 step's launches)
    hipGraph_t graph_loop = nullptr;
    hipGraphExec_t graph_loop_exec = nullptr;
    bool qkv_attn = false;
    bool lm_argmax = false;       // ... and the lm_head launch finds the greedy token and moves the loop state on
    uint64_t *lm_cand = nullptr;  // its candidate words (all ~0 between launches)
    int spin_limit = 400000;      // polls a consumer role makes before it gives up and raises the error word
    int handover_failures = 0;    // steps whose hand-over gave up; the executor then rebuilt itself with one op per launch
    // what build() had chosen before a give-up switched the shared launches off, and when they are tried again: after
    // rearm_after clean steps (doubled by every further give-up; 0 = never)
    bool shared_qkv_attn = false, shared_lm_argmax = false, fell_back = false;
    int rearm_after = 256;
    long clean_steps = 0;
    // streaming_kv: the ring inputs of the step in flight (host copies: the operators take them at launch time, as the
    // reference's kernels do), kv_position on the device, and the operators' [heads, S, D] tensors
    int ring_sink = 0, ring_window = 0, ring_start = 0, h_past = 0, h_active = 0;
    int64_t *d_kvpos = nullptr;
    void *q_ref = nullptr, *k_new = nullptr, *v_new = nullptr, *attn_ref = nullptr, *k_rot = nullptr;
    void *ring_ws = nullptr;      // ... and the scratch memory of the ring attention (rank-ordered rows, partial results)
    size_t ring_ws_bytes = 0;
    int last_status = 0;          // of the last model() call on this state
    void *warena = nullptr;       // weight_arena: every linear weight and scale of the model in one allocation, in execution order
    mynn_kv_pages *pages = nullptr;  // kv_page_rows: the session's page table (the caller's); k_cache / v_cache then are pools
    KvPaging paging;
    void *ws = nullptr;           // executors that dequantise a weight per call (M >= 16, no resident copy): their own workspace
    // per-launch record of the last enqueue (names + algorithmic bytes), events when profiling
    std::vector<Launch> record;
    bool profiling = false;
    std::vector<hipEvent_t> events;
};

static mynn_model_config g_cfg{};
static bool g_cfg_set = false;
static std::mutex g_mu;

static size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct ArenaPlan {
    size_t off = 0;
    size_t take(size_t bytes) {
        size_t o = off;
        off = align_up(off + bytes, 256);
        return o;
    }
};

static void note(Model &m, const char *name, double bytes, double flops = 0.0) {
    if (m.profiling) {
        // the launch that follows stamps these two with its own start and end
        hipEvent_t a, b;
        hipEventCreate(&a);
        hipEventCreate(&b);
        m.events.push_back(a);
        m.events.push_back(b);
        launch_timer() = LaunchTimer{a, b};
    }
    m.record.push_back({name, bytes, flops});
}

#define TRY(expr)            \
    do {                     \
        int rc__ = (expr);   \
        if (rc__) return rc__; \
    } while (0)

// one matrix-core GEMM against a resident dequantised weight
static int gemm_rows(Model &m, void *out, const void *act, const void *wt, const void *res, int M, int N, int K, int epi,
                     const char *name) {
    const double eb = 2.0, n_out = epi == GEMM_SWIGLU ? N / 2 : N;
    note(m, name, ((double)N * K + (double)M * K + (double)M * n_out * (epi == GEMM_RESIDUAL ? 2 : 1)) * eb, 2.0 * M * N * K);
    return gemm_nt_mfma(out, act, wt, res, M, N, K, m.cfg.dtype, epi, m.stream, m.cfg.gemm_tile);
}

template <typename T>
static int linear_rows(Model &m, void *out, const void *act, const Lin &l, int M, const char *name) {
    const double eb = sizeof(T);
    if (l.scale) {
        if (M >= 16 && l.K % 8 == 0) {
            // W_T = T(wq * scale) into the workspace, then the matrix-core product (two launches, two records)
            MYNN_REQUIRE(m.ws, MYNN_ERR_STATE, "decoder: no weight workspace for %s", name);
            note(m, "dequant_weight", (double)l.N * l.K * (1 + eb) + l.N * eb);
            TRY(dequant_weight_rows(m.ws, (const int8_t *)l.w, l.scale, l.N, l.K, m.cfg.dtype, 0, 0, m.stream));
            note(m, name, ((double)l.N * l.K + (double)M * l.K + (double)M * l.N) * eb, 2.0 * M * l.N * l.K);
            return gemm_nt_mfma(out, act, m.ws, nullptr, M, l.N, l.K, m.cfg.dtype, GEMM_PLAIN, m.stream, m.cfg.gemm_tile);
        }
        note(m, name, (double)l.N * l.K + l.N * eb + (double)M * l.K * eb + (double)M * l.N * eb, 2.0 * M * l.N * l.K);
        return dequant_gemv_dispatch(out, act, (const int8_t *)l.w, l.scale, M, l.N, l.K, m.cfg.dtype, m.cfg.dtype,
                                     m.stream);
    }
    note(m, name, ((double)l.N * l.K + (double)M * l.K + (double)M * l.N) * eb, 2.0 * M * l.N * l.K);
    MYNN_LAUNCH(dense_linear_kernel<T>, dim3(l.N, M), dim3(64), 0, m.stream, (T *)out, (const T *)act,
                       (const T *)l.w, l.N, l.K, l.N);
    return launch_status("dense_linear_kernel");
}

// one few-row GEMM against int8 weights (two launches: products, then sum/scale/store)
// next_norm (residual store): the weights of the RMSNorm that reads this output next; *normed = m.nrm holds it
static int skinny_rows(Model &m, void *out, const void *act, const Lin &l, const void *packed, const void *res, int M, int epi,
                       const char *name, const void *next_norm = nullptr, bool *normed = nullptr, const SkinnyRope *rope = nullptr,
                       bool *roped = nullptr) {
    const double eb = dtype_size(m.cfg.dtype), n_out = epi == GEMM_SWIGLU ? l.N / 2 : l.N;
    note(m, name, (double)l.N * l.K + l.N * eb + (double)M * l.K * eb + (double)M * n_out * eb * (epi == GEMM_RESIDUAL ? 2 : 1),
         2.0 * M * l.N * l.K);
    return dequant_gemm_skinny(out, act, (const int8_t *)(packed ? packed : l.w), packed != nullptr, l.scale, res, M, l.N, l.K,
                               m.cfg.dtype, epi, m.skinny_scratch, m.stream, next_norm, m.cfg.eps, m.nrm, normed, rope, roped);
}

// Options::quantize_activations: DynamicQuantizeLinear (per row, symmetric) then QuantizedMatMul.
// `fresh` = the activation changed since the last call (q/k/v and gate/up share one quantisation,
// as the pass caches it per value: quantize_activations.rs:121-130).
static int linear_w8a8(Model &m, void *out, const void *act, const Lin &l, int M, bool fresh, const char *name) {
    const double eb = dtype_size(m.cfg.dtype);
    if (fresh) {
        note(m, "dynamic_quantize", (double)M * l.K * (eb + 1) + M * eb);
        TRY(mynn_dynamic_quantize_linear(m.a8, m.a8_scale, nullptr, act, M, l.K, m.cfg.dtype, 1, m.stream));
    }
    note(m, name, (double)l.N * l.K + (double)M * l.K + l.N * eb + (double)M * l.N * eb, 2.0 * M * l.N * l.K);
    return mynn_quantized_matmul(out, nullptr, m.a8, m.a8_scale, (const int8_t *)l.w, l.scale, M, l.N, l.K, m.cfg.dtype,
                                 m.stream);
}

// W8A8 with the large int8 tiles: (RMSNorm +) per-row quantisation of the input, then the product with the
// store that the layer needs (plain, + residual, SwiGLU over interleaved gate/up rows)
static int qlinear_fused(Model &m, void *out, const void *act, const void *norm_w, const void *w, const void *scale, const void *res,
                         int M, int N, int K, int epi, const char *name) {
    const double eb = dtype_size(m.cfg.dtype);
    if (norm_w) {
        note(m, "rms_norm_quantize", (double)M * K * (eb + 1) + M * eb + K * eb);
        TRY(rms_norm_dynquant(m.a8, m.a8_scale, m.nrm, act, norm_w, M, K, m.cfg.eps, m.cfg.dtype, m.stream));
    } else {
        note(m, "dynamic_quantize", (double)M * K * (eb + 1) + M * eb);
        TRY(mynn_dynamic_quantize_linear(m.a8, m.a8_scale, nullptr, act, M, K, m.cfg.dtype, 1, m.stream));
    }
    const int n_out = epi == GEMM_SWIGLU ? N / 2 : N;
    note(m, name, (double)N * K + (double)M * K + N * eb + (double)M * n_out * eb * (res ? 2 : 1), 2.0 * M * N * K);
    return qgemm_dma(out, nullptr, m.a8, m.a8_scale, (const int8_t *)w, scale, res, M, N, K, m.cfg.dtype, epi, m.stream);
}

// The attention block of the streaming-KV graph, op for op (decoder.rs:281-347, 472-487): RoPE(q); k and v un-rotated
// into the caches through the sink + ring slot map; 16-bit KV: Rope over the whole K cache by kv_position, then
// Attention with the ring inputs; int8 KV: Attention rotates the dequantised keys itself (slots 10-12).
template <typename T>
static int streaming_attention(Model &m, Layer &L, float softmax_scale) {
    const mynn_model_config &c = m.cfg;
    const int S = c.seq_q, Hq = c.n_heads, Hkv = c.n_kv_heads, D = c.head_dim;
    const double eb = sizeof(T);
    hipStream_t s = m.stream;
    note(m, "streaming_rope_q_split", (double)S * (Hq + 2 * Hkv) * D * 2 * eb);
    MYNN_LAUNCH(stream_split_kernel<T>, dim3(S, Hq + 2 * Hkv), dim3(64), 0, s, (T *)m.q_ref, (T *)m.k_new, (T *)m.v_new,
                (const T *)m.qkv, (const T *)m.cos_t, (const T *)m.sin_t, m.d_pos, S, Hq, Hkv, D);
    TRY(launch_status("stream_split_kernel"));
    void *attn_out = S == 1 ? m.attn : m.attn_ref;  // (one row: [heads, 1, D] is the token-major row)
    if (c.quant_kv_cache) {
        note(m, "quantizing_kvcache_update_streaming", (double)S * 2 * Hkv * D * (eb + 1));
        TRY(mynn_quantizing_kvcache_update_streaming((int8_t *)L.k_cache, L.k_scale, m.k_new, m.h_past, Hkv, S, c.max_seq, D,
                                                     m.ring_sink, m.ring_window, m.ring_start, c.dtype, s));
        TRY(mynn_quantizing_kvcache_update_streaming((int8_t *)L.v_cache, L.v_scale, m.v_new, m.h_past, Hkv, S, c.max_seq, D,
                                                     m.ring_sink, m.ring_window, m.ring_start, c.dtype, s));
        note(m, "attention_streaming_rope", (double)S * 2.0 * Hq * D * eb);
        TRY(mynn_attention_streaming_ws(attn_out, m.q_ref, L.k_cache, L.v_cache, L.k_scale, L.v_scale, softmax_scale, S > 1, 1, S,
                                        m.h_active, c.max_seq, m.h_active - S, Hq, Hkv, D, c.dtype, 1, m.ring_sink, m.ring_window,
                                        m.ring_start, m.cos_t, m.sin_t, m.d_kvpos, m.ring_ws, m.ring_ws_bytes, s));
    } else {
        note(m, "kvcache_update_streaming", (double)S * 4 * Hkv * D * eb);
        TRY(mynn_kvcache_update_streaming(L.k_cache, m.k_new, m.h_past, Hkv, S, c.max_seq, D, m.ring_sink, m.ring_window,
                                          m.ring_start, c.dtype, s));
        TRY(mynn_kvcache_update_streaming(L.v_cache, m.v_new, m.h_past, Hkv, S, c.max_seq, D, m.ring_sink, m.ring_window,
                                          m.ring_start, c.dtype, s));
        note(m, "rope_k_cache", 2.0 * Hkv * c.max_seq * D * eb);
        TRY(mynn_rope(m.k_rot, L.k_cache, m.cos_t, m.sin_t, m.d_kvpos, Hkv, c.max_seq, D, c.dtype, s));
        note(m, "attention_streaming", (double)S * 2.0 * Hq * D * eb);
        TRY(mynn_attention_streaming_ws(attn_out, m.q_ref, m.k_rot, L.v_cache, nullptr, nullptr, softmax_scale, S > 1, 1, S,
                                        m.h_active, c.max_seq, m.h_active - S, Hq, Hkv, D, c.dtype, 0, m.ring_sink, m.ring_window,
                                        m.ring_start, nullptr, nullptr, nullptr, m.ring_ws, m.ring_ws_bytes, s));
    }
    if (S > 1) {
        const size_t n = (size_t)Hq * S * D;
        note(m, "heads_to_tokens", 2.0 * n * eb);
        MYNN_LAUNCH(heads_to_tokens_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (T *)m.attn, (const T *)m.attn_ref,
                    Hq, S, D);
        TRY(launch_status("heads_to_tokens_kernel"));
    }
    return 0;
}

template <typename T>
static int enqueue_step(Model &m) {
    const mynn_model_config &c = m.cfg;
    const int S = c.seq_q, B = c.batch, rows = B * S;
    const int H = c.hidden, Hq = c.n_heads, Hkv = c.n_kv_heads, D = c.head_dim, F = c.ffn, V = c.vocab;
    const int QD = Hq * D, KD = Hkv * D;
    const double eb = sizeof(T);
    const bool w8a8 = c.quantize_activations != 0, kv8 = c.quant_kv_cache != 0;
    const bool streaming = c.streaming_kv != 0;
    // batch-1 decode over int8 weights: the GEMVs carry RMSNorm, residual add and SwiGLU (also with an int8 KV cache, whose
    // attention block then runs as RoPE + quantising append and the int8-KV attention kernel)
    const bool fused = m.quant && rows == 1 && !w8a8 && !streaming;
    // batch-1 decode with quantize_activations: norm + quantiser + int8 GEMV + residual / SwiGLU of a linear in one launch
    const bool qfused = m.qgemv1 && rows == 1;
    auto qlinear1 = [&](void *out, const void *act, const void *norm_w, const Lin &l, const void *res, int epi, const char *name) {
        const int n_out = epi == GEMM_SWIGLU ? l.N / 2 : l.N;
        note(m, name, (double)l.N * l.K + l.K * eb + l.N * eb + (double)n_out * eb * (res ? 2 : 1) + (norm_w ? l.K * eb : 0.0), 2.0 * l.N * l.K);
        return qgemv_fused(out, act, norm_w, c.eps, (const int8_t *)l.w, l.scale, res, l.N, l.K, c.dtype, epi, m.stream);
    };
    hipStream_t s = m.stream;
    m.record.clear();
    for (hipEvent_t e : m.events) hipEventDestroy(e);
    m.events.clear();

    // embed: DequantizeLinear(table) -> Gather(ids), one row per token
    // (batch-1 decode with the fused launch: the first layer's launch makes the row itself)
    if (m.quant && rows == 1 && m.qkv_attn && !w8a8) {
    } else if (m.quant) {
        note(m, "embed_dequant", (double)rows * (H + eb + H * eb));
        TRY(embed_dequant<T>(m.x, (const int8_t *)m.embed.w, m.embed.scale, m.d_ids, rows, V, H, s));
    } else {
        note(m, "embed_gather", (double)rows * 2 * H * eb);
        TRY(mynn_gather_rows(m.x, m.embed.w, m.d_ids, rows, V, (size_t)H * sizeof(T), s));
    }
    const float softmax_scale = 1.0f / sqrtf((float)D);
    bool nrm_ready = false;  // m.nrm already holds the next RMSNorm's output (written by the launch that finished its input)
    for (size_t li = 0; li < m.layers.size(); li++) {
        Layer &L = m.layers[li];
        // ---- attention block
        bool roped = false;
        if (fused && m.qkv_attn) {
            // RMSNorm + q|k|v projection, RoPE, both cache appends and the attention in one launch
            note(m, li == 0 ? "embed_qkv_attention_o" : "qkv_attention_o", (double)L.qkv.N * H + L.qkv.N * eb + 2 * H * eb + 2.0 * KD * eb + (double)H * QD + H * eb + 2 * H * eb);
            QkvAttnParams p{};
            p.x = m.x; p.norm_w = L.norm1; p.eps = c.eps; p.wq = (const int8_t *)L.qkv.w; p.scale = L.qkv.scale;
            p.N = L.qkv.N; p.K = H; p.qkv = (uint64_t *)m.qkv; p.out = m.attn; p.k_cache = L.k_cache; p.v_cache = L.v_cache;
            p.k_scale = kv8 ? L.k_scale : nullptr; p.v_scale = kv8 ? L.v_scale : nullptr;
            p.cos_t = m.cos_t; p.sin_t = m.sin_t; p.d_pos = m.d_pos; p.d_active = m.d_active; p.d_past = m.d_past; p.Hq = Hq; p.Hkv = Hkv;
            p.max_seq = c.max_seq; p.softmax_scale = softmax_scale; p.err = m.d_past + 3; p.spin_limit = m.spin_limit;
            p.paging = m.paging;
            if (li == 0) {  // the input row of the first layer: the token's embedding
                p.embed_w = (const int8_t *)m.embed.w; p.embed_s = m.embed.scale; p.d_ids = m.d_ids; p.vocab = V;
            }
            // ... and the o projection + residual behind it: x2 = T(T(Wo . attn) + x)
            p.o_wq = (const int8_t *)L.o.w; p.o_scale = L.o.scale; p.o_out = m.x2; p.attn_words = (uint64_t *)m.attn;
            TRY(qkv_attention_launch(p, D, c.dtype, s));
        } else if (fused) {
            note(m, "gemv_norm_qkv", (double)L.qkv.N * H + L.qkv.N * eb + 2 * H * eb + L.qkv.N * eb);
            TRY(gemv_norm<T>(m.qkv, m.x, L.norm1, c.eps, (const int8_t *)L.qkv.w, L.qkv.scale, L.qkv.N, H, s));
        } else if (qfused) {
            TRY(qlinear1(m.qkv, m.x, L.norm1, L.qkv, nullptr, GEMM_PLAIN, "qgemv_norm_quant_qkv"));
        } else if (m.w8a8_fused) {
            TRY(qlinear_fused(m, m.qkv, m.x, L.norm1, L.qkv.w, L.qkv.scale, nullptr, rows, L.qkv.N, H, GEMM_PLAIN, "qlinear_qkv"));
        } else {
            if (!nrm_ready) {
                note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
                TRY(mynn_rms_norm(m.nrm, m.x, L.norm1, rows, H, c.eps, c.dtype, s));
            }
            nrm_ready = false;
            if (m.skinny) {
                // RoPE and both cache appends (an int8 cache: with its quantiser) ride on the launch that sums the projection's K ranges
                const SkinnyRope rp{m.q, L.k_cache, L.v_cache, m.cos_t, m.sin_t, m.d_pos, m.d_past, S, Hq, Hkv, D, c.max_seq, m.paging,
                                    kv8 ? L.k_scale : nullptr, kv8 ? L.v_scale : nullptr};
                TRY(skinny_rows(m, m.qkv, m.nrm, L.qkv, L.pk_qkv, nullptr, rows, GEMM_PLAIN, "linear_qkv", nullptr, nullptr,
                                (kv8 && D != 64 && D != 128) || streaming || L.qkv_b || c.unfused_decode ? nullptr : &rp, &roped));
            }
            else if (w8a8) TRY(linear_w8a8(m, m.qkv, m.nrm, L.qkv, rows, true, "qlinear_qkv"));
            else if (m.resident16) TRY(gemm_rows(m, m.qkv, m.nrm, L.wt_qkv, nullptr, rows, L.qkv.N, H, GEMM_PLAIN, "linear_qkv"));
            else TRY(linear_rows<T>(m, m.qkv, m.nrm, L.qkv, rows, "linear_qkv"));
        }
        if (L.qkv_b) {
            // the `{node}_bias` Add behind each projection (decoder.rs:167-184): the stored projection plus the bias, rounded again
            note(m, "add_qkv_bias", (double)rows * 2 * L.qkv.N * eb + (double)L.qkv.N * eb);
            TRY(add_bias_rows(m.qkv, L.qkv_b, rows, L.qkv.N, c.dtype, s));
        }
        if (streaming) {
            TRY(streaming_attention<T>(m, L, softmax_scale));
        } else if (!(fused && m.qkv_attn)) {
            AttnParams p{};
            p.out = m.attn; p.q = m.q; p.k = L.k_cache; p.v = L.v_cache; p.scale = softmax_scale;
            p.k_scale = L.k_scale; p.v_scale = L.v_scale;
            p.is_causal = S > 1; p.B = B; p.Sq = S; p.Hq = Hq; p.Hkv = Hkv; p.cache_len = c.max_seq;
            p.d_active = m.d_active; p.nsplit = m.nsplit; p.slice = m.slice; p.heads_per_wg = m.heads_per_wg;
            attn_token_major_layout(p, D);
            p.page_table = m.paging.table; p.page_shift = m.paging.shift; p.pages_per_seq = m.paging.pages_per_seq;
            // (an int8 cache: the form for a cache one workgroup covers quantises the new row itself)
            const bool fuse_attn = (fused || qfused) && !m.pages &&
                                   (kv8 ? attention_fused_kv8_supported(D, c.max_seq) : attention_fused_supported(D, Hq / Hkv));
            if (fuse_attn) {
                // RoPE(q), RoPE(k), both cache appends and the attention in one launch
                p.qkv = m.qkv; p.cos_t = m.cos_t; p.sin_t = m.sin_t; p.d_pos = m.d_pos; p.d_past = m.d_past;
                note(m, kv8 ? "attention_rope_quant_append" : "attention_rope_append", (double)(QD + 2 * KD) * eb + 2.0 * KD * (kv8 ? 1 + eb / D : eb) + QD * eb);
                TRY(attention_decode_launch(p, D, c.dtype, kv8 ? 1 : 0, m.attn_scratch, s));
            } else {
                // prefill on the matrix cores: the attention kernel rotates the queries itself, reading them from the
                // projection's output; the RoPE launch is left with the keys and the values
                // (a paged cache: that kernel for every prefill shape -- the per-row kernel has no paged form)
                const bool pf_kernel = S > 1 && (attention_prefill_supported(p, D, c.dtype, kv8) || m.pages);
                const bool pf = pf_kernel && !kv8 && !roped;
                const bool q_in_attn = pf && ((size_t)(QD + 2 * KD) * sizeof(T)) % 16 == 0 && aligned16(m.qkv);
                if (!roped) note(m, kv8 ? "rope_quant_kv_append" : q_in_attn ? "rope_kv_append_k_v" : "rope_kv_append",
                                 q_in_attn ? (double)rows * 2 * KD * 2 * eb : (double)rows * (QD + 2 * KD) * 2 * eb);
                if (roped) {
                } else if (kv8)
                    TRY(rope_quant_kv_append<T>(m.q, (int8_t *)L.k_cache, (int8_t *)L.v_cache, L.k_scale, L.v_scale, m.qkv,
                                                m.cos_t, m.sin_t, m.d_pos, m.d_past, B, S, Hq, Hkv, D, c.max_seq, s, m.paging));
                else
                    TRY(rope_kv_append<T>(q_in_attn ? nullptr : m.q, L.k_cache, L.v_cache, m.qkv, m.cos_t, m.sin_t, m.d_pos, m.d_past, 0, B, S,
                                          Hq, Hkv, D, c.max_seq, s, m.paging));
                if (q_in_attn) {
                    p.q = m.qkv; p.rope_q = 1; p.cos_t = m.cos_t; p.sin_t = m.sin_t; p.d_pos = m.d_pos;
                    p.q_bs = (long)S * (QD + 2 * KD); p.q_hs = D; p.q_rs = QD + 2 * KD;
                }
                // bytes: q in, out; the K/V rows read depend on the context, which the host does not
                // know under replay -- callers add 2*KD*eb per cached row when they report
                // flops: the causal half of QK^T and PV over the new rows alone (exact when past_len is 0)
                note(m, "attention", (double)rows * 2.0 * QD * eb, S > 1 ? 2.0 * B * Hq * D * (double)S * (S + 1) : 0.0);
                if (pf_kernel) TRY(attention_prefill_launch(p, D, c.dtype, s));
                else TRY(attention_decode_launch(p, D, c.dtype, kv8, m.attn_scratch, s));
            }
        }
        if (fused) {
            if (!m.qkv_attn) {
                note(m, "gemv_o_residual", (double)H * QD + H * eb + QD * eb + 2 * H * eb);
                TRY(gemv_residual<T>(m.x2, m.attn, (const int8_t *)L.o.w, L.o.scale, m.x, H, QD, s));
            }
            note(m, "gemv_norm_gateup_swiglu", (double)L.gu.N * H + L.gu.N * eb + 2 * H * eb + F * eb);
            // (after a fused launch the gate/up launch also empties its two hand-over vectors, m.qkv .. m.attn,
            // before their next use)
            uint64_t *fill = m.qkv_attn ? (uint64_t *)m.qkv : nullptr;
            const int fill_words = m.qkv_attn ? (int)(((char *)m.attn + (size_t)QD * sizeof(T) - (char *)m.qkv) / 8) : 0;
            TRY(gemv_norm_swiglu<T>(m.hmid, m.x2, L.norm2, c.eps, (const int8_t *)L.gu.w, L.gu.scale, L.gu.N, H, s, fill, fill_words));
            note(m, "gemv_down_residual", (double)H * F + H * eb + F * eb + 2 * H * eb);
            TRY(gemv_residual<T>(m.x, m.hmid, (const int8_t *)L.down.w, L.down.scale, m.x2, H, F, s));
        } else if (m.skinny) {
            bool normed = false;
            TRY(skinny_rows(m, m.x2, m.attn, L.o, L.pk_o, m.x, rows, GEMM_RESIDUAL, "linear_o_residual", L.norm2, &normed));
            if (!normed) {
                note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
                TRY(mynn_rms_norm(m.nrm, m.x2, L.norm2, rows, H, c.eps, c.dtype, s));
            }
            TRY(skinny_rows(m, m.hmid, m.nrm, L.gu, L.pk_gu, nullptr, rows, GEMM_SWIGLU, "linear_gateup_swiglu"));
            const void *next_norm = li + 1 < m.layers.size() ? m.layers[li + 1].norm1 : m.final_norm;
            TRY(skinny_rows(m, m.x, m.hmid, L.down, L.pk_down, m.x2, rows, GEMM_RESIDUAL, "linear_down_residual", next_norm, &nrm_ready));
        } else if (qfused) {
            TRY(qlinear1(m.x2, m.attn, nullptr, L.o, m.x, GEMM_RESIDUAL, "qgemv_quant_o_residual"));
            TRY(qlinear1(m.hmid, m.x2, L.norm2, L.gu, nullptr, GEMM_SWIGLU, "qgemv_norm_quant_gateup_swiglu"));
            TRY(qlinear1(m.x, m.hmid, nullptr, L.down, m.x2, GEMM_RESIDUAL, "qgemv_quant_down_residual"));
        } else if (m.w8a8_fused) {
            TRY(qlinear_fused(m, m.x2, m.attn, nullptr, L.o.w, L.o.scale, m.x, rows, H, QD, GEMM_RESIDUAL, "qlinear_o_residual"));
            TRY(qlinear_fused(m, m.hmid, m.x2, L.norm2, L.q8_gu, L.q8_gu_scale, nullptr, rows, 2 * F, H, GEMM_SWIGLU, "qlinear_gateup_swiglu"));
            TRY(qlinear_fused(m, m.x, m.hmid, nullptr, L.down.w, L.down.scale, m.x2, rows, H, F, GEMM_RESIDUAL, "qlinear_down_residual"));
        } else if (w8a8) {
            TRY(linear_w8a8(m, m.proj, m.attn, L.o, rows, true, "qlinear_o"));
            note(m, "add", 3.0 * rows * H * eb);
            TRY(mynn_add(m.x2, m.x, m.proj, (size_t)rows * H, c.dtype, s));
            note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
            TRY(mynn_rms_norm(m.nrm, m.x2, L.norm2, rows, H, c.eps, c.dtype, s));
            TRY(linear_w8a8(m, m.g, m.nrm, L.gate, rows, true, "qlinear_gate"));
            TRY(linear_w8a8(m, m.u, m.nrm, L.up, rows, false, "qlinear_up"));
            note(m, "swiglu", 3.0 * rows * F * eb);
            TRY(mynn_swiglu(m.hmid, m.g, m.u, (size_t)rows * F, c.dtype, s));
            TRY(linear_w8a8(m, m.proj, m.hmid, L.down, rows, true, "qlinear_down"));
            note(m, "add", 3.0 * rows * H * eb);
            TRY(mynn_add(m.x, m.x2, m.proj, (size_t)rows * H, c.dtype, s));
        } else if (m.resident16) {
            // residual adds and SwiGLU ride on the GEMM stores
            TRY(gemm_rows(m, m.x2, m.attn, L.wt_o, m.x, rows, H, QD, GEMM_RESIDUAL, "linear_o_residual"));
            note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
            TRY(mynn_rms_norm(m.nrm, m.x2, L.norm2, rows, H, c.eps, c.dtype, s));
            TRY(gemm_rows(m, m.hmid, m.nrm, L.wt_gu, nullptr, rows, 2 * F, H, GEMM_SWIGLU, "linear_gateup_swiglu"));
            TRY(gemm_rows(m, m.x, m.hmid, L.wt_down, m.x2, rows, H, F, GEMM_RESIDUAL, "linear_down_residual"));
        } else {
            TRY(linear_rows<T>(m, m.proj, m.attn, L.o, rows, "linear_o"));
            note(m, "add", 3.0 * rows * H * eb);
            TRY(mynn_add(m.x2, m.x, m.proj, (size_t)rows * H, c.dtype, s));
            note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
            TRY(mynn_rms_norm(m.nrm, m.x2, L.norm2, rows, H, c.eps, c.dtype, s));
            TRY(linear_rows<T>(m, m.g, m.nrm, L.gate, rows, "linear_gate"));
            TRY(linear_rows<T>(m, m.u, m.nrm, L.up, rows, "linear_up"));
            note(m, "swiglu", 3.0 * rows * F * eb);
            TRY(mynn_swiglu(m.hmid, m.g, m.u, (size_t)rows * F, c.dtype, s));
            TRY(linear_rows<T>(m, m.proj, m.hmid, L.down, rows, "linear_down"));
            note(m, "add", 3.0 * rows * H * eb);
            TRY(mynn_add(m.x, m.x2, m.proj, (size_t)rows * H, c.dtype, s));
        }
    }
    if (fused && m.lm_argmax) {
        note(m, "gemv_norm_lm_head_argmax", (double)V * H + V * eb + 2 * H * eb + V * eb);
        TRY(gemv_norm_argmax<T>(m.logits, m.x, m.final_norm, c.eps, (const int8_t *)m.lm_head.w, m.lm_head.scale, V, H, m.lm_cand,
                                m.d_next, AdvanceState{m.d_ids, m.d_pos, m.d_past, m.d_active, m.d_tokens, m.d_step, m.token_cap},
                                m.d_past + 3, m.spin_limit, s));
        launch_timer() = LaunchTimer{};
        m.launches = (int)m.record.size();
        return 0;
    } else if (fused) {
        note(m, "gemv_norm_lm_head", (double)V * H + V * eb + 2 * H * eb + V * eb);
        TRY(gemv_norm<T>(m.logits, m.x, m.final_norm, c.eps, (const int8_t *)m.lm_head.w, m.lm_head.scale, V, H, s));
    } else if (qfused) {
        TRY(qlinear1(m.logits, m.x, m.final_norm, m.lm_head, nullptr, GEMM_PLAIN, "qgemv_norm_quant_lm_head"));
    } else if (m.w8a8_fused) {
        TRY(qlinear_fused(m, m.logits, m.x, m.final_norm, m.lm_head.w, m.lm_head.scale, nullptr, rows, V, H, GEMM_PLAIN, "qlinear_lm_head"));
    } else {
        if (!nrm_ready) {
            note(m, "rms_norm", 2.0 * rows * H * eb + H * eb);
            TRY(mynn_rms_norm(m.nrm, m.x, m.final_norm, rows, H, c.eps, c.dtype, s));
        }
        if (m.skinny) TRY(skinny_rows(m, m.logits, m.nrm, m.lm_head, m.pk_lm_head, nullptr, rows, GEMM_PLAIN, "linear_lm_head"));
        else if (w8a8) TRY(linear_w8a8(m, m.logits, m.nrm, m.lm_head, rows, true, "qlinear_lm_head"));
        else if (m.resident16) TRY(gemm_rows(m, m.logits, m.nrm, m.wt_lm_head, nullptr, rows, V, H, GEMM_PLAIN, "linear_lm_head"));
        else TRY(linear_rows<T>(m, m.logits, m.nrm, m.lm_head, rows, "linear_lm_head"));
    }
    // greedy token of the last row of each sequence; for a batch-1 decode step the same launch
    // moves the device-side loop state on (token -> next input, position / past / active + 1)
    note(m, rows == 1 ? "argmax_advance" : "argmax_last", (double)B * V * eb);
    if (S == 1) {
        // the last (only) rows of all sequences are contiguous: one launch, one workgroup per sequence
        AdvanceState adv{};
        if (rows == 1) adv = AdvanceState{m.d_ids, m.d_pos, m.d_past, m.d_active, m.d_tokens, m.d_step, m.token_cap};
        TRY(argmax_rows<T>(m.d_next, m.logits, B, V, adv, s));
    } else {
        for (int b = 0; b < B; b++)
            TRY(argmax_rows<T>(m.d_next + b, (const T *)m.logits + ((size_t)b * S + (S - 1)) * V, 1, V, AdvanceState{}, s));
    }
    launch_timer() = LaunchTimer{};
    m.launches = (int)m.record.size();
    return 0;
}

static int enqueue(Model &m) {
    return dispatch_dtype16(m.cfg.dtype, [&](auto *t) {
        using T = std::remove_pointer_t<decltype(t)>;
        return enqueue_step<T>(m);
    });
}

// ---- weight repacking (explicit, at init, into library-owned buffers) --------------------------
static int concat_rows(void **out, const void *const *parts, const size_t *bytes, int n) {
    size_t total = 0;
    for (int i = 0; i < n; i++) total += bytes[i];
    MYNN_HIP(hipMalloc(out, total));
    size_t off = 0;
    for (int i = 0; i < n; i++) {
        MYNN_HIP(hipMemcpy((char *)*out + off, parts[i], bytes[i], hipMemcpyDeviceToDevice));
        off += bytes[i];
    }
    return 0;
}
static int interleave_rows(void **out, const void *a, const void *b, size_t rows, size_t row_bytes) {
    MYNN_HIP(hipMalloc(out, 2 * rows * row_bytes));
    MYNN_HIP(hipMemcpy2D(*out, 2 * row_bytes, a, row_bytes, row_bytes, rows, hipMemcpyDeviceToDevice));
    MYNN_HIP(hipMemcpy2D((char *)*out + row_bytes, 2 * row_bytes, b, row_bytes, row_bytes, rows, hipMemcpyDeviceToDevice));
    return 0;
}

static int host_rope_tables(Model &m);
static int capture_step(Model &m);

static int build(Model &m, void **init, void **state) {
    const mynn_model_config &c = m.cfg;
    const size_t eb = dtype_size(c.dtype);
    const int H = c.hidden, QD = c.n_heads * c.head_dim, KD = c.n_kv_heads * c.head_dim, F = c.ffn, V = c.vocab;
    const size_t wb = m.quant ? 1 : eb;  // bytes per weight element
    int i = 0;
    auto lin = [&](Lin &l, int N, int K) {
        l.w = init[i++];
        l.scale = m.quant ? init[i++] : (i++, nullptr);
        l.N = N;
        l.K = K;
    };
    WeightSet &ws = *m.wset;
    std::lock_guard<std::mutex> ws_lock(ws.mu);  // derived copies are made once per set, by whichever executor comes first
    // a stage that failed half-way (out of memory) left its flag unset: the next builder makes the stage again, over
    // whatever the failed one had allocated
    auto renew = [](void **p) {
        if (*p) (void)hipFree(*p);
        *p = nullptr;
    };
    if (!ws.repacked) ws.bytes_repack = 0;
    lin(m.embed, V, H);
    m.layers.resize(c.n_layers);
    for (int li = 0; li < c.n_layers; li++) {
        Layer &L = m.layers[li];
        L.norm1 = init[i++];
        Lin q, k, v;
        const void *qb = nullptr, *kb = nullptr, *vb = nullptr;
        lin(q, QD, H); if (c.qkv_bias) qb = init[i++];
        lin(k, KD, H); if (c.qkv_bias) kb = init[i++];
        lin(v, KD, H); if (c.qkv_bias) vb = init[i++];
        lin(L.o, H, QD);
        WeightLayer &W = ws.layers[li];
        if (c.qkv_bias) {
            MYNN_REQUIRE(qb && kb && vb, MYNN_ERR_INVALID, "model_init: null projection bias in layer %d", li);
            const void *bp[3] = {qb, kb, vb};
            const size_t bb[3] = {(size_t)QD * eb, (size_t)KD * eb, (size_t)KD * eb};
            if (!ws.repacked) {
                renew(&W.qkv_b);
                TRY(concat_rows(&W.qkv_b, bp, bb, 3));
                ws.bytes_repack += bb[0] + bb[1] + bb[2];
            }
            L.qkv_b = W.qkv_b;
        }
        L.norm2 = init[i++];
        lin(L.gate, F, H); lin(L.up, F, H); lin(L.down, H, F);
        MYNN_REQUIRE(L.norm1 && L.norm2 && q.w && k.w && v.w && L.o.w && L.gate.w && L.up.w && L.down.w,
                     MYNN_ERR_INVALID, "model_init: null weight in layer %d", li);
        MYNN_REQUIRE(!m.quant || (q.scale && k.scale && v.scale && L.o.scale && L.gate.scale && L.up.scale && L.down.scale),
                     MYNN_ERR_INVALID, "model_init: null scale in layer %d", li);
        const void *parts[3] = {q.w, k.w, v.w};
        const size_t pb[3] = {(size_t)QD * H * wb, (size_t)KD * H * wb, (size_t)KD * H * wb};
        if (!ws.repacked) {
            renew(&W.qkv_w);
            TRY(concat_rows(&W.qkv_w, parts, pb, 3));
            ws.bytes_repack += pb[0] + pb[1] + pb[2];
        }
        L.qkv.w = W.qkv_w; L.qkv.N = QD + 2 * KD; L.qkv.K = H;
        if (m.quant) {
            const void *sp[3] = {q.scale, k.scale, v.scale};
            const size_t sb[3] = {(size_t)QD * eb, (size_t)KD * eb, (size_t)KD * eb};
            if (!ws.repacked) {
                renew(&W.qkv_s); renew(&W.gu_w); renew(&W.gu_s);
                TRY(concat_rows(&W.qkv_s, sp, sb, 3));
                TRY(interleave_rows(&W.gu_w, L.gate.w, L.up.w, F, (size_t)H));
                TRY(interleave_rows(&W.gu_s, L.gate.scale, L.up.scale, F, eb));
                ws.bytes_repack += sb[0] + sb[1] + sb[2] + 2 * (size_t)F * H + 2 * (size_t)F * eb;
            }
            L.qkv.scale = W.qkv_s;
            L.gu.w = W.gu_w; L.gu.scale = W.gu_s; L.gu.N = 2 * F; L.gu.K = H;
        }
        const int per_layer = c.quant_kv_cache ? 4 : 2;
        L.k_cache = state[per_layer * li];
        L.v_cache = state[per_layer * li + 1];
        MYNN_REQUIRE(L.k_cache && L.v_cache, MYNN_ERR_INVALID, "model_init: null KV buffer in layer %d", li);
        if (c.quant_kv_cache) {
            L.k_scale = state[per_layer * li + 2];
            L.v_scale = state[per_layer * li + 3];
            MYNN_REQUIRE(L.k_scale && L.v_scale, MYNN_ERR_INVALID, "model_init: null KV scale buffer in layer %d", li);
        }
    }
    if (c.kv_page_rows) {
        m.pages = (mynn_kv_pages *)state[(c.quant_kv_cache ? 4 : 2) * c.n_layers];
        MYNN_REQUIRE(m.pages, MYNN_ERR_INVALID, "model_init: kv_page_rows without a page set after the pools in session_state");
        m.paging = kv_pages_paging(m.pages);
        MYNN_REQUIRE((1 << m.paging.shift) == c.kv_page_rows && m.paging.pages_per_seq * c.kv_page_rows == c.max_seq &&
                         kv_pages_batch(m.pages) == c.batch,
                     MYNN_ERR_INVALID, "model_init: the page set (batch %d, %d pages of %d rows) does not fit batch %d, max_seq %d, kv_page_rows %d",
                     kv_pages_batch(m.pages), m.paging.pages_per_seq, 1 << m.paging.shift, c.batch, c.max_seq, c.kv_page_rows);
    }
    ws.repacked = true;
    m.final_norm = init[i++];
    lin(m.lm_head, V, H);
    MYNN_REQUIRE(m.embed.w && m.final_norm && m.lm_head.w, MYNN_ERR_INVALID, "model_init: null embed/norm/lm_head");

    MYNN_HIP(hipStreamCreateWithFlags(&m.stream, hipStreamNonBlocking));
    TRY(host_rope_tables(m));

    if (c.weight_arena && m.quant) {
        // One allocation for every int8 linear weight and its scales, in the order a step reads them (the caller's o / down /
        // lm_head buffers are copied, like q|k|v and gate/up already are): an explicit repack, done once.
        struct Piece { const void **slot; size_t bytes; };
        std::vector<Piece> pieces;
        auto add = [&](Lin &l) {
            pieces.push_back({&l.w, (size_t)l.N * l.K});
            pieces.push_back({&l.scale, (size_t)l.N * eb});
        };
        for (Layer &L : m.layers) { add(L.qkv); add(L.o); add(L.gu); add(L.down); }
        add(m.lm_head);
        size_t total = 0;
        for (const Piece &pc : pieces) total += align_up(pc.bytes, 256);
        MYNN_HIP(hipMalloc(&m.warena, total));
        size_t off = 0;
        for (const Piece &pc : pieces) {
            MYNN_HIP(hipMemcpy((char *)m.warena + off, *pc.slot, pc.bytes, hipMemcpyDeviceToDevice));
            *pc.slot = (char *)m.warena + off;
            off += align_up(pc.bytes, 256);
        }
        // (the set keeps its repacked copies: other executors of the session may use them)
    }

    // ---- prefill executors keep every linear weight dequantised to the 16-bit type (2 bytes per weight
    // on top of the int8 originals): the matrix-core GEMM reads them directly, and the values are
    // those of the per-call dequantisation, T(wq * scale)
    {
        const int rows_ = c.batch * c.seq_q;
        m.skinny = m.quant && !c.quantize_activations && skinny_gemm_supported(rows_, QD + 2 * KD, H) &&
                   skinny_gemm_supported(rows_, H, QD) && skinny_gemm_supported(rows_, 2 * F, H) &&
                   skinny_gemm_supported(rows_, H, F) && skinny_gemm_supported(rows_, V, H);
    }
    if (m.skinny) {
        // one more int8 copy of every linear weight, tiled for sequential streaming (1 byte per weight)
        if (!ws.packed8) {
            ws.bytes_packed8 = 0;
            auto pack = [&](void **dst, const Lin &l) {
                renew(dst);
                MYNN_HIP(hipMalloc(dst, skinny_packed_bytes(l.N, l.K)));
                ws.bytes_packed8 += skinny_packed_bytes(l.N, l.K);
                return skinny_pack_weight(*dst, (const int8_t *)l.w, l.N, l.K, m.stream);
            };
            for (size_t li = 0; li < m.layers.size(); li++) {
                Layer &L = m.layers[li];
                WeightLayer &W = ws.layers[li];
                TRY(pack(&W.pk_qkv, L.qkv));
                TRY(pack(&W.pk_o, L.o));
                TRY(pack(&W.pk_gu, L.gu));
                TRY(pack(&W.pk_down, L.down));
            }
            TRY(pack(&ws.pk_lm_head, m.lm_head));
            MYNN_HIP(hipStreamSynchronize(m.stream));
            ws.packed8 = true;
        }
        for (size_t li = 0; li < m.layers.size(); li++) {
            Layer &L = m.layers[li];
            const WeightLayer &W = ws.layers[li];
            L.pk_qkv = W.pk_qkv; L.pk_o = W.pk_o; L.pk_gu = W.pk_gu; L.pk_down = W.pk_down;
        }
        m.pk_lm_head = ws.pk_lm_head;
    }
    if (m.quant && !m.skinny && !c.quantize_activations && c.batch * c.seq_q >= 16 && H % 8 == 0 && QD % 8 == 0 && F % 32 == 0) {
        if (!ws.resident16) {
            ws.bytes_resident16 = 0;
            auto resident = [&](void **dst, const Lin &l) {
                renew(dst);
                MYNN_HIP(hipMalloc(dst, gemm_weight_bytes(l.N, l.K)));
                ws.bytes_resident16 += gemm_weight_bytes(l.N, l.K);
                return dequant_weight_rows(*dst, (const int8_t *)l.w, l.scale, l.N, l.K, c.dtype, 0, 0, m.stream);
            };
            for (size_t li = 0; li < m.layers.size(); li++) {
                Layer &L = m.layers[li];
                WeightLayer &W = ws.layers[li];
                TRY(resident(&W.wt_qkv, L.qkv));
                TRY(resident(&W.wt_o, L.o));
                TRY(resident(&W.wt_down, L.down));
                renew(&W.wt_gu);
                MYNN_HIP(hipMalloc(&W.wt_gu, gemm_weight_bytes(2 * F, H)));
                ws.bytes_resident16 += gemm_weight_bytes(2 * F, H);
                TRY(dequant_weight_rows(W.wt_gu, (const int8_t *)L.gate.w, L.gate.scale, F, H, c.dtype, 32, 0, m.stream));
                TRY(dequant_weight_rows(W.wt_gu, (const int8_t *)L.up.w, L.up.scale, F, H, c.dtype, 32, 1, m.stream));
            }
            TRY(resident(&ws.wt_lm_head, m.lm_head));
            MYNN_HIP(hipStreamSynchronize(m.stream));
            ws.resident16 = true;
        }
        for (size_t li = 0; li < m.layers.size(); li++) {
            Layer &L = m.layers[li];
            const WeightLayer &W = ws.layers[li];
            L.wt_qkv = W.wt_qkv; L.wt_o = W.wt_o; L.wt_gu = W.wt_gu; L.wt_down = W.wt_down;
        }
        m.wt_lm_head = ws.wt_lm_head;
        m.resident16 = true;
    }

    if (m.quant && !m.skinny && !m.resident16 && !c.quantize_activations && c.batch * c.seq_q >= 16) {
        // a weight is dequantised per call: the executor's own workspace, sized for its largest linear (never shared
        // with another model or stream, never grown afterwards)
        size_t need = 0;
        auto grow = [&](const Lin &l) { if (l.K % 8 == 0) need = std::max(need, gemm_weight_bytes(l.N, l.K)); };
        for (Layer &L : m.layers) { grow(L.qkv); grow(L.o); grow(L.gate); grow(L.up); grow(L.down); }
        grow(m.lm_head);
        if (need) MYNN_HIP(hipMalloc(&m.ws, need));
    }

    // ---- W8A8 prefill executors: every linear is large enough for the 256-row int8 tiles; gate and up become one
    // product whose store applies SwiGLU, so their rows (and scales) are interleaved in groups of 32 once
    {
        const int rows_ = c.batch * c.seq_q;
        if (m.quant && c.quantize_activations && c.dtype != MYNN_F32 && F % 32 == 0 && qgemm_dma_supported(rows_, QD + 2 * KD, H) &&
            qgemm_dma_supported(rows_, H, QD) && qgemm_dma_supported(rows_, 2 * F, H) && qgemm_dma_supported(rows_, H, F) &&
            qgemm_dma_supported(rows_, V, H)) {
            const size_t seb = dtype_size(c.dtype);
            if (!ws.q8) ws.bytes_q8 = 0;
            for (size_t li = 0; li < m.layers.size() && !ws.q8; li++) {
                Layer &L = m.layers[li];
                WeightLayer &W = ws.layers[li];
                renew(&W.q8_gu); renew(&W.q8_gu_scale);
                MYNN_HIP(hipMalloc(&W.q8_gu, (size_t)2 * F * H));
                MYNN_HIP(hipMalloc(&W.q8_gu_scale, (size_t)2 * F * seb));
                ws.bytes_q8 += (size_t)2 * F * H + (size_t)2 * F * seb;
                TRY(interleave_row_groups(W.q8_gu, L.gate.w, F, (size_t)H, 32, 0, m.stream));
                TRY(interleave_row_groups(W.q8_gu, L.up.w, F, (size_t)H, 32, 1, m.stream));
                TRY(interleave_row_groups(W.q8_gu_scale, L.gate.scale, F, seb, 32, 0, m.stream));
                TRY(interleave_row_groups(W.q8_gu_scale, L.up.scale, F, seb, 32, 1, m.stream));
            }
            MYNN_HIP(hipStreamSynchronize(m.stream));
            ws.q8 = true;
            for (size_t li = 0; li < m.layers.size(); li++) {
                m.layers[li].q8_gu = ws.layers[li].q8_gu;
                m.layers[li].q8_gu_scale = ws.layers[li].q8_gu_scale;
            }
            m.w8a8_fused = true;
        }
    }

    // ---- arena: every activation of one step, the device scalars, attention split scratch
    const int rows = c.batch * c.seq_q;
    {
        const bool fused_attn = m.quant && rows == 1 && !c.quantize_activations && !c.quant_kv_cache && !m.pages &&
                                attention_fused_supported(c.head_dim, c.n_heads / c.n_kv_heads);
        attn_plan(c.batch, c.seq_q, c.n_heads, c.n_kv_heads, c.head_dim, c.dtype, c.quant_kv_cache, c.max_seq, c.max_seq, fused_attn,
                  &m.slice, &m.nsplit, &m.heads_per_wg);
        if (m.pages) {  // decode: the streaming kernel whatever the sizes; prefill: the matrix-core kernel, no key ranges
            m.slice = 0;
            m.nsplit = 1;
            m.heads_per_wg = c.n_heads / c.n_kv_heads;
            if (c.seq_q == 1) attn_stream_plan_paged(c.batch, c.n_kv_heads, c.max_seq, m.paging.shift, &m.slice, &m.nsplit);
        }
    }
    m.token_cap = c.max_seq + 8;
    ArenaPlan plan;
    size_t o_x = plan.take((size_t)rows * H * eb), o_x2 = plan.take((size_t)rows * H * eb);
    size_t o_n = plan.take((size_t)rows * H * eb), o_qkv = plan.take((size_t)rows * (QD + 2 * KD) * eb);
    size_t o_q = plan.take((size_t)rows * QD * eb), o_attn = plan.take((size_t)rows * QD * eb);
    size_t o_g = plan.take((size_t)rows * F * eb), o_u = plan.take((size_t)rows * F * eb);
    size_t o_h = plan.take((size_t)rows * F * eb), o_p = plan.take((size_t)rows * H * eb);
    size_t o_l = plan.take((size_t)rows * V * eb);
    const size_t kmax = (size_t)(F > H ? (F > QD ? F : QD) : (H > QD ? H : QD));
    size_t sk_bytes = 0;
    if (m.skinny) {
        const size_t cand[5] = {skinny_scratch_bytes(rows, QD + 2 * KD, H), skinny_scratch_bytes(rows, H, QD),
                                skinny_scratch_bytes(rows, 2 * F, H), skinny_scratch_bytes(rows, H, F),
                                skinny_scratch_bytes(rows, V, H)};
        for (size_t b : cand) sk_bytes = b > sk_bytes ? b : sk_bytes;
    }
    size_t o_sk = plan.take(sk_bytes);
    size_t o_a8 = plan.take(c.quantize_activations ? (size_t)rows * kmax : 0), o_a8s = plan.take((size_t)rows * eb);
    size_t o_ids = plan.take((size_t)rows * 8), o_pos = plan.take((size_t)c.seq_q * 8);
    size_t o_sc = plan.take(32 + (size_t)c.batch * 4), o_tok = plan.take((size_t)m.token_cap * 4);
    size_t o_as = plan.take(attn_scratch_bytes(c.batch, c.n_heads, c.seq_q, c.head_dim, m.nsplit));
    size_t o_cand = plan.take(rows == 1 ? (size_t)kGemvArgmaxWords * 8 : 0);
    const bool strm = c.streaming_kv != 0;
    size_t o_kvpos = plan.take(strm ? (size_t)c.max_seq * 8 : 0);
    size_t o_qref = plan.take(strm ? (size_t)rows * QD * eb : 0), o_knew = plan.take(strm ? (size_t)rows * KD * eb : 0);
    size_t o_vnew = plan.take(strm ? (size_t)rows * KD * eb : 0), o_aref = plan.take(strm ? (size_t)rows * QD * eb : 0);
    size_t o_krot = plan.take(strm && !c.quant_kv_cache ? (size_t)KD * c.max_seq * eb : 0);
    m.ring_ws_bytes = strm ? mynn_attention_streaming_workspace_bytes(1, c.seq_q, c.max_seq, c.n_heads, c.n_kv_heads, c.head_dim, c.dtype,
                                                                      c.quant_kv_cache, c.quant_kv_cache)
                           : 0;
    size_t o_ring = plan.take(m.ring_ws_bytes);
    m.arena_bytes = plan.off;
    MYNN_HIP(hipMalloc((void **)&m.arena, m.arena_bytes));
    MYNN_HIP(hipMemset(m.arena, 0, m.arena_bytes));
    m.x = m.arena + o_x; m.x2 = m.arena + o_x2; m.nrm = m.arena + o_n; m.qkv = m.arena + o_qkv; m.q = m.arena + o_q;
    m.attn = m.arena + o_attn; m.g = m.arena + o_g; m.u = m.arena + o_u; m.hmid = m.arena + o_h; m.proj = m.arena + o_p;
    m.logits = m.arena + o_l;
    m.a8 = (int8_t *)(m.arena + o_a8); m.a8_scale = m.arena + o_a8s;
    m.skinny_scratch = (float *)(m.arena + o_sk);
    m.d_ids = (int64_t *)(m.arena + o_ids); m.d_pos = (int64_t *)(m.arena + o_pos);
    m.d_past = (int32_t *)(m.arena + o_sc); m.d_active = m.d_past + 1; m.d_step = m.d_past + 2;
    m.d_next = m.d_past + 8;  // one token per sequence after the scalars
    m.d_tokens = (int32_t *)(m.arena + o_tok);
    m.attn_scratch = m.arena + o_as;
    m.lm_cand = (uint64_t *)(m.arena + o_cand);
    m.d_kvpos = (int64_t *)(m.arena + o_kvpos);
    m.q_ref = m.arena + o_qref; m.k_new = m.arena + o_knew; m.v_new = m.arena + o_vnew; m.attn_ref = m.arena + o_aref;
    m.k_rot = m.arena + o_krot;
    m.ring_ws = m.arena + o_ring;
    m.next_stage = align_up((size_t)c.batch * 4, 256);  // the sequences' next tokens live in the tail of the staging buffer
    m.stage_bytes = align_up((size_t)rows * 8 + (size_t)c.seq_q * 8 + 64 + (size_t)m.token_cap * 4 + (strm ? (size_t)c.max_seq * 8 : 0), 256) +
                    256 + m.next_stage;
    MYNN_HIP(hipHostMalloc((void **)&m.h_stage, m.stage_bytes, hipHostMallocDefault));
    MYNN_HIP(hipDeviceSynchronize());

    // ---- batch-1 decode: projection and attention in one launch when the shape allows
    m.spin_limit = c.handover_spin_limit > 0 ? c.handover_spin_limit : c.handover_spin_limit < 0 ? 0 : 400000;
    if (m.quant && rows == 1 && !c.quantize_activations && !c.unfused_decode && (!m.pages || m.paging.pages_per_seq <= 64) && !c.qkv_bias &&
        !c.streaming_kv && attention_fused_supported(c.head_dim, c.n_heads / c.n_kv_heads) &&
        (!c.quant_kv_cache || attention_fused_kv8_supported(c.head_dim, c.max_seq)) &&
        qkv_attention_supported(H, c.n_heads, c.n_kv_heads, c.head_dim, c.max_seq, c.dtype) && (QD + 2 * KD) * eb % 8 == 0) {
        bool ok = aligned16(m.qkv) && aligned16(m.x) && aligned16(m.attn) && aligned16(m.embed.w);
        for (const Layer &L : m.layers)
            ok = ok && aligned16(L.qkv.w) && aligned16(L.norm1) && aligned16(L.norm2) && aligned16(L.k_cache) && aligned16(L.v_cache) && aligned16(L.o.w);
        if (ok && (char *)m.attn > (char *)m.qkv && ((char *)m.attn + (size_t)QD * eb - (char *)m.qkv) % 8 == 0) {
            MYNN_HIP(hipMemset(m.qkv, 0xFF, (size_t)((char *)m.attn + (size_t)QD * eb - (char *)m.qkv)));
            m.lm_argmax = gemv_norm_argmax_supported(m.x, m.final_norm, (const int8_t *)m.lm_head.w, V, H);
            if (m.lm_argmax) MYNN_HIP(hipMemset(m.lm_cand, 0xFF, (size_t)kGemvArgmaxWords * 8));
            MYNN_HIP(hipDeviceSynchronize());
            m.qkv_attn = true;
        }
    }

    // ---- batch-1 decode with quantize_activations: one launch per linear (norm, quantiser, int8 GEMV, residual / SwiGLU)
    if (m.quant && rows == 1 && c.quantize_activations && !c.streaming_kv && !c.unfused_decode && c.dtype != MYNN_F32) {
        bool ok = qgemv_fused_supported(m.x, m.final_norm, (const int8_t *)m.lm_head.w, V, H) && aligned16(m.x2) && aligned16(m.attn) &&
                  aligned16(m.hmid);
        for (const Layer &L : m.layers)
            ok = ok && qgemv_fused_supported(m.x, L.norm1, (const int8_t *)L.qkv.w, L.qkv.N, H) &&
                 qgemv_fused_supported(m.attn, nullptr, (const int8_t *)L.o.w, H, QD) &&
                 qgemv_fused_supported(m.x2, L.norm2, (const int8_t *)L.gu.w, 2 * F, H) &&
                 qgemv_fused_supported(m.hmid, nullptr, (const int8_t *)L.down.w, H, F);
        m.qgemv1 = ok;
    }

    return capture_step(m);
}

// Captures the decode step once (one new token per sequence, any batch: every launch reads its positions and
// lengths from device memory).  Called again when the executor changes its launch plan.
constexpr int kLoopSteps = 32;
static int capture_step(Model &m) {
    if (m.graph_exec) (void)hipGraphExecDestroy(m.graph_exec);
    if (m.graph) (void)hipGraphDestroy(m.graph);
    if (m.graph_loop_exec) (void)hipGraphExecDestroy(m.graph_loop_exec);
    if (m.graph_loop) (void)hipGraphDestroy(m.graph_loop);
    m.graph_exec = m.graph_loop_exec = nullptr;
    m.graph = m.graph_loop = nullptr;
    m.use_graph = false;
    if (m.cfg.seq_q != 1 || m.cfg.streaming_kv) return 0;  // (the streaming operators take host scalars at launch time)
    hipError_t e = hipStreamBeginCapture(m.stream, hipStreamCaptureModeThreadLocal);
    if (e == hipSuccess) {
        int rc = enqueue(m);
        hipError_t e2 = hipStreamEndCapture(m.stream, &m.graph);
        if (rc == 0 && e2 == hipSuccess && hipGraphInstantiate(&m.graph_exec, m.graph, nullptr, nullptr, 0) == hipSuccess)
            m.use_graph = true;
        else {
            (void)hipGetLastError();
            if (rc) return rc;
        }
    } else (void)hipGetLastError();
    // batch-1 decode: several steps in one graph for the device-resident loop (every step leaves the next one's token,
    // position and lengths on the device, so the steps of a graph chain like separate launches of the one-step graph)
    if (m.use_graph && m.cfg.batch == 1 && hipStreamBeginCapture(m.stream, hipStreamCaptureModeThreadLocal) == hipSuccess) {
        int rc = 0;
        for (int i = 0; i < kLoopSteps && rc == 0; i++) rc = enqueue(m);
        hipError_t e2 = hipStreamEndCapture(m.stream, &m.graph_loop);
        if (rc != 0 || e2 != hipSuccess || hipGraphInstantiate(&m.graph_loop_exec, m.graph_loop, nullptr, nullptr, 0) != hipSuccess) {
            (void)hipGetLastError();
            if (m.graph_loop) (void)hipGraphDestroy(m.graph_loop);
            m.graph_loop = nullptr;
            m.graph_loop_exec = nullptr;
            if (rc) return rc;
        }
    } else (void)hipGetLastError();
    return 0;
}

static int host_rope_tables(Model &m) {
    const mynn_model_config &c = m.cfg;
    const size_t eb = dtype_size(c.dtype), n = (size_t)c.max_seq * c.head_dim;
    std::vector<char> hc(n * eb), hs(n * eb);
    TRY(mynn_rope_table(hc.data(), hs.data(), c.max_seq, c.head_dim, c.rope_theta, c.dtype));
    MYNN_HIP(hipMalloc(&m.cos_t, n * eb));
    MYNN_HIP(hipMalloc(&m.sin_t, n * eb));
    MYNN_HIP(hipMemcpy(m.cos_t, hc.data(), n * eb, hipMemcpyHostToDevice));
    MYNN_HIP(hipMemcpy(m.sin_t, hs.data(), n * eb, hipMemcpyHostToDevice));
    return 0;
}

static void destroy(Model *m) {
    if (!m) return;
    if (m->stream) hipStreamSynchronize(m->stream);
    for (hipEvent_t e : m->events) hipEventDestroy(e);
    if (m->graph_exec) hipGraphExecDestroy(m->graph_exec);
    if (m->graph) hipGraphDestroy(m->graph);
    if (m->graph_loop_exec) hipGraphExecDestroy(m->graph_loop_exec);
    if (m->graph_loop) hipGraphDestroy(m->graph_loop);
    weight_set_release(m->wset);
    if (m->ws) hipFree(m->ws);
    if (m->warena) hipFree(m->warena);
    if (m->cos_t) hipFree(m->cos_t);
    if (m->sin_t) hipFree(m->sin_t);
    if (m->arena) hipFree(m->arena);
    if (m->h_stage) hipHostFree(m->h_stage);
    if (m->stream) hipStreamDestroy(m->stream);
    delete m;
}

// H2D of one step's inputs (ids, positions, past_len, active, step counter = 0) in one copy
static int upload_inputs(Model &m, const int64_t *ids, const int64_t *pos, int64_t past, int64_t active) {
    const mynn_model_config &c = m.cfg;
    const int rows = c.batch * c.seq_q;
    // (streaming_kv: past_len is the session's unbounded stream position; the ring map folds it into the cache)
    MYNN_REQUIRE(past >= 0 && (c.streaming_kv ? past + c.seq_q <= INT32_MAX : past + c.seq_q <= c.max_seq), MYNN_ERR_TOO_LONG,
                 "past_len %lld + %d rows exceeds max_seq %d", (long long)past, c.seq_q, c.max_seq);
    MYNN_REQUIRE(active >= 1 && active <= c.max_seq, MYNN_ERR_INVALID, "active_seq_kv %lld out of range", (long long)active);
    // paged cache: every row the step writes or may read has a page before anything is launched
    if (m.pages) TRY(kv_pages_reserve(m.pages, std::max<long>(past + c.seq_q, active)));
    for (int s = 0; s < c.seq_q; s++)
        MYNN_REQUIRE(pos[s] >= 0 && pos[s] < c.max_seq, MYNN_ERR_INVALID, "position_id[%d]=%lld outside the RoPE table", s,
                     (long long)pos[s]);
    for (int r = 0; r < rows; r++)
        MYNN_REQUIRE(ids[r] >= -c.vocab && ids[r] < c.vocab, MYNN_ERR_INVALID, "input_ids[%d]=%lld outside the vocabulary", r,
                     (long long)ids[r]);
    int64_t *h_ids = (int64_t *)m.h_stage;
    int64_t *h_pos = h_ids + rows;
    int32_t *h_sc = (int32_t *)(h_pos + c.seq_q);
    memcpy(h_ids, ids, (size_t)rows * 8);
    memcpy(h_pos, pos, (size_t)c.seq_q * 8);
    h_sc[0] = (int32_t)past; h_sc[1] = (int32_t)active; h_sc[2] = 0;
    m.h_past = (int)past;
    m.h_active = (int)active;
    MYNN_HIP(hipMemcpyAsync(m.d_ids, h_ids, (size_t)rows * 8, hipMemcpyHostToDevice, m.stream));
    MYNN_HIP(hipMemcpyAsync(m.d_pos, h_pos, (size_t)c.seq_q * 8, hipMemcpyHostToDevice, m.stream));
    MYNN_HIP(hipMemcpyAsync(m.d_past, h_sc, 12, hipMemcpyHostToDevice, m.stream));
    return 0;
}

// A wait inside a fused launch ran out (the error word is set; read back after the stream has drained): the step's
// results -- logits, token, loop state, the KV row it appended -- are undefined.  The executor empties the hand-over
// vectors, gives up sharing launches for good (every op becomes a launch of its own: same arithmetic, bit-identical
// results, no workgroup ever waits for another) and captures its step again; the caller then repeats the step from
// its host-side inputs, which overwrites the KV row.
static int handover_recover(Model &m) {
    const mynn_model_config &c = m.cfg;
    MYNN_HIP(hipMemset(m.qkv, 0xFF, (size_t)((char *)m.attn + (size_t)c.n_heads * c.head_dim * dtype_size(c.dtype) - (char *)m.qkv)));
    MYNN_HIP(hipMemset(m.lm_cand, 0xFF, (size_t)kGemvArgmaxWords * 8));
    MYNN_HIP(hipMemset(m.d_past + 3, 0, 4));
    if (!m.fell_back && m.handover_failures == 0) {
        m.shared_qkv_attn = m.qkv_attn;
        m.shared_lm_argmax = m.lm_argmax;
    } else if (m.rearm_after > 0 && m.rearm_after < (1 << 20)) {
        m.rearm_after *= 2;  // it happened again after a re-arm: wait twice as long before the next try
    }
    m.handover_failures++;
    m.fell_back = true;
    m.clean_steps = 0;
    m.qkv_attn = false;
    m.lm_argmax = false;
    set_error("decode step: a stage of a fused launch waited too long for the stage before it (is the device shared?); "
              "the executor now runs one op per launch");
    return capture_step(m);
}

// `steps` more steps went through without a give-up (the stream is drained).  A model that fell back goes back to the
// shared launches once enough of them have: what made a producer late (another process on the device, a debugger, a
// serialising tool) is usually gone by then, and staying with one op per launch for the rest of a long-lived
// executor's life would cost it a third of its speed.  The hand-over vectors are emptied first: as ordinary
// activation buffers of the one-op-per-launch step they hold data.
static int handover_clean_steps(Model &m, long steps) {
    if (!m.fell_back || m.rearm_after <= 0) return 0;
    m.clean_steps += steps;
    if (m.clean_steps < m.rearm_after) return 0;
    const mynn_model_config &c = m.cfg;
    MYNN_HIP(hipMemset(m.qkv, 0xFF, (size_t)((char *)m.attn + (size_t)c.n_heads * c.head_dim * dtype_size(c.dtype) - (char *)m.qkv)));
    MYNN_HIP(hipMemset(m.lm_cand, 0xFF, (size_t)kGemvArgmaxWords * 8));
    MYNN_HIP(hipMemset(m.d_past + 3, 0, 4));
    m.qkv_attn = m.shared_qkv_attn;
    m.lm_argmax = m.shared_lm_argmax;
    m.fell_back = false;
    m.clean_steps = 0;
    return capture_step(m);
}

static int run_once(Model &m) {
    if (m.use_graph && !m.profiling) {
        MYNN_HIP(hipGraphLaunch(m.graph_exec, m.stream));
        return 0;
    }
    return enqueue(m);
}

}  // namespace mynn

using namespace mynn;

static int check_config(const mynn_model_config *cfg) {
    MYNN_REQUIRE(cfg, MYNN_ERR_INVALID, "model_configure: null config");
    MYNN_REQUIRE(cfg->n_layers > 0 && cfg->hidden > 0 && cfg->n_heads > 0 && cfg->n_kv_heads > 0 && cfg->head_dim > 0 &&
                     cfg->ffn > 0 && cfg->vocab > 0 && cfg->max_seq > 0 && cfg->seq_q > 0 && cfg->batch > 0,
                 MYNN_ERR_INVALID, "model_configure: non-positive dimension");
    MYNN_REQUIRE(cfg->hidden == cfg->n_heads * cfg->head_dim, MYNN_ERR_INVALID,
                 "model_configure: hidden %d != n_heads %d * head_dim %d", cfg->hidden, cfg->n_heads, cfg->head_dim);
    MYNN_REQUIRE(cfg->n_heads % cfg->n_kv_heads == 0, MYNN_ERR_INVALID, "model_configure: heads not a multiple of kv heads");
    MYNN_REQUIRE(cfg->dtype == MYNN_F16 || cfg->dtype == MYNN_BF16, MYNN_ERR_UNSUPPORTED,
                 "model_configure: dtype %d (fp16 or bf16 only)", cfg->dtype);
    MYNN_REQUIRE(!cfg->quantize_activations || (cfg->weights_int8 && cfg->hidden % 32 == 0 && cfg->ffn % 32 == 0),
                 MYNN_ERR_UNSUPPORTED, "model_configure: quantize_activations needs int8 weights and K %% 32 == 0");
    MYNN_REQUIRE(!cfg->quant_kv_cache || (cfg->head_dim % 2 == 0 && cfg->head_dim <= 128), MYNN_ERR_UNSUPPORTED,
                 "model_configure: quant_kv_cache needs an even head_dim <= 128 (got %d)", cfg->head_dim);
    MYNN_REQUIRE(cfg->seq_q <= cfg->max_seq, MYNN_ERR_INVALID, "model_configure: prefill_len %d > max_seq %d", cfg->seq_q,
                 cfg->max_seq);
    MYNN_REQUIRE(cfg->gemm_tile >= 0 && cfg->gemm_tile <= 4, MYNN_ERR_INVALID, "model_configure: gemm_tile %d (0..4)", cfg->gemm_tile);
    MYNN_REQUIRE(!cfg->streaming_kv || (cfg->batch == 1 && cfg->head_dim % 2 == 0), MYNN_ERR_UNSUPPORTED,
                 "model_configure: streaming_kv is a batch-1 graph (crates/llm) with an even head_dim");
    if (cfg->kv_page_rows) {
        const int P = cfg->kv_page_rows;
        MYNN_REQUIRE(P >= 64 && (P & (P - 1)) == 0 && cfg->max_seq % P == 0, MYNN_ERR_INVALID,
                     "model_configure: kv_page_rows %d (a power of two >= 64 that divides max_seq %d)", P, cfg->max_seq);
        MYNN_REQUIRE(!cfg->streaming_kv, MYNN_ERR_UNSUPPORTED, "model_configure: a paged KV cache does not take streaming_kv");
        MYNN_REQUIRE(!cfg->quant_kv_cache || cfg->seq_q == 1, MYNN_ERR_UNSUPPORTED,
                     "model_configure: a paged int8 KV cache serves decode models only (the prefill kernel reads 16-bit pages)");
        MYNN_REQUIRE(cfg->seq_q == 1 || cfg->max_seq / P <= 64, MYNN_ERR_UNSUPPORTED,
                     "model_configure: a prefill model reads at most 64 pages per sequence (max_seq %d, %d rows per page)", cfg->max_seq, P);
        MYNN_REQUIRE(attn_stream_paged_supported(1, cfg->n_heads, cfg->n_kv_heads, cfg->head_dim, cfg->dtype, P), MYNN_ERR_UNSUPPORTED,
                     "model_configure: a paged KV cache needs head_dim 64 or 128 and 1, 2, 4 or 8 query heads per kv head");
    }
    return 0;
}

extern "C" int mynn_model_configure(const mynn_model_config *cfg) {
    TRY(check_config(cfg));
    std::lock_guard<std::mutex> lk(g_mu);
    g_cfg = *cfg;
    g_cfg_set = true;
    return 0;
}

static void *model_create_with(const mynn_model_config *cfg, WeightSet *wset, void **session_state) {
    Model *m = new Model;
    m->cfg = *cfg;
    m->quant = cfg->weights_int8 != 0;
    m->wset = wset;  // (one reference is the model's from here on: destroy() lets it go)
    if (build(*m, wset->initializer.data(), session_state)) {
        destroy(m);
        return nullptr;
    }
    return m;
}

extern "C" void *mynn_model_create(const mynn_model_config *cfg, void **initializer, void **session_state) {
    if (check_config(cfg)) return nullptr;
    if (!initializer || !session_state) {
        fail(MYNN_ERR_INVALID, "model_create: null initializer / session_state array");
        return nullptr;
    }
    return model_create_with(cfg, weight_set_new(*cfg, initializer), session_state);  // a set of its own
}

extern "C" mynn_weight_set *mynn_weight_set_create(const mynn_model_config *cfg, void **initializer) {
    if (check_config(cfg)) return nullptr;
    if (!initializer) {
        fail(MYNN_ERR_INVALID, "weight_set_create: null initializer array");
        return nullptr;
    }
    return (mynn_weight_set *)weight_set_new(*cfg, initializer);
}
extern "C" void mynn_weight_set_destroy(mynn_weight_set *set) { weight_set_release((WeightSet *)set); }
extern "C" int mynn_weight_set_stats(mynn_weight_set *set, size_t *bytes /*[4]*/, int *holders) {
    MYNN_REQUIRE(set, MYNN_ERR_INVALID, "weight_set_stats: null set");
    WeightSet &w = *(WeightSet *)set;
    std::lock_guard<std::mutex> lk(w.mu);
    if (bytes) {
        bytes[0] = w.bytes_repack; bytes[1] = w.bytes_resident16; bytes[2] = w.bytes_packed8; bytes[3] = w.bytes_q8;
    }
    if (holders) *holders = w.refs;
    return 0;
}
extern "C" void *mynn_model_create_shared(const mynn_model_config *cfg, mynn_weight_set *set, void **session_state) {
    if (check_config(cfg)) return nullptr;
    if (!set || !session_state) {
        fail(MYNN_ERR_INVALID, "model_create_shared: null weight set / session_state array");
        return nullptr;
    }
    WeightSet *w = (WeightSet *)set;
    {
        std::lock_guard<std::mutex> lk(w->mu);
        if (!weight_set_fits(*w, *cfg)) {
            fail(MYNN_ERR_INVALID, "model_create_shared: the weight set was made for other shapes, another storage type or other weight options");
            return nullptr;
        }
        w->refs++;
    }
    return model_create_with(cfg, w, session_state);
}

extern "C" void *model_init(void **initializer, void **session_state) {
    mynn_model_config cfg;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (!g_cfg_set) {
            fail(MYNN_ERR_STATE, "model_init: call mynn_model_configure first");
            return nullptr;
        }
        cfg = g_cfg;
    }
    return mynn_model_create(&cfg, initializer, session_state);
}

extern "C" void model_destroy(void *state) { destroy((Model *)state); }
extern "C" void model_device_sync(void) { (void)hipDeviceSynchronize(); }
extern "C" int model_memcpy(void *dst, const void *src, size_t n, int kind) {
    return (int)hipMemcpy(dst, src, n, (hipMemcpyKind)kind);
}
extern "C" void *alloc_pinned(size_t n) {
    void *p = nullptr;
    if (hipHostMalloc(&p, n, hipHostMallocDefault) != hipSuccess) return nullptr;
    return p;
}
extern "C" void free_pinned(void *p) {
    if (p) (void)hipHostFree(p);
}

// one step; *handover_failed is set when a fused launch gave up (results undefined, error word still set)
static int step_once(Model &m, const int64_t *input_ids, const int64_t *position_id, int64_t past_len, int64_t active_seq_kv,
                     int32_t *next_token, void *logits_host, bool *handover_failed) {
    *handover_failed = false;
    TRY(upload_inputs(m, input_ids, position_id, past_len, active_seq_kv));
    TRY(run_once(m));
    const mynn_model_config &c = m.cfg;
    char *h_next = m.h_stage + m.stage_bytes - m.next_stage;
    // (fused projection + attention: the error word travels in the same copy, d_past[3] .. d_next[0])
    if (m.qkv_attn) MYNN_HIP(hipMemcpyAsync(h_next, m.d_past + 3, 24, hipMemcpyDeviceToHost, m.stream));
    else if (next_token) MYNN_HIP(hipMemcpyAsync(h_next, m.d_next, (size_t)c.batch * 4, hipMemcpyDeviceToHost, m.stream));
    if (logits_host)
        MYNN_HIP(hipMemcpyAsync(logits_host, m.logits, (size_t)c.batch * c.seq_q * c.vocab * dtype_size(c.dtype),
                                hipMemcpyDeviceToHost, m.stream));
    MYNN_HIP(hipStreamSynchronize(m.stream));
    if (m.qkv_attn) {
        if (*(const int32_t *)h_next) {
            *handover_failed = true;
            return 0;
        }
        if (next_token) memcpy(next_token, h_next + 20, 4);
        return 0;
    }
    if (next_token) memcpy(next_token, h_next, (size_t)c.batch * 4);
    return 0;
}

extern "C" int mynn_model_step(void *state, const int64_t *input_ids, const int64_t *position_id, int64_t past_len,
                               int64_t active_seq_kv, int32_t *next_token, void *logits_host) {
    MYNN_REQUIRE(state && input_ids && position_id, MYNN_ERR_INVALID, "model_step: null argument");
    Model &m = *(Model *)state;
    MYNN_REQUIRE(!m.cfg.streaming_kv, MYNN_ERR_STATE, "model_step: a streaming_kv model takes the ring inputs (mynn_model_step_streaming)");
    bool failed = false;
    TRY(step_once(m, input_ids, position_id, past_len, active_seq_kv, next_token, logits_host, &failed));
    if (!failed) return handover_clean_steps(m, 1);
    TRY(handover_recover(m));
    TRY(step_once(m, input_ids, position_id, past_len, active_seq_kv, next_token, logits_host, &failed));
    return failed ? fail(MYNN_ERR_STATE, "decode step: hand-over failure after recovery") : 0;
}

extern "C" int mynn_model_step_streaming(void *state, const int64_t *input_ids, const int64_t *position_id, int64_t past_len,
                                         int64_t active_seq_kv, int64_t ring_sink, int64_t ring_window, int64_t ring_start,
                                         const int64_t *kv_position, int32_t *next_token, void *logits_host) {
    MYNN_REQUIRE(state && input_ids && position_id && kv_position, MYNN_ERR_INVALID, "model_step_streaming: null argument");
    Model &m = *(Model *)state;
    const mynn_model_config &c = m.cfg;
    MYNN_REQUIRE(c.streaming_kv, MYNN_ERR_STATE, "model_step_streaming: the model was not built with streaming_kv");
    MYNN_REQUIRE(ring_sink >= 0 && ring_window > 0 && ring_sink + ring_window <= c.max_seq && ring_start >= 0 && ring_start < ring_window,
                 MYNN_ERR_INVALID, "model_step_streaming: ring sink=%lld window=%lld start=%lld (max_seq %d)", (long long)ring_sink,
                 (long long)ring_window, (long long)ring_start, c.max_seq);
    // past_len may lie past sink + window: the operators then apply the reference's own formulas to the session's
    // inputs (kvcache_update.cuh:21 maps past_len + t through ring_phys_index with the session's ring_start;
    // attention.cuh:397, 549 enumerate ranks through the same map), whatever slot that names.
    MYNN_REQUIRE(active_seq_kv >= c.seq_q && active_seq_kv <= ring_sink + ring_window, MYNN_ERR_INVALID,
                 "model_step_streaming: active_seq_kv %lld outside [%d, sink + window = %lld]", (long long)active_seq_kv, c.seq_q,
                 (long long)(ring_sink + ring_window));
    for (int r = 0; r < c.max_seq; r++)
        MYNN_REQUIRE(kv_position[r] >= 0 && kv_position[r] < c.max_seq, MYNN_ERR_INVALID, "kv_position[%d]=%lld outside the RoPE table",
                     r, (long long)kv_position[r]);
    m.ring_sink = (int)ring_sink;
    m.ring_window = (int)ring_window;
    m.ring_start = (int)ring_start;
    int64_t *h_kvpos = (int64_t *)(m.h_stage + align_up((size_t)c.batch * c.seq_q * 8 + (size_t)c.seq_q * 8 + 64 + (size_t)m.token_cap * 4, 8));
    memcpy(h_kvpos, kv_position, (size_t)c.max_seq * 8);
    MYNN_HIP(hipMemcpyAsync(m.d_kvpos, h_kvpos, (size_t)c.max_seq * 8, hipMemcpyHostToDevice, m.stream));
    bool failed = false;
    return step_once(m, input_ids, position_id, past_len, active_seq_kv, next_token, logits_host, &failed);
}

extern "C" int mynn_model_release_kv_pages(void *state) {
    MYNN_REQUIRE(state, MYNN_ERR_INVALID, "model_release_kv_pages: null state");
    Model &m = *(Model *)state;
    return m.pages ? mynn_kv_pages_release(m.pages) : 0;
}
extern "C" int mynn_model_handover_failures(void *state) { return state ? ((Model *)state)->handover_failures : 0; }
extern "C" int mynn_model_set_handover_rearm(void *state, int clean_steps) {
    MYNN_REQUIRE(state && clean_steps >= 0, MYNN_ERR_INVALID, "model_set_handover_rearm: bad argument");
    ((Model *)state)->rearm_after = clean_steps;
    return 0;
}
extern "C" int mynn_model_last_status(void *state) { return state ? ((Model *)state)->last_status : MYNN_ERR_INVALID; }

// Reference ABI: void, host pointers, synchronous.  A failure is reported on stderr, through mynn_last_error()
// and mynn_model_last_status(); it never exits the process.
extern "C" void model(void *state, void **output, void **input) {
    if (!state || !output || !input) {
        fail(MYNN_ERR_INVALID, "model: null argument");
        fprintf(stderr, "mynn model(): %s\n", mynn_last_error());
        if (state) ((Model *)state)->last_status = MYNN_ERR_INVALID;
        return;
    }
    Model &m = *(Model *)state;
    int rc;
    if (m.cfg.streaming_kv)
        rc = mynn_model_step_streaming(state, (const int64_t *)input[0], (const int64_t *)input[1], *(const int64_t *)input[2],
                                       *(const int64_t *)input[3], *(const int64_t *)input[4], *(const int64_t *)input[5],
                                       *(const int64_t *)input[6], (const int64_t *)input[7], nullptr, output[0]);
    else
        rc = mynn_model_step(state, (const int64_t *)input[0], (const int64_t *)input[1], *(const int64_t *)input[2],
                             *(const int64_t *)input[3], nullptr, output[0]);
    m.last_status = rc;
    if (rc) fprintf(stderr, "mynn model(): error %d: %s\n", rc, mynn_last_error());
}

extern "C" int mynn_model_argmax_row(void *state, int row, int32_t *token) {
    MYNN_REQUIRE(state && token, MYNN_ERR_INVALID, "model_argmax_row: null argument");
    Model &m = *(Model *)state;
    const mynn_model_config &c = m.cfg;
    MYNN_REQUIRE(row >= 0 && row < c.batch * c.seq_q, MYNN_ERR_INVALID, "model_argmax_row: row %d", row);
    const char *l = (const char *)m.logits + (size_t)row * c.vocab * dtype_size(c.dtype);
    TRY(mynn_argmax_last(m.d_next, l, c.vocab, c.dtype, m.stream));
    MYNN_HIP(hipMemcpyAsync(m.h_stage, m.d_next, 4, hipMemcpyDeviceToHost, m.stream));
    MYNN_HIP(hipStreamSynchronize(m.stream));
    memcpy(token, m.h_stage, 4);
    return 0;
}

extern "C" const void *mynn_model_logits_device(void *state) { return state ? ((Model *)state)->logits : nullptr; }

extern "C" int mynn_model_stats(void *state, size_t *arena_bytes, int *launches_per_step, int *graph) {
    MYNN_REQUIRE(state, MYNN_ERR_INVALID, "model_stats: null state");
    Model &m = *(Model *)state;
    if (arena_bytes) *arena_bytes = m.arena_bytes;
    if (launches_per_step) *launches_per_step = m.launches;
    if (graph) *graph = m.use_graph ? 1 : 0;
    return 0;
}

extern "C" int mynn_model_decode_loop(void *state, int32_t token, int64_t past_len, int n_steps, int32_t *out_tokens) {
    MYNN_REQUIRE(state && out_tokens && n_steps > 0, MYNN_ERR_INVALID, "decode_loop: bad argument");
    Model &m = *(Model *)state;
    const mynn_model_config &c = m.cfg;
    MYNN_REQUIRE(c.batch * c.seq_q == 1 && !c.streaming_kv, MYNN_ERR_STATE, "decode_loop: needs a batch-1 decode model without streaming_kv");
    MYNN_REQUIRE(past_len + n_steps <= c.max_seq && n_steps <= m.token_cap, MYNN_ERR_TOO_LONG,
                 "decode_loop: past_len %lld + %d steps exceeds max_seq %d", (long long)past_len, n_steps, c.max_seq);
    if (m.pages) TRY(kv_pages_reserve(m.pages, past_len + n_steps));
    for (int attempt = 0; attempt < 2; attempt++) {
        int64_t id = token, pos = past_len;
        TRY(upload_inputs(m, &id, &pos, past_len, past_len + 1));
        int done = 0;
        if (m.use_graph && !m.profiling && m.graph_loop_exec)
            for (; done + kLoopSteps <= n_steps; done += kLoopSteps) MYNN_HIP(hipGraphLaunch(m.graph_loop_exec, m.stream));
        for (; done < n_steps; done++) TRY(run_once(m));
        MYNN_HIP(hipMemcpyAsync(m.h_stage, m.d_tokens, (size_t)n_steps * 4, hipMemcpyDeviceToHost, m.stream));
        char *h_err = m.h_stage + m.stage_bytes - m.next_stage;
        if (m.qkv_attn) MYNN_HIP(hipMemcpyAsync(h_err, m.d_past + 3, 4, hipMemcpyDeviceToHost, m.stream));
        MYNN_HIP(hipStreamSynchronize(m.stream));
        if (m.qkv_attn && *(const int32_t *)h_err) {
            // some step's hand-over gave up: every later token is undefined.  Rebuild with one op per launch and run the
            // whole loop again from the same inputs (the KV rows are overwritten).
            TRY(handover_recover(m));
            continue;
        }
        memcpy(out_tokens, m.h_stage, (size_t)n_steps * 4);
        return handover_clean_steps(m, n_steps);
    }
    return fail(MYNN_ERR_STATE, "decode loop: hand-over failure after recovery");
}

static int profile_enqueue(Model &m, mynn_kernel_time *out, int cap) {
    for (hipEvent_t e : m.events) hipEventDestroy(e);
    m.events.clear();
    m.profiling = true;
    int rc = enqueue(m);
    m.profiling = false;
    launch_timer() = LaunchTimer{};
    if (rc) return rc;
    MYNN_HIP(hipStreamSynchronize(m.stream));
    int n = (int)m.record.size();
    for (int i = 0; i < n && i < cap; i++) {
        float ms = 0.f;
        // a record whose launch did not take the pair (or that made none) reports 0
        if (hipEventElapsedTime(&ms, m.events[2 * i], m.events[2 * i + 1]) != hipSuccess) {
            (void)hipGetLastError();
            ms = 0.f;
        }
        out[i].name = m.record[i].name;
        out[i].ms = ms;
        out[i].bytes = m.record[i].bytes;
        out[i].flops = m.record[i].flops;
    }
    return n < cap ? n : cap;
}

extern "C" int mynn_model_profile_step(void *state, int32_t token, int64_t past_len, mynn_kernel_time *out, int cap) {
    MYNN_REQUIRE(state && out && cap > 0, MYNN_ERR_INVALID, "profile_step: bad argument");
    Model &m = *(Model *)state;
    const mynn_model_config &c = m.cfg;
    MYNN_REQUIRE(c.batch * c.seq_q == 1, MYNN_ERR_STATE, "profile_step: needs a batch-1 decode model");
    int64_t id = token, pos = past_len;
    TRY(upload_inputs(m, &id, &pos, past_len, past_len + 1));
    return profile_enqueue(m, out, cap);
}

extern "C" int mynn_model_profile(void *state, const int64_t *input_ids, const int64_t *position_id, int64_t past_len,
                                  int64_t active_seq_kv, mynn_kernel_time *out, int cap) {
    MYNN_REQUIRE(state && input_ids && position_id && out && cap > 0, MYNN_ERR_INVALID, "profile: bad argument");
    Model &m = *(Model *)state;
    TRY(upload_inputs(m, input_ids, position_id, past_len, active_seq_kv));
    return profile_enqueue(m, out, cap);
}
