// Host side of crates/llm: the greedy generate loop of LlmSession (session.rs:311-537), the
// per-output-channel int8 weight quantiser (quantize.rs:124-169) and the RoPE tables
// (builder.rs:359-393).  Plain C++; nothing here touches the device except through the model ABI.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

#include "mynn_common.h"

using namespace mynn;

// ---- storage conversions on the host ----------------------------------------------------------
static inline void store_host(void *p, size_t i, float v, int dt) {
    switch (dt) {
    case MYNN_BF16: ((uint16_t *)p)[i] = f32_to_bf16_bits(v); break;
    case MYNN_F16: ((f16_t *)p)[i] = (f16_t)v; break;
    default: ((float *)p)[i] = v; break;
    }
}

extern "C" int mynn_quantize_per_channel(int8_t *q, void *scale, const float *w, size_t rows, size_t cols,
                                         int scale_dtype) {
    MYNN_REQUIRE(q && scale && w && rows > 0 && cols > 0, MYNN_ERR_INVALID, "quantize_per_channel: bad operand");
    MYNN_REQUIRE(dtype_ok(scale_dtype), MYNN_ERR_INVALID, "quantize_per_channel: dtype %d", scale_dtype);
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)rows; r++) {
        const float *row = w + (size_t)r * cols;
        float amax = 0.f;
        for (size_t c = 0; c < cols; c++) amax = fmaxf(amax, fabsf(row[c]));
        const float s = amax == 0.f ? 1.0f : amax / 127.0f;
        for (size_t c = 0; c < cols; c++) {
            float v = roundf(row[c] / s);  // half away from zero, like f32::round
            v = v < -128.f ? -128.f : (v > 127.f ? 127.f : v);
            q[(size_t)r * cols + c] = (int8_t)v;
        }
        store_host(scale, (size_t)r, s, scale_dtype);
    }
    return 0;
}

extern "C" int mynn_rope_table(void *cos_t, void *sin_t, int max_seq, int head_dim, float base, int dtype) {
    MYNN_REQUIRE(cos_t && sin_t && max_seq > 0 && head_dim > 0 && head_dim % 2 == 0, MYNN_ERR_INVALID,
                 "rope_table: bad operand");
    MYNN_REQUIRE(dtype_ok(dtype), MYNN_ERR_INVALID, "rope_table: dtype %d", dtype);
    const int half = head_dim / 2;
    std::vector<double> inv(half);
    for (int i = 0; i < half; i++) inv[i] = 1.0 / pow((double)base, 2.0 * i / head_dim);
    for (int p = 0; p < max_seq; p++)
        for (int j = 0; j < head_dim; j++) {
            const double ang = (double)p * inv[j % half];
            const float c = (float)cos(ang), s = (float)sin(ang);
            const size_t idx = (size_t)p * head_dim + j;
            if (dtype == MYNN_BF16) {
                // the reference narrows f64 initializers to bf16 by dropping the low 16 bits of the
                // f32 (src/session.rs:171-175), not by rounding
                ((uint16_t *)cos_t)[idx] = (uint16_t)(__builtin_bit_cast(uint32_t, c) >> 16);
                ((uint16_t *)sin_t)[idx] = (uint16_t)(__builtin_bit_cast(uint32_t, s) >> 16);
            } else {
                store_host(cos_t, idx, c, dtype);
                store_host(sin_t, idx, s, dtype);
            }
        }
    return 0;
}

// ---- LlmSession -------------------------------------------------------------------------------
struct mynn_llm {
    void *decode = nullptr, *prefill = nullptr;
    int prefill_len = 0, max_seq = 0;
    int64_t eos = -1, past_len = 0;
    mynn_step_fn step = nullptr;
    void *user = nullptr;
    int last_error = 0;
    bool streaming = false;  // DecodeKind::LlamaStreaming { sink, window }
    int sink = 0, window = 0;
};

// streaming_kv_position (session.rs:604-635): the recency rank of every cache slot -- sink slots keep their position,
// ring slots are walked in age order from ring_start, slots not written yet keep their own index
static void streaming_kv_position(std::vector<int64_t> &out, int64_t sink, int64_t window, int64_t stream_pos) {
    const int64_t max_active = sink + window;
    const int64_t ring_start = stream_pos < max_active ? 0 : (stream_pos - sink) % window;
    const int64_t in_ring = std::min<int64_t>(std::max<int64_t>(stream_pos - sink, 0), window);
    for (int64_t slot = 0; slot < (int64_t)out.size(); slot++) {
        int64_t v = slot;
        if (slot >= sink && slot < max_active) {
            const int64_t rel_age = (slot - sink + window - ring_start) % window;
            if (rel_age < in_ring) v = sink + rel_age;
        }
        out[slot] = v;
    }
}

extern "C" int mynn_llm_set_streaming(mynn_llm *l, int sink, int window) {
    MYNN_REQUIRE(l && !l->step, MYNN_ERR_INVALID, "llm_set_streaming: needs a Llama session");
    MYNN_REQUIRE(sink >= 0 && window > 0 && sink + window <= l->max_seq, MYNN_ERR_INVALID,
                 "llm_set_streaming: sink %d + window %d must fit max_seq %d, window > 0", sink, window, l->max_seq);
    MYNN_REQUIRE(!l->prefill || l->prefill_len <= window, MYNN_ERR_INVALID,
                 "llm_set_streaming: prefill_len (%d) must be <= window (%d) in streaming KV mode", l->prefill_len, window);
    l->streaming = true;
    l->sink = sink;
    l->window = window;
    return 0;
}

extern "C" mynn_llm *mynn_llm_create(void *decode_state, void *prefill_state, int prefill_len, int max_seq,
                                     int64_t eos_token_id) {
    if (!decode_state || max_seq <= 0 || (prefill_state && prefill_len <= 0)) {
        fail(MYNN_ERR_INVALID, "llm_create: bad argument");
        return nullptr;
    }
    mynn_llm *l = new mynn_llm;
    l->decode = decode_state;
    l->prefill = prefill_state;
    l->prefill_len = prefill_state ? prefill_len : 0;
    l->max_seq = max_seq;
    l->eos = eos_token_id;
    return l;
}
extern "C" mynn_llm *mynn_llm_create_with_step(mynn_step_fn step, void *user, int max_seq, int64_t eos_token_id) {
    if (!step || max_seq <= 0) {
        fail(MYNN_ERR_INVALID, "llm_create_with_step: bad argument");
        return nullptr;
    }
    mynn_llm *l = new mynn_llm;
    l->step = step;
    l->user = user;
    l->max_seq = max_seq;
    l->eos = eos_token_id;
    return l;
}
extern "C" void mynn_llm_destroy(mynn_llm *l) { delete l; }
// reset (session.rs:303-305): past_len = 0; a paged cache also gives its pages back to the pool (the prefill model shares
// the decode model's page set)
extern "C" void mynn_llm_reset(mynn_llm *l) {
    if (!l) return;
    l->past_len = 0;
    if (l->decode) (void)mynn_model_release_kv_pages(l->decode);
}
extern "C" int64_t mynn_llm_past_len(const mynn_llm *l) { return l ? l->past_len : -1; }
extern "C" void mynn_llm_set_past_len(mynn_llm *l, int64_t p) { if (l) l->past_len = p < 0 ? 0 : p; }

// decode_step (session.rs:508-537): inputs [token, position = past_len, past_len, active = past_len + 1]
static int decode_step(mynn_llm *l, int64_t token, int64_t *next) {
    if (l->step) {
        *next = l->step(l->user, token, l->past_len);
    } else {
        int32_t t = 0;
        int64_t pos = l->past_len;
        int rc;
        if (l->streaming) {
            // streaming_decode_inputs (session.rs:571-597): past_len is the unbounded stream position
            const int64_t max_active = l->sink + l->window, sp = l->past_len;
            pos = std::min(sp, max_active - 1);
            const int64_t ring_start = sp < max_active ? 0 : (sp - l->sink) % l->window;
            std::vector<int64_t> kvpos((size_t)l->max_seq);
            streaming_kv_position(kvpos, l->sink, l->window, sp);
            rc = mynn_model_step_streaming(l->decode, &token, &pos, sp, std::min(sp + 1, max_active), l->sink, l->window, ring_start,
                                           kvpos.data(), &t, nullptr);
        } else {
            rc = mynn_model_step(l->decode, &token, &pos, l->past_len, l->past_len + 1, &t, nullptr);
        }
        if (rc) return rc;
        *next = t;
    }
    l->past_len += 1;
    return 0;
}

// run_prefill_rec (session.rs:426-485): fixed-size chunks, the last one zero-padded; pad rows are
// overwritten by later tokens and hidden by the causal bound
static int run_prefill(mynn_llm *l, const int64_t *ids, size_t n, int64_t *next) {
    const size_t P = (size_t)l->prefill_len;
    std::vector<int64_t> padded(P), pos(P);
    while (n > 0) {
        const size_t chunk = n < P ? n : P;
        for (size_t i = 0; i < P; i++) {
            padded[i] = i < chunk ? ids[i] : 0;
            pos[i] = l->past_len + (int64_t)i;
        }
        int32_t t = 0;
        // the token wanted is that of row chunk-1; the model reports the last row, so the final
        // (possibly padded) chunk reads its logits back
        const bool last = chunk == n;
        const bool pick_row = last && chunk < P;
        int rc;
        if (l->streaming) {
            // streaming_prefill_inputs (session.rs:539-569)
            const int64_t max_active = l->sink + l->window, sp = l->past_len, after = sp + (int64_t)P;
            for (size_t i = 0; i < P; i++) pos[i] = std::min(sp + (int64_t)i, max_active - 1);
            const int64_t ring_start = after <= max_active ? 0 : (after - l->sink) % l->window;
            std::vector<int64_t> kvpos((size_t)l->max_seq);
            streaming_kv_position(kvpos, l->sink, l->window, after);
            rc = mynn_model_step_streaming(l->prefill, padded.data(), pos.data(), sp, std::min(after, max_active), l->sink, l->window,
                                           ring_start, kvpos.data(), pick_row ? nullptr : &t, nullptr);
        } else {
            rc = mynn_model_step(l->prefill, padded.data(), pos.data(), l->past_len, l->past_len + (int64_t)P, pick_row ? nullptr : &t,
                                 nullptr);
        }
        if (rc) return rc;
        if (pick_row) {
            // argmax of row chunk-1 on the device, from the device logits
            rc = mynn_model_argmax_row(l->prefill, (int)(chunk - 1), &t);
            if (rc) return rc;
        }
        l->past_len += (int64_t)chunk;
        if (last) *next = t;
        ids += chunk;
        n -= chunk;
    }
    return 0;
}

extern "C" int mynn_llm_generate_ids(mynn_llm *l, const int64_t *prompt_ids, size_t n_prompt, size_t max_new_tokens,
                                     int64_t *out) {
    MYNN_REQUIRE(l && (prompt_ids || n_prompt == 0) && (out || max_new_tokens == 0), MYNN_ERR_INVALID,
                 "llm_generate_ids: null argument");
    if (n_prompt == 0) return 0;
    const bool prefill_runs = l->prefill != nullptr;
    const int64_t needed = prefill_runs
        ? l->past_len + (int64_t)((n_prompt + l->prefill_len - 1) / l->prefill_len * l->prefill_len)
        : l->past_len + (int64_t)n_prompt;
    MYNN_REQUIRE(l->streaming || l->max_seq >= needed, MYNN_ERR_TOO_LONG, "prompt needs %lld cache rows, max_seq_len is %d (past_len %lld)",
                 (long long)needed, l->max_seq, (long long)l->past_len);
    int n_new = 0;
    // the executor's device-resident loop (mynn_model_decode_loop) serves runs of decode steps without a host round
    // trip per token; with an end-of-sequence id the runs are short, and what a run computed past that id is dropped
    // (its cache rows lie beyond past_len, where the next turn overwrites them)
    bool loop_ok = !l->step && !l->streaming && l->decode != nullptr;
    std::vector<int32_t> run;
    for (size_t i = 0; i < max_new_tokens;) {
        if (!l->streaming && l->max_seq < l->past_len + 1) break;
        int64_t tok = 0;
        int rc;
        if (i == 0) {
            if (prefill_runs) rc = run_prefill(l, prompt_ids, n_prompt, &tok);
            else {
                rc = 0;
                for (size_t j = 0; j < n_prompt && rc == 0; j++) rc = decode_step(l, prompt_ids[j], &tok);
            }
        } else {
            const int64_t room = l->max_seq - l->past_len;
            const size_t want = std::min<size_t>(std::min<size_t>(max_new_tokens - i, l->eos >= 0 ? 32 : 256), (size_t)room);
            if (loop_ok && want >= 4) {
                run.resize(want);
                if (mynn_model_decode_loop(l->decode, out[n_new - 1], l->past_len, (int)want, run.data()) == 0) {
                    size_t used = 0;
                    while (used < want) {
                        out[n_new++] = run[used++];
                        if (out[n_new - 1] == l->eos) break;
                    }
                    l->past_len += (int64_t)used;
                    i += used;
                    if (out[n_new - 1] == l->eos) break;
                    continue;
                }
                loop_ok = false;  // (a model without the loop, or no pages for the whole run: step by step from here)
            }
            rc = decode_step(l, out[n_new - 1], &tok);
        }
        if (rc) return rc > 0 ? -1000 - rc : rc;
        out[n_new++] = tok;
        i++;
        if (tok == l->eos) break;
    }
    return n_new;
}
