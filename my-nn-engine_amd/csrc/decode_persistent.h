// Single-launch decode step (decode_persistent.hip): one resident workgroup per CU runs the whole
// batch-1 step and the ops pass their output vectors through self-flagging hand-over buffers.
#pragma once
#include "kernels.h"

namespace mynn {

constexpr int kPdThreads = 512, kPdWaves = kPdThreads / 64;

struct PdLayer {
    const int8_t *qkv_w, *o_w, *gu_w, *down_w;  // [N, K] int8; gu = gate / up rows interleaved
    const void *qkv_s, *o_s, *gu_s, *down_s;    // per-row scales
    const void *norm1, *norm2;
    void *k_cache, *v_cache;                    // [Hkv, max_seq, D]
};

struct PdShape {
    int n_layers, H, Hq, Hkv, D, F, V, max_seq;
};

struct PdParams {
    const PdLayer *layers;  // device array
    int n_layers, H, Hq, Hkv, F, V, max_seq;
    float eps, softmax_scale;
    const int8_t *embed_w;
    const void *embed_s, *final_norm;
    const int8_t *lm_w;
    const void *lm_s, *cos_t, *sin_t;
    uint64_t *hand;   // two sets of hand-over words, all "empty" (~0) before the first step
    int set_words;    // words per set (decode_persistent_set_words)
    void *logits;
    int32_t *next;
    AdvanceState adv; // the device-side loop state the step reads and moves on
    unsigned *epoch;  // step counter: picks the set
    int *err;         // set to 1 by a wait that ran out
    int spin_limit;
    int act_floats;   // filled in by the launcher
};

bool decode_persistent_supported(const PdShape &s, int dtype, int cus);
size_t decode_persistent_set_words(const PdShape &s, int nb);
int decode_persistent_launch(PdParams p, const PdShape &s, int dtype, int nb, hipStream_t st);

}  // namespace mynn
