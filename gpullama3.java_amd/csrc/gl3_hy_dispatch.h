// gl3_hy_dispatch.h — what the generic entry points of the C-ABI do for a plan of the layer-list family.  Included by the translation
// unit that defines those entry points (gl3_api.hip, or gl3_api_lean.cpp in a build that carries only this family).
#pragma once
#include "gl3_hybrid.h"

// device_logits: compute the logits row (it stays in ctx->logits for the sampler) although no host copy is asked for
static inline int32_t hy_forward_decode(gl3_ctx* ctx, int32_t seq, int32_t token, int32_t pos, float* logits_out, int32_t* argmax_out, bool device_logits = false) {
    const int32_t w0 = 0;
    const bool want = logits_out || argmax_out || device_logits;
    int32_t r = gl3_hy_step(ctx, seq, &token, 1, pos, &w0, want ? 1 : 0, logits_out);
    if (r != GL3_OK) return r;
    return argmax_out ? gl3_hy_argmax(ctx, argmax_out) : GL3_OK;
}

static inline int32_t hy_forward_decode_sample(gl3_ctx* ctx, int32_t token, int32_t pos, float temperature, float topp, float coin, int32_t* token_out) {
    if (!token_out) GL3_FAIL(GL3_E_ARG, "null token_out");
    if (!(temperature >= 0.f)) GL3_FAIL(GL3_E_ARG, "temperature must be >= 0");
    if (temperature == 0.f) return hy_forward_decode(ctx, 0, token, pos, nullptr, token_out);
    if (!(coin >= 0.f && coin < 1.f)) GL3_FAIL(GL3_E_ARG, "coin must be in [0, 1)");
    int32_t r = hy_forward_decode(ctx, 0, token, pos, nullptr, nullptr, true);       // no host copy of the logits: the sampler reads them on the device
    if (r != GL3_OK) return r;
    return gl3_sample_run(ctx, ctx->logits, temperature, topp, coin, token_out);
}

// n sequences, one token each: the slots run one after the other (the family batches tokens of ONE sequence)
static inline int32_t hy_forward_decode_batch(gl3_ctx* ctx, const int32_t* tokens, const int32_t* seq_ids, const int32_t* positions, int32_t n, float* logits_out,
                                              int32_t* argmax_out) {
    if (n < 1 || !tokens || !seq_ids || !positions) GL3_FAIL(GL3_E_ARG, "null or empty batch");
    for (int i = 0; i < n; ++i) {
        int32_t r = hy_forward_decode(ctx, seq_ids[i], tokens[i], positions[i], logits_out ? logits_out + (size_t)i * ctx->d.vocab : nullptr,
                                      argmax_out ? argmax_out + i : nullptr);
        if (r != GL3_OK) return r;
    }
    return GL3_OK;
}
