// gl3_api_lean.cpp — the generic entry points of the C-ABI for a build that carries only the layer-list family (libgpullama_lean.so:
// gl3_hybrid.hip, gl3_modeldir.cpp, gl3_sample.hip).  The whole library defines the same symbols in gl3_api.hip, where they also serve
// the GGUF families; a host links against either.
#include <string>

#include "gl3_hy_dispatch.h"

static std::string g_create_err;
void gl3_set_create_error(const char* msg) { g_create_err = msg ? msg : ""; }
int32_t gl3_tp_check(gl3_ctx*) { return GL3_OK; }          // no tensor-parallel transport in this build

#define LEAN_CTX(c) do { if (!(c)) return GL3_E_ARG; if (!(c)->hy) return GL3_E_UNSUPPORTED; } while (0)

extern "C" {

const char* gl3_version(void) { return "gpullama3-hip (layer-list family only)"; }
const char* gl3_last_error(gl3_ctx* ctx) { return ctx ? ctx->err.c_str() : g_create_err.c_str(); }

int32_t gl3_create(const gl3_model_desc* desc, gl3_ctx** out) {
    if (!desc || !out) { g_create_err = "null argument"; return GL3_E_ARG; }
    if (desc->struct_size != sizeof(gl3_model_desc)) { g_create_err = "gl3_model_desc.struct_size mismatch"; return GL3_E_ARG; }
    if (desc->arch != GL3_ARCH_NODITAR) { g_create_err = "this build carries the layer-list family only"; return GL3_E_UNSUPPORTED; }
    return gl3_hy_create(desc, out, g_create_err);
}

void gl3_destroy(gl3_ctx* ctx) {
    if (!ctx) return;
    hipSetDevice(ctx->d.device);
    if (ctx->stream) hipStreamSynchronize(ctx->stream);
    gl3_hy_destroy(ctx);
    gl3_sample_free(ctx);
    if (ctx->argmax) hipFree(ctx->argmax);
    if (ctx->h_logits) hipHostFree(ctx->h_logits);
    if (ctx->h_argmax) hipHostFree(ctx->h_argmax);
    if (ctx->h_dyn) hipHostFree(ctx->h_dyn);
    if (ctx->stream) hipStreamDestroy(ctx->stream);
    delete ctx;
}

int32_t gl3_upload_tensor(gl3_ctx* ctx, int32_t id, int32_t layer, const void* host, uint64_t bytes, int32_t type) {
    LEAN_CTX(ctx);
    if (ctx->finalized) GL3_FAIL(GL3_E_STATE, "upload after finalize");
    return gl3_hy_upload(ctx, id, layer, host, bytes, type);
}
int32_t gl3_finalize(gl3_ctx* ctx) { LEAN_CTX(ctx); return ctx->finalized ? GL3_OK : gl3_hy_finalize(ctx); }
int32_t gl3_forward_decode(gl3_ctx* ctx, int32_t token, int32_t pos, float* logits_out, int32_t* argmax_out) {
    LEAN_CTX(ctx);
    return hy_forward_decode(ctx, 0, token, pos, logits_out, argmax_out);
}
int32_t gl3_forward_decode_sample(gl3_ctx* ctx, int32_t token, int32_t pos, float temperature, float topp, float coin, int32_t* token_out) {
    LEAN_CTX(ctx);
    return hy_forward_decode_sample(ctx, token, pos, temperature, topp, coin, token_out);
}
int32_t gl3_forward_prefill_seq(gl3_ctx* ctx, int32_t seq, const int32_t* tokens, int32_t n, int32_t start_pos) {
    LEAN_CTX(ctx);
    return n == 0 ? GL3_OK : gl3_hy_step(ctx, seq, tokens, n, start_pos, nullptr, 0, nullptr);
}
int32_t gl3_forward_prefill(gl3_ctx* ctx, const int32_t* tokens, int32_t n, int32_t start_pos) { return gl3_forward_prefill_seq(ctx, 0, tokens, n, start_pos); }
int32_t gl3_forward_decode_batch(gl3_ctx* ctx, const int32_t* tokens, const int32_t* seq_ids, const int32_t* positions, int32_t n, float* logits_out,
                                 int32_t* argmax_out) {
    LEAN_CTX(ctx);
    return hy_forward_decode_batch(ctx, tokens, seq_ids, positions, n, logits_out, argmax_out);
}
int32_t gl3_forward_step(gl3_ctx* ctx, int32_t seq, const int32_t* tokens, int32_t n, int32_t start_pos, const int32_t* want, int32_t n_want, float* logits_out) {
    LEAN_CTX(ctx);
    return gl3_hy_step(ctx, seq, tokens, n, start_pos, want, n_want, logits_out);
}
int32_t gl3_seq_acquire(gl3_ctx* ctx, int32_t* seq_out) { LEAN_CTX(ctx); return seq_out ? gl3_hy_seq_acquire(ctx, seq_out) : GL3_E_ARG; }
int32_t gl3_seq_release(gl3_ctx* ctx, int32_t seq) { LEAN_CTX(ctx); return gl3_hy_seq_release(ctx, seq); }
int32_t gl3_get_layer_rows(gl3_ctx* ctx, int32_t layer, float* out, int32_t n) { LEAN_CTX(ctx); return gl3_hy_layer_rows(ctx, layer, out, n); }
int32_t gl3_reset_kv(gl3_ctx* ctx) { LEAN_CTX(ctx); return gl3_hy_reset(ctx); }
int32_t gl3_get_sample_probs(gl3_ctx* ctx, float* out) { LEAN_CTX(ctx); return out ? gl3_sample_probs(ctx, out) : GL3_E_ARG; }
int32_t gl3_get_model_desc(gl3_ctx* ctx, gl3_model_desc* desc) {
    if (!ctx || !desc) return GL3_E_ARG;
    *desc = ctx->d;
    desc->layer_descs = nullptr;
    desc->n_seqs = ctx->n_seqs;
    return GL3_OK;
}
int32_t gl3_load_gguf(const char*, const gl3_model_desc*, gl3_ctx**) {
    g_create_err = "this build carries the layer-list family only: GGUF models need the whole library (make -C gpullama3.java_amd/csrc)";
    return GL3_E_UNSUPPORTED;
}
int32_t gl3_profile_hybrid_gemm(int32_t device, int32_t f32, int32_t rows, int32_t k, int32_t m, int32_t glu, int32_t iters, double* out_us) {
    return gl3_hy_profile_gemm(device, f32, rows, k, m, glu, iters, out_us);
}

}  // extern "C"
