// The decode step: Transformer.Forward (src/Transformer.cs:158-190) with
// MultiHeadAttention (:150-156) and the greedy branch of Sampler.Sample
// (src/Sampler.cs:44-47,69), issued on the library's stream.
#include "common.hpp"

#include <cmath>
#include <new>
#include <vector>

struct llama2_decoder {
    llama2_config cfg;
    std::vector<llama2_layer_weights> layers;
    llama2_transformer_weights w;
    llama2_run_state s;
    int mode;
    int kv_dim;
    int head_size;
};

using namespace l2;

namespace {

int check_qw(const llama2_qweight& q, const char* what, int layer)
{
    L2_CHECK(q.weight && q.zeros && q.scales, "llama2_decode_create: layer %d %s tensor has a null pointer", layer,
             what);
    return LLAMA2_OK;
}

#define L2_TRY(expr)          \
    do {                      \
        int rc_ = (expr);     \
        if (rc_ != LLAMA2_OK) \
            return rc_;       \
    } while (0)

// The ten module calls per layer, in the reference's order and with the
// reference's argument derivations (file:line beside each call).
int forward_modules(llama2_decoder* d, int position, int next_position)
{
    const llama2_config& c = d->cfg;
    const llama2_run_state& s = d->s;
    const int dim = c.dim, hidden = c.hidden_dim, hs = d->head_size, kv = d->kv_dim;
    const float scale = 1.0f / sqrtf(static_cast<float>(hs)); // Transformer.cs:161
    const int ss = ceil_div(dim, 128), ws = ceil_div(dim, 32) * 4, zs = ceil_div(ss, 8);
    const int hss = ceil_div(hidden, 128), hws = ceil_div(hidden, 32) * 4, hzs = ceil_div(hss, 8);

    L2_TRY(llama2_embedding(s.x, d->w.token_embedding_table, dim, s.tokens, position)); // :163
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = d->layers[i];
        L2_TRY(llama2_rmsnorm(s.xb, s.x, L.rms_attention, dim, 1e-5f)); // :167
        const size_t layer_offset = static_cast<size_t>(i) * c.seq_len * kv; // :169
        const size_t row = layer_offset + static_cast<size_t>(position) * kv; // QKVMatVec.cs:25
        L2_TRY(llama2_qkv_mat_vec(s.q, s.key_cache + row, s.value_cache + row, s.xb, L.query.weight, L.query.zeros,
                                  L.query.scales, L.key.weight, L.key.zeros, L.key.scales, L.value.weight,
                                  L.value.zeros, L.value.scales, dim, dim, zs, ss, ws)); // :171
        L2_TRY(llama2_rope(s.q, s.key_cache + row, c.n_kv_heads, hs, position, c.rope_theta, c.n_heads)); // :173
        const int seq = next_position; // :175
        L2_TRY(llama2_mat_vec_strided(s.attention, s.q, s.key_cache + layer_offset, hs, seq, hs, hs, dim, seq, scale,
                                      c.n_heads)); // :153, MatVecStrided.cs:18
        L2_TRY(llama2_softmax(s.attention, seq, c.n_heads)); // :154
        L2_TRY(llama2_vec_mat(s.xb, s.attention, s.value_cache + layer_offset, hs, seq, hs, hs, dim,
                              c.n_heads)); // :155, VecMat.cs:19
        L2_TRY(llama2_mat_vec_residual_int4(s.x, s.xb, L.output.weight, L.output.zeros, L.output.scales, dim, dim, zs,
                                            ss, ws)); // :177
        L2_TRY(llama2_rmsnorm(s.xb, s.x, L.rms_feed_forward, dim, 1e-5f)); // :179
        L2_TRY(llama2_mat_vec_swiglu(s.h, s.xb, L.gate.weight, L.gate.zeros, L.gate.scales, L.up.weight, L.up.zeros,
                                     L.up.scales, dim, hidden, zs, ss, ws)); // :181
        L2_TRY(llama2_mat_vec_residual_int4(s.x, s.h, L.down.weight, L.down.zeros, L.down.scales, hidden, dim, hzs,
                                            hss, hws)); // :183
    }
    L2_TRY(llama2_rmsnorm(s.x, s.x, d->w.rms_final_weight, dim, 1e-5f)); // :187
    L2_TRY(llama2_mat_vec(s.logits, s.x, d->w.classifier_weights, dim, c.vocab_size)); // :189
    return LLAMA2_OK;
}

} // namespace

extern "C" {

int llama2_decode_create(llama2_decoder** decoder, const llama2_config* config,
                         const llama2_transformer_weights* weights, const llama2_run_state* state, int mode)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_decode_create";
    L2_CHECK(decoder && config && weights && state, "%s: null argument", fn);
    *decoder = nullptr;
    const llama2_config& c = *config;
    L2_CHECK(c.dim > 0 && c.hidden_dim > 0 && c.n_layers > 0 && c.n_heads > 0 && c.n_kv_heads > 0 &&
                 c.vocab_size > 0 && c.seq_len > 0,
             "%s: non-positive field in config", fn);
    L2_CHECK(c.dim % c.n_heads == 0, "%s: dim=%d is not a multiple of n_heads=%d", fn, c.dim, c.n_heads);
    L2_CHECK(c.rope_theta == 10000.0f, "%s: Invalid model config (rope_theta=%g, expected 10000)", fn,
             static_cast<double>(c.rope_theta)); // src/Config.cs:27-28
    const int kv_dim = c.dim * c.n_kv_heads / c.n_heads;
    if (kv_dim != c.dim) // src/Transformer.cs:53-56
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: Differing kvDim dimention not currently supported (kv_dim=%d, dim=%d)",
                    fn, kv_dim, c.dim);
    if (c.seq_len > LLAMA2_MAX_SOFTMAX_SIZE)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: seq_len=%d exceeds the softmax limit %d", fn, c.seq_len,
                    LLAMA2_MAX_SOFTMAX_SIZE);
    L2_CHECK(mode == LLAMA2_DECODE_MODULES, "%s: unknown mode %d", fn, mode);
    L2_CHECK(weights->token_embedding_table && weights->classifier_weights && weights->rms_final_weight &&
                 weights->layers,
             "%s: null pointer in weights", fn);
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = weights->layers[i];
        L2_TRY(check_qw(L.query, "query", i));
        L2_TRY(check_qw(L.key, "key", i));
        L2_TRY(check_qw(L.value, "value", i));
        L2_TRY(check_qw(L.output, "output", i));
        L2_TRY(check_qw(L.gate, "gate", i));
        L2_TRY(check_qw(L.up, "up", i));
        L2_TRY(check_qw(L.down, "down", i));
        L2_CHECK(L.rms_attention && L.rms_feed_forward, "%s: layer %d has a null rmsnorm weight", fn, i);
    }
    L2_CHECK(state->x && state->xb && state->h && state->q && state->attention && state->logits &&
                 state->key_cache && state->value_cache && state->tokens,
             "%s: null pointer in run state", fn);
    llama2_decoder* d = new (std::nothrow) llama2_decoder();
    L2_CHECK(d, "%s: out of host memory", fn);
    d->cfg = c;
    d->layers.assign(weights->layers, weights->layers + c.n_layers);
    d->w = *weights;
    d->w.layers = d->layers.data();
    d->s = *state;
    d->mode = mode;
    d->kv_dim = kv_dim;
    d->head_size = c.dim / c.n_heads;
    *decoder = d;
    return LLAMA2_OK;
}

int llama2_decode_forward(llama2_decoder* d, int position, int next_position)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_forward: null decoder");
    L2_CHECK(position >= 0 && position < d->cfg.seq_len, "llama2_decode_forward: position=%d outside [0,%d)",
             position, d->cfg.seq_len);
    L2_CHECK(next_position == position + 1, "llama2_decode_forward: next_position=%d must be position+1=%d",
             next_position, position + 1);
    return forward_modules(d, position, next_position);
}

int llama2_decode_sample(llama2_decoder* d, int next_position, int generate_token, int* token)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d && token, "llama2_decode_sample: null argument");
    L2_CHECK(next_position >= 0 && next_position <= d->cfg.seq_len, "llama2_decode_sample: next_position=%d",
             next_position);
    L2_TRY(llama2_argmax(d->s.logits, d->cfg.vocab_size, d->s.tokens, next_position, generate_token));
    return llama2_memcpy_d2h(token, d->s.tokens, static_cast<size_t>(next_position) * sizeof(int), sizeof(int));
}

int llama2_decode_run(llama2_decoder* d, int position, int steps, int n_prompt)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_run: null decoder");
    L2_CHECK(position >= 0 && steps >= 0 && position + steps <= d->cfg.seq_len,
             "llama2_decode_run: position=%d steps=%d exceed seq_len=%d", position, steps, d->cfg.seq_len);
    for (int pos = position; pos < position + steps; ++pos) {
        L2_TRY(forward_modules(d, pos, pos + 1));
        L2_TRY(llama2_argmax(d->s.logits, d->cfg.vocab_size, d->s.tokens, pos + 1, pos + 1 >= n_prompt));
    }
    return LLAMA2_OK;
}

int llama2_decode_destroy(llama2_decoder* d)
{
    if (!d)
        return LLAMA2_OK;
    if (ctx().ready)
        L2_HIP(hipStreamSynchronize(ctx().stream));
    delete d;
    return LLAMA2_OK;
}

} // extern "C"
