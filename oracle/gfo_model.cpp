// CPU oracle (test infrastructure only, see gfo.h): a Gemma-3 shaped decoder stack run
// for a few contiguous rows against an fp16 KV ring, composed from the scalar operators.
//
// Follows:
//   src/engine/gemma_target_runtime.cpp:13-221   op order of one block:
//       u = rms(x, attn_norm); q,k,v = W u; q = headrms(q), k = headrms(k);
//       q = rope(q); K = f16(rope(k)); V = f16(v); a = attention(q, K, V);
//       x1 = x + rms(Wo a, post_attention_norm); u2 = rms(x1, ffn_norm);
//       h = gelu(Wg u2) * (Wu u2); x = x1 + rms(Wd h, post_ffw_norm); final rms(x, output_norm)
//   src/engine/gemma3_draft.mm:888-972           the drafter runs the same order
//   src/engine/gemma_target_runtime.cpp:238-271  per-layer attention schedule of contiguous rows
//   src/engine/model.cpp:599-619                 embedding scale sqrt(hidden); local/global policy
#include "gfo.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

extern "C" void gfo_forward_rows(const gfo_model_config* cfg, const gfo_layer* layers,
                                 int embed_dtype, const uint8_t* embed_w, const float* out_norm,
                                 const uint32_t* tokens, uint32_t rows, uint32_t position,
                                 uint16_t* priv_k, uint16_t* priv_v, float* out_hidden,
                                 uint32_t threads) {
    const uint32_t H = cfg->hidden, F = cfg->ffn, QW = cfg->q_heads * cfg->head_dim,
                   KW = cfg->kv_heads * cfg->head_dim;
    std::vector<float> x(size_t(rows) * H), u(size_t(rows) * H), q(size_t(rows) * QW),
        k(size_t(rows) * KW), v(size_t(rows) * KW), a(size_t(rows) * QW), o(size_t(rows) * H),
        x1(size_t(rows) * H), g(size_t(rows) * F), up(size_t(rows) * F), h(size_t(rows) * F);
    std::vector<uint32_t> positions(rows), ancestors(rows), schedule(size_t(rows) * 4);
    for (uint32_t r = 0; r < rows; ++r) { positions[r] = position + r; ancestors[r] = r; }

    gfo_embed(embed_dtype, embed_w, tokens, x.data(), rows, H, std::sqrt(static_cast<float>(H)));
    const float attn_scale = 1.0f / std::sqrt(static_cast<float>(cfg->head_dim));

    for (uint32_t l = 0; l < cfg->layers; ++l) {
        const gfo_layer& L = layers[l];
        const bool local = cfg->global_period > 1 && (l % cfg->global_period) != cfg->global_period - 1;
        const float base = local ? cfg->local_base : cfg->global_base;
        const float scale = local ? 1.0f : cfg->global_scale;
        const uint32_t ring_mask = (local ? cfg->ring_local : cfg->ring_global) - 1;
        uint16_t* pk = priv_k + size_t(l) * rows * KW;
        uint16_t* pv = priv_v + size_t(l) * rows * KW;

        gfo_rms_norm(x.data(), L.norm[0], u.data(), rows, H, cfg->eps);
        gfo_gemv_mt(L.dtype[0], L.w[0], u.data(), q.data(), rows, H, QW, threads);
        gfo_gemv_mt(L.dtype[1], L.w[1], u.data(), k.data(), rows, H, KW, threads);
        gfo_gemv_mt(L.dtype[2], L.w[2], u.data(), v.data(), rows, H, KW, threads);
        gfo_head_rms_norm(q.data(), L.norm[1], q.data(), rows, cfg->q_heads, cfg->head_dim, cfg->eps);
        gfo_head_rms_norm(k.data(), L.norm[2], k.data(), rows, cfg->kv_heads, cfg->head_dim, cfg->eps);
        gfo_rope_neox(q.data(), q.data(), positions.data(), rows, cfg->q_heads, cfg->head_dim,
                      cfg->head_dim, base, scale);
        gfo_kv_store_f16(k.data(), v.data(), positions.data(), pk, pv, rows, cfg->kv_heads,
                         cfg->head_dim, cfg->head_dim, base, scale);
        for (uint32_t r = 0; r < rows; ++r) {
            const uint32_t window_start = local && positions[r] >= cfg->sliding_window
                ? positions[r] + 1 - cfg->sliding_window : 0;
            const uint32_t base_start = std::min(position, window_start);
            const uint32_t private_start = window_start > position ? window_start - position : 0;
            schedule[4 * r + 0] = base_start;
            schedule[4 * r + 1] = position - base_start;
            schedule[4 * r + 2] = private_start;
            schedule[4 * r + 3] = r + 1 - private_start;
        }
        gfo_attention(q.data(), L.ring_k, L.ring_v, pk, pv, schedule.data(), ancestors.data(),
                      a.data(), rows, ring_mask, cfg->q_heads, cfg->kv_heads, cfg->head_dim, attn_scale);
        gfo_gemv_mt(L.dtype[3], L.w[3], a.data(), o.data(), rows, QW, H, threads);
        gfo_rms_norm_add(o.data(), L.norm[3], x.data(), x1.data(), rows, H, cfg->eps);
        gfo_rms_norm(x1.data(), L.norm[4], u.data(), rows, H, cfg->eps);
        gfo_gemv_mt(L.dtype[4], L.w[4], u.data(), g.data(), rows, H, F, threads);
        gfo_gemv_mt(L.dtype[5], L.w[5], u.data(), up.data(), rows, H, F, threads);
        gfo_geglu(g.data(), up.data(), h.data(), uint64_t(rows) * F);
        gfo_gemv_mt(L.dtype[6], L.w[6], h.data(), o.data(), rows, F, H, threads);
        gfo_rms_norm_add(o.data(), L.norm[5], x1.data(), x.data(), rows, H, cfg->eps);
    }
    gfo_rms_norm(x.data(), out_norm, out_hidden, rows, H, cfg->eps);
}
