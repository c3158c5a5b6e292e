// Runs the C++ host mirror (hgemm / hgemm_trans / attention / rope / sampling entry points, the model-level TextModel /
// KVCache / VisionModel drop-ins and their error behaviour) on the GPU and checks the results against the oracle library
// loaded beside it, or, for the model-level types, against the session entry points that the Python suite holds to the oracle.  Exit code 0 = all checks passed.
// Usage: host_mirror_check   (needs libmoonhip.so and libmoon_oracle.so on the link path; see test_gpu_cxx_mirror.py)
#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "moon_oracle.h"
#include "moonhip.hpp"

using moon::f16;
using moon::Tensor;

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float frand() { // xorshift, uniform in [-1, 1)
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (float)((rng_state >> 40) & 0xFFFFFF) / 8388608.0f - 1.0f;
}
static void fill(Tensor<f16> &t, float scale) {
    std::vector<float> tmp(t.data.size());
    for (auto &x : tmp) x = frand() * scale;
    orc_cast_f32_to_f16(tmp.data(), t.data.data(), tmp.size());
}
static double rel_fro(const std::vector<f16> &a, const std::vector<f16> &b) {
    std::vector<float> fa(a.size()), fb(b.size());
    orc_cast_f16_to_f32(a.data(), fa.data(), a.size());
    orc_cast_f16_to_f32(b.data(), fb.data(), b.size());
    double num = 0, den = 0;
    for (size_t i = 0; i < fa.size(); ++i) {
        double d = (double)fa[i] - fb[i];
        num += d * d;
        den += (double)fb[i] * fb[i];
    }
    return std::sqrt(num / (den > 0 ? den : 1));
}
static int failures = 0;
static void expect(bool ok, const char *what, double v = 0) {
    std::printf("%s %s (%.3g)\n", ok ? "ok  " : "FAIL", what, v);
    std::fflush(stdout);
    if (!ok) ++failures;
}

int main() {
    const double TOL = 1e-3; // relative Frobenius error against the f32-accumulated oracle
    {
        Tensor<f16> a({37, 200}), b({200, 91}), ref({37, 91});
        fill(a, 1.0f), fill(b, 0.1f);
        auto c = moon::hgemm::matmul(a, b);
        orc_hgemm_nn(a.data.data(), b.data.data(), ref.data.data(), 37, 91, 200);
        double e = rel_fro(c.data, ref.data);
        expect(e <= TOL, "hgemm.matmul 37x200x91", e);
    }
    for (size_t M : {size_t(1), size_t(5)}) {
        Tensor<f16> a({M, 2048}), bt({300, 2048}), ref({M, 300});
        fill(a, 1.0f), fill(bt, 0.05f);
        auto c = moon::hgemm_trans::matmul(a, bt);
        orc_hgemm_nt(a.data.data(), bt.data.data(), ref.data.data(), M, 300, 2048);
        double e = rel_fro(c.data, ref.data);
        expect(e <= TOL, M == 1 ? "hgemm_trans.matmul vector path" : "hgemm_trans.matmul M=5", e);
    }
    {
        const size_t H = 32, D = 64, q_len = 9, pos = 4, kv = pos + q_len;
        Tensor<f16> q({H, q_len, D}), k({H, kv, D}), v({H, kv, D}), ref({H, q_len, D});
        fill(q, 1.0f), fill(k, 1.0f), fill(v, 1.0f);
        auto mask = moon::attention::createAttentionMask(pos, q_len);
        auto o = moon::attention::multiMaskedSDPA(q, k, v, mask, H, D);
        orc_sdpa_multi(q.data.data(), k.data.data(), v.data.data(), mask.data.data(), kv, ref.data.data(), H, q_len, kv, D);
        double e = rel_fro(o.data, ref.data);
        expect(e <= TOL, "attention.multiMaskedSDPA causal with past", e);
        auto o2 = moon::attention::multiMasklessSDPA(H, D, q, k, v);
        orc_sdpa_multi(q.data.data(), k.data.data(), v.data.data(), nullptr, 0, ref.data.data(), H, q_len, kv, D);
        e = rel_fro(o2.data, ref.data);
        expect(e <= TOL, "attention.multiMasklessSDPA", e);
    }
    {
        const size_t H = 32, D = 64, kv = 300;
        Tensor<f16> q({H, 1, D}), k({H, kv, D}), v({H, kv, D}), ref({H, 1, D});
        fill(q, 1.0f), fill(k, 1.0f), fill(v, 1.0f);
        auto mask = moon::attention::createAttentionMask(kv - 1, 1);
        auto o = moon::attention::singleMaskedSDPA(q, k, v, mask);
        orc_sdpa_multi(q.data.data(), k.data.data(), v.data.data(), mask.data.data(), kv, ref.data.data(), H, 1, kv, D);
        double e = rel_fro(o.data, ref.data);
        expect(e <= TOL, "attention.singleMaskedSDPA", e);
    }
    // error behaviour: the reference's error names
    try {
        Tensor<f16> a({4, 8}), b({9, 4});
        moon::hgemm::matmul(a, b);
        expect(false, "hgemm.matmul inner-dimension mismatch must throw");
    } catch (const moon::IncompatibleTensorShapes &) { expect(true, "IncompatibleTensorShapes"); }
    try {
        Tensor<f16> a({4, 8, 2}), b({8, 4});
        moon::hgemm_trans::matmul(a, b);
        expect(false, "rank-3 operand must throw");
    } catch (const moon::InvalidTensorDimension &) { expect(true, "InvalidTensorDimension"); }
    try {
        Tensor<f16> q({32, 1, 64}), k({32, 2049, 64}), v({32, 2049, 64});
        Tensor<uint8_t> mask({1, 1, 2049});
        moon::attention::singleMaskedSDPA(q, k, v, mask);
        expect(false, "kv_len 2049 must throw");
    } catch (const moon::SequenceTooLong &) { expect(true, "SequenceTooLong"); }
    // sampling.sample: the oracle's index for draws in the middle of a candidate's interval (three equal top logits)
    {
        Tensor<f16> logits({1, 5000});
        fill(logits, 0.0f);
        const size_t top[3] = {40, 41, 4000};
        for (size_t i : top) logits.data[i] = orc_f2h(3.0f);
        moon::sampling::SamplingConfig cfg{moon::sampling::SamplingMethod::top_k};
        cfg.temperature = 1.0f;
        bool ok = true;
        for (int j = 0; j < 3; j++) {
            const float u = (j + 0.5f) / 3.0f;
            size_t want = 0;
            orc_sample_f16(logits.data.data(), logits.data.size(), 2, cfg.temperature, cfg.top_k, cfg.min_p, u, &want);
            ok = ok && want == top[j] && moon::sampling::sample(logits, cfg, u) == want;
        }
        expect(ok, "sampling.sample top_k");
        try {
            cfg.temperature = 0.0f;
            moon::sampling::sample(logits, cfg, 0.5f);
            expect(false, "temperature 0 must throw");
        } catch (const moon::InvalidTemperature &) { expect(true, "InvalidTemperature"); }
    }
    // vision.imagePatches: pixel 0 -> -1, 255 -> +1, 51 -> f16((f16(51/255) - 0.5) / 0.5) = -0.60009765625 (0xb8cd), each where
    // "b c (h p) (w q) -> b (h w) (c p q)" puts it, in both crops
    {
        const size_t H = 4, W = 6, C = 3, P = 2;
        Tensor<uint8_t> img({H, W, C});
        for (auto &v : img.data) v = 255;
        img.data[((2 * W) + 5) * C + 1] = 0;  // y 2, x 5, channel 1 -> patch (1, 2) = 5, column (1 * 2 + 0) * 2 + 1 = 5
        img.data[((1 * W) + 0) * C + 2] = 51; // y 1, x 0, channel 2 -> patch 0, column (2 * 2 + 1) * 2 + 0 = 10
        auto pt = moon::vision::imagePatches(img, P);
        const size_t T = 6, dim = 12;
        bool ok = pt.shape == std::vector<size_t>{2, T, dim};
        for (size_t b = 0; b < 2 && ok; b++)
            for (size_t t = 0; t < T; t++)
                for (size_t col = 0; col < dim; col++) {
                    const uint16_t want = (t == 5 && col == 5) ? 0xbc00 : (t == 0 && col == 10) ? 0xb8cd : 0x3c00;
                    ok = ok && pt.data[(b * T + t) * dim + col] == want;
                }
        expect(ok, "vision.imagePatches");
        try {
            Tensor<uint8_t> odd({5, 6, 3});
            moon::vision::imagePatches(odd, 2);
            expect(false, "5 rows of 2-pixel patches must throw");
        } catch (const moon::InvalidTensorDimension &) { expect(true, "InvalidPatchSize"); }
    }
    // model.TextModel / KVCache: the reference's loop (moondream.zig:323-368) over text_decoder / lm_head / text_encoder gives the
    // ids of the device loop on the same session; text_encoder returns the table's rows
    {
        moon::model::Config cfg;
        cfg.vocab = 512, cfg.dim = 128, cfg.hidden_dim = 256, cfg.n_layers = 2, cfg.n_heads = 2, cfg.head_dim = 64, cfg.seq_len = 64;
        moon::model::Weights w;
        const size_t L = cfg.n_layers, d = cfg.dim, f = cfg.hidden_dim, V = cfg.vocab;
        auto mk = [](Tensor<f16> &t, std::initializer_list<size_t> shape, float scale) {
            t = Tensor<f16>(shape);
            fill(t, scale);
        };
        mk(w.word_token_embedding, {V, d}, 0.5f), mk(w.t_ln_w, {L, d}, 1.0f), mk(w.t_ln_b, {L, d}, 0.1f);
        mk(w.t_Wqkv_w, {L, 3 * d, d}, 0.08f), mk(w.t_Wqkv_b, {L, 3 * d}, 0.05f), mk(w.t_out_proj_w, {L, d, d}, 0.08f);
        mk(w.t_out_proj_bias, {L, d}, 0.05f), mk(w.t_fc1_w, {L, f, d}, 0.08f), mk(w.t_fc1_b, {L, f}, 0.05f), mk(w.t_fc2_w, {L, d, f}, 0.08f);
        mk(w.t_fc2_b, {L, d}, 0.05f), mk(w.t_linear_w, {V, d}, 0.08f), mk(w.t_linear_b, {V}, 0.05f), mk(w.t_ln_out_w, {d}, 1.0f);
        mk(w.t_ln_out_b, {d}, 0.1f);
        moon::model::TextModel tm(cfg, w);
        Tensor<uint32_t> ids({6});
        const uint32_t prompt[6] = {3, 500, 17, 42, 255, 8};
        for (size_t i = 0; i < 6; i++) ids.data[i] = prompt[i];
        auto emb = tm.text_encoder(ids);
        bool rows = emb.shape == std::vector<size_t>{6, d};
        for (size_t i = 0; i < 6 && rows; i++)
            rows = std::memcmp(&emb.data[i * d], &w.word_token_embedding.data[prompt[i] * d], d * sizeof(f16)) == 0;
        expect(rows, "model.TextModel.text_encoder rows");
        moon::model::KVCache cache;
        std::vector<uint32_t> host_ids;
        auto r = tm.text_decoder(emb, &cache);
        for (int step = 0; step < 5; step++) {
            auto logits = tm.lm_head(r.output);
            const uint32_t tok = (uint32_t)moon::sampling::argmax(logits);
            host_ids.push_back(tok);
            Tensor<uint32_t> one({1});
            one.data[0] = tok;
            r = tm.text_decoder(tm.text_encoder(one), &cache);
        }
        expect(cache.getCurrentLen() == 11, "model.KVCache position after the loop", (double)cache.getCurrentLen());
        cache.reset();
        expect(cache.getCurrentLen() == 0, "model.KVCache.reset");
        uint32_t dev_ids[5] = {0, 0, 0, 0, 0};
        bool ok = moon_text_forward(tm.session(), prompt, 6) == MOON_OK && moon_text_greedy(tm.session(), 5, dev_ids) == MOON_OK;
        for (int i = 0; i < 5; i++) ok = ok && dev_ids[i] == host_ids[i];
        expect(ok, "model.TextModel host loop == device loop");
        cache.reset();
        moon_text_forward(tm.session(), prompt, 6);
        moon::sampling::SamplingConfig greedy{moon::sampling::SamplingMethod::greedy};
        expect(tm.next_token(greedy, 0.0f) == host_ids[0], "model.TextModel.next_token");
        try {
            Tensor<uint32_t> bad({1});
            bad.data[0] = (uint32_t)V;
            tm.text_encoder(bad);
            expect(false, "token id == vocab must throw");
        } catch (const moon::TokenIdOutOfBounds &) { expect(true, "TokenIdOutOfBounds"); }
    }
    // model.VisionModel: encode_image from the resized pixels = imagePatches + the session's encode_image on the patches
    {
        moon::model::Config cfg;
        cfg.img_dim = 8, cfg.patch_size = 2, cfg.vit_dim = 128, cfg.n_vit_layers = 2, cfg.n_vit_heads = 2, cfg.vit_head_dim = 64;
        cfg.hidden_features = 256;
        const size_t L = cfg.n_vit_layers, d = cfg.vit_dim, f = cfg.hidden_features, T = 16, pd = 12, ph = 96, od = 40;
        moon::model::Weights w;
        auto mk = [](Tensor<f16> &t, std::initializer_list<size_t> shape, float scale) {
            t = Tensor<f16>(shape);
            fill(t, scale);
        };
        mk(w.v_patch_embedding_linear_w, {pd, d}, 0.2f), mk(w.v_patch_embedding_linear_b, {d}, 0.05f), mk(w.v_pos_embedding, {1, T, d}, 0.1f);
        mk(w.v_Wqkv_w, {L, d, 3 * d}, 0.08f), mk(w.v_Wqkv_b, {L, 3 * d}, 0.05f), mk(w.v_out_proj_w, {L, d, d}, 0.08f), mk(w.v_out_proj_b, {L, d}, 0.05f);
        mk(w.v_fc1_w, {L, d, f}, 0.08f), mk(w.v_fc1_b, {L, f}, 0.05f), mk(w.v_fc2_w, {L, f, d}, 0.08f), mk(w.v_fc2_b, {L, d}, 0.05f);
        mk(w.v_norm1_w, {L, d}, 1.0f), mk(w.v_norm1_b, {L, d}, 0.1f), mk(w.v_norm2_w, {L, d}, 1.0f), mk(w.v_norm2_b, {L, d}, 0.1f);
        mk(w.v_norm_out_w, {d}, 1.0f), mk(w.v_norm_out_b, {d}, 0.1f), mk(w.v_proj_fc1_w, {2 * d, ph}, 0.08f), mk(w.v_proj_fc1_b, {ph}, 0.05f);
        mk(w.v_proj_fc2_w, {ph, od}, 0.08f), mk(w.v_proj_fc2_b, {od}, 0.05f);
        moon::model::VisionModel vm(cfg, w);
        Tensor<uint8_t> img({8, 8, 3});
        for (auto &px : img.data) px = (uint8_t)((rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull) >> 56);
        auto feats = vm.encode_image(img);
        auto patches = moon::vision::imagePatches(img, 2);
        Tensor<f16> want({T, od});
        bool ok = moon_vision_encode_image(vm.session(), patches.data.data(), want.data.data()) == MOON_OK &&
                  feats.shape == std::vector<size_t>{T, od} && std::memcmp(feats.data.data(), want.data.data(), want.data.size() * sizeof(f16)) == 0;
        std::vector<float> ff(feats.data.size());
        orc_cast_f16_to_f32(feats.data.data(), ff.data(), ff.size());
        double norm = 0;
        for (float x : ff) ok = ok && std::isfinite(x), norm += (double)x * x;
        expect(ok && norm > 0, "model.VisionModel.encode_image", norm);
        auto enc = vm.vision_encoder(patches);
        expect(enc.shape == std::vector<size_t>{2, T, d}, "model.VisionModel.vision_encoder shape");
        try {
            Tensor<f16> one_crop({1, T, pd});
            vm.vision_encoder(one_crop);
            expect(false, "one crop must throw");
        } catch (const moon::InvalidTensorDimension &) { expect(true, "UnexpectedBatchCount"); }
    }
    moon::attention::cleanupThreadPool();
    std::printf("%d failures\n", failures);
    return failures ? 1 : 0;
}
