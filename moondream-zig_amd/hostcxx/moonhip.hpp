// C++ host mirror of the reference's operator interface for the FP16 matmul / attention path, over the C ABI in
// moonhip.h.  The reference is Zig; where no Zig toolchain exists this header plays the part of the .zig shims in
// ../zig: same namespaces (hgemm, hgemm_trans, attention, rope, ops, sampling) and, in namespace model, the reference's
// TextModel / KVCache / VisionModel over device-resident sessions; same argument meaning, and the reference's error names as
// exception types.  Header-only; link libmoonhip.so.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <stdexcept>
#include <string>
#include <vector>

#include "moonhip.h"

namespace moon {

// The reference's error set (hgemm.zig:371,380; attention.zig:769; rope.zig:140-142; text_model.zig:127; ops.zig:1175).
struct Error : std::runtime_error {
    int status;
    Error(int s, const std::string &what) : std::runtime_error(what), status(s) {}
};
#define MOON_CXX_ERROR(Name)                                                                                                      \
    struct Name : Error {                                                                                                         \
        using Error::Error;                                                                                                       \
    }
MOON_CXX_ERROR(InvalidTensorDimension);
MOON_CXX_ERROR(IncompatibleTensorShapes);
MOON_CXX_ERROR(SequenceTooLong);
MOON_CXX_ERROR(OutOfMemory);
MOON_CXX_ERROR(InvalidRotationDimension);
MOON_CXX_ERROR(InvalidInputDimensions);
MOON_CXX_ERROR(TokenIdOutOfBounds);
MOON_CXX_ERROR(InvalidEpsilon);
MOON_CXX_ERROR(InvalidTemperature);
MOON_CXX_ERROR(NoGpuDevice);
MOON_CXX_ERROR(GpuFailure);
#undef MOON_CXX_ERROR

// Dense row-major tensor with an owned buffer, the shape of the reference's Tensor(T) (tensor.zig): `shape` and `data`.
template <class T> struct Tensor {
    std::vector<size_t> shape;
    std::vector<T> data;
    Tensor() = default;
    explicit Tensor(std::initializer_list<size_t> s) : shape(s) {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        data.assign(n, T());
    }
    explicit Tensor(const std::vector<size_t> &s) : shape(s) {
        size_t n = 1;
        for (size_t d : shape) n *= d;
        data.assign(n, T());
    }
};
using f16 = moon_f16; // binary16 bit pattern

class Context {
  public:
    explicit Context(int device = 0) {
        int rc = moon_ctx_create(device, &ctx_);
        if (rc != MOON_OK) raise(nullptr, rc);
    }
    ~Context() {
        if (ctx_) moon_ctx_destroy(ctx_);
    }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    moon_ctx *get() const { return ctx_; }
    void check(int rc) const {
        if (rc != MOON_OK) raise(ctx_, rc);
    }
    static Context &global() {
        static Context c(0);
        return c;
    }

  private:
    [[noreturn]] static void raise(const moon_ctx *ctx, int rc) {
        std::string msg = moon_last_error(ctx);
        switch (rc) {
        case MOON_EINVAL_DIM: throw InvalidTensorDimension(rc, msg);
        case MOON_ESHAPE: throw IncompatibleTensorShapes(rc, msg);
        case MOON_ESEQ_TOO_LONG: throw SequenceTooLong(rc, msg);
        case MOON_ENOMEM: throw OutOfMemory(rc, msg);
        case MOON_EROT_DIM: throw InvalidRotationDimension(rc, msg);
        case MOON_ETOKEN: throw TokenIdOutOfBounds(rc, msg);
        case MOON_EEPS: throw InvalidEpsilon(rc, msg);
        case MOON_ETEMPERATURE: throw InvalidTemperature(rc, msg);
        case MOON_ENODEVICE: throw NoGpuDevice(rc, msg);
        default: throw GpuFailure(rc, msg);
        }
    }
    moon_ctx *ctx_ = nullptr;
};

namespace hgemm {
// hgemm.matmul(a[M,K], b[K,N]) -> [M,N] (hgemm.zig:362-426)
inline Tensor<f16> matmul(const Tensor<f16> &a, const Tensor<f16> &b, Context &ctx = Context::global()) {
    if (a.shape.size() != 2 || b.shape.size() != 2) throw InvalidTensorDimension(MOON_EINVAL_DIM, "matmul needs rank-2 tensors");
    Tensor<f16> c({a.shape[0], b.shape[1]});
    ctx.check(moon_hgemm(ctx.get(), a.data.data(), a.shape[0], a.shape[1], b.data.data(), b.shape[0], b.shape[1], c.data.data()));
    return c;
}
} // namespace hgemm

namespace hgemm_trans {
// hgemm_trans.matmul(a[M,K], b_transposed[N,K]) -> [M,N] (hgemm_trans.zig:400-488)
inline Tensor<f16> matmul(const Tensor<f16> &a, const Tensor<f16> &b_t, Context &ctx = Context::global()) {
    if (a.shape.size() != 2 || b_t.shape.size() != 2)
        throw InvalidTensorDimension(MOON_EINVAL_DIM, "matmul needs rank-2 tensors");
    Tensor<f16> c({a.shape[0], b_t.shape[0]});
    ctx.check(
        moon_hgemm_trans(ctx.get(), a.data.data(), a.shape[0], a.shape[1], b_t.data.data(), b_t.shape[0], b_t.shape[1], c.data.data()));
    return c;
}
} // namespace hgemm_trans

namespace attention {
constexpr size_t MAX_KV_LEN = 2048; // attention.zig:252

// attention.createAttentionMask(pos, seq_len) -> bool[1, seq_len, pos + seq_len] (attention.zig:256-281)
inline Tensor<uint8_t> createAttentionMask(size_t pos, size_t seq_len) {
    Tensor<uint8_t> m({1, seq_len, pos + seq_len});
    for (size_t i = 0; i < seq_len; ++i)
        for (size_t j = 0; j < pos + seq_len; ++j) m.data[i * (pos + seq_len) + j] = j < pos || (j - pos) <= i;
    return m;
}

// attention.multiMasklessSDPA(n_heads, head_dim, q, k, v) (attention.zig:283-413)
inline Tensor<f16> multiMasklessSDPA(size_t n_heads, size_t head_dim, const Tensor<f16> &q, const Tensor<f16> &k, const Tensor<f16> &v,
                                     Context &ctx = Context::global()) {
    Tensor<f16> out({n_heads, q.shape.at(1), head_dim});
    ctx.check(moon_sdpa_maskless(ctx.get(), q.data.data(), k.data.data(), v.data.data(), out.data.data(), n_heads, q.shape.at(1),
                                 k.shape.at(1), head_dim));
    return out;
}

// attention.multiMaskedSDPA(q, k, v, mask, n_heads, head_dim) (attention.zig:416-541)
inline Tensor<f16> multiMaskedSDPA(const Tensor<f16> &q, const Tensor<f16> &k, const Tensor<f16> &v, const Tensor<uint8_t> &mask,
                                   size_t n_heads, size_t head_dim, Context &ctx = Context::global()) {
    Tensor<f16> out({n_heads, q.shape.at(1), head_dim});
    ctx.check(moon_sdpa_masked(ctx.get(), q.data.data(), k.data.data(), v.data.data(), mask.data.data(), mask.shape.at(2),
                               out.data.data(), n_heads, q.shape.at(1), k.shape.at(1), head_dim));
    return out;
}

// attention.singleMaskedSDPA(q, k, v, mask) (attention.zig:759-811)
inline Tensor<f16> singleMaskedSDPA(const Tensor<f16> &q, const Tensor<f16> &k, const Tensor<f16> &v, const Tensor<uint8_t> &mask,
                                    Context &ctx = Context::global()) {
    if (k.shape.at(1) > MAX_KV_LEN) throw SequenceTooLong(MOON_ESEQ_TOO_LONG, "kv_len exceeds 2048");
    Tensor<f16> out({q.shape.at(0), 1, q.shape.at(2)});
    ctx.check(moon_sdpa_single(ctx.get(), q.data.data(), k.data.data(), v.data.data(), mask.data.data(), out.data.data(), q.shape.at(0),
                               k.shape.at(1), q.shape.at(2)));
    return out;
}

inline void cleanupThreadPool(Context &ctx = Context::global()) { moon_cleanup(ctx.get()); }
} // namespace attention

namespace rope {
// rope.applyRotEmb(x, n_heads, head_dim, freqs_cis, position_ids, rot_dim) (rope.zig:130-272)
inline Tensor<f16> applyRotEmb(const Tensor<f16> &x, size_t n_heads, size_t head_dim, const Tensor<float> &freqs_cis,
                               const Tensor<size_t> &position_ids, size_t rot_dim, Context &ctx = Context::global()) {
    if (x.shape.size() != 3) throw InvalidInputDimensions(MOON_EINVAL_DIM, "applyRotEmb needs [n_heads, seq_len, head_dim]");
    Tensor<f16> out(x.shape);
    ctx.check(moon_rope_apply(ctx.get(), x.data.data(), out.data.data(), n_heads, x.shape[1], head_dim, freqs_cis.data.data(),
                              freqs_cis.shape.at(0), freqs_cis.shape.at(freqs_cis.shape.size() - 2), position_ids.data.data(), rot_dim));
    return out;
}
} // namespace rope

namespace ops {
// ops.layerNorm(f16, x, weight, bias, eps) (ops.zig:1063-1419)
inline Tensor<f16> layerNorm(const Tensor<f16> &x, const Tensor<f16> &weight, const Tensor<f16> &bias, float eps,
                             Context &ctx = Context::global()) {
    Tensor<f16> y(x.shape);
    size_t dim = x.shape.back();
    ctx.check(moon_layernorm(ctx.get(), x.data.data(), weight.data.data(), bias.data.data(), y.data.data(), x.data.size() / dim, dim, eps));
    return y;
}
// ops.gelu(f16, &x) in place (ops.zig:1635-1774)
inline void gelu(Tensor<f16> &x, Context &ctx = Context::global()) { ctx.check(moon_gelu(ctx.get(), x.data.data(), x.data.size())); }
// ops.broadcast_add_simd(&a, b) (ops.zig:1859-1913)
inline void broadcast_add_simd(Tensor<f16> &a, const Tensor<f16> &b, Context &ctx = Context::global()) {
    size_t cols = b.data.size();
    if (cols == 0 || a.data.size() % cols) throw IncompatibleTensorShapes(MOON_ESHAPE, "bias length does not divide the tensor");
    ctx.check(moon_bias_add(ctx.get(), a.data.data(), b.data.data(), a.data.size() / cols, cols));
}
// ops.add(f16, &a, b) (ops.zig:312-323)
inline void add(Tensor<f16> &a, const Tensor<f16> &b, Context &ctx = Context::global()) {
    if (a.data.size() != b.data.size()) throw IncompatibleTensorShapes(MOON_ESHAPE, "add needs equal sizes");
    ctx.check(moon_add(ctx.get(), a.data.data(), b.data.data(), a.data.size()));
}
} // namespace ops

namespace sampling {
// ops.argmax over the logits row (text_model.zig:385-387 feeding main.zig's greedy loop)
inline size_t argmax(const Tensor<f16> &logits, Context &ctx = Context::global()) {
    size_t idx = 0;
    ctx.check(moon_argmax(ctx.get(), logits.data.data(), logits.data.size(), &idx));
    return idx;
}
// sampling.SamplingMethod / SamplingConfig (sampling.zig:240-254), defaults included
enum class SamplingMethod { greedy = MOON_SAMPLE_GREEDY, multinomial = MOON_SAMPLE_MULTINOMIAL, top_k = MOON_SAMPLE_TOP_K, min_p = MOON_SAMPLE_MIN_P };
struct SamplingConfig {
    SamplingMethod method;
    float temperature = 0.5f;
    size_t top_k = 3;
    float min_p = 0.05f;
};
// sampling.sample (sampling.zig:353-389); u is the number the reference draws with rng.float(f32), one per call
inline size_t sample(const Tensor<f16> &logits, const SamplingConfig &config, float u, Context &ctx = Context::global()) {
    const moon_sampling_config cfg{static_cast<int>(config.method), config.temperature, config.top_k, config.min_p};
    size_t idx = 0;
    ctx.check(moon_sample(ctx.get(), logits.data.data(), logits.data.size(), &cfg, u, &idx));
    return idx;
}
} // namespace sampling

namespace vision {
// The steps of createPatches / encode_image between the resize and the encoder plus rearrangeBCHWtoBTC
// (vision_model.zig:129-184, reshape_handler.zig:5-129): image[H, W, C] u8 -> patches[2, (H/p)*(W/p), C*p*p]
inline Tensor<f16> imagePatches(const Tensor<uint8_t> &image, size_t patch_size, Context &ctx = Context::global()) {
    if (image.shape.size() != 3) throw InvalidTensorDimension(MOON_EINVAL_DIM, "imagePatches needs [H, W, C]");
    const size_t H = image.shape[0], W = image.shape[1], C = image.shape[2];
    if (!patch_size || H % patch_size || W % patch_size) throw InvalidTensorDimension(MOON_EINVAL_DIM, "InvalidPatchSize");
    Tensor<f16> out({2, (H / patch_size) * (W / patch_size), C * patch_size * patch_size});
    ctx.check(moon_image_patches(ctx.get(), image.data.data(), H, W, C, patch_size, out.data.data()));
    return out;
}
} // namespace vision

namespace model {
// The fields of the reference's Weights (weights.zig:16-60) that the two models read, in the moondream.bin layouts.
struct Weights {
    Tensor<f16> word_token_embedding, t_ln_w, t_ln_b, t_Wqkv_w, t_Wqkv_b, t_out_proj_w, t_out_proj_bias, t_fc1_w, t_fc1_b, t_fc2_w, t_fc2_b,
        t_linear_w, t_linear_b, t_ln_out_w, t_ln_out_b;
    Tensor<f16> v_patch_embedding_linear_w, v_patch_embedding_linear_b, v_pos_embedding, v_Wqkv_w, v_Wqkv_b, v_out_proj_w, v_out_proj_b, v_fc1_w,
        v_fc1_b, v_fc2_w, v_fc2_b, v_norm1_w, v_norm1_b, v_norm2_w, v_norm2_b, v_norm_out_w, v_norm_out_b, v_proj_fc1_w, v_proj_fc1_b, v_proj_fc2_w,
        v_proj_fc2_b;
};
// config.zig:76-107 (the fields the two models use)
struct Config {
    size_t vocab = 51200, dim = 2048, hidden_dim = 8192, n_layers = 24, n_heads = 32, head_dim = 64, seq_len = 2048;
    size_t img_channels = 3, img_dim = 378, patch_size = 14, vit_dim = 1152, n_vit_layers = 27, n_vit_heads = 16, vit_head_dim = 72,
           hidden_features = 4304;
};

class TextModel;
// KVCache(config) (text_model.zig:349-539): here a handle onto the cache that lives in the TextModel's device session (one live
// cache per TextModel); reset() empties it.
class KVCache {
  public:
    KVCache() = default;
    void reset() {
        if (bound()) moon_text_reset(bound());
    }
    size_t getCurrentLen() const { return bound() ? moon_text_position(bound()) : 0; }

  private:
    friend class TextModel;
    static moon_text_model *&bound() {
        static moon_text_model *m = nullptr;
        return m;
    }
};

// TextModel(config) (text_model.zig:22-345) over a device-resident session: text_encoder, text_decoder and lm_head keep the
// reference's meaning, so the generation loop of moondream.zig:323-368 runs unchanged on top of them.
class TextModel {
  public:
    TextModel(const Config &config, const Weights &w, Context &ctx = Context::global()) : config_(config), ctx_(ctx) {
        moon_text_config cfg;
        moon_text_config_default(&cfg);
        cfg.vocab = config.vocab, cfg.dim = config.dim, cfg.hidden_dim = config.hidden_dim, cfg.n_layers = config.n_layers;
        cfg.n_heads = config.n_heads, cfg.head_dim = config.head_dim, cfg.rot_dim = config.head_dim / 2, cfg.max_seq = config.seq_len;
        const moon_text_weights tw{w.word_token_embedding.data.data(), w.t_ln_w.data.data(), w.t_ln_b.data.data(), w.t_Wqkv_w.data.data(),
                                   w.t_Wqkv_b.data.data(), w.t_out_proj_w.data.data(), w.t_out_proj_bias.data.data(), w.t_fc1_w.data.data(),
                                   w.t_fc1_b.data.data(), w.t_fc2_w.data.data(), w.t_fc2_b.data.data(), w.t_linear_w.data.data(),
                                   w.t_linear_b.data.data(), w.t_ln_out_w.data.data(), w.t_ln_out_b.data.data()};
        ctx_.check(moon_text_model_create(ctx_.get(), &cfg, &tw, &session_));
        KVCache::bound() = session_;
    }
    ~TextModel() {
        if (KVCache::bound() == session_) KVCache::bound() = nullptr;
        moon_text_model_destroy(session_);
    }
    TextModel(const TextModel &) = delete;
    TextModel &operator=(const TextModel &) = delete;

    // text_model.zig:106-137
    Tensor<f16> text_encoder(const Tensor<uint32_t> &input_ids) const {
        if (input_ids.shape.size() != 1) throw InvalidTensorDimension(MOON_EINVAL_DIM, "InvalidInputShape");
        Tensor<f16> out({input_ids.shape[0], config_.dim});
        ctx_.check(moon_text_embed(session_, input_ids.data.data(), input_ids.data.size(), out.data.data()));
        return out;
    }
    // text_model.zig:139-180: the rows are appended at the cache's position (the cache argument is the session's own)
    struct DecoderResult {
        Tensor<f16> output;
        KVCache cache;
    };
    DecoderResult text_decoder(const Tensor<f16> &input_embeds, KVCache * /*kv_cache*/) const {
        if (input_embeds.shape.size() != 2) throw InvalidTensorDimension(MOON_EINVAL_DIM, "InvalidInputShape");
        const size_t n = input_embeds.shape[0];
        ctx_.check(moon_text_forward_embeds(session_, input_embeds.data.data(), n));
        DecoderResult r{Tensor<f16>({n, config_.dim}), KVCache()};
        ctx_.check(moon_text_hidden(session_, r.output.data.data(), n));
        return r;
    }
    // text_model.zig:325-345: logits of the last row of the latest text_decoder call
    Tensor<f16> lm_head(const Tensor<f16> &hidden) const {
        if (hidden.shape.size() != 2) throw InvalidTensorDimension(MOON_EINVAL_DIM, "InvalidInputShape");
        Tensor<f16> logits({1, config_.vocab});
        ctx_.check(moon_text_logits(session_, logits.data.data()));
        return logits;
    }
    // lm_head + sampling.sample in one call, the token alone comes back (not in the reference)
    uint32_t next_token(const sampling::SamplingConfig &config, float u) const {
        const moon_sampling_config cfg{static_cast<int>(config.method), config.temperature, config.top_k, config.min_p};
        uint32_t token = 0;
        ctx_.check(moon_text_next_token(session_, &cfg, u, &token));
        return token;
    }
    moon_text_model *session() const { return session_; }

  private:
    Config config_;
    Context &ctx_;
    moon_text_model *session_ = nullptr;
};

// VisionModel(config) (vision_model.zig:29-272) from the resized pixels on; decoding and resizing the file stay with the caller.
class VisionModel {
  public:
    VisionModel(const Config &config, const Weights &w, Context &ctx = Context::global()) : config_(config), ctx_(ctx) {
        moon_vision_config cfg;
        moon_vision_config_default(&cfg);
        cfg.dim = config.vit_dim, cfg.hidden_dim = config.hidden_features, cfg.n_layers = config.n_vit_layers, cfg.n_heads = config.n_vit_heads;
        cfg.head_dim = config.vit_head_dim;
        const moon_vision_weights vw{w.v_Wqkv_w.data.data(), w.v_Wqkv_b.data.data(), w.v_out_proj_w.data.data(), w.v_out_proj_b.data.data(),
                                     w.v_fc1_w.data.data(), w.v_fc1_b.data.data(), w.v_fc2_w.data.data(), w.v_fc2_b.data.data(),
                                     w.v_norm1_w.data.data(), w.v_norm1_b.data.data(), w.v_norm2_w.data.data(), w.v_norm2_b.data.data(),
                                     w.v_norm_out_w.data.data(), w.v_norm_out_b.data.data()};
        ctx_.check(moon_vision_model_create(ctx_.get(), &cfg, &vw, &session_));
        moon_vision_io_config io;
        moon_vision_io_config_default(&io);
        tokens_ = (config.img_dim / config.patch_size) * (config.img_dim / config.patch_size);
        io.patch_dim = config.patch_size * config.patch_size * config.img_channels, io.tokens = tokens_;
        io.proj_hidden = w.v_proj_fc1_w.shape.at(1), io.out_dim = out_dim_ = w.v_proj_fc2_w.shape.at(1);
        const moon_vision_io_weights iw{w.v_patch_embedding_linear_w.data.data(), w.v_patch_embedding_linear_b.data.data(),
                                        w.v_pos_embedding.data.data(), w.v_proj_fc1_w.data.data(), w.v_proj_fc1_b.data.data(),
                                        w.v_proj_fc2_w.data.data(), w.v_proj_fc2_b.data.data()};
        const int rc = moon_vision_io_attach(session_, &io, &iw);
        if (rc != MOON_OK) {
            moon_vision_model_destroy(session_);
            session_ = nullptr;
            ctx_.check(rc);
        }
    }
    ~VisionModel() {
        if (session_) moon_vision_model_destroy(session_);
    }
    VisionModel(const VisionModel &) = delete;
    VisionModel &operator=(const VisionModel &) = delete;

    // encode_image (vision_model.zig:160-202) from the resized image [img_dim, img_dim, 3] as stbir leaves it
    Tensor<f16> encode_image(const Tensor<uint8_t> &resized) const {
        if (resized.shape != std::vector<size_t>{config_.img_dim, config_.img_dim, 3}) throw InvalidTensorDimension(MOON_EINVAL_DIM, "resized image shape");
        Tensor<f16> out({tokens_, out_dim_});
        ctx_.check(moon_vision_encode_image_u8(session_, resized.data.data(), out.data.data()));
        return out;
    }
    // vision_encoder (vision_model.zig:204-271) behind rearrangeBCHWtoBTC: patches [2, tokens, patch_dim] -> [2, tokens, vit_dim]
    Tensor<f16> vision_encoder(const Tensor<f16> &patches) const {
        if (patches.shape.size() != 3 || patches.shape[0] != 2) throw InvalidTensorDimension(MOON_EINVAL_DIM, "UnexpectedBatchCount");
        Tensor<f16> out({2, tokens_, config_.vit_dim});
        ctx_.check(moon_vision_encoder(session_, patches.data.data(), out.data.data()));
        return out;
    }
    moon_vision_model *session() const { return session_; }

  private:
    Config config_;
    Context &ctx_;
    moon_vision_model *session_ = nullptr;
    size_t tokens_ = 0, out_dim_ = 0;
};
} // namespace model

} // namespace moon
