//! GPU drop-in for src/model/text_model.zig: TextModel(config) and KVCache(config) keep the pub signatures that
//! moondream.zig / moonchat.zig call (init, deinit, text_encoder, text_decoder, lm_head; KVCache.init / reset / deinit /
//! getLayerCache), so the generation loop of moondream.zig:323-368 compiles with only its import changed.  The work is
//! done by a device-resident session of libmoonhip (moon_text_*): the weights are uploaded once in init, the KV cache
//! and all activations stay in HBM, and what crosses the bus per call is what the reference's signatures carry: rows
//! of embeddings in, rows of hidden states / one row of logits out.
//!
//! Differences a caller can observe:
//!   * The KV cache lives in the session.  KVCache(config) is a handle onto it: one live cache per TextModel, and
//!     text_decoder appends to it whether or not the caller passes the handle (the reference's callers always do).
//!   * lm_head(hidden) answers for the last row of the latest text_decoder call; `hidden` is only looked at for its shape
//!     (the reference's callers pass exactly that tensor, moondream.zig:327-334).
//!   * text_decoder's `cache` result is an unused fresh handle, like the reference's (text_model.zig:143, 176-179).
const std = @import("std");
const Allocator = std.mem.Allocator;

const Weights = @import("../model/weights.zig").Weights;
const Config = @import("../model/config.zig").Config;
const Tensor = @import("../core/tensor.zig").Tensor;
const moon = @import("moonhip.zig");

pub fn TextModel(comptime model_config: Config) type {
    return struct {
        const Self = @This();
        const config = model_config;
        const KVCacheType = KVCache(config);
        pub const LayerCache = KVCacheType.LayerCache;

        comptime {
            if (config.head_dim * config.n_heads != config.dim) @compileError("Invalid head dimensions");
            if (config.seq_len == 0) @compileError("Sequence length must be greater than 0");
            if (config.vocab == 0) @compileError("Vocabulary size must be greater than 0");
            if (config.hidden_dim < config.dim) @compileError("Hidden dimension must be greater than or equal to model dimension");
        }

        weights: Weights,
        allocator: Allocator,
        session: *moon.c.moon_text_model,

        pub fn init(weights: Weights, allocator: Allocator) !Self {
            const ctx = try moon.context();
            var cfg: moon.c.moon_text_config = undefined;
            moon.c.moon_text_config_default(&cfg);
            cfg.vocab = config.vocab;
            cfg.dim = config.dim;
            cfg.hidden_dim = config.hidden_dim;
            cfg.n_layers = config.n_layers;
            cfg.n_heads = config.n_heads;
            cfg.head_dim = config.head_dim;
            cfg.rot_dim = config.head_dim / 2; // text_model.zig:56
            cfg.max_seq = 2048; // text_model.zig:353
            // the moondream.bin text layout is the session's own ([L, out, in] rows, weights.zig:439-454): no re-layout
            const w = moon.c.moon_text_weights{
                .word_token_embedding = moon.bits(weights.word_token_embedding.data.ptr),
                .t_ln_w = moon.bits(weights.t_ln_w.data.ptr),
                .t_ln_b = moon.bits(weights.t_ln_b.data.ptr),
                .t_Wqkv_w = moon.bits(weights.t_Wqkv_w.data.ptr),
                .t_Wqkv_b = moon.bits(weights.t_Wqkv_b.data.ptr),
                .t_out_proj_w = moon.bits(weights.t_out_proj_w.data.ptr),
                .t_out_proj_b = moon.bits(weights.t_out_proj_bias.data.ptr),
                .t_fc1_w = moon.bits(weights.t_fc1_w.data.ptr),
                .t_fc1_b = moon.bits(weights.t_fc1_b.data.ptr),
                .t_fc2_w = moon.bits(weights.t_fc2_w.data.ptr),
                .t_fc2_b = moon.bits(weights.t_fc2_b.data.ptr),
                .t_linear_w = moon.bits(weights.t_linear_w.data.ptr),
                .t_linear_b = moon.bits(weights.t_linear_b.data.ptr),
                .t_ln_out_w = moon.bits(weights.t_ln_out_w.data.ptr),
                .t_ln_out_b = moon.bits(weights.t_ln_out_b.data.ptr),
            };
            var session: ?*moon.c.moon_text_model = null;
            try moon.check(ctx, moon.c.moon_text_model_create(ctx, &cfg, &w, &session));
            KVCacheType.bound_session = session;
            return Self{ .weights = weights, .allocator = allocator, .session = session.? };
        }

        pub fn deinit(self: *Self) void {
            if (KVCacheType.bound_session == self.session) KVCacheType.bound_session = null;
            moon.c.moon_text_model_destroy(self.session);
            self.* = undefined;
        }

        /// text_model.zig:106-137
        pub fn text_encoder(self: Self, input_ids: Tensor(u32)) !Tensor(f16) {
            if (input_ids.shape.len != 1) return error.InvalidInputShape;
            const seq_length = input_ids.shape[0];
            if (seq_length > config.seq_len) return error.SequenceTooLong;
            const ctx = try moon.context();
            var output = try Tensor(f16).init(self.allocator, &[_]usize{ seq_length, config.dim });
            errdefer output.deinit();
            try moon.check(ctx, moon.c.moon_text_embed(self.session, input_ids.data.ptr, seq_length, moon.bitsMut(output.data.ptr)));
            return output;
        }

        /// text_model.zig:139-180: the rows are appended at the cache's position
        pub fn text_decoder(self: Self, input_embeds: Tensor(f16), kv_cache: ?*KVCacheType) !struct { output: Tensor(f16), cache: KVCacheType } {
            _ = kv_cache; // the session's own cache (see the head of this file)
            if (input_embeds.shape.len != 2) return error.InvalidInputShape;
            const ctx = try moon.context();
            const n = input_embeds.shape[0];
            try moon.check(ctx, moon.c.moon_text_forward_embeds(self.session, moon.bits(input_embeds.data.ptr), n));
            var output = try Tensor(f16).init(self.allocator, &[_]usize{ n, config.dim });
            errdefer output.deinit();
            try moon.check(ctx, moon.c.moon_text_hidden(self.session, moon.bitsMut(output.data.ptr), n));
            return .{ .output = output, .cache = try KVCacheType.init(self.allocator) };
        }

        /// text_model.zig:325-345
        pub fn lm_head(self: Self, hidden: Tensor(f16)) !Tensor(f16) {
            if (hidden.shape.len != 2) return error.InvalidInputShape;
            const ctx = try moon.context();
            var logits = try Tensor(f16).init(self.allocator, &[_]usize{ 1, config.vocab });
            errdefer logits.deinit();
            try moon.check(ctx, moon.c.moon_text_logits(self.session, moon.bitsMut(logits.data.ptr)));
            return logits;
        }

        /// Not in the reference: lm_head + sampling.sample on the device (moondream.zig:333-337 in one call; 4 bytes come
        /// back instead of the 100 KB row of logits).  u: one rng.float(f32), as sampling.sample would draw it.
        pub fn next_token(self: Self, cfg: moon.c.moon_sampling_config, u: f32) !u32 {
            const ctx = try moon.context();
            var token: u32 = 0;
            try moon.check(ctx, moon.c.moon_text_next_token(self.session, &cfg, u, &token));
            return token;
        }
    };
}

/// Handle onto the session's cache (text_model.zig:349-539).  The per-layer buffers of the reference do not exist on the
/// host; LayerCache only answers getCurrentLen / reset, which is what callers outside text_model.zig use.
pub fn KVCache(comptime model_config: Config) type {
    return struct {
        const Self = @This();
        const config = model_config;
        const n_layers: usize = config.n_layers;

        var bound_session: ?*moon.c.moon_text_model = null;
        var layer_handles: [n_layers]LayerCache = [_]LayerCache{.{}} ** n_layers;

        allocator: Allocator,

        pub const LayerCache = struct {
            pub fn getCurrentLen(self: *const LayerCache) usize {
                _ = self;
                return if (bound_session) |s| moon.c.moon_text_position(s) else 0;
            }
            pub fn reset(self: *LayerCache) void {
                _ = self;
                if (bound_session) |s| _ = moon.c.moon_text_reset(s);
            }
            pub fn deinit(self: *LayerCache) void {
                _ = self;
            }
        };

        pub fn init(allocator: Allocator) !Self {
            return Self{ .allocator = allocator };
        }

        pub fn deinit(self: *Self) void {
            self.* = undefined;
        }

        /// text_model.zig:526-530: empties the cache (the session's position goes back to 0)
        pub fn reset(self: *Self) void {
            _ = self;
            if (bound_session) |s| _ = moon.c.moon_text_reset(s);
        }

        pub fn getLayerCache(self: *Self, layer: usize) !*LayerCache {
            _ = self;
            if (layer >= n_layers) return error.LayerIndexOutOfBounds;
            return &layer_handles[layer];
        }
    };
}
