//! GPU drop-in for src/model/vision_model.zig: VisionModel(config) keeps init / deinit / createPatches / encode_image /
//! vision_encoder with the reference's signatures (vision_model.zig:71-272).  Decoding and resizing the file stay on the
//! host with stb_image exactly as in the reference (createPatches, :87-158); everything from the resized pixels on
//! (BHWC -> BCHW, /255, normalisation, patches, patch embedding, the 27 blocks, the projection MLP) runs in a
//! device-resident session of libmoonhip (moon_vision_*), whose weights are uploaded once in init.
const std = @import("std");
const Allocator = std.mem.Allocator;

const Weights = @import("../model/weights.zig").Weights;
const Config = @import("../model/config.zig").Config;
const Tensor = @import("../core/tensor.zig").Tensor;
const rearrangeBCHWtoBTC = @import("../utils/reshape_handler.zig").rearrangeBCHWtoBTC;
const moon = @import("moonhip.zig");

const c = @cImport({
    @cInclude("stb_image.h");
    @cInclude("stb_image_resize2.h");
    @cInclude("stdio.h");
});

pub fn VisionModel(comptime model_config: Config) type {
    return struct {
        const Self = @This();
        const config = model_config;
        const patches_per_image = (config.img_dim / config.patch_size) * (config.img_dim / config.patch_size);

        comptime {
            if (config.vit_head_dim * config.n_vit_heads != config.vit_dim) @compileError("Invalid head dimensions");
            if (config.img_dim % config.patch_size != 0) @compileError("Image dimension must be divisible by patch size");
        }

        weights: Weights,
        allocator: Allocator,
        session: *moon.c.moon_vision_model,

        pub fn init(weights: Weights, allocator: Allocator) !Self {
            const ctx = try moon.context();
            var cfg: moon.c.moon_vision_config = undefined;
            moon.c.moon_vision_config_default(&cfg);
            cfg.dim = config.vit_dim;
            cfg.hidden_dim = config.hidden_features;
            cfg.n_layers = config.n_vit_layers;
            cfg.n_heads = config.n_vit_heads;
            cfg.head_dim = config.vit_head_dim;
            // the moondream.bin vision layout [L, in, out] (weights.zig:459-474); the session re-lays it out once
            const w = moon.c.moon_vision_weights{
                .v_Wqkv_w = moon.bits(weights.v_Wqkv_w.data.ptr),
                .v_Wqkv_b = moon.bits(weights.v_Wqkv_b.data.ptr),
                .v_out_proj_w = moon.bits(weights.v_out_proj_w.data.ptr),
                .v_out_proj_b = moon.bits(weights.v_out_proj_b.data.ptr),
                .v_fc1_w = moon.bits(weights.v_fc1_w.data.ptr),
                .v_fc1_b = moon.bits(weights.v_fc1_b.data.ptr),
                .v_fc2_w = moon.bits(weights.v_fc2_w.data.ptr),
                .v_fc2_b = moon.bits(weights.v_fc2_b.data.ptr),
                .v_norm1_w = moon.bits(weights.v_norm1_w.data.ptr),
                .v_norm1_b = moon.bits(weights.v_norm1_b.data.ptr),
                .v_norm2_w = moon.bits(weights.v_norm2_w.data.ptr),
                .v_norm2_b = moon.bits(weights.v_norm2_b.data.ptr),
                .v_norm_out_w = moon.bits(weights.v_norm_out_w.data.ptr),
                .v_norm_out_b = moon.bits(weights.v_norm_out_b.data.ptr),
            };
            var session: ?*moon.c.moon_vision_model = null;
            try moon.check(ctx, moon.c.moon_vision_model_create(ctx, &cfg, &w, &session));
            errdefer moon.c.moon_vision_model_destroy(session);
            var io: moon.c.moon_vision_io_config = undefined;
            moon.c.moon_vision_io_config_default(&io);
            io.patch_dim = config.patch_size * config.patch_size * config.img_channels;
            io.tokens = patches_per_image;
            io.proj_hidden = weights.v_proj_fc1_w.shape[1];
            io.out_dim = weights.v_proj_fc2_w.shape[1];
            const iw = moon.c.moon_vision_io_weights{
                .v_patch_embedding_linear_w = moon.bits(weights.v_patch_embedding_linear_w.data.ptr),
                .v_patch_embedding_linear_b = moon.bits(weights.v_patch_embedding_linear_b.data.ptr),
                .v_pos_embedding = moon.bits(weights.v_pos_embedding.data.ptr),
                .v_proj_fc1_w = moon.bits(weights.v_proj_fc1_w.data.ptr),
                .v_proj_fc1_b = moon.bits(weights.v_proj_fc1_b.data.ptr),
                .v_proj_fc2_w = moon.bits(weights.v_proj_fc2_w.data.ptr),
                .v_proj_fc2_b = moon.bits(weights.v_proj_fc2_b.data.ptr),
            };
            try moon.check(ctx, moon.c.moon_vision_io_attach(session, &io, &iw));
            return Self{ .weights = weights, .allocator = allocator, .session = session.? };
        }

        pub fn deinit(self: *Self) void {
            moon.c.moon_vision_model_destroy(self.session);
            self.* = undefined;
        }

        /// The resized image as bytes [img_dim, img_dim, 3] (vision_model.zig:87-127: stb_image load + sRGB resize, unchanged).
        fn loadResized(self: Self, image_path: []const u8) ![]u8 {
            var normalized_path = try self.allocator.alloc(u8, image_path.len + 1);
            defer self.allocator.free(normalized_path);
            for (image_path, 0..) |ca, i| normalized_path[i] = if (ca == '\\') '/' else ca;
            normalized_path[image_path.len] = 0;
            var width: c_int = 0;
            var height: c_int = 0;
            var channels: c_int = 0;
            const img_data = c.stbi_load(normalized_path.ptr, &width, &height, &channels, 0);
            if (img_data == null) {
                std.debug.print("STB Image loading failed: {s}\n", .{c.stbi_failure_reason()});
                return error.ImageNotFound;
            }
            defer c.stbi_image_free(img_data);
            const ch: usize = @intCast(channels);
            const resized = try self.allocator.alloc(u8, config.img_dim * config.img_dim * ch);
            errdefer self.allocator.free(resized);
            const ok = c.stbir_resize_uint8_srgb(img_data, width, height, 0, resized.ptr, @intCast(config.img_dim), @intCast(config.img_dim), 0, if (channels == 3) c.STBIR_RGB else c.STBIR_RGBA);
            if (ok == 0) return error.FailedToResizeImage;
            if (ch == 3) return resized;
            // the encoder takes three channels (the reference's patch embedding has 588 = 14 * 14 * 3 inputs)
            const rgb = try self.allocator.alloc(u8, config.img_dim * config.img_dim * 3);
            for (0..config.img_dim * config.img_dim) |p| {
                for (0..3) |k| rgb[p * 3 + k] = resized[p * ch + k];
            }
            self.allocator.free(resized);
            return rgb;
        }

        /// vision_model.zig:87-158: [2, img_dim, img_dim, channels] f16, both crops the resized image
        pub fn createPatches(self: Self, image_path: []const u8) !Tensor(f16) {
            const pixels = try self.loadResized(image_path);
            defer self.allocator.free(pixels);
            var patches = try Tensor(f16).init(self.allocator, &[_]usize{ 2, config.img_dim, config.img_dim, 3 });
            errdefer patches.deinit();
            const n = config.img_dim * config.img_dim * 3;
            for (0..2) |b| {
                for (0..n) |i| patches.data[b * n + i] = @floatFromInt(pixels[i]);
            }
            return patches;
        }

        /// vision_model.zig:160-202: the features [patches_per_image, out_dim] of the image file.  From the resized pixels
        /// on, one call into the session (u8 up, the features down).
        pub fn encode_image(self: Self, image_path: []const u8) !Tensor(f16) {
            const ctx = try moon.context();
            const pixels = try self.loadResized(image_path);
            defer self.allocator.free(pixels);
            var out = try Tensor(f16).init(self.allocator, &[_]usize{ patches_per_image, self.weights.v_proj_fc2_w.shape[1] });
            errdefer out.deinit();
            try moon.check(ctx, moon.c.moon_vision_encode_image_u8(self.session, pixels.ptr, moon.bitsMut(out.data.ptr)));
            return out;
        }

        /// vision_model.zig:204-271: input [2, C, H, W] normalised -> [2, patches_per_image, vit_dim]
        pub fn vision_encoder(self: Self, input: Tensor(f16)) !Tensor(f16) {
            if (input.shape[0] != 2) {
                std.log.err("Expected batch size 2, got {d}\n", .{input.shape[0]});
                return error.UnexpectedBatchCount;
            }
            const ctx = try moon.context();
            var x = try rearrangeBCHWtoBTC(self.allocator, input, config.patch_size); // host helper of the reference, :210
            defer x.deinit();
            var out = try Tensor(f16).init(self.allocator, &[_]usize{ 2, patches_per_image, config.vit_dim });
            errdefer out.deinit();
            try moon.check(ctx, moon.c.moon_vision_encoder(self.session, moon.bits(x.data.ptr), moon.bitsMut(out.data.ptr)));
            return out;
        }
    };
}
