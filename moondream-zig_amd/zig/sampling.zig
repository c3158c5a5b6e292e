//! Drop-in for the sampling entry points of src/utils/sampling.zig that the generation loops call (moondream.zig:337,
//! moonchat.zig:597): the reference's names, signatures, configuration and error behaviour, the work done by libmoonhip
//! on the GPU.  The PRNG stays here: one rng.float(f32) per call, as in the reference.
const std = @import("std");
const Allocator = std.mem.Allocator;
const Tensor = @import("../core/tensor.zig").Tensor;
const moon = @import("moonhip.zig");

pub const SamplingMethod = enum(c_int) { greedy = 0, multinomial = 1, top_k = 2, min_p = 3 };

pub const SamplingConfig = struct {
    method: SamplingMethod,
    temperature: f32 = 0.5,
    top_k: ?usize = 3,
    min_p: ?f32 = 0.05,
    min_tokens_to_keep: usize = 1,
};

/// sampling.zig:257: argmax(comptime T, tensor).  f32 and f16 rows go to the device; other types keep the host loop.
pub fn argmax(comptime T: type, tensor: *const Tensor(T)) !usize {
    if (tensor.data.len == 0) return error.EmptyTensor;
    if (T != f32 and T != f16) {
        var max_idx: usize = 0;
        var max_val = tensor.data[0];
        for (tensor.data, 0..) |val, i| {
            if (val > max_val) {
                max_val = val;
                max_idx = i;
            }
        }
        return max_idx;
    }
    const ctx = try moon.context();
    var index: usize = 0;
    if (T == f32) {
        try moon.check(ctx, moon.c.moon_argmax_f32(ctx, tensor.data.ptr, tensor.data.len, &index));
    } else {
        try moon.check(ctx, moon.c.moon_argmax(ctx, moon.bits(tensor.data.ptr), tensor.data.len, &index));
    }
    return index;
}

/// sampling.zig:353: sample(tensor: *Tensor(f32), config, rng, allocator).  The allocator is unused (the working copy
/// of the row lives on the device); it is kept so that the call sites compile unchanged.
pub fn sample(tensor: *Tensor(f32), config: SamplingConfig, rng: std.rand.Random, allocator: Allocator) !usize {
    _ = allocator;
    if (tensor.data.len == 0) return error.EmptyTensor;
    const cfg = moon.c.moon_sampling_config{
        .method = @intFromEnum(config.method),
        .temperature = config.temperature,
        .top_k = if (config.method == .top_k) (config.top_k orelse return error.MissingTopKValue) else 0,
        .min_p = if (config.method == .min_p) (config.min_p orelse return error.MissingMinPValue) else 0,
    };
    const u: f32 = if (config.method == .greedy) 0 else rng.float(f32);
    const ctx = try moon.context();
    var index: usize = 0;
    try moon.check(ctx, moon.c.moon_sample_f32(ctx, tensor.data.ptr, tensor.data.len, &cfg, u, &index));
    return index;
}
