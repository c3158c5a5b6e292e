// Rounding-point helpers shared by the matrix-product kernels.  Each helper reproduces where the
// reference turns f32 into f16 (hgemm.zig:138 / hgemm_trans.zig:116,394 store; ops.zig:1892-1901 bias add;
// ops.zig:1717-1721 GELU), so a fused epilogue yields the same bits as the reference's separate passes.
#pragma once
#include "moon_internal.hpp"

// The compiler folds "f32 multiply, then convert to f16" into one v_fma_mixlo_f16 that rounds the exact
// product straight to f16, whatever the contraction setting.  Where the reference rounds to f32 first (and the
// host-side generator must be matched bit for bit), pass the f32 value through this no-op barrier.
__device__ __forceinline__ float f32_round(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

__device__ __forceinline__ float gelu_f32(float v) {
    // constants are the f16-rounded values the reference uses (ops.zig:1641-1642): c = 0.7978515625, alpha = 0.044708251953125
    // 0.5 v (1 + tanh(u)) = v / (1 + exp(-2u)), u = c (v + alpha v^3): one exp2 and one reciprocal of the hardware (each
    // within an ulp), no cancellation for negative v, the limits v and -0 come out exactly.  -2u / ln 2 is taken as
    // v * (k1 + k2 v^2) (a multiply, a fused multiply-add, a multiply): five plain instructions and the two transcendental
    // ones per element.  The error against the reference's f32 evaluation with a library tanh is a few f32 ulps of the
    // result: three orders below the f16 spacing.  (The library tanhf costs ~45 instructions per element, which made the
    // GELU epilogue of the vision fc1 GEMM 6 us of its 22.)
    constexpr float k1 = float(-0.7978515625 * 2.8853900817779268);                     // -2 c / ln 2
    constexpr float k2 = float(-0.7978515625 * 2.8853900817779268 * 0.044708251953125); // ... * alpha
    const float e = __builtin_amdgcn_exp2f(v * __builtin_fmaf(v * v, k2, k1));
    return f32_round(v * __builtin_amdgcn_rcpf(1.0f + e));
}

// epilogue with the bias value already in hand
// Internal epilogue value beside the public MOON_EPI_*: bias, then "+= into a residual" as the vision blocks do
// (x += attention_block(..), x += mlp(..): vision_model.zig:247, 261; ops.add rounds f16(x + y), ops.zig:320-322).
constexpr int MOON_EPI_BIAS_RESID = 3;
template <int EPI>
__device__ __forceinline__ half_t apply_residual(half_t t, const half_t *__restrict__ resid, size_t idx) {
    if (EPI == MOON_EPI_BIAS_RESID) t = (half_t)((float)resid[idx] + (float)t);
    return t;
}

template <int EPI>
__device__ __forceinline__ half_t apply_epilogue_v(float acc, half_t bias_n) {
    half_t t = (half_t)acc; // matmul result rounded to f16
    if (EPI >= MOON_EPI_BIAS) t = (half_t)((float)t + (float)bias_n);
    if (EPI == MOON_EPI_BIAS_GELU) t = (half_t)gelu_f32((float)t);
    return t;
}

template <int EPI>
__device__ __forceinline__ half_t apply_epilogue(float acc, const half_t *__restrict__ bias, size_t n) {
    return apply_epilogue_v<EPI>(acc, EPI >= MOON_EPI_BIAS ? bias[n] : (half_t)0.0f);
}

// One rotation of rope.applyRotEmb (rope.zig:223-224): separate multiplies and adds, one rounding to f16 each
__device__ __forceinline__ void rotate_pair(float xr, float xi, float c, float s, half_t &o_r, half_t &o_i) {
#pragma clang fp contract(off)
    o_r = (half_t)(xr * c - xi * s);
    o_i = (half_t)(xr * s + xi * c);
}

// Workgroup barrier for data exchanged through LDS only: waits for this wavefront's LDS operations, not for its
// outstanding global loads (which __syncthreads() would drain), so prefetched weights stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Accesses that are coherent across the whole device without cache maintenance: relaxed agent-scope atomics
// compile to loads/stores with the sc1 bit, which write through / miss in the per-XCD L2 and the per-CU L1.
// The persistent decode kernel moves all data that one workgroup produces and another consumes through
// these, so its device-wide barrier needs no L2 write-back or invalidate.  COH = false: plain accesses.
template <bool COH> __device__ __forceinline__ half_t ld_h(const half_t *p) {
    if (!COH) return *p;
    const unsigned short b = __hip_atomic_load(reinterpret_cast<const unsigned short *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(half_t, b);
}
template <bool COH> __device__ __forceinline__ void st_h(half_t *p, half_t v) {
    if (!COH) {
        *p = v;
        return;
    }
    __hip_atomic_store(reinterpret_cast<unsigned short *>(p), __builtin_bit_cast(unsigned short, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
template <bool COH> __device__ __forceinline__ float ld_f(const float *p) {
    if (!COH) return *p;
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool COH> __device__ __forceinline__ void st_f(float *p, float v) {
    if (!COH) {
        *p = v;
        return;
    }
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int ld_i_coh(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_i_coh(int *p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// 64-lane reductions on the DPP cross-lane path (no LDS crossbar): quad swaps (xor 1, xor 2), mirror within
// 8 lanes, mirror within the 16-lane row, then the four row results are read out and combined.  Fixed order,
// every lane returns the same bits.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
constexpr int DPP_QUAD_XOR1 = 0xB1, DPP_QUAD_XOR2 = 0x4E, DPP_ROW_HALF_MIRROR = 0x141, DPP_ROW_MIRROR = 0x140;

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<DPP_QUAD_XOR1>(v);
    v += dpp_move<DPP_QUAD_XOR2>(v);
    v += dpp_move<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_move<DPP_ROW_MIRROR>(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_move<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_move<DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_move<DPP_ROW_MIRROR>(v));
    return fmaxf(fmaxf(read_lane(v, 0), read_lane(v, 16)), fmaxf(read_lane(v, 32), read_lane(v, 48)));
}
