// Context, device memory, resident-weight registry, timers and the synthetic-data kernels.
#include <cstring>

#include "moon_internal.hpp"

static thread_local std::string g_create_error;

int moon_fail(moon_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    if (ctx)
        ctx->err = buf;
    else
        g_create_error = buf;
    return code;
}

int moon_grow(moon_ctx *ctx, GrowBuf &b, size_t bytes) {
    if (bytes <= b.cap) return MOON_OK;
    if (b.ptr) {
        // buffers may still be in use by queued kernels
        MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
        MOON_HIP(ctx, hipFree(b.ptr));
        b.ptr = nullptr;
        b.cap = 0;
        if (&b == &ctx->work[1]) { // the decode-attention counters lived there: a new allocation may return the same address
            ctx->attn_cnt_buf = nullptr;
            ctx->attn_cnt_launches = 0;
        }
    }
    size_t cap = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    MOON_HIP(ctx, hipMalloc(&b.ptr, cap));
    b.cap = cap;
    return MOON_OK;
}

extern "C" int moon_ctx_create(int device, moon_ctx **out) {
    if (!out) return moon_fail(nullptr, MOON_EINVAL, "moon_ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return moon_fail(nullptr, MOON_ENODEVICE, "no HIP device available (%s); this library has no CPU path",
                         e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count) return moon_fail(nullptr, MOON_EINVAL, "device %d out of range [0,%d)", device, count);
    e = hipSetDevice(device);
    if (e != hipSuccess) return moon_fail(nullptr, MOON_EHIP, "hipSetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return moon_fail(nullptr, MOON_EHIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0)
        return moon_fail(nullptr, MOON_ENODEVICE, "device %d is %s; the kernels are built for gfx950 only", device,
                         prop.gcnArchName);
    moon_ctx *ctx = new moon_ctx();
    if (const char *k = getenv("MOON_GEMM_KERNEL")) snprintf(ctx->gemm_kernel, sizeof ctx->gemm_kernel, "%s", k);
    ctx->device = device;
    ctx->cu_count = prop.multiProcessorCount;
    if ((e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess ||
        (e = hipEventCreate(&ctx->ev_start)) != hipSuccess || (e = hipEventCreate(&ctx->ev_stop)) != hipSuccess) {
        int rc = moon_fail(nullptr, MOON_EHIP, "stream/event creation: %s", hipGetErrorString(e));
        delete ctx;
        return rc;
    }
    if (int rc = decode_attention_static_init(ctx); rc != MOON_OK) { // the device is current here
        g_create_error = ctx->err;
        moon_ctx_destroy(ctx);
        return rc;
    }
    *out = ctx;
    return MOON_OK;
}

extern "C" void moon_cleanup(moon_ctx *ctx) {
    if (!ctx) return;
    std::lock_guard<std::mutex> lock(ctx->mu);
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &b : ctx->stage) {
        if (b.ptr) (void)hipFree(b.ptr);
        b = GrowBuf();
    }
    for (void *&p : ctx->pin_up) {
        if (p) (void)hipHostFree(p);
        p = nullptr;
    }
    if (ctx->pin_down) (void)hipHostFree(ctx->pin_down);
    ctx->pin_down = nullptr;
    for (auto &b : ctx->work) {
        if (b.ptr) (void)hipFree(b.ptr);
        b = GrowBuf();
    }
    // the per-head counters of the one-launch decode attention lived in work[1]: whatever is allocated next, at the same
    // address or not, starts from cleared counters
    ctx->attn_cnt_buf = nullptr;
    ctx->attn_cnt_heads = 0;
    ctx->attn_cnt_launches = 0;
}

extern "C" void moon_ctx_destroy(moon_ctx *ctx) {
    if (!ctx) return;
    moon_cleanup(ctx);
    for (auto &kv : ctx->resident) {
        (void)hipFree(kv.second.dptr);
        if (kv.second.dptr_t) (void)hipFree(kv.second.dptr_t);
    }
    ctx->resident.clear();
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

extern "C" int moon_set_gemm_kernel(moon_ctx *ctx, const char *name) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    static const char *const known[] = {"", "regs", "dma", "dma256", "w114", "w212", "w221"};
    if (!name) name = "";
    for (const char *k : known)
        if (!strcmp(name, k)) {
            snprintf(ctx->gemm_kernel, sizeof ctx->gemm_kernel, "%s", name);
            return MOON_OK;
        }
    return moon_fail(ctx, MOON_EINVAL, "moon_set_gemm_kernel: unknown kernel \"%s\"", name);
}

extern "C" const char *moon_last_kernel(const moon_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

extern "C" const char *moon_last_error(const moon_ctx *ctx) { return ctx ? ctx->err.c_str() : g_create_error.c_str(); }

extern "C" int moon_sync(moon_ctx *ctx) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

// ------------------------------------------------------------------ device memory
extern "C" int moon_dev_alloc(moon_ctx *ctx, size_t bytes, void **dptr) {
    if (!ctx || !dptr) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    *dptr = nullptr;
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    MOON_HIP(ctx, hipMalloc(dptr, bytes ? bytes : 1));
    return MOON_OK;
}

extern "C" int moon_dev_free(moon_ctx *ctx, void *dptr) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!dptr) return MOON_OK;
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    MOON_HIP(ctx, hipFree(dptr));
    return MOON_OK;
}

extern "C" int moon_dev_upload(moon_ctx *ctx, void *dptr, const void *host, size_t bytes) {
    if (!ctx || (!dptr && bytes) || (!host && bytes)) return moon_fail(ctx, MOON_EINVAL, "moon_dev_upload: null pointer");
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!bytes) return MOON_OK;
    MOON_HIP(ctx, hipMemcpyAsync(dptr, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

extern "C" int moon_dev_download(moon_ctx *ctx, void *host, const void *dptr, size_t bytes) {
    if (!ctx || (!dptr && bytes) || (!host && bytes)) return moon_fail(ctx, MOON_EINVAL, "moon_dev_download: null pointer");
    std::lock_guard<std::mutex> lock(ctx->mu);
    if (!bytes) return MOON_OK;
    MOON_HIP(ctx, hipMemcpyAsync(host, dptr, bytes, hipMemcpyDeviceToHost, ctx->stream));
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return MOON_OK;
}

// ------------------------------------------------------------------ resident weights
extern "C" int moon_weight_register(moon_ctx *ctx, const moon_f16 *host, size_t n_elems) {
    if (!ctx || !host || !n_elems) return moon_fail(ctx, MOON_EINVAL, "moon_weight_register: null or empty");
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->resident.find(host);
    if (it != ctx->resident.end()) {
        MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
        MOON_HIP(ctx, hipFree(it->second.dptr));
        if (it->second.dptr_t) MOON_HIP(ctx, hipFree(it->second.dptr_t));
        ctx->resident.erase(it);
    }
    void *d = nullptr;
    MOON_HIP(ctx, hipMalloc(&d, n_elems * sizeof(moon_f16)));
    hipError_t e = hipMemcpyAsync(d, host, n_elems * sizeof(moon_f16), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(d);
        return moon_fail(ctx, MOON_EHIP, "weight upload: %s", hipGetErrorString(e));
    }
    ctx->resident[host] = moon_ctx::Resident{d, n_elems};
    return MOON_OK;
}

extern "C" int moon_weight_unregister(moon_ctx *ctx, const moon_f16 *host) {
    if (!ctx || !host) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    auto it = ctx->resident.find(host);
    if (it == ctx->resident.end()) return moon_fail(ctx, MOON_EINVAL, "moon_weight_unregister: pointer was not registered");
    MOON_HIP(ctx, hipStreamSynchronize(ctx->stream));
    MOON_HIP(ctx, hipFree(it->second.dptr));
    if (it->second.dptr_t) MOON_HIP(ctx, hipFree(it->second.dptr_t));
    ctx->resident.erase(it);
    return MOON_OK;
}

// ------------------------------------------------------------------ timers
extern "C" int moon_timer_start(moon_ctx *ctx) {
    if (!ctx) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    MOON_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    return MOON_OK;
}

extern "C" int moon_timer_stop(moon_ctx *ctx, float *elapsed_ms) {
    if (!ctx || !elapsed_ms) return MOON_EINVAL;
    std::lock_guard<std::mutex> lock(ctx->mu);
    MOON_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    MOON_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
    MOON_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
    return MOON_OK;
}

// ------------------------------------------------------------------ synthetic data
// Counter-based generator: two splitmix64 words per element, the centred sum of their eight
// 16-bit fields (Irwin-Hall, integer exact) times one f32 scale, rounded to f16.  Integer
// arithmetic plus one IEEE multiply, so host and device produce identical bits.
__host__ __device__ static inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__host__ __device__ static inline uint64_t counter_word(uint64_t key, uint64_t ctr) {
    return mix64(key + 0x9E3779B97F4A7C15ull * (ctr + 1));
}
static inline uint64_t stream_key(uint64_t seed, uint64_t stream) {
    return mix64(mix64(seed + 0x9E3779B97F4A7C15ull) ^ (stream * 0xD1B54A32D192ED03ull + 0x2545F4914F6CDD1Dull));
}

__global__ void fill_normal_kernel(half_t *dst, size_t n, uint64_t key, float scale) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) {
        const uint64_t a = counter_word(key, 2 * i), b = counter_word(key, 2 * i + 1);
        uint32_t s = 0;
#pragma unroll
        for (int f = 0; f < 4; f++) {
            s += uint32_t((a >> (16 * f)) & 0xFFFF);
            s += uint32_t((b >> (16 * f)) & 0xFFFF);
        }
        const int32_t c = int32_t(s) - 262140;
        float f = float(c) * scale; // rounded to f32 first, then to f16, like the host generator
        asm volatile("" : "+v"(f));  // keeps the multiply from being folded into a single-rounding f16 convert
        dst[i] = (half_t)f;
    }
}

__global__ void fill_const_kernel(half_t *dst, size_t n, half_t v) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) dst[i] = v;
}

__global__ void fill_uniform_kernel(uint32_t *dst, size_t n, uint64_t key, uint32_t modulo) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) dst[i] = uint32_t((counter_word(key, i) >> 32) % modulo);
}

static inline unsigned fill_grid(size_t n) {
    size_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 16384 ? 16384 : g));
}

int launch_fill_normal(moon_ctx *ctx, half_t *dst, size_t n, uint64_t seed, uint64_t stream, float std_dev) {
    if (!n) return MOON_OK;
    const float scale = std_dev * (1.0f / 53510.105f);
    hipLaunchKernelGGL(fill_normal_kernel, dim3(fill_grid(n)), dim3(256), 0, ctx->stream, dst, n, stream_key(seed, stream), scale);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_fill_const(moon_ctx *ctx, half_t *dst, size_t n, float value) {
    if (!n) return MOON_OK;
    hipLaunchKernelGGL(fill_const_kernel, dim3(fill_grid(n)), dim3(256), 0, ctx->stream, dst, n, (half_t)value);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}
int launch_fill_uniform_u32(moon_ctx *ctx, uint32_t *dst, size_t n, uint64_t seed, uint64_t stream, uint32_t modulo) {
    if (!n) return MOON_OK;
    if (!modulo) return moon_fail(ctx, MOON_EINVAL, "fill_uniform: modulo is 0");
    hipLaunchKernelGGL(fill_uniform_kernel, dim3(fill_grid(n)), dim3(256), 0, ctx->stream, dst, n, stream_key(seed, stream), modulo);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// Plain device-to-device copy, 16 bytes per lane: reads n16 * 16 bytes and writes as many.  Besides its use as a copy
// it is the kernel of known traffic that hardware-counter readings are scaled against.
__global__ __launch_bounds__(256) void copy16_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

extern "C" int moon_dev_copy(moon_ctx *ctx, void *dst, const void *src, size_t bytes) {
    if (!ctx || ((!dst || !src) && bytes)) return moon_fail(ctx, MOON_EINVAL, "copy: null pointer");
    if (bytes % 16 || ((uintptr_t)dst | (uintptr_t)src) % 16) return moon_fail(ctx, MOON_EINVAL, "copy: pointers and size must be multiples of 16");
    if (!bytes) return MOON_OK;
    std::lock_guard<std::mutex> lock(ctx->mu);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    hipLaunchKernelGGL(copy16_kernel, dim3(fill_grid(bytes / 16)), dim3(256), 0, ctx->stream, (uint4 *)dst, (const uint4 *)src, bytes / 16);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

// Plain read of n16 * 16 bytes, eight 16-byte non-temporal loads in flight per lane, 1024 workgroups: what this device
// gives a kernel that does nothing but stream `bytes` from HBM in one launch -- the ceiling beside which a
// bandwidth-bound kernel of the same size is read.  The xor of everything lands in sink[0] only if it is a value that
// random data does not produce, so the loads stay and nothing is written.
typedef unsigned int read_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void read16_kernel(const read_u32x4 *__restrict__ src, size_t n16, uint32_t *sink) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        read_u32x4 v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = __builtin_nontemporal_load(src + i + k * stride);
#pragma unroll
        for (int k = 0; k < 8; k++) acc ^= v[k][0] ^ v[k][1] ^ v[k][2] ^ v[k][3];
    }
    for (; i < n16; i += stride) {
        const read_u32x4 v = __builtin_nontemporal_load(src + i);
        acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
    if (acc == 0x9e3779b9u && sink) sink[0] = acc;
}

extern "C" int moon_dev_read(moon_ctx *ctx, const void *src, size_t bytes, void *sink) {
    if (!ctx || (!src && bytes)) return moon_fail(ctx, MOON_EINVAL, "read: null pointer");
    if (bytes % 16 || (uintptr_t)src % 16) return moon_fail(ctx, MOON_EINVAL, "read: pointer and size must be multiples of 16");
    if (!bytes) return MOON_OK;
    std::lock_guard<std::mutex> lock(ctx->mu);
    MOON_HIP(ctx, hipSetDevice(ctx->device));
    const size_t n16 = bytes / 16, want = (n16 + 255) / 256;
    const unsigned grid = (unsigned)(want < 1024 ? want : 1024);
    hipLaunchKernelGGL(read16_kernel, dim3(grid), dim3(256), 0, ctx->stream, (const read_u32x4 *)src, n16, (uint32_t *)sink);
    MOON_HIP(ctx, hipGetLastError());
    return MOON_OK;
}

extern "C" int moon_dev_fill_normal_f16(moon_ctx *ctx, void *dptr, size_t n, uint64_t seed, uint64_t stream, float std_dev) {
    if (!ctx || (!dptr && n)) return moon_fail(ctx, MOON_EINVAL, "fill: null pointer");
    std::lock_guard<std::mutex> lock(ctx->mu);
    return launch_fill_normal(ctx, (half_t *)dptr, n, seed, stream, std_dev);
}
extern "C" int moon_dev_fill_const_f16(moon_ctx *ctx, void *dptr, size_t n, float value) {
    if (!ctx || (!dptr && n)) return moon_fail(ctx, MOON_EINVAL, "fill: null pointer");
    std::lock_guard<std::mutex> lock(ctx->mu);
    return launch_fill_const(ctx, (half_t *)dptr, n, value);
}
extern "C" int moon_dev_fill_uniform_u32(moon_ctx *ctx, void *dptr, size_t n, uint64_t seed, uint64_t stream, uint32_t modulo) {
    if (!ctx || (!dptr && n)) return moon_fail(ctx, MOON_EINVAL, "fill: null pointer");
    std::lock_guard<std::mutex> lock(ctx->mu);
    return launch_fill_uniform_u32(ctx, (uint32_t *)dptr, n, seed, stream, modulo);
}
