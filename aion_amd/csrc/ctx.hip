// Context, device memory and event helpers of libaion_hip.so: the C side of aion's
// Backend / Session / DeviceMemory vtables (backend/backend.zig:24-107,
// runtime/device_memory.zig:36-108).
#include "common.h"

#include <cxxabi.h>
#include <string>
#include <algorithm>

#include <cstring>
#include <mutex>
#include <new>

// Scratch for aionhip_step_matmul_static, the entry point that may not allocate: one copy per GPU the library runs on,
// held until the process ends. The name below is a host-side stand-in, not a device address: host code uses the
// address hipGetSymbolAddress returns for the current device (kept per device in g_static_scratch), never the name.
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
static std::mutex g_static_scratch_mutex;
static void *g_static_scratch[64];

// the current device's address of the array; looked up once per device, with that device current
static hipError_t static_scratch_address(int device, void **out) {
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    const bool cached = device >= 0 && device < 64;
    if (cached && g_static_scratch[device]) {
        *out = g_static_scratch[device];
        return hipSuccess;
    }
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    if (cached) g_static_scratch[device] = ptr;
    *out = ptr;
    return hipSuccess;
}

int set_err(aionhip_ctx *ctx, int status, const char *fmt, ...) {
    if (ctx) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        ctx->err = buf;
    }
    return status;
}

static void pool_release_cached(aionhip_ctx *ctx);

// Every internal device allocation goes through here: when the device is out of memory the pool's cached blocks are
// given back and the request is tried once more (not while a program is being recorded: releasing waits for the stream).
int dev_malloc(aionhip_ctx *ctx, void **out, size_t bytes, const char *what) {
    *out = nullptr;
    hipError_t e = hipMalloc(out, bytes);
    if (e == hipErrorOutOfMemory && ctx->pool_cached_bytes && !ctx->capturing) {
        (void)hipGetLastError();
        pool_release_cached(ctx);
        e = hipMalloc(out, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out = nullptr;
        return set_err(ctx, e == hipErrorOutOfMemory ? AIONHIP_OUT_OF_MEMORY : AIONHIP_EXECUTION_FAILED, "hipMalloc(%zu) for %s: %s", bytes, what, hipGetErrorString(e));
    }
    return AIONHIP_OK;
}

// Context-owned work buffers (prepared activations, GEMM staging, K-split meeting words, argmax tickets) grow by
// replacement. A recorded program holds the old address in its launches, so every replacement moves the context's
// buffer generation on and aionhip_program_execute refuses a program recorded under an earlier one.
int grow_work_buffer(aionhip_ctx *ctx, void **buf, size_t *have, size_t bytes, bool zeroed, const char *what) {
    if (bytes <= *have) return AIONHIP_OK;
    if (ctx->capturing)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s must grow to %zu bytes while a program is being recorded: run the steps once before recording", what, bytes);
    if (*buf) {
        // earlier launches may still read the old buffer
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        HIP_TRY(ctx, hipFree(*buf));
        *buf = nullptr;
        *have = 0;
        ctx->buffer_generation++;
    }
    size_t want = bytes + bytes / 4;
    want = (want + 4095) & ~(size_t)4095;
    int rc = dev_malloc(ctx, buf, want, what);
    if (rc) return rc;
    *have = want;
    if (zeroed) HIP_TRY(ctx, hipMemsetAsync(*buf, 0, want, ctx->stream));          // never inside a recording (checked above)
    return AIONHIP_OK;
}
int ensure_scratch(aionhip_ctx *ctx, size_t bytes) { return grow_work_buffer(ctx, &ctx->scratch, &ctx->scratch_bytes, bytes, false, "scratch"); }
int ensure_scratch2(aionhip_ctx *ctx, size_t bytes) { return grow_work_buffer(ctx, &ctx->scratch2, &ctx->scratch2_bytes, bytes, false, "GEMM staging"); }

static hipEvent_t take_event(aionhip_ctx *ctx) {
    if (!ctx->event_pool.empty()) {
        hipEvent_t e = ctx->event_pool.back();
        ctx->event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}
void prof_open(aionhip_ctx *ctx, hipEvent_t *start, hipEvent_t *stop) {
    ProfRecord r{ctx->prof_name, take_event(ctx), take_event(ctx), 0.f};
    ctx->prof.push_back(r);
    *start = r.start;
    *stop = r.stop;
}

int rope_table(aionhip_ctx *ctx, int pairs, float freq_step, float scale_factor, const float **out) {
    for (const auto &t : ctx->rope_tables)
        if (t.pairs == pairs && t.freq_step == freq_step && t.scale_factor == scale_factor) {
            *out = t.freq;
            return AIONHIP_OK;
        }
    if (ctx->capturing)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "a RoPE table cannot be built while a program is being recorded: run the steps once before recording");
    std::vector<float> host((size_t)(pairs > 0 ? pairs : 1));
    float f = scale_factor;
    for (int i = 0; i < pairs; ++i) {
        host[(size_t)i] = f;
        f *= freq_step;
    }
    void *dev = nullptr;
    const int rc = dev_malloc(ctx, &dev, host.size() * sizeof(float), "RoPE table");
    if (rc) return rc;
    hipError_t e = hipMemcpyAsync(dev, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return set_err(ctx, AIONHIP_EXECUTION_FAILED, "rope table upload: %s", hipGetErrorString(e));
    }
    ctx->rope_tables.push_back({pairs, freq_step, scale_factor, (float *)dev});
    *out = (const float *)dev;
    return AIONHIP_OK;
}

extern "C" {

int aionhip_set_attention_precise(aionhip_ctx *ctx, int on) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    ctx->attn_precise = on != 0;
    return AIONHIP_OK;
}

int aionhip_profile_start(aionhip_ctx *ctx) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    for (auto &r : ctx->prof) {
        ctx->event_pool.push_back(r.start);
        ctx->event_pool.push_back(r.stop);
    }
    ctx->prof.clear();
    ctx->profiling = true;
    return AIONHIP_OK;
}
int aionhip_profile_stop(aionhip_ctx *ctx, size_t *count) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    ctx->profiling = false;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    for (auto &r : ctx->prof) HIP_TRY(ctx, hipEventElapsedTime(&r.ms, r.start, r.stop));
    if (count) *count = ctx->prof.size();
    return AIONHIP_OK;
}
int aionhip_profile_entry(aionhip_ctx *ctx, size_t index, const char **name, float *ms) {
    if (!ctx || index >= ctx->prof.size()) return AIONHIP_INVALID_ARGUMENT;
    if (name) *name = ctx->prof[index].name;
    if (ms) *ms = ctx->prof[index].ms;
    return AIONHIP_OK;
}

const char *aionhip_name(void) { return "hip-gfx950"; }

int aionhip_create(int device, void *stream, aionhip_ctx **out) {
    if (!out) return AIONHIP_INVALID_ARGUMENT;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) return AIONHIP_UNSUPPORTED;
    if (hipSetDevice(device) != hipSuccess) return AIONHIP_EXECUTION_FAILED;
    aionhip_ctx *ctx = new (std::nothrow) aionhip_ctx();
    if (!ctx) return AIONHIP_OUT_OF_MEMORY;
    ctx->device = device;
    if (stream) {
        ctx->stream = (hipStream_t)stream;
    } else {
        if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
            delete ctx;
            return AIONHIP_EXECUTION_FAILED;
        }
        ctx->own_stream = true;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->cu_count = prop.multiProcessorCount;
    if (static_scratch_address(device, &ctx->static_scratch) != hipSuccess) {
        if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return AIONHIP_EXECUTION_FAILED;
    }
    *out = ctx;
    return AIONHIP_OK;
}

void aionhip_destroy(aionhip_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &r : ctx->prof) {
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    for (auto e : ctx->event_pool) (void)hipEventDestroy(e);
    for (auto &t : ctx->rope_tables) (void)hipFree(t.freq);
    for (auto &kv : ctx->bf16_copies) (void)hipFree(kv.second.first);
    if (ctx->scratch) (void)hipFree(ctx->scratch);
    if (ctx->scratch2) (void)hipFree(ctx->scratch2);
    if (ctx->ksplit) (void)hipFree(ctx->ksplit);
    if (ctx->tickets) (void)hipFree(ctx->tickets);
    pool_release_cached(ctx);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

int aionhip_sync(aionhip_ctx *ctx) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return AIONHIP_OK;
}

const char *aionhip_last_error(aionhip_ctx *ctx) { return ctx ? ctx->err.c_str() : "no context"; }
const char *aionhip_last_kernel(aionhip_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

int aionhip_last_launch(aionhip_ctx *ctx, char *instance, size_t instance_len, unsigned grid[3], unsigned block[3], size_t *lds_bytes) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!ctx->last_fn) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "last_launch: no kernel has been launched on this context");
    if (instance && instance_len) {
        // the device function's name as a kernel trace prints it: demangled, without the parameter list
        const char *mangled = hipKernelNameRefByPtr(ctx->last_fn, ctx->stream);
        (void)hipGetLastError();
        int status = -1;
        char *plain = mangled ? abi::__cxa_demangle(mangled, nullptr, nullptr, &status) : nullptr;
        std::string name = status == 0 && plain ? plain : (mangled ? mangled : "");
        free(plain);
        // cut "(args...)" of the outermost call: the last '(' at template depth 0
        int depth = 0;
        size_t cut = std::string::npos;
        for (size_t i = 0; i < name.size(); ++i) {
            const char ch = name[i];
            if (ch == '<') ++depth;
            else if (ch == '>') --depth;
            else if (ch == '(' && depth == 0 && name.compare(i, 21, "(anonymous namespace)") != 0) { cut = i; break; }
        }
        if (cut != std::string::npos) name.resize(cut);
        if (name.rfind("void ", 0) == 0) name.erase(0, 5);
        snprintf(instance, instance_len, "%s", name.c_str());
    }
    for (int i = 0; i < 3; ++i) {
        if (grid) grid[i] = ctx->last_grid[i];
        if (block) block[i] = ctx->last_block[i];
    }
    if (lds_bytes) *lds_bytes = ctx->last_lds;
    return AIONHIP_OK;
}
void *aionhip_stream(aionhip_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int aionhip_set_gemm_mode(aionhip_ctx *ctx, int mode) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (mode != AIONHIP_GEMM_EXACT_I8 && mode != AIONHIP_GEMM_BF16_MFMA && mode != AIONHIP_GEMM_BF16_MFMA_ALWAYS) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "unknown gemm mode %d", mode);
    ctx->gemm_mode = mode;
    return AIONHIP_OK;
}

int aionhip_device_info(aionhip_ctx *ctx, int *cu_count, int *wave_size, uint64_t *hbm_bytes, char *arch, size_t arch_len) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    hipDeviceProp_t prop;
    HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (wave_size) *wave_size = prop.warpSize;
    if (hbm_bytes) *hbm_bytes = (uint64_t)prop.totalGlobalMem;
    if (arch && arch_len) {
        std::strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return AIONHIP_OK;
}

// Size classes of the pool: multiples of an eighth of the power of two below the request (at least 256 bytes), so a
// block is at most 12.5 % larger than asked for and requests that differ a little share a class.
static size_t pool_class(size_t bytes) {
    if (bytes < 256) return 256;
    if (bytes > aionhip_ctx::POOL_MAX_BLOCK) return (bytes + 255) & ~(size_t)255;      // never cached: no class to share, no padding to pay
    size_t p2 = 256;
    while (p2 <= bytes / 2) p2 <<= 1;                      // largest power of two <= bytes
    const size_t step = p2 / 8 < 256 ? 256 : p2 / 8;
    return (bytes + step - 1) / step * step;
}

static void pool_release_cached(aionhip_ctx *ctx) {
    if (ctx->pool_cached_bytes == 0) return;
    (void)hipStreamSynchronize(ctx->stream);               // cached blocks may still be read by work in flight
    for (auto &kv : ctx->pool_free)
        for (void *p : kv.second) (void)hipFree(p);
    ctx->pool_free.clear();
    ctx->pool_cached_bytes = 0;
}

int aionhip_alloc(aionhip_ctx *ctx, size_t bytes, size_t alignment, aionhip_handle *out) {
    if (!ctx || !out) return AIONHIP_INVALID_ARGUMENT;
    *out = 0;
    if (alignment > 1 && (alignment & (alignment - 1)) != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "alignment %zu is not a power of two", alignment);
    const size_t cls = pool_class(bytes);
    void *p = nullptr;
    auto it = ctx->pool_free.find(cls);
    if (it != ctx->pool_free.end()) {
        // a cached block of this class that also meets the alignment (hipMalloc aligns to 256 bytes and in practice to pages)
        auto &v = it->second;
        for (size_t i = v.size(); i-- > 0;) {
            if (alignment <= 1 || ((uintptr_t)v[i] % alignment) == 0) {
                p = v[i];
                v.erase(v.begin() + (long)i);
                ctx->pool_cached_bytes -= cls;
                break;
            }
        }
        if (v.empty()) ctx->pool_free.erase(it);
    }
    if (!p) {
        const int rc = dev_malloc(ctx, &p, cls, "aionhip_alloc");
        if (rc) return rc;
        if (alignment > 1 && ((uintptr_t)p % alignment) != 0) {
            (void)hipFree(p);
            return set_err(ctx, AIONHIP_UNSUPPORTED, "cannot satisfy alignment %zu", alignment);
        }
    }
    ctx->pool_live[p] = cls;
    ctx->pool_live_bytes += cls;
    *out = (aionhip_handle)(uintptr_t)p;
    return AIONHIP_OK;
}

void aionhip_free(aionhip_ctx *ctx, aionhip_handle h) {
    if (!ctx || !h) return;
    void *p = (void *)(uintptr_t)h;
    auto it = ctx->pool_live.find(p);
    if (it == ctx->pool_live.end()) {                      // not from aionhip_alloc of this context: plain release
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(p);
        return;
    }
    const size_t cls = it->second;
    ctx->pool_live.erase(it);
    ctx->pool_live_bytes -= cls;
    if (cls <= aionhip_ctx::POOL_MAX_BLOCK) {
        ctx->pool_free[cls].push_back(p);
        ctx->pool_cached_bytes += cls;
    } else {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(p);
    }
}

int aionhip_trim(aionhip_ctx *ctx) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "trim waits for the stream and cannot be recorded into a program");
    pool_release_cached(ctx);
    return AIONHIP_OK;
}

int aionhip_memory_stats(aionhip_ctx *ctx, uint64_t *live_bytes, uint64_t *cached_bytes) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (live_bytes) *live_bytes = (uint64_t)ctx->pool_live_bytes;
    if (cached_bytes) *cached_bytes = (uint64_t)ctx->pool_cached_bytes;
    return AIONHIP_OK;
}

int aionhip_h2d(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, const void *src, size_t bytes) {
    if (!ctx || !dst || (!src && bytes)) return AIONHIP_INVALID_ARGUMENT;
    if (!bytes) return AIONHIP_OK;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "h2d synchronises and cannot be recorded into a program");
    // pageable source: hipMemcpyAsync stages and returns once `src` is consumed
    HIP_TRY(ctx, hipMemcpyAsync((char *)(uintptr_t)dst + dst_offset, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return AIONHIP_OK;
}

int aionhip_d2h(aionhip_ctx *ctx, void *dst, aionhip_handle src, size_t src_offset, size_t bytes) {
    if (!ctx || !src || (!dst && bytes)) return AIONHIP_INVALID_ARGUMENT;
    if (!bytes) return AIONHIP_OK;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "d2h synchronises and cannot be recorded into a program");
    HIP_TRY(ctx, hipMemcpyAsync(dst, (const char *)(uintptr_t)src + src_offset, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return AIONHIP_OK;
}

int aionhip_d2d(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, aionhip_handle src, size_t src_offset, size_t bytes) {
    if (!ctx || !dst || !src) return AIONHIP_INVALID_ARGUMENT;
    if (!bytes) return AIONHIP_OK;
    HIP_TRY(ctx, hipMemcpyAsync((char *)(uintptr_t)dst + dst_offset, (const char *)(uintptr_t)src + src_offset, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return AIONHIP_OK;
}

__global__ void fill_bytes_kernel(uint8_t *p, uint8_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

int aionhip_memset(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, int value, size_t bytes) {
    if (!ctx || !dst) return AIONHIP_INVALID_ARGUMENT;
    if (!bytes) return AIONHIP_OK;
    // a fill kernel rather than hipMemsetAsync so that the call can sit inside a captured graph
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fill_bytes_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((uint8_t *)(uintptr_t)dst + dst_offset, (uint8_t)value, bytes);
    LAUNCH_CHECK(ctx, "fill_bytes");
    return AIONHIP_OK;
}

int aionhip_event_create(aionhip_ctx *ctx, void **event) {
    if (!ctx || !event) return AIONHIP_INVALID_ARGUMENT;
    hipEvent_t e;
    HIP_TRY(ctx, hipEventCreate(&e));
    *event = (void *)e;
    return AIONHIP_OK;
}
int aionhip_event_record(aionhip_ctx *ctx, void *event) {
    if (!ctx || !event) return AIONHIP_INVALID_ARGUMENT;
    HIP_TRY(ctx, hipEventRecord((hipEvent_t)event, ctx->stream));
    return AIONHIP_OK;
}
int aionhip_event_elapsed_ms(aionhip_ctx *ctx, void *start, void *stop, float *ms) {
    if (!ctx || !start || !stop || !ms) return AIONHIP_INVALID_ARGUMENT;
    HIP_TRY(ctx, hipEventSynchronize((hipEvent_t)stop));
    HIP_TRY(ctx, hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return AIONHIP_OK;
}
void aionhip_event_destroy(aionhip_ctx *ctx, void *event) {
    (void)ctx;
    if (event) (void)hipEventDestroy((hipEvent_t)event);
}

}  // extern "C"
