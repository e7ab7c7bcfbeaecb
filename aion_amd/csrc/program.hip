// Programs: a fixed sequence of steps recorded once and replayed per token.
//
// aion compiles a model into an ExecutableProgram (a step list, runtime/executable.zig) and its
// WebGPU backend caches and replays the per-step dispatch state because a decode program is
// identical every token (backend/gpu/frame.zig:77-86, backend/gpu/backend.zig:616-638). Here the
// replayable form is a HIP graph: between aionhip_program_begin and aionhip_program_end the
// ordinary aionhip_step_* calls are captured instead of executed. Everything that varies per token
// (token id, positions, cache write index, kv length) lives in device buffers the steps read, so
// the same graph is valid for every token.
#include "common.h"

#include <new>

struct aionhip_program {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    size_t nodes = 0;
    uint64_t buffer_generation = 0;     // the context's work-buffer generation the launches were recorded under
};

namespace {
__global__ void add_i32_kernel(int *__restrict__ out, const int *__restrict__ a, const int *__restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}
struct AdvanceArgs {
    int *counter[8];
    int count;
};
// the loop state of a device-resident greedy decode in one launch: the produced token becomes the next input, the indices move on
// log (optional, n <= 64 so that one wavefront does everything): log[*log_index + i] = src[i], *log_index read before any
// counter moves (it may be one of them: the position a token was produced at)
__global__ void advance_state_kernel(int *__restrict__ dst, const int *__restrict__ src, size_t n, AdvanceArgs a, int delta,
                                     int *__restrict__ log, const int *__restrict__ log_index, int log_capacity) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    int at = -1;
    if (log) at = *log_index;
    if (i < n) {
        const int t = src[i];
        dst[i] = t;
        if (log && at >= 0 && (long)at + (long)i < (long)log_capacity) log[(size_t)at + i] = t;
    }
    __builtin_amdgcn_s_waitcnt(0);                  // the index has been read before a counter that may alias it moves
    if (blockIdx.x == 0 && (int)threadIdx.x < a.count) *a.counter[threadIdx.x] += delta;
}
}  // namespace

extern "C" {

int aionhip_step_advance_state(aionhip_ctx *ctx, aionhip_handle dst_tokens, aionhip_handle src_tokens, size_t n_tokens,
                               const aionhip_handle *counters, size_t n_counters, int delta) {
    return aionhip_step_advance_state_log(ctx, dst_tokens, src_tokens, n_tokens, counters, n_counters, delta, 0, 0, 0);
}

int aionhip_step_advance_state_log(aionhip_ctx *ctx, aionhip_handle dst_tokens, aionhip_handle src_tokens, size_t n_tokens,
                                   const aionhip_handle *counters, size_t n_counters, int delta,
                                   aionhip_handle log, aionhip_handle log_index, size_t log_capacity) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (log && (!log_index || (log & 3) || (log_index & 3) || n_tokens > 64 || log_capacity > 0x7FFFFFFFu))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "advance_state: a token log needs an aligned index, at most 64 tokens per step and a capacity below 2^31");
    if (n_counters > 8 || (n_counters && !counters) || (n_tokens && (!dst_tokens || !src_tokens)))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "advance_state: null operand or more than 8 counters");
    if (!n_tokens && !n_counters) return AIONHIP_OK;
    AdvanceArgs a{};
    a.count = (int)n_counters;
    for (size_t i = 0; i < n_counters; ++i) {
        if (!counters[i] || (counters[i] & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "advance_state: null or misaligned counter");
        for (size_t j = 0; j < i; ++j)
            if (counters[j] == counters[i]) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "advance_state: a counter is listed twice");
        a.counter[i] = (int *)(uintptr_t)counters[i];
    }
    const size_t blocks = n_tokens ? (n_tokens + 63) / 64 : 1;
    advance_state_kernel<<<dim3((unsigned)blocks), dim3(64), 0, ctx->stream>>>((int *)(uintptr_t)dst_tokens, (const int *)(uintptr_t)src_tokens, n_tokens, a, delta,
                                                                                    (int *)(uintptr_t)log, (const int *)(uintptr_t)log_index, (int)log_capacity);
    LAUNCH_CHECK(ctx, "advance_state");
    return AIONHIP_OK;
}

int aionhip_program_begin(aionhip_ctx *ctx) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "program_begin: already recording");
    if (ctx->profiling) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "program_begin: stop profiling first (events cannot be captured)");
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return AIONHIP_OK;
}

int aionhip_program_end(aionhip_ctx *ctx, aionhip_program **out) {
    if (!ctx || !out) return AIONHIP_INVALID_ARGUMENT;
    *out = nullptr;
    if (!ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "program_end: not recording");
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess || !graph) return set_err(ctx, AIONHIP_EXECUTION_FAILED, "hipStreamEndCapture: %s", hipGetErrorString(e));
    aionhip_program *p = new (std::nothrow) aionhip_program();
    if (!p) {
        (void)hipGraphDestroy(graph);
        return set_err(ctx, AIONHIP_OUT_OF_MEMORY, "host allocation failed");
    }
    p->graph = graph;
    p->buffer_generation = ctx->buffer_generation;
    (void)hipGraphGetNodes(graph, nullptr, &p->nodes);
    e = hipGraphInstantiate(&p->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        delete p;
        return set_err(ctx, AIONHIP_EXECUTION_FAILED, "hipGraphInstantiate: %s", hipGetErrorString(e));
    }
    *out = p;
    return AIONHIP_OK;
}

int aionhip_program_abort(aionhip_ctx *ctx) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!ctx->capturing) return AIONHIP_OK;
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(ctx->stream, &graph);      // also when a step failed mid-recording
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipGetLastError();                                            // an invalidated capture leaves a sticky error behind
    if (e != hipSuccess && e != hipErrorStreamCaptureInvalidated) return set_err(ctx, AIONHIP_EXECUTION_FAILED, "hipStreamEndCapture: %s", hipGetErrorString(e));
    return AIONHIP_OK;
}

int aionhip_program_execute(aionhip_ctx *ctx, aionhip_program *prog) {
    if (!ctx || !prog || !prog->exec) return AIONHIP_INVALID_ARGUMENT;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "program_execute: a recording is open");
    if (prog->buffer_generation != ctx->buffer_generation)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "program_execute: stale program - a work buffer of the context was replaced by a larger one after this program "
                                                      "was recorded (a later step needed more scratch); re-record it");
    HIP_TRY(ctx, hipGraphLaunch(prog->exec, ctx->stream));
    return AIONHIP_OK;
}

size_t aionhip_program_node_count(const aionhip_program *prog) { return prog ? prog->nodes : 0; }

int aionhip_program_is_current(const aionhip_ctx *ctx, const aionhip_program *prog) {
    return ctx && prog && prog->exec && prog->buffer_generation == ctx->buffer_generation ? 1 : 0;
}

void aionhip_program_destroy(aionhip_ctx *ctx, aionhip_program *prog) {
    if (!prog) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (prog->exec) (void)hipGraphExecDestroy(prog->exec);
    if (prog->graph) (void)hipGraphDestroy(prog->graph);
    delete prog;
}

int aionhip_step_add_i32(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !a || !b) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "add_i32: null operand");
    if (!n) return AIONHIP_OK;
    add_i32_kernel<<<dim3((unsigned)((n + 63) / 64)), dim3(64), 0, ctx->stream>>>((int *)(uintptr_t)out, (const int *)(uintptr_t)a, (const int *)(uintptr_t)b, n);
    LAUNCH_CHECK(ctx, "add_i32");
    return AIONHIP_OK;
}

}  // extern "C"
