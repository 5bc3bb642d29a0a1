// Context, device memory and stream plumbing behind the C boundary.
#include "hm_common.h"
#include "attention.h"

#include <cstdlib>
#include <mutex>

static std::mutex g_err_mutex;
static std::string g_init_error;

int hm_set_error(hm_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    if (ctx) {
        ctx->last_error = buf;
    } else {
        std::lock_guard<std::mutex> g(g_err_mutex);
        g_init_error = buf;
    }
    return code;
}

extern "C" {

const char *hm_version(void) { return "homura_amd 0.1 (gfx950)"; }

hm_ctx *hm_init(int device) {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        hm_set_error(nullptr, HM_ERR_HIP, "no HIP device available: %s",
                     e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        return nullptr;
    }
    if (device < 0 || device >= count) {
        hm_set_error(nullptr, HM_ERR_INVALID, "device %d out of range (have %d)", device, count);
        return nullptr;
    }
    if ((e = hipSetDevice(device)) != hipSuccess) {
        hm_set_error(nullptr, HM_ERR_HIP, "hipSetDevice: %s", hipGetErrorString(e));
        return nullptr;
    }
    hm_ctx *ctx = new hm_ctx();
    ctx->device = device;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) {
        ctx->num_cus = prop.multiProcessorCount;
        snprintf(ctx->device_name, sizeof(ctx->device_name), "%s (%s)", prop.name,
                 prop.gcnArchName);
    }
    // Default priority on purpose.
    if ((e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess) {
        hm_set_error(nullptr, HM_ERR_HIP, "hipStreamCreate: %s", hipGetErrorString(e));
        delete ctx;
        return nullptr;
    }
    ctx->workspace_bytes = (size_t)64 << 20;
    ctx->num_counters = 4096;
    if (hipMalloc(&ctx->workspace, ctx->workspace_bytes) != hipSuccess ||
        hipMalloc((void **)&ctx->counters, ctx->num_counters * sizeof(unsigned int)) !=
            hipSuccess) {
        hm_set_error(nullptr, HM_ERR_OOM, "workspace allocation failed");
        hm_destroy(ctx);
        return nullptr;
    }
    (void)hipMemsetAsync(ctx->counters, 0, ctx->num_counters * sizeof(unsigned int), ctx->stream);
    (void)hipStreamSynchronize(ctx->stream);
    if (gqa_attn_fixed_scratch_setup(ctx) != HM_OK) {
        hm_set_error(nullptr, HM_ERR_HIP, "%s", ctx->last_error.c_str());
        hm_destroy(ctx);
        return nullptr;
    }
    return ctx;
}

void hm_destroy(hm_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->counters) (void)hipFree(ctx->counters);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char *hm_last_error(hm_ctx *ctx) {
    if (ctx) return ctx->last_error.c_str();
    std::lock_guard<std::mutex> g(g_err_mutex);
    return g_init_error.c_str();
}

int hm_alloc(hm_ctx *ctx, size_t bytes, void **d_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, d_out != nullptr, "hm_alloc: d_out is NULL");
    *d_out = nullptr;
    if (bytes == 0) bytes = 16;  // zero-size tensors still get a valid pointer
    hipError_t e = hipMalloc(d_out, bytes);
    if (e != hipSuccess)
        return hm_set_error(ctx, HM_ERR_OOM, "hipMalloc(%zu) failed: %s", bytes,
                            hipGetErrorString(e));
    // HOMURA_ALLOC_FILL=<byte>: every new allocation starts filled with that byte (0xFF makes every float a
    // NaN), so that a kernel which reads memory nobody wrote shows in the results. For tests.
    static const int fill = [] {
        const char *v = std::getenv("HOMURA_ALLOC_FILL");
        return v ? (int)(std::strtol(v, nullptr, 0) & 0xFF) : -1;
    }();
    if (fill >= 0) HM_HIP(ctx, hipMemsetAsync(*d_out, fill, bytes, ctx->stream));
    return HM_OK;
}

int hm_free(hm_ctx *ctx, void *d_ptr) {
    HM_CHECK_CTX(ctx);
    if (!d_ptr) return HM_OK;
    HM_HIP(ctx, hipStreamSynchronize(ctx->stream));
    HM_HIP(ctx, hipFree(d_ptr));
    return HM_OK;
}

int hm_upload(hm_ctx *ctx, void *d_dst, const void *h_src, size_t bytes) {
    HM_CHECK_CTX(ctx);
    if (bytes == 0) return HM_OK;
    HM_REQUIRE(ctx, d_dst && h_src, "hm_upload: NULL pointer");
    HM_HIP(ctx, hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HM_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return HM_OK;
}

int hm_download(hm_ctx *ctx, void *h_dst, const void *d_src, size_t bytes) {
    HM_CHECK_CTX(ctx);
    if (bytes == 0) return HM_OK;
    HM_REQUIRE(ctx, h_dst && d_src, "hm_download: NULL pointer");
    HM_HIP(ctx, hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HM_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return HM_OK;
}

int hm_copy(hm_ctx *ctx, void *d_dst, const void *d_src, size_t bytes) {
    HM_CHECK_CTX(ctx);
    if (bytes == 0) return HM_OK;
    HM_REQUIRE(ctx, d_dst && d_src, "hm_copy: NULL pointer");
    HM_HIP(ctx, hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return HM_OK;
}

__global__ void fill_zero_kernel(uint32_t *p, size_t n_words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n_words; i += stride) p[i] = 0u;
}

int hm_fill_zero(hm_ctx *ctx, void *d_dst, size_t bytes) {
    HM_CHECK_CTX(ctx);
    if (bytes == 0) return HM_OK;
    HM_REQUIRE(ctx, d_dst != nullptr, "hm_fill_zero: NULL pointer");
    HM_REQUIRE(ctx, bytes % 4 == 0 && ((uintptr_t)d_dst % 4) == 0,
               "hm_fill_zero: pointer and size must be 4-byte aligned");
    size_t words = bytes / 4;
    int blocks = (int)((words + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, ctx->stream, (uint32_t *)d_dst,
                       words);
    HM_LAUNCH_CHECK(ctx);
    return HM_OK;
}

int hm_sync(hm_ctx *ctx) {
    HM_CHECK_CTX(ctx);
    HM_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return HM_OK;
}

void *hm_stream(hm_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int hm_device_name(hm_ctx *ctx, char *buf, size_t buflen) {
    HM_CHECK_CTX(ctx);
    if (!buf || buflen == 0) return HM_ERR_INVALID;
    snprintf(buf, buflen, "%s", ctx->device_name);
    return HM_OK;
}

// ── stream capture: callers with launch-bound inner loops record them once and replay ──

struct hm_graph_handle {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

int hm_graph_begin(hm_ctx *ctx) {
    HM_CHECK_CTX(ctx);
    HM_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    return HM_OK;
}

int hm_graph_end(hm_ctx *ctx, void **graph_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, graph_out != nullptr, "hm_graph_end: graph_out is NULL");
    *graph_out = nullptr;
    hipGraph_t g = nullptr;
    HM_HIP(ctx, hipStreamEndCapture(ctx->stream, &g));
    hm_graph_handle *h = new hm_graph_handle();
    h->graph = g;
    hipError_t e = hipGraphInstantiate(&h->exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        delete h;
        return hm_set_error(ctx, HM_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    *graph_out = h;
    return HM_OK;
}

int hm_graph_launch(hm_ctx *ctx, void *graph, int reps) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, graph != nullptr && reps >= 1, "hm_graph_launch: bad arguments");
    hm_graph_handle *h = (hm_graph_handle *)graph;
    for (int i = 0; i < reps; i++) HM_HIP(ctx, hipGraphLaunch(h->exec, ctx->stream));
    return HM_OK;
}

int hm_graph_destroy(hm_ctx *ctx, void *graph) {
    HM_CHECK_CTX(ctx);
    if (!graph) return HM_OK;
    hm_graph_handle *h = (hm_graph_handle *)graph;
    HM_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (h->exec) (void)hipGraphExecDestroy(h->exec);
    if (h->graph) (void)hipGraphDestroy(h->graph);
    delete h;
    return HM_OK;
}

int hm_event_create(hm_ctx *ctx, void **ev_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, ev_out != nullptr, "hm_event_create: ev_out is NULL");
    hipEvent_t ev;
    HM_HIP(ctx, hipEventCreate(&ev));
    *ev_out = (void *)ev;
    return HM_OK;
}

int hm_event_destroy(hm_ctx *ctx, void *ev) {
    HM_CHECK_CTX(ctx);
    if (ev) HM_HIP(ctx, hipEventDestroy((hipEvent_t)ev));
    return HM_OK;
}

int hm_event_record(hm_ctx *ctx, void *ev) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, ev != nullptr, "hm_event_record: NULL event");
    HM_HIP(ctx, hipEventRecord((hipEvent_t)ev, ctx->stream));
    return HM_OK;
}

int hm_event_elapsed_ms(hm_ctx *ctx, void *ev_start, void *ev_stop, float *ms_out) {
    HM_CHECK_CTX(ctx);
    HM_REQUIRE(ctx, ev_start && ev_stop && ms_out, "hm_event_elapsed_ms: NULL argument");
    HM_HIP(ctx, hipEventSynchronize((hipEvent_t)ev_stop));
    HM_HIP(ctx, hipEventElapsedTime(ms_out, (hipEvent_t)ev_start, (hipEvent_t)ev_stop));
    return HM_OK;
}

}  // extern "C"
