// context.hip — bridge lifecycle, device buffers, events, workspace, synthetic-data fills.
// Interface style after the reference's C-ABI (bridge/ane_bridge.h:11-98, bridge/ane_bridge.m:33-57,
// 233-251): idempotent init returning 0/-1, opaque handles, NULL-safe frees, one stderr line per error.
#include "common.h"

#include <stdarg.h>
#include <stdlib.h>

Mi355Ctx g_ctx = {};
static char g_err[512] = "";

int mi355_fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    fprintf(stderr, "mi355_bridge: %s\n", g_err);
    return -1;
}

bool mi355_ready(const char *who) {
    if (g_ctx.ready) return true;
    if (mi355_init() == 0) return true;
    mi355_fail("%s: no usable GPU (mi355_init failed)", who);
    return false;
}

bool mi355_outside_capture(const char *who) {
    if (!g_ctx.capturing) return true;
    mi355_fail("%s: not possible while a graph is being captured (it allocates, copies to the host or waits); "
               "run the sequence once before capturing so that workspaces and tables exist", who);
    return false;
}

void *mi355_ws(size_t bytes) {
    if (bytes <= g_ctx.ws_bytes && g_ctx.ws) return g_ctx.ws;
    if (!mi355_outside_capture("workspace growth")) return nullptr;
    size_t want = (bytes + 0xFFFFF) & ~(size_t)0xFFFFF;   // 1 MiB granules
    if (g_ctx.ws) {
        (void)hipStreamSynchronize(g_ctx.stream);
        (void)hipFree(g_ctx.ws);
        g_ctx.ws = nullptr;
        g_ctx.ws_bytes = 0;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
        mi355_fail("workspace hipMalloc(%zu): %s", want, hipGetErrorString(e));
        return nullptr;
    }
    g_ctx.ws = p;
    g_ctx.ws_bytes = want;
    g_ctx.alloc_epoch++;
    return p;
}

static Mi355Exchange g_xch = {nullptr, nullptr, nullptr};

bool mi355_exchange(Mi355Exchange *out) {
    if (!g_xch.slots) {
        if (!mi355_outside_capture("first use of a kernel whose workgroups exchange partial results (its exchange area "
                                   "is allocated)"))
            return false;
        const size_t slot_b = (size_t)XCH_MAX_BLOCKS * XCH_SLOT_STRIDE * sizeof(unsigned long long);
        const size_t cnt_b = (size_t)XCH_MAX_BLOCKS * sizeof(unsigned);
        char *p = nullptr;
        hipError_t e = hipMalloc((void **)&p, slot_b + cnt_b + 256);
        if (e != hipSuccess) { mi355_fail("exchange area hipMalloc: %s", hipGetErrorString(e)); return false; }
        // tags and counters must start equal: all zero
        e = hipMemsetAsync(p, 0, slot_b + cnt_b + 256, g_ctx.stream);
        if (e != hipSuccess) { (void)hipFree(p); mi355_fail("exchange area clear: %s", hipGetErrorString(e)); return false; }
        g_xch.slots = (unsigned long long *)p;
        g_xch.cnt = (unsigned *)(p + slot_b);
        g_xch.fallbacks = (int *)(p + slot_b + cnt_b);
    }
    *out = g_xch;
    return true;
}

// Watch over the cooperating kernels.  Their results do not depend on whether a partner's value arrived in time, so a
// device on which they keep missing one another (shared with other work, workgroups not resident together) would only
// show as launches that each take the bounded wait and then read their operands several times.  mi355_sync(), which
// waits anyway, therefore looks at the two counters after such kernels have run: when they have grown at three checks
// in a row with no tuning knob changed in between, the cooperating forms are switched off for the rest of the process
// (the single-workgroup RMSNorm tiles, the two-launch INT8 scale and quantizer, the three-launch cross-entropy take
// over) and one line says so.  A change of a tuning knob starts the count afresh, and the test mode that refuses every value is not
// counted.
static bool g_coop_launched = false, g_coop_rebase = true;
static long long g_coop_seen = 0;
static int g_coop_strikes = 0;

int mi355_exchange_spin_ticks(void) {
    g_coop_launched = true;
    if (g_ctx.xch_take_nothing > 0) return -1;
    return g_ctx.rms_cluster_spin == 0 ? 200000 : (g_ctx.rms_cluster_spin < 0 ? 0 : g_ctx.rms_cluster_spin);
}

// How many workgroups, since the library was loaded, gave up the bounded wait for a partner's value and computed it
// themselves.  The results are the same to the bit either way, so this count is the only sign of a device on which
// the cooperating workgroups are not resident together (each expiry costs the wait plus the recomputation).
MI355_API int mi355_exchange_stats(long long *shared_area, long long *softmax_ce) {
    if (!mi355_ready("exchange_stats")) return -1;
    if (!mi355_outside_capture("exchange_stats")) return -1;
    int a = 0, c = 0;
    HIP_OK(hipStreamSynchronize(g_ctx.stream));
    if (g_xch.fallbacks) HIP_OK(hipMemcpy(&a, g_xch.fallbacks, sizeof(int), hipMemcpyDeviceToHost));
    if (int *p = mi355_ce_fallbacks_dev()) HIP_OK(hipMemcpy(&c, p, sizeof(int), hipMemcpyDeviceToHost));
    if (shared_area) *shared_area = a;
    if (softmax_ce) *softmax_ce = c;
    return 0;
}

int mi355_ce_setup(void);        // softmax_ce.hip: locates its fixed scratch array on the current device

MI355_API int mi355_init(void) {
    if (g_ctx.ready) return 0;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return mi355_fail("init: no HIP device (%s)", e == hipSuccess ? "count 0" : hipGetErrorString(e));
    }
    HIP_OK(hipSetDevice(0));
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return mi355_fail("init: device 0 is %s; this library holds gfx950 code only", prop.gcnArchName);
    g_ctx.device = 0;
    g_ctx.num_cu = prop.multiProcessorCount;
    g_ctx.stream = nullptr;
    g_ctx.ws = nullptr;
    g_ctx.ws_bytes = 0;
    g_ctx.ready = true;
    if (mi355_ce_setup()) { g_ctx.ready = false; return -1; }
    g_err[0] = 0;
    return 0;
}

void mi355_free_caches(void);   // rope tables, host drop-in staging (other translation units)
void mi355_dw_free(void);       // queued weight-gradient reductions and their arena
void mi355_blas_free(void);     // rocBLAS handle of mi355_sgemm_dev
void mi355_ckpt_free(void);     // pinned staging buffer of the checkpoint reader/writer
void mi355_graph_shutdown(void);  // capture stream

MI355_API void mi355_shutdown(void) {
    if (!g_ctx.ready) return;
    (void)hipDeviceSynchronize();
    mi355_free_caches();
    mi355_dw_free();
    mi355_blas_free();
    mi355_ckpt_free();
    mi355_graph_shutdown();
    if (g_xch.slots) (void)hipFree(g_xch.slots);
    g_xch = Mi355Exchange{nullptr, nullptr, nullptr};
    g_coop_launched = false;                // (the shared area's counter starts from zero again after the next init)
    g_coop_rebase = true;
    g_coop_strikes = 0;
    if (g_ctx.ws) (void)hipFree(g_ctx.ws);
    g_ctx = Mi355Ctx{};
}

MI355_API const char *mi355_last_error(void) { return g_err; }

MI355_API int mi355_device_info(char *name, size_t name_len, double *peak_hbm_gbs, int *compute_units) {
    if (!mi355_ready("device_info")) return -1;
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, g_ctx.device));
    if (name && name_len) {
        // (some driver stacks leave the marketing name empty: the architecture string then stands alone)
        if (prop.name[0]) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
        else snprintf(name, name_len, "%s", prop.gcnArchName);
    }
    if (peak_hbm_gbs) {
        // memoryClockRate is in kHz, bus width in bits; HBM transfers twice per clock.
        *peak_hbm_gbs = 2.0 * (double)prop.memoryClockRate * 1e3 * ((double)prop.memoryBusWidth / 8.0) / 1e9;
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    return 0;
}

MI355_API int mi355_set_stream(void *hip_stream) {
    if (!mi355_ready("set_stream")) return -1;
    if (!mi355_outside_capture("set_stream")) return -1;
    if (mi355_dw_flush()) return -1;        // queued reductions belong to the old stream
    // Workspaces are shared by the ops of every stream and are freed behind a wait on the CURRENT stream only:
    // nothing may still be running on the stream that is left behind.
    HIP_OK(hipStreamSynchronize(g_ctx.stream));
    g_ctx.stream = (hipStream_t)hip_stream;
    return 0;
}

static int coop_check(void) {
    if (!g_coop_launched) return 0;
    g_coop_launched = false;
    int a = 0, c = 0;
    if (g_xch.fallbacks) HIP_OK(hipMemcpy(&a, g_xch.fallbacks, sizeof(int), hipMemcpyDeviceToHost));
    if (int *p = mi355_ce_fallbacks_dev()) HIP_OK(hipMemcpy(&c, p, sizeof(int), hipMemcpyDeviceToHost));
    const long long total = (long long)a + c;
    if (g_coop_rebase || g_ctx.xch_take_nothing > 0) {
        g_coop_rebase = false;
        g_coop_strikes = 0;
    } else if (total > g_coop_seen) {
        if (++g_coop_strikes >= 3 && (g_ctx.rms_cluster >= 0 || g_ctx.ce_resident >= 0)) {
            g_ctx.rms_cluster = -1;
            g_ctx.ce_resident = -1;
            fprintf(stderr, "mi355_bridge: workgroups of the cooperating kernels keep giving up their wait for one another "
                            "(%lld so far): is the GPU shared?  Switched to the non-cooperating forms "
                            "(mi355_tune_set(\"rms_cluster\", 0) and (\"ce_resident\", 0) switch back)\n", total);
        }
    } else {
        g_coop_strikes = 0;
    }
    g_coop_seen = total;
    return 0;
}

MI355_API int mi355_sync(void) {
    if (!mi355_ready("sync")) return -1;
    if (!mi355_outside_capture("sync")) return -1;
    if (mi355_dw_flush()) return -1;
    HIP_OK(hipStreamSynchronize(g_ctx.stream));
    return coop_check();
}

MI355_API int mi355_workspace_reserve(size_t bytes) {
    if (!mi355_ready("workspace_reserve")) return -1;
    return mi355_ws(bytes) ? 0 : -1;
}

MI355_API size_t mi355_workspace_size(void) { return g_ctx.ready ? g_ctx.ws_bytes : 0; }

MI355_API int mi355_tune_set(const char *key, int value) {
    if (!key) return -1;
    struct { const char *k; int *v; } tab[] = {
        {"rms_lpr", &g_ctx.rms_lpr}, {"rms_threads", &g_ctx.rms_threads},
        {"ew_unroll", &g_ctx.ew_unroll},
        {"ce_rows", &g_ctx.ce_rows}, {"ce_rows2", &g_ctx.ce_rows2}, {"buf_phase", &g_ctx.buf_phase}, {"qk_lpr", &g_ctx.qk_lpr}, {"qk_threads", &g_ctx.qk_threads},
        {"gemm_splitk", &g_ctx.gemm_splitk}, {"scatter_tree", &g_ctx.scatter_tree}, {"scatter_cols", &g_ctx.scatter_cols},
        {"rms_cluster", &g_ctx.rms_cluster}, {"rms_cluster_spin", &g_ctx.rms_cluster_spin},
        {"ce_resident", &g_ctx.ce_resident}, {"xch_take_nothing", &g_ctx.xch_take_nothing},
    };
    for (auto &t : tab)
        if (strcmp(t.k, key) == 0) { *t.v = value; g_coop_rebase = true; return 0; }
    return -1;
}

// ---------------------------------------------------------------------------------------------
// Buffers
// ---------------------------------------------------------------------------------------------
struct mi355_buf {
    void *base;     // what hipMalloc returned
    void *dev;      // what the caller sees
    size_t bytes;
};

MI355_API mi355_buf *mi355_buf_alloc(size_t bytes) {
    if (!mi355_ready("buf_alloc")) return nullptr;
    if (bytes == 0) { mi355_fail("buf_alloc: zero bytes"); return nullptr; }
    if (!mi355_outside_capture("buf_alloc")) return nullptr;
    // Large buffers start at a rotating multiple of 128 bytes within a 1 KiB group.  With S = 256 a row of an
    // activation is 1 KiB, so a workgroup of a column-reduction kernel, which reads the same 64 bytes of every row,
    // talks to one eighth of the memory channels, and one of those eighths is markedly slower under that pattern.
    // Operands that all start on a 2 MiB boundary put their slow strips into the same workgroups; rotated starts
    // spread them (RMSNorm backward at the Qwen3 shape: 16.1 -> 14.2 us).
    static unsigned counter = 0;
    size_t phase = 0;
    if (bytes >= ((size_t)1 << 20)) {
        if (g_ctx.buf_phase == 0) phase = (size_t)(counter++ % 8) * 128;
        else phase = (size_t)((g_ctx.buf_phase - 1) % 8) * 128;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes + phase);
    if (e != hipSuccess) { mi355_fail("buf_alloc(%zu): %s", bytes, hipGetErrorString(e)); return nullptr; }
    e = hipMemsetAsync(p, 0, bytes + phase, g_ctx.stream);
    if (e != hipSuccess) { (void)hipFree(p); mi355_fail("buf_alloc memset: %s", hipGetErrorString(e)); return nullptr; }
    mi355_buf *b = (mi355_buf *)malloc(sizeof(mi355_buf));
    if (!b) { (void)hipFree(p); return nullptr; }
    b->base = p;
    b->dev = (char *)p + phase;
    b->bytes = bytes;
    return b;
}

MI355_API void mi355_buf_free(mi355_buf *b) {
    if (!b) return;
    if (!mi355_outside_capture("buf_free")) return;
    if (g_ctx.ready && b->dev) {
        (void)hipStreamSynchronize(g_ctx.stream);
        (void)hipFree(b->base);
    }
    free(b);
}

MI355_API void *mi355_buf_devptr(mi355_buf *b) { return b ? b->dev : nullptr; }
MI355_API size_t mi355_buf_bytes(mi355_buf *b) { return b ? b->bytes : 0; }

MI355_API void mi355_buf_write(mi355_buf *b, size_t offset, const void *src, size_t bytes) {
    if (!b || !src || !g_ctx.ready || offset > b->bytes || bytes > b->bytes - offset || bytes == 0) return;
    if (!mi355_outside_capture("buf_write")) return;
    hipError_t e = hipMemcpyAsync((char *)b->dev + offset, src, bytes, hipMemcpyHostToDevice, g_ctx.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_ctx.stream);
    if (e != hipSuccess) mi355_fail("buf_write: %s", hipGetErrorString(e));
}

MI355_API void mi355_buf_read(mi355_buf *b, size_t offset, void *dst, size_t bytes) {
    if (!b || !dst || !g_ctx.ready || offset > b->bytes || bytes > b->bytes - offset || bytes == 0) return;
    if (!mi355_outside_capture("buf_read")) return;
    (void)mi355_dw_flush();                 // a read may be of a gradient that is still queued
    hipError_t e = hipMemcpyAsync(dst, (const char *)b->dev + offset, bytes, hipMemcpyDeviceToHost, g_ctx.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(g_ctx.stream);
    if (e != hipSuccess) mi355_fail("buf_read: %s", hipGetErrorString(e));
}

__global__ void fill_zero_kernel(v4f *p, size_t n4, char *tail, size_t ntail) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    v4f z = {0.f, 0.f, 0.f, 0.f};
    for (; i < n4; i += stride) p[i] = z;
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

MI355_API int mi355_buf_zero(mi355_buf *b) {
    if (!mi355_ready("buf_zero")) return -1;
    if (!b) return mi355_fail("buf_zero: NULL buffer");
    // a fill kernel rather than hipMemsetAsync, so the call is safe inside a captured graph
    size_t n4 = b->bytes / 16, ntail = b->bytes % 16;
    size_t blocks = ceil_div(n4 ? n4 : 1, 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, g_ctx.stream,
                       (v4f *)b->dev, n4, (char *)b->dev + n4 * 16, ntail);
    LAUNCH_OK("buf_zero");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Events
// ---------------------------------------------------------------------------------------------
struct mi355_event {
    hipEvent_t ev;
};

MI355_API mi355_event *mi355_event_create(void) {
    if (!mi355_ready("event_create")) return nullptr;
    mi355_event *e = (mi355_event *)malloc(sizeof(mi355_event));
    if (!e) return nullptr;
    if (hipEventCreate(&e->ev) != hipSuccess) { free(e); mi355_fail("event_create failed"); return nullptr; }
    return e;
}

MI355_API void mi355_event_destroy(mi355_event *e) {
    if (!e) return;
    if (g_ctx.ready) (void)hipEventDestroy(e->ev);
    free(e);
}

MI355_API int mi355_event_record(mi355_event *e) {
    if (!mi355_ready("event_record")) return -1;
    if (!e) return mi355_fail("event_record: NULL event");
    HIP_OK(hipEventRecord(e->ev, g_ctx.stream));
    return 0;
}

MI355_API float mi355_event_elapsed_ms(mi355_event *start, mi355_event *stop) {
    if (!g_ctx.ready || !start || !stop) return -1.0f;
    if (hipEventSynchronize(stop->ev) != hipSuccess) return -1.0f;
    float ms = -1.0f;
    if (hipEventElapsedTime(&ms, start->ev, stop->ev) != hipSuccess) return -1.0f;
    return ms;
}

// ---------------------------------------------------------------------------------------------
// Synthetic data: element i of stream `seed` is a pure function of (seed, i).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void fill_normal_kernel(float *p, size_t n, uint64_t seed, float mean, float std) {
    size_t pair = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t npair = (n + 1) / 2;
    for (; pair < npair; pair += stride) {
        uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + pair);
        float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777217.0f);   // (0,1)
        float u2 = (float)(uint32_t)((r >> 8) & 0xFFFFFF) * (1.0f / 16777216.0f);
        float rad = sqrtf(-2.0f * logf(u1));
        float sn, cs;
        sincosf(6.283185307179586f * u2, &sn, &cs);
        p[2 * pair] = mean + std * rad * cs;
        if (2 * pair + 1 < n) p[2 * pair + 1] = mean + std * rad * sn;
    }
}

__global__ void fill_randint_kernel(int32_t *p, size_t n, uint64_t seed, int32_t lo, uint32_t span) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + i);
        p[i] = lo + (int32_t)(((r >> 32) * (uint64_t)span) >> 32);
    }
}

MI355_API int mi355_fill_normal_dev(float *p, size_t n, uint64_t seed, float mean, float std) {
    if (!mi355_ready("fill_normal")) return -1;
    if (!p || n == 0) return mi355_fail("fill_normal: NULL pointer or empty");
    size_t blocks = ceil_div((n + 1) / 2, 256);
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(fill_normal_kernel, dim3((unsigned)blocks), dim3(256), 0, g_ctx.stream, p, n, seed, mean, std);
    LAUNCH_OK("fill_normal");
    return 0;
}

MI355_API int mi355_fill_randint_dev(int32_t *p, size_t n, uint64_t seed, int32_t lo, int32_t hi) {
    if (!mi355_ready("fill_randint")) return -1;
    if (!p || n == 0 || hi <= lo) return mi355_fail("fill_randint: bad arguments");
    size_t blocks = ceil_div(n, 256);
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(fill_randint_kernel, dim3((unsigned)blocks), dim3(256), 0, g_ctx.stream, p, n, seed, lo,
                       (uint32_t)(hi - lo));
    LAUNCH_OK("fill_randint");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Graphs: a launch-bound sequence of ops recorded once and replayed as one submission.
// Capture runs on a stream of the bridge's own (the default stream cannot be captured); replays go to the
// bridge stream.  Nothing recorded may allocate, wait or touch the host, so the sequence has to have run once
// before (workspaces sized, RoPE tables built).  No memset node is ever recorded: buffers are cleared by fill
// kernels.
// ---------------------------------------------------------------------------------------------
struct mi355_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
    unsigned epoch;     // g_ctx.alloc_epoch at capture: the recorded kernels hold workspace addresses of that time
};

static hipStream_t g_cap_stream = nullptr, g_saved_stream = nullptr;

void mi355_graph_shutdown(void) {
    if (g_cap_stream) (void)hipStreamDestroy(g_cap_stream);
    g_cap_stream = nullptr;
}

MI355_API int mi355_graph_begin(void) {
    if (!mi355_ready("graph_begin")) return -1;
    if (g_ctx.capturing) return mi355_fail("graph_begin: a capture is already open");
    if (mi355_dw_flush()) return -1;                       // queued reductions belong to the eager stream
    HIP_OK(hipStreamSynchronize(g_ctx.stream));            // the recording starts from a quiet device
    if (!g_cap_stream) HIP_OK(hipStreamCreate(&g_cap_stream));      // default flags and priority
    HIP_OK(hipStreamBeginCapture(g_cap_stream, hipStreamCaptureModeThreadLocal));
    g_saved_stream = g_ctx.stream;
    g_ctx.stream = g_cap_stream;
    g_ctx.capturing = true;
    return 0;
}

MI355_API mi355_graph *mi355_graph_end(void) {
    if (!g_ctx.ready || !g_ctx.capturing) { mi355_fail("graph_end: no capture is open"); return nullptr; }
    const int flushed = mi355_dw_flush();                   // queued reductions become part of the graph
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(g_cap_stream, &graph);
    g_ctx.stream = g_saved_stream;
    g_ctx.capturing = false;
    if (e != hipSuccess || !graph || flushed) {
        if (graph) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        if (e != hipSuccess || !graph) mi355_fail("graph_end: capture failed: %s", e == hipSuccess ? "empty graph" : hipGetErrorString(e));
        return nullptr;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        mi355_fail("graph_end: hipGraphInstantiate: %s", hipGetErrorString(e));
        return nullptr;
    }
    mi355_graph *g = (mi355_graph *)malloc(sizeof(mi355_graph));
    if (!g) { (void)hipGraphExecDestroy(exec); (void)hipGraphDestroy(graph); return nullptr; }
    g->graph = graph;
    g->exec = exec;
    g->epoch = g_ctx.alloc_epoch;
    return g;
}

MI355_API int mi355_graph_launch(mi355_graph *g) {
    if (!mi355_ready("graph_launch")) return -1;
    if (!g) return mi355_fail("graph_launch: NULL graph");
    if (!mi355_outside_capture("graph_launch")) return -1;
    if (g->epoch != g_ctx.alloc_epoch)
        return mi355_fail("graph_launch: a workspace was reallocated after this graph was recorded; record it again");
    if (mi355_dw_flush()) return -1;                        // keep eager reductions ahead of the replay
    HIP_OK(hipGraphLaunch(g->exec, g_ctx.stream));
    return 0;
}

MI355_API void mi355_graph_free(mi355_graph *g) {
    if (!g) return;
    if (g_ctx.ready) {
        (void)hipStreamSynchronize(g_ctx.stream);
        (void)hipGraphExecDestroy(g->exec);
        (void)hipGraphDestroy(g->graph);
    }
    free(g);
}
