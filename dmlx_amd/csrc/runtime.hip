// Runtime plumbing of libdmoe: error reporting, device selection, streams, device memory, workspaces.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "common.h"

namespace dmoe {

static std::mutex lds_limit_mutex;

int raise_lds_limit(LdsLimit &state, const void *kernel, int bytes) {
    int dev = 0;
    DMOE_HIP(hipGetDevice(&dev));
    DMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d is out of range", dev);
    std::lock_guard<std::mutex> lock(lds_limit_mutex);
    if (state.raised >> dev & 1ull) return DMOE_OK;
    DMOE_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    state.raised |= 1ull << dev;
    return DMOE_OK;
}

static thread_local char g_err[2048] = ""; // same size as the reference's mlx error buffer

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what) {
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return DMOE_ERR_HIP;
}

int workspace_reserve(dmoe_workspace ws, size_t bytes, Workspace **out) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    if (bytes > w->bytes) {
        DMOE_REQUIRE(!w->fixed, "this call needs %zu bytes of scratch memory, the static device scratch holds %zu",
                     bytes, w->bytes);
        // growth is rare (first call at a new size); in-flight work may still use the old block
        DMOE_HIP(hipDeviceSynchronize());
        if (w->base) DMOE_HIP(hipFree(w->base));
        w->base = nullptr;
        w->bytes = 0;
        size_t want = bytes + bytes / 4;
        DMOE_HIP(hipMalloc(&w->base, want));
        w->bytes = want;
    }
    *out = w;
    return DMOE_OK;
}

int side_stream_ready(Workspace *w) {
    if (w->side) return DMOE_OK;
    DMOE_REQUIRE(!w->fixed, "internal: a side stream was asked for on the static device scratch");
    DMOE_HIP(hipStreamCreateWithFlags(&w->side, hipStreamNonBlocking));
    DMOE_HIP(hipEventCreateWithFlags(&w->fork, hipEventDisableTiming));
    DMOE_HIP(hipEventCreateWithFlags(&w->join, hipEventDisableTiming));
    DMOE_HIP(hipEventCreateWithFlags(&w->packed, hipEventDisableTiming));
    DMOE_HIP(hipEventCreateWithFlags(&w->small_done, hipEventDisableTiming));
    return DMOE_OK;
}

int stage_flush(Workspace *w) {
    StageTimer &t = w->timer;
    for (int i = 0; i < DMOE_STAGE_COUNT; ++i) {
        // a stage whose start is recorded and whose stop is not keeps its slot: its ring is read at a later flush
        if (t.open[i]) continue;
        for (int k = 0; k < t.pending[i]; ++k) {
            DMOE_HIP(hipEventSynchronize(t.stop[i][k]));
            float ms = 0.0f;
            DMOE_HIP(hipEventElapsedTime(&ms, t.start[i][k], t.stop[i][k]));
            t.total_ms[i] += ms;
            t.samples[i] += 1;
        }
        t.pending[i] = 0;
    }
    return DMOE_OK;
}

int stage_begin(Workspace *w, int stage, hipStream_t st) {
    StageTimer &t = w->timer;
    if (!t.enabled) return DMOE_OK;
    if (t.pending[stage] == kStageRing) DMOE_TRY(stage_flush(w)); // the ring is full: read it out (waits for the device)
    DMOE_HIP(hipEventRecord(t.start[stage][t.pending[stage]], st));
    t.open[stage] = true;
    return DMOE_OK;
}

int stage_end(Workspace *w, int stage, hipStream_t st) {
    StageTimer &t = w->timer;
    if (!t.enabled || !t.open[stage]) return DMOE_OK;
    DMOE_HIP(hipEventRecord(t.stop[stage][t.pending[stage]], st));
    t.pending[stage] += 1;
    t.open[stage] = false;
    return DMOE_OK;
}

} // namespace dmoe

using namespace dmoe;

extern "C" {

int dmoe_version(void) { return DMOE_VERSION; }

const char *dmoe_last_error(void) { return g_err; }

int dmoe_quant_mode_from_string(const char *name) {
    if (!name) return -1;
    if (!strcmp(name, "affine")) return DMOE_QUANT_AFFINE;
    if (!strcmp(name, "mxfp4")) return DMOE_QUANT_MXFP4;
    if (!strcmp(name, "fp8")) return DMOE_QUANT_FP8_ROW;
    if (!strcmp(name, "none") || !strcmp(name, "bf16")) return DMOE_QUANT_NONE;
    return -1;
}

int dmoe_init(int device) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        set_error("no HIP device visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
        return DMOE_ERR_NO_DEVICE;
    }
    if (device >= 0) {
        DMOE_REQUIRE(device < n, "device %d out of range (%d visible)", device, n);
        DMOE_HIP(hipSetDevice(device));
    } else {
        DMOE_HIP(hipGetDevice(&device));
    }
    hipDeviceProp_t prop;
    DMOE_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
        return DMOE_ERR_NO_DEVICE;
    }
    // resolve this device's copy of the static scratch now, so that the allocation-free entry point finds it ready
    Workspace *unused = nullptr;
    DMOE_TRY(static_workspace(&unused));
    // and every GEMM kernel's dynamic-LDS limit: a first launch under stream capture or from another thread then has
    // no host-side set-up left
    DMOE_TRY(qgemm_wide_prepare());
    DMOE_TRY(qgemm_mfma_prepare());
    DMOE_TRY(qgemm_skinny_prepare());
    return DMOE_OK;
}

int dmoe_stream_create(dmoe_stream *out) {
    DMOE_REQUIRE(out != nullptr, "out is null");
    hipStream_t st;
    DMOE_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    out->ctx = (void *)st;
    return DMOE_OK;
}

int dmoe_stream_destroy(dmoe_stream s) {
    if (s.ctx) DMOE_HIP(hipStreamDestroy(to_hip(s)));
    return DMOE_OK;
}

int dmoe_stream_synchronize(dmoe_stream s) {
    DMOE_HIP(hipStreamSynchronize(to_hip(s)));
    return DMOE_OK;
}

int dmoe_malloc(void **out, size_t bytes) {
    DMOE_REQUIRE(out != nullptr, "out is null");
    *out = nullptr;
    if (bytes == 0) return DMOE_OK;
    DMOE_HIP(hipMalloc(out, bytes));
    return DMOE_OK;
}

int dmoe_free(void *p) {
    if (p) DMOE_HIP(hipFree(p));
    return DMOE_OK;
}

int dmoe_copy_to_device(void *dst, const void *src, size_t bytes, dmoe_stream s) {
    if (bytes == 0) return DMOE_OK;
    DMOE_REQUIRE(dst && src, "null pointer");
    DMOE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, to_hip(s)));
    // pageable host memory: the runtime may still read `src` after returning; wait so the caller may reuse it
    DMOE_HIP(hipStreamSynchronize(to_hip(s)));
    return DMOE_OK;
}

int dmoe_copy_to_host(void *dst, const void *src, size_t bytes, dmoe_stream s) {
    if (bytes == 0) return DMOE_OK;
    DMOE_REQUIRE(dst && src, "null pointer");
    DMOE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, to_hip(s)));
    DMOE_HIP(hipStreamSynchronize(to_hip(s)));
    return DMOE_OK;
}

int dmoe_workspace_create(dmoe_workspace *out, size_t initial_bytes) {
    DMOE_REQUIRE(out != nullptr, "out is null");
    Workspace *w = new Workspace();
    hipError_t e = hipGetDevice(&w->device);
    if (e != hipSuccess) {
        delete w;
        return hip_fail(e, "hipGetDevice");
    }
    e = hipMalloc((void **)&w->flags, 256);
    if (e == hipSuccess) e = hipMemset(w->flags, 0, 256);
    if (e != hipSuccess) {
        if (w->flags) (void)hipFree(w->flags);
        delete w;
        return hip_fail(e, "hipMalloc(workspace flags)");
    }
    out->ctx = w;
    if (initial_bytes) {
        Workspace *tmp;
        int rc = workspace_reserve(*out, initial_bytes, &tmp);
        if (rc != DMOE_OK) {
            (void)hipFree(w->flags);
            delete w;
            out->ctx = nullptr;
            return rc;
        }
    }
    return DMOE_OK;
}

int dmoe_workspace_set_stage_timing(dmoe_workspace ws, int enabled) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    StageTimer &t = w->timer;
    if (enabled && !t.start[0][0]) {
        for (int i = 0; i < DMOE_STAGE_COUNT; ++i)
            for (int k = 0; k < kStageRing; ++k) {
                DMOE_HIP(hipEventCreate(&t.start[i][k]));
                DMOE_HIP(hipEventCreate(&t.stop[i][k]));
            }
    }
    if (!enabled && t.enabled) DMOE_TRY(stage_flush(w));
    if (enabled && !t.enabled)
        for (int i = 0; i < DMOE_STAGE_COUNT; ++i) {
            t.total_ms[i] = 0.0f;
            t.samples[i] = 0;
            t.pending[i] = 0;
            t.open[i] = false;
        }
    t.enabled = enabled != 0;
    return DMOE_OK;
}

int dmoe_workspace_read_stage_times(float *h_out_total_ms, int *h_out_samples, dmoe_workspace ws) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w && h_out_total_ms && h_out_samples, "null argument");
    DMOE_TRY(stage_flush(w));
    for (int i = 0; i < DMOE_STAGE_COUNT; ++i) {
        h_out_total_ms[i] = w->timer.total_ms[i];
        h_out_samples[i] = w->timer.samples[i];
    }
    return DMOE_OK;
}

int dmoe_workspace_destroy(dmoe_workspace ws) {
    Workspace *w = (Workspace *)ws.ctx;
    if (!w) return DMOE_OK;
    for (int i = 0; i < DMOE_STAGE_COUNT; ++i)
        for (int k = 0; k < kStageRing; ++k) {
            if (w->timer.start[i][k]) (void)hipEventDestroy(w->timer.start[i][k]);
            if (w->timer.stop[i][k]) (void)hipEventDestroy(w->timer.stop[i][k]);
        }
    if (w->side) (void)hipStreamSynchronize(w->side);
    weight_cache_clear(w);
    if (w->fork) (void)hipEventDestroy(w->fork);
    if (w->join) (void)hipEventDestroy(w->join);
    if (w->packed) (void)hipEventDestroy(w->packed);
    if (w->small_done) (void)hipEventDestroy(w->small_done);
    if (w->side) (void)hipStreamDestroy(w->side);
    hipError_t e = w->base ? hipFree(w->base) : hipSuccess;
    if (w->flags) {
        hipError_t e2 = hipFree(w->flags);
        if (e == hipSuccess) e = e2;
    }
    delete w;
    if (e != hipSuccess) return hip_fail(e, "hipFree(workspace)");
    return DMOE_OK;
}

int dmoe_workspace_check(dmoe_workspace ws, dmoe_stream s) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    DMOE_HIP(hipStreamSynchronize(to_hip(s)));
    if (w->side) DMOE_HIP(hipStreamSynchronize(w->side));
    uint32_t flags[2] = {0, 0}; // [0] waits that gave up, [1] expert ids out of range
    DMOE_HIP(hipMemcpy(flags, w->flags, sizeof flags, hipMemcpyDeviceToHost));
    if (flags[0] || flags[1]) DMOE_HIP(hipMemset(w->flags, 0, sizeof flags));
    if (flags[0]) {
        // the paired launch relies on the order in which the hardware starts workgroups; after one failure this
        // workspace stays on the two-launch path, which waits for nothing
        w->paired = false;
        set_error("%u workgroup(s) gave up waiting for their tile's gate/up results: outputs since the last check are "
                  "invalid; this workspace now runs gate/up and down as two launches",
                  (unsigned)flags[0]);
        return DMOE_ERR_TIMEOUT;
    }
    if (flags[1]) {
        set_error("%u expert id(s) outside the layer's expert range reached the packing step (computed as the last "
                  "expert): outputs since the last check are invalid", (unsigned)flags[1]);
        return DMOE_ERR_INVALID;
    }
    return DMOE_OK;
}

int dmoe_workspace_set_weight_cache(dmoe_workspace ws, int enabled) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    DMOE_REQUIRE(!w->fixed, "the static device scratch keeps no weight cache");
    if (!enabled) {
        // copies may still be read by kernels in flight
        DMOE_HIP(hipDeviceSynchronize());
        weight_cache_clear(w);
    }
    w->cache_weights = enabled != 0;
    return DMOE_OK;
}

int dmoe_workspace_weight_cache_invalidate(dmoe_workspace ws, const dmoe_qweight *qw) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    return weight_cache_invalidate(w, qw);
}

int dmoe_workspace_set_weight_cache_limit(dmoe_workspace ws, size_t max_bytes) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    w->cache_limit_bytes = max_bytes;
    return DMOE_OK;
}

int dmoe_workspace_weight_cache_stats(size_t *out_bytes, int *out_stacks, dmoe_workspace ws) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    return weight_cache_stats(w, out_bytes, out_stacks);
}

int dmoe_workspace_set_paired_launch(dmoe_workspace ws, int enabled) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    w->paired = enabled != 0;
    return DMOE_OK;
}

int dmoe_workspace_set_wait_limit(dmoe_workspace ws, unsigned polls) {
    Workspace *w = (Workspace *)ws.ctx;
    DMOE_REQUIRE(w != nullptr, "workspace handle is null");
    w->spin_limit = polls;
    return DMOE_OK;
}

int dmoe_workspace_reserved(size_t *out_bytes, dmoe_workspace ws) {
    DMOE_REQUIRE(out_bytes && ws.ctx, "null argument");
    *out_bytes = ((Workspace *)ws.ctx)->bytes;
    return DMOE_OK;
}

} // extern "C"
