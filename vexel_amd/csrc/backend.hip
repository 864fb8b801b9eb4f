// Backend lifetime, memory, copies, stream capture. C ABI: include/vexel_hip.h.
#include <stdarg.h>
#include <string.h>

#include "common.h"

namespace vx {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int enter(vx_backend *be) {
    if (!be) {
        set_error("null backend");
        return VX_ERR_INVALID;
    }
    VX_CHECK_HIP(hipSetDevice(be->device));
    return VX_OK;
}

int ensure_ws(vx_backend *be, void **ptr, size_t *cap, size_t bytes, const char *what) {
    if (bytes <= *cap) return VX_OK;
    if (be->capturing) {
        set_error("%s scratch must grow to %zu bytes during graph capture; run the step once before capturing", what, bytes);
        return VX_ERR_INVALID;
    }
    // Earlier launches may still use the old buffer.
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    if (*ptr) VX_CHECK_HIP(hipFree(*ptr));
    *ptr = nullptr;
    *cap = 0;
    size_t want = bytes + bytes / 4;
    hipError_t e = hipMalloc(ptr, want);
    if (e != hipSuccess) {
        set_error("hipMalloc(%zu) for %s scratch failed: %s", want, what, hipGetErrorString(e));
        return VX_ERR_OOM;
    }
    *cap = want;
    be->scratch_gen++;
    return VX_OK;
}

}  // namespace vx

using namespace vx;

extern "C" {

const char *vx_last_error(void) { return g_err; }

uint64_t vx_scratch_generation(const vx_backend *be) { return be ? be->scratch_gen : 0; }

int vx_backend_create(int device_id, vx_backend **out) {
    if (!out) {
        set_error("out is null");
        return VX_ERR_INVALID;
    }
    int count = 0;
    VX_CHECK_HIP(hipGetDeviceCount(&count));
    VX_REQUIRE(device_id >= 0 && device_id < count, "device %d out of range (have %d)", device_id, count);
    VX_CHECK_HIP(hipSetDevice(device_id));
    hipDeviceProp_t prop;
    VX_CHECK_HIP(hipGetDeviceProperties(&prop, device_id));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library holds gfx950 code only", device_id, prop.gcnArchName);
        return VX_ERR_UNSUPPORTED;
    }
    vx_backend *be = new vx_backend();
    be->device = device_id;
    {
        int rc = attn_noalloc_init(be);
        if (rc) {
            delete be;
            return rc;
        }
    }
    VX_CHECK_HIP(hipStreamCreateWithFlags(&be->stream, hipStreamNonBlocking));
    VX_CHECK_HIP(hipEventCreate(&be->ev0));
    VX_CHECK_HIP(hipEventCreate(&be->ev1));
    be->host_stage_bytes = 1 << 20;
    VX_CHECK_HIP(hipHostMalloc(&be->host_stage, be->host_stage_bytes, hipHostMallocDefault));
    be->misc_ws_bytes = 1 << 20;
    VX_CHECK_HIP(hipMalloc(&be->misc_ws, be->misc_ws_bytes));
    VX_CHECK_HIP(hipMalloc(&be->rope_tab, (size_t)VX_ROPE_TAB_ROWS * VX_ROPE_TAB_PAIRS * 2 * sizeof(float)));
    VX_CHECK_HIP(hipMalloc((void **)&be->attn_cnt, VX_ATTN_CNT * sizeof(int32_t)));
    VX_CHECK_HIP(hipMemset(be->attn_cnt, 0, VX_ATTN_CNT * sizeof(int32_t)));  // (whoever arrives last at a counter puts it back to zero)
    VX_CHECK_HIP(hipMalloc(&be->prep_sync, VX_PREP_SYNC_BYTES));
    VX_CHECK_HIP(hipMemset(be->prep_sync, 0, VX_PREP_SYNC_BYTES));  // per-chunk sums of squares: every slot a prepare reads was written by the kernel before it
    {
        float ones[64];
        for (float &o : ones) o = 1.0f;
        VX_CHECK_HIP(hipMalloc((void **)&be->ones, sizeof ones));
        VX_CHECK_HIP(hipMemcpy(be->ones, ones, sizeof ones, hipMemcpyHostToDevice));
    }
    be->attn_merge = getenv("VEXEL_HIP_NO_ATTN_MERGE") == nullptr;
    *out = be;
    return VX_OK;
}

int vx_backend_set_attn_merge(vx_backend *be, int on) {
    if (!be) return VX_ERR_INVALID;
    be->attn_merge = on != 0;
    return VX_OK;
}

void vx_backend_destroy(vx_backend *be) {
    if (!be) return;
    (void)hipSetDevice(be->device);
    (void)hipStreamSynchronize(be->stream);
    stream_drop_all(be);
    for (auto &c : be->chunks) (void)hipFree(c.base);
    for (auto &kv : be->permanent) (void)hipFree(kv.first);
    if (be->gemm_ws) (void)hipFree(be->gemm_ws);
    if (be->part_ws) (void)hipFree(be->part_ws);
    if (be->part_ws2) (void)hipFree(be->part_ws2);
    if (be->attn_ws) (void)hipFree(be->attn_ws);
    if (be->sample_ws) (void)hipFree(be->sample_ws);
    if (be->items.buf) (void)hipFree(be->items.buf);
    if (be->misc_ws) (void)hipFree(be->misc_ws);
    if (be->prep_sync) (void)hipFree(be->prep_sync);
    if (be->rope_tab) (void)hipFree(be->rope_tab);
    if (be->shift_tab) (void)hipFree(be->shift_tab);
    if (be->attn_cnt) (void)hipFree(be->attn_cnt);
    if (be->ones) (void)hipFree(be->ones);
    if (be->host_stage) (void)hipHostFree(be->host_stage);
    if (be->ev0) (void)hipEventDestroy(be->ev0);
    if (be->ev1) (void)hipEventDestroy(be->ev1);
    if (be->stream) (void)hipStreamDestroy(be->stream);
    delete be;
}

int vx_backend_device(const vx_backend *be) { return be ? be->device : -1; }

void *vx_alloc(vx_backend *be, size_t bytes) {
    if (enter(be) != VX_OK || bytes == 0) return nullptr;
    const size_t align = 256;
    size_t need = (bytes + align - 1) / align * align;
    for (size_t i = be->cur_chunk; i < be->chunks.size(); i++) {
        PoolChunk &c = be->chunks[i];
        if (c.used + need <= c.size) {
            void *p = c.base + c.used;
            c.used += need;
            be->cur_chunk = i;
            return p;
        }
    }
    if (be->capturing) {
        set_error("vx_alloc(%zu) must grow the pool during graph capture", bytes);
        return nullptr;
    }
    size_t csize = need > ((size_t)64 << 20) ? need : ((size_t)64 << 20);
    void *base = nullptr;
    hipError_t e = hipMalloc(&base, csize);
    if (e != hipSuccess) {
        set_error("hipMalloc(%zu) failed: %s", csize, hipGetErrorString(e));
        return nullptr;
    }
    be->chunks.push_back(PoolChunk{(char *)base, csize, need});
    be->cur_chunk = be->chunks.size() - 1;
    return base;
}

void *vx_alloc_permanent(vx_backend *be, size_t bytes) {
    if (enter(be) != VX_OK || bytes == 0) return nullptr;
    if (be->capturing) {
        set_error("vx_alloc_permanent during graph capture");
        return nullptr;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        set_error("hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        return nullptr;
    }
    be->permanent[p] = bytes;
    return p;
}

void vx_free(vx_backend *be, void *ptr) {
    if (!ptr || enter(be) != VX_OK) return;
    auto it = be->permanent.find(ptr);
    if (it == be->permanent.end()) return;  // pool buffer: recycled by vx_reset_pool
    items_written(be, ptr, it->second);
    (void)hipStreamSynchronize(be->stream);
    stream_drop_packed(be, ptr);  // a packed copy of a matrix that started here goes with it
    (void)hipFree(ptr);
    be->permanent.erase(it);
}

void vx_reset_pool(vx_backend *be) {
    if (!be) return;
    for (auto &c : be->chunks) c.used = 0;
    be->cur_chunk = 0;
    be->items.valid = false;  // a kv_lens array taken from the pool is about to be reused
}

int vx_to_device(vx_backend *be, void *dst, const void *src_host, size_t bytes) {
    int rc = enter(be);
    if (rc) return rc;
    if (!dst || bytes == 0) return VX_OK;  // CPUBackend.ToDevice ignores nil / empty (cpu.go:57-63)
    VX_REQUIRE(src_host != nullptr, "vx_to_device: null source");
    VX_REQUIRE(!be->capturing, "vx_to_device during graph capture");
    items_written(be, dst, bytes);
    VX_CHECK_HIP(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, be->stream));
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    return VX_OK;
}

int vx_to_host(vx_backend *be, void *dst_host, const void *src, size_t bytes) {
    int rc = enter(be);
    if (rc) return rc;
    if (!src || bytes == 0) return VX_OK;
    VX_REQUIRE(dst_host != nullptr, "vx_to_host: null destination");
    VX_REQUIRE(!be->capturing, "vx_to_host during graph capture");
    VX_CHECK_HIP(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, be->stream));
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    return VX_OK;
}

int vx_sync(vx_backend *be) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(!be->capturing, "vx_sync during graph capture");
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    return VX_OK;
}

int vx_copy_buffer(vx_backend *be, const void *src, size_t src_off, void *dst, size_t dst_off, size_t bytes) {
    int rc = enter(be);
    if (rc) return rc;
    if (bytes == 0) return VX_OK;
    VX_REQUIRE(src && dst, "vx_copy_buffer: null pointer");
    items_written(be, (char *)dst + dst_off, bytes);
    VX_CHECK_HIP(hipMemcpyAsync((char *)dst + dst_off, (const char *)src + src_off, bytes,
                                hipMemcpyDeviceToDevice, be->stream));
    return VX_OK;
}

int vx_begin_batch(vx_backend *be) { return be ? VX_OK : VX_ERR_INVALID; }
int vx_end_batch(vx_backend *be) { return be ? VX_OK : VX_ERR_INVALID; }
int vx_memory_barrier(vx_backend *be) { return be ? VX_OK : VX_ERR_INVALID; }

int vx_graph_begin_capture(vx_backend *be) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(!be->capturing, "capture already active");
    VX_CHECK_HIP(hipStreamSynchronize(be->stream));
    VX_CHECK_HIP(hipStreamBeginCapture(be->stream, hipStreamCaptureModeThreadLocal));
    be->capturing = true;
    return VX_OK;
}

int vx_graph_end_capture(vx_backend *be, vx_graph **out) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(be->capturing, "no capture active");
    be->capturing = false;
    hipGraph_t graph = nullptr;
    VX_CHECK_HIP(hipStreamEndCapture(be->stream, &graph));
    VX_REQUIRE(out != nullptr, "out is null");
    vx_graph *g = new vx_graph();
    g->graph = graph;
    hipError_t e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
        (void)hipGraphDestroy(graph);
        delete g;
        return VX_ERR_HIP;
    }
    *out = g;
    return VX_OK;
}

int vx_graph_launch(vx_backend *be, vx_graph *g) {
    int rc = enter(be);
    if (rc) return rc;
    VX_REQUIRE(g && g->exec, "null graph");
    VX_CHECK_HIP(hipGraphLaunch(g->exec, be->stream));
    return VX_OK;
}

void vx_graph_destroy(vx_graph *g) {
    if (!g) return;
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    delete g;
}

int vx_timer_start(vx_backend *be) {
    int rc = enter(be);
    if (rc) return rc;
    VX_CHECK_HIP(hipEventRecord(be->ev0, be->stream));
    return VX_OK;
}

int vx_timer_stop_ms(vx_backend *be, float *ms) {
    int rc = enter(be);
    if (rc) return rc;
    VX_CHECK_HIP(hipEventRecord(be->ev1, be->stream));
    VX_CHECK_HIP(hipEventSynchronize(be->ev1));
    VX_CHECK_HIP(hipEventElapsedTime(ms, be->ev0, be->ev1));
    return VX_OK;
}

}  // extern "C"
