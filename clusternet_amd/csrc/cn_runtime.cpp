// Library state: status strings, per-device contexts, memory helpers.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "cn_internal.h"
#include "cn_xlut.h"

namespace cn {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

cn_status hip_fail(hipError_t e, const char *what, const char *file, int line) {
    set_error("%s failed: %s (%s:%d)", what, hipGetErrorString(e), file, line);
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) return CN_ERR_NO_DEVICE;
    return CN_ERR_HIP;
}

void host_table(float out[126]);

int g_reduction_fences = 0;

static Context g_ctx[kMaxDevices];
static std::mutex g_mutex;

size_t default_workspace_bytes() {
    size_t mib = 1024;
    if (const char *env = getenv("CNHIP_WORKSPACE_MB")) {
        long v = atol(env);
        if (v >= 16) mib = (size_t)v;
    }
    return mib << 20;
}

size_t planning_workspace_bytes(int device) {
    if (device >= 0 && device < kMaxDevices && g_ctx[device].ready) return g_ctx[device].workspace_bytes;
    return default_workspace_bytes();
}

static cn_status init_device(int device) {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        set_error("no HIP device available (%s)", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
        return CN_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= count || device >= kMaxDevices) {
        set_error("device %d out of range (%d visible)", device, count);
        return CN_ERR_NO_DEVICE;
    }
    Context &c = g_ctx[device];
    if (c.ready) return CN_OK;

    int previous = 0;
    CN_HIP(hipGetDevice(&previous));
    CN_HIP(hipSetDevice(device));
    // On any failure below: what was allocated so far is released, the context stays unready and the caller's
    // device is current again, so that a later attempt starts from nothing instead of leaking another set.
    struct Undo {
        Context &c;
        int previous;
        bool armed = true;
        ~Undo() {
            if (!armed) return;
            (void)hipFree(c.table);
            (void)hipFree(c.xsteps);
            (void)hipFree(c.quotient_table);
            (void)hipFree(c.workspace);
            (void)hipFree(c.reduce_scratch);
            (void)hipFree(c.tickets);
            (void)hipFree(c.sum_scratch);
            (void)hipFree(c.tile_queue);
            c = Context();
            (void)hipSetDevice(previous);
        }
    } undo{c, previous};
    hipDeviceProp_t prop;
    CN_HIP(hipGetDeviceProperties(&prop, device));
    c.device = device;
    c.num_cu = prop.multiProcessorCount;

    float table[126];
    host_table(table);
    CN_HIP(hipMalloc((void **)&c.table, sizeof(table)));
    CN_HIP(hipMemcpy(c.table, table, sizeof(table), hipMemcpyHostToDevice));

    {
        float slot[128];
        host_table(slot);
        slot[126] = 1.0f;
        slot[127] = 0.0f;
        static XStep steps[kXMaxSteps];
        const int count = xlut_collect_steps(slot, steps);
        if (count <= 0 || count + 2 > 256) { set_error("init: the encoder's step list could not be derived"); return CN_ERR_ARG; }
        c.xstep_count = count;
        CN_HIP(hipMalloc((void **)&c.xsteps, sizeof(steps)));
        CN_HIP(hipMemcpy(c.xsteps, steps, sizeof(steps), hipMemcpyHostToDevice));
        // the table for precision 1, where the quotient is the operand itself: the code as a function of the quotient
        static XEntry of_quotient[kXEntries];
        if (!xlut_build_from_steps(steps, count, 1.0f, slot, of_quotient)) {
            set_error("init: the encoder's table on the quotient could not be built");
            return CN_ERR_ARG;
        }
        CN_HIP(hipMalloc((void **)&c.quotient_table, sizeof(of_quotient)));
        CN_HIP(hipMemcpy(c.quotient_table, of_quotient, sizeof(of_quotient), hipMemcpyHostToDevice));
    }

    c.workspace_bytes = default_workspace_bytes();
    CN_HIP(hipMalloc(&c.workspace, c.workspace_bytes));

    CN_HIP(hipMalloc((void **)&c.reduce_scratch, (kReduceSlots + 64) * sizeof(uint32_t)));
    CN_HIP(hipMemset(c.reduce_scratch, 0, (kReduceSlots + 64) * sizeof(uint32_t)));
    CN_HIP(hipMalloc((void **)&c.tickets, kTicketWords * sizeof(uint32_t)));
    CN_HIP(hipMemset(c.tickets, 0, kTicketWords * sizeof(uint32_t)));
    CN_HIP(hipMalloc((void **)&c.sum_scratch, 1024 * sizeof(double)));
    CN_HIP(hipMalloc((void **)&c.tile_queue, kTileQueueWords * sizeof(uint32_t)));
    CN_HIP(hipMemset(c.tile_queue, 0, kTileQueueWords * sizeof(uint32_t)));
    {
        const cn_status located = gemm_static_setup(device);
        if (located != CN_OK) return located;
    }
    CN_HIP(hipDeviceSynchronize());
    CN_HIP(hipSetDevice(previous));
    undo.armed = false;
    c.ready = true;
    return CN_OK;
}

cn_status current_context(Context **out) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        set_error("no HIP device available (%s)", hipGetErrorString(e));
        return CN_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= kMaxDevices) {
        set_error("device %d out of range", device);
        return CN_ERR_NO_DEVICE;
    }
    if (!g_ctx[device].ready) {
        std::lock_guard<std::mutex> lock(g_mutex);
        cn_status s = init_device(device);
        if (s != CN_OK) return s;
    }
    *out = &g_ctx[device];
    return CN_OK;
}

Context *ready_context(int device) {
    return (device >= 0 && device < kMaxDevices && g_ctx[device].ready) ? &g_ctx[device] : nullptr;
}

static std::mutex g_slots_mutex;

uint32_t *Context::tile_counter_for(hipStream_t stream) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
        (void)hipGetLastError();  // the query's failure is not the caller's: the kernel simply does not draw
        return nullptr;
    }
    if (capture != hipStreamCaptureStatusNone) return nullptr;
    std::lock_guard<std::mutex> lock(g_slots_mutex);
    const int slot = tile_queue_owners.slot_for(stream);
    return slot < 0 ? nullptr : tile_queue + (size_t)slot * 32u;
}

}  // namespace cn

using namespace cn;

extern "C" {

// Test hook: the slots a fresh table of counter owners hands to the keys in turn (pure host logic).
void cn_host_stream_slots(const uint64_t *keys, int n, int *slots_out) {
    StreamSlots table;
    for (int i = 0; i < n; ++i) slots_out[i] = table.slot_for(reinterpret_cast<const void *>((uintptr_t)keys[i]));
}

const char *cn_status_string(cn_status s) {
    switch (s) {
        case CN_OK: return "CN_OK";
        case CN_ERR_NULL: return "CN_ERR_NULL";
        case CN_ERR_SHAPE: return "CN_ERR_SHAPE";
        case CN_ERR_NO_DEVICE: return "CN_ERR_NO_DEVICE";
        case CN_ERR_HIP: return "CN_ERR_HIP";
        case CN_ERR_WORKSPACE: return "CN_ERR_WORKSPACE";
        case CN_ERR_ARG: return "CN_ERR_ARG";
        default: return "CN_ERR_UNKNOWN";
    }
}

const char *cn_last_error(void) { return g_error; }

void cn_host_reduction_fences(int enabled) { g_reduction_fences = enabled != 0; }

// Test hook: after a device synchronisation, the number of ticket counters of the current device that are not zero
// (kernels that draw their tiles leave theirs at zero), or -1 if the device is not initialised.
int cn_host_tile_counters_in_use(void) {
    Context *c;
    if (current_context(&c) != CN_OK) return -1;
    uint32_t words[kTileQueueWords];
    if (hipDeviceSynchronize() != hipSuccess) return -1;
    if (hipMemcpy(words, c->tile_queue, sizeof(words), hipMemcpyDeviceToHost) != hipSuccess) return -1;
    int busy = 0;
    for (int q = 0; q < kTileQueues; ++q) busy += words[q * 32] != 0u;
    return busy;
}

cn_status cn_init(int device) {
    std::lock_guard<std::mutex> lock(g_mutex);
    return init_device(device);
}

cn_status cn_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    int previous = 0;
    bool have_prev = hipGetDevice(&previous) == hipSuccess;
    for (int d = 0; d < kMaxDevices; ++d) {
        Context &c = g_ctx[d];
        if (!c.ready) continue;
        CN_HIP(hipSetDevice(d));
        CN_HIP(hipDeviceSynchronize());
        CN_HIP(hipFree(c.table));
        CN_HIP(hipFree(c.xsteps));
        CN_HIP(hipFree(c.quotient_table));
        CN_HIP(hipFree(c.workspace));
        CN_HIP(hipFree(c.reduce_scratch));
        CN_HIP(hipFree(c.tickets));
        CN_HIP(hipFree(c.sum_scratch));
        CN_HIP(hipFree(c.tile_queue));
        c = Context();
    }
    if (have_prev) CN_HIP(hipSetDevice(previous));
    return CN_OK;
}

int cn_num_compute_units(void) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 0;
    return g_ctx[device].ready ? g_ctx[device].num_cu : 0;
}

cn_status cn_malloc(void **device_ptr, size_t bytes) {
    if (!device_ptr) { set_error("cn_malloc: NULL result pointer"); return CN_ERR_NULL; }
    *device_ptr = nullptr;
    if (bytes == 0) return CN_OK;
    CN_HIP(hipMalloc(device_ptr, bytes));
    return CN_OK;
}

cn_status cn_free(void *device_ptr) {
    if (!device_ptr) return CN_OK;
    CN_HIP(hipFree(device_ptr));
    return CN_OK;
}

cn_status cn_memcpy_h2d(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return CN_OK;
    if (!dst || !src) { set_error("cn_memcpy_h2d: NULL pointer"); return CN_ERR_NULL; }
    CN_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return CN_OK;
}

cn_status cn_memcpy_d2h(void *dst, const void *src, size_t bytes) {
    if (bytes == 0) return CN_OK;
    if (!dst || !src) { set_error("cn_memcpy_d2h: NULL pointer"); return CN_ERR_NULL; }
    CN_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return CN_OK;
}

cn_status cn_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return CN_OK;
    if (!dst || !src) { set_error("cn_memcpy_d2d: NULL pointer"); return CN_ERR_NULL; }
    CN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return CN_OK;
}

cn_status cn_synchronize(void *stream) {
    CN_HIP(hipStreamSynchronize((hipStream_t)stream));
    return CN_OK;
}

cn_status cn_table_get(float out_host[126]) {
    if (!out_host) { set_error("cn_table_get: NULL pointer"); return CN_ERR_NULL; }
    host_table(out_host);
    return CN_OK;
}

}  // extern "C"
