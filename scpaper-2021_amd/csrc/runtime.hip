// Device buffers, streams, events, fills and fp32<->fp16 conversion behind the
// C ABI, plus the status/error plumbing shared by every entry point.
#include <stdarg.h>

#include <new>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.hip.h"

namespace et {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return status;
}

int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return ET_OK;
    int status = ET_ERR_LAUNCH;
    if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) status = ET_ERR_ALLOC;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) status = ET_ERR_NO_DEVICE;
    return fail(status, "%s: %s", what, hipGetErrorString(e));
}

int check_launch(const char *kernel) { return check_hip(hipGetLastError(), kernel); }

template <typename T>
__global__ void fill_kernel(T *dst, size_t n, T value) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) dst[i] = value;
}

__global__ void f32_to_f16_kernel(_Float16 *dst, const float *src, size_t n) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) dst[i] = (_Float16)src[i];  // v_cvt_f16_f32: round-to-nearest-even
}

__global__ void f16_to_f32_kernel(float *dst, const _Float16 *src, size_t n) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) dst[i] = (float)src[i];
}

static inline unsigned grid_for(size_t n, unsigned block) {
    size_t g = (n + block - 1) / block;
    const size_t cap = 256u * 16u;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace et

using namespace et;

extern "C" {

const char *et_status_string(int status) {
    switch (status) {
        case ET_OK: return "ok";
        case ET_ERR_INVALID_ARG: return "invalid argument";
        case ET_ERR_UNSUPPORTED: return "unsupported shape";
        case ET_ERR_ALLOC: return "allocation failed";
        case ET_ERR_LAUNCH: return "HIP launch or copy failed";
        case ET_ERR_IO: return "file error";
        case ET_ERR_NO_DEVICE: return "no usable device";
        default: return "unknown status";
    }
}

const char *et_last_error(void) { return g_err; }

void et_set_last_error(const char *message) { set_error("%s", message ? message : ""); }

int et_device_info(char *name, int cap, int *num_cu, int *lds_bytes) {
    int dev = 0;
    ET_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    ET_HIP(hipGetDeviceProperties(&prop, dev));
    if (name && cap > 0) {
        snprintf(name, (size_t)cap, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (num_cu) *num_cu = prop.multiProcessorCount;
    if (lds_bytes) *lds_bytes = (int)prop.sharedMemPerBlock;
    return ET_OK;
}

// Device memory comes from slabs of 64 MiB.  Where the driver puts separate allocations of a few
// MiB each (a model makes a hundred of them) decides how they are mapped — translation fragments,
// memory channels — and the same encoder stack measured anything between 41.4 and 43.6 us per
// layer from one process start to the next, with the same kernels on the same inputs.  Inside a
// slab every buffer sits at a fixed distance from its neighbours and shares the slab's large
// pages.  A slab goes back to the driver when the last buffer cut from it has been freed and a
// newer slab has taken its place; requests of more than a quarter of a slab get an allocation of
// their own.
namespace {
constexpr size_t kSlabBytes = 64u << 20;
constexpr size_t kSlabAlign = 4096;
struct PrivateScope;
struct Slab {
    PrivateScope *owner = nullptr;  // the open private scope whose list holds this slab (nullptr: g_slabs, or none)
    char *base = nullptr;
    size_t used = 0;
    size_t live = 0;      // buffers cut from this slab and not yet freed
    size_t lead = 0;      // where cutting starts (a private scope may ask for a distance from the slab's start)
    bool current = true;  // still the slab its list cuts from
};
std::mutex g_pool_mu;
std::vector<Slab *> g_slabs;                       // the last one is the one being cut
std::unordered_map<void *, Slab *> g_owner;       // buffer -> its slab (nullptr: an allocation of its own)
// A private scope (et_pool_private_begin): the calling thread cuts from slabs of its own.
struct PrivateScope {
    std::vector<Slab *> slabs;
    size_t lead = 0;
};
thread_local PrivateScope *t_scope = nullptr;
}  // namespace

int et_pool_private_begin(size_t lead_bytes) {
    ET_REQUIRE(t_scope == nullptr, ET_ERR_INVALID_ARG, "et_pool_private_begin: a private scope is already open on this thread");
    ET_REQUIRE(lead_bytes % kSlabAlign == 0 && lead_bytes <= kSlabBytes / 2, ET_ERR_INVALID_ARG,
               "et_pool_private_begin: lead_bytes=%zu must be a multiple of %zu, at most %zu", lead_bytes, kSlabAlign,
               kSlabBytes / 2);
    t_scope = new PrivateScope;
    t_scope->lead = lead_bytes;
    return ET_OK;
}

int et_pool_private_end(void) {
    ET_REQUIRE(t_scope != nullptr, ET_ERR_INVALID_ARG, "et_pool_private_end: no private scope is open on this thread");
    std::vector<void *> release;
    {
        std::lock_guard<std::mutex> lk(g_pool_mu);
        for (Slab *slab : t_scope->slabs) {  // nothing cuts from them any more: each goes when its last buffer does
            slab->current = false;
            slab->owner = nullptr;
            if (slab->live == 0) {
                release.push_back(slab->base);
                delete slab;
            }
        }
    }
    delete t_scope;
    t_scope = nullptr;
    int status = ET_OK;  // every slab is released; the first failure is what the caller hears of
    for (void *p : release) {
        const int s = check_hip(hipFree(p), "hipFree");
        if (status == ET_OK) status = s;
    }
    return status;
}

int et_malloc(void **ptr, size_t bytes) {
    ET_REQUIRE(ptr != nullptr, ET_ERR_INVALID_ARG, "et_malloc: ptr is NULL");
    *ptr = nullptr;
    if (bytes == 0) bytes = 16;  // a valid, distinct pointer even for empty buffers
    void *p = nullptr;
    Slab *slab = nullptr;
    if (bytes <= kSlabBytes / 4) {
        std::lock_guard<std::mutex> lk(g_pool_mu);
        const size_t need = (bytes + kSlabAlign - 1) / kSlabAlign * kSlabAlign;
        std::vector<Slab *> &slabs = t_scope ? t_scope->slabs : g_slabs;
        if (slabs.empty() || slabs.back()->used + need > kSlabBytes) {
            if (!slabs.empty() && slabs.back()->live == 0) {  // nothing left in it: cut it again
                slabs.back()->used = slabs.back()->lead;
            } else {
                void *base = nullptr;
                ET_HIP(hipMalloc(&base, kSlabBytes));
                Slab *fresh = new Slab;
                fresh->base = static_cast<char *>(base);
                fresh->lead = fresh->used = (t_scope && slabs.empty()) ? t_scope->lead : 0;
                fresh->owner = t_scope;
                if (!slabs.empty()) slabs.back()->current = false;
                slabs.push_back(fresh);
            }
        }
        slab = slabs.back();
        p = slab->base + slab->used;
        slab->used += need;
        slab->live++;
        g_owner[p] = slab;
    } else {
        ET_HIP(hipMalloc(&p, bytes));
        std::lock_guard<std::mutex> lk(g_pool_mu);
        g_owner[p] = nullptr;
    }
    int s = check_hip(hipMemset(p, 0, bytes), "hipMemset");
    if (s != ET_OK) {
        (void)et_free(p);
        return s;
    }
    *ptr = p;
    return ET_OK;
}

int et_free(void *ptr) {
    if (!ptr) return ET_OK;
    // hipFree waits for the device before it releases memory; a buffer cut from a slab is handed out
    // again without the driver, so the wait is made here: work still running on the buffer ends first
    ET_HIP(hipDeviceSynchronize());
    void *release = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_pool_mu);
        auto it = g_owner.find(ptr);
        Slab *slab = it != g_owner.end() ? it->second : nullptr;  // memory from elsewhere goes to the driver as before
        if (it != g_owner.end()) g_owner.erase(it);
        if (!slab) {
            release = ptr;
        } else if (--slab->live == 0) {
            if (slab->current) {
                slab->used = slab->lead;  // empty again: cut from its start
            } else {
                release = slab->base;
                auto at = std::find(g_slabs.begin(), g_slabs.end(), slab);
                if (at != g_slabs.end()) g_slabs.erase(at);
                if (slab->owner) {  // a scope that is still open, on this thread or another: its list lets go of the slab
                    auto &theirs = slab->owner->slabs;
                    auto mine = std::find(theirs.begin(), theirs.end(), slab);
                    if (mine != theirs.end()) theirs.erase(mine);
                }
                delete slab;
            }
        }
    }
    if (release) ET_HIP(hipFree(release));
    return ET_OK;
}

int et_memset(void *ptr, int byte, size_t bytes, et_stream stream) {
    ET_REQUIRE(ptr != nullptr || bytes == 0, ET_ERR_INVALID_ARG, "et_memset: ptr is NULL");
    if (bytes == 0) return ET_OK;
    // A fill kernel rather than hipMemsetAsync, so that a caller may record
    // this call into a HIP graph.
    const uint32_t b = (uint32_t)(byte & 0xff);
    if ((reinterpret_cast<uintptr_t>(ptr) | bytes) % 4 == 0) {
        fill_kernel<uint32_t><<<grid_for(bytes / 4, 256), 256, 0, as_stream(stream)>>>(
            static_cast<uint32_t *>(ptr), bytes / 4, b * 0x01010101u);
    } else {
        fill_kernel<uint8_t><<<grid_for(bytes, 256), 256, 0, as_stream(stream)>>>(
            static_cast<uint8_t *>(ptr), bytes, (uint8_t)b);
    }
    return check_launch("fill_kernel<bytes>");
}

int et_memcpy_h2d(void *dst, const void *src_host, size_t bytes) {
    ET_REQUIRE((dst && src_host) || bytes == 0, ET_ERR_INVALID_ARG, "et_memcpy_h2d: NULL pointer");
    if (bytes == 0) return ET_OK;
    ET_HIP(hipMemcpy(dst, src_host, bytes, hipMemcpyHostToDevice));
    return ET_OK;
}

int et_memcpy_d2h(void *dst_host, const void *src, size_t bytes) {
    ET_REQUIRE((dst_host && src) || bytes == 0, ET_ERR_INVALID_ARG, "et_memcpy_d2h: NULL pointer");
    if (bytes == 0) return ET_OK;
    ET_HIP(hipMemcpy(dst_host, src, bytes, hipMemcpyDeviceToHost));
    return ET_OK;
}

int et_memcpy_auto(void *dst, const void *src, size_t bytes) {
    ET_REQUIRE((dst && src) || bytes == 0, ET_ERR_INVALID_ARG, "et_memcpy_auto: NULL pointer");
    if (bytes == 0) return ET_OK;
    // the runtime tells host from device memory by the address (unified addressing)
    ET_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDefault));
    return ET_OK;
}

int et_memcpy_d2d(void *dst, const void *src, size_t bytes, et_stream stream) {
    ET_REQUIRE((dst && src) || bytes == 0, ET_ERR_INVALID_ARG, "et_memcpy_d2d: NULL pointer");
    if (bytes == 0) return ET_OK;
    ET_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return ET_OK;
}

int et_fill_f16(et_f16 *dst, size_t n, et_f16 value, et_stream stream) {
    ET_REQUIRE(dst != nullptr || n == 0, ET_ERR_INVALID_ARG, "et_fill_f16: dst is NULL");
    if (n == 0) return ET_OK;
    fill_kernel<uint16_t><<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(dst, n, value);
    return check_launch("fill_kernel<u16>");
}

int et_fill_i32(int32_t *dst, size_t n, int32_t value, et_stream stream) {
    ET_REQUIRE(dst != nullptr || n == 0, ET_ERR_INVALID_ARG, "et_fill_i32: dst is NULL");
    if (n == 0) return ET_OK;
    fill_kernel<int32_t><<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(dst, n, value);
    return check_launch("fill_kernel<i32>");
}

int et_f32_to_f16(et_f16 *dst, const float *src, size_t n, et_stream stream) {
    ET_REQUIRE((dst && src) || n == 0, ET_ERR_INVALID_ARG, "et_f32_to_f16: NULL pointer");
    if (n == 0) return ET_OK;
    f32_to_f16_kernel<<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(dst), src, n);
    return check_launch("f32_to_f16_kernel");
}

int et_f16_to_f32(float *dst, const et_f16 *src, size_t n, et_stream stream) {
    ET_REQUIRE((dst && src) || n == 0, ET_ERR_INVALID_ARG, "et_f16_to_f32: NULL pointer");
    if (n == 0) return ET_OK;
    f16_to_f32_kernel<<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(
        dst, reinterpret_cast<const _Float16 *>(src), n);
    return check_launch("f16_to_f32_kernel");
}

int et_stream_create(et_stream *stream) {
    ET_REQUIRE(stream != nullptr, ET_ERR_INVALID_ARG, "et_stream_create: stream is NULL");
    hipStream_t s;
    ET_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return ET_OK;
}

int et_stream_destroy(et_stream stream) {
    if (!stream) return ET_OK;
    ET_HIP(hipStreamDestroy(as_stream(stream)));
    return ET_OK;
}

int et_stream_sync(et_stream stream) {
    ET_HIP(hipStreamSynchronize(as_stream(stream)));
    return ET_OK;
}

int et_device_sync(void) {
    ET_HIP(hipDeviceSynchronize());
    return ET_OK;
}

int et_graph_begin_capture(et_stream stream) {
    ET_REQUIRE(stream != nullptr, ET_ERR_INVALID_ARG,
               "et_graph_begin_capture: capture needs a stream from et_stream_create");
    ET_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeRelaxed));
    return ET_OK;
}

// An et_graph keeps the captured template together with its executable instance and destroys
// them in that order (instance first) at et_graph_destroy: the instance is never left referring
// to a template that is already gone.
struct GraphPair {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

int et_graph_end_capture(et_stream stream, et_graph *graph) {
    ET_REQUIRE(stream != nullptr && graph != nullptr, ET_ERR_INVALID_ARG,
               "et_graph_end_capture: NULL argument");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    ET_HIP(hipStreamEndCapture(as_stream(stream), &g));
    hipGraphExec_t exec = nullptr;
    int s = check_hip(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0), "hipGraphInstantiate");
    if (s != ET_OK) {
        (void)hipGraphDestroy(g);
        return s;
    }
    GraphPair *pair = new (std::nothrow) GraphPair;
    if (!pair) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(g);
        return fail(ET_ERR_ALLOC, "et_graph_end_capture: out of host memory");
    }
    pair->graph = g;
    pair->exec = exec;
    *graph = pair;
    return ET_OK;
}

int et_graph_launch(et_graph graph, et_stream stream) {
    ET_REQUIRE(graph != nullptr, ET_ERR_INVALID_ARG, "et_graph_launch: graph is NULL");
    ET_HIP(hipGraphLaunch(static_cast<GraphPair *>(graph)->exec, as_stream(stream)));
    return ET_OK;
}

int et_graph_destroy(et_graph graph) {
    if (!graph) return ET_OK;
    GraphPair *pair = static_cast<GraphPair *>(graph);
    // replays still in flight hold the instance's kernel arguments: drain before it goes
    hipError_t e0 = hipDeviceSynchronize();
    hipError_t e1 = hipGraphExecDestroy(pair->exec);
    hipError_t e2 = hipGraphDestroy(pair->graph);
    delete pair;
    ET_HIP(e0);
    ET_HIP(e1);
    ET_HIP(e2);
    return ET_OK;
}

int et_event_create(et_event *ev) {
    ET_REQUIRE(ev != nullptr, ET_ERR_INVALID_ARG, "et_event_create: ev is NULL");
    hipEvent_t e;
    ET_HIP(hipEventCreate(&e));
    *ev = e;
    return ET_OK;
}

int et_event_destroy(et_event ev) {
    if (!ev) return ET_OK;
    ET_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
    return ET_OK;
}

int et_event_record(et_event ev, et_stream stream) {
    ET_REQUIRE(ev != nullptr, ET_ERR_INVALID_ARG, "et_event_record: ev is NULL");
    ET_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(stream)));
    return ET_OK;
}

int et_event_sync(et_event ev) {
    ET_REQUIRE(ev != nullptr, ET_ERR_INVALID_ARG, "et_event_sync: ev is NULL");
    ET_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)));
    return ET_OK;
}

int et_event_elapsed_ms(float *ms, et_event start, et_event stop) {
    ET_REQUIRE(ms && start && stop, ET_ERR_INVALID_ARG, "et_event_elapsed_ms: NULL argument");
    ET_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                               reinterpret_cast<hipEvent_t>(stop)));
    return ET_OK;
}

}  // extern "C"
