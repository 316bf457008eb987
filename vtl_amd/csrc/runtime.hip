// Device, memory, transfer, stream and timing entry points of libvtlhip.so.
// These are the calls the V-side HipStorage makes where CudaStorage calls
// cudaMalloc / cudaMemcpy / cudaFree (storage/cuda_d_cuda.v:32-102).
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "common.hpp"

namespace vtlhip {

// per host thread, like HIP's current device: one host thread drives one device
static thread_local hipStream_t g_stream = nullptr;
static thread_local char g_last_error[256] = "";

hipStream_t current_stream() { return g_stream; }

int record_hip_error(hipError_t e, const char *what)
{
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s (%d)", what, hipGetErrorString(e), (int)e);
    (void)hipGetLastError();  // clear the sticky per-thread error
    if (e == hipErrorOutOfMemory)
        return VTL_HIP_ERR_OUT_OF_MEMORY;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice)
        return VTL_HIP_ERR_NO_DEVICE;
    return VTL_HIP_ERR_RUNTIME;
}

int check_launch(const char *kernel_name)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return record_hip_error(e, kernel_name);
    return VTL_HIP_OK;
}

// The switches are published as an immutable snapshot behind an atomic pointer:
// a launch that reads them while vtl_hip_reload_env() runs on another thread
// sees the old snapshot or the new one, never a half-written struct.  Replaced
// snapshots are not freed (a reader may still hold one; a reload is a test and
// tuning aid, a few dozen bytes each).
static std::atomic<const Tuning *> g_tuning{nullptr};
static std::mutex g_tuning_mutex;

static const Tuning *read_tuning(bool force)
{
    std::lock_guard<std::mutex> lock(g_tuning_mutex);  // two first callers at once: one reads, the other waits
    if (!force) {
        if (const Tuning *seen = g_tuning.load(std::memory_order_acquire))
            return seen;
    }
    Tuning *t = new Tuning;
    auto flag = [](const char *name) { return getenv(name) != nullptr; };
    auto number = [](const char *name, int unset) {
        const char *v = getenv(name);
        return v ? atoi(v) : unset;
    };
    t->no_gemv = flag("VTL_HIP_NO_GEMV");
    t->gemv_rows = number("VTL_HIP_GEMV_ROWS", -1);
    t->gemm_small = number("VTL_HIP_GEMM_SMALL", -1);
    if (const char *v = getenv("VTL_HIP_GEMM_CONFIG")) {
        int idx = -1, splits = 1;
        // a value that does not parse still takes the launch off the special-case kernels
        t->gemm_config = (sscanf(v, "%d,%d", &idx, &splits) >= 1 && idx >= 0) ? idx : 1 << 30;
        t->gemm_splits = splits;
    }
    t->no_fused_requant = flag("VTL_HIP_NO_FUSED_REQUANT");
    t->requant_wide = number("VTL_HIP_REQUANT_WIDE", 0);
    t->quant_four_launches = flag("VTL_HIP_QUANT_FOUR_LAUNCHES");
    t->no_fused_decode = flag("VTL_HIP_NO_FUSED_DECODE");
    t->stage_spin = number("VTL_HIP_STAGE_SPIN", 4096);
    if (t->stage_spin < 0 || t->stage_spin > (1 << 20))
        t->stage_spin = 4096;
    t->stream_weights_mib = number("VTL_HIP_STREAM_WEIGHTS_MIB", 48);
    if (t->stream_weights_mib < 0 || t->stream_weights_mib > (1 << 20))
        t->stream_weights_mib = 48;
    t->skinny_tiled = number("VTL_HIP_SKINNY_TILED", -1);
    t->skinny_waves = number("VTL_HIP_SKINNY_WAVES", 4);
    t->matmul_tile = number("VTL_HIP_MATMUL_TILE", 0);
    t->matmul_splits = number("VTL_HIP_MATMUL_SPLITS", -1);
    g_tuning.store(t, std::memory_order_release);
    return t;
}

const Tuning &tuning()
{
    const Tuning *t = g_tuning.load(std::memory_order_acquire);
    return t ? *t : *read_tuning(false);
}

// ---- scratch for callers that cannot allocate --------------------------------
// One array per device, part of the code object, so it exists from the moment
// the library is loaded on a device until the process ends.  Host code never
// uses the array's name as an address: static_scratch() asks the runtime for
// the device address (once per device) and everything else goes through that
// pointer.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices] = {};

static int current_device()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return -1;
    }
    return dev;
}

int stream_slot(hipStream_t st)
{
    struct Table {
        std::mutex lock;
        hipStream_t stream[kStreamSlots] = {};
        bool taken[kStreamSlots] = {};
    };
    static Table tables[kMaxDevices];
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    if (capturing != hipStreamCaptureStatusNone)
        return -1;
    const int dev = current_device();
    if (dev < 0)
        return -1;
    Table &t = tables[dev];
    std::lock_guard<std::mutex> hold(t.lock);
    for (int i = 0; i < kStreamSlots; i++)
        if (t.taken[i] && t.stream[i] == st)
            return i;
    for (int i = 0; i < kStreamSlots; i++)
        if (!t.taken[i]) {
            t.taken[i] = true;
            t.stream[i] = st;
            return i;
        }
    return -1;
}

void *static_scratch()
{
    const int dev = current_device();
    if (dev < 0)
        return nullptr;
    if (!g_scratch_ptr[dev].load(std::memory_order_acquire)) {   // two first callers resolve the same address
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            (void)record_hip_error(e, "hipGetSymbolAddress(scratch)");
            return nullptr;
        }
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    return g_scratch_ptr[dev].load(std::memory_order_acquire);
}

// While a ScratchArena is alive on this thread, library_workspace() hands out
// consecutive pieces of it instead of the library's own growing buffers.
static thread_local ScratchArena *g_arena = nullptr;
static thread_local int g_workspace_status = VTL_HIP_OK;

ScratchArena::ScratchArena(void *base_, size_t capacity_) : base(static_cast<char *>(base_)), capacity(capacity_)
{
    g_arena = this;
}

ScratchArena::~ScratchArena() { g_arena = nullptr; }

int workspace_status() { return g_workspace_status; }

void *library_workspace(size_t bytes, int slot)
{
    static void *bufs[3][kMaxDevices] = {};
    static size_t caps[3][kMaxDevices] = {};
    static bool captured[3][kMaxDevices] = {};   // the buffer's address is baked into a recorded graph
    g_workspace_status = VTL_HIP_OK;
    if (slot < 0 || slot > 2) {
        g_workspace_status = VTL_HIP_ERR_INVALID_ARG;
        return nullptr;
    }
    if (g_arena) {
        const size_t take = (bytes + 255) & ~(size_t)255;
        if (take > g_arena->capacity - g_arena->used) {
            snprintf(g_last_error, sizeof(g_last_error),
                     "call needs %zu more bytes of scratch, the static scratch of %zu bytes has %zu left", take,
                     g_arena->capacity, g_arena->capacity - g_arena->used);
            g_workspace_status = VTL_HIP_ERR_UNSUPPORTED;
            return nullptr;
        }
        void *p = g_arena->base + g_arena->used;
        g_arena->used += take;
        return p;
    }
    void **buf = bufs[slot];
    size_t *cap = caps[slot];
    bool *in_graph = captured[slot];
    const int dev = current_device();
    if (dev < 0) {
        g_workspace_status = VTL_HIP_ERR_NO_DEVICE;
        return nullptr;
    }
    // Is the current stream recording a graph?  A query that fails counts as "yes": the
    // cautious answer, since growing frees and allocates and neither may happen then.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(current_stream(), &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusActive;
    }
    const bool recording = capturing != hipStreamCaptureStatusNone;
    if (bytes > cap[dev]) {
        if (recording) {
            snprintf(g_last_error, sizeof(g_last_error),
                     "library scratch would have to grow to %zu bytes during a stream capture: pass a workspace "
                     "of your own, use the entry point that allocates nothing, or run the call once before "
                     "capturing",
                     bytes);
            g_workspace_status = VTL_HIP_ERR_UNSUPPORTED;
            return nullptr;
        }
        if (buf[dev] && !in_graph[dev]) {
            (void)hipDeviceSynchronize();   // every stream: the buffer is shared by all of them
            (void)hipFree(buf[dev]);
        }
        // A buffer that a recorded graph refers to is never freed: replays of that graph keep
        // writing to it.  It stays allocated until the process ends and a new one takes its place.
        buf[dev] = nullptr;
        cap[dev] = 0;
        in_graph[dev] = false;
        const size_t want = bytes < (size_t(32) << 20) ? (size_t(32) << 20) : bytes;
        if (hipMalloc(&buf[dev], want) != hipSuccess) {
            (void)hipGetLastError();
            buf[dev] = nullptr;
            g_workspace_status = VTL_HIP_ERR_OUT_OF_MEMORY;
            return nullptr;
        }
        cap[dev] = want;
    }
    if (recording)
        in_graph[dev] = true;
    return buf[dev];
}

// Byte fill as a kernel (a memset node recorded into a caller's graph is avoided this way):
// bytes up to the first 16-byte boundary, 16-byte vectors, remaining bytes.
__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char *p, unsigned word, size_t head, size_t nvec,
                                                         size_t tail)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nvec)
        reinterpret_cast<uint4 *>(p + head)[i] = make_uint4(word, word, word, word);
    if (i < head)
        p[i] = (unsigned char)word;
    if (i < tail)
        p[head + nvec * 16 + i] = (unsigned char)word;
}

}  // namespace vtlhip

using namespace vtlhip;

extern "C" {

int vtl_hip_device_count(int *n)
{
    if (!n)
        return VTL_HIP_ERR_INVALID_ARG;
    *n = 0;
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess)
        return record_hip_error(e, "hipGetDeviceCount");
    *n = c;
    return VTL_HIP_OK;
}

int vtl_hip_set_device(int device_id)
{
    int c = 0;
    int st = vtl_hip_device_count(&c);
    if (st != VTL_HIP_OK)
        return st;
    if (device_id < 0 || device_id >= c)
        return VTL_HIP_ERR_NO_DEVICE;
    VTL_HIP_TRY(hipSetDevice(device_id));
    (void)static_scratch();   // resolved here so that a later call under stream capture finds it ready
    return VTL_HIP_OK;
}

int vtl_hip_device_info(char *name, size_t name_cap, int *compute_units, int *clock_mhz)
{
    int dev = 0;
    VTL_HIP_TRY(hipGetDevice(&dev));
    hipDeviceProp_t p;
    VTL_HIP_TRY(hipGetDeviceProperties(&p, dev));
    if (name && name_cap) {
        // some driver stacks leave the marketing name empty
        snprintf(name, name_cap, "%s (%s)", p.name[0] ? p.name : "AMD GPU", p.gcnArchName);
    }
    if (compute_units)
        *compute_units = p.multiProcessorCount;
    if (clock_mhz)
        *clock_mhz = p.clockRate / 1000;
    return VTL_HIP_OK;
}

int vtl_hip_malloc(void **dptr, size_t bytes)
{
    if (!dptr || bytes == 0)
        return VTL_HIP_ERR_INVALID_ARG;
    *dptr = nullptr;
    VTL_HIP_TRY(hipMalloc(dptr, bytes));
    return VTL_HIP_OK;
}

int vtl_hip_free(void *dptr)
{
    if (!dptr)
        return VTL_HIP_OK;  // CudaStorage.release() skips nil too
    VTL_HIP_TRY(hipFree(dptr));
    return VTL_HIP_OK;
}

int vtl_hip_memcpy_h2d(void *dst_device, const void *src_host, size_t bytes)
{
    if (bytes == 0)
        return VTL_HIP_OK;
    if (!dst_device || !src_host)
        return VTL_HIP_ERR_INVALID_ARG;
    VTL_HIP_TRY(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, current_stream()));
    VTL_HIP_TRY(hipStreamSynchronize(current_stream()));
    return VTL_HIP_OK;
}

int vtl_hip_memcpy_d2h(void *dst_host, const void *src_device, size_t bytes)
{
    if (bytes == 0)
        return VTL_HIP_OK;
    if (!dst_host || !src_device)
        return VTL_HIP_ERR_INVALID_ARG;
    VTL_HIP_TRY(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, current_stream()));
    VTL_HIP_TRY(hipStreamSynchronize(current_stream()));
    return VTL_HIP_OK;
}

int vtl_hip_memcpy_d2d(void *dst_device, const void *src_device, size_t bytes)
{
    if (bytes == 0)
        return VTL_HIP_OK;
    if (!dst_device || !src_device)
        return VTL_HIP_ERR_INVALID_ARG;
    if (launch_copy(dst_device, src_device, bytes, current_stream()))
        return check_launch("copy_kernel");
    VTL_HIP_TRY(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, current_stream()));
    return VTL_HIP_OK;
}

int vtl_hip_memset(void *dst_device, int byte_value, size_t bytes)
{
    if (bytes == 0)
        return VTL_HIP_OK;
    if (!dst_device)
        return VTL_HIP_ERR_INVALID_ARG;
    unsigned char *p = static_cast<unsigned char *>(dst_device);
    size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15;
    if (head > bytes)
        head = bytes;
    const size_t nvec = (bytes - head) >> 4, tail = (bytes - head) & 15;
    const size_t blocks = ((nvec > 16 ? nvec : 16) + 255) / 256;
    if (blocks > 0x7fffffffULL)
        return VTL_HIP_ERR_UNSUPPORTED;
    const unsigned word = 0x01010101u * (unsigned)(byte_value & 0xff);
    hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, current_stream(), p, word, head, nvec,
                       tail);
    return check_launch("fill_bytes_kernel");
}

int vtl_hip_sync(void)
{
    VTL_HIP_TRY(hipStreamSynchronize(current_stream()));
    return VTL_HIP_OK;
}

int vtl_hip_set_stream(void *hip_stream)
{
    g_stream = (hipStream_t)hip_stream;
    return VTL_HIP_OK;
}

int vtl_hip_get_stream(void **hip_stream)
{
    if (!hip_stream)
        return VTL_HIP_ERR_INVALID_ARG;
    *hip_stream = (void *)g_stream;
    return VTL_HIP_OK;
}

int vtl_hip_event_create(void **event)
{
    if (!event)
        return VTL_HIP_ERR_INVALID_ARG;
    hipEvent_t e;
    VTL_HIP_TRY(hipEventCreate(&e));
    *event = (void *)e;
    return VTL_HIP_OK;
}

int vtl_hip_event_destroy(void *event)
{
    if (!event)
        return VTL_HIP_OK;
    VTL_HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return VTL_HIP_OK;
}

int vtl_hip_event_record(void *event)
{
    if (!event)
        return VTL_HIP_ERR_INVALID_ARG;
    VTL_HIP_TRY(hipEventRecord((hipEvent_t)event, current_stream()));
    return VTL_HIP_OK;
}

int vtl_hip_event_elapsed_ms(void *start, void *stop, float *ms)
{
    if (!start || !stop || !ms)
        return VTL_HIP_ERR_INVALID_ARG;
    VTL_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
    VTL_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return VTL_HIP_OK;
}

const char *vtl_hip_strerror(int status)
{
    switch (status) {
    case VTL_HIP_OK: return "success";
    case VTL_HIP_ERR_INVALID_ARG: return "invalid argument (null pointer, bad size or flag)";
    case VTL_HIP_ERR_NO_DEVICE: return "no usable HIP device";
    case VTL_HIP_ERR_RUNTIME: return "HIP runtime call failed";
    case VTL_HIP_ERR_OUT_OF_MEMORY: return "out of device memory";
    case VTL_HIP_ERR_UNSUPPORTED: return "shape not supported by the gfx950 kernels";
    default: return "unknown status";
    }
}

const char *vtl_hip_last_error(void) { return g_last_error; }

int vtl_hip_reload_env(void)
{
    (void)read_tuning(true);
    return VTL_HIP_OK;
}

const char *vtl_hip_version(void) { return "vtlhip 0.1 (gfx950)"; }

}  // extern "C"
