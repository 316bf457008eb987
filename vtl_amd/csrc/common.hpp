// Shared declarations of libvtlhip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vtl_hip.h"

namespace vtlhip {

// Stream every compute entry point enqueues on (nullptr = the null stream).
hipStream_t current_stream();

// Records a failed HIP runtime call for vtl_hip_last_error() and maps it to a
// status code of the C ABI.
int record_hip_error(hipError_t e, const char *what);

// Checks the launch that was just made.
int check_launch(const char *kernel_name);

// Streaming copy kernel (quant.hip); false when alignment or size do not qualify.
bool launch_copy(void *dst, const void *src, size_t bytes, hipStream_t st);

// Device scratch owned by the library: per device three independent buffers
// (slot 0: split-K partial sums and partial column sums; slot 1: quantized
// activations staged between the two launches of a dynamic-quantization call;
// slot 2: int8 operands repacked to a row length the fast kernels take),
// grown on demand and kept until the process ends.  Kernels enqueued on the
// current stream may use a slot until the next call that asks for it; nullptr
// when the allocation fails.  While the current stream records a graph a slot
// is handed out only if it is already large enough (growing would free and
// allocate), and a buffer handed out then is never freed afterwards, because
// replays of the graph keep using its address: a later, larger request gets a
// new buffer and the old one stays allocated.
void *library_workspace(size_t bytes, int slot = 0);
// Why the last library_workspace() call of this thread returned nullptr
// (VTL_HIP_ERR_OUT_OF_MEMORY, or VTL_HIP_ERR_UNSUPPORTED when the request does
// not fit the static scratch or would have to allocate during a stream capture).
int workspace_status();

// A small index (0 .. kStreamSlots - 1) that belongs to `st` on the current device, for code
// that keeps a little state in device memory between its launches and must not share it with
// work that may run at the same time: the first kStreamSlots streams that ask get one each, for
// as long as the process lives (a stream handle that is reused inherits its predecessor's
// index, which is as good).  -1 when none is left, when the stream is being captured into a
// graph (a replay would meet the state of another moment) or when that cannot be found out.
constexpr int kStreamSlots = 16;
int stream_slot(hipStream_t st);

// Static per-device scratch for the entry point that allocates nothing, and the
// scope during which library_workspace() serves from it.  static_scratch()
// returns the device address of the current device's array (nullptr on error).
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
void *static_scratch();
struct ScratchArena {
    char *base;
    size_t capacity, used = 0;
    ScratchArena(void *base_, size_t capacity_);
    ~ScratchArena();
    ScratchArena(const ScratchArena &) = delete;
    ScratchArena &operator=(const ScratchArena &) = delete;
};

// Tuning and test switches, taken from the environment once (first use) and
// again only when vtl_hip_reload_env() is called: the dispatch path of a launch
// reads this struct, never the environment.
struct Tuning {
    bool no_gemv = false;           // VTL_HIP_NO_GEMV: keep M <= 8 off the matrix-vector kernels
    int gemv_rows = -1;             // VTL_HIP_GEMV_ROWS: 1 / 0 force the few-token kernel on / off
    int gemm_small = -1;            // VTL_HIP_GEMM_SMALL: 1 / 0 force the small-product kernel on / off
    int gemm_config = -1;           // VTL_HIP_GEMM_CONFIG "<tile index>,<splits>"
    int gemm_splits = 1;
    bool no_fused_requant = false;  // VTL_HIP_NO_FUSED_REQUANT: linear, then the row quantizer
    int requant_wide = 0;           // VTL_HIP_REQUANT_WIDE: 1 row maxima in the tile kernel + wide quantizer, 0 one workgroup per row
    bool quant_four_launches = false;  // VTL_HIP_QUANT_FOUR_LAUNCHES: whole-tensor quantize as clear + absmax + scale + quantize (tests)
    bool no_fused_decode = false;   // VTL_HIP_NO_FUSED_DECODE: quantizer launch in front of the linear
    int stage_spin = 4096;          // VTL_HIP_STAGE_SPIN: polls a workgroup of the decode launch waits for the quantized rows (0: none, tests)
    int stream_weights_mib = 48;    // VTL_HIP_STREAM_WEIGHTS_MIB: weight matrices of this many MiB and more are read with non-temporal loads by the kernels for 2 to 32 rows (0: always)
    int skinny_tiled = -1;          // VTL_HIP_SKINNY_TILED: 1 / 0 force the 32x32-block weight-streaming kernel for M > 32
    int skinny_waves = 4;           // VTL_HIP_SKINNY_WAVES: 2, 4 or 8 waves (K ranges) per workgroup there
    int matmul_tile = 0;            // VTL_HIP_MATMUL_TILE: 128 / 64 force the f64-accumulating tile
    int matmul_splits = -1;         // VTL_HIP_MATMUL_SPLITS: K ranges of the f64-accumulating matmul
};
const Tuning &tuning();

constexpr int kWave = 64;

}  // namespace vtlhip

#define VTL_HIP_TRY(expr)                                                  \
    do {                                                                   \
        hipError_t vtl_e_ = (expr);                                        \
        if (vtl_e_ != hipSuccess)                                          \
            return ::vtlhip::record_hip_error(vtl_e_, #expr);              \
    } while (0)
