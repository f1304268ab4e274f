// The device behind an opaque handle: one HIP device, one compute stream, a VRAM budget, and the table of
// its allocations that every op checks its pointers against.  Mirrors the conventions of the reference's
// Device (gpu/core.hpp:649-979, check/SD_OP_BEGIN/END :426-435, op_span gpu/ops.hpp:4-26, checked sizes
// gpu/core.hpp:1415-1429) for the attention entry points only.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>
#include <utility>
#include <vector>

namespace sd {

// Every allocation carries this many spare bytes so an unaligned wide load at its end stays inside it
// (reference gpu/core.hpp:209-211).
constexpr size_t allocation_tail = 64;
// Page-locked staging for uploads and downloads (reference gpu/core.hpp:405: 32 MiB per device).
constexpr size_t io_arena_bytes = size_t(32) << 20;

extern thread_local std::string last_error;

inline const char* gpu_error_text(hipError_t error) {
    const char* text = hipGetErrorString(error);
    return text && *text ? text : "GPU error";
}

inline void check_at(hipError_t error, const char* file, int line) {
    if (error == hipSuccess) return;
    const std::string path(file);
    throw std::runtime_error(std::string(gpu_error_text(error)) + " (" + path.substr(path.find_last_of("/\\") + 1) + ":" +
                             std::to_string(line) + ", code " + std::to_string(int(error)) + ")");
}
#define SD_CHECK(error) ::sd::check_at((error), __FILE__, __LINE__)

struct Device {
    int ordinal = 0;
    hipStream_t stream = nullptr;
    size_t budget = 0, used = 0;
    std::map<const uint8_t*, size_t> allocations;   // base -> requested bytes
    std::mutex mutex;
    uint8_t* arena = nullptr;                       // page-locked staging, io_arena_bytes
    uint32_t kv_row = 272;                          // sd_kv_format: 272 (Q8_0) or 512 (FP16)
    unsigned compute_units = 0;
    // Query rows a wave of the prompt kernel holds at 128 columns: 64 (one wave a SIMD) or 32 (two); sdx_prefill_wave_rows.
    uint32_t prefill_wave_rows = 64;
    // Workspaces the attention ops own (allocated on first use, outside any graph capture).
    void* sequence_input = nullptr; size_t sequence_input_bytes = 0;
    void* sequence_output = nullptr; size_t sequence_output_bytes = 0;
    void* workspace = nullptr; size_t workspace_bytes = 0;
    // The attention rope table of a pass (sd_attention_turns_reserve / _arm): forward[row][pair] = (cosine, sine), then the
    // inverse turns at the same stride.  Armed for `turns_armed` rows, the next sd_op_norm_rope of that many rows fills it;
    // ready, the next sd_op_sparse_attention of those rows reads it instead of forming the angles again.
    double2* turns = nullptr;
    size_t turns_rows = 0, turns_pairs = 0, turns_armed = 0, turns_ready_rows = 0, turns_ready_pairs = 0;
    bool turns_ready = false;
    // Dynamic LDS limits raised so far, by kernel: the attribute belongs to this device's copy of the kernel, so each
    // handle raises it for itself (raise_shared_limit).
    std::map<const void*, size_t> shared_limits;
    // This device's address of the partial-result area the library itself holds for sdx_paged_attention_static.
    float* paged_static = nullptr;
    // The matrix-core indexer's radix histograms (index_topk.hip): all zero between calls.
    uint32_t* index_bins = nullptr; size_t index_bins_rows = 0; bool index_bins_dirty = false;
    // The lists of a short span's thinned index rows (block_index.hip), allocated at the first such call and kept.
    void* select_thin = nullptr;
    // Sequence state in mapped, page-locked host memory (sd_host_state): device pointer -> host pointer.  They are listed in
    // `allocations` too, so ops take them, but not counted in the VRAM budget.
    std::map<const void*, void*> host_states;
    // Host states page-locked and zeroed ahead of their use on a thread of their own (sd_host_states_prefetch): (bytes, host pointer).
    std::thread host_prefetch;
    std::vector<std::pair<size_t, void*>> host_ready;
    std::string host_prefetch_error;
    // The VRAM stage the host registered (sd_kv_stage) and whose rows it holds: a K/V cache, one of its sequences, and how many
    // of that sequence's pages from the first on are in it.
    void* kv_stage = nullptr; size_t kv_stage_bytes = 0;
    const void* kv_stage_owner = nullptr; size_t kv_stage_sequence = 0, kv_stage_pages = 0;
    // K/V pages move between HBM and host memory on a stream of their own (same priority), behind `kv_released` of the
    // compute stream; `kv_moved` marks the last move queued, and the compute stream waits for it before the next work
    // that touches pages (kv_settle).
    hipStream_t kv_stream = nullptr;
    hipEvent_t kv_released = nullptr, kv_moved = nullptr;
    bool kv_moving = false;
    // Page-locked host copies of sequence state (conversation checkpoints): pointer -> bytes.
    std::map<void*, size_t> checkpoints;
    // Recorded graphs of ops (sd_graph_begin / _end / _run), by the caller's key.
    struct Recorded { hipGraph_t graph = nullptr; hipGraphExec_t executable = nullptr; };
    std::map<uint64_t, Recorded> graphs;
    bool recording = false;
    std::vector<hipEvent_t> events;
    // Optional kernel timing for harnesses (sdx_profile): an event pair per launch of the op's main kernel (timed_launch).
    bool profile = false;
    std::vector<hipEvent_t> profile_events;
};

// Launches one kernel on the device's stream.  With the device's profiling on it goes through the extended launch, whose
// two events take the kernel's own start and end times (what a tracer reads), not the times of event packets around it.
template<typename... Params, typename... Args>
void timed_launch(Device& d, void (*kernel)(Params...), dim3 grid, dim3 block, size_t shared, Args... args) {
    hipEvent_t start = nullptr, stop = nullptr;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    const bool timed = d.profile && hipStreamIsCapturing(d.stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusNone;
    if (timed && (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess)) {
        if (start) (void)hipEventDestroy(start);
        start = stop = nullptr;
    }
    if (!start) { kernel<<<grid, block, shared, d.stream>>>(Params(args)...); return; }
    hipExtLaunchKernelGGL(kernel, grid, block, uint32_t(shared), d.stream, start, stop, 0, Params(args)...);
    d.profile_events.push_back(start);
    d.profile_events.push_back(stop);
}

// A kernel that asks for more dynamic LDS than the default limit has the limit raised first, once per handle and size.
inline void raise_shared_limit(Device& d, const void* kernel, size_t bytes) {
    size_t& have = d.shared_limits[kernel];
    if (bytes <= have) return;
    if (bytes > 160 * 1024) throw std::runtime_error("Straydog op: a kernel asks for more LDS than a compute unit has");
    const hipError_t error = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
    if (error != hipSuccess) throw std::runtime_error(std::string("Straydog op: ") + gpu_error_text(error));
    have = bytes;
}

// Work on the compute stream that reads or writes K/V pages comes after the page moves queued so far.  (A recording takes no
// wait on an event from outside it: sd_graph_begin settles first, and no move is queued while a graph is recorded.)
inline void kv_settle(Device& d) {
    if (!d.kv_moving) return;
    SD_CHECK(hipStreamWaitEvent(d.stream, d.kv_moved, 0));
    d.kv_moving = false;
}

Device& device(void* handle);                         // sets the HIP device of the handle; throws on null
void* allocate(Device& d, size_t bytes, bool zero);   // budget-checked hipMalloc (+ tail)
void release(Device& d, void* pointer);
void upload(Device& d, void* target, const void* data, size_t bytes);     // caller memory -> device, in stream order
void download(Device& d, void* output, const void* source, size_t bytes);  // device -> caller memory, waits
// A workspace of at least `bytes` that lives with the device; grows only outside graph capture.
void* workspace(Device& d, size_t bytes);
// Recorded graphs hold the addresses of the library's own buffers: when one of them moves, the graphs recorded so far go.
void drop_recorded_graphs(Device& d);

// [pointer, pointer + bytes) must lie inside one live allocation of this device.
void op_span(Device& d, const void* pointer, size_t bytes, const char* what);
// The same for a pointer that may carry the BF16 tag in bit 0: `count` values of 2 or 4 bytes.
void op_state_span(Device& d, const void* pointer, size_t count, const char* what);

inline bool state_bf16(const void* p) { return reinterpret_cast<uintptr_t>(p) & 1u; }
inline const void* state_base(const void* p) { return reinterpret_cast<const void*>(reinterpret_cast<uintptr_t>(p) & ~uintptr_t(1)); }

inline size_t checked_product(std::initializer_list<uint64_t> factors) {
    uint64_t total = 1;
    for (const uint64_t f : factors) {
        if (f && total > UINT64_MAX / f) throw std::runtime_error("Straydog op: a size overflows");
        total *= f;
    }
    if (total > (uint64_t(1) << 48)) throw std::runtime_error("Straydog op: a size overflows");
    return size_t(total);
}
inline size_t checked_floats(std::initializer_list<uint64_t> factors) { return checked_product({uint64_t(checked_product(factors)), 4}); }
inline unsigned checked_blocks(size_t count, unsigned threads = 256) {
    const size_t blocks = (count + threads - 1) / threads;
    if (!blocks || blocks > 0x7fffffffu) throw std::runtime_error("Straydog op: a launch is out of range");
    return unsigned(blocks);
}

}  // namespace sd

// The body of an extern "C" op: the device the handle names, failures as the thread's error text.
#define SD_OP_BEGIN try { ::sd::Device& value = ::sd::device(handle);
#define SD_OP_END SD_CHECK(hipGetLastError()); return 0; } catch (const std::exception& e) { ::sd::last_error = e.what(); return -1; }
