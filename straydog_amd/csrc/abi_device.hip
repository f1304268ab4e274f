// Devices, allocations and transfers of the C ABI (reference gpu/kernels.cpp:3511-3614 sd_create, :4555-4592 sd_buffer*,
// gpu/host_io.hpp:81-180 upload/download/allocate), for one MI355X per handle.
#include "device.hpp"

#include "../../include/straydog_gpu.h"
#include "../../include/straydog_gpu_ext.h"

#include <algorithm>
#include <cstring>

namespace sd {

thread_local std::string last_error;
void paged_attention_setup(Device& d);   // paged_attention.hip
void harness_setup(Device& d);           // harness.hip
void select_thin_reserve(Device& d);     // block_index.hip

// Recorded graphs hold the addresses their ops were given.  When a buffer the library owns moves (the workspace grows), the
// graphs recorded so far would replay on freed memory: they are dropped, sd_graph_run then answers 1 ("none stored under
// this key") and the caller records again -- what the reference does when its K/V views change (kv_clear_graphs,
// gpu/kv_stage.hpp:96-104).
void drop_recorded_graphs(Device& d) {
    for (auto& entry : d.graphs) {
        if (entry.second.executable) (void)hipGraphExecDestroy(entry.second.executable);
        if (entry.second.graph) (void)hipGraphDestroy(entry.second.graph);
    }
    d.graphs.clear();
}

Device& device(void* handle) {
    if (!handle) throw std::runtime_error("Straydog device handle is null");
    Device& d = *static_cast<Device*>(handle);
    SD_CHECK(hipSetDevice(d.ordinal));
    return d;
}

static std::string budget_exceeded(const Device& d, size_t bytes) {
    const size_t left = d.budget > d.used ? d.budget - d.used : 0;
    return "Straydog VRAM budget exceeded (" + std::to_string(bytes >> 20) + " MiB asked, " + std::to_string(left >> 20) + " MiB of " +
           std::to_string(d.budget >> 20) + " MiB left)";
}

void* allocate(Device& d, size_t bytes, bool zero) {
    const size_t available = d.budget > d.used ? d.budget - d.used : 0;
    if (!bytes || bytes > available || allocation_tail > available - bytes) throw std::runtime_error(budget_exceeded(d, bytes));
    void* pointer = nullptr;
    SD_CHECK(hipMalloc(&pointer, bytes + allocation_tail));
    {
        std::lock_guard<std::mutex> lock(d.mutex);
        d.allocations.emplace(static_cast<const uint8_t*>(pointer), bytes);
        d.used += bytes + allocation_tail;
    }
    if (zero) SD_CHECK(hipMemsetAsync(pointer, 0, bytes + allocation_tail, d.stream));
    else SD_CHECK(hipMemsetAsync(static_cast<uint8_t*>(pointer) + bytes, 0, allocation_tail, d.stream));
    return pointer;
}

void release(Device& d, void* pointer) {
    size_t bytes = 0;
    void* host = nullptr;
    {
        std::lock_guard<std::mutex> lock(d.mutex);
        const auto found = d.allocations.find(static_cast<const uint8_t*>(pointer));
        if (found == d.allocations.end()) throw std::runtime_error("Straydog release: not an allocation of this device");
        bytes = found->second;
        d.allocations.erase(found);
        const auto state = d.host_states.find(pointer);
        if (state != d.host_states.end()) { host = state->second; d.host_states.erase(state); }
        else d.used -= bytes + allocation_tail;
    }
    SD_CHECK(hipStreamSynchronize(d.stream));
    if (d.kv_stream) SD_CHECK(hipStreamSynchronize(d.kv_stream));
    if (pointer == d.kv_stage) {
        // (the stage's address is in recorded graphs that attend from it)
        drop_recorded_graphs(d);
        d.kv_stage = nullptr; d.kv_stage_bytes = 0; d.kv_stage_owner = nullptr; d.kv_stage_pages = 0;
    }
    if (host) SD_CHECK(hipHostFree(host));
    else SD_CHECK(hipFree(pointer));
}

// Caller memory goes through the page-locked arena a half at a time, so the caller's buffer is free on return and
// the bytes land in stream order; a half is reused only after the copy that read it has finished.
void upload(Device& d, void* target, const void* data, size_t bytes) {
    const size_t half = io_arena_bytes / 2;
    const uint8_t* from = static_cast<const uint8_t*>(data);
    uint8_t* to = static_cast<uint8_t*>(target);
    kv_settle(d);       // (the target may be pages a queued move still reads or writes)
    static thread_local int turn = 0;
    while (bytes) {
        const size_t part = std::min(bytes, half);
        uint8_t* slot = d.arena + (turn & 1) * half;
        hipEvent_t done = d.events[turn & 1];
        SD_CHECK(hipEventSynchronize(done));
        std::memcpy(slot, from, part);
        SD_CHECK(hipMemcpyAsync(to, slot, part, hipMemcpyHostToDevice, d.stream));
        SD_CHECK(hipEventRecord(done, d.stream));
        from += part; to += part; bytes -= part; ++turn;
    }
}

void download(Device& d, void* output, const void* source, size_t bytes) {
    uint8_t* to = static_cast<uint8_t*>(output);
    const uint8_t* from = static_cast<const uint8_t*>(source);
    // the bytes may be pages still on their way from host memory on the page stream
    kv_settle(d);
    // both halves may hold an upload in flight: wait for the stream once, then the arena is ours
    SD_CHECK(hipStreamSynchronize(d.stream));
    while (bytes) {
        const size_t part = std::min(bytes, io_arena_bytes);
        SD_CHECK(hipMemcpyAsync(d.arena, from, part, hipMemcpyDeviceToHost, d.stream));
        SD_CHECK(hipStreamSynchronize(d.stream));
        std::memcpy(to, d.arena, part);
        from += part; to += part; bytes -= part;
    }
}

void* workspace(Device& d, size_t bytes) {
    if (bytes <= d.workspace_bytes) return d.workspace;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    SD_CHECK(hipStreamIsCapturing(d.stream, &capturing));
    if (capturing != hipStreamCaptureStatusNone) throw std::runtime_error("Straydog attention workspace cannot grow while a graph is recorded");
    if (d.workspace) {
        drop_recorded_graphs(d);
        release(d, d.workspace);
    }
    d.workspace = nullptr; d.workspace_bytes = 0;
    const size_t rounded = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    d.workspace = allocate(d, rounded, true);
    d.workspace_bytes = rounded;
    return d.workspace;
}

void op_span(Device& d, const void* pointer, size_t bytes, const char* what) {
    const uint8_t* at = static_cast<const uint8_t*>(pointer);
    std::lock_guard<std::mutex> lock(d.mutex);
    auto next = d.allocations.upper_bound(at);
    if (at && next != d.allocations.begin()) {
        --next;
        const uint8_t* base = next->first;
        if (bytes <= next->second && size_t(at - base) <= next->second - bytes) return;
    }
    throw std::runtime_error(std::string("Straydog op: ") + what + " is outside this device's allocations");
}

void op_state_span(Device& d, const void* pointer, size_t count, const char* what) {
    op_span(d, state_base(pointer), checked_product({uint64_t(count), state_bf16(pointer) ? 2u : 4u}), what);
}

}  // namespace sd

using namespace sd;

extern "C" {

const char* sd_error(void) { return last_error.c_str(); }

int sd_device_count(void) {
    int count = 0;
    const hipError_t error = hipGetDeviceCount(&count);
    if (error != hipSuccess) { last_error = gpu_error_text(error); (void)hipGetLastError(); return error == hipErrorNoDevice ? 0 : -1; }
    return count;
}

int sd_device_info(int ordinal, char* name, size_t capacity, uint64_t* free_bytes, uint64_t* total_bytes) {
    try {
        hipDeviceProp_t properties;
        SD_CHECK(hipGetDeviceProperties(&properties, ordinal));
        if (name && capacity) { std::strncpy(name, properties.name, capacity - 1); name[capacity - 1] = '\0'; }
        SD_CHECK(hipSetDevice(ordinal));
        size_t free_now = 0, total = 0;
        SD_CHECK(hipMemGetInfo(&free_now, &total));
        if (free_bytes) *free_bytes = free_now;
        if (total_bytes) *total_bytes = total;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

void* sd_create(int ordinal, uint64_t budget) {
    Device* d = nullptr;
    try {
        int count = 0;
        SD_CHECK(hipGetDeviceCount(&count));
        if (ordinal < 0 || ordinal >= count) throw std::runtime_error("Straydog device ordinal out of range");
        SD_CHECK(hipSetDevice(ordinal));
        hipDeviceProp_t properties;
        SD_CHECK(hipGetDeviceProperties(&properties, ordinal));
        if (std::string(properties.gcnArchName).rfind("gfx950", 0) != 0)
            throw std::runtime_error(std::string("this Straydog attention library is built for gfx950 (MI355X) only; device is ") + properties.gcnArchName);
        d = new Device;
        d->ordinal = ordinal;
        d->budget = size_t(budget);
        d->compute_units = unsigned(properties.multiProcessorCount);
        SD_CHECK(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking));
        SD_CHECK(hipHostMalloc(reinterpret_cast<void**>(&d->arena), io_arena_bytes, hipHostMallocDefault));
        d->events.resize(2);
        for (auto& event : d->events) { SD_CHECK(hipEventCreateWithFlags(&event, hipEventDisableTiming)); SD_CHECK(hipEventRecord(event, d->stream)); }
        paged_attention_setup(*d);
        harness_setup(*d);
        return d;
    } catch (const std::exception& e) {
        last_error = e.what();
        if (d) sd_destroy(d);
        return nullptr;
    }
}

void sd_destroy(void* handle) {
    if (!handle) return;
    Device* d = static_cast<Device*>(handle);
    (void)hipSetDevice(d->ordinal);
    if (d->stream) (void)hipStreamSynchronize(d->stream);
    for (auto& entry : d->graphs) {
        if (entry.second.executable) (void)hipGraphExecDestroy(entry.second.executable);
        if (entry.second.graph) (void)hipGraphDestroy(entry.second.graph);
    }
    if (d->kv_stream) (void)hipStreamSynchronize(d->kv_stream);
    if (d->host_prefetch.joinable()) d->host_prefetch.join();
    for (const auto& held : d->host_ready) (void)hipHostFree(held.second);
    for (const auto& entry : d->host_states) { d->allocations.erase(static_cast<const uint8_t*>(entry.first)); (void)hipHostFree(entry.second); }
    for (const auto& entry : d->allocations) (void)hipFree(const_cast<uint8_t*>(entry.first));
    if (d->kv_released) (void)hipEventDestroy(d->kv_released);
    if (d->kv_moved) (void)hipEventDestroy(d->kv_moved);
    if (d->kv_stream) (void)hipStreamDestroy(d->kv_stream);
    for (auto& event : d->events) if (event) (void)hipEventDestroy(event);
    for (auto& event : d->profile_events) (void)hipEventDestroy(event);
    for (const auto& entry : d->checkpoints) (void)hipHostFree(entry.first);
    if (d->arena) (void)hipHostFree(d->arena);
    if (d->stream) (void)hipStreamDestroy(d->stream);
    delete d;
}

int sd_memory(void* handle, uint64_t* used, uint64_t* budget) {
    try {
        Device& d = device(handle);
        if (used) *used = d.used;
        if (budget) *budget = d.budget;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

void* sd_upload(void* handle, const void* data, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!data) throw std::runtime_error("invalid Straydog upload");
        void* pointer = allocate(d, size_t(bytes), false);
        upload(d, pointer, data, size_t(bytes));
        return pointer;
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

void* sd_allocate(void* handle, uint64_t bytes) {
    try { return allocate(device(handle), size_t(bytes), false); }
    catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sd_write(void* handle, void* pointer, const void* data, uint64_t bytes) {
    try {
        Device& d = device(handle);
        std::unique_lock<std::mutex> lock(d.mutex);
        const auto found = d.allocations.find(static_cast<const uint8_t*>(pointer));
        if (!data || found == d.allocations.end() || found->second != bytes) throw std::runtime_error("invalid Straydog write");
        lock.unlock();
        upload(d, pointer, data, size_t(bytes));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_release(void* handle, void* pointer) {
    try { release(device(handle), pointer); return 0; }
    catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_allocation_bytes(void* handle, const void* pointer, uint64_t* bytes) {
    try {
        Device& d = device(handle);
        std::lock_guard<std::mutex> lock(d.mutex);
        const auto found = d.allocations.find(static_cast<const uint8_t*>(pointer));
        if (found == d.allocations.end() || !bytes) throw std::runtime_error("Straydog: not an allocation of this device");
        *bytes = found->second + allocation_tail;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_zero(void* handle, void* pointer) {
    try {
        Device& d = device(handle);
        size_t bytes = 0;
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            const auto found = d.allocations.find(static_cast<const uint8_t*>(pointer));
            if (found == d.allocations.end()) throw std::runtime_error("Straydog zero: not an allocation of this device");
            bytes = found->second;
        }
        SD_CHECK(hipMemsetAsync(pointer, 0, bytes, d.stream));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_download(void* handle, void* pointer, void* output, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!output) throw std::runtime_error("invalid Straydog download");
        op_span(d, pointer, size_t(bytes), "a downloaded allocation");
        download(d, output, pointer, size_t(bytes));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

void* sd_buffer(void* handle, uint64_t bytes) {
    try {
        Device& d = device(handle);
        void* pointer = allocate(d, size_t(bytes), true);
        // Return only after the zeros land (reference gpu/kernels.cpp:4566-4568).
        SD_CHECK(hipStreamSynchronize(d.stream));
        return pointer;
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sd_buffer_write(void* handle, void* buffer, uint64_t offset, const void* data, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!data || offset > UINT64_MAX - bytes) throw std::runtime_error("invalid Straydog buffer write");
        op_span(d, static_cast<uint8_t*>(buffer) + offset, size_t(bytes), "a written buffer");
        upload(d, static_cast<uint8_t*>(buffer) + offset, data, size_t(bytes));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_buffer_read(void* handle, const void* buffer, uint64_t offset, void* output, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!output || offset > UINT64_MAX - bytes) throw std::runtime_error("invalid Straydog buffer read");
        op_span(d, static_cast<const uint8_t*>(buffer) + offset, size_t(bytes), "a read buffer");
        download(d, output, static_cast<const uint8_t*>(buffer) + offset, size_t(bytes));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

// Conversation checkpoints (reference gpu/kernels.cpp:3905-3915 sd_checkpoint_buffer, :3962-3990 sd_checkpoint_copy, :3951-3961
// sd_checkpoint_clone, :3996-4041 sd_state_copy): sequence state -- K/V pools, page tables, the block indexer's pooled blocks --
// saved to and restored from page-locked host memory.  With the rows resident in HBM a checkpoint is the only time they cross
// PCIe; whole allocations go as one copy each, a part of a state (a sequence's positions within a plane, one run per plane)
// as one strided copy.
void* sd_checkpoint_buffer(void* handle, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!bytes) throw std::runtime_error("invalid Straydog checkpoint buffer");
        void* host = nullptr;
        SD_CHECK(hipHostMalloc(&host, size_t(bytes), hipHostMallocDefault));
        try {
            std::lock_guard<std::mutex> lock(d.mutex);
            d.checkpoints.emplace(host, size_t(bytes));
        } catch (...) { (void)hipHostFree(host); throw; }
        return host;
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sdx_checkpoint_release(void* handle, void* buffer) {
    try {
        Device& d = device(handle);
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            if (!d.checkpoints.erase(buffer)) throw std::runtime_error("Straydog: not a checkpoint buffer of this device");
        }
        SD_CHECK(hipStreamSynchronize(d.stream));
        SD_CHECK(hipHostFree(buffer));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_checkpoint_copy(void* handle, int save, void* const* states, uint64_t count, void* buffer) {
    try {
        Device& d = device(handle);
        std::vector<size_t> sizes;
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            const auto found = d.checkpoints.find(buffer);
            if (found == d.checkpoints.end() || !states || !count || count > 4096) throw std::runtime_error("invalid Straydog checkpoint copy");
            size_t total = 0;
            for (uint64_t i = 0; i < count; ++i) {
                const auto state = d.allocations.find(static_cast<const uint8_t*>(states[i]));
                if (state == d.allocations.end() || state->second > found->second - total) throw std::runtime_error("invalid Straydog checkpoint state");
                sizes.push_back(state->second);
                total += state->second;
            }
        }
        auto* host = static_cast<uint8_t*>(buffer);
        kv_settle(d);
        for (uint64_t i = 0; i < count; ++i) {
            if (save) SD_CHECK(hipMemcpyAsync(host, states[i], sizes[i], hipMemcpyDeviceToHost, d.stream));
            else SD_CHECK(hipMemcpyAsync(states[i], host, sizes[i], hipMemcpyHostToDevice, d.stream));
            host += sizes[i];
        }
        SD_CHECK(hipStreamSynchronize(d.stream));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_checkpoint_clone(void* handle, void* from, void* to) {
    try {
        Device& d = device(handle);
        size_t bytes = 0;
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            const auto source = d.checkpoints.find(from), target = d.checkpoints.find(to);
            if (source == d.checkpoints.end() || target == d.checkpoints.end() || source->second != target->second || from == to)
                throw std::runtime_error("invalid Straydog checkpoint clone");
            bytes = source->second;
        }
        SD_CHECK(hipStreamSynchronize(d.stream));       // the copies into `from` among what the stream still had
        std::memcpy(to, from, bytes);
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_state_copy(void* handle, void* state, uint64_t offset, uint64_t pitch, uint64_t width, uint64_t height, float* host, uint64_t first, int save) {
    try {
        Device& d = device(handle);
        (void)first;        // (the reference truncates its VRAM mirrors of a host-resident K/V there; here the state is the only copy)
        size_t floats = 0;
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            const auto found = d.allocations.find(static_cast<const uint8_t*>(state));
            if (found == d.allocations.end() || !host || !width || !height || pitch < width) throw std::runtime_error("invalid Straydog state copy");
            floats = found->second / 4;
        }
        if (offset > floats || height - 1 > (floats - offset) / pitch || width > floats - offset - (height - 1) * pitch)
            throw std::runtime_error("Straydog state copy outside its state");
        float* base = static_cast<float*>(state) + offset;
        kv_settle(d);
        if (save) SD_CHECK(hipMemcpy2DAsync(host, width * 4, base, pitch * 4, width * 4, height, hipMemcpyDeviceToHost, d.stream));
        else SD_CHECK(hipMemcpy2DAsync(base, pitch * 4, host, width * 4, width * 4, height, hipMemcpyHostToDevice, d.stream));
        SD_CHECK(hipStreamSynchronize(d.stream));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_kv_format(void* handle, uint32_t row) {
    try {
        Device& d = device(handle);
        if (row != 512 && row != 272) throw std::runtime_error("invalid Straydog K/V format");
        d.kv_row = row;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

// Sequence state in mapped, page-locked host memory that kernels read and write over the bus (reference gpu/kernels.cpp:3876-3903
// sd_host_state, :4292-4300 sd_host_state_supported): owned like a device allocation -- ops take pointers into it, sd_release
// frees it -- but outside the VRAM budget.  A K/V pool may live there whole; the paged cache's host tier (kv_cache.hip) is the
// faster way to hold rows that are not being attended to.
// Page-locks and zeroes host states of these sizes on a thread of their own (reference gpu/kernels.cpp:3824-3847): sd_host_state then
// takes one of the right size, in any order, once the thread is done.
int sd_host_states_prefetch(void* handle, const uint64_t* sizes, uint64_t count) {
    try {
        Device& d = device(handle);
        if (!sizes || count > 4096 || d.host_prefetch.joinable() || !d.host_ready.empty()) throw std::runtime_error("invalid Straydog host state prefetch");
        std::vector<size_t> wanted(sizes, sizes + count);
        for (const size_t bytes : wanted) if (!bytes || bytes > (size_t(1) << 48)) throw std::runtime_error("invalid Straydog host state prefetch");
        const int ordinal = d.ordinal;
        d.host_prefetch_error.clear();
        d.host_prefetch = std::thread([&d, wanted, ordinal]() {
            try {
                SD_CHECK(hipSetDevice(ordinal));
                for (const size_t bytes : wanted) {
                    void* host = nullptr;
                    SD_CHECK(hipHostMalloc(&host, bytes + allocation_tail, hipHostMallocMapped));
                    d.host_ready.emplace_back(bytes, host);
                    std::memset(host, 0, bytes + allocation_tail);
                }
            } catch (const std::exception& e) { d.host_prefetch_error = e.what(); }
        });
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

void* sd_host_state(void* handle, uint64_t bytes) {
    try {
        Device& d = device(handle);
        if (!bytes || bytes > (uint64_t(1) << 48)) throw std::runtime_error("invalid Straydog host state");
        if (d.host_prefetch.joinable()) d.host_prefetch.join();
        if (!d.host_prefetch_error.empty()) {
            const std::string error = d.host_prefetch_error;
            d.host_prefetch_error.clear();
            throw std::runtime_error(error);
        }
        void* host = nullptr;
        const auto ready = std::find_if(d.host_ready.begin(), d.host_ready.end(), [&](const auto& held) { return held.first == size_t(bytes); });
        const bool zeroed = ready != d.host_ready.end();            // (the prefetch zeroed it)
        if (zeroed) { host = ready->second; d.host_ready.erase(ready); }
        else SD_CHECK(hipHostMalloc(&host, size_t(bytes) + allocation_tail, hipHostMallocMapped));
        try {
            if (!zeroed) std::memset(host, 0, size_t(bytes) + allocation_tail);
            void* pointer = nullptr;
            SD_CHECK(hipHostGetDevicePointer(&pointer, host, 0));
            std::lock_guard<std::mutex> lock(d.mutex);
            d.allocations.emplace(static_cast<const uint8_t*>(pointer), size_t(bytes));
            try { d.host_states.emplace(pointer, host); }
            catch (...) { d.allocations.erase(static_cast<const uint8_t*>(pointer)); throw; }
            return pointer;
        } catch (...) { (void)hipHostFree(host); throw; }
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sd_host_state_supported(void* handle) {
    try { (void)device(handle); return 1; }
    catch (const std::exception& e) { last_error = e.what(); return -1; }
}

// The VRAM stage (reference gpu/kernels.cpp:4277-4290): an allocation of the caller's, `rows` x 4096 bytes, that rows held in host
// memory are copied into to be attended from.  Registering it forgets what a former stage held and the graphs recorded so far.
int sd_kv_stage(void* handle, void* pointer, uint64_t rows) {
    try {
        Device& d = device(handle);
        {
            std::lock_guard<std::mutex> lock(d.mutex);
            const auto found = d.allocations.find(static_cast<const uint8_t*>(pointer));
            if (!rows || rows > (uint64_t(1) << 22) || found == d.allocations.end() || found->second != size_t(rows) * 1024 * 4 ||
                d.host_states.count(pointer))
                throw std::runtime_error("invalid Straydog K/V stage");
        }
        if (d.recording) throw std::runtime_error("invalid Straydog K/V stage");
        if (d.kv_stream) SD_CHECK(hipStreamSynchronize(d.kv_stream));
        d.kv_moving = false;
        drop_recorded_graphs(d);
        d.kv_stage = pointer; d.kv_stage_bytes = size_t(rows) * 1024 * 4;
        d.kv_stage_owner = nullptr; d.kv_stage_pages = 0;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

// ---- graphs of ops (reference gpu/kernels.cpp:4765-4813) ----
// Between begin and end the ops queued on the device's stream are recorded rather than run.  Only ops that take no host data and
// allocate nothing may be recorded; the ops that keep a workspace (see the extension header) are called once before.

int sd_graph_begin(void* handle) {
    try {
        Device& d = device(handle);
        if (d.recording) throw std::runtime_error("a Straydog graph is already being recorded");
        // (made here, not by the op that uses it: a capture takes no allocation; reference gpu/kernels.cpp:4769-4773)
        try { select_thin_reserve(d); } catch (const std::exception&) {}
        kv_settle(d);
        SD_CHECK(hipStreamBeginCapture(d.stream, hipStreamCaptureModeThreadLocal));
        d.recording = true;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_graph_end(void* handle, uint64_t key, int keep) {
    try {
        Device& d = device(handle);
        if (!d.recording) throw std::runtime_error("no Straydog graph is being recorded");
        d.recording = false;
        Device::Recorded made;
        SD_CHECK(hipStreamEndCapture(d.stream, &made.graph));
        if (!keep) {
            (void)hipGraphDestroy(made.graph);
            return 0;
        }
        const hipError_t instantiated = hipGraphInstantiate(&made.executable, made.graph, nullptr, nullptr, 0);
        if (instantiated != hipSuccess) {
            (void)hipGraphDestroy(made.graph);
            SD_CHECK(instantiated);
        }
        Device::Recorded& slot = d.graphs[key];
        if (slot.executable) (void)hipGraphExecDestroy(slot.executable);
        if (slot.graph) (void)hipGraphDestroy(slot.graph);
        slot = made;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sd_graph_run(void* handle, uint64_t key) {
    try {
        Device& d = device(handle);
        const auto found = d.graphs.find(key);
        if (found == d.graphs.end()) return 1;
        // page moves queued since the recording (a resume, a stage) come first: the graph's ops read the pages they fill
        kv_settle(d);
        SD_CHECK(hipGraphLaunch(found->second.executable, d.stream));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

// ---- extensions: stream waits and event timing for harnesses ----

int sdx_synchronize(void* handle) {
    try { Device& d = device(handle); SD_CHECK(hipStreamSynchronize(d.stream)); return 0; }
    catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int64_t sdx_event_record(void* handle) {
    try {
        Device& d = device(handle);
        hipEvent_t event;
        SD_CHECK(hipEventCreate(&event));
        SD_CHECK(hipEventRecord(event, d.stream));
        d.events.push_back(event);
        return int64_t(d.events.size() - 1);
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_event_elapsed(void* handle, int64_t begin, int64_t end, float* milliseconds) {
    try {
        Device& d = device(handle);
        if (begin < 2 || end < 2 || size_t(begin) >= d.events.size() || size_t(end) >= d.events.size() || !milliseconds)
            throw std::runtime_error("invalid Straydog event");
        SD_CHECK(hipEventSynchronize(d.events[size_t(end)]));
        SD_CHECK(hipEventElapsedTime(milliseconds, d.events[size_t(begin)], d.events[size_t(end)]));
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_events_clear(void* handle) {
    try {
        Device& d = device(handle);
        SD_CHECK(hipStreamSynchronize(d.stream));
        while (d.events.size() > 2) { SD_CHECK(hipEventDestroy(d.events.back())); d.events.pop_back(); }
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_profile(void* handle, int enable) {
    try {
        Device& d = device(handle);
        SD_CHECK(hipStreamSynchronize(d.stream));
        for (auto& event : d.profile_events) (void)hipEventDestroy(event);
        d.profile_events.clear();
        d.profile = enable != 0;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_profile_read(void* handle, double* milliseconds, uint64_t* launches) {
    try {
        Device& d = device(handle);
        SD_CHECK(hipStreamSynchronize(d.stream));
        double total = 0.0;
        for (size_t i = 0; i + 1 < d.profile_events.size(); i += 2) {
            float ms = 0.0f;
            SD_CHECK(hipEventElapsedTime(&ms, d.profile_events[i], d.profile_events[i + 1]));
            total += ms;
        }
        if (milliseconds) *milliseconds = total;
        if (launches) *launches = d.profile_events.size() / 2;
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_device_state(void* handle, uint64_t* values) {
    try {
        Device& d = device(handle);
        if (!values) throw std::runtime_error("invalid Straydog device query");
        size_t free_bytes = 0, total_bytes = 0;
        SD_CHECK(hipMemGetInfo(&free_bytes, &total_bytes));
        values[0] = free_bytes; values[1] = total_bytes; values[2] = d.workspace_bytes; values[3] = d.profile_events.size();
        return 0;
    } catch (const std::exception& e) { last_error = e.what(); return -1; }
}

int sdx_device_compute_units(void* handle) {
    try { return int(device(handle).compute_units); }
    catch (const std::exception& e) { last_error = e.what(); return -1; }
}

}  // extern "C"
