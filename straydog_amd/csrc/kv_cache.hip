// Where K/V rows live: a pool of pages in HBM and the sequences' page tables, kept by the library.
//
// The reference keeps a sequence's K/V in host memory and stages what attention needs into VRAM -- a mirror ring of the
// newest rows for decode, a layer's prefix for prefill, the union of the selected rows (gpu/kv_stage.hpp:1-184), and
// sd_kv_grow copies a whole state when a context outgrows it (gpu/straydog_gpu.h:105-109) -- because its cards hold 16-32 GB.
// With 288 GB of HBM the rows stay on the device, and what remains of that subsystem is bookkeeping: which pages a
// sequence owns.  Pages make growth free of copies (sd_kv_grow's job is `reserve`), a prompt prefix shared by several
// sequences is shared pages with a reference count (`fork` copies only the last, partial page), and a rejected
// speculation gives its pages back (`truncate`).  The page tables live in device memory in the layout the attention
// entry points take ([sequence][table_stride] int32); every change is uploaded in stream order, so attention queued after
// a call sees it, and nothing here waits for the device.
//
// Rows that are not in HBM.  A cache may be given a second tier of pages in page-locked host memory that the library
// allocates (`host`).  A sequence nobody is decoding is parked there (`park`: its pages leave on the move stream while the
// compute stream goes on with other sequences, and its HBM pages are free at once for others) and brought back before its
// next step (`resume`: the copies run on the move stream behind what the compute stream had queued, and the compute stream
// waits for them only at its next call that touches pages -- the reference's prefetch between two attention layers,
// gpu/kv_stage.hpp:62-85, kv_stage_settle :52-56).  A parked sequence can also be attended to where it is: `stage` copies
// its pages into the VRAM stage the host registered with sd_kv_stage (only the pages the stage does not already hold of
// it, gpu/kv_stage.hpp:146-149) and yields a pool / page-table view over the stage; rows appended through that view go
// back to the host pages with `unstage` (kv_after_prefill, gpu/kv_stage.hpp:151-155).  `grow` is sd_kv_grow's VRAM
// branch for a pool (gpu/kernels.cpp:4048-4140): a larger allocation, the pages copied on the device, the old one
// released, recorded graphs dropped.
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <algorithm>
#include <memory>

using namespace sd;

namespace sd {
void validate_pool(Device& d, const sdx_kv_pool* pool);
}

namespace {

struct KvCache {
    Device* device;
    sdx_kv_pool pool;
    int32_t* table;                       // device: [sequences][stride]
    size_t sequences, stride;
    std::vector<int32_t> pages_of;        // host copy of the table
    std::vector<uint32_t> held;           // pages a sequence holds
    std::vector<uint32_t> references;     // sequences that hold a page
    std::vector<int32_t> free_pages;      // a stack; the lowest page numbers are handed out first
    // The host tier: pages of the same layout in page-locked memory; a parked sequence's `pages_of` entries name these.
    uint8_t* host = nullptr;
    size_t host_pages = 0;
    std::vector<int32_t> free_host;
    std::vector<uint8_t> parked;
    int32_t* stage_table = nullptr;       // device: 0, 1, 2 ... stride-1, the page table of a staged sequence
};

size_t page_bytes(const KvCache& c) { return 2 * size_t(c.pool.kv_heads) * c.pool.page_tokens * c.pool.row_bytes; }

void check_resident(const KvCache& c, uint64_t sequence) {
    if (c.parked[sequence]) throw std::runtime_error("Straydog K/V cache: the sequence is parked in host memory");
}

// The move stream's next copies come after everything the compute stream holds now (the last readers and writers of the
// pages involved); made at the first move.
void begin_move(Device& d) {
    if (d.recording) throw std::runtime_error("Straydog K/V cache: pages cannot move while a graph is recorded");
    if (!d.kv_stream) {
        SD_CHECK(hipStreamCreateWithFlags(&d.kv_stream, hipStreamNonBlocking));
        SD_CHECK(hipEventCreateWithFlags(&d.kv_released, hipEventDisableTiming));
        SD_CHECK(hipEventCreateWithFlags(&d.kv_moved, hipEventDisableTiming));
    }
    SD_CHECK(hipEventRecord(d.kv_released, d.stream));
    SD_CHECK(hipStreamWaitEvent(d.kv_stream, d.kv_released, 0));
}

void end_move(Device& d) {
    SD_CHECK(hipEventRecord(d.kv_moved, d.kv_stream));
    d.kv_moving = true;
}

void forget_stage(Device& d, const KvCache& c, uint64_t sequence) {
    if (d.kv_stage_owner == &c && d.kv_stage_sequence == sequence) { d.kv_stage_owner = nullptr; d.kv_stage_pages = 0; }
}

KvCache& cache_of(Device& d, void* cache) {
    auto* c = static_cast<KvCache*>(cache);
    if (!c || c->device != &d) throw std::runtime_error("Straydog K/V cache: not a cache of this device");
    return *c;
}

size_t pages_for(const KvCache& c, uint64_t tokens) { return size_t((tokens + c.pool.page_tokens - 1) / c.pool.page_tokens); }

void check_sequence(const KvCache& c, uint64_t sequence) {
    if (sequence >= c.sequences) throw std::runtime_error("Straydog K/V cache: no such sequence");
}

int32_t take_page(KvCache& c) {
    const int32_t page = c.free_pages.back();
    c.free_pages.pop_back();
    c.references[size_t(page)] = 1;
    return page;
}

void drop_page(KvCache& c, int32_t page) {
    if (--c.references[size_t(page)] == 0) c.free_pages.push_back(page);
}

void upload_entries(KvCache& c, size_t sequence, size_t first, size_t count) {
    if (count) upload(*c.device, c.table + sequence * c.stride + first, c.pages_of.data() + sequence * c.stride + first, count * sizeof(int32_t));
}

// The first `rows` rows of every plane of page `source` into page `copy`, in stream order.
void copy_rows(KvCache& c, Device& d, int32_t source, int32_t copy, size_t rows) {
    const size_t plane = size_t(c.pool.page_tokens) * c.pool.row_bytes, planes = 2 * size_t(c.pool.kv_heads);
    auto* base = static_cast<uint8_t*>(c.pool.pages);
    for (size_t p = 0; p < planes; ++p)
        SD_CHECK(hipMemcpyAsync(base + (size_t(copy) * planes + p) * plane, base + (size_t(source) * planes + p) * plane, rows * c.pool.row_bytes,
                                hipMemcpyDeviceToDevice, d.stream));
}


// ---- the union gather (reference gpu/sparse_attention_compute.hpp:677-733) ------------------------------------------------
// Rows of a sequence whose pages are not in HBM would be read over the bus entry by entry, by every query row that names them.
// Instead the blocks of four rows that the rows' selections name are copied once, in block order, into the VRAM stage, and each
// selection is renumbered to the places there: a row reads the same keys and values in the same order, from HBM.

// marks[block] = 1 for every block of four positions that an entry which counts names (the rule of the selection-list attention:
// entry j < min(selected, counts[row]) counts iff 0 <= raw <= base + row and raw < context).  A workgroup a row.
__global__ void __launch_bounds__(256) union_mark_kernel(const float* indices, const float* counts, size_t selected, size_t first, size_t base, size_t context,
                                                         uint32_t* marks) {
    const size_t row = first + blockIdx.x;
    const float* list = indices + row * selected;
    const float stated = counts[row];
    const size_t count = stated > 0.0f ? min(selected, size_t(stated)) : 0;
    const float limit = float(base + row);
    for (size_t j = threadIdx.x; j < count; j += 256) {
        const float raw = list[j];
        if (raw >= 0.0f && raw <= limit && raw < float(context)) marks[size_t(raw) / 4] = 1u;
    }
}

// The union's places, in two launches of a workgroup per 1024 blocks: first each stretch's count of marked blocks, then
// marks[block] becomes the number of marked blocks before it, blocks[place] the block in that place, marks[end] the union's size.
__global__ void __launch_bounds__(1024) union_count_kernel(const uint32_t* marks, size_t end, uint32_t* stretch_counts) {
    __shared__ uint32_t wave_sums[16];
    const size_t block = size_t(blockIdx.x) * 1024 + threadIdx.x;
    const bool marked = block < end && marks[block] != 0;
    const uint64_t votes = __ballot(marked);
    if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = uint32_t(__popcll(votes));
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t total = 0;
        #pragma unroll
        for (int w = 0; w < 16; ++w) total += wave_sums[w];
        stretch_counts[blockIdx.x] = total;
    }
}
__global__ void __launch_bounds__(1024) union_place_kernel(uint32_t* marks, size_t end, const uint32_t* stretch_counts, uint32_t* blocks) {
    __shared__ uint32_t wave_sums[16];
    __shared__ uint32_t before_stretch;
    const unsigned lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t block = size_t(blockIdx.x) * 1024 + threadIdx.x;
    const bool marked = block < end && marks[block] != 0;
    const uint64_t votes = __ballot(marked);
    if (lane == 0) wave_sums[wave] = uint32_t(__popcll(votes));
    if (wave == 15) {
        // the stretches before this one, added up by one wave
        uint32_t sum = 0;
        for (unsigned i = lane; i < blockIdx.x; i += 64) sum += stretch_counts[i];
        #pragma unroll
        for (unsigned offset = 32; offset; offset >>= 1) sum += __shfl_xor(sum, offset);
        if (lane == 0) before_stretch = sum;
    }
    __syncthreads();
    uint32_t at = before_stretch + uint32_t(__popcll(votes & ((uint64_t(1) << lane) - 1)));
    #pragma unroll
    for (unsigned w = 0; w < 16; ++w) if (w < wave) at += wave_sums[w];
    if (block < end) {
        marks[block] = at;
        if (marked) blocks[at] = uint32_t(block);
    }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 1023) marks[end] = at + (marked ? 1u : 0u);
}

// Place p's four rows of every plane, from the sequence's pages (in HBM, or in the cache's host tier: over the bus) into
// positions 4p .. 4p + 3 of the stage, which has the pool's page layout.  A workgroup a place, 16 bytes a thread at a time (four
// rows of a plane follow one another and start on a 16-byte boundary: a block never straddles a page).
__global__ void __launch_bounds__(256) union_gather_kernel(const uint8_t* source, const int32_t* table, unsigned page_last, unsigned page_tokens, unsigned planes,
                                                           unsigned row_bytes, const uint32_t* blocks, uint8_t* stage) {
    const size_t place = blockIdx.x, block = blocks[place];
    const size_t pieces = size_t(4) * row_bytes / 16, plane_bytes = size_t(page_tokens) * row_bytes;
    const size_t from_token = block * 4, to_token = place * 4;
    const unsigned entry = unsigned(table[from_token / page_tokens]);
    const uint8_t* from = source + size_t(min(entry, page_last)) * planes * plane_bytes + (from_token % page_tokens) * row_bytes;
    uint8_t* to = stage + (to_token / page_tokens) * planes * plane_bytes + (to_token % page_tokens) * row_bytes;
    for (size_t i = threadIdx.x; i < planes * pieces; i += 256) {
        const size_t plane = i / pieces, piece = i % pieces;
        reinterpret_cast<uint4*>(to + plane * plane_bytes)[piece] = reinterpret_cast<const uint4*>(from + plane * plane_bytes)[piece];
    }
}

// The rows' lists renumbered to the union's places; an entry that does not count becomes -1 (which never counts).
__global__ void __launch_bounds__(256) union_renumber_kernel(const float* indices, const float* counts, size_t selected, size_t first, size_t base, size_t context,
                                                             const uint32_t* places, float* renumbered) {
    const size_t row = first + blockIdx.x;
    const float* list = indices + row * selected;
    float* out = renumbered + row * selected;
    const float stated = counts[row];
    const size_t count = stated > 0.0f ? min(selected, size_t(stated)) : 0;
    const float limit = float(base + row);
    for (size_t j = threadIdx.x; j < selected; j += 256) {
        const float raw = list[j];
        const bool counted = j < count && raw >= 0.0f && raw <= limit && raw < float(context);
        out[j] = counted ? float(size_t(places[size_t(raw) / 4]) * 4 + size_t(raw) % 4) : -1.0f;
    }
}

__global__ void __launch_bounds__(256) union_clear_kernel(uint32_t* words, size_t count) {
    const size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < count) words[i] = 0u;
}

}  // namespace

extern "C" {

void* sdx_kv_cache_create(void* handle, uint64_t pages, uint32_t page_tokens, uint32_t kv_heads, uint32_t dim, uint32_t row_bytes,
                          uint64_t sequences, uint64_t max_context) {
    try {
        Device& d = device(handle);
        if (!pages || pages > 0x7fffffffu || !sequences || sequences > 65535 || !max_context || !page_tokens)
            throw std::runtime_error("Straydog K/V cache: pages, sequences and max_context >= 1");
        auto cache = std::make_unique<KvCache>();
        cache->device = &d;
        cache->sequences = size_t(sequences);
        cache->stride = size_t((max_context + page_tokens - 1) / page_tokens);
        const size_t bytes = checked_product({pages, 2, kv_heads, page_tokens, row_bytes});
        cache->pool = sdx_kv_pool{nullptr, pages, page_tokens, kv_heads, dim, row_bytes};
        cache->pool.pages = allocate(d, bytes, true);
        try {
            validate_pool(d, &cache->pool);
            cache->table = static_cast<int32_t*>(allocate(d, checked_floats({sequences, uint64_t(cache->stride)}), true));
        } catch (...) {
            release(d, cache->pool.pages);
            throw;
        }
        cache->pages_of.assign(cache->sequences * cache->stride, 0);
        cache->held.assign(cache->sequences, 0);
        cache->references.assign(size_t(pages), 0);
        cache->free_pages.resize(size_t(pages));
        for (size_t i = 0; i < size_t(pages); ++i) cache->free_pages[i] = int32_t(pages - 1 - i);
        cache->parked.assign(cache->sequences, 0);
        return cache.release();
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sdx_kv_cache_destroy(void* handle, void* cache) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    if (value.kv_stage_owner == &c) { value.kv_stage_owner = nullptr; value.kv_stage_pages = 0; }
    release(value, c.table);            // (waits for both streams)
    release(value, c.pool.pages);
    if (c.stage_table) release(value, c.stage_table);
    if (c.host) SD_CHECK(hipHostFree(c.host));
    delete &c;
    SD_OP_END
}

int sdx_kv_cache_view(void* handle, void* cache, sdx_kv_pool* pool, const int32_t** page_table, uint64_t* table_stride) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    if (pool) *pool = c.pool;
    if (page_table) *page_table = c.table;
    if (table_stride) *table_stride = c.stride;
    SD_OP_END
}

int sdx_kv_cache_reserve(void* handle, void* cache, uint64_t sequence, uint64_t tokens) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    check_resident(c, sequence);
    kv_settle(value);           // (a page handed out here may still be on its way to host memory)
    const size_t need = pages_for(c, tokens), have = c.held[sequence];
    if (need > c.stride) throw std::runtime_error("Straydog K/V cache: a sequence longer than the cache's max_context");
    if (need > have) {
        if (need - have > c.free_pages.size()) throw std::runtime_error("Straydog K/V cache: out of pages");
        for (size_t i = have; i < need; ++i) c.pages_of[sequence * c.stride + i] = take_page(c);
        c.held[sequence] = uint32_t(need);
        upload_entries(c, sequence, have, need - have);
    }
    SD_OP_END
}

int sdx_kv_cache_truncate(void* handle, void* cache, uint64_t sequence, uint64_t tokens) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    const size_t keep = pages_for(c, tokens), rest = size_t(tokens % c.pool.page_tokens);
    if (c.parked[sequence]) {
        // a parked sequence shares nothing: its pages past the kept rows go back to the host tier
        for (size_t i = c.held[sequence]; i > keep; --i) c.free_host.push_back(c.pages_of[sequence * c.stride + i - 1]);
        c.held[sequence] = uint32_t(std::min<size_t>(c.held[sequence], keep));
        if (value.kv_stage_owner == &c && value.kv_stage_sequence == sequence) value.kv_stage_pages = std::min(value.kv_stage_pages, keep);
        return 0;
    }
    kv_settle(value);
    // Rows appended after a rewind land in the last kept page from row `rest` on.  If another sequence shares that page (a fork's
    // whole pages are shared by reference count), those rows are still the sibling's: this sequence continues on a copy of the
    // rows it keeps.  Without a free page for the copy nothing is changed.
    const bool shared_tail = rest && keep <= c.held[sequence] && keep && c.references[size_t(c.pages_of[sequence * c.stride + keep - 1])] > 1;
    if (shared_tail && c.free_pages.empty()) throw std::runtime_error("Straydog K/V cache: out of pages");
    for (size_t i = c.held[sequence]; i > keep; --i) drop_page(c, c.pages_of[sequence * c.stride + i - 1]);
    c.held[sequence] = uint32_t(std::min<size_t>(c.held[sequence], keep));
    if (shared_tail) {
        const int32_t source = c.pages_of[sequence * c.stride + keep - 1], copy = take_page(c);
        copy_rows(c, value, source, copy, rest);
        drop_page(c, source);
        c.pages_of[sequence * c.stride + keep - 1] = copy;
        upload_entries(c, sequence, keep - 1, 1);
    }
    SD_OP_END
}

int sdx_kv_cache_fork(void* handle, void* cache, uint64_t from, uint64_t to, uint64_t tokens) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, from);
    check_sequence(c, to);
    check_resident(c, from);
    check_resident(c, to);
    kv_settle(value);
    const size_t whole = size_t(tokens / c.pool.page_tokens), rest = size_t(tokens % c.pool.page_tokens), need = whole + (rest ? 1 : 0);
    if (from == to || c.held[to] || need > c.held[from]) throw std::runtime_error("Straydog K/V cache: a fork needs an empty target and a source that holds the prefix");
    if (rest && c.free_pages.empty()) throw std::runtime_error("Straydog K/V cache: out of pages");
    for (size_t i = 0; i < whole; ++i) {
        const int32_t page = c.pages_of[from * c.stride + i];
        ++c.references[size_t(page)];
        c.pages_of[to * c.stride + i] = page;
    }
    if (rest) {
        // the prefix's last page is written on by both sequences from here on: the target gets its own copy of the rows so far
        const int32_t source = c.pages_of[from * c.stride + whole], copy = take_page(c);
        c.pages_of[to * c.stride + whole] = copy;
        copy_rows(c, value, source, copy, rest);
    }
    c.held[to] = uint32_t(need);
    upload_entries(c, to, 0, need);
    SD_OP_END
}

int sdx_kv_cache_usage(void* handle, void* cache, uint64_t sequence, uint64_t* pages_held, uint64_t* pages_free) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    if (pages_held) {
        check_sequence(c, sequence);
        *pages_held = c.held[sequence];
    }
    if (pages_free) *pages_free = c.free_pages.size();
    SD_OP_END
}

int sdx_kv_cache_host(void* handle, void* cache, uint64_t host_pages) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    if (c.host || !host_pages || host_pages > 0x7fffffffu) throw std::runtime_error("Straydog K/V cache: one host tier of >= 1 pages");
    const size_t bytes = checked_product({host_pages, uint64_t(page_bytes(c))});
    const hipError_t error = hipHostMalloc(reinterpret_cast<void**>(&c.host), bytes, hipHostMallocDefault);
    if (error != hipSuccess) {
        (void)hipGetLastError();
        c.host = nullptr;
        throw std::runtime_error("not enough host memory for the K/V of this sequence");
    }
    c.host_pages = size_t(host_pages);
    c.free_host.resize(c.host_pages);
    for (size_t i = 0; i < c.host_pages; ++i) c.free_host[i] = int32_t(c.host_pages - 1 - i);
    SD_OP_END
}

int sdx_kv_cache_park(void* handle, void* cache, uint64_t sequence) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    check_resident(c, sequence);
    const size_t held = c.held[sequence], bytes = page_bytes(c);
    if (!c.host) throw std::runtime_error("Straydog K/V cache: no host tier");
    if (held > c.free_host.size()) throw std::runtime_error("not enough host memory for the K/V of this sequence");
    begin_move(value);
    for (size_t i = 0; i < held; ++i) {
        int32_t& entry = c.pages_of[sequence * c.stride + i];
        const int32_t page = entry, kept = c.free_host.back();
        c.free_host.pop_back();
        SD_CHECK(hipMemcpyAsync(c.host + size_t(kept) * bytes, static_cast<uint8_t*>(c.pool.pages) + size_t(page) * bytes, bytes,
                                hipMemcpyDeviceToHost, value.kv_stream));
        drop_page(c, page);     // (a page shared with a fork stays with the sibling)
        entry = kept;
    }
    end_move(value);
    c.parked[sequence] = 1;
    SD_OP_END
}

int sdx_kv_cache_resume(void* handle, void* cache, uint64_t sequence) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    if (!c.parked[sequence]) throw std::runtime_error("Straydog K/V cache: the sequence is not parked");
    const size_t held = c.held[sequence], bytes = page_bytes(c);
    if (held > c.free_pages.size()) throw std::runtime_error("Straydog K/V cache: out of pages");
    begin_move(value);
    for (size_t i = 0; i < held; ++i) {
        int32_t& entry = c.pages_of[sequence * c.stride + i];
        const int32_t kept = entry, page = take_page(c);
        SD_CHECK(hipMemcpyAsync(static_cast<uint8_t*>(c.pool.pages) + size_t(page) * bytes, c.host + size_t(kept) * bytes, bytes,
                                hipMemcpyHostToDevice, value.kv_stream));
        c.free_host.push_back(kept);
        entry = page;
    }
    end_move(value);
    c.parked[sequence] = 0;
    forget_stage(value, c, sequence);
    upload_entries(c, sequence, 0, held);
    SD_OP_END
}

int sdx_kv_cache_stage(void* handle, void* cache, uint64_t sequence, uint64_t tokens, sdx_kv_pool* pool, const int32_t** page_table,
                       uint64_t* table_stride) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    if (!c.parked[sequence]) throw std::runtime_error("Straydog K/V cache: only a parked sequence is staged");
    const size_t bytes = page_bytes(c), room = value.kv_stage ? value.kv_stage_bytes / bytes : 0, need = pages_for(c, tokens);
    if (!room) throw std::runtime_error("Straydog K/V cache: no K/V stage is registered (sd_kv_stage)");
    if (need > c.held[sequence] || need > room) throw std::runtime_error("Straydog K/V cache: the stage or the sequence holds fewer rows");
    if (!c.stage_table) {
        std::vector<int32_t> places(c.stride);
        for (size_t i = 0; i < c.stride; ++i) places[i] = int32_t(i);
        c.stage_table = static_cast<int32_t*>(allocate(value, c.stride * sizeof(int32_t), false));
        upload(value, c.stage_table, places.data(), c.stride * sizeof(int32_t));
    }
    if (value.kv_stage_owner != &c || value.kv_stage_sequence != sequence) {
        value.kv_stage_owner = &c; value.kv_stage_sequence = size_t(sequence); value.kv_stage_pages = 0;
    }
    if (need > value.kv_stage_pages) {
        begin_move(value);
        for (size_t i = value.kv_stage_pages; i < need; ++i)
            SD_CHECK(hipMemcpyAsync(static_cast<uint8_t*>(value.kv_stage) + i * bytes, c.host + size_t(c.pages_of[sequence * c.stride + i]) * bytes,
                                    bytes, hipMemcpyHostToDevice, value.kv_stream));
        end_move(value);
        value.kv_stage_pages = need;
    }
    if (pool) *pool = sdx_kv_pool{value.kv_stage, room, c.pool.page_tokens, c.pool.kv_heads, c.pool.dim, c.pool.row_bytes};
    if (page_table) *page_table = c.stage_table;
    if (table_stride) *table_stride = c.stride;
    SD_OP_END
}

int sdx_kv_cache_unstage(void* handle, void* cache, uint64_t sequence, uint64_t first, uint64_t count) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    if (!c.parked[sequence] || value.kv_stage_owner != &c || value.kv_stage_sequence != sequence)
        throw std::runtime_error("Straydog K/V cache: the stage does not hold this sequence");
    const size_t bytes = page_bytes(c), room = value.kv_stage_bytes / bytes, tokens = c.pool.page_tokens, row = c.pool.row_bytes;
    const size_t need = pages_for(c, first + count), have = c.held[sequence];
    // the rows before `first` are the ones the stage was given: it holds every page up to the one `first` falls in
    if (!count || first > uint64_t(value.kv_stage_pages) * tokens || need > room || need > c.stride)
        throw std::runtime_error("Straydog K/V cache: rows outside the stage");
    if (need > have && need - have > c.free_host.size()) throw std::runtime_error("not enough host memory for the K/V of this sequence");
    for (size_t i = have; i < need; ++i) { c.pages_of[sequence * c.stride + i] = c.free_host.back(); c.free_host.pop_back(); }
    c.held[sequence] = uint32_t(std::max(have, need));
    kv_settle(value);
    // in stream order behind the writes: each page's run of rows, one line per plane
    for (size_t at = size_t(first), end = size_t(first + count); at < end;) {
        const size_t page = at / tokens, from = at % tokens, run = std::min(end - at, tokens - from);
        SD_CHECK(hipMemcpy2DAsync(c.host + size_t(c.pages_of[sequence * c.stride + page]) * bytes + from * row, tokens * row,
                                  static_cast<uint8_t*>(value.kv_stage) + page * bytes + from * row, tokens * row, run * row,
                                  2 * size_t(c.pool.kv_heads), hipMemcpyDeviceToHost, value.stream));
        at += run;
    }
    value.kv_stage_pages = std::max(value.kv_stage_pages, need);
    SD_OP_END
}

int sdx_kv_cache_grow(void* handle, void* cache, uint64_t pages) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    const size_t had = size_t(c.pool.page_count), bytes = page_bytes(c);
    if (pages <= had || pages > 0x7fffffffu || value.recording) throw std::runtime_error("invalid Straydog K/V growth");
    kv_settle(value);
    void* grown = nullptr;
    try { grown = allocate(value, checked_product({pages, uint64_t(bytes)}), false); }
    catch (const std::exception&) { throw std::runtime_error("not enough VRAM for the K/V of this sequence"); }
    SD_CHECK(hipMemcpyAsync(grown, c.pool.pages, had * bytes, hipMemcpyDeviceToDevice, value.stream));
    SD_CHECK(hipMemsetAsync(static_cast<uint8_t*>(grown) + had * bytes, 0, (size_t(pages) - had) * bytes, value.stream));
    drop_recorded_graphs(value);
    release(value, c.pool.pages);
    c.pool.pages = grown;
    c.pool.page_count = pages;
    c.references.resize(size_t(pages), 0);
    // (the stack hands out its back first: the new, higher pages go under the ones that were free)
    std::vector<int32_t> stack;
    for (size_t page = size_t(pages); page > had; --page) stack.push_back(int32_t(page - 1));
    stack.insert(stack.end(), c.free_pages.begin(), c.free_pages.end());
    c.free_pages.swap(stack);
    SD_OP_END
}

int sdx_kv_cache_residency(void* handle, void* cache, uint64_t sequence, uint64_t* parked, uint64_t* host_pages_free, uint64_t* staged_pages) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    if (parked) *parked = c.parked[sequence];
    if (host_pages_free) *host_pages_free = c.free_host.size();
    if (staged_pages) *staged_pages = value.kv_stage_owner == &c && value.kv_stage_sequence == sequence ? value.kv_stage_pages : 0;
    SD_OP_END
}

int sdx_kv_cache_gather(void* handle, void* cache, uint64_t sequence, uint64_t context, uint64_t base, const float* indices, uint64_t selected,
                        const float* counts, uint64_t first, uint64_t rows, float* renumbered, uint64_t* taken, uint64_t* union_rows, sdx_kv_pool* pool,
                        const int32_t** page_table, uint64_t* table_stride) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    check_sequence(c, sequence);
    if (value.recording) throw std::runtime_error("Straydog K/V cache: the union gather reads its size back and cannot be recorded");
    const size_t bytes = page_bytes(c), room = value.kv_stage ? value.kv_stage_bytes / bytes : 0, tokens = c.pool.page_tokens;
    if (!room) throw std::runtime_error("Straydog K/V cache: no K/V stage is registered (sd_kv_stage)");
    if (!rows || rows > 65535 || !selected || selected > (uint64_t(1) << 20) || !context || context > (uint64_t(1) << 24) || !taken || first > (uint64_t(1) << 24) ||
        base > (uint64_t(1) << 24) || base + first + rows > context)
        throw std::runtime_error("invalid Straydog union gather");
    if (pages_for(c, context) > c.held[sequence]) throw std::runtime_error("Straydog K/V cache: the sequence holds fewer rows");
    op_span(value, indices, checked_floats({first + rows, selected}), "selection lists");
    op_span(value, counts, checked_floats({first + rows}), "selection counts");
    op_span(value, renumbered, checked_floats({first + rows, selected}), "renumbered selection lists");
    if (!c.stage_table) {
        std::vector<int32_t> places(c.stride);
        for (size_t i = 0; i < c.stride; ++i) places[i] = int32_t(i);
        c.stage_table = static_cast<int32_t*>(allocate(value, c.stride * sizeof(int32_t), false));
        upload(value, c.stage_table, places.data(), c.stride * sizeof(int32_t));
    }
    // where the sequence's pages are: the host tier (the device's table row then names host pages) or the pool
    const bool parked = c.parked[sequence] != 0;
    const uint8_t* source = parked ? c.host : static_cast<const uint8_t*>(c.pool.pages);
    const unsigned page_last = unsigned((parked ? c.host_pages : size_t(c.pool.page_count)) - 1);
    if (parked) upload_entries(c, sequence, 0, c.held[sequence]);
    kv_settle(value);                   // (a parked sequence's rows may still be on their way to the host tier)
    forget_stage(value, c, sequence);
    value.kv_stage_owner = nullptr; value.kv_stage_pages = 0;         // what the stage held, a prefix of some sequence, is gone
    const size_t end = size_t((base + first + rows - 1) / 4 + 1), capacity = room * tokens;
    const unsigned stretches = checked_blocks(end, 1024);
    uint32_t* marks = static_cast<uint32_t*>(workspace(value, checked_floats({2 * uint64_t(end) + 2 + stretches})));
    uint32_t* blocks = marks + end + 1;
    uint32_t* stretch_counts = blocks + end;
    // as many of the rows as the stage holds the union of: halved until it fits (the union's size is read back each time)
    size_t count = size_t(rows);
    uint32_t total = 0;
    for (;;) {
        union_clear_kernel<<<checked_blocks(end + 1), 256, 0, value.stream>>>(marks, end + 1);
        union_mark_kernel<<<unsigned(count), 256, 0, value.stream>>>(indices, counts, size_t(selected), size_t(first), size_t(base), size_t(context), marks);
        union_count_kernel<<<stretches, 1024, 0, value.stream>>>(marks, end, stretch_counts);
        union_place_kernel<<<stretches, 1024, 0, value.stream>>>(marks, end, stretch_counts, blocks);
        SD_CHECK(hipGetLastError());
        SD_CHECK(hipMemcpyAsync(value.arena, marks + end, 4, hipMemcpyDeviceToHost, value.stream));
        SD_CHECK(hipStreamSynchronize(value.stream));
        std::memcpy(&total, value.arena, 4);
        if (size_t(total) * 4 <= capacity || count == 1) break;
        count = (count + 1) / 2;
    }
    if (size_t(total) * 4 > capacity) count = 0;        // (a stage too small for one row's selection: nothing is gathered)
    if (count) {
        if (total)
            union_gather_kernel<<<total, 256, 0, value.stream>>>(source, c.table + size_t(sequence) * c.stride, page_last, c.pool.page_tokens, 2 * c.pool.kv_heads,
                                                                c.pool.row_bytes, blocks, static_cast<uint8_t*>(value.kv_stage));
        union_renumber_kernel<<<unsigned(count), 256, 0, value.stream>>>(indices, counts, size_t(selected), size_t(first), size_t(base), size_t(context), marks, renumbered);
    }
    *taken = count;
    if (union_rows) *union_rows = count ? uint64_t(total) * 4 : 0;
    if (pool) *pool = sdx_kv_pool{value.kv_stage, room, c.pool.page_tokens, c.pool.kv_heads, c.pool.dim, c.pool.row_bytes};
    if (page_table) *page_table = c.stage_table;
    if (table_stride) *table_stride = c.stride;
    SD_OP_END
}

}  // extern "C"
