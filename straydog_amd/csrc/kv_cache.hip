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

}  // extern "C"
