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
};

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
        return cache.release();
    } catch (const std::exception& e) { last_error = e.what(); return nullptr; }
}

int sdx_kv_cache_destroy(void* handle, void* cache) {
    SD_OP_BEGIN
    KvCache& c = cache_of(value, cache);
    release(value, c.table);
    release(value, c.pool.pages);
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

}  // extern "C"
