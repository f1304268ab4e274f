// Entry points for harnesses, none of them on the attention path: seeded device-side fills for synthetic workloads, a plain
// copy and read-only streaming probes (the measured memory ceilings a benchmark reports beside the roofline), a matrix-core
// probe (the measured dense FP16 ceiling).
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <hip/hip_fp16.h>

using namespace sd;

namespace sd { void validate_pool(Device& d, const sdx_kv_pool* pool); }

namespace {

// Seeded normal values from the generator family the reference's tests use: one xorshift64 stream (x ^= x << 13; x ^= x >> 7;
// x ^= x << 17, e.g. crates/straydog-engine/tests/fused_gpu.rs:39-53), two draws a Box-Muller pair as in
// gpu/tests/qsa_interval_test.cpp:12-18, value i of the stream at out[i].  The same family, not the same values: here a uniform is
// ((x >> 11) + 0.5) / 2^53 and both the cosine and the sine of a pair are kept, where that test seeds with seed * 0x9E3779B97F4A7C15
// + 12345, draws (next() >> 16) % 1000003 and keeps the cosine only, and fused_gpu.rs draws uniforms (x >> 40) / 2^24 - 0.5; a
// workload filled here reproduces no fixture of the reference.  The stream is sequential; the generator is linear over GF(2), so a
// thread reaches its own stretch of RUN pairs by jumping: jump[b] holds the matrix of 2 * RUN * 2^b steps as 64 columns, and the
// bits of the thread's number say which to apply.
constexpr int RUN = 64;                       // pairs a thread draws
__constant__ uint64_t jump[32][64];

__host__ __device__ inline uint64_t xorshift64(uint64_t x) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; return x; }

// The state of the stream 2 * RUN * stretch steps after `seed`.
__device__ __forceinline__ uint64_t jumped(uint64_t seed, size_t stretch) {
    uint64_t state = seed;
    for (int b = 0; b < 32 && stretch >> b; ++b) {
        if (!((stretch >> b) & 1)) continue;
        uint64_t moved = 0;
        #pragma unroll 8
        for (int j = 0; j < 64; ++j) moved ^= (0 - ((state >> j) & 1)) & jump[b][j];
        state = moved;
    }
    return state;
}

__global__ void __launch_bounds__(256) fill_normal_kernel(void* out, size_t count, uint64_t seed, int kind) {
    const size_t thread = size_t(blockIdx.x) * blockDim.x + threadIdx.x, first = thread * (2 * RUN);
    if (first >= count) return;
    uint64_t state = jumped(seed, thread);
    const auto store = [&](size_t i, double x) {
        const float value = float(x);
        if (kind == 0) static_cast<float*>(out)[i] = value;
        else if (kind == 1) static_cast<__half*>(out)[i] = __float2half_rn(value);
        else {
            const uint32_t bits = __float_as_uint(value);
            static_cast<uint16_t*>(out)[i] = uint16_t((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
        }
    };
    for (size_t i = first; i < min(count, first + 2 * RUN); i += 2) {
        state = xorshift64(state);
        const double u = (double(state >> 11) + 0.5) / 9007199254740992.0;
        state = xorshift64(state);
        const double v = (double(state >> 11) + 0.5) / 9007199254740992.0;
        const double r = sqrt(-2.0 * log(u));
        store(i, r * cos(6.283185307179586 * v));
        if (i + 1 < count) store(i + 1, r * sin(6.283185307179586 * v));
    }
}

// The jump matrices, worked out and uploaded once a device, when its handle is made (a first fill may be recorded into a graph,
// where a synchronous upload would fail): a matrix is its 64 columns (the images of the unit vectors).
void fill_normal_setup(Device& d) {
    static std::mutex mutex;
    static std::map<int, bool> ready;
    std::lock_guard<std::mutex> lock(mutex);
    if (ready[d.ordinal]) return;
    typedef std::vector<uint64_t> Matrix;
    const auto apply = [](const Matrix& m, uint64_t x) { uint64_t y = 0; for (int j = 0; j < 64; ++j) if ((x >> j) & 1) y ^= m[j]; return y; };
    const auto squared = [&](const Matrix& m) { Matrix r(64); for (int j = 0; j < 64; ++j) r[j] = apply(m, m[j]); return r; };
    Matrix m(64);
    for (int j = 0; j < 64; ++j) m[j] = xorshift64(uint64_t(1) << j);
    for (int steps = 1; steps < 2 * RUN; steps *= 2) m = squared(m);        // 2 * RUN steps: one thread's stretch
    std::vector<uint64_t> all;
    for (int b = 0; b < 32; ++b) { all.insert(all.end(), m.begin(), m.end()); m = squared(m); }
    SD_CHECK(hipMemcpyToSymbol(HIP_SYMBOL(jump), all.data(), all.size() * sizeof(uint64_t)));
    ready[d.ordinal] = true;
}

// Uniform values of the same stream, one draw each: lo + (hi - lo) * (x >> 40) / 2^24.
__global__ void __launch_bounds__(256) fill_uniform_kernel(float* out, size_t count, uint64_t seed, float lo, float hi) {
    const size_t thread = size_t(blockIdx.x) * blockDim.x + threadIdx.x, first = thread * (2 * RUN);
    if (first >= count) return;
    uint64_t state = jumped(seed, thread);
    for (size_t i = first; i < min(count, first + 2 * RUN); ++i) {
        state = xorshift64(state);
        out[i] = __fadd_rn(lo, __fmul_rn(hi - lo, float(double(state >> 40) / 16777216.0)));    // (two roundings, as the host's)
    }
}

// Plain streaming copy, 16 bytes a lane: the measured HBM ceiling and the calibration of byte counters.
__global__ void __launch_bounds__(256) copy_kernel(uint4* target, const uint4* source, size_t count) {
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x)
        target[i] = source[i];
}

// Read-only streaming probe: every lane reads UNROLL x 16 bytes per trip, block-contiguous, and folds them into one word
// that is stored only if it is a value that cannot occur (keeps the loads alive).  The measured read ceiling of the box.
typedef uint32_t probe_u4 __attribute__((ext_vector_type(4)));
template<int UNROLL>
__global__ void __launch_bounds__(256) read_probe_kernel(const probe_u4* __restrict__ source, size_t count, uint32_t* sink) {
    uint32_t fold = 0;
    const size_t stride = size_t(gridDim.x) * 256 * UNROLL;
    for (size_t base = size_t(blockIdx.x) * 256 * UNROLL + threadIdx.x; base < count; base += stride) {
        probe_u4 v[UNROLL];
        #pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = base + size_t(u) * 256 < count ? __builtin_nontemporal_load(source + base + size_t(u) * 256) : probe_u4{0, 0, 0, 0};
        #pragma unroll
        for (int u = 0; u < UNROLL; ++u) fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (fold == 0x9e3779b9u && sink) *sink = fold;
}

// The decode kernel's way through a pool, loads only: a workgroup of four waves takes one K/V head of a run of pages; on each
// page its waves take alternate steps of 32 tokens, a step's K slab and V slab (32 rows of a plane each, contiguous) copied by
// 1 KiB global->LDS loads into the wave's one stage, one word of the stage read back, then the next step.  What the pool's
// layout and this order of asking are worth by themselves, with no arithmetic and no operand reads beside them.
__global__ void __launch_bounds__(256) paged_stream_probe_kernel(const uint8_t* __restrict__ pages, unsigned page_count, unsigned page_tokens, unsigned kv_heads,
                                                                 unsigned row_bytes, unsigned pages_per_group, uint32_t* sink) {
    extern __shared__ __attribute__((aligned(16))) uint8_t probe_stage[];
    typedef __attribute__((address_space(3))) uint8_t* lds_bytes;
    const unsigned lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned kvh = blockIdx.x % kv_heads, first_page = (blockIdx.x / kv_heads) * pages_per_group;
    const unsigned slab = 32 * row_bytes, pieces = (slab + 1023) / 1024, steps_per_page = page_tokens / 32;
    const size_t plane = size_t(page_tokens) * row_bytes;
    const uint32_t mine = __builtin_amdgcn_readfirstlane(uint32_t(uintptr_t((lds_bytes)probe_stage))) + wave * 2 * slab;     // (a slab is whole 16-byte pieces)
    uint32_t fold = 0;
    for (unsigned page = first_page; page < min(first_page + pages_per_group, page_count); ++page)
        for (unsigned step = wave; step < steps_per_page; step += 4) {
            const uint8_t* k = pages + (size_t(page) * 2 * kv_heads + kvh) * plane + size_t(step) * slab + 16 * lane;
            for (unsigned part = 0; part < 2; ++part) {
                const uint8_t* from = k + (part ? size_t(kv_heads) * plane : 0);
                for (unsigned j = 0; j < pieces; ++j)
                    if (16 * lane + 1024 * j < slab) {
                        const uint32_t to = mine + part * slab + j * 1024;
                        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" :: "v"(from + 1024 * j), "s"(to) : "memory");
                    }
            }
            uint32_t word;
            asm volatile("s_waitcnt vmcnt(0)\n\tds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(word) : "v"(mine + lane * 4) : "memory");
            fold ^= word;
        }
    if (fold == 0x9e3779b9u && sink) *sink = fold;
}

// Matrix-core probe: every wave keeps eight independent chains of v_mfma_f32_16x16x32_f16 going on operands it holds in
// registers, two waves a SIMD, nothing else in the loop: the dense FP16 ceiling of the box at the clock it holds under
// that load.  The clock depends on the operands: with LIVE ones (pseudo-random values, another pair of registers for every
// product, as a kernel working on real data presents them) the matrix cores draw more and the shader clock settles well
// below what it holds for the tame constants of the other variant.
typedef _Float16 probe_half8 __attribute__((ext_vector_type(8)));
typedef float probe_float4 __attribute__((ext_vector_type(4)));
__device__ unsigned probe_mix(unsigned x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }
template<bool LIVE>
__global__ void __launch_bounds__(512) mfma_probe_kernel(unsigned trips, float* sink) {
    probe_half8 a[4], b[4];
    #pragma unroll
    for (int k = 0; k < 4; ++k)
        #pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (LIVE) {
                const unsigned h = probe_mix(threadIdx.x * 64 + k * 8 + i + blockIdx.x * 7919);
                a[k][i] = (_Float16)((float(h & 0xffff) / 65536.0f - 0.5f) * 4.0f);
                b[k][i] = (_Float16)((float(h >> 16) / 65536.0f - 0.5f) * 4.0f);
            } else { a[k][i] = (_Float16)(float(threadIdx.x % 7) * 0.125f); b[k][i] = (_Float16)(float(threadIdx.x % 5) * 0.25f); }
        }
    probe_float4 c[8];
    #pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = probe_float4{0.0f, 0.0f, 0.0f, 0.0f};
    for (unsigned trip = 0; trip < trips; ++trip) {
        #pragma unroll
        for (int i = 0; i < 32; ++i) c[i % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i % 4], b[(i / 4) % 4], c[i % 8], 0, 0, 0);
    }
    float fold = 0.0f;
    #pragma unroll
    for (int i = 0; i < 8; ++i) fold += c[i][0] + c[i][1] + c[i][2] + c[i][3];
    if (fold == -1.0f && sink) *sink = fold;       // never in practice; keeps the products
}

}  // namespace

namespace sd {
// Called once a device by sd_create: nothing is left to upload at a first fill, which may then be recorded into a graph.
void harness_setup(Device& d) { fill_normal_setup(d); }
}  // namespace sd

extern "C" {

int sdx_fill_normal(void* handle, void* out, uint64_t count, uint64_t seed, int out_kind) {
    SD_OP_BEGIN
    if (!count || out_kind < 0 || out_kind > 2) throw std::runtime_error("invalid Straydog fill");
    op_span(value, out, checked_product({count, out_kind == 0 ? 4u : 2u}), "a filled buffer");
    if (count > (uint64_t(1) << 38)) throw std::runtime_error("invalid Straydog fill");
    fill_normal_kernel<<<checked_blocks((size_t(count) + 2 * RUN - 1) / (2 * RUN)), 256, 0, value.stream>>>(out, size_t(count),
                                                                                                      seed ? seed : 0x9e3779b97f4a7c15ull, out_kind);
    SD_OP_END
}

int sdx_fill_uniform(void* handle, float* out, uint64_t count, uint64_t seed, float lo, float hi) {
    SD_OP_BEGIN
    if (!count) throw std::runtime_error("invalid Straydog fill");
    op_span(value, out, checked_floats({count}), "a filled buffer");
    if (count > (uint64_t(1) << 38)) throw std::runtime_error("invalid Straydog fill");
    fill_uniform_kernel<<<checked_blocks((size_t(count) + 2 * RUN - 1) / (2 * RUN)), 256, 0, value.stream>>>(out, size_t(count),
                                                                                                       seed ? seed : 0x9e3779b97f4a7c15ull, lo, hi);
    SD_OP_END
}

int sdx_read_probe(void* handle, const void* source, uint64_t bytes, uint32_t blocks_per_cu, uint32_t unroll) {
    SD_OP_BEGIN
    if (!bytes || bytes % 16 || !blocks_per_cu || blocks_per_cu > 64) throw std::runtime_error("invalid Straydog read probe");
    op_span(value, source, size_t(bytes), "a probe's source");
    const unsigned grid = value.compute_units * blocks_per_cu;
    uint32_t* sink = static_cast<uint32_t*>(workspace(value, 256));
    if (unroll >= 8) read_probe_kernel<8><<<grid, 256, 0, value.stream>>>(static_cast<const probe_u4*>(source), size_t(bytes / 16), sink);
    else if (unroll >= 4) read_probe_kernel<4><<<grid, 256, 0, value.stream>>>(static_cast<const probe_u4*>(source), size_t(bytes / 16), sink);
    else read_probe_kernel<2><<<grid, 256, 0, value.stream>>>(static_cast<const probe_u4*>(source), size_t(bytes / 16), sink);
    SD_OP_END
}

int sdx_paged_stream_probe(void* handle, const sdx_kv_pool* pool, uint64_t* bytes) {
    SD_OP_BEGIN
    validate_pool(value, pool);
    if (pool->page_count > (uint64_t(1) << 31)) throw std::runtime_error("invalid Straydog read probe");
    // as many workgroups as the decode kernel keeps resident (four a compute unit), each a K/V head of a run of pages
    const unsigned groups = std::max(1u, value.compute_units * 4 / pool->kv_heads);
    const unsigned pages_per_group = unsigned((pool->page_count + groups - 1) / groups);
    const unsigned grid = unsigned((pool->page_count + pages_per_group - 1) / pages_per_group) * pool->kv_heads;
    const size_t shared = size_t(4) * 2 * 32 * pool->row_bytes;
    uint32_t* sink = static_cast<uint32_t*>(workspace(value, 256));
    if (shared > 64 * 1024) raise_shared_limit(value, reinterpret_cast<const void*>(&paged_stream_probe_kernel), shared);
    paged_stream_probe_kernel<<<grid, 256, shared, value.stream>>>(static_cast<const uint8_t*>(pool->pages), unsigned(pool->page_count), pool->page_tokens, pool->kv_heads,
                                                                 pool->row_bytes, pages_per_group, sink);
    SD_CHECK(hipGetLastError());
    if (bytes) *bytes = pool->page_count * 2 * pool->kv_heads * pool->page_tokens * pool->row_bytes;
    SD_OP_END
}

int sdx_mfma_probe(void* handle, uint32_t trips, int live, double* flops) {
    SD_OP_BEGIN
    if (!trips || trips > (1u << 24)) throw std::runtime_error("invalid Straydog matrix probe");
    float* sink = static_cast<float*>(workspace(value, 256));
    const unsigned groups = value.compute_units;        // one workgroup of eight waves per compute unit
    if (live) mfma_probe_kernel<true><<<groups, 512, 0, value.stream>>>(trips, sink);
    else mfma_probe_kernel<false><<<groups, 512, 0, value.stream>>>(trips, sink);
    if (flops) *flops = double(groups) * 8 * double(trips) * 32 * (2.0 * 16 * 16 * 32);
    SD_OP_END
}

int sdx_copy(void* handle, void* target, const void* source, uint64_t bytes) {
    SD_OP_BEGIN
    if (!bytes || bytes % 16) throw std::runtime_error("invalid Straydog copy");
    op_span(value, target, size_t(bytes), "a copy's target");
    op_span(value, source, size_t(bytes), "a copy's source");
    kv_settle(value);
    copy_kernel<<<value.compute_units * 16, 256, 0, value.stream>>>(static_cast<uint4*>(target), static_cast<const uint4*>(source), size_t(bytes / 16));
    SD_OP_END
}

}  // extern "C"
