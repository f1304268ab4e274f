// Rows of the paged K/V cache as MFMA operands: the pieces shared by the decode kernel and the prefill kernel.
//
// Layouts (v_mfma_f32_16x16x32_f16 on gfx950, wave64): an A or B operand gives lane (l % 16, l / 16 = g) eight k-slots;
// a C tile gives lane column l % 16 and rows 4g..4g+3.  S^T = K . Q^T takes K rows as A operands (lane = token, eight
// consecutive columns per lane group), so the C layout (lane = query row, four tokens per lane group) is already the
// B-operand layout of O^T += V^T . P^T: probabilities never move between lanes.  A 32-token step is two such tiles; the
// eight k-slots of the second product are the lane's tokens {4g..4g+3, 16+4g..16+4g+3}.
#pragma once
#include "device.hpp"
#include "../../include/straydog_gpu_ext.h"

#include <hip/hip_fp16.h>

namespace sd { namespace paged {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;
typedef __attribute__((address_space(4))) const int32_t* table_ptr;   // read through the scalar cache: a page number is wave-uniform

constexpr int WAVES = 4, STEP = 32;
constexpr float NEG_BIG = -1.0e30f;   // a finite "nothing seen yet" maximum: exp2(NEG_BIG - m) is 0, no inf - inf anywhere

struct PagedArgs {
    const uint8_t* pages;
    unsigned page_tokens, kv_heads, heads, group, span;
    const int32_t* page_table;
    size_t table_stride;
    const int32_t* positions;
    const void* q;
    int q_f16;
    float scale_log2;      // softmax scale * log2(e): scores live in the base-2 domain
    float* partial;        // [workgroup + sequence * kv_heads + kv head][row][dim + 2]: one per segment of a workgroup's share
    unsigned rows, seqs;   // rows = span * group (query rows per K/V head)
    unsigned groups_max, share_min;   // the most workgroups that share the batch's tokens; the fewest 128-token units a share may have
    int max_context;       // positions[s] + span is clipped to this (the launch and the page table are sized for it)
    unsigned page_last;    // the pool's last page: a table entry outside the pool is taken as the nearest page of it
};

// A sequence's first query position as the kernels use it: the positions live on the device, where the host cannot check
// them, so one outside [0, max_context] is taken as the nearest end (and addresses nothing outside the page table).
__device__ __forceinline__ int first_position(const int32_t* positions, unsigned seq, int max_context) { return min(max(positions[seq], 0), max_context); }

// A page-table entry as the kernels use it: the table is device memory the host does not read, so an entry that names no page
// of the pool (negative, or past the last page) addresses the pool's last page instead of memory outside it.
__device__ __forceinline__ int pool_page(int entry, unsigned page_last) { return int(min(unsigned(entry), page_last)); }

// The maximum / the sum over the four lanes li, li + 16, li + 32, li + 48 (one query row's four lane groups), in all four.
// v_permlane16_swap exchanges the odd 16-lane rows of its first register with the even rows of its second, v_permlane32_swap
// the upper half of the first with the lower half of the second: with both registers holding the same values, each lane
// then finds its own value in one and its partner's in the other.  (Written as instructions: the compiler's builtin folds
// the two results into one when both operands are the same value.  The swap may not follow the write of its operands
// at once, hence the wait states.)
__device__ __forceinline__ void swap_rows(float& a, float& b) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void swap_halves(float& a, float& b) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ float row_max(float x) {
    float a = x, b = x;
    swap_rows(a, b);
    a = fmaxf(a, b); b = a;
    swap_halves(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float row_sum(float x) {
    float a = x, b = x;
    swap_rows(a, b);
    a += b; b = a;
    swap_halves(a, b);
    return a + b;
}

// LDS that global->LDS loads fill, read back and synchronised by hand.  The compiler guards every LDS read it can see
// against *all* outstanding global->LDS loads (a full vector-memory wait), and a __syncthreads() is a fence that waits for
// them too -- either would drain the ring of stages the loads are meant to keep full.  So the reads of such a stage are
// written as instructions (the caller has waited for exactly the loads it needs), and the barrier of a loop over the ring
// waits for the wave's LDS operations only.
typedef __attribute__((address_space(3))) const uint8_t* lds_bytes;
__device__ __forceinline__ uint32_t lds_address(const void* p) { return uint32_t(uintptr_t((lds_bytes)p)); }
__device__ __forceinline__ void ring_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// One global->LDS load: every lane's 16 bytes from its own address to LDS at to + 16 * lane (to is the wave's).  Written as
// instructions so that the compiler does not know of it -- the waits are the caller's (see above).  STREAM marks data
// that is read once (non-temporal).
template<bool STREAM>
__device__ __forceinline__ void load_to_lds(const void* from, const void* to) {
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_address(to));
    uint32_t keep;      // M0 names the LDS address; it is put back for whatever else the compiler keeps there
    if (STREAM) asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt\n\ts_mov_b32 m0, %0" : "=&s"(keep) : "v"(from), "s"(base) : "memory");
    else asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0" : "=&s"(keep) : "v"(from), "s"(base) : "memory");
}
// N (1 to 4) consecutive 1 KiB pieces as one run of instructions: `from` is an address the whole wave shares (it travels in scalar
// registers), a lane adds `lane_offset` (16 * lane, or that plus a constant), the pieces are told apart by the instruction's
// offset, which moves the global and the LDS address alike; M0 is set once.  No vector instruction forms an address.
template<bool STREAM, int N>
__device__ __forceinline__ void load_run_to_lds(const void* from, uint32_t to, uint32_t lane_offset) {
    static_assert(N >= 1 && N <= 4, "an instruction's offset reaches 4095 bytes");
    // (said to be the wave's in a way the compiler sees: where it cannot tell that the address is the same in every lane it would
    // hand over vector registers)
    const uint64_t given = uint64_t(uintptr_t(from));
    const uint64_t source = uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(given))))) |
                            uint64_t(uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(given >> 32))))) << 32;
    uint32_t keep;
#define SD_RUN_HEAD "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
#define SD_RUN_LOAD(offset, hint) "global_load_lds_dwordx4 %3, %2 offset:" #offset hint "\n\t"
#define SD_RUN_TAIL "s_mov_b32 m0, %0"
#define SD_RUN(body) asm volatile(SD_RUN_HEAD body SD_RUN_TAIL : "=&s"(keep) : "s"(to), "s"(source), "v"(lane_offset) : "memory")
    if (STREAM) {
        if (N == 1) SD_RUN(SD_RUN_LOAD(0, " nt"));
        if (N == 2) SD_RUN(SD_RUN_LOAD(0, " nt") SD_RUN_LOAD(1024, " nt"));
        if (N == 3) SD_RUN(SD_RUN_LOAD(0, " nt") SD_RUN_LOAD(1024, " nt") SD_RUN_LOAD(2048, " nt"));
        if (N == 4) SD_RUN(SD_RUN_LOAD(0, " nt") SD_RUN_LOAD(1024, " nt") SD_RUN_LOAD(2048, " nt") SD_RUN_LOAD(3072, " nt"));
    } else {
        if (N == 1) SD_RUN(SD_RUN_LOAD(0, ""));
        if (N == 2) SD_RUN(SD_RUN_LOAD(0, "") SD_RUN_LOAD(1024, ""));
        if (N == 3) SD_RUN(SD_RUN_LOAD(0, "") SD_RUN_LOAD(1024, "") SD_RUN_LOAD(2048, ""));
        if (N == 4) SD_RUN(SD_RUN_LOAD(0, "") SD_RUN_LOAD(1024, "") SD_RUN_LOAD(2048, "") SD_RUN_LOAD(3072, ""));
    }
#undef SD_RUN
#undef SD_RUN_TAIL
#undef SD_RUN_LOAD
#undef SD_RUN_HEAD
}
// The loads the compiler knows of (queries and the like) are waited for once, before the first hidden load is issued:
// its own wait for them would otherwise sit at their first use inside the loop and wait for the hidden loads as well.
__device__ __forceinline__ void settle_loads() { __builtin_amdgcn_s_waitcnt(0x0f70); }
typedef uint32_t words2 __attribute__((ext_vector_type(2)));
typedef uint32_t words4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2v as_half2(uint32_t bits) { return __builtin_bit_cast(half2v, bits); }

// v_perm_b32: byte i of the result is byte sel[i] of the 8 bytes {high, low} (0-3 = low's bytes, 4-7 = high's, 0x0c = 0x00).
__device__ __forceinline__ uint32_t byte_perm(uint32_t high, uint32_t low, uint32_t sel) { return __builtin_amdgcn_perm(high, low, sel); }

// Int8 bytes as the FP16 integers they are, then one rounding by the block scale (the reference's qsa_q8_half16,
// gpu/qsa_prompt_attention.hpp:15-33).  A byte is converted where it lies: v_cvt_f16_i16 with a byte of the source word
// sign-extended as its operand and one half of the result register as its destination (the other half kept) -- an
// instruction an element and no byte shuffling, against 1.25 an element for the bytes placed into 0x64uu patterns (v_perm, xor)
// and the patterns' bias subtracted.  Written as one run per operand: a register's two halves are written four instructions
// apart and a wait state follows the run, because a result written to half a register may not be read by the next vector
// instruction (the compiler keeps that distance for its own instructions, not for these).
#define SD_BYTE_LOW(to, from, byte) "v_cvt_f16_i16_sdwa " to ", sext(" from ") dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_" #byte "\n\t"
#define SD_BYTE_HIGH(to, from, byte) "v_cvt_f16_i16_sdwa " to ", sext(" from ") dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_" #byte "\n\t"
// the eight bytes of two words, in order
__device__ __forceinline__ void bytes_in_a_row(uint32_t low, uint32_t high, uint32_t (&pairs)[4]) {
    asm(SD_BYTE_LOW("%0", "%4", 0) SD_BYTE_LOW("%1", "%4", 2) SD_BYTE_LOW("%2", "%5", 0) SD_BYTE_LOW("%3", "%5", 2)
        SD_BYTE_HIGH("%0", "%4", 1) SD_BYTE_HIGH("%1", "%4", 3) SD_BYTE_HIGH("%2", "%5", 1) SD_BYTE_HIGH("%3", "%5", 3) "s_nop 0"
        : "=&v"(pairs[0]), "=&v"(pairs[1]), "=&v"(pairs[2]), "=&v"(pairs[3]) : "v"(low), "v"(high));
}
// byte BYTE of eight words, in order
template<int BYTE>
__device__ __forceinline__ void bytes_in_a_column(const uint32_t (&words)[8], uint32_t (&pairs)[4]) {
#define SD_COLUMN(byte) \
    asm(SD_BYTE_LOW("%0", "%4", byte) SD_BYTE_LOW("%1", "%6", byte) SD_BYTE_LOW("%2", "%8", byte) SD_BYTE_LOW("%3", "%10", byte) \
        SD_BYTE_HIGH("%0", "%5", byte) SD_BYTE_HIGH("%1", "%7", byte) SD_BYTE_HIGH("%2", "%9", byte) SD_BYTE_HIGH("%3", "%11", byte) "s_nop 0" \
        : "=&v"(pairs[0]), "=&v"(pairs[1]), "=&v"(pairs[2]), "=&v"(pairs[3]) \
        : "v"(words[0]), "v"(words[1]), "v"(words[2]), "v"(words[3]), "v"(words[4]), "v"(words[5]), "v"(words[6]), "v"(words[7]))
    if (BYTE == 0) SD_COLUMN(0);
    if (BYTE == 1) SD_COLUMN(1);
    if (BYTE == 2) SD_COLUMN(2);
    if (BYTE == 3) SD_COLUMN(3);
#undef SD_COLUMN
}
#undef SD_BYTE_HIGH
#undef SD_BYTE_LOW

template<int DIM, bool Q8> struct RowLoad;

// What one step needs from HBM, as raw words.  Q8_0: K tile t (16 tokens, lane li = token) gives each lane 8 columns of
// every 32-column block and the row's scales; V gives lane (li, g) the columns [W*li, W*li + W) (W = DIM/16) of its 8
// tokens {4g..4g+3, 16+4g..16+4g+3} and those columns' block scale.
template<int DIM> struct RowLoad<DIM, true> {
    static constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    uint2 k[2][BLOCKS];
    uint32_t kscale[2][BLOCKS / 2];
    uint32_t v[8][W / 4];
    uint16_t vscale[8];
};
// The rows lie in the wave's stage, 32 of each plane one after the other, so every piece is at a fixed distance from the
// lane's first K row (li) and first V row (4g).
template<int DIM>
__device__ __forceinline__ void load_step(RowLoad<DIM, true>& r, const uint8_t* kplane, const uint8_t* vplane, int li, int g) {
    constexpr int BLOCKS = DIM / 32, W = DIM / 16, ROW = DIM + DIM / 16;
    const uint8_t* krow = kplane + li * ROW;
    const uint8_t* vrow = vplane + 4 * g * ROW;
    #pragma unroll
    for (int t = 0; t < 2; ++t) {
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) r.k[t][b] = *reinterpret_cast<const uint2*>(krow + 16 * t * ROW + 8 * g + 32 * b);
        #pragma unroll
        for (int b = 0; b < BLOCKS / 2; ++b) r.kscale[t][b] = *reinterpret_cast<const uint32_t*>(krow + 16 * t * ROW + DIM + 4 * b);
    }
    #pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int token = e < 4 ? e : 12 + e;       // the lane's tokens are 4g + {0..3, 16..19}
        // (the lane's W bytes of a row lie at a multiple of W: one read, at a 16-bit distance from the lane's first row -- as single
        // words the reads pair up with 1 KiB of reach and every few rows want an address of their own)
        if (W == 8) {
            const uint2 words = *reinterpret_cast<const uint2*>(vrow + token * ROW + W * li);
            r.v[e][0] = words.x; r.v[e][1] = words.y;
        } else {
            const uint4 words = *reinterpret_cast<const uint4*>(vrow + token * ROW + W * li);
            r.v[e][0] = words.x; r.v[e][1] = words.y; r.v[e][W / 4 - 2] = words.z; r.v[e][W / 4 - 1] = words.w;
        }
        r.vscale[e] = *reinterpret_cast<const uint16_t*>(vrow + token * ROW + DIM + 2 * ((W * li) / 32));
    }
}

// FP16 rows: the same pieces, two bytes a value.
template<int DIM> struct RowLoad<DIM, false> {
    static constexpr int BLOCKS = DIM / 32, W = DIM / 16;
    half8 k[2][BLOCKS];
    uint32_t v[8][W / 2];
};
template<int DIM>
__device__ __forceinline__ void load_step(RowLoad<DIM, false>& r, const uint8_t* kplane, const uint8_t* vplane, int li, int g) {
    constexpr int BLOCKS = DIM / 32, W = DIM / 16, ROW = 2 * DIM;
    const uint8_t* krow = kplane + li * ROW;
    const uint8_t* vrow = vplane + 4 * g * ROW;
    #pragma unroll
    for (int t = 0; t < 2; ++t)
        #pragma unroll
        for (int b = 0; b < BLOCKS; ++b) r.k[t][b] = *reinterpret_cast<const half8*>(krow + 16 * t * ROW + 16 * g + 64 * b);
    #pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int token = e < 4 ? e : 12 + e;
        #pragma unroll
        for (int w = 0; w < W / 2; ++w) r.v[e][w] = *reinterpret_cast<const uint32_t*>(vrow + token * ROW + 2 * W * li + 4 * w);
    }
}

// The A operand of S^T = K . Q^T for tile t, block b.
template<int DIM>
__device__ __forceinline__ half8 key_operand(const RowLoad<DIM, true>& r, int t, int b) {
    const uint32_t scales = r.kscale[t][b / 2];
    const _Float16 one = (b & 1) ? as_half2(scales).y : as_half2(scales).x;      // (which half of the word a packed multiply reads is part of the instruction)
    const half2v scale = {one, one};
    uint32_t pairs[4];
    bytes_in_a_row(r.k[t][b].x, r.k[t][b].y, pairs);
    const half2v a0 = as_half2(pairs[0]) * scale, a1 = as_half2(pairs[1]) * scale, a2 = as_half2(pairs[2]) * scale, a3 = as_half2(pairs[3]) * scale;
    return half8{a0.x, a0.y, a1.x, a1.y, a2.x, a2.y, a3.x, a3.y};
}
template<int DIM>
__device__ __forceinline__ half8 key_operand(const RowLoad<DIM, false>& r, int t, int b) { return r.k[t][b]; }

// The scales of the lane's 8 tokens as 4 FP16 pairs (tokens e, e+1), formed once a step.
template<int DIM> struct ValueScales { half2v pair[4]; };
template<int DIM>
__device__ __forceinline__ void value_scales(const RowLoad<DIM, true>& r, ValueScales<DIM>& s) {
    #pragma unroll
    for (int e = 0; e < 8; e += 2) s.pair[e / 2] = as_half2(uint32_t(r.vscale[e]) | (uint32_t(r.vscale[e + 1]) << 16));
}
template<int DIM>
__device__ __forceinline__ void value_scales(const RowLoad<DIM, false>&, ValueScales<DIM>&) {}

// The A operand of O^T += V^T . P^T for output tile jj: column W*li + jj of the lane's 8 tokens.
template<int DIM>
__device__ __forceinline__ half8 value_operand(const RowLoad<DIM, true>& r, const ValueScales<DIM>& s, int jj) {
    const int word = jj / 4;
    const uint32_t words[8] = {r.v[0][word], r.v[1][word], r.v[2][word], r.v[3][word], r.v[4][word], r.v[5][word], r.v[6][word], r.v[7][word]};
    uint32_t pairs[4];
    switch (jj % 4) {
        case 0: bytes_in_a_column<0>(words, pairs); break;
        case 1: bytes_in_a_column<1>(words, pairs); break;
        case 2: bytes_in_a_column<2>(words, pairs); break;
        default: bytes_in_a_column<3>(words, pairs); break;
    }
    half2v out[4];
    #pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = as_half2(pairs[e]) * s.pair[e];
    return half8{out[0].x, out[0].y, out[1].x, out[1].y, out[2].x, out[2].y, out[3].x, out[3].y};
}
template<int DIM>
__device__ __forceinline__ half8 value_operand(const RowLoad<DIM, false>& r, const ValueScales<DIM>&, int jj) {
    half2v out[4];
    const int word = jj / 2;
    const uint32_t sel = (jj & 1) ? 0x07060302u : 0x05040100u;
    #pragma unroll
    for (int e = 0; e < 8; e += 2) out[e / 2] = as_half2(byte_perm(r.v[e + 1][word], r.v[e][word], sel));
    return half8{out[0].x, out[0].y, out[1].x, out[1].y, out[2].x, out[2].y, out[3].x, out[3].y};
}

}}  // namespace sd::paged
