// Building blocks of the grouped-GEMM kernel for gfx950 (grouped_gemm.hip): the 16-bit
// element types with their matrix instruction, buffer-descriptor addressing with direct global -> LDS loads, and the
// epilogue's transposing trip through LDS.
#pragma once

#include <type_traits>

#include "common.h"

namespace fmahip {
namespace gemm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;


constexpr int EPI_PLAIN = 0;
constexpr int EPI_SWIGLU = 1;      // stores the rounded pre-activation h and the activation
constexpr int EPI_SWIGLU_ACT = 2;  // the activation only (a forward pass that no backward follows)

// ---- the two 16-bit element types: conversions and the matrix instruction ------------------------------------------
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

struct ElemBf16 {
    using frag = bf16x8;
    using act_t = bf16_t;  // selects the activation's arithmetic (the one swiglu_forward uses for this dtype)
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {  // round to nearest even, lo in the low half
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ float round(float x) { return (float)(__bf16)x; }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return bf16_bits_to_float(b); }
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

struct ElemF16 {
    using frag = f16x8;
    using act_t = f16_t;
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f32x2 f = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ float round(float x) { return (float)(_Float16)x; }
    static __device__ __forceinline__ float from_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// ---- direct global -> LDS loaders ---------------------------------------------------------------------------------
// Every load is a buffer load to LDS (buffer_load_dwordx4 ... lds): the address is a 128-bit buffer descriptor held in
// scalar registers plus one per-lane byte offset that stays the same for the whole tile plus a scalar offset per
// instruction, so the K loop spends no vector instructions or registers on addresses. The descriptor's size field does
// the edge handling: a dword whose offset (lane + scalar part) is not below it is not read and lands in LDS as zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const uint16_t* p, uint32_t bytes) {
    // stride 0 (raw buffer), 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p), 0, (int)bytes, 0x00020000);
}
// The same load written in assembly, with its M0 set-up (M0 holds the LDS address the wavefront's 1 KB goes to). The
// compiler does not see that it writes LDS, so it places no waits of its own for it: the first loads of a tile are
// issued this way, partly while the previous tile's epilogue is still running, and waited for with an exact count.
__device__ __forceinline__ void buffer_load_lds_quiet(u32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) {
    // M0 is put back afterwards: the compiler keeps its own values in it and does not honour a clobber of it
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_addr));
}
__device__ __forceinline__ uint32_t lds_address(const uint8_t* p) {
    return (uint32_t)(uintptr_t)(lds_void*)const_cast<uint8_t*>(p);
}
// the descriptor make_rsrc() builds, as four plain words in scalar registers (p and bytes are the same in every lane)
__device__ __forceinline__ u32x4 make_rsrc_words(const uint16_t* p, uint32_t bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)p;
    u32x4 r;
    r.x = (uint32_t)a;
    r.y = (uint32_t)(a >> 32) & 0xffffu;
    r.z = bytes;
    r.w = 0x00020000u;
    return r;
}
__device__ __forceinline__ uint32_t uniform(uint32_t x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ uint64_t uniform(uint64_t x) {
    return ((uint64_t)uniform((uint32_t)(x >> 32)) << 32) | uniform((uint32_t)x);
}
constexpr uint32_t kOutOfRange = 0x80000000u;  // lane offset no descriptor of this kernel reaches (sizes stay < 2^31)


__device__ __forceinline__ s16x8 read_kc_frag(const uint8_t* p) { return *reinterpret_cast<const s16x8*>(p); }

// ---- epilogue staging: a wavefront transposes its accumulator sub-tile, half at a time, through 8 KB of LDS ----
// The MFMA leaves a lane with 4 consecutive columns of one row per 32x32 block, so storing straight from registers
// writes 8-byte pieces of 32 different rows per instruction. Staged through LDS as rows of ROWB bytes, every store
// instruction writes 16 bytes per lane and whole 64- or 128-byte row segments.
// Row m, 16-byte chunk c of the image sits at m*ROWB + ((c ^ key(m)) << 4), key(m) = (m / rows-per-256-B) mod chunks:
// the 8-byte writes of 32 consecutive rows conflict at most two ways, the 16-byte reads not at all.

// 16-byte buffer store of a staged piece. A lane whose offset is not below the descriptor's size stores nothing, so
// every lane always executes the instruction: the number of stores a wavefront issues per tile is a compile-time
// constant, which the wait for the next tile's first loads relies on.
// NT = the non-temporal hint. Measured both ways on the three benchmark layers: with the hint the six GEMMs ran 0.5 to
// 1.5 points of peak slower than with plain stores (22 of 24 comparisons), and streamed 64-byte pieces are not merged
// in the L2 and cost a read-modify-write each (SwiGLU epilogue: +35 % fetched and +28 % written bytes). No caller sets it.
template <bool NT>
__device__ __forceinline__ void store_tile16(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, (int)voff, 0, NT ? 2 : 0);
}
template <int ROWB>
__device__ __forceinline__ uint32_t stage_off(uint32_t m, uint32_t chunk16) {
    constexpr uint32_t kChunks = ROWB / 16;
    constexpr uint32_t kRowsPer256 = 256 / ROWB;
    return m * ROWB + ((chunk16 ^ ((m / kRowsPer256) & (kChunks - 1))) << 4);
}
// A wavefront's staging slice is made of the 1 KB pieces of LDS stage 1 that the wavefront itself fills when it loads
// operands (pieces wave, wave + NW, ... of the A array, then of the B array), so only its own loads ever overwrite its
// image and no workgroup barrier is needed between an epilogue and the next tile's loads into stage 1.
template <int NW>
struct StagingSlice {
    uint8_t* a;  // LDS stage 1, A array, this wavefront's first piece
    uint8_t* b;  // the same of the B array
    __device__ __forceinline__ uint8_t* at(uint32_t off) const {  // byte `off` of the image
        constexpr uint32_t kPieces = 32 / NW;                    // pieces per array
        const uint32_t piece = off >> 10;
        return (piece < kPieces ? a : b) + (piece % kPieces) * (uint32_t)(NW * 1024) + (off & 1023u);
    }
};
// lane's 4 columns [col, col+4) of image row m
template <int ROWB, typename Slice>
__device__ __forceinline__ void stage_put(const Slice& img, uint32_t m, uint32_t col, uint2 v) {
    *reinterpret_cast<uint2*>(img.at(stage_off<ROWB>(m, col >> 3) + ((col >> 2) & 1u) * 8u)) = v;
}
// Stores the image (ROWS rows of ROWB/2 columns) to origin[r * ld + c]; only the first rows_valid rows and cols_valid
// columns exist in the output (both may be 0). ld and cols_valid are multiples of 8 elements, so every 16-byte piece
// is wholly inside or outside. Issues exactly ROWS * ROWB / 1024 store instructions.
template <int ROWB, int ROWS, typename Slice>
__device__ __forceinline__ void stage_flush(const Slice& img, uint16_t* origin, uint32_t ld, uint32_t rows_valid,
                                            uint32_t cols_valid, uint32_t lane) {
    constexpr uint32_t kChunks = ROWB / 16;  // 16-byte pieces per image row
    constexpr uint32_t kRowsPerInst = 64 / kChunks;
    const uint32_t c16 = lane % kChunks;
    const uint32_t ldb = ld * 2u;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(origin, rows_valid * ldb);
    const bool col_ok = c16 * 8u < cols_valid;
#pragma unroll
    for (uint32_t it = 0; it < ROWS / kRowsPerInst; ++it) {
        const uint32_t r = it * kRowsPerInst + lane / kChunks;
        const uint4 v = *reinterpret_cast<const uint4*>(img.at(stage_off<ROWB>(r, c16)));
        store_tile16<false>(rsrc, col_ok ? r * ldb + c16 * 16u : kOutOfRange, v);
    }
}

// Like stage_flush for an image whose row holds two windows of HALF columns each: window 0 goes to columns 0.. of the
// origin's row, window 1 to columns second0.. of the same row (the "up" and "gate" halves of h).
template <int ROWB, int ROWS, int HALF, typename Slice>
__device__ __forceinline__ void stage_flush_split(const Slice& img, uint16_t* origin, uint32_t ld, uint32_t rows_valid,
                                                  uint32_t cols_valid, uint32_t second0, uint32_t lane) {
    constexpr uint32_t kChunks = ROWB / 16;
    constexpr uint32_t kRowsPerInst = 64 / kChunks;
    const uint32_t c16 = lane % kChunks;
    const uint32_t in_window = (c16 * 8u) % HALF;
    const uint32_t window = (c16 * 8u) / HALF;
    const uint32_t ldb = ld * 2u;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(origin, rows_valid * ldb);
    const bool col_ok = in_window < cols_valid;
#pragma unroll
    for (uint32_t it = 0; it < ROWS / kRowsPerInst; ++it) {
        const uint32_t r = it * kRowsPerInst + lane / kChunks;
        const uint4 v = *reinterpret_cast<const uint4*>(img.at(stage_off<ROWB>(r, c16)));
        store_tile16<false>(rsrc, col_ok ? r * ldb + (window * second0 + in_window) * 2u : kOutOfRange, v);
    }
}

// Scheduling hint for one k slice: MFMAS matrix instructions with READS LDS reads spread evenly between them.
template <int R, int MFMAS, int READS>
__device__ __forceinline__ void interleave_mfma_lds() {
    constexpr int kPairs = READS < MFMAS ? READS : MFMAS;
    constexpr int kPer = READS / kPairs;           // LDS reads after each of the first kPairs MFMAs
    constexpr int kExtra = READS - kPairs * kPer;  // the first kExtra of them get one more
    if constexpr (R < kPairs) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, kPer + (R < kExtra ? 1 : 0), 0);
        interleave_mfma_lds<R + 1, MFMAS, READS>();
    } else if constexpr (MFMAS - kPairs > 0) {
        __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - kPairs, 0);
    }
}

// Scheduling hint for one k slice: MFMAS matrix instructions, READS LDS reads spread between them, and LOADS buffer
// loads placed one after each of the first MFMAs.
template <int R, int MFMAS, int READS, int LOADS>
__device__ __forceinline__ void interleave3() {
    constexpr int kPairs = READS < MFMAS ? READS : MFMAS;
    constexpr int kPer = kPairs ? READS / kPairs : 0;
    constexpr int kExtra = READS - kPairs * kPer;
    if constexpr (R < MFMAS) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (R < kPairs) __builtin_amdgcn_sched_group_barrier(0x100, kPer + (R < kExtra ? 1 : 0), 0);
        if constexpr (R < LOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        interleave3<R + 1, MFMAS, READS, LOADS>();
    }
}

// Scheduling hint: MFMAS matrix instructions with LOADS buffer loads placed one after each of the first MFMAs.
template <int R, int MFMAS, int LOADS>
__device__ __forceinline__ void spread_mfma_vmem() {
    if constexpr (R < MFMAS) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (R < LOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        spread_mfma_vmem<R + 1, MFMAS, LOADS>();
    }
}

// Slow, layout-agnostic path for a group whose contiguous dimensions are not multiples of 8 elements.
template <typename EL, bool A_KC, bool B_KC, int TM, int TN>
__device__ void scalar_tile(const uint16_t* Ae, const uint16_t* Be, uint16_t* De, uint32_t Me, uint32_t Ne,
                            uint32_t Ke, uint32_t m0, uint32_t n0, float alpha, uint32_t nthreads) {
    for (uint32_t idx = threadIdx.x; idx < (uint32_t)(TM * TN); idx += nthreads) {
        const uint32_t m = m0 + idx / TN;
        const uint32_t n = n0 + idx % TN;
        if (m >= Me || n >= Ne) continue;
        float acc = 0.0f;
        for (uint32_t k = 0; k < Ke; ++k) {
            const uint16_t a = A_KC ? Ae[(uint64_t)m * Ke + k] : Ae[(uint64_t)k * Me + m];
            const uint16_t b = B_KC ? Be[(uint64_t)n * Ke + k] : Be[(uint64_t)k * Ne + n];
            acc = fmaf(EL::from_bits(a), EL::from_bits(b), acc);
        }
        De[(uint64_t)m * Ne + n] = (uint16_t)(EL::pack2(alpha * acc, 0.0f) & 0xffffu);
    }
}

}  // namespace gemm
}  // namespace fmahip
