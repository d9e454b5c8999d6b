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
typedef __attribute__((ext_vector_type(4))) float f32x4;
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
// the product is the gradient of a SwiGLU activation: the gradient of the packed pre-activation h is written instead
// (columns c and I + c of a row from column c of the product), with h read in the epilogue
constexpr int EPI_SWIGLU_BWD = 3;

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
    // 16x16 block over 32 k: at the same arithmetic rate the part sustains a higher clock on this shape (measured on
    // N(0,1) operands, matrix instructions only: 0.79 against 0.70 of the peak rate)
    static __device__ __forceinline__ f32x4 mfma16(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
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
    static __device__ __forceinline__ f32x4 mfma16(frag a, frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
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
// States that a value is the same in every lane (a no-op for a value the compiler already keeps in scalar registers).
// The assembly below needs its scalar operands in scalar registers whatever the compiler has decided about the
// computation that feeds them.
__device__ __forceinline__ uint32_t uniform(uint32_t x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ u32x4 uniform(u32x4 x) {
    return u32x4{uniform(x[0]), uniform(x[1]), uniform(x[2]), uniform(x[3])};
}
// The same load written in assembly, with its M0 set-up (M0 holds the LDS address the wavefront's 1 KB goes to). The
// compiler does not see that it writes LDS, so it places no waits of its own for it: the first loads of a tile are
// issued this way, partly while the previous tile's epilogue is still running, and waited for with an exact count.
// (s_nop 2: the scalar operands may come from a v_readfirstlane right in front of the assembly, and a vector-memory
// instruction must not read such a register within five wait states; the compiler does not check assembly for that.)
__device__ __forceinline__ void buffer_load_lds_quiet(u32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) {
    // M0 is put back afterwards: the compiler keeps its own values in it and does not honour a clobber of it
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %4\n\ts_nop 2\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(voff), "s"(uniform(rsrc)), "s"(uniform(soff)), "s"(uniform(lds_addr)));
}
// the 4-byte form of the same load (64 lanes x 4 bytes = 256 bytes of LDS per instruction)
__device__ __forceinline__ void buffer_load_lds_quiet_b32(u32x4 rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) {
    uint32_t saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %4\n\ts_nop 2\n\tbuffer_load_dword %1, %2, %3 offen lds\n\t"
                 "s_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "v"(voff), "s"(uniform(rsrc)), "s"(uniform(soff)), "s"(uniform(lds_addr)));
}
// LDS words at addr, addr + 256, addr + 512 and addr + 768 bytes, read in assembly and waited for here: for a table that
// only direct-to-LDS loads written in assembly fill, which the compiler therefore knows nothing about
__device__ __forceinline__ void lds_read4_stride64_quiet(uint32_t addr, uint32_t (&v)[4]) {
    uint2 a, b;
    asm volatile("ds_read2st64_b32 %0, %2 offset1:1\n\tds_read2st64_b32 %1, %2 offset0:2 offset1:3\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(a), "=&v"(b)
                 : "v"(addr));
    v[0] = a.x;
    v[1] = a.y;
    v[2] = b.x;
    v[3] = b.y;
}
__device__ __forceinline__ uint32_t lds_read1_quiet(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr));
    return v;
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
__device__ __forceinline__ uint64_t uniform(uint64_t x) {
    return ((uint64_t)uniform((uint32_t)(x >> 32)) << 32) | uniform((uint32_t)x);
}
constexpr uint32_t kOutOfRange = 0x80000000u;  // lane offset no descriptor of this kernel reaches (sizes stay < 2^31)


__device__ __forceinline__ s16x8 read_kc_frag(const uint8_t* p) { return *reinterpret_cast<const s16x8*>(p); }

// ---- epilogue staging: a wavefront transposes its accumulator sub-tile, half at a time, through 8 KB of LDS ----
// The MFMA leaves a lane with 4 consecutive columns of one row per accumulator block, so storing straight from registers
// writes 8-byte pieces of 16 or 32 different rows per instruction. Staged through LDS as rows of ROWB bytes, every store
// instruction writes 16 bytes per lane and whole 64- or 128-byte row segments.
// Row m, 16-byte chunk c of the image sits at m*ROWB + ((c ^ key(m)) << 4), key(m) = (m / rows-per-256-B) mod chunks:
// the 8-byte writes of 32 consecutive rows conflict at most two ways, the 16-byte reads not at all.

// 16-byte buffer store of a staged piece. A lane whose offset is not below the descriptor's size stores nothing, so
// every lane always executes the instruction: the number of stores a wavefront issues per tile is a compile-time
// constant, which the wait for the next tile's first loads relies on.
// NT = the non-temporal hint. Measured both ways on the three benchmark layers: hinted and plain stores of whole
// 128-byte lines run within 0.5 % of each other, except for weight-gradient tiles with a short reduction, which write
// much per flop and gain 1.5 to 4 % from the hint (the only caller that sets it); streamed 64-byte pieces are not merged
// in the L2 and cost a read-modify-write each (SwiGLU epilogue: +35 % fetched and +28 % written bytes).
template <bool NT>
__device__ __forceinline__ void store_tile16(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, (int)voff, 0, NT ? 2 : 0);
}
// The same store with the non-temporal hint, written in assembly: for an epilogue whose store COUNT the next tile's waits
// rely on, where nothing may merge, split or drop one. rsrc: the descriptor as four words (make_rsrc_words). A vector
// instruction that overwrites the data registers must not follow a 16-byte store directly; the compiler places that wait
// state behind its own stores only, so it is part of the assembly here.
__device__ __forceinline__ void store_tile16_quiet_nt(u32x4 rsrc, uint32_t voff, u32x4 v) {
    asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen nt\n\ts_nop 1" ::"v"(v), "v"(voff), "s"(uniform(rsrc)) : "memory");
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
    // The image is written as 8-byte and read as 16-byte vectors: two types that type-based alias analysis treats as
    // never overlapping, so without these fences the compiler may move the reads above the writes that feed them (or the
    // next image's writes above these reads). The LDS itself executes a wavefront's accesses in order.
    asm volatile("" ::: "memory");
#pragma unroll
    for (uint32_t it = 0; it < ROWS / kRowsPerInst; ++it) {
        const uint32_t r = it * kRowsPerInst + lane / kChunks;
        const uint4 v = *reinterpret_cast<const uint4*>(img.at(stage_off<ROWB>(r, c16)));
        store_tile16<false>(rsrc, col_ok ? r * ldb + c16 * 16u : kOutOfRange, v);
    }
    asm volatile("" ::: "memory");
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
    asm volatile("" ::: "memory");  // (see stage_flush)
#pragma unroll
    for (uint32_t it = 0; it < ROWS / kRowsPerInst; ++it) {
        const uint32_t r = it * kRowsPerInst + lane / kChunks;
        const uint4 v = *reinterpret_cast<const uint4*>(img.at(stage_off<ROWB>(r, c16)));
        store_tile16<false>(rsrc, col_ok ? r * ldb + (window * second0 + in_window) * 2u : kOutOfRange, v);
    }
    asm volatile("" ::: "memory");
}

// The same staging written in assembly, for an epilogue that runs while direct-to-LDS loads of the next tile are in
// flight: the compiler orders every LDS store of its own behind all such loads (s_waitcnt vmcnt), whatever LDS object they
// write, which would make the epilogue wait for the operands of the next tile. The LDS executes a wavefront's accesses
// in order, so the reads below see the writes above them without any wait; each flush waits for its own reads.
// `image` is the LDS byte address of the wavefront's staging slice.
template <int ROWB>
__device__ __forceinline__ void stage_put_quiet(uint32_t image, uint32_t m, uint32_t col, uint2 v) {
    const uint32_t addr = image + stage_off<ROWB>(m, col >> 3) + ((col >> 2) & 1u) * 8u;
    asm volatile("ds_write_b64 %0, %1" ::"v"(addr), "v"(__builtin_bit_cast(uint64_t, v)) : "memory");
}
// four 8-byte reads at LDS byte addresses a[0..3], complete on return (written in assembly for the same reason)
__device__ __forceinline__ void lds_read4x8_quiet(const uint32_t (&a)[4], uint2 (&v)[4]) {
    uint64_t r[4];
    asm volatile("ds_read_b64 %0, %4\n\tds_read_b64 %1, %5\n\tds_read_b64 %2, %6\n\tds_read_b64 %3, %7\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3])
                 : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3])
                 : "memory");
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_bit_cast(uint2, r[i]);
}
// two 16-byte reads of the image (at byte offsets off0 and off1), complete on return
__device__ __forceinline__ void stage_get2_quiet(uint32_t image, uint32_t off0, uint32_t off1, u32x4& v0, u32x4& v1) {
    asm volatile("ds_read_b128 %0, %2\n\tds_read_b128 %1, %3\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(v0), "=&v"(v1)
                 : "v"(image + off0), "v"(image + off1)
                 : "memory");
}
// stage_flush for images of exactly two store instructions (ROWS * ROWB == 2048)
// stream (the same in every lane): store with the non-temporal hint
template <int ROWB, int ROWS>
__device__ __forceinline__ void stage_flush_quiet(uint32_t image, uint16_t* origin, uint32_t ld, uint32_t rows_valid,
                                                  uint32_t cols_valid, uint32_t lane, bool stream = false) {
    constexpr uint32_t kChunks = ROWB / 16;
    constexpr uint32_t kRowsPerInst = 64 / kChunks;
    static_assert(ROWS == 2 * kRowsPerInst, "two store instructions per image");
    const uint32_t c16 = lane % kChunks;
    const uint32_t ldb = ld * 2u;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(origin, rows_valid * ldb);
    const bool col_ok = c16 * 8u < cols_valid;
    const uint32_t r0 = lane / kChunks, r1 = kRowsPerInst + lane / kChunks;
    u32x4 v0, v1;
    stage_get2_quiet(image, stage_off<ROWB>(r0, c16), stage_off<ROWB>(r1, c16), v0, v1);
    const uint32_t off0 = col_ok ? r0 * ldb + c16 * 16u : kOutOfRange, off1 = col_ok ? r1 * ldb + c16 * 16u : kOutOfRange;
    if (stream) {
        store_tile16<true>(rsrc, off0, __builtin_bit_cast(uint4, v0));
        store_tile16<true>(rsrc, off1, __builtin_bit_cast(uint4, v1));
    } else {
        store_tile16<false>(rsrc, off0, __builtin_bit_cast(uint4, v0));
        store_tile16<false>(rsrc, off1, __builtin_bit_cast(uint4, v1));
    }
}
template <int ROWB, int ROWS, int HALF>
__device__ __forceinline__ void stage_flush_split_quiet(uint32_t image, uint16_t* origin, uint32_t ld, uint32_t rows_valid,
                                                        uint32_t cols_valid, uint32_t second0, uint32_t lane) {
    constexpr uint32_t kChunks = ROWB / 16;
    constexpr uint32_t kRowsPerInst = 64 / kChunks;
    static_assert(ROWS == 2 * kRowsPerInst, "two store instructions per image");
    const uint32_t c16 = lane % kChunks;
    const uint32_t in_window = (c16 * 8u) % HALF;
    const uint32_t window = (c16 * 8u) / HALF;
    const uint32_t ldb = ld * 2u;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(origin, rows_valid * ldb);
    const bool col_ok = in_window < cols_valid;
    const uint32_t r0 = lane / kChunks, r1 = kRowsPerInst + lane / kChunks;
    const uint32_t col_off = (window * second0 + in_window) * 2u;
    u32x4 v0, v1;
    stage_get2_quiet(image, stage_off<ROWB>(r0, c16), stage_off<ROWB>(r1, c16), v0, v1);
    store_tile16<false>(rsrc, col_ok ? r0 * ldb + col_off : kOutOfRange, __builtin_bit_cast(uint4, v0));
    store_tile16<false>(rsrc, col_ok ? r1 * ldb + col_off : kOutOfRange, __builtin_bit_cast(uint4, v1));
}

// ---- tile geometry and the two LDS layouts of an operand tile ----------------------------------------------------
constexpr int BM = 256;
constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kRowBytes = BK * 2;           // 128: row of a [row][64 k] tile
constexpr int kTRowBytes = BM * 2;          // 512: row of a [64 k][256 out] tile
constexpr int kTileBytes = BM * kRowBytes;  // 32 KB per operand per stage, either layout
constexpr int kGroupM = 8;                  // m-tiles that share one column sweep of the tile order
constexpr int kXcds = 8;

__device__ __forceinline__ uint32_t phys_row(uint32_t r) { return (r & ~15u) | ((r & 7u) << 1) | ((r >> 3) & 1u); }
__device__ __forceinline__ uint32_t logical_row(uint32_t pr) {
    return (pr & ~15u) | ((pr & 15u) >> 1) | ((pr & 1u) << 3);
}
// [row][64 k] tile: byte offset of 16-byte chunk `chunk` of row r
__device__ __forceinline__ uint32_t kc_off(uint32_t r, uint32_t chunk) {
    return phys_row(r) * kRowBytes + ((chunk ^ (r & 7u)) << 4);
}
// [64 k][256 out] tile: byte offset, for k slice 0, of the first transposing read of the fragment that starts at out
// row r0 (a multiple of 32). Slice ks adds 16 rows, the second read of a fragment (k + 4) adds 4 rows.
__device__ __forceinline__ uint32_t mc_frag_off(uint32_t r0, uint32_t lane) {
    const uint32_t g = lane >> 4, j = lane & 15u;
    const uint32_t q = j & 3u, kr = j >> 2;
    const uint32_t chunk = (r0 >> 3) + 2u * (g & 1u) + (q >> 1);
    return (8u * (g >> 1) + kr) * kTRowBytes + ((chunk ^ (4u * kr)) << 4) + (q & 1u) * 8u;
}
// The same for fragments of the 16x16x32 instruction (16 out rows, a lane holds 8 consecutive k of one row, lanes
// 16g.. the g-th eight of the slice's 32 k): the fragment that starts at out row r0 (a multiple of 16), k slice 0 of two.
// Slice 1 adds 32 rows, the second read of a fragment (k + 4) adds 4 rows. For a tile written by LoaderT<NW, true>: the
// chunk position is also flipped by bit 3 of the k row, which keeps the reads of lanes 16..31 (k rows 8..15) off the
// banks of lanes 0..15.
__device__ __forceinline__ uint32_t mc_frag_off16(uint32_t r0, uint32_t lane) {
    const uint32_t g = lane >> 4, j = lane & 15u;
    const uint32_t q = j & 3u, kr = j >> 2;
    const uint32_t chunk = (r0 >> 3) + (q >> 1);
    return (8u * g + kr) * kTRowBytes + ((chunk ^ (4u * kr) ^ (2u * (g & 1u))) << 4) + (q & 1u) * 8u;
}

// Operand with the reduction dimension contiguous: tile [256 rows][64 k]. A wavefront instruction moves 8 physical rows
// (1 KB); NI instructions per wavefront and K step. SPLIT: tile rows 128..255 come from a second row range (base1).
template <int NW, bool SPLIT>
struct LoaderK {
    static constexpr int NI = 32 / NW;
    static constexpr uint32_t kRowsPerInst = NW * 8;
    const uint16_t* base0;  // first element of tile row 0
    const uint16_t* base1;  // SPLIT: first element of tile row 128
    uint32_t bytes;         // valid bytes from a base: rows inside the operand x row pitch
    uint32_t ldb;           // row pitch in bytes
    uint32_t voff;          // this lane's offset: its row of instruction 0, its 16-byte chunk
    uint32_t chunk;         // this lane's logical chunk (the same for every instruction)
    uint32_t kdim;
    uint32_t wave;

    // rows_valid: rows of the tile (of each half when SPLIT) that exist in the operand; the rest arrives as zeros
    __device__ __forceinline__ void setup(const uint16_t* b0, const uint16_t* b1, uint32_t rows_valid, uint32_t kdim_,
                                          uint32_t wave_, uint32_t lane) {
        static_assert(NW % 2 == 0, "chunk is per lane only for an even number of wavefronts");
        base0 = b0;
        base1 = b1;
        kdim = kdim_;
        wave = wave_;
        ldb = kdim_ * 2u;
        bytes = rows_valid * ldb;
        const uint32_t r = logical_row(wave_ * 8u + (lane >> 3));
        chunk = (lane & 7u) ^ (r & 7u);
        voff = r * ldb + chunk * 16u;
    }

    __device__ __forceinline__ void issue(uint8_t* tile, uint32_t k0) const { issue_range<0, NI>(tile, k0); }
    // instructions I0 .. I1-1 of the K step at k0
    template <int I0, int I1>
    __device__ __forceinline__ void issue_range(uint8_t* tile, uint32_t k0) const {
        uint32_t v = voff;
        // last, partial K step: chunks past the end of K are pushed out of range, which zero-fills them
        if (k0 + BK > kdim && k0 + chunk * 8u >= kdim) v = kOutOfRange;
        const __amdgpu_buffer_rsrc_t r0 = make_rsrc(base0, bytes);
        const __amdgpu_buffer_rsrc_t r1 = make_rsrc(SPLIT ? base1 : base0, bytes);
#pragma unroll
        for (int i = I0; i < I1; ++i) {
            const bool second = SPLIT && i >= NI / 2;
            const uint32_t row = (uint32_t)(second ? i - NI / 2 : i) * kRowsPerInst;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(second ? r1 : r0, (lds_void*)(tile + (i * NW + wave) * 1024), 16, v,
                                                     k0 * 2u + row * ldb, 0, 0);
        }
    }
    // the same NI loads through buffer_load_lds_quiet
    __device__ __forceinline__ void issue_quiet(uint8_t* tile, uint32_t k0) const {
        uint32_t v = voff;
        if (k0 + BK > kdim && k0 + chunk * 8u >= kdim) v = kOutOfRange;
        const u32x4 r0 = make_rsrc_words(base0, bytes);
        const u32x4 r1 = make_rsrc_words(SPLIT ? base1 : base0, bytes);
        const uint32_t lds0 = lds_address(tile) + wave * 1024u;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool second = SPLIT && i >= NI / 2;
            const uint32_t row = (uint32_t)(second ? i - NI / 2 : i) * kRowsPerInst;
            buffer_load_lds_quiet(second ? r1 : r0, v, k0 * 2u + row * ldb, lds0 + (uint32_t)(i * NW) * 1024u);
        }
    }
    // only the instruction that covers tile rows 0 .. NW*8-1, to the LDS address lds_base (a tile with few rows)
    __device__ __forceinline__ void issue_quiet_first_rows(uint32_t lds_base, uint32_t k0) const {
        uint32_t v = voff;
        if (k0 + BK > kdim && k0 + chunk * 8u >= kdim) v = kOutOfRange;
        buffer_load_lds_quiet(make_rsrc_words(base0, bytes), v, k0 * 2u, lds_base + wave * 1024u);
    }
    // the NI loads with the first half of the tile's 1 KB pieces going to lds_lo and the second half to lds_hi
    __device__ __forceinline__ void issue_quiet_halves(uint32_t lds_lo, uint32_t lds_hi, uint32_t k0) const {
        uint32_t v = voff;
        if (k0 + BK > kdim && k0 + chunk * 8u >= kdim) v = kOutOfRange;
        const u32x4 r0 = make_rsrc_words(base0, bytes);
        const u32x4 r1 = make_rsrc_words(SPLIT ? base1 : base0, bytes);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool second = SPLIT && i >= NI / 2;
            const uint32_t row = (uint32_t)(second ? i - NI / 2 : i) * kRowsPerInst;
            const uint32_t lds = (i < NI / 2 ? lds_lo + (uint32_t)(i * NW) * 1024u : lds_hi + (uint32_t)((i - NI / 2) * NW) * 1024u) + wave * 1024u;
            buffer_load_lds_quiet(second ? r1 : r0, v, k0 * 2u + row * ldb, lds);
        }
    }
};

// Operand stored [reduction][out] (out contiguous): tile [64 k][256 out]. A wavefront instruction moves two k rows
// (2 x 512 B). Rows past the end of the reduction are out of the descriptor's range (zeros); columns past the end of
// the operand's rows read whatever follows, which only reaches outputs that are never stored.
// SWZ16: the chunk positions that mc_frag_off16 reads (otherwise those of mc_frag_off).
template <int NW, bool SWZ16 = false>
struct LoaderT {
    static constexpr int NI = 32 / NW;
    const uint16_t* base;  // row 0 of the group's operand, first column of the tile
    uint32_t ldb;          // row pitch in bytes
    uint32_t col_bytes;    // byte offset of the tile's first column inside a row
    uint32_t voff;
    uint32_t kdim;
    uint32_t wave;

    __device__ __forceinline__ void setup(const uint16_t* group_base, uint32_t ld, uint32_t kdim_, uint32_t out0,
                                          uint32_t wave_, uint32_t lane) {
        base = group_base + out0;
        ldb = ld * 2u;
        col_bytes = out0 * 2u;
        kdim = kdim_;
        wave = wave_;
        const uint32_t khalf = lane >> 5;  // which of the two rows of an instruction this lane loads
        const uint32_t krow = wave_ * 2u + khalf;
        static_assert(!SWZ16 || NW == 8, "bit 3 of a lane's k row must be the same for every instruction");
        // (an instruction's rows are 16 i + krow: bit 3 of the k row is bit 3 of krow for every instruction i)
        const uint32_t flip = 4u * (krow & 3u) ^ (SWZ16 ? 2u * ((krow >> 3) & 1u) : 0u);
        voff = khalf * ldb + (((lane & 31u) ^ flip) << 4);
    }

    __device__ __forceinline__ void issue(uint8_t* tile, uint32_t k0) const { issue_range<0, NI>(tile, k0); }
    template <int I0, int I1>
    __device__ __forceinline__ void issue_range(uint8_t* tile, uint32_t k0) const {
        // rows of this K step that exist (none at all when the step lies past the end: everything is zero-filled)
        const uint32_t rows = k0 >= kdim ? 0u : (kdim - k0 < (uint32_t)BK ? kdim - k0 : (uint32_t)BK);
        const __amdgpu_buffer_rsrc_t r = make_rsrc(base + (uint64_t)k0 * (ldb / 2u), rows ? rows * ldb - col_bytes : 0u);
#pragma unroll
        for (int i = I0; i < I1; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)(tile + (i * NW + wave) * 1024), 16, voff,
                                                     (uint32_t)(i * NW + wave) * 2u * ldb, 0, 0);
        }
    }
    __device__ __forceinline__ void issue_quiet(uint8_t* tile, uint32_t k0) const {
        const uint32_t rows = k0 >= kdim ? 0u : (kdim - k0 < (uint32_t)BK ? kdim - k0 : (uint32_t)BK);
        const u32x4 r = make_rsrc_words(base + (uint64_t)k0 * (ldb / 2u), rows ? rows * ldb - col_bytes : 0u);
        const uint32_t lds0 = lds_address(tile) + wave * 1024u;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            buffer_load_lds_quiet(r, voff, (uint32_t)(i * NW + wave) * 2u * ldb, lds0 + (uint32_t)(i * NW) * 1024u);
        }
    }
    // the NI loads with k rows 0..31 of the step going to lds_lo and k rows 32..63 to lds_hi
    __device__ __forceinline__ void issue_quiet_halves(uint32_t lds_lo, uint32_t lds_hi, uint32_t k0) const {
        const uint32_t rows = k0 >= kdim ? 0u : (kdim - k0 < (uint32_t)BK ? kdim - k0 : (uint32_t)BK);
        const u32x4 r = make_rsrc_words(base + (uint64_t)k0 * (ldb / 2u), rows ? rows * ldb - col_bytes : 0u);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const uint32_t lds = (i < NI / 2 ? lds_lo + (uint32_t)(i * NW) * 1024u : lds_hi + (uint32_t)((i - NI / 2) * NW) * 1024u) + wave * 1024u;
            buffer_load_lds_quiet(r, voff, (uint32_t)(i * NW + wave) * 2u * ldb, lds);
        }
    }
};

__device__ __forceinline__ s16x8 read_tr_frag(const uint8_t* p) {
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * kTRowBytes));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
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
