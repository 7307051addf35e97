// K / V tile geometry, LDS swizzles and the asynchronous global -> LDS tile copy shared by the tiled kernels.
#pragma once
#include "acsr_plan.hpp"

namespace splat {

template <typename T, int D, bool KT, int BN = kBN>
struct TileGeom {
    static constexpr int ES = sizeof(T);
    static constexpr int EPC = 16 / ES;                       // elements per 16-byte chunk
    static constexpr int K_ROWB = KT ? BN * ES : D * ES;      // bytes per LDS row of the K tile (no padding)
    static constexpr int K_ROWS = KT ? D : BN;
    static constexpr int V_ROWB = D * ES;
    static constexpr int K_BYTES = K_ROWB * K_ROWS;
    static constexpr int V_BYTES = V_ROWB * BN;
    static constexpr int STAGE = K_BYTES + V_BYTES;
};

// XOR swizzle of the 16-byte chunk index of a row-major LDS tile with ROWB-byte rows, chosen so that 16
// lanes reading the same logical chunk of 16 consecutive rows hit 16 different bank groups.
template <int ROWB>
__device__ __forceinline__ constexpr int swz(int row) {
    constexpr int CPR = ROWB / 16;
    constexpr int CH = CPR < 16 ? CPR : 16;
    constexpr int RPB = ROWB >= 256 ? 1 : 256 / ROWB;
    return (row / RPB) & (CH - 1);
}
template <int ROWB, bool SWZ>
__device__ __forceinline__ int lds_off(int row, int byte_col) {
    if constexpr (SWZ)
        return row * ROWB + ((((byte_col >> 4) ^ swz<ROWB>(row)) << 4) | (byte_col & 15));
    else
        return row * ROWB + byte_col;
}

// Swizzle of the 64-byte block index for tiles read with the transposing read, whose 64 lanes touch 8
// consecutive rows x 64 bytes: 4 consecutive rows must fall into the 4 different 64-byte quadrants of the
// 256-byte bank space (what a row pitch of 256+64 bytes would give, which the 1 KiB LDS-DMA blocks rule out).
template <int ROWB>
__device__ __forceinline__ constexpr int swz64(int row) {
    return ROWB >= 256 ? (row & 3) : ((row >> 1) & 1);
}
// Swizzle for tiles that are read both ways: the 64-byte block index is rotated as for the transposing read, and the
// chunk inside the block by the next two row bits, so that the 16 rows a row-wise 16-byte read touches at once land on
// 16 different chunk positions of the 256-byte bank space (rows 16 apart share their pattern; rows 8 apart differ in
// the second bit of the chunk position).  The map is its own inverse.
template <int ROWB>
__device__ __forceinline__ constexpr int dual_chunk(int row, int c) {
    return (((c >> 2) ^ swz64<ROWB>(row)) << 2) | ((c & 3) ^ ((row >> 2) & 3));
}
// logical 16-byte chunk held at physical chunk position pc of `row`; MODE 0: none, 1: chunk XOR (b128 row reads),
// 2: 64-byte block XOR (transposing reads), 3: both kinds of read (dual_chunk)
template <int ROWB, int MODE>
__device__ __forceinline__ int logical_chunk(int row, int pc) {
    if constexpr (MODE == 1) return pc ^ swz<ROWB>(row);
    if constexpr (MODE == 2) return (((pc >> 2) ^ swz64<ROWB>(row)) << 2) | (pc & 3);
    if constexpr (MODE == 3) return dual_chunk<ROWB>(row, pc);
    return pc;
}

typedef __attribute__((address_space(1))) const void gptr_t;
typedef __attribute__((address_space(3))) void lptr_t;

// One wavefront-wide 1 KiB copy global -> LDS without passing through registers: lane i's 16 bytes land at
// lds_block + 16*i (lds_block must be wavefront-uniform).
//
// The copies are written as inline asm on purpose.  The compiler orders every LDS read behind every copy instruction it
// knows of (it cannot tell which LDS bytes a copy writes) and, while one is outstanding, turns all its counted waits
// into waits for everything; that would stall each tile on the copies of the next one.  Copies it does not see are
// ordered by the kernels themselves: wait_loads<N>() for this wavefront's copies, then a barrier, before any wavefront
// reads the stage.  The waits the compiler emits for loads it does know stay safe: loads complete in order, so extra
// copies in flight only make such a wait cover more than it needs to.
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
// per-lane 64-bit source address
__device__ __forceinline__ void dma16(const void* src, char* lds_block) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_address(lds_block)), "v"(src)
                 : "memory", "m0");
}
// wavefront-uniform 64-bit base + per-lane 32-bit byte offset
__device__ __forceinline__ void dma16_uniform(const void* base, uint32_t lane_off, char* lds_block) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_address(lds_block)), "v"(lane_off), "s"(base)
                 : "memory", "m0");
}
// One wavefront-wide 256-byte copy: lane i's 4 bytes from its own address land at lds_block + 4*i.
__device__ __forceinline__ void dma4(const void* src, char* lds_block) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :
                 : "s"(lds_address(lds_block)), "v"(src)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Copy a ROWS x ROWB-byte tile into LDS; row r comes from row_ptr(r) (16-byte aligned, ROWB readable bytes).
// Each wavefront issues ROWS*ROWB/4096 instructions of 1 KiB.
template <typename T, int ROWB, int ROWS, int SWZ, typename RowPtr>
__device__ __forceinline__ void dma_tile(char* tile, int wave, int lane, RowPtr row_ptr) {
    constexpr int NI = ROWS * ROWB / 1024;  // wavefront instructions per tile
    constexpr int CPR = ROWB / 16;          // chunks per row
    static_assert(NI % 4 == 0 && (1024 % ROWB == 0 || ROWB % 1024 == 0), "tile shape");
#pragma unroll
    for (int i = 0; i < NI / 4; ++i) {
        const int q = wave + 4 * i;
        const int flat = q * 64 + lane;  // chunk position in the tile
        const int row = flat / CPR, pc = flat % CPR;
        const int c = logical_chunk<ROWB, SWZ>(row, pc);
        dma16(reinterpret_cast<const char*>(row_ptr(row)) + c * 16, tile + q * 1024);
    }
}

// K fragment (8 consecutive contraction values of row `row`) from a swizzled row-major tile.
template <typename T, int ROWB>
__device__ __forceinline__ Frag<T> lds_frag_row_swz(const char* tile, int row, int elem_col) {
    Frag<T> f;
    if constexpr (sizeof(T) == 2) {
        u32x4 r = *reinterpret_cast<const u32x4*>(tile + lds_off<ROWB, true>(row, elem_col * 2));
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    } else {
        u32x4 r0 = *reinterpret_cast<const u32x4*>(tile + lds_off<ROWB, true>(row, elem_col * 4));
        u32x4 r1 = *reinterpret_cast<const u32x4*>(tile + lds_off<ROWB, true>(row, elem_col * 4 + 16));
        u32x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    }
    return f;
}

typedef __attribute__((address_space(3))) const u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) const float lds_f32;

__device__ __forceinline__ u32x4 lds_load128(uint32_t addr) { return *reinterpret_cast<lds_u32x4*>((uintptr_t)addr); }
__device__ __forceinline__ s16x4 lds_load_tr16(uint32_t addr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>((uintptr_t)addr));
}
__device__ __forceinline__ float lds_load_f32(uint32_t addr) { return *reinterpret_cast<lds_f32*>((uintptr_t)addr); }

// Wait until at most N of this wavefront's global loads (LDS-DMA copies included) are outstanding.
template <int N>
__device__ __forceinline__ void wait_loads() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace splat
