// Kernel arguments of the SpMM kernels (spmm.hip: every shape; spmm_thin.hip, spmm_tile.hip, spmm_t_thin.hip: 16-bit types, 64 / 128
// output columns).
#pragma once
#include "acsr_plan.hpp"

namespace splat {

struct SpmmParams {
    const void* p;
    const void* v;
    void* out;
    int64_t v_sb, v_sh, v_sl;
    int B, H, L, n_keys, n_out, T;
    int out_dtype;
    int out_vec;  // 16-byte stores are legal for every row of out
    int n_seg;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];
    int n_row_blocks, total, n_col_chunks;
    int v_vec;
    int row_stride;
    const PlanRec* plan;  // optional: the mask's plan table for 128-row blocks (gathered walks), else nullptr
};

// Launches the kernel of thin wavefronts when the problem has its shape (see spmm_thin.hip); returns 1 when it did, 0
// when the general kernel has to run, a negative code on errors.  `p` is complete except for the launch geometry.
int launch_spmm_thin(const char* who, const SpmmParams& p, int in_dtype, hipStream_t st);
// The same for rows that are short or not aligned (see spmm_tile.hip; launch_spmm_thin hands them over).
int launch_spmm_tile(const char* who, const SpmmParams& p, int in_dtype, hipStream_t st);

// ---- shared by the kernels of thin wavefronts ----
// Physical 16-byte chunk of logical chunk c of V tile row `row`: the 64-byte block index is XORed with the row's low bits
// (4 consecutive rows -> the 4 quadrants of the 256-byte bank space; for 128-byte rows two rows share a quadrant pair),
// and the halves of a block swap places in every second group of 8 rows.  Its own inverse.
template <int ROWB>
__device__ __forceinline__ constexpr int v_chunk(int row, int c) {
    const int blk = ROWB >= 256 ? (row & 3) : ((row >> 1) & 1);
    return (((c >> 2) ^ blk) << 2) | ((c & 3) ^ (((row >> 3) & 1) << 1));
}

// x shifted by k 16-bit elements towards higher element indices (k >= 0) or lower ones (k < 0), zeros moving in
__device__ __forceinline__ u32x4 shift_elements(u32x4 x, int k) {
    const uint64_t lo = (uint64_t)x[0] | ((uint64_t)x[1] << 32), hi = (uint64_t)x[2] | ((uint64_t)x[3] << 32);
    uint64_t rl, rh;
    if (k >= 0) {
        const int s = 16 * k;  // 0..128
        if (s == 0) {
            rl = lo, rh = hi;
        } else if (s < 64) {
            rl = lo << s, rh = (hi << s) | (lo >> (64 - s));
        } else if (s < 128) {
            rl = 0, rh = lo << (s - 64);
        } else {
            rl = 0, rh = 0;
        }
    } else {
        const int s = -16 * k;
        if (s < 64) {
            rl = (lo >> s) | (hi << (64 - s)), rh = hi >> s;
        } else if (s < 128) {
            rl = hi >> (s - 64), rh = 0;
        } else {
            rl = 0, rh = 0;
        }
    }
    return u32x4{(uint32_t)rl, (uint32_t)(rl >> 32), (uint32_t)rh, (uint32_t)(rh >> 32)};
}

// ---- the transposed product (spmm.hip: every shape; spmm_t_thin.hip: 16-bit types, 64 / 128 output columns) ----
struct SpmmTParams {
    const void* p;   // [BH, L, T] compressed, rows of the mask
    const void* x;   // [B, H, L, n_out] by strides, unit stride along the features
    void* out;       // [BH, Lt, n_out] contiguous
    int64_t x_sb, x_sh, x_sl;
    int B, H, L, Lt, n_out, T;
    int out_dtype, out_vec, x_vec;
    int n_seg;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];    // the mask: which columns row i keeps, and where
    SegPtrs seg_t[SPLAT_MAX_SEGMENTS];  // the transposed mask: which rows column j meets
    int n_row_blocks, total, n_col_chunks;
    int row_stride;  // of the transposed mask's ACSR
    int64_t p_elems;  // elements of p
    const PlanRec* plan_t;  // optional: the plan table of the transposed mask for 128-row blocks (gathered walks), else nullptr
};

// Row i's entries seen from a block of columns first + rs*m, m = 0..127.
struct BlockRow {
    RowWin w;  // unit step (lin == 1): live iff 0 <= m - lo < cnt, slot m - lo; lin > 1 (rs == 1 only): affine test in
               // columns as in dense plans; lin == 0: the row fits neither and is tested per entry from its map
    RowMap m;
};
__device__ __forceinline__ BlockRow block_row(const RowMap& m, int first, int rs) {
    BlockRow b;
    b.m = m;
    b.w.lo = 0, b.w.cnt = 0, b.w.lin = 1;
    if (m.cnt <= 0) return b;
    const int d0 = m.a - first;
    if (rs == 1) {
        b.w.lo = d0;
        b.w.lin = (m.cnt > 1) ? m.lin : 1;
        b.w.cnt = b.w.lin * (m.cnt - 1) + 1;
    } else if ((m.cnt == 1 || m.lin == rs) && d0 % rs == 0) {
        b.w.lo = d0 / rs;
        b.w.cnt = m.cnt;
    } else {
        b.w.lin = 0;
    }
    return b;
}
// the general test: entry of the row at column j, or zero
template <typename T>
__device__ __forceinline__ T entry_at_column(const T* row, const RowMap& m, int j) {
    const int u = j - m.a;
    if (u < 0 || m.cnt <= 0) return (T)0.f;
    if (u == 0) return row[0];
    if (m.cnt == 1 || u % m.lin != 0 || u / m.lin >= m.cnt) return (T)0.f;
    return row[u / m.lin];
}

// As launch_spmm_thin, for the transposed product (see spmm_t_thin.hip).
int launch_spmm_t_thin(const char* who, const SpmmTParams& p, int in_dtype, hipStream_t st);

}  // namespace splat
