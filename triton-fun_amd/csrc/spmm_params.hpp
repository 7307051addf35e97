// Kernel arguments of the SpMM kernels (spmm.hip: every shape; spmm_thin.hip: 16-bit types, 64 / 128 output columns).
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

}  // namespace splat
