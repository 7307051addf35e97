// Kernel arguments of the SDDMM kernels (sddmm.hip: every shape; sddmm_lines.hip: 16-bit types, d = 64 / 128).
#pragma once
#include "acsr_plan.hpp"

namespace splat {

struct SddmmParams {
    const void* q;
    const void* k;
    void* out;
    int64_t q_sb, q_sh, q_sl;
    int64_t k_sb, k_sh, k_sd, k_sl;
    int B, H, L, n_keys, d, T;
    float scale;
    const float* row_lse;  // optional [B*H, L]: the output is exp(scale * score - row_lse[row]) instead of scale * score
    int out_dtype;
    int n_seg;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];
    int n_row_blocks, total;
    int q_vec, k_vec;  // 16-byte loads are legal for q / k
    int out_vec;       // 16-bit outputs: every row's segment starts on a 16-byte boundary
    int row_stride;
    int key_split;  // workgroups per row block: each takes a contiguous share of every segment's tiles
    const PlanRec* plan;  // optional: the mask's plan table for 128-row blocks (variant for row-major K), else nullptr
};

// Launches the line-wise kernel when the problem has its shape (see sddmm_lines.hip); returns 1 when it did, 0 when the
// general kernel has to run, a negative code on errors.  `p` is complete except for key_split / total.
int launch_sddmm_lines(const char* who, const SddmmParams& p, int in_dtype, hipStream_t st);

}  // namespace splat
