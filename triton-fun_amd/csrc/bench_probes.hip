// Measurement aids (libsplat_bench.so, declared in include/splat_bench.h): nothing here is on the operator path.
//
//  * splat_bench_stream_copy: a plain copy with the access forms of the HBM-bound kernels (16 bytes per lane,
//    non-temporal, several requests in flight): the read + write streaming ceiling the row softmax is quoted against.
//  * splat_bench_mfma_lds_probe: the matrix work of the fused forward's tile loop with nothing else around it, in several
//    shapes.  Every wavefront runs, per 64-key tile at d = 128 in bf16, exactly the LDS fragment reads and MFMAs of both
//    products (scores, then output); no global loads in the loop, no copies into LDS, no exponentials, no barriers.  The
//    LDS holds the caller's data (random values give the switching activity of real operands; zeros do not).  What such
//    a loop sustains is what the chip can give any kernel of that shape: on a part that runs into its power limit the
//    clock drops under it, so the figure lies below the rated peak, which is quoted at the full clock.
//      shape 0: 32 x 32 x 16 MFMA, 32 query rows per wavefront, 2 wavefronts per SIMD (the fused forward's shape):
//               every MFMA takes a fresh 1 KiB fragment from LDS;
//      shape 1: 32 x 32 x 16 MFMA, 64 query rows per wavefront, 1 wavefront per SIMD: every fragment feeds two MFMAs,
//               half the LDS bytes per FLOP;
//      shape 2: 16 x 16 x 32 MFMA, 16 query rows per wavefront, 4 wavefronts per SIMD (128 registers): twice the LDS
//               bytes per FLOP, twice the wavefronts to hide latency with.
#include "../../include/splat_bench.h"
#include "tile_copy.hpp"

namespace splat {

typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int kPD = 128, kPBN = 64, kPROWB = kPD * 2, kPKB = kPBN * kPROWB, kPSTAGE = 2 * kPKB;

// shapes 0 and 1: RT = 32-row tiles per wavefront (1 or 2)
template <int RT>
__global__ __launch_bounds__(256, RT == 1 ? 2 : 1) void mfma_lds_probe_kernel(const bf16* data, float* out, int tiles) {
    constexpr int D = kPD, KS = D / 16, DT = D / 32, NT = kPBN / 32, ROWB = kPROWB, KBYTES = kPKB, STAGE = kPSTAGE;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, lm = lane & 31, g = lane >> 5;
    // two stages of (K tile, V tile) from the caller's 64 KiB
    for (int i = tid; i < 2 * STAGE / 16; i += 256)
        reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(data)[i];
    Frag<bf16> qf[RT][KS];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[r][ks] = global_frag<bf16>(data + ((tid + 37 * r) & 127) * D + 16 * ks + 8 * g);
    __syncthreads();
    const uint32_t smem_base = lds_address(smem);
    const int tr_row = (lane & 15) >> 2, tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t k_addr[KS], v_addr[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        v_addr[dt] = smem_base + KBYTES + (4 * g + tr_row) * ROWB + ((dt ^ swz64<ROWB>(4 * g + tr_row)) * 64) + tr_col * 2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = smem_base + lds_off<ROWB, true>(lm, (16 * ks + 8 * g) * 2);
    f32x16 o_acc[RT][DT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 16; ++j) o_acc[r][dt][j] = 0.f;
    int stage = 0;
    for (int it = 0; it < tiles; ++it) {
        f32x16 s_acc[RT][NT];
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 16; ++j) s_acc[r][nt][j] = 0.f;
        constexpr int NFR = NT * KS, K_AHEAD = 12;
        Frag<bf16> kfr[NFR];
        auto load_k = [&](int i) {
            Frag<bf16> kf;
            kf.v = __builtin_bit_cast(typename Frag<bf16>::vec, lds_load128(k_addr[i % KS] + 32 * (i / KS) * ROWB));
            return kf;
        };
#pragma unroll
        for (int i = 0; i < K_AHEAD; ++i) kfr[i] = load_k(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NFR; ++i) {
#pragma unroll
            for (int r = 0; r < RT; ++r) mma32(s_acc[r][i / KS], kfr[i], qf[r][i % KS]);
            if (i + K_AHEAD < NFR) {
                kfr[i + K_AHEAD] = load_k(i + K_AHEAD);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // scores to 16-bit operands of the second product, scaled so that the values stay of order one
        Frag<bf16> pf[RT][NT][2];
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 16; ++j) pf[r][nt][j >> 3].v[j & 7] = (bf16)(s_acc[r][nt][j] * 0.0884f);
        auto load_v = [&](int nt, int t, int dt) {
            const uint32_t a0 = v_addr[dt] + (32 * nt + 16 * t) * ROWB;
            return frag_from_tr<bf16>(lds_load_tr16(a0), lds_load_tr16(a0 + 8 * ROWB));
        };
        Frag<bf16> vfr[2][DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vfr[0][dt] = load_v(0, 0, dt);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 2 * NT; ++step) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int r = 0; r < RT; ++r) mma32(o_acc[r][dt], vfr[step & 1][dt], pf[r][step >> 1][step & 1]);
                if (step + 1 < 2 * NT) {
                    vfr[(step + 1) & 1][dt] = load_v((step + 1) >> 1, (step + 1) & 1, dt);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        stage ^= 1;
        const int delta = stage == 0 ? -STAGE : STAGE;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_addr[dt] += delta;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) k_addr[ks] += delta;
    }
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 16; ++j) sum += o_acc[r][dt][j];
    out[(int64_t)blockIdx.x * blockDim.x + tid] = sum;
}

// shape 2: 16 query rows per wavefront, 16 x 16 x 32 MFMA, 8 wavefronts per workgroup, 4 per SIMD.  K fragments: lane
// (key row i = lane % 16, g = lane / 16) reads the 16 bytes at d = 32 ks + 8 g of row 16 blk + i.  V^T fragments: lane s
// of 16-lane block g addresses key row 4 g + s / 4 and 4 elements at d = 16 db + 4 (s % 4) through the transposing read,
// and again 16 rows on; the 32-byte halves of a 64-byte block swap places for odd g so that the 16 rows a read touches
// spread over all banks.  The exponentials' results sit where the second product's B operand wants them: slots 0..3 of
// a 32-key step from score block 2t, slots 4..7 from block 2t + 1.
__global__ __launch_bounds__(512, 4) void mfma_lds_probe_thin_kernel(const bf16* data, float* out, int tiles) {
    constexpr int D = kPD, ROWB = kPROWB, KBYTES = kPKB, STAGE = kPSTAGE;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, g = lane >> 4;
    for (int i = tid; i < 2 * STAGE / 16; i += 512)
        reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(data)[i];
    Frag<bf16> qf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = global_frag<bf16>(data + (tid & 127) * D + 32 * ks + 8 * g);
    __syncthreads();
    const uint32_t smem_base = lds_address(smem);
    uint32_t k_addr[4], v_addr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) k_addr[ks] = smem_base + li * ROWB + (((4 * ks + g) ^ li) << 4);
    {
        const int row = 4 * g + (li >> 2);
#pragma unroll
        for (int dp = 0; dp < 4; ++dp) v_addr[dp] = smem_base + KBYTES + row * ROWB + ((dp ^ (row & 3)) * 64) + (4 * (li & 3)) * 2;
    }
    const uint32_t v_half = (g & 1) * 32;
    f32x4v o_acc[8];
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) o_acc[db][j] = 0.f;
    auto mma16 = [](f32x4v& acc, const Frag<bf16>& a, const Frag<bf16>& b) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
    };
    int stage = 0;
    for (int it = 0; it < tiles; ++it) {
        f32x4v s_acc[4];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int j = 0; j < 4; ++j) s_acc[blk][j] = 0.f;
        constexpr int K_AHEAD = 8, V_AHEAD = 4;
        Frag<bf16> kfr[16];
        auto load_k = [&](int i) {  // i = 4 blk + ks
            Frag<bf16> kf;
            kf.v = __builtin_bit_cast(typename Frag<bf16>::vec, lds_load128(k_addr[i & 3] + 16 * (i >> 2) * ROWB));
            return kf;
        };
#pragma unroll
        for (int i = 0; i < K_AHEAD; ++i) kfr[i] = load_k(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            mma16(s_acc[i >> 2], kfr[i], qf[i & 3]);
            if (i + K_AHEAD < 16) {
                kfr[i + K_AHEAD] = load_k(i + K_AHEAD);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        Frag<bf16> pf[2];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int j = 0; j < 4; ++j) pf[blk >> 1].v[4 * (blk & 1) + j] = (bf16)(s_acc[blk][j] * 0.0884f);
        auto load_v = [&](int t, int db) {
            const uint32_t a0 = (v_addr[db >> 1] + (((db & 1) * 32) ^ v_half)) + 32 * t * ROWB;
            return frag_from_tr<bf16>(lds_load_tr16(a0), lds_load_tr16(a0 + 16 * ROWB));
        };
        Frag<bf16> vfr[16];
#pragma unroll
        for (int i = 0; i < V_AHEAD; ++i) vfr[i] = load_v(i >> 3, i & 7);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; ++i) {  // i = 8 t + db
            mma16(o_acc[i & 7], vfr[i], pf[i >> 3]);
            if (i + V_AHEAD < 16) {
                vfr[i + V_AHEAD] = load_v((i + V_AHEAD) >> 3, (i + V_AHEAD) & 7);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        stage ^= 1;
        const int delta = stage == 0 ? -STAGE : STAGE;
#pragma unroll
        for (int dp = 0; dp < 4; ++dp) v_addr[dp] += delta;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) k_addr[ks] += delta;
    }
    float sum = 0.f;
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) sum += o_acc[db][j];
    out[(int64_t)blockIdx.x * blockDim.x + tid] = sum;
}

// The fused forward's tile loop at d = 64 with its exponentials: per 64-key tile both products out of LDS tiles and, per
// score, one multiply-add, one exponential, one add into the row sum and one conversion (what the kernel's loop does once
// every row has its reference); a workgroup barrier per tile, no loads, no masks.  Two shapes: 32 query rows per wavefront
// (32 x 32 x 16 MFMA, 4 wavefronts per workgroup) and 16 (16 x 16 x 32 MFMA, 8 wavefronts per workgroup), both launched
// with 53 KiB of LDS so that three workgroups share a compute unit (3 and 6 wavefronts per SIMD).
constexpr int kSD = 64, kSROWB = kSD * 2, kSKB = kPBN * kSROWB, kSSTAGE = 2 * kSKB, kSLDS = 53 * 1024;

template <bool EXP>
__global__ __launch_bounds__(256, 3) void softmax_loop_probe_wide_kernel(const bf16* data, float* out, int tiles) {
    constexpr int KS = kSD / 16, DT = kSD / 32, NT = kPBN / 32;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, lm = lane & 31, g = lane >> 5;
    for (int i = tid; i < 2 * kSSTAGE / 16; i += 256) reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(data)[i];
    Frag<bf16> qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag<bf16>(data + (tid & 127) * kSD + 16 * ks + 8 * g);
    __syncthreads();
    const uint32_t smem_base = lds_address(smem);
    const int tr_row = (lane & 15) >> 2, tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t k_addr[KS], v_addr[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        v_addr[dt] = smem_base + kSKB + (4 * g + tr_row) * kSROWB + ((dt ^ swz64<kSROWB>(4 * g + tr_row)) * 64) + tr_col * 2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = smem_base + lds_off<kSROWB, true>(lm, (16 * ks + 8 * g) * 2);
    f32x16 o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) o_acc[dt][j] = 0.f;
    float l_run = 0.f;
    const float m2 = 3.0f + 0.01f * lane;
    int stage = 0;
    for (int it = 0; it < tiles; ++it) {
        __syncthreads();  // (where the real loop hands a stage over)
        f32x16 s_acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 16; ++j) s_acc[nt][j] = 0.f;
        constexpr int NFR = NT * KS;
        Frag<bf16> kfr[NFR];
#pragma unroll
        for (int i = 0; i < NFR; ++i)
            kfr[i].v = __builtin_bit_cast(typename Frag<bf16>::vec, lds_load128(k_addr[i % KS] + 32 * (i / KS) * kSROWB));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NFR; ++i) mma32(s_acc[i / KS], kfr[i], qf[i % KS]);
        Frag<bf16> pf[NT][2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                float pv;
                if (EXP) {
                    pv = fast_exp2(fmaf(s_acc[nt][j], 0.18f, -m2));
                    l_run += pv;
                } else {
                    pv = s_acc[nt][j] * 0.0884f;
                }
                pf[nt][j >> 3].v[j & 7] = (bf16)pv;
            }
        auto load_v = [&](int nt, int t, int dt) {
            const uint32_t a0 = v_addr[dt] + (32 * nt + 16 * t) * kSROWB;
            return frag_from_tr<bf16>(lds_load_tr16(a0), lds_load_tr16(a0 + 8 * kSROWB));
        };
        Frag<bf16> vfr[2][DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vfr[0][dt] = load_v(0, 0, dt);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 2 * NT; ++step) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                mma32(o_acc[dt], vfr[step & 1][dt], pf[step >> 1][step & 1]);
                if (step + 1 < 2 * NT) {
                    vfr[(step + 1) & 1][dt] = load_v((step + 1) >> 1, (step + 1) & 1, dt);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        stage ^= 1;
        const int delta = stage == 0 ? -kSSTAGE : kSSTAGE;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_addr[dt] += delta;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) k_addr[ks] += delta;
    }
    float sum = l_run;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) sum += o_acc[dt][j];
    out[(int64_t)blockIdx.x * blockDim.x + tid] = sum;
}

template <bool EXP>
__global__ __launch_bounds__(512, 6) void softmax_loop_probe_thin_kernel(const bf16* data, float* out, int tiles) {
    constexpr int KS = kSD / 32, DB = kSD / 16;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, g = lane >> 4;
    for (int i = tid; i < 2 * kSSTAGE / 16; i += 512) reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(data)[i];
    Frag<bf16> qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag<bf16>(data + (tid & 127) * kSD + 32 * ks + 8 * g);
    __syncthreads();
    const uint32_t smem_base = lds_address(smem);
    uint32_t k_addr[KS], v_addr[kSD / 32];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = smem_base + li * kSROWB + (((4 * ks + g) ^ (li & 7)) << 4);
    {
        const int row = 4 * g + (li >> 2);
#pragma unroll
        for (int dp = 0; dp < kSD / 32; ++dp) v_addr[dp] = smem_base + kSKB + row * kSROWB + ((dp ^ (row & 1)) * 64) + (4 * (li & 3)) * 2;
    }
    const uint32_t v_half = (g & 1) * 32;
    f32x4v o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) o_acc[db][j] = 0.f;
    float l_run = 0.f;
    const float m2 = 3.0f + 0.01f * lane;
    int stage = 0;
    for (int it = 0; it < tiles; ++it) {
        __syncthreads();  // (where the real loop hands a stage over)
        f32x4v s_acc[4];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int j = 0; j < 4; ++j) s_acc[blk][j] = 0.f;
        constexpr int NFR = 4 * KS;
        Frag<bf16> kfr[NFR];
#pragma unroll
        for (int i = 0; i < NFR; ++i)  // i = KS blk + ks
            kfr[i].v = __builtin_bit_cast(typename Frag<bf16>::vec, lds_load128(k_addr[i % KS] + 16 * (i / KS) * kSROWB));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NFR; ++i) mma16(s_acc[i / KS], kfr[i], qf[i % KS]);
        Frag<bf16> pf[2];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float pv;
                if (EXP) {
                    pv = fast_exp2(fmaf(s_acc[blk][j], 0.18f, -m2));
                    l_run += pv;
                } else {
                    pv = s_acc[blk][j] * 0.0884f;
                }
                pf[blk >> 1].v[4 * (blk & 1) + j] = (bf16)pv;
            }
        auto load_v = [&](int t, int db) {
            const uint32_t a0 = (v_addr[db >> 1] + (((db & 1) * 32) ^ v_half)) + 32 * t * kSROWB;
            return frag_from_tr<bf16>(lds_load_tr16(a0), lds_load_tr16(a0 + 16 * kSROWB));
        };
        Frag<bf16> vfr[2 * DB];
#pragma unroll
        for (int i = 0; i < 2 * DB; ++i) vfr[i] = load_v(i / DB, i % DB);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2 * DB; ++i) mma16(o_acc[i % DB], vfr[i], pf[i / DB]);
        stage ^= 1;
        const int delta = stage == 0 ? -kSSTAGE : kSSTAGE;
#pragma unroll
        for (int dp = 0; dp < kSD / 32; ++dp) v_addr[dp] += delta;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) k_addr[ks] += delta;
    }
    float sum = l_run;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) sum += o_acc[db][j];
    out[(int64_t)blockIdx.x * blockDim.x + tid] = sum;
}

// The streaming ceiling the HBM-bound kernels are held against: a plain copy with the loads and stores the row softmax
// uses (16 bytes per lane, non-temporal, four requests in flight per lane), workgroups striding over the buffer.
__global__ __launch_bounds__(256) void stream_copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
    constexpr int UNROLL = 4;
    int64_t chunk = (int64_t)blockIdx.x * (UNROLL * 256);
    const int64_t stride = (int64_t)gridDim.x * (UNROLL * 256);
    for (; chunk + UNROLL * 256 <= n16; chunk += stride) {
        u32x4 r[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) r[u] = __builtin_nontemporal_load(src + chunk + u * 256 + threadIdx.x);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(r[u], dst + chunk + u * 256 + threadIdx.x);
    }
    // the tail that does not fill a whole chunk
    const int64_t n_full = n16 / (UNROLL * 256) * (UNROLL * 256);
    if (blockIdx.x == 0)
        for (int64_t i = n_full + threadIdx.x; i < n16; i += 256) dst[i] = src[i];
}

}  // namespace splat

using namespace splat;

extern "C" int splat_bench_version(void) { return SPLAT_BENCH_VERSION; }
extern "C" const char* splat_bench_last_error(void) { return splat_last_error(); }

extern "C" int splat_bench_stream_copy(const void* src, void* dst, int64_t bytes, void* stream) {
    begin_launch();
    if (!src || !dst) return fail(SPLAT_E_NULL, "splat_bench_stream_copy: null pointer argument");
    if (bytes <= 0 || (bytes & 15) != 0) return fail(SPLAT_E_SHAPE, "splat_bench_stream_copy: bytes must be a positive multiple of 16 (got %lld)", (long long)bytes);
    if (((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) != 0)
        return fail(SPLAT_E_ALIGN, "splat_bench_stream_copy: src and dst must be 16-byte aligned");
    stream_copy_kernel<<<8192, 256, 0, (hipStream_t)stream>>>(static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), bytes / 16);
    return check_launch("splat_bench_stream_copy");
}

extern "C" int64_t splat_bench_mfma_lds_probe_flops(int32_t shape, int32_t workgroups, int32_t tiles) {
    // per wavefront and tile: 2 products x 64 keys x rows x 128 x 2
    const int64_t rows_per_wg = shape == 1 ? 256 : 128;
    if (shape < 0 || shape > 2) return 0;
    return (int64_t)workgroups * tiles * rows_per_wg * 2 * 64 * 128 * 2;
}

extern "C" int splat_bench_mfma_lds_probe(const void* data, int64_t data_bytes, void* out, int64_t out_bytes, int32_t shape,
                                          int32_t workgroups, int32_t tiles, void* stream) {
    begin_launch();
    const char* who = "splat_bench_mfma_lds_probe";
    if (!data || !out) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (shape < 0 || shape > 2) return fail(SPLAT_E_UNSUPPORTED, "%s: shape must be 0, 1 or 2 (got %d)", who, shape);
    if (workgroups < 1 || workgroups > (1 << 20) || tiles < 1 || tiles > (1 << 20))
        return fail(SPLAT_E_SHAPE, "%s: workgroups and tiles must be 1..2^20 (got %d, %d)", who, workgroups, tiles);
    if (data_bytes < 65536) return fail(SPLAT_E_SHAPE, "%s: data must hold 65536 bytes (got %lld)", who, (long long)data_bytes);
    const int threads = shape == 2 ? 512 : 256;
    if (out_bytes < (int64_t)workgroups * threads * 4)
        return fail(SPLAT_E_SHAPE, "%s: out must hold %d bytes per workgroup (got %lld for %d)", who, threads * 4, (long long)out_bytes, workgroups);
    if ((reinterpret_cast<uintptr_t>(data) & 15) != 0 || (reinterpret_cast<uintptr_t>(out) & 3) != 0)
        return fail(SPLAT_E_ALIGN, "%s: data must be 16-byte aligned, out 4-byte aligned", who);
    const bf16* d = static_cast<const bf16*>(data);
    float* o = static_cast<float*>(out);
    hipStream_t st = (hipStream_t)stream;
    static uint64_t reserved[3] = {0, 0, 0};
    if (shape == 0) {
        if (int rc = reserve_dynamic_lds(&reserved[0], (const void*)mfma_lds_probe_kernel<1>, 65536, who)) return rc;
        mfma_lds_probe_kernel<1><<<workgroups, 256, 65536, st>>>(d, o, tiles);
    } else if (shape == 1) {
        if (int rc = reserve_dynamic_lds(&reserved[1], (const void*)mfma_lds_probe_kernel<2>, 65536, who)) return rc;
        mfma_lds_probe_kernel<2><<<workgroups, 256, 65536, st>>>(d, o, tiles);
    } else {
        if (int rc = reserve_dynamic_lds(&reserved[2], (const void*)mfma_lds_probe_thin_kernel, 65536, who)) return rc;
        mfma_lds_probe_thin_kernel<<<workgroups, 512, 65536, st>>>(d, o, tiles);
    }
    return check_launch(who);
}

extern "C" int64_t splat_bench_softmax_loop_probe_flops(int32_t workgroups, int32_t tiles) {
    return (int64_t)workgroups * tiles * 128 * 2 * 64 * kSD * 2;
}

extern "C" int splat_bench_softmax_loop_probe(const void* data, int64_t data_bytes, void* out, int64_t out_bytes, int32_t shape,
                                              int32_t exponentials, int32_t workgroups, int32_t tiles, void* stream) {
    begin_launch();
    const char* who = "splat_bench_softmax_loop_probe";
    if (!data || !out) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (shape < 0 || shape > 1) return fail(SPLAT_E_UNSUPPORTED, "%s: shape must be 0 or 1 (got %d)", who, shape);
    if (workgroups < 1 || workgroups > (1 << 20) || tiles < 1 || tiles > (1 << 20))
        return fail(SPLAT_E_SHAPE, "%s: workgroups and tiles must be 1..2^20 (got %d, %d)", who, workgroups, tiles);
    if (data_bytes < 65536) return fail(SPLAT_E_SHAPE, "%s: data must hold 65536 bytes (got %lld)", who, (long long)data_bytes);
    const int threads = shape == 1 ? 512 : 256;
    if (out_bytes < (int64_t)workgroups * threads * 4)
        return fail(SPLAT_E_SHAPE, "%s: out must hold %d bytes per workgroup (got %lld for %d)", who, threads * 4, (long long)out_bytes, workgroups);
    if ((reinterpret_cast<uintptr_t>(data) & 15) != 0 || (reinterpret_cast<uintptr_t>(out) & 3) != 0)
        return fail(SPLAT_E_ALIGN, "%s: data must be 16-byte aligned, out 4-byte aligned", who);
    const bf16* d = static_cast<const bf16*>(data);
    float* o = static_cast<float*>(out);
    hipStream_t st = (hipStream_t)stream;
    static uint64_t reserved[4] = {0, 0, 0, 0};
    auto go = [&](auto kern, uint64_t* res) -> int {
        if (int rc = reserve_dynamic_lds(res, (const void*)kern, kSLDS, who)) return rc;
        kern<<<workgroups, threads, kSLDS, st>>>(d, o, tiles);
        return 0;
    };
    int rc;
    if (shape == 0)
        rc = exponentials ? go(softmax_loop_probe_wide_kernel<true>, &reserved[0]) : go(softmax_loop_probe_wide_kernel<false>, &reserved[1]);
    else
        rc = exponentials ? go(softmax_loop_probe_thin_kernel<true>, &reserved[2]) : go(softmax_loop_probe_thin_kernel<false>, &reserved[3]);
    if (rc) return rc;
    return check_launch(who);
}
