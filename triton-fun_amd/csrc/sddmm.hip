// SDDMM on ACSR: out[bh, r, off + s] = scale * <q[bh, r, :], K[bh, c(r, s), :]> for the live slots only.
//
// A workgroup of 4 wavefronts owns 128 consecutive rows of one (batch, head); wavefront w owns rows
// 32w..32w+31.  The key positions its rows' spans cover are walked in tiles of 64 (see acsr_plan.hpp);
// K is staged through LDS in chunks of 64 contraction values, Q fragments stay in registers when the
// head dimension is <= 128 and are re-read from cache otherwise.  Scores are produced with 32x32x16
// MFMA in the orientation rows = queries, columns = keys, so that the 32 lanes of a half-wavefront hold
// 32 consecutive key positions of one row: with a uniform plan these are consecutive compressed slots
// and every store instruction writes two contiguous runs.  Dead positions are never stored.
// The kernel is bound by the compressed output (HBM), not by MFMA: 2*d flops per 2-4 output bytes.
#include "acsr_plan.hpp"

namespace splat {

constexpr int kDC = 64;  // contraction values per LDS chunk

struct SddmmParams {
    const void* q;
    const void* k;
    void* out;
    int64_t q_sb, q_sh, q_sl;
    int64_t k_sb, k_sh, k_sd, k_sl;
    int B, H, L, n_keys, d, T;
    float scale;
    int out_dtype;
    int n_seg;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];
    int n_row_blocks, total;
    int q_vec, k_vec;  // 16-byte loads are legal for q / k
    int row_stride;
};

// 8 consecutive contraction values of one row from global memory, zero beyond `d`.
template <typename T>
__device__ __forceinline__ Frag<T> load_q_frag(const T* row, int k0, int d, bool vec) {
    Frag<T> f;
    if (vec && k0 + 8 <= d) return global_frag<T>(row + k0);
#pragma unroll
    for (int e = 0; e < 8; ++e) f.v[e] = (k0 + e < d) ? row[k0 + e] : (T)0.f;
    return f;
}

template <typename T, bool KT, bool QREG>
__global__ __launch_bounds__(256) void sddmm_kernel(const SddmmParams p) {
    constexpr int ES = sizeof(T);
    constexpr int BM = 128;
    constexpr int NT = kBN / 32;
    constexpr int KSC = kDC / 16;                                       // MFMA steps per chunk
    constexpr int K_ROW = KT ? (kBN * ES + 64) : (kDC * ES + 16);       // bytes per LDS row
    constexpr int K_ROWS = KT ? kDC : kBN;
    constexpr int EPC = 16 / ES;
    constexpr int CPT = kBN * kDC * ES / 16 / 256;                      // 16-byte chunks per thread
    constexpr int CR = KT ? (kBN * ES / 16) : (kDC * ES / 16);          // chunks per LDS row
    constexpr int QF = QREG ? 8 : 1;

    __shared__ __attribute__((aligned(16))) char s_k[K_ROW * K_ROWS];
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ SegPtrs s_seg[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int bh = logical / p.n_row_blocks;
    const int rb = logical % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L, d = p.d;

    const T* qb = (const T*)p.q + b * p.q_sb + h * p.q_sh;
    const T* kb = (const T*)p.k + b * p.k_sb + h * p.k_sh;

    if (tid == 0) {
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) s_seg[k] = p.seg[k];
    }
    plan_segments<BM>(p.seg, p.n_seg, r0, rs, L, !KT, s_plan, &s_ps, tid);

    // A-operand rows of this lane: query row 32*wave + lm of the block
    const int q_row = min(r0 + rs * (32 * wave + lm), L - 1);
    const T* qr = qb + (int64_t)q_row * p.q_sl;
    Frag<T> qf[QF];
    if constexpr (QREG) {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = load_q_frag<T>(qr, 16 * ks + 8 * g, d, p.q_vec != 0);
    }
    const int n_chunks = (d + kDC - 1) / kDC;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        const SegPlan pl = s_plan[sg];
        if (pl.n_tiles == 0) continue;
        const int off = s_seg[sg].slot_offset;
        // the 16 output rows this lane holds (acc_row(j, g)), and the wavefront's span in positions
        RowWin win[16];
        int lmin = 0x3fffffff, hmax = -0x3fffffff;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            win[j] = make_row_win(cached_row_map<BM>(&s_ps, sg, 32 * wave + acc_row(j, g)), pl);
            if (win[j].cnt > 0) {
                lmin = min(lmin, win[j].lo);
                hmax = max(hmax, win[j].lo + win[j].cnt);
            }
        }
        lmin = wave_min_i(lmin);
        hmax = wave_max_i(hmax);

        for (int tile = 0; tile < pl.n_tiles; ++tile) {
            const int j0 = tile * kBN;
            const bool skip = (j0 + kBN <= lmin) || (j0 >= hmax);  // wavefront-uniform
            f32x16 acc[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[nt][j] = 0.f;

            // with Q in registers (d <= 128) the chunk loop has at most 2 trips and is fully unrolled, so that
            // the register array qf is only ever indexed by constants
#pragma unroll
            for (int ch = 0; ch < (QREG ? 2 : n_chunks); ++ch) {
                if (QREG && ch >= n_chunks) break;
                const int kd0 = ch * kDC;
                __syncthreads();  // previous chunk fully consumed
                // ---- stage the K chunk: positions j0..j0+63, contraction values kd0..kd0+63 ----
#pragma unroll
                for (int i = 0; i < CPT; ++i) {
                    const int idx = tid + 256 * i;
                    const int row = idx / CR, cc = idx % CR;
                    u32x4 val = {0u, 0u, 0u, 0u};
                    if constexpr (KT) {
                        // LDS row = contraction index, columns = key positions (dense walk, cs == 1)
                        const int kd = kd0 + row;
                        const int c = pl.c0 + j0 + cc * EPC;
                        if (kd < d) {
                            const T* src = kb + (int64_t)kd * p.k_sd;
                            if (p.k_vec && c + EPC <= p.n_keys) {
                                val = *reinterpret_cast<const u32x4*>(src + c);
                            } else {
                                T tmp[EPC];
#pragma unroll
                                for (int e = 0; e < EPC; ++e) tmp[e] = (c + e < p.n_keys) ? src[(int64_t)(c + e) * p.k_sl] : (T)0.f;
                                __builtin_memcpy(&val, tmp, 16);
                            }
                        }
                    } else {
                        const int n = min(max(pl.c0 + pl.cs * (j0 + row), 0), p.n_keys - 1);
                        const T* src = kb + (int64_t)n * p.k_sl;
                        const int kd = kd0 + cc * EPC;
                        if (p.k_vec && kd + EPC <= d) {
                            val = *reinterpret_cast<const u32x4*>(src + kd);
                        } else {
                            T tmp[EPC];
#pragma unroll
                            for (int e = 0; e < EPC; ++e) tmp[e] = (kd + e < d) ? src[(int64_t)(kd + e) * p.k_sd] : (T)0.f;
                            __builtin_memcpy(&val, tmp, 16);
                        }
                    }
                    *reinterpret_cast<u32x4*>(s_k + row * K_ROW + cc * 16) = val;
                }
                __syncthreads();
                if (skip) continue;
#pragma unroll
                for (int ks = 0; ks < KSC; ++ks) {
                    Frag<T> a;
                    if constexpr (QREG)
                        a = qf[(ch * KSC + ks) & 7];
                    else
                        a = load_q_frag<T>(qr, kd0 + 16 * ks + 8 * g, d, p.q_vec != 0);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        Frag<T> kf;
                        if constexpr (KT)
                            kf = lds_frag_cols<T>(s_k, K_ROW, 16 * ks + 8 * g, 16 * ks + 8 * g + 4, 32 * nt, lane);
                        else
                            kf = lds_frag_rowmajor<T>(s_k + (32 * nt + lm) * K_ROW + (16 * ks + 8 * g) * ES);
                        mma32(acc[nt], a, kf);
                    }
                }
            }
            if (skip) continue;
            // ---- scatter the live positions to their compressed slots ----
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int r = r0 + rs * (32 * wave + acc_row(j, g));
                const int64_t row_base = ((int64_t)bh * L + r) * p.T + off;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int jj = j0 + 32 * nt + lm;
                    if (win_live(win[j], jj)) store_as(p.out, row_base + win_slot(win[j], jj), acc[nt][j] * p.scale, p.out_dtype);
                }
            }
        }
    }
}

template <typename T>
static int launch_sddmm(SddmmParams p, bool kt, hipStream_t st) {
    p.n_row_blocks = count_row_blocks(p.L, 128, p.row_stride);
    p.total = p.B * p.H * p.n_row_blocks;
    const int grid = ((p.total + 7) / 8) * 8;
    const bool qreg = p.d <= 128;
    if (kt) {
        if (qreg)
            sddmm_kernel<T, true, true><<<grid, 256, 0, st>>>(p);
        else
            sddmm_kernel<T, true, false><<<grid, 256, 0, st>>>(p);
    } else {
        if (qreg)
            sddmm_kernel<T, false, true><<<grid, 256, 0, st>>>(p);
        else
            sddmm_kernel<T, false, false><<<grid, 256, 0, st>>>(p);
    }
    return check_launch("splat_sddmm");
}

}  // namespace splat

using namespace splat;

extern "C" int splat_sddmm(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb, int64_t k_sh,
                           int64_t k_sd, int64_t k_sl, void* out, const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H,
                           int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype, int32_t out_dtype,
                           void* stream) {
    if (!q || !kT || !out || !segs) return fail(SPLAT_E_NULL, "splat_sddmm: null pointer argument");
    if (B <= 0 || H <= 0 || L <= 0 || n_keys <= 0 || d <= 0 || T <= 0)
        return fail(SPLAT_E_SHAPE, "splat_sddmm: need B, H, L, n_keys, d, T > 0 (got %d, %d, %d, %d, %d, %d)", B, H, L, n_keys, d, T);
    if (L > (1 << 23) || n_keys > (1 << 23)) return fail(SPLAT_E_SHAPE, "splat_sddmm: L and n_keys are limited to 2^23");
    if (out_dtype != SPLAT_F32 && out_dtype != SPLAT_F16 && out_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "splat_sddmm: unknown out_dtype %d", out_dtype);
    if (in_dtype != SPLAT_F32 && in_dtype != SPLAT_F16 && in_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "splat_sddmm: unknown in_dtype %d", in_dtype);
    if (k_sd != 1 && k_sl != 1)
        return fail(SPLAT_E_ALIGN, "splat_sddmm: kT needs unit stride along d (k_sd == 1) or along keys (k_sl == 1); got k_sd=%lld k_sl=%lld",
                    (long long)k_sd, (long long)k_sl);
    SddmmParams p;
    p.q = q; p.k = kT; p.out = out;
    p.q_sb = q_sb; p.q_sh = q_sh; p.q_sl = q_sl;
    p.k_sb = k_sb; p.k_sh = k_sh; p.k_sd = k_sd; p.k_sl = k_sl;
    p.B = B; p.H = H; p.L = L; p.n_keys = n_keys; p.d = d; p.T = T;
    p.scale = scale;
    p.out_dtype = out_dtype;
    p.n_seg = n_seg;
    if (int rc = fill_segs("splat_sddmm", segs, n_seg, p.seg, T)) return rc;
    p.row_stride = common_row_stride(segs, n_seg);
    const int es = in_dtype == SPLAT_F32 ? 4 : 2;
    const int epc = 16 / es;
    auto al = [&](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    auto mul = [&](int64_t s) { return (s % epc) == 0; };
    // rows of K contiguous ([.., keys, d] memory) unless only the key stride is 1
    const bool kt = !(k_sd == 1);
    p.q_vec = (al(q) && mul(q_sb) && mul(q_sh) && mul(q_sl)) ? 1 : 0;
    p.k_vec = (al(kT) && mul(k_sb) && mul(k_sh) && mul(kt ? k_sd : k_sl)) ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    switch (in_dtype) {
        case SPLAT_F32: return launch_sddmm<float>(p, kt, st);
        case SPLAT_F16: return launch_sddmm<f16>(p, kt, st);
        default: return launch_sddmm<bf16>(p, kt, st);
    }
}
