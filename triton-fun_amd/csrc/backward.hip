// Pieces of the backward pass of ACSR sparse attention that the forward kernels do not already provide.
//
// With S~ the compressed scores, P~ = softmax(S~) and O = P~ . V (rows of P~ over the live columns of the row):
//   dP~ = SDDMM(dO, V^T)                       (splat_sddmm with x = dO, y = V viewed as [d, L])
//   dS~ = P~ o (dP~ - rowsum(P~ o dP~)) * scale (splat_softmax_bwd, below)
//   dQ  = SpMM(dS~, K)                          (splat_spmm with v = K)
//   dV  = P^T . dO,  dK = dS^T . Q              (splat_spmm on the ACSR of the transposed mask, after the compressed
//                                                matrix has been brought into that ACSR's layout by
//                                                splat_compressed_transpose, below)
// The reference has no backward pass (r_attention.py:77-100 is forward only).
#include "splat_common.hpp"

namespace splat {

struct BwdSegs {
    const float* nnz[SPLAT_MAX_SEGMENTS];
    int off[SPLAT_MAX_SEGMENTS];
    int n;
};

// One wavefront per compressed row: rs = sum over the live slots of p * dp, then ds = p * (dp - rs) * scale.
// Dead slots are neither read as data nor written.  ds may alias dp.  VEC: rows are read and written as 16-byte
// pieces where a piece lies inside a segment's live range (T a multiple of the piece, 16-byte aligned bases).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const T* __restrict__ p, const T* dp, T* ds, BwdSegs segs,
                                                          int64_t n_rows, int L, int Tdim, float scale) {
    constexpr int EPC = 16 / sizeof(T);
    typedef T vecT __attribute__((ext_vector_type(EPC)));
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int r = (int)(row % L);
    const T* pr = p + row * (int64_t)Tdim;
    const T* dpr = dp + row * (int64_t)Tdim;
    T* dsr = ds + row * (int64_t)Tdim;
    float rs = 0.f;
    for (int k = 0; k < segs.n; ++k) {
        const int lo = segs.off[k], hi = min(Tdim, lo + (int)segs.nnz[k][r]);
        if constexpr (VEC) {
            const int v_lo = (lo + EPC - 1) / EPC * EPC, v_hi = max(v_lo, hi / EPC * EPC);  // whole pieces
            for (int s = v_lo + lane * EPC; s < v_hi; s += 64 * EPC) {
                const vecT a = *reinterpret_cast<const vecT*>(pr + s), b = *reinterpret_cast<const vecT*>(dpr + s);
#pragma unroll
                for (int e = 0; e < EPC; ++e) rs += (float)a[e] * (float)b[e];
            }
            for (int s = lo + lane; s < min(v_lo, hi); s += 64) rs += (float)pr[s] * (float)dpr[s];
            for (int s = v_hi + lane; s < hi; s += 64) rs += (float)pr[s] * (float)dpr[s];
        } else {
            for (int s = lo + lane; s < hi; s += 64) rs += (float)pr[s] * (float)dpr[s];
        }
    }
    rs = wave_sum(rs);
    // every lane rewrites only the slots it reads here, so ds == dp is safe
    for (int k = 0; k < segs.n; ++k) {
        const int lo = segs.off[k], hi = min(Tdim, lo + (int)segs.nnz[k][r]);
        if constexpr (VEC) {
            const int v_lo = (lo + EPC - 1) / EPC * EPC, v_hi = max(v_lo, hi / EPC * EPC);
            for (int s = v_lo + lane * EPC; s < v_hi; s += 64 * EPC) {
                const vecT a = *reinterpret_cast<const vecT*>(pr + s), b = *reinterpret_cast<const vecT*>(dpr + s);
                vecT o;
#pragma unroll
                for (int e = 0; e < EPC; ++e) o[e] = (T)((float)a[e] * ((float)b[e] - rs) * scale);
                __builtin_nontemporal_store(o, reinterpret_cast<vecT*>(dsr + s));
            }
            for (int s = lo + lane; s < min(v_lo, hi); s += 64) dsr[s] = (T)((float)pr[s] * ((float)dpr[s] - rs) * scale);
            for (int s = v_hi + lane; s < hi; s += 64) dsr[s] = (T)((float)pr[s] * ((float)dpr[s] - rs) * scale);
        } else {
            for (int s = lo + lane; s < hi; s += 64) dsr[s] = (T)((float)pr[s] * ((float)dpr[s] - rs) * scale);
        }
    }
}

// Segment k of the mask and segment k of the transposed mask describe the same set of (row, column) pairs.
struct TransposeSeg {
    // rows of the mask: column of slot s of row i = a_i + lin_i * s
    const float* sTod_lin;
    const float* sTod_trans;
    const float* nnz;
    const int32_t* first_col;
    int off;
    // rows of the transposed mask (= columns of the mask): row of slot t of column j = a_j + lin_j * t
    const float* t_sTod_lin;
    const float* t_sTod_trans;
    const float* t_nnz;
    const int32_t* t_first_col;
    int t_off;
};
struct TransposeParams {
    const void* src;  // [BH, L, T]   compressed, rows of the mask
    void* dst;        // [BH, Lt, Tt] compressed, rows of the transposed mask
    int64_t BH;
    int L, T, Lt, Tt;
    int n_seg;
    TransposeSeg seg[SPLAT_MAX_SEGMENTS];
};

// dst[bh, j, t_off + t] = src[bh, i, off + s] where i is the row behind slot t of column j and s the slot of column
// j in row i.  A workgroup owns 64 consecutive columns j (rows of dst) of one (batch, head) and walks the rows i of
// src that hold any of them in chunks of 64 through an LDS tile [i][j]:
//   in:  lane = column; for each row i of the chunk the lanes whose column is live in that row read consecutive
//        slots of src (a coalesced run), the others write 0;
//   out: lane = row i; for each column j the lanes whose row is a slot of that column write consecutive slots of dst.
// Every element of src is read once and every element of dst written once, as runs of up to 64 elements.
// u / lin and whether it is exact, for 0 <= u < 2^24 and lin >= 1, with the reciprocal taken once per row (the
// float product is within one of the quotient, which the remainder test repairs); u < 0 gives q < 0.
__device__ __forceinline__ bool exact_quotient(int u, int lin, float inv, int& q) {
    int t = (int)((float)u * inv);
    int r = u - t * lin;
    if (r < 0) {
        t -= 1;
        r += lin;
    } else if (r >= lin) {
        t += 1;
        r -= lin;
    }
    q = t;
    return r == 0;
}

template <typename T>
__global__ __launch_bounds__(256) void compressed_transpose_kernel(const TransposeParams p) {
    constexpr int TJ = 64, TI = 64, PITCH = TJ + 2;
    __shared__ T tile[TI * PITCH];
    __shared__ int s_lo[4], s_hi[4];
    __shared__ int mj_a[TJ], mj_lin[TJ], mj_cnt[TJ];  // maps of the 64 columns (rows of dst)
    __shared__ int mi_a[TI], mi_lin[TI], mi_cnt[TI];  // maps of the chunk's 64 rows of src
    __shared__ float mj_inv[TJ], mi_inv[TI];          // 1 / lin
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_jt = (p.Lt + TJ - 1) / TJ;
    const int64_t bh = blockIdx.x / n_jt;
    const int j0 = (int)(blockIdx.x % n_jt) * TJ;
    const T* src = static_cast<const T*>(p.src) + bh * (int64_t)p.L * p.T;
    T* dst = static_cast<T*>(p.dst) + (bh * (int64_t)p.Lt) * p.Tt;

    for (int k = 0; k < p.n_seg; ++k) {
        const TransposeSeg& sg = p.seg[k];
        const int jc = j0 + lane;  // the column this lane stands for in the "in" phase
        RowMap mj = {0, 1, 0};
        if (jc < p.Lt) mj = load_row_map(sg.t_sTod_lin, sg.t_sTod_trans, sg.t_nnz, sg.t_first_col, jc);
        mj.cnt = min(mj.cnt, p.Tt - sg.t_off);  // never past the end of a compressed row, whatever the metadata says
        const int lo = wave_min_i(mj.cnt > 0 ? mj.a : 0x7fffffff);
        const int hi = wave_max_i(mj.cnt > 0 ? mj.a + mj.lin * (mj.cnt - 1) : -1);
        __syncthreads();  // the tile and the tables of the previous segment are done with
        if (wave == 0) mj_a[lane] = mj.a, mj_lin[lane] = mj.lin, mj_cnt[lane] = mj.cnt, mj_inv[lane] = 1.0f / (float)mj.lin;
        if (lane == 0) s_lo[wave] = lo, s_hi[wave] = hi;  // every wavefront holds the same 64 columns
        __syncthreads();
        const int i_min = max(s_lo[0], 0), i_max = min(s_hi[0], p.L - 1);
        for (int i0 = i_min; i0 <= i_max; i0 += TI) {
            if (wave == 0) {
                RowMap mi = {0, 1, 0};
                if (i0 + lane <= i_max) mi = load_row_map(sg.sTod_lin, sg.sTod_trans, sg.nnz, sg.first_col, i0 + lane);
                mi.cnt = min(mi.cnt, p.T - sg.off);
                mi_a[lane] = mi.a, mi_lin[lane] = mi.lin, mi_cnt[lane] = mi.cnt, mi_inv[lane] = 1.0f / (float)mi.lin;
            }
            __syncthreads();
            // ---- in: rows i0 + 16*wave .. + 15, lane = column ----
#pragma unroll 4
            for (int r = 0; r < TI / 4; ++r) {
                const int il = wave * (TI / 4) + r;
                const int a = mi_a[il], lin = mi_lin[il], cnt = mi_cnt[il];
                const int u = jc - a;
                int sl;
                const bool on_step = exact_quotient(u, lin, mi_inv[il], sl);
                T val = (T)0.f;
                if (on_step && u >= 0 && sl < cnt) val = src[(int64_t)(i0 + il) * p.T + sg.off + sl];
                tile[il * PITCH + lane] = val;
            }
            __syncthreads();
            // ---- out: columns j0 + 16*wave .. + 15, lane = row of the chunk ----
#pragma unroll 4
            for (int c = 0; c < TJ / 4; ++c) {
                const int jl = wave * (TJ / 4) + c;
                const int a = mj_a[jl], lin = mj_lin[jl], cnt = mj_cnt[jl];
                const int u = i0 + lane - a;
                int t;
                const bool on_step = exact_quotient(u, lin, mj_inv[jl], t);
                if (on_step && i0 + lane <= i_max && u >= 0 && t < cnt)
                    dst[(int64_t)(j0 + jl) * p.Tt + sg.t_off + t] = tile[lane * PITCH + jl];
            }
        }
    }
}

}  // namespace splat

using namespace splat;

extern "C" int splat_softmax_bwd(const void* p, const void* dp, void* ds, const splat_acsr_seg* segs, int32_t n_seg, int64_t BH,
                                 int32_t L, int32_t T, float scale, int32_t dtype, void* stream) {
    begin_launch();
    const char* who = "splat_softmax_bwd";
    if (!p || !dp || !ds || !segs) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (n_seg < 1 || n_seg > SPLAT_MAX_SEGMENTS) return fail(SPLAT_E_SHAPE, "%s: n_seg must be 1..%d (got %d)", who, SPLAT_MAX_SEGMENTS, n_seg);
    if (BH <= 0 || L <= 0 || T <= 0) return fail(SPLAT_E_SHAPE, "%s: need BH, L, T > 0 (got %lld, %d, %d)", who, (long long)BH, L, T);
    if (BH * (int64_t)L > ((int64_t)1 << 33)) return fail(SPLAT_E_SHAPE, "%s: too many rows", who);
    BwdSegs s;
    s.n = n_seg;
    for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) {
        s.nnz[k] = nullptr;
        s.off[k] = 0;
    }
    for (int k = 0; k < n_seg; ++k) {
        if (!segs[k].nnz) return fail(SPLAT_E_NULL, "%s: segment %d has a null nnz array", who, k);
        if (segs[k].slot_offset < 0 || segs[k].slot_offset >= T)
            return fail(SPLAT_E_SHAPE, "%s: segment %d slot_offset %d outside [0, T=%d)", who, k, segs[k].slot_offset, T);
        s.nnz[k] = segs[k].nnz;
        s.off[k] = segs[k].slot_offset;
    }
    const int64_t n_rows = BH * L;
    const unsigned grid = (unsigned)((n_rows + 3) / 4);
    hipStream_t st = (hipStream_t)stream;
    const bool aligned = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(dp) | reinterpret_cast<uintptr_t>(ds)) & 15) == 0;
    auto launch = [&](auto zero) {
        using E = decltype(zero);
        if (aligned && (T * (int)sizeof(E)) % 16 == 0)
            softmax_bwd_kernel<E, true><<<grid, 256, 0, st>>>((const E*)p, (const E*)dp, (E*)ds, s, n_rows, L, T, scale);
        else
            softmax_bwd_kernel<E, false><<<grid, 256, 0, st>>>((const E*)p, (const E*)dp, (E*)ds, s, n_rows, L, T, scale);
    };
    switch (dtype) {
        case SPLAT_F32: launch(0.0f); break;
        case SPLAT_F16: launch((f16)0); break;
        case SPLAT_BF16: launch((bf16)0); break;
        default: return fail(SPLAT_E_DTYPE, "%s: unknown dtype %d", who, dtype);
    }
    return check_launch(who);
}

extern "C" int splat_compressed_transpose(const void* src, void* dst, const splat_acsr_seg* segs, const splat_acsr_seg* segs_t,
                                          int32_t n_seg, int64_t BH, int32_t L, int32_t T, int32_t Lt, int32_t Tt, int32_t dtype,
                                          void* stream) {
    begin_launch();
    const char* who = "splat_compressed_transpose";
    if (!src || !dst || !segs || !segs_t) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (src == dst) return fail(SPLAT_E_UNSUPPORTED, "%s: not an in-place operation", who);
    if (n_seg < 1 || n_seg > SPLAT_MAX_SEGMENTS) return fail(SPLAT_E_SHAPE, "%s: n_seg must be 1..%d (got %d)", who, SPLAT_MAX_SEGMENTS, n_seg);
    if (BH <= 0 || L <= 0 || T <= 0 || Lt <= 0 || Tt <= 0)
        return fail(SPLAT_E_SHAPE, "%s: need BH, L, T, Lt, Tt > 0 (got %lld, %d, %d, %d, %d)", who, (long long)BH, L, T, Lt, Tt);
    if (BH * (int64_t)Lt > ((int64_t)1 << 33)) return fail(SPLAT_E_SHAPE, "%s: too many rows", who);
    TransposeParams p;
    p.src = src;
    p.dst = dst;
    p.BH = BH;
    p.L = L, p.T = T, p.Lt = Lt, p.Tt = Tt;
    p.n_seg = n_seg;
    for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) p.seg[k] = TransposeSeg{};
    for (int k = 0; k < n_seg; ++k) {
        const splat_acsr_seg &a = segs[k], &b = segs_t[k];
        if (!a.sTod_lin || !a.sTod_trans || !a.nnz || !b.sTod_lin || !b.sTod_trans || !b.nnz)
            return fail(SPLAT_E_NULL, "%s: segment %d lacks sTod_lin / sTod_trans / nnz", who, k);
        if (a.slot_offset < 0 || a.slot_offset >= T || b.slot_offset < 0 || b.slot_offset >= Tt)
            return fail(SPLAT_E_SHAPE, "%s: segment %d slot offsets %d / %d outside [0, %d) / [0, %d)", who, k, a.slot_offset,
                        b.slot_offset, T, Tt);
        p.seg[k] = TransposeSeg{a.sTod_lin, a.sTod_trans, a.nnz, a.first_col, a.slot_offset,
                                b.sTod_lin, b.sTod_trans, b.nnz, b.first_col, b.slot_offset};
    }
    const int64_t n_wg = BH * (int64_t)((Lt + 63) / 64);
    if (n_wg > 0x7fffffff) return fail(SPLAT_E_SHAPE, "%s: problem too large for one launch", who);
    const unsigned grid = (unsigned)n_wg;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case SPLAT_F32: compressed_transpose_kernel<float><<<grid, 256, 0, st>>>(p); break;
        case SPLAT_F16: compressed_transpose_kernel<f16><<<grid, 256, 0, st>>>(p); break;
        case SPLAT_BF16: compressed_transpose_kernel<bf16><<<grid, 256, 0, st>>>(p); break;
        default: return fail(SPLAT_E_DTYPE, "%s: unknown dtype %d", who, dtype);
    }
    return check_launch(who);
}
