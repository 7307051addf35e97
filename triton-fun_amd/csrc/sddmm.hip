// SDDMM on ACSR: out[bh, r, off + s] = scale * <q[bh, r, :], K[bh, c(r, s), :]> for the live slots only.
//
// A workgroup of 4 wavefronts owns 128 rows of one (batch, head) (rows first + rs*k, see acsr_plan.hpp);
// wavefront w owns rows 32w..32w+31 of the block.  The key positions its rows' spans cover are walked in tiles
// of 64.  Per tile the K rows are staged in LDS in chunks of DC contraction values (128 for 16-bit types, 64 for
// fp32; the copy of the next chunk is issued to registers before the math of the current one); Q fragments
// stay in registers when d <= DC and are re-read from cache otherwise.  Scores are produced transposed (rows =
// keys, columns = queries, 32x32x16 MFMA) so that one lane owns one query row; each 32-key half tile is then
// turned around in a per-wavefront LDS staging area so that a lane writes 8 consecutive positions of one row:
// with a uniform plan these are 8 consecutive compressed slots, one 16-byte store (any alignment).  Dead
// positions are never stored.  The kernel is bound by the compressed output (HBM), not by MFMA: 2*d flops per
// 2-4 output bytes.
#include <algorithm>
#include <type_traits>

#include "sddmm_params.hpp"

namespace splat {

template <typename T>
struct SddmmGeom {
    static constexpr int DC = sizeof(T) == 2 ? 128 : 64;  // contraction values per LDS chunk
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

// Store the scores of 8 consecutive tile positions jj..jj+7 of one row; `row_out` points at the row's first slot of
// the segment.  Unit-step rows: the positions are consecutive slots, written with one 16/32-byte store (any
// alignment) when all 8 are live and element by element under a range test at the two ends of the row's span;
// lanes whose positions miss the span altogether do nothing.  Other rows: the full affine test per position.
template <typename TO>
__device__ __forceinline__ void store_piece(TO* row_out, const RowWin& w, int jj, const float (&v)[8]) {
    const int u = jj - w.lo;
    if (w.lin == 1) {
        if (u >= 0 && u + 8 <= w.cnt) {
            typedef TO v8 __attribute__((ext_vector_type(8)));
            v8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = (TO)v[e];
            __builtin_memcpy(row_out + u, &t, 8 * sizeof(TO));
        } else if (u + 8 > 0 && u < w.cnt) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if ((unsigned)(u + e) < (unsigned)w.cnt) row_out[u + e] = (TO)v[e];
        }
    } else if (w.cnt > 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (win_live(w, jj + e)) row_out[win_slot(w, jj + e)] = (TO)v[e];
    }
}

// KSU: 0 = the contraction is longer than one LDS chunk (Q fragments are re-read per chunk); otherwise Q stays in
// registers, and KSU > 0 says at compile time how many MFMA steps hold data (-1: known at run time only).
template <typename T, bool KT, int KSU, bool PROBS>
__global__ __launch_bounds__(256, (KSU > 0 && KSU * 16 < SddmmGeom<T>::DC && !KT) ? 3 : 2) void sddmm_kernel(const SddmmParams p) {
    constexpr bool QREG = KSU != 0;
    constexpr int ES = sizeof(T);
    constexpr int BM = 128;
    constexpr int NT = kBN / 32;
    // one LDS chunk holds the whole contraction when its length is known to be shorter (d = 64 in a 16-bit type: half
    // the K tile, half the Q registers, and a third workgroup per CU)
    constexpr int DC = (KSU > 0 && !KT) ? KSU * 16 : SddmmGeom<T>::DC;
    constexpr int KSC = DC / 16;                                  // MFMA steps per chunk
    constexpr int K_ROW = KT ? (kBN * ES + 64) : (DC * ES + 16);  // bytes per LDS row
    constexpr int K_ROWS = KT ? DC : kBN;
    constexpr int EPC = 16 / ES;
    constexpr int CPT = kBN * DC * ES / 16 / 256;                 // 16-byte chunks per thread
    constexpr int CR = KT ? (kBN * ES / 16) : (DC * ES / 16);     // chunks per LDS row
    constexpr int S_ROW = 32 * 4 + 16;                            // staging row: 32 floats + pad

    __shared__ __attribute__((aligned(16))) char s_k[K_ROW * K_ROWS];
    // Per-wavefront staging: either the turn-around tile (32 rows of 32 floats) or, for 16-bit outputs of uniform plans,
    // a ring of 128 slots per row in which a row's scores collect until a whole 128-byte line of it can be stored
    // (+ 4 slots that mirror the ring's first 4, so that a read of 8 slots never wraps).
    constexpr int R_SLOTS = 128, R_ROW = (R_SLOTS + 4) * 2 + 8;
    constexpr int STG_BYTES = 32 * S_ROW > 32 * R_ROW ? 32 * S_ROW : 32 * R_ROW;
    __shared__ __attribute__((aligned(16))) char s_stage[4][STG_BYTES];
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ int s_off[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int ksp = logical % p.key_split;  // this workgroup's share of the row block's tiles
    const int bh = (logical / p.key_split) / p.n_row_blocks;
    const int rb = (logical / p.key_split) % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L, d = p.d;

    const T* qb = (const T*)p.q + b * p.q_sb + h * p.q_sh;
    const T* kb = (const T*)p.k + b * p.k_sb + h * p.k_sh;

    if (tid == 0) {
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) s_off[k] = p.seg[k].slot_offset;
    }
    plan_segments<BM>(p.seg, p.n_seg, r0, rs, L, !KT, s_plan, &s_ps, tid);

    // B-operand row of this lane: query row 32*wave + lm of the block
    const int q_row = min(r0 + rs * (32 * wave + lm), L - 1);
    const T* qr = qb + (int64_t)q_row * p.q_sl;
    // with a row statistic: exp(scale * s - lse) = exp2(s * exp_mul - exp_sub), stored as it is
    const float out_scale = PROBS ? 1.0f : p.scale;
    const float exp_mul = p.scale * 1.4426950408889634f;
    float exp_sub = 0.f;
    if constexpr (PROBS) exp_sub = p.row_lse[(int64_t)bh * L + q_row] * 1.4426950408889634f;
    Frag<T> qf[KSC];
    if constexpr (QREG) {
#pragma unroll
        for (int ks = 0; ks < KSC; ++ks) qf[ks] = load_q_frag<T>(qr, 16 * ks + 8 * g, d, p.q_vec != 0);
    }
    const int n_chunks = QREG ? 1 : (d + DC - 1) / DC;
    const int ks_used = QREG ? (d + 15) / 16 : KSC;  // MFMA steps that hold data when d <= DC

    // one 16-byte piece of the K chunk (positions j0.., contraction values kd0..) for this thread's slot i
    auto load_piece = [&](const SegPlan& pl, int j0, int kd0, int i) {
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
            } else if (kd < d) {
                T tmp[EPC];
#pragma unroll
                for (int e = 0; e < EPC; ++e) tmp[e] = (kd + e < d) ? src[(int64_t)(kd + e) * p.k_sd] : (T)0.f;
                __builtin_memcpy(&val, tmp, 16);
            }
        }
        return val;
    };

    char* stg = s_stage[wave];
    const int64_t out_bh = (int64_t)bh * L * p.T;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        const SegPlan pl = s_plan[sg];
        // output slots of different tiles are disjoint, so the tiles of a row block can be shared out freely
        const int t_begin = (int)(((int64_t)pl.n_tiles * ksp) / p.key_split);
        const int t_end = (int)(((int64_t)pl.n_tiles * (ksp + 1)) / p.key_split);
        if (t_begin >= t_end) continue;
        const int off = s_off[sg];
        // this lane's own row (source of the wavefront's span) and the 2 block rows it writes out
        const RowWin mine = make_row_win(cached_row_map<BM>(&s_ps, sg, 32 * wave + lm), pl);
        // tiles before lmin / from hmax on hold nothing for this wavefront; tiles from lo_max on and up to hi_min lie
        // inside every one of its rows' spans (never, if a row is empty or the plan is not uniform)
        const WaveSpan span = wave_span(mine, pl.uniform != 0);
        const int lmin = span.lo_min, hmax = span.hi_max;
        RowWin wr[2];
        int64_t wbase[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int rr = 32 * wave + 16 * c + (lane >> 2);
            wr[c] = make_row_win(cached_row_map<BM>(&s_ps, sg, rr), pl);
            const int r = r0 + rs * rr;
            if (r >= L) wr[c].cnt = 0;
            wbase[c] = out_bh + (int64_t)r * p.T + off;
        }

        // Tiles whose keys all exist need none of load_piece's clamping and 64-bit index arithmetic: a wavefront-uniform
        // base (the tile's first key) plus a per-lane byte offset that is fixed for the segment.
        const bool k_fast = !KT && QREG && p.k_vec && (d % EPC == 0) && ((int64_t)pl.cs * kBN * p.k_sl * ES < ((int64_t)1 << 31));
        uint32_t k_off[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int idx = tid + 256 * i;
            k_off[i] = (uint32_t)(((int64_t)pl.cs * (idx / CR) * p.k_sl + (idx % CR) * EPC) * ES);
        }
        auto load_tile_piece = [&](int tile, int i) {
            const int64_t key_first = pl.c0 + (int64_t)pl.cs * (tile * kBN), key_last = key_first + (int64_t)pl.cs * (kBN - 1);
            if (k_fast && key_first >= 0 && key_last < p.n_keys) {  // wavefront-uniform
                const char* base = reinterpret_cast<const char*>(kb + key_first * p.k_sl);
                u32x4 val = {0u, 0u, 0u, 0u};
                if (((tid + 256 * i) % CR) * EPC < d) val = *reinterpret_cast<const u32x4*>(base + k_off[i]);
                return val;
            }
            return load_piece(pl, tile * kBN, 0, i);
        };
        // ---- line-wise output (16-bit outputs, uniform plans, the whole row block in this workgroup) ----
        // Scores go from the accumulators into the row's ring at (slot + lo%4) mod 128, four consecutive slots at a time,
        // untested: a position outside the row's span lands on ring entries that are not waiting to be stored.  After each
        // tile every row stores the 64-slot lines that have become complete (and, once its last position has passed,
        // the rest), 8 lanes x 16 bytes per line: whole aligned lines instead of pieces that straddle them, which is
        // what lets them bypass the L2's write combining (non-temporal stores).
        // (measured: rows of four or five lines gain 13 % in launches of 4096 row blocks and lose 5 % in one of 2048)
        const bool use_ring = pl.uniform && p.key_split == 1 && p.out_dtype != SPLAT_F32 &&
                              (p.T >= 384 || (p.T >= 256 && p.total >= 4096));
        int f_lo[4], f_cnt[4], f_done[4];
        int64_t f_base[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int rr = 32 * wave + 8 * c + (lane >> 3);
            const RowWin w = make_row_win(cached_row_map<BM>(&s_ps, sg, rr), pl);
            const int r = r0 + rs * rr;
            f_lo[c] = w.lo;
            f_cnt[c] = (r < L) ? w.cnt : 0;
            f_done[c] = 0;
            f_base[c] = out_bh + (int64_t)r * p.T + off;
        }
        const int lo4 = mine.lo & ~3;
        u32x4 kreg[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) kreg[i] = QREG ? load_tile_piece(t_begin, i) : load_piece(pl, t_begin * kBN, 0, i);
        // Wait for them here: otherwise the compiler's wait for them sits at the top of the loop below, where on every
        // later iteration it can only mean "everything outstanding", the previous tile's stores included.
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int i = 0; i < CPT; ++i) asm volatile("" ::"v"(kreg[i]));
#endif

        for (int tile = t_begin; tile < t_end; ++tile) {
            const int j0 = tile * kBN;
            const bool skip = (j0 + kBN <= lmin) || (j0 >= hmax);  // wavefront-uniform
            f32x16 acc[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[nt][j] = 0.f;

            for (int ch = 0; ch < n_chunks; ++ch) {
                const int kd0 = ch * DC;
                lds_barrier();  // previous chunk fully consumed (the stores of the previous tile stay in flight)
#pragma unroll
                for (int i = 0; i < CPT; ++i) {
                    const int idx = tid + 256 * i;
                    *reinterpret_cast<u32x4*>(s_k + (idx / CR) * K_ROW + (idx % CR) * 16) = kreg[i];
                }
                // request the next chunk (of the next tile when this was the last chunk) while this one is used
                {
                    const bool last_ch = (ch + 1 == n_chunks);
                    const int nj0 = last_ch ? j0 + kBN : j0;
                    const int nkd0 = last_ch ? 0 : kd0 + DC;
                    if (!(last_ch && tile + 1 == t_end)) {
#pragma unroll
                        for (int i = 0; i < CPT; ++i) kreg[i] = QREG ? load_tile_piece(tile + 1, i) : load_piece(pl, nj0, nkd0, i);
                    }
                }
                lds_barrier();  // the chunk is in LDS (the loads just requested stay in flight)
                if (skip) continue;
                auto load_k = [&](int ks, int nt) {
                    if constexpr (KT)
                        return lds_frag_cols<T>(s_k, K_ROW, 16 * ks + 8 * g, 16 * ks + 8 * g + 4, 32 * nt, lane);
                    else
                        return lds_frag_rowmajor<T>(s_k + (32 * nt + lm) * K_ROW + (16 * ks + 8 * g) * ES);
                };
                if constexpr (KSU > 0 && !KT) {
                    // the step count is a constant: no test per step, and fragments are requested four MFMAs ahead
                    // (deeper read-ahead costs the third workgroup per CU its registers)
                                        constexpr int NF = KSU * NT, AHEAD = NF < 4 ? NF : 4;
                    Frag<T> kfr[NF];
#pragma unroll
                    for (int i = 0; i < AHEAD; ++i) kfr[i] = load_k(i / NT, i % NT);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = 0; i < NF; ++i) {
                        mma32(acc[i % NT], kfr[i], qf[i / NT]);  // rows = keys, columns = queries
                        if (i + AHEAD < NF) {
                            kfr[i + AHEAD] = load_k((i + AHEAD) / NT, (i + AHEAD) % NT);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                } else {
#pragma unroll
                    for (int ks = 0; ks < KSC; ++ks) {
                        if (QREG && ks >= ks_used) break;
                        Frag<T> qv;
                        if constexpr (QREG)
                            qv = qf[ks];
                        else
                            qv = load_q_frag<T>(qr, kd0 + 16 * ks + 8 * g, d, p.q_vec != 0);
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) mma32(acc[nt], load_k(ks, nt), qv);  // rows = keys, columns = queries
                    }
                }
            }
            // The K loads of the next tile have to be back before this tile's stores are issued: loads and stores
            // complete out of order with respect to each other, so a wait for the loads that comes after the stores
            // is a wait for the stores as well.
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
            for (int i = 0; i < CPT; ++i) asm volatile("" ::"v"(kreg[i]));
#endif
            if (skip) continue;
            if constexpr (PROBS) {  // probabilities of a softmax whose row statistic is known
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int j = 0; j < 16; ++j) acc[nt][j] = fast_exp2(fmaf(acc[nt][j], exp_mul, -exp_sub));
            }

            // every position of the tile is a slot of every row of this wavefront: no tests, one vector store per piece
            const bool full = (j0 >= span.lo_max) && (j0 + kBN <= span.hi_min);
            auto write_tile = [&](auto zero) {
                using TO = decltype(zero);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    // ---- turn the half tile around: lane (query lm, half g) holds positions 8jq + 4g + {0..3} ----
#pragma unroll
                    for (int jq = 0; jq < 4; ++jq) {
                        f32x4 v4 = {acc[nt][4 * jq] * out_scale, acc[nt][4 * jq + 1] * out_scale, acc[nt][4 * jq + 2] * out_scale,
                                    acc[nt][4 * jq + 3] * out_scale};
                        *reinterpret_cast<f32x4*>(stg + lm * S_ROW + (8 * jq + 4 * g) * 4) = v4;
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's LDS writes are visible to its own reads
                    // ---- lane writes positions 8*(lane%4) .. +7 of block rows 32w + 16c + lane/4 ----
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        const char* src = stg + (16 * c + (lane >> 2)) * S_ROW + (lane & 3) * 32;
                        const f32x4 a0 = *reinterpret_cast<const f32x4*>(src);
                        const f32x4 a1 = *reinterpret_cast<const f32x4*>(src + 16);
                        const float v[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
                        const int jj = j0 + 32 * nt + 8 * (lane & 3);
                        TO* const row_out = (TO*)p.out + wbase[c];
                        if (full) {
                            typedef TO v8 __attribute__((ext_vector_type(8)));
                            v8 t;
#pragma unroll
                            for (int e = 0; e < 8; ++e) t[e] = (TO)v[e];
                            __builtin_memcpy(row_out + (jj - wr[c].lo), &t, 8 * sizeof(TO));
                        } else {
                            store_piece<TO>(row_out, wr[c], jj, v);
                        }
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // staging reads done before it is overwritten
                }
            };
            auto ring_tile = [&](auto zero) {
                using TO = decltype(zero);
                typedef TO v4 __attribute__((ext_vector_type(4)));
                typedef TO v8 __attribute__((ext_vector_type(8)));
                char* const ring_row = stg + lm * R_ROW;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int jq = 0; jq < 4; ++jq) {
                        v4 t;
#pragma unroll
                        for (int i = 0; i < 4; ++i) t[i] = (TO)(acc[nt][4 * jq + i] * out_scale);
                        const int ri = (j0 + 32 * nt + 8 * jq + 4 * g - lo4) & (R_SLOTS - 1);
                        *reinterpret_cast<v4*>(ring_row + ri * 2) = t;
                        if (ri == 0) *reinterpret_cast<v4*>(ring_row + R_SLOTS * 2) = t;
                    }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's LDS writes are visible to its own reads
                // A tile that lies inside the span of every row of the wavefront adds 64 slots to each of them, so every
                // row completes exactly one line, and completes it: no tests, no branches (the tests below cost several
                // times the tile's MFMAs in scalar and branch instructions).  A row that ends with this tile may have a
                // last, shorter line to store as well: that tile takes the tests.
                if (__builtin_amdgcn_readfirstlane((full && j0 + kBN < span.hi_min) ? 1 : 0)) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int s0 = 64 * f_done[c] + 8 * (lane & 7);
                        const int rix = (s0 + (f_lo[c] & 3)) & (R_SLOTS - 1);
                        v8 val;
                        __builtin_memcpy(&val, stg + (8 * c + (lane >> 3)) * R_ROW + rix * 2, 16);
                        TO* const dst = (TO*)p.out + f_base[c] + s0;
                        if (p.out_vec) {
                            __builtin_nontemporal_store(val, reinterpret_cast<v8*>(dst));
                        } else {
                            __builtin_memcpy(dst, &val, 16);
                        }
                        f_done[c] += 1;
                    }
                    return;
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int u_end = j0 + kBN - f_lo[c];
                    const int final_slot = min(max(u_end, 0), f_cnt[c]);  // slots below it hold their scores
#pragma unroll
                    for (int rep = 0; rep < 2; ++rep) {
                        const int ls = 64 * f_done[c];
                        const bool line = (ls + 64 <= final_slot) || (u_end >= f_cnt[c] && ls < f_cnt[c]);
                        if (line) {
                            const int s0 = ls + 8 * (lane & 7);
                            const int rix = (s0 + (f_lo[c] & 3)) & (R_SLOTS - 1);
                            v8 val;
                            __builtin_memcpy(&val, stg + (8 * c + (lane >> 3)) * R_ROW + rix * 2, 16);
                            TO* const dst = (TO*)p.out + f_base[c] + s0;
                            const int n = f_cnt[c] - s0;
                            if (n >= 8) {
                                if (p.out_vec) {
                                    __builtin_nontemporal_store(val, reinterpret_cast<v8*>(dst));
                                } else {
                                    __builtin_memcpy(dst, &val, 16);
                                }
                            } else {
#pragma unroll
                                for (int e = 0; e < 8; ++e)
                                    if (e < n) dst[e] = val[e];
                            }
                            f_done[c] += 1;
                        }
                    }
                }
            };
            if (use_ring) {
                if (p.out_dtype == SPLAT_BF16)
                    ring_tile((bf16)0);
                else
                    ring_tile((f16)0);
            } else if (p.out_dtype == SPLAT_BF16) {
                write_tile((bf16)0);
            } else if (p.out_dtype == SPLAT_F16) {
                write_tile((f16)0);
            } else {
                write_tile(0.0f);
            }
        }
    }
}

template <typename T>
static int launch_sddmm(const char* who, SddmmParams p, bool kt, hipStream_t st) {
    begin_launch();
    p.n_row_blocks = count_row_blocks(p.L, 128, p.row_stride);
    // Few row blocks (one head of a short sequence, the reference's own benchmark shape) would leave most of the 256
    // compute units idle: share every row block's tiles out over several workgroups then.
    const int64_t blocks = (int64_t)p.B * p.H * p.n_row_blocks;
    if (blocks > 0x7ffffff0) return fail(SPLAT_E_SHAPE, "%s: problem too large for one launch", who);
    p.key_split = blocks >= 512 ? 1 : (int)std::min<int64_t>(32, (768 + blocks - 1) / blocks);
    p.total = (int)(blocks * p.key_split);
    const int grid = ((p.total + 7) / 8) * 8;
    constexpr int DC = SddmmGeom<T>::DC, KSC = DC / 16;
    const int steps = (p.d + 15) / 16;
    auto go = [&](auto probs_c) {
        constexpr bool PROBS = decltype(probs_c)::value;
        if (kt) {
            if (p.d <= DC)
                sddmm_kernel<T, true, -1, PROBS><<<grid, 256, 0, st>>>(p);
            else
                sddmm_kernel<T, true, 0, PROBS><<<grid, 256, 0, st>>>(p);
        } else {
            if (p.d > DC)
                sddmm_kernel<T, false, 0, PROBS><<<grid, 256, 0, st>>>(p);
            else if (steps == KSC)
                sddmm_kernel<T, false, KSC, PROBS><<<grid, 256, 0, st>>>(p);
            else if (steps == KSC / 2)
                sddmm_kernel<T, false, KSC / 2, PROBS><<<grid, 256, 0, st>>>(p);
            else
                sddmm_kernel<T, false, -1, PROBS><<<grid, 256, 0, st>>>(p);
        }
    };
    if (p.row_lse != nullptr)
        go(std::true_type{});
    else
        go(std::false_type{});
    return check_launch(who);
}

}  // namespace splat

using namespace splat;

static int sddmm_common(const char* who, const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb,
                        int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out, const splat_acsr_seg* segs, int32_t n_seg, int32_t B,
                        int32_t H, int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype,
                        int32_t out_dtype, const float* row_lse, const void* plan, int64_t plan_bytes, void* stream) {
    if (!q || !kT || !out || !segs) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (B <= 0 || H <= 0 || L <= 0 || n_keys <= 0 || d <= 0 || T <= 0)
        return fail(SPLAT_E_SHAPE, "%s: need B, H, L, n_keys, d, T > 0 (got %d, %d, %d, %d, %d, %d)", who, B, H, L, n_keys, d, T);
    if (L > (1 << 23) || n_keys > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: L and n_keys are limited to 2^23", who);
    if (out_dtype != SPLAT_F32 && out_dtype != SPLAT_F16 && out_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown out_dtype %d", who, out_dtype);
    if (in_dtype != SPLAT_F32 && in_dtype != SPLAT_F16 && in_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown in_dtype %d", who, in_dtype);
    if (k_sd != 1 && k_sl != 1)
        return fail(SPLAT_E_ALIGN, "%s: kT needs unit stride along d (k_sd == 1) or along keys (k_sl == 1); got k_sd=%lld k_sl=%lld", who,
                    (long long)k_sd, (long long)k_sl);
    SddmmParams p;
    p.q = q; p.k = kT; p.out = out;
    p.q_sb = q_sb; p.q_sh = q_sh; p.q_sl = q_sl;
    p.k_sb = k_sb; p.k_sh = k_sh; p.k_sd = k_sd; p.k_sl = k_sl;
    p.B = B; p.H = H; p.L = L; p.n_keys = n_keys; p.d = d; p.T = T;
    p.scale = scale;
    p.row_lse = row_lse;
    p.plan = nullptr;
    if (plan) {
        if ((reinterpret_cast<uintptr_t>(plan) & 15) != 0) return fail(SPLAT_E_ALIGN, "%s: the plan must be 16-byte aligned", who);
        const int64_t need = splat_attention_plan_bytes(segs, n_seg, L);
        if (need <= 0 || plan_bytes < need)
            return fail(SPLAT_E_SHAPE, "%s: the plan holds %lld bytes, this mask needs %lld", who, (long long)plan_bytes, (long long)need);
        p.plan = static_cast<const PlanRec*>(plan);  // the variant for rows of K that are contiguous comes first
    }
    p.out_dtype = out_dtype;
    p.n_seg = n_seg;
    if (int rc = fill_segs(who, segs, n_seg, p.seg, T)) return rc;
    p.row_stride = common_row_stride(segs, n_seg);
    const int es = in_dtype == SPLAT_F32 ? 4 : 2;
    const int epc = 16 / es;
    auto al = [&](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    auto mul = [&](int64_t s) { return (s % epc) == 0; };
    // rows of K contiguous ([.., keys, d] memory) unless only the key stride is 1
    const bool kt = !(k_sd == 1);
    p.q_vec = (al(q) && mul(q_sb) && mul(q_sh) && mul(q_sl)) ? 1 : 0;
    p.k_vec = (al(kT) && mul(k_sb) && mul(k_sh) && mul(kt ? k_sd : k_sl)) ? 1 : 0;
    p.out_vec = (al(out) && T % 8 == 0) ? 1 : 0;
    for (int k = 0; k < n_seg; ++k)
        if (segs[k].slot_offset % 8 != 0) p.out_vec = 0;
    hipStream_t st = (hipStream_t)stream;
    begin_launch();
    if (const int rc = launch_sddmm_lines(who, p, in_dtype, st)) return rc < 0 ? rc : check_launch(who);
    switch (in_dtype) {
        case SPLAT_F32: return launch_sddmm<float>(who, p, kt, st);
        case SPLAT_F16: return launch_sddmm<f16>(who, p, kt, st);
        default: return launch_sddmm<bf16>(who, p, kt, st);
    }
}

extern "C" int splat_sddmm(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb, int64_t k_sh,
                           int64_t k_sd, int64_t k_sl, void* out, const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H,
                           int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale, int32_t in_dtype, int32_t out_dtype,
                           void* stream) {
    return sddmm_common("splat_sddmm", q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, out, segs, n_seg, B, H, L, n_keys, d, T,
                        scale, in_dtype, out_dtype, nullptr, nullptr, 0, stream);
}

extern "C" int splat_sddmm_probs(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb,
                                 int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out, const splat_acsr_seg* segs, int32_t n_seg,
                                 int32_t B, int32_t H, int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale,
                                 int32_t in_dtype, int32_t out_dtype, const float* lse, void* stream) {
    const char* who = "splat_sddmm_probs";
    if (!lse) return fail(SPLAT_E_NULL, "%s: null lse", who);
    if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0) return fail(SPLAT_E_ALIGN, "%s: lse must be 4-byte aligned", who);
    return sddmm_common(who, q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, out, segs, n_seg, B, H, L, n_keys, d, T, scale,
                        in_dtype, out_dtype, lse, nullptr, 0, stream);
}

extern "C" int splat_sddmm_planned(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb,
                                   int64_t k_sh, int64_t k_sd, int64_t k_sl, void* out, const splat_acsr_seg* segs, int32_t n_seg,
                                   int32_t B, int32_t H, int32_t L, int32_t n_keys, int32_t d, int32_t T, float scale,
                                   int32_t in_dtype, int32_t out_dtype, const float* lse, const void* plan, int64_t plan_bytes,
                                   void* stream) {
    const char* who = "splat_sddmm_planned";
    if (!plan) return fail(SPLAT_E_NULL, "%s: null plan", who);
    if (lse && (reinterpret_cast<uintptr_t>(lse) & 3) != 0) return fail(SPLAT_E_ALIGN, "%s: lse must be 4-byte aligned", who);
    return sddmm_common(who, q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, out, segs, n_seg, B, H, L, n_keys, d, T, scale,
                        in_dtype, out_dtype, lse, plan, plan_bytes, stream);
}
