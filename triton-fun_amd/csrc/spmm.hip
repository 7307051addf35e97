// SpMM on ACSR: out[bh, r, :] = sum over live slots s of p[bh, r, off + s] * V[bh, c(r, s), :].
//
// A workgroup of 4 wavefronts owns 128 consecutive rows of one (batch, head) and a chunk of up to 128
// output columns; wavefront w owns rows 32w..32w+31.  Key positions are walked in tiles of 64 (see
// acsr_plan.hpp).  The V tile is staged row-major in LDS and read as MFMA B operand with the transposing
// LDS read; the A operand (probabilities) is read straight from the compressed rows: with a uniform
// plan 8 consecutive positions of a row are 8 consecutive slots, one (possibly unaligned) 16-byte load.
// Output orientation rows = queries, columns = output features, so stores are contiguous per row.
// Bound by reading the compressed probabilities (HBM), not by MFMA.
#include "spmm_params.hpp"

namespace splat {

// Write a wavefront's 32 x (32*DVT) block of accumulators to rows r0 + rs*(32*wave + k) of out[bh] ([rows, n_out],
// columns col0..).  An accumulator register holds one row's value at column lane%32: stored directly, a wavefront
// instruction writes 32 consecutive elements of two rows.  When rows of the output can take 16-byte stores (`wide`), each
// 32 x 32 tile is instead converted, turned around in the wavefront's staging area `stg` (32 rows of 144 bytes at
// least) and written as 16-byte pieces (8 or 4 per row).  With a staging area `rows_stg` of at least
// 32 x (32*DVT*element size + 16) bytes the whole 32 x (32*DVT) block is turned around at once and leaves as whole rows
// of the block (aligned runs, non-temporal) instead of one 64- or 128-byte piece of every row per 32-column tile.
template <int DVT>
__device__ __forceinline__ void store_block_rows(const f32x16 (&acc)[DVT], char* stg, char* rows_stg, int rows_stg_bytes, void* out,
                                                 int out_dtype, bool wide, int64_t bh, int n_rows, int n_out, int r0, int rs,
                                                 int wave, int lane, int col0) {
    const int lm = lane & 31, g = lane >> 5;
    const int es_out = (out_dtype == SPLAT_F32) ? 4 : 2;
    auto whole_rows = [&](auto zero) {
        using TO = decltype(zero);
        constexpr int ROW_B = 32 * DVT * (int)sizeof(TO) + 16, CPR = 2 * DVT * (int)sizeof(TO);  // staging row, pieces per row
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
            for (int j = 0; j < 16; ++j)
                *reinterpret_cast<TO*>(rows_stg + acc_row(j, g) * ROW_B + (32 * dt + lm) * sizeof(TO)) = (TO)acc[dt][j];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's LDS writes are visible to its own reads
#pragma unroll
        for (int i = 0; i < 32 * CPR / 64; ++i) {
            const int flat = i * 64 + lane;
            const int row = flat / CPR, c = flat % CPR;
            const int r = r0 + rs * (32 * wave + row);
            const u32x4 val = *reinterpret_cast<const u32x4*>(rows_stg + row * ROW_B + c * 16);
            if (r < n_rows) {
                char* orow = reinterpret_cast<char*>(out) + ((bh * n_rows + r) * n_out + col0) * sizeof(TO);
                __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(orow + c * 16));
            }
        }
    };
    if (wide && rows_stg != nullptr && 32 * (32 * DVT * es_out + 16) <= rows_stg_bytes) {
        if (out_dtype == SPLAT_BF16)
            whole_rows((bf16)0);
        else if (out_dtype == SPLAT_F16)
            whole_rows((f16)0);
        else
            whole_rows(0.0f);
        return;
    }
    if (wide) {
        const int row_b = 32 * es_out + 16;  // padded staging row
        const int cpr = 32 * es_out / 16;     // 16-byte pieces per row
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                char* dst = stg + acc_row(j, g) * row_b + lm * es_out;
                if (out_dtype == SPLAT_BF16)
                    *reinterpret_cast<bf16*>(dst) = (bf16)acc[dt][j];
                else if (out_dtype == SPLAT_F16)
                    *reinterpret_cast<f16*>(dst) = (f16)acc[dt][j];
                else
                    *reinterpret_cast<float*>(dst) = acc[dt][j];
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's LDS writes are visible to its own reads
            for (int flat = lane; flat < 32 * cpr; flat += 64) {
                const int row = flat / cpr, c = flat % cpr;
                const int r = r0 + rs * (32 * wave + row);
                const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * row_b + c * 16);
                if (r < n_rows) {
                    char* orow = reinterpret_cast<char*>(out) + ((bh * n_rows + r) * n_out + col0 + 32 * dt) * es_out;
                    *reinterpret_cast<u32x4*>(orow + c * 16) = val;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next tile overwrites the staging
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int r = r0 + rs * (32 * wave + acc_row(j, g));
        if (r < n_rows) {
            const int64_t base = (bh * n_rows + r) * n_out;
#pragma unroll
            for (int dt = 0; dt < DVT; ++dt) {
                const int c = col0 + 32 * dt + lm;
                if (c < n_out) store_as(out, base + c, acc[dt][j], out_dtype);
            }
        }
    }
}

template <typename T, int DVT>
__global__ __launch_bounds__(256, 2) void spmm_kernel(const SpmmParams p) {
    constexpr int ES = sizeof(T);
    constexpr int BM = 128;
    constexpr int DVC = 32 * DVT;           // output columns per workgroup
    constexpr int V_ROW = DVC * ES + 64;    // bytes per LDS row
    constexpr int EPC = 16 / ES;
    constexpr int CR = DVC * ES / 16;       // 16-byte chunks per LDS row
    constexpr int NCHUNK = kBN * CR;        // chunks per tile

    // Row of the probability staging tile.  16-bit types: 8 positions of margin on either side of the 64, because a piece
    // that straddles an end of its row's span is loaded from inside the span and written where it belongs.
    constexpr int P_MARGIN = (ES == 2) ? 8 : 0;
    constexpr int P_ROW = (kBN + 2 * P_MARGIN) * ES + 16;
    __shared__ __attribute__((aligned(16))) char s_v[V_ROW * kBN];
    constexpr int SP_BYTES = 32 * P_ROW;
    __shared__ __attribute__((aligned(16))) char s_p[4][SP_BYTES];
    static_assert(P_ROW >= 32 * 4 + 16, "the staging area also holds a 32 x 32 fp32 tile of the output");
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ SegPtrs s_seg[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int cchunk = logical % p.n_col_chunks;
    const int rest = logical / p.n_col_chunks;
    const int bh = rest / p.n_row_blocks;
    const int rb = rest % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L;
    const int col0 = cchunk * DVC;

    const T* vb = (const T*)p.v + b * p.v_sb + h * p.v_sh;
    const T* pb = (const T*)p.p + (int64_t)bh * L * p.T;

    if (tid == 0) {
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) s_seg[k] = p.seg[k];
    }
    plan_segments<BM>(p.seg, p.n_seg, r0, rs, L, true, s_plan, &s_ps, tid);

    f32x16 acc[DVT];
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[dt][j] = 0.f;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        const SegPlan pl = s_plan[sg];
        if (pl.n_tiles == 0) continue;
        const int off = s_seg[sg].slot_offset;

        const RowWin win = make_row_win(cached_row_map<BM>(&s_ps, sg, 32 * wave + lm), pl);
        RowWin wr[4];
        const T* wrow[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int rr = 32 * wave + 8 * c + (lane >> 3);
            wr[c] = make_row_win(cached_row_map<BM>(&s_ps, sg, rr), pl);
            const int r = r0 + rs * rr;
            if (r >= L) wr[c].cnt = 0;
            wrow[c] = pb + (int64_t)min(r, L - 1) * p.T + off;
        }
        // tiles before lmin / from hmax on hold nothing for this wavefront; tiles from lo_max on and up to hi_min lie
        // inside every one of its rows' spans (never, if a row is empty or not unit-step)
        const WaveSpan span = wave_span(win, __all(win.lin == 1) != 0);
        const int lmin = span.lo_min, hmax = span.hi_max;

        // one 16-byte piece of the V tile at positions j0.. for this thread's slot i
        auto load_piece = [&](int j0, int i) {
            const int idx = tid + 256 * i;
            const int row = idx / CR, cc = idx % CR;
            const int n = min(max(pl.c0 + pl.cs * (j0 + row), 0), p.n_keys - 1);
            const T* src = vb + (int64_t)n * p.v_sl;
            const int c = col0 + cc * EPC;
            u32x4 val = {0u, 0u, 0u, 0u};
            if (p.v_vec && c + EPC <= p.n_out) {
                val = *reinterpret_cast<const u32x4*>(src + c);
            } else if (c < p.n_out) {
                T tmp[EPC];
#pragma unroll
                for (int e = 0; e < EPC; ++e) tmp[e] = (c + e < p.n_out) ? src[c + e] : (T)0.f;
                __builtin_memcpy(&val, tmp, 16);
            }
            return val;
        };
        constexpr int CPT = NCHUNK / 256;
        static_assert(NCHUNK % 256 == 0, "tile shape");
        u32x4 vreg[CPT];
#pragma unroll
        for (int i = 0; i < CPT; ++i) vreg[i] = load_piece(0, i);
        // A tile's probabilities: lane (row 8c + lane/8 of the wavefront's 32, piece lane%8) fetches 8 consecutive
        // positions, so one instruction reads 8 rows x 64 consecutive slots; the pieces are turned into A fragments
        // (lane = row) through a per-wavefront staging tile.  Requested one tile ahead, like V.
        // 16-bit types, unit-step rows of at least 8 slots: a piece that straddles an end of the row's span is loaded as
        // the 8 slots at that end (one vector load like any other, no branch) and lands in the staging tile `shift`
        // positions off its own place, over zeros; where it overlaps the neighbouring piece both hold the same values.
        typedef T vec8 __attribute__((ext_vector_type(8)));
        struct Piece {
            vec8 v;
            int shift;   // positions between the piece's own place and where v belongs
            int state;   // 0: nothing live (zeros), 1: v is the whole piece, 2: zeros, then v at its shifted place
        };
        auto load_probs = [&](int j0, int c) {
            Piece pc;
            pc.shift = 0;
            pc.state = 1;
            const RowWin& w = wr[c];
            const int jj = j0 + 8 * (lane & 7);
            const int u = jj - w.lo;
            if ((j0 >= span.lo_max) && (j0 + kBN <= span.hi_min)) {  // wavefront-uniform: the tile is inside every span
                __builtin_memcpy(&pc.v, wrow[c] + u, 8 * ES);        // any alignment
            } else if (ES == 2 && w.lin == 1 && w.cnt >= 8) {
                const bool touches = (u + 8 > 0) && (u < w.cnt);
                const int uc = min(max(u, 0), w.cnt - 8);
                pc.shift = uc - u;
                pc.state = touches ? (pc.shift == 0 ? 1 : 2) : 0;
                if (touches) __builtin_memcpy(&pc.v, wrow[c] + uc, 8 * ES);  // any alignment
            } else if (w.lin == 1 && u >= 0 && u + 8 <= w.cnt) {
                __builtin_memcpy(&pc.v, wrow[c] + u, 8 * ES);  // any alignment
            } else if (w.lin == 1) {
                // an end of the row's span (or outside it): range test per slot, loads from a clamped slot so that
                // they need no branch
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const T x = wrow[c][min(max(u + e, 0), max(w.cnt - 1, 0))];
                    pc.v[e] = ((unsigned)(u + e) < (unsigned)w.cnt) ? x : (T)0.f;
                }
            } else {
                pc.v = gather_affine8<vec8>(wrow[c], w, jj);
            }
            return pc;
        };
        // the piece's place in the staging tile, and what goes there
        auto stage_piece = [&](char* stg, const Piece& pc, int c) {
            char* own = stg + (8 * c + (lane >> 3)) * P_ROW + (P_MARGIN + (lane & 7) * 8) * ES;
            if constexpr (ES == 2) {
                if (!__any(pc.state != 1)) {  // every piece of the instruction lies inside its row's span
                    *reinterpret_cast<vec8*>(own) = pc.v;
                } else {
                    vec8 zero;
#pragma unroll
                    for (int e = 0; e < 8; ++e) zero[e] = (T)0.f;
                    if (pc.state != 1) *reinterpret_cast<vec8*>(own) = zero;
                    if (pc.state != 0) __builtin_memcpy(own + pc.shift * ES, &pc.v, 8 * ES);
                }
            } else {
                *reinterpret_cast<vec8*>(own) = pc.v;
            }
        };
        Piece praw[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) praw[c] = load_probs(0, c);

        for (int tile = 0; tile < pl.n_tiles; ++tile) {
            const int j0 = tile * kBN;
            const bool skip = (j0 + kBN <= lmin) || (j0 >= hmax);  // wavefront-uniform
            __syncthreads();  // previous tile fully consumed
#pragma unroll
            for (int i = 0; i < CPT; ++i) {
                const int idx = tid + 256 * i;
                *reinterpret_cast<u32x4*>(s_v + (idx / CR) * V_ROW + (idx % CR) * 16) = vreg[i];
            }
            // while the tile settles in LDS: request the next V tile and this tile's probability fragments
            if (tile + 1 < pl.n_tiles) {
#pragma unroll
                for (int i = 0; i < CPT; ++i) vreg[i] = load_piece(j0 + kBN, i);
            }
            char* stg = s_p[wave];
#pragma unroll
            for (int c = 0; c < 4; ++c)
                stage_piece(stg, praw[c], c);
            if (tile + 1 < pl.n_tiles) {
#pragma unroll
                for (int c = 0; c < 4; ++c) praw[c] = load_probs(j0 + kBN, c);
            }
            __syncthreads();
            if (skip) continue;
            Frag<T> pf[kBN / 16];
#pragma unroll
            for (int t = 0; t < kBN / 16; ++t) pf[t] = lds_frag_rowmajor<T>(stg + lm * P_ROW + (P_MARGIN + 16 * t + 8 * g) * ES);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // fragments read before the next tile overwrites the staging
#pragma unroll
            for (int t = 0; t < kBN / 16; ++t) {
#pragma unroll
                for (int dt = 0; dt < DVT; ++dt) {
                    Frag<T> vf = lds_frag_cols<T>(s_v, V_ROW, 16 * t + 8 * g, 16 * t + 8 * g + 4, 32 * dt, lane);
                    mma32(acc[dt], pf[t], vf);
                }
            }
        }
    }

    __syncthreads();  // every wavefront is done with the staging areas and the V tile
    // whole-row staging: the wavefront's own area if it is large enough, else halves of the two tiles (all free now)
    constexpr int HALF = (2 * SP_BYTES < V_ROW * kBN / 2 ? 2 * SP_BYTES : V_ROW * kBN / 2) & ~15;  // per wavefront, two per tile
    char* const rows_stg = (wave < 2 ? &s_p[0][0] : s_v) + (wave & 1) * HALF;
    store_block_rows<DVT>(acc, s_p[wave], rows_stg, HALF, p.out, p.out_dtype, p.out_vec && (col0 + 32 * DVT <= p.n_out), bh, L,
                          p.n_out, r0, rs, wave, lane, col0);
}

template <typename T>
static int launch_spmm(SpmmParams p, hipStream_t st) {
    begin_launch();
    p.n_row_blocks = count_row_blocks(p.L, 128, p.row_stride);
    const int dvt = p.n_out > 64 ? 4 : (p.n_out > 32 ? 2 : 1);
    p.n_col_chunks = (p.n_out + 32 * dvt - 1) / (32 * dvt);
    const int64_t total = (int64_t)p.B * p.H * p.n_row_blocks * p.n_col_chunks;
    if (total > 0x7ffffff0) return fail(SPLAT_E_SHAPE, "splat_spmm: problem too large for one launch");
    p.total = (int)total;
    const int grid = ((p.total + 7) / 8) * 8;
    if (dvt == 4)
        spmm_kernel<T, 4><<<grid, 256, 0, st>>>(p);
    else if (dvt == 2)
        spmm_kernel<T, 2><<<grid, 256, 0, st>>>(p);
    else
        spmm_kernel<T, 1><<<grid, 256, 0, st>>>(p);
    return check_launch("splat_spmm");
}


// ---- transposed product: out[bh, j, :] = sum over the rows i that keep column j of p[bh, i, slot of j in row i] * x[bh, i, :]
// (the compressed matrix enters transposed without ever being stored that way; the backward pass needs P~^T.dO and
// dS~^T.Q).  A workgroup owns 128 columns j = first + rs*m of the mask = rows of the output (rs: the row stride of the
// transposed mask's ACSR, 1 unless its rows alternate column phase); the rows i that meet them are walked in tiles of 64,
// planned from that ACSR like any other row block.  Per tile, row i's entries at the block's 128 columns are read from
// its compressed row (consecutive slots when the row's column step is rs and its phase the block's) into an LDS tile
// [i][m], zero where row i does not keep the column, and read back as the A operand with the transposing LDS read,
// exactly as the x tile [i][feature] is read as the B operand.
template <typename T, int DVT>
__global__ __launch_bounds__(256, 2) void spmm_t_kernel(const SpmmTParams p) {
    constexpr int ES = sizeof(T);
    constexpr int BM = 128;
    constexpr int DVC = 32 * DVT;
    constexpr int X_ROW = DVC * ES + 64;   // bytes per LDS row of the x tile
    constexpr int PT_ROW = BM * ES + 64;   // bytes per LDS row of the probability tile
    constexpr int EPC = 16 / ES;
    constexpr int CR = DVC * ES / 16;
    constexpr int NCHUNK = kBN * CR;
    constexpr int CPT = NCHUNK / 256;
    static_assert(NCHUNK % 256 == 0, "tile shape");

    __shared__ __attribute__((aligned(16))) char s_x[X_ROW * kBN];
    __shared__ __attribute__((aligned(16))) char s_pt[PT_ROW * kBN];
    static_assert(PT_ROW * kBN >= 4 * 32 * (32 * 4 + 16), "the probability tile doubles as the output staging areas");
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ SegPtrs s_seg[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int cchunk = logical % p.n_col_chunks;
    const int rest = logical / p.n_col_chunks;
    const int bh = rest / p.n_row_blocks;
    const int rb = rest % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int j_first = block_first_row(rb, BM, rs);  // first column of the mask (row of the output) of this workgroup
    const int col0 = cchunk * DVC;

    const T* xb = (const T*)p.x + b * p.x_sb + h * p.x_sh;
    const T* pb = (const T*)p.p + (int64_t)bh * p.L * p.T;

    if (tid == 0) {
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) s_seg[k] = p.seg[k];
    }
    plan_segments<BM>(p.seg_t, p.n_seg, j_first, rs, p.Lt, true, s_plan, &s_ps, tid);

    f32x16 acc[DVT];
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[dt][j] = 0.f;

    // this thread's part of the probability tile: row prow, pieces pq, pq + 4, pq + 8, pq + 12 of 8 columns each
    const int prow = tid >> 2, pq = tid & 3;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        const SegPlan pl = s_plan[sg];
        if (pl.n_tiles == 0) continue;
        const SegPtrs src = s_seg[sg];

        // the rows i this wavefront's 32 columns meet, in walk positions
        const RowWin win = make_row_win(cached_row_map<BM>(&s_ps, sg, 32 * wave + lm), pl);
        int lmin = win.cnt > 0 ? win.lo : 0x3fffffff;
        int hmax = win.cnt > 0 ? win.lo + win.cnt : -0x3fffffff;
        lmin = wave_min_i(lmin);
        hmax = wave_max_i(hmax);

        // walk position -> row of the mask
        auto row_at = [&](int pos) { return pl.c0 + pl.cs * pos; };
        auto load_piece = [&](int pos0, int k) {
            const int idx = tid + 256 * k;
            const int row = idx / CR, cc = idx % CR;
            const int n = min(max(row_at(pos0 + row), 0), p.L - 1);
            const T* srow = xb + (int64_t)n * p.x_sl;
            const int c = col0 + cc * EPC;
            u32x4 val = {0u, 0u, 0u, 0u};
            if (p.x_vec && c + EPC <= p.n_out) {
                val = *reinterpret_cast<const u32x4*>(srow + c);
            } else if (c < p.n_out) {
                T tmp[EPC];
#pragma unroll
                for (int e = 0; e < EPC; ++e) tmp[e] = (c + e < p.n_out) ? srow[c + e] : (T)0.f;
                __builtin_memcpy(&val, tmp, 16);
            }
            return val;
        };
        // the map of the row at walk position pos0 + prow; rows that do not exist are empty
        auto load_map = [&](int pos0) {
            const int i = row_at(pos0 + prow);
            RowMap m = {0, 1, 0};
            if (i >= 0 && i < p.L) m = load_row_map(src, i);
            return m;
        };
        typedef T vec8 __attribute__((ext_vector_type(8)));
        // piece pq + 4c of that row: block columns 8*(pq + 4c) .. + 7
        auto load_probs = [&](const BlockRow& br, int pos0, int c) {
            vec8 v;
            const RowWin& w = br.w;
            const int i_row = min(max(row_at(pos0 + prow), 0), p.L - 1);
            const T* wrow = pb + (int64_t)i_row * p.T + src.slot_offset;
            const int jj = 8 * (pq + 4 * c);
            const int u = jj - w.lo;
            // A piece that straddles an end of the row's span is loaded like any other, as 16 bytes from where its first
            // position would be, and the positions outside the span are cleared afterwards: what lies there (dead
            // slots, the neighbouring row) is readable memory unless the piece leaves the whole buffer.  (Assembling
            // such a piece from element loads costs more than the loads: the compiler guards their registers with a
            // wait for every load in flight.)
            const int64_t e0 = ((int64_t)bh * p.L + i_row) * p.T + src.slot_offset + u;
            const bool touches = (u + 8 > 0) && (u < w.cnt);
            if (w.lin == 1 && touches && e0 >= 0 && e0 + 8 <= p.p_elems) {
                __builtin_memcpy(&v, wrow + u, 8 * ES);  // any alignment
                if (u < 0 || u + 8 > w.cnt) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if ((unsigned)(u + e) >= (unsigned)w.cnt) v[e] = (T)0.f;
                }
            } else if (w.lin == 1 && !touches) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (T)0.f;
            } else if (w.lin == 1) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const T x = wrow[min(max(u + e, 0), max(w.cnt - 1, 0))];
                    v[e] = ((unsigned)(u + e) < (unsigned)w.cnt) ? x : (T)0.f;
                }
            } else if (w.lin > 1) {
                v = gather_affine8<vec8>(wrow, w, jj);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = entry_at_column<T>(wrow, br.m, j_first + rs * (jj + e));
            }
            return v;
        };

        u32x4 xreg[CPT];
#pragma unroll
        for (int k = 0; k < CPT; ++k) xreg[k] = load_piece(0, k);
        RowMap m_next = load_map(kBN);  // requested two tiles ahead of its use, the probabilities one tile ahead
        vec8 praw[4];
        {
            const BlockRow br = block_row(load_map(0), j_first, rs);
#pragma unroll
            for (int c = 0; c < 4; ++c) praw[c] = load_probs(br, 0, c);
        }

        for (int tile = 0; tile < pl.n_tiles; ++tile) {
            const int pos0 = tile * kBN;
            const bool skip = (pos0 + kBN <= lmin) || (pos0 >= hmax);  // wavefront-uniform
            __syncthreads();  // previous tile fully consumed
#pragma unroll
            for (int k = 0; k < CPT; ++k) {
                const int idx = tid + 256 * k;
                *reinterpret_cast<u32x4*>(s_x + (idx / CR) * X_ROW + (idx % CR) * 16) = xreg[k];
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) *reinterpret_cast<vec8*>(s_pt + prow * PT_ROW + (pq + 4 * c) * 8 * ES) = praw[c];
            if (tile + 1 < pl.n_tiles) {
#pragma unroll
                for (int k = 0; k < CPT; ++k) xreg[k] = load_piece(pos0 + kBN, k);
                const BlockRow br = block_row(m_next, j_first, rs);
#pragma unroll
                for (int c = 0; c < 4; ++c) praw[c] = load_probs(br, pos0 + kBN, c);
                if (tile + 2 < pl.n_tiles) m_next = load_map(pos0 + 2 * kBN);
            }
            __syncthreads();
            if (skip) continue;
            Frag<T> pf[kBN / 16];
#pragma unroll
            for (int t = 0; t < kBN / 16; ++t) pf[t] = lds_frag_cols<T>(s_pt, PT_ROW, 16 * t + 8 * g, 16 * t + 8 * g + 4, 32 * wave, lane);
#pragma unroll
            for (int t = 0; t < kBN / 16; ++t) {
#pragma unroll
                for (int dt = 0; dt < DVT; ++dt) {
                    Frag<T> xf = lds_frag_cols<T>(s_x, X_ROW, 16 * t + 8 * g, 16 * t + 8 * g + 4, 32 * dt, lane);
                    mma32(acc[dt], pf[t], xf);
                }
            }
        }
    }

    __syncthreads();  // every wavefront is done with the tiles
    constexpr int HALF = ((PT_ROW < X_ROW ? PT_ROW : X_ROW) * kBN / 2) & ~15;  // per wavefront, two per tile
    char* const rows_stg = (wave < 2 ? s_pt : s_x) + (wave & 1) * HALF;
    store_block_rows<DVT>(acc, s_pt + wave * (32 * (32 * 4 + 16)), rows_stg, HALF, p.out, p.out_dtype,
                          p.out_vec && (col0 + 32 * DVT <= p.n_out), bh, p.Lt, p.n_out, j_first, rs, wave, lane, col0);
}

template <typename T>
static int launch_spmm_t(SpmmTParams p, hipStream_t st) {
    begin_launch();
    p.n_row_blocks = count_row_blocks(p.Lt, 128, p.row_stride);
    const int dvt = p.n_out > 64 ? 4 : (p.n_out > 32 ? 2 : 1);
    p.n_col_chunks = (p.n_out + 32 * dvt - 1) / (32 * dvt);
    const int64_t total = (int64_t)p.B * p.H * p.n_row_blocks * p.n_col_chunks;
    if (total > 0x7ffffff0) return fail(SPLAT_E_SHAPE, "splat_spmm_t: problem too large for one launch");
    p.total = (int)total;
    const int grid = ((p.total + 7) / 8) * 8;
    if (dvt == 4)
        spmm_t_kernel<T, 4><<<grid, 256, 0, st>>>(p);
    else if (dvt == 2)
        spmm_t_kernel<T, 2><<<grid, 256, 0, st>>>(p);
    else
        spmm_t_kernel<T, 1><<<grid, 256, 0, st>>>(p);
    return check_launch("splat_spmm_t");
}

}  // namespace splat

using namespace splat;

static int spmm_common(const char* who, const void* pp, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out,
                       const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t n_keys,
                       int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype, const void* plan, int64_t plan_bytes,
                       void* stream) {
    if (!pp || !v || !out || !segs) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (B <= 0 || H <= 0 || L <= 0 || n_keys <= 0 || n_out <= 0 || T <= 0)
        return fail(SPLAT_E_SHAPE, "%s: need B, H, L, n_keys, n_out, T > 0 (got %d, %d, %d, %d, %d, %d)", who, B, H, L, n_keys, n_out, T);
    if (L > (1 << 23) || n_keys > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: L and n_keys are limited to 2^23", who);
    if (out_dtype != SPLAT_F32 && out_dtype != SPLAT_F16 && out_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown out_dtype %d", who, out_dtype);
    if (in_dtype != SPLAT_F32 && in_dtype != SPLAT_F16 && in_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown in_dtype %d", who, in_dtype);
    if (v_sl < n_out) return fail(SPLAT_E_SHAPE, "%s: v row stride %lld < n_out %d", who, (long long)v_sl, n_out);
    SpmmParams p;
    p.p = pp; p.v = v; p.out = out;
    p.v_sb = v_sb; p.v_sh = v_sh; p.v_sl = v_sl;
    p.B = B; p.H = H; p.L = L; p.n_keys = n_keys; p.n_out = n_out; p.T = T;
    p.out_dtype = out_dtype;
    p.plan = nullptr;
    if (plan) {
        if ((reinterpret_cast<uintptr_t>(plan) & 15) != 0) return fail(SPLAT_E_ALIGN, "%s: the plan must be 16-byte aligned", who);
        const int64_t need = splat_attention_plan_bytes(segs, n_seg, L);
        if (need <= 0 || plan_bytes < need)
            return fail(SPLAT_E_SHAPE, "%s: the plan holds %lld bytes, this mask needs %lld", who, (long long)plan_bytes, (long long)need);
        p.plan = static_cast<const PlanRec*>(plan);  // the variant with gathered walks comes first
    }
    p.n_seg = n_seg;
    if (int rc = fill_segs(who, segs, n_seg, p.seg, T)) return rc;
    p.row_stride = common_row_stride(segs, n_seg);
    const int es = in_dtype == SPLAT_F32 ? 4 : 2;
    const int epc = 16 / es;
    p.v_vec = ((reinterpret_cast<uintptr_t>(v) & 15) == 0 && v_sb % epc == 0 && v_sh % epc == 0 && v_sl % epc == 0) ? 1 : 0;
    {
        const int es_out = out_dtype == SPLAT_F32 ? 4 : 2;
        p.out_vec = ((reinterpret_cast<uintptr_t>(out) & 15) == 0 && ((int64_t)n_out * es_out) % 16 == 0) ? 1 : 0;
    }
    hipStream_t st = (hipStream_t)stream;
    begin_launch();
    if (const int rc = launch_spmm_thin(who, p, in_dtype, st)) return rc < 0 ? rc : check_launch(who);
    switch (in_dtype) {
        case SPLAT_F32: return launch_spmm<float>(p, st);
        case SPLAT_F16: return launch_spmm<f16>(p, st);
        default: return launch_spmm<bf16>(p, st);
    }
}

extern "C" int splat_spmm(const void* pp, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out,
                          const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t n_keys,
                          int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype, void* stream) {
    return spmm_common("splat_spmm", pp, v, v_sb, v_sh, v_sl, out, segs, n_seg, B, H, L, n_keys, n_out, T, in_dtype, out_dtype,
                       nullptr, 0, stream);
}

extern "C" int splat_spmm_planned(const void* pp, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out,
                                  const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t n_keys,
                                  int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype, const void* plan,
                                  int64_t plan_bytes, void* stream) {
    if (!plan) return fail(SPLAT_E_NULL, "splat_spmm_planned: null plan");
    return spmm_common("splat_spmm_planned", pp, v, v_sb, v_sh, v_sl, out, segs, n_seg, B, H, L, n_keys, n_out, T, in_dtype,
                       out_dtype, plan, plan_bytes, stream);
}

static int spmm_t_common(const char* who, const void* pp, const void* x, int64_t x_sb, int64_t x_sh, int64_t x_sl, void* out,
                         const splat_acsr_seg* segs, const splat_acsr_seg* segs_t, int32_t n_seg, int32_t B, int32_t H,
                         int32_t L, int32_t Lt, int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype, const void* plan_t,
                         int64_t plan_bytes, void* stream) {
    if (!pp || !x || !out || !segs || !segs_t) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (B <= 0 || H <= 0 || L <= 0 || Lt <= 0 || n_out <= 0 || T <= 0)
        return fail(SPLAT_E_SHAPE, "%s: need B, H, L, Lt, n_out, T > 0 (got %d, %d, %d, %d, %d, %d)", who, B, H, L, Lt, n_out, T);
    if (L > (1 << 23) || Lt > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: L and Lt are limited to 2^23", who);
    if (out_dtype != SPLAT_F32 && out_dtype != SPLAT_F16 && out_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown out_dtype %d", who, out_dtype);
    if (in_dtype != SPLAT_F32 && in_dtype != SPLAT_F16 && in_dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown in_dtype %d", who, in_dtype);
    if (x_sl < n_out) return fail(SPLAT_E_SHAPE, "%s: x row stride %lld < n_out %d", who, (long long)x_sl, n_out);
    SpmmTParams p;
    p.p = pp; p.x = x; p.out = out;
    p.x_sb = x_sb; p.x_sh = x_sh; p.x_sl = x_sl;
    p.B = B; p.H = H; p.L = L; p.Lt = Lt; p.n_out = n_out; p.T = T;
    p.out_dtype = out_dtype;
    p.n_seg = n_seg;
    if (int rc = fill_segs(who, segs, n_seg, p.seg, T)) return rc;
    if (int rc = fill_segs(who, segs_t, n_seg, p.seg_t, -1)) return rc;
    p.row_stride = common_row_stride(segs_t, n_seg);
    p.p_elems = (int64_t)B * H * L * T;
    const int es = in_dtype == SPLAT_F32 ? 4 : 2;
    const int epc = 16 / es;
    p.x_vec = ((reinterpret_cast<uintptr_t>(x) & 15) == 0 && x_sb % epc == 0 && x_sh % epc == 0 && x_sl % epc == 0) ? 1 : 0;
    const int es_out = out_dtype == SPLAT_F32 ? 4 : 2;
    p.out_vec = ((reinterpret_cast<uintptr_t>(out) & 15) == 0 && ((int64_t)n_out * es_out) % 16 == 0) ? 1 : 0;
    p.plan_t = nullptr;
    if (plan_t) {
        if ((reinterpret_cast<uintptr_t>(plan_t) & 15) != 0) return fail(SPLAT_E_ALIGN, "%s: the plan must be 16-byte aligned", who);
        const int64_t need = splat_attention_plan_bytes(segs_t, n_seg, Lt);
        if (need <= 0 || plan_bytes < need)
            return fail(SPLAT_E_SHAPE, "%s: the plan holds %lld bytes, the transposed mask needs %lld", who, (long long)plan_bytes,
                        (long long)need);
        p.plan_t = static_cast<const PlanRec*>(plan_t);  // the variant with gathered walks comes first
    }
    hipStream_t st = (hipStream_t)stream;
    begin_launch();
    if (const int rc = launch_spmm_t_thin(who, p, in_dtype, st)) return rc < 0 ? rc : check_launch(who);
    switch (in_dtype) {
        case SPLAT_F32: return launch_spmm_t<float>(p, st);
        case SPLAT_F16: return launch_spmm_t<f16>(p, st);
        default: return launch_spmm_t<bf16>(p, st);
    }
}

extern "C" int splat_spmm_t(const void* pp, const void* x, int64_t x_sb, int64_t x_sh, int64_t x_sl, void* out,
                            const splat_acsr_seg* segs, const splat_acsr_seg* segs_t, int32_t n_seg, int32_t B, int32_t H,
                            int32_t L, int32_t Lt, int32_t n_out, int32_t T, int32_t in_dtype, int32_t out_dtype, void* stream) {
    return spmm_t_common("splat_spmm_t", pp, x, x_sb, x_sh, x_sl, out, segs, segs_t, n_seg, B, H, L, Lt, n_out, T, in_dtype,
                         out_dtype, nullptr, 0, stream);
}

extern "C" int splat_spmm_t_planned(const void* pp, const void* x, int64_t x_sb, int64_t x_sh, int64_t x_sl, void* out,
                                    const splat_acsr_seg* segs, const splat_acsr_seg* segs_t, int32_t n_seg, int32_t B,
                                    int32_t H, int32_t L, int32_t Lt, int32_t n_out, int32_t T, int32_t in_dtype,
                                    int32_t out_dtype, const void* plan_t, int64_t plan_bytes, void* stream) {
    if (!plan_t) return fail(SPLAT_E_NULL, "splat_spmm_t_planned: null plan");
    return spmm_t_common("splat_spmm_t_planned", pp, x, x_sb, x_sh, x_sl, out, segs, segs_t, n_seg, B, H, L, Lt, n_out, T,
                         in_dtype, out_dtype, plan_t, plan_bytes, stream);
}
