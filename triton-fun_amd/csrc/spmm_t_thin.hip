// Transposed SpMM on ACSR (out[bh, j, :] = sum over the rows i that keep column j of p[bh, i, slot of j] * x[bh, i, :]) for
// the common fast shape: 16-bit probabilities, x and output of one type, 64 or 128 output columns, 16-byte alignment, and
// the plan table of the transposed mask.
//
// A workgroup of 8 wavefronts owns 128 columns j = first + rs*m of the mask (rows of the output); a wavefront owns 32 of
// them and half of the features and accumulates out^T = x^T P with 16x16x32 MFMAs (rows = output features, columns =
// mask columns).  The wavefronts stay below 128 registers, so that four of them share a SIMD and cover each other's waits.
//
// The rows i that meet the block are walked in tiles of 64 as the table lists them.  Per tile the whole workgroup loads
// row i's entries at the block's 128 columns from its compressed row -- 16 pieces of 8 consecutive slots where the row's
// column step is rs, 16 bytes each at any alignment, cleared outside the row's span with a mask from a table in LDS --
// into an LDS tile [i][m], a few tiles ahead through register sets, and the x rows into a tile [i][feature] beside it.
// Where a row's slots begin in the block's columns and how many there are is worked out for 16 tiles at a time and kept
// in LDS, so that no global load of the tile loop waits for another.  Both tiles have two stages (one barrier per tile)
// and the permuted layout of the SpMM kernel's V tile, and both operands come out of them through the transposing read:
// the B operands 16 columns of the probability tile each, the A operands 16 features of the x tile.  Rows of
// another column step are left out of that loop and, if a segment has any, gathered entry by entry in a second walk.
// The output leaves through an LDS turn-around as whole rows, non-temporal.
#include <algorithm>
#include <type_traits>

#include "spmm_params.hpp"
#include "tile_copy.hpp"

namespace splat {

template <int D>
struct ThinTGeom {
    static constexpr int BM = 128;
    static constexpr int ROWB = D * 2;             // bytes per x row
    static constexpr int P_ROWB = BM * 2;          // bytes per row of the probability tile
    static constexpr int X_STAGE = kBN * ROWB;     // the x tile comes first in a stage
    static constexpr int STAGE = X_STAGE + kBN * P_ROWB;
    static constexpr int O_ROW = ROWB + 16;        // bytes per row of the output turn-around
    static constexpr int TILE_BYTES = 2 * STAGE > BM * O_ROW ? 2 * STAGE : BM * O_ROW;
    static constexpr int MASK_AT = TILE_BYTES;     // 81 masks of 16 bytes: [entries cleared at the low end][at the high end]
    static constexpr int MAPS_AT = MASK_AT + 81 * 16;
    static constexpr int CH = 16;                  // tiles per chunk of a walk: the rows of a chunk have their maps in LDS
    static constexpr int MAP_TILES = CH + 5;       // (the tile loop looks up to 4 tiles past a chunk's last)
    static constexpr int LDS_BYTES = MAPS_AT + MAP_TILES * kBN * 8;
};

// NB: register sets for probability pieces in flight (requested NB + 1 tiles before the tile they belong to is used)
template <typename T, int D, int NB>
__global__ __launch_bounds__(512, 4) void spmm_t_thin_kernel(const SpmmTParams p) {
    using G = ThinTGeom<D>;
    constexpr int BM = G::BM, ROWB = G::ROWB, P_ROWB = G::P_ROWB, X_STAGE = G::X_STAGE, STAGE = G::STAGE, O_ROW = G::O_ROW;
    constexpr int CPR = ROWB / 16;        // 16-byte chunks per x row
    constexpr int NI = kBN * CPR / 512;   // chunks of an x tile per thread
    constexpr int DT = D / 16;            // 16-feature blocks of the output
    static_assert(NI >= 1 && G::MASK_AT % 16 == 0, "tile shape");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const u32x4* const s_mask = reinterpret_cast<const u32x4*>(smem + G::MASK_AT);
    int2* const s_maps = reinterpret_cast<int2*>(smem + G::MAPS_AT);  // [tile of the chunk][row]: lo, cnt
    constexpr int CH = G::CH, MAP_TILES = G::MAP_TILES;
    static_assert(NB + 2 <= MAP_TILES - CH, "the tile loop looks NB + 1 tiles past a chunk's last");

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, g4 = lane >> 4;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int bh = logical / p.n_row_blocks;
    const int rb = logical % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int j_first = block_first_row(rb, BM, rs);
    const int L = p.L;

    const char* xbytes = reinterpret_cast<const char*>((const T*)p.x + b * p.x_sb + h * p.x_sh);
    const int64_t x_rowb = p.x_sl * 2;
    const T* pb = (const T*)p.p + (int64_t)bh * L * p.T;
    const PlanRec* const pt = p.plan_t;
    const int n_rb = p.n_row_blocks;
    // the only rows whose neighbours in memory may lie outside the buffer
    const bool first_bh = bh == 0, last_bh = bh == p.B * p.H - 1;
    const int rs_shift = (rs & (rs - 1)) == 0 ? __builtin_ctz(rs) : -1;

    // mask [lo][hi]: entries lo .. 7 - hi of a piece kept
    if (tid < 81) {
        const int lo = tid / 9, hi = tid % 9;
        const u32x4 ones = {~0u, ~0u, ~0u, ~0u};
        *reinterpret_cast<u32x4*>(smem + G::MASK_AT + tid * 16) = shift_elements(ones, lo) & shift_elements(ones, -hi);
    }
    lds_barrier();

    // this thread's chunks of every x tile: from walk row x_row, 16 bytes at x_col, to LDS offset x_lds of the stage
    int x_row[NI], x_col[NI], x_lds[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int id = tid + 512 * i;
        x_row[i] = id / CPR;
        x_col[i] = (id % CPR) * 16;
        x_lds[i] = x_row[i] * ROWB + v_chunk<ROWB>(x_row[i], id % CPR) * 16;
    }
    // this thread's pieces of every probability tile: walk row prow, block columns 8 (pq + 8 c) .. + 7, c = 0, 1
    const int prow = tid >> 3, pq = tid & 7;
    int p_lds[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) p_lds[c] = X_STAGE + prow * P_ROWB + v_chunk<P_ROWB>(prow, pq + 8 * c) * 16;

    // A wavefront owns 32 of the block's columns (two B operands) and half of the features (FD A operands): every
    // fragment read from LDS serves two MFMAs or FD of them.
    constexpr int FD = DT / 2;
    const int cg = wave & 3, fh = wave >> 2;
    // Operands through the transposing read: lane s of 16-lane block g4 addresses tile row 8 g4 + s / 4 (and 4 rows on)
    // and 4 columns of a 16-column block: 16 dt + 4 (s % 4) of the x tile, 32 cg + 16 cb + 4 (s % 4) of the probability tile
    int x_off[FD], p_off[2];
    {
        const int sq = li >> 2;
        const int in_half = 16 * ((li & 3) >> 1) + 8 * (li & 1);
        const int blk = ROWB >= 256 ? sq : (sq >> 1);
#pragma unroll
        for (int fd = 0; fd < FD; ++fd) {
            const int dt = FD * fh + fd;
            x_off[fd] = (8 * g4 + sq) * ROWB + in_half + 64 * ((dt >> 1) ^ blk) + 32 * ((dt & 1) ^ (g4 & 1));
        }
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
            p_off[cb] = X_STAGE + (8 * g4 + sq) * P_ROWB + in_half + 64 * (cg ^ sq) + 32 * (cb ^ (g4 & 1));
    }

    f32x4v acc[FD][2];
#pragma unroll
    for (int fd = 0; fd < FD; ++fd)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[fd][cb][j] = 0.f;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        SegPlan pl;
        {
            const PlanRec r = plan_uniform_load(pt + plan_seg_at(p.n_seg, rb, sg));
            pl = SegPlan{r[0], r[1], r[2], r[3]};
        }
        const int n_steps = pl.n_tiles;
        if (n_steps == 0) continue;  // workgroup-uniform
        const SegPtrs src = p.seg[sg];
        // walk positions in which some of this wavefront's 32 columns meet a row
        int lmin, hmax;
        {
            const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, sg, cg));
            lmin = r[0], hmax = r[3];
        }
        auto act = [&](int pos0) { return !(pos0 + 32 <= lmin || pos0 >= hmax); };

        bool seg_slow = false;  // this thread has met a row of another step

        auto row_at = [&](int pos) { return pl.c0 + pl.cs * pos; };
        auto load_x = [&](int t, u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int n = min(max(row_at(t * kBN + x_row[i]), 0), L - 1);
                reg[i] = *reinterpret_cast<const u32x4*>(xbytes + n * x_rowb + x_col[i]);
            }
        };
        auto write_x = [&](int stage, const u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<u32x4*>(smem + stage * STAGE + x_lds[i]) = reg[i];
        };
        auto write_p = [&](int stage, const u32x4 (&reg)[2]) {
#pragma unroll
            for (int c = 0; c < 2; ++c) *reinterpret_cast<u32x4*>(smem + stage * STAGE + p_lds[c]) = reg[c];
        };

        // The walk in chunks of CH tiles.  What the loads of a tile need to know of its rows goes into LDS for the whole
        // chunk first, so that the tile loop's global loads do not depend on one another: in the block's columns first + rs*m a
        // row whose column step is rs (or that has one column) holds consecutive slots from m = lo on, cnt of them, or none
        // when its phase is not the block's.  A row of another step (`slow`) is left out here and dealt with after the loop.
        for (int c0 = 0; c0 < n_steps; c0 += CH) {
            const int n_here = min(CH, n_steps - c0);
            for (int e = tid; e < MAP_TILES * kBN; e += 512) {
                const int te = e / kBN;
                const int i = row_at((c0 + te) * kBN + e % kBN);
                const int ic = min(max(i, 0), L - 1);
                const float lin_f = src.sTod_lin[ic], tr = src.sTod_trans[ic];
                const int n = (int)src.nnz[ic], fc = src.first_col[ic];
                const int lin = max((int)lin_f, 1);
                const int a = n == 1 ? fc : (int)rintf(lin_f * tr);
                int cnt = (te < n_here && i == ic) ? min(n, src.max_cnt) : 0;  // rows that do not exist are empty
                const int d0 = a - j_first;
                int lo;
                const bool slow = cnt > 1 && lin != rs;  // (rs == 1 asks for unit steps)
                if (rs == 1) {
                    lo = d0;
                } else {
                    int rem;
                    if (rs_shift >= 0)
                        lo = d0 >> rs_shift, rem = d0 & (rs - 1);
                    else
                        lo = d0 / rs, rem = d0 - lo * rs;
                    if (rem != 0) cnt = 0;
                }
                seg_slow |= slow;
                s_maps[e] = int2{lo, slow ? 0 : cnt};
            }
            lds_barrier();

            // Both pieces of the row at position prow of tile t of the chunk.  A piece that straddles an end of the row's
            // span is loaded like any other, as 16 bytes from where its first entry would be, and the entries outside the span
            // are cleared: what lies there (dead slots, the neighbouring row) is readable memory except before the first and
            // after the last row of the buffer, whose pieces are loaded from inside the row and shifted.
            auto load_probs = [&](int t, u32x4 (&out)[2]) {
                const int2 e = s_maps[t * kBN + prow];  // (tiles past the chunk's last: empty rows, nothing of theirs is read)
                const int lo = e.x, cnt = e.y;
                const int i_row = min(max(row_at((c0 + t) * kBN + prow), 0), L - 1);
                const T* wrow = pb + (int64_t)i_row * p.T + src.slot_offset;
                const bool risky = (first_bh && i_row == 0) || (last_bh && i_row == L - 1);
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int u = 8 * (pq + 8 * c) - lo;
                    const bool touches = u + 8 > 0 && u < cnt;
                    const int u_ld = risky ? min(max(u, -src.slot_offset), p.T - src.slot_offset - 8) : u;
                    const T* src_p = touches ? wrow + u_ld : pb;  // (the buffer's first 16 bytes: any readable address)
                    u32x4 raw;
                    __builtin_memcpy(&raw, src_p, 16);  // any alignment
                    if (u_ld != u) raw = shift_elements(raw, u_ld - u);
                    out[c] = raw & s_mask[min(max(-u, 0), 8) * 9 + min(max(u + 8 - cnt, 0), 8)];
                }
            };

            // ---- prologue: tile 0 into stage 0, x tile 1 and the probabilities of tiles 1 .. NB requested
            u32x4 xreg[NI];
            u32x4 praw[NB][2];  // [tile modulo NB]
            load_x(c0, xreg);
            load_probs(0, praw[0]);
            write_x(0, xreg);  // (everyone has left both stages at the barrier that ended the chunk before)
            write_p(0, praw[0]);
            if (n_here > 1) load_x(c0 + 1, xreg);
            static_for<NB>([&](auto u) {
                constexpr int k = decltype(u)::value + 1;
                load_probs(k, praw[k % NB]);
            });
            lds_barrier();

            auto step = [&](int s, auto idx_c) {
                constexpr int idx = decltype(idx_c)::value;  // s modulo UNROLL
                constexpr int par = idx & 1, set = (idx + 1) % NB;
                // tile s + 1 into the other stage (everyone has left it at the barrier that ended step s - 1); x tile s + 2
                // and the probabilities of tile s + 1 + NB requested into the registers this frees
                if (s + 1 < n_here) {
                    write_x(par ^ 1, xreg);
                    write_p(par ^ 1, praw[set]);
                    if (s + 2 < n_here) load_x(c0 + s + 2, xreg);
                }
                load_probs(s + 1 + NB, praw[set]);
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const int pos0 = (c0 + s) * kBN + 32 * hf;
                    if (!act(pos0)) continue;  // wavefront-uniform
                    Frag<T> pf[2];
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const char* pa = smem + p_off[cb] + (par * STAGE + 32 * hf * P_ROWB);
                        pf[cb] = frag_from_tr<T>(lds_tr16(pa), lds_tr16(pa + 4 * P_ROWB));
                    }
#pragma unroll
                    for (int fd = 0; fd < FD; ++fd) {
                        const char* a = smem + x_off[fd] + (par * STAGE + 32 * hf * ROWB);
                        const Frag<T> xf = frag_from_tr<T>(lds_tr16(a), lds_tr16(a + 4 * ROWB));
                        mma16(acc[fd][0], xf, pf[0]);
                        mma16(acc[fd][1], xf, pf[1]);
                    }
                }
                lds_barrier();
            };
            // the unrolled steps make the stage (s % 2) and the register set ((s + 1) % NB) compile-time constants
            constexpr int UNROLL = NB % 2 == 0 ? NB : 2 * NB;
            for (int s = 0; s < n_here; s += UNROLL) {
                static_for<UNROLL>([&](auto u) {
                    if (s + decltype(u)::value < n_here) step(s + decltype(u)::value, u);
                });
            }
        }

        // ---- rows of another column step, if the segment has any: one more walk with those rows alone (every other row
        // empty), gathered entry by entry from the row's map, one tile at a time
        if (__syncthreads_or(seg_slow ? 1 : 0)) {
            typedef T vec8 __attribute__((ext_vector_type(8)));
            for (int t = 0; t < n_steps; ++t) {
                const int i = row_at(t * kBN + prow);
                const int ic = min(max(i, 0), L - 1);
                RowMap m = load_row_map(src, ic);
                if (i != ic) m.cnt = 0;
                u32x4 pieces[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
                if (m.cnt > 1 && m.lin != rs) {  // (as above: rs == 1 asks for unit steps)
                    const T* wrow = pb + (int64_t)ic * p.T + src.slot_offset;
                    const BlockRow br = block_row(m, j_first, rs);
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        const int jj = 8 * (pq + 8 * c);
                        vec8 v;
                        if (br.w.lin > 1) {
                            v = gather_affine8<vec8>(wrow, br.w, jj);
                        } else {
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[e] = entry_at_column<T>(wrow, m, j_first + rs * (jj + e));
                        }
                        pieces[c] = __builtin_bit_cast(u32x4, v);
                    }
                }
                u32x4 xr[NI];
                load_x(t, xr);
                write_x(0, xr);  // (everyone has left the stage at the barrier before)
                write_p(0, pieces);
                lds_barrier();
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    if (!act(t * kBN + 32 * hf)) continue;  // wavefront-uniform
                    Frag<T> pf[2];
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const char* pa = smem + p_off[cb] + 32 * hf * P_ROWB;
                        pf[cb] = frag_from_tr<T>(lds_tr16(pa), lds_tr16(pa + 4 * P_ROWB));
                    }
#pragma unroll
                    for (int fd = 0; fd < FD; ++fd) {
                        const char* a = smem + x_off[fd] + 32 * hf * ROWB;
                        const Frag<T> xf = frag_from_tr<T>(lds_tr16(a), lds_tr16(a + 4 * ROWB));
                        mma16(acc[fd][0], xf, pf[0]);
                        mma16(acc[fd][1], xf, pf[1]);
                    }
                }
                lds_barrier();
            }
        }
    }

    // ---- output: out^T accumulators (lane: mask column 32 cg + 16 cb + li, features 16 (FD fh + fd) + 4 g4 .. + 3) turned
    // around in LDS, rows stored whole (every wavefront has passed the last barrier of the loop: the tiles are free)
    typedef T v4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int fd = 0; fd < FD; ++fd)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) {
            v4 t;
#pragma unroll
            for (int j = 0; j < 4; ++j) t[j] = (T)acc[fd][cb][j];
            *reinterpret_cast<v4*>(smem + (32 * cg + 16 * cb + li) * O_ROW + (16 * (FD * fh + fd) + 4 * g4) * 2) = t;
        }
    lds_barrier();  // a row's two halves come from two wavefronts
    const char* const o_stg = smem + (16 * wave) * O_ROW;
#pragma unroll
    for (int i = 0; i < 16 * CPR / 64; ++i) {
        const int flat = i * 64 + lane;
        const int row = flat / CPR, c = flat % CPR;
        const int j = j_first + rs * (16 * wave + row);
        const u32x4 val = *reinterpret_cast<const u32x4*>(o_stg + row * O_ROW + c * 16);
        if (j < p.Lt) {
            char* orow = reinterpret_cast<char*>(p.out) + ((int64_t)bh * p.Lt + j) * ROWB;
            __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(orow + c * 16));
        }
    }
}

template <typename T, int D>
static int launch_thin_t_variant(const char* who, SpmmTParams p, hipStream_t st) {
    using G = ThinTGeom<D>;
    static_assert(G::LDS_BYTES <= 80 * 1024, "two workgroups per compute unit");
    p.n_row_blocks = count_row_blocks(p.Lt, G::BM, p.row_stride);
    p.n_col_chunks = 1;
    const int64_t blocks = (int64_t)p.B * p.H * p.n_row_blocks;
    if (blocks > 0x7ffffff0) return 0;
    p.total = (int)blocks;
    static uint64_t reserved = 0;
    // (one register set: with two or three the pieces are requested earlier, but loads return in order, so a wavefront that
    // waits for its x rows waits for every piece requested before them anyway, and the registers are missed: +10-15 %)
    auto kern = spmm_t_thin_kernel<T, D, 1>;
    if (int rc = reserve_dynamic_lds(&reserved, reinterpret_cast<const void*>(kern), G::LDS_BYTES, who)) return rc;
    const int grid = ((p.total + 7) / 8) * 8;
    kern<<<grid, 512, G::LDS_BYTES, st>>>(p);
    return 1;
}

int launch_spmm_t_thin(const char* who, const SpmmTParams& p, int in_dtype, hipStream_t st) {
    if (!p.plan_t) return 0;  // this kernel starts from the transposed mask's plan table
    if (in_dtype == SPLAT_F32 || p.out_dtype != in_dtype) return 0;
    if (p.n_out != 64 && p.n_out != 128) return 0;
    if (!p.x_vec || !p.out_vec) return 0;
    if (p.T < 8) return 0;
    // (every row's first column is read as such, whatever the row's count)
    for (int k = 0; k < p.n_seg; ++k)
        if (!p.seg[k].first_col) return 0;
    auto by_d = [&](auto t) {
        using TT = decltype(t);
        return p.n_out == 128 ? launch_thin_t_variant<TT, 128>(who, p, st) : launch_thin_t_variant<TT, 64>(who, p, st);
    };
    return in_dtype == SPLAT_BF16 ? by_d(bf16{}) : by_d(f16{});
}

}  // namespace splat
