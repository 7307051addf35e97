// SpMM on ACSR for 16-bit launches with the mask's plan table, except those that spmm_thin.hip's rings take (long rows on
// 16-byte boundaries in a compressed matrix larger than the last-level cache): probabilities, V and output of one type, 64 or
// 128 output columns.
//
// A workgroup of 8 wavefronts owns 128 rows of one (batch, head) and walks their key positions in steps of 64 as the
// table lists them.  Per step the whole workgroup loads every row's 64 entries (8 pieces of 8 consecutive slots, 16 bytes
// each at any alignment, cleared outside the row's span with a mask from a table in LDS; every load is issued whatever
// the values, so that none waits for another) into an LDS tile [row][position] and the V rows into a tile [key][feature]
// beside it, a step ahead through registers, two stages, one barrier per step.  A wavefront owns 32 rows and half of the
// features and accumulates O^T = V^T P^T with 16x16x32 MFMAs: the B operands are 16-byte row reads of the probability tile
// (chunks permuted by the row so that a read covers all banks), the A operands transposing reads of the V tile (layout of
// spmm_thin.hip).  Plans whose rows step differently walk dense columns and gather element by element under the row's
// affine test.  The output leaves through an LDS turn-around as whole rows, non-temporal.
#include <algorithm>
#include <type_traits>

#include "spmm_params.hpp"
#include "tile_copy.hpp"

namespace splat {

template <int D>
struct PTileGeom {
    static constexpr int BM = 128;
    static constexpr int ROWB = D * 2;             // bytes per V row
    static constexpr int P_ROWB = kBN * 2;         // bytes per row of the probability tile: 64 positions
    static constexpr int V_STAGE = kBN * ROWB;     // the V tile comes first in a stage
    static constexpr int STAGE = V_STAGE + BM * P_ROWB;
    static constexpr int O_ROW = ROWB + 16;
    static constexpr int TILE_BYTES = 2 * STAGE > BM * O_ROW ? 2 * STAGE : BM * O_ROW;
    static constexpr int MASK_AT = TILE_BYTES;
    static constexpr int LDS_BYTES = MASK_AT + 81 * 16;
};

template <typename T, int D>
__global__ __launch_bounds__(512, 4) void spmm_tile_kernel(const SpmmParams p) {
    using G = PTileGeom<D>;
    constexpr int BM = G::BM, ROWB = G::ROWB, P_ROWB = G::P_ROWB, V_STAGE = G::V_STAGE, STAGE = G::STAGE, O_ROW = G::O_ROW;
    constexpr int CPR = ROWB / 16;
    constexpr int NI = kBN * CPR / 512;
    constexpr int DT = D / 16;
    constexpr int FD = DT / 2;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const u32x4* const s_mask = reinterpret_cast<const u32x4*>(smem + G::MASK_AT);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, g4 = lane >> 4;
    const int cg = wave & 3, fh = wave >> 2;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int bh = logical / p.n_row_blocks;
    const int rb = logical % p.n_row_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L;

    const char* vbytes = reinterpret_cast<const char*>((const T*)p.v + b * p.v_sb + h * p.v_sh);
    const int64_t v_rowb = p.v_sl * 2;
    const T* pb = (const T*)p.p + (int64_t)bh * L * p.T;
    const PlanRec* const pt = p.plan;
    const int n_rb = p.n_row_blocks;
    // the only rows whose neighbours in memory may lie outside the buffer
    const bool first_bh = bh == 0, last_bh = bh == p.B * p.H - 1;

    // mask [lo][hi]: entries lo .. 7 - hi of a piece kept
    if (tid < 81) {
        const int lo = tid / 9, hi = tid % 9;
        const u32x4 ones = {~0u, ~0u, ~0u, ~0u};
        *reinterpret_cast<u32x4*>(smem + G::MASK_AT + tid * 16) = shift_elements(ones, lo) & shift_elements(ones, -hi);
    }
    lds_barrier();

    // this thread's chunks of every V tile: from key row v_row, 16 bytes at v_col, to LDS offset v_lds of the stage
    int v_row[NI], v_col[NI], v_lds[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int id = tid + 512 * i;
        v_row[i] = id / CPR;
        v_col[i] = (id % CPR) * 16;
        v_lds[i] = v_row[i] * ROWB + v_chunk<ROWB>(v_row[i], id % CPR) * 16;
    }
    // this thread's pieces of every probability tile: block row prow, positions 8 (pq + 4 c) .. + 7 of the step, c = 0, 1;
    // chunk c of row r sits at physical chunk c ^ ((r >> 1) & 7): the 16 rows x 4 chunks of a fragment read cover all banks
    const int prow = tid >> 2, pq = tid & 3;
    const int my_row = r0 + rs * prow;
    int p_lds[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) p_lds[c] = V_STAGE + prow * P_ROWB + (((pq + 4 * c) ^ ((prow >> 1) & 7)) << 4);

    // A wavefront owns 32 of the block's rows (two B operands, cb) and half of the features (FD A operands): every fragment
    // read from LDS serves two MFMAs or FD of them.  B: lane (row li of the 16, positions 8 g4 .. + 7 of half step hf); A: lane s
    // of 16-lane block g4 addresses key row 8 g4 + s / 4 (and 4 rows on) and the 4 features 16 dt + 4 (s % 4)
    int v_off[FD], p_off[2][2];   // [cb][hf]
    {
        const int sq = li >> 2;
        const int in_half = 16 * ((li & 3) >> 1) + 8 * (li & 1);
        const int blk = ROWB >= 256 ? sq : (sq >> 1);
#pragma unroll
        for (int fd = 0; fd < FD; ++fd) {
            const int dt = FD * fh + fd;
            v_off[fd] = (8 * g4 + sq) * ROWB + in_half + 64 * ((dt >> 1) ^ blk) + 32 * ((dt & 1) ^ (g4 & 1));
        }
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int r = 32 * cg + 16 * cb + li;
                p_off[cb][hf] = V_STAGE + r * P_ROWB + (((4 * hf + g4) ^ ((r >> 1) & 7)) << 4);
            }
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
        if (n_steps == 0) continue;
        const int off = p.seg[sg].slot_offset;
        const bool uniform = pl.uniform != 0;
        // the row whose pieces this thread loads (counts are clamped to the slots the segment owns in this buffer, like the
        // ones read from the metadata)
        RowWin mine;
        {
            const PlanRec r = pt[plan_row_at(n_rb, p.n_seg, rb, sg, prow)];
            const int64_t most = uniform ? (int64_t)p.seg[sg].max_cnt : (int64_t)r[2] * (p.seg[sg].max_cnt - 1) + 1;
            mine = RowWin{r[0], (int)min((int64_t)r[1], most), r[2]};
        }
        if (my_row >= L) mine.cnt = 0;
        // key positions in which some of this wavefront's 32 rows have an entry
        int lmin, hmax;
        {
            const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, sg, cg));
            lmin = r[0], hmax = r[3];
        }
        auto act = [&](int pos0) { return !(pos0 + 32 <= lmin || pos0 >= hmax); };
        const int row_c = min(my_row, L - 1);
        const T* const prow_p = pb + (int64_t)row_c * p.T + off;
        const bool risky = (first_bh && row_c == 0) || (last_bh && row_c == L - 1);

        auto load_v = [&](int s, u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int n = min(max(pl.c0 + pl.cs * (s * kBN + v_row[i]), 0), p.n_keys - 1);
                reg[i] = *reinterpret_cast<const u32x4*>(vbytes + n * v_rowb + v_col[i]);
            }
        };
        auto write_v = [&](int stage, const u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<u32x4*>(smem + stage * STAGE + v_lds[i]) = reg[i];
        };
        auto write_p = [&](int stage, const u32x4 (&reg)[2]) {
#pragma unroll
            for (int c = 0; c < 2; ++c) *reinterpret_cast<u32x4*>(smem + stage * STAGE + p_lds[c]) = reg[c];
        };
        // This thread's two pieces of step s.  A piece that straddles an end of the row's span is loaded like any other, as 16
        // bytes from where its first entry would be, and the entries outside the span are cleared: what lies there (dead slots,
        // the neighbouring row) is readable memory except before the first and after the last row of the buffer, whose pieces
        // are loaded from inside the row and shifted.  (Steps past the last one hold nothing of any row: nothing is read.)
        auto load_probs = [&](int s, u32x4 (&out)[2]) {
            if (uniform) {
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const int u = s * kBN + 8 * (pq + 4 * c) - mine.lo;
                    const bool touches = u + 8 > 0 && u < mine.cnt;
                    const int u_ld = risky ? min(max(u, -off), p.T - off - 8) : u;
                    const T* src_p = touches ? prow_p + u_ld : pb;  // (the buffer's first 16 bytes: any readable address)
                    u32x4 raw;
                    __builtin_memcpy(&raw, src_p, 16);  // any alignment
                    if (u_ld != u) raw = shift_elements(raw, u_ld - u);
                    out[c] = raw & s_mask[min(max(-u, 0), 8) * 9 + min(max(u + 8 - mine.cnt, 0), 8)];
                }
            } else {
                typedef T vec8 __attribute__((ext_vector_type(8)));
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    vec8 v;
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = (T)0.f;
                    if (mine.cnt > 0) v = gather_affine8<vec8>(prow_p, mine, s * kBN + 8 * (pq + 4 * c));
                    out[c] = __builtin_bit_cast(u32x4, v);
                }
            }
        };

        // ---- prologue: tile 0 into stage 0, tile 1 requested (everyone has left both stages at the barrier that ended the
        // segment before)
        u32x4 vreg[NI];
        u32x4 praw[2];
        load_v(0, vreg);
        load_probs(0, praw);
        write_v(0, vreg);
        write_p(0, praw);
        if (n_steps > 1) load_v(1, vreg);
        load_probs(1, praw);
        lds_barrier();

        auto step = [&](int s, auto par_c) {
            constexpr int par = decltype(par_c)::value;
            // tile s + 1 into the other stage (everyone has left it at the barrier that ended step s - 1), tile s + 2 requested
            // into the registers this frees.  (One register set: loads return in order, so requesting the probabilities
            // earlier than the V rows of the same tile buys nothing.)
            if (s + 1 < n_steps) {
                write_v(par ^ 1, vreg);
                write_p(par ^ 1, praw);
                if (s + 2 < n_steps) load_v(s + 2, vreg);
            }
            load_probs(s + 2, praw);
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int pos0 = s * kBN + 32 * hf;
                if (!act(pos0)) continue;  // wavefront-uniform
                Frag<T> pf[2];
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
                    pf[cb].v = __builtin_bit_cast(typename Frag<T>::vec, *reinterpret_cast<const u32x4*>(smem + p_off[cb][hf] + par * STAGE));
#pragma unroll
                for (int fd = 0; fd < FD; ++fd) {
                    const char* a = smem + v_off[fd] + (par * STAGE + 32 * hf * ROWB);
                    const Frag<T> vf = frag_from_tr<T>(lds_tr16(a), lds_tr16(a + 4 * ROWB));
                    mma16(acc[fd][0], vf, pf[0]);
                    mma16(acc[fd][1], vf, pf[1]);
                }
            }
            lds_barrier();
        };
        for (int s = 0; s < n_steps; s += 2) {
            step(s, std::integral_constant<int, 0>{});
            if (s + 1 < n_steps) step(s + 1, std::integral_constant<int, 1>{});
        }
    }

    // ---- output: O^T accumulators (lane: row 32 cg + 16 cb + li, features 16 (FD fh + fd) + 4 g4 .. + 3) turned around in
    // LDS, rows stored whole (every wavefront has passed the last barrier of the loop: the tiles are free)
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
        const int r = r0 + rs * (16 * wave + row);
        const u32x4 val = *reinterpret_cast<const u32x4*>(o_stg + row * O_ROW + c * 16);
        if (r < L) {
            char* orow = reinterpret_cast<char*>(p.out) + ((int64_t)bh * L + r) * ROWB;
            __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(orow + c * 16));
        }
    }
}

template <typename T, int D>
static int launch_tile_variant(const char* who, SpmmParams p, hipStream_t st) {
    using G = PTileGeom<D>;
    static_assert(G::LDS_BYTES <= 80 * 1024, "two workgroups per compute unit");
    p.n_row_blocks = count_row_blocks(p.L, G::BM, p.row_stride);
    p.n_col_chunks = 1;
    const int64_t blocks = (int64_t)p.B * p.H * p.n_row_blocks;
    if (blocks > 0x7ffffff0) return 0;
    p.total = (int)blocks;
    static uint64_t reserved = 0;
    auto kern = spmm_tile_kernel<T, D>;
    if (int rc = reserve_dynamic_lds(&reserved, reinterpret_cast<const void*>(kern), G::LDS_BYTES, who)) return rc;
    const int grid = ((p.total + 7) / 8) * 8;
    kern<<<grid, 512, G::LDS_BYTES, st>>>(p);
    return 1;
}

int launch_spmm_tile(const char* who, const SpmmParams& p, int in_dtype, hipStream_t st) {
    if (!p.plan) return 0;  // this kernel starts from the mask's plan table
    if (in_dtype == SPLAT_F32 || p.out_dtype != in_dtype) return 0;
    if (p.n_out != 64 && p.n_out != 128) return 0;
    if (!p.v_vec || !p.out_vec) return 0;
    // a thread reads 16 bytes at a time from inside its row's share of a segment
    if (p.T < 8) return 0;
    for (int k = 0; k < p.n_seg; ++k)
        if (p.seg[k].max_cnt < 8) return 0;
    auto by_d = [&](auto t) {
        using TT = decltype(t);
        return p.n_out == 128 ? launch_tile_variant<TT, 128>(who, p, st) : launch_tile_variant<TT, 64>(who, p, st);
    };
    return in_dtype == SPLAT_BF16 ? by_d(bf16{}) : by_d(f16{});
}

}  // namespace splat
