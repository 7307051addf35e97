// SpMM on ACSR for 16-bit launches with long rows and a compressed matrix larger than the last-level
// cache: probabilities, V and output of one type, 64 or 128 output columns, 16-byte alignment,
// rows of at least 256 slots that start on 16-byte boundaries of the buffer, more than 192 MB of probabilities, the mask's
// plan table.  (Everything else with a plan table: spmm_tile.hip.)
//
// A workgroup of 8 wavefronts owns 128 rows of one (batch, head); wavefront w owns rows 16w..16w+15 and accumulates
// O^T = V^T P^T with 16x16x32 MFMAs (rows = output columns, columns = queries: a lane owns one query row).  Thin
// wavefronts stay below 128 registers, so that four of them share a SIMD and cover each other's waits.
//
// The B operand needs, per lane, 8 consecutive key positions of the lane's own row: with a uniform plan these are 8
// consecutive compressed slots.  A wavefront fetches its rows' slots as whole aligned 128-byte lines (non-temporal: they
// stream past the L2, where V stays), two steps ahead through registers into per-row rings of two
// lines in LDS, and every fragment is the funnel shift of two aligned 16-byte chunks of the lane's ring.  A wavefront
// whose rows all start on multiples of 8 positions (blocked masks) skips the rings: its fragments are aligned 16-byte
// loads straight from memory.  Other plans walk dense columns and gather element by element under the row's affine test.
//
// V tiles of 64 keys go through registers into one of two LDS stages (written a step ahead, one barrier per step), 64-byte
// blocks and their halves permuted so that the transposing reads of the A operand -- a lane block reads 4 key rows x
// 16 columns -- spread over all banks.  The output leaves through an LDS turn-around as whole rows, non-temporal.
#include <algorithm>
#include <type_traits>

#include "spmm_params.hpp"
#include "tile_copy.hpp"

namespace splat {

template <int D>
struct ThinGeom {
    static constexpr int BM = 128;
    static constexpr int ROWB = D * 2;            // bytes per V row
    static constexpr int STAGE = kBN * ROWB;      // bytes per V tile
    static constexpr int O_ROW = ROWB + 16;       // bytes per row of the output turn-around
    static constexpr int TILES_AT = 0;
    static constexpr int TILE_BYTES = 2 * STAGE > BM * O_ROW ? 2 * STAGE : BM * O_ROW;
    static constexpr int R_ROW = 128 * 2 + 16;     // bytes per row of the probability rings: two lines of 64 slots
    static constexpr int RING_AT = TILE_BYTES;
    static constexpr int LDS_BYTES = RING_AT + BM * R_ROW;
};

// NB: register sets for probabilities in flight: requested NB steps (rings) or NB - 1 steps (straight from memory) ahead
template <typename T, int D, int NB>
__global__ __launch_bounds__(512, 4) void spmm_thin_kernel(const SpmmParams p) {
    using G = ThinGeom<D>;
    constexpr int R_ROW = G::R_ROW;
    constexpr int BM = G::BM, ROWB = G::ROWB, STAGE = G::STAGE, O_ROW = G::O_ROW;
    constexpr int CPR = ROWB / 16;        // 16-byte chunks per V row
    constexpr int NI = kBN * CPR / 512;   // chunks of a V tile per thread
    constexpr int DT = D / 16;            // 16-column blocks of the output
    static_assert(NI >= 1 && G::RING_AT % 16 == 0, "tile shape");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char* const s_v = smem;
    char* const s_rings = smem + G::RING_AT;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, g4 = lane >> 4;

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

    const int my_rr = 16 * wave + li;
    const int my_r = r0 + rs * my_rr;

    // this thread's chunks of every V tile: from key row v_row, 16 bytes at v_col, to LDS offset v_lds of the stage
    int v_row[NI], v_col[NI], v_lds[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int id = tid + 512 * i;
        v_row[i] = id / CPR;
        v_col[i] = (id % CPR) * 16;
        v_lds[i] = v_row[i] * ROWB + v_chunk<ROWB>(v_row[i], id % CPR) * 16;
    }
    // A operand (V^T), 16-column block dt: lane s of 16-lane block g4 addresses key row 8 g4 + s / 4 (and 4 rows on) and
    // the 4 columns 16 dt + 4 (s % 4) through the transposing read
    int v_off[DT];
    {
        const int sq = li >> 2;
        const int base = (8 * g4 + sq) * ROWB + 16 * ((li & 3) >> 1) + 8 * (li & 1);
        const int blk = ROWB >= 256 ? sq : (sq >> 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_off[dt] = base + 64 * ((dt >> 1) ^ blk) + 32 * ((dt & 1) ^ (g4 & 1));
    }

    f32x4v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[dt][j] = 0.f;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        SegPlan pl;
        {
            const PlanRec r = plan_uniform_load(pt + plan_seg_at(p.n_seg, rb, sg));
            pl = SegPlan{r[0], r[1], r[2], r[3]};
        }
        const int n_steps = pl.n_tiles;
        if (n_steps == 0) continue;  // workgroup-uniform
        const int off = p.seg[sg].slot_offset;
        const bool uniform = pl.uniform != 0;

        RowWin mine;
        {
            // (counts are clamped to the slots the segment owns in this buffer, like the ones read from the metadata)
            const PlanRec r = pt[plan_row_at(n_rb, p.n_seg, rb, sg, my_rr)];
            const int64_t most = uniform ? (int64_t)p.seg[sg].max_cnt : (int64_t)r[2] * (p.seg[sg].max_cnt - 1) + 1;
            mine = RowWin{r[0], (int)min((int64_t)r[1], most), r[2]};
        }
        if (my_r >= L) mine.cnt = 0;
        WaveSpan span;
        {
            // the table holds the spans of 32 rows: wider than this wavefront's 16, which only makes the tests below pass less often
            const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, sg, wave >> 1));
            span = WaveSpan{r[0], r[1], r[2], r[3]};
        }
        const int lmin = span.lo_min, hmax = span.hi_max;
        const T* const prow = pb + (int64_t)min(my_r, L - 1) * p.T + off;
        // where a lane may read 16 bytes of its row: slots 0 .. row_last8 (the segment owns at least 8 slots of every row)
        const int row_last8 = p.seg[sg].max_cnt - 8;

        // Half steps: 32 positions from pos0 on.  `act`: some row of the wavefront has a position there; `full`: every row
        // has all of them.
        auto act = [&](int pos0) { return !(pos0 + 32 <= lmin || pos0 >= hmax); };
        auto full = [&](int pos0) { return pos0 >= span.lo_max && pos0 + 32 <= span.hi_min; };
        // ---- rings: the rows whose lines this lane fetches (8 lanes per row, 8 rows per instruction: two instructions
        // cover the wavefront's 16 rows; the two rows of 16 consecutive lanes are 8 apart, half the banks apart in the ring)
        // Step t needs slots 64 t - lo .. + 63 of a row, which lie in lines t + la and t + la + 1 (la = -ceil(lo / 64), a
        // line = 64 slots from the row's first): line t + la + 1 is requested NB steps ahead, written into the ring (line
        // index modulo 2) at the start of step t, over the line that step t - 1 was the last to need.
        int f_rr[2], f_la[2], f_cnt[2];
        const T* f_row[2];
        const int f_piece = lane & 7;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            f_rr[c] = 16 * wave + 4 * c + (lane >> 4) + 8 * ((lane >> 3) & 1);
            const PlanRec rec = pt[plan_row_at(n_rb, p.n_seg, rb, sg, f_rr[c])];
            const RowWin w = RowWin{rec[0], min(rec[1], p.seg[sg].max_cnt), rec[2]};
            const int r = r0 + rs * f_rr[c];
            f_la[c] = -((w.lo + 63) >> 6);
            f_cnt[c] = (r < L && uniform) ? w.cnt : 0;
            f_row[c] = pb + (int64_t)min(r, L - 1) * p.T + off;
        }
        // the 16 bytes of line t + la + 1 this lane fetches for row c (zeros where the line has nothing of the row)
        auto load_line = [&](int t, int c) {
            u32x4 raw = {0u, 0u, 0u, 0u};
            const int slot = 64 * (t + f_la[c] + 1) + 8 * f_piece;
            if (slot >= 0 && slot < f_cnt[c]) {  // 16-byte aligned
                // (this kernel's compressed matrices are too large for the last-level cache: they stream past the L2, where V stays)
                raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(f_row[c] + slot));
            }
            return raw;
        };
        auto write_line = [&](int t, int c, const u32x4& raw) {
            *reinterpret_cast<u32x4*>(s_rings + f_rr[c] * R_ROW + ((t + f_la[c] + 1) & 1) * 128 + f_piece * 16) = raw;
        };
        // The 8 entries at positions pos0 + 8 g4 .. + 7 of this lane's row out of its ring: slot s sits at ring element
        // s % 128, so the entries start k = -lo % 8 elements into an aligned 16-byte chunk; the two chunks around them are
        // read whole and shifted.
        const int ring_k = (-mine.lo) & 7;
        const char* const ring_mine = s_rings + my_rr * R_ROW;
        auto ring_frag = [&](int pos0) {
            const int u = pos0 + 8 * g4 - mine.lo;
            const int q = (u >> 3) & 15;
            const u32x4 a = *reinterpret_cast<const u32x4*>(ring_mine + q * 16);
            const u32x4 b = *reinterpret_cast<const u32x4*>(ring_mine + ((q + 1) & 15) * 16);
            const bool b1 = (ring_k & 2) != 0, b2 = (ring_k & 4) != 0;
            const uint32_t y0 = b1 ? a[1] : a[0], y1 = b1 ? a[2] : a[1], y2 = b1 ? a[3] : a[2], y3 = b1 ? b[0] : a[3];
            const uint32_t y4 = b1 ? b[1] : b[0], y5 = b1 ? b[2] : b[1], y6 = b1 ? b[3] : b[2];
            const uint32_t x0 = b2 ? y2 : y0, x1 = b2 ? y3 : y1, x2 = b2 ? y4 : y2, x3 = b2 ? y5 : y3, x4 = b2 ? y6 : y4;
            const uint32_t sh = (ring_k & 1) ? 16u : 0u;
            u32x4 raw;
            raw[0] = __builtin_amdgcn_alignbit(x1, x0, sh);
            raw[1] = __builtin_amdgcn_alignbit(x2, x1, sh);
            raw[2] = __builtin_amdgcn_alignbit(x3, x2, sh);
            raw[3] = __builtin_amdgcn_alignbit(x4, x3, sh);
            if (!full(pos0)) {  // wavefront-uniform: zero what lies outside the row's span
                const int low = min(max(-u, 0), 8), high = min(max(u + 8 - mine.cnt, 0), 8);
                const u32x4 ones = {~0u, ~0u, ~0u, ~0u};
                raw &= shift_elements(ones, low) & shift_elements(ones, -high);
            }
            Frag<T> f;
            f.v = __builtin_bit_cast(typename Frag<T>::vec, raw);
            return f;
        };

        auto load_v = [&](int s, u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int n = min(max(pl.c0 + pl.cs * (s * kBN + v_row[i]), 0), p.n_keys - 1);
                reg[i] = *reinterpret_cast<const u32x4*>(vbytes + n * v_rowb + v_col[i]);
            }
        };
        auto write_v = [&](int stage, const u32x4 (&reg)[NI]) {
#pragma unroll
            for (int i = 0; i < NI; ++i) *reinterpret_cast<u32x4*>(s_v + stage * STAGE + v_lds[i]) = reg[i];
        };
        // Straight from memory (wavefronts whose rows all start on multiples of 8 positions: every piece is 16-byte aligned): the
        // 8 entries at positions pos0 + 8 g4 .. + 7 of this lane's row as they come from memory -- the slots themselves where
        // the half step is full, else the 8 slots of the row nearest to them.
        auto load_p = [&](int pos0) {
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (!uniform || !act(pos0)) return raw;
            const int u = pos0 + 8 * g4 - mine.lo;
            if (full(pos0)) {
                __builtin_memcpy(&raw, prow + u, 16);
            } else {
                const int uc = min(max(u, 0), max(min(mine.cnt - 8, row_last8), 0));
                __builtin_memcpy(&raw, prow + uc, 16);
            }
            return raw;
        };
        // ... and as the B operand wants them: entry e is slot u + e, zero outside the row's span
        auto fix_p = [&](u32x4 raw, int pos0) {
            Frag<T> f;
            if (uniform) {
                if (!full(pos0)) {
                    const int u = pos0 + 8 * g4 - mine.lo;
                    const int uc = min(max(u, 0), max(min(mine.cnt - 8, row_last8), 0));
                    raw = shift_elements(raw, uc - u);
                    const int low = min(max(-u, 0), 8), high = min(max(u + 8 - mine.cnt, 0), 8);  // dead entries at either end
                    const u32x4 ones = {~0u, ~0u, ~0u, ~0u};
                    const u32x4 keep = shift_elements(ones, low) & shift_elements(ones, -high);
                    raw &= keep;
                }
            } else {
                typedef T vec8 __attribute__((ext_vector_type(8)));
                vec8 v;
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (T)0.f;
                if (mine.cnt > 0) v = gather_affine8<vec8>(prow, mine, pos0 + 8 * g4);
                raw = __builtin_bit_cast(u32x4, v);
            }
            f.v = __builtin_bit_cast(typename Frag<T>::vec, raw);
            return f;
        };

        // ---- prologue: V tile 0 into stage 0, V tile 1 and the probabilities of the first steps requested
        // Rings pay where rows start inside a 16-byte chunk of their positions' grid; a wavefront whose rows all start on
        // one (blocked masks) reads its aligned chunks straight from memory.  Wavefront-uniform: the rings are private.
        const bool ring = uniform && __any((mine.lo & 7) != 0 && mine.cnt > 0);
        u32x4 vreg[NI];
        u32x4 praw[NB][2];  // [step modulo NB][half (direct loads) or row (rings)]
        load_v(0, vreg);
        if (ring) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const u32x4 first = load_line(-1, c), second = load_line(0, c);
                write_line(-1, c, first);
                write_line(0, c, second);
            }
            static_for<NB>([&](auto u) {
                constexpr int k = decltype(u)::value;
                if constexpr (k >= 1) {
                    praw[k][0] = load_line(k, 0);
                    praw[k][1] = load_line(k, 1);
                }
            });
        } else {
            static_for<NB - 1>([&](auto u) {
                constexpr int k = decltype(u)::value;
                praw[k][0] = load_p(k * kBN);
                praw[k][1] = load_p(k * kBN + 32);
            });
        }
        write_v(0, vreg);
        if (n_steps > 1) load_v(1, vreg);
        lds_barrier();

        auto step = [&](int s, auto idx_c) {
            constexpr int idx = decltype(idx_c)::value;  // s modulo UNROLL
            constexpr int par = idx & 1, ri = idx % NB, rn = (idx + NB - 1) % NB;
            // tile s + 1 into the other stage (everyone has left it at the barrier that ended step s - 1), tile s + 2 and
            // the probabilities of a later step requested: into the registers step s - 1 has freed, or, with rings, into
            // those of this step once their line is in the ring
            if (s + 1 < n_steps) {
                write_v(par ^ 1, vreg);
                if (s + 2 < n_steps) load_v(s + 2, vreg);
            }
            if (ring) {
                if (s >= 1) {
                    write_line(s, 0, praw[ri][0]);
                    write_line(s, 1, praw[ri][1]);
                }
                praw[ri][0] = load_line(s + NB, 0);
                praw[ri][1] = load_line(s + NB, 1);
            }
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int pos0 = s * kBN + 32 * hf;
                if (!act(pos0)) continue;  // wavefront-uniform
                const Frag<T> pf = ring ? ring_frag(pos0) : fix_p(praw[ri][hf], pos0);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const char* a = s_v + v_off[dt] + (par * STAGE + 32 * hf * ROWB);
                    const Frag<T> vf = frag_from_tr<T>(lds_tr16(a), lds_tr16(a + 4 * ROWB));
                    mma16(acc[dt], vf, pf);
                }
            }
            if (!ring) {  // (kept out of the way of the ring path's schedule: after the products; nothing is read of steps past the last one: they are not active)
                praw[rn][0] = load_p((s + NB - 1) * kBN);
                praw[rn][1] = load_p((s + NB - 1) * kBN + 32);
            }
            lds_barrier();
        };
        // the unrolled steps make the stage (s % 2) and the register set (s % NB) compile-time constants
        static_assert(NB >= 2, "register sets");
        constexpr int UNROLL = NB % 2 == 0 ? NB : 2 * NB;
        for (int s = 0; s < n_steps; s += UNROLL) {
            static_for<UNROLL>([&](auto u) {
                if (s + decltype(u)::value < n_steps) step(s + decltype(u)::value, u);
            });
        }
    }

    // ---- output: O^T accumulators (lane: query li, columns 16 dt + 4 g4 .. + 3) turned around in LDS, rows stored whole
    // (every wavefront has passed the last barrier of the loop: the tiles are free)
    char* const o_stg = smem + (16 * wave) * O_ROW;
    typedef T v4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        v4 t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = (T)acc[dt][j];
        *reinterpret_cast<v4*>(o_stg + li * O_ROW + (16 * dt + 4 * g4) * 2) = t;
    }
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
static int launch_thin_variant(const char* who, SpmmParams p, hipStream_t st) {
    using G = ThinGeom<D>;
    static_assert(G::LDS_BYTES <= 80 * 1024, "two workgroups per compute unit");
    p.n_row_blocks = count_row_blocks(p.L, G::BM, p.row_stride);
    p.n_col_chunks = 1;
    const int64_t blocks = (int64_t)p.B * p.H * p.n_row_blocks;
    if (blocks > 0x7ffffff0) return 0;
    p.total = (int)blocks;
    static uint64_t reserved = 0;
    // (two register sets: more request the lines earlier, which buys nothing -- loads return in order, and the wait for a
    // step's V rows covers every line requested before them -- and costs registers: d = 64 with 3 / 4 / 6 sets is 2 / 5 / 20 %
    // slower, d = 128 spills with 3)
    auto kern = spmm_thin_kernel<T, D, 2>;
    if (int rc = reserve_dynamic_lds(&reserved, reinterpret_cast<const void*>(kern), G::LDS_BYTES, who)) return rc;
    const int grid = ((p.total + 7) / 8) * 8;
    kern<<<grid, 512, G::LDS_BYTES, st>>>(p);
    return 1;
}

int launch_spmm_thin(const char* who, const SpmmParams& p, int in_dtype, hipStream_t st) {
    if (!p.plan) return 0;  // this kernel starts from the mask's plan table
    if (in_dtype == SPLAT_F32 || p.out_dtype != in_dtype) return 0;
    if (p.n_out != 64 && p.n_out != 128) return 0;
    if (!p.v_vec || !p.out_vec) return 0;
    // a lane reads 16 bytes at a time from inside its row's share of a segment
    for (int k = 0; k < p.n_seg; ++k)
        if (p.seg[k].max_cnt < 8) return 0;
    // Rings: rows of the compressed matrix start on 16-byte boundaries, are long, and the matrix is too large for the 256 MB
    // last-level cache, so that whole lines fetched with non-temporal loads stream past the L2, where V stays (config 4's
    // 537 MB: 0.184 ms against 0.218 for the workgroup-wide tile of spmm_tile.hip).  A matrix that repeated launches find in
    // that cache (config 2's 134 MB), rows of one or two lines and rows anywhere else are better off with the tile (-7 to
    // -10 %).
    bool ring = (reinterpret_cast<uintptr_t>(p.p) & 15) == 0 && p.T % 8 == 0 && p.T >= 256 &&
                (int64_t)p.B * p.H * p.L * p.T * 2 > ((int64_t)192 << 20);
    for (int k = 0; k < p.n_seg; ++k)
        if (p.seg[k].slot_offset % 8 != 0) ring = false;
    if (!ring) return launch_spmm_tile(who, p, in_dtype, st);
    auto by_d = [&](auto t) {
        using TT = decltype(t);
        return p.n_out == 128 ? launch_thin_variant<TT, 128>(who, p, st) : launch_thin_variant<TT, 64>(who, p, st);
    };
    return in_dtype == SPLAT_BF16 ? by_d(bf16{}) : by_d(f16{});
}

}  // namespace splat
