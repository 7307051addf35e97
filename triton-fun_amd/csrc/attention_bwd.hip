// Fused backward of the ACSR attention: dQ, dK and dV without any compressed [B, H, L, T] matrix in memory.
//
// With S = scale * Q K^T on the live columns, P = exp(S - lse) (lse: the forward's row statistic), O = P V and the
// upstream gradient dO:  D = rowsum(dO * O),  dP = dO V^T,  dS = P * (dP - D),
//     dQ = scale * dS K        dK = scale * dS^T Q        dV = P^T dO.
// One kernel, four modes (d = 128: dQ, dK, dV, 8 products; d = 64: dQ, dK+dV, 7), built like the forward (attention.hip): a workgroup of 4 wavefronts owns 128 "rows", one
// lane one row (two lanes share it), and walks 64-position tiles of the rows' spans as the mask's plan table lists
// them; per tile two operand tiles X and Y arrive in LDS through the asynchronous copy ring.
//
//   mode  rows     positions  registers A, B   tile X   tile Y   per 32-position half
//   dQ    queries  keys       Q, dO            K        V        S^T = X A^T; P; dP^T = Y B^T; dS; acc^T += X^T dS^T
//   dK    keys     queries    K, V             Q        dO       the same with the mask's transpose
//   dV    keys     queries    K                Q        dO       S^T = X A^T; P;                 acc^T += Y^T P^T
//   dK+dV keys     queries    K, V             Q        dO       as dK, and acc2^T += Y^T P^T    (d = 64: both accumulators fit)
//
// dQ walks the mask's own plan, dK and dV the plan of the transposed mask (keys as rows).  The dQ launch comes first: its
// lanes hold their dO rows, so it also computes D (one more read of the lane's O row) and stores it for the other two.  lse
// and D belong to the queries: one value per lane in dQ, one per tile position otherwise (64 floats each per tile, copied into LDS beside
// the tiles).  The X tile of dQ / dK is read row-wise (16-byte fragments for S^T) and through the transposing read
// (for acc^T), hence the swizzle that serves both (tile_copy.hpp: dual_chunk).  Probabilities come straight from the
// statistic: no running maximum, no rescale, no second pass.  16-bit types, d = 64 or 128, rows of every operand
// contiguous.
#include <initializer_list>

#include "attn_tile.hpp"

namespace splat {

typedef float f32x4 __attribute__((ext_vector_type(4)));

enum { kBwdDQ = 0, kBwdDK = 1, kBwdDV = 2, kBwdDKV = 3 };

struct BwdParams {
    const void* a;  // register operand A, one row per lane: Q (dQ), K (dK, dV)
    const void* b;  // register operand B: dO (dQ), V (dK); unused (dV)
    const void* x;  // tile operand X: K (dQ), Q (dK, dV)
    const void* y;  // tile operand Y: V (dQ), dO (dK, dV)
    void* out;      // dQ, dK, dV
    void* out2;     // dK + dV in one launch: dV (same strides as out)
    int64_t a_sb, a_sh, a_sl, b_sb, b_sh, b_sl, x_sb, x_sh, x_sl, y_sb, y_sh, y_sl, o_sb, o_sh, o_sl;
    const float* lse;    // [B*H, L], natural log, per query
    const float* delta;  // [B*H, L], D per query (dK, dV: written by the dQ launch before them on the stream)
    const void* o;       // dQ only: the forward's output, from which that launch computes D = rowsum(dO * O) ...
    int64_t oo_sb, oo_sh, oo_sl;
    float* delta_w;      // ... and where it stores it
    int B, H, L;
    int Lr;               // rows of the launch: L, or the number of rows of a rectangular keys' side (dK, dV of selected keys)
    const int* row_map;   // [Lr] or null: the row of A / B that row r of the mask stands for (r itself when null)
    float scale, scale_log2e;
    int n_seg, n_row_blocks, total, row_stride;
    const PlanRec* plan;  // plan table of the mask (dQ) or of its transpose (dK, dV), first variant
};

template <typename T, int D, int MODE>
__global__ __launch_bounds__(256, 2) void attn_bwd_kernel(const BwdParams p) {
    constexpr int ES = 2, BM = 128, BN = 64;
    static_assert(sizeof(T) == ES, "16-bit element types");
    constexpr int KS = D / 16;  // contraction steps of the products over d
    constexpr int DT = D / 32;  // 32-row tiles of the transposed accumulator
    constexpr int ROWB = D * ES;
    constexpr int TILE = BN * ROWB;             // bytes of one operand tile
    constexpr int STAGE = 2 * TILE;               // X, Y
    constexpr int STATS = 2 * BN * 4;             // lse[64], D[64] of one stage
    constexpr int RING = 2 * STATS;               // both stages' statistics come first, then the ring of tiles
    constexpr int CPR = ROWB / 16, RPI = 1024 / ROWB;  // chunks per row, rows per 1 KiB copy block
    constexpr int NI = TILE / 4096;                   // copy blocks per wavefront and tile
    constexpr int NDMA = 2 * NI;
    constexpr bool POS_STATS = MODE != kBwdDQ;  // lse / D per tile position instead of per lane
    constexpr bool THREE = MODE != kBwdDV;      // the dP and dS steps
    constexpr bool BOTH = MODE == kBwdDKV;      // dK and dV from one walk: a second accumulator, fed with P^T and Y^T

    extern __shared__ __attribute__((aligned(1024))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int bh = logical / p.n_row_blocks;
    const int rb = p.n_row_blocks - 1 - (logical % p.n_row_blocks);
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L;

    const T* ab = (const T*)p.a + b * p.a_sb + h * p.a_sh;
    const T* bb = THREE ? (const T*)p.b + b * p.b_sb + h * p.b_sh : nullptr;
    const T* xb = (const T*)p.x + b * p.x_sb + h * p.x_sh;
    const T* yb = (const T*)p.y + b * p.y_sb + h * p.y_sh;
    T* ob = (T*)p.out + b * p.o_sb + h * p.o_sh;
    const float* lse_b = p.lse + (int64_t)bh * L;
    const float* del_b = p.delta + (int64_t)bh * L;

    // ---- register operands: fragments of this lane's row, resident for the whole kernel ----
    const int Lr = p.Lr;
    int my_row = min(r0 + rs * (wave * 32 + lm), Lr - 1);
    if constexpr (MODE != kBwdDQ) {
        if (p.row_map) my_row = min(max(p.row_map[my_row], 0), L - 1);
    }
    Frag<T> af[KS], bf[THREE ? KS : 1];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) af[ks] = global_frag<T>(ab + (int64_t)my_row * p.a_sl + 16 * ks + 8 * g);
    if constexpr (THREE) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) bf[ks] = global_frag<T>(bb + (int64_t)my_row * p.b_sl + 16 * ks + 8 * g);
    }
    const float c2 = p.scale_log2e;
    float row_lse2 = 0.f, row_delta = 0.f;  // dQ: the lane's own query
    if constexpr (!POS_STATS) {
        row_lse2 = lse_b[my_row] * 1.4426950408889634f;
        // D = rowsum(dO * O) of the lane's row (the two lanes of a row hold half of it each), kept for this launch and stored
        // for the dK and dV launches that follow it on the stream
        const T* orow = (const T*)p.o + b * p.oo_sb + h * p.oo_sh + (int64_t)my_row * p.oo_sl;
        Frag<T> of[KS];  // (all requested before any is used: the accumulators' registers are still free here)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) of[ks] = global_frag<T>(orow + 16 * ks + 8 * g);
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(of[ks].v));
#endif
        float s = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) s = fmaf((float)bf[ks].v[e], (float)of[ks].v[e], s);
        s += __shfl_xor(s, 32);
        row_delta = s;  // (stored after the tile loop: a store in flight would be waited for with the first tile's copies)
    }

    // ---- plan ----
    const PlanRec* const pt = p.plan;
    const int n_rb = p.n_row_blocks;
    auto seg_plan_of = [&](int sg) {
        const PlanRec r = plan_uniform_load(pt + plan_seg_at(p.n_seg, rb, sg));
        SegPlan t;
        t.c0 = r.x, t.cs = r.y, t.n_tiles = r.z, t.uniform = r.w;
        return t;
    };
    int total_tiles = 0;
    for (int sg = 0; sg < p.n_seg; ++sg) total_tiles += seg_plan_of(sg).n_tiles;
    total_tiles = __builtin_amdgcn_readfirstlane(total_tiles);

    // ---- tile walker (see attention.hip): 1 KiB copy blocks, block q = tile rows q*RPI .., wavefront w issues blocks
    // w, w+4, ...; lane i supplies physical chunk i of the block, which holds the logical chunk the swizzle assigns ----
    auto position_row = [&](const SegPlan& pl, int j) { return min(max(pl.c0 + pl.cs * j, 0), L - 1); };
    auto issue_tile_general = [&](const SegPlan& pl, int tile, int stage) {
        const int j0 = tile * BN;
        char* xs_w = smem + RING + stage * STAGE;
        char* ys_w = xs_w + TILE;
        dma_tile<T, ROWB, BN, 3>(xs_w, wave, lane, [&](int row) { return xb + (int64_t)position_row(pl, j0 + row) * p.x_sl; });
        dma_tile<T, ROWB, BN, 3>(ys_w, wave, lane, [&](int row) { return yb + (int64_t)position_row(pl, j0 + row) * p.y_sl; });
    };
    auto issue_stats = [&](const SegPlan& pl, int tile, int stage) {
        if constexpr (POS_STATS) {
            char* st_w = smem + stage * STATS;
            const int q = position_row(pl, tile * BN + lane);
            if (wave == 0) dma4(lse_b + q, st_w);
            if (wave == 1) dma4(del_b + q, st_w + BN * 4);
        }
    };
    uint32_t x_lane_off = 0, y_lane_off = 0;
    bool lane_off_fits = true;
    const char* x_next = nullptr;
    const char* y_next = nullptr;
    int64_t x_key = 0, y_key = 0;  // bytes from one tile position to the next
    auto set_lane_offsets = [&](const SegPlan& pl) {
        const int r = lane / CPR, pc = lane % CPR;
        const int lc = logical_chunk<ROWB, 3>(wave * RPI + r, pc);
        const int64_t x_far = (int64_t)pl.cs * (RPI - 1) * p.x_sl * ES + ROWB, y_far = (int64_t)pl.cs * (RPI - 1) * p.y_sl * ES + ROWB;
        lane_off_fits = x_far < ((int64_t)1 << 32) && y_far < ((int64_t)1 << 32);
        x_key = (int64_t)p.x_sl * ES * pl.cs;
        y_key = (int64_t)p.y_sl * ES * pl.cs;
        x_lane_off = (uint32_t)(x_key * r) + lc * 16;
        y_lane_off = (uint32_t)(y_key * r) + lc * 16;
        x_next = reinterpret_cast<const char*>(xb) + (int64_t)pl.c0 * p.x_sl * ES + (int64_t)wave * RPI * x_key;
        y_next = reinterpret_cast<const char*>(yb) + (int64_t)pl.c0 * p.y_sl * ES + (int64_t)wave * RPI * y_key;
    };
    auto tile_is_fast = [&](const SegPlan& pl, int tile) {
        const int j0 = tile * BN;
        // every position of the tile exists (the first one too: a walk may begin left of column 0)
        return lane_off_fits && pl.c0 + pl.cs * j0 >= 0 && pl.c0 + pl.cs * (j0 + BN - 1) < L;
    };
    auto issue_step = [&](int i, int stage) {
        char* xs_w = smem + RING + stage * STAGE;
        char* ys_w = xs_w + TILE;
        if (i < NI)
            dma16_uniform(x_next + (int64_t)(4 * RPI * i) * x_key, x_lane_off, xs_w + (wave + 4 * i) * 1024);
        else
            dma16_uniform(y_next + (int64_t)(4 * RPI * (i - NI)) * y_key, y_lane_off, ys_w + (wave + 4 * (i - NI)) * 1024);
    };
    int pf_seg = 0, pf_tile = 0;
    SegPlan ppl = {0, 1, 0, 1};
    auto pf_enter_segment = [&]() {
        pf_tile = 0;
        while (pf_seg < p.n_seg) {
            ppl = seg_plan_of(pf_seg);
            if (ppl.n_tiles > 0) break;
            ++pf_seg;
        }
        if (pf_seg < p.n_seg) set_lane_offsets(ppl);
    };
    auto advance_fetch = [&]() {
        x_next += BN * x_key;
        y_next += BN * y_key;
        if (++pf_tile >= ppl.n_tiles) {
            ++pf_seg;
            pf_enter_segment();
        }
    };

    // ---- LDS read addresses of stage 0; the stage offset is added once per tile ----
    const uint32_t smem_base = lds_address(smem);
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);  // element column inside a 32-element block
    // row-wise fragments: row lm (+32 for the second half: the swizzle repeats every 16 rows), logical chunk 2*ks + g
    uint32_t xr_addr[KS], yr_addr[THREE ? KS : 1];
    // transposing reads: rows 4g + tr_row and 8 rows further (whose swizzle differs), 64-byte block dt
    uint32_t tr_addr[DT], tr_addr8[DT];
    auto dual_off = [&](int row, int byte_col) { return row * ROWB + dual_chunk<ROWB>(row, byte_col >> 4) * 16 + (byte_col & 15); };
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        xr_addr[ks] = smem_base + RING + dual_off(lm, (16 * ks + 8 * g) * ES);
        if constexpr (THREE) yr_addr[ks] = smem_base + RING + TILE + dual_off(lm, (16 * ks + 8 * g) * ES);
    }
    constexpr int TR_BASE = RING + (THREE ? 0 : TILE);  // dQ, dK: transposed reads of X; dV: of Y; dK + dV: of both
    uint32_t ty_addr[BOTH ? DT : 1], ty_addr8[BOTH ? DT : 1];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        tr_addr[dt] = smem_base + TR_BASE + dual_off(4 * g + tr_row, (32 * dt + tr_col) * ES);
        tr_addr8[dt] = smem_base + TR_BASE + dual_off(4 * g + tr_row + 8, (32 * dt + tr_col) * ES);
        if constexpr (BOTH) {
            ty_addr[dt] = tr_addr[dt] + TILE;
            ty_addr8[dt] = tr_addr8[dt] + TILE;
        }
    }
    uint32_t st_addr = smem_base + 16 * g;  // lse of positions 4g.. of the stage; D is BN*4 bytes further

    // ---- first tile's copies, accumulators ----
    pf_seg = 0;
    pf_enter_segment();
    PlanRec win_rec = {0, 0, 1, 0};
    if (pf_seg < p.n_seg) win_rec = pt[plan_row_at(n_rb, p.n_seg, rb, pf_seg, wave * 32 + lm)];
    if (total_tiles > 0) {
        if (tile_is_fast(ppl, pf_tile)) {
#pragma unroll
            for (int s = 0; s < NDMA; ++s) issue_step(s, 0);
        } else {
            issue_tile_general(ppl, pf_tile, 0);
        }
        issue_stats(ppl, pf_tile, 0);
        advance_fetch();
    }
    f32x16 acc[DT], acc2[BOTH ? DT : 1];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            acc[dt][j] = 0.f;
            if constexpr (BOTH) acc2[dt][j] = 0.f;
        }

    int cur_seg = -1, cur_tile = 0;
    RowWin win = {0, 0, 1};
    int first = 0, dec = 0;
    uint64_t pat = ~0ull;
    int w_lo_min = 0, w_lo_max = 0, w_hi_min = 0, w_hi_max = 0;
    SegPlan cpl = {0, 1, 0, 1};
    int stage_it = 0, stage_pf = 1;
#if defined(__HIP_DEVICE_COMPILE__)
    // the register operands are in their registers before the loop, so that no wait of the compiler's for them ends up
    // inside it, where it would also wait for the copies in flight
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(af[ks].v));
    if constexpr (THREE) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(bf[ks].v));
    }
    asm volatile("" ::"v"(row_lse2), "v"(row_delta));
#endif

    for (int it = 0; it < total_tiles; ++it) {
        if (cur_seg < 0 || cur_tile >= cpl.n_tiles) {
            do {
                ++cur_seg;
                cpl = seg_plan_of(cur_seg);
            } while (cpl.n_tiles == 0);
            cur_tile = 0;
            if (it > 0) win_rec = pt[plan_row_at(n_rb, p.n_seg, rb, cur_seg, wave * 32 + lm)];
            win.lo = win_rec.x, win.cnt = win_rec.y, win.lin = win_rec.z;
            first = win_rec.w;
            const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, cur_seg, wave));
            if (!cpl.uniform) {
                dec = BN % win.lin;
                uint64_t pt_bits = 0;
                for (int q = 0; q < 64; q += win.lin) pt_bits |= 1ull << q;
                pat = pt_bits;
            } else {
                pat = ~0ull;
            }
            w_lo_min = r.x, w_lo_max = r.y, w_hi_min = r.z, w_hi_max = r.w;
            asm volatile("v_mov_b32 %0, %0" : "+v"(w_lo_min));
            asm volatile("v_mov_b32 %0, %0" : "+v"(w_lo_max));
            asm volatile("v_mov_b32 %0, %0" : "+v"(w_hi_min));
            asm volatile("v_mov_b32 %0, %0" : "+v"(w_hi_max));
        }
        const int j0 = cur_tile * BN;
        ++cur_tile;

        // this wavefront's copies of tile `it` have landed; after the barrier everybody's have, and everybody is done
        // with tile it - 1, whose stage the next fetch overwrites
        wait_loads<0>();
        __builtin_amdgcn_s_barrier();

        const bool fetch = (it + 1 < total_tiles);
        bool spread = false;
        if (fetch) {
            spread = tile_is_fast(ppl, pf_tile);
            if (!spread) issue_tile_general(ppl, pf_tile, stage_pf);
            issue_stats(ppl, pf_tile, stage_pf);
        }

        const bool skip = (j0 + BN <= w_lo_min) || (j0 >= w_hi_max);
        if (!skip) {
            const bool full = (j0 >= w_lo_max) && (j0 + BN <= w_hi_min);
            const uint64_t live = full ? ~0ull : row_live_bits(win, j0, first, pat);
            if constexpr (!THREE) {
                // ---- dV: two products only, so the whole 64-position tile fits the registers at once, as in the forward:
                // all score MFMAs with the fragments requested well ahead, then the exponentials, then the output MFMAs ----
                constexpr int NMMA = 2 * KS, AHEAD = NMMA < 12 ? NMMA : 12;
                f32x16 s2[2];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                    for (int j = 0; j < 16; ++j) s2[nt][j] = 0.f;
                Frag<T> xfr[NMMA];
                auto load_x = [&](int i) {
                    Frag<T> f;
                    f.v = __builtin_bit_cast(typename Frag<T>::vec, lds_load128(xr_addr[i % KS] + 32 * (i / KS) * ROWB));
                    return f;
                };
#pragma unroll
                for (int i = 0; i < AHEAD; ++i) xfr[i] = load_x(i);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < NMMA; ++i) {
                    mma32(s2[i / KS], xfr[i], af[i % KS]);
                    if (i + AHEAD < NMMA) {
                        xfr[i + AHEAD] = load_x(i + AHEAD);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (i < NDMA) {
                        if (spread) issue_step(i, stage_pf);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                Frag<T> pf2[2][2];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    if (!full) {
                        const uint32_t bits = (uint32_t)(live >> (32 * nt)) >> (4 * g);
#pragma unroll
                        for (int j = 0; j < 16; ++j) {
                            const int c = 8 * (j >> 2) + (j & 3);
                            s2[nt][j] = keep_or_mask(s2[nt][j], ((int)(bits << (31 - c))) >> 31);
                        }
                    }
#pragma unroll
                    for (int k4 = 0; k4 < 4; ++k4) {
                        const f32x4 lse4 = __builtin_bit_cast(f32x4, lds_load128(st_addr + (32 * nt + 8 * k4) * 4));
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int j = 4 * k4 + i;
                            pf2[nt][j >> 3].v[j & 7] = (T)fast_exp2(fmaf(s2[nt][j], c2, -1.4426950408889634f * lse4[i]));
                        }
                    }
                }
                auto load_t = [&](int step, int dt) {
                    const int roff = 16 * step * ROWB;
                    return frag_from_tr<T>(lds_load_tr16(tr_addr[dt] + roff), lds_load_tr16(tr_addr8[dt] + roff));
                };
                Frag<T> tf2[2][DT];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) tf2[0][dt] = load_t(0, dt);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int step = 0; step < 4; ++step) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        mma32(acc[dt], tf2[step & 1][dt], pf2[step >> 1][step & 1]);
                        if (step + 1 < 4) {
                            tf2[(step + 1) & 1][dt] = load_t(step + 1, dt);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            } else
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                // ---- S^T (32 positions x 32 rows) = X rows . A^T ----
                f32x16 s_acc;
#pragma unroll
                for (int j = 0; j < 16; ++j) s_acc[j] = 0.f;
                Frag<T> xfr[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    xfr[ks].v = __builtin_bit_cast(typename Frag<T>::vec, lds_load128(xr_addr[ks] + 32 * nt * ROWB));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    mma32(s_acc, xfr[ks], af[ks]);
                    // the copy instructions of the next tile go between these MFMAs
                    const int step = nt * KS + ks;  // 0 .. 2*KS - 1
                    if (step < NDMA) {
                        if (spread) issue_step(step, stage_pf);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if (!full) {
                    const uint32_t bits = (uint32_t)(live >> (32 * nt)) >> (4 * g);
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int c = 8 * (j >> 2) + (j & 3);
                        s_acc[j] = keep_or_mask(s_acc[j], ((int)(bits << (31 - c))) >> 31);
                    }
                }
                // ---- P^T = exp2(S^T * scale*log2e - lse*log2e); masked scores underflow to exactly 0 ----
                if constexpr (POS_STATS) {
#pragma unroll
                    for (int k4 = 0; k4 < 4; ++k4) {
                        // (the whole vector is reinterpreted: a bit cast of one element of an integer vector reads element 0)
                        const f32x4 lse4 = __builtin_bit_cast(f32x4, lds_load128(st_addr + (32 * nt + 8 * k4) * 4));
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            s_acc[4 * k4 + i] = fast_exp2(fmaf(s_acc[4 * k4 + i], c2, -1.4426950408889634f * lse4[i]));
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 16; ++j) s_acc[j] = fast_exp2(fmaf(s_acc[j], c2, -row_lse2));
                }
                Frag<T> pf[2];  // the second product's B operand: 16 positions each
                Frag<T> pp[BOTH ? 2 : 1];  // dK + dV: the probabilities themselves, dV's B operand
                if constexpr (THREE) {
                    // ---- dP^T = Y rows . B^T ----
                    f32x16 dp;
#pragma unroll
                    for (int j = 0; j < 16; ++j) dp[j] = 0.f;
                    Frag<T> yfr[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        yfr[ks].v = __builtin_bit_cast(typename Frag<T>::vec, lds_load128(yr_addr[ks] + 32 * nt * ROWB));
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) mma32(dp, yfr[ks], bf[ks]);
                    // ---- dS^T = P^T * (dP^T - D) * scale ----
                    if constexpr (POS_STATS) {
#pragma unroll
                        for (int k4 = 0; k4 < 4; ++k4) {
                            const f32x4 d4 = __builtin_bit_cast(f32x4, lds_load128(st_addr + BN * 4 + (32 * nt + 8 * k4) * 4));
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const int j = 4 * k4 + i;
                                pf[j >> 3].v[j & 7] = (T)(s_acc[j] * (dp[j] - d4[i]) * p.scale);
                            }
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 16; ++j) pf[j >> 3].v[j & 7] = (T)(s_acc[j] * (dp[j] - row_delta) * p.scale);
                    }
                    if constexpr (BOTH) {
#pragma unroll
                        for (int j = 0; j < 16; ++j) pp[j >> 3].v[j & 7] = (T)s_acc[j];
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 16; ++j) pf[j >> 3].v[j & 7] = (T)s_acc[j];
                }
                // ---- acc^T (d x 32 rows) += tile^T . pf: two steps of 16 positions ----
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    Frag<T> tf[DT];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const int roff = (32 * nt + 16 * t) * ROWB;
                        tf[dt] = frag_from_tr<T>(lds_load_tr16(tr_addr[dt] + roff), lds_load_tr16(tr_addr8[dt] + roff));
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) mma32(acc[dt], tf[dt], pf[t]);
                    if constexpr (BOTH) {
                        // ---- acc2^T += Y^T . P^T ----
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            const int roff = (32 * nt + 16 * t) * ROWB;
                            tf[dt] = frag_from_tr<T>(lds_load_tr16(ty_addr[dt] + roff), lds_load_tr16(ty_addr8[dt] + roff));
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) mma32(acc2[dt], tf[dt], pp[t]);
                    }
                }
            }
            if (2 * KS < NDMA && spread) {
#pragma unroll
                for (int s = 2 * KS; s < NDMA; ++s) issue_step(s, stage_pf);
            }
        } else if (spread) {
#pragma unroll
            for (int s = 0; s < NDMA; ++s) issue_step(s, stage_pf);
        }

        if (fetch) {
            advance_fetch();
            stage_pf ^= 1;
        }
        if (!cpl.uniform) {
            const int f = first - dec;
            first = f < 0 ? f + win.lin : f;
        }
        stage_it ^= 1;
        const int delta_b = stage_it == 0 ? -STAGE : STAGE;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            xr_addr[ks] += delta_b;
            if constexpr (THREE) yr_addr[ks] += delta_b;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            tr_addr[dt] += delta_b;
            tr_addr8[dt] += delta_b;
            if constexpr (BOTH) {
                ty_addr[dt] += delta_b;
                ty_addr8[dt] += delta_b;
            }
        }
        st_addr += stage_it == 0 ? -STATS : STATS;
    }
    // every wavefront has finished reading the last tile before the stages are reused for the output
    wait_loads<0>();
    __syncthreads();

    if constexpr (!POS_STATS) {
        if (g == 0 && r0 + rs * (wave * 32 + lm) < Lr) p.delta_w[(int64_t)bh * L + my_row] = row_delta;
    }

    // ---- epilogue: out = acc^T transposed through LDS, whole rows per store (each wavefront through a stretch of its own) ----
    {
        constexpr int OROW = D * ES + 16;
        static_assert(4 * 32 * OROW <= RING + 2 * STAGE, "staging space");
        char* stg = smem + wave * (32 * OROW);
        auto store_rows = [&](const f32x16 (&a)[DT], T* dst) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    typedef T vec4 __attribute__((ext_vector_type(4)));
                    vec4 o;
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[i] = (T)a[dt][4 * jj + i];
                    *reinterpret_cast<vec4*>(stg + lm * OROW + (32 * dt + 8 * jj + 4 * g) * ES) = o;
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            constexpr int OCPR = D * ES / 16;
#pragma unroll
            for (int i = 0; i < 32 * OCPR / 64; ++i) {
                const int flat = i * 64 + lane;
                const int row = flat / OCPR, c = flat % OCPR;
                const int r = r0 + rs * (wave * 32 + row);
                const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * OROW + c * 16);
                if (r < Lr) __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(reinterpret_cast<char*>(dst + (int64_t)r * p.o_sl) + c * 16));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (read out before the stretch is written again)
        };
        store_rows(acc, ob);
        if constexpr (BOTH) store_rows(acc2, (T*)p.out2 + b * p.o_sb + h * p.o_sh);
    }
}

template <typename T, int D, int MODE>
static int launch_bwd(BwdParams p, hipStream_t st) {
    begin_launch();
    constexpr int LDS_BYTES = 2 * (2 * 64 * D * 2) + 2 * (2 * 64 * 4);  // two stages of two tiles, two of statistics
    const int grid = ((p.total + 7) / 8) * 8;
    auto kern = attn_bwd_kernel<T, D, MODE>;
    static uint64_t lds_reserved = 0;
    if (int rc = reserve_dynamic_lds(&lds_reserved, reinterpret_cast<const void*>(kern), LDS_BYTES, "splat_attention_bwd")) return rc;
    kern<<<grid, 256, LDS_BYTES, st>>>(p);
    return check_launch("splat_attention_bwd");
}

// Adds the shares of listed rows onto the gradients of their keys: row k of every stretch (rows k + rps * s of the share
// buffers, [B*H, n_rows, D]) belongs to key key_of_row[k] (negative: padding).  One thread takes 8 features of one listed
// key of one (b, h) and one gradient (blockIdx.y: dk, dv), eight stretches' shares requested at a time, summing in fp32
// and rounding once.
template <typename T, int D>
__global__ __launch_bounds__(256) void bwd_rows_add_kernel(const T* __restrict__ dk_rows, const T* __restrict__ dv_rows, T* dk, T* dv,
                                                           const int* __restrict__ key_of_row, int n_rows, int rps, int L, int64_t total) {
    constexpr int CPR = D / 8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int c = (int)(idx % CPR);
    const int64_t r = idx / CPR;
    const int k = (int)(r % rps);
    const int64_t bh = r / rps;
    const int key = key_of_row[k];
    if (key < 0 || key >= L) return;
    const int n_stretches = n_rows / rps;
    const T* rows = (blockIdx.y ? dv_rows : dk_rows) + ((int64_t)bh * n_rows + k) * D + 8 * c;
    T* out = (blockIdx.y ? dv : dk) + ((int64_t)bh * L + key) * D + 8 * c;
    Frag<T> cur = global_frag<T>(out);
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = (float)cur.v[e];
    for (int st = 0; st < n_stretches; st += 8) {
        Frag<T> f[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) f[u] = global_frag<T>(rows + (int64_t)min(st + u, n_stretches - 1) * rps * D);  // (unconditional)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float w = st + u < n_stretches ? 1.f : 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(w, (float)f[u].v[e], acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) cur.v[e] = (T)acc[e];
    *reinterpret_cast<typename Frag<T>::vec*>(out) = cur.v;
}

template <typename T>
static int launch_rows_add(const void* dk_rows, const void* dv_rows, void* dk, void* dv, const int* key_of_row, int B, int H, int L,
                           int n_rows, int rps, int d, hipStream_t st) {
    begin_launch();
    const int64_t total = (int64_t)B * H * rps * (d / 8);
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7ffffff0) return fail(SPLAT_E_SHAPE, "splat_attention_bwd_keys: too many listed rows");
    if (d == 64)
        bwd_rows_add_kernel<T, 64><<<dim3((unsigned)blocks, 2), 256, 0, st>>>((const T*)dk_rows, (const T*)dv_rows, (T*)dk, (T*)dv, key_of_row, n_rows, rps, L, total);
    else
        bwd_rows_add_kernel<T, 128><<<dim3((unsigned)blocks, 2), 256, 0, st>>>((const T*)dk_rows, (const T*)dv_rows, (T*)dk, (T*)dv, key_of_row, n_rows, rps, L, total);
    return check_launch("splat_attention_bwd_keys");
}

// The keys' side: dK and dV of the rows of the transposed mask that `dk` describes (dv: the same launch geometry).
template <typename T>
static int run_bwd_keys(const BwdParams& dk, const BwdParams& dv, int d, hipStream_t st) {
    if (d == 64) {
        // both accumulators of the keys' side fit the registers at d = 64 (204 of 256; at d = 128 they would need over 300):
        // one walk, 4 products instead of 3 + 2, the scores and the exponentials once (config 2: 0.160 -> 0.133 ms)
        BwdParams dkv = dk;
        dkv.out2 = dv.out;
        return launch_bwd<T, 64, kBwdDKV>(dkv, st);
    }
    if (int rc = launch_bwd<T, 128, kBwdDK>(dk, st)) return rc;
    return launch_bwd<T, 128, kBwdDV>(dv, st);
}

template <typename T>
static int run_bwd(const BwdParams& dq, const BwdParams& dk, const BwdParams& dv, int d, hipStream_t st) {
    if (int rc = d == 64 ? launch_bwd<T, 64, kBwdDQ>(dq, st) : launch_bwd<T, 128, kBwdDQ>(dq, st)) return rc;
    return run_bwd_keys<T>(dk, dv, d, st);
}

struct Rows3 {
    const void* ptr;
    int64_t sb, sh, sl;
};

// Checks shared by the two entry points; `who` names the caller in messages.
static int check_bwd_common(const char* who, int B, int H, int L, int d, float scale, int dtype, std::initializer_list<Rows3> rows,
                            std::initializer_list<const void*> aligned16) {
    if (B <= 0 || H <= 0 || L <= 0) return fail(SPLAT_E_SHAPE, "%s: need B, H, L > 0 (got %d, %d, %d)", who, B, H, L);
    if (L > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: L is limited to 2^23 (got %d)", who, L);
    if (d != 64 && d != 128) return fail(SPLAT_E_UNSUPPORTED, "%s: head dim must be 64 or 128 (got %d)", who, d);
    if (dtype != SPLAT_F16 && dtype != SPLAT_BF16) return fail(SPLAT_E_UNSUPPORTED, "%s: 16-bit element types only (got dtype %d)", who, dtype);
    if (!(scale > 0.f)) return fail(SPLAT_E_UNSUPPORTED, "%s: scale must be > 0 (got %g)", who, (double)scale);
    auto mis = [&](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
    for (const Rows3& r : rows) {
        if (mis(r.ptr)) return fail(SPLAT_E_ALIGN, "%s: every tensor of rows must be 16-byte aligned", who);
        if ((r.sb % 8) != 0 || (r.sh % 8) != 0 || (r.sl % 8) != 0)
            return fail(SPLAT_E_ALIGN, "%s: every batch/head/row stride must be a multiple of 8 elements (16 bytes)", who);
        if (r.sl < d) return fail(SPLAT_E_SHAPE, "%s: row strides must be >= d", who);
    }
    for (const void* ptr : aligned16)
        if (mis(ptr)) return fail(SPLAT_E_ALIGN, "%s: the gradients and the plans must be 16-byte aligned", who);
    return 0;
}

static BwdParams bwd_base(const float* lse, const float* delta, int B, int H, int L, float scale) {
    BwdParams base;
    base.lse = lse; base.delta = delta;
    base.o = nullptr; base.oo_sb = base.oo_sh = base.oo_sl = 0; base.delta_w = nullptr; base.out2 = nullptr;
    base.B = B; base.H = H; base.L = L; base.Lr = L; base.row_map = nullptr;
    base.scale = scale; base.scale_log2e = scale * 1.4426950408889634f;
    return base;
}

// dK (and, as a copy with b = null and out = dV, dV): rows = `Lk` keys, the plan of the (transposed) mask's `n_seg_t` segments
// for those rows; outputs contiguous [B, H, Lk, d]
static BwdParams bwd_keys_params(const BwdParams& base, Rows3 q, Rows3 k, Rows3 v, Rows3 g, void* dk, const splat_acsr_seg* segs_t,
                                 int n_seg_t, const void* plan_t, int Lk, const int* row_map, int d) {
    BwdParams pk = base;
    pk.a = k.ptr; pk.a_sb = k.sb; pk.a_sh = k.sh; pk.a_sl = k.sl;
    pk.b = v.ptr; pk.b_sb = v.sb; pk.b_sh = v.sh; pk.b_sl = v.sl;
    pk.x = q.ptr; pk.x_sb = q.sb; pk.x_sh = q.sh; pk.x_sl = q.sl;
    pk.y = g.ptr; pk.y_sb = g.sb; pk.y_sh = g.sh; pk.y_sl = g.sl;
    pk.out = dk; pk.o_sb = (int64_t)base.H * Lk * d; pk.o_sh = (int64_t)Lk * d; pk.o_sl = d;
    pk.Lr = Lk; pk.row_map = row_map;
    pk.n_seg = n_seg_t; pk.row_stride = common_row_stride(segs_t, n_seg_t);
    pk.n_row_blocks = count_row_blocks(Lk, kPlanBM, pk.row_stride); pk.total = base.B * base.H * pk.n_row_blocks;
    pk.plan = static_cast<const PlanRec*>(plan_t);
    return pk;
}

}  // namespace splat

using namespace splat;

extern "C" int splat_attention_bwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* k, int64_t k_sb,
                                   int64_t k_sh, int64_t k_sl, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl,
                                   const void* out, int64_t o_sb, int64_t o_sh, int64_t o_sl, const void* dout, int64_t g_sb,
                                   int64_t g_sh, int64_t g_sl, const float* lse, float* delta, void* dq, void* dk, void* dv,
                                   const splat_acsr_seg* segs, int32_t n_seg, const void* plan, int64_t plan_bytes,
                                   const splat_acsr_seg* segs_t, int32_t n_seg_t, const void* plan_t, int64_t plan_t_bytes,
                                   int32_t B, int32_t H, int32_t L, int32_t d, float scale, int32_t dtype, void* stream) {
    const char* who = "splat_attention_bwd";
    if (!q || !k || !v || !out || !dout || !lse || !delta || !dq || !dk || !dv || !segs || !segs_t || !plan || !plan_t)
        return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    const Rows3 rq{q, q_sb, q_sh, q_sl}, rk{k, k_sb, k_sh, k_sl}, rv{v, v_sb, v_sh, v_sl}, ro{out, o_sb, o_sh, o_sl}, rg{dout, g_sb, g_sh, g_sl};
    if (int rc = check_bwd_common(who, B, H, L, d, scale, dtype, {rq, rk, rv, ro, rg}, {dq, dk, dv, plan, plan_t})) return rc;
    if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0 || (reinterpret_cast<uintptr_t>(delta) & 3) != 0)
        return fail(SPLAT_E_ALIGN, "%s: lse and delta must be 4-byte aligned", who);
    SegPtrs tmp[SPLAT_MAX_SEGMENTS];
    if (int rc = fill_segs(who, segs, n_seg, tmp, -1)) return rc;
    if (int rc = fill_segs(who, segs_t, n_seg_t, tmp, -1)) return rc;
    if (plan_bytes < splat_attention_plan_bytes(segs, n_seg, L) || plan_t_bytes < splat_attention_plan_bytes(segs_t, n_seg_t, L))
        return fail(SPLAT_E_SHAPE, "%s: a plan is smaller than its mask needs (%lld and %lld bytes given)", who, (long long)plan_bytes,
                    (long long)plan_t_bytes);
    if ((int64_t)B * H * std::max(count_row_blocks(L, kPlanBM, common_row_stride(segs, n_seg)),
                                  count_row_blocks(L, kPlanBM, common_row_stride(segs_t, n_seg_t))) > 0x7ffffff0)
        return fail(SPLAT_E_SHAPE, "%s: too many row blocks", who);
    hipStream_t st = (hipStream_t)stream;

    const BwdParams base = bwd_base(lse, delta, B, H, L, scale);
    // dQ: rows = queries, the mask's own plan
    BwdParams pq = base;
    pq.a = q; pq.a_sb = q_sb; pq.a_sh = q_sh; pq.a_sl = q_sl;
    pq.b = dout; pq.b_sb = g_sb; pq.b_sh = g_sh; pq.b_sl = g_sl;
    pq.x = k; pq.x_sb = k_sb; pq.x_sh = k_sh; pq.x_sl = k_sl;
    pq.y = v; pq.y_sb = v_sb; pq.y_sh = v_sh; pq.y_sl = v_sl;
    pq.out = dq; pq.o_sb = (int64_t)H * L * d; pq.o_sh = (int64_t)L * d; pq.o_sl = d;  // the gradients are contiguous [B, H, L, d]
    pq.n_seg = n_seg; pq.row_stride = common_row_stride(segs, n_seg);
    pq.n_row_blocks = count_row_blocks(L, kPlanBM, pq.row_stride); pq.total = B * H * pq.n_row_blocks;
    pq.plan = static_cast<const PlanRec*>(plan);
    pq.o = out; pq.oo_sb = o_sb; pq.oo_sh = o_sh; pq.oo_sl = o_sl; pq.delta_w = delta;  // D = rowsum(dO * O): computed and stored by this launch
    // dK, dV: rows = keys, the transposed mask's plan
    const BwdParams pk = bwd_keys_params(base, rq, rk, rv, rg, dk, segs_t, n_seg_t, plan_t, L, nullptr, d);
    BwdParams pv = pk;
    pv.b = nullptr;
    pv.out = dv;
    return dtype == SPLAT_F16 ? run_bwd<f16>(pq, pk, pv, d, st) : run_bwd<bf16>(pq, pk, pv, d, st);
}

extern "C" int splat_attention_bwd_keys(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* k, int64_t k_sb,
                                        int64_t k_sh, int64_t k_sl, const void* v, int64_t v_sb, int64_t v_sh, int64_t v_sl,
                                        const void* dout, int64_t g_sb, int64_t g_sh, int64_t g_sl, const float* lse,
                                        const float* delta, const int32_t* key_of_row, void* dk_rows, void* dv_rows,
                                        const splat_acsr_seg* segs_t, int32_t n_seg_t, const void* plan_t, int64_t plan_t_bytes,
                                        int32_t B, int32_t H, int32_t L, int32_t n_rows, int32_t d, float scale, int32_t dtype,
                                        void* dk, void* dv, int32_t rows_per_stretch, void* stream) {
    const char* who = "splat_attention_bwd_keys";
    if (!q || !k || !v || !dout || !lse || !delta || !key_of_row || !dk_rows || !dv_rows || !segs_t || !plan_t)
        return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    const Rows3 rq{q, q_sb, q_sh, q_sl}, rk{k, k_sb, k_sh, k_sl}, rv{v, v_sb, v_sh, v_sl}, rg{dout, g_sb, g_sh, g_sl};
    if (int rc = check_bwd_common(who, B, H, L, d, scale, dtype, {rq, rk, rv, rg}, {dk_rows, dv_rows, plan_t})) return rc;
    if (n_rows <= 0 || n_rows > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: need 0 < n_rows <= 2^23 (got %d)", who, n_rows);
    if ((dk == nullptr) != (dv == nullptr)) return fail(SPLAT_E_NULL, "%s: dk and dv go together (both or neither)", who);
    if (dk) {
        if ((reinterpret_cast<uintptr_t>(dk) & 15) != 0 || (reinterpret_cast<uintptr_t>(dv) & 15) != 0)
            return fail(SPLAT_E_ALIGN, "%s: dk and dv must be 16-byte aligned", who);
        if (rows_per_stretch <= 0 || n_rows % rows_per_stretch != 0)
            return fail(SPLAT_E_SHAPE, "%s: n_rows (%d) must be a multiple of rows_per_stretch (%d)", who, n_rows, rows_per_stretch);
    }
    if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0 || (reinterpret_cast<uintptr_t>(delta) & 3) != 0 ||
        (reinterpret_cast<uintptr_t>(key_of_row) & 3) != 0)
        return fail(SPLAT_E_ALIGN, "%s: lse, delta and key_of_row must be 4-byte aligned", who);
    SegPtrs tmp[SPLAT_MAX_SEGMENTS];
    if (int rc = fill_segs(who, segs_t, n_seg_t, tmp, -1)) return rc;
    if (plan_t_bytes < splat_attention_plan_bytes(segs_t, n_seg_t, n_rows))
        return fail(SPLAT_E_SHAPE, "%s: the plan is smaller than %d rows of this mask need (%lld bytes given)", who, n_rows,
                    (long long)plan_t_bytes);
    if ((int64_t)B * H * count_row_blocks(n_rows, kPlanBM, common_row_stride(segs_t, n_seg_t)) > 0x7ffffff0)
        return fail(SPLAT_E_SHAPE, "%s: too many row blocks", who);
    const BwdParams base = bwd_base(lse, delta, B, H, L, scale);
    const BwdParams pk = bwd_keys_params(base, rq, rk, rv, rg, dk_rows, segs_t, n_seg_t, plan_t, n_rows, key_of_row, d);
    BwdParams pv = pk;
    pv.b = nullptr;
    pv.out = dv_rows;
    hipStream_t st = (hipStream_t)stream;
    if (int rc = dtype == SPLAT_F16 ? run_bwd_keys<f16>(pk, pv, d, st) : run_bwd_keys<bf16>(pk, pv, d, st)) return rc;
    if (!dk) return 0;
    return dtype == SPLAT_F16 ? launch_rows_add<f16>(dk_rows, dv_rows, dk, dv, key_of_row, B, H, L, n_rows, rows_per_stretch, d, st)
                              : launch_rows_add<bf16>(dk_rows, dv_rows, dk, dv, key_of_row, B, H, L, n_rows, rows_per_stretch, d, st);
}
