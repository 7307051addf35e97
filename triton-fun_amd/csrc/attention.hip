// Fused ACSR sparse-attention forward (online softmax), gfx950.
//
// A workgroup of 4 wavefronts owns 128 query rows of one (batch, head).  It walks the key range its
// rows' affine spans cover in tiles of BN keys.  Per tile:
//   * the K and V tiles are copied global -> LDS without passing through registers (LDS-DMA), into a
//     ring of NSTAGE stages: the copy of tile t + NSTAGE - 1 is issued while tile t is computed, piecewise
//     between its score MFMAs;
//   * every wavefront computes the TRANSPOSED score tile S^T = K . Q^T for its 32 rows with
//     32x32x16 MFMA (A = K fragment from LDS, B = Q fragment held in registers for the whole kernel).
//     In the transposed product one lane owns one query row, so masking, the running max and the
//     running sum need no cross-lane traffic beyond one exchange with the lane that holds the other
//     half of the row;
//   * P^T (the exponentials, converted to the input type) is already laid out as the B operand of
//     O^T += V^T . P^T, whose A operand (V^T fragments) is read from the row-major V tile in LDS with
//     the transposing LDS read (ds_read_b64_tr_b16); K^T tiles ([d, keys] input layout) use the same read.
// The compressed score matrix never exists in memory: traffic is Q + K + V + O.
//
// Which keys a tile holds is decided per workgroup from the rows' (a, lin, cnt) maps: if all rows
// share the column step and phase, tiles enumerate exactly those columns (key index c0 + cs*j,
// gathered rows of K/V) and validity is a per-row range test in j; otherwise tiles are dense columns
// and validity is the full affine test (offset, step divisibility, count).  Each wavefront skips
// tiles that lie outside all of its rows' spans and drops the mask on tiles inside all of them.
#include <mutex>

#include "attn_tile.hpp"

namespace splat {

struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    int64_t q_sb, q_sh, q_sl;
    int64_t k_sb, k_sh, k_sd, k_sl;
    int64_t v_sb, v_sh, v_sl;
    int64_t o_sb, o_sh, o_sl;
    int B, H, L;
    float scale_log2e;
    int n_seg;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];
    int n_row_blocks;
    int total;
    int row_stride;
    const PlanRec* plan;  // plan table of this mask (PLANNED kernels), variant already selected
    float* lse;           // optional [B*H, L]: log of every row's sum of exponentials (natural log, scaled scores)
};

constexpr float kRescaleThreshold = 8.0f;  // in log2 units: exponentials stay below 2^8 before the reference moves

// Exponentials of one tile of scores against the rows' references (mb = reference * c2), as MFMA B fragments; returns
// the lane's sum.
template <int NT, typename T>
__device__ __forceinline__ float exp_tile(const f32x16 (&s)[NT], Frag<T> (&pf)[NT][2], float mb, float c2) {
    float rs = 0.f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float pv = fast_exp2(fmaf(s[nt][j], c2, -mb));
            rs += pv;
            pf[nt][j >> 3].v[j & 7] = (T)pv;
        }
    return rs;
}

// Fold one tile of 32*NT keys of (masked) scores of one 32-row tile into the running softmax state and emit the
// exponentials.  One lane owns one query row (half of its positions).  Returns whether every row of the wavefront
// has a real reference afterwards.
template <int NT, typename T, int DT>
__device__ __forceinline__ bool softmax_tile(f32x16 (&s)[NT], Frag<T> (&pf)[NT][2], float& m_ref, float& l_run,
                                             f32x16 (&o)[DT], float c2) {
    float mx = s[0][0];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int j = 0; j < 16; ++j) mx = fmaxf(mx, s[nt][j]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));  // the other half of the row lives in lane ^ 32
    // move the reference only when some row's maximum has outrun it by the threshold (always on the first
    // live tile); rows that do not move keep alpha = 1
    if (__any((mx - m_ref) * c2 > kRescaleThreshold)) {
        const float m_new = ((mx - m_ref) * c2 > kRescaleThreshold) ? mx : m_ref;
        const float alpha = fast_exp2((m_ref - m_new) * c2);
        const bool had_data = __any(m_ref > 0.5f * kNegBigA);  // otherwise O and l are still all zero
        m_ref = m_new;
        if (had_data) {
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int j = 0; j < 16; ++j) o[dt][j] *= alpha;
        }
    }
    // Masked scores are -1e30: their exponential underflows to exactly 0 as long as the reference is a real
    // score.  A row that has seen no live score yet keeps the -1e30 reference; give it offset 0 so that its
    // (all masked) entries still map to 0 instead of exp2(0).
    const bool real = m_ref > 0.5f * kNegBigA;
    l_run += exp_tile<NT, T>(s, pf, real ? m_ref * c2 : 0.f, c2);
    return !__any(!real);
}

template <typename T, int D, bool KT, int BN, int NSTAGE, bool PLANNED>
__global__ __launch_bounds__(256, sizeof(T) == 2 ? 2 : 1) void attn_fwd_kernel(const AttnParams p) {
    using G = TileGeom<T, D, KT, BN>;
    constexpr int ES = G::ES;
    constexpr int BM = 128;
    constexpr int KS = D / 16;  // contraction steps of the score product
    constexpr int DT = D / 32;  // 32-row tiles of O^T
    constexpr int NT = BN / 32;
    constexpr int PD = NSTAGE - 1;  // tiles whose copies run ahead of the tile being computed
    static_assert(NT == 1 || NT == 2, "tiles of 32 or 64 keys");
    static_assert(PD == 1 || PD == 3, "the wait ladder below covers 2 and 4 stages");
    constexpr bool FAST_DMA = (ES == 2);  // lane offsets of the LDS-DMA do not depend on the instruction index

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lm = lane & 31, g = lane >> 5;

    const int logical = xcd_remap(blockIdx.x, gridDim.x);
    if (logical >= p.total) return;
    const int bh = logical / p.n_row_blocks;
    // later row blocks of causal patterns carry the most keys: hand them out first
    const int rb = p.n_row_blocks - 1 - (logical % p.n_row_blocks);
    const int b = bh / p.H, h = bh % p.H;
    const int rs = p.row_stride;
    const int r0 = block_first_row(rb, BM, rs);
    const int L = p.L;

    const T* qb = (const T*)p.q + b * p.q_sb + h * p.q_sh;
    const T* kb = (const T*)p.k + b * p.k_sb + h * p.k_sh;
    const T* vb = (const T*)p.v + b * p.v_sb + h * p.v_sh;
    T* ob = (T*)p.o + b * p.o_sb + h * p.o_sh;

    // ---- Q fragments (B operand of S^T), resident for the whole kernel; requested before the plan so that
    // their latency overlaps the metadata loads (the plan's barriers wait for both) ------------------------
    Frag<T> qf[KS];
    {
        const int my_row = r0 + rs * (wave * 32 + lm);
        const T* qr = qb + (int64_t)min(my_row, L - 1) * p.q_sl;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag<T>(qr + 16 * ks + 8 * g);
    }
    // ---- plan: per segment, the column range and step of this row block; computed here from the rows' maps or
    // taken from the mask's plan table (scalar loads: no LDS, no barrier) ------------------------
    static_assert(!PLANNED || (BM == kPlanBM && PD == 1), "the plan table is laid out for 128-row blocks");
    const PlanRec* const pt = p.plan;
    const int n_rb = p.n_row_blocks;
    auto seg_plan_of = [&](int sg) {
        SegPlan t;
        if constexpr (PLANNED) {
            const PlanRec r = plan_uniform_load(pt + plan_seg_at(p.n_seg, rb, sg));
            t.c0 = r.x, t.cs = r.y, t.n_tiles = r.z, t.uniform = r.w;
        } else {
            const SegPlan l = s_plan[sg];  // the same for every lane: keep it in scalar registers
            t.c0 = __builtin_amdgcn_readfirstlane(l.c0);
            t.cs = __builtin_amdgcn_readfirstlane(l.cs);
            t.n_tiles = __builtin_amdgcn_readfirstlane(l.n_tiles);
            t.uniform = __builtin_amdgcn_readfirstlane(l.uniform);
        }
        return t;
    };
    if constexpr (!PLANNED) plan_segments<BM, BN>(p.seg, p.n_seg, r0, rs, L, !KT, s_plan, &s_ps, tid);

    int total_tiles = 0;
    for (int sg = 0; sg < p.n_seg; ++sg) total_tiles += seg_plan_of(sg).n_tiles;
    total_tiles = __builtin_amdgcn_readfirstlane(total_tiles);

    // ---- tile walker: asynchronous global -> LDS copies of a tile into a stage -------------------------
    // A tile is copied as 1 KiB blocks, one wavefront instruction each; block q holds tile rows q*RPI.. and
    // wavefront w issues blocks w, w+4, ...  Lane i of a block supplies physical chunk i, i.e. (row i / CPR,
    // chunk position i % CPR), and loads the logical chunk the tile's swizzle assigns to that position.  For
    // 16-bit types that assignment does not depend on the block, so a lane's source offset within a block is
    // a per-segment constant and the block's base is wavefront-uniform.
    constexpr int V_CPR = G::V_ROWB / 16, V_RPI = 1024 / G::V_ROWB;
    constexpr int K_CPR = G::K_ROWB / 16, K_RPI = 1024 / G::K_ROWB;
    constexpr int V_NI = BN * G::V_ROWB / 4096, K_NI = G::K_ROWS * G::K_ROWB / 4096;  // blocks per wavefront
    constexpr int NDMA = V_NI + K_NI;  // copy instructions per wavefront and tile, on every path
    static_assert(V_NI >= 1 && K_NI >= 1 && NDMA * (PD - 1) < 64, "tile shape");
    auto issue_tile_general = [&](const SegPlan& pl, int tile, int stage) {
        const int j0 = tile * BN;
        char* ks_w = smem + stage * G::STAGE;
        char* vs_w = ks_w + G::K_BYTES;
        auto key_row = [&](int row) { return min(max(pl.c0 + pl.cs * (j0 + row), 0), L - 1); };
        dma_tile<T, G::V_ROWB, BN, (ES == 2 ? 2 : 0)>(vs_w, wave, lane, [&](int row) { return vb + (int64_t)key_row(row) * p.v_sl; });
        if constexpr (KT) {
            // rows = contraction index, BN consecutive keys per row (dense walk); a chunk that would run past
            // the last key is replaced by the last whole chunk (those positions are never live)
#pragma unroll
            for (int i = 0; i < K_NI; ++i) {
                const int q = wave + 4 * i;
                const int flat = q * 64 + lane;
                const int row = flat / K_CPR, pc = flat % K_CPR;
                const int lc = logical_chunk<G::K_ROWB, (ES == 2 ? 2 : 0)>(row, pc);
                const int c = min(pl.c0 + j0 + lc * G::EPC, L - G::EPC);
                dma16(kb + (int64_t)row * p.k_sd + c, ks_w + q * 1024);
            }
        } else {
            dma_tile<T, G::K_ROWB, BN, 1>(ks_w, wave, lane, [&](int row) { return kb + (int64_t)key_row(row) * p.k_sl; });
        }
    };
    // FAST_DMA state for the segment being fetched: per-lane byte offsets inside a block, wavefront-uniform
    // running pointers to block `wave` of the next tile, and the byte distance between tile positions.
    uint32_t v_lane_off = 0, k_lane_off = 0;
    bool lane_off_fits = true;  // the copy instruction takes a 32-bit per-lane offset: wider ones go the general way
    const char* v_next = nullptr;
    const char* k_next = nullptr;
    int64_t v_key = 0, k_key = 0;  // bytes from one tile position to the next (K^T layout: from one d row to the next)
    auto set_lane_offsets = [&](const SegPlan& pl) {
        if constexpr (FAST_DMA) {
            const int vr = lane / V_CPR, vpc = lane % V_CPR;
            // the largest offsets of the segment: the last row of a block, with gathered rows pl.cs keys apart
            const int64_t v_far = (int64_t)pl.cs * (V_RPI - 1) * p.v_sl * ES + G::V_ROWB;
            const int64_t k_far = KT ? (int64_t)(K_RPI - 1) * p.k_sd * ES + G::K_ROWB : (int64_t)pl.cs * (K_RPI - 1) * p.k_sl * ES + G::K_ROWB;
            lane_off_fits = v_far < ((int64_t)1 << 32) && k_far < ((int64_t)1 << 32);
            v_lane_off = (uint32_t)((int64_t)pl.cs * vr * p.v_sl * ES) + logical_chunk<G::V_ROWB, 2>(vr, vpc) * 16;
            v_key = (int64_t)p.v_sl * ES * pl.cs;
            v_next = reinterpret_cast<const char*>(vb) + (int64_t)pl.c0 * p.v_sl * ES + (int64_t)wave * V_RPI * v_key;
            const int kr = lane / K_CPR, kpc = lane % K_CPR;
            if constexpr (KT) {
                k_lane_off = (uint32_t)((int64_t)kr * p.k_sd * ES) + logical_chunk<G::K_ROWB, 2>(kr, kpc) * 16;
                k_key = (int64_t)p.k_sd * ES;
                k_next = reinterpret_cast<const char*>(kb) + (int64_t)pl.c0 * ES + (int64_t)wave * K_RPI * k_key;
            } else {
                k_lane_off = (uint32_t)((int64_t)pl.cs * kr * p.k_sl * ES) +
                             logical_chunk<G::K_ROWB, 1>(wave * K_RPI + kr, kpc) * 16;
                k_key = (int64_t)p.k_sl * ES * pl.cs;
                k_next = reinterpret_cast<const char*>(kb) + (int64_t)pl.c0 * p.k_sl * ES + (int64_t)wave * K_RPI * k_key;
            }
        }
    };
    // whether every key of the tile exists, so that the running pointers can be used as they are
    auto tile_is_fast = [&](const SegPlan& pl, int tile) {
        const int j0 = tile * BN;
        const int key_first = pl.c0 + pl.cs * j0, key_last = pl.c0 + pl.cs * (j0 + BN - 1);
        bool fast = FAST_DMA && lane_off_fits && key_last < L;
        if constexpr (KT) fast = fast && (key_first + BN <= L);
        return fast;
    };
    // copy instruction i (0 .. NDMA-1) of the tile the running pointers stand at
    auto issue_step = [&](int i, int stage) {
        char* ks_w = smem + stage * G::STAGE;
        char* vs_w = ks_w + G::K_BYTES;
        if (i < V_NI)
            dma16_uniform(v_next + (int64_t)(4 * V_RPI * i) * v_key, v_lane_off, vs_w + (wave + 4 * i) * 1024);
        else
            dma16_uniform(k_next + (int64_t)(4 * K_RPI * (i - V_NI)) * k_key, k_lane_off, ks_w + (wave + 4 * (i - V_NI)) * 1024);
    };

    int pf_seg = 0, pf_tile = 0;  // position of the next tile to fetch
    SegPlan ppl = {0, 1, 0, 1};
    // move on to the first segment at or after pf_seg that has tiles and take its plan into scalar registers
    auto pf_enter_segment = [&]() {
        pf_tile = 0;
        while (pf_seg < p.n_seg) {
            ppl = seg_plan_of(pf_seg);
            if (ppl.n_tiles > 0) break;
            ++pf_seg;
        }
        if (pf_seg < p.n_seg) set_lane_offsets(ppl);
    };
    // Tiles of a segment are fetched in order, so the running pointers advance by one tile per fetch; LDS is
    // only consulted at the end of a segment.
    auto advance_fetch = [&]() {
        v_next += BN * v_key;
        k_next += KT ? (int64_t)(BN * ES) : BN * k_key;
        if (++pf_tile >= ppl.n_tiles) {
            ++pf_seg;
            pf_enter_segment();
        }
    };
    f32x16 o_acc[DT];
    float m_ref = kNegBigA, l_run = 0.f;

    // ---- LDS read addresses: lane-dependent part + current stage; tile constants go into the instruction's
    // immediate offset; the stage offset is added once per tile -------------------------------------------
    const uint32_t smem_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    // transposing reads: lane s of a 16-lane block addresses row s/4, 8 bytes at element column 16*(block%2) + 4*(s%4)
    const int tr_row = (lane & 15) >> 2;
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t k_addr[KT ? NT : KS];  // K tile: row-major: (row lm, swizzled chunk of step ks); K^T: (row 8g + tr_row, block nt)
    uint32_t v_addr[DT];            // V tile: (row 4g + tr_row, swizzled 64-byte block dt, column tr_col)
    if constexpr (ES == 2) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            v_addr[dt] = smem_base + G::K_BYTES + (4 * g + tr_row) * G::V_ROWB +
                         ((dt ^ swz64<G::V_ROWB>(4 * g + tr_row)) * 64) + tr_col * 2;
        if constexpr (KT) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                k_addr[nt] = smem_base + (8 * g + tr_row) * G::K_ROWB + ((nt ^ swz64<G::K_ROWB>(8 * g + tr_row)) * 64) + tr_col * 2;
        } else {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) k_addr[ks] = smem_base + lds_off<G::K_ROWB, true>(lm, (16 * ks + 8 * g) * ES);
        }
    } else {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_addr[dt] = smem_base + G::K_BYTES + (32 * dt + lm) * 4;
#pragma unroll
        for (int i = 0; i < (KT ? NT : KS); ++i) k_addr[i] = smem_base;
    }

    // Two ways to take a tile's exponentials.  The careful one tracks the row maxima and moves the reference (with a
    // rescale of O and l) when they outrun it.  Once every row of the wavefront has a reference, the fast one leaves the
    // references where they are: no maxima, no exchange between the half rows, no data-dependent branch between the
    // score MFMAs and the exponentials.  That is exact as long as nothing overflows (float range for 32-bit and bf16
    // probabilities, 65504 for fp16 ones); if a later score outruns a row's reference by more than that, the row's sum
    // or output turns infinite or NaN and stays so, which is checked after the last tile, and the workgroup then
    // repeats its tiles on the careful path alone.
    bool careful_only = false;
    int stage_it = 0;  // stage that holds the tile being computed (the LDS read addresses stand at it)
    for (;;) {
        pf_seg = 0;
        pf_enter_segment();
        // the row windows of the first segment with tiles: requested here, long before the loop needs them
        PlanRec win_rec = {0, 0, 1, 0};
        if constexpr (PLANNED) {
            if (pf_seg < p.n_seg) win_rec = pt[plan_row_at(n_rb, p.n_seg, rb, pf_seg, wave * 32 + lm)];
        }
#pragma unroll
        for (int i = 0; i < PD; ++i) {
            if (i < total_tiles) {
                if (tile_is_fast(ppl, pf_tile)) {
#pragma unroll
                    for (int s = 0; s < NDMA; ++s) issue_step(s, (stage_it + i) % NSTAGE);
                } else {
                    issue_tile_general(ppl, pf_tile, (stage_it + i) % NSTAGE);
                }
                advance_fetch();
            }
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 16; ++j) o_acc[dt][j] = 0.f;
        m_ref = kNegBigA;
        l_run = 0.f;

        // per-lane row map of the segment being computed
        int cur_seg = -1, cur_tile = 0;
        RowWin win = {0, 0, 1};
        int first = 0, dec = 0;  // periodic part of the row mask of dense plans: see row_live_bits
        uint64_t pat = ~0ull;
        int w_lo_min = 0, w_lo_max = 0, w_hi_min = 0, w_hi_max = 0;
        SegPlan cpl = {0, 1, 0, 1};
        const float c2 = p.scale_log2e;
        bool settled = false;         // every row of this wavefront has a reference
        int stage_pf = (stage_it + PD) % NSTAGE;  // stage the next fetch goes to
        // The Q fragments have to be in their registers before the loop: otherwise the compiler puts its waits for them
        // in front of the first score MFMAs of every tile, counted against the loads it knows of, and those waits would
        // then hold for the copies of the next tile that are in flight at that point.
#if defined(__HIP_DEVICE_COMPILE__)  // the register constraint means something else to the host pass
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(qf[ks].v));
#endif

        for (int it = 0; it < total_tiles; ++it) {
            // advance the compute position; reload the row map on a segment change
            if (cur_seg < 0 || cur_tile >= cpl.n_tiles) {
                do {
                    ++cur_seg;
                    cpl = seg_plan_of(cur_seg);
                } while (cpl.n_tiles == 0);
                cur_tile = 0;
                WaveSpan sp;
                if constexpr (PLANNED) {
                    if (it > 0) win_rec = pt[plan_row_at(n_rb, p.n_seg, rb, cur_seg, wave * 32 + lm)];
                    win.lo = win_rec.x, win.cnt = win_rec.y, win.lin = win_rec.z;
                    first = win_rec.w;
                    const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, cur_seg, wave));
                    sp.lo_min = r.x, sp.lo_max = r.y, sp.hi_min = r.z, sp.hi_max = r.w;
                } else {
                    win = make_row_win(cached_row_map<BM>(&s_ps, cur_seg, wave * 32 + lm), cpl);
                    first = cpl.uniform ? 0 : win_phase(win);
                    sp = wave_span(win, cpl.uniform != 0);
                }
                if (!cpl.uniform) {
                    // periodic part of the row's live positions (position 0 of the walk is column c0)
                    dec = BN % win.lin;
                    uint64_t pt_bits = 0;
                    for (int q = 0; q < 64; q += win.lin) pt_bits |= 1ull << q;
                    pat = pt_bits;
                } else {  // unit step: every position of the span
                    pat = ~0ull;
                }
                w_lo_min = sp.lo_min, w_lo_max = sp.lo_max, w_hi_min = sp.hi_min, w_hi_max = sp.hi_max;
                if constexpr (PLANNED) {
                    // keep the spans in vector registers, as the reductions of the other path leave them
                    asm volatile("v_mov_b32 %0, %0" : "+v"(w_lo_min));
                    asm volatile("v_mov_b32 %0, %0" : "+v"(w_lo_max));
                    asm volatile("v_mov_b32 %0, %0" : "+v"(w_hi_min));
                    asm volatile("v_mov_b32 %0, %0" : "+v"(w_hi_max));
                }
            }
            const int j0 = cur_tile * BN;
            ++cur_tile;

            // This wavefront's part of tile `it` has landed once at most the copies of the later tiles in flight
            // are outstanding; after the barrier every part has, and every wavefront is done with tile it - 1,
            // whose stage the next fetch overwrites.
            {
                const int later = total_tiles - 1 - it;
                if (PD == 1 || later == 0)
                    wait_loads<0>();
                else if (later == 1)
                    wait_loads<NDMA>();
                else
                    wait_loads<NDMA*(PD > 1 ? PD - 1 : 1)>();
            }
            __builtin_amdgcn_s_barrier();

            const bool fetch = (it + PD < total_tiles);
            bool spread = false;  // the fetch is issued piecewise between the matrix instructions below
            if (fetch) {
                spread = tile_is_fast(ppl, pf_tile);
                if (!spread) issue_tile_general(ppl, pf_tile, stage_pf);
            }

            const bool skip = (j0 + BN <= w_lo_min) || (j0 >= w_hi_max);
            if (!skip) {
                const bool full = (j0 >= w_lo_max) && (j0 + BN <= w_hi_min);

                // ---- S^T = K . Q^T ----
                // K fragments are requested from LDS a few MFMAs ahead of their use, never more than 12 read
                // instructions at a time: the counter that tracks them holds 15, and the compiler falls back to
                // waiting for every outstanding read once it could overflow.
                f32x16 s_acc[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int j = 0; j < 16; ++j) s_acc[nt][j] = 0.f;
                Frag<T> kfr[NT][KS];
                auto load_k = [&](int nt, int ks) {
                    Frag<T> kf;
                    if constexpr (ES == 2) {
                        if constexpr (KT) {
                            // rows 16ks + 8g + {0..3} and +4: multiples of 4 rows leave the lane's swizzle term alone
                            const uint32_t a0 = k_addr[nt] + 16 * ks * G::K_ROWB;
                            kf = frag_from_tr<T>(lds_load_tr16(a0), lds_load_tr16(a0 + 4 * G::K_ROWB));
                        } else {
                            kf.v = __builtin_bit_cast(typename Frag<T>::vec, lds_load128(k_addr[ks] + 32 * nt * G::K_ROWB));
                        }
                    } else {
                        const char* ks_l = smem + stage_it * G::STAGE;
                        if constexpr (KT) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                kf.v[e] = *reinterpret_cast<const float*>(ks_l + (16 * ks + 8 * g + e) * G::K_ROWB + (32 * nt + lm) * 4);
                        } else {
                            kf = lds_frag_row_swz<T, G::K_ROWB>(ks_l, 32 * nt + lm, 16 * ks + 8 * g);
                        }
                    }
                    return kf;
                };
                constexpr int NMMA = NT * KS;
                constexpr int K_AHEAD = (ES != 2) ? NMMA : ((KT ? 6 : 12) < NMMA ? (KT ? 6 : 12) : NMMA);  // fragments
#pragma unroll
                for (int i = 0; i < K_AHEAD; ++i) kfr[i / KS][i % KS] = load_k(i / KS, i % KS);
                __builtin_amdgcn_sched_barrier(0);  // keep the requests above the matrix work
                // the copy instructions of the fetch go between the MFMAs, so that the address path sees them at
                // the rate it can take instead of as one burst that stalls the wavefront
                constexpr int MMA_PER_DMA = (NMMA / NDMA) > 0 ? NMMA / NDMA : 1;
#pragma unroll
                for (int i = 0; i < NMMA; ++i) {
                    mma32(s_acc[i / KS], kfr[i / KS][i % KS], qf[i % KS]);
                    if (i + K_AHEAD < NMMA) {
                        kfr[(i + K_AHEAD) / KS][(i + K_AHEAD) % KS] = load_k((i + K_AHEAD) / KS, (i + K_AHEAD) % KS);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if constexpr (FAST_DMA) {
                        if ((i + 1) % MMA_PER_DMA == 0 && (i + 1) / MMA_PER_DMA <= NDMA) {
                            if (spread) issue_step((i + 1) / MMA_PER_DMA - 1, stage_pf);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                if constexpr (FAST_DMA && (NMMA / MMA_PER_DMA < NDMA)) {
                    if (spread) {
#pragma unroll
                        for (int s = NMMA / MMA_PER_DMA; s < NDMA; ++s) issue_step(s, stage_pf);
                    }
                }
                // ---- mask, online softmax against a lazily updated reference ----
                Frag<T> pf[NT][2];
                if (!full) mask_tile<NT>(s_acc, row_live_bits(win, j0, first, pat), g);
                if (settled && !careful_only)
                    l_run += exp_tile<NT, T>(s_acc, pf, m_ref * c2, c2);
                else
                    settled = softmax_tile<NT, T, DT>(s_acc, pf, m_ref, l_run, o_acc, c2);

                // ---- O^T += V^T . P^T ----
                // V fragments are requested one 16-key step (DT fragments) ahead of the MFMAs that consume them.
                auto load_v = [&](int nt, int t, int dt) {
                    Frag<T> vf;
                    if constexpr (ES == 2) {
                        const uint32_t a0 = v_addr[dt] + (32 * nt + 16 * t) * G::V_ROWB;
                        vf = frag_from_tr<T>(lds_load_tr16(a0), lds_load_tr16(a0 + 8 * G::V_ROWB));
                    } else {
                        const int rbase = 32 * nt + 16 * t + 4 * g;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            vf.v[e] = lds_load_f32(v_addr[dt] + (rbase + e) * G::V_ROWB);
                            vf.v[4 + e] = lds_load_f32(v_addr[dt] + (rbase + 8 + e) * G::V_ROWB);
                        }
                    }
                    return vf;
                };
                Frag<T> vfr[2][DT];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) vfr[0][dt] = load_v(0, 0, dt);
                __builtin_amdgcn_sched_barrier(0);  // keep the requests above the matrix work
#pragma unroll
                for (int step = 0; step < 2 * NT; ++step) {
                    const int nt = step >> 1, t = step & 1;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        mma32(o_acc[dt], vfr[step & 1][dt], pf[nt][t]);
                        if (step + 1 < 2 * NT) {
                            vfr[(step + 1) & 1][dt] = load_v((step + 1) >> 1, (step + 1) & 1, dt);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            } else if (spread) {
#pragma unroll
                for (int s = 0; s < NDMA; ++s) issue_step(s, stage_pf);
            }

            if (fetch) {
                advance_fetch();
                stage_pf = (stage_pf + 1 == NSTAGE) ? 0 : stage_pf + 1;
            }
            if (!cpl.uniform) {  // phase of the periodic mask at the next tile
                const int f = first - dec;
                first = f < 0 ? f + win.lin : f;
            }
            // the next stage becomes current
            stage_it = (stage_it + 1 == NSTAGE) ? 0 : stage_it + 1;
            const int delta = (stage_it == 0) ? -(NSTAGE - 1) * G::STAGE : G::STAGE;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) v_addr[dt] += delta;
#pragma unroll
            for (int i = 0; i < (KT ? NT : KS); ++i) k_addr[i] += delta;
        }
        // Every copy has been waited for (the last tile waits for all).  The barrier in here also makes the stages free
        // for the epilogue (or the second pass): every wavefront has finished reading the last tile.
        const bool bad = !careful_only && (!(l_run < 1.0e30f) || !(fabsf(o_acc[0][0]) < 1.0e30f));
        if (!__syncthreads_or(bad ? 1 : 0)) break;
        careful_only = true;  // the ring goes on from the stage it stands at
    }

    // ---- epilogue: O = O^T / l, transposed through LDS so that every global store is a contiguous run --------
    {
        constexpr int OROW = D * ES + 16;  // padded row of the staging tile
        static_assert(4 * 32 * OROW <= NSTAGE * G::STAGE, "staging space");
        char* stg = smem + wave * (32 * OROW);
        const float l_tot = l_run + __shfl_xor(l_run, 32);
        const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
        if (p.lse != nullptr && g == 0) {
            // probabilities are exp(scale * score - lse); a row without live columns gets +inf (every probability 0)
            const int my_row = r0 + rs * (wave * 32 + lm);
            const float lse = l_tot > 0.f ? (m_ref * p.scale_log2e + __log2f(l_tot)) * 0.6931471805599453f : __builtin_inff();
            if (my_row < L) p.lse[(int64_t)bh * L + my_row] = lse;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (T)(o_acc[dt][4 * jj + i] * inv);
                *reinterpret_cast<vec4*>(stg + lm * OROW + (32 * dt + 8 * jj + 4 * g) * ES) = o;
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wavefront's LDS writes are visible to its own reads
        constexpr int CPR = D * ES / 16;                    // 16-byte chunks per output row
#pragma unroll
        for (int i = 0; i < 32 * CPR / 64; ++i) {
            const int flat = i * 64 + lane;
            const int row = flat / CPR, c = flat % CPR;
            const int r = r0 + rs * (wave * 32 + row);
            const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * OROW + c * 16);
            // non-temporal: whole aligned rows that this kernel never reads back, so they need not pass through the L2
            if (r < L) __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(reinterpret_cast<char*>(ob + (int64_t)r * p.o_sl) + c * 16));
        }
    }
}

template <typename T, int D, bool KT, int BN, int NSTAGE, bool PLANNED>
static int launch_attn(const AttnParams& p0, hipStream_t st) {
    begin_launch();
    using G = TileGeom<T, D, KT, BN>;
    AttnParams p = p0;
    constexpr int BM = 128;
    p.n_row_blocks = count_row_blocks(p.L, BM, p.row_stride);
    p.total = p.B * p.H * p.n_row_blocks;
    if (PLANNED && KT) p.plan += plan_variant_recs(p.n_row_blocks, p.n_seg);  // the dense-walk variant
    const int grid = ((p.total + 7) / 8) * 8;
    const size_t lds = NSTAGE * (size_t)G::STAGE;
    auto kern = attn_fwd_kernel<T, D, KT, BN, NSTAGE, PLANNED>;
    static uint64_t lds_reserved = 0;  // per instantiation: devices whose copy of this kernel has the limit raised
    if (int rc = reserve_dynamic_lds(&lds_reserved, reinterpret_cast<const void*>(kern), lds, "splat_attention_fwd")) return rc;
    kern<<<grid, 256, lds, st>>>(p);
    return check_launch("splat_attention_fwd");
}

// One 32-row tile per wavefront (128 rows per workgroup): 16-bit kernels then fit two workgroups per CU, whose
// wavefronts hide part of each other's LDS, barrier and prologue latency.  Tiles of 64 keys, double buffered (the
// kernel also supports 32-key tiles in a ring of 4 stages; it measured slower at d = 128 and equal at d = 64).
template <typename T>
static int dispatch_attn(const AttnParams& p, int d, bool kt, hipStream_t st) {
    if (p.plan) {
        if (d == 64) return kt ? launch_attn<T, 64, true, 64, 2, true>(p, st) : launch_attn<T, 64, false, 64, 2, true>(p, st);
        return kt ? launch_attn<T, 128, true, 64, 2, true>(p, st) : launch_attn<T, 128, false, 64, 2, true>(p, st);
    }
    if (d == 64) return kt ? launch_attn<T, 64, true, 64, 2, false>(p, st) : launch_attn<T, 64, false, 64, 2, false>(p, st);
    return kt ? launch_attn<T, 128, true, 64, 2, false>(p, st) : launch_attn<T, 128, false, 64, 2, false>(p, st);
}

// One workgroup per (row block, variant): the same planning code the unplanned kernel runs in its prologue, with
// the results written to the table.
struct PlanParams {
    PlanRec* table;
    SegPtrs seg[SPLAT_MAX_SEGMENTS];
    int n_seg, L, rs, n_rb;
};
__global__ __launch_bounds__(256) void attn_plan_kernel(const PlanParams p) {
    constexpr int BM = kPlanBM, BN = 64;
    __shared__ SegPlan s_plan[SPLAT_MAX_SEGMENTS];
    __shared__ PlanScratch<BM> s_ps;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lm = lane & 31;
    const int rb = blockIdx.x, variant = blockIdx.y;
    const int n_seg = p.n_seg, n_rb = p.n_rb;
    PlanRec* const pt = p.table + variant * plan_variant_recs(n_rb, n_seg);
    plan_segments<BM, BN>(p.seg, n_seg, block_first_row(rb, BM, p.rs), p.rs, p.L, variant == 0, s_plan, &s_ps, tid);
    for (int sg = 0; sg < n_seg; ++sg) {
        const SegPlan pl = s_plan[sg];
        const RowWin win = make_row_win(cached_row_map<BM>(&s_ps, sg, wave * 32 + lm), pl);
        const WaveSpan sp = wave_span(win, pl.uniform != 0);
        if (tid == 0) pt[plan_seg_at(n_seg, rb, sg)] = PlanRec{pl.c0, pl.cs, pl.n_tiles, pl.uniform};
        if (lane == 0) pt[plan_span_at(n_rb, n_seg, rb, sg, wave)] = PlanRec{sp.lo_min, sp.lo_max, sp.hi_min, sp.hi_max};
        if (lane < 32)
            pt[plan_row_at(n_rb, n_seg, rb, sg, wave * 32 + lm)] = PlanRec{win.lo, win.cnt, win.lin, pl.uniform ? 0 : win_phase(win)};
    }
}

}  // namespace splat

using namespace splat;

static int attention_fwd_common(const char* who, const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v, int64_t v_sb,
                                int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb, int64_t o_sh, int64_t o_sl,
                                const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d,
                                float scale, int32_t dtype, const void* plan, int64_t plan_bytes, bool planned,
                                float* lse, void* stream) {
    if (!q || !kT || !v || !out || !segs) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (B <= 0 || H <= 0 || L <= 0) return fail(SPLAT_E_SHAPE, "%s: need B, H, L > 0 (got %d, %d, %d)", who, B, H, L);
    if (L > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: L is limited to 2^23 (got %d)", who, L);
    if (d != 64 && d != 128) return fail(SPLAT_E_UNSUPPORTED, "%s: head dim must be 64 or 128 (got %d)", who, d);
    if (dtype != SPLAT_F32 && dtype != SPLAT_F16 && dtype != SPLAT_BF16)
        return fail(SPLAT_E_DTYPE, "%s: unknown dtype %d", who, dtype);
    // the running max is taken over unscaled scores (needs scale >= 0) and masked scores are zeroed through
    // the underflow of exp2(-1e30 * scale) (needs scale > 0)
    if (!(scale > 0.f)) return fail(SPLAT_E_UNSUPPORTED, "%s: scale must be > 0 (got %g)", who, (double)scale);
    const int es = dtype == SPLAT_F32 ? 4 : 2;
    const int epc = 16 / es;
    bool kt;
    if (k_sd == 1 && (k_sl % epc) == 0 && k_sl >= d)
        kt = false;  // rows of K are contiguous: [.., L, d] memory viewed as [.., d, L]
    else if (k_sl == 1)
        kt = true;  // K^T contiguous: [.., d, L] memory
    else
        return fail(SPLAT_E_ALIGN, "%s: kT needs unit stride along d (k_sd == 1) or along keys (k_sl == 1); got k_sd=%lld k_sl=%lld", who,
                    (long long)k_sd, (long long)k_sl);
    if (kt && ((L % epc) != 0 || (k_sd % epc) != 0 || L < epc))
        return fail(SPLAT_E_ALIGN, "%s: with K^T contiguous along keys, L and the d-stride must be multiples of %d (got L=%d, k_sd=%lld)", who,
                    epc, L, (long long)k_sd);
    auto mis = [&](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
    auto bad = [&](int64_t s) { return (s % epc) != 0; };
    if (mis(q) || mis(kT) || mis(v) || mis(out)) return fail(SPLAT_E_ALIGN, "%s: q, kT, v and out must be 16-byte aligned", who);
    if (bad(q_sb) || bad(q_sh) || bad(q_sl) || bad(k_sb) || bad(k_sh) || bad(v_sb) || bad(v_sh) || bad(v_sl) || bad(o_sb) || bad(o_sh) || bad(o_sl))
        return fail(SPLAT_E_ALIGN, "%s: every batch/head/row stride must be a multiple of %d elements (16 bytes)", who, epc);
    if (q_sl < d || v_sl < d || o_sl < d) return fail(SPLAT_E_SHAPE, "%s: row strides must be >= d", who);

    AttnParams p;
    p.q = q; p.k = kT; p.v = v; p.o = out;
    p.q_sb = q_sb; p.q_sh = q_sh; p.q_sl = q_sl;
    p.k_sb = k_sb; p.k_sh = k_sh; p.k_sd = k_sd; p.k_sl = k_sl;
    p.v_sb = v_sb; p.v_sh = v_sh; p.v_sl = v_sl;
    p.o_sb = o_sb; p.o_sh = o_sh; p.o_sl = o_sl;
    p.B = B; p.H = H; p.L = L;
    p.scale_log2e = scale * 1.4426950408889634f;
    p.n_seg = n_seg;
    if (int rc = fill_segs(who, segs, n_seg, p.seg, -1)) return rc;
    p.row_stride = common_row_stride(segs, n_seg);
    p.plan = nullptr;
    p.lse = lse;
    if (planned) {
        if (!plan) return fail(SPLAT_E_NULL, "%s: null plan", who);
        if ((reinterpret_cast<uintptr_t>(plan) & 15) != 0) return fail(SPLAT_E_ALIGN, "%s: the plan must be 16-byte aligned", who);
        const int64_t need = splat_attention_plan_bytes(segs, n_seg, L);
        if (plan_bytes < need)
            return fail(SPLAT_E_SHAPE, "%s: the plan holds %lld bytes, this mask needs %lld", who, (long long)plan_bytes, (long long)need);
        p.plan = static_cast<const PlanRec*>(plan);
    }
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case SPLAT_F32: return dispatch_attn<float>(p, d, kt, st);
        case SPLAT_F16: return dispatch_attn<f16>(p, d, kt, st);
        default: return dispatch_attn<bf16>(p, d, kt, st);
    }
}

extern "C" int splat_attention_fwd(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT, int64_t k_sb,
                                   int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v, int64_t v_sb, int64_t v_sh,
                                   int64_t v_sl, void* out, int64_t o_sb, int64_t o_sh, int64_t o_sl,
                                   const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H, int32_t L, int32_t d,
                                   float scale, int32_t dtype, void* stream) {
    return attention_fwd_common("splat_attention_fwd", q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, v, v_sb, v_sh, v_sl, out,
                                o_sb, o_sh, o_sl, segs, n_seg, B, H, L, d, scale, dtype, nullptr, 0, false, nullptr, stream);
}

extern "C" int splat_attention_fwd_planned(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                           int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                                           int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb, int64_t o_sh,
                                           int64_t o_sl, const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H,
                                           int32_t L, int32_t d, float scale, int32_t dtype, const void* plan,
                                           int64_t plan_bytes, void* stream) {
    return attention_fwd_common("splat_attention_fwd_planned", q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, v, v_sb, v_sh,
                                v_sl, out, o_sb, o_sh, o_sl, segs, n_seg, B, H, L, d, scale, dtype, plan, plan_bytes, true,
                                nullptr, stream);
}

extern "C" int splat_attention_fwd_stats(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                         int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                                         int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb, int64_t o_sh,
                                         int64_t o_sl, const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H,
                                         int32_t L, int32_t d, float scale, int32_t dtype, const void* plan,
                                         int64_t plan_bytes, float* lse, void* stream) {
    const char* who = "splat_attention_fwd_stats";
    if (!lse) return fail(SPLAT_E_NULL, "%s: null lse", who);
    if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0) return fail(SPLAT_E_ALIGN, "%s: lse must be 4-byte aligned", who);
    return attention_fwd_common(who, q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, v, v_sb, v_sh, v_sl, out, o_sb, o_sh,
                                o_sl, segs, n_seg, B, H, L, d, scale, dtype, plan, plan_bytes, plan != nullptr, lse, stream);
}

// ---- the forward for callers that cannot allocate: the plan lives in a file-scope device array ----------------
constexpr int64_t kStaticPlanBytes = SPLAT_STATIC_PLAN_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticPlanBytes];
// Host code must not use the array's name as an address: each device holds its own copy, whose address the runtime
// hands out.  Resolved once per device, with that device current.
static std::mutex g_scratch_lock;
static void* g_scratch_ptr[64] = {};
static int static_plan_buffer(const char* who, void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(SPLAT_E_UNSUPPORTED, "%s: device ordinal %d is beyond the 64 this table holds", who, dev);
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(e != hipSuccess ? (int)e : SPLAT_E_NULL, "%s: cannot resolve the plan buffer on device %d: %s", who, dev,
                        hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

extern "C" int64_t splat_attention_plan_bytes(const splat_acsr_seg* segs, int32_t n_seg, int32_t L) {
    if (!segs || n_seg < 1 || n_seg > SPLAT_MAX_SEGMENTS || L <= 0) return 0;
    const int n_rb = count_row_blocks(L, kPlanBM, common_row_stride(segs, n_seg));
    return 2 * plan_variant_recs(n_rb, n_seg) * (int64_t)sizeof(PlanRec);
}

extern "C" int splat_attention_plan(const splat_acsr_seg* segs, int32_t n_seg, int32_t L, void* plan, int64_t plan_bytes,
                                    void* stream) {
    begin_launch();
    const char* who = "splat_attention_plan";
    if (!segs || !plan) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (L <= 0 || L > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: need 0 < L <= 2^23 (got %d)", who, L);
    if ((reinterpret_cast<uintptr_t>(plan) & 15) != 0) return fail(SPLAT_E_ALIGN, "%s: the plan must be 16-byte aligned", who);
    PlanParams p;
    if (int rc = fill_segs(who, segs, n_seg, p.seg, -1)) return rc;
    const int64_t need = splat_attention_plan_bytes(segs, n_seg, L);
    if (plan_bytes < need)
        return fail(SPLAT_E_SHAPE, "%s: the plan needs %lld bytes for this mask, got %lld", who, (long long)need, (long long)plan_bytes);
    p.table = static_cast<PlanRec*>(plan);
    p.n_seg = n_seg;
    p.L = L;
    p.rs = common_row_stride(segs, n_seg);
    p.n_rb = count_row_blocks(L, kPlanBM, p.rs);
    attn_plan_kernel<<<dim3(p.n_rb, 2), 256, 0, (hipStream_t)stream>>>(p);
    return check_launch(who);
}

extern "C" int splat_attention_fwd_noalloc(const void* q, int64_t q_sb, int64_t q_sh, int64_t q_sl, const void* kT,
                                           int64_t k_sb, int64_t k_sh, int64_t k_sd, int64_t k_sl, const void* v,
                                           int64_t v_sb, int64_t v_sh, int64_t v_sl, void* out, int64_t o_sb, int64_t o_sh,
                                           int64_t o_sl, const splat_acsr_seg* segs, int32_t n_seg, int32_t B, int32_t H,
                                           int32_t L, int32_t d, float scale, int32_t dtype, void* stream) {
    const char* who = "splat_attention_fwd_noalloc";
    if (!segs) return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (L <= 0 || L > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: need 0 < L <= 2^23 (got %d)", who, L);
    const int64_t need = splat_attention_plan_bytes(segs, n_seg, L);
    if (need <= 0) return fail(SPLAT_E_SHAPE, "%s: no plan for n_seg=%d, L=%d", who, n_seg, L);
    if (need > kStaticPlanBytes)
        return fail(SPLAT_E_SHAPE,
                    "%s: this mask's plan needs %lld bytes, the built-in buffer holds %lld (about %lld row blocks of 128 rows "
                    "times segments); use splat_attention_plan + splat_attention_fwd_planned with a buffer of your own",
                    who, (long long)need, (long long)kStaticPlanBytes,
                    (long long)(kStaticPlanBytes / (2 * plan_variant_recs(1, 1) * (int64_t)sizeof(PlanRec))));
    void* plan = nullptr;
    if (int rc = static_plan_buffer(who, &plan)) return rc;
    // the plan kernel rewrites every record this mask's forward reads, so nothing of an earlier call's plan is seen;
    // the forward follows on the same stream
    if (int rc = splat_attention_plan(segs, n_seg, L, plan, kStaticPlanBytes, stream)) return rc;
    return attention_fwd_common(who, q, q_sb, q_sh, q_sl, kT, k_sb, k_sh, k_sd, k_sl, v, v_sb, v_sh, v_sl, out, o_sb, o_sh, o_sl,
                                segs, n_seg, B, H, L, d, scale, dtype, plan, kStaticPlanBytes, true, nullptr, stream);
}
