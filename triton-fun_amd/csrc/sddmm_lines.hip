// SDDMM on ACSR for the common fast shape: 16-bit inputs and outputs of one type, d = 64 or 128, rows of K contiguous,
// 16-byte alignment everywhere, at least 256 row blocks in the launch or rows of at most 256 slots.
//
// A workgroup of 8 wavefronts owns 128 rows of one (batch, head); wavefront w owns rows 16w..16w+15 and computes
// S^T = K Q^T with 16x16x32 MFMAs (rows = keys, columns = queries: a lane owns one query row and, per 16-key block, 4
// consecutive key positions).  Thin wavefronts keep the register count below 128, so that four of them share a SIMD:
// the kernel is a chain of latencies (copy, barrier, LDS reads, stores), and what hides them is wavefronts in flight.
//
// K reaches LDS without passing through registers (global_load_lds, 1 KiB per wavefront instruction) in steps of 64
// keys through a ring of NST stages, NST - 1 steps ahead, one barrier per step.  Loads complete in order, stores complete
// in order, but the two kinds overtake each other and share one counter: a wait for "all but n" operations proves that
// the copy of the current step has landed only if n is at most the number of copy instructions issued after it.  That
// many stores of the previous half lines may then still be in flight, as long as the younger copies have landed too,
// which they normally have.
//
// Output, uniform plans (every row of the block has the plan's column step and phase, so tile positions are slots): per
// 32 positions the scores go from the accumulators into a per-row ring of 64 slots in LDS (four consecutive slots per
// write, no tests: a position outside the row's span lands on ring entries that are not waiting to be stored), and each
// row stores the 32-slot half lines that have become complete -- 4 lanes x 16 bytes, aligned, non-temporal -- and its
// remainder once its last position has passed.  The ring is filled at position granularity and read at slot granularity:
// a lane reads the 24 aligned bytes around its 8 slots and shifts (a 16-byte LDS read at a 2-byte offset costs several
// times an aligned one).  Other plans (rows with differing steps) walk dense columns and store element by element under
// the row's affine test.
#include <algorithm>
#include <type_traits>

#include "sddmm_params.hpp"
#include "tile_copy.hpp"

namespace splat {

// KEYS: keys per step (64 or 32); HL: slots per store unit (64: whole 128-byte lines, 32: halves of lines)
template <int D, int NST, int KEYS, int HL, int BM_, bool PLANNED>
struct LinesGeom {
    static constexpr int BM = BM_;
    static constexpr int NW = BM / 16;          // wavefronts per workgroup
    static constexpr int ROWB = D * 2;          // bytes per key row
    static constexpr int STAGE = KEYS * ROWB;   // bytes per step
    static constexpr int R_SLOTS = 2 * HL;      // ring slots per row: what waits for its unit to fill up, plus a unit's worth
    // bytes per ring row: 36 or 68 banks, so that the rows one store instruction reads at a time (4 rows 4 apart for
    // half lines, 2 rows 8 apart for lines) spread over all the banks
    static constexpr int R_ROW = R_SLOTS * 2 + 16;
    static constexpr int RING_AT = NST * STAGE;
    static constexpr int PLAN_AT = RING_AT + BM * R_ROW;
    static constexpr int LDS_BYTES = PLANNED ? PLAN_AT : PLAN_AT + (int)sizeof(PlanScratch<BM>) + SPLAT_MAX_SEGMENTS * ((int)sizeof(SegPlan) + 4);
};

template <typename T, int D, int NST, int KEYS, int HL, int BM_, bool PROBS, bool PLANNED>
__global__ __launch_bounds__(BM_ * 4, 4) void sddmm_lines_kernel(const SddmmParams p) {
    using G = LinesGeom<D, NST, KEYS, HL, BM_, PLANNED>;
    static_assert(!PLANNED || BM_ == kPlanBM, "the plan table is laid out for 128-row blocks");
    constexpr int NW = G::NW;
    constexpr int NH = KEYS / 32;  // halves of 32 positions per step
    static_assert(G::STAGE % (NW * 1024) == 0, "every wavefront copies whole kilobytes");
    constexpr int NC = HL / 32;  // store instructions per unit and wavefront (16 or 8 rows each)
    constexpr int BM = G::BM, ROWB = G::ROWB, STAGE = G::STAGE, R_SLOTS = G::R_SLOTS, R_ROW = G::R_ROW;
    constexpr int KS = D / 32;          // MFMA steps over the contraction
    constexpr int CPR = ROWB / 16;      // 16-byte chunks per key row
    constexpr int NI = STAGE / (NW * 1024);  // copy instructions per wavefront and step
    constexpr int AFTER = (NST - 2) * NI;  // copy instructions issued after those of the step that is waited for
    static_assert(G::PLAN_AT % 16 == 0, "plan scratch alignment");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    char* const s_kring = smem;
    char* const s_rings = smem + G::RING_AT;
    PlanScratch<BM>* const s_ps = reinterpret_cast<PlanScratch<BM>*>(smem + G::PLAN_AT);
    SegPlan* const s_plan = reinterpret_cast<SegPlan*>(s_ps + 1);
    int* const s_off = reinterpret_cast<int*>(s_plan + SPLAT_MAX_SEGMENTS);

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

    const T* qb = (const T*)p.q + b * p.q_sb + h * p.q_sh;
    const char* kbytes = reinterpret_cast<const char*>((const T*)p.k + b * p.k_sb + h * p.k_sh);
    const int64_t k_rowb = p.k_sl * 2;

    // B operand: this lane's query row, contraction values 32 ks + 8 g4 .. + 7 (requested before the planning, whose
    // loads and barriers then hide the latency)
    const int my_rr = 16 * wave + li;
    const int my_r = r0 + rs * my_rr;
    const T* qr = qb + (int64_t)min(my_r, L - 1) * p.q_sl;
    Frag<T> qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag<T>(qr + 32 * ks + 8 * g4);
    const float out_scale = PROBS ? 1.0f : p.scale;
    const float exp_mul = p.scale * 1.4426950408889634f;
    float exp_sub = 0.f;
    if constexpr (PROBS) exp_sub = p.row_lse[(int64_t)bh * L + min(my_r, L - 1)] * 1.4426950408889634f;

    // the plan: computed here from the rows' maps, or taken from the mask's plan table (scalar loads for what the copies
    // need, so that they can start at once; no LDS, no barrier)
    if constexpr (!PLANNED) {
        if (tid < SPLAT_MAX_SEGMENTS) s_off[tid] = p.seg[tid].slot_offset;
        plan_segments<BM>(p.seg, p.n_seg, r0, rs, L, true, s_plan, s_ps, tid);
    }
    const PlanRec* const pt = p.plan;
    const int n_rb = p.n_row_blocks;

    // this lane's 16 bytes of each of the step's copy instructions: chunk position `flat` of the stage
    int d_row[NI], d_col[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int flat = (wave + NW * i) * 64 + lane;
        d_row[i] = flat / CPR;
        d_col[i] = logical_chunk<ROWB, 1>(d_row[i], flat % CPR) * 16;
    }
    // fragment addresses: key row li of a 16-key block, chunk 4 ks + g4; rows li and li + 16 k share their swizzle (it
    // depends on the row modulo 16 or, for 128-byte rows, on row / 2 modulo 8)
    static_assert(ROWB == 256 || ROWB == 128, "swizzle period");
    int a_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a_off[ks] = lds_off<ROWB, true>(li, (32 * ks + 8 * g4) * 2);

    char* const ring_mine = s_rings + my_rr * R_ROW;
    // the rows whose units this lane helps to store: HL / 8 lanes per row, 16 or 8 rows per store instruction, picked so
    // that the rows of 16 consecutive lanes spread over all the banks
    int f_rr[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c)
        f_rr[c] = 16 * wave + (HL == 32 ? (lane >> 4) + 4 * ((lane >> 2) & 3) : 4 * c + (lane >> 4) + 8 * ((lane >> 3) & 1));
    const int f_piece = lane & (HL / 8 - 1);
    const int64_t out_bh = (int64_t)bh * L * p.T;

    for (int sg = 0; sg < p.n_seg; ++sg) {
        SegPlan pl;
        if constexpr (PLANNED) {
            const PlanRec r = plan_uniform_load(pt + plan_seg_at(p.n_seg, rb, sg));
            pl = SegPlan{r[0], r[1], r[2], r[3]};
        } else {
            pl = s_plan[sg];
        }
        const int n_steps = pl.n_tiles * (kBN / KEYS);
        if (n_steps == 0) continue;  // workgroup-uniform
        const int off = PLANNED ? p.seg[sg].slot_offset : s_off[sg];
        const bool uniform = pl.uniform != 0;

        auto row_win = [&](int rr) {
            RowWin w;
            if constexpr (PLANNED) {
                // (counts are clamped to the slots the segment owns in this buffer, like the ones read from the metadata)
                const PlanRec r = pt[plan_row_at(n_rb, p.n_seg, rb, sg, rr)];
                const int64_t most = uniform ? (int64_t)p.seg[sg].max_cnt : (int64_t)r[2] * (p.seg[sg].max_cnt - 1) + 1;
                w = RowWin{r[0], (int)min((int64_t)r[1], most), r[2]};
            } else {
                w = make_row_win(cached_row_map<BM>(s_ps, sg, rr), pl);
            }
            if (r0 + rs * rr >= L) w.cnt = 0;
            return w;
        };
        const RowWin mine = row_win(my_rr);
        WaveSpan span;
        if constexpr (PLANNED) {
            // the table holds the spans of 32 rows: wider than this wavefront's 16, which only makes the tests below pass less often
            const PlanRec r = plan_uniform_load(pt + plan_span_at(n_rb, p.n_seg, rb, sg, wave >> 1));
            span = WaveSpan{r[0], r[1], r[2], r[3]};
        } else {
            span = wave_span(mine, uniform);
        }
        const int lmin = span.lo_min, hmax = span.hi_max;
        const int lo4 = mine.lo & ~3;
        const int64_t my_base = out_bh + (int64_t)my_r * p.T + off;

        int f_lo[NC], f_cnt[NC], f_done[NC];
        int64_t f_base[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const RowWin w = row_win(f_rr[c]);
            f_lo[c] = w.lo;
            f_cnt[c] = w.cnt;
            f_done[c] = 0;
            f_base[c] = out_bh + (int64_t)(r0 + rs * f_rr[c]) * p.T + off;
        }

        // Steps whose keys all exist copy from a wavefront-uniform base (the step's first key) plus a per-lane byte offset
        // that is fixed for the segment; the others clamp the key index per lane.
        const bool fast_copy = (int64_t)pl.cs * (KEYS - 1) * k_rowb + ROWB < ((int64_t)1 << 31);
        uint32_t d_off[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) d_off[i] = (uint32_t)((int64_t)pl.cs * d_row[i] * k_rowb + d_col[i]);
        auto issue = [&](int s, auto stage_c) {
            constexpr int stage = decltype(stage_c)::value;
            const int64_t key_first = pl.c0 + (int64_t)pl.cs * (s * KEYS), key_last = key_first + (int64_t)pl.cs * (KEYS - 1);
            if (fast_copy && key_first >= 0 && key_last < p.n_keys) {  // workgroup-uniform
                const char* base = kbytes + key_first * k_rowb;
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    dma16_uniform(base, d_off[i], s_kring + stage * STAGE + (wave + NW * i) * 1024);
                return;
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int n = min(max(pl.c0 + pl.cs * (s * KEYS + d_row[i]), 0), p.n_keys - 1);
                dma16(kbytes + n * k_rowb + d_col[i], s_kring + stage * STAGE + (wave + NW * i) * 1024);
            }
        };

        // every wavefront has finished with the stages of the previous segment
        __builtin_amdgcn_s_barrier();
        int pend_from = -1;  // first position whose scores went into the rings since the last look for units (wavefront-uniform)
        // the stage of a step is its index modulo NST: the loop below is unrolled NST times, so that every LDS address is a
        // per-lane register plus a constant
        static_for<NST - 1>([&](auto u) {
            if (decltype(u)::value < n_steps) issue(decltype(u)::value, u);
        });
        auto step = [&](int s, auto stage_c) {
            constexpr int stage = decltype(stage_c)::value;
            if (s + NST - 2 < n_steps)
                wait_loads<AFTER>();
            else
                wait_loads<0>();
            __builtin_amdgcn_s_barrier();  // step s has landed for everyone, and nobody reads step s - 1 any more
            if (s + NST - 1 < n_steps) issue(s + NST - 1, std::integral_constant<int, (stage + NST - 1) % NST>{});
            typedef T v4 __attribute__((ext_vector_type(4)));
            // wavefront-uniform: which halves of the step hold positions of this wavefront's rows
            const int posA = s * KEYS, posB = posA + 32;
            const bool actA = !(posA + 32 <= lmin || posA >= hmax), actB = NH == 2 && !(posB + 32 <= lmin || posB >= hmax);

            Frag<T> fr[2][2 * KS];
            auto read_frags = [&](int half) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
                        fr[half][2 * ks + kt].v = __builtin_bit_cast(
                            typename Frag<T>::vec, *reinterpret_cast<const u32x4*>(s_kring + a_off[ks] + (stage * STAGE + (32 * half + 16 * kt) * ROWB)));
            };
            f32x4v acc[2][2];
            auto products = [&](int half) {
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[half][kt][j] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt) {
                        mma16(acc[half][kt], fr[half][2 * ks + kt], qf[ks]);
                    }
            };
            // scores of 32 positions into the rows' rings (uniform plans) or straight to their slots (other plans)
            auto put = [&](int half, int pos0) {
                if constexpr (PROBS) {
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int j = 0; j < 4; ++j) acc[half][kt][j] = fast_exp2(fmaf(acc[half][kt][j], exp_mul, -exp_sub));
                }
                if (!uniform) {  // workgroup-uniform
                    T* const row_out = (T*)p.out + my_base;
                    if (mine.cnt > 0) {
#pragma unroll
                        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                const int pos = pos0 + 16 * kt + 4 * g4 + j;
                                if (win_live(mine, pos)) row_out[win_slot(mine, pos)] = (T)(acc[half][kt][j] * out_scale);
                            }
                    }
                    return;
                }
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    v4 t;
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[j] = (T)(acc[half][kt][j] * out_scale);
                    const int ri = (pos0 + 16 * kt + 4 * g4 - lo4) & (R_SLOTS - 1);
                    *reinterpret_cast<v4*>(ring_mine + ri * 2) = t;
                }
            };
            // 8 slots of row f_rr[c] from ring entry s0 + f_lo % 4 on (slot s sits at ring entry (s + f_lo % 4) % R_SLOTS:
            // the ring is filled at position granularity): the 24 aligned bytes around them, shifted by 0..3 elements
            auto take = [&](int c, int s0) {
                const char* const ring = s_rings + f_rr[c] * R_ROW;
                const u32x4 lo = *reinterpret_cast<const u32x4*>(ring + (s0 & (R_SLOTS - 1)) * 2);
                const u32x2 hi = *reinterpret_cast<const u32x2*>(ring + ((s0 + 8) & (R_SLOTS - 1)) * 2);
                const bool dw = (f_lo[c] & 2) != 0;
                const uint32_t x0 = dw ? lo[1] : lo[0], x1 = dw ? lo[2] : lo[1], x2 = dw ? lo[3] : lo[2];
                const uint32_t x3 = dw ? hi[0] : lo[3], x4 = dw ? hi[1] : hi[0];
                const uint32_t sh = (f_lo[c] & 1) ? 16u : 0u;
                u32x4 r;
                r[0] = __builtin_amdgcn_alignbit(x1, x0, sh);
                r[1] = __builtin_amdgcn_alignbit(x2, x1, sh);
                r[2] = __builtin_amdgcn_alignbit(x3, x2, sh);
                r[3] = __builtin_amdgcn_alignbit(x4, x3, sh);
                return r;
            };
            // store the units that the positions from pos0 up to pos1 (the first HL of them since the last call) have
            // completed
            auto flush = [&](int pos0, int pos1) {
                if (!uniform) return;
                // all of them inside the span of every row of the wavefront, and not the last of any: each row has exactly
                // one unit to store, a whole one
                if (pos1 - pos0 == HL && pos0 >= span.lo_max && pos1 < span.hi_min) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int s0 = HL * f_done[c] + 8 * f_piece;
                        const u32x4 val = take(c, s0);
                        __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>((T*)p.out + f_base[c] + s0));
                        f_done[c] += 1;
                    }
                    return;
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const int u_end = pos1 - f_lo[c];
                    const int final_slot = min(max(u_end, 0), f_cnt[c]);  // slots below it hold their scores
#pragma unroll
                    for (int rep = 0; rep < 2; ++rep) {
                        const int ls = HL * f_done[c];
                        const bool unit = (ls + HL <= final_slot) || (u_end >= f_cnt[c] && ls < f_cnt[c]);
                        if (unit) {
                            const int s0 = ls + 8 * f_piece;
                            const u32x4 val = take(c, s0);
                            T* const dst = (T*)p.out + f_base[c] + s0;
                            const int n = f_cnt[c] - s0;
                            if (n >= 8) {
                                __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(dst));
                            } else {
                                typedef T v8 __attribute__((ext_vector_type(8)));
                                const v8 e8 = __builtin_bit_cast(v8, val);
#pragma unroll
                                for (int e = 0; e < 8; ++e)
                                    if (e < n) dst[e] = e8[e];
                            }
                            f_done[c] += 1;
                        }
                    }
                }
            };
            // Units are looked for once HL positions have been put since the last look, and when this wavefront's rows end.
            auto do_half = [&](int h, int pos0) {
                read_frags(h);
                products(h);
                put(h, pos0);
                if (pend_from < 0) pend_from = pos0;
                if (pos0 + 32 - pend_from >= HL || pos0 + 32 >= hmax) {
                    flush(pend_from, pos0 + 32);
                    pend_from = -1;
                }
            };
            if (actA) do_half(0, posA);
            if (actB) do_half(1, posB);
        };
        for (int s = 0; s < n_steps; s += NST) {
            static_for<NST>([&](auto u) {
                if (s + decltype(u)::value < n_steps) step(s + decltype(u)::value, u);
            });
        }
    }
}

template <typename T, int D, int NST, int KEYS, int HL, int BM, bool PROBS, bool PLANNED>
static int launch_lines_variant(const char* who, SddmmParams p, hipStream_t st) {
    using G = LinesGeom<D, NST, KEYS, HL, BM, PLANNED>;
    static_assert(G::LDS_BYTES * (256 / BM) <= 160 * 1024, "16 wavefronts per compute unit");
    p.n_row_blocks = count_row_blocks(p.L, BM, p.row_stride);
    const int64_t blocks = (int64_t)p.B * p.H * p.n_row_blocks;
    if (blocks > 0x7ffffff0) return 0;
    p.key_split = 1;
    p.total = (int)blocks;
    static uint64_t reserved = 0;
    auto kern = sddmm_lines_kernel<T, D, NST, KEYS, HL, BM, PROBS, PLANNED>;
    if (int rc = reserve_dynamic_lds(&reserved, reinterpret_cast<const void*>(kern), G::LDS_BYTES, who)) return rc;
    const int grid = ((p.total + 7) / 8) * 8;
    kern<<<grid, BM * 4, G::LDS_BYTES, st>>>(p);
    return 1;
}

// Whole 128-byte lines are what the memory system likes best (a blocked mask at d = 128: 0.25 ms against 0.34 ms with
// halves), but their rings take 34 KiB of LDS, which at d = 128 leaves room for steps of 32 keys only (two barriers per
// 64 keys).  Short rows (one or two lines) are better off with halves and steps of 64 keys.
template <typename T, bool PROBS, bool PLANNED>
static int launch_lines_typed(const char* who, const SddmmParams& p, hipStream_t st) {
    if (p.d == 128) {
        if (p.T >= 256) return launch_lines_variant<T, 128, PLANNED ? 5 : 4, 32, 64, 128, PROBS, PLANNED>(who, p, st);
        return launch_lines_variant<T, 128, 3, 64, 32, 128, PROBS, PLANNED>(who, p, st);
    }
    if (p.T >= 128) return launch_lines_variant<T, 64, 4, 64, 64, 128, PROBS, PLANNED>(who, p, st);
    return launch_lines_variant<T, 64, 4, 64, 32, 128, PROBS, PLANNED>(who, p, st);
}

int launch_sddmm_lines(const char* who, const SddmmParams& p_in, int in_dtype, hipStream_t st) {
    if (in_dtype == SPLAT_F32 || p_in.out_dtype != in_dtype) return 0;
    if (p_in.d != 64 && p_in.d != 128) return 0;
    if (p_in.k_sd != 1 || !p_in.q_vec || !p_in.k_vec || !p_in.out_vec) return 0;
    const SddmmParams& p = p_in;
    // Few row blocks with long rows are better off with the general kernel, which splits a block's key range over several
    // workgroups (64 blocks of 1024 slots: 0.021 against 0.029 ms; of 256 slots: 0.016 against 0.013).
    if ((int64_t)p.B * p.H * count_row_blocks(p.L, 128, p.row_stride) < 256 && p.T > 256) return 0;
    const bool probs = p.row_lse != nullptr;
    const SddmmParams& pp = p;
    auto go = [&](auto t, auto probs_c, auto planned_c) {
        return launch_lines_typed<decltype(t), decltype(probs_c)::value, decltype(planned_c)::value>(who, pp, st);
    };
    auto by_plan = [&](auto t, auto probs_c) { return pp.plan ? go(t, probs_c, std::true_type{}) : go(t, probs_c, std::false_type{}); };
    auto by_probs = [&](auto t) { return probs ? by_plan(t, std::true_type{}) : by_plan(t, std::false_type{}); };
    return in_dtype == SPLAT_BF16 ? by_probs(bf16{}) : by_probs(f16{});
}

}  // namespace splat
