// Per-workgroup planning shared by the SDDMM, SpMM and fused attention kernels: from the affine maps of
// the workgroup's rows decide which key positions the tiles enumerate and how a row tests validity.
#pragma once
#include "splat_common.hpp"

namespace splat {

constexpr int kBN = 64;  // key positions per tile

// Device pointers of one segment (kernel-argument form of splat_acsr_seg).
struct SegPtrs {
    const float* sTod_lin;
    const float* sTod_trans;
    const float* nnz;
    const int32_t* first_col;
    int slot_offset;
    int max_cnt;  // slots the segment may own in a compressed row (T - slot_offset); INT32_MAX where no buffer has rows of T slots
};

// Per-workgroup plan of one segment.
struct SegPlan {
    int c0;       // dense column of tile position j = 0
    int cs;       // column step between consecutive tile positions
    int n_tiles;  // tiles (of the kernel's tile size, kBN unless stated) to walk
    int uniform;  // 1: all rows share step and phase -> position j of row r is slot j - lo_r;
                  // 0: positions are dense columns and a row applies the full affine test
};

// A row's count is clamped to the slots its segment owns, so that metadata that disagrees with the buffer's trailing
// dimension cannot send a kernel past the end of a compressed row.
__device__ __forceinline__ RowMap load_row_map(const SegPtrs& s, int r) {
    RowMap m = load_row_map(s.sTod_lin, s.sTod_trans, s.nnz, s.first_col, r);
    m.cnt = min(m.cnt, s.max_cnt);
    return m;
}

// LDS the planner needs: per-wavefront partial reductions, and the rows' integer maps for later reuse.
template <int BM>
struct PlanScratch {
    int part[4][SPLAT_MAX_SEGMENTS][4];  // [wave][segment]: amin, cmax, linmin, linmax
    int flag[4][SPLAT_MAX_SEGMENTS];     // [wave][segment]: some row breaks the common step / phase
    int row_a[SPLAT_MAX_SEGMENTS][BM];
    int row_lin[SPLAT_MAX_SEGMENTS][BM];
    int row_cnt[SPLAT_MAX_SEGMENTS][BM];
};

template <int BM>
__device__ __forceinline__ RowMap cached_row_map(const PlanScratch<BM>* ps, int sg, int rr) {
    RowMap m;
    m.a = ps->row_a[sg][rr];
    m.lin = ps->row_lin[sg][rr];
    m.cnt = ps->row_cnt[sg][rr];
    return m;
}

// Gather the maps of rows r0 + rs*k, k in [0, BM), of every segment into LDS and reduce what the plans need.  Called by
// every thread of the workgroup (threads 0..255 take one row each, BM <= 256; further wavefronts only take part in
// the barriers); contains two barriers.  Afterwards segment_plan() may be evaluated by any thread.
template <int BM>
__device__ __forceinline__ void gather_row_maps(const SegPtrs* seg, int n_seg, int r0, int rs, int n_rows,
                                                PlanScratch<BM>* ps, int tid) {
    static_assert(BM <= 256, "one row per thread");
    const int lane = tid & 63, wave = tid >> 6;
    // wavefronts that hold no row leave neutral partial results and only take part in the barriers
    const bool has_rows = (wave * 64 < BM);  // wavefront-uniform
    RowMap mine[SPLAT_MAX_SEGMENTS];
    if (has_rows) {
#pragma unroll
        for (int sg = 0; sg < SPLAT_MAX_SEGMENTS; ++sg) {
            RowMap m = {0, 1, 0};
            if (sg < n_seg && tid < BM && r0 + rs * tid < n_rows) m = load_row_map(seg[sg], r0 + rs * tid);
            mine[sg] = m;
            if (sg < n_seg) {
                if (tid < BM) {
                    ps->row_a[sg][tid] = m.a;
                    ps->row_lin[sg][tid] = m.lin;
                    ps->row_cnt[sg][tid] = m.cnt;
                }
                const int amin = wave_min_i(m.cnt > 0 ? m.a : 0x7fffffff);
                const int cmax = wave_max_i(m.cnt > 0 ? m.a + m.lin * (m.cnt - 1) : -1);
                const int linmin = wave_min_i(m.cnt > 1 ? m.lin : 0x7fffffff);
                const int linmax = wave_max_i(m.cnt > 1 ? m.lin : 0);
                if (lane == 0) {
                    ps->part[wave][sg][0] = amin;
                    ps->part[wave][sg][1] = cmax;
                    ps->part[wave][sg][2] = linmin;
                    ps->part[wave][sg][3] = linmax;
                }
            }
        }
    } else if (lane < SPLAT_MAX_SEGMENTS && wave < 4) {
        ps->part[wave][lane][0] = 0x7fffffff;
        ps->part[wave][lane][1] = -1;
        ps->part[wave][lane][2] = 0x7fffffff;
        ps->part[wave][lane][3] = 0;
        ps->flag[wave][lane] = 0;
    }
    __syncthreads();
    if (has_rows) {
#pragma unroll
        for (int sg = 0; sg < SPLAT_MAX_SEGMENTS; ++sg) {
            if (sg < n_seg) {
                int amin = 0x7fffffff, linmin = 0x7fffffff, linmax = 0;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    amin = min(amin, ps->part[w][sg][0]);
                    linmin = min(linmin, ps->part[w][sg][2]);
                    linmax = max(linmax, ps->part[w][sg][3]);
                }
                bool bad = (linmax != 0 && linmin != linmax);
                const int step = (linmax == 0) ? 1 : linmin;  // no row with 2+ columns: any step fits
                if (!bad && step > 1) bad = mine[sg].cnt > 0 && ((mine[sg].a - amin) % step) != 0;
                const int any_bad = __any(bad) ? 1 : 0;
                if (lane == 0) ps->flag[wave][sg] = any_bad;
            }
        }
    }
    __syncthreads();
}

// The workgroup's plan for segment sg (valid after gather_row_maps).  `allow_gather` = false forces dense walks.
template <int BM, int BN = kBN>
__device__ __forceinline__ SegPlan segment_plan(const PlanScratch<BM>* ps, int sg, bool allow_gather) {
    int amin = 0x7fffffff, cmax = -1, linmin = 0x7fffffff, linmax = 0, bad = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        amin = min(amin, ps->part[w][sg][0]);
        cmax = max(cmax, ps->part[w][sg][1]);
        linmin = min(linmin, ps->part[w][sg][2]);
        linmax = max(linmax, ps->part[w][sg][3]);
        bad |= ps->flag[w][sg];
    }
    SegPlan pl;
    if (cmax < 0) {
        pl.c0 = 0;
        pl.cs = 1;
        pl.n_tiles = 0;
        pl.uniform = 1;
        return pl;
    }
    const int step = (linmax == 0) ? 1 : linmin;
    const bool uni = (bad == 0) && (allow_gather || step == 1);
    pl.uniform = uni ? 1 : 0;
    pl.cs = uni ? step : 1;
    // dense walks start on a tile boundary (keeps 16-byte K^T loads aligned and lets neighbouring row blocks
    // share cache lines); gathered walks start at the first live column
    pl.c0 = (pl.cs == 1) ? (amin & ~(BN - 1)) : amin;
    const int n_pos = (cmax - pl.c0) / pl.cs + 1;
    pl.n_tiles = (n_pos + BN - 1) / BN;
    return pl;
}

// gather_row_maps + one SegPlan per segment in LDS (plan[0..n_seg)); ends with a barrier.
template <int BM, int BN = kBN>
__device__ __forceinline__ void plan_segments(const SegPtrs* seg, int n_seg, int r0, int rs, int n_rows,
                                              bool allow_gather, SegPlan* plan, PlanScratch<BM>* ps, int tid) {
    gather_row_maps<BM>(seg, n_seg, r0, rs, n_rows, ps, tid);
    if (tid < n_seg) plan[tid] = segment_plan<BM, BN>(ps, tid, allow_gather);
    __syncthreads();
}

// Row blocks.  With row stride rs a workgroup owns the BM rows first + rs*k: the rows of one column phase out
// of BM*rs consecutive ones (rs = 1: BM consecutive rows).  Patterns whose rows alternate phase (dilated
// windows) then get uniform plans.  Block index -> first row.
__device__ __forceinline__ int block_first_row(int block, int BM, int rs) { return (block / rs) * BM * rs + (block % rs); }
inline int count_row_blocks(int n_rows, int BM, int rs) { return ((n_rows + BM * rs - 1) / (BM * rs)) * rs; }
// The row stride the segments agree on (their hints are equal and > 1), else 1.
inline int common_row_stride(const splat_acsr_seg* segs, int n_seg) {
    int rs = segs[0].row_stride_hint;
    for (int k = 1; k < n_seg; ++k)
        if (segs[k].row_stride_hint != rs) return 1;
    return (rs > 1 && rs <= 64) ? rs : 1;
}

// How one row tests a tile position j (relative to the plan's c0/cs).
//   uniform plan: live iff 0 <= j - lo < cnt, slot = j - lo
//   dense plan:   u = j - lo is the column offset from the row's first column; live iff 0 <= u < cnt
//                 (cnt = extent in columns) and u % lin == 0, slot = u / lin
struct RowWin {
    int lo, cnt, lin;
};

__device__ __forceinline__ RowWin make_row_win(const RowMap& m, const SegPlan& pl) {
    RowWin w;
    if (m.cnt <= 0) {
        w.lo = 0;
        w.cnt = 0;
        w.lin = 1;
    } else if (pl.uniform) {
        w.lo = (m.a - pl.c0) / pl.cs;
        w.cnt = m.cnt;
        w.lin = 1;
    } else {
        w.lo = m.a - pl.c0;
        w.lin = (m.cnt > 1) ? m.lin : 1;
        w.cnt = w.lin * (m.cnt - 1) + 1;
    }
    return w;
}

__device__ __forceinline__ bool win_live(const RowWin& w, int j) {
    const int u = j - w.lo;
    return (unsigned)u < (unsigned)w.cnt && (w.lin == 1 || ((unsigned)u % (unsigned)w.lin) == 0u);
}
__device__ __forceinline__ int win_slot(const RowWin& w, int j) {
    const int u = j - w.lo;
    return (w.lin == 1) ? u : u / w.lin;
}

// The entries of one compressed row at the 8 consecutive positions jj..jj+7 of a dense walk, zero where the row has no
// slot (`row` points at the row's first slot of the segment).  Two integer divisions per call: the first live position
// and its slot; the following ones are `lin` positions and one slot further each.
template <typename V, typename T>
__device__ __forceinline__ V gather_affine8(const T* row, const RowWin& w, int jj) {
    V v;
    const int u0 = jj - w.lo;
    int r = u0 % w.lin;
    if (r < 0) r += w.lin;
    int next = (r == 0) ? 0 : w.lin - r;  // offset of the first position congruent to the row's first column
    int slot = (u0 + next) / w.lin;       // exact; negative before the row's first column
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const bool hit = (e == next);
        const bool live = hit && (unsigned)(u0 + e) < (unsigned)w.cnt;
        v[e] = live ? row[slot] : (T)0.f;
        if (hit) {
            next += w.lin;
            ++slot;
        }
    }
    return v;
}

// Width of a wavefront's rows in tile positions: the tiles before lo_min / from hi_max on hold nothing for it, the
// tiles from lo_max on and up to hi_min need no mask.
struct WaveSpan {
    int lo_min, lo_max, hi_min, hi_max;
};
// Evaluated by the 64 lanes of a wavefront, each holding the window of one of its rows (both halves of the wavefront
// hold the same 32 rows).
__device__ __forceinline__ WaveSpan wave_span(const RowWin& win, bool uniform) {
    const bool empty = win.cnt <= 0;
    WaveSpan s;
    s.lo_min = wave_min_i(empty ? 0x3fffffff : win.lo);
    s.lo_max = wave_max_i(empty ? -0x3fffffff : win.lo);
    s.hi_min = wave_min_i(empty ? 0x3fffffff : win.lo + win.cnt);
    s.hi_max = wave_max_i(empty ? -0x3fffffff : win.lo + win.cnt);
    if (__any(empty) || !uniform) s.lo_max = 0x3fffffff;  // such a wavefront never drops the mask
    return s;
}
// smallest offset >= 0 from position 0 of the walk that is congruent to the row's first position modulo its step
__device__ __forceinline__ int win_phase(const RowWin& w) {
    const int f = w.lo % w.lin;
    return f < 0 ? f + w.lin : f;
}

// ---- plan table: what a workgroup of the fused kernel derives from the ACSR metadata, stored once per mask ----
// 16-byte records, two variants (0: gathered walks allowed, 1: dense walks only, for K^T-contiguous keys), each
//   seg  [row block][segment]            SegPlan
//   span [row block][segment][wavefront] WaveSpan
//   row  [segment][row block][row k]     RowWin + phase (row k of the block is row first + stride * k)
typedef int PlanRec __attribute__((ext_vector_type(4)));
constexpr int kPlanBM = 128;  // rows per row block of the fused kernel

__host__ __device__ inline int64_t plan_variant_recs(int n_rb, int n_seg) { return (int64_t)n_rb * n_seg * (5 + kPlanBM); }
__host__ __device__ inline int64_t plan_seg_at(int n_seg, int rb, int sg) { return (int64_t)rb * n_seg + sg; }
__host__ __device__ inline int64_t plan_span_at(int n_rb, int n_seg, int rb, int sg, int wave) {
    return (int64_t)n_rb * n_seg + ((int64_t)rb * n_seg + sg) * 4 + wave;
}
__host__ __device__ inline int64_t plan_row_at(int n_rb, int n_seg, int rb, int sg, int k) {
    return (int64_t)n_rb * n_seg * 5 + ((int64_t)sg * n_rb + rb) * kPlanBM + k;
}
// A record whose address is the same for the whole wavefront, through the scalar (constant) load path.
typedef __attribute__((address_space(4))) const PlanRec const_plan_rec;
__device__ __forceinline__ PlanRec plan_uniform_load(const PlanRec* p) {
    return *reinterpret_cast<const_plan_rec*>(reinterpret_cast<uintptr_t>(p));
}

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// Transposing LDS read: the 16 lanes of a block address 4 rows x 16 columns of 16-bit elements (lane s:
// row s/4, columns 4*(s%4)..+3); lane i of the block receives column i of the 4 rows.
__device__ __forceinline__ s16x4 lds_tr16(const char* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
}

template <typename T>
__device__ __forceinline__ Frag<T> frag_from_tr(s16x4 lo, s16x4 hi) {
    Frag<T> f;
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    s16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    return f;
}

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

// Fragment whose 8 contraction slots sit in 8 consecutive LDS elements.
template <typename T>
__device__ __forceinline__ Frag<T> lds_frag_rowmajor(const char* p) {
    Frag<T> f;
    if constexpr (sizeof(T) == 2) {
        u32x4 r = *reinterpret_cast<const u32x4*>(p);
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    } else {
        u32x4 r0 = *reinterpret_cast<const u32x4*>(p);
        u32x4 r1 = *reinterpret_cast<const u32x4*>(p + 16);
        u32x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    }
    return f;
}

// Fragment whose contraction index runs down the rows of an LDS tile: slots 0..3 are rows r0..r0+3,
// slots 4..7 rows r1..r1+3, all at column col0 + lane%32.  16-bit types use two transposing reads,
// fp32 reads 8 scalars.
template <typename T>
__device__ __forceinline__ Frag<T> lds_frag_cols(const char* tile, int row_bytes, int r0, int r1, int col0, int lane) {
    Frag<T> f;
    if constexpr (sizeof(T) == 2) {
        const int s = lane & 15;
        const int col = col0 + 16 * ((lane >> 4) & 1) + 4 * (s & 3);
        const char* p0 = tile + (r0 + (s >> 2)) * row_bytes + col * 2;
        const char* p1 = tile + (r1 + (s >> 2)) * row_bytes + col * 2;
        f = frag_from_tr<T>(lds_tr16(p0), lds_tr16(p1));
    } else {
        const int col = col0 + (lane & 31);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            f.v[e] = *reinterpret_cast<const float*>(tile + (r0 + e) * row_bytes + col * 4);
            f.v[4 + e] = *reinterpret_cast<const float*>(tile + (r1 + e) * row_bytes + col * 4);
        }
    }
    return f;
}

// 8 consecutive elements from global memory (16-byte aligned).
template <typename T>
__device__ __forceinline__ Frag<T> global_frag(const T* p) {
    Frag<T> f;
    if constexpr (sizeof(T) == 2) {
        u32x4 r = *reinterpret_cast<const u32x4*>(p);
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    } else {
        u32x4 r0 = *reinterpret_cast<const u32x4*>(p);
        u32x4 r1 = *reinterpret_cast<const u32x4*>(p + 4);
        u32x8 r = __builtin_shufflevector(r0, r1, 0, 1, 2, 3, 4, 5, 6, 7);
        f.v = __builtin_bit_cast(typename Frag<T>::vec, r);
    }
    return f;
}

// Fill a SegPtrs array from the host-side segment descriptors; returns 0 or a negative code.
inline int fill_segs(const char* who, const splat_acsr_seg* segs, int n_seg, SegPtrs* out, int T) {
    if (n_seg < 1 || n_seg > SPLAT_MAX_SEGMENTS)
        return fail(SPLAT_E_SHAPE, "%s: n_seg must be 1..%d (got %d)", who, SPLAT_MAX_SEGMENTS, n_seg);
    for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) out[k] = SegPtrs{nullptr, nullptr, nullptr, nullptr, 0, 0};
    for (int k = 0; k < n_seg; ++k) {
        if (!segs[k].sTod_lin || !segs[k].sTod_trans || !segs[k].nnz)
            return fail(SPLAT_E_NULL, "%s: segment %d lacks sTod_lin / sTod_trans / nnz", who, k);
        if (T >= 0 && (segs[k].slot_offset < 0 || segs[k].slot_offset >= T))
            return fail(SPLAT_E_SHAPE, "%s: segment %d slot_offset %d outside [0, T=%d)", who, k, segs[k].slot_offset, T);
        out[k] = SegPtrs{segs[k].sTod_lin, segs[k].sTod_trans, segs[k].nnz, segs[k].first_col, segs[k].slot_offset,
                         T >= 0 ? T - segs[k].slot_offset : 0x7fffffff};
    }
    return 0;
}

}  // namespace splat
