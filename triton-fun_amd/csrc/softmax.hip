// Row softmax over the live slots of compressed [BH, L, T] score rows.
//
// One wavefront owns one row.  The row's live slots are read once with 16/32-byte loads (8 elements
// per lane per step), kept in registers, reduced with wavefront shuffles (max, then sum of
// exp2((x - max) * log2 e)) and written back once; dead slots (s >= nnz) are neither read as data nor
// written.  HBM-bound: 2 * live slots * element size bytes per row.  Rows whose length is not a multiple of 8 start
// at any element of an 8-element chunk: they are read as the aligned chunks that cover them (a chunk at a row's end
// also holds its neighbour's first slots, which are discarded) and written whole where a chunk is all theirs, element by
// element at the two ends.  Rows longer than 2048 slots take a three-pass kernel that re-reads the row from cache.
#include "splat_common.hpp"

namespace splat {

struct SoftmaxSegs {
    const float* nnz[SPLAT_MAX_SEGMENTS];
    int off[SPLAT_MAX_SEGMENTS];
    int n;
};

struct LiveRanges {
    int lo[SPLAT_MAX_SEGMENTS], hi[SPLAT_MAX_SEGMENTS];
    int n;
    __device__ __forceinline__ void load(const SoftmaxSegs& s, int row, int T) {
        n = s.n;
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) {
            lo[k] = hi[k] = 0;
            if (k < s.n) {
                lo[k] = s.off[k];
                hi[k] = min(T, s.off[k] + (int)s.nnz[k][row]);
            }
        }
    }
    __device__ __forceinline__ bool live(int slot) const {
        bool v = false;
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) v |= (k < n) && slot >= lo[k] && slot < hi[k];
        return v;
    }
    // 8-bit liveness of slots [s0, s0+8); s0 may be negative (a chunk that begins before the row does)
    __device__ __forceinline__ uint32_t live8(int s0) const {
        uint32_t m = 0;
#pragma unroll
        for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) {
            if (k < n) {
                int a = max(lo[k], s0) - s0, b = min(hi[k], s0 + 8) - s0;
                if (b > a) m |= ((1u << b) - 1u) & ~((1u << a) - 1u);
            }
        }
        return m;
    }
};

template <typename T>
struct Vec8 {
    typedef T type __attribute__((ext_vector_type(8)));
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;

// LPR lanes share one row (64 / LPR rows per wavefront): rows shorter than 512 slots still fill every lane.  A wavefront
// takes RIF such row groups at once and requests all of their chunks before it looks at any (bytes in flight per
// wavefront are what a streaming kernel lives on).
// SHIFT: T is not a multiple of 8, so row r begins (r * T) % 8 elements into an aligned chunk.
template <typename Tin, typename Tout, int NCH, int LPR, int RIF, bool SHIFT>
__global__ __launch_bounds__(256) void softmax_rows_vec(const Tin* __restrict__ x, Tout* __restrict__ y, SoftmaxSegs segs,
                                                        int64_t n_rows, int L, int T) {
    typedef typename Vec8<Tin>::type vin;
    typedef typename Vec8<Tout>::type vout;
    constexpr int RPW = 64 / LPR;  // rows per wavefront and group
    const int lane = threadIdx.x & (LPR - 1);
    const int64_t row0 = (((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RIF) * RPW + ((threadIdx.x & 63) / LPR);
    if (RPW == 1 && row0 >= n_rows) return;
    const int64_t total = n_rows * (int64_t)T;

    // the loads do not wait for the rows' live counts: a chunk inside the row is fetched whole and the dead
    // slots in it are discarded afterwards
    vin raw[RIF][NCH];
    bool row_ok[RIF];
    int64_t row[RIF];
    int shift[RIF], nchunk[RIF];  // elements of the first chunk that precede the row; chunks that cover the row
#pragma unroll
    for (int i = 0; i < RIF; ++i) {
        const int64_t row_raw = row0 + (int64_t)i * RPW;
        row_ok[i] = row_raw < n_rows;
        row[i] = row_ok[i] ? row_raw : n_rows - 1;  // surplus lane groups shadow the last row and store nothing
        const int64_t first = row[i] * (int64_t)T;
        shift[i] = SHIFT ? (int)(first & 7) : 0;
        nchunk[i] = (T + shift[i] + 7) >> 3;
        const Tin* xr = x + (first - shift[i]);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int ch = lane + LPR * c;
            if (ch < nchunk[i]) {
                if constexpr (!SHIFT) {
                    raw[i][c] = __builtin_nontemporal_load(reinterpret_cast<const vin*>(xr + (ch << 3)));
                } else if (first - shift[i] + (ch << 3) + 8 <= total) {
                    // rows share the lines at their ends with their neighbours: through the cache, not around it
                    raw[i][c] = *reinterpret_cast<const vin*>(xr + (ch << 3));
                } else {  // the last chunk of the buffer ends beyond it: only the elements that exist
#pragma unroll
                    for (int e = 0; e < 8; ++e) raw[i][c][e] = first - shift[i] + (ch << 3) + e < total ? xr[(ch << 3) + e] : (Tin)0.f;
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RIF; ++i) {
        LiveRanges lr;
        lr.load(segs, (int)(row[i] % L), T);
        Tout* yr = y + (row[i] * (int64_t)T - shift[i]);  // chunk ch of the row = elements 8*ch .. 8*ch+7 from here
        float v[NCH][8];
        uint32_t live[NCH];
        float mx = kNegBig;
        bool whole = true;  // every chunk of this lane is live in all 8 slots
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int ch = lane + LPR * c;
            live[c] = (ch < nchunk[i]) ? lr.live8((ch << 3) - shift[i]) : 0u;
            whole = whole && live[c] == 0xffu;
        }
        // the common case, decided for the whole wavefront: no dead slot anywhere in its rows, so no per-slot selects
        const bool all_whole = !__any(!whole);
        float sum = 0.f;
        if (all_whole) {
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const vin t = raw[i][c];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    v[c][e] = (float)t[e];
                    mx = fmaxf(mx, v[c][e]);
                }
            }
#pragma unroll
            for (int o = LPR / 2; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            const float mb = mx * kLog2e;
#pragma unroll
            for (int c = 0; c < NCH; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    v[c][e] = fast_exp2(fmaf(v[c][e], kLog2e, -mb));
                    sum += v[c][e];
                }
        } else {
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                if (live[c]) {
                    const vin t = raw[i][c];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        v[c][e] = ((live[c] >> e) & 1u) ? (float)t[e] : kNegBig;
                        mx = fmaxf(mx, v[c][e]);
                    }
                }
            }
#pragma unroll
            for (int o = LPR / 2; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            const float mb = mx * kLog2e;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                if (live[c]) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        // dead slots hold -1e30 and underflow to exactly 0 against any real maximum; a row without live
                        // slots stores nothing, so what its lanes compute does not matter
                        float p = fast_exp2(fmaf(v[c][e], kLog2e, -mb));
                        v[c][e] = p;
                        sum += p;
                    }
                }
            }
        }
#pragma unroll
        for (int o = LPR / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
        const float inv = sum > 0.f ? 1.0f / sum : 0.f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (live[c] && row_ok[i]) {
                const int ch = lane + LPR * c;
                if (live[c] == 0xffu) {
                    vout o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[e] = (Tout)(v[c][e] * inv);
                    if constexpr (SHIFT)
                        *reinterpret_cast<vout*>(yr + (ch << 3)) = o;
                    else
                        __builtin_nontemporal_store(o, reinterpret_cast<vout*>(yr + (ch << 3)));
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if ((live[c] >> e) & 1u) yr[(ch << 3) + e] = (Tout)(v[c][e] * inv);
                }
            }
        }
    }
}

template <typename Tin, typename Tout>
__global__ __launch_bounds__(256) void softmax_rows_any(const Tin* __restrict__ x, Tout* __restrict__ y, SoftmaxSegs segs,
                                                        int64_t n_rows, int L, int T) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    LiveRanges lr;
    lr.load(segs, (int)(row % L), T);
    const Tin* xr = x + row * (int64_t)T;
    Tout* yr = y + row * (int64_t)T;
    float mx = kNegBig;
    for (int s = lane; s < T; s += 64)
        if (lr.live(s)) mx = fmaxf(mx, (float)xr[s]);
    mx = wave_max(mx);
    const float mb = mx * kLog2e;
    float sum = 0.f;
    for (int s = lane; s < T; s += 64)
        if (lr.live(s)) sum += fast_exp2(fmaf((float)xr[s], kLog2e, -mb));
    sum = wave_sum(sum);
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;
    // in-place safe: every lane rewrites only the slots it reads in this loop
    for (int s = lane; s < T; s += 64)
        if (lr.live(s)) yr[s] = (Tout)(fast_exp2(fmaf((float)xr[s], kLog2e, -mb)) * inv);
}

template <typename Tin, typename Tout>
static int launch_softmax(const void* x, void* y, const SoftmaxSegs& segs, int64_t n_rows, int L, int T, hipStream_t st) {
    begin_launch();
    unsigned grid = (unsigned)((n_rows + 3) / 4);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 31) == 0;
    const Tin* xi = (const Tin*)x;
    Tout* yo = (Tout*)y;
    if (aligned && (T & 7) != 0 && T <= 2032) {
        // rows that start anywhere in a chunk: up to T/8 + 2 chunks cover one
        const int chunks = T / 8 + 2;
        auto groups = [&](int rows_per_wave) { return (unsigned)((n_rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave)); };
        if (chunks <= 16)
            softmax_rows_vec<Tin, Tout, 1, 16, 1, true><<<groups(4), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (chunks <= 32)
            // 8 lanes and four chunks per row, eight rows per wavefront: the per-row work (live counts, masks, two
            // reductions, the element-wise stores at a row's ends) is what such short rows cost, and eight rows share
            // every instruction of it (+46 % over 32 lanes per row at T = 191)
            softmax_rows_vec<Tin, Tout, 4, 8, 1, true><<<groups(8), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (chunks <= 64)
            softmax_rows_vec<Tin, Tout, 1, 64, 4, true><<<groups(4), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (chunks <= 128)
            softmax_rows_vec<Tin, Tout, 2, 64, 1, true><<<groups(1), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else
            softmax_rows_vec<Tin, Tout, 4, 64, 1, true><<<groups(1), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
    } else if (aligned && (T & 7) == 0 && T <= 2048) {
        const int nch = (T / 8 + 63) / 64;
        // row groups in flight per wavefront: 4 where a row is 512 bytes or more (+7 % at T = 512, +4 % at T = 256 over
        // one group, measured), one for shorter rows (more was slower there)
        auto groups = [&](int rows_per_wave) { return (unsigned)((n_rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave)); };
        if (T <= 128)
            softmax_rows_vec<Tin, Tout, 1, 16, 1, false><<<groups(4), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (T <= 256)
            softmax_rows_vec<Tin, Tout, 1, 32, 4, false><<<groups(2 * 4), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (nch <= 1)
            softmax_rows_vec<Tin, Tout, 1, 64, 4, false><<<groups(4), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else if (nch <= 2)
            softmax_rows_vec<Tin, Tout, 2, 64, 1, false><<<groups(1), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
        else
            softmax_rows_vec<Tin, Tout, 4, 64, 1, false><<<groups(1), 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
    } else {
        softmax_rows_any<Tin, Tout><<<grid, 256, 0, st>>>(xi, yo, segs, n_rows, L, T);
    }
    return check_launch("splat_softmax");
}

template <typename Tin>
static int dispatch_out(const void* x, void* y, const SoftmaxSegs& segs, int64_t n_rows, int L, int T, int out_dtype, hipStream_t st) {
    switch (out_dtype) {
        case SPLAT_F32: return launch_softmax<Tin, float>(x, y, segs, n_rows, L, T, st);
        case SPLAT_F16: return launch_softmax<Tin, f16>(x, y, segs, n_rows, L, T, st);
        case SPLAT_BF16: return launch_softmax<Tin, bf16>(x, y, segs, n_rows, L, T, st);
    }
    return fail(SPLAT_E_DTYPE, "splat_softmax: unknown out_dtype %d", out_dtype);
}

}  // namespace splat

using namespace splat;

extern "C" int splat_softmax(const void* x, void* y, const splat_acsr_seg* segs, int32_t n_seg, int64_t BH, int32_t L,
                             int32_t T, int32_t in_dtype, int32_t out_dtype, void* stream) {
    if (!x || !y || !segs) return fail(SPLAT_E_NULL, "splat_softmax: null pointer argument");
    if (n_seg < 1 || n_seg > SPLAT_MAX_SEGMENTS) return fail(SPLAT_E_SHAPE, "splat_softmax: n_seg must be 1..%d (got %d)", SPLAT_MAX_SEGMENTS, n_seg);
    if (BH <= 0 || L <= 0 || T <= 0) return fail(SPLAT_E_SHAPE, "splat_softmax: need BH, L, T > 0 (got %lld, %d, %d)", (long long)BH, L, T);
    if (BH * (int64_t)L > ((int64_t)1 << 33)) return fail(SPLAT_E_SHAPE, "splat_softmax: too many rows");
    SoftmaxSegs s;
    s.n = n_seg;
    for (int k = 0; k < SPLAT_MAX_SEGMENTS; ++k) {
        s.nnz[k] = nullptr;
        s.off[k] = 0;
    }
    for (int k = 0; k < n_seg; ++k) {
        if (!segs[k].nnz) return fail(SPLAT_E_NULL, "splat_softmax: segment %d has a null nnz array", k);
        if (segs[k].slot_offset < 0 || segs[k].slot_offset >= T)
            return fail(SPLAT_E_SHAPE, "splat_softmax: segment %d slot_offset %d outside [0, T=%d)", k, segs[k].slot_offset, T);
        s.nnz[k] = segs[k].nnz;
        s.off[k] = segs[k].slot_offset;
    }
    const int64_t n_rows = BH * L;
    hipStream_t st = (hipStream_t)stream;
    switch (in_dtype) {
        case SPLAT_F32: return dispatch_out<float>(x, y, s, n_rows, L, T, out_dtype, st);
        case SPLAT_F16: return dispatch_out<f16>(x, y, s, n_rows, L, T, out_dtype, st);
        case SPLAT_BF16: return dispatch_out<bf16>(x, y, s, n_rows, L, T, out_dtype, st);
    }
    return fail(SPLAT_E_DTYPE, "splat_softmax: unknown in_dtype %d", in_dtype);
}
