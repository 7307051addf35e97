// ACSR builder and mask generators.
//
// splat_acsr_build: one wavefront (short rows) or one workgroup (rows >= 4 KiB) per mask row streams the row once
// (16-byte loads), reducing the
// byte sum (nnz), the first two columns whose byte equals 1 (the affine map's anchors a < b) and the
// first/last nonzero column.  Lane 0 then evaluates the 2x2 solve of acsr_helpers.py:122 in closed
// form in double precision and rounds to float32, which is what the reference's
// float64 -> torch.FloatTensor conversion stores.  A second, tiny kernel folds rows into the
// per-row-block span pairs (acsr_helpers.py:135-140).  HBM-bound: rows*ld bytes in, 28*rows out.
#include "splat_common.hpp"

namespace splat {

constexpr int kInf = 0x7fffffff;

// 0x80 in every byte of y that is zero (exact, no borrow artefacts).
__device__ __forceinline__ uint32_t zero_bytes(uint32_t y) {
    return ~(((y & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | y | 0x7F7F7F7Fu);
}

struct RowScan {
    uint32_t sum;  // sum of byte values
    int m1, m2;    // two smallest columns whose byte == 1
    int first, last;  // first / last nonzero column

    __device__ __forceinline__ void init() {
        sum = 0;
        m1 = m2 = first = kInf;
        last = -1;
    }
    __device__ __forceinline__ void add_one(int col) {
        if (col < m1) {
            m2 = m1;
            m1 = col;
        } else if (col < m2 && col != m1) {
            m2 = col;
        }
    }
    __device__ __forceinline__ void dword(uint32_t x, int col0) {
        if (x == 0) return;
        sum = __builtin_amdgcn_sad_u8(x, 0u, sum);
        uint32_t nz = ~zero_bytes(x) & 0x80808080u;  // bytes that are nonzero
        int lo = (__builtin_ctz(nz) >> 3), hi = ((31 - __builtin_clz(nz)) >> 3);
        first = min(first, col0 + lo);
        last = max(last, col0 + hi);
        if (m2 == kInf) {
            uint32_t eq = zero_bytes(x ^ 0x01010101u);  // bytes equal to 1
            while (eq) {
                int b = __builtin_ctz(eq) >> 3;
                add_one(col0 + b);
                eq &= eq - 1;
            }
        }
    }
    __device__ __forceinline__ void byte(uint32_t x, int col) {
        if (x == 0) return;
        sum += x;
        first = min(first, col);
        last = max(last, col);
        if (x == 1) add_one(col);
    }
    __device__ __forceinline__ void wave_reduce() {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            uint32_t s2 = __shfl_xor(sum, o);
            int a1 = __shfl_xor(m1, o), a2 = __shfl_xor(m2, o);
            int f2 = __shfl_xor(first, o), l2 = __shfl_xor(last, o);
            sum += s2;
            int n1 = min(m1, a1);
            int n2 = min(max(m1, a1), min(m2, a2));
            m1 = n1;
            m2 = n2;
            first = min(first, f2);
            last = max(last, l2);
        }
    }
};

// The summary's starting values, written by the first workgroup of the rows kernel (no kernel of its own): the rows
// kernels themselves never touch the summary otherwise, the span kernel that follows them reduces into it.
__device__ __forceinline__ void init_summary(int32_t* summary) {
    if (blockIdx.x == 0 && threadIdx.x < 8) summary[threadIdx.x] = (threadIdx.x == 2) ? 0x7fffffff : 0;
}
constexpr float kUnpackFailed = 0.0f;  // stored as a row's sTod_lin (a real step is >= 1) until the span kernel has counted it

// What one row contributes once its scan is reduced: the closed-form 2x2 solve.  (The summary extrema are
// reduced by the span kernel: per-row atomics on one address cost more than streaming the whole mask.)
__device__ __forceinline__ void finish_row(const RowScan& s, int row, int cols, float* dTos_lin, float* dTos_trans,
                                           float* sTod_lin, float* sTod_trans, float* nnz_out, int32_t* row_first,
                                           int32_t* row_last) {
    const int nnz = (int)s.sum;
    double x0 = 1.0, x1 = 0.0;
    int step = 1;
    bool failed = false;
    if (nnz > 1) {
        if (s.m1 == kInf || s.m2 == kInf) {
            failed = true;  // the reference asserts here (acsr_helpers.py:119); counted by the span kernel
        } else {
            step = s.m2 - s.m1;
            x0 = 1.0 / (double)step;
            // the solve yields +0.0 (not -0.0) for a == 0
            x1 = (s.m1 == 0) ? 0.0 : -(double)s.m1 / (double)step;
        }
    }
    dTos_lin[row] = (float)x0;
    dTos_trans[row] = (float)x1;
    sTod_lin[row] = failed ? kUnpackFailed : (float)step;
    sTod_trans[row] = (float)fabs(x1);
    nnz_out[row] = (float)nnz;
    if (row_first) row_first[row] = (s.first == kInf) ? cols : s.first;
    if (row_last) row_last[row] = s.last;
}

__device__ __forceinline__ void scan_chunk(RowScan& s, const u32x4& x, int c) {
    if ((x.x | x.y | x.z | x.w) == 0) return;
    s.dword(x.x, c);
    s.dword(x.y, c + 4);
    s.dword(x.z, c + 8);
    s.dword(x.w, c + 12);
}

// Short rows: one wavefront per row, four rows per workgroup.
__global__ __launch_bounds__(256) void acsr_rows_kernel(const uint8_t* __restrict__ mask, int rows, int cols,
                                                        int64_t ld, int vec_ok, float* __restrict__ dTos_lin,
                                                        float* __restrict__ dTos_trans, float* __restrict__ sTod_lin,
                                                        float* __restrict__ sTod_trans, float* __restrict__ nnz_out,
                                                        int32_t* __restrict__ row_first,
                                                        int32_t* __restrict__ row_last, int32_t* __restrict__ summary) {
    init_summary(summary);
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint8_t* p = mask + (int64_t)row * ld;
    RowScan s;
    s.init();
    int done = 0;
    if (vec_ok) {
        const int nvec = cols >> 4;
        const u32x4* pv = reinterpret_cast<const u32x4*>(p);
        for (int i = lane; i < nvec; i += 64) scan_chunk(s, pv[i], i << 4);
        done = nvec << 4;
    }
    for (int c = done + lane; c < cols; c += 64) s.byte(p[c], c);
    s.wave_reduce();
    if (lane == 0) finish_row(s, row, cols, dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnz_out, row_first, row_last);
}

// Long rows (>= 4 KiB, 16-byte aligned): one workgroup per row, so that the memory system sees a few thousand
// sequential 4 KiB-wide streams instead of tens of thousands of 1 KiB-wide ones; up to 8 loads in flight per lane.
__global__ __launch_bounds__(256) void acsr_rows_wide_kernel(const uint8_t* __restrict__ mask, int rows, int cols,
                                                             int64_t ld, float* __restrict__ dTos_lin,
                                                             float* __restrict__ dTos_trans, float* __restrict__ sTod_lin,
                                                             float* __restrict__ sTod_trans, float* __restrict__ nnz_out,
                                                             int32_t* __restrict__ row_first,
                                                             int32_t* __restrict__ row_last, int32_t* __restrict__ summary) {
    init_summary(summary);
    __shared__ uint32_t s_sum[4];
    __shared__ int s_m1[4], s_m2[4], s_first[4], s_last[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = blockIdx.x;
    const uint8_t* p = mask + (int64_t)row * ld;
    RowScan s;
    s.init();
    const int nvec = cols >> 4;
    const u32x4* pv = reinterpret_cast<const u32x4*>(p);
    int i = tid;
    for (; i + 7 * 256 < nvec; i += 8 * 256) {
        u32x4 xs[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) xs[u] = __builtin_nontemporal_load(pv + i + 256 * u);
#pragma unroll
        for (int u = 0; u < 8; ++u) scan_chunk(s, xs[u], (i + 256 * u) << 4);
    }
    for (; i + 3 * 256 < nvec; i += 4 * 256) {
        u32x4 xs[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) xs[u] = __builtin_nontemporal_load(pv + i + 256 * u);
#pragma unroll
        for (int u = 0; u < 4; ++u) scan_chunk(s, xs[u], (i + 256 * u) << 4);
    }
    for (; i < nvec; i += 256) scan_chunk(s, pv[i], i << 4);
    for (int c = (nvec << 4) + tid; c < cols; c += 256) s.byte(p[c], c);
    s.wave_reduce();
    if (lane == 0) {
        s_sum[wave] = s.sum;
        s_m1[wave] = s.m1;
        s_m2[wave] = s.m2;
        s_first[wave] = s.first;
        s_last[wave] = s.last;
    }
    __syncthreads();
    if (tid == 0) {
        RowScan t;
        t.init();
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            t.sum += s_sum[w];
            const int n1 = min(t.m1, s_m1[w]);
            const int n2 = min(max(t.m1, s_m1[w]), min(t.m2, s_m2[w]));
            t.m1 = n1;
            t.m2 = n2;
            t.first = min(t.first, s_first[w]);
            t.last = max(t.last, s_last[w]);
        }
        finish_row(t, row, cols, dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnz_out, row_first, row_last);
    }
}

// Long rows, one wavefront per row: a wavefront takes its rows one after the other (consecutive wavefronts hold
// consecutive rows at any time), each row in batches of eight 16-byte chunks per lane with the next batch requested
// before the current one is scanned; no cross-wavefront reduction, no barrier, no LDS.
__global__ __launch_bounds__(256) void acsr_rows_stream_kernel(const uint8_t* __restrict__ mask, int rows, int cols,
                                                               int64_t ld, float* __restrict__ dTos_lin,
                                                               float* __restrict__ dTos_trans, float* __restrict__ sTod_lin,
                                                               float* __restrict__ sTod_trans, float* __restrict__ nnz_out,
                                                               int32_t* __restrict__ row_first,
                                                               int32_t* __restrict__ row_last, int32_t* __restrict__ summary) {
    init_summary(summary);
    const int lane = threadIdx.x & 63;
    const int n_waves = gridDim.x * 4;
    const int nvec = cols >> 4;
    constexpr int NB = 8;
    auto load_batch = [&](u32x4 (&xs)[NB], const u32x4* pv, int i0) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int i = i0 + 64 * u;
            xs[u] = i < nvec ? __builtin_nontemporal_load(pv + i) : u32x4{0, 0, 0, 0};
        }
    };
    for (int row = blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += n_waves) {
        const uint8_t* p = mask + (int64_t)row * ld;
        const u32x4* pv = reinterpret_cast<const u32x4*>(p);
        RowScan s;
        s.init();
        u32x4 cur[NB], nxt[NB];
        load_batch(cur, pv, lane);
        for (int i0 = lane; i0 < nvec; i0 += 64 * NB) {
            const bool more = i0 + 64 * NB < nvec;
            if (more) load_batch(nxt, pv, i0 + 64 * NB);
#pragma unroll
            for (int u = 0; u < NB; ++u) scan_chunk(s, cur[u], (i0 + 64 * u) << 4);
            if (more) {
#pragma unroll
                for (int u = 0; u < NB; ++u) cur[u] = nxt[u];
            }
        }
        for (int c = (nvec << 4) + lane; c < cols; c += 64) s.byte(p[c], c);
        s.wave_reduce();
        if (lane == 0) finish_row(s, row, cols, dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnz_out, row_first, row_last);
    }
}

// One thread per row block: span_start = min(cols, min_r trans_r), span_end = max(-1, max_r nnz_r*lin_r + trans_r)
// evaluated in double from the exact integers (a, lin, nnz) and rounded once to float32.  The same pass reduces
// the summary: T = max nnz, smallest / largest column step over rows with nnz > 1, and how many rows with
// nnz > 1 have a first column that is not congruent to the row index modulo their step.
__global__ __launch_bounds__(256) void acsr_spans_kernel(float* __restrict__ sTod_lin,
                                                         const float* __restrict__ sTod_trans,
                                                         const float* __restrict__ nnz, int rows, int cols,
                                                         int block_height, float* __restrict__ span_start,
                                                         float* __restrict__ span_end, int32_t* __restrict__ summary) {
    const int g = blockIdx.x * blockDim.x + threadIdx.x;
    const int n_blocks = (rows + block_height - 1) / block_height;
    int t_max = 0, step_min = 0x7fffffff, step_max = 0, off_phase = 0, failed = 0;
    if (g < n_blocks) {
        double lo = (double)cols, hi = -1.0;
        const int r1 = min(rows, (g + 1) * block_height);
        for (int r = g * block_height; r < r1; ++r) {
            float linf = sTod_lin[r];
            if (linf == kUnpackFailed) {  // a row the reference would have asserted on: counted, then stored as (1, 0) like
                ++failed;                 // the rows with at most one live column
                linf = 1.0f;
                sTod_lin[r] = linf;
            }
            const int lin = (int)linf;
            const int a = (int)rintf(linf * sTod_trans[r]);
            const int cnt = (int)nnz[r];
            const double t = (double)a / (double)lin;
            lo = fmin(lo, t);
            hi = fmax(hi, (double)((int64_t)cnt * lin) + t);
            t_max = max(t_max, cnt);
            if (cnt > 1) {
                step_min = min(step_min, lin);
                step_max = max(step_max, lin);
                off_phase += ((a - r) % lin) != 0;
            }
        }
        span_start[g] = (float)lo;
        span_end[g] = (float)hi;
    }
    t_max = wave_max_i(t_max);
    step_min = wave_min_i(step_min);
    step_max = wave_max_i(step_max);
    off_phase = (int)wave_sum((float)off_phase);  // at most 64 * block_height per wavefront: exact in float
    failed = (int)wave_sum((float)failed);
    if ((threadIdx.x & 63) == 0) {
        if (failed) atomicAdd(&summary[1], failed);
        atomicMax(&summary[0], t_max);
        atomicMin(&summary[2], step_min);
        atomicMax(&summary[3], step_max);
        if (off_phase) atomicAdd(&summary[4], off_phase);
    }
}

__device__ __forceinline__ bool mask_pred(int pattern, int64_t i, int64_t j, int64_t p0, int64_t p1) {
    if (pattern & SPLAT_MASK_TRANSPOSED) {  // entry (i, j) of the transposed pattern is entry (j, i) of the pattern
        const int64_t t = i;
        i = j;
        j = t;
        pattern &= ~SPLAT_MASK_TRANSPOSED;
    }
    switch (pattern) {
        case SPLAT_MASK_BLOCKED: {
            if (i < p0) return j < p0;
            int64_t start = (i / p0 - 1) * p0;
            return start <= j && j < start + 2 * p0;
        }
        case SPLAT_MASK_WINDOWED:
            return i - p0 <= j && j <= i + p0;
        case SPLAT_MASK_CAUSAL_WINDOWED:
            return i - p0 <= j && j <= i;
        case SPLAT_MASK_DILATED: {
            int64_t rel = j - (i - (p0 * p1) / 2);
            return rel >= 0 && rel < p0 * p1 && rel % p1 == 0;
        }
        case SPLAT_MASK_STRIDED_LOCAL:
            return j <= i && j > i - p0;
        case SPLAT_MASK_STRIDED_FAR:
            return j <= i - p0 && j % p1 == p1 - 1;
    }
    return false;
}

// What a scan of row i of the s x s pattern would find, in closed form: every pattern's row is an arithmetic
// progression of columns (first, step, count), clipped to [0, s).
__device__ __forceinline__ RowScan pattern_row(int pattern, int64_t i, int64_t s, int64_t p0, int64_t p1) {
    int64_t first = 0, step = 1, count = 0;
    switch (pattern) {
        case SPLAT_MASK_BLOCKED: {
            const int64_t start = (i < p0) ? 0 : (i / p0 - 1) * p0;
            const int64_t end = (i < p0) ? p0 : start + 2 * p0;  // exclusive
            first = start;
            count = min(end, s) - start;
            break;
        }
        case SPLAT_MASK_WINDOWED:
            first = max((int64_t)0, i - p0);
            count = min(s - 1, i + p0) - first + 1;
            break;
        case SPLAT_MASK_CAUSAL_WINDOWED:
            first = max((int64_t)0, i - p0);
            count = min(s - 1, i) - first + 1;
            break;
        case SPLAT_MASK_STRIDED_LOCAL:
            first = max((int64_t)0, i - p0 + 1);
            count = min(s - 1, i) - first + 1;
            break;
        case SPLAT_MASK_DILATED: {
            const int64_t base = i - (p0 * p1) / 2;  // column of t = 0; columns base + t * p1, t in [0, p0)
            const int64_t t_lo = base < 0 ? (-base + p1 - 1) / p1 : 0;
            const int64_t room = s - 1 - base;
            const int64_t t_hi = room < 0 ? -1 : min(p0 - 1, room / p1);
            step = p1;
            first = base + t_lo * p1;
            count = t_hi - t_lo + 1;
            break;
        }
        case SPLAT_MASK_STRIDED_FAR: {
            const int64_t room = min(i - p0, s - 1) - (p1 - 1);  // columns p1 - 1 + t * p1 <= i - p0
            step = p1;
            first = p1 - 1;
            count = room < 0 ? 0 : room / p1 + 1;
            break;
        }
        // ---- rows of the transposed patterns = columns of the patterns: which rows keep column i ----
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_BLOCKED: {
            // row block b >= 1 keeps column blocks b - 1 and b, row block 0 keeps column block 0: column block c is kept
            // by row blocks c and c + 1
            const int64_t c = i / p0;
            first = c * p0;
            count = min((c + 2) * p0, s) - first;
            break;
        }
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_WINDOWED:
            first = max((int64_t)0, i - p0);
            count = min(s - 1, i + p0) - first + 1;
            break;
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_CAUSAL_WINDOWED:
            first = i;
            count = min(s - 1, i + p0) - first + 1;
            break;
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_STRIDED_LOCAL:
            first = i;
            count = min(s - 1, i + p0 - 1) - first + 1;
            break;
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_DILATED: {
            // row r keeps column r - h + t * p1, t in [0, p0), h = p0 * p1 / 2: column i is kept by rows i + h - t * p1,
            // in ascending order base + u * p1, u in [0, p0)
            const int64_t base = i + (p0 * p1) / 2 - (p0 - 1) * p1;
            const int64_t u_lo = base < 0 ? (-base + p1 - 1) / p1 : 0;
            const int64_t room = s - 1 - base;
            const int64_t u_hi = room < 0 ? -1 : min(p0 - 1, room / p1);
            step = p1;
            first = base + u_lo * p1;
            count = u_hi - u_lo + 1;
            break;
        }
        case SPLAT_MASK_TRANSPOSED | SPLAT_MASK_STRIDED_FAR:
            // only columns congruent to p1 - 1 are kept, by every row from i + p0 on
            first = i + p0;
            count = (i % p1 == p1 - 1) ? s - first : 0;
            break;
    }
    RowScan r;
    r.init();
    if (count > 0) {
        r.sum = (uint32_t)count;
        r.m1 = r.first = (int)first;
        if (count > 1) r.m2 = (int)(first + step);
        r.last = (int)(first + (count - 1) * step);
    }
    return r;
}

__global__ __launch_bounds__(256) void acsr_rows_pattern_kernel(int pattern, int s, int64_t p0, int64_t p1,
                                                                float* __restrict__ dTos_lin, float* __restrict__ dTos_trans,
                                                                float* __restrict__ sTod_lin, float* __restrict__ sTod_trans,
                                                                float* __restrict__ nnz_out, int32_t* __restrict__ row_first,
                                                                int32_t* __restrict__ row_last, int32_t* __restrict__ summary) {
    init_summary(summary);
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= s) return;
    finish_row(pattern_row(pattern, row, s, p0, p1), row, s, dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnz_out, row_first,
               row_last);
}

__global__ __launch_bounds__(256) void mask_generate_kernel(uint8_t* __restrict__ mask, int rows, int cols,
                                                            int64_t ld, int pattern, int64_t p0, int64_t p1,
                                                            int vec_ok) {
    const int chunks = (cols + 15) >> 4;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (int64_t)rows * chunks) return;
    const int i = (int)(id / chunks);
    const int c0 = (int)(id % chunks) << 4;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int b = 0; b < 16; ++b) {
        int j = c0 + b;
        if (j < cols && mask_pred(pattern, i, j, p0, p1)) w[b >> 2] |= 1u << ((b & 3) * 8);
    }
    uint8_t* dst = mask + (int64_t)i * ld + c0;
    if (vec_ok && c0 + 16 <= cols) {
        *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        for (int b = 0; b < 16 && c0 + b < cols; ++b) dst[b] = (uint8_t)((w[b >> 2] >> ((b & 3) * 8)) & 0xff);
    }
}

}  // namespace splat

using namespace splat;

extern "C" int splat_acsr_build(const uint8_t* mask, int64_t rows, int64_t cols, int64_t ld, int32_t block_height,
                                float* dTos_lin, float* dTos_trans, float* sTod_lin, float* sTod_trans, float* nnz,
                                float* span_start, float* span_end, int32_t* row_first, int32_t* row_last,
                                int32_t* summary, void* stream) {
    begin_launch();
    if (!mask || !dTos_lin || !dTos_trans || !sTod_lin || !sTod_trans || !nnz || !span_start || !span_end || !summary)
        return fail(SPLAT_E_NULL, "splat_acsr_build: null pointer argument");
    if (rows <= 0 || cols <= 0 || ld < cols || block_height <= 0)
        return fail(SPLAT_E_SHAPE, "splat_acsr_build: need rows > 0, cols > 0, ld >= cols, block_height > 0 (got %lld, %lld, %lld, %d)",
                    (long long)rows, (long long)cols, (long long)ld, block_height);
    // a row sum must fit int32 and columns must be exactly representable in float32 metadata
    if (rows > (1 << 23) || cols > (1 << 23))
        return fail(SPLAT_E_SHAPE, "splat_acsr_build: rows and cols are limited to 2^23 (got %lld, %lld)", (long long)rows, (long long)cols);
    hipStream_t st = (hipStream_t)stream;
    const int vec_ok = ((reinterpret_cast<uintptr_t>(mask) & 15) == 0 && (ld & 15) == 0) ? 1 : 0;
    // rows of 16 KiB and more: a workgroup per row; 4 to 16 KiB: a wavefront per row, each wavefront taking several rows
    // (at 8 KiB rows 0.028 against 0.038 ms with caches flushed; at 16 KiB the two are equal and the workgroup form is
    // 5 % faster on a mask that is found in the caches)
    if (vec_ok && cols >= 4096 && cols < 16384)
        acsr_rows_stream_kernel<<<(unsigned)min((int64_t)1024, (rows + 3) / 4), 256, 0, st>>>(mask, (int)rows, (int)cols, ld, dTos_lin, dTos_trans, sTod_lin,
                                                              sTod_trans, nnz, row_first, row_last, summary);
    else if (vec_ok && cols >= 4096)
        acsr_rows_wide_kernel<<<(unsigned)rows, 256, 0, st>>>(mask, (int)rows, (int)cols, ld, dTos_lin, dTos_trans, sTod_lin,
                                                              sTod_trans, nnz, row_first, row_last, summary);
    else
        acsr_rows_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, st>>>(mask, (int)rows, (int)cols, ld, vec_ok, dTos_lin, dTos_trans,
                                                                     sTod_lin, sTod_trans, nnz, row_first, row_last, summary);
    const int n_blocks = (int)((rows + block_height - 1) / block_height);
    acsr_spans_kernel<<<(n_blocks + 255) / 256, 256, 0, st>>>(sTod_lin, sTod_trans, nnz, (int)rows, (int)cols, block_height,
                                                               span_start, span_end, summary);
    return check_launch("splat_acsr_build");
}

static int check_pattern(const char* who, int64_t s, int32_t pattern, int64_t p0, int64_t p1) {
    if (s <= 0 || s > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: need 0 < s <= 2^23 (got %lld)", who, (long long)s);
    const int base = pattern & ~SPLAT_MASK_TRANSPOSED;
    if (pattern < 0 || base < SPLAT_MASK_BLOCKED || base > SPLAT_MASK_STRIDED_FAR)
        return fail(SPLAT_E_UNSUPPORTED, "%s: unknown pattern %d", who, pattern);
    const bool needs_p1 = base == SPLAT_MASK_DILATED || base == SPLAT_MASK_STRIDED_FAR;
    if (p0 < 0 || (base == SPLAT_MASK_BLOCKED && p0 <= 0) || (needs_p1 && p1 <= 0))
        return fail(SPLAT_E_SHAPE, "%s: bad pattern parameters p0=%lld p1=%lld", who, (long long)p0, (long long)p1);
    return 0;
}

extern "C" int splat_acsr_build_pattern(int32_t pattern, int64_t s, int64_t p0, int64_t p1, int32_t block_height,
                                        float* dTos_lin, float* dTos_trans, float* sTod_lin, float* sTod_trans, float* nnz,
                                        float* span_start, float* span_end, int32_t* row_first, int32_t* row_last,
                                        int32_t* summary, void* stream) {
    begin_launch();
    const char* who = "splat_acsr_build_pattern";
    if (!dTos_lin || !dTos_trans || !sTod_lin || !sTod_trans || !nnz || !span_start || !span_end || !summary)
        return fail(SPLAT_E_NULL, "%s: null pointer argument", who);
    if (block_height <= 0) return fail(SPLAT_E_SHAPE, "%s: block_height must be > 0 (got %d)", who, block_height);
    if (int rc = check_pattern(who, s, pattern, p0, p1)) return rc;
    if (p0 > (1 << 23) || p1 > (1 << 23)) return fail(SPLAT_E_SHAPE, "%s: pattern parameters are limited to 2^23", who);
    hipStream_t st = (hipStream_t)stream;
    acsr_rows_pattern_kernel<<<(unsigned)((s + 255) / 256), 256, 0, st>>>(pattern, (int)s, p0, p1, dTos_lin, dTos_trans, sTod_lin,
                                                                         sTod_trans, nnz, row_first, row_last, summary);
    const int n_blocks = (int)((s + block_height - 1) / block_height);
    acsr_spans_kernel<<<(n_blocks + 255) / 256, 256, 0, st>>>(sTod_lin, sTod_trans, nnz, (int)s, (int)s, block_height, span_start,
                                                               span_end, summary);
    return check_launch(who);
}

extern "C" int splat_mask_generate(uint8_t* mask, int64_t rows, int64_t cols, int64_t ld, int32_t pattern, int64_t p0,
                                   int64_t p1, void* stream) {
    begin_launch();
    if (!mask) return fail(SPLAT_E_NULL, "splat_mask_generate: null mask");
    if (rows <= 0 || cols <= 0 || ld < cols || rows > (1 << 23) || cols > (1 << 23))
        return fail(SPLAT_E_SHAPE, "splat_mask_generate: bad shape rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols, (long long)ld);
    {
        const int base = pattern & ~SPLAT_MASK_TRANSPOSED;
        if (pattern < 0 || base < SPLAT_MASK_BLOCKED || base > SPLAT_MASK_STRIDED_FAR)
            return fail(SPLAT_E_UNSUPPORTED, "splat_mask_generate: unknown pattern %d", pattern);
        const bool needs_p1 = base == SPLAT_MASK_DILATED || base == SPLAT_MASK_STRIDED_FAR;
        if (p0 < 0 || (base == SPLAT_MASK_BLOCKED && p0 <= 0) || (needs_p1 && p1 <= 0))
            return fail(SPLAT_E_SHAPE, "splat_mask_generate: bad pattern parameters p0=%lld p1=%lld", (long long)p0, (long long)p1);
    }
    const int vec_ok = ((reinterpret_cast<uintptr_t>(mask) & 15) == 0 && (ld & 15) == 0) ? 1 : 0;
    const int64_t n = rows * ((cols + 15) >> 4);
    mask_generate_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(mask, (int)rows, (int)cols, ld, pattern, p0, p1, vec_ok);
    return check_launch("splat_mask_generate");
}
