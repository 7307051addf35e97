// K^T [B, H, d, L] with the keys contiguous (the reference's layout, r_sddmm.py:230-231) -> K [B, H, L, d] with rows
// contiguous, which is what the kernels read without waste when rows step over columns (a dilated window's every second
// key, a strided far field's every 128th): there they fetch only the keys a tile needs, while K^T can only be read in
// dense runs of keys.  A pure streaming kernel: every byte read once and written once, in whole 16-byte pieces on both
// sides; the turn goes through a 64 x 64 LDS tile.
#include "splat_common.hpp"

namespace splat {

struct TransposeParams {
    const void* src;
    void* dst;
    int64_t s_sb, s_sh, s_sd;  // element strides of the source's batch, head and d index; keys have stride 1
    int B, H, L, d;
    int vec;  // 16-byte loads are legal for every source row
};

// One workgroup: 64 keys x 64 values of d of one (batch, head).  LDS tile [d index][key], read back key by key.
template <typename T>
__global__ __launch_bounds__(256) void transpose_keys_kernel(const TransposeParams p) {
    constexpr int ES = sizeof(T), EPC = 16 / ES;  // elements per 16-byte piece
    constexpr int TK = 64, TD = 64;
    constexpr int PITCH = TK * ES + 4;            // odd number of banks between rows: the column reads spread out
    __shared__ __attribute__((aligned(16))) char tile[TD * PITCH];
    const int tid = threadIdx.x;
    const int n_kt = (p.L + TK - 1) / TK, n_dt = (p.d + TD - 1) / TD;
    int blk = blockIdx.x;
    const int kt = blk % n_kt;
    blk /= n_kt;
    const int dt = blk % n_dt;
    const int bh = blk / n_dt;
    const int b = bh / p.H, h = bh % p.H;
    const int k0 = kt * TK, d0 = dt * TD;
    const T* src = (const T*)p.src + (int64_t)b * p.s_sb + (int64_t)h * p.s_sh;
    T* dst = (T*)p.dst + (int64_t)bh * p.L * p.d;

    // in: rows = d index, 64 keys each
    constexpr int PPR = TK / EPC;  // pieces per row
#pragma unroll
    for (int i = 0; i < TD * PPR / 256; ++i) {
        const int idx = tid + 256 * i, row = idx / PPR, pc = idx % PPR;
        const int dd = d0 + row, kk = k0 + pc * EPC;
        T v[EPC];
        if (dd < p.d && p.vec && kk + EPC <= p.L) {
            __builtin_memcpy(v, __builtin_assume_aligned(src + (int64_t)dd * p.s_sd + kk, 16), 16);
        } else {
#pragma unroll
            for (int e = 0; e < EPC; ++e) v[e] = (dd < p.d && kk + e < p.L) ? src[(int64_t)dd * p.s_sd + kk + e] : (T)0.f;
        }
#pragma unroll
        for (int e = 0; e < EPC; ++e) *reinterpret_cast<T*>(tile + row * PITCH + (pc * EPC + e) * ES) = v[e];
    }
    __syncthreads();
    // out: rows = keys, 64 values of d each (one 16-byte piece per thread and pass)
    constexpr int PPK = TD / EPC;  // pieces per key
    const bool dvec = (p.d % EPC) == 0;  // every destination piece starts on a 16-byte boundary
#pragma unroll
    for (int i = 0; i < TK * PPK / 256; ++i) {
        const int idx = tid + 256 * i, key = idx / PPK, pc = idx % PPK;
        const int kk = k0 + key, dd = d0 + pc * EPC;
        if (kk >= p.L || dd >= p.d) continue;
        T v[EPC];
#pragma unroll
        for (int e = 0; e < EPC; ++e) v[e] = *reinterpret_cast<const T*>(tile + (pc * EPC + e) * PITCH + key * ES);
        T* out = dst + (int64_t)kk * p.d + dd;
        if (dvec && dd + EPC <= p.d) {
            __builtin_memcpy(__builtin_assume_aligned(out, 16), v, 16);
        } else {
#pragma unroll
            for (int e = 0; e < EPC; ++e)
                if (dd + e < p.d) out[e] = v[e];
        }
    }
}

}  // namespace splat

using namespace splat;

extern "C" int splat_transpose_keys(const void* kT, int64_t kT_sb, int64_t kT_sh, int64_t kT_sd, void* k_rows, int32_t B,
                                    int32_t H, int32_t L, int32_t d, int32_t dtype, void* stream) {
    begin_launch();
    if (!kT || !k_rows) return fail(SPLAT_E_NULL, "splat_transpose_keys: null pointer argument");
    if (B <= 0 || H <= 0 || L <= 0 || d <= 0) return fail(SPLAT_E_SHAPE, "splat_transpose_keys: need B, H, L, d > 0 (got %d, %d, %d, %d)", B, H, L, d);
    if (kT_sd < L) return fail(SPLAT_E_SHAPE, "splat_transpose_keys: the stride of the d index (%lld) is shorter than a row of %d keys", (long long)kT_sd, L);
    const int es = dtype == SPLAT_F32 ? 4 : 2;
    if (dtype != SPLAT_F32 && dtype != SPLAT_F16 && dtype != SPLAT_BF16) return fail(SPLAT_E_DTYPE, "splat_transpose_keys: unknown dtype %d", dtype);
    if ((reinterpret_cast<uintptr_t>(k_rows) & 15) != 0) return fail(SPLAT_E_ALIGN, "splat_transpose_keys: k_rows must be 16-byte aligned");
    if ((reinterpret_cast<uintptr_t>(kT) & (es - 1)) != 0) return fail(SPLAT_E_ALIGN, "splat_transpose_keys: kT is not aligned to its element size");
    const int64_t blocks = (int64_t)B * H * ((L + 63) / 64) * ((d + 63) / 64);
    if (blocks > 0x7ffffff0) return fail(SPLAT_E_SHAPE, "splat_transpose_keys: problem too large for one launch");
    TransposeParams p;
    p.src = kT, p.dst = k_rows;
    p.s_sb = kT_sb, p.s_sh = kT_sh, p.s_sd = kT_sd;
    p.B = B, p.H = H, p.L = L, p.d = d;
    const int epc = 16 / es;
    p.vec = ((reinterpret_cast<uintptr_t>(kT) & 15) == 0) && kT_sb % epc == 0 && kT_sh % epc == 0 && kT_sd % epc == 0;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == SPLAT_F32)
        transpose_keys_kernel<float><<<(int)blocks, 256, 0, st>>>(p);
    else  // the two 16-bit types move alike
        transpose_keys_kernel<bf16><<<(int)blocks, 256, 0, st>>>(p);
    return check_launch("splat_transpose_keys");
}
