// Measurement aid: the matrix work of the fused forward's tile loop with nothing else around it.
//
// Every wavefront runs, per tile, exactly the LDS reads and MFMAs of one 64-key tile of the fused kernel at d = 128
// and a 16-bit type: 16 row-wise 16-byte reads + 16 MFMAs (scores), then 32 transposing reads + 16 MFMAs (output).
// There are no global loads in the loop, no copies into LDS, no exponentials and no barriers; the LDS holds the
// caller's data (random values give the switching activity of real operands; zeros do not).  What this loop sustains
// is what the chip can give any kernel of this shape: on a part that runs into its power limit the clock drops under
// such a loop, so the figure lies below the rated peak, which is quoted at the full clock.  bench.py reports it next
// to the fused forward.
#include "tile_copy.hpp"

namespace splat {

__global__ __launch_bounds__(256, 2) void mfma_lds_probe_kernel(const bf16* data, float* out, int tiles) {
    constexpr int D = 128, BN = 64, KS = D / 16, DT = D / 32, NT = BN / 32, ROWB = D * 2, KBYTES = BN * ROWB, STAGE = 2 * KBYTES;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int tid = threadIdx.x, lane = tid & 63, lm = lane & 31, g = lane >> 5;
    // two stages of (K tile, V tile) from the caller's 64 KiB
    for (int i = tid; i < 2 * STAGE / 16; i += 256)
        reinterpret_cast<u32x4*>(smem)[i] = reinterpret_cast<const u32x4*>(data)[i];
    Frag<bf16> qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = global_frag<bf16>(data + (tid & 127) * D + 16 * ks + 8 * g);
    __syncthreads();
    const uint32_t smem_base = lds_address(smem);
    const int tr_row = (lane & 15) >> 2, tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    uint32_t k_addr[KS], v_addr[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        v_addr[dt] = smem_base + KBYTES + (4 * g + tr_row) * ROWB + ((dt ^ swz64<ROWB>(4 * g + tr_row)) * 64) + tr_col * 2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_addr[ks] = smem_base + lds_off<ROWB, true>(lm, (16 * ks + 8 * g) * 2);
    f32x16 o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) o_acc[dt][j] = 0.f;
    int stage = 0;
    for (int it = 0; it < tiles; ++it) {
        f32x16 s_acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 16; ++j) s_acc[nt][j] = 0.f;
        constexpr int NMMA = NT * KS, K_AHEAD = 12;
        Frag<bf16> kfr[NMMA];
        auto load_k = [&](int i) {
            Frag<bf16> kf;
            kf.v = __builtin_bit_cast(typename Frag<bf16>::vec, lds_load128(k_addr[i % KS] + 32 * (i / KS) * ROWB));
            return kf;
        };
#pragma unroll
        for (int i = 0; i < K_AHEAD; ++i) kfr[i] = load_k(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NMMA; ++i) {
            mma32(s_acc[i / KS], kfr[i], qf[i % KS]);
            if (i + K_AHEAD < NMMA) {
                kfr[i + K_AHEAD] = load_k(i + K_AHEAD);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // scores to 16-bit operands of the second product, scaled so that the values stay of order one
        Frag<bf16> pf[NT][2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 16; ++j) pf[nt][j >> 3].v[j & 7] = (bf16)(s_acc[nt][j] * 0.0884f);
        auto load_v = [&](int nt, int t, int dt) {
            const uint32_t a0 = v_addr[dt] + (32 * nt + 16 * t) * ROWB;
            return frag_from_tr<bf16>(lds_load_tr16(a0), lds_load_tr16(a0 + 8 * ROWB));
        };
        Frag<bf16> vfr[2][DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vfr[0][dt] = load_v(0, 0, dt);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 2 * NT; ++step) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                mma32(o_acc[dt], vfr[step & 1][dt], pf[step >> 1][step & 1]);
                if (step + 1 < 2 * NT) {
                    vfr[(step + 1) & 1][dt] = load_v((step + 1) >> 1, (step + 1) & 1, dt);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        stage ^= 1;
        const int delta = stage == 0 ? -STAGE : STAGE;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_addr[dt] += delta;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) k_addr[ks] += delta;
    }
    float sum = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 16; ++j) sum += o_acc[dt][j];
    out[(int64_t)blockIdx.x * 256 + tid] = sum;
}

}  // namespace splat

using namespace splat;

extern "C" int splat_mfma_lds_probe(const void* data, int64_t data_bytes, void* out, int64_t out_bytes, int32_t workgroups,
                                    int32_t tiles, void* stream) {
    begin_launch();
    if (!data || !out) return fail(SPLAT_E_NULL, "splat_mfma_lds_probe: null pointer argument");
    if (workgroups < 1 || workgroups > (1 << 20) || tiles < 1 || tiles > (1 << 20))
        return fail(SPLAT_E_SHAPE, "splat_mfma_lds_probe: workgroups and tiles must be 1..2^20 (got %d, %d)", workgroups, tiles);
    if (data_bytes < 65536) return fail(SPLAT_E_SHAPE, "splat_mfma_lds_probe: data must hold 65536 bytes (got %lld)", (long long)data_bytes);
    if (out_bytes < (int64_t)workgroups * 256 * 4)
        return fail(SPLAT_E_SHAPE, "splat_mfma_lds_probe: out must hold 1024 bytes per workgroup (got %lld for %d)", (long long)out_bytes, workgroups);
    if ((reinterpret_cast<uintptr_t>(data) & 15) != 0 || (reinterpret_cast<uintptr_t>(out) & 3) != 0)
        return fail(SPLAT_E_ALIGN, "splat_mfma_lds_probe: data must be 16-byte aligned, out 4-byte aligned");
    static uint64_t lds_reserved = 0;
    if (int rc = reserve_dynamic_lds(&lds_reserved, (const void*)mfma_lds_probe_kernel, 65536, "splat_mfma_lds_probe")) return rc;
    mfma_lds_probe_kernel<<<workgroups, 256, 65536, (hipStream_t)stream>>>(static_cast<const bf16*>(data), static_cast<float*>(out), tiles);
    return check_launch("splat_mfma_lds_probe");
}
