// Shared device/host helpers for the gfx950 SPLAT kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/splat_hip.h"

namespace splat {

using bf16 = __bf16;
using f16 = _Float16;

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- host side error plumbing (defined in api_common.cpp) ---------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
void begin_launch();  // first statement of every function that launches and then calls check_launch
int check_launch(const char* what);

// Raise a kernel's dynamic LDS limit once per device (the attribute belongs to the device's copy of the kernel, so a
// process that uses several GPUs needs it on each): `done` is a bit mask over device ordinals, one per kernel.
int reserve_dynamic_lds(uint64_t* done, const void* kernel, size_t bytes, const char* who);

constexpr int kWave = 64;

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, int I = 0, typename F>
__host__ __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

template <typename T>
struct ElemTraits;
template <>
struct ElemTraits<float> {
    static constexpr int kDtype = SPLAT_F32;
};
template <>
struct ElemTraits<f16> {
    static constexpr int kDtype = SPLAT_F16;
};
template <>
struct ElemTraits<bf16> {
    static constexpr int kDtype = SPLAT_BF16;
};

// An MFMA operand fragment: what one lane feeds into one 32x32 x (16 contraction values) step.
// Lane (i = lane%32, g = lane/32) holds contraction slots 8g..8g+7 of row/column i.
template <typename T>
struct Frag {
    typedef T vec __attribute__((ext_vector_type(8)));
    vec v;
};

// acc[32x32] += A[32x16] * B[16x32]; A fragment rows = output rows, B fragment rows = output cols.
// Output layout: lane (n = lane%32, g = lane/32), register j holds row 8*(j/4) + 4*g + j%4, col n.
__device__ __forceinline__ void mma32(f32x16& acc, const Frag<bf16>& a, const Frag<bf16>& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma32(f32x16& acc, const Frag<f16>& a, const Frag<f16>& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma32(f32x16& acc, const Frag<float>& a, const Frag<float>& b) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[j], b.v[j], acc, 0, 0, 0);
}

// acc[16x16] += A[16x32] * B[32x16].  Lane (i = lane%16, g = lane/16) holds contraction slots 8g..8g+7 of row i (A) or
// column i (B); of the output, lane (n = lane%16, g = lane/16) holds rows 4g..4g+3 of column n.
typedef float f32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void mma16(f32x4v& acc, const Frag<bf16>& a, const Frag<bf16>& b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma16(f32x4v& acc, const Frag<f16>& a, const Frag<f16>& b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, acc, 0, 0, 0);
}

// Row (within a 32-row tile) held by accumulator register j of lane group g.
__device__ __forceinline__ constexpr int acc_row(int j, int g) { return 8 * (j >> 2) + 4 * g + (j & 3); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <typename T>
__device__ __forceinline__ T from_float(float x) {
    return (T)x;
}
template <typename T>
__device__ __forceinline__ float to_float(T x) {
    return (float)x;
}

// Store a float as element `idx` of a buffer whose element type is chosen at run time.
__device__ __forceinline__ void store_as(void* base, int64_t idx, float x, int dtype) {
    if (dtype == SPLAT_BF16)
        ((bf16*)base)[idx] = (bf16)x;
    else if (dtype == SPLAT_F16)
        ((f16*)base)[idx] = (f16)x;
    else
        ((float*)base)[idx] = x;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o));
    return v;
}

// Integer view of one row's affine map, recovered from the float32 metadata.
//   a   = first live dense column, lin = column step, cnt = live slots.
// sTod_trans stores a/lin rounded to float32, so a = rint(lin * trans) is exact for a < 2^23.
struct RowMap {
    int a, lin, cnt;
};
__device__ __forceinline__ RowMap load_row_map(const float* sTod_lin, const float* sTod_trans, const float* nnz,
                                               const int32_t* first_col, int r) {
    RowMap m;
    m.cnt = (int)nnz[r];
    float lin = sTod_lin[r];
    m.lin = max((int)lin, 1);
    m.a = (int)rintf(lin * sTod_trans[r]);
    if (first_col != nullptr && m.cnt == 1) m.a = first_col[r];
    return m;
}

// Workgroup barrier that hands LDS contents over and nothing else: it waits for this wavefront's LDS traffic, not for
// its global loads and stores.  __syncthreads() waits for both counters, which serialises a kernel whose loads of the
// next tile or stores of the previous one are meant to stay in flight across the barrier.  (The empty statements keep
// the compiler from moving memory accesses across the barrier.)
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Map a launch-order workgroup id onto a logical id so that logically consecutive ids run on the
// same XCD (hardware deals consecutive workgroup ids round-robin over the 8 XCDs, each with its own
// L2).  gridDim.x must be 8 * chunk; ids >= total are idle.
__device__ __forceinline__ int xcd_remap(int wg, int grid) {
    const int chunk = grid >> 3;
    return (wg & 7) * chunk + (wg >> 3);
}

}  // namespace splat
