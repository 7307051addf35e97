// Pieces of the fused attention kernels (forward and backward) that work on one tile of scores.
#pragma once
#include "tile_copy.hpp"

namespace splat {

constexpr float kNegBigA = -1.0e30f;

// Live positions of one row in the tile that starts at position j0, one bit per position (bit b = position j0 + b):
// the row's span [lo, lo + cnt) intersected with its periodic pattern.  `first` is the smallest offset >= 0 in the tile
// whose position is congruent to the row's first one modulo its step (0 for unit step) and `pat` has a bit at every
// multiple of the step below 64.
__device__ __forceinline__ uint64_t row_live_bits(const RowWin& w, int j0, int first, uint64_t pat) {
    const int a = w.lo - j0, b = a + w.cnt;  // live range [a, b) in tile offsets
    const uint64_t lo_m = a <= 0 ? ~0ull : (a >= 64 ? 0ull : ~0ull << a);
    const uint64_t hi_m = b >= 64 ? ~0ull : (b <= 0 ? 0ull : (1ull << b) - 1ull);
    const uint64_t per = first < 64 ? pat << first : 0ull;
    return lo_m & hi_m & per;
}

// x where keep is -1, the masked score -1e30 where keep is 0 (one bit-field insert)
__device__ __forceinline__ float keep_or_mask(float x, int keep) {
    const uint32_t xb = __builtin_bit_cast(uint32_t, x), nb = __builtin_bit_cast(uint32_t, kNegBigA);
    return __builtin_bit_cast(float, (xb & (uint32_t)keep) | (nb & ~(uint32_t)keep));
}

// Accumulator register j of 32-key half nt of a lane holds position 32*nt + 8*(j/4) + 4*g + j%4 of the tile; its bit
// of `live` (see row_live_bits) says whether the score is kept.
template <int NT>
__device__ __forceinline__ void mask_tile(f32x16 (&s)[NT], uint64_t live, int g) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t bits = (uint32_t)(live >> (32 * nt)) >> (4 * g);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int c = 8 * (j >> 2) + (j & 3);
            s[nt][j] = keep_or_mask(s[nt][j], ((int)(bits << (31 - c))) >> 31);
        }
    }
}

}  // namespace splat
