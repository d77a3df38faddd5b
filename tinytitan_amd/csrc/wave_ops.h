// Cross-lane reductions over the 2 (32-row tiles) or 4 (16-row tiles) lanes that share a query
// row, with gfx950's v_permlane32_swap / v_permlane16_swap: no lane-index register, no LDS trip.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

namespace tt {

// v_permlane32_swap(x, x): first result = lanes 0-31 of x in both halves, second = lanes 32-63.
__device__ __forceinline__ void halves_of(float x, float &lo, float &hi) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    lo = __builtin_bit_cast(float, (unsigned)r[0]);
    hi = __builtin_bit_cast(float, (unsigned)r[1]);
}
// v_permlane16_swap(x, x): first result = rows 0,0,2,2 of x (a row is 16 lanes), second = rows 1,1,3,3.
__device__ __forceinline__ void row_pairs_of(float x, float &even, float &odd) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    even = __builtin_bit_cast(float, (unsigned)r[0]);
    odd = __builtin_bit_cast(float, (unsigned)r[1]);
}

// Lanes l and l ^ 32.
__device__ __forceinline__ float max_across_halves(float x) {
    float lo, hi;
    halves_of(x, lo, hi);
    return fmaxf(lo, hi);
}
__device__ __forceinline__ float sum_across_halves(float x) {
    float lo, hi;
    halves_of(x, lo, hi);
    return lo + hi;
}
// Lanes l, l ^ 16, l ^ 32, l ^ 48.
__device__ __forceinline__ float max_across_quarters(float x) {
    float a, b;
    row_pairs_of(x, a, b);
    return max_across_halves(fmaxf(a, b));
}
__device__ __forceinline__ float sum_across_quarters(float x) {
    float a, b;
    row_pairs_of(x, a, b);
    return sum_across_halves(a + b);
}

// The largest value of the 64 lanes, in every lane, by data-parallel-primitive moves: within a row of 16 lanes by
// row_shr 1, 2, 4, 8, then lane 15 of every row into the row after it (row_bcast15) and lane 31 into the upper half
// (row_bcast31) -- a lane takes a step's value only where the move had a source -- then lane 63's.
__device__ __forceinline__ float wave_max_f32(float x, int lane) {
    const int in_row = lane & 15;
    auto moved = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    float t;
    t = moved(x, std::integral_constant<int, 0x111>{});
    if (in_row >= 1) x = fmaxf(x, t);
    t = moved(x, std::integral_constant<int, 0x112>{});
    if (in_row >= 2) x = fmaxf(x, t);
    t = moved(x, std::integral_constant<int, 0x114>{});
    if (in_row >= 4) x = fmaxf(x, t);
    t = moved(x, std::integral_constant<int, 0x118>{});
    if (in_row >= 8) x = fmaxf(x, t);
    t = moved(x, std::integral_constant<int, 0x142>{});
    if ((lane & 31) >= 16) x = fmaxf(x, t);
    t = moved(x, std::integral_constant<int, 0x143>{});
    if (lane >= 32) x = fmaxf(x, t);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

// The sum of the 64 lanes, in lane 63 (other lanes hold partial sums): row_shr 1, 2, 4, 8 inside the rows of 16, then
// row_bcast15 and row_bcast31; a lane whose move has no source adds zero.  Six vector instructions, no trip through LDS.
__device__ __forceinline__ float wave_sum_in_lane63(float x) {
    auto moved = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    x += moved(x, std::integral_constant<int, 0x111>{});
    x += moved(x, std::integral_constant<int, 0x112>{});
    x += moved(x, std::integral_constant<int, 0x114>{});
    x += moved(x, std::integral_constant<int, 0x118>{});
    x += moved(x, std::integral_constant<int, 0x142>{});
    x += moved(x, std::integral_constant<int, 0x143>{});
    return x;
}

// Sums, minima and maxima over aligned groups of 8, 16 or 32 lanes, every lane of a group getting the result, by DPP
// moves: quad_perm [1,0,3,2] and [2,3,0,1] inside a quad; then row_half_mirror (lane i <-> 7 - i: the other quad,
// whose lanes all hold that quad's value by now) and row_mirror (i <-> 15 - i: the other eight); the other row of 16 by
// v_permlane16_swap.  No trip through LDS.
template <int CTRL>
__device__ __forceinline__ float dpp_moved(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LANES, typename Op>
__device__ __forceinline__ float group_reduce(float x, Op op) {
    static_assert(LANES == 4 || LANES == 8 || LANES == 16 || LANES == 32, "a group of 4, 8, 16 or 32 lanes");
    x = op(x, dpp_moved<0xB1>(x));
    x = op(x, dpp_moved<0x4E>(x));
    if constexpr (LANES >= 8) x = op(x, dpp_moved<0x141>(x));
    if constexpr (LANES >= 16) x = op(x, dpp_moved<0x140>(x));
    if constexpr (LANES >= 32) {
        float even, odd;
        row_pairs_of(x, even, odd);
        x = op(even, odd);
    }
    return x;
}
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
    return group_reduce<LANES>(x, [](float a, float b) { return a + b; });
}
template <int LANES>
__device__ __forceinline__ float group_min(float x) {
    return group_reduce<LANES>(x, [](float a, float b) { return fminf(a, b); });
}
template <int LANES>
__device__ __forceinline__ float group_max(float x) {
    return group_reduce<LANES>(x, [](float a, float b) { return fmaxf(a, b); });
}

}  // namespace tt
