// Sums across the lanes of a wave64 with DPP (data-parallel primitives: an operand of a vector
// instruction is taken from another lane of the same wavefront, no LDS traffic, no barrier).
//
// wave_group_sum<W>(v): the lanes of a wavefront are split into groups of W consecutive lanes (W a
// power of two, 2..64); the LAST lane of every group returns the sum of its group's values, the other
// lanes partial sums.  Steps: row_shr:1,2,4,8 add, within each row of 16 lanes, the value 1, 2, 4, 8
// lanes to the left (lanes without such a neighbour add 0), which leaves the total of the window of
// 2, 4, 8, 16 lanes that ends at a lane; row_bcast:15 adds lane 15 of rows 0 and 2 to every lane of
// rows 1 and 3, row_bcast:31 adds lane 31 to rows 2 and 3 -- so lane 31 ends with the total of lanes
// 0..31 and lane 63 with the total of the wavefront.
//
// block_group_sum<W>(v, scratch): groups of W = 128..1024 consecutive threads of a workgroup (whole
// wavefronts); wavefront totals meet in LDS.  All threads of the workgroup must call it together.
//
// wave_group_reduce<W, OP> / block_group_reduce<W, OP> are the same for another operation (max_op, min_op): a lane
// without a neighbour contributes the operation's identity instead of 0.
#ifndef TIRAMISU_AMD_WAVE_REDUCE_HIP_H
#define TIRAMISU_AMD_WAVE_REDUCE_HIP_H
#include <hip/hip_runtime.h>
#include <limits>

namespace twave {

// The operations: apply() and the value that changes nothing (what a lane without a neighbour contributes).
struct sum_op {
    template <class T> static __device__ __forceinline__ T identity() { return (T)0; }
    template <class T> static __device__ __forceinline__ T apply(T a, T b) { return a + b; }
};
struct max_op {
    template <class T> static __device__ __forceinline__ T identity() {
        return std::numeric_limits<T>::has_infinity ? -std::numeric_limits<T>::infinity() : std::numeric_limits<T>::lowest();
    }
    template <class T> static __device__ __forceinline__ T apply(T a, T b) { return a > b ? a : b; }
};
struct min_op {
    template <class T> static __device__ __forceinline__ T identity() {
        return std::numeric_limits<T>::has_infinity ? std::numeric_limits<T>::infinity() : std::numeric_limits<T>::max();
    }
    template <class T> static __device__ __forceinline__ T apply(T a, T b) { return a < b ? a : b; }
};

// T: float, double, or a 32- or 64-bit integer.  The value of the lane that the control word names, `fill` where there is
// no such lane or the row is masked out.  DPP moves 32-bit lanes, so a 64-bit value travels as its two halves.
template <int CTRL, int ROW_MASK, class T>
__device__ __forceinline__ T dpp_from(T v, T fill) {
    static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit values");
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill), __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
    } else {
        const unsigned long long bits = __builtin_bit_cast(unsigned long long, v), fbits = __builtin_bit_cast(unsigned long long, fill);
        const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp((int)(unsigned)fbits, (int)(unsigned)bits, CTRL, ROW_MASK, 0xf, false);
        const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp((int)(unsigned)(fbits >> 32), (int)(unsigned)(bits >> 32), CTRL, ROW_MASK, 0xf, false);
        return __builtin_bit_cast(T, ((unsigned long long)hi << 32) | lo);
    }
}

template <int W, class OP, class T>
__device__ __forceinline__ T wave_group_reduce(T v) {
    static_assert(W >= 2 && W <= 64 && (W & (W - 1)) == 0, "group width must be a power of two up to the wavefront size");
    const T e = OP::template identity<T>();
    if (W >= 2) v = OP::apply(v, dpp_from<0x111, 0xf>(v, e));    // row_shr:1
    if (W >= 4) v = OP::apply(v, dpp_from<0x112, 0xf>(v, e));    // row_shr:2
    if (W >= 8) v = OP::apply(v, dpp_from<0x114, 0xf>(v, e));    // row_shr:4
    if (W >= 16) v = OP::apply(v, dpp_from<0x118, 0xf>(v, e));   // row_shr:8
    if (W >= 32) v = OP::apply(v, dpp_from<0x142, 0xa>(v, e));   // row_bcast:15 into rows 1 and 3
    if (W >= 64) v = OP::apply(v, dpp_from<0x143, 0xc>(v, e));   // row_bcast:31 into rows 2 and 3
    return v;
}

// `scratch` holds one value per wavefront of the workgroup; `linear` is the thread's linear id.
template <int W, class OP, class T>
__device__ __forceinline__ T block_group_reduce(T v, T *scratch, int linear) {
    static_assert(W % 64 == 0 && W >= 128 && W <= 1024, "group width must be whole wavefronts");
    v = wave_group_reduce<64, OP>(v);
    if ((linear & 63) == 63) scratch[linear >> 6] = v;
    __syncthreads();
    T total = OP::template identity<T>();
    if ((linear % W) == W - 1) {
        const int last = linear >> 6;
#pragma unroll
        for (int w = W / 64 - 1; w >= 0; w--) total = OP::apply(total, scratch[last - w]);
    }
    __syncthreads();
    return total;
}

template <int W, class T> __device__ __forceinline__ T wave_group_sum(T v) { return wave_group_reduce<W, sum_op>(v); }
template <int W, class T> __device__ __forceinline__ T block_group_sum(T v, T *scratch, int linear) { return block_group_reduce<W, sum_op>(v, scratch, linear); }

}  // namespace twave
#endif
