// Running min / max of a tensor kept by the kernel that produces it, so that a
// dynamic quantizer downstream needs no pass of its own over the tensor.
//
// A range buffer is kRangeWords 32-bit words: word 0 = number of partial slots
// in use, then kRangeSlots minima and kRangeSlots maxima.  Every block of the
// producing kernel writes its own slot (no atomics, nothing to initialise);
// the consumer reduces the slots.  fminf / fmaxf drop NaNs, so a block that saw
// a NaN stores NaN in both of its slots and the reduction propagates it (the
// reference's reductions propagate NaN, lucid/_C/backend/cpu/Reduce.cpp:87-125).
// min and max are exact and order-independent, so the result is bit-identical
// to a separate min / max pass.
#pragma once
#include "common.hpp"

namespace lq {

constexpr int kRangeSlots = 16384;
constexpr int kRangeWords = 4 + 2 * kRangeSlots;

// Folds one (lo, hi, nan) per lane of a block (up to 1024 threads) into the
// block's slot.  All threads of the block must call it; gridDim.x * gridDim.y
// must not exceed kRangeSlots.
__device__ __forceinline__ void range_block_store(float* range, float lo, float hi, int nan) {
    __shared__ float s_lo[16], s_hi[16];
    __shared__ int s_nan[16];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        lo = fminf(lo, __shfl_xor(lo, d, 64));
        hi = fmaxf(hi, __shfl_xor(hi, d, 64));
        nan |= __shfl_xor(nan, d, 64);
    }
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if ((threadIdx.x & 63) == 0) s_lo[wave] = lo, s_hi[wave] = hi, s_nan[wave] = nan;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < nw; ++w) {
            lo = fminf(lo, s_lo[w]);
            hi = fmaxf(hi, s_hi[w]);
            nan |= s_nan[w];
        }
        if (nan) lo = hi = __builtin_nanf("");
        const unsigned slot = blockIdx.y * gridDim.x + blockIdx.x;
        range[4 + slot] = lo;
        range[4 + kRangeSlots + slot] = hi;
        if (slot == 0) reinterpret_cast<unsigned*>(range)[0] = gridDim.x * gridDim.y;
    }
}

}  // namespace lq
