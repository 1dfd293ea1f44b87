// Running min / max of a tensor kept by the kernel that produces it, so that a
// dynamic quantizer downstream needs no pass of its own over the tensor.
//
// The range lives in four 32-bit words: {min key, max key, NaN flag, unused}.
// A key is the float's bit pattern mapped to an unsigned integer that orders
// the same way (negative floats reversed, sign bit flipped), so atomicMin /
// atomicMax on the keys are an exact, order-independent float min / max.
// fminf / fmaxf drop NaNs; a NaN anywhere sets the flag instead, and decoding
// then yields NaN for both ends (the reference's reductions propagate NaN,
// lucid/_C/backend/cpu/Reduce.cpp:87-125).
#pragma once
#include "common.hpp"

namespace lq {

constexpr uint32_t kRangeMinIdentity = 0xff800000u;  // key of +inf
constexpr uint32_t kRangeMaxIdentity = 0x007fffffu;  // key of -inf

__device__ __forceinline__ uint32_t range_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}

__device__ __forceinline__ float range_unkey(uint32_t k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

// Folds one value per lane of a block (any block size up to 1024) into the keys:
// butterfly inside the wavefront, LDS across wavefronts, one lane does the atomics.
// All threads of the block must call it.
__device__ __forceinline__ void range_block_update(uint32_t* keys, float lo, float hi, int nan) {
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
        atomicMin(&keys[0], range_key(lo));
        atomicMax(&keys[1], range_key(hi));
        if (nan) atomicOr(&keys[2], 1u);
    }
}

}  // namespace lq
