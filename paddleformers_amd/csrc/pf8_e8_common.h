// pf8_e8_common.h -- what the kernels whose 256x256 accumulator tile is the whole AGPR file share: the LDS swizzle key,
// the global -> LDS copy, the fragment read and the literal accumulator-register accessors.
#pragma once
#include <type_traits>

#include "pf8_device.h"

namespace pf8 {

__device__ __forceinline__ int e8_keyp(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// 16 bytes per lane global -> LDS, scalar base + 32-bit lane offset; tracked by vmcnt only
__device__ __forceinline__ void e8_dma16(uint32_t voff, const uint8_t* sbase, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_dst) : "memory");
}
__device__ __forceinline__ i32x8 e8_frag(const uint8_t* p0, const uint8_t* p1) {
    i32x4 lo = *reinterpret_cast<const i32x4*>(p0);
    i32x4 hi = *reinterpret_cast<const i32x4*>(p1);
    return (i32x8){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

template <int IDX>
__device__ __forceinline__ void e8_acc_zero4() {
    asm volatile("v_accvgpr_write_b32 a[%0], 0\n\tv_accvgpr_write_b32 a[%1], 0\n\tv_accvgpr_write_b32 a[%2], 0\n\tv_accvgpr_write_b32 a[%3], 0"
                 : : "n"(4 * IDX), "n"(4 * IDX + 1), "n"(4 * IDX + 2), "n"(4 * IDX + 3));
}
template <int R>
__device__ __forceinline__ float e8_acc_get() {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(R));
    return v;
}
template <int N, typename F>
__device__ __forceinline__ void e8_static_for(F&& f) {
    if constexpr (N > 0) {
        e8_static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

}  // namespace pf8
