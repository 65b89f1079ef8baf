// pf8_gemm_common.h -- what the block-scaled FP8 GEMM kernel files share: the argument block, the LDS swizzle, the
// global -> LDS copy instructions and the fragment read.
#pragma once
#include <type_traits>

#include "pf8_device.h"

namespace pf8 {

enum { MODE_FWD = 0, MODE_WGRAD = 1 };
enum { GROUP_NONE = 0, GROUP_CONTIG = 1, GROUP_MASKED = 2, GROUP_WGRAD = 3 };

struct GemmArgs {
    const uint8_t* p;      // P operand [Prows, red]
    const uint8_t* q;      // Q operand [Qrows, red]
    const float* sp;       // P scales
    const float* sq;       // Q scales
    void* out;
    int64_t Prows, Qrows;  // output is [Qrows, Prows]
    int64_t red;           // reduction length (elements = bytes)
    int64_t ldo;           // output row stride (elements)
    int sq_layout;         // forward only: 0 = [Qrows, KB], 1 = [KB, Qrows]
    int accumulate;        // wgrad only
    int group;             // GROUP_*
    int E;
    const int32_t* m_indices;   // GROUP_CONTIG: expert per row
    const int32_t* masked_m;    // GROUP_MASKED: valid rows per expert
    int32_t tile_start[257];    // GROUP_WGRAD: first 128-row block of each expert along the reduction axis
    int64_t ldsq;               // UE8M0 forward: bytes between the K blocks of sq (0 = Qrows)
    const int32_t* pair_list;   // UE8M0 forward: when set, the kernel runs only if the paired-tile kernel declines
    int cus;                    //   (header of its work-item list, compute units both assume)
    int pow2_scales;            // wgrad: every scale is a power of two (applied inside the MFMA)
    uint32_t wgrad_skip[8];     // GROUP_WGRAD: bit e set = expert e is another kernel's (the 256x256-tile launch)
    // fused up+gate -> SwiGLU -> 1x128 requantization (k_gemm_fwd_deep<.., .., 1>): P holds [gate rows | up rows],
    // Prows = 2 * inter; `out` (bf16 [Qrows, 2 inter]) may be null
    int64_t inter;              // I: columns of the quantized activation
    const float* probs;         // per-row factor or null
    uint8_t* q2;                // e4m3 [Qrows, inter]
    float* s2;                  // fp32 [Qrows, inter / 128]
    int pow2_out;               // bit 0: power-of-two scale rule of the requantization; bit 1: s2 stored [inter / 128, Qrows]
};

// 16-byte chunk c of LDS row `row` lives at chunk c ^ swz_key(row): the 16 rows a fragment read touches
// then fall on 16 different bank groups of the 64-bank LDS
__device__ __forceinline__ int swz_key(int row) { return (row & 7) ^ ((row >> 3) & 1); }
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ swz_key(row)) << 4); }

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

// 16 bytes per lane, global -> LDS without passing through registers.  lds_dst is the wave-uniform
// LDS byte address of the 1 KB the instruction fills (lane l writes bytes [16 l, 16 l + 16)).
// Written as inline assembly on purpose: the compiler's wait-count pass treats a visible
// global_load_lds as a pending FLAT access and then turns every later LDS wait into a full drain
// (lgkmcnt(0)), which serialises the fragment reads of a K block with its first MFMA.  The copy
// is tracked by vmcnt in hardware; the K loop waits for it explicitly before its barrier.
// M0 is written here without being listed as clobbered: this compiler treats M0 as a reserved register (a clobber
// entry for it is rejected with a warning and ignored), never allocates it, and sets it itself only directly in
// front of an instruction that reads it, so no value of the compiler's lives in M0 across this statement.
__device__ __forceinline__ void dma16_to_lds(const uint8_t* src, uint32_t lds_dst) {
    const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(m0v) : "memory");
}

__device__ __forceinline__ i32x8 ld_frag_lds(const uint8_t* p0, const uint8_t* p1) {
    i32x4 lo = *reinterpret_cast<const i32x4*>(p0);
    i32x4 hi = *reinterpret_cast<const i32x4*>(p1);
    return (i32x8){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

// the same copy with a scalar base and one 32-bit lane offset; lds_dst is wave-uniform
__device__ __forceinline__ void dma16_s(uint32_t voff, const uint8_t* sbase, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_dst) : "memory");
}

// 4 bytes per lane: 256 B per instruction, lane l writes bytes [4 l, 4 l + 4) behind lds_dst
__device__ __forceinline__ void dma4_s(uint32_t voff, const uint8_t* sbase, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_dst) : "memory");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), unrolled at compile time
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

}  // namespace pf8
