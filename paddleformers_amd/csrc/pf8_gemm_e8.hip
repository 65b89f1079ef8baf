// pf8_gemm_e8.hip -- FP8 GEMMs whose block scales are powers of two, stored as UE8M0 exponent bytes
// (scale = 2^(byte - 127)): the forward / dgrad GEMM of the path when every operand was quantized
// with pow2 scales.  gfx950's block-scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4) applies both
// operands' scales inside the instruction, so a K block's product is accumulated by the matrix pipe
// itself instead of being folded in by vector FMAs.  That removes the product registers and the
// VALU work of the fp32-scale kernels and lets the accumulator tile fill the whole AGPR file.
//
// Geometry: 256(Q, output rows) x 256(P, output columns) x 128(K) blocks, 256 threads = 4 wavefronts
// (2 along Q x 2 along P), each owning 128 x 128 = 8 x 8 MFMA tiles = 256 accumulator registers.
// Per K block a compute unit moves 64 KB L2 -> LDS and reads 128 KB of fragments for 256 MFMAs:
// two thirds of the LDS traffic per MFMA of the 128 x 256 fp32-scale kernels.
//   * One persistent workgroup per compute unit; 128 KB of LDS is two slots of [P 32 KB | Q 32 KB].
//     The P fragments of a block (64 registers) are read once, behind the previous block's barrier,
//     and held; the Q fragments stream through a ring of four, three ahead of their MFMAs.
//   * One barrier per block, before MFMA 44 of 64: by then every fragment read of the block has
//     been issued, so the slot is free, and the wavefront's copies of the next block have landed.
//     Behind it the copies of the block after next go into the freed slot, one between every other
//     MFMA, running on into the next block; the ring runs on across tile boundaries.
//   * The accumulator tile IS the AGPR file: element (i, j) lives in a[4(8i+j) .. +3], named
//     literally in every instruction that touches it, so the register allocator never sees it
//     (left to the allocator, the tile gets split between both register files and copied back and
//     forth).  One empty statement that clobbers a255 makes the kernel descriptor reserve all 256.
//   * Q row r of a wavefront's fragment j is row 8 (r) + j of its 128, so the eight scale bytes a lane
//     needs per block are contiguous (one 8-byte load) and op_sel picks the byte per MFMA.
//   * Grouped layout: expert segments are padded to 128 rows, so a 256-row tile is made of two
//     128-row blocks of the SAME expert that need not be neighbours.  A one-workgroup pre-pass pairs
//     the blocks of every expert (an odd one out gets a half-empty tile, padding blocks get none) and
//     writes the list the GEMM walks.  Without a list the kernel walks aligned 256-row tiles and
//     visits a tile that holds two experts twice, once per expert, each pass storing its own half.
#include <atomic>
#include <type_traits>

#include "pf8_device.h"
#include "pf8_e8_common.h"
#include "pf8_host.h"

namespace pf8 {

struct E8Args {
    const uint8_t* p;      // [E][Prows, red]  weights: output columns
    const uint8_t* q;      // [Qrows, red]     activations: output rows
    const uint8_t* sp8;    // [E][Prows/128, KB] exponent bytes
    const uint8_t* sq8;    // [KB, ldsq] exponent bytes (1x128 scales, K-block major)
    void* out;             // bf16 [Qrows, ldo]
    int64_t Prows, Qrows, red, ldo, ldsq;
    int grouped;
    const int32_t* m_indices;
    const int32_t* items;   // grouped: {n, blocks, -, -} then {block0, block1 or -1, expert, -} per item; may be null
    int cus;
    int force;              // with items: run them here whatever the list's header says
};

// acc[IDX] += (2^(sa-127) A) (2^(sb.byte[OB]-127) B): A = P fragment (one scale per block), B = Q fragment
template <int IDX, int OB>
__device__ __forceinline__ void e8_mfma(const i32x8& a, const i32x8& b, int sa, int sb) {
    if constexpr (OB == 0) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel_hi:[0,0,0]" : : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(4 * IDX), "n"(4 * IDX + 3));
    if constexpr (OB == 1) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel:[0,1,0] op_sel_hi:[0,0,0]" : : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(4 * IDX), "n"(4 * IDX + 3));
    if constexpr (OB == 2) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel_hi:[0,1,0]" : : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(4 * IDX), "n"(4 * IDX + 3));
    if constexpr (OB == 3) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(4 * IDX), "n"(4 * IDX + 3));
}

__global__ __launch_bounds__(256, 1) void k_gemm_e8(const E8Args a) {
    constexpr int SLOT = 65536, Q_OFS = 32768, EP_OFS = 131072, EP_LD = 272;
    constexpr int BAR = 44, CSTEP = 2;     // barrier position; MFMAs between two copies
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    asm volatile("" ::: "a255");
    if (a.items && !a.force && !e8_paired_tiles_win(a.items, a.Prows / 256, a.cus)) return;   // left to the 128-row-tile kernel
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = wave >> 1, wp = wave & 1;
    const int li = lane & 15, kg = lane >> 4;

    // Prows = 256 t + 128: the last column tile has one 128-row half; its second half re-reads the first
    // (as a missing Q half does) and the wavefronts that own it store nothing
    const int64_t p_tiles = (a.Prows + 255) / 256, q_tiles = a.items ? (int64_t)__builtin_amdgcn_readfirstlane(a.items[0]) : (a.Qrows + 255) / 256;
    const int64_t T = p_tiles * q_tiles;
    // consecutive workgroups go round-robin to the 8 XCDs: every XCD owns a contiguous run of
    // logical tiles (groups of 8 q-tiles x all p-tiles), walked W tiles at a time by its W workgroups
    const int64_t per_xcd = (T + 7) / 8;
    const int64_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, W = gridDim.x >> 3;
    const int64_t KB = a.red / 128, PB = a.Prows / 128;

    auto tile_coords = [&](int64_t n, int64_t& q_tile, int64_t& p_tile) -> bool {
        constexpr int G = 8;
        const int64_t loc = slot + n * W, logical = xcd * per_xcd + loc;
        if (loc >= per_xcd || logical >= T) return false;
        const int64_t grp = logical / (G * p_tiles), rem = logical % (G * p_tiles);
        const int64_t gq = q_tiles - grp * G < G ? q_tiles - grp * G : G;
        q_tile = grp * G + rem % gq;
        p_tile = rem / gq;
        return true;
    };
    // which expert's weights a tile multiplies and which 128-row halves it stores.  A half of padding
    // rows (index < 0) or past the end stores nothing; two different experts need a second pass.
    auto classify = [&](int e0, int e1, int& e, int& mask, int& second_e) {
        second_e = -1;
        if (e0 < 0 && e1 < 0) { e = 0; mask = 0; }
        else if (e0 < 0) { e = e1; mask = 2; }
        else if (e1 < 0 || e0 == e1) { e = e0; mask = e1 < 0 ? 1 : 3; }
        else { e = e0; mask = 1; second_e = e1; }
    };
    auto has_tail = [&](int64_t qt) -> bool { return qt * 256 + 128 >= a.Qrows; };
    auto p_tail = [&](int64_t pt) -> bool { return pt * 256 + 128 >= a.Prows; };

    // work item = (tile, expert, halves to store); c_* current, n_* next; all wave-uniform
    int64_t cq = 0, cp = 0, nq = 0, np = 0, tn = 0;
    if (!tile_coords(0, cq, cp)) return;
    int c_mask, c_second = -1, n_mask = 0, n_second = -1;
    int64_t c_orow, n_orow = 0;                 // first output row of this wavefront's half
    const uint8_t *c_ptile, *c_ptile2, *c_qtile, *c_qtile2, *c_sq, *c_sp;
    // aligned tile qt of expert e
    auto setup = [&](int64_t qt, int64_t pt, int e, const uint8_t*& ptile, const uint8_t*& ptile2, const uint8_t*& qtile, const uint8_t*& qtile2,
                     const uint8_t*& sq, const uint8_t*& sp, int64_t& orow) {
        const bool tail = has_tail(qt);
        ptile = a.p + ((int64_t)e * a.Prows + pt * 256) * a.red;
        ptile2 = p_tail(pt) ? ptile : ptile + 128 * a.red;
        qtile = a.q + qt * 256 * a.red;
        qtile2 = tail ? qtile : qtile + 128 * a.red;     // a missing second half re-reads the first
        sq = a.sq8 + qt * 256 + ((wq && !tail) ? 128 : 0);
        sp = a.sp8 + ((int64_t)e * PB + pt * 2 + (p_tail(pt) ? 0 : wp)) * KB;
        orow = qt * 256 + wq * 128;
    };
    // listed item {block0, block1 or -1, expert}
    auto setup_item = [&](i32x4 it, int64_t pt, int& mask, const uint8_t*& ptile, const uint8_t*& ptile2, const uint8_t*& qtile, const uint8_t*& qtile2,
                          const uint8_t*& sq, const uint8_t*& sp, int64_t& orow) {
        const int64_t b0 = it.x, b1 = it.y < 0 ? it.x : it.y;
        mask = it.y < 0 ? 1 : 3;
        ptile = a.p + ((int64_t)it.z * a.Prows + pt * 256) * a.red;
        ptile2 = p_tail(pt) ? ptile : ptile + 128 * a.red;
        qtile = a.q + b0 * 128 * a.red;
        qtile2 = a.q + b1 * 128 * a.red;
        sq = a.sq8 + (wq ? b1 : b0) * 128;
        sp = a.sp8 + ((int64_t)it.z * PB + pt * 2 + (p_tail(pt) ? 0 : wp)) * KB;
        orow = (wq ? b1 : b0) * 128;
    };
    if (a.items) {
        const int32_t* ip = a.items + 4 + 4 * cq;
        setup_item((i32x4){__builtin_amdgcn_readfirstlane(ip[0]), __builtin_amdgcn_readfirstlane(ip[1]), __builtin_amdgcn_readfirstlane(ip[2]), 0}, cp, c_mask, c_ptile, c_ptile2, c_qtile, c_qtile2, c_sq, c_sp, c_orow);
    } else {
        int e0 = 0, e1 = has_tail(cq) ? -1 : 0, c_e;
        if (a.grouped) {
            e0 = __builtin_amdgcn_readfirstlane(a.m_indices[cq * 256]);
            if (!has_tail(cq)) e1 = __builtin_amdgcn_readfirstlane(a.m_indices[cq * 256 + 128]);
        }
        classify(e0, e1, c_e, c_mask, c_second);
        setup(cq, cp, c_e, c_ptile, c_ptile2, c_qtile, c_qtile2, c_sq, c_sp, c_orow);
    }
    int ld_e0 = 0, ld_e1 = 0;      // expert ids of the next tile's halves
    i32x4 ld_item = {0, 0, 0, 0};  // or its list entry
    const uint8_t *n_ptile = c_ptile, *n_ptile2 = c_ptile2, *n_qtile = c_qtile, *n_qtile2 = c_qtile2, *n_sq = c_sq, *n_sp = c_sp;
    bool n_valid = false;

    // copy c of a wavefront fills rows (4 c + wave) * 8 + (lane >> 3) of the stacked [P; Q] block.  P rows
    // are swizzled by e8_keyp(row), Q rows by e8_keyp(row >> 3): a Q fragment's 16 lanes read rows 8 apart
    const int crow = lane >> 3, cpos = lane & 7;
    const uint32_t c_off_p = (uint32_t)((wave * 8 + crow) * a.red + ((cpos ^ e8_keyp(wave * 8 + crow)) << 4));
    uint32_t c_off_q[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) c_off_q[v] = (uint32_t)((wave * 8 + crow) * a.red + ((cpos ^ e8_keyp(4 * v + wave)) << 4));
    const int64_t copy_step = 32 * a.red;
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    int fp_ofs[2], fq_ofs[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int prow = wp * 128 + li;
        fp_ofs[h] = prow * 128 + (((2 * kg + h) ^ e8_keyp(prow)) << 4);
        fq_ofs[h] = Q_OFS + (wq * 128 + li * 8) * 128 + (((2 * kg + h) ^ e8_keyp(li)) << 4);
    }
    const uint32_t s_off = (uint32_t)(li * 8);
    uint32_t zero_off = 0;
    asm volatile("" : "+v"(zero_off));     // a VGPR holding 0 (the address form needs one)

#define E8_COPY(c_, pt_, pt2_, qt_, qt2_, slot_)                                                       \
    do {                                                                                               \
        if ((c_) < 4) e8_dma16(c_off_p, (pt_) + (c_) * copy_step, lds_base + (slot_) * SLOT + ((c_) * 4 + wave) * 1024); \
        else if ((c_) < 8) e8_dma16(c_off_p, (pt2_) + ((c_) - 4) * copy_step, lds_base + (slot_) * SLOT + ((c_) * 4 + wave) * 1024); \
        else if ((c_) < 12) e8_dma16(c_off_q[(c_) & 3], (qt_) + ((c_) - 8) * copy_step, lds_base + (slot_) * SLOT + Q_OFS + (((c_) - 8) * 4 + wave) * 1024); \
        else e8_dma16(c_off_q[(c_) & 3], (qt2_) + ((c_) - 12) * copy_step, lds_base + (slot_) * SLOT + Q_OFS + (((c_) - 8) * 4 + wave) * 1024); \
    } while (0)
    // the scale bytes of a block, straight into the VGPRs the MFMAs take them from: eight Q exponents per
    // lane and the P block's exponent (every lane the same byte).  Vector loads on purpose: the value of
    // an asynchronous load may not be touched before its wait, and the compiler, which cannot know that,
    // is free to copy or spill a scalar register at any point, but leaves these VGPRs alone.
#define E8_LOAD_S(sq_, sp_)                                                                            \
    do {                                                                                               \
        asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(sq_nxt) : "v"(s_off), "s"(sq_) : "memory"); \
        asm volatile("global_load_ubyte %0, %1, %2" : "=v"(sp_nxt) : "v"(zero_off), "s"(sp_) : "memory"); \
    } while (0)

    i32x8 pf[2][8], qf[4];
    u32x2 sq_nxt = {0, 0};
    uint32_t sp_nxt = 0;

    e8_static_for<64>([&](auto ix) { e8_acc_zero4<decltype(ix)::value>(); });
    {
        E8_LOAD_S(c_sq, c_sp);
#pragma unroll
        for (int c = 0; c < 16; ++c) E8_COPY(c, c_ptile, c_ptile2, c_qtile, c_qtile2, 0);
#pragma unroll
        for (int c = 0; c < 16; ++c)
            if (c * CSTEP < 64 - BAR) E8_COPY(c, c_ptile + 128, c_ptile2 + 128, c_qtile + 128, c_qtile2 + 128, 1);
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : "+v"(sq_nxt), "+v"(sp_nxt) : : "memory");
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[0][i] = e8_frag(lds + fp_ofs[0] + i * 2048, lds + fp_ofs[1] + i * 2048);
#pragma unroll
        for (int j = 0; j < 3; ++j) qf[j] = e8_frag(lds + fq_ofs[0] + j * 128, lds + fq_ofs[1] + j * 128);
    }
    int64_t kb = 0;

    // one K block; PAR = parity of the block in this workgroup's stream of blocks = its LDS slot and
    // the half of pf[] that holds its P fragments.  Returns true after the last work item.
    auto blk = [&](auto par_c) -> bool {
        constexpr int PAR = decltype(par_c)::value;
        if (kb == 0) {
            // the item after this one: the same tile again for its second expert, or the next tile, whose
            // list entry / expert ids are fetched here (scalar loads, waited for on the spot: once per item)
            n_valid = c_second >= 0 ? true : tile_coords(tn + 1, nq, np);
            if (c_second < 0 && n_valid) {
                if (a.items) {
                    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ld_item) : "s"(a.items + 4 + 4 * nq) : "memory");
                } else if (a.grouped) {
                    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ld_e0) : "s"(a.m_indices + nq * 256) : "memory");
                    if (!has_tail(nq))
                        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ld_e1) : "s"(a.m_indices + nq * 256 + 128) : "memory");
                }
            }
        }
        if (kb == 1) {
            if (c_second >= 0) {
                nq = cq; np = cp; n_mask = 2; n_second = -1;
                setup(nq, np, c_second, n_ptile, n_ptile2, n_qtile, n_qtile2, n_sq, n_sp, n_orow);
            } else if (n_valid && a.items) {
                setup_item(ld_item, np, n_mask, n_ptile, n_ptile2, n_qtile, n_qtile2, n_sq, n_sp, n_orow);
            } else if (n_valid) {
                const int e0 = a.grouped ? ld_e0 : 0, e1 = has_tail(nq) ? -1 : (a.grouped ? ld_e1 : 0);
                int ne;
                classify(e0, e1, ne, n_mask, n_second);
                setup(nq, np, ne, n_ptile, n_ptile2, n_qtile, n_qtile2, n_sq, n_sp, n_orow);
            } else {
                // past the last item the copies and scale loads re-read this item's first blocks
                n_ptile = c_ptile; n_ptile2 = c_ptile2; n_qtile = c_qtile; n_qtile2 = c_qtile2; n_sq = c_sq; n_sp = c_sp;
            }
        }
        const u32x2 sq_cur = sq_nxt;
        const uint32_t sp_cur = sp_nxt;
        const bool in1 = kb + 1 < KB, in2 = kb + 2 < KB;
        const int64_t o1 = (in1 ? kb + 1 : kb + 1 - KB) * 128, o2 = (in2 ? kb + 2 : kb + 2 - KB) * 128;
        const uint8_t* s_sq = in1 ? c_sq + (kb + 1) * a.ldsq : n_sq;
        const uint8_t* s_sp = in1 ? c_sp + (kb + 1) : n_sp;
        const uint8_t* cp1_p = (in1 ? c_ptile : n_ptile) + o1;
        const uint8_t* cp1_p2 = (in1 ? c_ptile2 : n_ptile2) + o1;
        const uint8_t* cp1_q = (in1 ? c_qtile : n_qtile) + o1;
        const uint8_t* cp1_q2 = (in1 ? c_qtile2 : n_qtile2) + o1;
        const uint8_t* cp2_p = (in2 ? c_ptile : n_ptile) + o2;
        const uint8_t* cp2_p2 = (in2 ? c_ptile2 : n_ptile2) + o2;
        const uint8_t* cp2_q = (in2 ? c_qtile : n_qtile) + o2;
        const uint8_t* cp2_q2 = (in2 ? c_qtile2 : n_qtile2) + o2;
        E8_LOAD_S(s_sq, s_sp);
        const uint8_t* pbase = lds + PAR * SLOT;
        const uint8_t* nbase = lds + (PAR ^ 1) * SLOT;
        __builtin_amdgcn_sched_barrier(0);
        e8_static_for<64>([&](auto mc) {
            constexpr int m = decltype(mc)::value;
            constexpr int j = m >> 3, i = m & 7;
            if constexpr (m == BAR) {
                // every fragment read of this block has been issued (the last at MFMA 32) and the next
                // block's copies were all issued by MFMA 12: once both have returned, meet the others
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : "+v"(sq_nxt), "+v"(sp_nxt) : : "memory");
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (i == 0 && j + 3 < 8) {
                qf[(j + 3) % 4] = e8_frag(pbase + fq_ofs[0] + (j + 3) * 128, pbase + fq_ofs[1] + (j + 3) * 128);
                __builtin_amdgcn_sched_barrier(0);
            }
            e8_mfma<8 * i + j, (j & 3)>(pf[PAR][i], qf[j % 4], (int)sp_cur, (int)(j < 4 ? sq_cur.x : sq_cur.y));
            __builtin_amdgcn_sched_barrier(0);
            // copies: the block after next into the slot this block has just left, continued in the
            // next block before its barrier
            if constexpr (m >= BAR && (m - BAR) % CSTEP == 0 && (m - BAR) / CSTEP < 16) {
                E8_COPY((m - BAR) / CSTEP, cp2_p, cp2_p2, cp2_q, cp2_q2, PAR);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (m < BAR && (m + 64 - BAR) % CSTEP == 0 && (m + 64 - BAR) / CSTEP < 16) {
                E8_COPY((m + 64 - BAR) / CSTEP, cp1_p, cp1_p2, cp1_q, cp1_q2, PAR ^ 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the next block's P fragments and first Q fragments, from the slot just declared landed
            if constexpr (m >= 48 && m < 56) {
                pf[PAR ^ 1][m - 48] = e8_frag(nbase + fp_ofs[0] + (m - 48) * 2048, nbase + fp_ofs[1] + (m - 48) * 2048);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (m == 57 || m == 59 || m == 61) {
                constexpr int jj = (m - 57) / 2;
                qf[jj] = e8_frag(nbase + fq_ofs[0] + jj * 128, nbase + fq_ofs[1] + jj * 128);
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        ++kb;
        if (kb < KB) return false;

        // ---- item finished: the wavefronts whose half is stored write it out through a private LDS
        // slice, one Q fragment (16 rows x 128 columns) at a time, as whole 256-byte rows
        if (((c_mask >> wq) & 1) && !(wp && p_tail(cp))) {
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written back before they are read
            uint8_t* ep = lds + EP_OFS + wave * (16 * EP_LD);
            const int er = lane >> 4, ec = lane & 15;
            const uint32_t vo = (uint32_t)((er * 8 * a.ldo + ec * 8) * 2);
            const uint32_t vo_step = (uint32_t)(32 * a.ldo * 2);
            uint8_t* tile_out = reinterpret_cast<uint8_t*>(a.out) + (c_orow * a.ldo + cp * 256 + wp * 128) * 2;
            e8_static_for<8>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                e8_static_for<8>([&](auto icn) {
                    constexpr int i = decltype(icn)::value;
                    constexpr int R = 4 * (8 * i + j);
                    uint2 o;
                    o.x = pack_bf16(e8_acc_get<R>(), e8_acc_get<R + 1>());
                    o.y = pack_bf16(e8_acc_get<R + 2>(), e8_acc_get<R + 3>());
                    *reinterpret_cast<uint2*>(ep + li * EP_LD + (i * 16 + 4 * kg) * 2) = o;
                });
                uint8_t* row_out = tile_out + j * a.ldo * 2;
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rl = er + 4 * it;                        // staged row = li of the producer
                    const uint4 v = *reinterpret_cast<const uint4*>(ep + rl * EP_LD + ec * 16);
                    st16(row_out + vo + it * vo_step, v);
                }
            });
        }
        if (!n_valid) return true;
        e8_static_for<64>([&](auto ix) { e8_acc_zero4<decltype(ix)::value>(); });
        if (c_second < 0) ++tn;
        cq = nq; cp = np; c_mask = n_mask; c_second = n_second; c_orow = n_orow;
        c_ptile = n_ptile; c_ptile2 = n_ptile2; c_qtile = n_qtile; c_qtile2 = n_qtile2; c_sq = n_sq; c_sp = n_sp;
        kb = 0;
        return false;
    };
    for (;;) {
        if (blk(std::integral_constant<int, 0>{})) break;
        if (blk(std::integral_constant<int, 1>{})) break;
    }
    __builtin_amdgcn_s_waitcnt(0);   // the copies issued past the end must land before the LDS is released
#undef E8_COPY
#undef E8_LOAD_S
}

// Pairs the 128-row blocks of every expert of a contiguous grouped layout into 256-row work items.
// One workgroup of 1024 threads, each walking a contiguous run of blocks; two scans over the threads:
// the parity of a block inside its expert's segment (a composition of {reset, flip} functions), then
// the number of items opened before it (an item opens at every even block of a segment).
// items = {n, number of 128-row blocks, 0, 0} followed by {block0, block1 or -1, expert, 0} per item.
__global__ __launch_bounds__(1024) void k_e8_build_items(const int32_t* __restrict__ m_indices, int64_t NB, int32_t* __restrict__ items) {
    constexpr int CACHE = 8192;                 // expert ids of the first blocks, read from memory once
    __shared__ int s_scan[2][1024];
    __shared__ int s_e[CACHE];
    const int tid = threadIdx.x;
    for (int64_t b = tid; b < NB && b < CACHE; b += 1024) s_e[b] = m_indices[b * 128];
    __syncthreads();
    const int64_t chunk = (NB + 1023) / 1024;
    const int64_t lo = tid * chunk < NB ? tid * chunk : NB, hi = lo + chunk < NB ? lo + chunk : NB;
    auto expert = [&](int64_t b) -> int { return (b < 0 || b >= NB) ? -2 : (b < CACHE ? s_e[b] : m_indices[b * 128]); };
    // function codes: bit 1 = constant, bit 0 = its value (constant) or flip (otherwise); g after f:
    auto then = [](int f, int g) -> int { return (g & 2) ? g : (f ^ (g & 1)); };
    auto step_fn = [&](int prev_e, int e) -> int { return e < 0 ? 3 : (e != prev_e ? 2 : 1); };
    int f = 0, pe = expert(lo - 1);
    for (int64_t b = lo; b < hi; ++b) { const int e = expert(b); f = then(f, step_fn(pe, e)); pe = e; }
    // inclusive scan of the function composition (Hillis-Steele)
    int cur = 0;
    s_scan[0][tid] = f;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int v = tid >= d ? then(s_scan[cur][tid - d], s_scan[cur][tid]) : s_scan[cur][tid];
        s_scan[cur ^ 1][tid] = v;
        cur ^= 1;
        __syncthreads();
    }
    const int f_in = tid ? s_scan[cur][tid - 1] : 0;
    const int par = (f_in & 2) ? (f_in & 1) : (1 ^ (f_in & 1));     // parity of the block before `lo` (1 = none open)
    __syncthreads();
    // items opened in this run of blocks
    int opened = 0, p = par;
    pe = expert(lo - 1);
    for (int64_t b = lo; b < hi; ++b) {
        const int e = expert(b);
        p = e < 0 ? 1 : (e != pe ? 0 : p ^ 1);
        opened += (e >= 0 && p == 0);
        pe = e;
    }
    cur = 0;
    s_scan[0][tid] = opened;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int v = tid >= d ? s_scan[cur][tid - d] + s_scan[cur][tid] : s_scan[cur][tid];
        s_scan[cur ^ 1][tid] = v;
        cur ^= 1;
        __syncthreads();
    }
    int t = (tid ? s_scan[cur][tid - 1] : 0) - 1;     // index of the item open before `lo`
    if (tid == 1023) { items[0] = s_scan[cur][1023]; items[1] = (int32_t)NB; items[2] = 0; items[3] = 0; }
    p = par;
    pe = expert(lo - 1);
    for (int64_t b = lo; b < hi; ++b) {
        const int e = expert(b);
        p = e < 0 ? 1 : (e != pe ? 0 : p ^ 1);
        if (e >= 0) {
            if (p == 0) {
                ++t;
                items[4 + 4 * t] = (int32_t)b;
                items[4 + 4 * t + 2] = e;
                items[4 + 4 * t + 3] = 0;
                if (expert(b + 1) != e) items[4 + 4 * t + 1] = -1;
            } else {
                items[4 + 4 * t + 1] = (int32_t)b;
            }
        }
        pe = e;
    }
}

// fp32 scales that are powers of two -> exponent bytes; *bad counts the scales that are not
__global__ void k_scales_to_ue8m0(const float* __restrict__ s, int64_t n, uint8_t* __restrict__ out, int* bad) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint32_t b = f2u(s[i]);
    out[i] = (uint8_t)(b >> 23);
    if (bad && ((b & 0x807FFFFFu) != 0 || (b >> 23) == 0xFF || (b >> 23) == 0)) atomicAdd(bad, 1);
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

static constexpr int E8_LDS_BYTES = 131072 + 4 * 16 * 272;

static int launch_e8(const E8Args& a, int64_t max_q_tiles, int cus, hipStream_t st, const char* where) {
    // the LDS opt-in, once per device (a bit per device; a race sets the same attribute twice)
    static std::atomic<uint64_t> attr_done{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
    const uint64_t bit = 1ull << (dev & 63);
    if (!(attr_done.load(std::memory_order_acquire) & bit)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_e8), hipFuncAttributeMaxDynamicSharedMemorySize, E8_LDS_BYTES);
        if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
        attr_done.fetch_or(bit, std::memory_order_release);
    }
    const int64_t T = ((a.Prows + 255) / 256) * max_q_tiles, per_xcd = (T + 7) / 8;
    int64_t w = cus / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    hipLaunchKernelGGL(k_gemm_e8, dim3((unsigned)(8 * w)), dim3(256), E8_LDS_BYTES, st, a);
    return pf8_check_launch(where);
}

static int check_e8_shapes(const char* where, int64_t M, int64_t N, int64_t K, int64_t ldsa) {
    if (M % 128 != 0) return pf8_fail(PF8_EINVAL, where, "M must be a multiple of 128");
    if (N % 128 != 0 || (N != 0 && N < 256)) return pf8_fail(PF8_EINVAL, where, "N must be a multiple of 128 and at least 256");
    if (K % 128 != 0 || K < 384) return pf8_fail(PF8_EINVAL, where, "K must be a multiple of 128 and at least 384");
    if (ldsa < M || ldsa % 8 != 0) return pf8_fail(PF8_EINVAL, where, "ldsa must be >= M and a multiple of 8");
    if (K > (1ll << 24)) return pf8_fail(PF8_EINVAL, where, "K too large");
    return PF8_OK;
}

extern "C" int pf8_gemm_nt_ue8m0(const uint8_t* a, const uint8_t* sa, int64_t ldsa, const uint8_t* b, const uint8_t* sb, int64_t M,
                                 int64_t N, int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative shape");
    int rc = check_e8_shapes(__func__, M, N, K, ldsa);
    if (rc) return rc;
    if (M == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && out, "null pointer");
    PF8_REQUIRE(ldo >= N && ldo % 8 == 0, "ldo must be >= N and a multiple of 8");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && PF8_ALIGNED16(out) && (reinterpret_cast<uintptr_t>(sa) & 7u) == 0,
                "a, b, out must be 16-byte aligned and sa 8-byte aligned");
    PF8_REQUIRE(ldo * 2 * 128 <= 0x7FFFFFFFll, "ldo too large");
    E8Args g = {};
    g.p = b; g.q = a; g.sp8 = sb; g.sq8 = sa; g.out = out;
    g.Prows = N; g.Qrows = M; g.red = K; g.ldo = ldo; g.ldsq = ldsa; g.grouped = 0;
    return launch_e8(g, (M + 255) / 256, pf8_effective_cus(), (hipStream_t)stream, __func__);
}

extern "C" int pf8_grouped_gemm_nt_contiguous_ue8m0(const uint8_t* a, const uint8_t* sa, int64_t ldsa, const uint8_t* b,
                                                    const uint8_t* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                                    const int32_t* m_indices, const int32_t* items, uint16_t* out,
                                                    pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Mtot >= 0 && N >= 0 && K >= 0, "negative shape");
    int rc = check_e8_shapes(__func__, Mtot, N, K, ldsa);
    if (rc) return rc;
    if (Mtot == 0 || N == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && out && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && PF8_ALIGNED16(out) && (reinterpret_cast<uintptr_t>(sa) & 7u) == 0,
                "a, b, out must be 16-byte aligned and sa 8-byte aligned");
    PF8_REQUIRE(N * 2 * 128 <= 0x7FFFFFFFll, "N too large");
    E8Args g = {};
    g.p = b; g.q = a; g.sp8 = sb; g.sq8 = sa; g.out = out;
    g.Prows = N; g.Qrows = Mtot; g.red = K; g.ldo = N; g.ldsq = ldsa; g.grouped = 1; g.m_indices = m_indices;
    // the compute-unit budget is read once: both launches size their grids by it and both kernels weigh
    // the expert load with it, so a pf8_set_num_cus from another thread cannot make them disagree
    const int cus = pf8_effective_cus();
    if (items) {
        // both kernels are launched; each decides on entry, from the list's header, whether this expert
        // load is its own, and the other returns at once
        PF8_REQUIRE((reinterpret_cast<uintptr_t>(items) & 15u) == 0, "items must be 16-byte aligned");
        g.items = items;
        g.cus = cus;
        g.force = N % 256 != 0;      // the 128x256-tile kernel takes whole 256-column tiles only
        rc = launch_e8(g, Mtot / 128, cus, (hipStream_t)stream, __func__);
        if (rc || g.force) return rc;
        return pf8_launch_deep_ue8m0(b, a, sb, sa, ldsa, out, N, Mtot, K, E, m_indices, items, cus, (hipStream_t)stream, __func__);
    }
    return launch_e8(g, (Mtot + 255) / 256, cus, (hipStream_t)stream, __func__);
}

// ---------------------------------------------------------------------------------------------
// The grouped UE8M0 GEMM for callers that cannot allocate: the work-item list lives in a file-scope
// device array instead of a caller buffer.  Every GPU holds its own copy of the array at its own
// address; the name `scratch` is only a host-side handle for hipGetSymbolAddress, which is asked once
// per device (with that device current) and whose answer is what every launch passes on.
// ---------------------------------------------------------------------------------------------
static constexpr int64_t NOALLOC_MAX_BLOCKS = 8192;                 // 128-row blocks: 1,048,576 rows
static __device__ __align__(256) int32_t scratch[4 + 4 * NOALLOC_MAX_BLOCKS];    // 131,088 bytes per GPU, held until the process ends

static int noalloc_scratch(const char* where, int32_t** out) {
    static std::atomic<int32_t*> ptrs[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return pf8_fail(PF8_EINVAL, where, "device ordinal beyond 63");
    int32_t* p = ptrs[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !sym) return pf8_fail(PF8_ELAUNCH, where, e != hipSuccess ? hipGetErrorString(e) : "hipGetSymbolAddress returned a null address");
        p = static_cast<int32_t*>(sym);
        ptrs[dev].store(p, std::memory_order_release);     // two threads racing here store the same address
    }
    *out = p;
    return PF8_OK;
}

extern "C" int pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc(const uint8_t* a, const uint8_t* sa, int64_t ldsa, const uint8_t* b,
                                                            const uint8_t* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                                            const int32_t* m_indices, uint16_t* out, pf8_stream_t stream) {
    PF8_REQUIRE(Mtot >= 0 && Mtot % 128 == 0, "Mtot must be a non-negative multiple of 128");
    PF8_REQUIRE(Mtot / 128 <= NOALLOC_MAX_BLOCKS, "Mtot beyond the 1,048,576 rows the built-in work-item list holds: build a list with pf8_grouped_items_build and call pf8_grouped_gemm_nt_contiguous_ue8m0");
    if (Mtot == 0 || N == 0 || E == 0) return pf8_grouped_gemm_nt_contiguous_ue8m0(a, sa, ldsa, b, sb, E, Mtot, N, K, m_indices, nullptr, out, stream);
    PF8_REQUIRE(m_indices, "null pointer");
    int32_t* items = nullptr;
    int rc = noalloc_scratch(__func__, &items);
    if (rc) return rc;
    // the list builder writes the header and every field of every item it counts, and the GEMM reads
    // no further than that count: nothing in the array has to start at zero, stale items of an earlier,
    // longer call are never looked at
    hipLaunchKernelGGL(k_e8_build_items, dim3(1), dim3(1024), 0, (hipStream_t)stream, m_indices, Mtot / 128, items);
    rc = pf8_check_launch(__func__);
    if (rc) return rc;
    return pf8_grouped_gemm_nt_contiguous_ue8m0(a, sa, ldsa, b, sb, E, Mtot, N, K, m_indices, items, out, stream);
}

extern "C" int pf8_grouped_items_build(const int32_t* m_indices, int64_t Mtot, int32_t* items, pf8_stream_t stream) {
    PF8_REQUIRE(Mtot >= 0 && Mtot % 128 == 0, "Mtot must be a non-negative multiple of 128");
    PF8_REQUIRE(items && (reinterpret_cast<uintptr_t>(items) & 15u) == 0, "items must be a 16-byte aligned buffer");
    PF8_REQUIRE(Mtot == 0 || m_indices, "null pointer");
    PF8_REQUIRE(Mtot / 128 <= 0x3FFFFFFFll, "too many rows");
    hipLaunchKernelGGL(k_e8_build_items, dim3(1), dim3(1024), 0, (hipStream_t)stream, m_indices, Mtot / 128, items);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_scales_to_ue8m0(const float* s, int64_t n, uint8_t* out, int* not_pow2, pf8_stream_t stream) {
    PF8_REQUIRE(n >= 0, "negative length");
    if (n == 0) return PF8_OK;
    PF8_REQUIRE(s && out, "null pointer");
    PF8_REQUIRE((n + 255) / 256 <= 0x7FFFFFFFll, "too many scales");
    hipLaunchKernelGGL(k_scales_to_ue8m0, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, s, n, out, not_pow2);
    return pf8_check_launch(__func__);
}
