// pf8_wgrad_e8.hip -- the grouped weight gradient of the experts with a long reduction axis, on the 256x256
// accumulator tile of the UE8M0 forward kernel (pf8_gemm_e8.hip): dW[e] [Q rows, P rows] (+)= Q_e . P_e^T with BOTH
// operands 1x128-scaled along the reduction axis by powers of two, fp32 output.
//
// The 128x128-tile kernel (k_gemm_wgrad) runs two workgroups per compute unit and reads 64 KB of fragments per 64 MFMAs
// and wavefront pair; it is the right shape for the many experts whose reduction is a handful of blocks (their time is
// the read-modify-write of the gradient), but an expert with dozens of blocks is bound by that LDS traffic.  Here one
// persistent workgroup per compute unit holds a 256x256 tile in the AGPR file (half the fragment bytes per MFMA), the
// copy ring runs on across tile boundaries, and both operands' exponents go into the block-scaled MFMA per lane:
//   * P fragment i of a wavefront is rows 16 i + l of its 128 (l = lane % 16): eight 4-byte scale loads per block;
//     Q fragment j is rows 8 l + j: the eight scales are two 16-byte loads.  The exponent fields are packed four to a
//     register and op_sel picks the byte per MFMA on both sides.
//   * Work items are (expert, tile); the experts differ in length, so tiles are handed out dynamically: every XCD owns
//     the same slice of every expert's tile grid (its L2 then holds a few operand panels of one expert at a time) and
//     its workgroups draw tickets from a counter of their XCD.  The ticket for the next item is drawn three blocks
//     ahead of where its first copies are issued, so its latency is never waited for.
//   * The counters live in a file-scope device array of 64 slots; a launch takes the next slot and the last workgroup
//     to finish clears it, so launches that overlap on one device (different streams) never share counters.
//   * Epilogue: the accumulators go through a wavefront-private 4 KB LDS slice, 16 rows x 64 columns at a time, and
//     are added to the old gradient rows, whose loads run four passes ahead.
// Results are bit-identical to k_gemm_wgrad<true>: the same instruction accumulates the same blocks in the same order.
#include <atomic>
#include <type_traits>

#include "pf8_device.h"
#include "pf8_e8_common.h"
#include "pf8_host.h"

namespace pf8 {

struct WgE8Args {
    const uint8_t* p;      // packed per expert: [Prows, M_e] at Prows * (rows before e)
    const uint8_t* q;      // [Qrows, M_e] at Qrows * (rows before e)
    const float* sp;       // [blocks, Prows], an expert's blocks start at (rows before e) / 128
    const float* sq;       // [blocks, Qrows]
    float* out;            // [E, Qrows, ldo]
    int64_t Prows, Qrows, ldo;
    int accumulate;
    int n_items;
    int gq;                // q-tiles per group of the tile order
    int32_t* tickets;      // [0..7] per-XCD ticket counters, [8] workgroups finished; all zero at launch
    int32_t item_t0[kWgE8MaxItems];   // first 128-row block of the item's expert along the reduction axis
    int32_t item_kb[kWgE8MaxItems];   // its number of blocks (>= 4)
    int32_t item_e[kWgE8MaxItems];    // the expert
};

// acc[IDX] += (2^(sa.byte[OA]-127) A) (2^(sb.byte[OB]-127) B): A = P fragment, B = Q fragment
template <int IDX, int OA, int OB>
__device__ __forceinline__ void wg8_mfma(const i32x8& a, const i32x8& b, uint32_t sa, uint32_t sb) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%4:%5], %0, %1, a[%4:%5], %2, %3 op_sel:[%6,%7,0] op_sel_hi:[%8,%9,0]"
                 : : "v"(a), "v"(b), "v"(sa), "v"(sb), "n"(4 * IDX), "n"(4 * IDX + 3), "n"(OA & 1), "n"(OB & 1), "n"(OA >> 1), "n"(OB >> 1));
}

// exponent fields of four positive fp32 scales, packed low byte first
__device__ __forceinline__ uint32_t wg8_pack_exp(float a, float b, float c, float d) {
    return (f2u(a) >> 23) | ((f2u(b) >> 23) << 8) | ((f2u(c) >> 23) << 16) | ((f2u(d) >> 23) << 24);
}

// ACC: add to the old gradient (a compile-time switch: a branch around the loads of the old rows would make the compiler
// wait for all of them at the first use instead of counting them)
template <bool ACC>
__global__ __launch_bounds__(256, 1) void k_wgrad_e8(const WgE8Args a) {
    constexpr int SLOT = 65536, Q_OFS = 32768, EP_OFS = 131072, TKT_OFS = EP_OFS + 4 * 4096;
    constexpr int BAR = 44, CSTEP = 2;     // barrier position; MFMAs between two copies
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    asm volatile("" ::: "a255");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = wave >> 1, wp = wave & 1;
    const int li = lane & 15, kg = lane >> 4;

    // every workgroup leaves through here: the last one clears the slot for the launch that takes it next
    auto finish = [&]() {
        if (tid == 0) {
            const int done = __hip_atomic_fetch_add(a.tickets + 8, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (done == (int)gridDim.x - 1) {
#pragma unroll
                for (int i = 0; i < 9; ++i) __hip_atomic_store(a.tickets + i, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    };

    // Prows / Qrows = 256 t + 128: the last tile along that axis has one 128-row half; its second half re-reads the
    // first and the wavefronts that own it store nothing
    const int64_t p_tiles = (a.Prows + 255) / 256, q_tiles = (a.Qrows + 255) / 256;
    const int64_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, W = gridDim.x >> 3;
    // this XCD's slice of every item's tile grid: an eighth of its tiles in the order "groups of gq q-tiles x all p-tiles,
    // q fastest", so a slice is about gq q-tiles x T / (8 gq) p-tiles and every XCD gets the same number of tiles (the
    // host picks the gq that makes the slice squarest: fewest operand panels per tile).  Its queue: the slices of all
    // items, longest reduction first.
    const int64_t T_item = p_tiles * q_tiles;
    const int64_t lo_x = xcd * T_item / 8, n_x = (xcd + 1) * T_item / 8 - lo_x;
    const int64_t total_x = n_x * a.n_items;
    if (slot >= total_x) { finish(); return; }
    int32_t* const my_counter = a.tickets + xcd;

    auto p_tail = [&](int64_t pt) -> bool { return pt * 256 + 128 >= a.Prows; };
    auto q_tail = [&](int64_t qt) -> bool { return qt * 256 + 128 >= a.Qrows; };

    // work item = (expert, tile); c_* current, n_* next; all wave-uniform
    struct Item {
        const uint8_t *ptile, *ptile2, *qtile, *qtile2;
        const float *sq, *sp;      // block 0, first row of this wavefront's half
        float* out;                // first output row / column of this wavefront's quarter
        int32_t red, kb;           // reduction length in bytes and in blocks
        int32_t store;             // this wavefront stores its quarter
    };
    auto setup = [&](int64_t u, Item& it) {
        // (32-bit divisions run on the vector unit: their wave-uniform results are moved to scalar registers by hand)
        const uint32_t item = (uint32_t)__builtin_amdgcn_readfirstlane((int)((uint32_t)u / (uint32_t)n_x));
        const uint32_t v = (uint32_t)lo_x + ((uint32_t)u - item * (uint32_t)n_x);
        const uint32_t per_group = (uint32_t)(a.gq * p_tiles);
        const uint32_t grp = (uint32_t)__builtin_amdgcn_readfirstlane((int)(v / per_group)), r = v - grp * per_group;
        const uint32_t left = (uint32_t)q_tiles - grp * (uint32_t)a.gq, gsize = left < (uint32_t)a.gq ? left : (uint32_t)a.gq;
        const uint32_t r_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(r / gsize)), r_lo = r - r_hi * gsize;
        const int64_t qt = (int64_t)grp * a.gq + r_lo, pt = r_hi;
        const int64_t t0 = a.item_t0[item], kbn = a.item_kb[item], e = a.item_e[item];
        const int64_t red = kbn * 128;
        const bool pt_tail = p_tail(pt), qt_tail = q_tail(qt);
        it.red = (int32_t)red;
        it.kb = (int32_t)kbn;
        it.ptile = a.p + a.Prows * 128 * t0 + pt * 256 * red;
        it.ptile2 = pt_tail ? it.ptile : it.ptile + 128 * red;
        it.qtile = a.q + a.Qrows * 128 * t0 + qt * 256 * red;
        it.qtile2 = qt_tail ? it.qtile : it.qtile + 128 * red;
        it.sq = a.sq + t0 * a.Qrows + qt * 256 + ((wq && !qt_tail) ? 128 : 0);
        it.sp = a.sp + t0 * a.Prows + pt * 256 + ((wp && !pt_tail) ? 128 : 0);
        it.out = a.out + (e * a.Qrows + qt * 256 + wq * 128) * a.ldo + pt * 256 + wp * 128;
        it.store = !(wq && qt_tail) && !(wp && pt_tail);
    };
    Item c, n;
    setup(slot, c);
    n = c;
    bool n_valid = false;

    // copy k of a wavefront fills rows (4 k + wave) * 8 + (lane >> 3) of the stacked [P; Q] block.  P rows
    // are swizzled by e8_keyp(row), Q rows by e8_keyp(row >> 3): a Q fragment's 16 lanes read rows 8 apart
    const int crow = lane >> 3, cpos = lane & 7;
    const uint32_t c_row = (uint32_t)(wave * 8 + crow);
    const uint32_t c_ch_p = (uint32_t)((cpos ^ e8_keyp(wave * 8 + crow)) << 4);
    uint32_t c_ch_q[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) c_ch_q[v] = (uint32_t)((cpos ^ e8_keyp(4 * v + wave)) << 4);
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    int fp_ofs[2], fq_ofs[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int prow = wp * 128 + li;
        fp_ofs[h] = prow * 128 + (((2 * kg + h) ^ e8_keyp(prow)) << 4);
        fq_ofs[h] = Q_OFS + (wq * 128 + li * 8) * 128 + (((2 * kg + h) ^ e8_keyp(li)) << 4);
    }
    const uint32_t sq_off = (uint32_t)(li * 32), sp_off = (uint32_t)(li * 4);
    uint32_t zero_off = 0;
    asm volatile("" : "+v"(zero_off));     // a VGPR holding 0 (the address form needs one)

    // red_: reduction length (= row stride in bytes) of the item the block belongs to
#define WG8_COPY(k_, red_, pt_, pt2_, qt_, qt2_, slot_)                                                \
    do {                                                                                               \
        const int64_t step_ = 32 * (int64_t)(red_);                                                    \
        if ((k_) < 4) e8_dma16(c_row * (uint32_t)(red_) + c_ch_p, (pt_) + (k_) * step_, lds_base + (slot_) * SLOT + ((k_) * 4 + wave) * 1024); \
        else if ((k_) < 8) e8_dma16(c_row * (uint32_t)(red_) + c_ch_p, (pt2_) + ((k_) - 4) * step_, lds_base + (slot_) * SLOT + ((k_) * 4 + wave) * 1024); \
        else if ((k_) < 12) e8_dma16(c_row * (uint32_t)(red_) + c_ch_q[(k_) & 3], (qt_) + ((k_) - 8) * step_, lds_base + (slot_) * SLOT + Q_OFS + (((k_) - 8) * 4 + wave) * 1024); \
        else e8_dma16(c_row * (uint32_t)(red_) + c_ch_q[(k_) & 3], (qt2_) + ((k_) - 12) * step_, lds_base + (slot_) * SLOT + Q_OFS + (((k_) - 8) * 4 + wave) * 1024); \
    } while (0)
    // the scales of a block, straight into VGPRs: eight Q scales per lane (rows 8 l .. 8 l + 7) and the eight P scales
    // of rows l, l + 16, ...  Asynchronous: not touched before the wait in front of the block's barrier.
#define WG8_LOAD_S(sq_, sp_)                                                                           \
    do {                                                                                               \
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sq_r0) : "v"(sq_off), "s"(sq_) : "memory"); \
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=v"(sq_r1) : "v"(sq_off), "s"(sq_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2" : "=v"(sp_r[0]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:64" : "=v"(sp_r[1]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:128" : "=v"(sp_r[2]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:192" : "=v"(sp_r[3]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:256" : "=v"(sp_r[4]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:320" : "=v"(sp_r[5]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:384" : "=v"(sp_r[6]) : "v"(sp_off), "s"(sp_) : "memory"); \
        asm volatile("global_load_dword %0, %1, %2 offset:448" : "=v"(sp_r[7]) : "v"(sp_off), "s"(sp_) : "memory"); \
    } while (0)
#define WG8_WAIT_ALL()                                                                                 \
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)"                                                       \
                 : "+v"(sq_r0), "+v"(sq_r1), "+v"(sp_r[0]), "+v"(sp_r[1]), "+v"(sp_r[2]), "+v"(sp_r[3]), "+v"(sp_r[4]), "+v"(sp_r[5]), \
                   "+v"(sp_r[6]), "+v"(sp_r[7]), "+v"(tkt) : : "memory")

    i32x8 pf[2][8], qf[4];
    f32x4 sq_r0 = {1.f, 1.f, 1.f, 1.f}, sq_r1 = {1.f, 1.f, 1.f, 1.f};
    float sp_r[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
    uint32_t tkt = 0;                      // wave 0, lane 0: the ticket drawn at the first block of an item
    volatile uint32_t* const lds_tkt = reinterpret_cast<volatile uint32_t*>(lds + TKT_OFS);

    e8_static_for<64>([&](auto ix) { e8_acc_zero4<decltype(ix)::value>(); });
    {
        WG8_LOAD_S(c.sq, c.sp);
#pragma unroll
        for (int k = 0; k < 16; ++k) WG8_COPY(k, c.red, c.ptile, c.ptile2, c.qtile, c.qtile2, 0);
#pragma unroll
        for (int k = 0; k < 16; ++k)
            if (k * CSTEP < 64 - BAR) WG8_COPY(k, c.red, c.ptile + 128, c.ptile2 + 128, c.qtile + 128, c.qtile2 + 128, 1);
        WG8_WAIT_ALL();
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) pf[0][i] = e8_frag(lds + fp_ofs[0] + i * 2048, lds + fp_ofs[1] + i * 2048);
#pragma unroll
        for (int j = 0; j < 3; ++j) qf[j] = e8_frag(lds + fq_ofs[0] + j * 128, lds + fq_ofs[1] + j * 128);
    }
    int32_t kb = 0;

    // one K block; PAR = parity of the block in this workgroup's stream of blocks = its LDS slot and
    // the half of pf[] that holds its P fragments.  Returns true after the last work item.
    auto blk = [&](auto par_c) -> bool {
        constexpr int PAR = decltype(par_c)::value;
        // the item after this one: a ticket is drawn during the first block, handed to the other wavefronts through
        // LDS behind the second block's barrier and turned into addresses at the third (an item has at least four
        // blocks; the first copies for the next item are issued in its last but one)
        // (the empty statements keep the lanes' reconvergence in a block of its own: merged into the join of the three
        // cases, it would make every wave-uniform value that differs between the cases look divergent to the compiler)
        if (kb == 0) {
            if (wave == 0) {
                if (lane == 0) {
                    uint32_t one = 1;
                    // (s_nop: the counter's address may have been moved into its scalar registers by the vector unit just
                    // before this statement, and a memory instruction may read such registers five wait states later at the
                    // earliest; the compiler pads its own instructions but not inline assembly)
                    asm volatile("s_nop 4\n\tglobal_atomic_add %0, %1, %2, %3 sc0" : "=v"(tkt) : "v"(zero_off), "v"(one), "s"(my_counter) : "memory");
                }
                asm volatile("" ::: "memory");
            }
        } else if (kb == 1) {
            if (wave == 0) {
                if (lane == 0) *lds_tkt = tkt;
                asm volatile("" ::: "memory");
            }
        } else if (kb == 2) {
            const int64_t u = W + (int64_t)__builtin_amdgcn_readfirstlane(*lds_tkt);
            n_valid = u < total_x;
            if (n_valid) setup(u, n);
            else n = c;                    // past the last item the copies and scale loads re-read this item's first blocks
        }
        // the exponents of this block's scales, four to a register
        const uint32_t sq_cur0 = wg8_pack_exp(sq_r0[0], sq_r0[1], sq_r0[2], sq_r0[3]), sq_cur1 = wg8_pack_exp(sq_r1[0], sq_r1[1], sq_r1[2], sq_r1[3]);
        const uint32_t sp_cur0 = wg8_pack_exp(sp_r[0], sp_r[1], sp_r[2], sp_r[3]), sp_cur1 = wg8_pack_exp(sp_r[4], sp_r[5], sp_r[6], sp_r[7]);
        const int32_t KB = c.kb;
        const bool in1 = kb + 1 < KB, in2 = kb + 2 < KB;
        const int32_t o1 = (in1 ? kb + 1 : kb + 1 - KB) * 128, o2 = (in2 ? kb + 2 : kb + 2 - KB) * 128;
        const float* s_sq = in1 ? c.sq + (uint64_t)(uint32_t)(kb + 1) * (uint32_t)a.Qrows : n.sq;
        const float* s_sp = in1 ? c.sp + (uint64_t)(uint32_t)(kb + 1) * (uint32_t)a.Prows : n.sp;
        const int32_t red1 = in1 ? c.red : n.red, red2 = in2 ? c.red : n.red;
        const uint8_t* cp1_p = (in1 ? c.ptile : n.ptile) + o1;
        const uint8_t* cp1_p2 = (in1 ? c.ptile2 : n.ptile2) + o1;
        const uint8_t* cp1_q = (in1 ? c.qtile : n.qtile) + o1;
        const uint8_t* cp1_q2 = (in1 ? c.qtile2 : n.qtile2) + o1;
        const uint8_t* cp2_p = (in2 ? c.ptile : n.ptile) + o2;
        const uint8_t* cp2_p2 = (in2 ? c.ptile2 : n.ptile2) + o2;
        const uint8_t* cp2_q = (in2 ? c.qtile : n.qtile) + o2;
        const uint8_t* cp2_q2 = (in2 ? c.qtile2 : n.qtile2) + o2;
        __builtin_amdgcn_sched_barrier(0);
        WG8_LOAD_S(s_sq, s_sp);
        const uint8_t* pbase = lds + PAR * SLOT;
        const uint8_t* nbase = lds + (PAR ^ 1) * SLOT;
        __builtin_amdgcn_sched_barrier(0);
        e8_static_for<64>([&](auto mc) {
            constexpr int m = decltype(mc)::value;
            constexpr int j = m >> 3, i = m & 7;
            if constexpr (m == BAR) {
                // every fragment read of this block has been issued (the last at MFMA 32) and the next
                // block's copies were all issued by MFMA 12: once both have returned, meet the others
                WG8_WAIT_ALL();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (i == 0 && j + 3 < 8) {
                qf[(j + 3) % 4] = e8_frag(pbase + fq_ofs[0] + (j + 3) * 128, pbase + fq_ofs[1] + (j + 3) * 128);
                __builtin_amdgcn_sched_barrier(0);
            }
            wg8_mfma<8 * i + j, (i & 3), (j & 3)>(pf[PAR][i], qf[j % 4], i < 4 ? sp_cur0 : sp_cur1, j < 4 ? sq_cur0 : sq_cur1);
            __builtin_amdgcn_sched_barrier(0);
            // copies: the block after next into the slot this block has just left, continued in the
            // next block before its barrier
            if constexpr (m >= BAR && (m - BAR) % CSTEP == 0 && (m - BAR) / CSTEP < 16) {
                WG8_COPY((m - BAR) / CSTEP, red2, cp2_p, cp2_p2, cp2_q, cp2_q2, PAR);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (m < BAR && (m + 64 - BAR) % CSTEP == 0 && (m + 64 - BAR) / CSTEP < 16) {
                WG8_COPY((m + 64 - BAR) / CSTEP, red1, cp1_p, cp1_p2, cp1_q, cp1_q2, PAR ^ 1);
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

        // ---- item finished: fp32 read-modify-write of this wavefront's 128 x 128 quarter.  Pass t stages the 16 rows
        // 8 r + j (r = 0..15: the lanes' Q rows of fragment j = t / 2) x 64 columns (P fragments 4 h .. 4 h + 3, h = t % 2)
        // in the wavefront's LDS slice, 16-byte chunk k of row r at chunk k ^ r, and adds them to the old rows as whole
        // 256-byte pieces; the old rows of pass t + 4 are requested before pass t is added.
        if (c.store) {
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written back before they are read
            uint8_t* ep = lds + EP_OFS + wave * 4096;
            const int er = lane >> 4, ec = lane & 15;
            // byte address of a row piece = wave-uniform (row 32 it + j of the quarter, column 64 h) + one lane offset
            // (row 8 er, column 4 ec); all products fit 32 bits (128 rows of ldo floats are below 2 GB)
            const uint32_t ldo4 = (uint32_t)a.ldo * 4u;
            const uint32_t lane_off = (uint32_t)(8 * er) * ldo4 + (uint32_t)(16 * ec);
            uint8_t* const quarter = reinterpret_cast<uint8_t*>(c.out);
            constexpr int AHEAD = 4;                 // passes whose old rows are in flight
            f32x4 old[AHEAD][4];
            auto request = [&](auto tc) {
                constexpr int t = decltype(tc)::value, j = t >> 1, h = t & 1;
                if constexpr (ACC) {
#pragma unroll
                    for (int it = 0; it < 4; ++it) {
                        const uint4 ow = ld16(quarter + (uint64_t)((uint32_t)(32 * it + j) * ldo4 + 256u * h) + lane_off);
                        old[t % AHEAD][it] = (f32x4){u2f(ow.x), u2f(ow.y), u2f(ow.z), u2f(ow.w)};
                    }
                } else {
#pragma unroll
                    for (int it = 0; it < 4; ++it) old[t % AHEAD][it] = (f32x4){0.f, 0.f, 0.f, 0.f};
                }
            };
            e8_static_for<AHEAD>([&](auto tc) { request(tc); });
            __builtin_amdgcn_sched_barrier(0);
            e8_static_for<16>([&](auto tc) {
                constexpr int t = decltype(tc)::value, j = t >> 1, h = t & 1;
                e8_static_for<4>([&](auto ic) {
                    constexpr int i = 4 * h + decltype(ic)::value;
                    constexpr int R = 4 * (8 * i + j);
                    const f32x4 v = {e8_acc_get<R>(), e8_acc_get<R + 1>(), e8_acc_get<R + 2>(), e8_acc_get<R + 3>()};
                    *reinterpret_cast<f32x4*>(ep + li * 256 + (((decltype(ic)::value * 4 + kg) ^ li) << 4)) = v;
                });
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rl = er + 4 * it;                        // staged row = l of the producer
                    const f32x4 v = *reinterpret_cast<const f32x4*>(ep + rl * 256 + ((ec ^ rl) << 4));
                    const f32x4 o = old[t % AHEAD][it];
                    const f32x4 w = {o.x + v.x, o.y + v.y, o.z + v.z, o.w + v.w};
                    uint8_t* dst = quarter + (uint64_t)((uint32_t)(32 * it + j) * ldo4 + 256u * h) + lane_off;
                    st16(dst, make_uint4(f2u(w.x), f2u(w.y), f2u(w.z), f2u(w.w)));
                }
                if constexpr (t + AHEAD < 16) request(std::integral_constant<int, t + AHEAD>{});
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        if (!n_valid) return true;
        e8_static_for<64>([&](auto ix) { e8_acc_zero4<decltype(ix)::value>(); });
        c = n;
        kb = 0;
        return false;
    };
    for (;;) {
        if (blk(std::integral_constant<int, 0>{})) break;
        if (blk(std::integral_constant<int, 1>{})) break;
    }
    __builtin_amdgcn_s_waitcnt(0);   // the copies issued past the end must land before the LDS is released
    finish();
#undef WG8_COPY
#undef WG8_LOAD_S
#undef WG8_WAIT_ALL
}

}  // namespace pf8

using namespace pf8;

static constexpr int WG8_LDS_BYTES = 131072 + 4 * 4096 + 16;
static constexpr int WG8_SLOTS = 64;
// ticket counters of the launches in flight: slot s = 16 ints (8 XCD counters, the count of finished workgroups), zero
// whenever no launch is using it.  Every GPU holds its own copy at its own address.
static __device__ __align__(256) int32_t wg8_tickets[WG8_SLOTS * 16];

static int wg8_ticket_slot(const char* where, int32_t** out) {
    static std::atomic<int32_t*> ptrs[64];
    static std::atomic<uint32_t> seq{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return pf8_fail(PF8_EINVAL, where, "device ordinal beyond 63");
    int32_t* p = ptrs[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        e = hipGetSymbolAddress(&sym, HIP_SYMBOL(wg8_tickets));
        if (e != hipSuccess || !sym) return pf8_fail(PF8_ELAUNCH, where, e != hipSuccess ? hipGetErrorString(e) : "hipGetSymbolAddress returned a null address");
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_wgrad_e8<true>), hipFuncAttributeMaxDynamicSharedMemorySize, WG8_LDS_BYTES);
        if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_wgrad_e8<false>), hipFuncAttributeMaxDynamicSharedMemorySize, WG8_LDS_BYTES);
        if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
        p = static_cast<int32_t*>(sym);
        ptrs[dev].store(p, std::memory_order_release);     // two threads racing here store the same address
    }
    *out = p + 16 * (seq.fetch_add(1, std::memory_order_relaxed) % WG8_SLOTS);
    return PF8_OK;
}

// Launches the 256x256-tile kernel on the listed experts (longest reduction first).  The caller has checked the shapes:
// Prows, Qrows multiples of 128 and at least 256, every listed expert at least four blocks long, 16-byte aligned scales.
int pf8_launch_wgrad_e8(const uint8_t* p, const uint8_t* q, const float* sp, const float* sq, float* out, int64_t Prows, int64_t Qrows,
                        int64_t ldo, int accumulate, int n_items, const int32_t* item_t0, const int32_t* item_kb, const uint8_t* item_e,
                        int cus, hipStream_t stream, const char* where) {
    if (n_items <= 0) return PF8_OK;
    if (n_items > kWgE8MaxItems) return pf8_fail(PF8_EINVAL, where, "too many experts for the 256x256-tile weight-gradient kernel");
    WgE8Args g = {};
    g.p = p; g.q = q; g.sp = sp; g.sq = sq; g.out = out;
    g.Prows = Prows; g.Qrows = Qrows; g.ldo = ldo; g.accumulate = accumulate; g.n_items = n_items;
    for (int i = 0; i < n_items; ++i) {
        if (item_kb[i] < 4) return pf8_fail(PF8_EINVAL, where, "an expert of fewer than four blocks was listed for the 256x256-tile kernel");
        g.item_t0[i] = item_t0[i]; g.item_kb[i] = item_kb[i]; g.item_e[i] = item_e[i];
    }
    int rc = wg8_ticket_slot(where, &g.tickets);
    if (rc) return rc;
    // q-tiles per group: a slice of T / 8 tiles touches about gq Q panels and T / (8 gq) P panels; the divisor of the q-tile
    // count that makes that sum smallest
    const int64_t tq = (Qrows + 255) / 256, tp = (Prows + 255) / 256, T_item = tq * tp;
    double best = -1.0;
    for (int64_t gq = 1; gq <= tq; ++gq) {
        if (tq % gq) continue;
        const double cost = (double)gq + (double)T_item / (8.0 * (double)gq);
        if (best < 0 || cost < best) { best = cost; g.gq = (int)gq; }
    }
    const int64_t per_xcd = ((T_item + 7) / 8) * n_items;
    int64_t w = cus / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    if (accumulate) hipLaunchKernelGGL(k_wgrad_e8<true>, dim3((unsigned)(8 * w)), dim3(256), WG8_LDS_BYTES, stream, g);
    else hipLaunchKernelGGL(k_wgrad_e8<false>, dim3((unsigned)(8 * w)), dim3(256), WG8_LDS_BYTES, stream, g);
    return pf8_check_launch(where);
}
