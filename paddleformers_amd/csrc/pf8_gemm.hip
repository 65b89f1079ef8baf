// pf8_gemm.hip -- block-scaled FP8 GEMMs for gfx950 (v_mfma_f32_16x16x128_f8f6f4) and their C entry
// points: dense NT, grouped contiguous, grouped masked, the 1x128-by-1x128 weight-gradient GEMM and
// its per-expert grouped form.
//
// One MFMA consumes a 128-wide slice of the reduction axis, which is exactly one scale block: the
// product of a K block goes into a scratch accumulator (C = 0) and is folded into the fp32 master
// accumulator with one FMA per element, scaled by sa*sb of that block.
//
// Naming: the "P" operand feeds the MFMA A port (its rows become the CONTIGUOUS axis of the output),
// the "Q" operand feeds the B port (its rows become output rows).  Each lane then owns 4 consecutive
// output elements of one output row, so stores are 8 B (bf16) or 16 B (fp32) per lane.
//   forward / dgrad : P = weights [N,K] (128x128 scales), Q = activations [M,K] (1x128 scales)
//   weight gradient : P = dout^T [N,M], Q = x^T [Kin,M], both 1x128-scaled along M
//
// Two kernels: k_gemm_fwd128 (forward / dgrad, 128x256x128 tiles, described at its definition) and
// k_gemm (the weight-gradient form: 256 threads = 4 wavefronts in a 2x2 arrangement, tile
// 128(P) x 128(Q) x 128(K), each wavefront 64x64 = 4x4 MFMA tiles, operands staged through
// registers into two 32 KB LDS stages).  LDS rows are 128 B with their 16-byte chunks XOR-swizzled
// so that fragment reads (16 rows x 32 B per quarter-wave) are bank-conflict free.
#include <atomic>
#include <type_traits>

#include "pf8_gemm_common.h"
#include "pf8_host.h"

namespace pf8 {

// ---------------------------------------------------------------------------------------------
// Forward / dgrad kernel: 128(Q) x 256(P) x 128(K) tiles, 256 threads = 4 wavefronts (2 along Q x
// 2 along P), each owning 64(Q) x 128(P) = 4 x 8 MFMA tiles (128 accumulator registers).
//
// Budget per compute unit and 128-wide K block (two workgroups resident): 2048 cycles of MFMA work
// per SIMD against 96 KB of L2->LDS traffic (1536 cycles at 64 B/clk) and 8 x 12 fragment reads of
// 2 KB (LDS delivers 128 B/clk, measured: 1536 cycles, plus 768 for the incoming copies).  LDS is
// as busy as the matrix pipe, so the schedule is built to overlap them:
//   * both operand tiles go global -> LDS with global_load_lds_dwordx4 (no staging registers; the
//     16-byte chunk each lane fetches is chosen so that the linear 1 KB an instruction writes lands
//     XOR-swizzled, which the fragment reads see conflict-free);
//   * 80 KB of LDS per workgroup so that TWO workgroups share a compute unit: while one sits at a
//     barrier or waits for its first fragments, the other keeps the matrix pipe busy.  The P tile
//     is double-buffered (2 x 32 KB); the Q tile (16 KB) is single-buffered: its fragments are read
//     into registers at the head of a K block, and once every wavefront has done so (second
//     barrier, placed after the first eight MFMAs) the buffer is refilled for the next block;
//   * fragment reads are issued in the order the MFMAs consume them (P0, Q0..Q3, P1, then one P
//     fragment two steps ahead), so the first MFMA of a block waits for two fragments only;
//   * the four scale-FMAs that fold product j-2 into the fp32 accumulators sit between MFMA j and
//     j+1 (scheduling barriers pin this: left alone, the scheduler pairs every MFMA with its own
//     FMAs and waits out the MFMA latency 32 times per block).
// Tried and dropped: a 256x256 tile with 8 wavefronts in one workgroup per compute unit (fewer LDS
// bytes per MFMA, but its single barrier domain left the matrix pipe idle at every block boundary:
// 1.7-1.9 PFLOP/s dense against 1.8-2.0 here, and 0.85 against 1.4 on short expert segments), and
// reading the activation fragments straight from global memory (16 rows per load instruction
// defeat the coalescer).
// A 128-row tile never straddles two experts of the grouped layout.
// ---------------------------------------------------------------------------------------------
template <int SQL>
__global__ __launch_bounds__(256, 2) void k_gemm_fwd128(const GemmArgs a) {
    constexpr int BQ = 128, NPS = 8;
    constexpr int P_STAGE = 32768, Q_OFS = 65536;   // [P stage 0 | P stage 1 | Q]
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int64_t p_tiles = (a.Prows + 255) / 256, q_tiles = (a.Qrows + BQ - 1) / BQ;
    const int64_t T = p_tiles * q_tiles;
    // consecutive workgroups go round-robin to the 8 XCDs: give every XCD a contiguous run of logical
    // tiles, ordered in groups of 16 q-tiles x all p-tiles.  The grid normally holds one workgroup per
    // tile; under a compute-unit budget it is smaller and a workgroup walks its XCD's run in strides.
    const int64_t per_xcd = (T + 7) / 8;
    for (int64_t loc = blockIdx.x >> 3; loc < per_xcd; loc += gridDim.x >> 3) {
    // the lane's coordinates are formed anew for every tile from a value the compiler cannot see through: hoisted
    // out of the loop, everything a tile's set-up derives from them would stay live across the whole tile (39
    // registers more than the file holds)
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6;
    const int wq = wave >> 1, wp = wave & 1;
    const int li = lane & 15, kg = lane >> 4;
    const int64_t logical = (int64_t)(blockIdx.x & 7) * per_xcd + loc;
    if (logical >= T) break;
    constexpr int G = 16;
    const int64_t grp = logical / (G * p_tiles), rem = logical % (G * p_tiles);
    const int64_t gq = q_tiles - grp * G < G ? q_tiles - grp * G : G;
    const int64_t q_tile = grp * G + rem % gq, p_tile = rem / gq;
    const int64_t p0 = p_tile * 256, q0 = q_tile * BQ;

    int64_t KB = a.red / 128;
    asm volatile("" : "+s"(KB));          // per tile as well: a flag derived from it was kept in a register across the loop
    const int64_t PB = (a.Prows + 127) / 128;
    const uint8_t* qbase = a.q;
    const float* sqb = a.sq;
    uint8_t* outb = reinterpret_cast<uint8_t*>(a.out);
    const int64_t q_rows_total = a.Qrows;
    int e = 0, row_hi = BQ;
    if (a.group == GROUP_CONTIG) {
        e = a.m_indices[q0];
        if (e < 0) continue;
    } else if (a.group == GROUP_MASKED) {
        e = blockIdx.y;
        const int64_t valid = a.masked_m[e];
        if (q0 >= valid) continue;
        row_hi = valid - q0 < BQ ? (int)(valid - q0) : BQ;
        qbase += (int64_t)e * a.Qrows * a.red;
        sqb += (int64_t)e * a.Qrows * KB;
        outb += (int64_t)e * a.Qrows * a.ldo * 2;
    }

    // global -> LDS: P tile = 32 copies of 1 KB (8 per wavefront), Q tile = 16 copies (4 per wavefront)
    const int crow = lane >> 3, cpos = lane & 7;
    uint32_t p_src[8], q_src[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = (i * 4 + wave) * 8 + crow;             // 0..255
        const int chunk = cpos ^ swz_key(row);
        int64_t pr = p0 + row; if (pr > a.Prows - 1) pr = a.Prows - 1;
        p_src[i] = (uint32_t)((pr - p0) * a.red + chunk * 16);
        if (i < 4) {
            int64_t qr = q0 + row; if (qr > q_rows_total - 1) qr = q_rows_total - 1;   // row < 128 for i < 4
            q_src[i] = (uint32_t)((qr - q0) * a.red + chunk * 16);
        }
    }
    const uint8_t* qtile = qbase + q0 * a.red;
    const uint8_t* ptile = a.p + ((int64_t)e * a.Prows + p0) * a.red;
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    int fp_ofs[2], fq_ofs[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        fp_ofs[h] = swz(wp * 128 + li, 2 * kg + h);
        fq_ofs[h] = Q_OFS + swz(wq * 64 + li, 2 * kg + h);
    }
    int64_t qrow_g[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        int64_t r = q0 + wq * 64 + t * 16 + li;
        if (r > q_rows_total - 1) r = q_rows_total - 1;
        qrow_g[t] = r;
    }
    int64_t pblk = p_tile * 2 + wp;
    if (pblk > PB - 1) pblk = PB - 1;
    const float* spb = a.sp + ((int64_t)e * PB + pblk) * KB;

    f32x4 acc[NPS][4];
#pragma unroll
    for (int i = 0; i < NPS; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float fq_nxt[4], fpb_nxt = 0.f;

#define PF8_DMA_P(kb_, stage_)                                                                         \
    _Pragma("unroll") for (int i = 0; i < 8; ++i)                                                      \
        dma16_to_lds(ptile + p_src[i] + (kb_) * 128, lds_base + (stage_) * P_STAGE + (i * 4 + wave) * 1024);
#define PF8_DMA_Q(kb_)                                                                                 \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                      \
        dma16_to_lds(qtile + q_src[i] + (kb_) * 128, lds_base + Q_OFS + (i * 4 + wave) * 1024);
#define PF8_LOAD_S(kb_)                                                                                \
    _Pragma("unroll") for (int t = 0; t < 4; ++t)                                                      \
        fq_nxt[t] = SQL == 0 ? sqb[qrow_g[t] * KB + (kb_)] : sqb[(kb_) * q_rows_total + qrow_g[t]];
#define PF8_PFRAG(ps_) ld_frag_lds(pbase + fp_ofs[0] + (ps_) * 2048, pbase + fp_ofs[1] + (ps_) * 2048)
#define PF8_QFRAG(qs_) ld_frag_lds(lds + fq_ofs[0] + (qs_) * 2048, lds + fq_ofs[1] + (qs_) * 2048)

    if (KB > 0) {
        PF8_DMA_P(0, 0)
        PF8_DMA_Q(0)
        PF8_LOAD_S(0)
        fpb_nxt = spb[0];
    }
    for (int64_t kb = 0; kb < KB; ++kb) {
        const int cur = (int)(kb & 1);
        __builtin_amdgcn_s_waitcnt(0);   // this wave's copies and scale loads have landed
        __syncthreads();                 // everyone's copies landed; everyone is done with P stage cur^1
        float fq_cur[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) fq_cur[t] = fq_nxt[t] * fpb_nxt;
        const int64_t kbn = kb + 1 < KB ? kb + 1 : kb;
        PF8_DMA_P(kbn, cur ^ 1)
        PF8_LOAD_S(kbn)
        const uint8_t* pbase = lds + cur * P_STAGE;
        i32x8 pf[3], qf[4];
        f32x4 d[3];
        pf[0] = PF8_PFRAG(0);
        __builtin_amdgcn_sched_barrier(0);
        qf[0] = PF8_QFRAG(0);
        __builtin_amdgcn_sched_barrier(0);
        qf[1] = PF8_QFRAG(1);
        __builtin_amdgcn_sched_barrier(0);
        qf[2] = PF8_QFRAG(2);
        __builtin_amdgcn_sched_barrier(0);
        qf[3] = PF8_QFRAG(3);
        __builtin_amdgcn_sched_barrier(0);
        pf[1] = PF8_PFRAG(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NPS * 4; ++j) {
            const int ps = j >> 2, qs = j & 3;
            d[j % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ps % 3], qf[qs], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (qs == 0 && ps + 2 < NPS) {
                pf[(ps + 2) % 3] = PF8_PFRAG(ps + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (j == 7) {
                // every wavefront has its four Q fragments in registers by now: refill the Q buffer
                __syncthreads();
                PF8_DMA_Q(kbn)
                __builtin_amdgcn_sched_barrier(0);
            }
            if (j >= 2) {
                const int jj = j - 2;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[jj >> 2][jj & 3][r] = __builtin_fmaf(d[jj % 3][r], fq_cur[jj & 3], acc[jj >> 2][jj & 3][r]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int jj = NPS * 4 - 2; jj < NPS * 4; ++jj)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                acc[jj >> 2][jj & 3][r] = __builtin_fmaf(d[jj % 3][r], fq_cur[jj & 3], acc[jj >> 2][jj & 3][r]);
        __builtin_amdgcn_sched_barrier(0);
        // the block scale of P is a scalar load; scalar loads share the LDS wait counter and return
        // out of order, so issuing it any earlier would turn every fragment wait of this block
        // into a full drain
        fpb_nxt = spb[kbn];
    }
    __builtin_amdgcn_s_waitcnt(0);

    // ---- epilogue: bf16 through LDS so that every store instruction writes whole 256-byte rows
    // (straight from the MFMA layout a lane owns 4 consecutive outputs and a store instruction
    // covers 32-byte row pieces: measured 17% of the kernel's time on the dense configuration) ----
    constexpr int EP_LD = 272;                   // 128 bf16 per row + 16 B pad
    __syncthreads();                             // everyone is done reading fragments
    uint8_t* ep = lds + wave * (64 * EP_LD);
#pragma unroll
    for (int qs = 0; qs < 4; ++qs)
#pragma unroll
        for (int ps = 0; ps < NPS; ++ps) {
            uint2 o;
            o.x = pack_bf16(acc[ps][qs][0], acc[ps][qs][1]);
            o.y = pack_bf16(acc[ps][qs][2], acc[ps][qs][3]);
            *reinterpret_cast<uint2*>(ep + (qs * 16 + li) * EP_LD + (ps * 16 + 4 * kg) * 2) = o;
        }
    // LDS operations of one wavefront execute in order: the reads below see the writes above
    const int er = lane >> 4, ec = lane & 15;
    const int64_t col = p0 + wp * 128 + ec * 8;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int rt = wq * 64 + er + 4 * i;     // row inside the tile
        const int64_t row = q0 + rt;
        const uint4 v = *reinterpret_cast<const uint4*>(ep + (er + 4 * i) * EP_LD + ec * 16);
        if (rt >= row_hi || row >= q_rows_total) continue;
        uint8_t* dst = outb + (row * a.ldo + col) * 2;
        if (col + 8 <= a.Prows) {
            st16(dst, v);
        } else if (col + 4 <= a.Prows) {
            *reinterpret_cast<uint2*>(dst) = make_uint2(v.x, v.y);
        }
    }
    __syncthreads();   // the staging rows are dead before the next tile's copies land on them
    }
#undef PF8_DMA_P
#undef PF8_DMA_Q
#undef PF8_LOAD_S
#undef PF8_PFRAG
#undef PF8_QFRAG
}

// ---------------------------------------------------------------------------------------------
// Deep-pipeline forward kernel for shapes without ragged tiles: Qrows % 128 == 0, Prows % 128 == 0 and at least 256
// (a last column tile may be half new), at least three K blocks; dense, contiguous-grouped and masked layouts.
//   * One persistent workgroup per compute unit walks its XCD's run of 128x256 tiles; 144 KB of LDS
//     is a three-stage ring of [P 32 KB | Q 16 KB] blocks that runs on ACROSS tile boundaries: the
//     copies of the block two ahead are issued during the current block, one between every other
//     MFMA, whether that block belongs to this tile or the next.  A tile therefore has no fill
//     phase of its own, and a copy has two block times to land.
//   * One barrier per block, placed before MFMA 24 of 32: by then every fragment read of the block
//     has been issued, and behind the barrier the first fragments of the next block are read into
//     the registers that come free (P6 and P7 are interleaved at the end for that), so the matrix
//     pipe does not drain at a block boundary.
//   * All global addresses are a scalar base plus one per-lane 32-bit offset (the swizzled chunk a
//     lane fetches does not depend on the copy index): 224 registers, MFMA results stay in VGPRs.
//   * Every memory instruction of the loop is inline assembly so that vmcnt is counted by hand: per
//     block a wavefront issues 5 scale loads and then 12 copies, loads retire in issue order, and
//     the wait before the barrier leaves exactly the 12 youngest copies outstanding (the stores of a
//     finished tile are older than those and simply retire with them).  The scales land in VGPRs,
//     the P block's too (every lane loads the same word): a value in flight may not be touched
//     before its wait, and the compiler, unaware of the load, copies scalar registers freely.
//   * The epilogue stages bf16 rows in the LDS stage the tile's last block has just left, 32 rows
//     per wavefront at a time, and writes whole 256-byte rows.
// ---------------------------------------------------------------------------------------------
// SF = 1: the scales are UE8M0 exponent bytes (sq [KB, ldsq], sp [E][Prows/128, KB]) instead of floats;
// the kernel is the same, a scale is decoded where the block's factors are formed.
__device__ __forceinline__ float e8m0_to_f32(uint32_t b) { return u2f(b ? b << 23 : 0x00400000u); }

// FUSE = 1: the up+gate GEMM of the MoE MLP with SwiGLU, the probability factor and the 1x128 requantization in its
// epilogue.  A tile's 256 weight rows are 128 gate rows and the 128 up rows of the same output columns (two row ranges
// of the stacked [gate | up] weight, nothing is re-laid out), so the wavefront pair (wq, 0) / (wq, 1) holds gate and up
// of the same 64 x 128 outputs.  Both round to bf16 (that IS o1, stored as well when the caller wants it), meet in the
// LDS staging rows, and each wavefront turns 16 rows per pass into e4m3 bytes and one scale per row: a row of 128
// outputs is the 16 lanes of a DPP row, exactly the tile of the standalone SwiGLU quantizer, whose arithmetic is
// restated operation for operation (bf16(silu(g) * u), bf16(. * p), amax, scale, quotient), so bytes and scales are
// bit-identical to the un-fused pair of launches.
// Capacities of the persistent kernel's LDS tables, shared by the kernel and by the host code that decides which
// launches it may take: row tiles whose expert order is tabulated, experts of a masked launch, dynamic LDS of the ring.
constexpr int kDeepSegTiles = 2048, kDeepMaskedExperts = 256, kDeepDynLds = 147456;

template <int SQL, int SF = 0, int FUSE = 0, int MASKED = 0>
__global__ __launch_bounds__(256, 2) void k_gemm_fwd_deep(const GemmArgs a) {
    using ST = typename std::conditional<SF == 1, uint8_t, float>::type;
    if (SF == 1 && a.pair_list && e8_paired_tiles_win(a.pair_list, a.Prows / 256, a.cus)) return;
    const ST* const sp_base = reinterpret_cast<const ST*>(a.sp);
    const ST* const sq_base = reinterpret_cast<const ST*>(a.sq);
    constexpr int BQ = 128, NPS = 8;
    constexpr int STAGE = 49152, Q_OFS = 32768;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wq = wave >> 1, wp = wave & 1;
    const int li = lane & 15, kg = lane >> 4;

    // Prows may be 256 t + 128: the last column tile then covers the last 256 weight rows, i.e. it repeats the 128
    // columns before it (those wavefronts store nothing) beside the 128 new ones.  Not with FUSE.
    const int64_t p_tiles = (a.Prows + 255) / 256;
    int64_t q_tiles = a.Qrows / BQ;          // masked layout: row tiles per expert here, valid row tiles of all experts below
    const int64_t p_last0 = a.Prows - 256;                                   // first weight row of that tile
    auto p_row0 = [&](int64_t pt) -> int64_t { return FUSE ? pt * 128 : (pt * 256 < p_last0 ? pt * 256 : p_last0); };
    // FUSE: tile p takes weight rows [128 p, 128 p + 128) (gate) and inter + the same (up)
    const int64_t up_off = FUSE ? a.inter * a.red : 128 * a.red;      // bytes from a tile's first half to its second
    const int64_t IB = FUSE ? a.inter / 128 : 0;
    // consecutive workgroups go round-robin to the 8 XCDs: every XCD owns a contiguous run of
    // logical tiles (groups of q-tiles x all p-tiles, see below), walked W tiles at a time by its W workgroups
    const int64_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, W = gridDim.x >> 3;
    const int64_t KB = a.red / 128;
    const int64_t PB = a.Prows / 128;
    const int64_t q_rows_total = a.Qrows;
    const bool grouped = a.group == GROUP_CONTIG;
    constexpr bool masked = MASKED != 0;       // its own instantiation: the extra state costs the others registers

    // Grouped layout with at most 2048 row tiles: every expert's run of row tiles is cut into groups of at most 12
    // tiles (no group spans two experts), and the tiles of a group are walked q fastest, p slowest.  The 32 workgroups
    // of an XCD then work on one or two weight strips of ONE expert at a time and on the few activation strips of
    // that group, instead of on 16 activation strips that belong to a dozen experts.  Measured on config 3 (32
    // experts, Zipf load) against groups of 16 row tiles cut without regard to experts: the L2s miss 1.33 GB instead
    // of 1.74 GB per up+gate launch (hit rate 64% against 53%) and 0.74 GB instead of 0.96 GB on the down GEMM; the
    // launches get 3% and 2% shorter.  seg_tab[q] = first tile of q's group | tiles in it << 16; every workgroup
    // builds the table for itself: the first tile of each run by a prefix maximum over the tiles, 256 at a time.
    __shared__ uint32_t seg_tab[kDeepSegTiles];
    __shared__ int16_t seg_eid[MASKED ? 2 : kDeepSegTiles + 2];   // expert of every row tile (one global load each), -1 = padding
    __shared__ int seg_wave_max[2][4];
    __shared__ int seg_valid[MASKED ? kDeepMaskedExperts : 1];
    __shared__ int seg_total;
    static_assert(sizeof(seg_tab) + sizeof(seg_eid) + sizeof(seg_wave_max) + sizeof(seg_valid) + sizeof(int) + kDeepDynLds <= 163840,
                  "static tables plus the dynamic ring exceed the 160 KB of LDS a workgroup can have");
    const bool ordered = !MASKED && grouped && q_tiles <= kDeepSegTiles && a.E <= 32767;
    if (ordered) {
        constexpr int CAP = 12;
        const int qt = (int)q_tiles;
        for (int t = tid; t < qt; t += 256) {
            const int e = a.m_indices[(int64_t)t * BQ];
            seg_eid[t + 1] = (int16_t)(e < 0 ? -1 : e);
        }
        if (tid == 0) { seg_eid[0] = -2; seg_eid[qt + 1] = -2; }
        __syncthreads();
        int carry = 0;                                     // first tile of the run the previous chunk ended in
        for (int c0 = 0, par = 0; c0 < qt; c0 += 256, par ^= 1) {
            const int t = c0 + tid;
            const int e = t < qt ? seg_eid[t + 1] : -2;
            int v = (t < qt && t > 0 && seg_eid[t] != e) ? t : 0;
#pragma unroll
            for (int dlt = 1; dlt < 64; dlt <<= 1) {
                const int o = __shfl_up(v, dlt, 64);
                if (lane >= dlt && o > v) v = o;
            }
            if (lane == 63) seg_wave_max[par][wave] = v;
            __syncthreads();                               // the buffers alternate: one barrier per chunk
            int all = carry;
            for (int w = 0; w < 4; ++w) {
                const int m = seg_wave_max[par][w];
                if (w < wave && m > v) v = m;
                if (m > all) all = m;
            }
            if (carry > v) v = carry;
            carry = all;
            if (t < qt) {
                const int gs = v + (t - v) / CAP * CAP;    // v = first tile of this tile's run
                int hi = t + 1;
                while (hi < gs + CAP && seg_eid[hi + 1] == e) ++hi;     // stops at the end marker behind the last tile
                seg_tab[t] = (uint32_t)gs | (uint32_t)(hi - gs) << 16;
            }
        }
        __syncthreads();
    }

    // Masked layout (a [E, Mmax, K], masked_m[e] valid rows; at most 256 experts and 2048 row tiles): only the row tiles
    // that hold valid rows are walked.  Every workgroup lists them for itself: seg_tab[slot] = expert | tile << 16,
    // seg_valid[e] = valid rows; a row tile of expert e is row tile e * (Mmax / 128) + tile of the [E * Mmax, K] matrix.
    const int mt = (int)(a.Qrows / BQ);                    // row tiles per expert (masked)
    if (masked) {
        int valid = 0, cnt = 0;
        if (tid < a.E) {
            valid = a.masked_m[tid];
            valid = valid < 0 ? 0 : (valid > (int)a.Qrows ? (int)a.Qrows : valid);
            cnt = (valid + BQ - 1) / BQ;
            seg_valid[tid] = valid;
        }
        int incl = cnt;                                    // inclusive prefix sum over the 256 threads
#pragma unroll
        for (int dlt = 1; dlt < 64; dlt <<= 1) {
            const int o = __shfl_up(incl, dlt, 64);
            if (lane >= dlt) incl += o;
        }
        if (lane == 63) seg_wave_max[0][wave] = incl;
        __syncthreads();
        int before = 0;
        for (int w = 0; w < wave; ++w) before += seg_wave_max[0][w];
        if (tid == 0) seg_total = seg_wave_max[0][0] + seg_wave_max[0][1] + seg_wave_max[0][2] + seg_wave_max[0][3];
        const int first = before + incl - cnt;
        for (int i = 0; i < cnt; ++i) seg_tab[first + i] = (uint32_t)tid | (uint32_t)i << 16;
        __syncthreads();
        q_tiles = seg_total;
    }
    const int64_t T = p_tiles * q_tiles;
    const int64_t per_xcd = (T + 7) / 8;
    int t_e = 0, t_rows = BQ;                              // masked: expert and valid rows of the tile tile_coords returned last

    auto tile_coords = [&](int64_t n, int64_t& q_tile, int64_t& p_tile) -> bool {
        constexpr int G = 16;
        const int64_t loc = slot + n * W, logical = xcd * per_xcd + loc;
        if (loc >= per_xcd || logical >= T) return false;
        if (ordered) {
            const uint32_t sg = (uint32_t)__builtin_amdgcn_readfirstlane((int)seg_tab[(int)(logical / p_tiles)]);
            const int gs = (int)(sg & 0xFFFFu), gl = (int)(sg >> 16);
            const int j = (int)(logical - (int64_t)gs * p_tiles);
            p_tile = j / gl;
            q_tile = gs + j % gl;
            return true;
        }
        const int64_t grp = logical / (G * p_tiles), rem = logical % (G * p_tiles);
        const int64_t gq = q_tiles - grp * G < G ? q_tiles - grp * G : G;
        q_tile = grp * G + rem % gq;
        p_tile = rem / gq;
        if (masked) {
            const uint32_t sg = (uint32_t)__builtin_amdgcn_readfirstlane((int)seg_tab[(int)q_tile]);
            t_e = (int)(sg & 0xFFFFu);
            const int lt = (int)(sg >> 16);
            const int left = __builtin_amdgcn_readfirstlane(seg_valid[t_e]) - lt * BQ;
            t_rows = left < BQ ? left : BQ;
            q_tile = (int64_t)t_e * mt + lt;
        }
        return true;
    };

    // current tile (c_*) and next tile (n_*): everything here is wave-uniform
    int64_t cq = 0, cp = 0, nq = 0, np = 0;
    if (!tile_coords(0, cq, cp)) return;
    int ce = 0;
    if (grouped) ce = __builtin_amdgcn_readfirstlane(a.m_indices[cq * BQ]);
    if (masked) ce = t_e;
    int c_rows = ce < 0 ? 0 : (masked ? t_rows : BQ);   // rows of the tile that are stored (none for a padding tile)
    if (ce < 0) ce = 0;
    const uint8_t* c_ptile = a.p + ((int64_t)ce * a.Prows + p_row0(cp)) * a.red;
    const uint8_t* c_qtile = a.q + cq * BQ * a.red;
    const ST* c_spb = sp_base + ((int64_t)ce * PB + (FUSE ? cp + wp * IB : p_row0(cp) / 128 + wp)) * KB;
    const ST* c_sq0 = SQL == 0 ? sq_base + (cq * BQ + wq * 64) * KB : sq_base + cq * BQ + wq * 64;
    const uint8_t* n_ptile = c_ptile;
    const uint8_t* n_qtile = c_qtile;
    const ST* n_spb = c_spb;
    const ST* n_sq0 = c_sq0;
    int n_rows = 0;

    // copy i of a wavefront fills rows (4 i + wave) * 8 + (lane >> 3) of the tile; the 16-byte chunk a
    // lane fetches is (lane & 7) ^ swz_key(row), and swz_key depends on lane and wave only
    const int crow = lane >> 3, cpos = lane & 7;
    const uint32_t c_off = (uint32_t)((wave * 8 + crow) * a.red + ((cpos ^ swz_key(wave * 8 + crow)) << 4));
    const int64_t copy_step = 32 * a.red;                       // 32 rows between copy i and i+1
    const int64_t sq_t = SQL == 0 ? 16 * KB : 16;               // floats between the scale rows of t and t+1
    const int64_t sq_k = SQL == 0 ? 1 : (SF == 1 && a.ldsq ? a.ldsq : q_rows_total);   // scales between K blocks
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    int fp_ofs[2], fq_ofs[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        fp_ofs[h] = swz(wp * 128 + li, 2 * kg + h);
        fq_ofs[h] = Q_OFS + swz(wq * 64 + li, 2 * kg + h);
    }
    const uint32_t s_off = (SQL == 0 ? (uint32_t)(li * KB) : (uint32_t)li) * (uint32_t)sizeof(ST);
    uint32_t zero_off = 0;
    asm volatile("" : "+v"(zero_off));     // a VGPR holding 0 for the scalar-base address form

    f32x4 acc[NPS][4];
    float fq_nxt[4], fpb_nxt = 0.f;

#define PF8_COPY(i_, pt_, qt_, stage_)                                                                 \
    do {                                                                                               \
        if ((i_) < 4) dma16_s(c_off, (pt_) + (i_) * copy_step, lds_base + (stage_) * STAGE + ((i_) * 4 + wave) * 1024); \
        else if ((i_) < 8) dma16_s(c_off, (pt_) + up_off + ((i_) - 4) * copy_step, lds_base + (stage_) * STAGE + ((i_) * 4 + wave) * 1024); \
        else dma16_s(c_off, (qt_) + ((i_) - 8) * copy_step, lds_base + (stage_) * STAGE + Q_OFS + (((i_) - 8) * 4 + wave) * 1024); \
    } while (0)
#define PF8_LOAD_S(sq_, sp_)                                                                           \
    _Pragma("unroll") for (int t = 0; t < 4; ++t)                                                      \
        if (SF == 1) asm volatile("global_load_ubyte %0, %1, %2" : "=v"(fq_nxt[t]) : "v"(s_off), "s"((sq_) + t * sq_t) : "memory"); \
        else asm volatile("global_load_dword %0, %1, %2" : "=v"(fq_nxt[t]) : "v"(s_off), "s"((sq_) + t * sq_t) : "memory"); \
    if (SF == 1) asm volatile("global_load_ubyte %0, %1, %2" : "=v"(fpb_nxt) : "v"(zero_off), "s"(sp_) : "memory"); \
    else asm volatile("global_load_dword %0, %1, %2" : "=v"(fpb_nxt) : "v"(zero_off), "s"(sp_) : "memory");
#define PF8_PFRAG(ps_) ld_frag_lds(pbase + fp_ofs[0] + (ps_) * 2048, pbase + fp_ofs[1] + (ps_) * 2048)
#define PF8_QFRAG(qs_) ld_frag_lds(pbase + fq_ofs[0] + (qs_) * 2048, pbase + fq_ofs[1] + (qs_) * 2048)

    i32x8 pf[4], qf[4];
    {
        // fill: blocks 0 and 1 of the first tile
#pragma unroll
        for (int i = 0; i < 12; ++i) PF8_COPY(i, c_ptile, c_qtile, 0);
        PF8_LOAD_S(c_sq0, c_spb)
#pragma unroll
        for (int i = 0; i < 12; ++i) PF8_COPY(i, c_ptile + 128, c_qtile + 128, 1);
        asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)"
                     : "+v"(fq_nxt[0]), "+v"(fq_nxt[1]), "+v"(fq_nxt[2]), "+v"(fq_nxt[3]), "+v"(fpb_nxt) : : "memory");
        __syncthreads();
        const uint8_t* pbase = lds;
        pf[0] = PF8_PFRAG(0);
        qf[0] = PF8_QFRAG(0);
        qf[1] = PF8_QFRAG(1);
        pf[1] = PF8_PFRAG(1);
        qf[2] = PF8_QFRAG(2);
    }
    int cur = 0;
    for (int64_t n = 0;; ++n) {
        // coordinates of the next tile; its expert id is fetched by a scalar load that is waited for on
        // the spot (once per tile), and its addresses are formed at the head of block 1
        const bool n_valid = tile_coords(n + 1, nq, np);
        int ne = 0;
        if (n_valid && grouped) asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ne) : "s"(a.m_indices + nq * BQ) : "memory");
        const int ne_rows = t_rows;
        if (masked) ne = t_e;
#pragma unroll
        for (int i = 0; i < NPS; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

        for (int64_t kb = 0; kb < KB; ++kb) {
            if (kb == 1) {
                if (n_valid) {
                    n_rows = ne < 0 ? 0 : (masked ? ne_rows : BQ);
                    const int e = ne < 0 ? 0 : ne;
                    n_ptile = a.p + ((int64_t)e * a.Prows + p_row0(np)) * a.red;
                    n_qtile = a.q + nq * BQ * a.red;
                    n_spb = sp_base + ((int64_t)e * PB + (FUSE ? np + wp * IB : p_row0(np) / 128 + wp)) * KB;
                    n_sq0 = SQL == 0 ? sq_base + (nq * BQ + wq * 64) * KB : sq_base + nq * BQ + wq * 64;
                } else {
                    // past the last tile the copies and scale loads re-read this tile's first blocks:
                    // the same instruction count in every block keeps the vmcnt arithmetic fixed
                    n_ptile = c_ptile; n_qtile = c_qtile; n_spb = c_spb; n_sq0 = c_sq0; n_rows = 0;
                }
            }
            float fq_cur[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                fq_cur[t] = SF == 1 ? e8m0_to_f32(f2u(fq_nxt[t])) * e8m0_to_f32(f2u(fpb_nxt)) : fq_nxt[t] * fpb_nxt;
            const int nxt1 = cur == 2 ? 0 : cur + 1;         // stage of the next block
            const int nxt2 = cur >= 1 ? cur - 1 : cur + 2;   // stage the previous block used
            // scales of the next block, copies of the block after it: this tile's, or the next tile's
            const bool in1 = kb + 1 < KB, in2 = kb + 2 < KB;
            const ST* s_sq = in1 ? c_sq0 + (kb + 1) * sq_k : n_sq0;
            const ST* s_sp = in1 ? c_spb + (kb + 1) : n_spb;
            const uint8_t* cp_p = in2 ? c_ptile + (kb + 2) * 128 : n_ptile + (kb + 2 - KB) * 128;
            const uint8_t* cp_q = in2 ? c_qtile + (kb + 2) * 128 : n_qtile + (kb + 2 - KB) * 128;
            PF8_LOAD_S(s_sq, s_sp)
            const uint8_t* pbase = lds + cur * STAGE;
            const uint8_t* nbase = lds + nxt1 * STAGE;
            f32x4 d[3];
            qf[3] = PF8_QFRAG(3);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NPS * 4; ++j) {
                const int ps = j < 24 ? (j >> 2) : 6 + (j & 1), qs = j < 24 ? (j & 3) : ((j - 24) >> 1);
                if (j == 24) {
                    // every fragment read of this block has been issued (the last at MFMA 20): once
                    // they have returned, and this wavefront's copies of the next block with them,
                    // meet the other wavefronts
                    asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)"
                                 : "+v"(fq_nxt[0]), "+v"(fq_nxt[1]), "+v"(fq_nxt[2]), "+v"(fq_nxt[3]), "+v"(fpb_nxt) : : "memory");
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                }
                d[j % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ps % 4], qf[qs], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (j < 24 && qs == 0 && ps + 2 < NPS) {
                    pf[(ps + 2) % 4] = PF8_PFRAG(ps + 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if ((j & 1) == 1 && j < 24) {
                    // no branch here: control flow inside the MFMA sequence lets the compiler sink
                    // the scale-FMAs out of it
                    PF8_COPY(j >> 1, cp_p, cp_q, nxt2);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the next block's first fragments, from the stage that has just been declared landed
                if (j == 24) { pf[0] = ld_frag_lds(nbase + fp_ofs[0], nbase + fp_ofs[1]); __builtin_amdgcn_sched_barrier(0); }
                if (j == 25) { qf[0] = ld_frag_lds(nbase + fq_ofs[0], nbase + fq_ofs[1]); __builtin_amdgcn_sched_barrier(0); }
                if (j == 26) { pf[1] = ld_frag_lds(nbase + fp_ofs[0] + 2048, nbase + fp_ofs[1] + 2048); __builtin_amdgcn_sched_barrier(0); }
                if (j == 27) { qf[1] = ld_frag_lds(nbase + fq_ofs[0] + 2048, nbase + fq_ofs[1] + 2048); __builtin_amdgcn_sched_barrier(0); }
                if (j == 29) { qf[2] = ld_frag_lds(nbase + fq_ofs[0] + 4096, nbase + fq_ofs[1] + 4096); __builtin_amdgcn_sched_barrier(0); }
                if (j >= 2) {
                    const int jj = j - 2;
                    const int pj = jj < 24 ? (jj >> 2) : 6 + (jj & 1), qj = jj < 24 ? (jj & 3) : ((jj - 24) >> 1);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[pj][qj][r] = __builtin_fmaf(d[jj % 3][r], fq_cur[qj], acc[pj][qj][r]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int jj = NPS * 4 - 2; jj < NPS * 4; ++jj) {
                const int pj = 6 + (jj & 1), qj = (jj - 24) >> 1;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[pj][qj][r] = __builtin_fmaf(d[jj % 3][r], fq_cur[qj], acc[pj][qj][r]);
            }
            __builtin_amdgcn_sched_barrier(0);
            cur = nxt1;
        }

        // ---- epilogue of this tile.  Its last block's stage is free: every wavefront passed that
        // block's barrier with its fragment reads returned, and no copy targets the stage before the
        // next block starts.  Each wavefront stages 32 of its 64 rows at a time in a private slice
        // (LDS operations of one wavefront execute in order) and stores whole 256-byte rows.
        if (FUSE) {
            constexpr int EP_LD = 272;                   // 128 bf16 per row + 16 B pad
            const int last = cur == 0 ? 2 : cur - 1;
            uint8_t* ep0 = lds + last * STAGE;
            uint8_t* ep = ep0 + wave * (32 * EP_LD);                             // this wavefront's rows: gate (wp = 0) or up (wp = 1)
            const uint8_t* ep_g = ep0 + (wq * 2) * (32 * EP_LD);                 // the pair's gate rows
            const uint8_t* ep_u = ep0 + (wq * 2 + 1) * (32 * EP_LD);             // the pair's up rows
            uint8_t* outb = reinterpret_cast<uint8_t*>(a.out);
            const int er = lane >> 4, ec = lane & 15;
            const int64_t col = (wp ? a.inter : 0) + cp * 128 + ec * 8;          // column of o1
            const bool has_p = a.probs != nullptr;
            const ExpPoly poly = exp_poly_in_registers();
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int qh = 0; qh < 2; ++qh) {
                    const int qs = half * 2 + qh;
#pragma unroll
                    for (int ps = 0; ps < NPS; ++ps) {
                        uint2 o;
                        o.x = pack_bf16(acc[ps][qs][0], acc[ps][qs][1]);
                        o.y = pack_bf16(acc[ps][qs][2], acc[ps][qs][3]);
                        *reinterpret_cast<uint2*>(ep + (qh * 16 + li) * EP_LD + (ps * 16 + 4 * kg) * 2) = o;
                    }
                }
                if (outb) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int rl = er + 4 * i;
                        const int64_t row = cq * BQ + wq * 64 + half * 32 + rl;
                        const uint4 v = *reinterpret_cast<const uint4*>(ep + rl * EP_LD + ec * 16);
                        if (c_rows) st16(outb + (row * a.ldo + col) * 2, v);
                    }
                }
                __syncthreads();      // the pair's gate and up rows are both staged
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int rl = wp * 16 + it * 4 + er;                         // this wavefront's 16 of the pass's 32 rows
                    const int64_t row = cq * BQ + wq * 64 + half * 32 + rl;
                    const uint4 wg = *reinterpret_cast<const uint4*>(ep_g + rl * EP_LD + ec * 16);
                    const uint4 wu = *reinterpret_cast<const uint4*>(ep_u + rl * EP_LD + ec * 16);
                    const float pr = has_p ? a.probs[row] : 1.0f;
                    // as in k_swiglu_quant: products rounded to bf16 in pairs, amax on the packed magnitudes
                    const uint32_t gw[4] = {wg.x, wg.y, wg.z, wg.w}, uw[4] = {wu.x, wu.y, wu.z, wu.w};
                    uint32_t pk[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        uint32_t w = pack_bf16(silu_exact(bf16_lo(gw[i]), poly) * bf16_lo(uw[i]), silu_exact(bf16_hi(gw[i]), poly) * bf16_hi(uw[i]));
                        pk[i] = pack_bf16(bf16_lo(w) * pr, bf16_hi(w) * pr);         // pr = 1 without probabilities: the product is exact
                    }
                    const uint32_t m = pkmax_u16(pkmax_u16(pk[0] & 0x7FFF7FFFu, pk[1] & 0x7FFF7FFFu), pkmax_u16(pk[2] & 0x7FFF7FFFu, pk[3] & 0x7FFF7FFFu));
                    const TileScale t = make_scale(row16_max(umax(m << 16, m & 0xFFFF0000u)), (a.pow2_out & 1) != 0);
                    float v[8];
                    unpack8(make_uint4(pk[0], pk[1], pk[2], pk[3]), v);
                    const uint2 o = quant8(v, t);
                    if (c_rows) {
                        st8(a.q2 + row * a.inter + cp * 128 + ec * 8, o);
                        if (ec == 0) {
                            if (a.pow2_out & 2) a.s2[(int64_t)cp * a.Qrows + row] = t.s;      // scales stored [I/128, rows]
                            else a.s2[row * IB + cp] = t.s;
                        }
                    }
                }
                if (half == 0) __syncthreads();      // everyone has read the first pass's rows before they are overwritten
            }
        } else {
            constexpr int EP_LD = 272;                   // 128 bf16 per row + 16 B pad
            const int last = cur == 0 ? 2 : cur - 1;
            uint8_t* ep = lds + last * STAGE + wave * (32 * EP_LD);
            uint8_t* outb = reinterpret_cast<uint8_t*>(a.out);
            const int er = lane >> 4, ec = lane & 15;
            const int64_t col = p_row0(cp) + wp * 128 + ec * 8;
            const bool store = c_rows && !(cp * 256 > p_last0 && wp == 0);     // not a padding tile, not the repeated half of a last half tile
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int qh = 0; qh < 2; ++qh) {
                    const int qs = half * 2 + qh;
#pragma unroll
                    for (int ps = 0; ps < NPS; ++ps) {
                        uint2 o;
                        o.x = pack_bf16(acc[ps][qs][0], acc[ps][qs][1]);
                        o.y = pack_bf16(acc[ps][qs][2], acc[ps][qs][3]);
                        *reinterpret_cast<uint2*>(ep + (qh * 16 + li) * EP_LD + (ps * 16 + 4 * kg) * 2) = o;
                    }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int rl = er + 4 * i;                        // row inside the 32-row slice
                    const int64_t row = cq * BQ + wq * 64 + half * 32 + rl;
                    const uint4 v = *reinterpret_cast<const uint4*>(ep + rl * EP_LD + ec * 16);
                    if (store && (!masked || rl < c_rows - wq * 64 - half * 32)) st16(outb + (row * a.ldo + col) * 2, v);
                }
            }
        }
        if (!n_valid) break;
        __syncthreads();   // the staging slices are dead before any copy of the next block lands there
        cq = nq; cp = np; c_rows = n_rows;
        c_ptile = n_ptile; c_qtile = n_qtile; c_spb = n_spb; c_sq0 = n_sq0;
    }
    __builtin_amdgcn_s_waitcnt(0);   // the copies issued past the end must land before the LDS is released
#undef PF8_COPY
#undef PF8_LOAD_S
#undef PF8_PFRAG
#undef PF8_QFRAG
}

// ---------------------------------------------------------------------------------------------
// Weight-gradient kernel: out[Q rows, P rows] (+)= Q . P^T with BOTH operands 1x128-scaled along the
// reduction axis, fp32 output.  128(Q) x 128(P) x 128(K) tiles, 256 threads = 4 wavefronts (2 x 2,
// 64x64 each), two double-buffered 32 KB LDS stages (64 KB: two workgroups per compute unit), the
// same global->LDS copies, fragment order and pinned MFMA/FMA interleave as the forward kernel.
// Every product needs two scales, sq[row] * sp[col], so eight VALU operations follow each MFMA
// (one multiply and one FMA per element): this kernel is bound by the vector ALU at about half
// the MFMA rate, and on the grouped layout by the fp32 read-modify-write of the gradients.
// The per-lane scales of the next K block are loaded BEFORE that block's copies are issued: vector
// memory operations complete in order, so a scale load issued after the copies would make every
// later wait on it wait for the copies as well.
// ---------------------------------------------------------------------------------------------
template <bool POW2>
__global__ __launch_bounds__(256, 2) void k_gemm_wgrad(const GemmArgs a) {
    constexpr int NPS = 4, STAGE = 32768, Q_OFS = 16384;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wq = wave >> 1, wp = wave & 1;
    const int li = lane & 15, kg = lane >> 4;

    // (tile arithmetic in 32 bits: the host admits at most 2^31 tiles, and 64-bit divisions are hundreds of dependent scalar
    // instructions in front of every tile)
    const uint32_t p_tiles = (uint32_t)((a.Prows + 127) / 128), q_tiles = (uint32_t)((a.Qrows + 127) / 128);
    const uint32_t T = p_tiles * q_tiles;
    const uint32_t per_xcd = (T + 7u) / 8u;
    const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (logical >= T) return;
    // tiles are walked in strips eight P tiles wide, P fastest inside a strip: the 64 workgroups an XCD
    // runs at a time then cover about 8 x 8 tiles and share 16 operand panels in its L2 instead of 34
    const uint32_t strip_w = 8u * q_tiles, strip = logical / strip_w, in_strip = logical - strip * strip_w;
    const uint32_t strip_p = p_tiles - strip * 8u < 8u ? p_tiles - strip * 8u : 8u;
    const uint32_t q_tile32 = in_strip / strip_p;
    const int64_t p_tile = strip * 8u + (in_strip - q_tile32 * strip_p), q_tile = q_tile32;
    const int64_t p0 = p_tile * 128, q0 = q_tile * 128;

    const uint8_t* pbase = a.p;
    const uint8_t* qbase = a.q;
    const float* spb = a.sp;
    const float* sqb = a.sq;
    uint8_t* outb = reinterpret_cast<uint8_t*>(a.out);
    int64_t ld = a.red;             // row stride of both operands = reduction length
    int64_t KB = a.red / 128;
    if (a.group == GROUP_WGRAD) {
        const int e = blockIdx.y;
        if ((a.wgrad_skip[e >> 5] >> (e & 31)) & 1u) return;
        const int64_t t0 = a.tile_start[e], t1 = a.tile_start[e + 1];
        // packed per-expert operands: [rows, M_e] at rows*128*t0, scales [M_e/128, rows] at t0*rows
        pbase += a.Prows * 128 * t0;
        qbase += a.Qrows * 128 * t0;
        spb += t0 * a.Prows;
        sqb += t0 * a.Qrows;
        outb += (int64_t)e * a.Qrows * a.ldo * 4;
        ld = (t1 - t0) * 128;
        KB = t1 - t0;
        if (KB == 0 && a.accumulate) return;
    }

    const int crow = lane >> 3, cpos = lane & 7;
    uint32_t p_src[4], q_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (i * 4 + wave) * 8 + crow;             // 0..127
        const int chunk = cpos ^ swz_key(row);
        int64_t pr = p0 + row; if (pr > a.Prows - 1) pr = a.Prows - 1;
        int64_t qr = q0 + row; if (qr > a.Qrows - 1) qr = a.Qrows - 1;
        p_src[i] = (uint32_t)((pr - p0) * ld + chunk * 16);
        q_src[i] = (uint32_t)((qr - q0) * ld + chunk * 16);
    }
    const uint8_t* ptile = pbase + p0 * ld;
    const uint8_t* qtile = qbase + q0 * ld;
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    int fp_ofs[2], fq_ofs[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        fp_ofs[h] = swz(wp * 64 + li, 2 * kg + h);
        fq_ofs[h] = Q_OFS + swz(wq * 64 + li, 2 * kg + h);
    }
    // scale addresses: one Q row per q sub-tile, four consecutive P rows per p sub-tile
    const float* sq_ptr[4];
    const float* sp_ptr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        int64_t r = q0 + wq * 64 + t * 16 + li;
        if (r > a.Qrows - 1) r = a.Qrows - 1;
        sq_ptr[t] = sqb + r;
        int64_t c = p0 + wp * 64 + t * 16 + 4 * kg;
        if (c > a.Prows - 4) c = a.Prows - 4;
        sp_ptr[t] = spb + c;
    }

    // POW2: the block-scaled MFMA wants, from lane l, the scale of A row l % 16 (a P row) and of B
    // column l % 16 (a Q row): one scalar per fragment and lane on both sides
    const float* sp1_ptr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        int64_t c = p0 + wp * 64 + t * 16 + li;
        if (c > a.Prows - 1) c = a.Prows - 1;
        sp1_ptr[t] = spb + c;
    }

    f32x4 acc[NPS][4];
#pragma unroll
    for (int i = 0; i < NPS; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float fq_nxt[4], fp1_nxt[4];
    f32x4 fp_nxt[4];

#define PF8_DMA(kb_, stage_)                                                                           \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                      \
        dma16_to_lds(ptile + p_src[i] + (kb_) * 128, lds_base + (stage_) * STAGE + (i * 4 + wave) * 1024); \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                      \
        dma16_to_lds(qtile + q_src[i] + (kb_) * 128, lds_base + (stage_) * STAGE + Q_OFS + (i * 4 + wave) * 1024);
#define PF8_LOAD_S(kb_)                                                                                \
    _Pragma("unroll") for (int t = 0; t < 4; ++t) {                                                    \
        fq_nxt[t] = sq_ptr[t][(kb_) * a.Qrows];                                                        \
        if (POW2) fp1_nxt[t] = sp1_ptr[t][(kb_) * a.Prows];                                            \
        else fp_nxt[t] = *reinterpret_cast<const f32x4*>(sp_ptr[t] + (kb_) * a.Prows);                 \
    }
#define PF8_PFRAG(ps_) ld_frag_lds(base + fp_ofs[0] + (ps_) * 2048, base + fp_ofs[1] + (ps_) * 2048)
#define PF8_QFRAG(qs_) ld_frag_lds(base + fq_ofs[0] + (qs_) * 2048, base + fq_ofs[1] + (qs_) * 2048)

    if (KB > 0) {
        PF8_LOAD_S(0)
        __builtin_amdgcn_sched_barrier(0);
        PF8_DMA(0, 0)
    }
    for (int64_t kb = 0; kb < KB; ++kb) {
        const int cur = (int)(kb & 1);
        __builtin_amdgcn_s_waitcnt(0);   // this wave's copies and scale loads have landed
        __syncthreads();                 // everyone's copies landed; everyone is done with stage cur^1
        float fq_cur[4];
        f32x4 fp_cur[4];
        int eq_cur[4], ep_cur[4];      // POW2: the scales' exponent fields = UE8M0 bytes
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            fq_cur[t] = fq_nxt[t];
            if (POW2) { eq_cur[t] = (int)(f2u(fq_nxt[t]) >> 23); ep_cur[t] = (int)(f2u(fp1_nxt[t]) >> 23); }
            else fp_cur[t] = fp_nxt[t];
        }
        const int64_t kbn = kb + 1 < KB ? kb + 1 : kb;
        PF8_LOAD_S(kbn)
        __builtin_amdgcn_sched_barrier(0);
        PF8_DMA(kbn, cur ^ 1)
        const uint8_t* base = lds + cur * STAGE;
        i32x8 pf[NPS], qf[4];
        f32x4 d[3];
        pf[0] = PF8_PFRAG(0);
        __builtin_amdgcn_sched_barrier(0);
        qf[0] = PF8_QFRAG(0);
        __builtin_amdgcn_sched_barrier(0);
        qf[1] = PF8_QFRAG(1);
        __builtin_amdgcn_sched_barrier(0);
        qf[2] = PF8_QFRAG(2);
        __builtin_amdgcn_sched_barrier(0);
        qf[3] = PF8_QFRAG(3);
        __builtin_amdgcn_sched_barrier(0);
        pf[1] = PF8_PFRAG(1);
        __builtin_amdgcn_sched_barrier(0);
        pf[2] = PF8_PFRAG(2);
        __builtin_amdgcn_sched_barrier(0);
        pf[3] = PF8_PFRAG(3);
        __builtin_amdgcn_sched_barrier(0);
        if (POW2) {
            // both operands' power-of-two scales go into the MFMA, which accumulates the block itself
#pragma unroll
            for (int j = 0; j < NPS * 4; ++j) {
                const int ps = j >> 2, qs = j & 3;
                acc[ps][qs] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ps], qf[qs], acc[ps][qs], 0, 0, 0, ep_cur[ps], 0, eq_cur[qs]);
                __builtin_amdgcn_sched_barrier(0);
            }
            continue;
        }
#pragma unroll
        for (int j = 0; j < NPS * 4; ++j) {
            const int ps = j >> 2, qs = j & 3;
            d[j % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ps], qf[qs], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (j >= 2) {
                const int jj = j - 2;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[jj >> 2][jj & 3][r] = __builtin_fmaf(d[jj % 3][r] * fq_cur[jj & 3], fp_cur[jj >> 2][r], acc[jj >> 2][jj & 3][r]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#pragma unroll
        for (int jj = NPS * 4 - 2; jj < NPS * 4; ++jj)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                acc[jj >> 2][jj & 3][r] = __builtin_fmaf(d[jj % 3][r] * fq_cur[jj & 3], fp_cur[jj >> 2][r], acc[jj >> 2][jj & 3][r]);
    }
    __builtin_amdgcn_s_waitcnt(0);

    // ---- epilogue: fp32 through LDS so that every load/store instruction touches whole 256-byte
    // rows of the gradient; optional read-modify-write ----
    constexpr int EP_LD = 272;                   // 64 fp32 per row + 16 B pad
    __syncthreads();                             // everyone is done reading fragments
    uint8_t* ep = lds + wave * (64 * EP_LD);
#pragma unroll
    for (int qs = 0; qs < 4; ++qs)
#pragma unroll
        for (int ps = 0; ps < NPS; ++ps)
            *reinterpret_cast<f32x4*>(ep + (qs * 16 + li) * EP_LD + (ps * 16 + 4 * kg) * 4) = acc[ps][qs];
    const int er = lane >> 4, ec = lane & 15;
    const int64_t col = p0 + wp * 64 + ec * 4;
    const bool col_ok = col + 4 <= a.Prows;
    const int64_t col_c = col_ok ? col : a.Prows - 4;
    // read-modify-write: all 16 loads of the old gradient rows are in flight before the first add
    // (one load-add-store round trip per row would cost sixteen memory latencies per tile)
    f32x4 old[16];
    if (a.accumulate) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int64_t row = q0 + wq * 64 + er + 4 * i;
            if (row > a.Qrows - 1) row = a.Qrows - 1;
            { const uint4 ow = ld16(outb + (row * a.ldo + col_c) * 4); old[i] = (f32x4){u2f(ow.x), u2f(ow.y), u2f(ow.z), u2f(ow.w)}; }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) old[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t row = q0 + wq * 64 + er + 4 * i;
        const f32x4 v = *reinterpret_cast<const f32x4*>(ep + (er + 4 * i) * EP_LD + ec * 16);
        const f32x4 o = (f32x4){old[i].x + v.x, old[i].y + v.y, old[i].z + v.z, old[i].w + v.w};
        if (row < a.Qrows && col_ok) st16(outb + (row * a.ldo + col) * 4, make_uint4(f2u(o.x), f2u(o.y), f2u(o.z), f2u(o.w)));
    }
#undef PF8_DMA
#undef PF8_LOAD_S
#undef PF8_PFRAG
#undef PF8_QFRAG
}

static int launch_gemm(const GemmArgs& a, int mode, dim3 grid, hipStream_t st, const char* where) {
    const size_t lds_bytes = 69632;   // two 32 KB stages; the fp32 epilogue staging needs 4 x 64 x 272 B
    if (mode == MODE_FWD) {
        const int64_t T128 = ((a.Prows + 255) / 256) * ((a.Qrows + 127) / 128);
        // the grid is padded to a multiple of 8 so that every XCD gets an equal run of tiles
        dim3 g128((unsigned)(((T128 + 7) / 8) * 8), grid.y);
        // The persistent deep-pipeline kernel takes every shape it can tile (128-row tiles, 256-column tiles of which the
        // last may be half new, at least three K blocks; dense, contiguous-grouped or masked).  Measured on MI355X
        // against the two-workgroup kernel: +14..24% when all tiles fit one round of compute units, +21% / +8% on the
        // up+gate / down GEMMs of 32 experts with a skewed 8192-row load, +2% on those of 128 experts with 131072 rows,
        // within 3% either way on dense products from 3 to 64 K blocks and up to 32 rounds of tiles.
        const bool aligned = a.Prows % 128 == 0 && a.Prows >= 256 && a.Qrows % 128 == 0 && a.red >= 384 &&
                             (a.group != GROUP_MASKED || (a.E <= kDeepMaskedExperts && (int64_t)a.E * (a.Qrows / 128) <= kDeepSegTiles));
        const int64_t cus = pf8_effective_cus();
        const bool deep = aligned;
        if (a.group == GROUP_MASKED && !aligned && a.Prows % 128 == 0 && a.Prows >= 256 && a.Qrows % 128 == 0 && a.red >= 384)
            pf8_note_once(PF8_NOTE_MASKED_TABLE, "masked grouped GEMM beyond 256 experts or 2048 row tiles: taking the two-workgroup kernel "
                                                 "(one grid row per expert) instead of the persistent one");
        if (deep && a.group == GROUP_CONTIG && a.Qrows / 128 > kDeepSegTiles)
            pf8_note_once(PF8_NOTE_GROUPED_ORDER, "contiguous grouped GEMM with more than 2048 row tiles: tiles are walked in plain groups of 16 "
                                                  "row tiles instead of expert by expert (more weight re-reads per XCD)");
        if (deep) {
            // persistent: one workgroup per compute unit (or per tile of an XCD's run, if fewer); the masked layout is
            // one launch over all experts (the kernel walks the row tiles that hold valid rows)
            const int64_t per_xcd = (T128 * (a.group == GROUP_MASKED ? a.E : 1) + 7) / 8;
            int64_t w = cus / 8;
            if (w < 1) w = 1;
            if (w > per_xcd) w = per_xcd;
            dim3 gd((unsigned)(8 * w), 1);
            if (a.group == GROUP_MASKED) hipLaunchKernelGGL((k_gemm_fwd_deep<0, 0, 0, 1>), gd, dim3(256), kDeepDynLds, st, a);
            else if (a.sq_layout == 0) hipLaunchKernelGGL((k_gemm_fwd_deep<0>), gd, dim3(256), kDeepDynLds, st, a);
            else hipLaunchKernelGGL((k_gemm_fwd_deep<1>), gd, dim3(256), kDeepDynLds, st, a);
        } else {
            // under a compute-unit budget: two workgroups per budgeted unit, each walking several tiles
            if (pf8_cus_capped()) {
                int64_t w = 2 * cus / 8;
                if (w < 1) w = 1;
                if (8 * w < (int64_t)g128.x) g128.x = (unsigned)(8 * w);
            }
            if (a.sq_layout == 0) hipLaunchKernelGGL((k_gemm_fwd128<0>), g128, dim3(256), 81920, st, a);
            else hipLaunchKernelGGL((k_gemm_fwd128<1>), g128, dim3(256), 81920, st, a);
        }
    } else {
        const int64_t Tw = ((a.Prows + 127) / 128) * ((a.Qrows + 127) / 128);
        dim3 gw((unsigned)(((Tw + 7) / 8) * 8), grid.y);
        if (a.pow2_scales) hipLaunchKernelGGL(k_gemm_wgrad<true>, gw, dim3(256), lds_bytes, st, a);
        else hipLaunchKernelGGL(k_gemm_wgrad<false>, gw, dim3(256), lds_bytes, st, a);
    }
    return pf8_check_launch(where);
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

static int ensure_lds_attr() {
    // more than 64 KB of dynamic LDS needs the opt-in attribute, once per kernel instantiation and device
    // (a bit per device; two threads racing here both set the same attributes, which is harmless)
    static std::atomic<uint64_t> done{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, "pf8_gemm", hipGetErrorString(e));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return PF8_OK;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_wgrad<false>), hipFuncAttributeMaxDynamicSharedMemorySize, 69632);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_wgrad<true>), hipFuncAttributeMaxDynamicSharedMemorySize, 69632);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd128<0>), hipFuncAttributeMaxDynamicSharedMemorySize, 81920);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd128<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 81920);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<0>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<1>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<1, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<0, 0, 0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<0, 0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fwd_deep<1, 0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kDeepDynLds);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, "pf8_gemm", hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return PF8_OK;
}

int pf8_launch_deep_ue8m0(const uint8_t* p, const uint8_t* q, const uint8_t* sp8, const uint8_t* sq8, int64_t ldsq, void* out,
                          int64_t Prows, int64_t Qrows, int64_t red, int E, const int32_t* m_indices, const int32_t* pair_list,
                          int cus, hipStream_t stream, const char* where) {
    if (Prows % 256 != 0 || Qrows % 128 != 0 || red % 128 != 0 || red < 384) return pf8_fail(PF8_EINVAL, where, "shape outside the persistent kernel's tiling");
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = p; g.q = q; g.sp = reinterpret_cast<const float*>(sp8); g.sq = reinterpret_cast<const float*>(sq8); g.out = out;
    g.Prows = Prows; g.Qrows = Qrows; g.red = red; g.ldo = Prows; g.sq_layout = 1; g.group = GROUP_CONTIG; g.E = E;
    g.m_indices = m_indices; g.ldsq = ldsq; g.pair_list = pair_list; g.cus = cus;
    const int64_t T128 = (Prows / 256) * (Qrows / 128), per_xcd = (T128 + 7) / 8;
    int64_t w = cus / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    hipLaunchKernelGGL((k_gemm_fwd_deep<1, 1>), dim3((unsigned)(8 * w)), dim3(256), kDeepDynLds, stream, g);
    return pf8_check_launch(where);
}

extern "C" int pf8_gemm_nt(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b, const float* sb, int64_t M,
                           int64_t N, int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0, "K must be a multiple of 128");
    PF8_REQUIRE(N % 4 == 0, "N must be a multiple of 4");
    if (M == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && out, "null pointer");
    PF8_REQUIRE(ldo >= N && ldo % 4 == 0, "ldo must be >= N and a multiple of 4");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b; g.q = a; g.sp = sb; g.sq = sa; g.out = out;
    g.Prows = N; g.Qrows = M; g.red = K; g.ldo = ldo; g.sq_layout = sa_layout; g.group = GROUP_NONE;
    const int64_t tiles = ((N + 127) / 128) * ((M + 127) / 128);
    PF8_REQUIRE(tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_FWD, dim3((unsigned)tiles), (hipStream_t)stream, __func__);
}

extern "C" int pf8_grouped_gemm_nt_contiguous(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b, const float* sb,
                                              int E, int64_t Mtot, int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out,
                                              pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Mtot >= 0 && N >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0, "K must be a multiple of 128");
    PF8_REQUIRE(N % 4 == 0, "N must be a multiple of 4");
    PF8_REQUIRE(Mtot % 128 == 0, "Mtot must be a multiple of 128 (expert segments are padded to 128 rows)");
    if (Mtot == 0 || N == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && out && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b; g.q = a; g.sp = sb; g.sq = sa; g.out = out;
    g.Prows = N; g.Qrows = Mtot; g.red = K; g.ldo = N; g.sq_layout = sa_layout; g.group = GROUP_CONTIG; g.E = E;
    g.m_indices = m_indices;
    const int64_t tiles = ((N + 127) / 128) * (Mtot / 128);
    PF8_REQUIRE(tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_FWD, dim3((unsigned)tiles), (hipStream_t)stream, __func__);
}

extern "C" int pf8_grouped_gemm_swiglu_quant_nt_contiguous(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b,
                                                           const float* sb, int E, int64_t Mtot, int64_t I, int64_t K,
                                                           const int32_t* m_indices, const float* probs, uint16_t* o1, uint8_t* q,
                                                           float* s, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Mtot >= 0 && I >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0 && K >= 384, "K must be a multiple of 128 and at least 384");
    PF8_REQUIRE(I % 128 == 0, "I must be a multiple of 128");
    PF8_REQUIRE(Mtot % 128 == 0, "Mtot must be a multiple of 128 (expert segments are padded to 128 rows)");
    if (Mtot == 0 || I == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && q && s && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && PF8_ALIGNED16(o1) && (reinterpret_cast<uintptr_t>(q) & 7u) == 0,
                "a, b, o1 must be 16-byte aligned and q 8-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    PF8_REQUIRE(K <= (1ll << 24) && I <= (1ll << 24), "shape too large");
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b; g.q = a; g.sp = sb; g.sq = sa; g.out = o1;
    g.Prows = 2 * I; g.Qrows = Mtot; g.red = K; g.ldo = 2 * I; g.sq_layout = sa_layout; g.group = GROUP_CONTIG; g.E = E;
    g.m_indices = m_indices;
    g.inter = I; g.probs = probs; g.q2 = q; g.s2 = s; g.pow2_out = pow2;
    const int64_t T128 = (I / 128) * (Mtot / 128), per_xcd = (T128 + 7) / 8;
    PF8_REQUIRE(T128 <= 0x7FFFFFFF, "too many tiles");
    int64_t w = pf8_effective_cus() / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    dim3 gd((unsigned)(8 * w), 1);
    if (sa_layout == 0) hipLaunchKernelGGL((k_gemm_fwd_deep<0, 0, 1>), gd, dim3(256), kDeepDynLds, (hipStream_t)stream, g);
    else hipLaunchKernelGGL((k_gemm_fwd_deep<1, 0, 1>), gd, dim3(256), kDeepDynLds, (hipStream_t)stream, g);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_grouped_gemm_nt_masked(const uint8_t* a, const float* sa, const uint8_t* b, const float* sb, int E, int64_t Mmax,
                                          int64_t N, int64_t K, const int32_t* masked_m, int expected_m, uint16_t* out,
                                          pf8_stream_t stream) {
    (void)expected_m;   // scheduling hint in the reference API; the grid covers Mmax and exits early
    PF8_REQUIRE(E >= 0 && Mmax >= 0 && N >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0, "K must be a multiple of 128");
    PF8_REQUIRE(N % 4 == 0, "N must be a multiple of 4");
    PF8_REQUIRE(E <= 65535, "too many experts");
    if (Mmax == 0 || N == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(a && sa && b && sb && out && masked_m, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0, "pointers must be 16-byte aligned");
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b; g.q = a; g.sp = sb; g.sq = sa; g.out = out;
    g.Prows = N; g.Qrows = Mmax; g.red = K; g.ldo = N; g.sq_layout = 0; g.group = GROUP_MASKED; g.E = E;
    g.masked_m = masked_m;
    const int64_t tiles = ((N + 127) / 128) * ((Mmax + 127) / 128);
    PF8_REQUIRE(tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_FWD, dim3((unsigned)tiles, (unsigned)E), (hipStream_t)stream, __func__);
}

#define PF8_REQUIRE_AT(where, cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, where, msg); } while (0)

static int gemm_nt_1d1d_f32(const char* where, const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                            int64_t Kin, int64_t N, int64_t M, float* out, int accumulate, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE_AT(where, Kin >= 0 && N >= 0 && M >= 0, "negative shape");
    PF8_REQUIRE_AT(where, M % 128 == 0, "M (the reduction axis) must be a multiple of 128");
    PF8_REQUIRE_AT(where, N % 4 == 0, "N must be a multiple of 4");
    if (Kin == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE_AT(where, out, "null pointer");
    PF8_REQUIRE_AT(where, M == 0 || (a_t && sa_t && b_t && sb_t), "null pointer");
    PF8_REQUIRE_AT(where, PF8_ALIGNED16(a_t) && PF8_ALIGNED16(b_t) && PF8_ALIGNED16(out) && PF8_ALIGNED16(sb_t), "pointers must be 16-byte aligned");
    if (M == 0 && accumulate) return PF8_OK;
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b_t; g.q = a_t; g.sp = sb_t; g.sq = sa_t; g.out = out;
    g.Prows = N; g.Qrows = Kin; g.red = M; g.ldo = N; g.accumulate = accumulate; g.group = GROUP_NONE; g.pow2_scales = pow2;
    const int64_t tiles = ((N + 127) / 128) * ((Kin + 127) / 128);
    PF8_REQUIRE_AT(where, tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_WGRAD, dim3((unsigned)tiles), (hipStream_t)stream, where);
}

extern "C" int pf8_gemm_nt_1d1d_f32(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t, int64_t Kin,
                                    int64_t N, int64_t M, float* out, int accumulate, pf8_stream_t stream) {
    return gemm_nt_1d1d_f32(__func__, a_t, sa_t, b_t, sb_t, Kin, N, M, out, accumulate, 0, stream);
}

extern "C" int pf8_gemm_nt_1d1d_f32_pow2(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t, int64_t Kin,
                                         int64_t N, int64_t M, float* out, int accumulate, pf8_stream_t stream) {
    return gemm_nt_1d1d_f32(__func__, a_t, sa_t, b_t, sb_t, Kin, N, M, out, accumulate, 1, stream);
}

static int grouped_wgrad(const char* where, const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                         const int64_t* rows_per_expert, int E, int64_t Kin, int64_t N, float* out, int accumulate, int pow2,
                         pf8_stream_t stream) {
    PF8_REQUIRE_AT(where, E >= 0 && Kin >= 0 && N >= 0, "negative shape");
    PF8_REQUIRE_AT(where, E <= 256, "at most 256 experts per call");
    PF8_REQUIRE_AT(where, N % 4 == 0, "N must be a multiple of 4");
    if (E == 0 || Kin == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE_AT(where, rows_per_expert && out, "null pointer");
    GemmArgs g = {};
    int64_t total = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE_AT(where, rows_per_expert[e] >= 0 && rows_per_expert[e] % 128 == 0, "rows_per_expert entries must be non-negative multiples of 128");
        g.tile_start[e] = (int32_t)(total / 128);
        total += rows_per_expert[e];
    }
    g.tile_start[E] = (int32_t)(total / 128);
    PF8_REQUIRE_AT(where, total == 0 || (a_t && sa_t && b_t && sb_t), "null pointer");
    PF8_REQUIRE_AT(where, PF8_ALIGNED16(a_t) && PF8_ALIGNED16(b_t) && PF8_ALIGNED16(out) && PF8_ALIGNED16(sb_t), "pointers must be 16-byte aligned");
    if (total == 0 && accumulate) return PF8_OK;
    int rc = ensure_lds_attr();
    if (rc) return rc;
    g.p = b_t; g.q = a_t; g.sp = sb_t; g.sq = sa_t; g.out = out;
    g.Prows = N; g.Qrows = Kin; g.red = 0; g.ldo = N; g.accumulate = accumulate; g.group = GROUP_WGRAD; g.E = E; g.pow2_scales = pow2;
    const int64_t tiles = ((N + 127) / 128) * ((Kin + 127) / 128);
    PF8_REQUIRE_AT(where, tiles <= 0x7FFFFFFF, "too many tiles");
    // The experts with a long reduction axis (power-of-two scales, shapes the 256x256 tile takes) go to the kernel that
    // holds the tile in the AGPR file, longest first; the others stay here, where two workgroups per compute unit
    // overlap one tile's gradient read-modify-write with the other's blocks.  Only when the long experts fill the
    // device at least once: a handful of 256x256 tiles would leave most compute units idle.
    const int min_blocks = pf8_wgrad_tile256_min_blocks();
    if (pow2 && min_blocks > 0 && N % 128 == 0 && N >= 256 && Kin % 128 == 0 && Kin >= 256 && PF8_ALIGNED16(sa_t) &&
        N * 128 * 4 <= 0x7FFFFFFFll) {
        int32_t t0[kWgE8MaxItems], kb[kWgE8MaxItems];
        uint8_t ex[kWgE8MaxItems];
        int n = 0;
        for (int e = 0; e < E; ++e) {
            const int32_t blocks = g.tile_start[e + 1] - g.tile_start[e];
            if (blocks < (min_blocks < 4 ? 4 : min_blocks) || (int64_t)blocks * 128 > (1ll << 24)) continue;
            int i = n++;
            for (; i > 0 && kb[i - 1] < blocks; --i) { t0[i] = t0[i - 1]; kb[i] = kb[i - 1]; ex[i] = ex[i - 1]; }   // longest first
            t0[i] = g.tile_start[e]; kb[i] = blocks; ex[i] = (uint8_t)e;
        }
        const int cus = pf8_effective_cus();
        const int64_t tiles256 = ((N + 255) / 256) * ((Kin + 255) / 256);
        if (n > 0 && tiles256 * n >= cus) {
            rc = pf8_launch_wgrad_e8(b_t, a_t, sb_t, sa_t, out, N, Kin, N, accumulate, n, t0, kb, ex, cus, (hipStream_t)stream, where);
            if (rc) return rc;
            if (n == E) return PF8_OK;
            for (int i = 0; i < n; ++i) g.wgrad_skip[ex[i] >> 5] |= 1u << (ex[i] & 31);
        }
    }
    return launch_gemm(g, MODE_WGRAD, dim3((unsigned)tiles, (unsigned)E), (hipStream_t)stream, where);
}

extern "C" int pf8_grouped_wgrad(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                                 const int64_t* rows_per_expert, int E, int64_t Kin, int64_t N, float* out, int accumulate,
                                 pf8_stream_t stream) {
    return grouped_wgrad(__func__, a_t, sa_t, b_t, sb_t, rows_per_expert, E, Kin, N, out, accumulate, 0, stream);
}

extern "C" int pf8_grouped_wgrad_pow2(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                                      const int64_t* rows_per_expert, int E, int64_t Kin, int64_t N, float* out, int accumulate,
                                      pf8_stream_t stream) {
    return grouped_wgrad(__func__, a_t, sa_t, b_t, sb_t, rows_per_expert, E, Kin, N, out, accumulate, 1, stream);
}
