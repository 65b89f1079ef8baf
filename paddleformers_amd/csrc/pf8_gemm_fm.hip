// pf8_gemm_fm.hip -- forward / dgrad block-scaled FP8 GEMM on FRAGMENT-MAJOR weights.
//
// The FP8 weights of this path are written by this library (the stacked-weight quantizers) and read only by its
// GEMMs, so their byte order is the library's to choose.  `pf8_weight_to_fragment_major` re-orders a quantized weight
// [E][N, K] into the order in which a wavefront's matrix instructions consume it:
//     wf[e][n / 64][k / 128][pf = 0..1][kh = 0..1][h = 0..1][lane = 0..63][16 bytes]
// where the 16 bytes are k = 128 kb + 64 kh + 32 (lane / 32) + 16 h .. + 15 of weight row n = 64 (n / 64) + 32 pf + lane % 32.
// The 8 KB of one (64-row panel, K block) are exactly the four A-operand fragments (32 rows x 64 k each) of
// v_mfma_f32_32x32x64_f8f6f4 that cover it, and consecutive K blocks of a panel are contiguous.
//
// With that order a wavefront fetches its weight fragments with whole 1 KB global loads STRAIGHT INTO REGISTERS: no
// LDS write, no LDS read, no swizzle, and a perfectly sequential stream per wavefront.  The registers are accumulation
// VGPRs (AGPRs): gfx950 loads into them directly and the MFMA takes its A operand from them, so a ring of three K blocks
// of weight fragments (96 AGPRs) costs no architectural VGPR, and the weights are prefetched two blocks ahead.
//
// Geometry: workgroup tile 128 (Q = activation rows) x 256 (P = weight rows) x 128 (K, one scale block), 256 threads =
// 4 wavefronts side by side along P: wavefront w owns weight rows [64 w, 64 w + 64) of the tile and ALL 128 activation
// rows, 2 x 4 MFMA tiles of 32 x 32 = 128 accumulator VGPRs.  No two wavefronts load the same weight byte.  Per K block
// a compute unit takes in 32 KB of weights (global -> AGPR) and 16 KB of activations (global -> LDS) and reads 64 KB of
// activation fragments from LDS: 80 KB of LDS traffic against the 144 KB of the kernels that stage both operands in LDS.
//
// Why the 32x32x64 instruction: a wavefront's instruction stream, not the matrix pipe, bounds the fp32-scale kernels.
// Every product element needs one VALU FMA (acc += product * sa * sb), i.e. 128 FMAs = 512 issue cycles per K block
// against 1024 cycles of matrix work, and issuing an MFMA costs the stream about 16 cycles whatever its shape.  Measured
// on one wavefront per SIMD: 16x16x128 (32 cycles of matrix work) followed by its 4 FMAs takes 39 cycles, 33 with three
// FMAs: no slack at all, every copy, LDS read or scalar instruction lengthens the block.  32x32x64 does twice the work
// per issue: with its 8 FMAs and the LDS reads of the loop it takes 66 cycles against 64, and 12 FMAs still fit.  A
// K block's product is two chained instructions (k 0..63, then k 64..127 accumulated onto it inside the matrix pipe).
//
//   * Activations go global -> LDS (global_load_lds_dwordx4) into a ring of three 16 KB stages.  Tile row r is stored in
//     LDS row 32 (r % 4) + r / 4, so fragment j (LDS rows 32 j .. 32 j + 31) holds tile rows 4 i + j and the four
//     activation scales a lane needs per block (rows 4 x .. 4 x + 3) are 16 contiguous bytes.
//   * The scales of a block travel with it: 128 activation scales and the two weight-block scales are copied into the
//     stage (global_load_lds_dword, one instruction per wavefront) and read from LDS after the barrier that declares
//     the stage landed.  Every memory instruction of the loop is therefore issued two blocks ahead of its use, and
//     the one counted wait per block (vmcnt(13): the block's own 13 instructions may stay in flight) never waits for
//     anything issued in the current block.  Vector loads retire in order, so a younger load a block needs early
//     would otherwise drag the whole prefetch queue with it.
//   * One barrier per block (before MFMA 12 of 16), behind it the first fragments and the scales of the next block
//     are read; all rings run on across tile boundaries.  The loop is unrolled by the three ring positions and a tile
//     may end at any of them, so K needs no particular divisibility.
//   * The MFMAs are inline assembly (the AGPR operand has to be named), so the compiler does not see them as matrix
//     instructions and inserts no wait states for their results.  The schedule provides them: the 16 FMAs of a product
//     follow the first and second MFMA issued behind it (products alternate between two register sets): the first
//     eight result registers are read one MFMA behind, the other eight two behind, which the measured write-back times
//     (in the loop) allow with four wait states to spare.  A block's last product is folded in behind the first two
//     MFMAs of the next block, and a tile's very last behind an explicit wait.
//   * Epilogue: each wavefront stages 32 rows x 64 columns of bf16 at a time in a private LDS slice and stores
//     128-byte row pieces.
// Needs Prows % 128 == 0 and Prows >= 256, Qrows % 128 == 0 and K % 128 == 0, K >= 384; dense and contiguous-grouped layouts.
#include <atomic>

#include "pf8_gemm_common.h"
#include "pf8_host.h"

namespace pf8 {

typedef float f32x16 __attribute__((ext_vector_type(16)));

struct FmArgs {
    const uint8_t* pf;     // fragment-major weights [E][Prows / 64][KB][8192]
    const uint8_t* q;      // activations [Qrows, red]
    const float* sp;       // [E][Prows / 128, KB]
    const float* sq;       // sq_layout 0: [Qrows, KB], 1: [KB, Qrows]
    uint16_t* out;         // bf16 [Qrows, ldo]
    int64_t Prows, Qrows, red, ldo;
    int grouped, E;
    const int32_t* m_indices;
    // GATHER instantiation: q is the token matrix [T, red] and output row r multiplies token src_row[r]; sq holds the scales
    // of the OUTPUT rows (gathered beforehand: 4 bytes per row and K block against 128), zero for a row whose src_row is
    // negative (a padding row: it reads token 0's bytes with a zero factor, its output is zero); Qrows counts output rows
    const int32_t* src_row;
    int64_t* cycles;       // TRACE instantiation only: [workgroups][8] cycle sums of wavefront 0 (see pf8_debug_grouped_gemm_fm_cycles)
};

constexpr int kFmSegTiles = 2048;                 // row tiles whose expert order is tabulated in LDS
constexpr int kFmStages = 3, kFmStage = 16384 + 1024, kFmEpLd = 144;
constexpr int kFmDynLds = kFmStages * kFmStage + 4 * 32 * kFmEpLd;

// AGPR ring: position S (block counter % 3) holds fragment (pf, kh), half h in a[32 S + 16 pf + 8 kh + 4 h .. + 3]
template <int A, int IMM>
__device__ __forceinline__ void fm_pload(uint32_t voff, const uint8_t* sbase) {
    asm volatile("global_load_dwordx4 a[%2:%3], %0, %1 offset:%4" : : "v"(voff), "s"(sbase), "n"(A), "n"(A + 3), "n"(IMM) : "memory");
}
// d = A . B (k 0..63 of the block)
template <int A>
__device__ __forceinline__ void fm_mfma_first(f32x16& d, const i32x8& q) {
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, a[%2:%3], %1, 0" : "=&v"(d) : "v"(q), "n"(A), "n"(A + 7));
}
// d += A . B (k 64..127), accumulated inside the matrix pipe
template <int A>
__device__ __forceinline__ void fm_mfma_second(f32x16& d, const i32x8& q) {
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, a[%2:%3], %1, %0" : "+v"(d) : "v"(q), "n"(A), "n"(A + 7));
}

template <int SQL, int TRACE = 0, int GATHER = 0>
__global__ __launch_bounds__(256, 1) void k_gemm_fm(const FmArgs a) {
    constexpr int BQ = 128;
    constexpr int STAGE = kFmStage, S_OFS = 16384, SP_OFS = 16384 + 512, EP_OFS = kFmStages * kFmStage, EP_LD = kFmEpLd;
    constexpr int BAR = 12;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    asm volatile("" ::: "a95");           // the kernel descriptor reserves a0..a95: the weight-fragment ring, named literally below
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int x = lane & 31, hh = lane >> 5;

    // a last column tile may be half new (Prows = 256 t + 128): it covers the LAST 256 weight rows, and the two wavefronts
    // that repeat the previous tile's columns store nothing
    const int64_t p_tiles = (a.Prows + 255) / 256, q_tiles = a.Qrows / BQ;
    const int64_t KB = a.red / 128, PB = a.Prows / 128, P64 = a.Prows / 64;
    const int64_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, W = gridDim.x >> 3;
    const bool grouped = a.grouped != 0;

    // Tile order (as in the other persistent kernels): every XCD owns a contiguous run of logical tiles, walked W at a
    // time by its W workgroups.  Grouped launches with at most kFmSegTiles row tiles cut every expert's run of row tiles
    // into groups of at most 12 (no group spans two experts) and walk a group's tiles q fastest, p slowest, so that the
    // workgroups of an XCD share one or two weight strips of ONE expert at a time.  seg_tab[q] = first tile of q's
    // group | tiles in it << 16, built by every workgroup for itself with a prefix maximum over the row tiles.
    __shared__ uint32_t seg_tab[kFmSegTiles];
    __shared__ int16_t seg_eid[kFmSegTiles + 2];
    __shared__ int seg_wave_max[2][4];
    static_assert(sizeof(seg_tab) + sizeof(seg_eid) + sizeof(seg_wave_max) + kFmDynLds <= 163840, "LDS budget");
    const bool ordered = grouped && q_tiles <= kFmSegTiles && a.E <= 32767;
    if (ordered) {
        constexpr int CAP = 12;
        const int qt = (int)q_tiles;
        for (int t = tid; t < qt; t += 256) {
            const int e = a.m_indices[(int64_t)t * BQ];
            seg_eid[t + 1] = (int16_t)(e < 0 ? -1 : e);
        }
        if (tid == 0) { seg_eid[0] = -2; seg_eid[qt + 1] = -2; }
        __syncthreads();
        int carry = 0;
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
            __syncthreads();
            int all = carry;
            for (int w = 0; w < 4; ++w) {
                const int m = seg_wave_max[par][w];
                if (w < wave && m > v) v = m;
                if (m > all) all = m;
            }
            if (carry > v) v = carry;
            carry = all;
            if (t < qt) {
                const int gs = v + (t - v) / CAP * CAP;
                int hi = t + 1;
                while (hi < gs + CAP && seg_eid[hi + 1] == e) ++hi;
                seg_tab[t] = (uint32_t)gs | (uint32_t)(hi - gs) << 16;
            }
        }
        __syncthreads();
    }
    const int64_t T = p_tiles * q_tiles;
    const int64_t per_xcd = (T + 7) / 8;
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
        return true;
    };

    // ---- per-lane constants
    // activation copy c (0..3) of wavefront w fills LDS rows (4 c + w) * 8 + (lane >> 3) = fragment c, fragment row
    // 8 w + (lane >> 3), i.e. tile row 32 w + 4 (lane >> 3) + c; the swizzle key of that LDS row is (lane >> 3) ^ (w & 1)
    const int crow = lane >> 3, cpos = lane & 7;
    const uint32_t q_chunk = (uint32_t)((cpos ^ (crow ^ (wave & 1))) << 4);
    const uint32_t q_off = (uint32_t)((32 * wave + 4 * crow) * a.red) + q_chunk;
    const int64_t q_cstep = a.red;
    const uint32_t p_voff0 = (uint32_t)lane * 16u, p_voff1 = (uint32_t)lane * 16u + 4096u;
    // scale copy: wavefronts 0 / 1 bring in the activation scales of tile rows [64 w, 64 w + 64), wavefront 2 the scales of
    // the tile's two weight blocks (odd lanes the second), wavefront 3 repeats that into a spare slice (every wavefront
    // issues the same number of memory instructions: one wait count fits all)
    const int64_t sq_k = SQL == 1 ? a.Qrows : 1;                  // floats between K blocks of one row's scales
    const uint32_t s_voff = wave < 2 ? (uint32_t)((64 * wave + lane) * (SQL == 1 ? 1 : KB) * 4) : (uint32_t)((lane & 1) * KB * 4);
    const int64_t s_kstep = wave < 2 ? sq_k * 4 : 4;              // bytes between K blocks in this wavefront's scale stream
    const uint32_t s_lds = (uint32_t)(S_OFS + wave * 256);
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    // fragment (j, kh): LDS row 32 j + x, 16-byte chunks 4 kh + 2 hh and the one after it; kh flips bit 6 of the offset
    const int fq_ofs0 = swz(x, 2 * hh), fq_ofs1 = swz(x, 2 * hh + 1);
    const int sq_rd = S_OFS + x * 16, sp_rd = SP_OFS + (wave >> 1) * 4;

    // ---- current / next tile (wave-uniform)
    int64_t cq = 0, cp = 0, nq = 0, np = 0, tn = 0;
    if (!tile_coords(0, cq, cp)) return;
    auto expert_of = [&](int64_t qt) -> int {
        int e = 0;
        // the tile index is the same in every lane, but comes out of a 64-bit division the compiler may carry out in vector
        // registers: hand it to the scalar load as a scalar
        const int qt_s = __builtin_amdgcn_readfirstlane((int)qt);
        if (grouped) asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(a.m_indices + (int64_t)qt_s * BQ) : "memory");
        return e;
    };
    const uint8_t *c_p, *c_q, *c_s, *n_p, *n_q, *n_s;
    int c_store, n_store = 0;
    bool n_valid = false;
    // GATHER: per tile and lane, the byte offsets of the four token rows its activation copies fetch (copy c: tile row
    // 32 w + 4 (lane >> 3) + c); c_* current tile, n_* next
    uint32_t c_qoff[4] = {0, 0, 0, 0}, n_qoff[4] = {0, 0, 0, 0};
    auto gather_setup = [&](int64_t qt, uint32_t (&qoff)[4]) {
        const int4 rc = *reinterpret_cast<const int4*>(a.src_row + qt * BQ + 32 * wave + 4 * crow);
        const int rcv[4] = {rc.x, rc.y, rc.z, rc.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) qoff[c] = (uint32_t)(rcv[c] < 0 ? 0 : rcv[c]) * (uint32_t)a.red + q_chunk;
    };
    auto setup = [&](int64_t qt, int64_t pt, const uint8_t*& pp, const uint8_t*& qp, const uint8_t*& sp_, int& store) {
        int e = expert_of(qt);
        store = e >= 0;
        if (e < 0) e = 0;                  // a padding tile is computed on expert 0's weights and not stored
        if constexpr (TRACE & 64) { pt = 0; qt = 0; e = 0; }        // timing experiment: every tile reads the operands of tile (0, 0)
        const int64_t p0 = pt * 256 + 256 <= a.Prows ? pt * 256 : a.Prows - 256;       // first weight row of the tile
        if (pt * 256 != p0 && wave < 2) store = 0;
        pp = a.pf + (((int64_t)e * P64 + p0 / 64 + wave) * KB) * 8192;
        qp = GATHER ? a.q : a.q + qt * BQ * a.red;
        if (wave < 2) sp_ = reinterpret_cast<const uint8_t*>(a.sq + (SQL == 1 ? qt * BQ : qt * BQ * KB));
        else sp_ = reinterpret_cast<const uint8_t*>(a.sp + ((int64_t)e * PB + p0 / 128) * KB);
    };
    setup(cq, cp, c_p, c_q, c_s, c_store);
    if constexpr (GATHER) gather_setup(cq, c_qoff);
    n_p = c_p; n_q = c_q; n_s = c_s;

    // the 13 memory instructions that bring in one K block, for ring position TT: 0 = scales, 1..8 = weight fragments
    // (1 KB each, in the order they lie in memory), 9..12 = activation copies
    auto issue = [&](auto tc, auto ic, const uint8_t* pp, const uint8_t* qp, const uint8_t* sp_, const uint32_t (&qoff)[4]) {
        constexpr int TT = decltype(tc)::value, I = decltype(ic)::value;
        if constexpr (I == 0) {
            if constexpr (!(TRACE & 4)) dma4_s(s_voff, sp_, lds_base + TT * STAGE + s_lds);
        } else if constexpr (I <= 8) {
            constexpr int t = I - 1;
            if constexpr (!(TRACE & 2)) fm_pload<32 * TT + 4 * t, (t & 3) * 1024>(t < 4 ? p_voff0 : p_voff1, pp);
        } else {
            constexpr int c = I - 9;
            if constexpr (!(TRACE & 4)) {
                if constexpr (GATHER) dma16_s(qoff[c], qp, lds_base + TT * STAGE + (4 * c + wave) * 1024);
                else dma16_s(q_off, qp + c * q_cstep, lds_base + TT * STAGE + (4 * c + wave) * 1024);
            }
        }
    };
    auto issue_all = [&](auto tc, const uint8_t* pp, const uint8_t* qp, const uint8_t* sp_) {
        static_for<13>([&](auto ic) { issue(tc, ic, pp, qp, sp_, c_qoff); });
    };
    auto qfrag = [&](const uint8_t* base, int j, int kh) -> i32x8 {
        return ld_frag_lds(base + j * 4096 + (fq_ofs0 ^ (kh * 64)), base + j * 4096 + (fq_ofs1 ^ (kh * 64)));
    };

    f32x16 acc[2][4];          // [pf][j]: element r = weight row 32 pf + 8 (r / 4) + 4 hh + r % 4 of the wavefront's 64, tile row 4 x + j
    // products in flight alternate between two register sets
    f32x16 d[2];
    float fq_last = 0.f;       // factor of the previous block's products of fragment 3 (zero at the head of a tile)
    i32x8 qf[4];               // fragment (j, kh) in qf[(2 j + kh) & 3]
    f32x4 sq_nxt;
    float sp_nxt;
    auto read_scales = [&](const uint8_t* base) {
        sq_nxt = *reinterpret_cast<const f32x4*>(base + sq_rd);
        sp_nxt = *reinterpret_cast<const float*>(base + sp_rd);
    };
    // zeroed by instructions the compiler cannot fold into a shared constant: given one, it parks a zero tuple in AGPRs
    // (free registers in its view) and copies from there, on top of the weight-fragment ring
    auto zero16 = [&](f32x16& v) {
#pragma unroll
        for (int r = 0; r < 16; ++r) asm volatile("v_mov_b32 %0, 0" : "=v"(v[r]));
    };
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) zero16(acc[i][j]);
    };

    // ---- fill: blocks 0 and 1 of the first tile
    issue_all(std::integral_constant<int, 0>{}, c_p, c_q, c_s);
    issue_all(std::integral_constant<int, 1>{}, c_p + 8192, c_q + 128, c_s + s_kstep);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    qf[0] = qfrag(lds, 0, 0);
    qf[1] = qfrag(lds, 0, 1);
    read_scales(lds);
    zero_acc();
#pragma unroll
    for (int i = 0; i < 2; ++i) zero16(d[i]);

    // TRACE: shader-clock sums over all K blocks of this wavefront: [0] MFMAs 0..11 with their copies and reads, [1] the
    // counted wait for the next block's data, [2] the barrier, [3] MFMAs 12..15 with the next block's first reads,
    // [4] epilogues, [5] blocks, [6] tiles.  Reading the clock is a scalar load waited for on the spot, which also drains
    // the LDS queue: the traced kernel is a few percent slower than the plain one.
    int64_t tr[7] = {0, 0, 0, 0, 0, 0, 0};
    auto now = [&]() -> int64_t {
        int64_t t = 0;
        if constexpr (TRACE) asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t) : : "memory");
        return t;
    };

    int64_t kb = 0;
    // one K block at ring position PH (= the workgroup's block counter % 3); returns true after the last tile
    auto blk = [&](auto phc) -> bool {
        constexpr int PH = decltype(phc)::value, NX = (PH + 1) % 3, PT = (PH + 2) % 3;
        const int64_t t0 = now();
        int64_t t1 = 0, t2 = 0, t3 = 0;
        if (kb == 0) {
            // the tile after this one (its first blocks are prefetched from this tile's last two)
            n_valid = tile_coords(tn + 1, nq, np);
            if (n_valid) setup(nq, np, n_p, n_q, n_s, n_store);
            else { n_p = c_p; n_q = c_q; n_s = c_s; n_store = 0; }      // past the last tile the prefetch re-reads this tile's first blocks
            if constexpr (GATHER) {
                if (n_valid) gather_setup(nq, n_qoff);
                else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) n_qoff[c] = c_qoff[c];
                }
            }
        }
        float fq_cur[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) fq_cur[t] = sq_nxt[t] * sp_nxt;
        const int64_t k2 = kb + 2;
        const bool in2 = k2 < KB;
        const int64_t kk = in2 ? k2 : k2 - KB;
        const uint8_t* pp = (in2 ? c_p : n_p) + kk * 8192;
        const uint8_t* qp = (in2 ? c_q : n_q) + kk * 128;
        const uint8_t* sp_ = (in2 ? c_s : n_s) + kk * s_kstep;
        uint32_t p_qoff[4] = {0, 0, 0, 0};                        // GATHER: the lane offsets of the tile the prefetched block belongs to
        if constexpr (GATHER) {
#pragma unroll
            for (int c = 0; c < 4; ++c) p_qoff[c] = in2 ? c_qoff[c] : n_qoff[c];
        }
        const uint8_t* sbase = lds + PH * STAGE;
        const uint8_t* nbase = lds + NX * STAGE;
        __builtin_amdgcn_sched_barrier(0);
        static_for<16>([&](auto mc) {
            constexpr int m = decltype(mc)::value, j = m >> 2, pf = (m >> 1) & 1, kh = m & 1, t = m >> 1;
            if constexpr (m == BAR) {
                // every fragment read of this block has been issued (the last before MFMA 8), and of the memory
                // instructions in flight only the 13 youngest (this block's) may still be out: the next block is
                // complete.  Behind the barrier everybody's share of it is.
                if constexpr (TRACE) { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); t1 = now(); }
                if constexpr (TRACE & 6) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // ablations: instruction counts differ
                else asm volatile("s_waitcnt vmcnt(13) lgkmcnt(0)" ::: "memory");
                if constexpr (TRACE) t2 = now();
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if constexpr (TRACE) t3 = now();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr ((m & 3) == 0 && j + 1 < 4 && !(TRACE & 16)) {
                qf[(2 * (j + 1)) & 3] = qfrag(sbase, j + 1, 0);
                qf[(2 * (j + 1) + 1) & 3] = qfrag(sbase, j + 1, 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (kh == 0) fm_mfma_first<32 * PH + 16 * pf>(d[t & 1], qf[(2 * j) & 3]);
            else fm_mfma_second<32 * PH + 16 * pf + 8>(d[t & 1], qf[(2 * j + 1) & 3]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (m < 12) {
                if constexpr (m == 0) issue(std::integral_constant<int, PT>{}, std::integral_constant<int, 0>{}, pp, qp, sp_, p_qoff);
                issue(std::integral_constant<int, PT>{}, std::integral_constant<int, m + 1>{}, pp, qp, sp_, p_qoff);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (m == 12 && !(TRACE & 16)) { qf[0] = qfrag(nbase, 0, 0); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (m == 13 && !(TRACE & 16)) { qf[1] = qfrag(nbase, 0, 1); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (m == 14) { read_scales(nbase); __builtin_amdgcn_sched_barrier(0); }
            // FMAs of product tt (MFMAs 2 tt, 2 tt + 1): registers 0..7 behind MFMA 2 tt + 2, registers 8..15 behind MFMA
            // 2 tt + 3.  Measured on this hardware: the matrix pipe writes a 32x32 result four registers at a time, registers
            // 0..7 twelve wait states after the MFMA was issued and 12..15 twenty after; the next MFMA is issued sixteen
            // wait states behind it, so behind ONE further MFMA registers 0..11 are there (12..15 four wait states later)
            // and behind two all are.  m = 0, 1: product 7 of the previous block.
            {
                constexpr bool prev = m < 2;
                constexpr int tp = prev ? 7 : ((m & 1) ? (m - 3) / 2 : (m - 2) / 2), half = m & 1;
                constexpr int aj = tp >> 1, ap = tp & 1;
                const float f = prev ? fq_last : fq_cur[aj];
                if constexpr (!(TRACE & 8))
#pragma unroll
                for (int r = 8 * half; r < 8 * half + 8; ++r) acc[ap][aj][r] = __builtin_fmaf(d[tp & 1][r], f, acc[ap][aj][r]);
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        fq_last = fq_cur[3];     // product 7 is folded in behind the next block's first two MFMAs
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (TRACE) {
            const int64_t t4 = now();
            tr[0] += t1 - t0; tr[1] += t2 - t1; tr[2] += t3 - t2; tr[3] += t4 - t3; tr[5] += 1;
        }
        ++kb;
        if (kb < KB) return false;

        // ---- tile finished.  Its last products: nothing follows them in the matrix pipe, so wait out the MFMA latency by
        // hand (the compiler does not know these registers come from matrix instructions)
        const int64_t te0 = now();
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(d[1]) : : "memory");      // 32 wait states; the last registers need 20
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[1][3][r] = __builtin_fmaf(d[1][r], fq_last, acc[1][3][r]);
        fq_last = 0.f;
        // epilogue: fragment j of this wavefront = tile rows 4 i + j (i = 0..31) x its 64 columns, staged as 32 rows of
        // 128 bytes in a private slice (LDS operations of one wavefront execute in order), stored 8 rows per instruction
        if (c_store) {
            // the lane's coordinates are formed anew from a value the compiler cannot see through: hoisted out of the K loop,
            // the epilogue's addresses would stay live across it, in registers the loop needs
            int tid_e = threadIdx.x;
            asm volatile("" : "+v"(tid_e));
            const int lane_e = tid_e & 63, x_e = lane_e & 31, hh_e = lane_e >> 5;
            uint8_t* ep = lds + EP_OFS + wave * (32 * EP_LD);
            const int er = lane_e >> 3, ec = lane_e & 7;
            const int64_t p0_e = cp * 256 + 256 <= a.Prows ? cp * 256 : a.Prows - 256;
            uint8_t* tile_out = reinterpret_cast<uint8_t*>(a.out) + ((cq * BQ) * a.ldo + p0_e + wave * 64 + ec * 8) * 2;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int pf = 0; pf < 2; ++pf)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        uint2 o;
                        o.x = pack_bf16(acc[pf][j][4 * g], acc[pf][j][4 * g + 1]);
                        o.y = pack_bf16(acc[pf][j][4 * g + 2], acc[pf][j][4 * g + 3]);
                        *reinterpret_cast<uint2*>(ep + x_e * EP_LD + (32 * pf + 8 * g + 4 * hh_e) * 2) = o;
                    }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int rl = er + 8 * i;                       // staged row = x of the producer = tile row 4 rl + j
                    const uint4 v = *reinterpret_cast<const uint4*>(ep + rl * EP_LD + ec * 16);
                    st16(tile_out + (int64_t)(4 * rl + j) * a.ldo * 2, v);
                }
            }
        }
        if constexpr (TRACE) { tr[4] += now() - te0; tr[6] += 1; }
        if (!n_valid) return true;
        zero_acc();
        ++tn;
        kb = 0;
        cq = nq; cp = np; c_p = n_p; c_q = n_q; c_s = n_s; c_store = n_store;
        if constexpr (GATHER) {
#pragma unroll
            for (int c = 0; c < 4; ++c) c_qoff[c] = n_qoff[c];
        }
        return false;
    };
    for (;;) {
        if (blk(std::integral_constant<int, 0>{})) break;
        if (blk(std::integral_constant<int, 1>{})) break;
        if (blk(std::integral_constant<int, 2>{})) break;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the copies issued past the end must land before the LDS is released
    if constexpr (TRACE) {
        if (tid == 0 && a.cycles)
#pragma unroll
            for (int i = 0; i < 7; ++i) a.cycles[(int64_t)blockIdx.x * 8 + i] = tr[i];
    }
}

// Re-orders quantized weights [E][N, K] (row-major) into the fragment-major order described at the top: one
// workgroup of 512 threads per 8 KB block, 16 bytes per thread.
__global__ __launch_bounds__(512) void k_weight_to_fm(const uint8_t* __restrict__ w, uint8_t* __restrict__ wf, int64_t N, int64_t K) {
    const int64_t KB = K / 128;
    const int64_t blk = blockIdx.x;                 // ((e * N / 64 + n64) * KB + kb)
    const int64_t kb = blk % KB, pn = blk / KB;     // pn = e * N / 64 + n64: weight row 64 pn of the stacked [E * N, K] matrix
    const int t = threadIdx.x, pf = t >> 8, kh = (t >> 7) & 1, h = (t >> 6) & 1, lane = t & 63, x = lane & 31, hh = lane >> 5;
    (void)N;
    const uint4 v = *reinterpret_cast<const uint4*>(w + (pn * 64 + pf * 32 + x) * K + kb * 128 + kh * 64 + hh * 32 + h * 16);
    *reinterpret_cast<uint4*>(wf + blk * 8192 + t * 16) = v;
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

static int fm_lds_attr() {
    static std::atomic<uint64_t> done{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, "pf8_gemm_fm", hipGetErrorString(e));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return PF8_OK;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fm<0>), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fm<1>), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fm<1, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fm<0, 0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm_fm<1, 0, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, "pf8_gemm_fm", hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return PF8_OK;
}

extern "C" int pf8_weight_to_fragment_major(const uint8_t* w, int E, int64_t N, int64_t K, uint8_t* wf, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && N >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(N % 64 == 0 && K % 128 == 0, "N must be a multiple of 64 and K of 128");
    if (E == 0 || N == 0 || K == 0) return PF8_OK;
    PF8_REQUIRE(w && wf, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(w) && PF8_ALIGNED16(wf), "pointers must be 16-byte aligned");
    const int64_t blocks = (int64_t)E * (N / 64) * (K / 128);
    PF8_REQUIRE(blocks <= 0x7FFFFFFF, "too many blocks");
    hipLaunchKernelGGL(k_weight_to_fm, dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream, w, wf, N, K);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_gemm_fm_supported(int64_t M, int64_t N, int64_t K) {
    return M > 0 && M % 128 == 0 && N >= 256 && N % 128 == 0 && K >= 384 && K % 128 == 0;
}

static int launch_fm(const char* where, const uint8_t* a, const float* sa, int sa_layout, const uint8_t* wf, const float* sb, int E,
                     int64_t M, int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out, int64_t ldo, pf8_stream_t stream,
                     int64_t* cycles = nullptr, int64_t cycles_rows = 0, int ablate = 0, const int32_t* src_row = nullptr) {
    int rc = fm_lds_attr();
    if (rc) return rc;
    FmArgs g = {};
    g.pf = wf; g.q = a; g.sp = sb; g.sq = sa; g.out = out;
    g.Prows = N; g.Qrows = M; g.red = K; g.ldo = ldo; g.grouped = m_indices != nullptr; g.E = E; g.m_indices = m_indices;
    const int64_t T = ((N + 255) / 256) * (M / 128), per_xcd = (T + 7) / 8;
    if (T > 0x7FFFFFFF) return pf8_fail(PF8_EINVAL, where, "too many tiles");
    int64_t w = pf8_effective_cus() / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    if (cycles) {
        if (cycles_rows < 8 * w) return pf8_fail(PF8_EINVAL, where, "cycles must hold 8 values for each of the launch's workgroups (8 per 8 compute units)");
        if (sa_layout != 1) return pf8_fail(PF8_EINVAL, where, "the traced instantiation reads K-block-major activation scales (sa_layout 1)");
        g.cycles = cycles;
        void (*k)(const FmArgs) = nullptr;
        switch (ablate) {
            case 0: k = k_gemm_fm<1, 1>; break;
            case 6: k = k_gemm_fm<1, 1 | 6>; break;
            case 8: k = k_gemm_fm<1, 1 | 8>; break;
            case 14: k = k_gemm_fm<1, 1 | 14>; break;
            case 30: k = k_gemm_fm<1, 1 | 30>; break;
            case 64: k = k_gemm_fm<1, 1 | 64>; break;
            default: return pf8_fail(PF8_EINVAL, where, "unknown ablation");
        }
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, kFmDynLds);
        if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, where, hipGetErrorString(e));
        hipLaunchKernelGGL(k, dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
        return pf8_check_launch(where);
    }
    if (src_row) {
        g.src_row = src_row;
        if (sa_layout == 0) hipLaunchKernelGGL((k_gemm_fm<0, 0, 1>), dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
        else hipLaunchKernelGGL((k_gemm_fm<1, 0, 1>), dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
    } else if (sa_layout == 0) hipLaunchKernelGGL(k_gemm_fm<0>, dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
    else hipLaunchKernelGGL(k_gemm_fm<1>, dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
    return pf8_check_launch(where);
}

extern "C" int pf8_gemm_nt_fm(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b_fm, const float* sb, int64_t M, int64_t N,
                              int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative shape");
    if (M == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(pf8_gemm_fm_supported(M, N, K), "needs M % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0 and K >= 384");
    PF8_REQUIRE(a && sa && b_fm && sb && out, "null pointer");
    PF8_REQUIRE(ldo >= N && ldo % 8 == 0, "ldo must be >= N and a multiple of 8");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b_fm) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    PF8_REQUIRE(K <= (1ll << 24), "K too large");
    return launch_fm(__func__, a, sa, sa_layout, b_fm, sb, 1, M, N, K, nullptr, out, ldo, stream);
}

extern "C" int pf8_grouped_gemm_nt_contiguous_fm(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b_fm, const float* sb,
                                                 int E, int64_t Mtot, int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out,
                                                 pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Mtot >= 0 && N >= 0 && K >= 0, "negative shape");
    if (Mtot == 0 || N == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(pf8_gemm_fm_supported(Mtot, N, K), "needs Mtot % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0 and K >= 384");
    PF8_REQUIRE(a && sa && b_fm && sb && out && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b_fm) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    PF8_REQUIRE(K <= (1ll << 24), "K too large");
    return launch_fm(__func__, a, sa, sa_layout, b_fm, sb, E, Mtot, N, K, m_indices, out, N, stream);
}

extern "C" int pf8_debug_grouped_gemm_fm_cycles(const uint8_t* a, const float* sa, const uint8_t* b_fm, const float* sb, int E, int64_t Mtot,
                                                int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out, int64_t* cycles,
                                                int64_t workgroups, int ablate, pf8_stream_t stream) {
    PF8_REQUIRE(E > 0 && pf8_gemm_fm_supported(Mtot, N, K), "needs Mtot % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0 and K >= 384");
    PF8_REQUIRE(a && sa && b_fm && sb && out && m_indices && cycles, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b_fm) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    return launch_fm(__func__, a, sa, 1, b_fm, sb, E, Mtot, N, K, m_indices, out, N, stream, cycles, workgroups, ablate);
}

extern "C" int pf8_grouped_gemm_nt_contiguous_fm_gather(const uint8_t* tokens, int64_t T, const int32_t* src_row, const float* sa, int sa_layout,
                                                        const uint8_t* b_fm, const float* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                                        const int32_t* m_indices, uint16_t* out, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Mtot >= 0 && N >= 0 && K >= 0 && T >= 0, "negative shape");
    if (Mtot == 0 || N == 0 || E == 0) return PF8_OK;
    PF8_REQUIRE(pf8_gemm_fm_supported(Mtot, N, K), "needs Mtot % 128 == 0, N % 128 == 0, N >= 256, K % 128 == 0 and K >= 384");
    PF8_REQUIRE(T > 0 && tokens && sa && src_row && b_fm && sb && out && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(tokens) && PF8_ALIGNED16(b_fm) && PF8_ALIGNED16(out) && PF8_ALIGNED16(src_row), "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    PF8_REQUIRE(K <= (1ll << 24) && T * K < (1ll << 31), "the token matrix must stay below 2 GiB");
    return launch_fm(__func__, tokens, sa, sa_layout, b_fm, sb, E, Mtot, N, K, m_indices, out, N, stream, nullptr, 0, 0, src_row);
}
