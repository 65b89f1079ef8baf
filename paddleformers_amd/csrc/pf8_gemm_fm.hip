// pf8_gemm_fm.hip -- forward / dgrad block-scaled FP8 GEMM on FRAGMENT-MAJOR weights.
//
// The FP8 weights of this path are written by this library (the stacked-weight quantizers) and read only by its
// GEMMs, so their byte order is the library's to choose.  `pf8_weight_to_fragment_major` re-orders a quantized weight
// [E][N, K] into the order in which a wavefront's matrix instructions consume it:
//     wf[e][n / 64][k / 128][ps = 0..3][h = 0..1][lane = 0..63][16 bytes]
// where the 16 bytes are k = 128 kb + 32 (lane / 16) + 16 h .. + 15 of weight row n = 64 (n / 64) + 16 ps + lane % 16.
// The 8 KB of one (64-row panel, K block) are exactly the four A-operand fragments (16 rows x 128 k each) of
// v_mfma_f32_16x16x128_f8f6f4, and consecutive K blocks of a panel are contiguous.
//
// With that order a wavefront fetches its weight fragments with whole 1 KB global loads STRAIGHT INTO REGISTERS: no
// LDS write, no LDS read, no swizzle, and a perfectly sequential stream per wavefront.  The registers are accumulation
// VGPRs (AGPRs): gfx950 loads into them directly and the MFMA takes its A operand from them, so a ring of four K blocks
// of weight fragments (128 AGPRs) costs no architectural VGPR, and the weights are prefetched three blocks ahead.
//
// Geometry: workgroup tile 128 (Q = activation rows) x 256 (P = weight rows) x 128 (K, one scale block), 256 threads =
// 4 wavefronts side by side along P: wavefront w owns weight rows [64 w, 64 w + 64) of the tile (4 fragments) and ALL
// 128 activation rows (8 fragments), 4 x 8 MFMA tiles = 128 accumulator VGPRs.  No two wavefronts load the same weight
// byte.  Per K block a compute unit takes in 32 KB of weights (global -> AGPR) and 16 KB of activations (global -> LDS)
// and reads 64 KB of activation fragments from LDS: 80 KB of LDS traffic against the 144 KB of the kernels that stage
// both operands in LDS, for the same 32 MFMAs per wavefront.
//
//   * Activations go global -> LDS (global_load_lds_dwordx4) into a ring of four 16 KB stages.  Tile row r is stored in
//     LDS row 16 (r % 8) + r / 8, so fragment j (LDS rows 16 j .. 16 j + 15) holds tile rows 8 i + j: the eight
//     activation scales a lane needs per block (rows 8 li .. 8 li + 7) are then 32 contiguous bytes.
//   * The scales of a block travel with it: 128 activation scales and the two weight-block scales are copied into the
//     stage (global_load_lds_dword, one instruction per wavefront) and read from LDS after the barrier that declares
//     the stage landed.  Every memory instruction of the loop is therefore issued three blocks ahead of its use,
//     and the one counted wait per block (vmcnt(26): two blocks of 13 instructions may stay in flight) never waits for
//     anything issued less than a block and a half ago.  Vector loads retire in order, so a younger load a block needs
//     early would otherwise drag the whole prefetch queue with it.
//   * One barrier per block (before MFMA 24 of 32), behind it the first fragments and the scales of the next block
//     are read; the rings run on across tile boundaries.
//   * The product of a K block (MFMA with C = 0) is folded into the fp32 accumulators by one FMA per element with
//     sa * sb of the block, two MFMAs behind, as in the other fp32-scale kernels.  The MFMAs are inline assembly
//     (the AGPR operand has to be named), so the compiler does not see them as matrix instructions and inserts no wait
//     states for their results: nothing reads a product before two further MFMAs have been issued behind it (64
//     cycles; the product is written after about 32).  The last two products of a block are therefore folded in
//     behind the first two MFMAs of the next block, and a tile's very last two behind an explicit wait.
//   * Epilogue: each wavefront stages 16 rows x 64 columns of bf16 at a time in a private LDS slice and stores
//     128-byte row pieces.
// Needs Prows % 256 == 0, Qrows % 128 == 0 and K % 512 == 0 (the four-deep rings are unrolled by four blocks); dense
// and contiguous-grouped layouts.
#include <atomic>

#include "pf8_gemm_common.h"
#include "pf8_host.h"

namespace pf8 {

struct FmArgs {
    const uint8_t* pf;     // fragment-major weights [E][Prows / 64][KB][8192]
    const uint8_t* q;      // activations [Qrows, red]
    const float* sp;       // [E][Prows / 128, KB]
    const float* sq;       // sq_layout 0: [Qrows, KB], 1: [KB, Qrows]
    uint16_t* out;         // bf16 [Qrows, ldo]
    int64_t Prows, Qrows, red, ldo;
    int grouped, E;
    const int32_t* m_indices;
};

constexpr int kFmSegTiles = 2048;                 // row tiles whose expert order is tabulated in LDS
constexpr int kFmStages = 4, kFmStage = 16384 + 1024, kFmEpLd = 144;
constexpr int kFmDynLds = kFmStages * kFmStage + 4 * 16 * kFmEpLd;

// AGPR ring: slot S (block index % 4) holds fragment ps, half h in a[32 S + 8 ps + 4 h .. + 3]
template <int A, int IMM>
__device__ __forceinline__ void fm_pload(uint32_t voff, const uint8_t* sbase) {
    asm volatile("global_load_dwordx4 a[%2:%3], %0, %1 offset:%4" : : "v"(voff), "s"(sbase), "n"(A), "n"(A + 3), "n"(IMM) : "memory");
}
template <int A>
__device__ __forceinline__ void fm_mfma(f32x4& d, const i32x8& q) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, a[%2:%3], %1, 0" : "=&v"(d) : "v"(q), "n"(A), "n"(A + 7));
}

template <int SQL>
__global__ __launch_bounds__(256, 1) void k_gemm_fm(const FmArgs a) {
    constexpr int BQ = 128;
    constexpr int STAGE = kFmStage, S_OFS = 16384, SP_OFS = 16384 + 512, EP_OFS = kFmStages * kFmStage, EP_LD = kFmEpLd;
    constexpr int BAR = 24;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    asm volatile("" ::: "a127");          // the kernel descriptor reserves a0..a127: the weight-fragment ring, named literally below
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, kg = lane >> 4;

    const int64_t p_tiles = a.Prows / 256, q_tiles = a.Qrows / BQ;
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
    // activation copy c (0..3) of wavefront w fills LDS rows (4 c + w) * 8 + (lane >> 3) = fragment (4 c + w) / 2, fragment
    // row 8 (w & 1) + (lane >> 3), i.e. tile row 64 (w & 1) + 8 (lane >> 3) + 2 c + (w >> 1); the swizzle key of that LDS
    // row is (lane >> 3) ^ (w & 1) whatever c
    const int crow = lane >> 3, cpos = lane & 7;
    const uint32_t q_off = (uint32_t)((64 * (wave & 1) + 8 * crow + (wave >> 1)) * a.red + ((cpos ^ (crow ^ (wave & 1))) << 4));
    const int64_t q_cstep = 2 * a.red;
    const uint32_t p_voff0 = (uint32_t)lane * 16u, p_voff1 = (uint32_t)lane * 16u + 4096u;
    // scale copy: wavefronts 0 / 1 bring in the activation scales of tile rows [64 w, 64 w + 64), wavefront 2 the scales of
    // the tile's two weight blocks (odd lanes the second), wavefront 3 repeats that into a spare slice (every wavefront
    // issues the same number of memory instructions: one wait count fits all)
    const int64_t sq_k = SQL == 1 ? a.Qrows : 1;                  // floats between K blocks of one row's scales
    const uint32_t s_voff = wave < 2 ? (uint32_t)((64 * wave + lane) * (SQL == 1 ? 1 : KB) * 4) : (uint32_t)((lane & 1) * KB * 4);
    const int64_t s_kstep = wave < 2 ? sq_k * 4 : 4;              // bytes between K blocks in this wavefront's scale stream
    const uint32_t s_lds = (uint32_t)(S_OFS + wave * 256);
    const uint32_t lds_base = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const int fq_ofs0 = swz(li, 2 * kg), fq_ofs1 = swz(li, 2 * kg + 1);
    const int sq_rd = S_OFS + li * 32, sp_rd = SP_OFS + (wave >> 1) * 4;

    // ---- current / next tile (wave-uniform)
    int64_t cq = 0, cp = 0, nq = 0, np = 0;
    if (!tile_coords(0, cq, cp)) return;
    auto expert_of = [&](int64_t qt) -> int {
        int e = 0;
        if (grouped) asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(a.m_indices + qt * BQ) : "memory");
        return e;
    };
    const uint8_t *c_p, *c_q, *c_s, *n_p, *n_q, *n_s;
    int c_store, n_store = 0;
    auto setup = [&](int64_t qt, int64_t pt, const uint8_t*& pp, const uint8_t*& qp, const uint8_t*& sp_, int& store) {
        int e = expert_of(qt);
        store = e >= 0;
        if (e < 0) e = 0;                  // a padding tile is computed on expert 0's weights and not stored
        pp = a.pf + (((int64_t)e * P64 + pt * 4 + wave) * KB) * 8192;
        qp = a.q + qt * BQ * a.red;
        if (wave < 2) sp_ = reinterpret_cast<const uint8_t*>(a.sq + (SQL == 1 ? qt * BQ : qt * BQ * KB));
        else sp_ = reinterpret_cast<const uint8_t*>(a.sp + ((int64_t)e * PB + pt * 2) * KB);
    };
    setup(cq, cp, c_p, c_q, c_s, c_store);

    // the 13 memory instructions that bring in one K block, for ring position T: 0 = scales, 1..8 = weight fragments
    // (ps = (i - 1) / 2, h = (i - 1) % 2), 9..12 = activation copies
    auto issue = [&](auto tc, auto ic, const uint8_t* pp, const uint8_t* qp, const uint8_t* sp_) {
        constexpr int TT = decltype(tc)::value, I = decltype(ic)::value;
        if constexpr (I == 0) {
            dma4_s(s_voff, sp_, lds_base + TT * STAGE + s_lds);
        } else if constexpr (I <= 8) {
            constexpr int ps = (I - 1) >> 1, h = (I - 1) & 1;
            fm_pload<32 * TT + 8 * ps + 4 * h, (ps & 1) * 2048 + h * 1024>(ps < 2 ? p_voff0 : p_voff1, pp);
        } else {
            constexpr int c = I - 9;
            dma16_s(q_off, qp + c * q_cstep, lds_base + TT * STAGE + (4 * c + wave) * 1024);
        }
    };
    auto issue_all = [&](auto tc, const uint8_t* pp, const uint8_t* qp, const uint8_t* sp_) {
        static_for<13>([&](auto ic) { issue(tc, ic, pp, qp, sp_); });
    };
    auto qfrag = [&](const uint8_t* base, int j) -> i32x8 { return ld_frag_lds(base + fq_ofs0 + j * 2048, base + fq_ofs1 + j * 2048); };

    f32x4 acc[4][8];
    // products in flight: MFMA j of a block writes d[j % 4] and the FMAs that fold it in follow MFMA j + 2, so products 30
    // and 31 of a block are folded in behind MFMAs 0 and 1 of the NEXT block, with the factor of their own block (fq_last)
    f32x4 d[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) d[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float fq_last = 0.f;
    i32x8 qf[4];
    f32x4 sq_nxt[2];
    float sp_nxt;
    auto read_scales = [&](const uint8_t* base) {
        sq_nxt[0] = *reinterpret_cast<const f32x4*>(base + sq_rd);
        sq_nxt[1] = *reinterpret_cast<const f32x4*>(base + sq_rd + 16);
        sp_nxt = *reinterpret_cast<const float*>(base + sp_rd);
    };

    // ---- fill: blocks 0, 1, 2 of the first tile
    issue_all(std::integral_constant<int, 0>{}, c_p, c_q, c_s);
    issue_all(std::integral_constant<int, 1>{}, c_p + 8192, c_q + 128, c_s + s_kstep);
    issue_all(std::integral_constant<int, 2>{}, c_p + 2 * 8192, c_q + 2 * 128, c_s + 2 * s_kstep);
    asm volatile("s_waitcnt vmcnt(26)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    qf[0] = qfrag(lds, 0);
    qf[1] = qfrag(lds, 1);
    qf[2] = qfrag(lds, 2);
    read_scales(lds);

    // one K block; U = its ring position.  kb = its index inside the current tile.
    auto blk = [&](auto uc, int64_t kb) {
        constexpr int U = decltype(uc)::value, NX = (U + 1) & 3, PT = (U + 3) & 3;
        float fq_cur[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) { fq_cur[t] = sq_nxt[0][t] * sp_nxt; fq_cur[4 + t] = sq_nxt[1][t] * sp_nxt; }
        // the block three ahead: this tile's, or one of the next tile's first three
        const int64_t k3 = kb + 3;
        const bool in3 = k3 < KB;
        const int64_t kk = in3 ? k3 : k3 - KB;
        const uint8_t* pp = (in3 ? c_p : n_p) + kk * 8192;
        const uint8_t* qp = (in3 ? c_q : n_q) + kk * 128;
        const uint8_t* sp_ = (in3 ? c_s : n_s) + kk * s_kstep;
        const uint8_t* sbase = lds + U * STAGE;
        const uint8_t* nbase = lds + NX * STAGE;
        __builtin_amdgcn_sched_barrier(0);
        static_for<32>([&](auto jc) {
            constexpr int j = decltype(jc)::value, qs = j >> 2, ps = j & 3;
            if constexpr (j == BAR) {
                // every fragment read of this block has been issued (the last before MFMA 16), and of the memory
                // instructions in flight only the 26 youngest (this block's and the previous one's) may still be out:
                // the next block is complete.  Behind the barrier everybody's share of it is.
                asm volatile("s_waitcnt vmcnt(26) lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (ps == 0 && qs + 3 < 8) {
                qf[(qs + 3) & 3] = qfrag(sbase, qs + 3);
                __builtin_amdgcn_sched_barrier(0);
            }
            fm_mfma<32 * U + 8 * ps>(d[j & 3], qf[qs & 3]);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr ((j & 1) == 1 && j < 24) {
                constexpr int sl = j >> 1;                       // 12 issue slots for 13 instructions
                if constexpr (sl == 0) issue(std::integral_constant<int, PT>{}, std::integral_constant<int, 0>{}, pp, qp, sp_);
                issue(std::integral_constant<int, PT>{}, std::integral_constant<int, sl + 1>{}, pp, qp, sp_);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (j == 24) { qf[0] = qfrag(nbase, 0); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (j == 25) { qf[1] = qfrag(nbase, 1); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (j == 26) { read_scales(nbase); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (j == 28) { qf[2] = qfrag(nbase, 2); __builtin_amdgcn_sched_barrier(0); }
            if constexpr (j >= 2) {
                constexpr int jj = j - 2, qj = jj >> 2, pj = jj & 3;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[pj][qj][r] = __builtin_fmaf(d[jj & 3][r], fq_cur[qj], acc[pj][qj][r]);
                __builtin_amdgcn_sched_barrier(0);
            } else {
                // the previous block's products 30 / 31 (at the head of a tile fq_last is zero and d finite: adds nothing)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[2 + j][7][r] = __builtin_fmaf(d[2 + j][r], fq_last, acc[2 + j][7][r]);
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        fq_last = fq_cur[7];
        __builtin_amdgcn_sched_barrier(0);
    };

    for (int64_t n = 0;; ++n) {
        const bool n_valid = tile_coords(n + 1, nq, np);
        if (n_valid) setup(nq, np, n_p, n_q, n_s, n_store);
        else { n_p = c_p; n_q = c_q; n_s = c_s; n_store = 0; }     // past the last tile the prefetch re-reads this tile's first blocks
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        for (int64_t kb = 0; kb < KB; kb += 4) {
            blk(std::integral_constant<int, 0>{}, kb);
            blk(std::integral_constant<int, 1>{}, kb + 1);
            blk(std::integral_constant<int, 2>{}, kb + 2);
            blk(std::integral_constant<int, 3>{}, kb + 3);
        }
        // the tile's last two products: nothing follows them in the matrix pipe, so wait out the MFMA latency by hand
        // (the compiler does not know these registers come from matrix instructions)
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" : "+v"(d[2]), "+v"(d[3]) : : "memory");
#pragma unroll
        for (int t = 2; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][7][r] = __builtin_fmaf(d[t][r], fq_last, acc[t][7][r]);
        fq_last = 0.f;
        // ---- epilogue: fragment j of this wavefront = tile rows 8 i + j (i = 0..15) x its 64 columns, staged as 16 rows of
        // 128 bytes in a private slice (LDS operations of one wavefront execute in order), stored 8 rows per instruction
        if (c_store) {
            uint8_t* ep = lds + EP_OFS + wave * (16 * EP_LD);
            const int er = lane >> 3, ec = lane & 7;
            uint8_t* tile_out = reinterpret_cast<uint8_t*>(a.out) + ((cq * BQ) * a.ldo + cp * 256 + wave * 64 + ec * 8) * 2;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
#pragma unroll
                for (int ps = 0; ps < 4; ++ps) {
                    uint2 o;
                    o.x = pack_bf16(acc[ps][j][0], acc[ps][j][1]);
                    o.y = pack_bf16(acc[ps][j][2], acc[ps][j][3]);
                    *reinterpret_cast<uint2*>(ep + li * EP_LD + (ps * 16 + 4 * kg) * 2) = o;
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int rl = er + 8 * i;                       // staged row = li of the producer = tile row 8 rl + j
                    const uint4 v = *reinterpret_cast<const uint4*>(ep + rl * EP_LD + ec * 16);
                    st16(tile_out + (int64_t)(8 * rl + j) * a.ldo * 2, v);
                }
            }
        }
        if (!n_valid) break;
        cq = nq; cp = np; c_p = n_p; c_q = n_q; c_s = n_s; c_store = n_store;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the copies issued past the end must land before the LDS is released
}

// Re-orders quantized weights [E][N, K] (row-major) into the fragment-major order described at the top: one
// workgroup of 512 threads per 8 KB block, 16 bytes per thread.
__global__ __launch_bounds__(512) void k_weight_to_fm(const uint8_t* __restrict__ w, uint8_t* __restrict__ wf, int64_t N, int64_t K) {
    const int64_t KB = K / 128, P64 = N / 64;
    const int64_t blk = blockIdx.x;                 // ((e * P64 + n64) * KB + kb)
    const int64_t kb = blk % KB, pn = blk / KB;     // pn = e * P64 + n64: weight row 64 pn of the stacked [E * N, K] matrix
    const int t = threadIdx.x, ps = t >> 7, h = (t >> 6) & 1, lane = t & 63, li = lane & 15, kg = lane >> 4;
    (void)P64;
    const uint4 v = *reinterpret_cast<const uint4*>(w + (pn * 64 + ps * 16 + li) * K + kb * 128 + kg * 32 + h * 16);
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
    return M > 0 && M % 128 == 0 && N >= 256 && N % 256 == 0 && K >= 512 && K % 512 == 0;
}

static int launch_fm(const char* where, const uint8_t* a, const float* sa, int sa_layout, const uint8_t* wf, const float* sb, int E,
                     int64_t M, int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out, int64_t ldo, pf8_stream_t stream) {
    int rc = fm_lds_attr();
    if (rc) return rc;
    FmArgs g = {};
    g.pf = wf; g.q = a; g.sp = sb; g.sq = sa; g.out = out;
    g.Prows = N; g.Qrows = M; g.red = K; g.ldo = ldo; g.grouped = m_indices != nullptr; g.E = E; g.m_indices = m_indices;
    const int64_t T = (N / 256) * (M / 128), per_xcd = (T + 7) / 8;
    if (T > 0x7FFFFFFF) return pf8_fail(PF8_EINVAL, where, "too many tiles");
    int64_t w = pf8_effective_cus() / 8;
    if (w < 1) w = 1;
    if (w > per_xcd) w = per_xcd;
    if (sa_layout == 0) hipLaunchKernelGGL(k_gemm_fm<0>, dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
    else hipLaunchKernelGGL(k_gemm_fm<1>, dim3((unsigned)(8 * w)), dim3(256), kFmDynLds, (hipStream_t)stream, g);
    return pf8_check_launch(where);
}

extern "C" int pf8_gemm_nt_fm(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b_fm, const float* sb, int64_t M, int64_t N,
                              int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative shape");
    if (M == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(pf8_gemm_fm_supported(M, N, K), "needs M % 128 == 0, N % 256 == 0 and K % 512 == 0");
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
    PF8_REQUIRE(pf8_gemm_fm_supported(Mtot, N, K), "needs Mtot % 128 == 0, N % 256 == 0 and K % 512 == 0");
    PF8_REQUIRE(a && sa && b_fm && sb && out && m_indices, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a) && PF8_ALIGNED16(b_fm) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    PF8_REQUIRE(sa_layout == 0 || sa_layout == 1, "sa_layout must be 0 or 1");
    PF8_REQUIRE(K <= (1ll << 24), "K too large");
    return launch_fm(__func__, a, sa, sa_layout, b_fm, sb, E, Mtot, N, K, m_indices, out, N, stream);
}
