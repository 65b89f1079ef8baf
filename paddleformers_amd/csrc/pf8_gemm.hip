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
// Workgroup: 256 threads = 4 wavefronts in a 2x2 arrangement, tile 128(P) x 128(Q) x 128(K);
// each wavefront owns 64x64 = 4x4 MFMA tiles.  LDS: two stages of P and Q tiles (64 KB), rows of
// 128 B with the 16-byte chunks XOR-swizzled by (row>>1)&7 so both the 16 B global->LDS writes and
// the fragment reads are bank-conflict free.
#include "pf8_device.h"
#include "pf8_host.h"

namespace pf8 {

constexpr int TILE = 128;

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
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

template <int MODE, int SQL>
__global__ __launch_bounds__(256, 2) void k_gemm(const GemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // lds: [stage][P tile 16 KB | Q tile 16 KB]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wp = wave & 1, wq = wave >> 1;
    const int li = lane & 15, kg = lane >> 4;

    const int64_t p_tiles = (a.Prows + TILE - 1) / TILE;
    const int64_t p_tile = blockIdx.x % p_tiles, q_tile = blockIdx.x / p_tiles;
    const int64_t p0 = p_tile * TILE, q0 = q_tile * TILE;

    const uint8_t* pbase = a.p;
    const uint8_t* qbase = a.q;
    const float* spb = a.sp;
    const float* sqb = a.sq;
    uint8_t* outb = reinterpret_cast<uint8_t*>(a.out);
    int64_t ldp = a.red, ldq = a.red;        // row strides of the operands (bytes)
    int64_t KBn = a.red / 128;               // K blocks to reduce over
    int64_t q_valid = a.Qrows;               // rows of Q that may be stored
    int64_t KBs = KBn;                       // K blocks per row in the scale tensors (forward)
    const int64_t PB = (a.Prows + 127) / 128;

    if (MODE == MODE_FWD) {
        if (a.group == GROUP_CONTIG) {
            const int e = a.m_indices[q0];
            if (e < 0) return;
            pbase += (int64_t)e * a.Prows * a.red;
            spb += (int64_t)e * PB * KBs;
        } else if (a.group == GROUP_MASKED) {
            const int e = blockIdx.y;
            const int64_t valid = a.masked_m[e];
            if (q0 >= valid) return;
            q_valid = valid;
            pbase += (int64_t)e * a.Prows * a.red;
            spb += (int64_t)e * PB * KBs;
            qbase += (int64_t)e * a.Qrows * a.red;
            sqb += (int64_t)e * a.Qrows * KBs;
            outb += (int64_t)e * a.Qrows * a.ldo * 2;
        }
    } else {
        if (a.group == GROUP_WGRAD) {
            const int e = blockIdx.y;
            const int64_t t0 = a.tile_start[e], t1 = a.tile_start[e + 1];
            const int64_t Me = (t1 - t0) * 128;
            // packed per-expert operands: [rows, Me] at rows*128*t0, scales [Me/128, rows] at t0*rows
            pbase += a.Prows * 128 * t0;
            qbase += a.Qrows * 128 * t0;
            spb += t0 * a.Prows;
            sqb += t0 * a.Qrows;
            outb += (int64_t)e * a.Qrows * a.ldo * 4;
            ldp = ldq = Me;
            KBn = t1 - t0;
            if (KBn == 0 && a.accumulate) return;
        }
    }

    // ---- global -> LDS staging: thread copies chunk (tid&7) of rows (tid>>3) + 32*i ------------
    const int crow = tid >> 3, cchunk = tid & 7;
    const uint8_t* gp[4];
    const uint8_t* gq[4];
    int lofs[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = crow + 32 * i;
        int64_t pr = p0 + row; if (pr > a.Prows - 1) pr = a.Prows - 1;
        int64_t qr = q0 + row; if (qr > a.Qrows - 1) qr = a.Qrows - 1;
        gp[i] = pbase + pr * ldp + cchunk * 16;
        gq[i] = qbase + qr * ldq + cchunk * 16;
        lofs[i] = swz(row, cchunk);
    }
    uint4 rp[4], rq[4];
#define PF8_G_LOAD(kb_)                                                          \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                              \
        rp[i] = *reinterpret_cast<const uint4*>(gp[i] + (kb_) * 128);            \
        rq[i] = *reinterpret_cast<const uint4*>(gq[i] + (kb_) * 128);            \
    }
#define PF8_L_STORE(stage_)                                                      \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                              \
        *reinterpret_cast<uint4*>(lds + (stage_) * 32768 + lofs[i]) = rp[i];     \
        *reinterpret_cast<uint4*>(lds + (stage_) * 32768 + 16384 + lofs[i]) = rq[i]; \
    }

    // ---- fragment addresses --------------------------------------------------------------------
    int fofs_p[4][2], fofs_q[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int prow = wp * 64 + t * 16 + li, qrow = wq * 64 + t * 16 + li;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            fofs_p[t][h] = swz(prow, 2 * kg + h);
            fofs_q[t][h] = 16384 + swz(qrow, 2 * kg + h);
        }
    }

    // ---- scale addressing ----------------------------------------------------------------------
    // forward: lane needs sq of its 4 output rows (one per q sub-tile) and the block scale of P
    // wgrad  : lane needs sq of its 4 output rows and sp of its 16 output columns (4 x float4)
    int64_t qrow_g[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        int64_t r = q0 + wq * 64 + t * 16 + li;
        if (r > a.Qrows - 1) r = a.Qrows - 1;
        qrow_g[t] = r;
    }
    int64_t pcol_g[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        int64_t c = p0 + wp * 64 + t * 16 + 4 * kg;
        if (c > a.Prows - 4) c = a.Prows - 4;
        pcol_g[t] = c;
    }
    float fq[4];
    f32x4 fp4[4];
    float fpb = 0.0f;
    auto s_load = [&](int64_t kb) {
        if (MODE == MODE_FWD) {
#pragma unroll
            for (int t = 0; t < 4; ++t) fq[t] = SQL == 0 ? sqb[qrow_g[t] * KBs + kb] : sqb[kb * a.Qrows + qrow_g[t]];
            fpb = spb[p_tile * KBs + kb];
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                fq[t] = sqb[kb * a.Qrows + qrow_g[t]];
                fp4[t] = *reinterpret_cast<const f32x4*>(spb + kb * a.Prows + pcol_g[t]);
            }
        }
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    if (KBn > 0) {
        PF8_G_LOAD(0)
        PF8_L_STORE(0)
    }
    __syncthreads();

    for (int64_t kb = 0; kb < KBn; ++kb) {
        const int cur = (int)(kb & 1);
        // prefetch the next K block into registers (the last iteration re-reads its own block:
        // no branch, so the staging registers never leave the register file)
        const int64_t kbn = kb + 1 < KBn ? kb + 1 : kb;
        PF8_G_LOAD(kbn)
        s_load(kb);
        const uint8_t* base = lds + cur * 32768;
        i32x8 pf[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            i32x4 lo = *reinterpret_cast<const i32x4*>(base + fofs_p[t][0]);
            i32x4 hi = *reinterpret_cast<const i32x4*>(base + fofs_p[t][1]);
            pf[t] = (i32x8){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
#pragma unroll
        for (int qs = 0; qs < 4; ++qs) {
            i32x4 lo = *reinterpret_cast<const i32x4*>(base + fofs_q[qs][0]);
            i32x4 hi = *reinterpret_cast<const i32x4*>(base + fofs_q[qs][1]);
            i32x8 qf = (i32x8){lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            float f = MODE == MODE_FWD ? fq[qs] * fpb : fq[qs];
#pragma unroll
            for (int ps = 0; ps < 4; ++ps) {
                f32x4 d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ps], qf, (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                if (MODE == MODE_FWD) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[ps][qs][r] = __builtin_fmaf(d[r], f, acc[ps][qs][r]);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[ps][qs][r] = __builtin_fmaf(d[r] * f, fp4[ps][r], acc[ps][qs][r]);
                }
            }
        }
        PF8_L_STORE(cur ^ 1)
        __syncthreads();
    }

    // ---- epilogue ------------------------------------------------------------------------------
#pragma unroll
    for (int qs = 0; qs < 4; ++qs) {
        const int64_t row = q0 + wq * 64 + qs * 16 + li;
        if (row >= q_valid) continue;
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) {
            const int64_t col = p0 + wp * 64 + ps * 16 + 4 * kg;
            if (col + 4 > a.Prows) continue;
            if (MODE == MODE_FWD) {
                uint2 o;
                o.x = pack_bf16(acc[ps][qs][0], acc[ps][qs][1]);
                o.y = pack_bf16(acc[ps][qs][2], acc[ps][qs][3]);
                *reinterpret_cast<uint2*>(outb + (row * a.ldo + col) * 2) = o;
            } else {
                f32x4* dst = reinterpret_cast<f32x4*>(outb + (row * a.ldo + col) * 4);
                f32x4 v = acc[ps][qs];
                if (a.accumulate) { f32x4 old = *dst; v = (f32x4){old.x + v.x, old.y + v.y, old.z + v.z, old.w + v.w}; }
                *dst = v;
            }
        }
    }
}

static int launch_gemm(const GemmArgs& a, int mode, dim3 grid, hipStream_t st, const char* where) {
    const size_t lds_bytes = 65536;
    if (mode == MODE_FWD) {
        if (a.sq_layout == 0) hipLaunchKernelGGL((k_gemm<MODE_FWD, 0>), grid, dim3(256), lds_bytes, st, a);
        else hipLaunchKernelGGL((k_gemm<MODE_FWD, 1>), grid, dim3(256), lds_bytes, st, a);
    } else {
        hipLaunchKernelGGL((k_gemm<MODE_WGRAD, 1>), grid, dim3(256), lds_bytes, st, a);
    }
    return pf8_check_launch(where);
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

static int ensure_lds_attr() {
    // 64 KB of dynamic LDS needs the opt-in attribute once per kernel instantiation
    static int done = 0;
    if (done) return PF8_OK;
    hipError_t e = hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm<MODE_FWD, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm<MODE_FWD, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_gemm<MODE_WGRAD, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    if (e != hipSuccess) return pf8_fail(PF8_ELAUNCH, "pf8_gemm", hipGetErrorString(e));
    done = 1;
    return PF8_OK;
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

extern "C" int pf8_gemm_nt_1d1d_f32(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t, int64_t Kin,
                                    int64_t N, int64_t M, float* out, int accumulate, pf8_stream_t stream) {
    PF8_REQUIRE(Kin >= 0 && N >= 0 && M >= 0, "negative shape");
    PF8_REQUIRE(M % 128 == 0, "M (the reduction axis) must be a multiple of 128");
    PF8_REQUIRE(N % 4 == 0, "N must be a multiple of 4");
    if (Kin == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(out, "null pointer");
    PF8_REQUIRE(M == 0 || (a_t && sa_t && b_t && sb_t), "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a_t) && PF8_ALIGNED16(b_t) && PF8_ALIGNED16(out) && PF8_ALIGNED16(sb_t), "pointers must be 16-byte aligned");
    if (M == 0 && accumulate) return PF8_OK;
    int rc = ensure_lds_attr();
    if (rc) return rc;
    GemmArgs g = {};
    g.p = b_t; g.q = a_t; g.sp = sb_t; g.sq = sa_t; g.out = out;
    g.Prows = N; g.Qrows = Kin; g.red = M; g.ldo = N; g.accumulate = accumulate; g.group = GROUP_NONE;
    const int64_t tiles = ((N + 127) / 128) * ((Kin + 127) / 128);
    PF8_REQUIRE(tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_WGRAD, dim3((unsigned)tiles), (hipStream_t)stream, __func__);
}

extern "C" int pf8_grouped_wgrad(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                                 const int64_t* rows_per_expert, int E, int64_t Kin, int64_t N, float* out, int accumulate,
                                 pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && Kin >= 0 && N >= 0, "negative shape");
    PF8_REQUIRE(E <= 256, "at most 256 experts per call");
    PF8_REQUIRE(N % 4 == 0, "N must be a multiple of 4");
    if (E == 0 || Kin == 0 || N == 0) return PF8_OK;
    PF8_REQUIRE(rows_per_expert && out, "null pointer");
    GemmArgs g = {};
    int64_t total = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE(rows_per_expert[e] >= 0 && rows_per_expert[e] % 128 == 0, "rows_per_expert entries must be non-negative multiples of 128");
        g.tile_start[e] = (int32_t)(total / 128);
        total += rows_per_expert[e];
    }
    g.tile_start[E] = (int32_t)(total / 128);
    PF8_REQUIRE(total == 0 || (a_t && sa_t && b_t && sb_t), "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(a_t) && PF8_ALIGNED16(b_t) && PF8_ALIGNED16(out) && PF8_ALIGNED16(sb_t), "pointers must be 16-byte aligned");
    if (total == 0 && accumulate) return PF8_OK;
    int rc = ensure_lds_attr();
    if (rc) return rc;
    g.p = b_t; g.q = a_t; g.sp = sb_t; g.sq = sa_t; g.out = out;
    g.Prows = N; g.Qrows = Kin; g.red = 0; g.ldo = N; g.accumulate = accumulate; g.group = GROUP_WGRAD; g.E = E;
    const int64_t tiles = ((N + 127) / 128) * ((Kin + 127) / 128);
    PF8_REQUIRE(tiles <= 0x7FFFFFFF, "too many tiles");
    return launch_gemm(g, MODE_WGRAD, dim3((unsigned)tiles, (unsigned)E), (hipStream_t)stream, __func__);
}
