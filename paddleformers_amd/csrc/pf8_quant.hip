// pf8_quant.hip -- bandwidth-bound block quantizers for gfx950 and their C entry points.
//
// Data layout in HBM: activations bf16 row-major [rows, K]; e4m3 bytes in the same shape; scales
// fp32 either [rows, K/128] or [K/128, rows].  One 1x128 tile = 256 B of bf16 = 16 lanes x 16 B, i.e.
// exactly one DPP row of a 64-wide wavefront, so the tile amax is four DPP max steps and never
// touches LDS.  2-D work (128x128 weight tiles, the fused row+column quantizer, the per-expert
// transposing quantizer) stages one 128x128 tile per 256-thread workgroup in registers (8x8
// elements per thread) and uses LDS only to turn the column-scaled bytes into 16-byte coalesced
// rows of the transposed output.
#include "pf8_device.h"
#include "pf8_host.h"

namespace pf8 {

// ---------------------------------------------------------------------------------------------
// 1x128 quantizer: one wavefront per row, four tiles per load instruction
// ---------------------------------------------------------------------------------------------

// grid.x = column chunks of 16 tiles, grid.y = groups of 4 rows; every lane issues its four 16-byte
// loads before any arithmetic, so a wavefront is one load phase, one compute phase, one store phase.
// The arithmetic has to hide behind the memory stream, so the bookkeeping around it is kept off the
// vector pipe:
//   * the row is wave-uniform: every address is a scalar base plus one 32-bit lane offset;
//   * the scales of a lane group's four tiles are computed in ONE pass (lane q of every quad takes
//     tile q; the IEEE divides for the scale and for its reciprocal run once, not four times) and come back through
//     quad-broadcast DPP operands.
template <int LAYOUT, int U>
__global__ __launch_bounds__(256) void k_quant_1x128(const uint16_t* __restrict__ x, int64_t M, int64_t m0, int KB, int64_t ldx,
                                                     uint8_t* __restrict__ q, float* __restrict__ s, int pow2) {
    static_assert(U == 4, "one quad lane per tile");
    const int lane = threadIdx.x & 63, g = lane >> 4, l = lane & 15;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t r = m0 + (int64_t)blockIdx.y * 4 + wave;   // m0: first row of this launch's slab
    if (r >= M) return;
    const int kb0 = blockIdx.x * 16;
    const uint8_t* xr = reinterpret_cast<const uint8_t*>(x + r * ldx);
    uint8_t* qr = q + r * (int64_t)KB * 128;
    const uint32_t in_off = (uint32_t)((kb0 + g) * 256 + l * 16);    // tile u adds u * 1024
    const uint32_t out_off = (uint32_t)((kb0 + g) * 128 + l * 8);    // tile u adds u * 512
    uint4 w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        w[u] = make_uint4(0, 0, 0, 0);
        if (kb0 + 4 * u + g < KB) w[u] = ld16(xr + in_off + u * 1024);
    }
    uint32_t am[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) am[u] = row16_max(amax_bits8(w[u]));
    const int ql = l & 3;
    const uint32_t am_sel = ql == 0 ? am[0] : ql == 1 ? am[1] : ql == 2 ? am[2] : am[3];
    const float sc = scale_of(am_sel, pow2 != 0);       // lane q of a quad: scale of tile q
    // its reciprocal: exponent arithmetic for a power of two, else ONE IEEE division per tile
    const bool slow = !(sc >= kMinFastScale);
    const float y = pow2 ? pow2_recip(sc) : 1.0f / (slow ? 1.0f : sc);
    if (l < 4) {
        const int kb = kb0 + 4 * l + g;
        if (kb < KB) {
            if (LAYOUT == 0) s[r * KB + kb] = sc;
            else if (LAYOUT == 1) s[(int64_t)kb * M + r] = sc;
            else reinterpret_cast<uint8_t*>(s)[(int64_t)kb * M + r] = (uint8_t)(f2u(sc) >> 23);     // UE8M0: the exponent field of a power of two
        }
    }
    // cross-lane reads see only active lanes: every broadcast happens while the wavefront is whole
    uint2 o[4];
    if (pow2) {
        float v[8];
        unpack8(w[0], v); o[0] = quant8_exact(v, quad_bcast<0>(y));
        unpack8(w[1], v); o[1] = quant8_exact(v, quad_bcast<1>(y));
        unpack8(w[2], v); o[2] = quant8_exact(v, quad_bcast<2>(y));
        unpack8(w[3], v); o[3] = quant8_exact(v, quad_bcast<3>(y));
    } else {
        float v[8];
        const float s0 = quad_bcast<0>(sc), s1 = quad_bcast<1>(sc), s2 = quad_bcast<2>(sc), s3 = quad_bcast<3>(sc);
        unpack8(w[0], v); o[0] = quant8_r(v, s0, quad_bcast<0>(y), !(s0 >= kMinFastScale));
        unpack8(w[1], v); o[1] = quant8_r(v, s1, quad_bcast<1>(y), !(s1 >= kMinFastScale));
        unpack8(w[2], v); o[2] = quant8_r(v, s2, quad_bcast<2>(y), !(s2 >= kMinFastScale));
        unpack8(w[3], v); o[3] = quant8_r(v, s3, quad_bcast<3>(y), !(s3 >= kMinFastScale));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (kb0 + 4 * u + g < KB) st8(qr + out_off + u * 512, o[u]);
}

// ---------------------------------------------------------------------------------------------
// fused SwiGLU (+probs) + 1x128 quantizer: one wavefront per row
// ---------------------------------------------------------------------------------------------

// Per output the kernel spends about 29 vector instructions, 17 of them SiLU (the exponential's short fixed sequence, one
// v_rcp_f32 and the three-instruction exact quotient).  Products are rounded to bf16 in pairs by the hardware convert and
// stay packed: the optional bf16 copy is stored as they are and amax runs on packed 16-bit magnitudes.
// U: 128-column blocks per lane group (a wavefront covers 4 U of them); the host picks the U that leaves fewer idle lane
// groups in a row's last wavefront (I = 1408: 11 blocks are three wavefronts of 4, not two of 8 with five groups idle).
template <int LAYOUT, bool HAS_P, int U>
__global__ __launch_bounds__(256) void k_swiglu_quant(const uint16_t* __restrict__ o1, const float* __restrict__ probs,
                                                      int64_t M, int64_t m0, int IB, uint8_t* __restrict__ q,
                                                      float* __restrict__ s, uint16_t* __restrict__ o2, int pow2) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, l = lane & 15;
    const int64_t r = m0 + (int64_t)blockIdx.y * 4 + wave;
    if (r >= M) return;
    const int kb0 = blockIdx.x * (4 * U);
    const int64_t I = (int64_t)IB * 128;
    const uint4* gr = reinterpret_cast<const uint4*>(o1 + r * 2 * I);
    const uint4* ur = reinterpret_cast<const uint4*>(o1 + r * 2 * I + I);
    uint2* qr = reinterpret_cast<uint2*>(q + r * I);
    const float p = HAS_P ? probs[r] : 1.0f;
    const ExpPoly poly = exp_poly_in_registers();
    uint4 wg[U], wu[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int kb = kb0 + 4 * u + g;
        wg[u] = make_uint4(0, 0, 0, 0);
        wu[u] = make_uint4(0, 0, 0, 0);
        if (kb < IB) {
            wg[u] = ld16(gr + kb * 16 + l);
            wu[u] = ld16(ur + kb * 16 + l);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int kb = kb0 + 4 * u + g;
        if (kb < IB) {
            const uint32_t gw[4] = {wg[u].x, wg[u].y, wg[u].z, wg[u].w}, uw[4] = {wu[u].x, wu[u].y, wu[u].z, wu[u].w};
            uint32_t pk[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t w = pack_bf16(silu_exact(bf16_lo(gw[i]), poly) * bf16_lo(uw[i]), silu_exact(bf16_hi(gw[i]), poly) * bf16_hi(uw[i]));
                if (HAS_P) w = pack_bf16(bf16_lo(w) * p, bf16_hi(w) * p);
                pk[i] = w;
            }
            if (o2) st16(o2 + r * I + kb * 128 + l * 8, make_uint4(pk[0], pk[1], pk[2], pk[3]));
            const uint32_t m = pkmax_u16(pkmax_u16(pk[0] & 0x7FFF7FFFu, pk[1] & 0x7FFF7FFFu), pkmax_u16(pk[2] & 0x7FFF7FFFu, pk[3] & 0x7FFF7FFFu));
            TileScale t = make_scale(row16_max(umax(m << 16, m & 0xFFFF0000u)), pow2 != 0);
            float v[8];
            unpack8(make_uint4(pk[0], pk[1], pk[2], pk[3]), v);
            uint2 o = quant8(v, t);
            st8(qr + kb * 16 + l, o);
            if (l == 0) {
                if (LAYOUT == 0) s[r * IB + kb] = t.s;
                else if (LAYOUT == 1) s[(int64_t)kb * M + r] = t.s;
                else reinterpret_cast<uint8_t*>(s)[(int64_t)kb * M + r] = (uint8_t)(f2u(t.s) >> 23);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// SwiGLU backward with probs: one wavefront per row
// ---------------------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void k_swiglu_bwd(const uint16_t* __restrict__ o1, const uint16_t* __restrict__ do2_s,
                                                    const float* __restrict__ probs, int64_t M, int64_t I,
                                                    uint16_t* __restrict__ do1, float* __restrict__ probs_grad,
                                                    uint16_t* __restrict__ o2_s) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + wave;
    if (r >= M) return;
    const float p = probs[r];
    const uint4* gr = reinterpret_cast<const uint4*>(o1 + r * 2 * I);
    const uint4* ur = reinterpret_cast<const uint4*>(o1 + r * 2 * I + I);
    const uint4* dr = reinterpret_cast<const uint4*>(do2_s + r * I);
    uint4* dgr = reinterpret_cast<uint4*>(do1 + r * 2 * I);
    uint4* dur = reinterpret_cast<uint4*>(do1 + r * 2 * I + I);
    uint4* osr = reinterpret_cast<uint4*>(o2_s + r * I);
    const int chunks = (int)(I / 8);
    const ExpPoly poly = exp_poly_in_registers();
    float pg = 0.0f;
    for (int c = lane; c < chunks; c += 64) {
        const uint4 wg = ld16(gr + c), wu = ld16(ur + c), wd = ld16(dr + c);
        float gv[8], uv[8], dv[8], dg[8], du[8], os[8];
        unpack8(wg, gv);
        unpack8(wu, uv);
        unpack8(wd, dv);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const SiluSigmoid ss = silu_and_sigmoid(gv[i], poly);       // g / den and 1 / den without the IEEE division sequence
            const float sl = ss.silu;
            float o2f = round_bf16(sl * uv[i]);
            os[i] = o2f * p;
            float do2 = round_bf16(dv[i] * p);
            pg += dv[i] * o2f;
            const float sig = ss.sigmoid;
            float t1 = 1.0f - sig;
            float t2 = gv[i] * t1;
            float t3 = 1.0f + t2;
            float t4 = sig * t3;
            float t5 = do2 * uv[i];
            dg[i] = t5 * t4;
            du[i] = do2 * sl;
        }
        uint4 a, b, o;
        a.x = pack_bf16(dg[0], dg[1]); a.y = pack_bf16(dg[2], dg[3]); a.z = pack_bf16(dg[4], dg[5]); a.w = pack_bf16(dg[6], dg[7]);
        b.x = pack_bf16(du[0], du[1]); b.y = pack_bf16(du[2], du[3]); b.z = pack_bf16(du[4], du[5]); b.w = pack_bf16(du[6], du[7]);
        o.x = pack_bf16(os[0], os[1]); o.y = pack_bf16(os[2], os[3]); o.z = pack_bf16(os[4], os[5]); o.w = pack_bf16(os[6], os[7]);
        st16(dgr + c, a);
        st16(dur + c, b);
        st16(osr + c, o);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) pg += __shfl_xor(pg, off);
    if (lane == 0) probs_grad[r] = pg;
}

// ---------------------------------------------------------------------------------------------
// 128x128-tile kernels: 256 threads, thread (g = tid/16, l = tid%16) owns rows 8g..8g+7 and
// columns 8l..8l+7 of the tile
// ---------------------------------------------------------------------------------------------

constexpr int LDT = 33;   // dwords per row of the transposed byte tile in LDS (128 B + 4 B pad)

// write one thread's column-major bytes (column 8l+j, rows 8g..8g+7) into the LDS tile
__device__ __forceinline__ void lds_put_col(uint32_t* lds_t, int l, int g, int j, uint2 bytes) {
    uint32_t* p = lds_t + (8 * l + j) * LDT + 2 * g;
    p[0] = bytes.x;
    p[1] = bytes.y;
}
// after a barrier: thread reads 16 bytes of transposed row c = (tid>>3) + 32*i
__device__ __forceinline__ uint4 lds_get_row(const uint32_t* lds_t, int c, int seg) {
    const uint32_t* p = lds_t + c * LDT + 4 * seg;
    return make_uint4(p[0], p[1], p[2], p[3]);
}

struct TileSrc {
    const uint16_t* x;     // bf16 source (or nullptr when the source is e4m3)
    const uint8_t* xq;     // e4m3 source
    const float* xs;       // scales of the e4m3 source: [rows, K/128] (xs_layout 0) or [K/128, rows] (1)
    int64_t ld;            // row stride in elements
    int64_t rows;          // total rows (for xs_layout 1)
    int xs_layout;
    const int32_t* src_row;   // row r of the tile grid is row src_row[r] of the source (negative = a row of zeros); null = r
};

// load this thread's 8x8 patch as fp32 values; amax bit patterns per row chunk go to rmax[i]
__device__ __forceinline__ void load_patch(const TileSrc& src, int64_t row0, int64_t col0, int g, int l, float (&v)[8][8]) {
    if (src.x) {
        uint4 w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            w[i] = ld16(src.x + (row0 + 8 * g + i) * src.ld + col0 + 8 * l);
#pragma unroll
        for (int i = 0; i < 8; ++i) unpack8(w[i], v[i]);
    } else {
        uint2 w[8];
        float sc[8];
        const int64_t KB = src.ld / 128;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int64_t r = row0 + 8 * g + i;
            w[i] = ld8(src.xq + r * src.ld + col0 + 8 * l);
            sc[i] = src.xs_layout == 0 ? src.xs[r * KB + col0 / 128] : src.xs[(col0 / 128) * src.rows + r];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float f[8];
            e4m3x4_to_f32(w[i].x, f);
            e4m3x4_to_f32(w[i].y, f + 4);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] = round_bf16(f[j] * sc[i]);
        }
    }
}

// reduce a per-thread value over the whole 256-thread workgroup (max of unsigned)
__device__ __forceinline__ uint32_t block_max(uint32_t v, uint32_t* lds4) {
    v = row16_max(v);
    v = umax(v, (uint32_t)__shfl_xor((int)v, 16));
    v = umax(v, (uint32_t)__shfl_xor((int)v, 32));
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
    __syncthreads();
    v = umax(umax(lds4[0], lds4[1]), umax(lds4[2], lds4[3]));
    return v;
}

struct StackArgs {
    const uint16_t* w[256];
};

// One staged 128x128 byte tile (row n of the LDS tile = weight row n0 + n, its 128 bytes = K block kb) written as the two
// 8 KB fragment-major blocks it fills (the order pf8_gemm_fm.hip describes and k_weight_to_fm produces from the plain
// bytes): chunk t = pf<<8 | kh<<7 | h<<6 | hh<<5 | x of a block is bytes 64 kh + 32 hh + 16 h .. + 15 of row 32 pf + x of its
// 64-row panel.  wf: the expert's fragment-major matrix, KB its K blocks per row.  A workgroup writes 4 KB per pass.
__device__ __forceinline__ void store_tile_fragment_major(const uint32_t* lds, uint8_t* __restrict__ wf, int64_t n0, int64_t KB, int64_t kb) {
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int ch = it * 256 + threadIdx.x;
        const int panel = ch >> 9, pf = (ch >> 8) & 1, kh = (ch >> 7) & 1, h = (ch >> 6) & 1, hh = (ch >> 5) & 1, x = ch & 31;
        const uint4 o = lds_get_row(lds, panel * 64 + pf * 32 + x, kh * 4 + hh * 2 + h);
        st16(wf + ((n0 / 64 + panel) * KB + kb) * 8192 + (ch & 511) * 16, o);
    }
}

// 128x128 block-scaled quantizer.  Source tile (tr, tc) of expert e; writes q (same orientation)
// and/or qt (transposed).  STACK: sources come from a pointer table, outputs are stacked per expert.
// FM: also the fragment-major copies of q and / or qt (q_fm, qt_fm; either may be null), made from the same registers.
template <bool STACK, bool FM = false>
__global__ __launch_bounds__(256) void k_quant_128x128(const uint16_t* __restrict__ w, StackArgs ptrs, int64_t R, int64_t C,
                                                       uint8_t* __restrict__ q, float* __restrict__ s, uint8_t* __restrict__ qt,
                                                       float* __restrict__ st, int pow2, uint8_t* __restrict__ q_fm,
                                                       uint8_t* __restrict__ qt_fm) {
    __shared__ uint32_t lds_t[128 * LDT];
    __shared__ uint32_t lds_r[FM ? 128 * LDT : 1];
    __shared__ uint32_t lds4[4];
    const int tid = threadIdx.x, g = tid >> 4, l = tid & 15;
    const int64_t CB = C / 128, RB = R / 128;
    const int64_t tc = blockIdx.x, tr = blockIdx.y, e = blockIdx.z;
    TileSrc src;
    src.x = STACK ? ptrs.w[e] : w;
    src.xq = nullptr; src.xs = nullptr; src.ld = C; src.rows = R; src.xs_layout = 0; src.src_row = nullptr;
    const int64_t row0 = tr * 128, col0 = tc * 128;
    float v[8][8];
    load_patch(src, row0, col0, g, l, v);
    uint32_t am = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) am = umax(am, f2u(v[i][j]) & 0x7FFFFFFFu);
    am = block_max(am, lds4);
    TileScale t = make_scale(am, pow2 != 0);
    const int64_t ebase = e * R * C;
    if (q) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint2 o = quant8(v[i], t);
            st8(q + ebase + (row0 + 8 * g + i) * C + col0 + 8 * l, o);
            if (FM && q_fm) {
                lds_r[(8 * g + i) * LDT + 2 * l] = o.x;
                lds_r[(8 * g + i) * LDT + 2 * l + 1] = o.y;
            }
        }
        if (tid == 0) s[e * RB * CB + tr * CB + tc] = t.s;
    }
    if (qt) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float col[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) col[i] = v[i][j];
            lds_put_col(lds_t, l, g, j, quant8(col, t));
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int c = (tid >> 3) + 32 * i, seg = tid & 7;
            uint4 o = lds_get_row(lds_t, c, seg);
            st16(qt + ebase + (col0 + c) * R + row0 + 16 * seg, o);
        }
        if (tid == 0) st[e * RB * CB + tc * RB + tr] = t.s;
        if (FM && qt_fm) store_tile_fragment_major(lds_t, qt_fm + ebase, col0, RB, tr);     // [C, R]: weight rows = columns here
    }
    if (FM && q && q_fm) {
        if (!qt) __syncthreads();              // with qt the barrier above has covered the row tile's writes as well
        store_tile_fragment_major(lds_r, q_fm + ebase, row0, CB, tc);
    }
}

struct SplitArgs {
    int32_t tile_start[257];   // first 128-row tile of each expert (prefix sums), tile_start[E] = total
    int32_t E;
};

// this thread's 8x8 patch as packed bf16 (one 16-byte chunk per row); an e4m3 source is dequantised
// to bf16 first (q * s rounded to nearest even), which is what the un-fused chain feeds the quantizer
__device__ __forceinline__ void load_patch_packed(const TileSrc& src, int64_t row0, int64_t col0, int g, int l, uint4 (&w)[8]) {
    if (src.x) {
        if (src.src_row) {
            // the thread's eight rows are consecutive: their sources are two 16-byte loads (row0 is a multiple of 128)
            const int4 r0 = *reinterpret_cast<const int4*>(src.src_row + row0 + 8 * g), r1 = *reinterpret_cast<const int4*>(src.src_row + row0 + 8 * g + 4);
            const int rr[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w[i] = rr[i] < 0 ? make_uint4(0, 0, 0, 0) : ld16(src.x + (int64_t)rr[i] * src.ld + col0 + 8 * l);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = ld16(src.x + (row0 + 8 * g + i) * src.ld + col0 + 8 * l);
        }
    } else {
        uint2 q[8];
        float sc[8];
        const int64_t KB = src.ld / 128;
        int rr[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (src.src_row) {
            const int4 r0 = *reinterpret_cast<const int4*>(src.src_row + row0 + 8 * g), r1 = *reinterpret_cast<const int4*>(src.src_row + row0 + 8 * g + 4);
            rr[0] = r0.x; rr[1] = r0.y; rr[2] = r0.z; rr[3] = r0.w; rr[4] = r1.x; rr[5] = r1.y; rr[6] = r1.z; rr[7] = r1.w;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int64_t r = row0 + 8 * g + i;
            if (src.src_row) r = rr[i];
            if (r < 0) {                // a zero byte times a zero scale, as the copied padding row holds them
                q[i] = make_uint2(0, 0);
                sc[i] = 0.0f;
                continue;
            }
            q[i] = ld8(src.xq + r * src.ld + col0 + 8 * l);
            if (src.xs_layout == 2) sc[i] = u2f((uint32_t)reinterpret_cast<const uint8_t*>(src.xs)[(col0 / 128) * src.rows + r] << 23);
            else sc[i] = src.xs_layout == 0 ? src.xs[r * KB + col0 / 128] : src.xs[(col0 / 128) * src.rows + r];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // hardware e4m3 -> fp32 (exact), two bytes per instruction
            const f32x2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[i].x, false), a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[i].x, true);
            const f32x2 b0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[i].y, false), b1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[i].y, true);
            const float f[8] = {a0[0] * sc[i], a0[1] * sc[i], a1[0] * sc[i], a1[1] * sc[i],
                                b0[0] * sc[i], b0[1] * sc[i], b1[0] * sc[i], b1[1] * sc[i]};
            w[i] = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
        }
    }
}

// Row-scaled copy (optional) + column-scaled transposed copy of one 128x128 tile.
//   SPLIT=false: q[M,K] + s, qt[K,M] + st                (fused quant+transpose)
//   SPLIT=true : qt / st packed per expert               (transpose-split-quant), source bf16 or e4m3
// pow2: bit 0 = power-of-two scales for the transposed copy, bit 1 = for the row-scaled copy.
// Per element the kernel spends one masked copy, two packed-u16 max (row and column amax), one
// unpack and two reciprocal-based quantizations; the 128 row scales and 128 column scales are each computed
// once (threads 0..127 / 128..255) and handed round through LDS instead of sixteen times over.
// LDS of one tile's quantization: the transposed byte tile, the per-wave packed column maxima, the row maxima and
// (s, 1/s, -, slow) for rows 0..127 / columns 128..255
struct RowColLds {
    uint32_t t[128 * LDT];
    uint32_t cm[4 * 64];
    uint32_t rm[128];
    float4 sc[256];
};

// expert of row tile tr: the last e with tile_start[e] <= tr, by bisection of the prefix table (E <= 256, uniform per
// workgroup; a linear scan is up to 255 dependent scalar loads)
__device__ __forceinline__ int split_expert_of(const SplitArgs& sp, int64_t tr) {
    int e = 0;
#pragma unroll
    for (int step = 128; step >= 1; step >>= 1)
        if (e + step < sp.E && (int64_t)sp.tile_start[e + step] <= tr) e += step;
    return e;
}

// The quantization of one tile whose packed bf16 patch the thread holds in w (rows 8g..8g+7, columns 8l..8l+7 of tile
// (tr, tc)), as k_quant_rowcol describes it.  Three barriers; a caller that runs it again on another patch needs none in
// between (the arrays a call writes first are read last two barriers earlier).  SPLIT: e_known is the expert of the row
// tile when the caller has looked it up already (-1: looked up here); the expert is returned.
template <bool SPLIT, int LAYOUT>
__device__ __forceinline__ int quant_rowcol_tile(const uint4 (&w)[8], int64_t tr, int64_t tc, int64_t M, int64_t K, uint8_t* __restrict__ q,
                                                  float* __restrict__ s, uint8_t* __restrict__ qt, float* __restrict__ st,
                                                  const SplitArgs& sp, int pow2, bool want_rows, RowColLds& L, int e_known = -1) {
    uint32_t* const lds_t = L.t;
    uint32_t* const lds_cm = L.cm;
    uint32_t* const lds_rm = L.rm;
    float4* const lds_sc = L.sc;
    const int tid = threadIdx.x, g = tid >> 4, l = tid & 15, wave = tid >> 6, lane = tid & 63;
    const int64_t KB = K / 128, MB = M / 128;
    const int64_t row0 = tr * 128, col0 = tc * 128;
    // ---- amax on the packed magnitudes ----
    uint32_t cmx = 0, cmy = 0, cmz = 0, cmw = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t ax = w[i].x & 0x7FFF7FFFu, ay = w[i].y & 0x7FFF7FFFu, az = w[i].z & 0x7FFF7FFFu, aw = w[i].w & 0x7FFF7FFFu;
        cmx = pkmax_u16(cmx, ax); cmy = pkmax_u16(cmy, ay); cmz = pkmax_u16(cmz, az); cmw = pkmax_u16(cmw, aw);
        if (want_rows) {
            const uint32_t m = pkmax_u16(pkmax_u16(ax, ay), pkmax_u16(az, aw));
            const uint32_t rm = row16_max(umax(m << 16, m & 0xFFFF0000u));
            if (l == i) lds_rm[8 * g + i] = rm;
        }
    }
    // columns: the 4 row groups of this wave, then the 4 waves through LDS
    cmx = pkmax_u16(cmx, (uint32_t)__shfl_xor((int)cmx, 16)); cmx = pkmax_u16(cmx, (uint32_t)__shfl_xor((int)cmx, 32));
    cmy = pkmax_u16(cmy, (uint32_t)__shfl_xor((int)cmy, 16)); cmy = pkmax_u16(cmy, (uint32_t)__shfl_xor((int)cmy, 32));
    cmz = pkmax_u16(cmz, (uint32_t)__shfl_xor((int)cmz, 16)); cmz = pkmax_u16(cmz, (uint32_t)__shfl_xor((int)cmz, 32));
    cmw = pkmax_u16(cmw, (uint32_t)__shfl_xor((int)cmw, 16)); cmw = pkmax_u16(cmw, (uint32_t)__shfl_xor((int)cmw, 32));
    if (lane < 16) {
        uint32_t* p = lds_cm + wave * 64 + 4 * l;
        p[0] = cmx; p[1] = cmy; p[2] = cmz; p[3] = cmw;
    }
    __syncthreads();

    // ---- one scale per row (threads 0..127) and per column (threads 128..255) ----
    {
        uint32_t am;
        if (tid < 128) {
            am = lds_rm[tid];
        } else {
            const int c = tid - 128;
            const uint32_t pk = pkmax_u16(pkmax_u16(lds_cm[c >> 1], lds_cm[64 + (c >> 1)]), pkmax_u16(lds_cm[128 + (c >> 1)], lds_cm[192 + (c >> 1)]));
            am = (c & 1) ? (pk & 0xFFFF0000u) : (pk << 16);
        }
        if (tid >= 128 || want_rows) {
            const TileScale t = make_scale(am, (pow2 & (tid < 128 ? 2 : 1)) != 0);
            lds_sc[tid] = make_float4(t.s, t.y, 0.0f, t.slow ? 1.0f : 0.0f);
        }
    }
    __syncthreads();

    // ---- quantise: rows straight to memory, columns into the transposed LDS tile.  Values are
    // unpacked from the packed patch where they are used (twice per element) instead of keeping 64
    // floats live: the kernel stays under 128 registers, so four workgroups share a compute unit.
    if (want_rows) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float4 f = lds_sc[8 * g + i];
            TileScale t; t.s = f.x; t.y = f.y; t.slow = f.w != 0.0f; t.exact = (pow2 & 2) != 0;
            const int64_t r = row0 + 8 * g + i;
            float v[8];
            unpack8(w[i], v);
            st8(q + r * K + col0 + 8 * l, quant8(v, t));
            if (l == i) {
                if (LAYOUT == 0) s[r * KB + tc] = t.s;
                else if (pow2 & 4) reinterpret_cast<uint8_t*>(s)[tc * M + r] = (uint8_t)(f2u(t.s) >> 23);      // UE8M0 bytes [K/128, M]
                else s[tc * M + r] = t.s;
            }
        }
    }
    float cs[8];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t d = k == 0 ? w[i].x : k == 1 ? w[i].y : k == 2 ? w[i].z : w[i].w;
            lo[i] = bf16_lo(d);
            hi[i] = bf16_hi(d);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = 2 * k + h;
            const float4 f = lds_sc[128 + 8 * l + j];
            TileScale t; t.s = f.x; t.y = f.y; t.slow = f.w != 0.0f; t.exact = (pow2 & 1) != 0;
            cs[j] = t.s;
            lds_put_col(lds_t, l, g, j, h == 0 ? quant8(lo, t) : quant8(hi, t));
        }
    }
    __syncthreads();

    // destination of the transposed tile
    int64_t qt_base, ldq;
    int e = e_known;
    if (SPLIT) {
        if (e < 0) e = split_expert_of(sp, tr);
        const int64_t off = (int64_t)sp.tile_start[e] * 128;                       // rows before this expert
        const int64_t Me = (int64_t)(sp.tile_start[e + 1] - sp.tile_start[e]) * 128;
        qt_base = off * K + (row0 - off);      // + c*Me
        ldq = Me;
    } else {
        qt_base = row0;
        ldq = M;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int c = (tid >> 3) + 32 * i, seg = tid & 7;
        uint4 o = lds_get_row(lds_t, c, seg);
        st16(qt + qt_base + (col0 + c) * ldq + 16 * seg, o);
    }
    if (g == 0) {
        if (LAYOUT == 1 || SPLIT) {
            // scale rows are tile rows, globally numbered (an expert's block starts at its first tile)
            float4* p = reinterpret_cast<float4*>(st + tr * K + col0 + 8 * l);
            p[0] = make_float4(cs[0], cs[1], cs[2], cs[3]);
            p[1] = make_float4(cs[4], cs[5], cs[6], cs[7]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) st[(col0 + 8 * l + j) * MB + tr] = cs[j];
        }
    }
    return e;
}

template <bool SPLIT, int LAYOUT>
__global__ __launch_bounds__(256, 4) void k_quant_rowcol(TileSrc src, int64_t M, int64_t K, uint8_t* __restrict__ q,
                                                      float* __restrict__ s, uint8_t* __restrict__ qt, float* __restrict__ st,
                                                      SplitArgs sp, int pow2) {
    __shared__ RowColLds L;
    const int tid = threadIdx.x, g = tid >> 4, l = tid & 15;
    const int64_t KB = K / 128, MB = M / 128;
    // Consecutive workgroups go round-robin to the 8 XCDs: every XCD gets a contiguous run of tiles, walked in bands of four
    // row tiles x all column tiles, row tile fastest.  The four workgroups that run side by side on an XCD then write four
    // adjacent 128-byte pieces of every transposed row and four consecutive row bands of the row-scaled copy, which its L2
    // hands to memory as longer runs than the 128-byte pieces of a plain grid (adjacent column tiles on eight different
    // XCDs): 103 -> 95 us on [16384, 7168].
    // (32-bit arithmetic: the host admits at most 2^31 tiles, and four 64-bit divisions are several hundred dependent
    // scalar instructions in front of every tile)
    const uint32_t nt = (uint32_t)(KB * MB), per_xcd = (nt + 7u) / 8u;
    const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= per_xcd || logical >= nt) return;
    const uint32_t band_w = 4u * (uint32_t)KB, band = logical / band_w, in_band = logical - band * band_w;
    const uint32_t band_h = (uint32_t)MB - band * 4u < 4u ? (uint32_t)MB - band * 4u : 4u;
    const uint32_t tc32 = in_band / band_h;
    const int64_t tr = band * 4u + (in_band - tc32 * band_h), tc = tc32;
    uint4 w[8];
    load_patch_packed(src, tr * 128, tc * 128, g, l, w);
    quant_rowcol_tile<SPLIT, LAYOUT>(w, tr, tc, M, K, q, s, qt, st, sp, pow2, q != nullptr, L);
}

// makes the four words values the compiler has to hold in registers at this point of the program
__device__ __forceinline__ void pin_words(uint4& w) {
    asm volatile("" : "+v"(w.x), "+v"(w.y), "+v"(w.z), "+v"(w.w));
}

// SwiGLU backward with probs on one 128x128 tile of the [M, I] grid, its three results quantized where they are made:
// do1 = [d gate | d up] ([M, 2I]) row-scaled (q, s) and column-scaled, transposed per expert (qt, st); o2_s ([M, I])
// column-scaled, transposed per expert (oqt, ost).  Every value takes the arithmetic of k_swiglu_bwd and is rounded to
// bf16 before it is quantized, so the bytes and scales are those of k_quant_rowcol<true, 1> on the tensors k_swiglu_bwd
// writes; neither tensor exists in memory here.  probs_grad leaves as one partial sum per row and column tile
// (pg_part [I/128, M]) that k_sum_row_partials adds up in the order of the tiles.  LAYOUT: do1's row scales as [M, 2I/128]
// (0) or [2I/128, M] (1).
// (three workgroups per compute unit; the row-major scale stores of LAYOUT 0 need a few registers more than that leaves)
template <int LAYOUT>
__global__ __launch_bounds__(256, LAYOUT == 1 ? 3 : 2) void k_swiglu_bwd_quant(const uint16_t* __restrict__ o1, const uint16_t* __restrict__ do2_s,
                                                          const float* __restrict__ probs, int64_t M, int64_t I,
                                                          uint8_t* __restrict__ q, float* __restrict__ s, uint8_t* __restrict__ qt,
                                                          float* __restrict__ st, uint8_t* __restrict__ oqt, float* __restrict__ ost,
                                                          float* __restrict__ pg_part, SplitArgs sp, int pow2) {
    __shared__ RowColLds L;
    const int tid = threadIdx.x, g = tid >> 4, l = tid & 15;
    const int64_t IB = I / 128, MB = M / 128;
    // tile order of k_quant_rowcol: a contiguous run of tiles per XCD, bands of four row tiles, row tile fastest
    const uint32_t nt = (uint32_t)(IB * MB), per_xcd = (nt + 7u) / 8u;
    const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= per_xcd || logical >= nt) return;
    const uint32_t band_w = 4u * (uint32_t)IB, band = logical / band_w, in_band = logical - band * band_w;
    const uint32_t band_h = (uint32_t)MB - band * 4u < 4u ? (uint32_t)MB - band * 4u : 4u;
    const uint32_t tc32 = in_band / band_h;
    const int64_t tr = band * 4u + (in_band - tc32 * band_h), tc = tc32;
    const int64_t r0 = tr * 128 + 8 * g, c0 = tc * 128 + 8 * l;       // this thread's first row and column

    uint4 wg[8], wu[8], wd[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        wg[i] = ld16(o1 + (r0 + i) * 2 * I + c0);
        wu[i] = ld16(o1 + (r0 + i) * 2 * I + I + c0);
        wd[i] = ld16(do2_s + (r0 + i) * I + c0);
    }
    const float4 p0 = *reinterpret_cast<const float4*>(probs + r0), p1 = *reinterpret_cast<const float4*>(probs + r0 + 4);
    const float pr[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
    const int e = split_expert_of(sp, tr);
    const ExpPoly poly = exp_poly_in_registers();

    uint4 a[8], b[8], o[8];       // d gate, d up and o2_s of the patch, packed bf16
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float gv[8], uv[8], dv[8], dg[8], du[8], os[8];
        unpack8(wg[i], gv);
        unpack8(wu[i], uv);
        unpack8(wd[i], dv);
        const float p = pr[i];
        float pg = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const SiluSigmoid ss = silu_and_sigmoid(gv[j], poly);
            const float sl = ss.silu;
            const float o2f = round_bf16(sl * uv[j]);
            os[j] = o2f * p;
            const float do2 = round_bf16(dv[j] * p);
            pg += dv[j] * o2f;
            const float sig = ss.sigmoid;
            const float t1 = 1.0f - sig;
            const float t2 = gv[j] * t1;
            const float t3 = 1.0f + t2;
            const float t4 = sig * t3;
            const float t5 = do2 * uv[j];
            dg[j] = t5 * t4;
            du[j] = do2 * sl;
        }
        a[i].x = pack_bf16(dg[0], dg[1]); a[i].y = pack_bf16(dg[2], dg[3]); a[i].z = pack_bf16(dg[4], dg[5]); a[i].w = pack_bf16(dg[6], dg[7]);
        b[i].x = pack_bf16(du[0], du[1]); b[i].y = pack_bf16(du[2], du[3]); b[i].z = pack_bf16(du[4], du[5]); b[i].w = pack_bf16(du[6], du[7]);
        o[i].x = pack_bf16(os[0], os[1]); o[i].y = pack_bf16(os[2], os[3]); o[i].z = pack_bf16(os[4], os[5]); o[i].w = pack_bf16(os[6], os[7]);
        // the packed words are made here: left to itself the compiler sinks the arithmetic behind them into the three
        // quantizations and keeps every element's intermediate values alive instead (hundreds of registers)
        pin_words(a[i]);
        pin_words(b[i]);
        pin_words(o[i]);
        // the row's 128 terms of this tile: eight per lane, then the sixteen lanes of the row group
        pg += __shfl_xor(pg, 1);
        pg += __shfl_xor(pg, 2);
        pg += __shfl_xor(pg, 4);
        pg += __shfl_xor(pg, 8);
        if (l == i) pg_part[tc * M + r0 + i] = pg;
        // one row at a time: interleaved, the eight rows' temporaries do not fit the register file next to the patches
        __builtin_amdgcn_sched_barrier(0);
    }
    quant_rowcol_tile<true, LAYOUT>(a, tr, tc, M, 2 * I, q, s, qt, st, sp, pow2, true, L, e);
    quant_rowcol_tile<true, LAYOUT>(b, tr, tc + IB, M, 2 * I, q, s, qt, st, sp, pow2, true, L, e);
    quant_rowcol_tile<true, 1>(o, tr, tc, M, I, nullptr, nullptr, oqt, ost, sp, pow2 & 1, false, L, e);
}

// out[r] = part[0][r] + part[1][r] + ... + part[n-1][r], added in that order
__global__ __launch_bounds__(256) void k_sum_row_partials(const float* __restrict__ part, int n, int64_t M, float* __restrict__ out) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= M) return;
    float acc = part[r];
    for (int k = 1; k < n; ++k) acc += part[(int64_t)k * M + r];
    out[r] = acc;
}

// ---------------------------------------------------------------------------------------------
// dequantizers
// ---------------------------------------------------------------------------------------------

// 1x128 dequant: one thread per 8 bytes.  IDX: integer type of the index arithmetic, 32-bit whenever the tensor allows it
// (a 64-bit division per thread is emulated and costs more than the data movement)
template <int LAYOUT, typename IDX>
__global__ __launch_bounds__(256) void k_act_dequant(const uint8_t* __restrict__ q, const float* __restrict__ s, int64_t M,
                                                     int64_t K, uint16_t* __restrict__ out) {
    const IDX idx = (IDX)blockIdx.x * 256 + threadIdx.x;   // 8-byte chunk index
    const IDX cpr = (IDX)(K / 8);
    if ((int64_t)idx >= M * (K / 8)) return;
    const IDX r32 = idx / cpr, c8 = idx - r32 * cpr;
    const int64_t r = r32;
    const int64_t kb = c8 / 16, KB = K / 128;
    const float sc = LAYOUT == 0 ? s[r * KB + kb] : s[kb * M + r];
    const uint2 w = ld8(q + (int64_t)idx * 8);
    float f[8];
    e4m3x4_to_f32(w.x, f);
    e4m3x4_to_f32(w.y, f + 4);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] *= sc;
    uint4 o;
    o.x = pack_bf16(f[0], f[1]); o.y = pack_bf16(f[2], f[3]); o.z = pack_bf16(f[4], f[5]); o.w = pack_bf16(f[6], f[7]);
    st16(out + (int64_t)idx * 8, o);
}

// ---------------------------------------------------------------------------------------------
// Block-FP8 checkpoint dequantization: out = cast(e4m3(q) * scale(block)), any block geometry on the
// last two axes, partial trailing blocks cropped, scales as UE8M0 exponent bytes or fp32/bf16/fp16.
// One thread per 16 consecutive bytes of a row; HBM-bound (1 B in, 2 or 4 B out).  IDX is the
// integer type of the index arithmetic: 32-bit whenever the tensor allows it (64-bit divisions are
// emulated and would cost more than the data movement).
// ---------------------------------------------------------------------------------------------
enum { SCALE_F32 = 0, SCALE_UE8M0 = 1, SCALE_BF16 = 2, SCALE_F16 = 3 };

__device__ __forceinline__ float load_block_scale(const void* s, int fmt, int64_t i) {
    if (fmt == SCALE_F32) return reinterpret_cast<const float*>(s)[i];
    if (fmt == SCALE_UE8M0) {
        const uint32_t e = reinterpret_cast<const uint8_t*>(s)[i];
        // 2^(e-127): exponent field e, e == 0 is the subnormal 2^-127, e == 255 decodes to +inf
        return e == 0u ? u2f(0x00400000u) : u2f(e << 23);
    }
    if (fmt == SCALE_BF16) return u2f((uint32_t)reinterpret_cast<const uint16_t*>(s)[i] << 16);
    return (float)reinterpret_cast<const _Float16*>(s)[i];
}

template <int OUT_F32, typename IDX>
__global__ __launch_bounds__(256) void k_block_dequant(const uint8_t* __restrict__ q, const void* __restrict__ s, int fmt, int64_t B,
                                                       int64_t R, int64_t C, int64_t br, int64_t bc, void* __restrict__ out) {
    const IDX chunks = (IDX)((C + 15) / 16);
    const IDX idx = (IDX)blockIdx.x * 256 + threadIdx.x;
    if ((int64_t)idx >= B * R * (int64_t)chunks) return;
    const IDX ch = idx % chunks, row = idx / chunks;               // row runs over B * R
    const IDX b = row / (IDX)R, r = row % (IDX)R;
    const IDX gr = (IDX)((R + br - 1) / br), gc = (IDX)((C + bc - 1) / bc);
    const IDX c0 = ch * 16;
    const int n = (IDX)C - c0 < 16 ? (int)((IDX)C - c0) : 16;
    const int64_t srow = ((int64_t)b * gr + r / (IDX)br) * gc;
    const IDX cb0 = c0 / (IDX)bc, cb1 = (c0 + n - 1) / (IDX)bc;
    const uint8_t* qp = q + (int64_t)row * C + c0;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    const bool vec = n == 16 && ((reinterpret_cast<uintptr_t>(qp) & 15u) == 0);
    if (vec) {
        const uint4 v = ld16(qp);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else {
        for (int i = 0; i < n; ++i) w[i >> 2] |= (uint32_t)qp[i] << (8 * (i & 3));
    }
    float f[16];
    const bool one_scale = cb0 == cb1;
    const float s0 = load_block_scale(s, fmt, srow + cb0);
#pragma unroll
    for (int i = 0; i < 4; ++i) e4m3x4_to_f32(w[i], f + 4 * i);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        float sc = s0;
        if (!one_scale && i < n) sc = load_block_scale(s, fmt, srow + (c0 + i) / (IDX)bc);
        f[i] *= sc;
    }
    if (OUT_F32) {
        float* op = reinterpret_cast<float*>(out) + (int64_t)row * C + c0;
        if (vec && (reinterpret_cast<uintptr_t>(op) & 15u) == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) reinterpret_cast<f32x4*>(op)[i] = (f32x4){f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]};
        } else {
            for (int i = 0; i < n; ++i) op[i] = f[i];
        }
    } else {
        uint16_t* op = reinterpret_cast<uint16_t*>(out) + (int64_t)row * C + c0;
        if (vec && (reinterpret_cast<uintptr_t>(op) & 15u) == 0) {
            // plain stores: a lane writes 32 bytes as two halves, so one store instruction leaves every 128-byte line half
            // written, and with the non-temporal hint the halves reach memory apart (0.87 against 0.51 ms on 2.8 GB)
            uint4* o4 = reinterpret_cast<uint4*>(op);
            o4[0] = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
            o4[1] = make_uint4(pack_bf16(f[8], f[9]), pack_bf16(f[10], f[11]), pack_bf16(f[12], f[13]), pack_bf16(f[14], f[15]));
        } else {
            for (int i = 0; i < n; ++i) op[i] = (uint16_t)(pack_bf16(f[i], 0.0f) & 0xFFFFu);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// self-test kernels
// ---------------------------------------------------------------------------------------------

// plain 16-byte-per-lane copy of known size: the yardstick the HBM traffic counters are scaled by
__global__ __launch_bounds__(256) void k_debug_copy(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) st16(dst + i, ld16(src + i));      // the yardstick carries the same non-temporal hints as the kernels measured against it
}
__global__ void k_debug_encode(const float* v, int64_t n, uint8_t* out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (uint8_t)(cvt_e4m3_lo(v[i], 0.0f, 0u) & 0xFFu);
}
__global__ void k_debug_div_encode(const float* x, const float* s, int64_t n, uint8_t* out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    TileScale t = make_scale_from(s[i]);
    float v[8] = {x[i], 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    uint2 o = quant8(v, t);
    out[i] = (uint8_t)(o.x & 0xFFu);
}
__global__ void k_debug_silu(const float* x, int64_t n, float* out, float* out_sigmoid) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    out[i] = silu_exact(x[i]);
    if (out_sigmoid) out_sigmoid[i] = silu_and_sigmoid(x[i], exp_poly()).sigmoid;
}

}  // namespace pf8

using namespace pf8;

// ---------------------------------------------------------------------------------------------
// C entry points
// ---------------------------------------------------------------------------------------------

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

extern "C" int pf8_quant_1x128(const uint16_t* x, int64_t M, int64_t K, int64_t ldx, uint8_t* q, float* s, int scale_layout,
                               int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0, "K must be a multiple of 128");
    if (M == 0 || K == 0) return PF8_OK;
    PF8_REQUIRE(x && q && s, "null pointer");
    PF8_REQUIRE(ldx >= K && ldx % 8 == 0, "ldx must be >= K and a multiple of 8");
    PF8_REQUIRE(PF8_ALIGNED16(x) && PF8_ALIGNED16(q) && (scale_layout == 2 || (reinterpret_cast<uintptr_t>(s) & 3u) == 0), "pointers must be 16-byte aligned");
    PF8_REQUIRE(scale_layout >= 0 && scale_layout <= 2, "scale_layout must be 0, 1 or 2");
    PF8_REQUIRE(scale_layout != 2 || pow2, "UE8M0 scale bytes (scale_layout 2) need power-of-two scales");
    PF8_REQUIRE(K / 128 <= 0x7FFFFF, "shape too large");
    hipStream_t st = (hipStream_t)stream;
    const int KB = (int)(K / 128);
    constexpr int U = 4;
    // grid.y is limited to 65535 workgroups of 4 rows: larger inputs are walked in slabs
    const int64_t slab = (int64_t)65535 * 4;
    for (int64_t m0 = 0; m0 < M; m0 += slab) {
        const int64_t m = M - m0 < slab ? M - m0 : slab;
        dim3 grid((unsigned)((KB + 4 * U - 1) / (4 * U)), (unsigned)((m + 3) / 4)), block(256);
        if (scale_layout == 0) hipLaunchKernelGGL((k_quant_1x128<0, U>), grid, block, 0, st, x, M, m0, KB, ldx, q, s, pow2);
        else if (scale_layout == 1) hipLaunchKernelGGL((k_quant_1x128<1, U>), grid, block, 0, st, x, M, m0, KB, ldx, q, s, pow2);
        else hipLaunchKernelGGL((k_quant_1x128<2, U>), grid, block, 0, st, x, M, m0, KB, ldx, q, s, pow2);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    return PF8_OK;
}

extern "C" int pf8_quant_128x128(const uint16_t* w, int64_t R, int64_t C, uint8_t* q, float* s, uint8_t* q_t, float* s_t,
                                 int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(R >= 0 && C >= 0, "negative shape");
    PF8_REQUIRE(R % 128 == 0 && C % 128 == 0, "R and C must be multiples of 128");
    if (R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(w, "null pointer");
    PF8_REQUIRE((q != nullptr) == (s != nullptr) && (q_t != nullptr) == (s_t != nullptr), "q/s and q_t/s_t come in pairs");
    PF8_REQUIRE(q || q_t, "no output requested");
    PF8_REQUIRE(PF8_ALIGNED16(w) && PF8_ALIGNED16(q) && PF8_ALIGNED16(q_t), "pointers must be 16-byte aligned");
    PF8_REQUIRE(R / 128 <= 65535 && C / 128 <= 0x7FFFFFFF, "shape too large");
    dim3 grid((unsigned)(C / 128), (unsigned)(R / 128), 1), block(256);
    StackArgs none = {};
    hipLaunchKernelGGL(k_quant_128x128<false>, grid, block, 0, (hipStream_t)stream, w, none, R, C, q, s, q_t, s_t, pow2, (uint8_t*)nullptr,
                       (uint8_t*)nullptr);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_stack_transpose_quant(const uint16_t* const* w_list, int E, int64_t R, int64_t C, int transpose, uint8_t* q,
                                         float* s, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && R >= 0 && C >= 0, "negative shape");
    PF8_REQUIRE(R % 128 == 0 && C % 128 == 0, "R and C must be multiples of 128");
    if (E == 0 || R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(w_list && q && s, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(q), "pointers must be 16-byte aligned");
    PF8_REQUIRE(R / 128 <= 65535, "shape too large");
    for (int e = 0; e < E; ++e) PF8_REQUIRE(w_list[e] && PF8_ALIGNED16(w_list[e]), "null or misaligned weight pointer");
    const int64_t per_q = R * C, per_s = (R / 128) * (C / 128);
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int n = E - e0 < 256 ? E - e0 : 256;
        StackArgs a = {};
        for (int i = 0; i < n; ++i) a.w[i] = w_list[e0 + i];
        dim3 grid((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)n), block(256);
        uint8_t* qe = q + (int64_t)e0 * per_q;
        float* se = s + (int64_t)e0 * per_s;
        if (transpose)
            hipLaunchKernelGGL(k_quant_128x128<true>, grid, block, 0, (hipStream_t)stream, nullptr, a, R, C, (uint8_t*)nullptr,
                               (float*)nullptr, qe, se, pow2, (uint8_t*)nullptr, (uint8_t*)nullptr);
        else
            hipLaunchKernelGGL(k_quant_128x128<true>, grid, block, 0, (hipStream_t)stream, nullptr, a, R, C, qe, se,
                               (uint8_t*)nullptr, (float*)nullptr, pow2, (uint8_t*)nullptr, (uint8_t*)nullptr);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    return PF8_OK;
}

extern "C" int pf8_stack_quant_both(const uint16_t* const* w_list, int E, int64_t R, int64_t C, uint8_t* q, float* s,
                                    uint8_t* q_t, float* s_t, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && R >= 0 && C >= 0, "negative shape");
    PF8_REQUIRE(R % 128 == 0 && C % 128 == 0, "R and C must be multiples of 128");
    if (E == 0 || R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(w_list && q && s && q_t && s_t, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(q) && PF8_ALIGNED16(q_t), "pointers must be 16-byte aligned");
    PF8_REQUIRE(R / 128 <= 65535, "shape too large");
    for (int e = 0; e < E; ++e) PF8_REQUIRE(w_list[e] && PF8_ALIGNED16(w_list[e]), "null or misaligned weight pointer");
    const int64_t per_q = R * C, per_s = (R / 128) * (C / 128);
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int n = E - e0 < 256 ? E - e0 : 256;
        StackArgs a = {};
        for (int i = 0; i < n; ++i) a.w[i] = w_list[e0 + i];
        dim3 grid((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)n), block(256);
        hipLaunchKernelGGL(k_quant_128x128<true>, grid, block, 0, (hipStream_t)stream, nullptr, a, R, C,
                           q + (int64_t)e0 * per_q, s + (int64_t)e0 * per_s, q_t + (int64_t)e0 * per_q, s_t + (int64_t)e0 * per_s, pow2,
                           (uint8_t*)nullptr, (uint8_t*)nullptr);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    return PF8_OK;
}

extern "C" int pf8_stack_quant_both_fm(const uint16_t* const* w_list, int E, int64_t R, int64_t C, uint8_t* q, float* s,
                                       uint8_t* q_t, float* s_t, uint8_t* q_fm, uint8_t* q_t_fm, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && R >= 0 && C >= 0, "negative shape");
    PF8_REQUIRE(R % 128 == 0 && C % 128 == 0, "R and C must be multiples of 128");
    if (E == 0 || R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(w_list && q && s && q_t && s_t, "null pointer");
    PF8_REQUIRE(q_fm || q_t_fm, "no fragment-major output asked for (pf8_stack_quant_both makes the plain copies)");
    PF8_REQUIRE(PF8_ALIGNED16(q) && PF8_ALIGNED16(q_t) && PF8_ALIGNED16(q_fm) && PF8_ALIGNED16(q_t_fm), "pointers must be 16-byte aligned");
    PF8_REQUIRE(R / 128 <= 65535, "shape too large");
    for (int e = 0; e < E; ++e) PF8_REQUIRE(w_list[e] && PF8_ALIGNED16(w_list[e]), "null or misaligned weight pointer");
    const int64_t per_q = R * C, per_s = (R / 128) * (C / 128);
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int n = E - e0 < 256 ? E - e0 : 256;
        StackArgs a = {};
        for (int i = 0; i < n; ++i) a.w[i] = w_list[e0 + i];
        dim3 grid((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)n), block(256);
        hipLaunchKernelGGL((k_quant_128x128<true, true>), grid, block, 0, (hipStream_t)stream, nullptr, a, R, C,
                           q + (int64_t)e0 * per_q, s + (int64_t)e0 * per_s, q_t + (int64_t)e0 * per_q, s_t + (int64_t)e0 * per_s, pow2,
                           q_fm ? q_fm + (int64_t)e0 * per_q : nullptr, q_t_fm ? q_t_fm + (int64_t)e0 * per_q : nullptr);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    return PF8_OK;
}

extern "C" int pf8_quant_transpose(const uint16_t* x, int64_t M, int64_t K, uint8_t* q, float* s, uint8_t* q_t, float* s_t,
                                   int scale_layout, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(M % 128 == 0 && K % 128 == 0, "M and K must be multiples of 128");
    if (M == 0 || K == 0) return PF8_OK;
    PF8_REQUIRE(x && q_t && s_t, "null pointer");
    PF8_REQUIRE((q != nullptr) == (s != nullptr), "q and s come as a pair");
    PF8_REQUIRE(PF8_ALIGNED16(x) && PF8_ALIGNED16(q) && PF8_ALIGNED16(q_t) && PF8_ALIGNED16(s_t), "pointers must be 16-byte aligned");
    PF8_REQUIRE(scale_layout == 0 || scale_layout == 1, "scale_layout must be 0 or 1");
    PF8_REQUIRE((K / 128) * (M / 128) <= 0x7FFFFFF0ll, "too many tiles");
    TileSrc src = {x, nullptr, nullptr, K, M, 0, nullptr};
    SplitArgs sp = {};
    dim3 grid((unsigned)(((K / 128) * (M / 128) + 7) / 8 * 8)), block(256);
    if (scale_layout == 0)
        hipLaunchKernelGGL((k_quant_rowcol<false, 0>), grid, block, 0, (hipStream_t)stream, src, M, K, q, s, q_t, s_t, sp, pow2 ? 3 : 0);
    else
        hipLaunchKernelGGL((k_quant_rowcol<false, 1>), grid, block, 0, (hipStream_t)stream, src, M, K, q, s, q_t, s_t, sp, pow2 ? 3 : 0);
    return pf8_check_launch(__func__);
}

// shared by pf8_transpose_split_quant and pf8_quant_and_transpose_split: q/s null = no row-scaled copy
static int transpose_split_quant(const char* where, const void* x, const float* xs, int x_is_fp8, int xs_layout,
                                 const int64_t* rows_per_expert, int E, int64_t K, uint8_t* q, float* s, uint8_t* q_t, float* s_t,
                                 int pow2_bits, pf8_stream_t stream, const int32_t* src_row = nullptr, int64_t src_rows = 0) {
#define PF8_REQUIRE_AT(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, where, msg); } while (0)
    PF8_REQUIRE_AT(xs_layout >= 0 && xs_layout <= 2, "xs_layout must be 0, 1 or 2");
    PF8_REQUIRE_AT(E >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE_AT(K % 128 == 0, "K must be a multiple of 128");
    PF8_REQUIRE_AT(E <= 256, "at most 256 experts per call");
    if (E == 0 || K == 0) return PF8_OK;
    PF8_REQUIRE_AT(rows_per_expert, "null pointer");
    SplitArgs sp = {};
    int64_t total = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE_AT(rows_per_expert[e] >= 0 && rows_per_expert[e] % 128 == 0, "rows_per_expert entries must be non-negative multiples of 128");
        sp.tile_start[e] = (int32_t)(total / 128);
        total += rows_per_expert[e];
    }
    PF8_REQUIRE_AT(total / 128 <= 65535 && (K / 128) * (total / 128) <= 0x7FFFFFF0ll, "too many rows");
    sp.tile_start[E] = (int32_t)(total / 128);
    sp.E = E;
    if (total == 0) return PF8_OK;
    PF8_REQUIRE_AT(x && q_t && s_t, "null pointer");
    PF8_REQUIRE_AT(!x_is_fp8 || xs, "fp8 input needs its scales");
    PF8_REQUIRE_AT(PF8_ALIGNED16(x) && PF8_ALIGNED16(q_t) && PF8_ALIGNED16(s_t) && PF8_ALIGNED16(q), "pointers must be 16-byte aligned");
#undef PF8_REQUIRE_AT
    TileSrc src;
    src.x = x_is_fp8 ? nullptr : (const uint16_t*)x;
    src.xq = x_is_fp8 ? (const uint8_t*)x : nullptr;
    src.xs = xs;
    src.ld = K;
    src.rows = src_row ? src_rows : total;
    src.xs_layout = xs_layout;
    src.src_row = src_row;
    dim3 grid((unsigned)(((K / 128) * (total / 128) + 7) / 8 * 8)), block(256);
    hipLaunchKernelGGL((k_quant_rowcol<true, 1>), grid, block, 0, (hipStream_t)stream, src, total, K, q, s, q_t, s_t, sp, pow2_bits);
    return pf8_check_launch(where);
}

extern "C" int pf8_transpose_split_quant(const void* x, const float* xs, int x_is_fp8, int xs_layout, const int64_t* rows_per_expert,
                                         int E, int64_t K, uint8_t* q_t, float* s_t, int pow2, pf8_stream_t stream) {
    return transpose_split_quant(__func__, x, xs, x_is_fp8, xs_layout, rows_per_expert, E, K, nullptr, nullptr, q_t, s_t, pow2 ? 1 : 0, stream);
}

extern "C" int pf8_transpose_split_quant_gather(const void* tokens, const float* token_scales, int x_is_fp8, int xs_layout, int64_t T,
                                                const int32_t* src_row, const int64_t* rows_per_expert, int E, int64_t K, uint8_t* q_t,
                                                float* s_t, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(T > 0, "the token matrix is empty");
    PF8_REQUIRE(src_row && PF8_ALIGNED16(src_row), "src_row must be a 16-byte aligned device pointer");
    return transpose_split_quant(__func__, tokens, token_scales, x_is_fp8, xs_layout, rows_per_expert, E, K, nullptr, nullptr, q_t, s_t,
                                 pow2 ? 1 : 0, stream, src_row, T);
}

extern "C" int pf8_quant_and_transpose_split(const uint16_t* x, const int64_t* rows_per_expert, int E, int64_t K, uint8_t* q, float* s,
                                             int pow2_rows, uint8_t* q_t, float* s_t, int pow2_t, pf8_stream_t stream) {
    PF8_REQUIRE(q && s, "null pointer");
    // pow2_rows == 2: the row scales (powers of two) are written as UE8M0 bytes [K/128, Mtot] into s
    return transpose_split_quant(__func__, x, nullptr, 0, 0, rows_per_expert, E, K, q, s, q_t, s_t,
                                 (pow2_t ? 1 : 0) | (pow2_rows ? 2 : 0) | (pow2_rows == 2 ? 4 : 0), stream);
}

extern "C" int pf8_swiglu_weighted_quant(const uint16_t* o1, const float* probs, int64_t M, int64_t I, uint8_t* q, float* s,
                                         uint16_t* o2, int scale_layout, int pow2, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && I >= 0, "negative shape");
    PF8_REQUIRE(I % 128 == 0, "I must be a multiple of 128");
    if (M == 0 || I == 0) return PF8_OK;
    PF8_REQUIRE(o1 && q && s, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(o1) && PF8_ALIGNED16(q) && PF8_ALIGNED16(o2), "pointers must be 16-byte aligned");
    PF8_REQUIRE(scale_layout >= 0 && scale_layout <= 2, "scale_layout must be 0, 1 or 2");
    PF8_REQUIRE(scale_layout != 2 || pow2, "UE8M0 scale bytes (scale_layout 2) need power-of-two scales");
    PF8_REQUIRE(I / 128 <= 0x7FFFFF, "shape too large");
    const int IB = (int)(I / 128);
    const int64_t slab = (int64_t)65535 * 4;
    for (int64_t m0 = 0; m0 < M; m0 += slab) {
        const int64_t m = M - m0 < slab ? M - m0 : slab;
        // blocks per wavefront: 8, or 4 when that wastes fewer lane groups on the row's last wavefront
        const int u = ((IB + 7) / 8) * 8 > ((IB + 3) / 4) * 4 ? 1 : 2;
        dim3 grid((unsigned)((IB + 4 * u - 1) / (4 * u)), (unsigned)((m + 3) / 4)), block(256);
        void (*k)(const uint16_t*, const float*, int64_t, int64_t, int, uint8_t*, float*, uint16_t*, int) = nullptr;
#define PF8_PICK(L, P) (u == 2 ? k_swiglu_quant<L, P, 2> : k_swiglu_quant<L, P, 1>)
        if (scale_layout == 0) k = probs ? PF8_PICK(0, true) : PF8_PICK(0, false);
        else if (scale_layout == 1) k = probs ? PF8_PICK(1, true) : PF8_PICK(1, false);
        else k = probs ? PF8_PICK(2, true) : PF8_PICK(2, false);
#undef PF8_PICK
        hipLaunchKernelGGL(k, grid, block, 0, (hipStream_t)stream, o1, probs, M, m0, IB, q, s, o2, pow2);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    return PF8_OK;
}

extern "C" int pf8_swiglu_weighted_bwd(const uint16_t* o1, const uint16_t* do2_s, const float* probs, int64_t M, int64_t I,
                                       uint16_t* do1, float* probs_grad, uint16_t* o2_s, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && I >= 0, "negative shape");
    PF8_REQUIRE(I % 8 == 0, "I must be a multiple of 8");
    if (M == 0) return PF8_OK;
    PF8_REQUIRE(I > 0, "I must be positive");
    PF8_REQUIRE(o1 && do2_s && probs && do1 && probs_grad && o2_s, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(o1) && PF8_ALIGNED16(do2_s) && PF8_ALIGNED16(do1) && PF8_ALIGNED16(o2_s), "pointers must be 16-byte aligned");
    dim3 grid((unsigned)((M + 3) / 4)), block(256);
    hipLaunchKernelGGL(k_swiglu_bwd, grid, block, 0, (hipStream_t)stream, o1, do2_s, probs, M, I, do1, probs_grad, o2_s);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_swiglu_weighted_bwd_quant(const uint16_t* o1, const uint16_t* do2_s, const float* probs, const int64_t* rows_per_expert,
                                             int E, int64_t I, uint8_t* do1_q, float* do1_s, int scale_layout, int pow2_rows, uint8_t* do1_q_t,
                                             float* do1_s_t, uint8_t* o2s_q_t, float* o2s_s_t, int pow2_t, float* probs_grad,
                                             float* pg_partial, pf8_stream_t stream) {
    PF8_REQUIRE(E >= 0 && I >= 0, "negative shape");
    PF8_REQUIRE(I % 128 == 0, "I must be a multiple of 128");
    PF8_REQUIRE(E <= 256, "at most 256 experts per call");
    PF8_REQUIRE(scale_layout == 0 || scale_layout == 1, "scale_layout must be 0 ([M, 2I/128]) or 1 ([2I/128, M])");
    PF8_REQUIRE(pow2_rows != 2 || scale_layout == 1, "UE8M0 row scales (pow2_rows 2) are written [2I/128, M] (scale_layout 1)");
    if (E == 0) return PF8_OK;
    PF8_REQUIRE(rows_per_expert, "null pointer");
    SplitArgs sp = {};
    int64_t total = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE(rows_per_expert[e] >= 0 && rows_per_expert[e] % 128 == 0, "rows_per_expert entries must be non-negative multiples of 128");
        sp.tile_start[e] = (int32_t)(total / 128);
        total += rows_per_expert[e];
    }
    PF8_REQUIRE(total / 128 <= 65535 && (2 * I / 128) * (total / 128) <= 0x7FFFFFF0ll, "too many rows");
    sp.tile_start[E] = (int32_t)(total / 128);
    sp.E = E;
    if (total == 0) return PF8_OK;
    PF8_REQUIRE(I > 0, "I must be positive");
    PF8_REQUIRE(o1 && do2_s && probs && do1_q && do1_s && do1_q_t && do1_s_t && o2s_q_t && o2s_s_t && probs_grad && pg_partial, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(o1) && PF8_ALIGNED16(do2_s) && PF8_ALIGNED16(probs) && PF8_ALIGNED16(do1_q) && PF8_ALIGNED16(do1_q_t) &&
                PF8_ALIGNED16(do1_s_t) && PF8_ALIGNED16(o2s_q_t) && PF8_ALIGNED16(o2s_s_t), "pointers must be 16-byte aligned");
    // pow2 bits of k_quant_rowcol: 1 = transposed copies, 2 = row-scaled copy, 4 = its scales as UE8M0 bytes [2I/128, M]
    const int pow2_bits = (pow2_t ? 1 : 0) | (pow2_rows ? 2 : 0) | (pow2_rows == 2 ? 4 : 0);
    dim3 grid((unsigned)(((I / 128) * (total / 128) + 7) / 8 * 8)), block(256);
    if (scale_layout == 0)
        hipLaunchKernelGGL(k_swiglu_bwd_quant<0>, grid, block, 0, (hipStream_t)stream, o1, do2_s, probs, total, I, do1_q, do1_s, do1_q_t,
                           do1_s_t, o2s_q_t, o2s_s_t, pg_partial, sp, pow2_bits);
    else
        hipLaunchKernelGGL(k_swiglu_bwd_quant<1>, grid, block, 0, (hipStream_t)stream, o1, do2_s, probs, total, I, do1_q, do1_s, do1_q_t,
                           do1_s_t, o2s_q_t, o2s_s_t, pg_partial, sp, pow2_bits);
    int rc = pf8_check_launch(__func__);
    if (rc) return rc;
    hipLaunchKernelGGL(k_sum_row_partials, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, pg_partial,
                       (int)(I / 128), total, probs_grad);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_act_dequant(const uint8_t* q, const float* s, int scale_layout, int64_t M, int64_t K, uint16_t* out,
                               pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && K >= 0, "negative shape");
    PF8_REQUIRE(K % 128 == 0, "K must be a multiple of 128");
    if (M == 0 || K == 0) return PF8_OK;
    PF8_REQUIRE(q && s && out, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(q) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    PF8_REQUIRE(scale_layout == 0 || scale_layout == 1, "scale_layout must be 0 or 1");
    const int64_t chunks = M * (K / 8);
    dim3 grid((unsigned)((chunks + 255) / 256)), block(256);
    if (chunks < 0x7FFFFF00ll) {
        if (scale_layout == 0) hipLaunchKernelGGL((k_act_dequant<0, uint32_t>), grid, block, 0, (hipStream_t)stream, q, s, M, K, out);
        else hipLaunchKernelGGL((k_act_dequant<1, uint32_t>), grid, block, 0, (hipStream_t)stream, q, s, M, K, out);
    } else {
        if (scale_layout == 0) hipLaunchKernelGGL((k_act_dequant<0, int64_t>), grid, block, 0, (hipStream_t)stream, q, s, M, K, out);
        else hipLaunchKernelGGL((k_act_dequant<1, int64_t>), grid, block, 0, (hipStream_t)stream, q, s, M, K, out);
    }
    return pf8_check_launch(__func__);
}

extern "C" int pf8_block_dequant(const uint8_t* q, const void* scale, int scale_format, int64_t B, int64_t R, int64_t C,
                                 int64_t block_r, int64_t block_c, void* out, int out_f32, pf8_stream_t stream) {
    PF8_REQUIRE(B >= 0 && R >= 0 && C >= 0, "negative shape");
    PF8_REQUIRE(block_r > 0 && block_c > 0, "block sizes must be positive");
    PF8_REQUIRE(scale_format >= 0 && scale_format <= 3, "scale_format must be 0 (fp32), 1 (ue8m0), 2 (bf16) or 3 (fp16)");
    if (B == 0 || R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(q && scale && out, "null pointer");
    PF8_REQUIRE(B * R < (1LL << 40) && C < (1LL << 40), "tensor too large");
    const int64_t threads = B * R * ((C + 15) / 16);
    PF8_REQUIRE((threads + 255) / 256 <= 0x7FFFFFFF, "tensor too large for one launch");
    dim3 grid((unsigned)((threads + 255) / 256)), block(256);
    const bool small = threads + 256 < (1LL << 31) && C + 16 < (1LL << 31) && block_r < (1LL << 31) && block_c < (1LL << 31);
    hipStream_t st = (hipStream_t)stream;
    if (out_f32 && small) hipLaunchKernelGGL((k_block_dequant<1, uint32_t>), grid, block, 0, st, q, scale, scale_format, B, R, C, block_r, block_c, out);
    else if (out_f32) hipLaunchKernelGGL((k_block_dequant<1, int64_t>), grid, block, 0, st, q, scale, scale_format, B, R, C, block_r, block_c, out);
    else if (small) hipLaunchKernelGGL((k_block_dequant<0, uint32_t>), grid, block, 0, st, q, scale, scale_format, B, R, C, block_r, block_c, out);
    else hipLaunchKernelGGL((k_block_dequant<0, int64_t>), grid, block, 0, st, q, scale, scale_format, B, R, C, block_r, block_c, out);
    return pf8_check_launch(__func__);
}

// 128x128-block dequant to bf16: the block dequantizer with fp32 scales and one 128x128 geometry
extern "C" int pf8_weight_dequant(const uint8_t* q, const float* s, int64_t R, int64_t C, uint16_t* out, pf8_stream_t stream) {
    PF8_REQUIRE(R >= 0 && C >= 0, "negative shape");
    if (R == 0 || C == 0) return PF8_OK;
    PF8_REQUIRE(q && s && out, "null pointer");
    return pf8_block_dequant(q, s, SCALE_F32, 1, R, C, 128, 128, out, 0, stream);
}

extern "C" int pf8_debug_copy(const void* src, void* dst, int64_t nbytes, pf8_stream_t stream) {
    PF8_REQUIRE(nbytes >= 0 && nbytes % 16 == 0, "nbytes must be a non-negative multiple of 16");
    if (nbytes == 0) return PF8_OK;
    PF8_REQUIRE(src && dst && PF8_ALIGNED16(src) && PF8_ALIGNED16(dst), "null or misaligned pointer");
    const int64_t n16 = nbytes / 16;
    PF8_REQUIRE((n16 + 255) / 256 <= 0x7FFFFFFF, "too large");
    hipLaunchKernelGGL(k_debug_copy, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)src, (uint4*)dst, n16);
    return pf8_check_launch(__func__);
}
extern "C" int pf8_debug_encode(const float* v, int64_t n, uint8_t* out, pf8_stream_t stream) {
    if (n <= 0) return PF8_OK;
    PF8_REQUIRE(v && out, "null pointer");
    hipLaunchKernelGGL(k_debug_encode, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, v, n, out);
    return pf8_check_launch(__func__);
}
extern "C" int pf8_debug_div_encode(const float* x, const float* s, int64_t n, uint8_t* out, pf8_stream_t stream) {
    if (n <= 0) return PF8_OK;
    PF8_REQUIRE(x && s && out, "null pointer");
    hipLaunchKernelGGL(k_debug_div_encode, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, s, n, out);
    return pf8_check_launch(__func__);
}
extern "C" int pf8_debug_silu(const float* x, int64_t n, float* out, pf8_stream_t stream) {
    if (n <= 0) return PF8_OK;
    PF8_REQUIRE(x && out, "null pointer");
    hipLaunchKernelGGL(k_debug_silu, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, n, out, (float*)nullptr);
    return pf8_check_launch(__func__);
}
extern "C" int pf8_debug_silu_sigmoid(const float* x, int64_t n, float* out_silu, float* out_sigmoid, pf8_stream_t stream) {
    if (n <= 0) return PF8_OK;
    PF8_REQUIRE(x && out_silu && out_sigmoid, "null pointer");
    hipLaunchKernelGGL(k_debug_silu, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, n, out_silu, out_sigmoid);
    return pf8_check_launch(__func__);
}
