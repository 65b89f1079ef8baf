// pf8_device.h -- device-side scalar helpers shared by the gfx950 kernels: bf16 unpack/round,
// OCP e4m3 packing through the hardware converter, the 16-lane (one DPP row = one 1x128 tile)
// amax reduction, the scale rule and the tile quantizer with its fast exact-division path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pf8 {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// a dword holds two bf16: element 0 in the low half
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }

// two fp32 -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// one fp32 -> bf16 -> fp32 (the value a bf16 tensor would hold)
__device__ __forceinline__ float round_bf16(float f) { return bf16_lo(pack_bf16(f, 0.0f)); }

// unsigned max with the other operand fetched from a lane `ror` positions away inside the 16-lane
// DPP row; magnitudes of non-NaN floats order like their bit patterns, so amax runs on integers
// (no NaN-canonicalisation instructions in the way).
template <int ROR>
__device__ __forceinline__ uint32_t row_max_step(uint32_t v) {
    uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x120 + ROR, 0xF, 0xF, false);
    return v > o ? v : o;
}
// all 16 lanes of a DPP row end with the row maximum
__device__ __forceinline__ uint32_t row16_max(uint32_t v) {
    v = row_max_step<8>(v);
    v = row_max_step<4>(v);
    v = row_max_step<2>(v);
    v = row_max_step<1>(v);
    return v;
}

// 16-byte / 8-byte global accesses
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 ld16(const void* p) {
    u32x4 v = *reinterpret_cast<const u32x4*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void* p, uint4 o) {
    u32x4 v = {o.x, o.y, o.z, o.w};
    *reinterpret_cast<u32x4*>(p) = v;
}
__device__ __forceinline__ void st8(void* p, uint2 o) {
    u32x2 v = {o.x, o.y};
    *reinterpret_cast<u32x2*>(p) = v;
}

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
// element-wise max of the two 16-bit halves (v_pk_max_u16)
__device__ __forceinline__ uint32_t pkmax_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}

// |.| bit patterns of the 8 bf16 in a 16-byte chunk, reduced to one fp32-positioned pattern
__device__ __forceinline__ uint32_t amax_bits8(uint4 w) {
    uint32_t m = pkmax_u16(pkmax_u16(w.x & 0x7FFF7FFFu, w.y & 0x7FFF7FFFu),
                           pkmax_u16(w.z & 0x7FFF7FFFu, w.w & 0x7FFF7FFFu));
    return umax(m << 16, m & 0xFFFF0000u);
}

struct TileScale {
    float s;      // decode scale stored next to the bytes
    float r_lo;   // reciprocal of s nudged down by 2^-20 (relative)
    float r_hi;   // reciprocal of s nudged up by 2^-20
    bool slow;    // tile must take the IEEE division path (scale too small for a finite reciprocal)
    bool exact;   // s is a power of two: r_lo == r_hi == 1/s exactly, and v * r_lo IS the correctly rounded v / s
};

// s = amax/448 (IEEE divide), amax == 0 -> 1; pow2: decode scale rounded up to a power of two.
__device__ __forceinline__ TileScale make_scale_from(float s) {
    TileScale t;
    t.s = s;
    const float r = __builtin_amdgcn_rcpf(s);
    t.r_lo = r * 0.99999904632568359375f;   // 1 - 2^-20
    t.r_hi = r * 1.00000095367431640625f;   // 1 + 2^-20
    t.slow = !(s >= 1.0e-30f);
    t.exact = false;
    return t;
}
// 1/s of a power of two s = 2^k, k in [-126, 126] (what the pow2 rule below yields), by exponent arithmetic
__device__ __forceinline__ float pow2_recip(float s) { return u2f(0x7F000000u - f2u(s)); }
__device__ __forceinline__ TileScale make_scale(uint32_t amax_bits, bool pow2) {
    float amax = u2f(amax_bits);
    float s = amax / 448.0f;
    if (pow2) s = u2f((f2u(s) + 0x007FFFFFu) & 0x7F800000u);
    if (amax_bits == 0u) s = 1.0f;
    if (pow2) {
        // dividing by a power of two is multiplying by its (exact) reciprocal: the product is the
        // correctly rounded quotient, so one conversion per element and no bracket to check.  (With
        // the bracket every exact e4m3 tie, one bf16 value in 32, would take the division path.)
        TileScale t;
        t.s = s;
        t.r_lo = t.r_hi = pow2_recip(s);
        t.slow = false;
        t.exact = true;
        return t;
    }
    return make_scale_from(s);
}

// two fp32 -> two e4m3 codes in the low / high half of a dword (hardware OCP convert, RNE)
__device__ __forceinline__ uint32_t cvt_e4m3_lo(float a, float b, uint32_t old) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}
__device__ __forceinline__ uint32_t cvt_e4m3_hi(float a, float b, uint32_t old) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true);
}
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    return cvt_e4m3_hi(c, d, cvt_e4m3_lo(a, b, 0u));
}

// Quantise 8 values of one tile: bytes == e4m3_rne(v / s) with v / s the correctly rounded fp32
// quotient.  Fast path: the quotient is bracketed by v*r_lo and v*r_hi (the reciprocal is good to
// 1 ulp, the nudges are 2^-20, so the bracket holds with a wide margin); rounding is monotone, so
// where both ends convert to the same e4m3 code that is the code of the exact quotient.  Where they
// differ a rounding boundary lies inside the 2^-19-wide bracket and that ELEMENT is redone with the
// IEEE division.  This is not rare: s = amax/448 carries an fp32 rounding error, so every element
// for which 448 v / amax is an exact e4m3 tie in real arithmetic (bf16 inputs make these common,
// about one element in a thousand) sits 2^-24 from a boundary.  Most wavefronts therefore visit
// the fallback for one or two elements, and it is written to cost one division, not eight.
__device__ __forceinline__ uint32_t nonzero_bytes(uint32_t d) {   // 0x80 in every byte of d that is not zero
    return (((d & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | d) & 0x80808080u;
}
__device__ __forceinline__ void quant8_fix(const float (&v)[8], float s, uint2& lo, const uint2 hi) {
    const uint32_t dx = lo.x ^ hi.x, dy = lo.y ^ hi.y;
    if (__builtin_expect((dx | dy) != 0u, 0)) {
        const uint32_t zx = nonzero_bytes(dx), zy = nonzero_bytes(dy);
        if (__builtin_popcount(zx) + __builtin_popcount(zy) == 1) {
            // the usual case, one element: pick it without branching on its index
            const int idx = zx ? (__builtin_ctz(zx) >> 3) : 4 + (__builtin_ctz(zy) >> 3);
            const float a = (idx & 1) ? v[1] : v[0], b = (idx & 1) ? v[3] : v[2];
            const float c = (idx & 1) ? v[5] : v[4], d = (idx & 1) ? v[7] : v[6];
            const float e = (idx & 2) ? b : a, f = (idx & 2) ? d : c;
            const float qv = ((idx & 4) ? f : e) / s;
            const uint32_t code = cvt_e4m3_lo(qv, qv, 0u) & 0xFFu;
            const int sh = 8 * (idx & 3);
            const uint32_t keep = ~(0xFFu << sh), put = code << sh;
            if (idx & 4) lo.y = (lo.y & keep) | put;
            else lo.x = (lo.x & keep) | put;
        } else {
            // a tile whose amax makes exact ties common (e.g. amax = 448 * 2^k: one value in eight)
            lo.x = pack4_e4m3(v[0] / s, v[1] / s, v[2] / s, v[3] / s);
            lo.y = pack4_e4m3(v[4] / s, v[5] / s, v[6] / s, v[7] / s);
        }
    }
}
__device__ __forceinline__ uint2 quant8_exact(const float (&v)[8], float r) {
    uint2 o;
    o.x = pack4_e4m3(v[0] * r, v[1] * r, v[2] * r, v[3] * r);
    o.y = pack4_e4m3(v[4] * r, v[5] * r, v[6] * r, v[7] * r);
    return o;
}
__device__ __forceinline__ uint2 quant8(const float (&v)[8], const TileScale& t) {
    if (t.exact) return quant8_exact(v, t.r_lo);
    uint2 lo, hi;
    const float r_lo = t.slow ? 0.0f : t.r_lo, r_hi = t.slow ? __builtin_inff() : t.r_hi;   // slow: every element differs
    lo.x = pack4_e4m3(v[0] * r_lo, v[1] * r_lo, v[2] * r_lo, v[3] * r_lo);
    lo.y = pack4_e4m3(v[4] * r_lo, v[5] * r_lo, v[6] * r_lo, v[7] * r_lo);
    hi.x = pack4_e4m3(v[0] * r_hi, v[1] * r_hi, v[2] * r_hi, v[3] * r_hi);
    hi.y = pack4_e4m3(v[4] * r_hi, v[5] * r_hi, v[6] * r_hi, v[7] * r_hi);
    quant8_fix(v, t.s, lo, hi);
    return lo;
}

// ---- quantizers that hold several tiles per lane: scales for up to four tiles in one pass ----
// value of lane Q of every quad, for all four lanes of the quad (folds into the consuming VALU op)
template <int Q>
__device__ __forceinline__ float quad_bcast(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), Q * 0x55, 0xF, 0xF, false));
}
// Reciprocal pair of a scale; a scale too small for a finite reciprocal gets (0, inf), which makes
// the two conversions of any element disagree and sends the tile down the division path.
__device__ __forceinline__ void scale_recips(float s, float& r_lo, float& r_hi) {
    const float r = __builtin_amdgcn_rcpf(s);
    const bool ok = s >= 1.0e-30f;
    r_lo = ok ? r * 0.99999904632568359375f : 0.0f;          // 1 - 2^-20
    r_hi = ok ? r * 1.00000095367431640625f : __builtin_inff();   // 1 + 2^-20
}
__device__ __forceinline__ float scale_of(uint32_t amax_bits, bool pow2) {
    float s = u2f(amax_bits) / 448.0f;
    if (pow2) s = u2f((f2u(s) + 0x007FFFFFu) & 0x7F800000u);
    return amax_bits == 0u ? 1.0f : s;
}
// 8 values against a reciprocal pair; elements whose two conversions differ are redone by division
__device__ __forceinline__ uint2 quant8_r(const float (&v)[8], float r_lo, float r_hi, float s) {
    uint2 lo, hi;
    lo.x = pack4_e4m3(v[0] * r_lo, v[1] * r_lo, v[2] * r_lo, v[3] * r_lo);
    lo.y = pack4_e4m3(v[4] * r_lo, v[5] * r_lo, v[6] * r_lo, v[7] * r_lo);
    hi.x = pack4_e4m3(v[0] * r_hi, v[1] * r_hi, v[2] * r_hi, v[3] * r_hi);
    hi.y = pack4_e4m3(v[4] * r_hi, v[5] * r_hi, v[6] * r_hi, v[7] * r_hi);
    quant8_fix(v, s, lo, hi);
    return lo;
}

__device__ __forceinline__ void unpack8(uint4 w, float (&v)[8]) {
    v[0] = bf16_lo(w.x); v[1] = bf16_hi(w.x);
    v[2] = bf16_lo(w.y); v[3] = bf16_hi(w.y);
    v[4] = bf16_lo(w.z); v[5] = bf16_hi(w.z);
    v[6] = bf16_lo(w.w); v[7] = bf16_hi(w.w);
}

// four e4m3 codes of one word -> fp32 with the hardware convert (exact, two bytes per instruction)
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float* f) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    f[0] = lo[0]; f[1] = lo[1]; f[2] = hi[0]; f[3] = hi[1];
}

// expf restated operation for operation from the CPU checker: clamp, Cody-Waite reduction with two
// fused steps, degree-5 Horner polynomial with fused multiply-adds, exact power-of-two scaling.
__device__ __forceinline__ float expf_fixed(float x) {
    x = __builtin_fminf(__builtin_fmaxf(x, -87.0f), 88.5f);
    float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    float y = __builtin_fmaf(p, r2, r);
    y = y + 1.0f;
    return __builtin_ldexpf(y, (int)n);
}

// silu(g) = g / (1 + exp(-g)), IEEE division
__device__ __forceinline__ float silu_exact(float g) { return g / (1.0f + expf_fixed(-g)); }

// Contiguous-grouped GEMM with UE8M0 scales: which of the two kernels takes an expert load, from the
// work-item list's header {paired 256-row items, 128-row blocks}.  Rounds of tiles per compute unit,
// a 256x256 block costing 1.6 times a 128x256 one (measured): few blocks per expert leave many
// paired tiles half empty, and then the smaller tile wins.  Both kernels evaluate this on entry and
// the one that loses returns (a host-side choice would need the row counts).
__device__ __forceinline__ bool e8_paired_tiles_win(const int32_t* list_header, int64_t p_tiles, int64_t cus) {
    const int64_t n = list_header[0], nb = list_header[1];
    const int64_t rounds_pair = (n * p_tiles + cus - 1) / cus, rounds_128 = (nb * p_tiles + cus - 1) / cus;
    return 16 * rounds_pair <= 10 * rounds_128;
}

}  // namespace pf8
