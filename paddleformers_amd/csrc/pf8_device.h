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
// The streaming kernels touch every byte once: loads and stores carry the non-temporal hint, which keeps them from
// displacing each other in the caches (a plain copy of 89 MB: 16.0 us with the hint on both sides, 17.8 us without;
// 477 MB: 77.5 against 80.6 us).
__device__ __forceinline__ uint4 ld16(const void* p) {
    u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ld8(const void* p) {
    u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ void st16(void* p, uint4 o) {
    u32x4 v = {o.x, o.y, o.z, o.w};
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ void st8(void* p, uint2 o) {
    u32x2 v = {o.x, o.y};
    __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
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
    float y;      // its correctly rounded reciprocal (IEEE 1/s); exact when s is a power of two
    bool slow;    // scale too small for a finite, normal reciprocal: the tile takes the IEEE division
    bool exact;   // s is a power of two: v * y IS the correctly rounded v / s
};

// Scales below this have no usable reciprocal (1/s overflows or s is subnormal): such tiles divide.
constexpr float kMinFastScale = 1.0e-30f;

// 1/s of a power of two s = 2^k, k in [-126, 126] (what the pow2 rule below yields), by exponent arithmetic
__device__ __forceinline__ float pow2_recip(float s) { return u2f(0x7F000000u - f2u(s)); }

__device__ __forceinline__ TileScale make_scale_from(float s) {
    TileScale t;
    t.s = s;
    t.slow = !(s >= kMinFastScale);
    t.y = 1.0f / (t.slow ? 1.0f : s);
    t.exact = false;
    return t;
}
// s = amax/448 (IEEE divide), amax == 0 -> 1; pow2: decode scale rounded up to a power of two.
// For a bf16-valued amax m 2^E with a normal quotient the rounded-up power of two needs no division: 448 = 1.75 2^8, so
// it is 2^(E-8) when m <= 1.75 and 2^(E-7) above (the next bf16 mantissa after 1.75 is 2^-7 away, far from where the fp32
// rounding of the quotient could reach a power of two), i.e. the exponent field of amax + 0x1FFFFF less 8.  Any other
// amax (not a bf16 value, or so small that the quotient is subnormal) takes the division.
__device__ __forceinline__ float scale_of(uint32_t amax_bits, bool pow2) {
    if (pow2 && __builtin_expect(amax_bits >= 0x04800000u && (amax_bits & 0xFFFFu) == 0u, 1))
        return u2f(((amax_bits + 0x001FFFFFu) & 0x7F800000u) - 0x04000000u);
    float s = u2f(amax_bits) / 448.0f;
    if (pow2) s = u2f((f2u(s) + 0x007FFFFFu) & 0x7F800000u);
    return amax_bits == 0u ? 1.0f : s;
}
__device__ __forceinline__ TileScale make_scale(uint32_t amax_bits, bool pow2) {
    const float s = scale_of(amax_bits, pow2);
    if (pow2) {
        // dividing by a power of two is multiplying by its (exact) reciprocal: the product is the
        // correctly rounded quotient, one multiply and one conversion per element
        TileScale t;
        t.s = s;
        t.y = pow2_recip(s);
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
// quotient, without dividing per element.  With y = RN(1/s) (one IEEE division per tile):
//     q0 = v * y;   r = fma(-q0, s, v);   q = fma(r, y, q0)
// q0 is within an ulp or two of the quotient, the residual r = v - q0 s is exact in fp32, and the
// corrected q rounds to the same e4m3 code as the IEEE quotient.  That is not taken on faith: the
// inputs of every quantizer here are bf16 values and s = amax/448 of a bf16 amax, a finite set, and
// the CPU test suite walks ALL (amax, v) pairs of it (522 million, |v| <= amax, s >= kMinFastScale),
// comparing the codes of this sequence with those of the division; it also holds on 2.5e9 random
// pairs of an arbitrary fp32 scale and a bf16 value.  (The fp32 quotients themselves differ only
// where the residual underflows, quotients below 2^-27, which encode as zero either way.)
// One input needs care: v = -0 gives q0 = -0, r = +0 and q = (+0) + (-0) = +0, while -0 / s is -0 (code
// 0x80).  The quotient always carries the sign of v (s > 0), so the sign is copied over (one v_bfi_b32).
__device__ __forceinline__ float div_by_recip(float v, float s, float y) {
    const float q0 = v * y;
    const float r = __builtin_fmaf(-q0, s, v);
    return __builtin_copysignf(__builtin_fmaf(r, y, q0), v);
}
__device__ __forceinline__ uint2 quant8_exact(const float (&v)[8], float y) {
    uint2 o;
    o.x = pack4_e4m3(v[0] * y, v[1] * y, v[2] * y, v[3] * y);
    o.y = pack4_e4m3(v[4] * y, v[5] * y, v[6] * y, v[7] * y);
    return o;
}
__device__ __forceinline__ uint2 quant8_divide(const float (&v)[8], float s) {
    uint2 o;
    o.x = pack4_e4m3(v[0] / s, v[1] / s, v[2] / s, v[3] / s);
    o.y = pack4_e4m3(v[4] / s, v[5] / s, v[6] / s, v[7] / s);
    return o;
}
// 8 values against a scale and its reciprocal; `slow` tiles (tiny scales) divide
__device__ __forceinline__ uint2 quant8_r(const float (&v)[8], float s, float y, bool slow) {
    if (__builtin_expect(slow, 0)) return quant8_divide(v, s);
    uint2 o;
    o.x = pack4_e4m3(div_by_recip(v[0], s, y), div_by_recip(v[1], s, y), div_by_recip(v[2], s, y), div_by_recip(v[3], s, y));
    o.y = pack4_e4m3(div_by_recip(v[4], s, y), div_by_recip(v[5], s, y), div_by_recip(v[6], s, y), div_by_recip(v[7], s, y));
    return o;
}
__device__ __forceinline__ uint2 quant8(const float (&v)[8], const TileScale& t) {
    if (t.exact) return quant8_exact(v, t.y);
    return quant8_r(v, t.s, t.y, t.slow);
}

// value of lane Q of every quad, for all four lanes of the quad (folds into the consuming VALU op)
template <int Q>
__device__ __forceinline__ float quad_bcast(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), Q * 0x55, 0xF, 0xF, false));
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

// expf restated operation for operation from the CPU checker: t = x log2(e) clamped to [-125, 126], n = t rounded by adding
// and subtracting 1.5 * 2^23, 2^(t - n) by a degree-4 Horner polynomial with fused multiply-adds, n added to the exponent
// field straight from the low bits of the rounded sum.  Ten instructions; relative error below 2^-17.
// The polynomial's coefficients as values the compiler has to keep in registers: handed to expf_fixed / silu_exact by a
// kernel that evaluates many of them, they turn the Horner steps into three-operand multiply-adds with no constant to
// re-materialise in between.
struct ExpPoly { float c4, c3, c2, c1; };
__device__ __forceinline__ ExpPoly exp_poly() {
    return ExpPoly{9.584701620042324e-3f, 5.590607970952988e-2f, 2.4024060368537903e-1f, 6.931242942810059e-1f};
}
__device__ __forceinline__ ExpPoly exp_poly_in_registers() {
    ExpPoly k = exp_poly();
    asm volatile("" : "+v"(k.c4), "+v"(k.c3), "+v"(k.c2), "+v"(k.c1));
    return k;
}
__device__ __forceinline__ float expf_fixed(float x, const ExpPoly& k) {
    // the clamp as one median-of-three (a NaN comes out as the lower bound, as fminf(fmaxf()) leaves it)
    const float t = __builtin_amdgcn_fmed3f(x * 1.44269504088896341f, -125.0f, 126.0f);
    const float s = t + 12582912.0f;
    const float n = s - 12582912.0f;
    const float f = t - n;
    float p = __builtin_fmaf(k.c4, f, k.c3);
    p = __builtin_fmaf(p, f, k.c2);
    p = __builtin_fmaf(p, f, k.c1);
    p = __builtin_fmaf(p, f, 1.0f);
    return u2f(f2u(p) + (f2u(s) << 23));
}
__device__ __forceinline__ float expf_fixed(float x) { return expf_fixed(x, exp_poly()); }

// silu(g) = g / (1 + exp(-g)) with the correctly rounded quotient, without the IEEE division sequence: y = v_rcp_f32 of
// the denominator (within one unit in the last place), q0 = g y, r = fma(-q0, den, g), q = fma(r, y, q0), and the sign of g
// copied over (g = -0).  The denominator lies in [1, 2^126], so the reciprocal is a normal number.  g is always a bf16
// value in this library and the denominator a function of g: the GPU test suite compares this routine with the CPU
// checker's division on every one of the 65,536 bf16 inputs, bit for bit.
__device__ __forceinline__ float silu_exact(float g, const ExpPoly& k) {
    const float den = 1.0f + expf_fixed(-g, k);
    const float y = __builtin_amdgcn_rcpf(den);
    const float q0 = g * y;
    const float r = __builtin_fmaf(-q0, den, g);
    return __builtin_copysignf(__builtin_fmaf(r, y, q0), g);
}
__device__ __forceinline__ float silu_exact(float g) { return silu_exact(g, exp_poly()); }

// The two quotients of the SwiGLU backward from one hardware reciprocal: g / den (silu_exact's sequence) and 1 / den
// (y = v_rcp_f32(den), r = fma(-y, den, 1), y + r y), den = 1 + exp(-g).  Both are the correctly rounded quotients for
// every bf16 g: the GPU test suite compares them with the CPU checker's divisions on all 65,536 inputs.
struct SiluSigmoid { float silu, sigmoid; };
__device__ __forceinline__ SiluSigmoid silu_and_sigmoid(float g, const ExpPoly& k) {
    const float den = 1.0f + expf_fixed(-g, k);
    const float y = __builtin_amdgcn_rcpf(den);
    const float q0 = g * y;
    SiluSigmoid o;
    o.silu = __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-q0, den, g), y, q0), g);
    o.sigmoid = __builtin_fmaf(__builtin_fmaf(-y, den, 1.0f), y, y);
    return o;
}

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
