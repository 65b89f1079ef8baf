/*
 * pf8_oracle.c -- CPU restatement of the PaddleFormers FP8 block-quant / block-scaled GEMM path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing shipped may link, import or call this file: it is the checker
 * the HIP kernels are compared against (tests/, the smoke check and the CPU leg of the benchmark).
 *
 * Every function cites the reference lines (paths relative to the PaddleFormers checkout) whose
 * arithmetic it restates.  The reference has no native code and its kernels live in third-party
 * CUDA binaries (paddlepaddle-gpu nightly, paddlefleet==0.4.0.post20260909+08dd2e727b0 / DeepGEMM),
 * so the restatement follows the in-repo Triton formulation and the un-fused fallback chains.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   e4m3 decode        reference KATs 0x00,0x01,0x38,0x7E,0xFE,0x7F; closed form; torch cast
 *   e4m3 encode        brute-force nearest-even search over the decode table; torch cast
 *   bf16 round         torch cast over a bit-pattern sweep
 *   quant 1x128/128x128  float64 brute force on small inputs; 448-byte invariant; pow2 scaling
 *                      invariance; transpose identity quant(W^T) == quant(W)^T
 *   quant_transpose    equals two separate quantizations (by construction here; checked vs numpy)
 *   stack/split        equals stack -> transpose -> quant chains written in numpy
 *   expf / silu        float64 libm to <= 1 ulp(fp32) / <= 1 ulp(bf16)
 *   swiglu bwd         float64 finite differences
 *   gemm               exact integer matmul special case; float64 dequant-matmul
 * Parity UNPINNED against the real third-party kernels (no golden vectors exist in the reference):
 *   fp8_quant_blockwise op order (divide vs reciprocal-multiply) and amax==0 behaviour,
 *   fused_weighted_swiglu_act_quant internal precision, fused_transpose_split_quant fp8-input
 *   rounding, DeepGEMM accumulation order.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off; explicit fmaf where a fused op is meant)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define PF8O_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------ */
/* scalar codecs                                                                              */
/* ------------------------------------------------------------------------------------------ */

/* OCP float8_e4m3fn decode.  quantization/checkpoint_dequant.py:80-90 (_build_e4m3_lut):
 * exponent==0 -> m*2^-9, else (1+m/8)*2^(e-7); S.1111.111 is NaN; no infinities. */
PF8O_API float pf8o_e4m3_decode(uint8_t c) {
    int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if (e == 0xF && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

/* fp32 -> e4m3fn, round-to-nearest-even on the value grid, sign kept (so -tiny -> 0x80).
 * This is the cast `y.to(float8_e4m3fn)` of cli/train/deepseek_v3_pretrain/kernel.py:46-47.
 * Finite |v| above 448 saturates to 448 (the Triton cast on NVIDIA is cvt.rn.satfinite); a
 * well-formed tile never gets there because |x/s| <= 448*(1+2^-23).  NaN -> 0x7F. */
PF8O_API uint8_t pf8o_e4m3_encode(float v) {
    uint32_t bits; memcpy(&bits, &v, 4);
    uint8_t sign = (uint8_t)((bits >> 24) & 0x80);
    float a = fabsf(v);
    if (isnan(v)) return (uint8_t)(sign | 0x7F);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7E);
    if (a < 0.015625f) {                  /* below 2^-6: subnormal grid, spacing 2^-9 */
        /* a * 512 is exact (power-of-two scaling), rintf is RNE in the default mode */
        int m = (int)rintf(a * 512.0f);   /* 0..8 ; 8 means 2^-6 = 0x08 */
        return (uint8_t)(sign | (uint8_t)m);
    }
    /* normal: 2^e * (1 + m/8).  Work on the fp32 bit pattern: keep 3 mantissa bits, RNE. */
    uint32_t ab = bits & 0x7FFFFFFFu;
    uint32_t lsb = (ab >> 20) & 1u;
    ab += 0x7FFFFu + lsb;                 /* round half to even at bit 20 */
    int e = (int)(ab >> 23) - 127;        /* may have carried into the exponent */
    int m = (int)((ab >> 20) & 7u);
    if (e > 8 || (e == 8 && m == 7)) return (uint8_t)(sign | 0x7E);   /* cannot happen below 448 */
    return (uint8_t)(sign | (uint8_t)(((e + 7) << 3) | m));
}

PF8O_API float pf8o_bf16_to_f32(uint16_t h) {
    uint32_t b = (uint32_t)h << 16; float f; memcpy(&f, &b, 4); return f;
}

/* fp32 -> bf16 round-to-nearest-even; this is the `.cast(paddle.bfloat16)` of the un-fused chains
 * (ernie token_dispatcher/fp8_utils.py:998).  NaN stays NaN (quiet bit forced). */
PF8O_API uint16_t pf8o_f32_to_bf16(float f) {
    uint32_t b; memcpy(&b, &f, 4);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

/* expf with a fixed, portable operation sequence that the device code restates bit for bit, chosen short (the fused
 * SwiGLU quantizer is bound by its arithmetic): t = x * log2(e) clamped to [-125, 126]; n = round-to-nearest-even of t by
 * adding and subtracting 1.5 * 2^23; f = t - n (exact, |f| <= 0.5); 2^f by a degree-4 polynomial (minimax for the relative
 * error, 2^-18.4, constant term 1) in Horner form with fused multiply-adds; the scaling by 2^n adds n to the exponent
 * field, n taken from the low bits of the rounded sum.  Relative error below 2^-17 over the clamp range (the product
 * x * log2(e) is rounded once); outside it the value is the clamp's.
 * The reference only says `F.silu(x) * y` (transformers/fp8_utils.py:26-29); which expf Paddle's CUDA swiglu uses is not
 * visible, so this definition is the build's own (parity unpinned); its results are rounded to bf16 (relative 2^-8). */
PF8O_API float pf8o_expf(float x) {
    float t = x * 1.44269504088896341f;
    t = fminf(fmaxf(t, -125.0f), 126.0f);
    float s = t + 12582912.0f;
    float n = s - 12582912.0f;
    float f = t - n;
    float p = 9.584701620042324e-3f;
    p = fmaf(p, f, 5.590607970952988e-2f);
    p = fmaf(p, f, 2.4024060368537903e-1f);
    p = fmaf(p, f, 6.931242942810059e-1f);
    p = fmaf(p, f, 1.0f);
    uint32_t pb, sb;
    memcpy(&pb, &p, 4);
    memcpy(&sb, &s, 4);
    pb += sb << 23;
    memcpy(&p, &pb, 4);
    return p;
}

/* silu(g) = g / (1 + exp(-g)) in fp32.  transformers/fp8_utils.py:26-29, nn/mlp.py:21-23. */
PF8O_API float pf8o_silu(float g) { return g / (1.0f + pf8o_expf(-g)); }

/* ------------------------------------------------------------------------------------------ */
/* scale rule                                                                                 */
/* ------------------------------------------------------------------------------------------ */

/* s = amax / 448 (kernel.py:44).  amax == 0 is defined as s = 1 (the literal formula gives 0/0).
 * pow2: round the decode scale UP to a power of two with the bit trick of
 * utils/upcast_downcast_triton.py:71-85. */
static float scale_from_amax(float amax, int pow2) {
    if (amax == 0.0f) return 1.0f;
    float s = amax / 448.0f;
    if (pow2) {
        uint32_t b; memcpy(&b, &s, 4);
        b = (b + 0x007FFFFFu) & 0x7F800000u;
        memcpy(&s, &b, 4);
    }
    return s;
}
PF8O_API float pf8o_scale_from_amax(float amax, int pow2) { return scale_from_amax(amax, pow2); }

/* ------------------------------------------------------------------------------------------ */
/* quantizers                                                                                 */
/* ------------------------------------------------------------------------------------------ */

/* 1x128 quantization.  kernel.py:41-48 (act_quant_kernel): per tile s = max|x|/448, y = x/s,
 * cast to e4m3.  scale_layout 0: s[M, K/128] row-major (output_scale_transpose=False);
 * 1: s[K/128, M] (output_scale_transpose=True, transformers/fp8_utils.py:262-268). */
PF8O_API void pf8o_quant_1x128(const uint16_t* x, int64_t M, int64_t K, int64_t ldx, uint8_t* q,
                               float* s, int scale_layout, int pow2) {
    int64_t KB = K / 128;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r) {
        for (int64_t b = 0; b < KB; ++b) {
            const uint16_t* xp = x + r * ldx + b * 128;
            float amax = 0.0f;
            for (int j = 0; j < 128; ++j) amax = fmaxf(amax, fabsf(pf8o_bf16_to_f32(xp[j])));
            float sc = scale_from_amax(amax, pow2);
            for (int j = 0; j < 128; ++j)
                q[r * K + b * 128 + j] = pf8o_e4m3_encode(pf8o_bf16_to_f32(xp[j]) / sc);
            if (scale_layout == 0) s[r * KB + b] = sc; else s[b * M + r] = sc;
        }
    }
}

/* 128x128 quantization of a weight.  transformers/fp8_utils.py:105-131 (weight_quant): same
 * amax/448 rule over a 2-D tile; the transposed outputs are the exact transposes (:110, :123).
 * Any of (q,s) / (qt,st) may be NULL. */
PF8O_API void pf8o_quant_128x128(const uint16_t* w, int64_t R, int64_t C, uint8_t* q, float* s,
                                 uint8_t* qt, float* st, int pow2) {
    int64_t RB = R / 128, CB = C / 128;
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t rb = 0; rb < RB; ++rb) {
        for (int64_t cb = 0; cb < CB; ++cb) {
            float amax = 0.0f;
            for (int i = 0; i < 128; ++i)
                for (int j = 0; j < 128; ++j)
                    amax = fmaxf(amax, fabsf(pf8o_bf16_to_f32(w[(rb * 128 + i) * C + cb * 128 + j])));
            float sc = scale_from_amax(amax, pow2);
            for (int i = 0; i < 128; ++i)
                for (int j = 0; j < 128; ++j) {
                    int64_t r = rb * 128 + i, c = cb * 128 + j;
                    uint8_t v = pf8o_e4m3_encode(pf8o_bf16_to_f32(w[r * C + c]) / sc);
                    if (q) q[r * C + c] = v;
                    if (qt) qt[c * R + r] = v;
                }
            if (s) s[rb * CB + cb] = sc;
            if (st) st[cb * RB + rb] = sc;
        }
    }
}

static uint16_t* transpose_bf16(const uint16_t* x, int64_t M, int64_t K) {
    uint16_t* t = (uint16_t*)malloc((size_t)(M * K) * 2 + 2);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r)
        for (int64_t c = 0; c < K; ++c) t[c * M + r] = x[r * K + c];
    return t;
}

/* Fused quant+transpose.  transformers/fp8_utils.py:155-174 (padding_and_quant_input) treats
 * the fused call and two separate quantizations as interchangeable, so this IS two separate
 * 1x128 quantizations: of x (q[M,K]) and of x^T (qt[K,M]).  scale_layout applies to both
 * (1: s[K/128,M], st[M/128,K]; 0: s[M,K/128], st[K,M/128]).  (q,s) may be NULL. */
PF8O_API void pf8o_quant_transpose(const uint16_t* x, int64_t M, int64_t K, uint8_t* q, float* s,
                                   uint8_t* qt, float* st, int scale_layout, int pow2) {
    if (q) pf8o_quant_1x128(x, M, K, K, q, s, scale_layout, pow2);
    if (qt) {
        uint16_t* t = transpose_bf16(x, M, K);
        pf8o_quant_1x128(t, K, M, M, qt, st, scale_layout, pow2);
        free(t);
    }
}

/* Stack E weights, optional per-expert transpose, 128x128 quant.  Un-fused definition:
 * ernie token_dispatcher/fp8_utils.py:276-287 (stack -> transpose [0,2,1] -> reshape -> quant).
 * transpose=0: q[E*R, C], s[E*R/128, C/128]; transpose=1: q[E*C, R], s[E*C/128, R/128]. */
PF8O_API void pf8o_stack_transpose_quant(const uint16_t* const* w_list, int E, int64_t R, int64_t C,
                                         int transpose, uint8_t* q, float* s, int pow2) {
    for (int e = 0; e < E; ++e) {
        if (!transpose) {
            pf8o_quant_128x128(w_list[e], R, C, q + (int64_t)e * R * C, s + (int64_t)e * (R / 128) * (C / 128),
                               NULL, NULL, pow2);
        } else {
            uint16_t* t = transpose_bf16(w_list[e], R, C);
            pf8o_quant_128x128(t, C, R, q + (int64_t)e * R * C, s + (int64_t)e * (R / 128) * (C / 128),
                               NULL, NULL, pow2);
            free(t);
        }
    }
}

/* Fused SwiGLU (+ optional per-row probs) + 1x128 quant.  Un-fused definition:
 * ernie token_dispatcher/fp8_utils.py:996-1004: o2 = swiglu(o1) [bf16]; o2 = (o2*probs).cast(bf16);
 * quant 1x128.  Gate is the first half (transformers/fp8_utils.py:26-29, nn/experts.py:63).
 * o2_out (bf16, may be NULL) receives the pre-quant activations. */
PF8O_API void pf8o_swiglu_weighted_quant(const uint16_t* o1, const float* probs, int64_t M, int64_t I,
                                         uint8_t* q, float* s, int scale_layout, int pow2,
                                         uint16_t* o2_out) {
    uint16_t* o2 = o2_out ? o2_out : (uint16_t*)malloc((size_t)(M * I) * 2 + 2);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r) {
        for (int64_t j = 0; j < I; ++j) {
            float g = pf8o_bf16_to_f32(o1[r * 2 * I + j]);
            float u = pf8o_bf16_to_f32(o1[r * 2 * I + I + j]);
            float sg = pf8o_silu(g);
            uint16_t h = pf8o_f32_to_bf16(sg * u);
            if (probs) h = pf8o_f32_to_bf16(pf8o_bf16_to_f32(h) * probs[r]);
            o2[r * I + j] = h;
        }
    }
    if (q) pf8o_quant_1x128(o2, M, I, I, q, s, scale_layout, pow2);
    if (!o2_out) free(o2);
}

/* 1x128 dequant to bf16.  transformers/fp8_utils.py:136-138; kernel.py:87-97. */
PF8O_API void pf8o_act_dequant(const uint8_t* q, const float* s, int scale_layout, int64_t M, int64_t K,
                               uint16_t* out) {
    int64_t KB = K / 128;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r)
        for (int64_t c = 0; c < K; ++c) {
            float sc = scale_layout == 0 ? s[r * KB + c / 128] : s[(c / 128) * M + r];
            out[r * K + c] = pf8o_f32_to_bf16(pf8o_e4m3_decode(q[r * K + c]) * sc);
        }
}

/* 128x128 dequant to bf16.  kernel.py:73-118 (weight_dequant);
 * quantization/checkpoint_dequant.py:148-174, 277-292 (partial trailing blocks are cropped). */
PF8O_API void pf8o_weight_dequant(const uint8_t* q, const float* s, int64_t R, int64_t C, uint16_t* out) {
    int64_t CB = (C + 127) / 128;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r)
        for (int64_t c = 0; c < C; ++c)
            out[r * C + c] = pf8o_f32_to_bf16(pf8o_e4m3_decode(q[r * C + c]) * s[(r / 128) * CB + c / 128]);
}

/* Per-expert split -> transpose -> 1x128 quant along tokens.  Un-fused definition:
 * ernie token_dispatcher/fp8_utils.py:1199-1210.  With fp8 input the rows are first dequantised
 * to bf16 (transformers/fp8_utils.py:779-788 does fused_act_dequant -> quant on the dense path).
 * Outputs are packed: expert e's qt[K, M_e] starts at K*off_e, st[M_e/128, K] at (off_e/128)*K,
 * off_e = sum of earlier experts' rows.  xs is [Mtot, K/128] row-major (xs_layout 0) or
 * [K/128, Mtot] (xs_layout 1, the cached input_scale of transformers/fp8_utils.py:941). */
PF8O_API void pf8o_transpose_split_quant(const void* x, const float* xs, int x_is_fp8, int xs_layout,
                                         const int64_t* rows, int E, int64_t K, uint8_t* qt, float* st, int pow2) {
    int64_t off = 0, Mtot = 0;
    float* xs_rm = NULL;   /* scales re-laid row-major [Mtot, K/128] */
    for (int e = 0; e < E; ++e) Mtot += rows[e];
    if (x_is_fp8 && xs_layout == 1) {
        xs_rm = (float*)malloc((size_t)(Mtot * (K / 128)) * 4 + 4);
        for (int64_t r = 0; r < Mtot; ++r)
            for (int64_t b = 0; b < K / 128; ++b) xs_rm[r * (K / 128) + b] = xs[b * Mtot + r];
        xs = xs_rm;
    }
    for (int e = 0; e < E; ++e) {
        int64_t Me = rows[e];
        if (Me == 0) continue;
        uint16_t* xe = (uint16_t*)malloc((size_t)(Me * K) * 2);
        if (x_is_fp8) {
            pf8o_act_dequant((const uint8_t*)x + off * K, xs + off * (K / 128), 0, Me, K, xe);
        } else {
            memcpy(xe, (const uint16_t*)x + off * K, (size_t)(Me * K) * 2);
        }
        uint16_t* t = transpose_bf16(xe, Me, K);
        pf8o_quant_1x128(t, K, Me, Me, qt + off * K, st + (off / 128) * K, 1, pow2);
        free(t); free(xe);
        off += Me;
    }
    free(xs_rm);
}

/* SwiGLU backward with probs.  Un-fused definition: ernie token_dispatcher/fp8_utils.py:1088-1092;
 * swiglu_grad with sigma = 1/(1+exp(-g)): d_g = do2*u*sigma*(1+g*(1-sigma)), d_u = do2*silu(g).
 * probs_grad is summed in float64 and rounded once (the kernel's sum order is unspecified). */
PF8O_API void pf8o_swiglu_weighted_bwd(const uint16_t* o1, const uint16_t* do2_s, const float* probs,
                                       int64_t M, int64_t I, uint16_t* do1, float* probs_grad,
                                       uint16_t* o2_s) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < M; ++r) {
        double pg = 0.0;
        float p = probs[r];
        for (int64_t j = 0; j < I; ++j) {
            float g = pf8o_bf16_to_f32(o1[r * 2 * I + j]);
            float u = pf8o_bf16_to_f32(o1[r * 2 * I + I + j]);
            float e = pf8o_expf(-g);
            float den = 1.0f + e;
            float sl = g / den;
            uint16_t o2 = pf8o_f32_to_bf16(sl * u);
            float o2f = pf8o_bf16_to_f32(o2);
            o2_s[r * I + j] = pf8o_f32_to_bf16(o2f * p);
            float ds = pf8o_bf16_to_f32(do2_s[r * I + j]);
            float do2 = pf8o_bf16_to_f32(pf8o_f32_to_bf16(ds * p));
            pg += (double)ds * (double)o2f;
            float sig = 1.0f / den;
            float t1 = 1.0f - sig;
            float t2 = g * t1;
            float t3 = 1.0f + t2;
            float t4 = sig * t3;
            float t5 = do2 * u;
            do1[r * 2 * I + j] = pf8o_f32_to_bf16(t5 * t4);
            do1[r * 2 * I + I + j] = pf8o_f32_to_bf16(do2 * sl);
        }
        probs_grad[r] = (float)pg;
    }
}

/* ------------------------------------------------------------------------------------------ */
/* GEMMs                                                                                      */
/* ------------------------------------------------------------------------------------------ */

static float* decode_all(const uint8_t* q, int64_t n) {
    float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = pf8o_e4m3_decode((uint8_t)i);
    float* f = (float*)malloc((size_t)n * 4 + 4);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) f[i] = lut[q[i]];
    return f;
}

/* exact dot product of 128 e4m3 pairs: every product is exact in fp32 and the 128-term sum spans
 * < 53 bits, so a float64 sum is exact whatever the order. */
static inline double dot128(const float* a, const float* b) {
    double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    for (int k = 0; k < 128; k += 4) {
        s0 += (double)(a[k] * b[k]);
        s1 += (double)(a[k + 1] * b[k + 1]);
        s2 += (double)(a[k + 2] * b[k + 2]);
        s3 += (double)(a[k + 3] * b[k + 3]);
    }
    return (s0 + s1) + (s2 + s3);
}

static void gemm_nt_rows(const float* af, const float* sa, int sa_layout, int64_t sa_ld,
                         const float* bf, const float* sb, int64_t m0, int64_t m1, int64_t N, int64_t K,
                         uint16_t* out_bf16, float* out_f32, int64_t ldo) {
    int64_t KB = K / 128, NBs = (N + 127) / 128;
    (void)NBs;
#pragma omp parallel for schedule(static)
    for (int64_t m = m0; m < m1; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int64_t kb = 0; kb < KB; ++kb) {
                float d = (float)dot128(af + m * K + kb * 128, bf + n * K + kb * 128);
                float sA = sa_layout == 0 ? sa[m * KB + kb] : sa[kb * sa_ld + m];
                float sB = sb[(n / 128) * KB + kb];
                acc += d * sA * sB;
            }
            if (out_bf16) out_bf16[m * ldo + n] = pf8o_f32_to_bf16(acc);
            else out_f32[m * ldo + n] = acc;
        }
    }
}

/* Block-scaled NT GEMM.  kernel.py:160-187 (fp8_gemm_kernel): for each 128-wide K block
 * acc += dot(a_blk, b_blk) * a_s[:,None] * b_s[None,:] in fp32, then cast to bf16.
 * a[M,K], b[N,K] e4m3; sa layout 0: [M,K/128], 1: [K/128,M]; sb[ceil(N/128),K/128]. */
PF8O_API void pf8o_gemm_nt(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b, const float* sb,
                           int64_t M, int64_t N, int64_t K, uint16_t* out) {
    float* af = decode_all(a, M * K);
    float* bf = decode_all(b, N * K);
    gemm_nt_rows(af, sa, sa_layout, M, bf, sb, 0, M, N, K, out, NULL, N);
    free(af); free(bf);
}

/* The tolerance oracle named by the task: bf16( dequant(a) @ dequant(b)^T ) with the matmul in
 * float64 (dequantised values are fp32 products q*s, as in transformers/fp8_utils.py:136-138). */
PF8O_API void pf8o_gemm_nt_dequant_ref(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b,
                                       const float* sb, int64_t M, int64_t N, int64_t K, uint16_t* out) {
    int64_t KB = K / 128;
    float* af = decode_all(a, M * K);
    float* bf = decode_all(b, N * K);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k)
            af[m * K + k] *= (sa_layout == 0 ? sa[m * KB + k / 128] : sa[(k / 128) * M + m]);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) bf[n * K + k] *= sb[(n / 128) * KB + k / 128];
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
            const float* ap = af + m * K; const float* bp = bf + n * K;
            for (int64_t k = 0; k < K; k += 4) {
                s0 += (double)ap[k] * bp[k]; s1 += (double)ap[k + 1] * bp[k + 1];
                s2 += (double)ap[k + 2] * bp[k + 2]; s3 += (double)ap[k + 3] * bp[k + 3];
            }
            out[m * N + n] = pf8o_f32_to_bf16((float)((s0 + s1) + (s2 + s3)));
        }
    free(af); free(bf);
}

/* wgrad GEMM, both operands 1x128-scaled along the reduction dim, fp32 out, optional accumulate.
 * transformers/fp8_utils.py:176-221 (kitchen_gemm): out[Kin,N] (+)= x_t[Kin,M] . dout_t[N,M]^T with
 * x_t_scale[M/128,Kin], dout_t_scale[M/128,N]. */
PF8O_API void pf8o_gemm_nt_1d1d_f32(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                                    int64_t Kin, int64_t N, int64_t M, float* out, int accumulate) {
    int64_t MB = M / 128;
    float* af = decode_all(a_t, Kin * M);
    float* bf = decode_all(b_t, N * M);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < Kin; ++i)
        for (int64_t j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int64_t mb = 0; mb < MB; ++mb) {
                float d = (float)dot128(af + i * M + mb * 128, bf + j * M + mb * 128);
                acc += d * sa_t[mb * Kin + i] * sb_t[mb * N + j];
            }
            out[i * N + j] = accumulate ? out[i * N + j] + acc : acc;
        }
    free(af); free(bf);
}

/* Grouped GEMM, contiguous layout, restated as the per-expert loop the reference itself offers:
 * transformers/fp8_utils.py:853-870 (split_group_gemm); m_indices from :906-911.  Rows with
 * m_indices < 0 are left untouched. */
PF8O_API void pf8o_grouped_gemm_nt_contiguous(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b,
                                              const float* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                              const int32_t* m_indices, uint16_t* out) {
    int64_t KB = K / 128, NB = (N + 127) / 128;
    float* af = decode_all(a, Mtot * K);
    for (int e = 0; e < E; ++e) {
        float* bf = NULL;
        int64_t m = 0;
        while (m < Mtot) {
            if (m_indices[m] != e) { ++m; continue; }
            int64_t m1 = m;
            while (m1 < Mtot && m_indices[m1] == e) ++m1;
            if (!bf) bf = decode_all(b + (int64_t)e * N * K, N * K);
            gemm_nt_rows(af, sa, sa_layout, Mtot, bf, sb + (int64_t)e * NB * KB, m, m1, N, K, out, NULL, N);
            m = m1;
        }
        free(bf);
    }
    free(af);
}

/* Grouped GEMM, masked layout.  ernie token_dispatcher/fp8_utils.py:227-233: a[E,Mmax,K],
 * sa[E,Mmax,K/128], rows >= masked_m[e] ignored (left untouched in out[E,Mmax,N]). */
PF8O_API void pf8o_grouped_gemm_nt_masked(const uint8_t* a, const float* sa, const uint8_t* b, const float* sb,
                                          int E, int64_t Mmax, int64_t N, int64_t K, const int32_t* masked_m,
                                          uint16_t* out) {
    int64_t KB = K / 128, NB = (N + 127) / 128;
    for (int e = 0; e < E; ++e) {
        if (masked_m[e] <= 0) continue;
        float* af = decode_all(a + (int64_t)e * Mmax * K, Mmax * K);
        float* bf = decode_all(b + (int64_t)e * N * K, N * K);
        gemm_nt_rows(af, sa + (int64_t)e * Mmax * KB, 0, Mmax, bf, sb + (int64_t)e * NB * KB, 0, masked_m[e], N, K,
                     out + (int64_t)e * Mmax * N, NULL, N);
        free(af); free(bf);
    }
}

/* array forms of the scalar functions (for exhaustive sweeps in the tests) */
PF8O_API void pf8o_e4m3_encode_array(const float* v, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = pf8o_e4m3_encode(v[i]);
}
/* Checker for the device kernels' division-free quantizer step.  The formulation is q = x / s with an
 * IEEE divide per element (kernel.py:45-47); the kernels instead form y = 1/s once per tile and take
 *     q0 = x * y;  r = fma(-q0, s, x);  q = fma(r, y, q0)
 * per element.  Every quantizer input is a bf16 value and s = amax/448 of a bf16 amax, a finite set:
 * this walks ALL pairs (amax > 0 a finite bf16 magnitude, 0 <= x <= amax a bf16 magnitude; the device
 * copies the sign of x onto the result, which is what makes negative inputs, -0 included, symmetric) whose scale is at least min_scale (smaller ones take the divide on the device as well) and
 * counts, in out[0..2]: pairs visited, pairs whose e4m3 CODE differs between the two ways, pairs whose
 * fp32 quotient differs (those are quotients far below the e4m3 grid, where the residual underflows). */
PF8O_API void pf8o_check_reciprocal_division(int pow2, float min_scale, int64_t* out) {
    int64_t total = 0, bad_code = 0, bad_q = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : total, bad_code, bad_q)
    for (int ab = 1; ab < 0x7F80; ++ab) {
        const float amax = pf8o_bf16_to_f32((uint16_t)ab);
        const float s = scale_from_amax(amax, pow2);
        if (!(s >= min_scale)) continue;
        volatile float yv = 1.0f / s;
        const float y = yv;
        for (int xb = 0; xb <= ab; ++xb) {
            const float x = pf8o_bf16_to_f32((uint16_t)xb);
            volatile float qv = x / s;
            const float q = qv;
            const float q0 = x * y;
            const float r = fmaf(-q0, s, x);
            const float q1 = fmaf(r, y, q0);
            total++;
            if (pf8o_e4m3_encode(q1) != pf8o_e4m3_encode(q)) bad_code++;
            if (memcmp(&q1, &q, 4) != 0) bad_q++;
        }
    }
    out[0] = total; out[1] = bad_code; out[2] = bad_q;
}

PF8O_API void pf8o_div_encode_array(const float* x, const float* s, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = pf8o_e4m3_encode(x[i] / s[i]);
}
PF8O_API void pf8o_expf_array(const float* v, int64_t n, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = pf8o_expf(v[i]);
}
PF8O_API void pf8o_silu_array(const float* v, int64_t n, float* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = pf8o_silu(v[i]);
}
PF8O_API void pf8o_f32_to_bf16_array(const float* v, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < n; ++i) out[i] = pf8o_f32_to_bf16(v[i]);
}

PF8O_API int pf8o_version(void) { return 1; }
