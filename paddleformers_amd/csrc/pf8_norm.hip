// pf8_norm.hip -- RMSNorm forward and backward for the FP8 MLP with norm recompute
// (FusedNormFP8MLPFunction): y = bf16(x * invar * w), invar = 1/sqrt(mean(x^2) + eps) per row.
// HBM-bound row kernels: one workgroup per row forward; backward, a fixed number of workgroups walk the
// rows with a stride, each keeps its share of the weight gradient in registers and writes it to a
// row of a caller-provided workspace, which a second kernel sums into dw (without a workspace the
// partial sums go to dw by atomics: every workgroup then adds to the same H addresses, and on
// [16384, 7168] that alone takes four times as long as moving the data).
#include "pf8_device.h"
#include "pf8_host.h"
#include "../../include/pf8.h"

namespace pf8 {

__device__ __forceinline__ float block_sum(float v, float* lds4) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    const int wave = threadIdx.x >> 6;
    __syncthreads();                       // lds4 may still be read from the previous call
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}

template <int MAXC>   // column chunks (of 8) per thread, kept packed in registers between the two passes (0: re-read)
__global__ __launch_bounds__(256) void k_rms_norm_fwd(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, float eps, int64_t M,
                                                      int64_t H, uint16_t* __restrict__ y, float* __restrict__ invar) {
    __shared__ float lds4[4];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    const int64_t chunks = H / 8;
    const uint4* xr = reinterpret_cast<const uint4*>(x + r * H);
    uint4 xp[MAXC > 0 ? MAXC : 1];
    float ss = 0.0f;
    if (MAXC > 0) {
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int64_t c = tid + 256 * j;
            xp[j] = c < chunks ? ld16(xr + c) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            float v[8];
            unpack8(xp[j], v);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __builtin_fmaf(v[i], v[i], ss);
        }
    } else {
        for (int64_t c = tid; c < chunks; c += 256) {
            float v[8];
            unpack8(ld16(xr + c), v);
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = __builtin_fmaf(v[i], v[i], ss);
        }
    }
    ss = block_sum(ss, lds4);
    const float iv = 1.0f / __builtin_sqrtf(ss / (float)H + eps);
    if (tid == 0) invar[r] = iv;
    uint4* yr = reinterpret_cast<uint4*>(y + r * H);
    const uint4* wr = reinterpret_cast<const uint4*>(w);
    auto emit = [&](int64_t c, uint4 xw) {
        float v[8], g[8];
        unpack8(xw, v);
        unpack8(wr[c], g);
        uint4 o;
        o.x = pack_bf16(v[0] * iv * g[0], v[1] * iv * g[1]);
        o.y = pack_bf16(v[2] * iv * g[2], v[3] * iv * g[3]);
        o.z = pack_bf16(v[4] * iv * g[4], v[5] * iv * g[5]);
        o.w = pack_bf16(v[6] * iv * g[6], v[7] * iv * g[7]);
        st16(yr + c, o);
    };
    if (MAXC > 0) {
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int64_t c = tid + 256 * j;
            if (c < chunks) emit(c, xp[j]);
        }
    } else {
        for (int64_t c = tid; c < chunks; c += 256) emit(c, xr[c]);
    }
}

// dx = invar * (g - x * invar^2 * mean(g * x)),  g = dy * w;   dw += sum_rows dy * x * invar
template <int MAXC>   // column chunks (of 8) per thread whose weight gradient lives in registers
__global__ __launch_bounds__(256) void k_rms_norm_bwd(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                      const float* __restrict__ invar, const uint16_t* __restrict__ dy, int64_t M, int64_t H,
                                                      uint16_t* __restrict__ dx, float* __restrict__ dw, float* __restrict__ ws) {
    __shared__ float lds4[4];
    const int tid = threadIdx.x;
    const int64_t chunks = H / 8;
    const uint4* wr = reinterpret_cast<const uint4*>(w);
    float dwa[MAXC][8];
#pragma unroll
    for (int j = 0; j < MAXC; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) dwa[j][i] = 0.0f;
    for (int64_t r = blockIdx.x; r < M; r += gridDim.x) {
        const uint4* xr = reinterpret_cast<const uint4*>(x + r * H);
        const uint4* dr = reinterpret_cast<const uint4*>(dy + r * H);
        const float iv = invar[r];
        float s1 = 0.0f;
        uint4 xp[MAXC], dp[MAXC];          // the row stays in registers (packed) between the two passes
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int64_t c = tid + 256 * j;
            xp[j] = make_uint4(0, 0, 0, 0);
            dp[j] = make_uint4(0, 0, 0, 0);
            if (c < chunks) {
                xp[j] = ld16(xr + c);
                dp[j] = ld16(dr + c);
            }
        }
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int64_t c = tid + 256 * j;
            if (c < chunks) {
                float xv[8], dv[8], gv[8];
                unpack8(xp[j], xv);
                unpack8(dp[j], dv);
                unpack8(wr[c], gv);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    s1 = __builtin_fmaf(dv[i] * gv[i], xv[i], s1);
                    dwa[j][i] = __builtin_fmaf(dv[i] * xv[i], iv, dwa[j][i]);
                }
            }
        }
        s1 = block_sum(s1, lds4);
        const float k = iv * iv * iv * (s1 / (float)H);
        uint4* oxr = reinterpret_cast<uint4*>(dx + r * H);
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int64_t c = tid + 256 * j;
            if (c < chunks) {
                float xv[8], dv[8], gv[8], o[8];
                unpack8(xp[j], xv);
                unpack8(dp[j], dv);
                unpack8(wr[c], gv);
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = dv[i] * gv[i] * iv - xv[i] * k;
                st16(oxr + c, make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7])));
            }
        }
    }
#pragma unroll
    for (int j = 0; j < MAXC; ++j) {
        const int64_t c = tid + 256 * j;
        if (c < chunks) {
            if (ws) {
                float* o = ws + (int64_t)blockIdx.x * H + c * 8;
                *reinterpret_cast<f32x4*>(o) = (f32x4){dwa[j][0], dwa[j][1], dwa[j][2], dwa[j][3]};
                *reinterpret_cast<f32x4*>(o + 4) = (f32x4){dwa[j][4], dwa[j][5], dwa[j][6], dwa[j][7]};
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) atomicAdd(dw + c * 8 + i, dwa[j][i]);
            }
        }
    }
}

// dw[c] += sum over the workspace rows, in a fixed order (the result does not depend on scheduling). A workgroup
// owns 64 columns: 16 lanes of four floats across, 64 row slots down; a slot sums the rows r = slot, slot + 64, ...
// and the slots are folded through LDS in slot order.
__global__ __launch_bounds__(1024) void k_rms_norm_dw_reduce(const float* __restrict__ ws, int rows, int64_t H, float* __restrict__ dw) {
    __shared__ f32x4 part[64][16];
    const int lane = threadIdx.x & 15, slot = threadIdx.x >> 4;
    const int64_t c4 = (int64_t)blockIdx.x * 16 + lane;
    const bool live = c4 * 4 < H;
    f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
    if (live) {
        const float* col = ws + c4 * 4;
        int r = slot;
        for (; r + 192 < rows; r += 256) {
            const f32x4 v0 = *reinterpret_cast<const f32x4*>(col + (int64_t)r * H);
            const f32x4 v1 = *reinterpret_cast<const f32x4*>(col + (int64_t)(r + 64) * H);
            const f32x4 v2 = *reinterpret_cast<const f32x4*>(col + (int64_t)(r + 128) * H);
            const f32x4 v3 = *reinterpret_cast<const f32x4*>(col + (int64_t)(r + 192) * H);
            s0 += v0; s1 += v1; s2 += v2; s3 += v3;
        }
        for (; r < rows; r += 64) s0 += *reinterpret_cast<const f32x4*>(col + (int64_t)r * H);
    }
    part[slot][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (threadIdx.x < 64) {
        const int64_t c = (int64_t)blockIdx.x * 64 + threadIdx.x;
        if (c < H) {
            const float* pl = reinterpret_cast<const float*>(&part[0][0]) + threadIdx.x;
            float t0 = 0.0f, t1 = 0.0f, t2 = 0.0f, t3 = 0.0f;
#pragma unroll
            for (int k = 0; k < 64; k += 4) {
                t0 += pl[k * 64];
                t1 += pl[(k + 1) * 64];
                t2 += pl[(k + 2) * 64];
                t3 += pl[(k + 3) * 64];
            }
            dw[c] += (t0 + t1) + (t2 + t3);
        }
    }
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

extern "C" int pf8_rms_norm_fwd(const uint16_t* x, const uint16_t* w, float eps, int64_t M, int64_t H, uint16_t* y, float* invar,
                                pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && H > 0 && H % 8 == 0, "H must be a positive multiple of 8");
    if (M == 0) return PF8_OK;
    PF8_REQUIRE(M <= 0x7FFFFFFF, "too many rows");
    PF8_REQUIRE(x && w && y && invar, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(x) && PF8_ALIGNED16(w) && PF8_ALIGNED16(y), "pointers must be 16-byte aligned");
    const int64_t chunks = H / 8;
    hipStream_t st = (hipStream_t)stream;
    if (chunks <= 256 * 2) hipLaunchKernelGGL(k_rms_norm_fwd<2>, dim3((unsigned)M), dim3(256), 0, st, x, w, eps, M, H, y, invar);
    else if (chunks <= 256 * 4) hipLaunchKernelGGL(k_rms_norm_fwd<4>, dim3((unsigned)M), dim3(256), 0, st, x, w, eps, M, H, y, invar);
    else if (chunks <= 256 * 8) hipLaunchKernelGGL(k_rms_norm_fwd<8>, dim3((unsigned)M), dim3(256), 0, st, x, w, eps, M, H, y, invar);
    else hipLaunchKernelGGL(k_rms_norm_fwd<0>, dim3((unsigned)M), dim3(256), 0, st, x, w, eps, M, H, y, invar);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_rms_norm_bwd(const uint16_t* x, const uint16_t* w, const float* invar, const uint16_t* dy, int64_t M, int64_t H,
                                uint16_t* dx, float* dw, float* ws, int64_t ws_rows, pf8_stream_t stream) {
    PF8_REQUIRE(M >= 0 && H > 0 && H % 8 == 0, "H must be a positive multiple of 8");
    PF8_REQUIRE(H <= 8 * 256 * 8, "H larger than 16384 is not supported");
    if (M == 0) return PF8_OK;
    PF8_REQUIRE(x && w && invar && dy && dx && dw, "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(x) && PF8_ALIGNED16(w) && PF8_ALIGNED16(dy) && PF8_ALIGNED16(dx), "pointers must be 16-byte aligned");
    PF8_REQUIRE(!ws || (ws_rows >= 1 && PF8_ALIGNED16(ws)), "the workspace must be 16-byte aligned and hold at least one row");
    // with a workspace: as many workgroups as it has rows (1024 fill the device four deep); without: one per
    // compute unit, to keep the atomics on dw few
    int64_t wgs = ws ? (ws_rows < 1024 ? ws_rows : 1024) : 256;
    if (wgs > M) wgs = M;
    const int64_t chunks = H / 8;
    hipStream_t st = (hipStream_t)stream;
    if (chunks <= 256 * 2) hipLaunchKernelGGL(k_rms_norm_bwd<2>, dim3((unsigned)wgs), dim3(256), 0, st, x, w, invar, dy, M, H, dx, dw, ws);
    else if (chunks <= 256 * 4) hipLaunchKernelGGL(k_rms_norm_bwd<4>, dim3((unsigned)wgs), dim3(256), 0, st, x, w, invar, dy, M, H, dx, dw, ws);
    else hipLaunchKernelGGL(k_rms_norm_bwd<8>, dim3((unsigned)wgs), dim3(256), 0, st, x, w, invar, dy, M, H, dx, dw, ws);
    int rc = pf8_check_launch(__func__);
    if (rc || !ws) return rc;
    hipLaunchKernelGGL(k_rms_norm_dw_reduce, dim3((unsigned)((H + 63) / 64)), dim3(1024), 0, st, ws, (int)wgs, H, dw);
    return pf8_check_launch(__func__);
}
