// pf8_permute.hip -- the token reordering either side of the grouped GEMMs: moe_permute gathers the
// routed copies of every token into expert-sorted order with each expert's segment padded to a
// multiple of `padding_alignment` rows (zero rows), moe_unpermute sums them back per token.
// Pure data movement, HBM-bound: every token row is read once and written once per routed copy.
#include "pf8_device.h"
#include "pf8_host.h"
#include "../../include/pf8.h"

namespace pf8 {

struct PermuteArgs {
    int64_t row_start[257];   // first output row of each expert's segment; row_start[E] = total padded rows
    int32_t count[256];       // routed rows of each expert (the rest of its segment is padding)
    int32_t E;
};

// One workgroup per expert: rank the tokens routed to it (stable in token order) with wave ballots
// and a running offset, fill its column of the row map, clear its padding rows' probabilities.
template <int TOPK>   // compile-time top-k (a multiple of 4: the routing row is read as 16-byte words), 0 = generic
__global__ __launch_bounds__(1024) void k_permute_rowmap(const int32_t* __restrict__ routemap, int64_t T, int topk, PermuteArgs pa,
                                                        int32_t* __restrict__ rowmap, float* __restrict__ out_probs,
                                                        int32_t* __restrict__ overflow, uint8_t* __restrict__ out_x, int64_t row_bytes,
                                                        float* __restrict__ out_xs, int64_t scale_cols) {
    // every thread ranks J tokens per step (token = step base + j * 1024 + tid, so rank order is
    // j-major): the J x topk loads of a step are in flight together and a step costs one barrier
    constexpr int J = 4;
    __shared__ int wave_cnt[2][J][16];    // double-buffered: one barrier per step
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int E = pa.E;
    int64_t base = pa.row_start[e];
    const int64_t limit = base + pa.count[e];
    int buf = 0;
    for (int64_t t0 = 0; t0 < T; t0 += 1024 * J, buf ^= 1) {
        bool hit[J];
        uint64_t m[J];
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int64_t t = t0 + j * 1024 + tid;
            hit[j] = false;
            if (t < T) {
                if (TOPK > 0) {
#pragma unroll
                    for (int k = 0; k < TOPK; k += 4) {
                        const int4 v = *reinterpret_cast<const int4*>(routemap + t * TOPK + k);
                        hit[j] |= v.x == e || v.y == e || v.z == e || v.w == e;
                    }
                } else {
                    for (int k = 0; k < topk; ++k) hit[j] |= routemap[t * topk + k] == e;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            m[j] = __ballot(hit[j]);
            if (lane == 0) wave_cnt[buf][j][wave] = __popcll(m[j]);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < J; ++j) {
            int before = __popcll(m[j] & ((1ull << lane) - 1ull)), total = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                const int c = wave_cnt[buf][j][w];
                before += w < wave ? c : 0;
                total += c;
            }
            const int64_t t = t0 + j * 1024 + tid;
            if (t < T) {
                int64_t row = hit[j] ? base + before : -1;
                if (row >= limit) { row = -1; atomicOr(overflow, 1); }      // more routed rows than tokens_per_expert says
                rowmap[t * E + e] = (int32_t)row;
            }
            base += total;
        }
    }
    if (out_probs)
        for (int64_t r = limit + tid; r < pa.row_start[e + 1]; r += 1024) out_probs[r] = 0.0f;
    // fewer routed rows than tokens_per_expert says: rows [base, limit) receive no token.  They are
    // flagged and cleared here, so that nothing uninitialised flows into the quantizers and GEMMs.
    if (base < limit) {
        if (tid == 0) atomicOr(overflow, 2);
        for (int64_t r = base; r < limit; ++r) {
            uint4* dst = reinterpret_cast<uint4*>(out_x + r * row_bytes);
            if (out_x)
                for (int64_t i = tid; i < row_bytes / 16; i += 1024) st16(dst + i, make_uint4(0, 0, 0, 0));
            if (out_xs)
                for (int64_t i = tid; i < scale_cols; i += 1024) out_xs[r * scale_cols + i] = 0.0f;
            if (out_probs && tid == 0) out_probs[r] = 0.0f;
        }
    }
}

// One workgroup per padding row: zero the row of tokens (and of scales).
__global__ __launch_bounds__(256) void k_permute_zero_pad(PermuteArgs pa, int64_t row_bytes, uint8_t* __restrict__ out_x,
                                                          int64_t scale_cols, float* __restrict__ out_xs) {
    // blockIdx.y = expert, blockIdx.x = padding row of that expert
    const int e = blockIdx.y;
    const int64_t r = pa.row_start[e] + pa.count[e] + blockIdx.x;
    if (r >= pa.row_start[e + 1]) return;
    uint4* dst = reinterpret_cast<uint4*>(out_x + r * row_bytes);
    for (int64_t i = threadIdx.x; i < row_bytes / 16; i += 256) st16(dst + i, make_uint4(0, 0, 0, 0));
    if (out_xs)
        for (int64_t i = threadIdx.x; i < scale_cols; i += 256) out_xs[r * scale_cols + i] = 0.0f;
}

// One workgroup per token: its row is read once into registers and written to every routed copy.
template <int MAXV>   // 16-byte chunks per thread held in registers
__global__ __launch_bounds__(256) void k_permute_gather(const uint8_t* __restrict__ x, const float* __restrict__ xs,
                                                        const int32_t* __restrict__ routemap, const float* __restrict__ probs,
                                                        const int32_t* __restrict__ rowmap, int64_t T, int64_t row_bytes, int64_t scale_cols,
                                                        int topk, int E, uint8_t* __restrict__ out_x, float* __restrict__ out_xs,
                                                        float* __restrict__ out_probs) {
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    const int64_t chunks = row_bytes / 16;
    uint4 v[MAXV];
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
        const int64_t c = tid + 256 * i;
        if (c < chunks) v[i] = ld16(reinterpret_cast<const uint4*>(x + t * row_bytes) + c);
    }
    for (int k = 0; k < topk; ++k) {
        const int e = routemap[t * topk + k];
        if (e < 0 || e >= E) continue;
        const int64_t r = rowmap[t * E + e];
        if (r < 0) continue;
        uint4* dst = reinterpret_cast<uint4*>(out_x + r * row_bytes);
#pragma unroll
        for (int i = 0; i < MAXV; ++i) {
            const int64_t c = tid + 256 * i;
            if (c < chunks) st16(dst + c, v[i]);
        }
        for (int64_t c = tid + 256 * (int64_t)MAXV; c < chunks; c += 256) st16(dst + c, *(reinterpret_cast<const uint4*>(x + t * row_bytes) + c));
        if (xs)
            for (int64_t c = tid; c < scale_cols; c += 256) out_xs[r * scale_cols + c] = xs[t * scale_cols + c];
        if (out_probs && tid == 0) out_probs[r] = probs ? probs[t * topk + k] : 0.0f;
    }
}

// The map-only form of the gather: one thread per routing slot writes the slot's token index (and probability) at the
// slot's row; rows no slot claims keep the -1 the fill kernel wrote.
__global__ __launch_bounds__(256) void k_fill_i32(int32_t* __restrict__ p, int64_t n, int32_t v) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

__global__ __launch_bounds__(256) void k_permute_source_rows(const int32_t* __restrict__ routemap, const float* __restrict__ probs,
                                                             const int32_t* __restrict__ rowmap, int64_t T, int topk, int E,
                                                             int32_t* __restrict__ src_row, float* __restrict__ out_probs) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= T * topk) return;
    const int64_t t = i / topk;
    const int e = routemap[i];
    if (e < 0 || e >= E) return;
    const int64_t r = rowmap[t * E + e];
    if (r < 0) return;
    src_row[r] = (int32_t)t;
    if (out_probs) out_probs[r] = probs ? probs[i] : 0.0f;
}

// The scales of rows that are read through a source map, gathered on their own (4 bytes per row and K block against the 128
// bytes they scale): out[r, kb] = xs[src_row[r], kb], 0 for a negative src_row; one thread per output element, row fastest.
template <int LAYOUT>
__global__ __launch_bounds__(256) void k_gather_row_scales(const float* __restrict__ xs, const int32_t* __restrict__ src_row, int64_t rows,
                                                           int64_t KB, float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * KB) return;
    const int64_t kb = i / rows, r = i % rows;
    const int t = src_row[r];
    const float v = t < 0 ? 0.0f : xs[(int64_t)t * KB + kb];
    if (LAYOUT == 1) out[kb * rows + r] = v;
    else out[r * KB + kb] = v;
}

// One workgroup per token: fp32 sum of its routed copies in slot order, bf16 out; probabilities back
// into [T, topk] order.
__global__ __launch_bounds__(256) void k_unpermute(const uint16_t* __restrict__ u, const int32_t* __restrict__ rowmap,
                                                   const int32_t* __restrict__ routemap, const float* __restrict__ probs_u, int64_t T,
                                                   int64_t H, int topk, int E, uint16_t* __restrict__ out, float* __restrict__ out_probs) {
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    for (int64_t c0 = (int64_t)tid * 8; c0 < H; c0 += 256 * 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < topk; ++k) {
            const int e = routemap[t * topk + k];
            if (e < 0 || e >= E) continue;
            const int64_t r = rowmap[t * E + e];
            if (r < 0) continue;
            const uint4 w = ld16(u + r * H + c0);
            float f[8];
            unpack8(w, f);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] += f[i];
        }
        st16(out + t * H + c0, make_uint4(pack_bf16(acc[0], acc[1]), pack_bf16(acc[2], acc[3]), pack_bf16(acc[4], acc[5]),
                                          pack_bf16(acc[6], acc[7])));
    }
    if (out_probs && tid < topk) {
        const int e = routemap[t * topk + tid];
        float p = 0.0f;
        if (e >= 0 && e < E) {
            const int64_t r = rowmap[t * E + e];
            if (r >= 0 && probs_u) p = probs_u[r];
        }
        out_probs[t * topk + tid] = p;
    }
}

}  // namespace pf8

using namespace pf8;

#define PF8_REQUIRE(cond, msg) do { if (!(cond)) return pf8_fail(PF8_EINVAL, __func__, msg); } while (0)
#define PF8_ALIGNED16(p) ((reinterpret_cast<uintptr_t>(p) & 15u) == 0)

extern "C" int pf8_moe_permute(const void* x, int x_is_fp8, const float* xs, const int32_t* routemap, const float* probs, int64_t T,
                               int64_t H, int topk, int E, const int64_t* tokens_per_expert, int padding_alignment, void* out_x,
                               int32_t* rowmap, float* out_probs, float* out_xs, int32_t* overflow, pf8_stream_t stream) {
    PF8_REQUIRE(T >= 0 && H >= 0 && topk > 0 && E > 0, "bad shape");
    PF8_REQUIRE(E <= 256, "at most 256 experts");
    PF8_REQUIRE(padding_alignment > 0, "padding_alignment must be positive");
    PF8_REQUIRE(tokens_per_expert, "tokens_per_expert is a host array of E counts");
    const int64_t row_bytes = x_is_fp8 ? H : 2 * H;
    PF8_REQUIRE(row_bytes % 16 == 0, "rows must be a multiple of 16 bytes");
    PF8_REQUIRE(!x_is_fp8 || H % 128 == 0, "fp8 tokens carry one scale per 128 columns");
    PF8_REQUIRE((xs != nullptr) == (out_xs != nullptr), "scale in and scale out come together");
    PermuteArgs pa = {};
    pa.E = E;
    int64_t total = 0, max_pad = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE(tokens_per_expert[e] >= 0 && tokens_per_expert[e] <= 0x7FFFFFFF, "bad tokens_per_expert");
        pa.row_start[e] = total;
        pa.count[e] = (int32_t)tokens_per_expert[e];
        const int64_t padded = (tokens_per_expert[e] + padding_alignment - 1) / padding_alignment * padding_alignment;
        if (padded - tokens_per_expert[e] > max_pad) max_pad = padded - tokens_per_expert[e];
        total += padded;
    }
    pa.row_start[E] = total;
    PF8_REQUIRE(total <= 0x7FFFFFFF, "too many rows");
    if (total == 0 && T == 0) return PF8_OK;
    PF8_REQUIRE(rowmap && overflow, "null pointer");
    PF8_REQUIRE(total == 0 || (out_x && PF8_ALIGNED16(out_x)), "null or misaligned output");
    PF8_REQUIRE(T == 0 || (x && routemap && PF8_ALIGNED16(x)), "null or misaligned input");
    hipStream_t st = (hipStream_t)stream;
    const int64_t scale_cols = xs ? H / 128 : 0;
    const bool rm16 = (reinterpret_cast<uintptr_t>(routemap) & 15u) == 0;
    // (the row-map kernel also clears the rows of an expert whose count overstates its routed tokens)
    if (topk == 8 && rm16) hipLaunchKernelGGL(k_permute_rowmap<8>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)out_x, row_bytes, out_xs, scale_cols);
    else if (topk == 4 && rm16) hipLaunchKernelGGL(k_permute_rowmap<4>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)out_x, row_bytes, out_xs, scale_cols);
    else hipLaunchKernelGGL(k_permute_rowmap<0>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)out_x, row_bytes, out_xs, scale_cols);
    int rc = pf8_check_launch(__func__);
    if (rc) return rc;
    if (max_pad > 0 && row_bytes > 0) {
        PF8_REQUIRE(max_pad <= 0x7FFFFFFF, "padding too large");
        hipLaunchKernelGGL(k_permute_zero_pad, dim3((unsigned)max_pad, (unsigned)E), dim3(256), 0, st, pa, row_bytes, (uint8_t*)out_x,
                           scale_cols, out_xs);
        rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    if (T > 0 && row_bytes > 0) {
        PF8_REQUIRE(T <= 0x7FFFFFFF, "too many tokens");
        const int64_t chunks = row_bytes / 16;
        if (chunks <= 256 * 2)
            hipLaunchKernelGGL(k_permute_gather<2>, dim3((unsigned)T), dim3(256), 0, st, (const uint8_t*)x, xs, routemap, probs, rowmap, T,
                               row_bytes, scale_cols, topk, E, (uint8_t*)out_x, out_xs, out_probs);
        else
            hipLaunchKernelGGL(k_permute_gather<4>, dim3((unsigned)T), dim3(256), 0, st, (const uint8_t*)x, xs, routemap, probs, rowmap, T,
                               row_bytes, scale_cols, topk, E, (uint8_t*)out_x, out_xs, out_probs);
        rc = pf8_check_launch(__func__);
    }
    return rc;
}

extern "C" int pf8_moe_permute_map(const int32_t* routemap, const float* probs, int64_t T, int topk, int E, const int64_t* tokens_per_expert,
                                   int padding_alignment, int32_t* rowmap, int32_t* src_row, float* out_probs, int32_t* overflow,
                                   pf8_stream_t stream) {
    PF8_REQUIRE(T >= 0 && topk > 0 && E > 0, "bad shape");
    PF8_REQUIRE(E <= 256, "at most 256 experts");
    PF8_REQUIRE(padding_alignment > 0, "padding_alignment must be positive");
    PF8_REQUIRE(tokens_per_expert, "tokens_per_expert is a host array of E counts");
    PermuteArgs pa = {};
    pa.E = E;
    int64_t total = 0;
    for (int e = 0; e < E; ++e) {
        PF8_REQUIRE(tokens_per_expert[e] >= 0 && tokens_per_expert[e] <= 0x7FFFFFFF, "bad tokens_per_expert");
        pa.row_start[e] = total;
        pa.count[e] = (int32_t)tokens_per_expert[e];
        total += (tokens_per_expert[e] + padding_alignment - 1) / padding_alignment * padding_alignment;
    }
    pa.row_start[E] = total;
    PF8_REQUIRE(total <= 0x7FFFFFFF && T <= 0x7FFFFFFF && T * topk <= 0x7FFFFFFFll * 256, "too many rows");
    if (total == 0 && T == 0) return PF8_OK;
    PF8_REQUIRE(rowmap && overflow && (total == 0 || src_row), "null pointer");
    PF8_REQUIRE(T == 0 || routemap, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (total > 0) {
        hipLaunchKernelGGL(k_fill_i32, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, src_row, total, -1);
        int rc = pf8_check_launch(__func__);
        if (rc) return rc;
    }
    const bool rm16 = (reinterpret_cast<uintptr_t>(routemap) & 15u) == 0;
    // no token rows to clear: the rows of an expert whose count overstates its routed tokens keep source -1 (read as zeros)
    if (topk == 8 && rm16) hipLaunchKernelGGL(k_permute_rowmap<8>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)nullptr, (int64_t)0, (float*)nullptr, (int64_t)0);
    else if (topk == 4 && rm16) hipLaunchKernelGGL(k_permute_rowmap<4>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)nullptr, (int64_t)0, (float*)nullptr, (int64_t)0);
    else hipLaunchKernelGGL(k_permute_rowmap<0>, dim3(E), dim3(1024), 0, st, routemap, T, topk, pa, rowmap, out_probs, overflow, (uint8_t*)nullptr, (int64_t)0, (float*)nullptr, (int64_t)0);
    int rc = pf8_check_launch(__func__);
    if (rc || T == 0) return rc;
    hipLaunchKernelGGL(k_permute_source_rows, dim3((unsigned)((T * topk + 255) / 256)), dim3(256), 0, st, routemap, probs, rowmap, T, topk, E,
                       src_row, out_probs);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_gather_row_scales(const float* xs, int64_t T, int64_t KB, const int32_t* src_row, int64_t rows, float* out, int out_layout,
                                     pf8_stream_t stream) {
    PF8_REQUIRE(T >= 0 && KB >= 0 && rows >= 0, "negative shape");
    PF8_REQUIRE(out_layout == 0 || out_layout == 1, "out_layout must be 0 or 1");
    if (rows == 0 || KB == 0) return PF8_OK;
    PF8_REQUIRE(src_row && out && (xs || T == 0), "null pointer");
    PF8_REQUIRE(rows * KB <= 0x7FFFFFFFll * 256, "too many scales");
    const dim3 grid((unsigned)((rows * KB + 255) / 256));
    if (out_layout == 1) hipLaunchKernelGGL(k_gather_row_scales<1>, grid, dim3(256), 0, (hipStream_t)stream, xs, src_row, rows, KB, out);
    else hipLaunchKernelGGL(k_gather_row_scales<0>, grid, dim3(256), 0, (hipStream_t)stream, xs, src_row, rows, KB, out);
    return pf8_check_launch(__func__);
}

extern "C" int pf8_moe_unpermute(const uint16_t* unzipped, const int32_t* rowmap, const int32_t* routemap, const float* probs_unzipped,
                                 int64_t T, int64_t H, int topk, int E, uint16_t* out, float* out_probs, pf8_stream_t stream) {
    PF8_REQUIRE(T >= 0 && H >= 0 && topk > 0 && E > 0, "bad shape");
    PF8_REQUIRE(topk <= 256, "topk too large");
    PF8_REQUIRE(H % 8 == 0, "H must be a multiple of 8");
    if (T == 0) return PF8_OK;
    PF8_REQUIRE(T <= 0x7FFFFFFF, "too many tokens");
    PF8_REQUIRE(rowmap && routemap && out && (unzipped || H == 0), "null pointer");
    PF8_REQUIRE(PF8_ALIGNED16(unzipped) && PF8_ALIGNED16(out), "pointers must be 16-byte aligned");
    hipLaunchKernelGGL(k_unpermute, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, unzipped, rowmap, routemap, probs_unzipped, T, H,
                       topk, E, out, out_probs);
    return pf8_check_launch(__func__);
}
