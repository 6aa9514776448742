// The GEMV dispatcher's other block formats: Q8_0 (34 B per 32 values), Q5_K (176 B per 256) and Q5_0 (22 B per 32),
// fp32 activations, as the reference's q8_0_gemv_avx2 / q5k_gemv_avx2 / q5_0_gemv_scalar compute them
// (torch/io/cpu_quant_gemv.h:784-826, :1091-1185, :1572-1630), and the dequantisers of the first two
// (torch/io/gguf_dequant.h:237-255, :348-388).  A Qwen3 / Llama Q4_K_M file holds none of these, so the kernels are
// plain: one wave per row, a lane per run of 32 values (a Q8_0 / Q5_0 block, or one of the eight sub-blocks of a
// Q5_K block), the lane's runs striding the row by 64, x read through the cache, one wave reduction per row.
#include "ptm_common.h"

namespace ptm {

struct __attribute__((packed, aligned(2))) u32_a2 { uint32_t v; };

// Σ q_i x_i over 32 values whose quants are 32 consecutive signed bytes at a 2-byte aligned address
__device__ __forceinline__ float dot32_i8(const uint8_t* __restrict__ q, const float* __restrict__ x) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const uint32_t v = reinterpret_cast<const u32_a2*>(q + 4 * w)->v;
        const float4 xv = *reinterpret_cast<const float4*>(x + 4 * w);
        s = fmaf((float)(int8_t)(v & 0xffu), xv.x, s);
        s = fmaf((float)(int8_t)((v >> 8) & 0xffu), xv.y, s);
        s = fmaf((float)(int8_t)((v >> 16) & 0xffu), xv.z, s);
        s = fmaf((float)(int8_t)(v >> 24), xv.w, s);
    }
    return s;
}

struct FmtQ8_0 {
    static constexpr int UNIT_BYTES = 34, UNITS_PER_BLOCK = 1, BLOCK_BYTES = 34;
    // contribution of run u (32 values) of a row
    static __device__ __forceinline__ float term(const uint8_t* __restrict__ row, int u, const float* __restrict__ x) {
        const uint8_t* p = row + (int64_t)u * 34;
        const float d = h2f(reinterpret_cast<const u16_a2*>(p)->v);
        return d * dot32_i8(p + 2, x + 32 * u);
    }
    static __device__ __forceinline__ float value(const uint8_t* __restrict__ blocks, int64_t e) {
        const uint8_t* p = blocks + (e >> 5) * 34;
        return h2f(reinterpret_cast<const u16_a2*>(p)->v) * (float)(int8_t)p[2 + (e & 31)];
    }
};

struct FmtQ5_0 {
    static constexpr int BLOCK_BYTES = 22;
    static __device__ __forceinline__ float term(const uint8_t* __restrict__ row, int u, const float* __restrict__ x) {
        const uint8_t* p = row + (int64_t)u * 22;
        const float d = h2f(reinterpret_cast<const u16_a2*>(p)->v);
        const uint32_t qh = reinterpret_cast<const u32_a2*>(p + 2)->v;
        const float* xb = x + 32 * u;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t v = reinterpret_cast<const u32_a2*>(p + 6 + 4 * w)->v;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = 4 * w + i;
                const uint32_t b = (v >> (8 * i)) & 0xffu;
                const int q0 = (int)((b & 0xfu) | (((qh >> j) & 1u) << 4)) - 16;
                const int q1 = (int)((b >> 4) | (((qh >> (j + 16)) & 1u) << 4)) - 16;
                s = fmaf((float)q0, xb[j], s);
                s = fmaf((float)q1, xb[j + 16], s);
            }
        }
        return d * s;
    }
};

struct FmtQ5_K {
    static constexpr int BLOCK_BYTES = 176;
    // scale and min of sub-block sb from the 12 packed bytes at p + 4 (get_scale_min_k4, gguf_dequant.h:289-297)
    static __device__ __forceinline__ void scale_min(const uint8_t* __restrict__ p, int sb, int& sc, int& mn) {
        const uint32_t* s = reinterpret_cast<const uint32_t*>(p + 4);
        q4k_scale_min(s[0], s[1], s[2], sb, sc, mn);
    }
    static __device__ __forceinline__ float term(const uint8_t* __restrict__ row, int u, const float* __restrict__ x) {
        const int sb = u & 7, pair = sb >> 1, hi = sb & 1;
        const uint8_t* p = row + (int64_t)(u >> 3) * 176;
        const uint32_t dd = *reinterpret_cast<const uint32_t*>(p);
        int sc, mn;
        scale_min(p, sb, sc, mn);
        const float ds = h2f(dd) * (float)sc, ms = h2f(dd >> 16) * (float)mn;
        const float* xb = x + 32 * u;
        float sq = 0.0f, sx = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const uint32_t nib = (*reinterpret_cast<const uint32_t*>(p + 48 + 32 * pair + 4 * w) >> (4 * hi)) & 0x0f0f0f0fu;
            const uint32_t bit = (*reinterpret_cast<const uint32_t*>(p + 16 + 4 * w) >> (2 * pair + hi)) & 0x01010101u;
            const uint32_t q = nib | (bit << 4);
            const float4 xv = *reinterpret_cast<const float4*>(xb + 4 * w);
            sq = fmaf((float)(q & 0xffu), xv.x, sq);
            sq = fmaf((float)((q >> 8) & 0xffu), xv.y, sq);
            sq = fmaf((float)((q >> 16) & 0xffu), xv.z, sq);
            sq = fmaf((float)(q >> 24), xv.w, sq);
            sx += (xv.x + xv.y) + (xv.z + xv.w);
        }
        return fmaf(ds, sq, -(ms * sx));
    }
    static __device__ __forceinline__ float value(const uint8_t* __restrict__ blocks, int64_t e) {
        const uint8_t* p = blocks + (e >> 8) * 176;
        const int r = (int)(e & 255), sb = r >> 5, pair = sb >> 1, hi = sb & 1, l = r & 31;
        const uint32_t dd = *reinterpret_cast<const uint32_t*>(p);
        int sc, mn;
        scale_min(p, sb, sc, mn);
        const float ds = h2f(dd) * (float)sc, ms = h2f(dd >> 16) * (float)mn;
        const uint32_t b = p[48 + 32 * pair + l];
        const int q = (int)((hi ? (b >> 4) : (b & 0xfu)) + (((p[16 + l] >> (2 * pair + hi)) & 1u) ? 16u : 0u));
        return ds * (float)q - ms;   // as the reference: d1 * q - m1, two roundings
    }
};

// Q4_K with fp32 activations, as the reference computes it where it has no AVX2 (q4k_gemv_scalar, cpu_quant_gemv.h:689-767):
// every weight is dequantised as fma(d * sc, q, -(dmin * m)) and multiplied with x, no Q8 rounding of the activations.
// The exact-math cross-check of the Q8-activation kernel, not a path of the decoder.  Run u is sub-block u & 7 of
// super-block u >> 3: 32 nibbles of one 32-byte group (low nibbles for even, high for odd sub-blocks).
struct FmtQ4_K_F32 {
    static constexpr int BLOCK_BYTES = 144;
    static __device__ __forceinline__ float term(const uint8_t* __restrict__ row, int u, const float* __restrict__ x) {
        const int sb = u & 7, hi = sb & 1;
        const uint8_t* p = row + (int64_t)(u >> 3) * 144;
        const uint4 hdr = *reinterpret_cast<const uint4*>(p);
        int sc, mn;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, sb, sc, mn);
        const float d1 = h2f(hdr.x) * (float)sc, m1 = h2f(hdr.x >> 16) * (float)mn;
        const uint8_t* qs = p + 16 + 32 * (sb >> 1);
        const float* xb = x + 32 * u;
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const uint32_t q = (*reinterpret_cast<const uint32_t*>(qs + 4 * w) >> (4 * hi)) & 0x0f0f0f0fu;
            const float4 xv = *reinterpret_cast<const float4*>(xb + 4 * w);
            s = fmaf(fmaf(d1, (float)(q & 0xffu), -m1), xv.x, s);
            s = fmaf(fmaf(d1, (float)((q >> 8) & 0xffu), -m1), xv.y, s);
            s = fmaf(fmaf(d1, (float)((q >> 16) & 0xffu), -m1), xv.z, s);
            s = fmaf(fmaf(d1, (float)(q >> 24), -m1), xv.w, s);
        }
        return s;
    }
};

// y[r] (+)= sum over the row's runs of 32; one wave per row, four rows per workgroup
template <typename Fmt, bool ACC>
__global__ __launch_bounds__(256) void rowwave_gemv_kernel(const uint8_t* __restrict__ W, const float* __restrict__ x,
                                                           float* __restrict__ y, int K, int N, int64_t stride) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= N) return;  // wave-uniform
    const uint8_t* row = W + (int64_t)r * stride;
    const int units = K / 32;
    float acc = 0.0f;
    for (int u = lane; u < units; u += 64) acc += Fmt::term(row, u, x);
    acc = sum64(acc);
    if (lane == 0) {
        if constexpr (ACC) y[r] += acc;
        else y[r] = acc;
    }
}

template <typename Fmt>
__global__ __launch_bounds__(256) void elementwise_dequant_kernel(const uint8_t* __restrict__ blocks, float* __restrict__ out,
                                                                  int64_t n) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n) out[e] = Fmt::value(blocks, e);
}

template <typename Fmt>
static int rowwave_launch(const void* W, const float* x, float* y, int K, int N, int64_t stride, int per_block,
                          int w_align, bool accumulate, hipStream_t s) {
    if (!W || !x || !y) return PTM_E_NULL;
    if (K <= 0 || N <= 0 || (K % per_block) != 0) return PTM_E_SHAPE;
    if (stride < (int64_t)(K / per_block) * Fmt::BLOCK_BYTES) return PTM_E_SHAPE;
    if ((stride % w_align) != 0 || (reinterpret_cast<uintptr_t>(W) % w_align) != 0 || !aligned16(x) ||
        (reinterpret_cast<uintptr_t>(y) & 3u))
        return PTM_E_ALIGN;
    const dim3 grid((N + 3) / 4), block(256);
    const uint8_t* w = static_cast<const uint8_t*>(W);
    if (accumulate) hipLaunchKernelGGL((rowwave_gemv_kernel<Fmt, true>), grid, block, 0, s, w, x, y, K, N, stride);
    else hipLaunchKernelGGL((rowwave_gemv_kernel<Fmt, false>), grid, block, 0, s, w, x, y, K, N, stride);
    return launch_status();
}

template <typename Fmt>
static int dequant_launch(const void* blocks, float* out, int64_t n, int per_block, int align, hipStream_t s) {
    if (!blocks || !out) return PTM_E_NULL;
    if (n < 0 || (n % per_block) != 0) return PTM_E_SHAPE;
    if ((reinterpret_cast<uintptr_t>(blocks) % align) != 0 || (reinterpret_cast<uintptr_t>(out) & 3u)) return PTM_E_ALIGN;
    if (n == 0) return PTM_OK;
    if ((n + 255) / 256 > 0x7fffffff) return PTM_E_UNSUPPORTED;
    hipLaunchKernelGGL((elementwise_dequant_kernel<Fmt>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                       static_cast<const uint8_t*>(blocks), out, n);
    return launch_status();
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_q8_0_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                  ptm_stream_t stream) {
    return rowwave_launch<FmtQ8_0>(W, x, y, K, N, row_stride_bytes, 32, 2, accumulate != 0, as_stream(stream));
}

int ptm_q5_0_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                  ptm_stream_t stream) {
    return rowwave_launch<FmtQ5_0>(W, x, y, K, N, row_stride_bytes, 32, 2, accumulate != 0, as_stream(stream));
}

int ptm_q5k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                 ptm_stream_t stream) {
    return rowwave_launch<FmtQ5_K>(W, x, y, K, N, row_stride_bytes, 256, 4, accumulate != 0, as_stream(stream));
}

int ptm_q4k_gemv_f32act(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                        ptm_stream_t stream) {
    return rowwave_launch<FmtQ4_K_F32>(W, x, y, K, N, row_stride_bytes, 256, 16, accumulate != 0, as_stream(stream));
}

int ptm_dequant_q8_0(const void* blocks, float* out, int64_t n, ptm_stream_t stream) {
    return dequant_launch<FmtQ8_0>(blocks, out, n, 32, 2, as_stream(stream));
}

int ptm_dequant_q5k(const void* blocks, float* out, int64_t n, ptm_stream_t stream) {
    return dequant_launch<FmtQ5_K>(blocks, out, n, 256, 4, as_stream(stream));
}

}  // extern "C"
