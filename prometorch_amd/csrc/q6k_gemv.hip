// Q6_K dequant-fused GEMV for gfx950 (wave64), fp32 activations as in the reference CPU
// kernel (torch/io/cpu_quant_gemv.h:883-1020): y = sum_k (d*scale*(q-32)) * x_k, fp32 accumulate.
//
// A row is swept by an aligned group of 8 lanes.  Per 210-byte super-block lane j fetches
//   ql[16j .. 16j+16)            16 low nibbles  -> group (j%4)/2   of half j/4
//                                16 high nibbles -> group (j%4)/2+2 of half j/4
//   qh[32*(j/4) + 16*(j%2) ..+16) the 2-bit planes of those 32 weights
//   scales[16] and d             (same for the 8 lanes)
// with 128-bit loads (blocks are only 2-byte aligned; gfx950 global loads take that).
// Weights are assembled four at a time in a dword (q = nibble | twobits<<4, 0..63), converted
// with v_cvt_f32_ubyteN and multiplied with x from LDS; the "-32" offset is applied once per
// 16 weights through the per-16 sums of x kept in LDS:  sum (q-32) x = sum q x - 32 sum x.
#include "ptm_common.h"

namespace ptm {

struct Q6KArgs {
    const uint8_t* W;
    const float* x;
    float* y;        // may be NULL when only the argmax is wanted
    int K, N;
    int64_t stride;
    float* part_val; // ARGMAX: per-workgroup best value / index
    int* part_idx;
};

enum { Q6K_THREADS = 256, Q6K_ROWS_PER_WG = 32 };

__device__ __forceinline__ float dot4_u8(uint32_t q, float4 x, float acc) {
    acc = fmaf((float)(q & 0xffu), x.x, acc);
    acc = fmaf((float)((q >> 8) & 0xffu), x.y, acc);
    acc = fmaf((float)((q >> 16) & 0xffu), x.z, acc);
    acc = fmaf((float)(q >> 24), x.w, acc);
    return acc;
}

template <int U>
__device__ __forceinline__ float q6k_row_partial(const uint8_t* __restrict__ row, int nblk,
                                                 const float* __restrict__ xf, const float* __restrict__ xsum16,
                                                 int j) {
    const int half = j >> 2, jj = j & 3, which32 = jj >> 1, l16 = jj & 1;
    const int qh_off = 128 + 32 * half + 16 * l16;
    const int sc_lo_i = 8 * half + 2 * which32 + l16;  // scale of the low-nibble 16; high-nibble one is +4
    const int hshift = 2 * which32;
    const int xo = 128 * half + 32 * which32 + 16 * l16;  // x offset of the low-nibble 16; high-nibble +64
    float acc = 0.0f;
    for (int b0 = 0; b0 < nblk; b0 += U) {
        uint4 ql[U], qh[U], sc[U];
        uint32_t dd[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int b = min(b0 + u, nblk - 1);
            const uint8_t* p = row + (int64_t)b * 210;
            ql[u] = ld16_a2(p + 16 * j);
            qh[u] = ld16_a2(p + qh_off);
            sc[u] = ld16_a2(p + 192);
            dd[u] = reinterpret_cast<const u16_a2*>(p + 208)->v;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int b = b0 + u;
            if (b < nblk) {
                const float* xb = xf + b * 256 + xo;
                float s_lo = 0.0f, s_hi = 0.0f;
                const uint32_t qlw[4] = {ql[u].x, ql[u].y, ql[u].z, ql[u].w};
                const uint32_t qhw[4] = {qh[u].x, qh[u].y, qh[u].z, qh[u].w};
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t hs = qhw[w] >> hshift;
                    const uint32_t q_lo = (qlw[w] & 0x0f0f0f0fu) | ((hs << 4) & 0x30303030u);
                    const uint32_t q_hi = ((qlw[w] >> 4) & 0x0f0f0f0fu) | (hs & 0x30303030u);
                    const float4 x_lo = *reinterpret_cast<const float4*>(xb + 4 * w);
                    const float4 x_hi = *reinterpret_cast<const float4*>(xb + 64 + 4 * w);
                    s_lo = dot4_u8(q_lo, x_lo, s_lo);
                    s_hi = dot4_u8(q_hi, x_hi, s_hi);
                }
                const int xi = (b * 256 + xo) >> 4;
                s_lo = fmaf(-32.0f, xsum16[xi], s_lo);
                s_hi = fmaf(-32.0f, xsum16[xi + 4], s_hi);
                const uint32_t scw[4] = {sc[u].x, sc[u].y, sc[u].z, sc[u].w};
                const uint32_t w_lo = scw[sc_lo_i >> 2] >> (8 * (sc_lo_i & 3));
                const uint32_t w_hi = scw[(sc_lo_i + 4) >> 2] >> (8 * (sc_lo_i & 3));
                const float d = h2f(dd[u]);
                const float f_lo = d * (float)(int)(int8_t)(w_lo & 0xffu);
                const float f_hi = d * (float)(int)(int8_t)(w_hi & 0xffu);
                acc = fmaf(f_lo, s_lo, acc);
                acc = fmaf(f_hi, s_hi, acc);
            }
        }
    }
    return acc;
}

template <bool ACC, bool ARGMAX, int U>
__global__ __launch_bounds__(Q6K_THREADS) void q6k_gemv_kernel(const Q6KArgs a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    float* xf = reinterpret_cast<float*>(lds_raw);
    float* xsum16 = xf + a.K;
    const int tid = threadIdx.x;
    // stage x and its per-16 sums: 4 consecutive float4 slots (4 lanes) make one 16-group
    const float4* x4 = reinterpret_cast<const float4*>(a.x);
    for (int i = tid; i < a.K / 4; i += Q6K_THREADS) {
        const float4 v = x4[i];
        reinterpret_cast<float4*>(xf)[i] = v;
        float s = (v.x + v.y) + (v.z + v.w);
        s += dpp_f<0xB1>(s);
        s += dpp_f<0x4E>(s);
        if ((tid & 3) == 0) xsum16[i >> 2] = s;
    }
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6, j = lane & 7;
    const int r = blockIdx.x * Q6K_ROWS_PER_WG + wave * 8 + (lane >> 3);
    const bool live = r < a.N;
    const int rr = live ? r : a.N - 1;
    float p = q6k_row_partial<U>(a.W + (int64_t)rr * a.stride, a.K / 256, xf, xsum16, j);
    p = sum8(p);
    if (live && j == 0 && a.y) {
        if constexpr (ACC) a.y[rr] += p;
        else a.y[rr] = p;
    }
    if constexpr (ARGMAX) {
        // best (value, lowest index) of this workgroup's 32 rows
        __shared__ float bv[4];
        __shared__ int bi[4];
        float v = live ? p : -INFINITY;
        int idx = rr;
        for (int off = 8; off < 64; off <<= 1) {
            const float ov = __shfl_xor(v, off, 64);
            const int oi = __shfl_xor(idx, off, 64);
            if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
        }
        if (lane == 0) { bv[wave] = v; bi[wave] = idx; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < 4; ++w)
                if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
            a.part_val[blockIdx.x] = v;
            a.part_idx[blockIdx.x] = idx;
        }
    }
}

__global__ __launch_bounds__(256) void argmax_partials_kernel(const float* pv, const int* pi, int n, int64_t* out) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float ov = pv[i];
        const int oi = pi[i];
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
        *out = (int64_t)idx;
    }
}

static int q6k_check(const void* W, const void* x, int K, int N, int64_t stride) {
    if (!W || !x) return PTM_E_NULL;
    if (K <= 0 || N <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (K > 32768) return PTM_E_UNSUPPORTED;  // x + per-16 sums must fit LDS (K*4.25 bytes <= 136 KB)
    if (stride < (int64_t)(K / 256) * 210) return PTM_E_SHAPE;
    if ((stride & 1) != 0 || (reinterpret_cast<uintptr_t>(W) & 1u) || !aligned16(x)) return PTM_E_ALIGN;
    return PTM_OK;
}

template <bool ACC, bool ARGMAX>
static int q6k_launch(const Q6KArgs& a, hipStream_t s) {
    const int grid = (a.N + Q6K_ROWS_PER_WG - 1) / Q6K_ROWS_PER_WG;
    const size_t lds = (size_t)a.K * 4 + (size_t)a.K / 4;
    static bool attr_done = false;  // raise the dynamic-LDS cap once, outside any capture
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_kernel<false, false, 5>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_kernel<true, false, 5>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_kernel<false, true, 5>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
        attr_done = true;
    }
    hipLaunchKernelGGL((q6k_gemv_kernel<ACC, ARGMAX, 5>), dim3(grid), dim3(Q6K_THREADS), lds, s, a);
    return launch_status();
}

int q6k_gemv_impl(const void* W, const float* x, float* y, int K, int N, int64_t stride, bool accumulate,
                  hipStream_t s) {
    const int rc = q6k_check(W, x, K, N, stride);
    if (rc != PTM_OK) return rc;
    if (!y) return PTM_E_NULL;
    Q6KArgs a{static_cast<const uint8_t*>(W), x, y, K, N, stride, nullptr, nullptr};
    return accumulate ? q6k_launch<true, false>(a, s) : q6k_launch<false, false>(a, s);
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_q6k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t stride, int accumulate,
                 ptm_stream_t stream) {
    return q6k_gemv_impl(W, x, y, K, N, stride, accumulate != 0, as_stream(stream));
}

int64_t ptm_argmax_workspace_bytes(int N) {
    const int64_t g = (N + Q6K_ROWS_PER_WG - 1) / Q6K_ROWS_PER_WG;
    return g * 8;
}

int ptm_q6k_gemv_argmax(const void* W, const float* x, float* logits, int K, int N, int64_t stride,
                        int64_t* out_index, void* workspace, ptm_stream_t stream) {
    const int rc = q6k_check(W, x, K, N, stride);
    if (rc != PTM_OK) return rc;
    if (!out_index || !workspace) return PTM_E_NULL;
    const int grid = (N + Q6K_ROWS_PER_WG - 1) / Q6K_ROWS_PER_WG;
    Q6KArgs a{static_cast<const uint8_t*>(W), x, logits, K, N, stride, static_cast<float*>(workspace),
              reinterpret_cast<int*>(static_cast<float*>(workspace) + grid)};
    const int rc2 = q6k_launch<false, true>(a, as_stream(stream));
    if (rc2 != PTM_OK) return rc2;
    hipLaunchKernelGGL(argmax_partials_kernel, dim3(1), dim3(256), 0, as_stream(stream), a.part_val, a.part_idx,
                       grid, out_index);
    return launch_status();
}

}  // extern "C"
