// Prefill: quantised-weight GEMM  Y[M,N] = X[M,K] . W[N,K]^T  on the matrix cores (gfx950 MFMA).
//
// The reference has no such kernel: for M > 1 rows matmul_q runs M independent GEMVs
// (torch/io/gguf_model.h:7029-7036, :7056-7061), re-reading the weights M times.  These kernels keep the
// GEMV's arithmetic per output row and read each weight tile once per 64 rows of X.
//
// Q4_K (reference row semantics: torch/io/cpu_quant_gemv.h:505-685)
//   rows of X are quantised to Q8 blocks of 32 (same rule as the GEMV), and for every 32-wide sub-block
//   v_mfma_i32_16x16x32_i8 produces the exact integer dots of a 16x16 (m x n) tile: K = 32 of the
//   instruction is exactly one sub-block, so each result is scaled on the VALU by
//   fma(d*sc*dx[m], isum, -(dmin*mn*sx[m])) and added to the even/odd sub-block chains in the
//   reference's order (the result is bit-identical to the reference's per-row GEMV).
//   4-bit weights are unpacked in registers (an 8-byte slice of qs gives the B fragments of the low-
//   and high-nibble sub-blocks), Q8 activations of a 64-row x 256-column chunk are staged in LDS.
// Q6_K (reference row semantics: cpu_quant_gemv.h:883-1020, fp32 activations)
//   v_mfma_f32_16x16x16_bf16: K = 16 is exactly one scale group of Q6_K.  (q - 32) is exact in bf16 and
//   X is bf16 by contract, so products are exact; each 16-group sum is scaled by d*scale[n] in fp32.
#include "ptm_common.h"

namespace ptm {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));

enum { QG_NT = 2, QG_MT = 4, QG_MCHUNK = 16 * QG_MT, QG_NBLOCK = 4 * 16 * QG_NT, QG_PITCH8 = 256 + 8, QG_PITCH16 = 512 + 8 };

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__host__ __device__ inline int qg_mpad(int M) { return (M + QG_MCHUNK - 1) / QG_MCHUNK * QG_MCHUNK; }

// ---- rows of X (bf16) -> Q8 blocks: qs[Mpad][K], dT[K/32][Mpad], sT[K/32][Mpad]; rows >= M are zero ----
__global__ __launch_bounds__(256) void qgemm_quantize_rows_kernel(const uint16_t* __restrict__ X, int8_t* __restrict__ qs,
                                                                  float* __restrict__ dT, float* __restrict__ sT, int M,
                                                                  int Mpad, int K) {
    const int m = blockIdx.x;
    const int n4 = K / 4;
    for (int i = threadIdx.x; i < n4; i += 256) {  // K % 256 == 0: whole waves stay together
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m < M) {
            const uint2 raw = *reinterpret_cast<const uint2*>(X + (int64_t)m * K + 4 * i);
            v.x = bf16_to_f32(raw.x & 0xffffu);
            v.y = bf16_to_f32(raw.x >> 16);
            v.z = bf16_to_f32(raw.y & 0xffffu);
            v.w = bf16_to_f32(raw.y >> 16);
        }
        float d, s;
        const uint32_t packed = q8_quantize4(v, d, s);
        reinterpret_cast<uint32_t*>(qs + (int64_t)m * K)[i] = packed;
        if ((threadIdx.x & 7) == 0) {
            dT[(int64_t)(i >> 3) * Mpad + m] = d;
            sT[(int64_t)(i >> 3) * Mpad + m] = s;
        }
    }
}

// ---- Q4_K x Q8 on int8 MFMA ----------------------------------------------------------------------
// grid (ceil(N/128), Mpad/64), 256 threads; wave w owns columns [128*bx + 32*w, +32) as two 16-wide tiles.
__global__ __launch_bounds__(256) void qgemm_q4k_kernel(const uint8_t* __restrict__ W, int64_t stride,
                                                        const int8_t* __restrict__ qs, const float* __restrict__ dT,
                                                        const float* __restrict__ sT, float* __restrict__ Y, int M,
                                                        int Mpad, int K, int N) {
    __shared__ __align__(16) uint8_t s_x[QG_MCHUNK * QG_PITCH8];
    __shared__ __align__(16) float s_d[8][QG_MCHUNK];
    __shared__ __align__(16) float s_s[8][QG_MCHUNK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, kq = lane >> 4;  // MFMA: lane = (row or column) + 16 * (k / 8)
    const int m0 = blockIdx.y * QG_MCHUNK;
    const int nblk = K / 256;
    int ncol[QG_NT];
    const uint8_t* wrow[QG_NT];
#pragma unroll
    for (int t = 0; t < QG_NT; ++t) {
        ncol[t] = blockIdx.x * QG_NBLOCK + wave * (16 * QG_NT) + 16 * t + col;
        wrow[t] = W + (int64_t)min(ncol[t], N - 1) * stride;
    }
    float acc_a[QG_NT][QG_MT][4], acc_b[QG_NT][QG_MT][4];
#pragma unroll
    for (int t = 0; t < QG_NT; ++t)
#pragma unroll
        for (int mt = 0; mt < QG_MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc_a[t][mt][r] = acc_b[t][mt][r] = 0.0f;

    for (int b = 0; b < nblk; ++b) {
        // weights of this super-block for the lane's two columns
        uint4 hdr[QG_NT];
        uint2 raw[QG_NT][4];
#pragma unroll
        for (int t = 0; t < QG_NT; ++t) {
            const uint8_t* p = wrow[t] + (int64_t)b * 144;
            hdr[t] = *reinterpret_cast<const uint4*>(p);
#pragma unroll
            for (int g = 0; g < 4; ++g) raw[t][g] = *reinterpret_cast<const uint2*>(p + 16 + 32 * g + 8 * kq);
        }
        __syncthreads();  // previous chunk fully consumed
        // Q8 activations of rows [m0, m0+64), columns [256b, 256b+256): 64 x 256 B, 16 B per thread x 4
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int row = (tid >> 4) + 16 * it, cb = (tid & 15) * 16;
            *reinterpret_cast<uint4*>(s_x + row * QG_PITCH8 + cb) =
                *reinterpret_cast<const uint4*>(qs + (int64_t)(m0 + row) * K + b * 256 + cb);
        }
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int e = tid + 256 * it, sb = e >> 6, m = e & 63;
            s_d[sb][m] = dT[(int64_t)(b * 8 + sb) * Mpad + m0 + m];
            s_s[sb][m] = sT[(int64_t)(b * 8 + sb) * Mpad + m0 + m];
        }
        __syncthreads();

        float dsc[QG_NT][8], dmn[QG_NT][8];
#pragma unroll
        for (int t = 0; t < QG_NT; ++t) {
            const float d = h2f(hdr[t].x), dmin = h2f(hdr[t].x >> 16);
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                int sc, mn;
                q4k_scale_min(hdr[t].y, hdr[t].z, hdr[t].w, sb, sc, mn);
                dsc[t][sb] = d * (float)sc;
                dmn[t][sb] = dmin * (float)mn;
            }
        }
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) {
            const int g = sb >> 1;
            long bfrag[QG_NT];
#pragma unroll
            for (int t = 0; t < QG_NT; ++t) {
                const uint32_t lo = (sb & 1) ? ((raw[t][g].x >> 4) & 0x0f0f0f0fu) : (raw[t][g].x & 0x0f0f0f0fu);
                const uint32_t hi = (sb & 1) ? ((raw[t][g].y >> 4) & 0x0f0f0f0fu) : (raw[t][g].y & 0x0f0f0f0fu);
                bfrag[t] = (long)(((uint64_t)hi << 32) | lo);
            }
#pragma unroll
            for (int mt = 0; mt < QG_MT; ++mt) {
                const long afrag = *reinterpret_cast<const long*>(s_x + (mt * 16 + col) * QG_PITCH8 + sb * 32 + 8 * kq);
                const float4 dx = *reinterpret_cast<const float4*>(&s_d[sb][mt * 16 + 4 * kq]);
                const float4 sx = *reinterpret_cast<const float4*>(&s_s[sb][mt * 16 + 4 * kq]);
                const float dxr[4] = {dx.x, dx.y, dx.z, dx.w}, sxr[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                for (int t = 0; t < QG_NT; ++t) {
                    const v4i zero = {0, 0, 0, 0};
                    const v4i c = __builtin_amdgcn_mfma_i32_16x16x32_i8(afrag, bfrag[t], zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float w = dsc[t][sb] * dxr[r];
                        const float cm = dmn[t][sb] * sxr[r];
                        const float term = fmaf(w, (float)c[r], -cm);
                        if (sb & 1) acc_b[t][mt][r] += term;
                        else acc_a[t][mt][r] += term;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < QG_NT; ++t)
#pragma unroll
        for (int mt = 0; mt < QG_MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + mt * 16 + 4 * kq + r;
                if (m < M && ncol[t] < N) Y[(int64_t)m * N + ncol[t]] = acc_a[t][mt][r] + acc_b[t][mt][r];
            }
}

// ---- Q6_K x bf16 on bf16 MFMA --------------------------------------------------------------------
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t* p) {
    struct __attribute__((packed, aligned(2))) u32a2 { uint32_t v; };
    return reinterpret_cast<const u32a2*>(p)->v;
}
// two (q - 32) values (bytes b0, b1 of q in 0..63) as a packed pair of bf16
__device__ __forceinline__ uint32_t q_pair_bf16(uint32_t b0, uint32_t b1) {
    const float f0 = (float)(int)b0 - 32.0f, f1 = (float)(int)b1 - 32.0f;
    return (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xffff0000u);
}

__global__ __launch_bounds__(256) void qgemm_q6k_kernel(const uint8_t* __restrict__ W, int64_t stride,
                                                        const uint16_t* __restrict__ X, float* __restrict__ Y, int M,
                                                        int K, int N) {
    __shared__ __align__(16) uint8_t s_x[QG_MCHUNK * QG_PITCH16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, kq = lane >> 4;  // MFMA 16x16x16: lane = (row or column) + 16 * (k / 4)
    const int m0 = blockIdx.y * QG_MCHUNK;
    const int nblk = K / 256;
    int ncol[QG_NT];
    const uint8_t* wrow[QG_NT];
#pragma unroll
    for (int t = 0; t < QG_NT; ++t) {
        ncol[t] = blockIdx.x * QG_NBLOCK + wave * (16 * QG_NT) + 16 * t + col;
        wrow[t] = W + (int64_t)min(ncol[t], N - 1) * stride;
    }
    float acc[QG_NT][QG_MT][4];
#pragma unroll
    for (int t = 0; t < QG_NT; ++t)
#pragma unroll
        for (int mt = 0; mt < QG_MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][mt][r] = 0.0f;

    for (int b = 0; b < nblk; ++b) {
        // B fragments: for scale group s (16 weights) the lane holds elements 16s + 4kq + {0..3} of column n
        v4s bfrag[QG_NT][16];
        float fsc[QG_NT][16];
#pragma unroll
        for (int t = 0; t < QG_NT; ++t) {
            const uint8_t* p = wrow[t] + (int64_t)b * 210;
            const float d = h2f(reinterpret_cast<const u16_a2*>(p + 208)->v);
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                const int e = 16 * s + 4 * kq;  // first of the lane's four consecutive elements
                const int half = e >> 7, r = e & 127, grp = r >> 5, l5 = r & 31;
                const uint32_t ql = ld_u32_a2(p + 64 * half + 32 * (grp & 1) + l5);
                const uint32_t qh = ld_u32_a2(p + 128 + 32 * half + l5);
                const uint32_t q4 = (ql >> (4 * (grp >> 1))) & 0x0f0f0f0fu;
                const uint32_t q = q4 | (((qh >> (2 * grp)) & 0x03030303u) << 4);
                const uint32_t p01 = q_pair_bf16(q & 0xffu, (q >> 8) & 0xffu);
                const uint32_t p23 = q_pair_bf16((q >> 16) & 0xffu, q >> 24);
                v4s f;
                f[0] = (short)(p01 & 0xffffu); f[1] = (short)(p01 >> 16);
                f[2] = (short)(p23 & 0xffffu); f[3] = (short)(p23 >> 16);
                bfrag[t][s] = f;
                // scale index of element e: 8*half + 2*grp + l5/16
                fsc[t][s] = d * (float)(int)(int8_t)p[192 + 8 * half + 2 * grp + (l5 >> 4)];
            }
        }
        __syncthreads();
        // bf16 activations of rows [m0, m0+64), columns [256b, +256): 64 x 512 B, 16 B per thread x 8
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int row = (tid >> 5) + 8 * it, cb = (tid & 31) * 16;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m0 + row < M) v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(X) + ((int64_t)(m0 + row) * K + b * 256) * 2 + cb);
            *reinterpret_cast<uint4*>(s_x + row * QG_PITCH16 + cb) = v;
        }
        __syncthreads();
#pragma unroll
        for (int s = 0; s < 16; ++s) {
#pragma unroll
            for (int mt = 0; mt < QG_MT; ++mt) {
                const v4s afrag = *reinterpret_cast<const v4s*>(s_x + (mt * 16 + col) * QG_PITCH16 + (16 * s + 4 * kq) * 2);
#pragma unroll
                for (int t = 0; t < QG_NT; ++t) {
                    const v4f zero = {0.f, 0.f, 0.f, 0.f};
                    const v4f c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(afrag, bfrag[t][s], zero, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[t][mt][r] = fmaf(fsc[t][s], c[r], acc[t][mt][r]);
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < QG_NT; ++t)
#pragma unroll
        for (int mt = 0; mt < QG_MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + mt * 16 + 4 * kq + r;
                if (m < M && ncol[t] < N) Y[(int64_t)m * N + ncol[t]] = acc[t][mt][r];
            }
}

static int qgemm_check(const void* W, const void* X, const void* Y, int M, int K, int N, int64_t stride, int blk_bytes) {
    if (!W || !X || !Y) return PTM_E_NULL;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (stride < (int64_t)(K / 256) * blk_bytes) return PTM_E_SHAPE;
    if (!aligned16(X) || (reinterpret_cast<uintptr_t>(Y) & 3u)) return PTM_E_ALIGN;
    if ((int64_t)qg_mpad(M) / QG_MCHUNK > 65535) return PTM_E_UNSUPPORTED;
    return PTM_OK;
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int64_t ptm_qgemm_workspace_bytes(int M, int K) {
    if (M <= 0 || K <= 0) return 0;
    const int64_t mp = qg_mpad(M);
    return mp * K + 2 * (int64_t)(K / 32) * mp * 4;
}

int ptm_qgemm_q4k(const void* W, const void* X_bf16, float* Y, int M, int K, int N, int64_t stride, void* workspace,
                  ptm_stream_t stream) {
    int rc = qgemm_check(W, X_bf16, Y, M, K, N, stride, 144);
    if (rc != PTM_OK) return rc;
    if (!workspace) return PTM_E_NULL;
    if (!aligned16(W) || (stride & 15) || !aligned16(workspace)) return PTM_E_ALIGN;
    const int mp = qg_mpad(M);
    int8_t* qs = static_cast<int8_t*>(workspace);
    float* dT = reinterpret_cast<float*>(qs + (int64_t)mp * K);
    float* sT = dT + (int64_t)(K / 32) * mp;
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(qgemm_quantize_rows_kernel, dim3(mp), dim3(256), 0, s, static_cast<const uint16_t*>(X_bf16), qs, dT,
                       sT, M, mp, K);
    if ((rc = launch_status()) != PTM_OK) return rc;
    const dim3 grid((N + QG_NBLOCK - 1) / QG_NBLOCK, mp / QG_MCHUNK);
    hipLaunchKernelGGL(qgemm_q4k_kernel, grid, dim3(256), 0, s, static_cast<const uint8_t*>(W), stride, qs, dT, sT, Y, M, mp,
                       K, N);
    return launch_status();
}

int ptm_qgemm_q6k(const void* W, const void* X_bf16, float* Y, int M, int K, int N, int64_t stride, void* workspace,
                  ptm_stream_t stream) {
    (void)workspace;  // Q6_K consumes the bf16 activations directly
    const int rc = qgemm_check(W, X_bf16, Y, M, K, N, stride, 210);
    if (rc != PTM_OK) return rc;
    if ((stride & 1) || (reinterpret_cast<uintptr_t>(W) & 1u)) return PTM_E_ALIGN;
    const int mp = qg_mpad(M);
    const dim3 grid((N + QG_NBLOCK - 1) / QG_NBLOCK, mp / QG_MCHUNK);
    hipLaunchKernelGGL(qgemm_q6k_kernel, grid, dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(W), stride,
                       static_cast<const uint16_t*>(X_bf16), Y, M, K, N);
    return launch_status();
}

}  // extern "C"
