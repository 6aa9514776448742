// Prefill: quantised-weight GEMM  Y[M,N] = X[M,K] . W[N,K]^T  on the matrix cores (gfx950 MFMA).
//
// The reference has no such kernel: for M > 1 rows matmul_q runs M independent GEMVs
// (torch/io/gguf_model.h:7029-7036, :7056-7061), re-reading the weights M times.  Two families:
//   * exact kernels (below): the GEMV's arithmetic per output row, each weight tile read once per 64 rows of X;
//   * a fast kernel (second half of this file): fp16 MFMA on weights dequantised in registers.
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

#include <mutex>

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

// =================================================================================================
// Fast path: fp16 MFMA on dequantised weights.
//   Activations: each row of X is rounded to the reference's Q8 values (d * q per block of 32, the rounding the
//   CPU GEMV applies) and stored as fp16, scaled by a power of two per row so that it cannot overflow.
//   Weights: dequantised in registers to their exact fp32 value, then rounded to fp16 (round toward zero, one
//   instruction per pair).  v_mfma_f32_32x32x16_f16 accumulates in fp32 over the whole K, so there is NO per-sub-
//   block epilogue: VALU work is the dequantisation only, and it is amortised over the 128 rows of X a workgroup
//   owns.  Result = reference GEMV up to fp16 rounding of the operands (relative 2^-12 per element).
//   Workgroup: 128 rows of X x 256 columns (wave w: columns 64w..64w+63 = two 32-wide MFMA tiles, all 128 rows =
//   four 32-high tiles; 8 accumulator tiles = 128 VGPRs).  A 128 x 32 fp16 tile of X per sub-block step is shared
//   through LDS (double-buffered); each wave dequantises only its own columns.
//   The summation index of the MFMA is free to permute: lane half kh takes the 16 CONSECUTIVE elements
//   [16 kh, 16 kh + 16) of a 32-wide sub-block (first 8 in k-step 0, next 8 in k-step 1), for A and B alike, so a
//   lane's weights of one sub-block come from one 16-byte load.
// =================================================================================================
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// LDS holds the fp16 X tile of a whole super-block step: 128 rows x 256 k, row pitch 528 B (16 consecutive lanes
// x 16 B then hit all 64 banks once), double-buffered: 2 x 66 KB of the CU's 160 KB.
enum { QF_TM = 128, QF_TN = 256, QF_PITCH = 528 };

__host__ __device__ inline int qf_mpad(int M) { return (M + QF_TM - 1) / QF_TM * QF_TM; }

// rows of X (bf16, or fp32 when XF32) -> fp16 rows Xh[Mpad][K] (Q8ROUND: first rounded to the reference's Q8 values d*q per block of
// 32, the rounding its Q4_K GEMV applies; otherwise the bf16 value itself, as its Q6_K GEMV uses), divided by a
// power of two per row (returned in rowscale) so that fp16 cannot overflow
template <bool XF32>
__device__ __forceinline__ float4 load_x4(const void* row, int i) {
    if constexpr (XF32) {
        return reinterpret_cast<const float4*>(row)[i];
    } else {
        const uint2 raw = reinterpret_cast<const uint2*>(row)[i];
        return make_float4(bf16_to_f32(raw.x & 0xffffu), bf16_to_f32(raw.x >> 16), bf16_to_f32(raw.y & 0xffffu),
                           bf16_to_f32(raw.y >> 16));
    }
}

template <bool Q8ROUND, bool XF32>
__global__ __launch_bounds__(256) void qgemm_prepare_rows_f16_kernel(const void* __restrict__ X, _Float16* __restrict__ Xh,
                                                                     float* __restrict__ rowscale, int M, int K) {
    __shared__ float red[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    const int n4 = K / 4;
    _Float16* dst = Xh + (int64_t)m * K;
    if (m >= M) {  // padding rows: zeros
        for (int i = tid; i < n4; i += 256) reinterpret_cast<uint2*>(dst)[i] = make_uint2(0, 0);
        return;
    }
    const void* src = static_cast<const uint8_t*>(X) + (int64_t)m * K * (XF32 ? 4 : 2);
    float amax = 0.0f;
    for (int i = tid; i < n4; i += 256) {
        const float4 v = load_x4<XF32>(src, i);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    amax = max64(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // power of two that brings the row below 2^14 (fp16 tops out at 65504); 1 for ordinary activations
    int e = 0;
    if (amax > 16384.0f) { (void)frexpf(amax, &e); e -= 14; }
    const float down = ldexpf(1.0f, -e);
    if (tid == 0) rowscale[m] = ldexpf(1.0f, e);
    for (int i = tid; i < n4; i += 256) {  // K % 256 == 0: whole waves, aligned groups of 8 lanes = one Q8 block
        float4 v = load_x4<XF32>(src, i);
        if constexpr (Q8ROUND) {
            float d, sm;
            const uint32_t pk = q8_quantize4(v, d, sm);
            v.x = d * (float)(int)(int8_t)(pk & 0xff);
            v.y = d * (float)(int)(int8_t)((pk >> 8) & 0xff);
            v.z = d * (float)(int)(int8_t)((pk >> 16) & 0xff);
            v.w = d * (float)(int)(int8_t)(pk >> 24);
        }
        union { _Float16 h[4]; uint2 u; } o;
        o.h[0] = (_Float16)(v.x * down);  // power-of-two scaling: exact
        o.h[1] = (_Float16)(v.y * down);
        o.h[2] = (_Float16)(v.z * down);
        o.h[3] = (_Float16)(v.w * down);
        reinterpret_cast<uint2*>(dst)[i] = o.u;
    }
}

// The same conversion fused with what precedes a projection in the prompt pass, so that the fp32 intermediate is never
// written: PRE 1 = RMSNorm of the row (x * rs * (gamma + add_one), the arithmetic and reduction order of
// rms_norm_kernel), PRE 2 = SiLU(gate) * up (the arithmetic of silu_mul_kernel), or tanh-GELU(gate) * up (that of
// gelu_mul_kernel) when add_one, which has no other meaning for PRE 2, is set.  Writes the Q8-rounded form (for Q4_K
// matrices) and / or the plain form (for Q6_K matrices) in one pass; either output may be NULL.
// THREADS: 256, or 1024 for PRE 2 on short prompts (one workgroup per row: with few rows the launch lasts as long as one
// row's dependent chain, which four times the threads shorten; the row maximum does not depend on the thread count).
template <int PRE, int THREADS = 256>
__global__ __launch_bounds__(THREADS) void qgemm_prepare_fused_kernel(const float* __restrict__ X, const float* __restrict__ X2,
                                                                  float eps, int add_one, _Float16* __restrict__ Xh_round,
                                                                  float* __restrict__ rs_round, _Float16* __restrict__ Xh_plain,
                                                                  float* __restrict__ rs_plain, int M, int K) {
    static_assert(PRE == 2 || THREADS == 256, "the RMSNorm sum keeps the 256-thread reduction order");
    __shared__ float red[4];
    __shared__ float red2[THREADS / 64];
    const int m = blockIdx.x, tid = threadIdx.x;
    const int n4 = K / 4;
    if (m >= M) {  // padding rows: zeros
        for (int i = tid; i < n4; i += THREADS) {
            if (Xh_round) reinterpret_cast<uint2*>(Xh_round + (int64_t)m * K)[i] = make_uint2(0, 0);
            if (Xh_plain) reinterpret_cast<uint2*>(Xh_plain + (int64_t)m * K)[i] = make_uint2(0, 0);
        }
        return;
    }
    const float* x = X + (int64_t)m * K;
    const float* x2 = PRE == 2 ? X2 + (int64_t)m * K : X2;
    float rs = 1.0f;
    const float one = add_one ? 1.0f : 0.0f;
    if constexpr (PRE == 1) {
        float ss = 0.0f;
        for (int i = tid; i < K; i += THREADS) ss = fmaf(x[i], x[i], ss);
        ss = block_sum256(ss, red);
        rs = 1.0f / sqrtf(ss / (float)K + eps);
    }
    auto value4 = [&](int i) {
        const float4 a = reinterpret_cast<const float4*>(x)[i], b = reinterpret_cast<const float4*>(x2)[i];
        float4 r;
        if constexpr (PRE == 1) {
            r.x = a.x * rs * (b.x + one); r.y = a.y * rs * (b.y + one); r.z = a.z * rs * (b.z + one); r.w = a.w * rs * (b.w + one);
        } else {
            const bool gelu = add_one != 0;
            auto silu_mul = [gelu](float g, float u) {
                if (gelu) {
                    const float x3 = g * g * g;
                    const float t = tanhf(0.7978845608028654f * (g + 0.044715f * x3));
                    return 0.5f * g * (1.0f + t) * u;
                }
                float ng = 0.0f - g;
                ng = fminf(fmaxf(ng, -88.0f), 88.0f);
                return (g * (1.0f / (1.0f + expf(ng)))) * u;
            };
            r.x = silu_mul(a.x, b.x); r.y = silu_mul(a.y, b.y); r.z = silu_mul(a.z, b.z); r.w = silu_mul(a.w, b.w);
        }
        return r;
    };
    // Rows of up to 16384 values are computed once and kept in registers between the maximum and the store pass: all of a
    // thread's loads go out together, and the exponentials of PRE 2 are paid once (the pass is otherwise two dependent
    // sweeps over 2 x 4 K bytes per row).
    constexpr int HOLD = 4096 / THREADS;
    const bool held = n4 <= HOLD * THREADS;
    float4 hv[HOLD];
    float amax = 0.0f;
    if (held) {
#pragma unroll
        for (int u = 0; u < HOLD; ++u) {
            const int i = tid + THREADS * u;
            hv[u] = i < n4 ? value4(i) : make_float4(0.f, 0.f, 0.f, 0.f);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(hv[u].x), fabsf(hv[u].y)), fmaxf(fabsf(hv[u].z), fabsf(hv[u].w))));
        }
    } else {
        for (int i = tid; i < n4; i += THREADS) {
            const float4 v = value4(i);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    amax = max64(amax);
    if ((tid & 63) == 0) red2[tid >> 6] = amax;
    __syncthreads();
    {
        float t = red2[0];
#pragma unroll
        for (int w = 1; w < THREADS / 64; ++w) t = fmaxf(t, red2[w]);
        amax = t;
    }
    int e = 0;
    if (amax > 16384.0f) { (void)frexpf(amax, &e); e -= 14; }
    const float down = ldexpf(1.0f, -e);
    if (tid == 0) {
        if (rs_round) rs_round[m] = ldexpf(1.0f, e);
        if (rs_plain) rs_plain[m] = ldexpf(1.0f, e);
    }
    auto store4 = [&](_Float16* dst, int i, float4 v) {
        union { _Float16 h[4]; uint2 u; } o;
        o.h[0] = (_Float16)(v.x * down);
        o.h[1] = (_Float16)(v.y * down);
        o.h[2] = (_Float16)(v.z * down);
        o.h[3] = (_Float16)(v.w * down);
        reinterpret_cast<uint2*>(dst)[i] = o.u;
    };
    auto emit4 = [&](int i, float4 v) {  // K % 256 == 0: whole waves, aligned groups of 8 lanes = one Q8 block
        if (Xh_plain) store4(Xh_plain + (int64_t)m * K, i, v);
        if (Xh_round) {
            float d, sm;
            const uint32_t pk = q8_quantize4(v, d, sm);
            float4 q;
            q.x = d * (float)(int)(int8_t)(pk & 0xff);
            q.y = d * (float)(int)(int8_t)((pk >> 8) & 0xff);
            q.z = d * (float)(int)(int8_t)((pk >> 16) & 0xff);
            q.w = d * (float)(int)(int8_t)(pk >> 24);
            store4(Xh_round + (int64_t)m * K, i, q);
        }
    };
    if (held) {
#pragma unroll
        for (int u = 0; u < HOLD; ++u) {
            const int i = tid + THREADS * u;
            if (i < n4) emit4(i, hv[u]);  // wave-uniform: n4 is a multiple of 64
        }
    } else {
        for (int i = tid; i < n4; i += THREADS) emit4(i, value4(i));
    }
}

// The K-split partial sums of a projection into the residual stream, folded into the conversion that follows it:
// X[m] (+)= P[0][m] + P[1][m] + ... (the order of qgemm_split_reduce_kernel), then RMSNorm of the new row and its fp16
// forms as qgemm_prepare_fused_kernel<1> produces them (same arithmetic, same reduction order: the row is staged in LDS
// and walked with that kernel's two lane mappings).  One launch and one pass over the row instead of a reduction launch
// and three sweeps of the conversion.
template <int B>  // partial sums fetched per batch
__global__ __launch_bounds__(256) void qgemm_reduce_norm_prepare_kernel(const float* __restrict__ P, int splits, float* __restrict__ X,
                                                                        int accumulate, const float* __restrict__ gamma, float eps,
                                                                        int add_one, _Float16* __restrict__ Xh_round,
                                                                        float* __restrict__ rs_round, _Float16* __restrict__ Xh_plain,
                                                                        float* __restrict__ rs_plain, int M, int K) {
    extern __shared__ __align__(16) float rn_row[];  // K floats
    __shared__ float red[4];
    __shared__ float red2[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    const int n4 = K / 4;
    if (m >= M) {  // padding rows: zeros
        for (int i = tid; i < n4; i += 256) {
            if (Xh_round) reinterpret_cast<uint2*>(Xh_round + (int64_t)m * K)[i] = make_uint2(0, 0);
            if (Xh_plain) reinterpret_cast<uint2*>(Xh_plain + (int64_t)m * K)[i] = make_uint2(0, 0);
        }
        return;
    }
    const int64_t total = (int64_t)M * K;
    float4* x4 = reinterpret_cast<float4*>(X + (int64_t)m * K);
    for (int i = tid; i < n4; i += 256) {
        // B partial sums per batch, fetched unconditionally (the index clamped) so that they are in flight together; B = 4
        // where there are at most four slabs (half the clamped re-reads of the last one)
        const float4 o = accumulate ? x4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int z0 = 0; z0 < splits; z0 += B) {
            float4 b[B];
#pragma unroll
            for (int u = 0; u < B; ++u) b[u] = reinterpret_cast<const float4*>(P + min(z0 + u, splits - 1) * total + (int64_t)m * K)[i];
#pragma unroll
            for (int u = 0; u < B; ++u) {
                if (z0 + u == 0) a = b[u];
                else if (z0 + u < splits) { a.x += b[u].x; a.y += b[u].y; a.z += b[u].z; a.w += b[u].w; }
            }
        }
        if (accumulate) { a.x += o.x; a.y += o.y; a.z += o.z; a.w += o.w; }
        x4[i] = a;
        reinterpret_cast<float4*>(rn_row)[i] = a;
    }
    __syncthreads();
    float ss = 0.0f;
    for (int i = tid; i < K; i += 256) ss = fmaf(rn_row[i], rn_row[i], ss);
    ss = block_sum256(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)K + eps);
    const float one = add_one ? 1.0f : 0.0f;
    auto value4 = [&](int i) {
        const float4 a = reinterpret_cast<const float4*>(rn_row)[i], b = reinterpret_cast<const float4*>(gamma)[i];
        float4 r;
        r.x = a.x * rs * (b.x + one); r.y = a.y * rs * (b.y + one); r.z = a.z * rs * (b.z + one); r.w = a.w * rs * (b.w + one);
        return r;
    };
    float amax = 0.0f;
    for (int i = tid; i < n4; i += 256) {
        const float4 v = value4(i);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    amax = max64(amax);
    if ((tid & 63) == 0) red2[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red2[0], red2[1]), fmaxf(red2[2], red2[3]));
    int e = 0;
    if (amax > 16384.0f) { (void)frexpf(amax, &e); e -= 14; }
    const float down = ldexpf(1.0f, -e);
    if (tid == 0) {
        if (rs_round) rs_round[m] = ldexpf(1.0f, e);
        if (rs_plain) rs_plain[m] = ldexpf(1.0f, e);
    }
    auto store4 = [&](_Float16* dst, int i, float4 v) {
        union { _Float16 h[4]; uint2 u; } o;
        o.h[0] = (_Float16)(v.x * down);
        o.h[1] = (_Float16)(v.y * down);
        o.h[2] = (_Float16)(v.z * down);
        o.h[3] = (_Float16)(v.w * down);
        reinterpret_cast<uint2*>(dst)[i] = o.u;
    };
    for (int i = tid; i < n4; i += 256) {  // K % 256 == 0: whole waves, aligned groups of 8 lanes = one Q8 block
        const float4 v = value4(i);
        if (Xh_plain) store4(Xh_plain + (int64_t)m * K, i, v);
        if (Xh_round) {
            float d, sm;
            const uint32_t pk = q8_quantize4(v, d, sm);
            float4 q;
            q.x = d * (float)(int)(int8_t)(pk & 0xff);
            q.y = d * (float)(int)(int8_t)((pk >> 8) & 0xff);
            q.z = d * (float)(int)(int8_t)((pk >> 16) & 0xff);
            q.w = d * (float)(int)(int8_t)(pk >> 24);
            store4(Xh_round + (int64_t)m * K, i, q);
        }
    }
}

// 16 small integers (4 dwords of bytes, each < 1024) -> two fragments of 8 fp16 holding (byte - bias) * scale + offset.
// A byte b becomes the fp16 number 1024 + b by writing it under the exponent byte 0x64 (one v_perm per pair); the
// subtraction of 1024 + bias is exact, and one packed fp16 FMA applies scale and offset: 2.5 instructions per pair.
__device__ __forceinline__ void bytes_to_frags(const uint32_t (&b)[4], float bias, float scale, float offset, h8& f0, h8& f1) {
    const h2 sub = {(_Float16)(1024.0f + bias), (_Float16)(1024.0f + bias)};
    const h2 sc = {(_Float16)scale, (_Float16)scale};
    const h2 of = {(_Float16)offset, (_Float16)offset};
    uint32_t o[8];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const uint32_t hq = __builtin_amdgcn_perm(0x64646464u, b[w], p ? 0x04030402u : 0x04010400u);
            h2 q;
            __builtin_memcpy(&q, &hq, 4);
            const h2 v = __builtin_elementwise_fma(q - sub, sc, of);
            __builtin_memcpy(&o[2 * w + p], &v, 4);
        }
    }
    __builtin_memcpy(&f0, &o[0], 16);
    __builtin_memcpy(&f1, &o[4], 16);
}

__device__ __forceinline__ void pin4(uint4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }

// ---- per-type weight access: what a lane (column n, element half kh) fetches of a 256-wide super-block ----
struct Q4Tile {  // Q4_K: header + the lane's 16 bytes of each of the 4 groups of 64
    uint4 hdr;
    uint4 qs[4];
    __device__ __forceinline__ void load(const uint8_t* blk, int kh) {
        hdr = *reinterpret_cast<const uint4*>(blk);
#pragma unroll
        for (int g = 0; g < 4; ++g) qs[g] = *reinterpret_cast<const uint4*>(blk + 16 + 32 * g + 16 * kh);
    }
    // sub-block s (0..7) of the block -> two fragments
    __device__ __forceinline__ void frags(int s, int /*kh*/, h8& f0, h8& f1) const {
        int sc, mn;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, s, sc, mn);
        const float dsc = h2f(hdr.x) * (float)sc, dmn = h2f(hdr.x >> 16) * (float)mn;
        const uint4 r = qs[s >> 1];
        const int sh = 4 * (s & 1);
        const uint32_t b[4] = {(r.x >> sh) & 0x0f0f0f0fu, (r.y >> sh) & 0x0f0f0f0fu, (r.z >> sh) & 0x0f0f0f0fu,
                               (r.w >> sh) & 0x0f0f0f0fu};
        bytes_to_frags(b, 0.0f, dsc, -dmn, f0, f1);  // (d*sc)*q - dmin*m, the dequantised value (gguf_dequant.h:304-341)
    }
    // Nothing computed from these registers may be scheduled above this point: without it the scheduler fills the vector
    // slots behind the first MFMAs of a block with the scale arithmetic of the block that was requested an instant
    // before, and every block starts with a wait for its successor's weights.
    __device__ __forceinline__ void pin() {
        pin4(hdr);
#pragma unroll
        for (int g = 0; g < 4; ++g) pin4(qs[g]);
    }
    static constexpr int kBlockBytes = 144;
    static constexpr bool kQ8Round = true;
};
struct Q6Tile {  // Q6_K: the lane's 16 bytes of ql for each (half, pair), of qh for each half, scales, d
    uint4 ql[4], qh[2], sc;
    uint32_t d;
    __device__ __forceinline__ void load(const uint8_t* blk, int kh) {
#pragma unroll
        for (int c = 0; c < 4; ++c) ql[c] = ld16_a2(blk + 64 * (c >> 1) + 32 * (c & 1) + 16 * kh);
#pragma unroll
        for (int h = 0; h < 2; ++h) qh[h] = ld16_a2(blk + 128 + 32 * h + 16 * kh);
        sc = ld16_a2(blk + 192);
        d = reinterpret_cast<const u16_a2*>(blk + 208)->v;
    }
    // step s (0..7): elements 32 s + 16 kh + (0..15) = half s/4, group gq = s%4, one scale (index 2 s + kh)
    __device__ __forceinline__ void frags(int s, int kh, h8& f0, h8& f1) const {
        const int half = s >> 2, gq = s & 3;
        const uint4 l = ql[2 * half + (gq & 1)], hq = qh[half];
        const int lsh = 4 * (gq >> 1), hsh = 2 * gq;
        const uint32_t lw[4] = {l.x, l.y, l.z, l.w}, hw[4] = {hq.x, hq.y, hq.z, hq.w};
        uint32_t b[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) b[w] = ((lw[w] >> lsh) & 0x0f0f0f0fu) | ((((hw[w] >> hsh) & 0x03030303u)) << 4);
        const uint32_t scw[4] = {sc.x, sc.y, sc.z, sc.w};
        const uint32_t pair = scw[s >> 1] >> (16 * (s & 1));            // scales 2s and 2s+1
        const int sv = (int)(int8_t)((kh ? pair >> 8 : pair) & 0xffu);
        bytes_to_frags(b, 32.0f, h2f(d) * (float)sv, 0.0f, f0, f1);     // d*scale*(q-32) (gguf_dequant.h:395-430)
    }
    __device__ __forceinline__ void pin() {
#pragma unroll
        for (int c = 0; c < 4; ++c) pin4(ql[c]);
        pin4(qh[0]); pin4(qh[1]); pin4(sc);
        asm volatile("" : "+v"(d));
    }
    static constexpr int kBlockBytes = 210;
    static constexpr bool kQ8Round = false;
};

// X tile of a super-block step in LDS.  The pieces a thread owns of the NEXT block's tile are fetched during the first
// steps of the current block, followed by the next block's weights, and written to the other LDS buffer during the
// later steps, so the block ends with the next tile complete behind the only workgroup barrier of the block.  (After the
// last block the same code re-fetches the last tile into the idle buffer: no conditionals in the steady-state loop.)
// WAVES = 8 (what is launched, for every tile height): waves w and w + 4 own one 32-column strip each of the same 64
// columns and all MT row tiles, so a SIMD holds two waves and one's dequantisation and LDS reads run under the other's
// MFMAs (the two pipes of a single wave barely overlap); no weight is dequantised twice, the X tile in LDS is read by twice
// as many waves.  WAVES = 4 (a wave owns both strips) is the layout this grew from: slower at every height.
// (bx, by, bz) = (column tile, row tile, K split) of this workgroup; s_a = its dynamic LDS
template <typename Tile, int MT, int WAVES>
__device__ __forceinline__ void qgemm_f16_body(const uint8_t* W, int64_t stride, const _Float16* Xh,
                                               const float* __restrict__ rowscale, float* Y, int M, int K, int N,
                                               int accumulate, int blocks_per_split, float* partials, int bx, int by, int bz,
                                               uint8_t* s_a) {
    // W and Xh are deliberately not __restrict__: loads through a restrict pointer may be moved across the
    // compiler fences below, and the prefetch distance of this loop depends on those fences
    constexpr int TM = 32 * MT;                     // rows of X per workgroup (MT tiles of 32)
    constexpr int NT = 2 / (WAVES / 4);             // 32-column tiles per wave
    constexpr int RS = 2 * WAVES;                   // rows of the X tile that one fetch instruction of the workgroup covers
    constexpr int NPIECE = TM / RS;                 // 16-byte pieces of the X tile per thread
    static_assert(WAVES == 4 || (WAVES == 8 && (MT == 4 || MT == 2 || MT == 1)), "wave layouts");
    static_assert(NPIECE == 2 || NPIECE == 4 || NPIECE == 8 || NPIECE == 16, "pieces per thread");
    const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3;  // s_a: [2][TM * QF_PITCH]
    const int j = lane & 31, kh = lane >> 5;
    const int m0 = by * TM;
    const int n_base = bx * QF_TN + wave * 64 + (WAVES == 8 ? 32 * (tid >> 8) : 0);
    // split K: workgroup z of the grid sums super-blocks [blk0, blk0 + nblk) into its own M x N partial
    const int blk0 = bz * blocks_per_split;
    const int nblk = min(K / 256 - blk0, blocks_per_split);
    const uint8_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
        wrow[t] = W + (int64_t)min(n_base + 32 * t + j, N - 1) * stride + (int64_t)blk0 * Tile::kBlockBytes;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][t][r] = 0.0f;

    // X tile of a block = 128 rows x 512 B = 4096 pieces of 16 B; piece q = 256 i + tid (i = 0..15) is row q / 32, bytes
    // 16 (q % 32): a wave fetches two whole rows per instruction and writes LDS without bank conflicts
    const int64_t x_row_bytes = (int64_t)K * 2;
    const uint8_t* x_src = reinterpret_cast<const uint8_t*>(Xh) + (int64_t)(m0 + (tid >> 5)) * x_row_bytes + 16 * (tid & 31) +
                           (int64_t)blk0 * 512;
    uint8_t* x_dst = s_a + (tid >> 5) * QF_PITCH + 16 * (tid & 31);
    float* s_rs = reinterpret_cast<float*>(s_a + 2 * TM * QF_PITCH);  // the tile's TM row scales (every padded row has one)
    if (tid < TM) s_rs[tid] = rowscale[m0 + tid];
    // the 16 pieces of the next tile in flight (scalars, not an array: they must stay in registers)
    static_assert(MT == 1 || MT == 2 || MT == 4, "row tiles per workgroup");
    uint4 x0, x1, x2, x3, x4, x5, x6, x7, x8, x9, x10, x11, x12, x13, x14, x15;
    // prologue: tile of block 0 -> LDS buffer 0, weights of block 0, fragments of step 0.  The weight loads go out behind
    // the tile's, before anything waits: one memory round trip for both, not two (a launch of two or three blocks per
    // workgroup, as the K splits of the narrow projections are, is mostly this prologue)
#define QF_LD0(p) (*reinterpret_cast<const uint4*>(x_src + RS * (p) * x_row_bytes))
#define QF_ST0(p, v) (*reinterpret_cast<uint4*>(x_dst + RS * (p) * QF_PITCH) = (v))
    x0 = QF_LD0(0); x1 = QF_LD0(1);
    if constexpr (NPIECE >= 4) { x2 = QF_LD0(2); x3 = QF_LD0(3); }
    if constexpr (NPIECE >= 8) { x4 = QF_LD0(4); x5 = QF_LD0(5); x6 = QF_LD0(6); x7 = QF_LD0(7); }
    if constexpr (NPIECE >= 16) {
        x8 = QF_LD0(8); x9 = QF_LD0(9); x10 = QF_LD0(10); x11 = QF_LD0(11); x12 = QF_LD0(12);
        x13 = QF_LD0(13); x14 = QF_LD0(14); x15 = QF_LD0(15);
    }
    issue_order_fence();
    Tile cur[NT], nxt[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) cur[t].load(wrow[t], kh);
    issue_order_fence();
    QF_ST0(0, x0); QF_ST0(1, x1);
    if constexpr (NPIECE >= 4) { QF_ST0(2, x2); QF_ST0(3, x3); }
    if constexpr (NPIECE >= 8) { QF_ST0(4, x4); QF_ST0(5, x5); QF_ST0(6, x6); QF_ST0(7, x7); }
    if constexpr (NPIECE >= 16) {
        QF_ST0(8, x8); QF_ST0(9, x9); QF_ST0(10, x10); QF_ST0(11, x11); QF_ST0(12, x12);
        QF_ST0(13, x13); QF_ST0(14, x14); QF_ST0(15, x15);
    }
#undef QF_LD0
#undef QF_ST0
    h8 bf[NT][2], bn[NT][2];
#pragma unroll
    for (int t = 0; t < NT; ++t) cur[t].frags(0, kh, bf[t][0], bf[t][1]);
    __syncthreads();

    for (int blk = 0; blk < nblk; ++blk) {
        const int nb = min(blk + 1, nblk - 1);  // block whose tile and weights are fetched during this one
        const uint8_t* a_cur = s_a + (blk & 1) * (TM * QF_PITCH);
        uint8_t* x_nxt = x_dst + ((blk & 1) ^ 1) * (TM * QF_PITCH);
        const uint8_t* x_from = x_src + (int64_t)nb * 512;
        h8 af[2][MT];  // X fragments of step 0 of this block (the tile became visible at the barrier)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                af[ks][mt] = *reinterpret_cast<const h8*>(a_cur + (mt * 32 + j) * QF_PITCH + 32 * kh + 16 * ks);
#pragma unroll
        for (int s = 0; s < 8; ++s) {  // unrolled: the sub-block index selects registers
#define QF_LD(p) (*reinterpret_cast<const uint4*>(x_from + RS * (p) * x_row_bytes))
#define QF_ST(p, v) (*reinterpret_cast<uint4*>(x_nxt + RS * (p) * QF_PITCH) = (v))
            // For the 128-row tile the fetches of the next block are spread over steps 0..3 and the LDS stores of the tile pieces
            // over steps 4..7: issued in one burst at step 0 they held up the vector-memory path for everything behind them
            // (512 x 4096 x 14336: 75.6 -> 72.1 us; a 2048-token prompt 26.3 -> 25.6 ms; prompts of up to 64 rows were 2 % slower
            // with their few pieces spread, so the small tiles keep the burst).  Tile pieces go FIRST and the weights last (step 3):
            // loads return in order, so a wait for a piece must not have the weight loads (HBM latency, one cache line per
            // lane) in front of it; the weights are first needed at step 7.
#define QF_W() _Pragma("unroll") for (int t = 0; t < NT; ++t) nxt[t].load(wrow[t] + (int64_t)nb * Tile::kBlockBytes, kh)
            if constexpr (NPIECE == 8) {
                if (s == 0) { x0 = QF_LD(0); x1 = QF_LD(1); }
                if (s == 1) { x2 = QF_LD(2); x3 = QF_LD(3); }
                if (s == 2) { x4 = QF_LD(4); x5 = QF_LD(5); }
                if (s == 3) { x6 = QF_LD(6); x7 = QF_LD(7); issue_order_fence(); QF_W(); }
                if (s == 4) { QF_ST(0, x0); QF_ST(1, x1); }
                if (s == 5) { QF_ST(2, x2); QF_ST(3, x3); }
                if (s == 6) { QF_ST(4, x4); QF_ST(5, x5); }
                if (s == 7) { QF_ST(6, x6); QF_ST(7, x7); }
            } else if constexpr (NPIECE <= 4) {  // the 64- and 32-row tiles: one burst and one step of stores measured faster there
                if (s == 0) {
                    x0 = QF_LD(0); x1 = QF_LD(1);
                    if constexpr (NPIECE == 4) { x2 = QF_LD(2); x3 = QF_LD(3); }
                    issue_order_fence();
                    QF_W();
                }
                if (s == 3) {
                    QF_ST(0, x0); QF_ST(1, x1);
                    if constexpr (NPIECE == 4) { QF_ST(2, x2); QF_ST(3, x3); }
                }
            } else {  // 16 pieces (the four-wave 128-row layout): one burst at step 0, stores in steps 3..6
                if (s == 0) {
                    x0 = QF_LD(0); x1 = QF_LD(1); x2 = QF_LD(2); x3 = QF_LD(3); x4 = QF_LD(4); x5 = QF_LD(5); x6 = QF_LD(6); x7 = QF_LD(7);
                    x8 = QF_LD(8); x9 = QF_LD(9); x10 = QF_LD(10); x11 = QF_LD(11); x12 = QF_LD(12);
                    x13 = QF_LD(13); x14 = QF_LD(14); x15 = QF_LD(15);
                    issue_order_fence();
                    QF_W();
                }
                if (s == 3) { QF_ST(0, x0); QF_ST(1, x1); QF_ST(2, x2); QF_ST(3, x3); }
                if (s == 4) { QF_ST(4, x4); QF_ST(5, x5); QF_ST(6, x6); QF_ST(7, x7); }
                if (s == 5) { QF_ST(8, x8); QF_ST(9, x9); QF_ST(10, x10); QF_ST(11, x11); }
                if (s == 6) { QF_ST(12, x12); QF_ST(13, x13); QF_ST(14, x14); QF_ST(15, x15); }
            }
#undef QF_W
#undef QF_LD
#undef QF_ST
            issue_order_fence();  // the fetches stay HERE, two steps ahead of their use (the compiler would sink them to it)
            // This step's X fragments were read from LDS during the previous step; nothing that consumes them may be hoisted
            // above this point.  (An MFMA is no memory operation: without this the scheduler moves each MFMA up to right
            // behind the LDS read of its operand, the fragments share ONE register quad, and every MFMA waits out the
            // LDS latency of its own operand.)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(af[ks][mt]));
            // X fragments of the NEXT step are read from LDS now and weight fragments of the next step are prepared
            // while this step's 16 MFMAs (all operands already in registers) run
            h8 an[2][MT];
            if (s < 7) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        an[ks][mt] = *reinterpret_cast<const h8*>(a_cur + (mt * 32 + j) * QF_PITCH + 64 * (s + 1) + 32 * kh + 16 * ks);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (s < 7) cur[t].frags(s + 1, kh, bn[t][0], bn[t][1]);
                else { nxt[t].pin(); nxt[t].frags(0, kh, bn[t][0], bn[t][1]); }
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                        acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[ks][mt], bf[t][ks], acc[mt][t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NT; ++t) { bf[t][0] = bn[t][0]; bf[t][1] = bn[t][1]; }
            if (s < 7) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) af[ks][mt] = an[ks][mt];
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) cur[t] = nxt[t];
        __syncthreads();  // next tile complete, this tile no longer read
    }
    // C layout of the 32x32 tile: column j = lane % 32, rows 8 (r / 4) + 4 (lane / 32) + r % 4.  The row scales come from
    // LDS (staged in the prologue), and when accumulating the 16 old values of a tile are fetched together before its 16
    // stores: a load issued behind a store the compiler cannot tell apart from it is one serial memory round trip per value,
    // more than the main loop of a launch with few blocks per workgroup takes.
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int n = n_base + 32 * t + j;
        const bool n_ok = n < N;
        const int nc = n_ok ? n : N - 1;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float old[16];
            if (!partials && accumulate) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = min(m0 + mt * 32 + 8 * (r >> 2) + 4 * kh + (r & 3), M - 1);
                    old[r] = Y[(int64_t)m * N + nc];
                }
                issue_order_fence();
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) old[r] = 0.0f;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int lr = mt * 32 + 8 * (r >> 2) + 4 * kh + (r & 3);
                const int m = m0 + lr;
                const float v = acc[mt][t][r] * s_rs[lr];
                if (m < M && n_ok) {
                    if (partials) __builtin_nontemporal_store(v, &partials[((int64_t)bz * M + m) * N + n]);
                    else __builtin_nontemporal_store(accumulate ? old[r] + v : v, &Y[(int64_t)m * N + n]);
                }
            }
        }
    }
}

// Which tile a workgroup takes.  The hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each with its own
// L2; taken as they come, the workgroups of one XCD are scattered over all column tiles, row tiles and K splits and share
// almost nothing (the down projection of a 512-row prompt, 10 x 4 tiles x 6 splits, then pulls 200 MB through the L2s for
// 30 MB of operands).  Here the workgroups an XCD receives form one contiguous run of the order "row tile fastest, then
// column tile (or slot) within a band of 4 row tiles, then band, then K split": the 32 or so workgroups an XCD runs at a time
// are then about 4 row tiles x 8 column tiles, so each weight piece serves 4 of them and each X tile 8 from one L2.
__device__ __forceinline__ int qf_xcd_order(int hw, int nwg) {
    const int xcd = hw & 7, slot = hw >> 3, per = nwg >> 3, rem = nwg & 7;
    return xcd * per + (xcd < rem ? xcd : rem) + slot;
}
// position L of that order -> (column tile or slot, row tile, K split) on a gx x gy x gz grid
__device__ __forceinline__ void qf_tile_of(int L, int gx, int gy, int& bx, int& by, int& bz) {
    const int plane = gx * gy;
    bz = L / plane;
    const int r = L - bz * plane;
    const int band = r / (4 * gx);
    const int rows = min(4, gy - 4 * band);
    const int within = r - band * 4 * gx;
    by = 4 * band + within % rows;
    bx = within / rows;
}

template <typename Tile, int MT, int WAVES = 4>
__global__ __launch_bounds__(64 * WAVES, (WAVES == 8 ? 1 : (MT <= 2 ? 2 : 1))) void qgemm_f16_kernel(const uint8_t* W, int64_t stride, const _Float16* Xh,
                                                        const float* __restrict__ rowscale, float* Y, int M, int K, int N,
                                                        int accumulate, int blocks_per_split, float* partials) {
    extern __shared__ __align__(16) uint8_t qf_lds[];
    const int hw = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int L = qf_xcd_order(hw, gridDim.x * gridDim.y * gridDim.z);
    int bx, by, bz;
    qf_tile_of(L, gridDim.x, gridDim.y, bx, by, bz);
    qgemm_f16_body<Tile, MT, WAVES>(W, stride, Xh, rowscale, Y, M, K, N, accumulate, blocks_per_split, partials, bx, by, bz, qf_lds);
}

// Up to three projections of the same rows in ONE launch of the eight-wave 128-row tile (q, k, v of a layer: in a Q4_K_M
// file two Q4_K matrices and a Q6_K one).  Each matrix brings its own prepared rows (Q8-rounded for Q4_K, plain for
// Q6_K), column tiles and K splits; blockIdx.x walks the (column tile, split) slots of the matrices one after the other.
// Three narrow launches of two or three blocks per workgroup are mostly launch, prologue and epilogue; one launch pays
// them once and fills the chip.
struct QfMat {
    const uint8_t* W;
    int64_t stride;
    const _Float16* Xh;
    const float* rowscale;
    float* Y;
    float* partials;  // NULL: one split, written to Y
    int N, bps, ntiles, slot_end, q6;
};
struct QfMulti { QfMat m[3]; int n_mat; };

template <int MT, int WAVES>
__global__ __launch_bounds__(64 * WAVES, (WAVES == 8 ? 1 : 2)) void qgemm_f16_multi_kernel(const QfMulti a, int M, int K) {
    extern __shared__ __align__(16) uint8_t qf_lds[];
    const int L = qf_xcd_order(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x * gridDim.y);
    int sx, by, unused;
    qf_tile_of(L, gridDim.x, gridDim.y, sx, by, unused);  // sx: the (matrix, split, column tile) slot
    int i = 0;
    if (a.n_mat > 1 && sx >= a.m[0].slot_end) i = 1;
    if (a.n_mat > 2 && sx >= a.m[1].slot_end) i = 2;
    const QfMat& q = i == 0 ? a.m[0] : (i == 1 ? a.m[1] : a.m[2]);
    const int local = sx - (i == 0 ? 0 : (i == 1 ? a.m[0].slot_end : a.m[1].slot_end));
    const int bx = local % q.ntiles, bz = local / q.ntiles;
    if (q.q6) qgemm_f16_body<Q6Tile, MT, WAVES>(q.W, q.stride, q.Xh, q.rowscale, q.Y, M, K, q.N, 0, q.bps, q.partials, bx, by, bz, qf_lds);
    else qgemm_f16_body<Q4Tile, MT, WAVES>(q.W, q.stride, q.Xh, q.rowscale, q.Y, M, K, q.N, 0, q.bps, q.partials, bx, by, bz, qf_lds);
}

// Y (+)= partials[0] + partials[1] + ... in that fixed order (deterministic, unlike atomics)
__global__ __launch_bounds__(256) void qgemm_split_reduce_kernel(const float* __restrict__ P, int splits, float* __restrict__ Y,
                                                                 int64_t total, int accumulate) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    if (i + 4 <= total && (total & 3) == 0) {
        float4 a = *reinterpret_cast<const float4*>(P + i);
        for (int z = 1; z < splits; ++z) {
            const float4 b = *reinterpret_cast<const float4*>(P + z * total + i);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        float4* y = reinterpret_cast<float4*>(Y + i);
        if (accumulate) { const float4 o = *y; a.x += o.x; a.y += o.y; a.z += o.z; a.w += o.w; }
        *y = a;
    } else {
        for (int64_t e = i; e < total && e < i + 4; ++e) {
            float a = P[e];
            for (int z = 1; z < splits; ++z) a += P[z * total + e];
            Y[e] = accumulate ? Y[e] + a : a;
        }
    }
}

// the same for the matrices of a multi-matrix launch: blockIdx.x walks the segments' 1024-element pieces
struct QfRedSeg { const float* P; float* Y; int64_t total; int splits, blk_end; };
struct QfRedMulti { QfRedSeg s[3]; int n; };
__global__ __launch_bounds__(256) void qgemm_split_reduce_multi_kernel(const QfRedMulti a) {
    int k = 0;
    if (a.n > 1 && (int)blockIdx.x >= a.s[0].blk_end) k = 1;
    if (a.n > 2 && (int)blockIdx.x >= a.s[1].blk_end) k = 2;
    const QfRedSeg& g = k == 0 ? a.s[0] : (k == 1 ? a.s[1] : a.s[2]);
    const int b = (int)blockIdx.x - (k == 0 ? 0 : (k == 1 ? a.s[0].blk_end : a.s[1].blk_end));
    const int64_t i = ((int64_t)b * 256 + threadIdx.x) * 4;
    if (i >= g.total) return;
    if (i + 4 <= g.total && (g.total & 3) == 0) {
        float4 v = *reinterpret_cast<const float4*>(g.P + i);
        for (int z = 1; z < g.splits; ++z) {
            const float4 w = *reinterpret_cast<const float4*>(g.P + z * g.total + i);
            v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
        }
        *reinterpret_cast<float4*>(g.Y + i) = v;
    } else {
        for (int64_t e = i; e < g.total && e < i + 4; ++e) {
            float v = g.P[e];
            for (int z = 1; z < g.splits; ++z) v += g.P[z * g.total + e];
            g.Y[e] = v;
        }
    }
}

// Row classes of the split rules: up to 128 rows, up to 256, up to 1024, more (2048-row chunks of long prompts: with 16 row
// tiles per column tile, as many splits as a 512-row launch wants only multiply the partial sums).
static inline int qf_row_class(int M) { return M <= 128 ? 1 : (M <= 256 ? 2 : (M <= 1024 ? 4 : 8)); }

// K splits for an N x K weight matrix and M rows: enough workgroups to fill the chip when N alone gives few column
// tiles (a 2560-wide projection is 10 tiles).  M enters only through its class (up to 128 rows, up to 256, up to 1024, more), so
// that the summation order of a row does not change with how many rows share the launch within a class; short
// prompts (one row tile) get up to 16 splits, because there the launch is bound by how many workgroups stream weights.
int qgemm_f16_splits(int N, int K, int M) {
    const int ntiles = (N + QF_TN - 1) / QF_TN, nblk = K / 256;
    const int row_tiles = qf_row_class(M);
    int s = 256 / (ntiles * row_tiles);
    const int cap = row_tiles == 1 ? 16 : 8;
    s = s > cap ? cap : s;
    s = s > nblk / 2 ? nblk / 2 : s;
    return s < 1 ? 1 : s;
}

// K splits of the matrices of a multi-matrix launch.  All (column tile, split) slots of all matrices must fit one round of
// the chip (256 workgroups over the row tiles of M's class, as above), and the launch lasts as long as its slowest
// workgroup: starting from one split each, the matrix whose workgroups have the most work (blocks per split, a Q6_K block
// weighing 1.6 Q4_K blocks: measured 8 against 5 us) gets its next split count until the slots run out.  A function of
// the shapes, the types and M's class only, like qgemm_f16_splits.
void qgemm_f16_multi_plan(int n, const int* N, const uint32_t* types, int K, int M, int* splits) {
    const int nblk = K / 256;
    const int row_tiles = qf_row_class(M);
    const int budget = 256 / row_tiles;
    const int cap = (row_tiles == 1 ? 16 : 8) < nblk / 2 ? (row_tiles == 1 ? 16 : 8) : (nblk / 2 < 1 ? 1 : nblk / 2);
    int ntile[3], slots = 0;
    for (int i = 0; i < n; ++i) { splits[i] = 1; ntile[i] = (N[i] + QF_TN - 1) / QF_TN; slots += ntile[i]; }
    for (;;) {
        int j = -1;
        float worst = 0.0f;
        for (int i = 0; i < n; ++i) {
            const float est = (float)((nblk + splits[i] - 1) / splits[i]) * (types[i] == PTM_TYPE_Q6_K ? 1.6f : 1.0f);
            if (est > worst) { worst = est; j = i; }
        }
        if (j < 0) break;
        const int bps = (nblk + splits[j] - 1) / splits[j];
        if (bps <= 1) break;
        const int next = (nblk + bps - 2) / (bps - 1);  // the fewest splits with fewer blocks each
        if (next > cap || slots + ntile[j] * (next - splits[j]) > budget) break;
        slots += ntile[j] * (next - splits[j]);
        splits[j] = next;
    }
}

// Rows per workgroup in tiles of 32: 4 (128 rows: each dequantised weight serves twice as many products) unless that
// leaves most of the chip idle; then 2 (64 rows: twice the workgroups).  Prompts of up to 64 / 32 rows take the 64- / 32-row
// tile: a quarter of the X tile traffic, LDS reads and MFMAs per block.  A row's sum does not depend on the choice (same K
// order).  Threshold swept on the Qwen3-4B shapes: 128 workgroups, Q4_K only, is the best or tied at every prompt length.
static int qgemm_f16_row_tiles(bool q4, int M, int N, int splits) {
    if (M <= 32) return 1;
    if (M <= 64) return 2;
    const int wgs = ((N + QF_TN - 1) / QF_TN) * ((M + 127) / 128) * splits;
    return (q4 && wgs < 128) ? 2 : 4;  // 512 x 2560 x 9728 (152 workgroups): 60 us with 128 rows, 70 with 64; 512 x 4096 x 4096 (64): 80 / 68
}

static int qgemm_check(const void* W, const void* X, const void* Y, int M, int K, int N, int64_t stride, int blk_bytes) {
    if (!W || !X || !Y) return PTM_E_NULL;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (stride < (int64_t)(K / 256) * blk_bytes) return PTM_E_SHAPE;
    if (!aligned16(X) || (reinterpret_cast<uintptr_t>(Y) & 3u)) return PTM_E_ALIGN;
    if ((int64_t)qg_mpad(M) / QG_MCHUNK > 65535) return PTM_E_UNSUPPORTED;
    return PTM_OK;
}

// Y (+)= X . W^T with X bf16 or fp32 rows; shared by the C entry points and the prefill runtime.
int qgemm_f16_impl(uint32_t ggml_type, const void* W, const void* X, bool x_is_f32, float* Y, int M, int K, int N,
                   int64_t stride, void* workspace, bool accumulate, float* split_ws, size_t split_ws_bytes, bool reuse_rows,
                   hipStream_t s, int* deferred_splits) {
    // deferred_splits (optional): where K was split, the partial sums are left in split_ws for the caller's next kernel to
    // fold in (qgemm_f16_reduce_norm_prepare) and their count is returned here; 0 = Y is complete
    // reuse_rows: the workspace already holds these rows of X prepared by the previous call for a matrix of the
    // same type (same rounding rule), so the conversion pass is skipped
    if (ggml_type != PTM_TYPE_Q4_K && ggml_type != PTM_TYPE_Q6_K) return PTM_E_UNSUPPORTED;
    const int blk = ggml_type == PTM_TYPE_Q4_K ? 144 : 210;
    const int rc = qgemm_check(W, X, Y, M, K, N, stride, blk);
    if (rc != PTM_OK) return rc;
    if (!workspace) return PTM_E_NULL;
    if (!aligned16(workspace)) return PTM_E_ALIGN;
    if (ggml_type == PTM_TYPE_Q4_K ? (!aligned16(W) || (stride & 15)) : ((stride & 1) || (reinterpret_cast<uintptr_t>(W) & 1u)))
        return PTM_E_ALIGN;
    const int mp = qf_mpad(M);
    if (mp / 32 > 65535) return PTM_E_UNSUPPORTED;
    _Float16* Xh = static_cast<_Float16*>(workspace);
    float* rowscale = reinterpret_cast<float*>(Xh + (int64_t)mp * K);
    const int nblk = K / 256;
    int splits = split_ws ? qgemm_f16_splits(N, K, M) : 1;
    while (splits > 1 && (size_t)splits * M * N * sizeof(float) > split_ws_bytes) --splits;
    const int bps = (nblk + splits - 1) / splits;
    splits = (nblk + bps - 1) / bps;  // no empty split
    float* partials = splits > 1 ? split_ws : nullptr;
    const int acc = accumulate ? 1 : 0;
    const bool q4 = ggml_type == PTM_TYPE_Q4_K;
    if (!reuse_rows) {
        if (q4 && x_is_f32) hipLaunchKernelGGL((qgemm_prepare_rows_f16_kernel<true, true>), dim3(mp), dim3(256), 0, s, X, Xh, rowscale, M, K);
        else if (q4) hipLaunchKernelGGL((qgemm_prepare_rows_f16_kernel<true, false>), dim3(mp), dim3(256), 0, s, X, Xh, rowscale, M, K);
        else if (x_is_f32) hipLaunchKernelGGL((qgemm_prepare_rows_f16_kernel<false, true>), dim3(mp), dim3(256), 0, s, X, Xh, rowscale, M, K);
        else hipLaunchKernelGGL((qgemm_prepare_rows_f16_kernel<false, false>), dim3(mp), dim3(256), 0, s, X, Xh, rowscale, M, K);
    }
    // rows per workgroup: 32, 64 or 128 (see qgemm_f16_row_tiles)
    const int MT = qgemm_f16_row_tiles(q4, M, N, splits);
    const int tm = 32 * MT;
    const size_t lds = 2 * (size_t)tm * QF_PITCH + 4 * (size_t)tm;  // 132 KB / 66 KB (two X tiles) + the row scales: above the default 64 KB cap of dynamic LDS
    static std::once_flag raised;  // two host threads may get here at once: the second waits until the caps are raised
    std::call_once(raised, [] {
        const int big = 2 * 128 * QF_PITCH + 4 * 128, small = 2 * 64 * QF_PITCH + 4 * 64;
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_kernel<Q4Tile, 4, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, big);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_kernel<Q6Tile, 4, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, big);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_kernel<Q4Tile, 2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, small);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_kernel<Q6Tile, 2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize, small);
    });
    const dim3 grid((N + QF_TN - 1) / QF_TN, (M + tm - 1) / tm, splits);
    const uint8_t* Wb = static_cast<const uint8_t*>(W);
    // Every tile height runs with eight waves (two per SIMD, one 32-column strip each): against four waves owning two strips
    // each, 512 x 4096 x 14336 104 -> 92 us (128 rows), 512 x 4096 x 4096 59.8 -> 45.3 us and 96 x 4096 x 2560 57.0 -> 42.7 us
    // (64 rows), a 16-token prompt 4.09 -> 3.86 ms (32 rows); the 64-row Q6_K tile no longer spills.
#define PTM_QF(TILE, MTV) hipLaunchKernelGGL((qgemm_f16_kernel<TILE, MTV, 8>), grid, dim3(512), lds, s, Wb, stride, Xh, rowscale, Y, M, K, N, acc, bps, partials)
    if (q4) {
        if (MT == 4) PTM_QF(Q4Tile, 4);
        else if (MT == 2) PTM_QF(Q4Tile, 2);
        else PTM_QF(Q4Tile, 1);
    } else {
        if (MT == 4) PTM_QF(Q6Tile, 4);
        else if (MT == 2) PTM_QF(Q6Tile, 2);
        else PTM_QF(Q6Tile, 1);
    }
#undef PTM_QF
    if (deferred_splits) *deferred_splits = partials ? splits : 0;
    if (partials && !deferred_splits) {
        const int64_t total = (int64_t)M * N;
        hipLaunchKernelGGL(qgemm_split_reduce_kernel, dim3((unsigned)((total + 1023) / 1024)), dim3(256), 0, s, partials, splits,
                           Y, total, acc);
    }
    return launch_status();
}

// X (+)= the `splits` partial sums a deferred qgemm_f16_impl left in P, then RMSNorm(X; gamma) into the row workspaces
// (ws_round for Q4_K matrices, ws_plain for Q6_K ones; either may be NULL), as qgemm_f16_prepare_fused(1, ...) fills them.
int qgemm_f16_reduce_norm_prepare(const float* P, int splits, float* X, bool accumulate, const float* gamma, float eps,
                                  int add_one, void* ws_round, void* ws_plain, int M, int K, hipStream_t s) {
    if (!P || !X || !gamma || (!ws_round && !ws_plain)) return PTM_E_NULL;
    if (M <= 0 || K <= 0 || (K % 256) != 0 || splits < 1) return PTM_E_SHAPE;
    if (K > 12288) return PTM_E_UNSUPPORTED;  // the row is staged in LDS (48 KB, within the default cap)
    if (!aligned16(P) || !aligned16(X) || !aligned16(gamma) || !aligned16(ws_round) || !aligned16(ws_plain)) return PTM_E_ALIGN;
    const int mp = qf_mpad(M);
    _Float16* hr = static_cast<_Float16*>(ws_round);
    _Float16* hp = static_cast<_Float16*>(ws_plain);
    float* rr = hr ? reinterpret_cast<float*>(hr + (int64_t)mp * K) : nullptr;
    float* rp = hp ? reinterpret_cast<float*>(hp + (int64_t)mp * K) : nullptr;
    if (splits <= 4)
        hipLaunchKernelGGL(qgemm_reduce_norm_prepare_kernel<4>, dim3(mp), dim3(256), (size_t)K * 4, s, P, splits, X, accumulate ? 1 : 0,
                           gamma, eps, add_one, hr, rr, hp, rp, M, K);
    else
        hipLaunchKernelGGL(qgemm_reduce_norm_prepare_kernel<8>, dim3(mp), dim3(256), (size_t)K * 4, s, P, splits, X, accumulate ? 1 : 0,
                           gamma, eps, add_one, hr, rr, hp, rp, M, K);
    return launch_status();
}

// Y[i] = X . W[i]^T for up to three Q4_K / Q6_K matrices over the same K whose rows are already prepared (ws_round for the
// Q4_K ones, ws_plain for the Q6_K ones, as qgemm_f16_prepare_fused leaves them), in one launch plus one reduction.
size_t qgemm_f16_multi_split_bytes(int n, const int* N, const uint32_t* types, int K, int M) {
    int sp[3];
    qgemm_f16_multi_plan(n, N, types, K, M, sp);
    size_t e = 0;
    for (int i = 0; i < n; ++i) if (sp[i] > 1) e += (size_t)sp[i] * M * N[i];
    return 4 * e;
}

// deferred_P / deferred_splits (optional, n entries each): instead of the reduction launch, where matrix i's partial sums lie
// (its finished rows Y[i] when it was not split) and how many slabs there are, for the caller's next kernel to fold in.
int qgemm_f16_multi(int n, const uint32_t* types, const void* const* W, const int64_t* strides, const int* N, float* const* Y,
                    int M, int K, void* ws_round, void* ws_plain, float* split_ws, size_t split_ws_bytes, hipStream_t s,
                    const float** deferred_P, int* deferred_splits) {
    if (n < 1 || n > 3) return PTM_E_SHAPE;
    if (M <= 0 || K <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    const int mp = qf_mpad(M);
    if (mp / 128 > 65535) return PTM_E_UNSUPPORTED;
    if (qgemm_f16_multi_split_bytes(n, N, types, K, M) > split_ws_bytes || !split_ws) return PTM_E_SHAPE;
    int sp[3];
    qgemm_f16_multi_plan(n, N, types, K, M, sp);
    const int nblk = K / 256;
    QfMulti a{};
    QfRedMulti r{};
    a.n_mat = n;
    int slots = 0, red_blocks = 0;
    float* part = split_ws;
    // the Q6_K matrices first: their workgroups take longest and should be the first ones placed
    int order[3], k = 0;
    for (int i = 0; i < n; ++i) if (types[i] == PTM_TYPE_Q6_K) order[k++] = i;
    for (int i = 0; i < n; ++i) if (types[i] != PTM_TYPE_Q6_K) order[k++] = i;
    for (int o = 0; o < n; ++o) {
        const int i = order[o];
        const bool q6 = types[i] == PTM_TYPE_Q6_K;
        if (!q6 && types[i] != PTM_TYPE_Q4_K) return PTM_E_UNSUPPORTED;
        void* ws = q6 ? ws_plain : ws_round;
        if (!W[i] || !Y[i] || !ws) return PTM_E_NULL;
        if (N[i] <= 0 || strides[i] < (int64_t)nblk * (q6 ? 210 : 144)) return PTM_E_SHAPE;
        if (q6 ? ((strides[i] & 1) || (reinterpret_cast<uintptr_t>(W[i]) & 1u)) : (!aligned16(W[i]) || (strides[i] & 15))) return PTM_E_ALIGN;
        if (!aligned16(ws) || (reinterpret_cast<uintptr_t>(Y[i]) & 15u)) return PTM_E_ALIGN;
        QfMat& m = a.m[o];
        m.W = static_cast<const uint8_t*>(W[i]);
        m.stride = strides[i];
        m.Xh = static_cast<const _Float16*>(ws);
        m.rowscale = reinterpret_cast<const float*>(m.Xh + (int64_t)mp * K);
        m.Y = Y[i];
        m.N = N[i];
        m.bps = (nblk + sp[i] - 1) / sp[i];
        const int splits = (nblk + m.bps - 1) / m.bps;  // no empty split
        m.ntiles = (N[i] + QF_TN - 1) / QF_TN;
        m.q6 = q6 ? 1 : 0;
        m.partials = splits > 1 ? part : nullptr;
        if (deferred_P) { deferred_P[i] = splits > 1 ? part : Y[i]; deferred_splits[i] = splits; }
        slots += m.ntiles * splits;
        m.slot_end = slots;
        if (splits > 1) {
            QfRedSeg& g = r.s[r.n++];
            g.P = part;
            g.Y = Y[i];
            g.total = (int64_t)M * N[i];
            g.splits = splits;
            red_blocks += (int)((g.total + 1023) / 1024);
            g.blk_end = red_blocks;
            part += (size_t)splits * M * N[i];
        }
    }
    static std::once_flag raised;
    std::call_once(raised, [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_multi_kernel<4, 8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  2 * 128 * QF_PITCH + 4 * 128);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qgemm_f16_multi_kernel<2, 8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  2 * 64 * QF_PITCH + 4 * 64);
    });
    if (M <= 32)  // short prompts: the 32-row tile (see qgemm_f16_row_tiles)
        hipLaunchKernelGGL((qgemm_f16_multi_kernel<1, 8>), dim3(slots, 1), dim3(512), 2 * (size_t)32 * QF_PITCH + 4 * 32, s, a, M, K);
    else if (M <= 64)
        hipLaunchKernelGGL((qgemm_f16_multi_kernel<2, 8>), dim3(slots, 1), dim3(512), 2 * (size_t)64 * QF_PITCH + 4 * 64, s, a, M, K);
    else
        hipLaunchKernelGGL((qgemm_f16_multi_kernel<4, 8>), dim3(slots, (M + 127) / 128), dim3(512), 2 * (size_t)128 * QF_PITCH + 4 * 128, s, a, M, K);
    if (r.n > 0 && !deferred_P) hipLaunchKernelGGL(qgemm_split_reduce_multi_kernel, dim3(red_blocks), dim3(256), 0, s, r);
    return launch_status();
}

// Fills the row workspaces of qgemm_f16_impl (call it with reuse_rows afterwards): pre 1 = RMSNorm(X; gamma = X2), pre 2 =
// SiLU(X) * X2.  ws_round serves Q4_K matrices, ws_plain Q6_K ones; either may be NULL.
int qgemm_f16_prepare_fused(int pre, const float* X, const float* X2, float eps, int add_one, void* ws_round, void* ws_plain,
                            int M, int K, hipStream_t s) {
    if (!X || !X2 || (!ws_round && !ws_plain)) return PTM_E_NULL;
    if (M <= 0 || K <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (!aligned16(X) || !aligned16(X2) || !aligned16(ws_round) || !aligned16(ws_plain)) return PTM_E_ALIGN;
    const int mp = qf_mpad(M);
    _Float16* hr = static_cast<_Float16*>(ws_round);
    _Float16* hp = static_cast<_Float16*>(ws_plain);
    float* rr = hr ? reinterpret_cast<float*>(hr + (int64_t)mp * K) : nullptr;
    float* rp = hp ? reinterpret_cast<float*>(hp + (int64_t)mp * K) : nullptr;
    if (pre == 1) hipLaunchKernelGGL(qgemm_prepare_fused_kernel<1>, dim3(mp), dim3(256), 0, s, X, X2, eps, add_one, hr, rr, hp, rp, M, K);
    else if (pre == 2 && M <= 128) hipLaunchKernelGGL((qgemm_prepare_fused_kernel<2, 1024>), dim3(mp), dim3(1024), 0, s, X, X2, eps, add_one, hr, rr, hp, rp, M, K);
    else if (pre == 2) hipLaunchKernelGGL(qgemm_prepare_fused_kernel<2>, dim3(mp), dim3(256), 0, s, X, X2, eps, add_one, hr, rr, hp, rp, M, K);
    else return PTM_E_UNSUPPORTED;
    return launch_status();
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

int64_t ptm_qgemm_f16_workspace_bytes(int M, int K) {
    if (M <= 0 || K <= 0) return 0;
    const int64_t mp = qf_mpad(M);
    return mp * K * 2 + mp * 4;
}

int ptm_qgemm_f16(uint32_t ggml_type, const void* W, const void* X_bf16, float* Y, int M, int K, int N, int64_t stride,
                  void* workspace, ptm_stream_t stream) {
    return qgemm_f16_impl(ggml_type, W, X_bf16, false, Y, M, K, N, stride, workspace, false, nullptr, 0, false, as_stream(stream),
                          nullptr);
}

int64_t ptm_qgemm_f16_f32_workspace_bytes(int M, int K, int N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    const int64_t base = (ptm_qgemm_f16_workspace_bytes(M, K) + 255) & ~(int64_t)255;
    const int splits = qgemm_f16_splits(N, K, M);
    return base + (splits > 1 ? (int64_t)splits * M * N * 4 : 0);
}

int ptm_qgemm_f16_f32(uint32_t ggml_type, const void* W, const float* X_f32, float* Y, int M, int K, int N, int64_t stride,
                      void* workspace, int accumulate, ptm_stream_t stream) {
    if (M <= 0 || K <= 0 || N <= 0) return PTM_E_SHAPE;
    if (!workspace) return PTM_E_NULL;
    const int64_t base = (ptm_qgemm_f16_workspace_bytes(M, K) + 255) & ~(int64_t)255;
    const int splits = qgemm_f16_splits(N, K, M);
    return qgemm_f16_impl(ggml_type, W, X_f32, true, Y, M, K, N, stride, workspace, accumulate != 0,
                          splits > 1 ? reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + base) : nullptr,
                          splits > 1 ? (size_t)splits * M * N * 4 : 0, false, as_stream(stream), nullptr);
}

}  // extern "C"
