// Shared device helpers for the gfx950 kernels (wave64, DPP cross-lane ops, block decode).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/ptm.h"

#define PTM_WAVE 64

namespace ptm {

// ---- error plumbing -------------------------------------------------------------------
extern thread_local int g_last_hip_error;
inline int hip_status(hipError_t e) {
    if (e == hipSuccess) return PTM_OK;
    g_last_hip_error = (int)e;
    return PTM_E_HIP;
}
inline int launch_status() { return hip_status(hipGetLastError()); }
inline hipStream_t as_stream(ptm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- DPP lane exchanges (row = 16 lanes) ------------------------------------------------
// quad_perm encodings: [1,0,3,2] = 0xB1 (xor 1), [2,3,0,1] = 0x4E (xor 2);
// 0x141 = row_half_mirror (lane i <-> 7-i inside each 8), 0x140 = row_mirror (i <-> 15-i).
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// all-reduce (sum / max) over aligned groups of 8 lanes
__device__ __forceinline__ float sum8(float v) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    return v;
}
__device__ __forceinline__ int sum8i(int v) {
    v += dpp_i<0xB1>(v);
    v += dpp_i<0x4E>(v);
    v += dpp_i<0x141>(v);
    return v;
}
__device__ __forceinline__ float max8(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    return v;
}
__device__ __forceinline__ float sum16(float v) {
    v = sum8(v);
    v += dpp_f<0x140>(v);
    return v;
}
// all-reduce over the whole wave64
__device__ __forceinline__ float sum64(float v) {
    v = sum16(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float max64(float v) {
    v = max8(v);
    v = fmaxf(v, dpp_f<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// ---- fp16 ---------------------------------------------------------------------------
__device__ __forceinline__ float h2f(uint32_t bits16) {
    return __half2float(__ushort_as_half((unsigned short)(bits16 & 0xffffu)));
}
__device__ __forceinline__ unsigned short f2h_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

// ---- Q4_K header decode: 12 packed bytes (3 dwords) -> (scale, min) of sub-block j ------
// Same mapping as get_scale_min_k4 (reference: torch/io/gguf_dequant.h:289-297).
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, int& sc, int& mn) {
    const int sh = 8 * (j & 3);
    const uint32_t b0 = (s0 >> sh) & 0xffu, b1 = (s1 >> sh) & 0xffu, b2 = (s2 >> sh) & 0xffu;
    const int sc_lo = b0 & 63u, mn_lo = b1 & 63u;
    const int sc_hi = (b2 & 0x0fu) | ((b0 >> 6) << 4);
    const int mn_hi = (b2 >> 4) | ((b1 >> 6) << 4);
    sc = j < 4 ? sc_lo : sc_hi;
    mn = j < 4 ? mn_lo : mn_hi;
}

// 16-byte load from an address that is only 2-byte aligned (Q6_K blocks are 210 B).
struct __attribute__((packed, aligned(2))) u128_a2 { uint32_t v[4]; };
__device__ __forceinline__ uint4 ld16_a2(const uint8_t* p) {
    const u128_a2 t = *reinterpret_cast<const u128_a2*>(p);
    return make_uint4(t.v[0], t.v[1], t.v[2], t.v[3]);
}
struct __attribute__((packed, aligned(2))) u16_a2 { uint16_t v; };

// Q8 activation layout in memory: int8 qs[K] | float d[K/32] | float sum[K/32]
__host__ __device__ inline int64_t q8_bytes(int K) { return (int64_t)K + K / 4; }

// Quantise the 32 floats held as float4 by the 8 lanes of an aligned lane group.
// Returns the packed 4 int8 of this lane; d and sum (d * sum q) are group-uniform.
// Same rule as quantize_x_q8 (reference: torch/io/cpu_quant_gemv.h:147-198).
__device__ __forceinline__ uint32_t q8_quantize4(float4 v, float& d, float& sum) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = max8(amax);
    d = amax / 127.0f;
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    int q0 = (int)rintf(v.x * id), q1 = (int)rintf(v.y * id), q2 = (int)rintf(v.z * id), q3 = (int)rintf(v.w * id);
    q0 = max(-127, min(127, q0));
    q1 = max(-127, min(127, q1));
    q2 = max(-127, min(127, q2));
    q3 = max(-127, min(127, q3));
    const int s = sum8i(q0 + q1 + q2 + q3);
    sum = d * (float)s;
    return (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) |
           ((uint32_t)(q3 & 0xff) << 24);
}

// Block-wide sum for blockDim.x = 256 (4 waves); red is 4 floats of LDS.
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = sum64(v);
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// ---- activation staging --------------------------------------------------------------------------
// A 256-thread workgroup walks x[K] as float4 slots i = tid + 256*u.  Loads are issued four slots
// at a time BEFORE any of them is consumed, so a staging pass costs one memory round trip per 4096
// values instead of one per 1024.  For K <= 4096 the slots stay in registers between the
// sum-of-squares pass and the normalise pass.
struct XChunk { float4 v[4]; };

__device__ __forceinline__ XChunk load_chunk(const float4* __restrict__ p, int base, int n4) {
    XChunk c;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = base + (int)threadIdx.x + 256 * u;
        c.v[u] = i < n4 ? p[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    return c;
}

__device__ __forceinline__ float chunk_sumsq(const XChunk& c, float ss) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        ss = fmaf(c.v[u].x, c.v[u].x, ss);
        ss = fmaf(c.v[u].y, c.v[u].y, ss);
        ss = fmaf(c.v[u].z, c.v[u].z, ss);
        ss = fmaf(c.v[u].w, c.v[u].w, ss);
    }
    return ss;
}

// x * rs * (gamma [+1]) in the reference's order (cpu_quant_gemv.h:2599)
__device__ __forceinline__ float4 norm4(float4 v, float4 g, float rs, float one) {
    v.x = v.x * rs * (g.x + one);
    v.y = v.y * rs * (g.y + one);
    v.z = v.z * rs * (g.z + one);
    v.w = v.w * rs * (g.w + one);
    return v;
}

// Staging is split in two so that a kernel can put its (few) activation loads in front of its (many)
// weight loads: vector loads complete in issue order, so activation loads issued behind the weight
// prefetch could only be consumed after every weight had arrived.
//   XStage st = stage_issue<NORM>(x, gamma, K);      // loads of the first 4096 values (+ gamma)
//   ... issue weight loads ...
//   stage_finish<NORM>(st, x, gamma, K, eps, add_one, red, emit);
// emit(i, value) is called for every float4 slot i of x (RMS-normalised with gamma when NORM), all 256
// threads taking part; emit may use cross-lane ops (slots are handed out wave-uniformly: K % 256 == 0).
struct XStage { XChunk x0, g0; };

template <bool NORM>
__device__ __forceinline__ XStage stage_issue(const float* __restrict__ x, const float* __restrict__ gamma, int K) {
    XStage st;
    st.x0 = load_chunk(reinterpret_cast<const float4*>(x), 0, K / 4);
    if constexpr (NORM) st.g0 = load_chunk(reinterpret_cast<const float4*>(gamma), 0, K / 4);
    return st;
}

template <bool NORM, typename Emit>
__device__ __forceinline__ void stage_finish(const XStage& st, const float* __restrict__ x,
                                             const float* __restrict__ gamma, int K, float eps, int add_one,
                                             float* red4, Emit emit) {
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const float4* g4 = reinterpret_cast<const float4*>(gamma);
    const int n4 = K / 4;
    const float one = add_one ? 1.0f : 0.0f;
    float rs = 1.0f;
    if constexpr (NORM) {
        float ss = chunk_sumsq(st.x0, 0.0f);
        for (int base = 1024; base < n4; base += 1024) ss = chunk_sumsq(load_chunk(x4, base, n4), ss);
        ss = block_sum256(ss, red4);
        rs = 1.0f / sqrtf(ss / (float)K + eps);
    }
    for (int base = 0; base < n4; base += 1024) {
        XChunk c = st.x0, g = st.g0;
        if (base > 0) {
            c = load_chunk(x4, base, n4);
            if constexpr (NORM) g = load_chunk(g4, base, n4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + (int)threadIdx.x + 256 * u;
            if (i < n4) {
                float4 v = c.v[u];
                if constexpr (NORM) v = norm4(v, g.v[u], rs, one);
                emit(i, v);
            }
        }
    }
}

}  // namespace ptm
