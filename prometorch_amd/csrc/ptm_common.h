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

// Bookkeeping of a decode step done by the thread that finishes the argmax (all NULL: plain argmax):
// publish the token, feed it back as the next input, advance the position.
struct ArgmaxAdvance {
    int* d_token;
    int64_t* d_past;
    int* d_step;
    int64_t* tokens_out;
    int cap;
};

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
// all-reduce over each half of the wave (lanes 0..31, 32..63)
__device__ __forceinline__ float sum32(float v) {
    v = sum16(v);
    v += __shfl_xor(v, 16, 64);
    return v;
}
// sum over groups of LPP = 8, 16 or 32 consecutive lanes
template <int LPP>
__device__ __forceinline__ float sum_lanes(float v) {
    static_assert(LPP == 8 || LPP == 16 || LPP == 32, "lane group of 8, 16 or 32");
    if constexpr (LPP == 8) return sum8(v);
    else if constexpr (LPP == 16) return sum16(v);
    else return sum32(v);
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

// Activations are fetched with buffer loads: the hardware range check returns zeros for slots past the end of
// the vector, so the load needs no predicate.  (A predicated global load is compiled to a branch around the
// load; the compiler can then no longer count the loads in flight and waits for ALL of them, the weight
// prefetch included, before the first use of x.)
// Compiler-only fence: memory operations are neither moved nor scheduled across it.  Used to pin the ISSUE
// order of loads (activations, then weights), which decides the order in which their data can be consumed.
__device__ __forceinline__ void issue_order_fence() { asm volatile("" ::: "memory"); }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ XChunk load_chunk(__amdgpu_buffer_rsrc_t rs, int base) {
    XChunk c;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = base + (int)threadIdx.x + 256 * u;
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, i * 16, 0, 0);
        c.v[u] = make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
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
//   XStage<NCH> st = stage_issue<NORM, NCH>(x, gamma, K, eps, add_one, red, emit);   // loads of the first NCH*4096 values
//   ... issue weight loads ...
//   stage_finish<NORM, NCH>(st, K, eps, add_one, red, emit);
// emit(i, value) is called for every float4 slot i of x (RMS-normalised with gamma when NORM), all 256
// threads taking part; emit may use cross-lane ops (slots are handed out wave-uniformly: K % 256 == 0).
// Between the two calls only unconditional loads may be issued, and stage_finish issues none: the compiler
// can then count the loads in flight and wait for exactly the activation loads.  Vectors longer than
// NCH*4096 values take a slow path that stages the part beyond the register window first, inside stage_issue.
template <int NCH = 1>
struct XStage { XChunk x[NCH], g[NCH]; float rs; };

template <bool NORM, typename Emit>
__device__ __forceinline__ void emit_chunk(const XChunk& c, const XChunk& g, int base, int n4, float rs, float one,
                                           Emit& emit) {
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

template <bool NORM, int NCH = 1, typename Emit>
__device__ __forceinline__ XStage<NCH> stage_issue(const float* __restrict__ x, const float* __restrict__ gamma, int K,
                                                   float eps, int add_one, float* red4, Emit emit) {
    const __amdgpu_buffer_rsrc_t x4 = make_rsrc(x, K * 4);
    const __amdgpu_buffer_rsrc_t g4 = make_rsrc(NORM ? gamma : x, K * 4);
    const int n4 = K / 4;
    XStage<NCH> st;
    st.rs = 1.0f;
    // Slow path first, while no other load is in flight: the compiler cannot count loads across this loop and
    // waits for everything outstanding where the paths join, which costs nothing here.
    if (n4 > 1024 * NCH) {
        if constexpr (NORM) {
            float ss = 0.0f;
            for (int base = 0; base < n4; base += 1024) ss = chunk_sumsq(load_chunk(x4, base), ss);
            ss = block_sum256(ss, red4);
            st.rs = 1.0f / sqrtf(ss / (float)K + eps);
        }
        for (int base = 1024 * NCH; base < n4; base += 1024) {
            const XChunk c = load_chunk(x4, base);
            XChunk g = c;
            if constexpr (NORM) g = load_chunk(g4, base);
            emit_chunk<NORM>(c, g, base, n4, st.rs, add_one ? 1.0f : 0.0f, emit);
        }
    }
    issue_order_fence();  // keep the loads below from being hoisted above the slow path
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        st.x[c] = load_chunk(x4, 1024 * c);
        if constexpr (NORM) st.g[c] = load_chunk(g4, 1024 * c);
    }
    return st;
}

template <bool NORM, int NCH = 1, typename Emit>
__device__ __forceinline__ void stage_finish(const XStage<NCH>& st, int K, float eps, int add_one, float* red4,
                                             Emit emit) {
    const int n4 = K / 4;
    float rs = st.rs;
    if constexpr (NORM) {
        if (n4 <= 1024 * NCH) {
            float ss = 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) ss = chunk_sumsq(st.x[c], ss);
            ss = block_sum256(ss, red4);
            rs = 1.0f / sqrtf(ss / (float)K + eps);
        }
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c)
        if (1024 * c < n4) emit_chunk<NORM>(st.x[c], st.g[c], 1024 * c, n4, rs, add_one ? 1.0f : 0.0f, emit);
}

// The same staging with a deferred post-norm in front (K <= 4096, one chunk): the vector that is normalised is
// x + RMSNorm(h) * w, formed by every workgroup from x, the branch output h and the post-norm weight w; pre_out (NULL in all
// but one workgroup) receives that sum.  Slots past the end of the vectors load as zeros and stay zero.
struct XStagePre { XChunk x, g, h, w; };

__device__ __forceinline__ XStagePre stage_issue_pre(const float* x, const float* gamma, const float* h, const float* w, int K) {
    XStagePre st;
    st.h = load_chunk(make_rsrc(h, K * 4), 0);  // the branch output first: its sum of squares is the first thing needed
    st.w = load_chunk(make_rsrc(w, K * 4), 0);
    st.x = load_chunk(make_rsrc(x, K * 4), 0);
    st.g = load_chunk(make_rsrc(gamma, K * 4), 0);
    return st;
}

template <typename Emit>
__device__ __forceinline__ void stage_finish_pre(const XStagePre& st, int K, float eps, int add_one, float* red4,
                                                 float* pre_out, Emit emit) {
    const int n4 = K / 4;
    const float one = add_one ? 1.0f : 0.0f;
    const float ssh = block_sum256(chunk_sumsq(st.h, 0.0f), red4);
    const float rsh = 1.0f / sqrtf(ssh / (float)K + eps);
    XChunk xe;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        xe.v[u].x = st.x.v[u].x + st.h.v[u].x * rsh * (st.w.v[u].x + one);
        xe.v[u].y = st.x.v[u].y + st.h.v[u].y * rsh * (st.w.v[u].y + one);
        xe.v[u].z = st.x.v[u].z + st.h.v[u].z * rsh * (st.w.v[u].z + one);
        xe.v[u].w = st.x.v[u].w + st.h.v[u].w * rsh * (st.w.v[u].w + one);
        const int i = (int)threadIdx.x + 256 * u;
        if (pre_out && i < n4) reinterpret_cast<float4*>(pre_out)[i] = xe.v[u];
    }
    const float ss = block_sum256(chunk_sumsq(xe, 0.0f), red4);
    const float rs = 1.0f / sqrtf(ss / (float)K + eps);
    emit_chunk<true>(xe, st.g, 0, n4, rs, one, emit);
}

// Blocks per pass for a lane group that owns nb_max blocks: the candidate (from a small set, so that the
// number of kernel instances stays small) that wastes the fewest padded block slots; ties go to the larger.
inline int pick_blocks_per_pass(int nb_max, const int* cand, int n_cand) {
    int best = cand[0], best_waste = 1 << 30;
    for (int i = 0; i < n_cand; ++i) {
        const int waste = (nb_max + cand[i] - 1) / cand[i] * cand[i] - nb_max;
        if (waste < best_waste || (waste == best_waste && cand[i] > best)) { best = cand[i]; best_waste = waste; }
    }
    return best;
}

}  // namespace ptm
