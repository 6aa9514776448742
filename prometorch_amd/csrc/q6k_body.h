// Device code of the Q6_K dequant-fused GEMV (see q6k_gemv.hip for the design notes); kept in a
// header so that a launch mixing Q4_K and Q6_K projections can call it per workgroup.
#pragma once
#include "ptm_common.h"

namespace ptm {

struct Q6KArgs {
    const uint8_t* W;
    const float* x;
    float* y;        // may be NULL when only the argmax is wanted
    int K, N;
    int log2S;       // lane groups per row = 1 << log2S
    int64_t stride;
    float* part_val; // ARGMAX: per-workgroup best value / index
    int* part_idx;
    const float* gamma;  // NORM: RMSNorm weight applied to x while staging
    float eps;
    int add_one;
    float* xn_out;       // NORM: if not NULL, workgroup 0 also stores the normalised x[K] here
    // PRE (with NORM, K <= 4096): a deferred post-norm and residual add in front of the RMSNorm, x + RMSNorm(pre_h) * pre_w;
    // workgroup 0 stores that sum to pre_out (not x: other workgroups still read x)
    const float* pre_h;
    const float* pre_w;
    float* pre_out;
};

enum { Q6K_THREADS = 256, Q6K_U = 5 };

__device__ __forceinline__ float dot4_u8(uint32_t q, float4 x, float acc) {
    acc = fmaf((float)(q & 0xffu), x.x, acc);
    acc = fmaf((float)((q >> 8) & 0xffu), x.y, acc);
    acc = fmaf((float)((q >> 16) & 0xffu), x.z, acc);
    acc = fmaf((float)(q >> 24), x.w, acc);
    return acc;
}

// What one lane fetches of a block.  Blocks are 210 bytes, so every other block of a row starts 2 bytes off a
// dword boundary, and 16-byte loads from such addresses run at a fraction of the aligned rate.  The ql / qh
// pieces are therefore fetched as the dword-aligned 16 bytes at (address - mis), mis = 0 or 2, plus the
// piece's last two bytes, and shifted into place with v_alignbyte.  The lane's two scales are fetched as single
// signed bytes (no extraction arithmetic), d as a half word.
struct Q6Blk { uint4 ql, qh; uint32_t ql_t, qh_t; int sc_lo, sc_hi; uint32_t d; uint32_t mis; };

struct __attribute__((packed, aligned(4))) u128_a4 { uint32_t v[4]; };

__device__ __forceinline__ Q6Blk q6k_load(const uint8_t* __restrict__ p, int j, int qh_off, int sc_off) {
    Q6Blk r;
    r.mis = (uint32_t)reinterpret_cast<uintptr_t>(p) & 2u;
    const uint8_t* pa = p - r.mis;  // same dword as p, hence same page: never faults even at the first byte of an allocation
    const u128_a4 l = *reinterpret_cast<const u128_a4*>(pa + 16 * j);
    const u128_a4 h = *reinterpret_cast<const u128_a4*>(pa + qh_off);
    r.ql = make_uint4(l.v[0], l.v[1], l.v[2], l.v[3]);
    r.qh = make_uint4(h.v[0], h.v[1], h.v[2], h.v[3]);
    r.ql_t = reinterpret_cast<const u16_a2*>(p + 16 * j + 14)->v;
    r.qh_t = reinterpret_cast<const u16_a2*>(p + qh_off + 14)->v;
    r.sc_lo = reinterpret_cast<const int8_t*>(p)[sc_off];
    r.sc_hi = reinterpret_cast<const int8_t*>(p)[sc_off + 4];
    r.d = reinterpret_cast<const u16_a2*>(p + 208)->v;
    return r;
}

// the 16 bytes that start `mis` bytes into {w, tail}
__device__ __forceinline__ void realign16(const uint4 w, uint32_t tail, uint32_t mis, uint32_t (&out)[4]) {
    out[0] = __builtin_amdgcn_alignbyte(w.y, w.x, mis);
    out[1] = __builtin_amdgcn_alignbyte(w.z, w.y, mis);
    out[2] = __builtin_amdgcn_alignbyte(w.w, w.z, mis);
    out[3] = __builtin_amdgcn_alignbyte(tail, w.w, mis);
}

// x in LDS: float4 slot i of the vector sits at slot i + i / 32 (one spare slot behind every 128 values).  A lane group
// reads 16-byte pieces 128 values apart (the two halves of a super-block) and neighbouring groups read blocks 256
// values apart: unpadded, the 16 lanes one ds_read_b128 pass serves would hit 4 of the 16 bank quads, four lanes each
// (measured on the 2560 x 9728 down projection: 68 % of the LDS cycles were bank conflicts).
__device__ __forceinline__ int q6k_xslot(int i4) { return i4 + (i4 >> 5); }
inline __host__ __device__ int q6k_x_floats(int K) { return K + K / 32; }              // padded length of x in LDS
inline size_t q6k_x_lds_bytes(int K) { return (size_t)q6k_x_floats(K) * 4 + (size_t)K / 4; }  // x and its per-16 sums

// contribution of block b to lane j's chain
__device__ __forceinline__ float q6k_block_term(const Q6Blk& k, const float* __restrict__ xf,
                                                const float* __restrict__ xsum16, int b, int j) {
    const int half = j >> 2, jj = j & 3, which32 = jj >> 1, l16 = jj & 1;
    const int hshift = 2 * which32;
    const int xo = 128 * half + 32 * which32 + 16 * l16;  // x offset of the low-nibble 16; high-nibble +64
    const float* xb = xf + 4 * q6k_xslot((b * 256 + xo) >> 2);  // the 32 slots of a half block share one shift
    float s_lo = 0.0f, s_hi = 0.0f;
    uint32_t qlw[4], qhw[4];
    realign16(k.ql, k.ql_t, k.mis, qlw);
    realign16(k.qh, k.qh_t, k.mis, qhw);
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
    const float d = h2f(k.d);
    const float f_lo = d * (float)k.sc_lo;  // scale of the low-nibble 16; the high-nibble one is 4 further
    const float f_hi = d * (float)k.sc_hi;
    return fmaf(f_hi, s_hi, f_lo * s_lo);
}

// XCH: chunks of 4096 activations whose loads go out before the weight prefetch (the rest trail it).
// NB:  super-blocks per lane group and pass.  Every pass issues exactly NB block loads, unconditionally
//      (block indices past the row's end are clamped and their terms dropped), so that the number of loads
//      in flight is known at compile time and each block is consumed as soon as IT has arrived.
template <bool ACC, bool ARGMAX, bool NORM, int XCH, int NB, bool PRE = false>
__device__ __forceinline__ void q6k_gemv_body(const Q6KArgs a, uint8_t* lds_raw, int wg) {
    float* xf = reinterpret_cast<float*>(lds_raw);
    float* xsum16 = xf + q6k_x_floats(a.K);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6, j = lane & 7, grp = lane >> 3;
    const int S = 1 << a.log2S;
    const int sub = grp & (S - 1);
    const int rows_per_wave = 8 >> a.log2S;
    const int r = (wg * 4 + wave) * rows_per_wave + (grp >> a.log2S);
    const bool live = r < a.N;
    const int rr = live ? r : a.N - 1;
    const int nblk = a.K / 256;
    const int nb_max = (nblk + S - 1) >> a.log2S;
    const uint8_t* row = a.W + (int64_t)rr * a.stride;
    const int qh_off = 128 + 32 * (j >> 2) + 16 * (j & 1);
    const int sc_off = 192 + 8 * (j >> 2) + 2 * ((j & 3) >> 1) + (j & 1);  // the lane's low-nibble scale

    // x (optionally RMS-normalised) goes to LDS with its per-16 sums: 4 consecutive float4 slots make one 16-group
    __shared__ float red[4];
    auto emit = [&](int i, float4 v) {
        reinterpret_cast<float4*>(xf)[q6k_xslot(i)] = v;
        if constexpr (NORM) {
            if (wg == 0 && a.xn_out) reinterpret_cast<float4*>(a.xn_out)[i] = v;
        }
        float sm = (v.x + v.y) + (v.z + v.w);
        sm += dpp_f<0xB1>(sm);
        sm += dpp_f<0x4E>(sm);
        if ((tid & 3) == 0) xsum16[i >> 2] = sm;
    };
    // activation loads first (loads complete in issue order), then the first pass of weight loads
    static_assert(!PRE || (NORM && XCH == 1), "the deferred post-norm comes with the RMSNorm prologue of short vectors");
    Q6Blk blk[NB];
    if constexpr (PRE) {
        const XStagePre stg = stage_issue_pre(a.x, a.gamma, a.pre_h, a.pre_w, a.K);
        issue_order_fence();
#pragma unroll
        for (int u = 0; u < NB; ++u) blk[u] = q6k_load(row + (int64_t)min(sub + (u << a.log2S), nblk - 1) * 210, j, qh_off, sc_off);
        issue_order_fence();
        stage_finish_pre(stg, a.K, a.eps, a.add_one, red, wg == 0 ? a.pre_out : nullptr, emit);
    } else {
        const XStage<XCH> stg = stage_issue<NORM, XCH>(a.x, a.gamma, a.K, a.eps, a.add_one, red, emit);
        issue_order_fence();
#pragma unroll
        for (int u = 0; u < NB; ++u) blk[u] = q6k_load(row + (int64_t)min(sub + (u << a.log2S), nblk - 1) * 210, j, qh_off, sc_off);
        issue_order_fence();
        stage_finish<NORM, XCH>(stg, a.K, a.eps, a.add_one, red, emit);
    }
    __syncthreads();

    // Passes roll: as soon as a block of pass p has been consumed its registers are refilled with the same slot of
    // pass p + 1, so a lane group keeps NB - 1 .. NB blocks in flight while it computes; the last pass only consumes.
    float acc = 0.0f;
    int i0 = 0;
    for (; i0 + NB < nb_max; i0 += NB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int b = sub + ((i0 + u) << a.log2S);
            const float t = q6k_block_term(blk[u], xf, xsum16, min(b, nblk - 1), j);
            acc += b < nblk ? t : 0.0f;
            blk[u] = q6k_load(row + (int64_t)min(sub + ((i0 + NB + u) << a.log2S), nblk - 1) * 210, j, qh_off, sc_off);
        }
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const int b = sub + ((i0 + u) << a.log2S);
        const float t = q6k_block_term(blk[u], xf, xsum16, min(b, nblk - 1), j);
        acc += b < nblk ? t : 0.0f;
    }
    float p = sum8(acc);
    if (S >= 2) p += dpp_f<0x128>(p);
    if (S >= 4) p += __shfl_xor(p, 16, 64);
    if (S >= 8) p += __shfl_xor(p, 32, 64);
    if (live && sub == 0 && j == 0 && a.y) {
        if constexpr (ACC) a.y[rr] += p;
        else a.y[rr] = p;
    }
    if constexpr (ARGMAX) {
        // best (value, lowest index) of this workgroup's rows
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
            a.part_val[wg] = v;
            a.part_idx[wg] = idx;
        }
    }
}

// Lane groups per row: the fewest that still give the chip enough workgroups, with a group's blocks in at most two
// rolling passes (the vocabulary projection 151936 x 2560 then runs one group per row, two passes of 5 blocks:
// 94 -> 88 us with the argmax against two groups per row and one pass, for half the stagings of x).
inline int q6k_pick_log2S(int rows, int nblk) {
    int l = 0;
    while (l < 3) {
        const int S = 1 << l;
        const int wgs = (rows * S + 31) / 32;
        const int nb = (nblk + S - 1) / S;
        if (nb <= 2 * Q6K_U && wgs >= 600) break;
        if (nb <= 1) break;
        ++l;
    }
    return l;
}
inline int q6k_workgroups(int N, int K) {
    const int l = q6k_pick_log2S(N, K / 256);
    const int rows_per_wg = 32 >> l;
    return (N + rows_per_wg - 1) / rows_per_wg;
}

inline int q6k_blocks_per_pass(int N, int K) {
    static const int cand[] = {2, 3, 5};
    const int l = q6k_pick_log2S(N, K / 256);
    return pick_blocks_per_pass((K / 256 + (1 << l) - 1) >> l, cand, 3);
}

}  // namespace ptm
