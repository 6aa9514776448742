// Device code of the Q4_K dequant-fused GEMV (see q4k_gemv.hip for the design notes); kept in a
// header so that a launch mixing Q4_K and Q6_K projections can call it per workgroup.
#pragma once
#include "ptm_common.h"

namespace ptm {

struct Q4KArgs {
    const uint8_t* W[3];
    float* y[3];
    int row_end[3];  // cumulative row counts of the (up to 3) matrices
    int n_mat;
    int total_rows;  // MODE 1: 2*N interleaved (gate row r, up row r)
    int K;
    int log2S;       // lane groups per row = 1 << log2S
    int64_t stride;
    int tiles_per_wg;    // row tiles (of 32 >> log2S rows) a workgroup walks with ONE staging of x (0 or 1: one tile)
    const void* x;       // fp32 x[K] (XQ8 == false) or Q8 blocks (XQ8 == true)
    const float* gamma;  // RMSNorm weight (NORM)
    float eps;
    int add_one;
    int gelu;            // MODE 1: tanh-GELU(gate) * up (gemma) instead of SiLU(gate) * up
    // PRE (with NORM, K <= 4096): the branch output of the previous projection still waits for its post-norm and residual
    // add (gemma's post-attention / post-feed-forward norms, gguf_model.h:3656-3680, :3787-3807).  Every workgroup forms
    // x + RMSNorm(pre_h) * pre_w itself before its own RMSNorm; workgroup 0 also stores that sum to pre_out, which must not
    // be x (other workgroups still read x).
    const float* pre_h;
    const float* pre_w;
    float* pre_out;
};

enum { Q4K_THREADS = 256, Q4K_U = 10 };

// ---- prologue: bring the Q8 activation into LDS; loads first (q4k_stage_issue), the arithmetic after the
// weight prefetch has been issued (q4k_stage_finish) --------------------------------------------------
// fp32 x: thread t owns the 16 consecutive values [16t, 16t+16), i.e. half a Q8 block (lanes t, t^1 share a
// block), so the two exact divisions of the Q8 rule are paid once per 16 values.  Every workgroup quantises the
// whole vector, so this prologue is kept short: its instructions are issued by every wave of the launch.
struct Q4KStage { float4 x[4], g[4], h[4], w[4]; float rs; u32x4 q8[2]; };

__device__ __forceinline__ void q4k_load16(__amdgpu_buffer_rsrc_t r, int first, float4 (&v)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(r, (first + 4 * u) * 4, 0, 0);  // zeros past the end
        v[u] = make_float4(__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w));
    }
}
__device__ __forceinline__ float q4k_sumsq16(const float4 (&v)[4], float ss) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        ss = fmaf(v[u].x, v[u].x, ss);
        ss = fmaf(v[u].y, v[u].y, ss);
        ss = fmaf(v[u].z, v[u].z, ss);
        ss = fmaf(v[u].w, v[u].w, ss);
    }
    return ss;
}
// Q8 rule of quantize_x_q8 (reference: torch/io/cpu_quant_gemv.h:147-198) on the half block `unit` (16 values).
template <bool NORM>
__device__ __forceinline__ void q4k_quantize16_store(const float4 (&xv)[4], const float4 (&gv)[4], float rs, float one,
                                                     int unit, uint8_t* lds, int K) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        float4 t = xv[u];
        if constexpr (NORM) t = norm4(t, gv[u], rs, one);
        v[4 * u] = t.x; v[4 * u + 1] = t.y; v[4 * u + 2] = t.z; v[4 * u + 3] = t.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, dpp_f<0xB1>(amax));
    const float d = amax / 127.0f;
    const float id = d > 0.0f ? 1.0f / d : 0.0f;
    int isum = 0;
    uint32_t w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        uint32_t pk = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = max(-127, min(127, (int)rintf(v[4 * u + i] * id)));
            isum += q;
            pk |= (uint32_t)(q & 0xff) << (8 * i);
        }
        w[u] = pk;
    }
    isum += dpp_i<0xB1>(isum);
    *reinterpret_cast<uint4*>(lds + 16 * unit) = make_uint4(w[0], w[1], w[2], w[3]);
    if ((unit & 1) == 0) {
        float* xd = reinterpret_cast<float*>(lds + K);
        xd[unit >> 1] = d;
        xd[K / 32 + (unit >> 1)] = d * (float)isum;
    }
}

template <bool XQ8, bool NORM, bool PRE = false>
__device__ __forceinline__ Q4KStage q4k_stage_issue(const Q4KArgs a, uint8_t* lds, float* red) {
    static_assert(!PRE || (NORM && !XQ8), "the deferred post-norm comes with the RMSNorm prologue");
    Q4KStage st;
    const int tid = threadIdx.x;
    st.rs = 1.0f;
    if constexpr (XQ8) {
        const uint4* src = reinterpret_cast<const uint4*>(a.x);
        uint4* dst = reinterpret_cast<uint4*>(lds);
        const int n16 = (a.K + a.K / 4) / 16;
        // beyond the register window (K > 6553): copied first, while no other load is in flight
        for (int i = tid + 2 * Q4K_THREADS; i < n16; i += Q4K_THREADS) dst[i] = src[i];
        issue_order_fence();  // keep the loads below from being hoisted above that loop
        const __amdgpu_buffer_rsrc_t r = make_rsrc(a.x, n16 * 16);
#pragma unroll
        for (int u = 0; u < 2; ++u) st.q8[u] = __builtin_amdgcn_raw_buffer_load_b128(r, (tid + Q4K_THREADS * u) * 16, 0, 0);
    } else {
        const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, a.K * 4);
        const __amdgpu_buffer_rsrc_t rg = make_rsrc(NORM ? static_cast<const void*>(a.gamma) : a.x, a.K * 4);
        const float one = a.add_one ? 1.0f : 0.0f;
        // Slow path (K > 4096, beyond the 16 values per thread kept in registers) first, while no other load is in
        // flight: the compiler cannot count loads across these loops and waits for everything where the paths join.
        if (a.K > 16 * Q4K_THREADS) {
            if constexpr (NORM) {
                float ss = 0.0f;
                for (int base = 0; base < a.K; base += 16 * Q4K_THREADS) {
                    float4 t[4];
                    q4k_load16(rx, base + 16 * tid, t);
                    ss = q4k_sumsq16(t, ss);
                }
                ss = block_sum256(ss, red);
                st.rs = 1.0f / sqrtf(ss / (float)a.K + a.eps);
            }
            for (int base = 16 * Q4K_THREADS; base < a.K; base += 16 * Q4K_THREADS) {
                float4 t[4], g[4];
                q4k_load16(rx, base + 16 * tid, t);
                if constexpr (NORM) q4k_load16(rg, base + 16 * tid, g);
                if (base + 16 * tid < a.K) q4k_quantize16_store<NORM>(t, g, st.rs, one, base / 16 + tid, lds, a.K);
            }
        }
        issue_order_fence();
        if constexpr (PRE) {  // the branch output first: its sum of squares is the first thing needed
            q4k_load16(make_rsrc(a.pre_h, a.K * 4), 16 * tid, st.h);
            q4k_load16(make_rsrc(a.pre_w, a.K * 4), 16 * tid, st.w);
        }
        q4k_load16(rx, 16 * tid, st.x);
        if constexpr (NORM) q4k_load16(rg, 16 * tid, st.g);
    }
    return st;
}

template <bool XQ8, bool NORM, bool PRE = false>
__device__ __forceinline__ void q4k_stage_finish(const Q4KStage& st, const Q4KArgs a, uint8_t* lds, float* red, int wg = 0) {
    const int tid = threadIdx.x;
    if constexpr (XQ8) {
        uint4* dst = reinterpret_cast<uint4*>(lds);
        const int n16 = (a.K + a.K / 4) / 16;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int i = tid + Q4K_THREADS * u;
            if (i < n16) dst[i] = make_uint4(st.q8[u].x, st.q8[u].y, st.q8[u].z, st.q8[u].w);
        }
    } else if constexpr (PRE) {
        // x + RMSNorm(h) * w first (threads past the end hold zeros), then the kernel's own RMSNorm of that sum
        const float one = a.add_one ? 1.0f : 0.0f;
        const float ssh = block_sum256(q4k_sumsq16(st.h, 0.0f), red);
        const float rsh = 1.0f / sqrtf(ssh / (float)a.K + a.eps);
        float4 xv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            xv[u].x = st.x[u].x + st.h[u].x * rsh * (st.w[u].x + one);
            xv[u].y = st.x[u].y + st.h[u].y * rsh * (st.w[u].y + one);
            xv[u].z = st.x[u].z + st.h[u].z * rsh * (st.w[u].z + one);
            xv[u].w = st.x[u].w + st.h[u].w * rsh * (st.w[u].w + one);
        }
        if (wg == 0 && a.pre_out && 16 * tid < a.K) {
#pragma unroll
            for (int u = 0; u < 4; ++u) reinterpret_cast<float4*>(a.pre_out)[4 * tid + u] = xv[u];
        }
        const float ss = block_sum256(q4k_sumsq16(xv, 0.0f), red);
        const float rs = 1.0f / sqrtf(ss / (float)a.K + a.eps);
        if (16 * tid < a.K) q4k_quantize16_store<true>(xv, st.g, rs, one, tid, lds, a.K);
    } else {
        float rs = st.rs;
        if constexpr (NORM) {
            if (a.K <= 16 * Q4K_THREADS) {
                const float ss = block_sum256(q4k_sumsq16(st.x, 0.0f), red);
                rs = 1.0f / sqrtf(ss / (float)a.K + a.eps);
            }
        }
        if (16 * tid < a.K) q4k_quantize16_store<NORM>(st.x, st.g, rs, a.add_one ? 1.0f : 0.0f, tid, lds, a.K);
    }
    __syncthreads();
}

// contribution of one super-block to lane j's chain (sub-block j of the block)
__device__ __forceinline__ float q4k_block_term(const uint4 hdr, const uint4 qv, const uint8_t* __restrict__ lds,
                                                int K, int b, int j) {
    const int8_t* xq = reinterpret_cast<const int8_t*>(lds);
    const float* xd = reinterpret_cast<const float*>(lds + K);
    const float* xs = xd + K / 32;
    const int half = j & 1;
    const int xoff = (j >> 1) * 64 + half * 16;  // low-nibble activations; high-nibble ones are +32
    const int4 xl = *reinterpret_cast<const int4*>(xq + b * 256 + xoff);
    const int4 xh = *reinterpret_cast<const int4*>(xq + b * 256 + xoff + 32);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_sdot4((int)(qv.x & 0x0f0f0f0fu), xl.x, lo, false);
    lo = __builtin_amdgcn_sdot4((int)(qv.y & 0x0f0f0f0fu), xl.y, lo, false);
    lo = __builtin_amdgcn_sdot4((int)(qv.z & 0x0f0f0f0fu), xl.z, lo, false);
    lo = __builtin_amdgcn_sdot4((int)(qv.w & 0x0f0f0f0fu), xl.w, lo, false);
    hi = __builtin_amdgcn_sdot4((int)((qv.x >> 4) & 0x0f0f0f0fu), xh.x, hi, false);
    hi = __builtin_amdgcn_sdot4((int)((qv.y >> 4) & 0x0f0f0f0fu), xh.y, hi, false);
    hi = __builtin_amdgcn_sdot4((int)((qv.z >> 4) & 0x0f0f0f0fu), xh.z, hi, false);
    hi = __builtin_amdgcn_sdot4((int)((qv.w >> 4) & 0x0f0f0f0fu), xh.w, hi, false);
    // even lane keeps the low-nibble half-dot and receives its partner's; odd lane the high one
    const int keep = half ? hi : lo;
    const int give = half ? lo : hi;
    const int isum = keep + dpp_i<0xB1>(give);
    int sc, mn;
    q4k_scale_min(hdr.y, hdr.z, hdr.w, j, sc, mn);
    const float d = h2f(hdr.x), dmin = h2f(hdr.x >> 16);
    const float w = d * (float)sc * xd[b * 8 + j];
    const float c = dmin * (float)mn * xs[b * 8 + j];
    return fmaf(w, (float)isum, -c);
}

__device__ __forceinline__ float gelu_mul_ref(float g, float u) {
    // reference: gguf_model.h:3730-3738
    const float x3 = g * g * g;
    const float t = tanhf(0.7978845608028654f * (g + 0.044715f * x3));
    return 0.5f * g * (1.0f + t) * u;
}

__device__ __forceinline__ float silu_mul_ref(float g, float u) {
    // reference: gguf_model.h:3741-3755 (clamp, libm exp, 1/(1+e), g*sig, *u)
    float ng = 0.0f - g;
    ng = fminf(fmaxf(ng, -88.0f), 88.0f);
    const float sig = 1.0f / (1.0f + expf(ng));
    return (g * sig) * u;
}

// MODE 0: y = or += W.x for up to three matrices over a flattened row space
// MODE 1: gate/up pair with SiLU over interleaved virtual rows (2r = gate row r, 2r+1 = up row r):
//         y[0][r] = silu(Wg[r].x) * (Wu[r].x)
// NB: super-blocks per lane group and pass; every pass issues exactly NB block loads, unconditionally (indices
//     past the row's end are clamped, their terms dropped), so the count of loads in flight is static and a
//     block is consumed as soon as it has arrived instead of after the whole prefetch.
// ROLLT (very tall matrices: a workgroup walks several row tiles, each a single pass of NB blocks per lane group): the
//     passes roll ACROSS tiles - a consumed block's registers are refilled with the same slot of the NEXT tile's row, so a
//     wave never stands with nothing in flight between two tiles (behind the last tile the refills repeat that tile: their
//     number stays static, the lines are in cache, nothing consumes them).
template <bool XQ8, bool NORM, bool ACC, int MODE, int NB, bool ROLLT = false, bool PRE = false>
__device__ __forceinline__ void q4k_gemv_body(const Q4KArgs a, uint8_t* lds, int wg) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 7, grp = lane >> 3;
    const int S = 1 << a.log2S;
    const int sub = grp & (S - 1);
    const int rows_per_wave = 8 >> a.log2S;
    const int nblk = a.K / 256;
    const int nb_max = (nblk + S - 1) >> a.log2S;  // passes are sized for the group with the most blocks
    const int tpw = a.tiles_per_wg > 1 ? a.tiles_per_wg : 1;
    const int n_tiles = (a.total_rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave);

    // One row tile: first pass of weight loads, `between` (the activation prologue on the first tile, nothing on the
    // others), block terms, reduction, store.
    auto run_tile = [&](int tile, auto&& between) {
        const int r = (tile * 4 + wave) * rows_per_wave + (grp >> a.log2S);
        const bool live = r < a.total_rows;
        const int rr = live ? r : a.total_rows - 1;
        int mat = 0, local = rr;
        if constexpr (MODE == 1) {
            mat = rr & 1;
            local = rr >> 1;
        } else {
            if (a.n_mat > 1 && rr >= a.row_end[0]) { mat = 1; local = rr - a.row_end[0]; }
            if (a.n_mat > 2 && rr >= a.row_end[1]) { mat = 2; local = rr - a.row_end[1]; }
        }
        const uint8_t* row = (mat == 0 ? a.W[0] : (mat == 1 ? a.W[1] : a.W[2])) + (int64_t)local * a.stride;
        uint4 hdr[NB], qv[NB];
        issue_order_fence();
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const uint8_t* p = row + (int64_t)min(sub + (u << a.log2S), nblk - 1) * 144;
            hdr[u] = *reinterpret_cast<const uint4*>(p);
            qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
        }
        issue_order_fence();
        between();

        // passes roll: a consumed block's registers are refilled from the next pass at once, so a lane group keeps
        // NB - 1 .. NB blocks in flight while it computes; the last pass only consumes
        float acc = 0.0f;
        int i0 = 0;
        for (; i0 + NB < nb_max; i0 += NB) {
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int b = sub + ((i0 + u) << a.log2S);
                const float t = q4k_block_term(hdr[u], qv[u], lds, a.K, min(b, nblk - 1), j);
                acc += b < nblk ? t : 0.0f;
                const uint8_t* p = row + (int64_t)min(sub + ((i0 + NB + u) << a.log2S), nblk - 1) * 144;
                hdr[u] = *reinterpret_cast<const uint4*>(p);
                qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int b = sub + ((i0 + u) << a.log2S);
            const float t = q4k_block_term(hdr[u], qv[u], lds, a.K, min(b, nblk - 1), j);
            acc += b < nblk ? t : 0.0f;
        }
        // reduce: 8 lanes of the group, then the S groups of the row
        float p = sum8(acc);
        if (S >= 2) p += dpp_f<0x128>(p);  // row_ror:8 = the other 8-lane half of the 16-lane row
        if (S >= 4) p += __shfl_xor(p, 16, 64);
        if (S >= 8) p += __shfl_xor(p, 32, 64);

        if constexpr (MODE == 1) {
            // gate and up of one row sit S groups apart
            float other;
            if (S == 1) other = dpp_f<0x128>(p);
            else if (S == 2) other = __shfl_xor(p, 16, 64);
            else other = __shfl_xor(p, 32, 64);
            if (live && mat == 0 && sub == 0 && j == 0) a.y[0][local] = a.gelu ? gelu_mul_ref(p, other) : silu_mul_ref(p, other);
        } else {
            float* y = mat == 0 ? a.y[0] : (mat == 1 ? a.y[1] : a.y[2]);
            if (live && sub == 0 && j == 0) {
                if constexpr (ACC) y[local] += p;
                else y[local] = p;
            }
        }
    };

    // ---- activation loads first, then the first tile's weight loads, then the activation prologue ----
    __shared__ float red[4];
    static_assert(!(PRE && ROLLT), "the deferred post-norm is built into the one-tile-at-a-time form only");
    const Q4KStage stg = q4k_stage_issue<XQ8, NORM, PRE>(a, lds, red);
    if constexpr (ROLLT) {
        // MODE 0: one matrix (a.W[0], a.y[0]); MODE 1: virtual row 2 r = gate row r (a.W[0]), 2 r + 1 = up row r (a.W[1]).
        // The pointers are taken out of the argument struct once: a select over its arrays per tile would push it to scratch.
        const uint8_t* const W0 = a.W[0];
        const uint8_t* const W1 = MODE == 1 ? a.W[1] : a.W[0];
        float* const y0 = a.y[0];
        auto row_ptr = [&](int rv) {   // virtual row (clamped) -> first byte of its weights
            const int rc = min(rv, a.total_rows - 1);
            if constexpr (MODE == 1) return ((rc & 1) ? W1 : W0) + (int64_t)(rc >> 1) * a.stride;
            else return W0 + (int64_t)rc * a.stride;
        };
        const int total_rows = a.total_rows, log2S = a.log2S;
        const int boff = sub * 144, bstep = 144 << log2S;
        int tile = wg * tpw;
        const int tile_end = min(tile + tpw, n_tiles);  // workgroup-uniform; the grid holds no workgroup without a tile
        int r = (tile * 4 + wave) * rows_per_wave + (grp >> log2S);
        const uint8_t* row = row_ptr(r);
        uint4 hdr[NB], qv[NB];
        issue_order_fence();
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const uint8_t* p = row + min(boff + u * bstep, (nblk - 1) * 144);
            hdr[u] = *reinterpret_cast<const uint4*>(p);
            qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
        }
        issue_order_fence();
        q4k_stage_finish<XQ8, NORM>(stg, a, lds, red);
        for (; tile < tile_end; ++tile) {
            const int r_next = tile + 1 < tile_end ? r + 4 * rows_per_wave : r;
            const uint8_t* row_next = row_ptr(r_next);
            float acc = 0.0f;
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int b = sub + (u << log2S);
                const float t = q4k_block_term(hdr[u], qv[u], lds, a.K, min(b, nblk - 1), j);
                acc += b < nblk ? t : 0.0f;
                const uint8_t* p = row_next + min(boff + u * bstep, (nblk - 1) * 144);
                hdr[u] = *reinterpret_cast<const uint4*>(p);
                qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
            }
            float p = sum8(acc);
            if (S >= 2) p += dpp_f<0x128>(p);
            if (S >= 4) p += __shfl_xor(p, 16, 64);
            if (S >= 8) p += __shfl_xor(p, 32, 64);
            if constexpr (MODE == 1) {
                // gate and up of one row sit S groups apart
                float other;
                if (S == 1) other = dpp_f<0x128>(p);
                else if (S == 2) other = __shfl_xor(p, 16, 64);
                else other = __shfl_xor(p, 32, 64);
                if (r < total_rows && (r & 1) == 0 && sub == 0 && j == 0)
                    y0[r >> 1] = a.gelu ? gelu_mul_ref(p, other) : silu_mul_ref(p, other);
            } else {
                if (r < total_rows && sub == 0 && j == 0) {
                    if constexpr (ACC) y0[r] += p;
                    else y0[r] = p;
                }
            }
            r = r_next;
        }
        return;
    }
    run_tile(wg * tpw, [&] { q4k_stage_finish<XQ8, NORM, PRE>(stg, a, lds, red, wg); });
    // further tiles reuse the staged activations: the quantisation of x is paid once per workgroup
    for (int k = 1; k < tpw; ++k) {
        const int tile = wg * tpw + k;
        if (tile >= n_tiles) break;
        run_tile(tile, [] {});
    }
}

// lane groups per row: enough workgroups to cover the chip, and all of a group's blocks in one pass
inline int q4k_pick_log2S(int total_rows, int nblk, int max_log2S) {
    int l = 0;
    while (l < max_log2S) {
        const int S = 1 << l;
        const int wgs = (total_rows * S + 31) / 32;
        const int nb = (nblk + S - 1) / S;
        if (nb <= 5 && wgs >= 600) break;  // 5 blocks in flight per group: measured better than 10 (registers -> occupancy)
        if (nb <= 1) break;
        ++l;
    }
    return l;
}
inline int q4k_workgroups(int total_rows, int log2S) {
    const int rows_per_wg = 32 >> log2S;
    return (total_rows + rows_per_wg - 1) / rows_per_wg;
}
// Row tiles per workgroup: beyond ~1200 tiles a workgroup walks several, so that the activation prologue (every
// workgroup quantises the whole vector) is amortised.
inline int q4k_tiles_per_wg(int n_tiles) {
    const int max_wgs = 1280;
    int t = 1;
    while (t < 8 && (n_tiles + t - 1) / t > max_wgs) ++t;
    return t;
}
// The same for the kernel whose loads roll across a workgroup's tiles (q4k_gemv_tall_kernel): at most 768 workgroups, all
// resident at once (151936 x 2560: 9496 tiles; 2048 / 1024 / 768 / 512 workgroups measured 42.2 / 41.7 / 41.5 / 41.0 us).
inline int q4k_tiles_per_wg_rolling(int n_tiles) {
    const int t = (n_tiles + 767) / 768;
    return t > 16 ? 16 : t;
}
inline int q4k_blocks_per_pass(int nblk, int log2S) {
    static const int cand[] = {2, 3, 4, 5, 10};
    return pick_blocks_per_pass((nblk + (1 << log2S) - 1) >> log2S, cand, 5);
}

}  // namespace ptm
