// Split-KV single-token GQA attention for gfx950 (wave64).
//
// Same mathematics as the reference's single-token attention (torch/io/gguf_model.h:3510-3636:
// s_t = (q.k_t)*scale, softmax over t in [0, total), out = sum_t p_t v_t) and the same split /
// merge structure as its flash-decode kernels (aten/src/ATen/cuda/FlashDecoding.cu:33-200),
// re-laid out for MI355X:
//   * one workgroup per (kv head, chunk of 64 positions) serves ALL query heads of the GQA
//     group, so each K/V row is fetched once instead of once per query head;
//   * a K/V row of head_dim halfs is fetched by head_dim/8 lanes with 128-bit loads (a wave
//     covers 4 rows of 128 halfs per load), q lives in registers;
//   * the position count is read from device memory so the launch is graph-replayable;
//     workgroups past the end exit at once.
#include "ptm_common.h"

namespace ptm {

enum { FD_CHUNK = 64, FD_THREADS = 256 };
enum { FD_LONG_SPLITS = 64 };   // partials per head of the looping kernel for long caches (attn_decode_mfma_long_kernel)

// e^x through the hardware base-2 exponential (v_exp_f32, 1 ulp): softmax weights need no more, and the libm
// expf expands to a dozen instructions on a path whose cost is instruction count.  -inf gives 0.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }
// 1/sqrt(x) through v_rsq_f32 (1 ulp) for the per-head RMS scale.
__device__ __forceinline__ float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }

template <bool KV16>
__device__ __forceinline__ void load8(const void* base, int64_t elem_off, float (&o)[8]) {
    if constexpr (KV16) {
        const uint4 r = *reinterpret_cast<const uint4*>(static_cast<const __half*>(base) + elem_off);
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = h2f(w[i]);
            o[2 * i + 1] = h2f(w[i] >> 16);
        }
    } else {
        const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + elem_off);
        const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + elem_off + 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
        o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
}

// Workgroup index -> (chunk, kv head).  Workgroups are dispatched in index order.  Chunks run fastest within a head (the
// workgroups that start together then read rows far apart: with the head fastest, eight of them read adjacent 256-byte
// pieces of the same rows and the launch took 0.6 us longer), but only in blocks of 64 chunks: all heads' chunks 0..63
// come before any head's chunk 64, so that with a cache far longer than the context the live chunks of every head start
// before the thousands of workgroups that only look at the position and leave.
enum { FD_ORDER_BLOCK = 64 };
__device__ __forceinline__ int fd_lin(int bx, int by, int gx) { return bx + gx * by; }
__device__ __forceinline__ int fd_split_of(int bx, int by, int gx, int gy) {
    const int lin = fd_lin(bx, by, gx), per = FD_ORDER_BLOCK * gy;
    const int blk = lin / per, r = lin - blk * per;
    const int width = min(FD_ORDER_BLOCK, gx - blk * FD_ORDER_BLOCK);   // chunks in this block (the last may be narrower)
    return blk * FD_ORDER_BLOCK + r % width;
}
__device__ __forceinline__ int fd_head_of(int bx, int by, int gx, int gy) {
    const int lin = fd_lin(bx, by, gx), per = FD_ORDER_BLOCK * gy;
    const int blk = lin / per, r = lin - blk * per;
    const int width = min(FD_ORDER_BLOCK, gx - blk * FD_ORDER_BLOCK);
    return r / width;
}

// What a FUSED launch of the kernel below does first: per-head RMSNorm (optional) + rotation of the raw q heads and, in
// the workgroup whose chunk holds the new position, of the raw k row, and the K/V append.
struct FdFuse {
    const float *K, *V, *qw, *kw, *rope;  // raw new k / v rows [kv_dim], norm weights (both or neither), table [max_seq][HD]
    float eps;
    int add_one, rope_interleaved;
};

// Raw values of one item of the FUSED prologue (a query head or the new k row) as a lane holds them: rotation pairs
// lane and lane + 64 (clamped into the head where the head has fewer pairs), their norm weights, the rotation row, and the
// v row's values at the same places.
struct FdItem { float x0[2], x1[2], n0[2], n1[2], c[2], s[2], v0[2], v1[2]; };
template <int HD>
__device__ __forceinline__ FdItem fd_item_load(const float* src, const float* nw, const float* cs, const float* vrow,
                                               int interleaved, int lane) {
    constexpr int HALF = HD / 2;
    const float* nwp = nw ? nw : src;  // a valid address either way; unused without norm weights
    FdItem e;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int t = min(lane + 64 * j, HALF - 1);
        const int i0 = interleaved ? 2 * t : t, i1 = interleaved ? 2 * t + 1 : t + HALF;
        e.x0[j] = src[i0];
        e.x1[j] = src[i1];
        e.n0[j] = nwp[i0];
        e.n1[j] = nwp[i1];
        e.c[j] = cs[t];
        e.s[j] = cs[HALF + t];
        e.v0[j] = vrow[t];
        e.v1[j] = vrow[t + HALF];
    }
    return e;
}

// grid (max_splits, n_kv_heads); G = query heads per kv head; HD = head_dim.  FUSED: Q holds the raw projections and
// the caches are appended to (the one-launch form for heads wider than the fused kernel further down covers).
template <bool KV16, int HD, int G, bool FUSED = false>
__global__ __launch_bounds__(FD_THREADS) void flash_decode_partial_kernel(
    const float* __restrict__ Q, void* __restrict__ Kc, void* __restrict__ Vc,
    float* __restrict__ pO, float* __restrict__ pL, float* __restrict__ pM, int n_heads, int n_kv_heads,
    const int64_t* __restrict__ d_past, int64_t past_host, int max_seq, float scale, int window, const FdFuse f) {
    constexpr int LPP = HD / 8;         // lanes per position (each lane owns 8 dims)
    constexpr int PPW = 64 / LPP;       // positions per wave per pass
    constexpr int PPB = PPW * 4;        // positions per workgroup per pass
    constexpr int NPASS = FD_CHUNK / PPB;
    __shared__ float s_p[G][FD_CHUNK];
    __shared__ float s_o[4][G][HD];
    __shared__ float s_q[FUSED ? G : 1][FUSED ? HD : 1];
    __shared__ float s_new[2][FUSED ? HD : 1];

    // d_past == NULL: the position is the host argument (launch_flash_decode's total_seq, CUDAOps.h:543-549)
    int64_t total = (d_past ? *d_past : past_host) + 1;
    if constexpr (FUSED) {
        if (total <= 0 || total > max_seq) return;  // never touch memory outside the cache
    }
    if (total > max_seq) total = max_seq;
    const int split = fd_split_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y), kvh = fd_head_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y);
    const int64_t t0 = (int64_t)split * FD_CHUNK;
    if (t0 >= total) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // window > 0: only positions [total - window, total) count; a chunk wholly in front of them leaves an empty partial
    const int64_t t_begin = (window > 0 && total > window) ? total - window : 0;
    if (t0 + FD_CHUNK <= t_begin) {
        for (int e = tid; e < G * HD; e += FD_THREADS) {
            const int g = e / HD, d = e % HD;
            const int64_t oi = (int64_t)split * n_heads + kvh * G + g;
            pO[oi * HD + d] = 0.0f;
            if (d == 0) { pM[oi] = -INFINITY; pL[oi] = 0.0f; }
        }
        return;
    }
    const int dl = lane % LPP, pl = lane / LPP;
    const int kv_dim = n_kv_heads * HD;
    const int64_t col = (int64_t)kvh * HD + dl * 8;
    const int64_t past = total - 1;

    // FUSED: what this wave's first item of the prologue needs (wave w prepares query heads w, w + 4, ..., then, in the
    // workgroup that owns the new position, the new k row; a lane owns rotation pairs lane and lane + 64) is requested
    // FIRST and unconditionally, from addresses that are valid for every wave: loads return in order, so behind the cache
    // rows these few values would wait for all of them, and under a branch the compiler would wait for everything in flight.
    static_assert(!FUSED || HD == 256, "the fused prologue is laid out for heads of 256 (two rotation pairs per lane)");
    constexpr int HALF = HD / 2;
    FdItem first{};
    if constexpr (FUSED) {
        const bool k_item = wave >= G;  // waves past the query heads fetch the k row (used by the owner's wave G only)
        first = fd_item_load<HD>(k_item ? f.K + (int64_t)kvh * HD : Q + (int64_t)(kvh * G + wave) * HD, k_item ? f.kw : f.qw,
                                 f.rope + past * HD, f.V + (int64_t)kvh * HD, f.rope_interleaved, lane);
        issue_order_fence();
    }

    // ---- all K and V rows of the chunk are requested up front: one HBM round trip (FUSED: the new position's row is
    // not in the cache yet, it comes from LDS below) ----
    float kreg[NPASS][8], vreg[NPASS][8];
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int64_t t = t0 + pass * PPB + wave * PPW + pl;
        const int64_t last = FUSED ? (past > 0 ? past - 1 : 0) : total - 1;
        const int64_t tc = t <= last ? t : last;
        load8<KV16>(Kc, tc * kv_dim + col, kreg[pass]);
        load8<KV16>(Vc, tc * kv_dim + col, vreg[pass]);
    }

    float q[G][8];
    if constexpr (FUSED) {
        issue_order_fence();
        const bool owner = past >= t0 && past < t0 + FD_CHUNK;
        const float one = f.add_one ? 1.0f : 0.0f;
        // norm + rotation of one item from its loaded values; query heads go to s_q, the k row (with the v row) to the cache
        // and to s_new
        auto finish = [&](int it, FdItem& e) {
            const bool is_k = it == G;
            if ((is_k ? f.kw : f.qw) != nullptr) {
                float ss = fmaf(e.x0[0], e.x0[0], 0.0f);
                ss = fmaf(e.x1[0], e.x1[0], ss);
                ss = fmaf(e.x0[1], e.x0[1], ss);
                ss = fmaf(e.x1[1], e.x1[1], ss);
                ss = sum64(ss);
                const float rs = 1.0f / sqrtf(ss / (float)HD + f.eps);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    e.x0[j] = e.x0[j] * rs * (e.n0[j] + one);
                    e.x1[j] = e.x1[j] * rs * (e.n1[j] + one);
                }
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int t = lane + 64 * j;
                if (t >= HALF) continue;
                const int i0 = f.rope_interleaved ? 2 * t : t, i1 = f.rope_interleaved ? 2 * t + 1 : t + HALF;
                float r0 = fmaf(e.x0[j], e.c[j], -(e.x1[j] * e.s[j])), r1 = fmaf(e.x0[j], e.s[j], e.x1[j] * e.c[j]);
                if (!is_k) {
                    s_q[it][i0] = r0;
                    s_q[it][i1] = r1;
                } else {
                    const int64_t rowoff = past * kv_dim + (int64_t)kvh * HD;
                    float v0 = e.v0[j], v1 = e.v1[j];
                    if constexpr (KV16) {
                        const __half h0 = __float2half_rn(r0), h1 = __float2half_rn(r1), g0 = __float2half_rn(v0), g1 = __float2half_rn(v1);
                        __half* kc = static_cast<__half*>(Kc) + rowoff;
                        __half* vc = static_cast<__half*>(Vc) + rowoff;
                        kc[i0] = h0; kc[i1] = h1; vc[t] = g0; vc[t + HALF] = g1;
                        r0 = __half2float(h0); r1 = __half2float(h1); v0 = __half2float(g0); v1 = __half2float(g1);
                    } else {
                        float* kc = static_cast<float*>(Kc) + rowoff;
                        float* vc = static_cast<float*>(Vc) + rowoff;
                        kc[i0] = r0; kc[i1] = r1; vc[t] = v0; vc[t + HALF] = v1;
                    }
                    s_new[0][i0] = r0; s_new[0][i1] = r1;
                    s_new[1][t] = v0; s_new[1][t + HALF] = v1;
                }
            }
        };
        const int n_items = G + (owner ? 1 : 0);
        if (wave < n_items) finish(wave, first);
        for (int it = wave + 4; it < n_items; it += 4) {  // more than three query heads per kv head: further items, fetched here
            const bool is_k = it == G;
            FdItem e = fd_item_load<HD>(is_k ? f.K + (int64_t)kvh * HD : Q + (int64_t)(kvh * G + it) * HD, is_k ? f.kw : f.qw,
                                        f.rope + past * HD, f.V + (int64_t)kvh * HD, f.rope_interleaved, lane);
            finish(it, e);
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 8; ++i) q[g][i] = s_q[g][dl * 8 + i];
#pragma unroll
        for (int pass = 0; pass < NPASS; ++pass) {
            if (t0 + pass * PPB + wave * PPW + pl == past) {
#pragma unroll
                for (int i = 0; i < 8; ++i) { kreg[pass][i] = s_new[0][dl * 8 + i]; vreg[pass][i] = s_new[1][dl * 8 + i]; }
            }
        }
    } else {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float4 a = *reinterpret_cast<const float4*>(Q + (int64_t)(kvh * G + g) * HD + dl * 8);
            const float4 b = *reinterpret_cast<const float4*>(Q + (int64_t)(kvh * G + g) * HD + dl * 8 + 4);
            q[g][0] = a.x; q[g][1] = a.y; q[g][2] = a.z; q[g][3] = a.w;
            q[g][4] = b.x; q[g][5] = b.y; q[g][6] = b.z; q[g][7] = b.w;
        }
    }

    // ---- scores ----
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int tl = pass * PPB + wave * PPW + pl;
        const bool valid = t0 + tl < total && t0 + tl >= t_begin;
        if (!valid) {  // a position that does not count holds a clamped row, possibly never written: 0 * garbage must not be NaN
#pragma unroll
            for (int i = 0; i < 8; ++i) vreg[pass][i] = 0.0f;
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) d = fmaf(q[g][i], kreg[pass][i], d);
            d = sum_lanes<LPP>(d);
            if (dl == 0) s_p[g][tl] = valid ? d * scale : -INFINITY;
        }
    }
    __syncthreads();

    // ---- chunk softmax statistics: wave w handles heads w, w+4, ... ; lane = position ----
    for (int g = wave; g < G; g += 4) {
        const float s = s_p[g][lane];
        const float m = max64(s);
        const float p = expf(s - m);  // -inf - m -> 0
        const float l = sum64(p);
        s_p[g][lane] = p;
        if (lane == 0) {
            const int64_t o = (int64_t)split * n_heads + kvh * G + g;
            pM[o] = m;
            pL[o] = l;
        }
    }
    __syncthreads();

    // ---- weighted V ----
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int tl = pass * PPB + wave * PPW + pl;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float p = s_p[g][tl];
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(p, vreg[pass][i], acc[g][i]);
        }
    }
    // reduce over the PPW position slots of the wave (lanes with equal dl), then over waves
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float a = acc[g][i];
            for (int off = LPP; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
            acc[g][i] = a;
        }
    if (pl == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 8; ++i) s_o[wave][g][dl * 8 + i] = acc[g][i];
    }
    __syncthreads();
    for (int e = tid; e < G * HD; e += FD_THREADS) {
        const int g = e / HD, d = e % HD;
        const float o = (s_o[0][g][d] + s_o[1][g][d]) + (s_o[2][g][d] + s_o[3][g][d]);
        pO[((int64_t)split * n_heads + kvh * G + g) * HD + d] = o;
    }
}

// Merge of the active splits: grid n_heads, 256 threads = NSLOT split-slots x HD/4 float4 outputs.
// Slot r sums splits r, r+NSLOT, ... in batches of 8 independent loads (the first batch is issued
// before the max/denominator reductions so its latency overlaps them); slot sums are then added in
// slot order, so the result does not depend on timing.
template <int HD>
__global__ __launch_bounds__(256) void flash_decode_merge_kernel(const float* __restrict__ pO,
                                                                 const float* __restrict__ pL,
                                                                 const float* __restrict__ pM, float* __restrict__ O,
                                                                 int n_heads, const int64_t* __restrict__ d_past,
                                                                 int64_t past_host, int max_seq,
                                                                 uint8_t* __restrict__ q8_out, int chunk_shift, int log2_units) {
    constexpr int NOUT = HD / 4, NSLOT = 256 / NOUT;
    __shared__ __align__(16) float4 s_stage[256];
    __shared__ float s_red[8];
    const int h = blockIdx.x, tid = threadIdx.x;
    const int o_idx = tid % NOUT, slot = tid / NOUT;
    const float4* pO4 = reinterpret_cast<const float4*>(pO);
    // Every load of the common case goes out before the position is known: chunk slots past the last active one
    // are clamped into the allocation (ns_max chunks) and dropped by selects below, so the kernel makes one
    // memory round trip, not one for the position and a second for the data.
    // chunk_shift < 0: the partials of the looping kernel (at most FD_LONG_SPLITS of them, cpw chunks of 64 positions each)
    const bool long_mode = chunk_shift < 0;
    const int chunk = long_mode ? FD_CHUNK : 1 << chunk_shift;  // positions per chunk
    const int cs_ = long_mode ? 6 : chunk_shift;
    const int ns_max = long_mode ? min((max_seq + chunk - 1) >> cs_, (int)FD_LONG_SPLITS) : (max_seq + chunk - 1) >> cs_;
    const int64_t past = d_past ? *d_past : past_host;
    // partial maxima are natural-log scores, or base-2 ones (log2_units) from the matrix-core kernel
    const float ek = log2_units ? 1.0f : 1.44269504088896340736f;
    auto wexp = [ek](float x) { return __builtin_amdgcn_exp2f(x * ek); };
    float4 v[8];
    float mm[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int sc = min(slot + u * NSLOT, ns_max - 1);
        v[u] = pO4[((int64_t)sc * n_heads + h) * NOUT + o_idx];
        mm[u] = pM[(int64_t)sc * n_heads + h];
    }
    const int s_first = min(tid, ns_max - 1);
    const float pm_first = pM[(int64_t)s_first * n_heads + h], pl_first = pL[(int64_t)s_first * n_heads + h];
    int64_t total = past + 1;
    if (total > max_seq) total = max_seq;
    if (total <= 0) return;
    const int n_chunks = (int)((total + chunk - 1) >> cs_);
    const int cpw_ = long_mode ? (n_chunks + (int)FD_LONG_SPLITS - 1) / (int)FD_LONG_SPLITS : 1;
    const int ns = long_mode ? (n_chunks + cpw_ - 1) / cpw_ : n_chunks;
    float m = tid < ns ? pm_first : -INFINITY;
    for (int sI = tid + 256; sI < ns; sI += 256) m = fmaxf(m, pM[(int64_t)sI * n_heads + h]);
    m = max64(m);
    if ((tid & 63) == 0) s_red[tid >> 6] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    float den = tid < ns ? wexp(pm_first - M) * pl_first : 0.0f;
    for (int sI = tid + 256; sI < ns; sI += 256)
        den = fmaf(wexp(pM[(int64_t)sI * n_heads + h] - M), pL[(int64_t)sI * n_heads + h], den);
    den = sum64(den);
    if ((tid & 63) == 0) s_red[4 + (tid >> 6)] = den;
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = slot; s0 < ns; s0 += NSLOT * 8) {
        if (s0 != slot) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int sc = min(s0 + u * NSLOT, ns - 1);
                v[u] = pO4[((int64_t)sc * n_heads + h) * NOUT + o_idx];
                mm[u] = pM[(int64_t)sc * n_heads + h];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const bool on = (s0 + u * NSLOT) < ns;  // a select, not a zero weight: inactive slots may hold anything
            const float w = wexp(mm[u] - M);
            sum.x = on ? fmaf(w, v[u].x, sum.x) : sum.x;
            sum.y = on ? fmaf(w, v[u].y, sum.y) : sum.y;
            sum.z = on ? fmaf(w, v[u].z, sum.z) : sum.z;
            sum.w = on ? fmaf(w, v[u].w, sum.w) : sum.w;
        }
    }
    s_stage[slot * NOUT + o_idx] = sum;
    __syncthreads();
    if (tid < NOUT) {
        float4 t = s_stage[tid];
        for (int r = 1; r < NSLOT; ++r) {
            const float4 u = s_stage[r * NOUT + tid];
            t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
        }
        const float dsum = (s_red[4] + s_red[5]) + (s_red[6] + s_red[7]);
        const float inv = 1.0f / (dsum + 1e-10f);  // reference: inv_sum = 1/(sum_exp + 1e-10f), gguf_model.h:3589
        const float4 o4 = make_float4(t.x * inv, t.y * inv, t.z * inv, t.w * inv);
        reinterpret_cast<float4*>(O)[(int64_t)h * NOUT + tid] = o4;
        if (q8_out) {
            // the same vector as Q8 blocks (int8 qs[K] | float d[K/32] | float sum[K/32], K = n_heads * HD) for a Q4_K
            // output projection, whose prologue then copies 1.25 bytes per value instead of quantising 4
            const int K = n_heads * HD;
            float d, sm;
            const uint32_t packed = q8_quantize4(o4, d, sm);  // 8 consecutive lanes hold one block of 32
            reinterpret_cast<uint32_t*>(q8_out)[(int64_t)h * NOUT + tid] = packed;
            if ((tid & 7) == 0) {
                float* dd = reinterpret_cast<float*>(q8_out + K);
                const int blk = h * (HD / 32) + (tid >> 3);
                dd[blk] = d;
                dd[K / 32 + blk] = sm;
            }
        }
    }
}

static int fd_merge(int head_dim, int n_heads, hipStream_t s, const float* pO, const float* pL, const float* pM, float* O,
                    const int64_t* d_past, int max_seq, uint8_t* q8_out = nullptr, int64_t past_host = 0,
                    int chunk = FD_CHUNK, int log2_units = 0) {
    const int chunk_shift = chunk < 0 ? -1 : chunk == 128 ? 7 : 6;
    if (head_dim == 256)
        hipLaunchKernelGGL(flash_decode_merge_kernel<256>, dim3(n_heads), dim3(256), 0, s, pO, pL, pM, O, n_heads, d_past, past_host, max_seq, q8_out, chunk_shift, log2_units);
    else if (head_dim == 128)
        hipLaunchKernelGGL(flash_decode_merge_kernel<128>, dim3(n_heads), dim3(256), 0, s, pO, pL, pM, O, n_heads, d_past, past_host, max_seq, q8_out, chunk_shift, log2_units);
    else
        hipLaunchKernelGGL(flash_decode_merge_kernel<64>, dim3(n_heads), dim3(256), 0, s, pO, pL, pM, O, n_heads, d_past, past_host, max_seq, q8_out, chunk_shift, log2_units);
    return launch_status();
}

// ---------------------------------------------------------------------------------------------
// Front half of the attention step of one token in ONE launch: per-head QK-norm + NeoX RoPE of q and
// of the new k row, K/V cache append, and the split-KV partial attention over the cache.
//   * every workgroup normalises/rotates the 4..8 query heads it needs itself (512..1024 values);
//   * the workgroup whose chunk contains the new position also produces the new K/V row, writes it
//     to the cache and uses it from LDS (the cache row is not yet visible to its own loads).
// The split merge stays a second, small launch.  Doing it in the workgroup of a kv head that arrives last was measured
// twice on MI355X and lost both times: with device-scope release/acquire fences in all ~270 workgroups (an L2 write-back per
// fence across the 8 XCDs), and with write-through partial stores, a relaxed device-scope arrival counter and one round of
// 20 write-through-coherent loads per thread (store acknowledgement + atomic + load round trip behind the slowest workgroup:
// 1579 against 1568 us per Qwen3-4B token with the second launch).
// The kernel's cost is instruction latency (about one wave per SIMD, each with a long dependent chain), not the
// 8.6 MB of KV it reads, so the arithmetic is kept short: hardware exp2 / rsq, no barrier before the final merge.
// ---------------------------------------------------------------------------------------------
struct AttnArgs {
    const float *Q, *K, *V, *qw, *kw, *rope;
    void *Kc, *Vc;
    float *pO, *pL, *pM;
    const int64_t* d_past;
    int n_heads, n_kv_heads, max_seq, add_one;
    float scale, eps;
    int rope_interleaved;  // 0: NeoX pairs (d, d + HD/2); 1: pairs (2d, 2d + 1) as llama / mistral rotate (hot_loops.cpp:1962-2030)
    int window;            // > 0: only the last `window` positions are attended to (gemma3 local layers, gguf_model.h:3490-3500)
    // biases of the q / k / v projections (qwen2, gguf_model.h:3419-3431), added to the raw vectors before norm and rotation
    // by the kernels instantiated with BIAS; null otherwise
    const float *qb, *kb, *vb;
};

// one wave: RMSNorm (optional) + NeoX rotation of a head held as pairs (t, t+HD/2); results to dst[HD]
template <int HD>
__device__ __forceinline__ void head_norm_rope(const float* __restrict__ src, const float* __restrict__ w,
                                               const float* __restrict__ cs, float eps, int add_one, int lane,
                                               float& r0, float& r1) {
    constexpr int HALF = HD / 2;
    const bool on = lane < HALF;
    float x0 = on ? src[lane] : 0.0f, x1 = on ? src[lane + HALF] : 0.0f;
    if (w) {
        float ss = fmaf(x0, x0, 0.0f);
        ss = fmaf(x1, x1, ss);
        ss = sum64(ss);
        const float rs = 1.0f / sqrtf(ss / (float)HD + eps);
        const float one = add_one ? 1.0f : 0.0f;
        if (on) {
            x0 = x0 * rs * (w[lane] + one);
            x1 = x1 * rs * (w[lane + HALF] + one);
        }
    }
    const float c = on ? cs[lane] : 1.0f, s = on ? cs[HALF + lane] : 0.0f;
    r0 = fmaf(x0, c, -(x1 * s));
    r1 = fmaf(x0, s, x1 * c);
}

// Sum of N accumulators over the position slots of a wave (lanes with equal dl = lane % LPP), without LDS
// traffic.  v_permlane32_swap exchanges lanes 32..63 of one register with lanes 0..31 of another, so ONE swap
// and ONE add reduce TWO accumulators over the two wave halves (the first then lives in lanes 0..31, the second
// in lanes 32..63); v_permlane16_swap does the same for odd/even rows of 16 lanes.  After both steps register k
// of the result holds, in row r of the wave, the total of accumulator 4k + {0, 2, 1, 3}[r].
template <int N, int LPP>
__device__ __forceinline__ void reduce_position_slots(float (&acc)[N], float (&out)[N / 4]) {
    static_assert(N % 4 == 0, "accumulator count must be a multiple of 4");
    if constexpr (LPP == 8) {
#pragma unroll
        for (int k = 0; k < N; ++k) acc[k] += dpp_f<0x128>(acc[k]);  // row_ror:8 adds the other 8-lane half of the row
    }
    float half[N / 2];
#pragma unroll
    for (int k = 0; k < N / 2; ++k) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[2 * k]), __float_as_uint(acc[2 * k + 1]), false, false);
        half[k] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
#pragma unroll
    for (int k = 0; k < N / 4; ++k) {
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(half[2 * k]), __float_as_uint(half[2 * k + 1]), false, false);
        out[k] = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
}

// Every wave works on its own 16 (HD 128) or 32 (HD 64) positions of the chunk from the loads to a wave-local
// softmax partial (max, sum, weighted V); the four partials are merged through LDS behind a workgroup barrier.  The
// query heads are prepared once per workgroup (wave w takes heads w, w + 4, ...; one more barrier, measured 0.1 us better
// than every wave preparing all of them); the new K/V row each wave prepares for itself.
template <bool KV16, int HD, int G>
__global__ __launch_bounds__(FD_THREADS) void attn_decode_fused_kernel(const AttnArgs a) {
    constexpr int LPP = HD / 8, PPW = 64 / LPP, PPB = PPW * 4, NPASS = FD_CHUNK / PPB, HALF = HD / 2;
    __shared__ float s_q[G][HD];
    __shared__ float s_new[4][2][HD];
    __shared__ float s_o[4][G][HD];
    __shared__ float s_m[4][G], s_l[4][G];

    const int64_t past = *a.d_past;
    if (past < 0 || past >= a.max_seq) return;          // never touch memory outside the cache
    const int64_t total = past + 1;
    const int split = fd_split_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y), kvh = fd_head_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y);
    const int64_t t0 = (int64_t)split * FD_CHUNK;
    if (t0 >= total) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t t_begin = (a.window > 0 && total > a.window) ? total - a.window : 0;
    if (t0 + FD_CHUNK <= t_begin) {
        // a chunk wholly in front of the window: an empty partial (weight exp(-inf - M) = 0 in the merge)
        for (int e = tid; e < G * HD; e += FD_THREADS) {
            const int g = e / HD, d = e % HD;
            const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
            a.pO[oi * HD + d] = 0.0f;
            if (d == 0) { a.pM[oi] = -INFINITY; a.pL[oi] = 0.0f; }
        }
        return;
    }
    const int dl = lane % LPP, pl = lane / LPP;
    const int kv_dim = a.n_kv_heads * HD;
    const int64_t col = (int64_t)kvh * HD + dl * 8;
    const bool owner = past >= t0 && past < t0 + FD_CHUNK;
    const bool on = lane < HALF;
    const int lh = lane & (HALF - 1);
    const bool has_norm = a.qw != nullptr;

    // ---- loads, all unconditional so that their count is static: first the few values of the prologue ... ----
    const float* cs = a.rope + past * HD;
    const float* qwp = has_norm ? a.qw : a.Q;  // a valid address either way; unused without norm weights
    const float* kwp = has_norm ? a.kw : a.Q;
    // lane lh owns rotation pair lh: elements (i0, i1) of a head
    const int i0 = a.rope_interleaved ? 2 * lh : lh, i1 = a.rope_interleaved ? 2 * lh + 1 : lh + HALF;
    float qx0[G], qx1[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float* src = a.Q + (int64_t)(kvh * G + g) * HD;
        qx0[g] = src[i0];
        qx1[g] = src[i1];
    }
    const float qn0 = qwp[i0], qn1 = qwp[i1], kn0 = kwp[i0], kn1 = kwp[i1];
    const float rc = cs[lh], rsn = cs[HALF + lh];
    float kx0 = a.K[(int64_t)kvh * HD + i0], kx1 = a.K[(int64_t)kvh * HD + i1];
    float vx0 = a.V[(int64_t)kvh * HD + lh], vx1 = a.V[(int64_t)kvh * HD + lh + HALF];
    issue_order_fence();
    // ---- ... then the cached K/V rows of this wave's positions (the new position is not cached: clamp below it) ----
    float kreg[NPASS][8], vreg[NPASS][8];
    const int64_t last_cached = past > 0 ? past - 1 : 0;
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int64_t t = t0 + pass * PPB + wave * PPW + pl;
        const int64_t tc = t < past ? t : last_cached;
        load8<KV16>(a.Kc, tc * kv_dim + col, kreg[pass]);
        load8<KV16>(a.Vc, tc * kv_dim + col, vreg[pass]);
    }
    issue_order_fence();

    // ---- per-head RMSNorm + NeoX rotation of the G query heads and of the new K row; V row as is ----
    const float one = a.add_one ? 1.0f : 0.0f;
    // wave w prepares query heads w, w + 4, ... for the whole workgroup
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if ((g & 3) != wave) continue;  // wave-uniform
        float x0 = on ? qx0[g] : 0.0f, x1 = on ? qx1[g] : 0.0f;
        if (has_norm) {
            float ss = fmaf(x0, x0, 0.0f);
            ss = fmaf(x1, x1, ss);
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
            x0 = x0 * rs * (qn0 + one);
            x1 = x1 * rs * (qn1 + one);
        }
        if (on) {
            s_q[g][i0] = fmaf(x0, rc, -(x1 * rsn));
            s_q[g][i1] = fmaf(x0, rsn, x1 * rc);
        }
    }
    if (owner) {  // workgroup-uniform
        float x0 = on ? kx0 : 0.0f, x1 = on ? kx1 : 0.0f;
        if (has_norm) {
            float ss = fmaf(x0, x0, 0.0f);
            ss = fmaf(x1, x1, ss);
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
            x0 = x0 * rs * (kn0 + one);
            x1 = x1 * rs * (kn1 + one);
        }
        float r0 = fmaf(x0, rc, -(x1 * rsn)), r1 = fmaf(x0, rsn, x1 * rc);
        const int64_t rowoff = past * kv_dim + (int64_t)kvh * HD;
        if constexpr (KV16) {
            const __half h0 = __float2half_rn(r0), h1 = __float2half_rn(r1), g0 = __float2half_rn(vx0), g1 = __float2half_rn(vx1);
            if (on && wave == 0) {
                static_cast<__half*>(a.Kc)[rowoff + i0] = h0;
                static_cast<__half*>(a.Kc)[rowoff + i1] = h1;
                static_cast<__half*>(a.Vc)[rowoff + lane] = g0;
                static_cast<__half*>(a.Vc)[rowoff + lane + HALF] = g1;
            }
            r0 = __half2float(h0); r1 = __half2float(h1); vx0 = __half2float(g0); vx1 = __half2float(g1);
        } else {
            if (on && wave == 0) {
                static_cast<float*>(a.Kc)[rowoff + i0] = r0;
                static_cast<float*>(a.Kc)[rowoff + i1] = r1;
                static_cast<float*>(a.Vc)[rowoff + lane] = vx0;
                static_cast<float*>(a.Vc)[rowoff + lane + HALF] = vx1;
            }
        }
        if (on) {
            s_new[wave][0][i0] = r0;
            s_new[wave][0][i1] = r1;
            s_new[wave][1][lane] = vx0;
            s_new[wave][1][lane + HALF] = vx1;
        }
    }
    __syncthreads();  // the query heads come from the other waves (the new row's values stay within their wave)

    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) q[g][i] = s_q[g][dl * 8 + i];

    // ---- scores of this wave's positions; every lane of a position's lane group ends up with the score ----
    float sc[G][NPASS];
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int64_t t = t0 + pass * PPB + wave * PPW + pl;
        if (t == past) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { kreg[pass][i] = s_new[wave][0][dl * 8 + i]; vreg[pass][i] = s_new[wave][1][dl * 8 + i]; }
        }
        const bool valid = t < total && t >= t_begin;
        if (!valid) {  // rows past the end or in front of the window carry weight 0; keep 0 * garbage from producing NaN
#pragma unroll
            for (int i = 0; i < 8; ++i) vreg[pass][i] = 0.0f;
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) d = fmaf(q[g][i], kreg[pass][i], d);
            d = sum_lanes<LPP>(d);
            sc[g][pass] = valid ? d * a.scale : -INFINITY;
        }
    }
    // ---- wave-local softmax statistics and weighted V ----
    float acc[G * 8];
    float wm[G], wl[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float m = sc[g][0];
#pragma unroll
        for (int pass = 1; pass < NPASS; ++pass) m = fmaxf(m, sc[g][pass]);
        for (int off = LPP; off < 64; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        const float ms = m == -INFINITY ? 0.0f : m;  // a wave without valid positions contributes nothing
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g * 8 + i] = 0.0f;
#pragma unroll
        for (int pass = 0; pass < NPASS; ++pass) {
            const float p = fast_exp(sc[g][pass] - ms);  // -inf -> 0
            l += p;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g * 8 + i] = fmaf(p, vreg[pass][i], acc[g * 8 + i]);
        }
        for (int off = LPP; off < 64; off <<= 1) l += __shfl_xor(l, off, 64);
        wm[g] = m;
        wl[g] = l;
    }
    float red[G * 2];
    reduce_position_slots<G * 8, LPP>(acc, red);
    {
        const int row = lane >> 4;                       // 16-lane row of the wave
        const int sel = ((row & 1) << 1) | (row >> 1);   // {0, 2, 1, 3}[row]
        if (LPP == 16 || (lane & 8) == 0) {
#pragma unroll
            for (int k = 0; k < G * 2; ++k) {
                const int idx = 4 * k + sel;             // accumulator g*8 + i
                s_o[wave][idx >> 3][dl * 8 + (idx & 7)] = red[k];
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) { s_m[wave][g] = wm[g]; s_l[wave][g] = wl[g]; }
        }
    }
    __syncthreads();
    // ---- merge the four wave partials into the chunk's partial ----
    for (int e = tid; e < G * HD; e += FD_THREADS) {
        const int g = e / HD, d = e % HD;
        const float m0 = s_m[0][g], m1 = s_m[1][g], m2 = s_m[2][g], m3 = s_m[3][g];
        const float M = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));  // finite: the chunk holds at least one valid position
        const float w0 = fast_exp(m0 - M), w1 = fast_exp(m1 - M), w2 = fast_exp(m2 - M), w3 = fast_exp(m3 - M);
        const float o = (w0 * s_o[0][g][d] + w1 * s_o[1][g][d]) + (w2 * s_o[2][g][d] + w3 * s_o[3][g][d]);
        const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
        a.pO[oi * HD + d] = o;
        if (d == 0) {
            a.pM[oi] = M;
            a.pL[oi] = (w0 * s_l[0][g] + w1 * s_l[1][g]) + (w2 * s_l[2][g] + w3 * s_l[3][g]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The same front half on the matrix cores, for an fp16 cache.  The vector kernel above spends ~1400 instructions per
// wave on 16 positions x G heads, three quarters of them conversions, cross-lane sums and address arithmetic around 264
// FMAs, and the launch lasts as long as that chain whatever the context length (512 positions: 9.3 us for attention +
// merge, 2240: 10.5 us).  Here a wave's positions are MFMA tiles:
//   S^T[16 positions][16 head columns] = K tile . Q^T   v_mfma_f32_16x16x32_f16, A = the K rows exactly as they lie in the
//       cache (lane l: row l % 16, elements 32 s + 8 (l / 16) .. +7 of step s: one 16-byte load, no conversion), B = the
//       query heads as fp16 (columns past G repeat head 0 and are never stored);
//   O[16 head rows][HD] = P . V                        A = the probabilities in the layout the first product left them in
//       (lane l: head l % 16, positions 4 (l / 16) .. +3), B = V^T fragments from a wave-private LDS copy of the V rows through
//       the transposing read ds_read_b64_tr_b16.
// fp32 accuracy is kept by splitting the fp32 operands into two fp16 terms (q = q_hi + q_lo, p = p_hi + p_lo, 22 mantissa
// bits; K and V are fp16 already, products are exact, accumulation is fp32), so the result stays within the vector kernel's
// bar.  Scores are kept in base 2 (q is scaled by scale * log2 e before the split); the partial maxima are stored in those
// units and the merge kernel is told so.  A wave takes TPW tiles of 16 positions, a workgroup a chunk of 64 TPW positions.
// ---------------------------------------------------------------------------------------------
typedef _Float16 fd_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 fd_h4 __attribute__((ext_vector_type(4)));
typedef short fd_s4 __attribute__((ext_vector_type(4)));
typedef float fd_f4 __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i passes the address of four 16-bit values (row i / 4 of a 4-row
// block, columns 4 (i % 4) .. +3 of a 16-column block) and receives column i of the four rows.
__device__ __forceinline__ fd_h4 fd_lds_read_tr16(const uint8_t* p) {
    typedef __attribute__((address_space(3))) fd_s4 lds_s4;
    return __builtin_bit_cast(fd_h4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)p));
}
// max / sum over the four 16-lane rows of the wave (lanes with equal lane % 16), result in every lane
__device__ __forceinline__ float fd_rows_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float fd_rows_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int HD, int G, int TPW, bool BIAS = false>
__global__ __launch_bounds__(FD_THREADS) void attn_decode_mfma_kernel(const AttnArgs a) {
    constexpr int HALF = HD / 2;
    constexpr int KS = HD / 32;          // QK steps (32 head-dim elements each)
    constexpr int DT = HD / 16;          // 16-wide tiles of the output's head dimension
    constexpr int LPR = HD / 8;          // lanes per V row (16-byte pieces)
    constexpr int RPL = 64 / LPR;        // V rows per load instruction of a wave
    constexpr int VL = 16 / RPL;         // V loads per tile
    constexpr int VP = HD * 2 + 64;      // LDS pitch of a V row: the four rows of a transposing read fall on different banks
    constexpr int GP = G <= 4 ? 4 : 8;   // head slots of the wave partials
    constexpr int CH = 64 * TPW;         // positions per workgroup
    constexpr int PP = (HALF + 63) / 64; // rotation pairs a lane holds in the prologue: pairs lane and (heads of 256) lane + 64
    static_assert(G >= 1 && G <= 8 && (HD == 64 || HD == 128 || (HD == 256 && G <= 4)) && (TPW == 1 || TPW == 2), "shape");
    __shared__ __align__(16) _Float16 s_qh[G][HD];
    __shared__ __align__(16) _Float16 s_ql[G][HD];
    __shared__ __align__(16) _Float16 s_nk[HD];
    __shared__ __align__(16) uint8_t s_v[4][TPW][16 * VP];
    __shared__ __align__(16) float s_o[4][HD][GP];
    __shared__ float s_m[4][GP], s_l[4][GP];

    const int64_t past = *a.d_past;
    if (past < 0 || past >= a.max_seq) return;          // never touch memory outside the cache
    const int64_t total = past + 1;
    const int split = fd_split_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y), kvh = fd_head_of(blockIdx.x, blockIdx.y, gridDim.x, gridDim.y);
    const int64_t t0 = (int64_t)split * CH;
    if (t0 >= total) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t_begin = (a.window > 0 && total > a.window) ? total - a.window : 0;
    if (t0 + CH <= t_begin) {
        // a chunk wholly in front of the window: an empty partial (weight 2^(-inf - M) = 0 in the merge)
        for (int e = tid; e < G * HD; e += FD_THREADS) {
            const int g = e / HD, d = e % HD;
            const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
            a.pO[oi * HD + d] = 0.0f;
            if (d == 0) { a.pM[oi] = -INFINITY; a.pL[oi] = 0.0f; }
        }
        return;
    }
    const int j = lane & 15, rg = lane >> 4;
    const int kv_dim = a.n_kv_heads * HD;
    bool on[PP];
    int lh[PP];
#pragma unroll
    for (int p = 0; p < PP; ++p) {
        on[p] = lane + 64 * p < HALF;
        lh[p] = (lane + 64 * p) & (HALF - 1);
    }
    const bool has_norm = a.qw != nullptr;
    const int64_t wt0 = t0 + (int64_t)wave * (16 * TPW);            // first position of this wave
    const bool owner = past >= wt0 && past < wt0 + 16 * TPW;       // wave-uniform: this wave's tiles hold the new position

    // ---- loads, all unconditional so that their count is static: first the few values of the prologue ... ----
    const float* cs = a.rope + past * HD;
    const float* qwp = has_norm ? a.qw : a.Q;  // a valid address either way; unused without norm weights
    const float* kwp = has_norm ? a.kw : a.Q;
    int i0[PP], i1[PP];
#pragma unroll
    for (int p = 0; p < PP; ++p) {
        i0[p] = a.rope_interleaved ? 2 * lh[p] : lh[p];
        i1[p] = a.rope_interleaved ? 2 * lh[p] + 1 : lh[p] + HALF;
    }
    constexpr int NQ = (G + 3) / 4;  // query heads a wave prepares: wave, wave + 4
    float qx0[NQ][PP], qx1[NQ][PP], qb0[NQ][PP], qb1[NQ][PP];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        const int g = wave + 4 * n < G ? wave + 4 * n : 0;
        const float* src = a.Q + (int64_t)(kvh * G + g) * HD;
#pragma unroll
        for (int p = 0; p < PP; ++p) {
            qx0[n][p] = src[i0[p]];
            qx1[n][p] = src[i1[p]];
            if constexpr (BIAS) {
                qb0[n][p] = a.qb[(kvh * G + g) * HD + i0[p]];
                qb1[n][p] = a.qb[(kvh * G + g) * HD + i1[p]];
            }
        }
    }
    float qn0[PP], qn1[PP], kn0[PP], kn1[PP], rc[PP], rsn[PP], kx0[PP], kx1[PP], vx0[PP], vx1[PP], kb0[PP], kb1[PP], vb0[PP], vb1[PP];
#pragma unroll
    for (int p = 0; p < PP; ++p) {
        qn0[p] = qwp[i0[p]];
        qn1[p] = qwp[i1[p]];
        kn0[p] = kwp[i0[p]];
        kn1[p] = kwp[i1[p]];
        rc[p] = cs[lh[p]];
        rsn[p] = cs[HALF + lh[p]];
        kx0[p] = a.K[(int64_t)kvh * HD + i0[p]];
        kx1[p] = a.K[(int64_t)kvh * HD + i1[p]];
        vx0[p] = a.V[(int64_t)kvh * HD + lh[p]];
        vx1[p] = a.V[(int64_t)kvh * HD + lh[p] + HALF];
        kb0[p] = kb1[p] = vb0[p] = vb1[p] = 0.0f;
        if constexpr (BIAS) {
            kb0[p] = a.kb[kvh * HD + i0[p]];
            kb1[p] = a.kb[kvh * HD + i1[p]];
            vb0[p] = a.vb[kvh * HD + lh[p]];
            vb1[p] = a.vb[kvh * HD + lh[p] + HALF];
        }
    }
    issue_order_fence();
    // ---- ... then the cached K/V rows of this wave's tiles (the new position is not cached: clamp below it) ----
    uint4 kreg[TPW][KS], vreg[TPW][VL];
    const int64_t last_cached = past > 0 ? past - 1 : 0;
    const __half* Kh = static_cast<const __half*>(a.Kc) + (int64_t)kvh * HD;
    const __half* Vh = static_cast<const __half*>(a.Vc) + (int64_t)kvh * HD;
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int64_t tk = wt0 + 16 * u + j;
        const int64_t tkc = tk < past ? tk : last_cached;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            kreg[u][s] = *reinterpret_cast<const uint4*>(Kh + tkc * kv_dim + 32 * s + 8 * rg);
    }
#pragma unroll
    for (int u = 0; u < TPW; ++u)
#pragma unroll
        for (int vl = 0; vl < VL; ++vl) {
            const int64_t tv = wt0 + 16 * u + vl * RPL + lane / LPR;
            const int64_t tvc = tv < past ? tv : last_cached;
            vreg[u][vl] = *reinterpret_cast<const uint4*>(Vh + tvc * kv_dim + 8 * (lane % LPR));
        }
    issue_order_fence();

    // ---- per-head RMSNorm + rotation of this wave's query heads, scaled into base-2 score units, as two fp16 terms ----
    const float one = a.add_one ? 1.0f : 0.0f;
    const float qs = a.scale * 1.44269504088896340736f;
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        const int g = wave + 4 * n;
        if (g >= G) continue;  // wave-uniform
        float x0[PP], x1[PP];
        float ss = 0.0f;
#pragma unroll
        for (int p = 0; p < PP; ++p) {
            if constexpr (BIAS) { qx0[n][p] += qb0[n][p]; qx1[n][p] += qb1[n][p]; }
            x0[p] = on[p] ? qx0[n][p] : 0.0f;
            x1[p] = on[p] ? qx1[n][p] : 0.0f;
            ss = fmaf(x0[p], x0[p], ss);
            ss = fmaf(x1[p], x1[p], ss);
        }
        if (has_norm) {
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
#pragma unroll
            for (int p = 0; p < PP; ++p) {
                x0[p] = x0[p] * rs * (qn0[p] + one);
                x1[p] = x1[p] * rs * (qn1[p] + one);
            }
        }
#pragma unroll
        for (int p = 0; p < PP; ++p) {
            if (on[p]) {
                const float r0 = fmaf(x0[p], rc[p], -(x1[p] * rsn[p])) * qs, r1 = fmaf(x0[p], rsn[p], x1[p] * rc[p]) * qs;
                const _Float16 h0 = (_Float16)r0, h1 = (_Float16)r1;
                s_qh[g][i0[p]] = h0;
                s_qh[g][i1[p]] = h1;
                s_ql[g][i0[p]] = (_Float16)(r0 - (float)h0);
                s_ql[g][i1[p]] = (_Float16)(r1 - (float)h1);
            }
        }
    }
    __half nv0[PP], nv1[PP];
#pragma unroll
    for (int p = 0; p < PP; ++p) nv0[p] = nv1[p] = __float2half_rn(0.0f);
    if (owner) {  // the new K row: normalised, rotated, rounded as the cache holds it; the new V row
        float x0[PP], x1[PP];
        float ss = 0.0f;
#pragma unroll
        for (int p = 0; p < PP; ++p) {
            if constexpr (BIAS) { kx0[p] += kb0[p]; kx1[p] += kb1[p]; vx0[p] += vb0[p]; vx1[p] += vb1[p]; }
            x0[p] = on[p] ? kx0[p] : 0.0f;
            x1[p] = on[p] ? kx1[p] : 0.0f;
            ss = fmaf(x0[p], x0[p], ss);
            ss = fmaf(x1[p], x1[p], ss);
        }
        if (has_norm) {
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
#pragma unroll
            for (int p = 0; p < PP; ++p) {
                x0[p] = x0[p] * rs * (kn0[p] + one);
                x1[p] = x1[p] * rs * (kn1[p] + one);
            }
        }
        const int64_t rowoff = past * kv_dim + (int64_t)kvh * HD;
#pragma unroll
        for (int p = 0; p < PP; ++p) {
            const __half h0 = __float2half_rn(fmaf(x0[p], rc[p], -(x1[p] * rsn[p]))), h1 = __float2half_rn(fmaf(x0[p], rsn[p], x1[p] * rc[p]));
            nv0[p] = __float2half_rn(vx0[p]);
            nv1[p] = __float2half_rn(vx1[p]);
            if (on[p]) {
                static_cast<__half*>(a.Kc)[rowoff + i0[p]] = h0;
                static_cast<__half*>(a.Kc)[rowoff + i1[p]] = h1;
                static_cast<__half*>(a.Vc)[rowoff + lh[p]] = nv0[p];
                static_cast<__half*>(a.Vc)[rowoff + lh[p] + HALF] = nv1[p];
                reinterpret_cast<__half*>(s_nk)[i0[p]] = h0;
                reinterpret_cast<__half*>(s_nk)[i1[p]] = h1;
            }
        }
    }
    __syncthreads();  // the query heads come from the other waves (the new row stays within its wave)

    // ---- B operands: head column j (columns past G repeat head 0), both terms ----
    fd_h8 qh[KS], ql[KS];
    {
        const int jq = j < G ? j : 0;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            qh[s] = *reinterpret_cast<const fd_h8*>(&s_qh[jq][32 * s + 8 * rg]);
            ql[s] = *reinterpret_cast<const fd_h8*>(&s_ql[jq][32 * s + 8 * rg]);
        }
    }
    // ---- scores (base 2) of this wave's tiles: lane = (head j, positions 4 rg .. +3 of each tile) ----
    fd_f4 sc[TPW];
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int64_t tt0 = wt0 + 16 * u;
        if (owner && past >= tt0 && past < tt0 + 16 && j == (int)(past - tt0)) {
#pragma unroll
            for (int s = 0; s < KS; ++s) kreg[u][s] = *reinterpret_cast<const uint4*>(&s_nk[32 * s + 8 * rg]);
        }
        fd_f4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const fd_h8 kf = __builtin_bit_cast(fd_h8, kreg[u][s]);
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qh[s], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, ql[s], c, 0, 0, 0);
        }
        // only a tile that reaches the new position or the window's edge holds positions that do not count (wave-uniform)
        if (tt0 + 16 > past || tt0 < t_begin) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t t = tt0 + 4 * rg + r;
                c[r] = (t < total && t >= t_begin) ? c[r] : -INFINITY;
            }
        }
        sc[u] = c;
    }
    // ---- this wave's V rows into its LDS tile, row-major; rows that do not count are zeroed (0 * garbage must not be NaN) ----
#pragma unroll
    for (int u = 0; u < TPW; ++u) {
        const int64_t tt0 = wt0 + 16 * u;
        const bool edge = tt0 + 16 > past || tt0 < t_begin;  // wave-uniform
#pragma unroll
        for (int vl = 0; vl < VL; ++vl) {
            const int row = vl * RPL + lane / LPR;
            uint4 v = vreg[u][vl];
            if (edge) {
                const int64_t t = tt0 + row;
                if (!(t < past && t >= t_begin)) v = make_uint4(0u, 0u, 0u, 0u);
            }
            *reinterpret_cast<uint4*>(&s_v[wave][u][row * VP + 16 * (lane % LPR)]) = v;
        }
        if (owner && past >= tt0 && past < tt0 + 16) {
            __half* vrow = reinterpret_cast<__half*>(&s_v[wave][u][(int)(past - tt0) * VP]);
#pragma unroll
            for (int p = 0; p < PP; ++p) {
                if (on[p]) {
                    vrow[lh[p]] = nv0[p];
                    vrow[lh[p] + HALF] = nv1[p];
                }
            }
        }
    }
    // the V^T fragments are requested before the softmax arithmetic, which covers the LDS round trip
    fd_h4 vb[DT][TPW];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int u = 0; u < TPW; ++u)
            vb[dt][u] = fd_lds_read_tr16(&s_v[wave][u][(4 * rg + (j >> 2)) * VP + (16 * dt + 4 * (j & 3)) * 2]);
    // ---- wave-local softmax statistics ----
    float m = fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3]));
    if constexpr (TPW == 2) m = fmaxf(m, fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
    m = fd_rows_max(m);
    const float ms = m == -INFINITY ? 0.0f : m;  // a wave without valid positions contributes nothing
    float l = 0.0f;
    fd_h4 ph[TPW], pl[TPW];
#pragma unroll
    for (int u = 0; u < TPW; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = __builtin_amdgcn_exp2f(sc[u][r] - ms);  // -inf -> 0
            l += p;
            const _Float16 h = (_Float16)p;
            ph[u][r] = h;
            pl[u][r] = (_Float16)(p - (float)h);
        }
    l = fd_rows_sum(l);
    // ---- O[head][dim] += P . V ----
    fd_f4 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        fd_f4 c = {0.0f, 0.0f, 0.0f, 0.0f};
        if constexpr (TPW == 1) {
            c = __builtin_amdgcn_mfma_f32_16x16x16f16(ph[0], vb[dt][0], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_16x16x16f16(pl[0], vb[dt][0], c, 0, 0, 0);
        } else {
            // the 32 positions of both tiles in one product: summation index 8 rg + 4 u + r <-> position 16 u + 4 rg + r
            const fd_h4 v0 = vb[dt][0], v1 = vb[dt][TPW - 1];
            const fd_h8 b8 = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
            const fd_h8 ah = {ph[0][0], ph[0][1], ph[0][2], ph[0][3], ph[TPW - 1][0], ph[TPW - 1][1], ph[TPW - 1][2], ph[TPW - 1][3]};
            const fd_h8 al = {pl[0][0], pl[0][1], pl[0][2], pl[0][3], pl[TPW - 1][0], pl[TPW - 1][1], pl[TPW - 1][2], pl[TPW - 1][3]};
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, b8, c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, b8, c, 0, 0, 0);
        }
        acc[dt] = c;
    }
    // lane (j, rg) holds O[head 4 rg + r][dim 16 dt + j]: head rows past G are the repeated columns' and are dropped
    if (4 * rg < G) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<float4*>(&s_o[wave][16 * dt + j][4 * rg]) = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
    }
    if (rg == 0 && j < G) { s_m[wave][j] = m; s_l[wave][j] = l; }
    __syncthreads();
    // ---- merge the four wave partials into the chunk's partial ----
    for (int e = tid; e < G * HD; e += FD_THREADS) {
        const int g = e / HD, d = e % HD;
        const float m0 = s_m[0][g], m1 = s_m[1][g], m2 = s_m[2][g], m3 = s_m[3][g];
        const float M = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));  // finite: the chunk holds at least one valid position
        const float w0 = __builtin_amdgcn_exp2f(m0 - M), w1 = __builtin_amdgcn_exp2f(m1 - M),
                    w2 = __builtin_amdgcn_exp2f(m2 - M), w3 = __builtin_amdgcn_exp2f(m3 - M);
        const float o = (w0 * s_o[0][d][g] + w1 * s_o[1][d][g]) + (w2 * s_o[2][d][g] + w3 * s_o[3][d][g]);
        const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
        a.pO[oi * HD + d] = o;
        if (d == 0) {
            a.pM[oi] = M;
            a.pL[oi] = (w0 * s_l[0][g] + w1 * s_l[1][g]) + (w2 * s_l[2][g] + w3 * s_l[3][g]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Long caches (more than FD_LONG_SPLITS chunks of 64 positions fit): the same matrix-core kernel as a loop.  A launch always
// has FD_LONG_SPLITS workgroups per kv head; workgroup s walks the chunks [s cpw, (s + 1) cpw), cpw = ceil(chunks in use /
// FD_LONG_SPLITS), with a running maximum / sum / output per wave (online softmax) and leaves ONE partial.  Against one
// workgroup per chunk this bounds the partials (64 per head instead of 512 at 32 k positions: the merge launch took 8.9 of
// the 37 us there, and the partials 8 MB of traffic per layer) and the grid (a cache of 33 k positions launched 4128
// workgroups of which 264 had work at 2 k: +1.4 us).  The next chunk's rows are in flight while the current one is worked on.
// ---------------------------------------------------------------------------------------------
__host__ __device__ inline int fd_long_cpw(int n_chunks) { return (n_chunks + FD_LONG_SPLITS - 1) / FD_LONG_SPLITS; }

template <int HD, int G, bool BIAS = false>
__global__ __launch_bounds__(FD_THREADS) void attn_decode_mfma_long_kernel(const AttnArgs a) {
    constexpr int HALF = HD / 2, KS = HD / 32, DT = HD / 16, LPR = HD / 8, RPL = 64 / LPR, VL = 16 / RPL, VP = HD * 2 + 64;
    constexpr int GP = G <= 4 ? 4 : 8;
    static_assert(G >= 1 && G <= 8 && (HD == 64 || HD == 128), "shape");
    __shared__ __align__(16) _Float16 s_qh[G][HD];
    __shared__ __align__(16) _Float16 s_ql[G][HD];
    __shared__ __align__(16) _Float16 s_nk[HD];
    __shared__ __align__(16) uint8_t s_v[4][16 * VP];
    __shared__ __align__(16) float s_o[4][HD][GP];
    __shared__ float s_m[4][GP], s_l[4][GP];

    const int64_t past = *a.d_past;
    if (past < 0 || past >= a.max_seq) return;          // never touch memory outside the cache
    const int64_t total = past + 1;
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int n_chunks = (int)((total + FD_CHUNK - 1) / FD_CHUNK);
    const int cpw = fd_long_cpw(n_chunks);
    const int c_first = split * cpw;
    if (c_first >= n_chunks) return;
    const int c_end = min(c_first + cpw, n_chunks);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t_begin = (a.window > 0 && total > a.window) ? total - a.window : 0;
    const int c_lo = max(c_first, (int)(t_begin / FD_CHUNK));   // chunks wholly in front of the window are skipped
    if (c_lo >= c_end) {
        for (int e = tid; e < G * HD; e += FD_THREADS) {
            const int g = e / HD, d = e % HD;
            const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
            a.pO[oi * HD + d] = 0.0f;
            if (d == 0) { a.pM[oi] = -INFINITY; a.pL[oi] = 0.0f; }
        }
        return;
    }
    const int j = lane & 15, rg = lane >> 4;
    const int kv_dim = a.n_kv_heads * HD;
    const bool on = lane < HALF;
    const int lh = lane & (HALF - 1);
    const bool has_norm = a.qw != nullptr;
    const int pc = (int)(past / FD_CHUNK);                                        // the chunk that holds the new position
    const bool owner = pc >= c_lo && pc < c_end && (int)((past - (int64_t)pc * FD_CHUNK) / 16) == wave;  // wave-uniform

    // ---- prologue loads (static count), then the first chunk's rows ----
    const float* cs = a.rope + past * HD;
    const float* qwp = has_norm ? a.qw : a.Q;
    const float* kwp = has_norm ? a.kw : a.Q;
    const int i0 = a.rope_interleaved ? 2 * lh : lh, i1 = a.rope_interleaved ? 2 * lh + 1 : lh + HALF;
    constexpr int NQ = (G + 3) / 4;
    float qx0[NQ], qx1[NQ], qb0[NQ], qb1[NQ];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        const int g = wave + 4 * n < G ? wave + 4 * n : 0;
        const float* src = a.Q + (int64_t)(kvh * G + g) * HD;
        qx0[n] = src[i0];
        qx1[n] = src[i1];
        if constexpr (BIAS) {
            qb0[n] = a.qb[(kvh * G + g) * HD + i0];
            qb1[n] = a.qb[(kvh * G + g) * HD + i1];
        }
    }
    const float qn0 = qwp[i0], qn1 = qwp[i1], kn0 = kwp[i0], kn1 = kwp[i1];
    const float rc = cs[lh], rsn = cs[HALF + lh];
    float kx0 = a.K[(int64_t)kvh * HD + i0], kx1 = a.K[(int64_t)kvh * HD + i1];
    float vx0 = a.V[(int64_t)kvh * HD + lh], vx1 = a.V[(int64_t)kvh * HD + lh + HALF];
    float kb0 = 0.0f, kb1 = 0.0f, vb0 = 0.0f, vb1 = 0.0f;
    if constexpr (BIAS) {
        kb0 = a.kb[kvh * HD + i0];
        kb1 = a.kb[kvh * HD + i1];
        vb0 = a.vb[kvh * HD + lh];
        vb1 = a.vb[kvh * HD + lh + HALF];
    }
    issue_order_fence();
    const int64_t last_cached = past > 0 ? past - 1 : 0;
    const __half* Kh = static_cast<const __half*>(a.Kc) + (int64_t)kvh * HD;
    const __half* Vh = static_cast<const __half*>(a.Vc) + (int64_t)kvh * HD;
    auto fetch = [&](int c, uint4 (&kr)[KS], uint4 (&vr)[VL]) {   // this wave's 16 positions of chunk c; all loads unconditional
        const int64_t wt0 = (int64_t)c * FD_CHUNK + 16 * wave;
        const int64_t tk = wt0 + j;
        const int64_t tkc = tk < past ? tk : last_cached;
#pragma unroll
        for (int s = 0; s < KS; ++s) kr[s] = *reinterpret_cast<const uint4*>(Kh + tkc * kv_dim + 32 * s + 8 * rg);
#pragma unroll
        for (int vl = 0; vl < VL; ++vl) {
            const int64_t tv = wt0 + vl * RPL + lane / LPR;
            const int64_t tvc = tv < past ? tv : last_cached;
            vr[vl] = *reinterpret_cast<const uint4*>(Vh + tvc * kv_dim + 8 * (lane % LPR));
        }
    };
    uint4 kreg[KS], vreg[VL], knext[KS], vnext[VL];
    fetch(c_lo, kreg, vreg);
    issue_order_fence();

    // ---- query heads (and, in the wave that owns it, the new K/V row) as in attn_decode_mfma_kernel ----
    const float one = a.add_one ? 1.0f : 0.0f;
    const float qs = a.scale * 1.44269504088896340736f;
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
        const int g = wave + 4 * n;
        if (g >= G) continue;  // wave-uniform
        if constexpr (BIAS) { qx0[n] += qb0[n]; qx1[n] += qb1[n]; }
        float x0 = on ? qx0[n] : 0.0f, x1 = on ? qx1[n] : 0.0f;
        if (has_norm) {
            float ss = fmaf(x0, x0, 0.0f);
            ss = fmaf(x1, x1, ss);
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
            x0 = x0 * rs * (qn0 + one);
            x1 = x1 * rs * (qn1 + one);
        }
        if (on) {
            const float r0 = fmaf(x0, rc, -(x1 * rsn)) * qs, r1 = fmaf(x0, rsn, x1 * rc) * qs;
            const _Float16 h0 = (_Float16)r0, h1 = (_Float16)r1;
            s_qh[g][i0] = h0;
            s_qh[g][i1] = h1;
            s_ql[g][i0] = (_Float16)(r0 - (float)h0);
            s_ql[g][i1] = (_Float16)(r1 - (float)h1);
        }
    }
    __half nv0 = __float2half_rn(0.0f), nv1 = nv0;
    if (owner) {
        if constexpr (BIAS) { kx0 += kb0; kx1 += kb1; vx0 += vb0; vx1 += vb1; }
        float x0 = on ? kx0 : 0.0f, x1 = on ? kx1 : 0.0f;
        if (has_norm) {
            float ss = fmaf(x0, x0, 0.0f);
            ss = fmaf(x1, x1, ss);
            ss = sum64(ss);
            const float rs = fast_rsqrt(ss * (1.0f / (float)HD) + a.eps);
            x0 = x0 * rs * (kn0 + one);
            x1 = x1 * rs * (kn1 + one);
        }
        const __half h0 = __float2half_rn(fmaf(x0, rc, -(x1 * rsn))), h1 = __float2half_rn(fmaf(x0, rsn, x1 * rc));
        nv0 = __float2half_rn(vx0);
        nv1 = __float2half_rn(vx1);
        if (on) {
            const int64_t rowoff = past * kv_dim + (int64_t)kvh * HD;
            static_cast<__half*>(a.Kc)[rowoff + i0] = h0;
            static_cast<__half*>(a.Kc)[rowoff + i1] = h1;
            static_cast<__half*>(a.Vc)[rowoff + lh] = nv0;
            static_cast<__half*>(a.Vc)[rowoff + lh + HALF] = nv1;
            reinterpret_cast<__half*>(s_nk)[i0] = h0;
            reinterpret_cast<__half*>(s_nk)[i1] = h1;
        }
    }
    __syncthreads();
    fd_h8 qh[KS], ql[KS];
    {
        const int jq = j < G ? j : 0;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            qh[s] = *reinterpret_cast<const fd_h8*>(&s_qh[jq][32 * s + 8 * rg]);
            ql[s] = *reinterpret_cast<const fd_h8*>(&s_ql[jq][32 * s + 8 * rg]);
        }
    }

    // ---- the chunks of this workgroup: running maximum m_run / sum l_run of head j (score layout), output acc (head rows) ----
    float m_run = -INFINITY, l_run = 0.0f;
    fd_f4 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = fd_f4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = c_lo;; ++c) {
        // the next chunk's rows travel while this one is worked on.  After the last chunk the loads still go out (a load under
        // a branch would cost the compiler its count of the loads in flight) but every lane asks for the last cached row -
        // a chunk index past the position clamps there - so they move a few bytes, and nobody waits for them
        fetch(c + 1 < c_end ? c + 1 : pc + 1, knext, vnext);
        issue_order_fence();
        const int64_t tt0 = (int64_t)c * FD_CHUNK + 16 * wave;
        const bool has_new = owner && c == pc;                     // wave-uniform: this tile holds the new position
        const bool edge = tt0 + 16 > past || tt0 < t_begin;       // wave-uniform: some of its positions do not count
        if (has_new && j == (int)(past - tt0)) {
#pragma unroll
            for (int s = 0; s < KS; ++s) kreg[s] = *reinterpret_cast<const uint4*>(&s_nk[32 * s + 8 * rg]);
        }
        fd_f4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const fd_h8 kf = __builtin_bit_cast(fd_h8, kreg[s]);
            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qh[s], sc, 0, 0, 0);
            sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, ql[s], sc, 0, 0, 0);
        }
        if (edge) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t t = tt0 + 4 * rg + r;
                sc[r] = (t < total && t >= t_begin) ? sc[r] : -INFINITY;
            }
        }
#pragma unroll
        for (int vl = 0; vl < VL; ++vl) {
            const int row = vl * RPL + lane / LPR;
            uint4 v = vreg[vl];
            if (edge) {
                const int64_t t = tt0 + row;
                if (!(t < past && t >= t_begin)) v = make_uint4(0u, 0u, 0u, 0u);
            }
            *reinterpret_cast<uint4*>(&s_v[wave][row * VP + 16 * (lane % LPR)]) = v;
        }
        if (has_new && on) {
            __half* vrow = reinterpret_cast<__half*>(&s_v[wave][(int)(past - tt0) * VP]);
            vrow[lh] = nv0;
            vrow[lh + HALF] = nv1;
        }
        fd_h4 vb[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vb[dt] = fd_lds_read_tr16(&s_v[wave][(4 * rg + (j >> 2)) * VP + (16 * dt + 4 * (j & 3)) * 2]);
        // online softmax: new maximum, correction of what has been summed so far
        float m = fd_rows_max(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])));
        const float m_new = fmaxf(m_run, m);
        const float ms = m_new == -INFINITY ? 0.0f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m_run - ms);   // first chunk: 2^(-inf) = 0
        float l = 0.0f;
        fd_h4 ph, pl;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = __builtin_amdgcn_exp2f(sc[r] - ms);
            l += p;
            const _Float16 h = (_Float16)p;
            ph[r] = h;
            pl[r] = (_Float16)(p - (float)h);
        }
        l_run = fmaf(l_run, corr, fd_rows_sum(l));
        m_run = m_new;
        // the output rows of this lane are heads 4 rg + r: their corrections sit in lanes 4 rg + r of the lane's own row
        float cr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, (lane & 48) | ((4 * rg + r) & 15), 64);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            fd_f4 cacc = {acc[dt][0] * cr[0], acc[dt][1] * cr[1], acc[dt][2] * cr[2], acc[dt][3] * cr[3]};
            cacc = __builtin_amdgcn_mfma_f32_16x16x16f16(ph, vb[dt], cacc, 0, 0, 0);
            cacc = __builtin_amdgcn_mfma_f32_16x16x16f16(pl, vb[dt], cacc, 0, 0, 0);
            acc[dt] = cacc;
        }
        if (c + 1 >= c_end) break;
#pragma unroll
        for (int s = 0; s < KS; ++s) kreg[s] = knext[s];
#pragma unroll
        for (int vl = 0; vl < VL; ++vl) vreg[vl] = vnext[vl];
    }
    if (4 * rg < G) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<float4*>(&s_o[wave][16 * dt + j][4 * rg]) = make_float4(acc[dt][0], acc[dt][1], acc[dt][2], acc[dt][3]);
    }
    if (rg == 0 && j < G) { s_m[wave][j] = m_run; s_l[wave][j] = l_run; }
    __syncthreads();
    for (int e = tid; e < G * HD; e += FD_THREADS) {
        const int g = e / HD, d = e % HD;
        const float m0 = s_m[0][g], m1 = s_m[1][g], m2 = s_m[2][g], m3 = s_m[3][g];
        const float M = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));  // finite: the chunks hold at least one valid position
        const float w0 = __builtin_amdgcn_exp2f(m0 - M), w1 = __builtin_amdgcn_exp2f(m1 - M),
                    w2 = __builtin_amdgcn_exp2f(m2 - M), w3 = __builtin_amdgcn_exp2f(m3 - M);
        const float o = (w0 * s_o[0][d][g] + w1 * s_o[1][d][g]) + (w2 * s_o[2][d][g] + w3 * s_o[3][d][g]);
        const int64_t oi = (int64_t)split * a.n_heads + kvh * G + g;
        a.pO[oi * HD + d] = o;
        if (d == 0) {
            a.pM[oi] = M;
            a.pL[oi] = (w0 * s_l[0][g] + w1 * s_l[1][g]) + (w2 * s_l[2][g] + w3 * s_l[3][g]);
        }
    }
}

template <int HD, bool BIAS>
static int attn_mfma_long_launch_g(int G, dim3 grid, hipStream_t s, const AttnArgs& a) {
#define PTM_AL(GG) hipLaunchKernelGGL((attn_decode_mfma_long_kernel<HD, GG, BIAS>), grid, dim3(FD_THREADS), 0, s, a)
    switch (G) {
        case 1: PTM_AL(1); break;
        case 2: PTM_AL(2); break;
        case 3: PTM_AL(3); break;
        case 4: PTM_AL(4); break;
        case 5: PTM_AL(5); break;
        case 6: PTM_AL(6); break;
        case 7: PTM_AL(7); break;
        case 8: PTM_AL(8); break;
        default: return PTM_E_UNSUPPORTED;
    }
#undef PTM_AL
    return launch_status();
}

template <int HD, int TPW, bool BIAS>
static int attn_mfma_launch_g(int G, dim3 grid, hipStream_t s, const AttnArgs& a) {
#define PTM_AM(GG) hipLaunchKernelGGL((attn_decode_mfma_kernel<HD, GG, TPW, BIAS>), grid, dim3(FD_THREADS), 0, s, a)
    if constexpr (HD == 256) {  // up to four query heads per kv head (the wave partials of more would not fit the static LDS)
        switch (G) {
            case 1: PTM_AM(1); break;
            case 2: PTM_AM(2); break;
            case 3: PTM_AM(3); break;
            case 4: PTM_AM(4); break;
            default: return PTM_E_UNSUPPORTED;
        }
    } else {
        switch (G) {
            case 1: PTM_AM(1); break;
            case 2: PTM_AM(2); break;
            case 3: PTM_AM(3); break;
            case 4: PTM_AM(4); break;
            case 5: PTM_AM(5); break;
            case 6: PTM_AM(6); break;
            case 7: PTM_AM(7); break;
            case 8: PTM_AM(8); break;
            default: return PTM_E_UNSUPPORTED;
        }
    }
#undef PTM_AM
    return launch_status();
}

template <bool KV16, int HD>
static int attn_launch_g(int G, dim3 grid, hipStream_t s, const AttnArgs& a) {
#define PTM_AT(GG) hipLaunchKernelGGL((attn_decode_fused_kernel<KV16, HD, GG>), grid, dim3(FD_THREADS), 0, s, a)
    switch (G) {
        case 1: PTM_AT(1); break;
        case 2: PTM_AT(2); break;
        case 3: PTM_AT(3); break;
        case 4: PTM_AT(4); break;
        case 5: PTM_AT(5); break;
        case 6: PTM_AT(6); break;
        case 7: PTM_AT(7); break;
        case 8: PTM_AT(8); break;
        default: return PTM_E_UNSUPPORTED;
    }
#undef PTM_AT
    return launch_status();
}

template <bool KV16, int HD, bool FUSED = false>
static int fd_launch_g(int G, dim3 grid, hipStream_t s, const float* Q, const void* Kc, const void* Vc, float* pO,
                       float* pL, float* pM, int n_heads, int n_kv_heads, const int64_t* d_past, int max_seq,
                       float scale, int window = 0, const FdFuse& f = FdFuse{}, int64_t past_host = 0) {
#define PTM_FD(GG)                                                                                                     \
    hipLaunchKernelGGL((flash_decode_partial_kernel<KV16, HD, GG, FUSED>), grid, dim3(FD_THREADS), 0, s, Q,             \
                       const_cast<void*>(Kc), const_cast<void*>(Vc), pO, pL, pM, n_heads, n_kv_heads, d_past, past_host, \
                       max_seq, scale, window, f)
    switch (G) {
        case 1: PTM_FD(1); break;
        case 2: PTM_FD(2); break;
        case 3: PTM_FD(3); break;
        case 4: PTM_FD(4); break;
        case 5: PTM_FD(5); break;
        case 6: PTM_FD(6); break;
        case 7: PTM_FD(7); break;
        case 8: PTM_FD(8); break;
        default: return PTM_E_UNSUPPORTED;
    }
#undef PTM_FD
    return launch_status();
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_flash_decode_kv_chunk_size(void) { return FD_CHUNK; }
int ptm_flash_decode_num_splits(int total_seq) { return total_seq <= 0 ? 0 : (total_seq + FD_CHUNK - 1) / FD_CHUNK; }

int ptm_flash_decode(const float* Q, const void* K_cache, const void* V_cache, float* O, float* partial_O,
                     float* partial_lse, float* partial_max, int n_heads, int n_kv_heads, int head_dim,
                     const int64_t* d_past_len, int max_seq, float scale, int kv_fp16, ptm_stream_t stream) {
    return ptm_flash_decode_window(Q, K_cache, V_cache, O, nullptr, partial_O, partial_lse, partial_max, n_heads, n_kv_heads,
                                   head_dim, d_past_len, max_seq, scale, kv_fp16, 0, stream);
}

static int flash_decode_any(const float* Q, const void* K_cache, const void* V_cache, float* O, void* o_q8,
                            float* partial_O, float* partial_lse, float* partial_max, int n_heads, int n_kv_heads,
                            int head_dim, const int64_t* d_past_len, int64_t past_host, int max_seq, float scale, int kv_fp16,
                            int window, ptm_stream_t stream) {
    if (!Q || !K_cache || !V_cache || !O || !partial_O || !partial_lse || !partial_max)
        return PTM_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || (n_heads % n_kv_heads) != 0) return PTM_E_SHAPE;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return PTM_E_UNSUPPORTED;
    if (!aligned16(Q) || !aligned16(K_cache) || !aligned16(V_cache)) return PTM_E_ALIGN;
    if (o_q8 && (reinterpret_cast<uintptr_t>(o_q8) & 15u)) return PTM_E_ALIGN;
    if (window < 0) window = 0;
    const int G = n_heads / n_kv_heads;
    const dim3 grid(ptm_flash_decode_num_splits(max_seq), n_kv_heads);
    hipStream_t s = as_stream(stream);
    int rc;
#define PTM_FDW(KV, HDV) fd_launch_g<KV, HDV>(G, grid, s, Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale, window, FdFuse{}, past_host)
    if (kv_fp16) rc = head_dim == 256 ? PTM_FDW(true, 256) : head_dim == 128 ? PTM_FDW(true, 128) : PTM_FDW(true, 64);
    else rc = head_dim == 256 ? PTM_FDW(false, 256) : head_dim == 128 ? PTM_FDW(false, 128) : PTM_FDW(false, 64);
#undef PTM_FDW
    if (rc != PTM_OK) return rc;
    return fd_merge(head_dim, n_heads, s, partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                    static_cast<uint8_t*>(o_q8), past_host);
}

int ptm_flash_decode_window(const float* Q, const void* K_cache, const void* V_cache, float* O, void* o_q8,
                            float* partial_O, float* partial_lse, float* partial_max, int n_heads, int n_kv_heads,
                            int head_dim, const int64_t* d_past_len, int max_seq, float scale, int kv_fp16, int window,
                            ptm_stream_t stream) {
    if (!d_past_len) return PTM_E_NULL;
    return flash_decode_any(Q, K_cache, V_cache, O, o_q8, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, head_dim,
                            d_past_len, 0, max_seq, scale, kv_fp16, window, stream);
}

// Position from the host: attends rows [0, total_seq) of caches that hold at least total_seq rows.
int ptm_flash_decode_pos(const float* Q, const void* K_cache, const void* V_cache, float* O, float* partial_O,
                         float* partial_lse, float* partial_max, int n_heads, int n_kv_heads, int head_dim, int total_seq,
                         float scale, int kv_fp16, ptm_stream_t stream) {
    if (total_seq <= 0) return PTM_E_RANGE;
    return flash_decode_any(Q, K_cache, V_cache, O, nullptr, partial_O, partial_lse, partial_max, n_heads, n_kv_heads,
                            head_dim, nullptr, (int64_t)total_seq - 1, total_seq, scale, kv_fp16, 0, stream);
}

// ptm_attn_decode_fused that can also leave the output as Q8 activation blocks (o_q8, may be NULL) for a Q4_K output
// projection.  The decode runtime's entry; not declared in the public header.
// window > 0: only the last `window` positions (the new one included) are attended to.
// 1 when ptm_attn_decode_fused_bias adds the projection biases itself for this cache type and head size
int ptm_attn_decode_folds_bias(int head_dim, int kv_fp16) { return kv_fp16 && (head_dim == 64 || head_dim == 128); }

// As ptm_attn_decode_fused_win with the biases of the q / k / v projections (all three or none) added to the raw vectors
// before norm and rotation; only where ptm_attn_decode_folds_bias says so.
int ptm_attn_decode_fused_bias(const float* Q, const float* K, const float* V, const float* q_bias, const float* k_bias,
                               const float* v_bias, const float* q_norm_w,
                               const float* k_norm_w, void* K_cache, void* V_cache, float* O, void* o_q8, float* partial_O,
                               float* partial_lse, float* partial_max, const float* rope_table,
                               int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                               float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, int window,
                               ptm_stream_t stream) {
    const bool bias = q_bias != nullptr;
    if (bias != (k_bias != nullptr) || bias != (v_bias != nullptr)) return PTM_E_NULL;
    if (bias && !ptm_attn_decode_folds_bias(head_dim, kv_fp16)) return PTM_E_UNSUPPORTED;
    if (!Q || !K || !V || !K_cache || !V_cache || !O || !partial_O || !partial_lse || !partial_max ||
        !rope_table || !d_past_len)
        return PTM_E_NULL;
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) return PTM_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || (n_heads % n_kv_heads) != 0) return PTM_E_SHAPE;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return PTM_E_UNSUPPORTED;
    if (!aligned16(K_cache) || !aligned16(V_cache) || !aligned16(partial_O) || !aligned16(O)) return PTM_E_ALIGN;
    if (head_dim == 256 && kv_fp16 && !bias && n_heads / n_kv_heads <= 4 && ptm_flash_decode_num_splits(max_seq) <= FD_LONG_SPLITS) {
        // heads of 256 (gemma3), fp16 cache of up to 4096 positions: the matrix-core kernel, two rotation pairs per lane
        if (o_q8 && (reinterpret_cast<uintptr_t>(o_q8) & 15u)) return PTM_E_ALIGN;
        AttnArgs a256{Q, K, V, q_norm_w, k_norm_w, rope_table, K_cache, V_cache, partial_O, partial_lse, partial_max,
                      d_past_len, n_heads, n_kv_heads, max_seq, add_one, scale, eps, rope_interleaved ? 1 : 0,
                      window > 0 ? window : 0, nullptr, nullptr, nullptr};
        const dim3 grid256(ptm_flash_decode_num_splits(max_seq), n_kv_heads);
        const int rc256 = attn_mfma_launch_g<256, 1, false>(n_heads / n_kv_heads, grid256, as_stream(stream), a256);
        if (rc256 != PTM_OK) return rc256;
        return fd_merge(head_dim, n_heads, as_stream(stream), partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                        static_cast<uint8_t*>(o_q8), 0, FD_CHUNK, 1);
    }
    if (head_dim == 256) {
        // heads this wide with an fp32 cache, more query heads per kv head or a longer cache: the plain split-KV kernel with
        // the norm / rotation / append prologue in front
        if (o_q8 && (reinterpret_cast<uintptr_t>(o_q8) & 15u)) return PTM_E_ALIGN;
        const FdFuse f{K, V, q_norm_w, k_norm_w, rope_table, eps, add_one, rope_interleaved ? 1 : 0};
        const dim3 grid256(ptm_flash_decode_num_splits(max_seq), n_kv_heads);
        const int G256 = n_heads / n_kv_heads;
        const int w = window > 0 ? window : 0;
        const int rc256 = kv_fp16 ? fd_launch_g<true, 256, true>(G256, grid256, as_stream(stream), Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale, w, f)
                                  : fd_launch_g<false, 256, true>(G256, grid256, as_stream(stream), Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale, w, f);
        if (rc256 != PTM_OK) return rc256;
        return fd_merge(head_dim, n_heads, as_stream(stream), partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                        static_cast<uint8_t*>(o_q8));
    }
    AttnArgs a{Q, K, V, q_norm_w, k_norm_w, rope_table, K_cache, V_cache, partial_O, partial_lse, partial_max,
               d_past_len, n_heads, n_kv_heads, max_seq, add_one, scale, eps, rope_interleaved ? 1 : 0, window > 0 ? window : 0,
               q_bias, k_bias, v_bias};
    const int G = n_heads / n_kv_heads;
    const dim3 grid(ptm_flash_decode_num_splits(max_seq), n_kv_heads);
    hipStream_t s = as_stream(stream);
    int rc;
    if (o_q8 && (reinterpret_cast<uintptr_t>(o_q8) & 15u)) return PTM_E_ALIGN;
    if (kv_fp16) {
        // fp16 cache: the matrix-core kernel, chunks of 64 positions; partial maxima in base-2 units
        if (ptm_flash_decode_num_splits(max_seq) > FD_LONG_SPLITS) {
            // a cache of more than 4096 positions: the looping kernel, at most FD_LONG_SPLITS partials per head
            const dim3 grid_long(FD_LONG_SPLITS, n_kv_heads);
            if (bias) rc = head_dim == 128 ? attn_mfma_long_launch_g<128, true>(G, grid_long, s, a) : attn_mfma_long_launch_g<64, true>(G, grid_long, s, a);
            else rc = head_dim == 128 ? attn_mfma_long_launch_g<128, false>(G, grid_long, s, a) : attn_mfma_long_launch_g<64, false>(G, grid_long, s, a);
            if (rc != PTM_OK) return rc;
            return fd_merge(head_dim, n_heads, s, partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                            static_cast<uint8_t*>(o_q8), 0, -1, 1);
        }
        if (bias) rc = head_dim == 128 ? attn_mfma_launch_g<128, 1, true>(G, grid, s, a) : attn_mfma_launch_g<64, 1, true>(G, grid, s, a);
        else rc = head_dim == 128 ? attn_mfma_launch_g<128, 1, false>(G, grid, s, a) : attn_mfma_launch_g<64, 1, false>(G, grid, s, a);
        if (rc != PTM_OK) return rc;
        return fd_merge(head_dim, n_heads, s, partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                        static_cast<uint8_t*>(o_q8), 0, FD_CHUNK, 1);
    }
    rc = head_dim == 128 ? attn_launch_g<false, 128>(G, grid, s, a) : attn_launch_g<false, 64>(G, grid, s, a);
    if (rc != PTM_OK) return rc;
    return fd_merge(head_dim, n_heads, s, partial_O, partial_lse, partial_max, O, d_past_len, max_seq,
                    static_cast<uint8_t*>(o_q8));
}

int ptm_attn_decode_fused_win(const float* Q, const float* K, const float* V, const float* q_norm_w,
                              const float* k_norm_w, void* K_cache, void* V_cache, float* O, void* o_q8, float* partial_O,
                              float* partial_lse, float* partial_max, const float* rope_table,
                              int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                              float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, int window,
                              ptm_stream_t stream) {
    return ptm_attn_decode_fused_bias(Q, K, V, nullptr, nullptr, nullptr, q_norm_w, k_norm_w, K_cache, V_cache, O, o_q8,
                                      partial_O, partial_lse, partial_max, rope_table, n_heads, n_kv_heads, head_dim,
                                      d_past_len, max_seq, scale, eps, add_one, kv_fp16, rope_interleaved, window, stream);
}

int ptm_attn_decode_fused_q8(const float* Q, const float* K, const float* V, const float* q_norm_w,
                             const float* k_norm_w, void* K_cache, void* V_cache, float* O, void* o_q8, float* partial_O,
                             float* partial_lse, float* partial_max, const float* rope_table,
                             int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                             float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, ptm_stream_t stream) {
    return ptm_attn_decode_fused_win(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, O, o_q8, partial_O, partial_lse,
                                     partial_max, rope_table, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale,
                                     eps, add_one, kv_fp16, rope_interleaved, 0, stream);
}

int ptm_attn_decode_fused(const float* Q, const float* K, const float* V, const float* q_norm_w,
                          const float* k_norm_w, void* K_cache, void* V_cache, float* O, float* partial_O,
                          float* partial_lse, float* partial_max, const float* rope_table,
                          int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                          float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, ptm_stream_t stream) {
    return ptm_attn_decode_fused_q8(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, O, nullptr, partial_O, partial_lse,
                                    partial_max, rope_table, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale,
                                    eps, add_one, kv_fp16, rope_interleaved, stream);
}

int ptm_attn_decode_fused_window(const float* Q, const float* K, const float* V, const float* q_norm_w,
                                 const float* k_norm_w, void* K_cache, void* V_cache, float* O, float* partial_O,
                                 float* partial_lse, float* partial_max, const float* rope_table,
                                 int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                                 float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, int window,
                                 ptm_stream_t stream) {
    return ptm_attn_decode_fused_win(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, O, nullptr, partial_O, partial_lse,
                                     partial_max, rope_table, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale,
                                     eps, add_one, kv_fp16, rope_interleaved, window, stream);
}

}  // extern "C"
