// Prefill of M prompt tokens at once: the row-batched counterparts of the decode-step glue.
//
// The reference's prefill (GGUFModel::forward(tokens, use_cache), torch/io/gguf_model.h:2510-2571, layer body
// transformer_layer :7300-7460) runs the layer
// over all prompt rows: RMSNorm per row, matmul_q per projection, per-head QK-norm + RoPE at each row's position,
// KV append, causal attention, residual adds.  Row m of the result is what M single-token decode steps give for
// token m (same formulas as the decode kernels; positions past + m), so parity is checked against the CPU oracle
// stepping the prompt token by token.
//   embedding_rows        one embedding row per prompt token (fp32 table, or Q6_K rows dequantised on the fly)
//   qknorm_rope_kv_rows   per (row, head): RMSNorm over the head, NeoX rotation at position pos0 + row; K and V rows
//                         are appended to the cache (fp16 or fp32)
//   prefill_attn          causal GQA attention of row m over cache positions [0, pos0 + m]: one wave per (row, kv
//                         head) serves the G query heads; every lane group keeps its own online-softmax state over
//                         the positions it visits (no cross-lane traffic inside the loop), merged once at the end
//   prefill_attn_mfma     the same attention on the matrix cores for an fp16 cache and 16 or more rows: a workgroup
//                         owns one kv head and 128 query vectors (128 / G rows x G heads), walks the cache in tiles
//                         of 32 positions staged through LDS, S^T = K . Q^T and O^T += V^T . P^T with
//                         v_mfma_f32_32x32x16_f16, online softmax in the accumulator layout (a lane owns one query
//                         vector's column).  Q and P are rounded to fp16: ~1e-3 of the output's scale.
#include "ptm_common.h"

namespace ptm {

enum { PTM_PREFILL_MFMA_MIN_ROWS = 16 };  // fewer rows: the exact fp32 kernel (too few workgroups for the tiled one to pay)

__device__ __forceinline__ float pf_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// Q6_K element e (0..255) of a block (reference: dequantize_q6_k, torch/io/gguf_dequant.h:395-430)
__device__ __forceinline__ float pf_q6k_elem(const uint8_t* blk, int e) {
    const int half = e >> 7, r = e & 127, grp = r >> 5, l = r & 31;
    const uint32_t ql = blk[64 * half + 32 * (grp & 1) + l], qh = blk[128 + 32 * half + l];
    const int q = (int)(((ql >> (4 * (grp >> 1))) & 0xfu) | (((qh >> (2 * grp)) & 3u) << 4)) - 32;
    const float d = h2f(reinterpret_cast<const u16_a2*>(blk + 208)->v);
    const int sc = (int)(int8_t)blk[192 + 8 * half + 2 * grp + (l >> 4)];
    return d * (float)sc * (float)q;
}

__global__ __launch_bounds__(256) void embedding_rows_kernel(const float* __restrict__ table_f32,
                                                             const uint8_t* __restrict__ table_q6k, int64_t stride,
                                                             const int* __restrict__ tokens, int hidden, int vocab,
                                                             float* __restrict__ out) {
    const int m = blockIdx.y;
    int tok = tokens[m];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);  // ids are validated on the host; never read outside the table
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= hidden) return;
    float v;
    if (table_f32) v = table_f32[(int64_t)tok * hidden + i];
    else v = pf_q6k_elem(table_q6k + (int64_t)tok * stride + (int64_t)(i >> 8) * 210, i & 255);
    out[(int64_t)m * hidden + i] = v;
}

// PART: q, k and v arrive as the K-split partial sums a multi-matrix GEMM launch left (per matrix: `splits` slabs of
// rows x width floats, summed here in slab order, then the optional bias: the arithmetic of the split reduction and of
// add_qkv_bias_kernel), and only what the attention reads is written: the rotated q rows and the cache rows.
struct QkvParts {
    const float* P[3];  // q, k, v; a matrix that was not split points at its finished rows (splits 1)
    int splits[3];
    const float* bias[3];  // NULL: none
};
__device__ __forceinline__ float qkv_part_load(const float* __restrict__ P, int splits, int64_t total, int64_t idx,
                                               const float* __restrict__ bias, int col) {
    // four slabs per batch, fetched unconditionally (the slab index clamped) so that they are in flight together
    float a = 0.0f;
    for (int z0 = 0; z0 < splits; z0 += 4) {
        float b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) b[u] = P[(int64_t)min(z0 + u, splits - 1) * total + idx];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (z0 + u == 0) a = b[u];
            else if (z0 + u < splits) a += b[u];
        }
    }
    return bias ? a + bias[col] : a;
}

// grid (rows, n_heads + n_kv_heads), one wave; lane t owns the rotation pair (t, t + head_dim/2)
template <bool KV16, bool PART>
__global__ __launch_bounds__(64) void qknorm_rope_kv_rows_kernel(float* __restrict__ Q, float* __restrict__ K,
                                                                 const float* __restrict__ V, const float* __restrict__ qw,
                                                                 const float* __restrict__ kw, void* __restrict__ Kc,
                                                                 void* __restrict__ Vc, const float* __restrict__ rope,
                                                                 int n_heads, int n_kv_heads, int head_dim, int64_t pos0,
                                                                 float eps, int add_one, int rope_interleaved,
                                                                 const QkvParts parts) {
    const int m = blockIdx.x, hb = blockIdx.y;
    const bool is_k = hb >= n_heads;
    const int h = is_k ? hb - n_heads : hb;
    const int64_t pos = pos0 + m;
    const int kv_dim = n_kv_heads * head_dim;
    float* vec = is_k ? K + (int64_t)m * kv_dim + (int64_t)h * head_dim
                      : Q + ((int64_t)m * n_heads + h) * head_dim;
    const float* nw = is_k ? kw : qw;
    const int half = head_dim / 2;
    const float* cs = rope + pos * head_dim;
    const int rows = gridDim.x;
    const int width = is_k ? kv_dim : n_heads * head_dim;       // row width of the matrix this head belongs to
    const int64_t row_off = (int64_t)m * width + (int64_t)h * head_dim;
    auto src = [&](int i) {
        if constexpr (PART) {
            const int w = is_k ? 1 : 0;
            return qkv_part_load(parts.P[w], parts.splits[w], (int64_t)rows * width, row_off + i, parts.bias[w], h * head_dim + i);
        } else {
            return vec[i];
        }
    };
    // thread t owns rotation pairs t and t + 64 (the second only for heads wider than 128)
    float x0[2], x1[2];
    int i0[2], i1[2];
    bool on[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int t = threadIdx.x + 64 * j;
        on[j] = t < half;
        i0[j] = rope_interleaved ? 2 * t : t;
        i1[j] = rope_interleaved ? 2 * t + 1 : t + half;
        x0[j] = on[j] ? src(i0[j]) : 0.0f;
        x1[j] = on[j] ? src(i1[j]) : 0.0f;
    }
    if (nw) {
        float ss = fmaf(x0[0], x0[0], 0.0f);
        ss = fmaf(x1[0], x1[0], ss);
        ss = fmaf(x0[1], x0[1], ss);
        ss = fmaf(x1[1], x1[1], ss);
        ss = sum64(ss);
        const float rs = 1.0f / sqrtf(ss / (float)head_dim + eps);
        const float one = add_one ? 1.0f : 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            if (on[j]) {
                x0[j] = x0[j] * rs * (nw[i0[j]] + one);
                x1[j] = x1[j] * rs * (nw[i1[j]] + one);
            }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        if (!on[j]) continue;
        const int t = threadIdx.x + 64 * j;
        const float c = cs[t], s = cs[half + t];
        const float r0 = fmaf(x0[j], c, -(x1[j] * s)), r1 = fmaf(x0[j], s, x1[j] * c);  // hot_loops.cpp:2035-2061
        if (!PART || !is_k) {  // the rotated fp32 K rows have no reader in the prompt pass
            vec[i0[j]] = r0;
            vec[i1[j]] = r1;
        }
        if (is_k) {
            const int64_t off = pos * kv_dim + (int64_t)h * head_dim;
            float v0, v1;
            if constexpr (PART) {
                v0 = qkv_part_load(parts.P[2], parts.splits[2], (int64_t)rows * kv_dim, row_off + t, parts.bias[2], h * head_dim + t);
                v1 = qkv_part_load(parts.P[2], parts.splits[2], (int64_t)rows * kv_dim, row_off + t + half, parts.bias[2], h * head_dim + t + half);
            } else {
                v0 = V[(int64_t)m * kv_dim + (int64_t)h * head_dim + t];
                v1 = V[(int64_t)m * kv_dim + (int64_t)h * head_dim + t + half];
            }
            if constexpr (KV16) {
                __half* kc = static_cast<__half*>(Kc) + off;
                __half* vc = static_cast<__half*>(Vc) + off;
                kc[i0[j]] = __float2half_rn(r0);
                kc[i1[j]] = __float2half_rn(r1);
                vc[t] = __float2half_rn(v0);
                vc[t + half] = __float2half_rn(v1);
            } else {
                float* kc = static_cast<float*>(Kc) + off;
                float* vc = static_cast<float*>(Vc) + off;
                kc[i0[j]] = r0;
                kc[i1[j]] = r1;
                vc[t] = v0;
                vc[t + half] = v1;
            }
        }
    }
}

// Four values of a q / k / v row that may still be K-split partial sums: slab z holds them at P + z * total + idx
__device__ __forceinline__ float4 qkv_part_load4(const float* __restrict__ P, int splits, int64_t total, int64_t idx,
                                                 const float* __restrict__ bias, int col) {
    float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (int z0 = 0; z0 < splits; z0 += 4) {  // four slabs per batch, the slab index clamped: in flight together
        float4 b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) b[u] = *reinterpret_cast<const float4*>(P + (int64_t)min(z0 + u, splits - 1) * total + idx);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (z0 + u == 0) a = b[u];
            else if (z0 + u < splits) { a.x += b[u].x; a.y += b[u].y; a.z += b[u].z; a.w += b[u].w; }
        }
    }
    if (bias) {
        const float4 bb = *reinterpret_cast<const float4*>(bias + col);
        a.x += bb.x; a.y += bb.y; a.z += bb.z; a.w += bb.w;
    }
    return a;
}

// The same work with head_dim / 8 lanes per head (head_dim 32, 64, 128 or 256) and 16-byte accesses: a lane owns four
// rotation pairs (two runs of four elements), a wave 64 / (head_dim / 8) heads of one row.  grid (rows, q head blocks + kv
// head blocks), one wave.  With one wave per (row, head) and 4-byte accesses the launch was bound by the number of
// workgroups and requests: 82 k single-wave workgroups for 2048 rows of 40 heads.
template <bool KV16, bool PART>
__global__ __launch_bounds__(64) void qknorm_rope_kv_rows_quad_kernel(float* __restrict__ Q, float* __restrict__ K,
                                                                      const float* __restrict__ V, const float* __restrict__ qw,
                                                                      const float* __restrict__ kw, void* __restrict__ Kc,
                                                                      void* __restrict__ Vc, const float* __restrict__ rope,
                                                                      int n_heads, int n_kv_heads, int head_dim, int64_t pos0,
                                                                      float eps, int add_one, int rope_interleaved,
                                                                      const QkvParts parts) {
    const int m = blockIdx.x, rows = gridDim.x;
    const int lph = head_dim >> 3, hpw = 64 / lph;  // lanes per head, heads per wave
    const int q_blocks = (n_heads + hpw - 1) / hpw;
    const bool is_k = (int)blockIdx.y >= q_blocks;
    const int hblk = is_k ? blockIdx.y - q_blocks : blockIdx.y;
    const int lane = threadIdx.x, l = lane & (lph - 1);
    const int nh = is_k ? n_kv_heads : n_heads;
    const int h_raw = hblk * hpw + lane / lph;
    const bool live = h_raw < nh;
    const int h = live ? h_raw : nh - 1;  // idle lanes of the last block read the last head and store nothing
    const int half = head_dim / 2, kv_dim = n_kv_heads * head_dim;
    const int64_t pos = pos0 + m;
    // the lane's two runs: NeoX pairs (4 l + e, half + 4 l + e); interleaved pairs (8 l + 2 e, 8 l + 2 e + 1) lie in
    // elements 8 l .. 8 l + 7.  Either way they are the pairs 4 l .. 4 l + 3 of the rotation table.
    const int e0 = rope_interleaved ? 8 * l : 4 * l, e1 = rope_interleaved ? 8 * l + 4 : half + 4 * l;
    const int width = is_k ? kv_dim : n_heads * head_dim;
    const int64_t row_off = (int64_t)m * width + (int64_t)h * head_dim;
    float* vec = (is_k ? K : Q) + row_off;
    const int w = is_k ? 1 : 0;
    float4 a, b, va, vb;
    va = vb = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if constexpr (PART) {
        const int64_t total = (int64_t)rows * width;
        a = qkv_part_load4(parts.P[w], parts.splits[w], total, row_off + e0, parts.bias[w], h * head_dim + e0);
        b = qkv_part_load4(parts.P[w], parts.splits[w], total, row_off + e1, parts.bias[w], h * head_dim + e1);
        if (is_k) {
            va = qkv_part_load4(parts.P[2], parts.splits[2], total, row_off + e0, parts.bias[2], h * head_dim + e0);
            vb = qkv_part_load4(parts.P[2], parts.splits[2], total, row_off + e1, parts.bias[2], h * head_dim + e1);
        }
    } else {
        a = *reinterpret_cast<const float4*>(vec + e0);
        b = *reinterpret_cast<const float4*>(vec + e1);
        if (is_k) {
            va = *reinterpret_cast<const float4*>(V + row_off + e0);
            vb = *reinterpret_cast<const float4*>(V + row_off + e1);
        }
    }
    const float* cs = rope + pos * head_dim;
    const float4 c4 = *reinterpret_cast<const float4*>(cs + 4 * l), s4 = *reinterpret_cast<const float4*>(cs + half + 4 * l);
    const float* nw = is_k ? kw : qw;
    if (nw) {
        float ss = fmaf(a.x, a.x, 0.0f);
        ss = fmaf(a.y, a.y, ss); ss = fmaf(a.z, a.z, ss); ss = fmaf(a.w, a.w, ss);
        ss = fmaf(b.x, b.x, ss); ss = fmaf(b.y, b.y, ss); ss = fmaf(b.z, b.z, ss); ss = fmaf(b.w, b.w, ss);
        for (int o = lph >> 1; o >= 1; o >>= 1) ss += __shfl_xor(ss, o, 64);  // within the head's lanes
        const float rs = 1.0f / sqrtf(ss / (float)head_dim + eps);
        const float one = add_one ? 1.0f : 0.0f;
        const float4 wa = *reinterpret_cast<const float4*>(nw + e0), wb = *reinterpret_cast<const float4*>(nw + e1);
        a.x = a.x * rs * (wa.x + one); a.y = a.y * rs * (wa.y + one); a.z = a.z * rs * (wa.z + one); a.w = a.w * rs * (wa.w + one);
        b.x = b.x * rs * (wb.x + one); b.y = b.y * rs * (wb.y + one); b.z = b.z * rs * (wb.z + one); b.w = b.w * rs * (wb.w + one);
    }
    // rotation of pair (x0, x1) by (c, s): (x0 c - x1 s, x0 s + x1 c)  (hot_loops.cpp:2035-2061)
    auto rot = [](float& x0, float& x1, float c, float s) {
        const float r0 = fmaf(x0, c, -(x1 * s)), r1 = fmaf(x0, s, x1 * c);
        x0 = r0;
        x1 = r1;
    };
    if (rope_interleaved) {
        rot(a.x, a.y, c4.x, s4.x); rot(a.z, a.w, c4.y, s4.y); rot(b.x, b.y, c4.z, s4.z); rot(b.z, b.w, c4.w, s4.w);
    } else {
        rot(a.x, b.x, c4.x, s4.x); rot(a.y, b.y, c4.y, s4.y); rot(a.z, b.z, c4.z, s4.z); rot(a.w, b.w, c4.w, s4.w);
    }
    if (!live) return;
    if (!PART || !is_k) {  // the rotated fp32 K rows have no reader in the prompt pass
        *reinterpret_cast<float4*>(vec + e0) = a;
        *reinterpret_cast<float4*>(vec + e1) = b;
    }
    if (is_k) {
        const int64_t off = pos * kv_dim + (int64_t)h * head_dim;
        if constexpr (KV16) {
            auto pack = [](const float4& v) {
                const __half2 lo = __floats2half2_rn(v.x, v.y), hi = __floats2half2_rn(v.z, v.w);
                uint2 r;
                __builtin_memcpy(&r.x, &lo, 4);
                __builtin_memcpy(&r.y, &hi, 4);
                return r;
            };
            __half* kc = static_cast<__half*>(Kc) + off;
            __half* vc = static_cast<__half*>(Vc) + off;
            *reinterpret_cast<uint2*>(kc + e0) = pack(a);
            *reinterpret_cast<uint2*>(kc + e1) = pack(b);
            *reinterpret_cast<uint2*>(vc + e0) = pack(va);
            *reinterpret_cast<uint2*>(vc + e1) = pack(vb);
        } else {
            float* kc = static_cast<float*>(Kc) + off;
            float* vc = static_cast<float*>(Vc) + off;
            *reinterpret_cast<float4*>(kc + e0) = a;
            *reinterpret_cast<float4*>(kc + e1) = b;
            *reinterpret_cast<float4*>(vc + e0) = va;
            *reinterpret_cast<float4*>(vc + e1) = vb;
        }
    }
}

// launches the 16-byte kernel when the shape and the pointers allow it, the one-wave-per-head kernel otherwise
template <bool PART>
static int qknorm_rope_kv_rows_launch(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                      void* K_cache, void* V_cache, const float* rope_table, int rows, int n_heads,
                                      int n_kv_heads, int head_dim, int64_t pos0, float eps, int add_one, int kv_fp16,
                                      int rope_interleaved, const QkvParts& parts, hipStream_t s) {
    bool quad = head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256;
    quad = quad && aligned16(Q) && aligned16(K) && aligned16(V) && aligned16(q_norm_w) && aligned16(k_norm_w) &&
           aligned16(K_cache) && aligned16(V_cache) && aligned16(rope_table);
    for (int i = 0; i < 3; ++i) quad = quad && aligned16(parts.P[i]) && aligned16(parts.bias[i]);
#define PTM_QK(KERNEL, KV16, GRID)                                                                                         \
    hipLaunchKernelGGL((KERNEL<KV16, PART>), GRID, dim3(64), 0, s, Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, rope_table, \
                       n_heads, n_kv_heads, head_dim, pos0, eps, add_one, rope_interleaved ? 1 : 0, parts)
    if (quad) {
        const int hpw = 64 / (head_dim / 8);
        const dim3 grid(rows, (n_heads + hpw - 1) / hpw + (n_kv_heads + hpw - 1) / hpw);
        if (kv_fp16) PTM_QK(qknorm_rope_kv_rows_quad_kernel, true, grid);
        else PTM_QK(qknorm_rope_kv_rows_quad_kernel, false, grid);
    } else {
        const dim3 grid(rows, n_heads + n_kv_heads);
        if (kv_fp16) PTM_QK(qknorm_rope_kv_rows_kernel, true, grid);
        else PTM_QK(qknorm_rope_kv_rows_kernel, false, grid);
    }
#undef PTM_QK
    return launch_status();
}

template <bool KV16>
__device__ __forceinline__ void pf_load8(const void* base, int64_t elem_off, float (&o)[8]) {
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

// grid (ceil(rows / 4), n_kv_heads), 4 waves = 4 consecutive rows of one kv head
template <bool KV16, int HD, int G>
__global__ __launch_bounds__(256) void prefill_attn_kernel(const float* __restrict__ Q, const void* __restrict__ Kc,
                                                           const void* __restrict__ Vc, float* __restrict__ O, int rows,
                                                           int n_heads, int n_kv_heads, int64_t pos0, float scale,
                                                           int window) {
    constexpr int LPP = HD / 8, PPW = 64 / LPP;  // lanes per position, positions per wave and pass
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = blockIdx.x * 4 + wave, kvh = blockIdx.y;
    if (m >= rows) return;  // wave-uniform; no barriers below
    const int dl = lane % LPP, pl = lane / LPP;
    const int kv_dim = n_kv_heads * HD;
    const int64_t col = (int64_t)kvh * HD + dl * 8;
    const int64_t limit = pos0 + m;  // last position this row may attend to (itself)
    // window > 0: the row sees positions (limit - window, limit] only (gemma3 local layers, gguf_model.h:3490-3500)
    const int64_t lo = (window > 0 && limit + 1 > window) ? limit + 1 - window : 0;

    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float* src = Q + ((int64_t)m * n_heads + kvh * G + g) * HD + dl * 8;
        const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
        q[g][0] = a.x; q[g][1] = a.y; q[g][2] = a.z; q[g][3] = a.w;
        q[g][4] = b.x; q[g][5] = b.y; q[g][6] = b.z; q[g][7] = b.w;
    }
    float mrun[G], lsum[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        mrun[g] = -INFINITY;
        lsum[g] = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
    }
    const int64_t n_pass = limit / PPW + 1, pass0 = lo / PPW;
    float kn[8], vn[8];
    {
        const int64_t tf = pass0 * PPW + pl;
        const int64_t tc = tf <= limit ? tf : limit;
        pf_load8<KV16>(Kc, tc * kv_dim + col, kn);
        pf_load8<KV16>(Vc, tc * kv_dim + col, vn);
    }
    for (int64_t pass = pass0; pass < n_pass; ++pass) {
        float k[8], v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { k[i] = kn[i]; v[i] = vn[i]; }
        const int64_t t = pass * PPW + pl;
        if (pass + 1 < n_pass) {  // next pass's rows are requested before this pass's arithmetic
            const int64_t tn = t + PPW;
            const int64_t tc = tn <= limit ? tn : limit;
            pf_load8<KV16>(Kc, tc * kv_dim + col, kn);
            pf_load8<KV16>(Vc, tc * kv_dim + col, vn);
        }
        const bool valid = t <= limit && t >= lo;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) d = fmaf(q[g][i], k[i], d);
            d = sum_lanes<LPP>(d);
            const float s = valid ? d * scale : -INFINITY;
            const float mnew = fmaxf(mrun[g], s);
            const float muse = mnew == -INFINITY ? 0.0f : mnew;
            const float corr = pf_exp(mrun[g] - muse);  // -inf -> 0 on the first valid position
            const float p = pf_exp(s - muse);
            lsum[g] = fmaf(lsum[g], corr, p);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[g][i] = fmaf(acc[g][i], corr, p * v[i]);
            mrun[g] = mnew;
        }
    }
    // merge the PPW position slots of the wave (lanes with equal dl)
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float M = mrun[g];
        for (int off = LPP; off < 64; off <<= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
        const float w = pf_exp(mrun[g] - M);  // M is finite: the row's own position is valid for one of the slots
        float l = lsum[g] * w;
        for (int off = LPP; off < 64; off <<= 1) l += __shfl_xor(l, off, 64);
        const float inv = 1.0f / (l + 1e-10f);  // reference: inv_sum = 1/(sum_exp + 1e-10f), gguf_model.h:3589
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float a = acc[g][i] * w;
            for (int off = LPP; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
            acc[g][i] = a * inv;
        }
        if (pl == 0) {
            float* dst = O + ((int64_t)m * n_heads + kvh * G + g) * HD + dl * 8;
            *reinterpret_cast<float4*>(dst) = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
        }
    }
}

// ---- matrix-core version (fp16 cache) ----------------------------------------------------------------------------
typedef _Float16 pf_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 pf_h4 __attribute__((ext_vector_type(4)));
typedef short pf_s4 __attribute__((ext_vector_type(4)));
// ds_read_b64_tr_b16: within each group of 16 lanes, lane i passes the address of four 16-bit values (a row i / 4 of the caller's
// choice, columns 4 (i % 4) .. +3 of a 16-column block) and receives column i of the four rows: the transposition a V tile stored
// position-major needs to become the A operand V^T[d][positions] of the MFMA.
__device__ __forceinline__ pf_h4 lds_read_tr16(const uint8_t* p) {
    typedef __attribute__((address_space(3))) pf_s4 lds_s4;
    return __builtin_bit_cast(pf_h4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)p));
}
typedef float pf_f16v __attribute__((ext_vector_type(16)));

// v_mfma_f32_32x32x16_f16 operand layout used below: A (32 x 16): lane l holds row l % 32, summation indices
// 8 (l / 32) + 0..7; B (16 x 32): lane l holds column l % 32, the same indices; C (32 x 32): lane l holds column
// l % 32, rows 8 (r / 4) + 4 (l / 32) + r % 4 for r = 0..15.  The summation index may be permuted freely as long as A
// and B agree, which is used twice: the 16 head-dim elements of a step are [16 ks + 8 kh, +8) for lane half kh,
// and the 16 positions of a P.V step are the ones the lane already holds in its S^T accumulator.
// NG groups of four waves (256 NG threads): every group holds the same 32 G-head query rows; with two groups, group g takes
// the pairs of 32-position tiles (4 s + 2 g, 4 s + 2 g + 1) into its own staging buffers (the barriers are shared) and the two
// online-softmax states are merged through LDS at the end, which halves the number of steps of a row block's chain and gives
// each SIMD a second wave.  Tile indices are absolute, so with a given NG a row's arithmetic does not depend on how the prompt
// was chunked.
// G query heads per kv head: a row takes GP = the next power of two slots of a wave's 32 query vectors (G = 3: 4, G = 5..7: 8);
// the slots past G repeat the last head and are not stored.  window > 0: a query at position p attends to (p - window, p]
// only: the tile walk starts at the first tile any query of the workgroup can see, and the tiles that reach below some
// query's window are masked like the diagonal ones.
// DS = 2 (head dimension 256, one group): waves w and w + 4 hold the same 32 query vectors and each computes all scores but
// only one half of the output's head dimension, staging the tiles together.  A wave with the whole 256-wide output would
// need 128 accumulator registers beside 64 of q fragments and 64 of tile pieces in flight: one wave per SIMD; with the
// output split a SIMD holds two, and the repeated score MFMAs (half of a tile's work) cost less than the idle pipes would.
template <int HD, int G, int NG, int DS = 1>
__global__ __launch_bounds__(256 * NG * DS) void prefill_attn_mfma_kernel(const float* __restrict__ Q, const __half* __restrict__ Kc,
                                                                const __half* __restrict__ Vc, float* __restrict__ O, int rows,
                                                                int n_heads, int n_kv_heads, int64_t pos0, float scale, int window) {
    constexpr int GP = G <= 1 ? 1 : G <= 2 ? 2 : G <= 4 ? 4 : 8;   // head slots per row
    constexpr int RPW = 32 / GP;       // rows per wave (each with its GP head slots: 32 query vectors)
    constexpr int BM = 4 * RPW;        // rows per workgroup
    constexpr int KS = HD / 16;        // MFMA steps over the head dimension
    constexpr int DT = HD / 32 / DS;   // 32-wide tiles of the output's head dimension that this wave accumulates
    static_assert(DS == 1 || (DS == 2 && NG == 1), "the output is split over the two wave sets of a single group");
    constexpr int KP = HD * 2 + 16;    // LDS pitch of a K row (bytes)
    constexpr int VP = HD * 2 + 64;    // LDS pitch of a V row: 16 of the 64 banks on: the 32 lanes served together by a transposing
                                       // read (4 rows x 2 blocks of 16 columns) cover all banks (measured: 191 ns per 64 KB against 238 with + 32)
    constexpr int SN = 256 * DS;            // threads that stage a group's tiles
    constexpr int PCS = 32 * HD / 8 / SN;   // 16-byte pieces of a 32-position tile per thread (1 or 2)
    static_assert(PCS == 1 || PCS == 2, "tile smaller than the workgroup");
    // LDS: per group two K tiles and two V tiles; the merge buffer (group 1's accumulators, running maximum and sum,
    // lane-contiguous) takes the same memory once the tiles are done, which keeps a workgroup under half the CU's LDS
    constexpr int K_BYTES = 32 * KP, VT_BYTES = 32 * VP, STAGE_BYTES = 2 * NG * (K_BYTES + VT_BYTES);
    constexpr int MERGE_BYTES = NG == 2 ? 4 * (16 * DT + 2) * 64 * 4 : 0;
    __shared__ __align__(16) uint8_t s_raw[STAGE_BYTES > MERGE_BYTES ? STAGE_BYTES : MERGE_BYTES];
    float (*s_merge)[16 * DT + 2][64] = reinterpret_cast<float (*)[16 * DT + 2][64]>(s_raw);
    const int grp = NG == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;  // wave-uniform: tile counters stay scalar
    uint8_t* const s_k = s_raw + grp * 2 * (K_BYTES + VT_BYTES);  // the group's two K tiles, then its two V tiles
    uint8_t* const s_vt = s_k + 2 * K_BYTES;
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, kh = lane >> 5;
    const int dh = DS == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;  // which half of the output's head dimension
    const int stid = DS == 2 ? (int)threadIdx.x : tid;                              // index among the staging threads
    // Workgroups start in the order of their linear index, and a row block's work grows with its first row: the index runs
    // over the kv heads fastest and from the last row block down, so the longest workgroups of ALL heads start first and the
    // short ones fill the tail (with the heads outermost, a late head's longest blocks would start after the early heads'
    // short ones and run alone at the end).  With 8 kv heads a head's workgroups also share one XCD and its L2.
    const int wg = blockIdx.x + gridDim.x * blockIdx.y;
    const int kvh = wg % (int)gridDim.y;
    const int m_base = ((int)gridDim.x - 1 - wg / (int)gridDim.y) * BM;
    const int kv_dim = n_kv_heads * HD;

    const int slot = j % GP;
    const bool dead = slot >= G;       // a padding slot: computed like its row's last head, never stored
    const int row = m_base + wave * RPW + j / GP, head = kvh * G + (dead ? G - 1 : slot);
    const int row_c = row < rows ? row : rows - 1;
    const int64_t limit = pos0 + row_c;  // last position this query attends to
    const int64_t lowest = window > 0 ? limit - window + 1 : 0;   // first one
    // scores are kept in base 2: q is scaled by scale * log2(e) before its rounding to fp16
    const float qs = scale * 1.44269504088896340736f;
    pf_h8 qf[KS];
    {
        const float* src = Q + ((int64_t)row_c * n_heads + head) * HD + 8 * kh;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const float4 a = *reinterpret_cast<const float4*>(src + 16 * ks), b = *reinterpret_cast<const float4*>(src + 16 * ks + 4);
            qf[ks] = pf_h8{(_Float16)(a.x * qs), (_Float16)(a.y * qs), (_Float16)(a.z * qs), (_Float16)(a.w * qs),
                           (_Float16)(b.x * qs), (_Float16)(b.y * qs), (_Float16)(b.z * qs), (_Float16)(b.w * qs)};
        }
    }
    pf_f16v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    const int last_row = (m_base + BM < rows ? m_base + BM : rows) - 1;
    const int64_t t_end = pos0 + last_row;  // last position any query of this workgroup attends to
    const int ntiles = (int)(t_end / 32) + 1;
    // with a window: the first position any query of the workgroup sees (its first row's), and the first position ALL of
    // them see (its last row's): tiles below the former are skipped, tiles below the latter are masked
    const int64_t t_first = window > 0 && pos0 + m_base - window + 1 > 0 ? pos0 + m_base - window + 1 : 0;
    const int64_t t_all = window > 0 ? t_end - window + 1 : 0;
    // The group's next pair of tiles is in flight in registers (sets A and B) while the current pair is worked on: the rows
    // come from HBM or L2.  Every fetch is unconditional (tile indices past the end are clamped), so the number of loads in
    // flight at each wait is static.
    uint4 kA0, kA1, vA0, vA1, kB0, kB1, vB0, vB1;  // scalars, not arrays: they must stay in registers across the loop
    kA1 = vA1 = kB1 = vB1 = make_uint4(0, 0, 0, 0);
    // Piece i of a thread, for K and V alike: position (stid + SN i) / (HD / 8), elements 8 ((stid + SN i) % (HD / 8)) .. +8 (a
    // wave reads whole rows).  Byte offsets into the caches fit 32 bits (checked at launch); a piece's offset for a tile is its
    // offset in tile 0 plus the tile's, clamped to the same piece of the last visible position: rows past the end are masked
    // below and nothing is read past the appended rows.
    uint32_t pc_off[PCS], pc_max[PCS], pc_lds_k[PCS], pc_lds_v[PCS];
#pragma unroll
    for (int i = 0; i < PCS; ++i) {
        const int q = stid + SN * i, p = q / (HD / 8), c = q % (HD / 8);
        const uint32_t col = (uint32_t)(kvh * HD + 8 * c);
        pc_off[i] = ((uint32_t)p * (uint32_t)kv_dim + col) * 2u;
        pc_max[i] = ((uint32_t)t_end * (uint32_t)kv_dim + col) * 2u;
        pc_lds_k[i] = p * KP + 16 * c;
        pc_lds_v[i] = p * VP + 16 * c;
    }
    const uint32_t tile_bytes = 32u * (uint32_t)kv_dim * 2u;
    const char* const Kb = reinterpret_cast<const char*>(Kc);
    const char* const Vb = reinterpret_cast<const char*>(Vc);
    auto fetch_from = [&](const char* base, int tile, uint4& r0, uint4& r1) {
        tile = tile < ntiles ? tile : ntiles - 1;
        const uint32_t tb = (uint32_t)tile * tile_bytes;
        r0 = *reinterpret_cast<const uint4*>(base + min(pc_off[0] + tb, pc_max[0]));
        if constexpr (PCS > 1) r1 = *reinterpret_cast<const uint4*>(base + min(pc_off[1] + tb, pc_max[1]));
    };
    auto fetch = [&](int tile, uint4& k0, uint4& v0, uint4& k1, uint4& v1) {
        fetch_from(Kb, tile, k0, k1);
        fetch_from(Vb, tile, v0, v1);
    };
    auto stage = [&](int buf, int i, const uint4& kr, const uint4& vr) {
        *reinterpret_cast<uint4*>(s_k + buf * K_BYTES + pc_lds_k[i]) = kr;
        *reinterpret_cast<uint4*>(s_vt + buf * VT_BYTES + pc_lds_v[i]) = vr;
    };
    // One step = two adjacent tiles of the group (64 positions): both are staged behind one pair of barriers, their score
    // MFMA chains are independent (the matrix pipe runs one while the other's operands arrive), and they share one pass of the
    // online softmax (one maximum, one correction, one rescale test).  The register sets are refilled with the group's next
    // pair during the step.
    auto do_step = [&](int t0) {
        __syncthreads();  // every wave has finished reading the previous pair
        stage(0, 0, kA0, vA0);
        if constexpr (PCS > 1) stage(0, 1, kA1, vA1);
        stage(1, 0, kB0, vB0);
        if constexpr (PCS > 1) stage(1, 1, kB1, vB1);
        __syncthreads();
        // the next pair's K pieces are requested here, its V pieces behind the score MFMAs: one burst of eight loads per
        // lane held up the LDS reads queued behind it (2048 rows 63.8 -> 62.1 us, 512 rows at position 1536 50.5 -> 46.3)
        fetch_from(Kb, t0 + 2 * NG, kA0, kA1);
        fetch_from(Kb, t0 + 2 * NG + 1, kB0, kB1);
        issue_order_fence();

        // S^T tiles: rows = a tile's 32 positions, column = this lane's query vector.  K fragments are read four at a time, so
        // the MFMAs wait for a batch instead of each for its own read.
        pf_f16v sc[2];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[u][r] = 0.0f;
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += 4)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                pf_h8 ka[4];
#pragma unroll
                for (int w = 0; w < 4; ++w) ka[w] = *reinterpret_cast<const pf_h8*>(s_k + u * K_BYTES + j * KP + (16 * (k0 + w) + 8 * kh) * 2);
#pragma unroll
                for (int w = 0; w < 4; ++w) asm volatile("" : "+v"(ka[w]));  // no MFMA is moved up to behind its own read
#pragma unroll
                for (int w = 0; w < 4; ++w) sc[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[w], qf[k0 + w], sc[u], 0, 0, 0);
            }
        issue_order_fence();
        fetch_from(Vb, t0 + 2 * NG, vA0, vA1);
        fetch_from(Vb, t0 + 2 * NG + 1, vB0, vB1);
        issue_order_fence();
        // only the tiles on the diagonal hold positions some query of the workgroup must not see (workgroup-uniform)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int tile = t0 + u;
            if ((int64_t)tile * 32 + 31 > pos0 + m_base) {
                issue_order_fence();  // keeps this a branch: as selects it would cost every tile 50 instructions
                const int lim = (int)(limit - (int64_t)tile * 32) - 4 * kh;  // position offsets of this lane: 8 (r / 4) + r % 4
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[u][r] = 8 * (r >> 2) + (r & 3) <= lim ? sc[u][r] : -INFINITY;
            }
            if ((int64_t)tile * 32 < t_all) {   // the window's lower edge (workgroup-uniform; never taken without a window)
                issue_order_fence();
                const int64_t lo64 = lowest - (int64_t)tile * 32 - 4 * kh;
                const int lo = lo64 > 64 ? 64 : (int)lo64;
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[u][r] = 8 * (r >> 2) + (r & 3) >= lo ? sc[u][r] : -INFINITY;
            }
        }
        // v_max3_f32 by hand: fmaxf() first quiets each MFMA result with an instruction of its own (no NaN can occur here)
        float mx = sc[0][0];
        asm("v_max_f32 %0, %0, %1" : "+v"(mx) : "v"(sc[1][0]));
#pragma unroll
        for (int r = 1; r < 16; ++r) asm("v_max3_f32 %0, %0, %1, %2" : "+v"(mx) : "v"(sc[0][r]), "v"(sc[1][r]));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));  // the column's other positions
        const float m_new = fmaxf(m_run, mx);
        // group 1 may have seen no visible position of a query yet (-inf): exponentials then take 0 as the reference and are 0
        const float ms = m_new == -INFINITY ? 0.0f : m_new;
        const float corr = __builtin_amdgcn_exp2f(m_run - ms);
        float psum = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                sc[u][r] = __builtin_amdgcn_exp2f(sc[u][r] - ms);
                psum += sc[u][r];
            }
        l_run = fmaf(l_run, corr, psum);  // this lane's positions; the two lane halves are added at the end
        // a running maximum that no lane of the wave has raised leaves every correction at exactly 1: the rescale is skipped
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(m_new != m_run) != 0, 0)) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[dt][r] *= corr;
        }
        m_run = m_new;
        // O^T += V^T . P^T: step ks of a tile sums the positions of its accumulator registers 8 ks .. 8 ks + 7
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const pf_h8 pb0 = {(_Float16)sc[u][0], (_Float16)sc[u][1], (_Float16)sc[u][2], (_Float16)sc[u][3],
                               (_Float16)sc[u][4], (_Float16)sc[u][5], (_Float16)sc[u][6], (_Float16)sc[u][7]};
            const pf_h8 pb1 = {(_Float16)sc[u][8], (_Float16)sc[u][9], (_Float16)sc[u][10], (_Float16)sc[u][11],
                               (_Float16)sc[u][12], (_Float16)sc[u][13], (_Float16)sc[u][14], (_Float16)sc[u][15]};
            pf_h4 vlo[2][DT], vhi[2][DT];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    // positions 16 ks + 4 kh .. +3 and the same + 8 of V column 32 dt + j (the lane's S^T rows)
                    const uint8_t* vrow = s_vt + u * VT_BYTES + (16 * ks + 4 * kh + ((lane & 15) >> 2)) * VP +
                                          (32 * (dt + DT * dh) + (j & 16) + 4 * (lane & 3)) * 2;
                    vlo[ks][dt] = lds_read_tr16(vrow);
                    vhi[ks][dt] = lds_read_tr16(vrow + 8 * VP);
                }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const pf_h4 lo = vlo[ks][dt], hi = vhi[ks][dt];
                    const pf_h8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, ks ? pb1 : pb0, acc[dt], 0, 0, 0);
                }
        }
    };
    // Group g takes the tile pairs (4 s + 2 g, 4 s + 2 g + 1); a tile index past the end is a tile of masked positions (its
    // fetch is clamped, its probabilities are exact zeros), so both groups run the same number of steps and meet at every
    // barrier; nothing is conditional between the steps, so the count of loads in flight at each wait stays static.
    const int st0 = (int)(t_first / 32) / (2 * NG);   // the step that holds the first visible tile
    fetch(2 * NG * st0 + 2 * grp, kA0, vA0, kA1, vA1);
    fetch(2 * NG * st0 + 2 * grp + 1, kB0, vB0, kB1, vB1);
    const int nsteps = (ntiles + 2 * NG - 1) / (2 * NG);
    for (int st = st0; st < nsteps; ++st) do_step(2 * NG * st + 2 * grp);
    // ---- merge the two groups' states (same lane of waves w and w + 4 = same query vector, same output elements) ----
    if constexpr (NG == 2) {
    __syncthreads();  // the merge buffer overlays the tiles: every wave has finished its last tile
    if (grp == 1) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) s_merge[wave][16 * dt + r][lane] = acc[dt][r];
        s_merge[wave][16 * DT][lane] = m_run;
        s_merge[wave][16 * DT + 1][lane] = l_run;
    }
    __syncthreads();
    if (grp == 1) return;
    {
        const float m1 = s_merge[wave][16 * DT][lane], l1 = s_merge[wave][16 * DT + 1][lane];
        const float mm0 = fmaxf(m_run, m1);  // finite unless a window hides every tile of one group from this query
        const float mm = mm0 == -INFINITY ? 0.0f : mm0;
        const float c0 = __builtin_amdgcn_exp2f(m_run - mm), c1 = __builtin_amdgcn_exp2f(m1 - mm);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] = fmaf(acc[dt][r], c0, s_merge[wave][16 * dt + r][lane] * c1);
        l_run = fmaf(l_run, c0, l1 * c1);
    }
    }
    const float l = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / (l + 1e-10f);  // reference: inv_sum = 1/(sum_exp + 1e-10f), gguf_model.h:3589
    if (row < rows && !dead) {
        float* dst = O + ((int64_t)row * n_heads + head) * HD + 32 * DT * dh + 4 * kh;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq)
                *reinterpret_cast<float4*>(dst + 32 * dt + 8 * rq) =
                    make_float4(acc[dt][4 * rq] * inv, acc[dt][4 * rq + 1] * inv, acc[dt][4 * rq + 2] * inv, acc[dt][4 * rq + 3] * inv);
    }
}

template <int HD>
static int prefill_attn_mfma_launch(int G, hipStream_t s, const float* Q, const void* Kc, const void* Vc, float* O, int rows,
                                    int n_heads, int n_kv_heads, int64_t pos0, float scale, int window) {
    const int gp = G <= 1 ? 1 : G <= 2 ? 2 : G <= 4 ? 4 : 8;
    const int bm = 128 / gp;
    const dim3 grid((rows + bm - 1) / bm, n_kv_heads);
    // Two groups halve the chain of a row block's tiles and cost a merge and twice the threads to start: with at most 16
    // tiles per row block (the chunk ends within the first 512 positions) one group is faster (192 / 256 / 384 rows from
    // position 0: 9.8 / 11.1 / 13.8 us against 12.5 / 12.6 / 14.9; 512 rows: 17.0 / 17.2), beyond it two are (768 rows: 21.8
    // against 22.7; 256 rows at position 1024: 27.8 against 31.4)
    // (with a window a row block walks at most window + its own rows)
    const int64_t span = window > 0 && window + bm < pos0 + rows ? window + bm : pos0 + rows;
    const bool one = span <= 512;
#define PTM_PA(GG)                                                                                                          \
    if constexpr (HD == 256)                                                                                                \
        hipLaunchKernelGGL((prefill_attn_mfma_kernel<HD, GG, 1, 2>), grid, dim3(512), 0, s, Q, static_cast<const __half*>(Kc), \
                           static_cast<const __half*>(Vc), O, rows, n_heads, n_kv_heads, pos0, scale, window);              \
    else if (one)                                                                                                                \
        hipLaunchKernelGGL((prefill_attn_mfma_kernel<HD, GG, 1>), grid, dim3(256), 0, s, Q, static_cast<const __half*>(Kc), \
                           static_cast<const __half*>(Vc), O, rows, n_heads, n_kv_heads, pos0, scale, window);              \
    else                                                                                                                    \
        hipLaunchKernelGGL((prefill_attn_mfma_kernel<HD, GG, 2>), grid, dim3(512), 0, s, Q, static_cast<const __half*>(Kc), \
                           static_cast<const __half*>(Vc), O, rows, n_heads, n_kv_heads, pos0, scale, window)
    switch (G) {
        case 1: PTM_PA(1); break;
        case 2: PTM_PA(2); break;
        case 3: PTM_PA(3); break;
        case 4: PTM_PA(4); break;
        case 5: PTM_PA(5); break;
        case 6: PTM_PA(6); break;
        case 7: PTM_PA(7); break;
        case 8: PTM_PA(8); break;
        default: return PTM_E_UNSUPPORTED;
    }
#undef PTM_PA
    return launch_status();
}

template <bool KV16, int HD>
static int prefill_attn_launch(int G, dim3 grid, hipStream_t s, const float* Q, const void* Kc, const void* Vc, float* O,
                               int rows, int n_heads, int n_kv_heads, int64_t pos0, float scale, int window) {
#define PTM_PA(GG) hipLaunchKernelGGL((prefill_attn_kernel<KV16, HD, GG>), grid, dim3(256), 0, s, Q, Kc, Vc, O, rows, n_heads, n_kv_heads, pos0, scale, window)
    switch (G) {
        case 1: PTM_PA(1); break;
        case 2: PTM_PA(2); break;
        case 3: PTM_PA(3); break;
        case 4: PTM_PA(4); break;
        case 5: PTM_PA(5); break;
        case 6: PTM_PA(6); break;
        case 7: PTM_PA(7); break;
        case 8: PTM_PA(8); break;
        default: return PTM_E_UNSUPPORTED;
    }
#undef PTM_PA
    return launch_status();
}

// QK-norm + rotation + cache append of M rows whose q, k, v are still K-split partial sums (P[i]: splits[i] slabs of
// M x width_i floats; splits 1 = finished rows), optionally with biases: writes Q (rotated) and the cache rows only.
int qknorm_rope_kv_rows_from_parts(const float* const* P, const int* splits, const float* const* bias, float* Q,
                                   const float* q_norm_w, const float* k_norm_w, void* K_cache, void* V_cache,
                                   const float* rope_table, int rows, int n_heads, int n_kv_heads, int head_dim, int64_t pos0,
                                   int max_seq, float eps, int add_one, int kv_fp16, int rope_interleaved, hipStream_t s) {
    if (!P || !splits || !Q || !K_cache || !V_cache || !rope_table) return PTM_E_NULL;
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) return PTM_E_NULL;
    if (rows <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || head_dim <= 0 || (head_dim & 1) || head_dim > 256)
        return PTM_E_SHAPE;
    if (pos0 < 0 || pos0 + rows > max_seq) return PTM_E_RANGE;  // never write outside the cache
    if (n_heads + n_kv_heads > 65535) return PTM_E_UNSUPPORTED;
    QkvParts parts{};
    for (int i = 0; i < 3; ++i) {
        if (!P[i]) return PTM_E_NULL;
        if (splits[i] < 1) return PTM_E_SHAPE;
        parts.P[i] = P[i];
        parts.splits[i] = splits[i];
        parts.bias[i] = bias ? bias[i] : nullptr;
    }
    return qknorm_rope_kv_rows_launch<true>(Q, Q, Q, q_norm_w, k_norm_w, K_cache, V_cache, rope_table, rows, n_heads, n_kv_heads,
                                            head_dim, pos0, eps, add_one, kv_fp16, rope_interleaved, parts, s);
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_embedding_rows(const float* table_f32, const void* table_q6k, int64_t q6k_row_stride_bytes, const int* d_tokens,
                       int rows, int hidden, int vocab, float* out, ptm_stream_t stream) {
    if ((!table_f32 && !table_q6k) || !d_tokens || !out) return PTM_E_NULL;
    if (rows <= 0 || hidden <= 0 || vocab <= 0 || rows > 65535) return PTM_E_SHAPE;
    if (!table_f32 && ((hidden % 256) != 0 || q6k_row_stride_bytes < (int64_t)(hidden / 256) * 210)) return PTM_E_SHAPE;
    hipLaunchKernelGGL(embedding_rows_kernel, dim3((hidden + 255) / 256, rows), dim3(256), 0, as_stream(stream), table_f32,
                       static_cast<const uint8_t*>(table_q6k), q6k_row_stride_bytes, d_tokens, hidden, vocab, out);
    return launch_status();
}

int ptm_qknorm_rope_kvwrite_rows(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                 void* K_cache, void* V_cache, const float* rope_table, int rows, int n_heads,
                                 int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float eps, int add_one,
                                 int kv_fp16, int rope_interleaved, ptm_stream_t stream) {
    if (!Q || !K || !V || !K_cache || !V_cache || !rope_table) return PTM_E_NULL;
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) return PTM_E_NULL;
    if (rows <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || head_dim <= 0 || (head_dim & 1) || head_dim > 256)
        return PTM_E_SHAPE;
    if (pos0 < 0 || pos0 + rows > max_seq) return PTM_E_RANGE;  // never write outside the cache
    if (n_heads + n_kv_heads > 65535) return PTM_E_UNSUPPORTED;
    return qknorm_rope_kv_rows_launch<false>(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, rope_table, rows, n_heads, n_kv_heads,
                                             head_dim, pos0, eps, add_one, kv_fp16, rope_interleaved, QkvParts{}, as_stream(stream));
}

int ptm_prefill_attention(const float* Q, const void* K_cache, const void* V_cache, float* O, int rows, int n_heads,
                          int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float scale, int kv_fp16,
                          ptm_stream_t stream) {
    return ptm_prefill_attention_window(Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, head_dim, pos0, max_seq, scale,
                                        kv_fp16, 0, stream);
}

int ptm_prefill_attention_window(const float* Q, const void* K_cache, const void* V_cache, float* O, int rows, int n_heads,
                                 int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float scale, int kv_fp16,
                                 int window, ptm_stream_t stream) {
    if (!Q || !K_cache || !V_cache || !O) return PTM_E_NULL;
    if (rows <= 0 || n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || (n_heads % n_kv_heads) != 0) return PTM_E_SHAPE;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return PTM_E_UNSUPPORTED;
    if (pos0 < 0 || pos0 + rows > max_seq) return PTM_E_RANGE;
    if (!aligned16(Q) || !aligned16(K_cache) || !aligned16(V_cache) || !aligned16(O)) return PTM_E_ALIGN;
    if (n_kv_heads > 65535) return PTM_E_UNSUPPORTED;
    const int G = n_heads / n_kv_heads;
    const dim3 grid((rows + 3) / 4, n_kv_heads);
    hipStream_t s = as_stream(stream);
    if (window < 0) window = 0;
    // the MFMA kernel addresses the caches with 32-bit byte offsets (computed for up to two tiles past the last position
    // before they are clamped)
    const bool offsets_fit = (pos0 + rows + 64) * (int64_t)n_kv_heads * head_dim * 2 < ((int64_t)1 << 32);
    if (head_dim == 256) {  // wide heads (gemma3)
        if (kv_fp16 && offsets_fit && rows >= PTM_PREFILL_MFMA_MIN_ROWS && G <= 8)
            return prefill_attn_mfma_launch<256>(G, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window);
        return kv_fp16 ? prefill_attn_launch<true, 256>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window)
                       : prefill_attn_launch<false, 256>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window);
    }
    if (kv_fp16 && offsets_fit && rows >= PTM_PREFILL_MFMA_MIN_ROWS && G <= 8)
        return head_dim == 128 ? prefill_attn_mfma_launch<128>(G, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window)
                               : prefill_attn_mfma_launch<64>(G, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window);
    if (kv_fp16)
        return head_dim == 128 ? prefill_attn_launch<true, 128>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window)
                               : prefill_attn_launch<true, 64>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window);
    return head_dim == 128 ? prefill_attn_launch<false, 128>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window)
                           : prefill_attn_launch<false, 64>(G, grid, s, Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, pos0, scale, window);
}

}  // extern "C"
