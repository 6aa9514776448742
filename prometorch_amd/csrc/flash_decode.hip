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

// grid (max_splits, n_kv_heads); G = query heads per kv head; HD = head_dim
template <bool KV16, int HD, int G>
__global__ __launch_bounds__(FD_THREADS) void flash_decode_partial_kernel(
    const float* __restrict__ Q, const void* __restrict__ Kc, const void* __restrict__ Vc,
    float* __restrict__ pO, float* __restrict__ pL, float* __restrict__ pM, int n_heads, int n_kv_heads,
    const int64_t* __restrict__ d_past, int max_seq, float scale) {
    constexpr int LPP = HD / 8;         // lanes per position (each lane owns 8 dims)
    constexpr int PPW = 64 / LPP;       // positions per wave per pass
    constexpr int PPB = PPW * 4;        // positions per workgroup per pass
    constexpr int NPASS = FD_CHUNK / PPB;
    __shared__ float s_p[G][FD_CHUNK];
    __shared__ float s_o[4][G][HD];

    int64_t total = *d_past + 1;
    if (total > max_seq) total = max_seq;
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int64_t t0 = (int64_t)split * FD_CHUNK;
    if (t0 >= total) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dl = lane % LPP, pl = lane / LPP;
    const int kv_dim = n_kv_heads * HD;
    const int64_t col = (int64_t)kvh * HD + dl * 8;

    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const float4 a = *reinterpret_cast<const float4*>(Q + (int64_t)(kvh * G + g) * HD + dl * 8);
        const float4 b = *reinterpret_cast<const float4*>(Q + (int64_t)(kvh * G + g) * HD + dl * 8 + 4);
        q[g][0] = a.x; q[g][1] = a.y; q[g][2] = a.z; q[g][3] = a.w;
        q[g][4] = b.x; q[g][5] = b.y; q[g][6] = b.z; q[g][7] = b.w;
    }

    // ---- all K and V rows of the chunk are requested up front: one HBM round trip ----
    float kreg[NPASS][8], vreg[NPASS][8];
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int64_t t = t0 + pass * PPB + wave * PPW + pl;
        const int64_t tc = t < total ? t : total - 1;
        load8<KV16>(Kc, tc * kv_dim + col, kreg[pass]);
        load8<KV16>(Vc, tc * kv_dim + col, vreg[pass]);
    }

    // ---- scores ----
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        const int tl = pass * PPB + wave * PPW + pl;
        const bool valid = t0 + tl < total;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) d = fmaf(q[g][i], kreg[pass][i], d);
            d = (LPP == 16) ? sum16(d) : sum8(d);
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

// grid n_heads, 256 threads: merge the active splits.  Thread (slot = tid / head_dim-quarter...) layout:
// the 256 threads form R = 256/head_dim split-slots x head_dim dims; slot r sums splits r, r+R, ...
// (independent loads, all in flight), then the R slot sums are added in slot order.
__global__ __launch_bounds__(256) void flash_decode_reduce_kernel(const float* __restrict__ pO,
                                                                  const float* __restrict__ pL,
                                                                  const float* __restrict__ pM, float* __restrict__ O,
                                                                  int n_heads, int head_dim,
                                                                  const int64_t* __restrict__ d_past, int max_seq) {
    __shared__ float s_w[256];     // per-split weight exp(m_s - M)
    __shared__ float s_num[256];
    __shared__ float s_red[8];
    int64_t total = *d_past + 1;
    if (total > max_seq) total = max_seq;
    const int ns = (int)((total + FD_CHUNK - 1) / FD_CHUNK);
    const int h = blockIdx.x, tid = threadIdx.x;
    // global max and denominator over splits (ns may exceed 256: strided)
    float m = -INFINITY;
    for (int s = tid; s < ns; s += 256) m = fmaxf(m, pM[(int64_t)s * n_heads + h]);
    m = max64(m);
    if ((tid & 63) == 0) s_red[tid >> 6] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    float den = 0.0f;
    for (int s = tid; s < ns; s += 256) den = fmaf(expf(pM[(int64_t)s * n_heads + h] - M), pL[(int64_t)s * n_heads + h], den);
    den = sum64(den);
    if ((tid & 63) == 0) s_red[4 + (tid >> 6)] = den;
    const int R = 256 / head_dim, slot = tid / head_dim, d = tid % head_dim;
    float num = 0.0f;
    for (int s0 = 0; s0 < ns; s0 += 256) {
        __syncthreads();
        if (s0 + tid < ns) s_w[tid] = expf(pM[(int64_t)(s0 + tid) * n_heads + h] - M);
        __syncthreads();
        const int lim = min(256, ns - s0);
        for (int s = slot; s < lim; s += R)
            num = fmaf(s_w[s], pO[((int64_t)(s0 + s) * n_heads + h) * head_dim + d], num);
    }
    s_num[tid] = num;
    __syncthreads();
    if (tid < head_dim) {
        float t = s_num[tid];
        for (int r = 1; r < R; ++r) t += s_num[r * head_dim + tid];
        const float dsum = (s_red[4] + s_red[5]) + (s_red[6] + s_red[7]);
        // reference: inv_sum = 1/(sum_exp + 1e-10f), gguf_model.h:3589
        O[(int64_t)h * head_dim + tid] = t * (1.0f / (dsum + 1e-10f));
    }
}

template <bool KV16, int HD>
static int fd_launch_g(int G, dim3 grid, hipStream_t s, const float* Q, const void* Kc, const void* Vc, float* pO,
                       float* pL, float* pM, int n_heads, int n_kv_heads, const int64_t* d_past, int max_seq,
                       float scale) {
#define PTM_FD(GG)                                                                                              \
    hipLaunchKernelGGL((flash_decode_partial_kernel<KV16, HD, GG>), grid, dim3(FD_THREADS), 0, s, Q, Kc, Vc, pO, \
                       pL, pM, n_heads, n_kv_heads, d_past, max_seq, scale)
    switch (G) {
        case 1: PTM_FD(1); break;
        case 2: PTM_FD(2); break;
        case 4: PTM_FD(4); break;
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
    if (!Q || !K_cache || !V_cache || !O || !partial_O || !partial_lse || !partial_max || !d_past_len)
        return PTM_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || (n_heads % n_kv_heads) != 0) return PTM_E_SHAPE;
    if (head_dim != 64 && head_dim != 128) return PTM_E_UNSUPPORTED;
    if (!aligned16(Q) || !aligned16(K_cache) || !aligned16(V_cache)) return PTM_E_ALIGN;
    const int G = n_heads / n_kv_heads;
    const dim3 grid(ptm_flash_decode_num_splits(max_seq), n_kv_heads);
    hipStream_t s = as_stream(stream);
    int rc;
    if (kv_fp16) {
        rc = head_dim == 128 ? fd_launch_g<true, 128>(G, grid, s, Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale)
                             : fd_launch_g<true, 64>(G, grid, s, Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale);
    } else {
        rc = head_dim == 128 ? fd_launch_g<false, 128>(G, grid, s, Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale)
                             : fd_launch_g<false, 64>(G, grid, s, Q, K_cache, V_cache, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, d_past_len, max_seq, scale);
    }
    if (rc != PTM_OK) return rc;
    hipLaunchKernelGGL(flash_decode_reduce_kernel, dim3(n_heads), dim3(256), 0, s, partial_O, partial_lse,
                       partial_max, O, n_heads, head_dim, d_past_len, max_seq);
    return launch_status();
}

}  // extern "C"
