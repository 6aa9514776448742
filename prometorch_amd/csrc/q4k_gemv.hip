// Q4_K dequant-fused GEMV for gfx950 (wave64).
//
// Arithmetic follows the reference CPU kernel (torch/io/cpu_quant_gemv.h:505-685): the
// activation vector is quantised to Q8 blocks of 32 (cpu_quant_gemv.h:147-198), each 32-wide
// sub-block contributes  fma(d*sc*dx, (float)isum, -(dmin*m*sx))  with isum the exact int32
// dot of 4-bit weights and int8 activations; only the order in which the per-sub-block terms
// are added differs (per-lane chains + a cross-lane tree instead of two scalar chains).
//
// Data movement: a super-block (144 B) is fetched by an aligned group of 8 lanes: lane j takes
// the 16-byte header {d, dmin, scales[12]} and the j-th 16-byte slice of qs[128] with 128-bit
// loads, so every fetched byte is used.  A slice holds 16 low nibbles (sub-block 2*(j/2)) and
// 16 high nibbles (sub-block 2*(j/2)+1); lane pairs swap halves through one DPP move so that
// lane j ends up owning the complete integer dot of sub-block j.
// A row is shared by S lane groups (S = 1, 2, 4 or 8 - a whole wave), group s taking blocks
// s, s+S, ...; S is chosen on the host so that a launch has several hundred workgroups even for
// short-and-wide matrices (o-proj: 2560 rows) and so that each group's blocks are all in flight
// at once.  The first pass of weight loads is issued BEFORE the activation vector is staged
// (RMSNorm, Q8 quantisation, LDS), so HBM latency overlaps the prologue.
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
    const void* x;       // fp32 x[K] (XQ8 == false) or Q8 blocks (XQ8 == true)
    const float* gamma;  // RMSNorm weight (NORM)
    float eps;
    int add_one;
};

enum { Q4K_THREADS = 256, Q4K_U = 10 };

// ---- prologue: bring the Q8 activation into LDS -------------------------------------------
template <bool XQ8, bool NORM>
__device__ __forceinline__ void q4k_stage_x(const Q4KArgs& a, uint8_t* lds) {
    const int K = a.K;
    const int tid = threadIdx.x;
    if constexpr (XQ8) {
        const uint4* src = reinterpret_cast<const uint4*>(a.x);
        uint4* dst = reinterpret_cast<uint4*>(lds);
        const int n16 = (K + K / 4) / 16;
        for (int i = tid; i < n16; i += Q4K_THREADS) dst[i] = src[i];
    } else {
        __shared__ float red[4];
        int8_t* qs = reinterpret_cast<int8_t*>(lds);
        float* xd = reinterpret_cast<float*>(lds + K);
        float* xs = xd + K / 32;
        // 8 consecutive float4 slots (8 lanes) = one Q8 block
        stage_x_slots<NORM>(static_cast<const float*>(a.x), a.gamma, K, a.eps, a.add_one, red, [&](int i, float4 v) {
            float d, sm;
            const uint32_t packed = q8_quantize4(v, d, sm);
            reinterpret_cast<uint32_t*>(qs)[i] = packed;
            if ((tid & 7) == 0) {
                xd[i >> 3] = d;
                xs[i >> 3] = sm;
            }
        });
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
template <bool XQ8, bool NORM, bool ACC, int MODE>
__global__ __launch_bounds__(Q4K_THREADS) void q4k_gemv_kernel(const Q4KArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 7, grp = lane >> 3;
    const int S = 1 << a.log2S;
    const int sub = grp & (S - 1);
    const int rows_per_wave = 8 >> a.log2S;
    const int r = (blockIdx.x * 4 + wave) * rows_per_wave + (grp >> a.log2S);
    const bool live = r < a.total_rows;
    const int rr = live ? r : a.total_rows - 1;
    const int nblk = a.K / 256;
    const int nb_max = (nblk + S - 1) >> a.log2S;  // passes are sized for the group with the most blocks

    int mat = 0, local = rr;
    if constexpr (MODE == 1) {
        mat = rr & 1;
        local = rr >> 1;
    } else {
        if (a.n_mat > 1 && rr >= a.row_end[0]) { mat = 1; local = rr - a.row_end[0]; }
        if (a.n_mat > 2 && rr >= a.row_end[1]) { mat = 2; local = rr - a.row_end[1]; }
    }
    const uint8_t* row = (mat == 0 ? a.W[0] : (mat == 1 ? a.W[1] : a.W[2])) + (int64_t)local * a.stride;

    // ---- first pass of weight loads, issued before the activation prologue ----
    uint4 hdr[Q4K_U], qv[Q4K_U];
    const int cnt0 = min(Q4K_U, nb_max);
#pragma unroll
    for (int u = 0; u < Q4K_U; ++u) {
        if (u < cnt0) {
            const int b = min(sub + (u << a.log2S), nblk - 1);
            const uint8_t* p = row + (int64_t)b * 144;
            hdr[u] = *reinterpret_cast<const uint4*>(p);
            qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
        }
    }

    q4k_stage_x<XQ8, NORM>(a, lds);

    float acc = 0.0f;
    for (int i0 = 0; i0 < nb_max; i0 += Q4K_U) {
        const int cnt = min(Q4K_U, nb_max - i0);
        if (i0 > 0) {
#pragma unroll
            for (int u = 0; u < Q4K_U; ++u) {
                if (u < cnt) {
                    const int b = min(sub + ((i0 + u) << a.log2S), nblk - 1);
                    const uint8_t* p = row + (int64_t)b * 144;
                    hdr[u] = *reinterpret_cast<const uint4*>(p);
                    qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < Q4K_U; ++u) {
            if (u < cnt) {
                const int b = sub + ((i0 + u) << a.log2S);
                const float t = q4k_block_term(hdr[u], qv[u], lds, a.K, min(b, nblk - 1), j);
                acc += b < nblk ? t : 0.0f;
            }
        }
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
        if (live && mat == 0 && sub == 0 && j == 0) a.y[0][local] = silu_mul_ref(p, other);
    } else {
        float* y = mat == 0 ? a.y[0] : (mat == 1 ? a.y[1] : a.y[2]);
        if (live && sub == 0 && j == 0) {
            if constexpr (ACC) y[local] += p;
            else y[local] = p;
        }
    }
}

// lane groups per row: enough workgroups to cover the chip, and all of a group's blocks in one pass
static int q4k_pick_log2S(int total_rows, int nblk, int max_log2S) {
    int l = 0;
    while (l < max_log2S) {
        const int S = 1 << l;
        const int wgs = (total_rows * S + 31) / 32;
        const int nb = (nblk + S - 1) / S;
        if (nb <= Q4K_U && wgs >= 600) break;
        if (nb <= 1) break;
        ++l;
    }
    return l;
}

template <bool XQ8, bool NORM, bool ACC, int MODE>
static int q4k_launch(Q4KArgs& a, hipStream_t s) {
    a.log2S = q4k_pick_log2S(a.total_rows, a.K / 256, MODE == 1 ? 2 : 3);
    const int rows_per_wg = 32 >> a.log2S;
    const int grid = (a.total_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t lds = (size_t)q8_bytes(a.K);
    hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE>), dim3(grid), dim3(Q4K_THREADS), lds, s, a);
    return launch_status();
}

static int q4k_check(const void* W, const void* x, const void* y, int K, int N, int64_t stride) {
    if (!W || !x || !y) return PTM_E_NULL;
    if (K <= 0 || N <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (K > 32768) return PTM_E_UNSUPPORTED;  // Q8 activations must fit the 40 KB LDS budget used here
    if (stride < (int64_t)(K / 256) * 144) return PTM_E_SHAPE;
    if ((stride & 15) != 0 || !aligned16(W) || !aligned16(x) || (reinterpret_cast<uintptr_t>(y) & 3u)) return PTM_E_ALIGN;
    return PTM_OK;
}

// Shared by the C entry points and the decode runtime.
int q4k_gemv_multi(int n_mat, const void* const* W, float* const* y, const int* N, const void* x, bool x_is_q8,
                   const float* gamma, float eps, int add_one, int K, int64_t stride, bool accumulate,
                   hipStream_t s) {
    Q4KArgs a{};
    int total = 0;
    for (int i = 0; i < n_mat; ++i) {
        const int rc = q4k_check(W[i], x, y[i], K, N[i], stride);
        if (rc != PTM_OK) return rc;
        a.W[i] = static_cast<const uint8_t*>(W[i]);
        a.y[i] = y[i];
        total += N[i];
        a.row_end[i] = total;
    }
    a.n_mat = n_mat;
    a.total_rows = total;
    a.K = K;
    a.stride = stride;
    a.x = x;
    a.gamma = gamma;
    a.eps = eps;
    a.add_one = add_one;
    if (gamma) {
        if (x_is_q8) return PTM_E_UNSUPPORTED;
        if (!aligned16(gamma)) return PTM_E_ALIGN;
        return accumulate ? q4k_launch<false, true, true, 0>(a, s) : q4k_launch<false, true, false, 0>(a, s);
    }
    if (x_is_q8) return accumulate ? q4k_launch<true, false, true, 0>(a, s) : q4k_launch<true, false, false, 0>(a, s);
    return accumulate ? q4k_launch<false, false, true, 0>(a, s) : q4k_launch<false, false, false, 0>(a, s);
}

int q4k_gate_up_silu(const void* wg, const void* wu, const void* x, bool x_is_q8, const float* gamma, float eps,
                     int add_one, float* act, int K, int N, int64_t stride, hipStream_t s) {
    int rc = q4k_check(wg, x, act, K, N, stride);
    if (rc != PTM_OK) return rc;
    rc = q4k_check(wu, x, act, K, N, stride);
    if (rc != PTM_OK) return rc;
    if (N > 0x3fffffff) return PTM_E_UNSUPPORTED;
    Q4KArgs a{};
    a.W[0] = static_cast<const uint8_t*>(wg);
    a.W[1] = static_cast<const uint8_t*>(wu);
    a.y[0] = act;
    a.n_mat = 2;
    a.row_end[0] = N;
    a.total_rows = 2 * N;
    a.K = K;
    a.stride = stride;
    a.x = x;
    a.gamma = gamma;
    a.eps = eps;
    a.add_one = add_one;
    if (gamma) {
        if (x_is_q8) return PTM_E_UNSUPPORTED;
        if (!aligned16(gamma)) return PTM_E_ALIGN;
        return q4k_launch<false, true, false, 1>(a, s);
    }
    return x_is_q8 ? q4k_launch<true, false, false, 1>(a, s) : q4k_launch<false, false, false, 1>(a, s);
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_q4k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t stride, int accumulate,
                 ptm_stream_t stream) {
    return q4k_gemv_multi(1, &W, &y, &N, x, false, nullptr, 0.f, 0, K, stride, accumulate != 0, as_stream(stream));
}

int ptm_q4k_gemv_q8(const void* W, const void* x_q8, float* y, int K, int N, int64_t stride, int accumulate,
                    ptm_stream_t stream) {
    return q4k_gemv_multi(1, &W, &y, &N, x_q8, true, nullptr, 0.f, 0, K, stride, accumulate != 0, as_stream(stream));
}

int ptm_q4k_fused_gate_up_gemv(const void* w_gate, const void* w_up, const float* x, float* y_gate, float* y_up,
                               int K, int N_gate, int N_up, int64_t stride, ptm_stream_t stream) {
    const void* W[2] = {w_gate, w_up};
    float* y[2] = {y_gate, y_up};
    const int N[2] = {N_gate, N_up};
    return q4k_gemv_multi(2, W, y, N, x, false, nullptr, 0.f, 0, K, stride, false, as_stream(stream));
}

int ptm_q4k_fused_qkv_gemv(const void* w_q, const void* w_k, const void* w_v, const float* x, float* out_q,
                           float* out_k, float* out_v, int K, int N_q, int N_k, int N_v, int64_t stride,
                           ptm_stream_t stream) {
    const void* W[3] = {w_q, w_k, w_v};
    float* y[3] = {out_q, out_k, out_v};
    const int N[3] = {N_q, N_k, N_v};
    return q4k_gemv_multi(3, W, y, N, x, false, nullptr, 0.f, 0, K, stride, false, as_stream(stream));
}

int ptm_q4k_fused_rmsnorm_gemv(const float* x, const float* norm_w, const void* W, float* y, int K, int N,
                               int64_t stride, float eps, int add_one, ptm_stream_t stream) {
    if (!norm_w) return PTM_E_NULL;
    return q4k_gemv_multi(1, &W, &y, &N, x, false, norm_w, eps, add_one, K, stride, false, as_stream(stream));
}

int ptm_q4k_fused_rmsnorm_qkv_gemv(const float* x, const float* norm_w, const void* w_q, const void* w_k,
                                   const void* w_v, float* out_q, float* out_k, float* out_v, int K, int N_q,
                                   int N_k, int N_v, int64_t stride, float eps, int add_one,
                                   ptm_stream_t stream) {
    if (!norm_w) return PTM_E_NULL;
    const void* W[3] = {w_q, w_k, w_v};
    float* y[3] = {out_q, out_k, out_v};
    const int N[3] = {N_q, N_k, N_v};
    return q4k_gemv_multi(3, W, y, N, x, false, norm_w, eps, add_one, K, stride, false, as_stream(stream));
}

int ptm_q4k_fused_rmsnorm_gate_up_gemv(const float* x, const float* norm_w, const void* w_gate,
                                       const void* w_up, float* y_gate, float* y_up, int K, int N_gate,
                                       int N_up, int64_t stride, float eps, int add_one, ptm_stream_t stream) {
    if (!norm_w) return PTM_E_NULL;
    const void* W[2] = {w_gate, w_up};
    float* y[2] = {y_gate, y_up};
    const int N[2] = {N_gate, N_up};
    return q4k_gemv_multi(2, W, y, N, x, false, norm_w, eps, add_one, K, stride, false, as_stream(stream));
}

int ptm_q4k_fused_rmsnorm_gate_up_silu(const float* x, const float* norm_w, const void* w_gate,
                                       const void* w_up, float* act, int K, int N, int64_t stride, float eps,
                                       int add_one, ptm_stream_t stream) {
    if (!norm_w) return PTM_E_NULL;
    return q4k_gate_up_silu(w_gate, w_up, x, false, norm_w, eps, add_one, act, K, N, stride, as_stream(stream));
}

}  // extern "C"
