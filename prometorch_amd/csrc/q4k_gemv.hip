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
// at once (five per group measured best: fewer registers, more waves per SIMD).  The first pass of
// weight loads is issued BEFORE the activation vector is staged (RMSNorm, Q8 quantisation, LDS), so HBM
// latency overlaps the prologue; every pass issues a fixed number of loads (template NB) and activations
// come through range-checked buffer loads, so no load sits under a branch and the compiler can wait for
// exactly the block it is about to use.  Very tall matrices let a workgroup walk several row tiles with
// one staging of x; where a tile is a single pass, the block loads roll across the tiles (q4k_gemv_tall_kernel: a consumed
// block's registers are refilled from the next tile's row, 151936 x 2560: 44.5 -> 41.6 us).
#include "q4k_body.h"

namespace ptm {

template <bool XQ8, bool NORM, bool ACC, int MODE, int NB>
__global__ __launch_bounds__(Q4K_THREADS) void q4k_gemv_kernel(const Q4KArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    q4k_gemv_body<XQ8, NORM, ACC, MODE, NB>(a, lds, blockIdx.x);
}

// a workgroup walks several row tiles, every tile one pass of NB blocks per lane group: the passes roll across the tiles
template <bool XQ8, bool NORM, bool ACC, int MODE, int NB>
__global__ __launch_bounds__(Q4K_THREADS) void q4k_gemv_tall_kernel(const Q4KArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    q4k_gemv_body<XQ8, NORM, ACC, MODE, NB, true>(a, lds, blockIdx.x);
}

// Few rows, long rows (a Q4_K down projection: 2560 x 9728, as in the layers of a Q4_K_M file whose ffn_down is Q4_K): with
// four rows per workgroup, 640 workgroups would each quantise the whole 9728-value activation vector for four rows' worth
// of weights.  Here a workgroup is `waves` waves of one row each (the row's super-blocks strided over the wave's 8 lane
// groups, two or three blocks of a group in flight, passes rolling), sized so that the launch is one workgroup per CU (two
// for 17 to 32 rows per CU): x is quantised once per workgroup, one to three half blocks of 16 values per thread.
// Block-to-lane assignment and reduction order are those of q4k_gemv_body with 8 lane groups per row, so the result is
// bit-identical to that kernel's.  Against that kernel: 3584 x 18944 15.2 -> 11.3 us, 4096 x 14336 12.0 -> 9.8,
// 5120 x 17408 15.9 -> 14.2, 8192 x 28672 31.1 -> 28.1.
enum { Q4K_LONGROW_MAX_WAVES = 16 };
// XL: half blocks of x a thread quantises (rows longer than 16 values per thread: up to three rounds); MAXW: the most waves
// an instantiation is launched with
template <bool ACC, int NB, int XL = 1, int MAXW = 12>
__global__ __launch_bounds__(64 * MAXW) void q4k_gemv_longrow_kernel(const uint8_t* __restrict__ W, int64_t stride,
                                                                  const float* __restrict__ x, float* y, int N, int K) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, nthr = blockDim.x, lane = tid & 63, wave = tid >> 6, j = lane & 7, sub = lane >> 3;
    const int nblk = K / 256;
    const int r = blockIdx.x * (nthr >> 6) + wave;
    const bool live = r < N;
    const uint8_t* row = W + (int64_t)(live ? r : N - 1) * stride;
    // activation loads first (range-checked: zeros past the end), then the weights, then the Q8 arithmetic
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, K * 4);
    float4 xv[XL][4];
#pragma unroll
    for (int u = 0; u < XL; ++u) q4k_load16(rx, 16 * (tid + nthr * u), xv[u]);
    issue_order_fence();
    uint4 hdr[NB], qv[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const uint8_t* p = row + (int64_t)min(sub + 8 * u, nblk - 1) * 144;
        hdr[u] = *reinterpret_cast<const uint4*>(p);
        qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
    }
    issue_order_fence();
#pragma unroll
    for (int u = 0; u < XL; ++u) {  // lanes t, t ^ 1 share a block: both inside or both outside (nthr is a multiple of 64)
        const int unit = tid + nthr * u;
        if (16 * unit < K) q4k_quantize16_store<false>(xv[u], xv[u], 1.0f, 0.0f, unit, lds, K);
    }
    __syncthreads();
    // passes roll as in q4k_gemv_body: a consumed block's registers are refilled from the next pass at once
    const int nb_max = (nblk + 7) >> 3;
    float acc = 0.0f;
    int i0 = 0;
    for (; i0 + NB < nb_max; i0 += NB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int b = sub + 8 * (i0 + u);
            const float t = q4k_block_term(hdr[u], qv[u], lds, K, min(b, nblk - 1), j);
            acc += b < nblk ? t : 0.0f;
            const uint8_t* p = row + (int64_t)min(sub + 8 * (i0 + NB + u), nblk - 1) * 144;
            hdr[u] = *reinterpret_cast<const uint4*>(p);
            qv[u] = *reinterpret_cast<const uint4*>(p + 16 + 16 * j);
        }
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const int b = sub + 8 * (i0 + u);
        const float t = q4k_block_term(hdr[u], qv[u], lds, K, min(b, nblk - 1), j);
        acc += b < nblk ? t : 0.0f;
    }
    float p = sum8(acc);
    p += dpp_f<0x128>(p);
    p += __shfl_xor(p, 16, 64);
    p += __shfl_xor(p, 32, 64);
    if (live && lane == 0) {
        if constexpr (ACC) y[r] += p;
        else y[r] = p;
    }
}

// waves per workgroup and half blocks of x per thread of that launch, or waves = 0 when the shape is not one for it.  Up to
// 16 rows per CU make one workgroup per CU, up to 32 two (each quantises x for itself).
struct Q4KLongrow { int waves, xl; };
static Q4KLongrow q4k_longrow_shape(int N, int K) {
    if (K < 4096) return {0, 0};                                  // long rows
    const int rows_per_cu = (N + 255) / 256;
    const int per_cu = (rows_per_cu + Q4K_LONGROW_MAX_WAVES - 1) / Q4K_LONGROW_MAX_WAVES;
    if (per_cu > 2) return {0, 0};
    const int waves = (rows_per_cu + per_cu - 1) / per_cu;
    if (waves < 2) return {0, 0};
    const int xl = (K / 16 + 64 * waves - 1) / (64 * waves);
    if (xl > 3) return {0, 0};
    return {waves, xl};
}

template <bool ACC, int NB>
static int q4k_launch_longrow_nb(const void* W, int64_t stride, const float* x, float* y, int N, int K, Q4KLongrow sh, hipStream_t s) {
    const dim3 grid((N + sh.waves - 1) / sh.waves), block(64 * sh.waves);
    const size_t lds = (size_t)q8_bytes(K);
    const uint8_t* Wb = static_cast<const uint8_t*>(W);
#define PTM_LR(XL, MAXW) hipLaunchKernelGGL((q4k_gemv_longrow_kernel<ACC, NB, XL, MAXW>), grid, block, lds, s, Wb, stride, x, y, N, K)
    if (sh.waves <= 12) {
        if (sh.xl == 1) PTM_LR(1, 12);
        else if (sh.xl == 2) PTM_LR(2, 12);
        else PTM_LR(3, 12);
    } else {
        if (sh.xl == 1) PTM_LR(1, 16);
        else if (sh.xl == 2) PTM_LR(2, 16);
        else PTM_LR(3, 16);
    }
#undef PTM_LR
    return launch_status();
}

template <bool ACC>
static int q4k_launch_longrow(const void* W, int64_t stride, const float* x, float* y, int N, int K, Q4KLongrow sh, hipStream_t s) {
    // blocks in flight per lane group: two; three for workgroups of up to ten waves (2560 x 9728, 10 waves, five blocks per
    // group: 1 / 2 / 3 / 5 in flight 7.5 / 7.0 / 6.9 / 7.0 us; 2048 x 11008, 8 waves: 2 / 3 in flight 6.6 / 6.2;
    // 3072 x 8192, 12 waves: 5.9 / 6.5; 3584 x 18944, 14 waves: 1 / 2 / 3 in flight 12.8 / 11.3 / 12.2)
    const int nb = (K / 256 + 7) / 8;
    if (nb > 2 && sh.waves <= 10) return q4k_launch_longrow_nb<ACC, 3>(W, stride, x, y, N, K, sh, s);
    return q4k_launch_longrow_nb<ACC, 2>(W, stride, x, y, N, K, sh, s);
}

template <bool XQ8, bool NORM, bool ACC, int MODE>
static int q4k_launch(Q4KArgs& a, hipStream_t s) {
    a.log2S = q4k_pick_log2S(a.total_rows, a.K / 256, MODE == 1 ? 2 : 3);
    const int n_tiles = q4k_workgroups(a.total_rows, a.log2S);
    a.tiles_per_wg = q4k_tiles_per_wg(n_tiles);
    const dim3 block(Q4K_THREADS);
    const size_t lds = (size_t)q8_bytes(a.K);
    const int nb = q4k_blocks_per_pass(a.K / 256, a.log2S);
    {
        // a very tall matrix (or gate / up pair) whose lane groups hold a row's blocks in a single pass: the loads roll
        // across the tiles
        const int nb_max = (a.K / 256 + (1 << a.log2S) - 1) >> a.log2S;
                // (only beyond 1280 tiles: the Qwen3-4B gate / up pair, 1216 tiles, as 608 workgroups of two rolling tiles measured
        // 9.88 us against 9.45 with one tile per workgroup)
        if ((MODE == 1 || a.n_mat == 1) && a.tiles_per_wg > 1 && nb_max <= nb && nb <= 5) {
            a.tiles_per_wg = q4k_tiles_per_wg_rolling(n_tiles);
            const dim3 grid((n_tiles + a.tiles_per_wg - 1) / a.tiles_per_wg);
            switch (nb) {
                case 2: hipLaunchKernelGGL((q4k_gemv_tall_kernel<XQ8, NORM, ACC, MODE, 2>), grid, block, lds, s, a); break;
                case 3: hipLaunchKernelGGL((q4k_gemv_tall_kernel<XQ8, NORM, ACC, MODE, 3>), grid, block, lds, s, a); break;
                case 4: hipLaunchKernelGGL((q4k_gemv_tall_kernel<XQ8, NORM, ACC, MODE, 4>), grid, block, lds, s, a); break;
                default: hipLaunchKernelGGL((q4k_gemv_tall_kernel<XQ8, NORM, ACC, MODE, 5>), grid, block, lds, s, a); break;
            }
            return launch_status();
        }
    }
    const dim3 grid((n_tiles + a.tiles_per_wg - 1) / a.tiles_per_wg);
    switch (nb) {
        case 2: hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE, 2>), grid, block, lds, s, a); break;
        case 3: hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE, 3>), grid, block, lds, s, a); break;
        case 4: hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE, 4>), grid, block, lds, s, a); break;
        case 5: hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE, 5>), grid, block, lds, s, a); break;
        default: hipLaunchKernelGGL((q4k_gemv_kernel<XQ8, NORM, ACC, MODE, 10>), grid, block, lds, s, a); break;
    }
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
    if (n_mat == 1) {
        const Q4KLongrow sh = q4k_longrow_shape(N[0], K);
        if (sh.waves > 0)
            return accumulate ? q4k_launch_longrow<true>(W[0], stride, static_cast<const float*>(x), y[0], N[0], K, sh, s)
                              : q4k_launch_longrow<false>(W[0], stride, static_cast<const float*>(x), y[0], N[0], K, sh, s);
    }
    return accumulate ? q4k_launch<false, false, true, 0>(a, s) : q4k_launch<false, false, false, 0>(a, s);
}

int q4k_gate_up_silu(const void* wg, const void* wu, const void* x, bool x_is_q8, const float* gamma, float eps,
                     int add_one, float* act, int K, int N, int64_t stride, hipStream_t s, bool gelu) {
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
    a.gelu = gelu ? 1 : 0;
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
    return q4k_gate_up_silu(w_gate, w_up, x, false, norm_w, eps, add_one, act, K, N, stride, as_stream(stream), false);
}

}  // extern "C"
