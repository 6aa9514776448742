// One launch for projections of the same activation vector that come in different quant types:
// in a Q4_K_M file attn_q / attn_k are Q4_K while attn_v is Q6_K, so the reference issues three
// GEMVs after one RMSNorm (torch/io/gguf_model.h:2750-2764).  Here workgroups [0, n6) run the
// Q6_K body on the Q6_K matrix and the rest run the Q4_K body on up to three Q4_K matrices; each
// workgroup recomputes the RMSNorm of x in its prologue, so no separate norm launch is needed.
#include "q4k_body.h"
#include "q6k_body.h"

namespace ptm {

// PRE: a deferred post-norm and residual add in front of the RMSNorm (x + RMSNorm(pre_h) * pre_w, formed by every workgroup;
// workgroup 0, a Q6_K one, stores it)
template <int NB4, int NB6, bool PRE = false>
__global__ __launch_bounds__(256) void rmsnorm_mixed_gemv_kernel(const Q4KArgs a4, const Q6KArgs a6, int n6_wgs) {
    extern __shared__ __align__(16) uint8_t lds[];
    if ((int)blockIdx.x < n6_wgs) q6k_gemv_body<false, false, true, 1, NB6, PRE>(a6, lds, blockIdx.x);
    else q4k_gemv_body<false, true, false, 0, NB4, false, PRE>(a4, lds, (int)blockIdx.x - n6_wgs);
}

template <int NB4, bool PRE>
static void mixed_launch6(int nb6, dim3 grid, size_t lds, hipStream_t s, const Q4KArgs& a4, const Q6KArgs& a6, int n6) {
    switch (nb6) {
        case 2: hipLaunchKernelGGL((rmsnorm_mixed_gemv_kernel<NB4, 2, PRE>), grid, dim3(256), lds, s, a4, a6, n6); break;
        case 3: hipLaunchKernelGGL((rmsnorm_mixed_gemv_kernel<NB4, 3, PRE>), grid, dim3(256), lds, s, a4, a6, n6); break;
        default: hipLaunchKernelGGL((rmsnorm_mixed_gemv_kernel<NB4, 5, PRE>), grid, dim3(256), lds, s, a4, a6, n6); break;
    }
}

template <bool PRE>
static void mixed_launch4(int nb4, int nb6, dim3 grid, size_t lds, hipStream_t s, const Q4KArgs& a4, const Q6KArgs& a6, int n6) {
    switch (nb4) {
        case 2: mixed_launch6<2, PRE>(nb6, grid, lds, s, a4, a6, n6); break;
        case 3: mixed_launch6<3, PRE>(nb6, grid, lds, s, a4, a6, n6); break;
        case 4: mixed_launch6<4, PRE>(nb6, grid, lds, s, a4, a6, n6); break;
        case 5: mixed_launch6<5, PRE>(nb6, grid, lds, s, a4, a6, n6); break;
        default: mixed_launch6<10, PRE>(nb6, grid, lds, s, a4, a6, n6); break;
    }
}

// y4[i] = W4[i] . norm(x) for the n4 Q4_K matrices (same K and stride), y6 = W6 . norm(x) (Q6_K, same K).
// pre_h / pre_w / pre_out (all or none; K <= 4096): x stands for x + RMSNorm(pre_h) * pre_w, which is also stored to pre_out.
int rmsnorm_mixed_gemv(int n4, const void* const* W4, float* const* y4, const int* N4, int64_t stride4,
                       const void* W6, float* y6, int N6, int64_t stride6, const float* x, const float* gamma,
                       float eps, int add_one, int K, hipStream_t s, const float* pre_h, const float* pre_w, float* pre_out) {
    if (!x || !gamma || !W6 || !y6) return PTM_E_NULL;
    const bool pre = pre_h != nullptr;
    if (pre != (pre_w != nullptr) || pre != (pre_out != nullptr)) return PTM_E_NULL;
    if (pre && (K > 4096 || pre_out == x)) return PTM_E_UNSUPPORTED;
    if (pre && (!aligned16(pre_h) || !aligned16(pre_w) || !aligned16(pre_out))) return PTM_E_ALIGN;
    if (n4 < 1 || n4 > 3 || K <= 0 || (K % 256) != 0 || N6 <= 0) return PTM_E_SHAPE;
    if (K > 16384) return PTM_E_UNSUPPORTED;  // 64 KB of dynamic LDS without raising the cap
    if (!aligned16(x) || !aligned16(gamma) || (stride4 & 15) || (stride6 & 1)) return PTM_E_ALIGN;
    if (stride4 < (int64_t)(K / 256) * 144 || stride6 < (int64_t)(K / 256) * 210) return PTM_E_SHAPE;
    Q4KArgs a4{};
    int total = 0;
    for (int i = 0; i < n4; ++i) {
        if (!W4[i] || !y4[i]) return PTM_E_NULL;
        if (N4[i] <= 0) return PTM_E_SHAPE;
        if (!aligned16(W4[i])) return PTM_E_ALIGN;
        a4.W[i] = static_cast<const uint8_t*>(W4[i]);
        a4.y[i] = y4[i];
        total += N4[i];
        a4.row_end[i] = total;
    }
    a4.n_mat = n4;
    a4.total_rows = total;
    a4.K = K;
    a4.stride = stride4;
    a4.x = x;
    a4.gamma = gamma;
    a4.eps = eps;
    a4.add_one = add_one;
    // Lane groups per row of the two parts.  Every workgroup stages x and gamma (20 KB for 2560 values) for a few KB of
    // weights, so the launch wants few, fat workgroups: the smallest split that still gives the chip 1.5 workgroups
    // per CU, the Q6_K rows (fewer, and more arithmetic per byte) one step finer than the Q4_K ones.  Qwen3-4B and
    // Llama-3-8B shapes both land on 2 and 4 groups per row (448 workgroups): 617 -> 633 tok/s and 518 -> 523 tok/s
    // against the per-kernel rules of the single-type GEMVs (4 and 8 groups, 896 workgroups).
    int l4 = 3, l6 = 3;
    for (int l = 0; l <= 3; ++l) {
        const int t6 = l + 1 < 3 ? l + 1 : 3;
        if ((total + (32 >> l) - 1) / (32 >> l) + (N6 + (32 >> t6) - 1) / (32 >> t6) >= 384 || l == 3) {
            l4 = l;
            l6 = t6;
            break;
        }
    }
    a4.log2S = l4;
    Q6KArgs a6{static_cast<const uint8_t*>(W6), x, y6, K, N6, l6, stride6, nullptr, nullptr,
               gamma, eps, add_one, nullptr, pre_h, pre_w, pre_out};
    a4.pre_h = pre_h;
    a4.pre_w = pre_w;
    a4.pre_out = nullptr;  // the Q6_K workgroup 0 stores the sum
    const int n6 = (N6 + (32 >> l6) - 1) / (32 >> l6), n4w = q4k_workgroups(total, a4.log2S);
    const size_t lds = q6k_x_lds_bytes(K);  // the Q6_K body's fp32 x + per-16 sums; Q4_K needs less
    static const int cand6[] = {2, 3, 5};
    const int nb6 = pick_blocks_per_pass((K / 256 + (1 << l6) - 1) >> l6, cand6, 3);
    const dim3 grid(n6 + n4w);
    const int nb4 = q4k_blocks_per_pass(K / 256, a4.log2S);
    if (pre) mixed_launch4<true>(nb4, nb6, grid, lds, s, a4, a6, n6);
    else mixed_launch4<false>(nb4, nb6, grid, lds, s, a4, a6, n6);
    return launch_status();
}

}  // namespace ptm
