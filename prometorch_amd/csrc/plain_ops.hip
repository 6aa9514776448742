// The unquantised operators the reference's decode and prefill host code calls beside the k-quant kernels
// (aten/src/ATen/cuda/CUDAInference.cu, CUDAQuantGemv.cu:1212-1330, CUDABlas.cu:532, CUDAKernels.cu:768): fp32 and fp16
// weight GEMVs (models whose output or embedding matrix is stored unquantised), rotation of a row block, KV row copy,
// row concatenation, out-of-place scaling.  None of them is on the Q4_K_M hot path; they exist so that every launcher the
// reference's forward_decode / forward name has a counterpart.  One wave per output row, lanes striding the row with
// 16-byte loads; x is read through the cache.
#include "ptm_common.h"

namespace ptm {

__global__ __launch_bounds__(256) void mul_scalar_kernel(const float* __restrict__ a, float s, float* __restrict__ o, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) o[i] = a[i] * s;
}

__global__ __launch_bounds__(256) void kv_rows_copy_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n,
                                                           int64_t dst_off) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[dst_off + i] = src[i];
}

__global__ __launch_bounds__(256) void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          float* __restrict__ o, int64_t na, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) o[i] = i < na ? a[i] : b[i - na];
}

// data [seq_len][n_heads * head_dim]; row s is rotated at position position_offset + s.  A thread owns one rotation pair:
// interleaved (2d, 2d + 1) as the reference's rope_kernel (CUDAInference.cu:149-175), or NeoX (d, d + head_dim / 2).
// Angles from `table` ([rows][head_dim]: cos[0..hd/2), sin[0..hd/2) per position) when given, else computed here.
__global__ __launch_bounds__(256) void rope_rows_kernel(float* __restrict__ data, int64_t total_pairs, int n_heads, int head_dim,
                                                        int position_offset, float base, const float* __restrict__ table,
                                                        int neox) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total_pairs) return;
    const int half = head_dim / 2;
    const int d = (int)(idx % half);
    const int64_t hs = idx / half;  // s * n_heads + h
    const int64_t s = hs / n_heads;
    const int64_t pos = position_offset + s;
    float c, sn;
    if (table) {
        c = table[pos * head_dim + d];
        sn = table[pos * head_dim + half + d];
    } else {
        const float inv = 1.0f / powf(base, 2.0f * (float)d / (float)head_dim);
        const float th = (float)pos * inv;
        c = cosf(th);
        sn = sinf(th);
    }
    float* v = data + hs * head_dim;
    const int i0 = neox ? d : 2 * d, i1 = neox ? d + half : 2 * d + 1;
    const float x0 = v[i0], x1 = v[i1];
    v[i0] = fmaf(x0, c, -(x1 * sn));
    v[i1] = fmaf(x0, sn, x1 * c);
}

// y[n] = sum_k W[n][k] x[k], W row-major fp32 (launch_gemv, CUDABlas.cu:532) or fp16 (launch_fp16_gemv,
// CUDAQuantGemv.cu:1306-1330; XH: x rounded to fp16 first, as launch_cublas_hgemv does, :1212-1269).
template <typename WT, bool XH>
__global__ __launch_bounds__(256) void rowmajor_gemv_kernel(const WT* __restrict__ W, const float* __restrict__ x,
                                                            float* __restrict__ y, int K, int N) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const WT* row = W + (int64_t)n * K;
    float acc = 0.0f;
    for (int k = lane; k < K; k += 64) {
        float xv = x[k];
        if constexpr (XH) xv = __half2float(__float2half_rn(xv));
        float wv;
        if constexpr (sizeof(WT) == 2) wv = __half2float(row[k]);
        else wv = row[k];
        acc = fmaf(wv, xv, acc);
    }
    acc = sum64(acc);
    if (lane == 0) y[n] = acc;
}

// y[n] = sum_k W[k][n] x[k]: the [K][N] layout of launch_inference_gemv (fp32, CUDAInference.cu:426-470) and of
// launch_cublas_hgemv's default, column-major [N][K] with lda = N, which is what launch_dequant_q4k_to_fp16 writes.
// A thread owns one output; consecutive threads read consecutive words of a row of W.
template <typename WT, bool XH>
__global__ __launch_bounds__(256) void kmajor_gemv_kernel(const WT* __restrict__ W, const float* __restrict__ x,
                                                          float* __restrict__ y, int K, int N) {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) {
        float xv = x[k];
        if constexpr (XH) xv = __half2float(__float2half_rn(xv));
        float wv;
        if constexpr (sizeof(WT) == 2) wv = __half2float(W[(int64_t)k * N + n]);
        else wv = W[(int64_t)k * N + n];
        acc = fmaf(wv, xv, acc);
    }
    y[n] = acc;
}

}  // namespace ptm

using namespace ptm;

static inline unsigned blocks256(int64_t n) { return (unsigned)((n + 255) / 256); }

extern "C" {

int ptm_mul_scalar(const float* a, float factor, float* out, int64_t n, ptm_stream_t stream) {
    if (!a || !out) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(mul_scalar_kernel, dim3(blocks256(n)), dim3(256), 0, as_stream(stream), a, factor, out, n);
    return launch_status();
}

int ptm_kv_cache_write(const float* src, float* dst_cache, int64_t num_new_rows, int64_t cols, int64_t offset_row,
                       ptm_stream_t stream) {
    if (!src || !dst_cache) return PTM_E_NULL;
    if (num_new_rows < 0 || cols <= 0 || offset_row < 0) return PTM_E_SHAPE;
    if (num_new_rows == 0) return PTM_OK;
    hipLaunchKernelGGL(kv_rows_copy_kernel, dim3(blocks256(num_new_rows * cols)), dim3(256), 0, as_stream(stream), src,
                       dst_cache, num_new_rows * cols, offset_row * cols);
    return launch_status();
}

int ptm_concat_rows(const float* a, const float* b, float* out, int64_t a_rows, int64_t b_rows, int64_t cols,
                    ptm_stream_t stream) {
    if (!out || (a_rows > 0 && !a) || (b_rows > 0 && !b)) return PTM_E_NULL;
    if (a_rows < 0 || b_rows < 0 || cols <= 0) return PTM_E_SHAPE;
    const int64_t n = (a_rows + b_rows) * cols;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(concat_rows_kernel, dim3(blocks256(n)), dim3(256), 0, as_stream(stream), a, b, out, a_rows * cols, n);
    return launch_status();
}

int ptm_rope(float* data, int seq_len, int n_heads, int head_dim, int position_offset, float rope_freq_base,
             const float* rope_table, int table_rows, int neox, ptm_stream_t stream) {
    if (!data) return PTM_E_NULL;
    if (seq_len < 0 || n_heads <= 0 || head_dim <= 0 || (head_dim & 1)) return PTM_E_SHAPE;
    if (position_offset < 0 || (rope_table && (int64_t)position_offset + seq_len > table_rows)) return PTM_E_RANGE;
    if (seq_len == 0) return PTM_OK;
    const int64_t pairs = (int64_t)seq_len * n_heads * (head_dim / 2);
    hipLaunchKernelGGL(rope_rows_kernel, dim3(blocks256(pairs)), dim3(256), 0, as_stream(stream), data, pairs, n_heads,
                       head_dim, position_offset, rope_freq_base, rope_table, neox);
    return launch_status();
}

int ptm_f32_gemv(const float* W, const float* x, float* y, int K, int N, int k_major, ptm_stream_t stream) {
    if (!W || !x || !y) return PTM_E_NULL;
    if (K <= 0 || N <= 0) return PTM_E_SHAPE;
    if (k_major)
        hipLaunchKernelGGL((kmajor_gemv_kernel<float, false>), dim3(blocks256(N)), dim3(256), 0, as_stream(stream), W, x, y, K, N);
    else
        hipLaunchKernelGGL((rowmajor_gemv_kernel<float, false>), dim3((N + 3) / 4), dim3(256), 0, as_stream(stream), W, x, y, K, N);
    return launch_status();
}

int ptm_f16_gemv(const void* W_fp16, const float* x, float* y, int K, int N, int k_major, int round_x, ptm_stream_t stream) {
    if (!W_fp16 || !x || !y) return PTM_E_NULL;
    if (K <= 0 || N <= 0) return PTM_E_SHAPE;
    if (reinterpret_cast<uintptr_t>(W_fp16) & 1u) return PTM_E_ALIGN;
    const __half* W = static_cast<const __half*>(W_fp16);
    hipStream_t s = as_stream(stream);
    if (k_major) {
        if (round_x) hipLaunchKernelGGL((kmajor_gemv_kernel<__half, true>), dim3(blocks256(N)), dim3(256), 0, s, W, x, y, K, N);
        else hipLaunchKernelGGL((kmajor_gemv_kernel<__half, false>), dim3(blocks256(N)), dim3(256), 0, s, W, x, y, K, N);
    } else {
        if (round_x) hipLaunchKernelGGL((rowmajor_gemv_kernel<__half, true>), dim3((N + 3) / 4), dim3(256), 0, s, W, x, y, K, N);
        else hipLaunchKernelGGL((rowmajor_gemv_kernel<__half, false>), dim3((N + 3) / 4), dim3(256), 0, s, W, x, y, K, N);
    }
    return launch_status();
}

}  // extern "C"
