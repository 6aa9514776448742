// Quant-type dispatcher of the GEMV operator (reference: cpu_quant_gemv, torch/io/cpu_quant_gemv.h:1635-1688,
// and gemv_scratch, torch/io/gguf_model.h:3117-3140).
#include "ptm_common.h"

extern "C" int ptm_quant_gemv(uint32_t ggml_type, const void* W, const float* x, float* y, int K, int N,
                              int64_t row_stride_bytes, int accumulate, ptm_stream_t stream) {
    switch (ggml_type) {
        case PTM_TYPE_Q4_K: return ptm_q4k_gemv(W, x, y, K, N, row_stride_bytes, accumulate, stream);
        case PTM_TYPE_Q6_K: return ptm_q6k_gemv(W, x, y, K, N, row_stride_bytes, accumulate, stream);
        case PTM_TYPE_Q5_K: return ptm_q5k_gemv(W, x, y, K, N, row_stride_bytes, accumulate, stream);
        case PTM_TYPE_Q8_0: return ptm_q8_0_gemv(W, x, y, K, N, row_stride_bytes, accumulate, stream);
        case PTM_TYPE_Q5_0: return ptm_q5_0_gemv(W, x, y, K, N, row_stride_bytes, accumulate, stream);
        default: return PTM_E_UNSUPPORTED;  // the reference silently does nothing here
    }
}

// cpu_quant_gemv_supported, torch/io/cpu_quant_gemv.h:1691-1694
extern "C" int ptm_quant_gemv_supported(uint32_t t) {
    return t == PTM_TYPE_Q4_K || t == PTM_TYPE_Q8_0 || t == PTM_TYPE_Q6_K || t == PTM_TYPE_Q5_K || t == PTM_TYPE_Q5_0;
}
