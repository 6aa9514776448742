// placeholder until the MFMA prefill GEMM lands
#include "ptm_common.h"
extern "C" {
int64_t ptm_qgemm_workspace_bytes(int M, int K) { return (int64_t)M * (K + K / 4); }
int ptm_qgemm_q4k(const void*, const void*, float*, int, int, int, int64_t, void*, ptm_stream_t) { return PTM_E_UNSUPPORTED; }
int ptm_qgemm_q6k(const void*, const void*, float*, int, int, int, int64_t, void*, ptm_stream_t) { return PTM_E_UNSUPPORTED; }
}
