// Measurement aid for bench.py, not part of libptm_hip.so: a pure streaming read, the ceiling a weight-streaming kernel of
// the same footprint is measured against.  Built into libptm_bench.so beside bench.py.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

// Streaming read of `n16` 16-byte words: the ceiling a weight-streaming kernel of the same footprint is measured
// against.  Eight independent 16-byte loads per lane, consecutive lanes on consecutive words; the XOR of a
// workgroup's words is its one output, so the loads cannot be dropped and the result can be checked.
enum { STREAM_READ_WORDS_PER_LANE = 8, STREAM_READ_WORDS_PER_WG = 256 * STREAM_READ_WORDS_PER_LANE };
static __global__ __launch_bounds__(256) void stream_read_xor_kernel(const uint4* __restrict__ p, int64_t n16,
                                                              uint32_t* __restrict__ out) {
    __shared__ uint32_t part[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t base = (int64_t)blockIdx.x * STREAM_READ_WORDS_PER_WG + wave * (64 * STREAM_READ_WORDS_PER_LANE) + lane;
    uint4 v[STREAM_READ_WORDS_PER_LANE];
#pragma unroll
    for (int i = 0; i < STREAM_READ_WORDS_PER_LANE; ++i) {
        const int64_t idx = base + i * 64;
        v[i] = idx < n16 ? p[idx] : make_uint4(0, 0, 0, 0);
    }
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < STREAM_READ_WORDS_PER_LANE; ++i) s ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s ^= __shfl_xor(s, o);
    if (lane == 0) part[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

}  // namespace

extern "C" {

// number of 32 KiB spans of `bytes` (one partial XOR each)
int64_t bench_stream_read_partials(int64_t bytes) {
    return bytes <= 0 ? 0 : (bytes / 16 + STREAM_READ_WORDS_PER_WG - 1) / STREAM_READ_WORDS_PER_WG;
}

// out_partials[i] = XOR of all 32-bit words of the i-th 32 KiB span of src (bytes a multiple of 16, src 16-byte aligned);
// 0 on success, -1 on a bad argument, -2 when the launch failed
int bench_stream_read_xor(const void* src, int64_t bytes, uint32_t* out_partials, void* stream) {
    if (!src || !out_partials || bytes <= 0 || bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(src) & 15) != 0) return -1;
    const int64_t wgs = bench_stream_read_partials(bytes);
    if (wgs > 0x7fffffff) return -1;
    hipLaunchKernelGGL(stream_read_xor_kernel, dim3((unsigned)wgs), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(src), bytes / 16, out_partials);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

}  // extern "C"
