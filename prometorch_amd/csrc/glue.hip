// Decode-step glue kernels for gfx950: dequantisation, Q8 activation quantiser, RMSNorm,
// per-head QK-norm + RoPE + KV append, SiLU*up, embedding row, argmax, add/copy.
#include "ptm_common.h"

#include <cmath>

namespace ptm {

thread_local int g_last_hip_error = 0;

// ---------------------------------------------------------------------------------------
// Dequantisation (bit-exact with reference: torch/io/gguf_dequant.h:304-341, :395-430)
// ---------------------------------------------------------------------------------------
// one thread per 4 consecutive weights of a Q4_K block (64 threads per block)
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst,
                                                          int64_t nblocks) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t b = t >> 6;
    if (b >= nblocks) return;
    const int e = (int)(t & 63) * 4;  // element offset in block
    const uint8_t* p = src + b * 144;
    const uint4 hdr = *reinterpret_cast<const uint4*>(p);
    const int sb = e >> 5, l = e & 31;
    int sc, mn;
    q4k_scale_min(hdr.y, hdr.z, hdr.w, sb, sc, mn);
    const float ds = h2f(hdr.x) * (float)sc, ms = h2f(hdr.x >> 16) * (float)mn;
    const uint32_t qw = *reinterpret_cast<const uint32_t*>(p + 16 + 32 * (sb >> 1) + l);
    const uint32_t nib = (sb & 1) ? (qw >> 4) : qw;
    float4 o;
    o.x = ds * (float)(nib & 0xfu) - ms;
    o.y = ds * (float)((nib >> 8) & 0xfu) - ms;
    o.z = ds * (float)((nib >> 16) & 0xfu) - ms;
    o.w = ds * (float)((nib >> 24) & 0xfu) - ms;
    *reinterpret_cast<float4*>(dst + b * 256 + e) = o;
}

__device__ __forceinline__ float q6k_elem(const uint8_t* p, int e) {
    const int half = e >> 7, r = e & 127, grp = r >> 5, l = r & 31;
    const uint32_t lo = p[64 * half + 32 * (grp & 1) + l];
    const uint32_t hi = p[128 + 32 * half + l];
    const int nib = (grp & 2) ? (lo >> 4) : (lo & 0xf);
    const int q = (nib | (((hi >> (2 * grp)) & 3) << 4)) - 32;
    const int sc = (int)(int8_t)p[192 + 8 * half + 2 * grp + (l >> 4)];
    const float d = h2f((uint32_t)p[208] | ((uint32_t)p[209] << 8));
    return d * (float)sc * (float)q;
}

__global__ __launch_bounds__(256) void dequant_q6k_kernel(const uint8_t* __restrict__ src, float* __restrict__ dst,
                                                          int64_t nblocks) {
    const int64_t b = blockIdx.x;
    if (b >= nblocks) return;
    dst[b * 256 + threadIdx.x] = q6k_elem(src + b * 210, threadIdx.x);
}

// Q4_K -> fp16 column-major out[k*N + n] (reference: CUDAQuantGemv.cu:1115-1190)
__global__ __launch_bounds__(256) void dequant_q4k_fp16_kernel(const uint8_t* __restrict__ W, __half* __restrict__ out,
                                                               int K, int N, int64_t stride) {
    const int n = blockIdx.x, b = blockIdx.y, e = threadIdx.x;
    const uint8_t* p = W + (int64_t)n * stride + (int64_t)b * 144;
    const uint4 hdr = *reinterpret_cast<const uint4*>(p);
    const int sb = e >> 5, l = e & 31;
    int sc, mn;
    q4k_scale_min(hdr.y, hdr.z, hdr.w, sb, sc, mn);
    const uint32_t byte = p[16 + 32 * (sb >> 1) + l];
    const float q = (float)((sb & 1) ? (byte >> 4) : (byte & 0xf));
    const float v = h2f(hdr.x) * (float)sc * q - h2f(hdr.x >> 16) * (float)mn;
    out[(int64_t)(b * 256 + e) * N + n] = __float2half_rn(v);
}

// ---------------------------------------------------------------------------------------
// Q8 activation quantiser (reference: torch/io/cpu_quant_gemv.h:147-198)
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void quantize_q8_kernel(const float* __restrict__ x, uint8_t* __restrict__ q8, int K) {
    const int i = blockIdx.x * 256 + threadIdx.x;  // float4 slot; K/4 is a multiple of 64
    if (i >= K / 4) return;
    const float4 v = reinterpret_cast<const float4*>(x)[i];
    float d, s;
    const uint32_t packed = q8_quantize4(v, d, s);
    reinterpret_cast<uint32_t*>(q8)[i] = packed;
    if ((threadIdx.x & 7) == 0) {
        float* xd = reinterpret_cast<float*>(q8 + K);
        xd[i >> 3] = d;
        xd[K / 32 + (i >> 3)] = s;
    }
}

// ---------------------------------------------------------------------------------------
// RMSNorm (reference: CUDAInference.cu:19-76; CPU order x*rms*w as cpu_quant_gemv.h:2567-2610)
// ---------------------------------------------------------------------------------------
template <bool Q8OUT>
__global__ __launch_bounds__(256) void rms_norm_kernel(const float* __restrict__ in, const float* __restrict__ w,
                                                       float* __restrict__ out, int hidden, float eps, int add_one,
                                                       uint8_t* __restrict__ q8) {
    __shared__ float red[4];
    const float* x = in + (int64_t)blockIdx.x * hidden;
    float* o = out + (int64_t)blockIdx.x * hidden;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < hidden; i += 256) ss = fmaf(x[i], x[i], ss);
    ss = block_sum256(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)hidden + eps);
    const float one = add_one ? 1.0f : 0.0f;
    if constexpr (Q8OUT) {
        for (int i = threadIdx.x; i < hidden / 4; i += 256) {
            const float4 v = reinterpret_cast<const float4*>(x)[i];
            const float4 g = reinterpret_cast<const float4*>(w)[i];
            float4 r;
            r.x = v.x * rs * (g.x + one);
            r.y = v.y * rs * (g.y + one);
            r.z = v.z * rs * (g.z + one);
            r.w = v.w * rs * (g.w + one);
            reinterpret_cast<float4*>(o)[i] = r;
            float d, s;
            const uint32_t packed = q8_quantize4(r, d, s);
            reinterpret_cast<uint32_t*>(q8)[i] = packed;
            if ((threadIdx.x & 7) == 0) {
                float* xd = reinterpret_cast<float*>(q8 + hidden);
                xd[i >> 3] = d;
                xd[hidden / 32 + (i >> 3)] = s;
            }
        }
    } else {
        for (int i = threadIdx.x; i < hidden; i += 256) o[i] = x[i] * rs * (w[i] + one);
    }
}

// x[r][:] += RMSNorm(h[r][:]) * w: the post-norm of a gemma2 / gemma3 branch and its residual add
// (gguf_model.h:3656-3680, :3787-3807); one workgroup per row
__global__ __launch_bounds__(256) void rms_norm_add_kernel(const float* __restrict__ h, const float* __restrict__ w,
                                                           float* __restrict__ x, int hidden, float eps, int add_one) {
    __shared__ float red[4];
    const float* hr = h + (int64_t)blockIdx.x * hidden;
    float* xr = x + (int64_t)blockIdx.x * hidden;
    const float one = add_one ? 1.0f : 0.0f;
    if ((hidden & 3) == 0 && hidden <= 4 * 256 * 4) {
        // rows of up to 4096 values: every load goes out before the reduction, one memory round trip
        const int nv = hidden >> 2;
        float4 hv[4], xv[4], wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = threadIdx.x + 256 * j;
            const int ic = i < nv ? i : 0;
            hv[j] = reinterpret_cast<const float4*>(hr)[ic];
            xv[j] = reinterpret_cast<const float4*>(xr)[ic];
            wv[j] = reinterpret_cast<const float4*>(w)[ic];
        }
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (threadIdx.x + 256 * j < nv) {
                ss = fmaf(hv[j].x, hv[j].x, ss);
                ss = fmaf(hv[j].y, hv[j].y, ss);
                ss = fmaf(hv[j].z, hv[j].z, ss);
                ss = fmaf(hv[j].w, hv[j].w, ss);
            }
        }
        ss = block_sum256(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < nv) {
                float4 r;
                r.x = xv[j].x + hv[j].x * rs * (wv[j].x + one);
                r.y = xv[j].y + hv[j].y * rs * (wv[j].y + one);
                r.z = xv[j].z + hv[j].z * rs * (wv[j].z + one);
                r.w = xv[j].w + hv[j].w * rs * (wv[j].w + one);
                reinterpret_cast<float4*>(xr)[i] = r;
            }
        }
        return;
    }
    float ss = 0.0f;
    for (int i = threadIdx.x; i < hidden; i += 256) ss = fmaf(hr[i], hr[i], ss);
    ss = block_sum256(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += 256) xr[i] = xr[i] + hr[i] * rs * (w[i] + one);
}

__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ x, float s, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] *= s;
}

// tanh-approximated GELU(gate) * up, the expression of gguf_model.h:3730-3738
__global__ __launch_bounds__(256) void gelu_mul_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                       float* __restrict__ o, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float x = g[i];
    const float x3 = x * x * x;
    const float t = tanhf(0.7978845608028654f * (x + 0.044715f * x3));
    o[i] = 0.5f * x * (1.0f + t) * u[i];
}

// in-place per-head RMSNorm: one wave per (row, head)
__global__ __launch_bounds__(64) void per_head_rms_norm_kernel(float* __restrict__ data, const float* __restrict__ w,
                                                               int head_dim, float eps, int add_one) {
    float* x = data + (int64_t)blockIdx.x * head_dim;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < head_dim; i += 64) ss = fmaf(x[i], x[i], ss);
    ss = sum64(ss);
    const float rs = 1.0f / sqrtf(ss / (float)head_dim + eps);
    const float one = add_one ? 1.0f : 0.0f;
    for (int i = threadIdx.x; i < head_dim; i += 64) x[i] = x[i] * rs * (w[i] + one);
}

// ---------------------------------------------------------------------------------------
// Fused QK-norm + RoPE + KV append (reference: FlashDecoding.cu:256-395, :641-744; CPU order
// gguf_model.h:3441-3479 and hot_loops.cpp:1853-1876, :2035-2061)
// grid = n_heads + n_kv_heads blocks of one wave; thread t owns the rotation pair t
// (NeoX: (t, t+hd/2); interleaved: (2t, 2t+1)); K-head blocks also append K and V.
// ---------------------------------------------------------------------------------------
template <bool KV16>
__global__ __launch_bounds__(64) void qknorm_rope_kvwrite_kernel(float* __restrict__ Q, float* __restrict__ K,
                                                                 const float* __restrict__ V,
                                                                 const float* __restrict__ qw,
                                                                 const float* __restrict__ kw, void* __restrict__ Kc,
                                                                 void* __restrict__ Vc, int n_heads, int n_kv_heads,
                                                                 int head_dim, const int64_t* __restrict__ d_past,
                                                                 int64_t pos_host, int64_t row_host,
                                                                 int max_seq, float base, const float* __restrict__ table,
                                                                 float eps, int add_one, int neox) {
    // d_past != NULL: position and cache row both come from device memory (graph-replayable); otherwise from the host
    // arguments, where the rotation position and the cache row may differ (launch_fused_qknorm_rope_kvwrite's
    // `position` / `cache_offset_row`, CUDAOps.h:563-570)
    const int64_t pos = d_past ? *d_past : pos_host;
    const int64_t crow = d_past ? pos : row_host;
    if (pos < 0 || crow < 0 || crow >= max_seq || (table && pos >= max_seq)) return;  // never touch memory outside the cache / table
    const int hb = blockIdx.x;
    const bool is_k = hb >= n_heads;
    const int h = is_k ? hb - n_heads : hb;
    float* vec = (is_k ? K : Q) + (int64_t)h * head_dim;
    const float* nw = is_k ? kw : qw;
    const int half = head_dim / 2;
    // thread t owns rotation pairs t and t + 64 (the second only for heads wider than 128)
    float x0[2], x1[2];
    int i0[2], i1[2];
    bool on[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int t = threadIdx.x + 64 * j;
        on[j] = t < half;
        i0[j] = neox ? t : 2 * t;
        i1[j] = neox ? t + half : 2 * t + 1;
        x0[j] = on[j] ? vec[i0[j]] : 0.0f;
        x1[j] = on[j] ? vec[i1[j]] : 0.0f;
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
        float c, s;
        if (table) {
            c = table[pos * head_dim + t];
            s = table[pos * head_dim + half + t];
        } else {
            const float inv = 1.0f / powf(base, 2.0f * (float)t / (float)head_dim);
            const float th = (float)pos * inv;
            c = cosf(th);
            s = sinf(th);
        }
        const float r0 = fmaf(x0[j], c, -(x1[j] * s));
        const float r1 = fmaf(x0[j], s, x1[j] * c);
        vec[i0[j]] = r0;
        vec[i1[j]] = r1;
        if (is_k) {
            const int64_t row = crow * (int64_t)(n_kv_heads * head_dim) + (int64_t)h * head_dim;
            const float v0 = V[h * head_dim + i0[j]], v1 = V[h * head_dim + i1[j]];
            if constexpr (KV16) {
                __half* kc = static_cast<__half*>(Kc) + row;
                __half* vc = static_cast<__half*>(Vc) + row;
                kc[i0[j]] = __float2half_rn(r0);
                kc[i1[j]] = __float2half_rn(r1);
                vc[i0[j]] = __float2half_rn(v0);
                vc[i1[j]] = __float2half_rn(v1);
            } else {
                float* kc = static_cast<float*>(Kc) + row;
                float* vc = static_cast<float*>(Vc) + row;
                kc[i0[j]] = r0;
                kc[i1[j]] = r1;
                vc[i0[j]] = v0;
                vc[i1[j]] = v1;
            }
        }
    }
}

__global__ __launch_bounds__(256) void fp16_kv_write_kernel(const float* __restrict__ src, __half* __restrict__ dst,
                                                            int64_t n, int64_t dst_off) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[dst_off + i] = __float2half_rn(src[i]);
}

// ---------------------------------------------------------------------------------------
// Elementwise
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                       float* __restrict__ o, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    // reference CPU order (gguf_model.h:3741-3755): clamp(-g), exp, 1/(1+e), g*sig, *u
    const float gv = g[i];
    float ng = 0.0f - gv;
    ng = fminf(fmaxf(ng, -88.0f), 88.0f);
    const float sig = 1.0f / (1.0f + expf(ng));
    o[i] = (gv * sig) * u[i];
}

__global__ __launch_bounds__(256) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                  float* __restrict__ o, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) o[i] = a[i] + b[i];
}

// Q[r][j] += bq[j], K[r][j] += bk[j], V[r][j] += bv[j] for `rows` rows in one launch (element e of a row of
// q_dim + 2 kv_dim values picks its segment)
__global__ __launch_bounds__(256) void qkv_bias_kernel(float* __restrict__ Q, float* __restrict__ K, float* __restrict__ V,
                                                       const float* __restrict__ bq, const float* __restrict__ bk,
                                                       const float* __restrict__ bv, int64_t rows, int q_dim, int kv_dim) {
    const int w = q_dim + 2 * kv_dim;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= rows * w) return;
    const int64_t r = e / w;
    const int j = (int)(e - r * w);
    if (j < q_dim) Q[r * q_dim + j] += bq[j];
    else if (j < q_dim + kv_dim) K[r * kv_dim + (j - q_dim)] += bk[j - q_dim];
    else V[r * kv_dim + (j - q_dim - kv_dim)] += bv[j - q_dim - kv_dim];
}

__global__ __launch_bounds__(256) void copy_kernel(const float* __restrict__ a, float* __restrict__ o, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) o[i] = a[i];
}

__global__ __launch_bounds__(256) void embedding_row_kernel(const float* __restrict__ table, float* __restrict__ out,
                                                            const int* __restrict__ d_tok, int hidden) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < hidden) out[i] = table[(int64_t)(*d_tok) * hidden + i];
}

__global__ __launch_bounds__(256) void embedding_row_q6k_kernel(const uint8_t* __restrict__ table, float* __restrict__ out,
                                                                const int* __restrict__ d_tok, int hidden, int64_t stride) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < hidden) out[i] = q6k_elem(table + (int64_t)(*d_tok) * stride + (int64_t)(i >> 8) * 210, i & 255);
}

// single-workgroup argmax, strict '>' with lowest index on ties (reference: CUDAReduce.cu:447-479)
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ in, int64_t* __restrict__ out, int64_t n) {
    __shared__ float bv[16];
    __shared__ int64_t bi[16];
    float v = -INFINITY;
    int64_t idx = INT64_MAX;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const float x = in[i];
        if (x > v) { v = x; idx = i; }  // ascending i per thread: first maximum kept
    }
    for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int64_t oi = __shfl_xor(idx, off, 64);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
        *out = idx == INT64_MAX ? 0 : idx;
    }
}

}  // namespace ptm

using namespace ptm;

static inline unsigned nblk256(int64_t n) { return (unsigned)((n + 255) / 256); }

extern "C" {

const char* ptm_strerror(int code) {
    switch (code) {
        case PTM_OK: return "ok";
        case PTM_E_NULL: return "required pointer is NULL";
        case PTM_E_SHAPE: return "bad shape (K must be a positive multiple of 256, sizes positive, stride >= row bytes)";
        case PTM_E_ALIGN: return "alignment precondition violated";
        case PTM_E_UNSUPPORTED: return "unsupported type or size";
        case PTM_E_HIP: return "HIP runtime error";
        case PTM_E_RANGE: return "index out of range";
        case PTM_E_STATE: return "invalid object state";
        case PTM_E_IO: return "file cannot be opened or mapped";
        case PTM_E_FORMAT: return "malformed GGUF file or missing / mistyped key";
        case PTM_E_NOT_FOUND: return "no tensor or key of that name";
        default: return "unknown error";
    }
}
int ptm_last_hip_error(void) { return g_last_hip_error; }
int ptm_version(void) { return 100; }
int ptm_device_cus(void) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return cus;
}

int ptm_dequant_q4k(const void* blocks, float* out, int64_t n, ptm_stream_t stream) {
    if (!blocks || !out) return PTM_E_NULL;
    if (n < 0 || (n % 256) != 0) return PTM_E_SHAPE;
    if (!aligned16(blocks) || !aligned16(out)) return PTM_E_ALIGN;
    if (n == 0) return PTM_OK;
    const int64_t nb = n / 256;
    hipLaunchKernelGGL(dequant_q4k_kernel, dim3(nblk256(nb * 64)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(blocks), out, nb);
    return launch_status();
}

int ptm_dequant_q6k(const void* blocks, float* out, int64_t n, ptm_stream_t stream) {
    if (!blocks || !out) return PTM_E_NULL;
    if (n < 0 || (n % 256) != 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    if (n / 256 > 0x7fffffff) return PTM_E_UNSUPPORTED;
    hipLaunchKernelGGL(dequant_q6k_kernel, dim3((unsigned)(n / 256)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(blocks), out, n / 256);
    return launch_status();
}

int ptm_dequant_q4k_to_fp16(const void* W, void* out, int K, int N, int64_t stride, ptm_stream_t stream) {
    if (!W || !out) return PTM_E_NULL;
    if (K <= 0 || N <= 0 || (K % 256) != 0 || stride < (int64_t)(K / 256) * 144) return PTM_E_SHAPE;
    if (!aligned16(W) || (stride & 15)) return PTM_E_ALIGN;
    if (K / 256 > 65535) return PTM_E_UNSUPPORTED;
    hipLaunchKernelGGL(dequant_q4k_fp16_kernel, dim3(N, K / 256), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(W), static_cast<__half*>(out), K, N, stride);
    return launch_status();
}

int64_t ptm_q8_bytes(int K) { return q8_bytes(K); }

int ptm_quantize_q8(const float* x, void* q8, int K, ptm_stream_t stream) {
    if (!x || !q8) return PTM_E_NULL;
    if (K <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (!aligned16(x) || !aligned16(q8)) return PTM_E_ALIGN;
    hipLaunchKernelGGL(quantize_q8_kernel, dim3(nblk256(K / 4)), dim3(256), 0, as_stream(stream), x,
                       static_cast<uint8_t*>(q8), K);
    return launch_status();
}

int ptm_rms_norm(const float* in, const float* weight, float* out, int rows, int hidden, float eps, int add_one,
                 void* q8_out, ptm_stream_t stream) {
    if (!in || !weight || !out) return PTM_E_NULL;
    if (rows <= 0 || hidden <= 0) return PTM_E_SHAPE;
    if (q8_out) {
        if (rows != 1 || (hidden % 256) != 0) return PTM_E_SHAPE;
        if (!aligned16(in) || !aligned16(weight) || !aligned16(out) || !aligned16(q8_out)) return PTM_E_ALIGN;
        hipLaunchKernelGGL(rms_norm_kernel<true>, dim3(1), dim3(256), 0, as_stream(stream), in, weight, out, hidden,
                           eps, add_one, static_cast<uint8_t*>(q8_out));
    } else {
        hipLaunchKernelGGL(rms_norm_kernel<false>, dim3(rows), dim3(256), 0, as_stream(stream), in, weight, out,
                           hidden, eps, add_one, static_cast<uint8_t*>(nullptr));
    }
    return launch_status();
}

int ptm_per_head_rms_norm(float* data, const float* weight, int rows, int n_heads, int head_dim, float eps,
                          int add_one, ptm_stream_t stream) {
    if (!data || !weight) return PTM_E_NULL;
    if (rows <= 0 || n_heads <= 0 || head_dim <= 0) return PTM_E_SHAPE;
    hipLaunchKernelGGL(per_head_rms_norm_kernel, dim3(rows * n_heads), dim3(64), 0, as_stream(stream), data, weight,
                       head_dim, eps, add_one);
    return launch_status();
}

static int qknorm_rope_kvwrite_any(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                   void* K_cache, void* V_cache, int n_heads, int n_kv_heads, int head_dim,
                                   const int64_t* d_past_len, int64_t pos_host, int64_t row_host, int max_seq,
                                   float rope_freq_base, const float* rope_table, float eps, int add_one, int neox,
                                   int kv_fp16, ptm_stream_t stream) {
    if (!Q || !K || !V || !K_cache || !V_cache) return PTM_E_NULL;
    if ((q_norm_w == nullptr) != (k_norm_w == nullptr)) return PTM_E_NULL;
    if (n_heads <= 0 || n_kv_heads <= 0 || max_seq <= 0 || head_dim <= 0 || (head_dim & 1)) return PTM_E_SHAPE;
    if (head_dim > 256) return PTM_E_UNSUPPORTED;
    const dim3 grid(n_heads + n_kv_heads);
    if (kv_fp16)
        hipLaunchKernelGGL(qknorm_rope_kvwrite_kernel<true>, grid, dim3(64), 0, as_stream(stream), Q, K, V, q_norm_w,
                           k_norm_w, K_cache, V_cache, n_heads, n_kv_heads, head_dim, d_past_len, pos_host, row_host, max_seq,
                           rope_freq_base, rope_table, eps, add_one, neox);
    else
        hipLaunchKernelGGL(qknorm_rope_kvwrite_kernel<false>, grid, dim3(64), 0, as_stream(stream), Q, K, V, q_norm_w,
                           k_norm_w, K_cache, V_cache, n_heads, n_kv_heads, head_dim, d_past_len, pos_host, row_host, max_seq,
                           rope_freq_base, rope_table, eps, add_one, neox);
    return launch_status();
}

int ptm_qknorm_rope_kvwrite(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                            void* K_cache, void* V_cache, int n_heads, int n_kv_heads, int head_dim,
                            const int64_t* d_past_len, int max_seq, float rope_freq_base, const float* rope_table,
                            float eps, int add_one, int neox, int kv_fp16, ptm_stream_t stream) {
    if (!d_past_len) return PTM_E_NULL;
    return qknorm_rope_kvwrite_any(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, n_heads, n_kv_heads, head_dim, d_past_len,
                                   0, 0, max_seq, rope_freq_base, rope_table, eps, add_one, neox, kv_fp16, stream);
}

int ptm_qknorm_rope_kvwrite_pos(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                void* K_cache, void* V_cache, int n_heads, int n_kv_heads, int head_dim, int position,
                                int64_t cache_offset_row, int max_seq, float rope_freq_base, const float* rope_table,
                                float eps, int add_one, int neox, int kv_fp16, ptm_stream_t stream) {
    if (position < 0 || cache_offset_row < 0 || cache_offset_row >= max_seq || (rope_table && position >= max_seq))
        return PTM_E_RANGE;
    return qknorm_rope_kvwrite_any(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, n_heads, n_kv_heads, head_dim, nullptr,
                                   position, cache_offset_row, max_seq, rope_freq_base, rope_table, eps, add_one, neox,
                                   kv_fp16, stream);
}

int ptm_rope_table_host(float* table, int max_seq, int head_dim, float base) {
    return ptm_rope_table_host_scaled(table, max_seq, head_dim, base, 1.0f);
}

int ptm_rope_table_host_scaled(float* table, int max_seq, int head_dim, float base, float scale) {
    return ptm_rope_table_host_factors(table, max_seq, head_dim, base, scale, nullptr, nullptr, 0, 1.0f);
}

int ptm_rope_table_host_factors(float* table, int max_seq, int head_dim, float base, float scale, const float* factors_short,
                                const float* factors_long, int orig_ctx, float attn_factor) {
    if (!table) return PTM_E_NULL;
    if (max_seq <= 0 || head_dim <= 0 || (head_dim & 1)) return PTM_E_SHAPE;
    const int half = head_dim / 2;
    const bool scaled = scale > 0.0f && scale != 1.0f;                 // hot_loops.cpp:1858-1860
    const bool apply_af = attn_factor > 0.0f && attn_factor != 1.0f;   // hot_loops.cpp:1861
    for (int pos = 0; pos < max_seq; ++pos) {
        const float p = scaled ? (float)pos / scale : (float)pos;
        // the reference picks the set by the sequence length after this token (gguf_model.h:285-296, called with past + 1)
        const float* factors = orig_ctx <= 0 ? nullptr : (pos + 1 <= orig_ctx ? factors_short : factors_long);
        for (int d = 0; d < half; ++d) {
            float inv = 1.0f / std::pow(base, 2.0f * (float)d / (float)head_dim);
            if (factors) inv /= factors[d];
            const float th = p * inv;
            float c = std::cos(th), s = std::sin(th);
            if (apply_af) { c *= attn_factor; s *= attn_factor; }
            table[(int64_t)pos * head_dim + d] = c;
            table[(int64_t)pos * head_dim + half + d] = s;
        }
    }
    return PTM_OK;
}

int ptm_fp16_kv_cache_write(const float* src, void* dst, int64_t rows, int64_t cols, int64_t offset_row,
                            ptm_stream_t stream) {
    if (!src || !dst) return PTM_E_NULL;
    if (rows < 0 || cols <= 0 || offset_row < 0) return PTM_E_SHAPE;
    if (rows == 0) return PTM_OK;
    hipLaunchKernelGGL(fp16_kv_write_kernel, dim3(nblk256(rows * cols)), dim3(256), 0, as_stream(stream), src,
                       static_cast<__half*>(dst), rows * cols, offset_row * cols);
    return launch_status();
}

int ptm_silu_mul(const float* gate, const float* up, float* out, int64_t n, ptm_stream_t stream) {
    if (!gate || !up || !out) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(silu_mul_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), gate, up, out, n);
    return launch_status();
}

int ptm_embedding_row(const float* table, float* out, const int* d_token_id, int hidden, ptm_stream_t stream) {
    if (!table || !out || !d_token_id) return PTM_E_NULL;
    if (hidden <= 0) return PTM_E_SHAPE;
    hipLaunchKernelGGL(embedding_row_kernel, dim3(nblk256(hidden)), dim3(256), 0, as_stream(stream), table, out,
                       d_token_id, hidden);
    return launch_status();
}

int ptm_embedding_row_q6k(const void* table, float* out, const int* d_token_id, int hidden, int64_t stride,
                          ptm_stream_t stream) {
    if (!table || !out || !d_token_id) return PTM_E_NULL;
    if (hidden <= 0 || (hidden % 256) != 0 || stride < (int64_t)(hidden / 256) * 210) return PTM_E_SHAPE;
    hipLaunchKernelGGL(embedding_row_q6k_kernel, dim3(nblk256(hidden)), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(table), out, d_token_id, hidden, stride);
    return launch_status();
}

int ptm_argmax(const float* in, int64_t* out, int64_t n, ptm_stream_t stream) {
    if (!in || !out) return PTM_E_NULL;
    if (n <= 0) return PTM_E_SHAPE;
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, as_stream(stream), in, out, n);
    return launch_status();
}

int ptm_rms_norm_add(const float* h, const float* weight, float* x, int rows, int hidden, float eps, int add_one,
                     ptm_stream_t stream) {
    if (!h || !weight || !x) return PTM_E_NULL;
    if (rows < 0 || hidden <= 0) return PTM_E_SHAPE;
    if ((hidden & 3) == 0 && (!aligned16(h) || !aligned16(weight) || !aligned16(x))) return PTM_E_ALIGN;
    if (rows == 0) return PTM_OK;
    hipLaunchKernelGGL(rms_norm_add_kernel, dim3(rows), dim3(256), 0, as_stream(stream), h, weight, x, hidden, eps, add_one);
    return launch_status();
}

int ptm_scale(float* x, float factor, int64_t n, ptm_stream_t stream) {
    if (!x) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(scale_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), x, factor, n);
    return launch_status();
}

int ptm_gelu_mul(const float* gate, const float* up, float* out, int64_t n, ptm_stream_t stream) {
    if (!gate || !up || !out) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(gelu_mul_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), gate, up, out, n);
    return launch_status();
}

int ptm_add(const float* a, const float* b, float* out, int64_t n, ptm_stream_t stream) {
    if (!a || !b || !out) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(add_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), a, b, out, n);
    return launch_status();
}

int ptm_add_qkv_bias(float* Q, float* K, float* V, const float* q_bias, const float* k_bias, const float* v_bias, int rows,
                     int q_dim, int kv_dim, ptm_stream_t stream) {
    if (!Q || !K || !V || !q_bias || !k_bias || !v_bias) return PTM_E_NULL;
    if (rows < 0 || q_dim <= 0 || kv_dim <= 0) return PTM_E_SHAPE;
    if (rows == 0) return PTM_OK;
    const int64_t n = (int64_t)rows * (q_dim + 2 * (int64_t)kv_dim);
    hipLaunchKernelGGL(qkv_bias_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), Q, K, V, q_bias, k_bias, v_bias,
                       (int64_t)rows, q_dim, kv_dim);
    return launch_status();
}

int ptm_copy(const float* in, float* out, int64_t n, ptm_stream_t stream) {
    if (!in || !out) return PTM_E_NULL;
    if (n < 0) return PTM_E_SHAPE;
    if (n == 0) return PTM_OK;
    hipLaunchKernelGGL(copy_kernel, dim3(nblk256(n)), dim3(256), 0, as_stream(stream), in, out, n);
    return launch_status();
}

}  // extern "C"
