/* TEST INFRASTRUCTURE ONLY — see ptm_oracle.h.
 *
 * Restates, on the CPU, the arithmetic the reference's x86/AVX2 build performs on the
 * GGUF k-quant decode path, in the same fp32 operation order (so that, compiled with
 * the flags in oracle/Makefile, results are bit-identical to the compiled reference).
 * Build: gcc -O2 -mavx2 -mfma -ffp-contract=off -fopenmp (fused multiply-adds are
 * written out as fmaf()/_mm256_fmadd_ps exactly where the reference build has them).
 */
#include "ptm_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int po_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- fp16 <-> fp32 (reference: torch/io/gguf_dequant.h:73-106) ------------------ */
float po_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1f, man = h & 0x3ffu;
    uint32_t bits;
    if (e == 0x1f) {
        bits = sign | 0x7f800000u | (man << 13);
    } else if (e != 0) {
        bits = sign | ((e + 112u) << 23) | (man << 13);
    } else if (man == 0) {
        bits = sign;
    } else { /* subnormal half = man * 2^-24: renormalise */
        const int lz = __builtin_clz(man) - 21; /* shifts needed to bring bit 10 up */
        const uint32_t m2 = (man << lz) & 0x3ffu;
        bits = sign | ((uint32_t)(113 - lz) << 23) | (m2 << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t po_fp32_to_fp16(float f) {
    /* F16C conversion, round-to-nearest-even: what an fp16 KV cache stores. */
    return (uint16_t)_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}

/* ---- 6-bit scale/min unpack (reference: gguf_dequant.h:289-297) ----------------- */
void po_get_scale_min_k4(int j, const uint8_t* q, uint8_t* sc, uint8_t* m) {
    if (j >= 4) {
        *sc = (uint8_t)((q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    } else {
        *sc = q[j] & 0x3f;
        *m = q[j + 4] & 0x3f;
    }
}

static inline float ld_f16(const uint8_t* p) {
    uint16_t b;
    memcpy(&b, p, 2);
    return po_fp16_to_fp32(b);
}

/* ---- dequantisation (reference: gguf_dequant.h:304-341, :395-430) ---------------- */
void po_dequantize_q4_k(const void* src, float* dst, int64_t n) {
    const uint8_t* p = (const uint8_t*)src;
    for (int64_t b = 0; b < n / 256; ++b, p += 144, dst += 256) {
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        for (int sb = 0; sb < 8; ++sb) {
            uint8_t sc, m;
            po_get_scale_min_k4(sb, p + 4, &sc, &m);
            const float ds = d * (float)sc, ms = dmin * (float)m;
            const uint8_t* qs = p + 16 + 32 * (sb >> 1);
            const int shift = (sb & 1) * 4;
            for (int l = 0; l < 32; ++l)
                dst[32 * sb + l] = ds * (float)((qs[l] >> shift) & 0xf) - ms;
        }
    }
}

void po_dequantize_q6_k(const void* src, float* dst, int64_t n) {
    const uint8_t* p = (const uint8_t*)src;
    for (int64_t b = 0; b < n / 256; ++b, p += 210, dst += 256) {
        const int8_t* sc = (const int8_t*)(p + 192);
        const float d = ld_f16(p + 208);
        for (int e = 0; e < 256; ++e) {
            const int half = e >> 7, r = e & 127, grp = r >> 5, l = r & 31;
            const uint8_t lo = p[64 * half + 32 * (grp & 1) + l];
            const uint8_t hi = p[128 + 32 * half + l];
            const int nib = (grp & 2) ? (lo >> 4) : (lo & 0xf);
            const int q = (nib | (((hi >> (2 * grp)) & 3) << 4)) - 32;
            dst[e] = d * (float)sc[8 * half + 2 * grp + (l >> 4)] * (float)q;
        }
    }
}

/* ---- Q8 activation quantiser (reference: cpu_quant_gemv.h:147-198) --------------- */
void po_quantize_x_q8(const float* x, int64_t K, float* d_out, float* sum_out, int8_t* qs) {
    for (int64_t b = 0; b < K / 32; ++b) {
        const float* xb = x + 32 * b;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) {
            const float a = fabsf(xb[i]);
            if (a > amax) amax = a;
        }
        const float d = amax / 127.0f;
        const float id = d > 0.0f ? 1.0f / d : 0.0f;
        int32_t s = 0;
        for (int i = 0; i < 32; ++i) {
            /* cvtps_epi32 under the default MXCSR = round-half-to-even */
            int32_t v = (int32_t)_mm_cvtss_si32(_mm_set_ss(xb[i] * id));
            v = v < -127 ? -127 : (v > 127 ? 127 : v);
            qs[32 * b + i] = (int8_t)v;
            s += v;
        }
        d_out[b] = d;
        sum_out[b] = d * (float)s;
    }
}

/* exact int32 dot of 32 4-bit weights (one nibble plane of 32 bytes) with 32 int8 */
static inline int32_t dot32_nib(const uint8_t* qs, int shift, const int8_t* x8) {
    const __m256i raw = _mm256_loadu_si256((const __m256i*)qs);
    const __m256i nib = _mm256_and_si256(shift ? _mm256_srli_epi16(raw, 4) : raw, _mm256_set1_epi8(0x0f));
    const __m256i xv = _mm256_loadu_si256((const __m256i*)x8);
    const __m256i p32 = _mm256_madd_epi16(_mm256_maddubs_epi16(nib, xv), _mm256_set1_epi16(1));
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(p32), _mm256_extracti128_si256(p32, 1));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4e));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xb1));
    return _mm_cvtsi128_si32(s);
}

void po_q4k_row_isums(const void* row, const int8_t* qs8, int64_t K, int32_t* isum) {
    const uint8_t* p = (const uint8_t*)row;
    for (int64_t b = 0; b < K / 256; ++b, p += 144)
        for (int sb = 0; sb < 8; ++sb)
            isum[8 * b + sb] = dot32_nib(p + 16 + 32 * (sb >> 1), sb & 1, qs8 + 256 * b + 32 * sb);
}

/* One Q4_K row against Q8 x, paired-row formula (reference: cpu_quant_gemv.h:555-671):
 * even sub-blocks accumulate into one chain, odd ones into another, y = a + b.
 * The compiled reference fuses "w*isum - c" into one FMA; the min term is rounded first. */
static float q4k_row_dot(const uint8_t* row, int64_t nblk, const float* xd, const float* xs, const int8_t* xq) {
    float acc[2] = {0.0f, 0.0f};
    for (int64_t b = 0; b < nblk; ++b) {
        const uint8_t* p = row + 144 * b;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        for (int sb = 0; sb < 8; ++sb) {
            uint8_t sc, m;
            po_get_scale_min_k4(sb, p + 4, &sc, &m);
            const int64_t xb = 8 * b + sb;
            const int32_t is = dot32_nib(p + 16 + 32 * (sb >> 1), sb & 1, xq + 32 * xb);
            const float w = d * (float)sc * xd[xb];
            const float c = dmin * (float)m * xs[xb];
            acc[sb & 1] += fmaf(w, (float)is, -c);
        }
    }
    return acc[0] + acc[1];
}

/* Unpaired last row of an odd N (reference: q4k_q8_dot_avx2, cpu_quant_gemv.h:220-296):
 * one chain per super-block, super-block partials added in order. */
static float q4k_row_dot_odd(const uint8_t* row, int64_t nblk, const float* xd, const float* xs, const int8_t* xq) {
    float total = 0.0f;
    for (int64_t b = 0; b < nblk; ++b) {
        const uint8_t* p = row + 144 * b;
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        float sumf = 0.0f;
        for (int sb = 0; sb < 8; ++sb) {
            uint8_t sc, m;
            po_get_scale_min_k4(sb, p + 4, &sc, &m);
            const int64_t xb = 8 * b + sb;
            const int32_t is = dot32_nib(p + 16 + 32 * (sb >> 1), sb & 1, xq + 32 * xb);
            const float w = d * (float)sc * xd[xb];
            const float c = dmin * (float)m * xs[xb];
            sumf += fmaf(w, (float)is, -c);
        }
        total += sumf;
    }
    return total;
}

void po_q4k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const int64_t nb8 = K / 32;
    float* xd = (float*)malloc(sizeof(float) * 2 * nb8);
    float* xs = xd + nb8;
    int8_t* xq = (int8_t*)malloc(K);
    po_quantize_x_q8(x, K, xd, xs, xq);
    const uint8_t* base = (const uint8_t*)W;
    const int64_t n_even = N & ~(int64_t)1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < n_even; ++n)
        y[n] = q4k_row_dot(base + n * stride, K / 256, xd, xs, xq);
    if (N & 1) y[N - 1] = q4k_row_dot_odd(base + (N - 1) * stride, K / 256, xd, xs, xq);
    free(xd);
    free(xq);
}

/* fp32-activation Q4_K (reference scalar path, cpu_quant_gemv.h:689-767): exact-math cross-check */
void po_q4k_gemv_f32(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* p = base + n * stride;
        float dot = 0.0f;
        for (int64_t b = 0; b < K / 256; ++b, p += 144) {
            const float d = ld_f16(p), dmin = ld_f16(p + 2);
            for (int g = 0; g < 4; ++g) {
                uint8_t sc, m;
                po_get_scale_min_k4(2 * g, p + 4, &sc, &m);
                const float d1 = d * (float)sc, m1 = dmin * (float)m;
                po_get_scale_min_k4(2 * g + 1, p + 4, &sc, &m);
                const float d2 = d * (float)sc, m2 = dmin * (float)m;
                const uint8_t* qs = p + 16 + 32 * g;
                const float* xx = x + 256 * b + 64 * g;
                for (int l = 0; l < 32; ++l) {
                    dot = fmaf(fmaf(d1, (float)(qs[l] & 0xf), -m1), xx[l], dot);
                    dot = fmaf(fmaf(d2, (float)(qs[l] >> 4), -m2), xx[32 + l], dot);
                }
            }
        }
        y[n] = dot;
    }
}

static inline float hsum8(__m256 v) { /* (lo+hi) then pairwise, as reference hsum_avx */
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_hadd_ps(s, s);
    s = _mm_hadd_ps(s, s);
    return _mm_cvtss_f32(s);
}

/* eight consecutive 6-bit quants (minus 32) of one Q6_K group as floats */
static inline __m256 q6_group8(const uint8_t* ql, const uint8_t* qh, int grp) {
    const __m256i lo = _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i*)ql));
    const __m256i hi = _mm256_cvtepu8_epi32(_mm_loadl_epi64((const __m128i*)qh));
    const __m256i nib = (grp & 2) ? _mm256_srli_epi32(lo, 4) : _mm256_and_si256(lo, _mm256_set1_epi32(0xf));
    const __m256i two = _mm256_and_si256(_mm256_srli_epi32(hi, 2 * grp), _mm256_set1_epi32(3));
    const __m256i q = _mm256_sub_epi32(_mm256_or_si256(nib, _mm256_slli_epi32(two, 4)), _mm256_set1_epi32(32));
    return _mm256_cvtepi32_ps(q);
}

/* Q6_K GEMV, fp32 activations, 8-lane accumulator (reference: cpu_quant_gemv.h:883-1020) */
void po_q6k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* p = base + n * stride;
        __m256 acc = _mm256_setzero_ps();
        for (int64_t b = 0; b < K / 256; ++b, p += 210) {
            const int8_t* sc = (const int8_t*)(p + 192);
            const float d = ld_f16(p + 208);
            for (int half = 0; half < 2; ++half) {
                const uint8_t* ql = p + 64 * half;
                const uint8_t* qh = p + 128 + 32 * half;
                const float* xx = x + 256 * b + 128 * half;
                for (int l = 0; l < 32; l += 8) {
                    for (int grp = 0; grp < 4; ++grp) {
                        const float s = d * (float)sc[8 * half + 2 * grp + (l >> 4)];
                        const __m256 w = _mm256_mul_ps(_mm256_set1_ps(s), q6_group8(ql + 32 * (grp & 1) + l, qh + l, grp));
                        acc = _mm256_fmadd_ps(w, _mm256_loadu_ps(xx + 32 * grp + l), acc);
                    }
                }
            }
        }
        y[n] = hsum8(acc);
    }
}

/* sequential fp32 Q6_K (reference scalar path, cpu_quant_gemv.h:1024-1078): cross-check */
void po_q6k_gemv_f32(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
    float* row = (float*)malloc(sizeof(float) * K);
    for (int64_t n = 0; n < N; ++n) {
        po_dequantize_q6_k(base + n * stride, row, K);
        double dot = 0.0;
        for (int64_t k = 0; k < K; ++k) dot += (double)row[k] * (double)x[k];
        y[n] = (float)dot;
    }
    free(row);
}

/* ---- the dispatcher's other block formats: Q8_0 (34 B / 32 values), Q5_K (176 B / 256), Q5_0 (22 B / 32) ----------
 * fp32 activations in all three.  The 8-lane sums are written lane by lane: lane i of the reference's vector
 * accumulator sees elements i, i+8, ... of each run of 32, and the lanes meet in the order of its hsum_avx. */
static inline float hsum8_lanes(const float* a) { /* ((a0+a4)+(a1+a5)) + ((a2+a6)+(a3+a7)) */
    const float s0 = a[0] + a[4], s1 = a[1] + a[5], s2 = a[2] + a[6], s3 = a[3] + a[7];
    return (s0 + s1) + (s2 + s3);
}

/* reference: gguf_dequant.h:237-255 */
void po_dequantize_q8_0(const void* src, float* dst, int64_t n) {
    const uint8_t* p = (const uint8_t*)src;
    for (int64_t b = 0; b < n / 32; ++b, p += 34, dst += 32) {
        const float d = ld_f16(p);
        const int8_t* q = (const int8_t*)(p + 2);
        for (int j = 0; j < 32; ++j) dst[j] = d * (float)q[j];
    }
}

/* the 5-bit quant e (0..255) of a Q5_K block: nibble from qs, fifth bit from qh */
static inline int q5k_quant(const uint8_t* p, int e) {
    const int pair = e >> 6, hi = (e >> 5) & 1, l = e & 31;
    const uint8_t b = p[48 + 32 * pair + l];
    const int nib = hi ? (b >> 4) : (b & 0xf);
    return nib + (((p[16 + l] >> (2 * pair + hi)) & 1) ? 16 : 0);
}

/* reference: gguf_dequant.h:348-388 */
void po_dequantize_q5_k(const void* src, float* dst, int64_t n) {
    const uint8_t* p = (const uint8_t*)src;
    for (int64_t b = 0; b < n / 256; ++b, p += 176, dst += 256) {
        const float d = ld_f16(p), dmin = ld_f16(p + 2);
        for (int sb = 0; sb < 8; ++sb) {
            uint8_t sc, m;
            po_get_scale_min_k4(sb, p + 4, &sc, &m);
            const float ds = d * (float)sc, ms = dmin * (float)m;
            for (int l = 0; l < 32; ++l) dst[32 * sb + l] = ds * (float)q5k_quant(p, 32 * sb + l) - ms;
        }
    }
}

/* reference: cpu_quant_gemv.h:784-826 (acc += (d*q) * x per lane, fused) */
void po_q8_0_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* p = base + n * stride;
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int64_t b = 0; b < K / 32; ++b, p += 34) {
            const float d = ld_f16(p);
            const int8_t* q = (const int8_t*)(p + 2);
            for (int l = 0; l < 32; l += 8)
                for (int i = 0; i < 8; ++i) acc[i] = fmaf(d * (float)q[l + i], x[32 * b + l + i], acc[i]);
        }
        y[n] = hsum8_lanes(acc);
    }
}

/* reference: cpu_quant_gemv.h:1091-1185.  Per 32-wide sub-block the lanes first gather sum(q*x) and sum(x), then
 * acc += d_sb * sum(q*x); acc -= m_sb * sum(x), low-nibble sub-block before the high-nibble one of each pair. */
void po_q5k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* p = base + n * stride;
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int64_t b = 0; b < K / 256; ++b, p += 176) {
            const float d = ld_f16(p), dmin = ld_f16(p + 2);
            for (int sb = 0; sb < 8; ++sb) {
                uint8_t sc, m;
                po_get_scale_min_k4(sb, p + 4, &sc, &m);
                const float ds = d * (float)sc, ms = dmin * (float)m;
                const float* xx = x + 256 * b + 32 * sb;
                float qx[8] = {0, 0, 0, 0, 0, 0, 0, 0}, sx[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int l = 0; l < 32; l += 8)
                    for (int i = 0; i < 8; ++i) {
                        qx[i] = fmaf((float)q5k_quant(p, 32 * sb + l + i), xx[l + i], qx[i]);
                        sx[i] = sx[i] + xx[l + i];
                    }
                for (int i = 0; i < 8; ++i) {
                    acc[i] = fmaf(ds, qx[i], acc[i]);
                    acc[i] = fmaf(-ms, sx[i], acc[i]);
                }
            }
        }
        y[n] = hsum8_lanes(acc);
    }
}

/* reference: cpu_quant_gemv.h:1572-1630: one running sum per row, elements j and j+16 of a block alternating;
 * d*q is exact in fp32 (11-bit by 5-bit), and the reference build (g++ -O2 -mfma, contraction on) fuses the
 * multiply by x with the add */
void po_q5_0_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    const uint8_t* base = (const uint8_t*)W;
    for (int64_t n = 0; n < N; ++n) {
        const uint8_t* p = base + n * stride;
        float acc = 0.0f;
        for (int64_t b = 0; b < K / 32; ++b, p += 22) {
            const float d = ld_f16(p);
            uint32_t qh;
            memcpy(&qh, p + 2, 4);
            for (int j = 0; j < 16; ++j) {
                const int q0 = ((p[6 + j] & 0xf) | (((qh >> j) & 1) << 4)) - 16;
                const int q1 = ((p[6 + j] >> 4) | (((qh >> (j + 16)) & 1) << 4)) - 16;
                acc = fmaf(d * (float)q0, x[32 * b + j], acc);
                acc = fmaf(d * (float)q1, x[32 * b + j + 16], acc);
            }
        }
        y[n] = acc;
    }
}

void po_cpu_quant_gemv(uint32_t type, const void* W, const float* x, float* y,
                       int64_t K, int64_t N, int64_t stride) {
    if (type == PO_Q4_K) po_q4k_gemv(W, x, y, K, N, stride);
    else if (type == PO_Q6_K) po_q6k_gemv(W, x, y, K, N, stride);
    else if (type == PO_Q8_0) po_q8_0_gemv(W, x, y, K, N, stride);
    else if (type == PO_Q5_K) po_q5k_gemv(W, x, y, K, N, stride);
    else if (type == PO_Q5_0) po_q5_0_gemv(W, x, y, K, N, stride);
    /* any other type: no-op, as reference cpu_quant_gemv.h:1684-1686 */
}

/* ---- RMSNorm --------------------------------------------------------------------- */
/* sequential-sum variant: the attention-norm fallback taken when q/k/v quant types differ
 * (reference: gguf_model.h:3387-3394) */
void po_rmsnorm_seq(const float* x, const float* gamma, float eps, int add_one, int64_t H, float* out) {
    float ss = 0.0f;
    for (int64_t j = 0; j < H; ++j) ss = fmaf(x[j], x[j], ss);
    const float r = 1.0f / sqrtf(ss / (float)H + eps);
    for (int64_t j = 0; j < H; ++j) out[j] = x[j] * r * (add_one ? 1.0f + gamma[j] : gamma[j]);
}
/* 8-lane variant (reference: cpu_quant_gemv.h:2567-2610 and :2438-2469) */
void po_rmsnorm_vec(const float* x, const float* gamma, float eps, int add_one, int64_t H, float* out) {
    __m256 v = _mm256_setzero_ps();
    int64_t j = 0;
    for (; j + 8 <= H; j += 8) {
        const __m256 a = _mm256_loadu_ps(x + j);
        v = _mm256_fmadd_ps(a, a, v);
    }
    float ss = hsum8(v);
    for (; j < H; ++j) ss = fmaf(x[j], x[j], ss);
    const float r = 1.0f / sqrtf(ss / (float)H + eps);
    for (j = 0; j < H; ++j) out[j] = x[j] * r * (add_one ? 1.0f + gamma[j] : gamma[j]);
}

/* ---- RoPE (reference: hot_loops.cpp:1853-1876, :2035-2061) ----------------------- */
void po_rope_precompute(float* c, float* s, int64_t pos, int64_t head_dim, float base) {
    po_rope_precompute_scaled(c, s, pos, head_dim, base, 1.0f);
}
/* linear position scaling: theta = (pos / scale) * freq when scale is positive and not 1 (hot_loops.cpp:1858-1860) */
void po_rope_precompute_scaled(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale) {
    po_rope_precompute_factors(c, s, pos, head_dim, base, scale, NULL, 1.0f);
}
/* per-frequency factors (phi3 LongRoPE: inv_freq[d] /= factor[d]) and the attention factor that scales cos and sin
 * (hot_loops.cpp:1861-1873) */
void po_rope_precompute_factors(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale,
                                const float* factors, float attn_factor) {
    const float p = (scale > 0.0f && scale != 1.0f) ? (float)pos / scale : (float)pos;
    const int apply_af = attn_factor > 0.0f && attn_factor != 1.0f;
    for (int64_t d = 0; d < head_dim / 2; ++d) {
        float inv = 1.0f / powf(base, 2.0f * (float)d / (float)head_dim);
        if (factors) inv /= factors[d];
        const float th = p * inv;
        float cv = cosf(th), sv = sinf(th);
        if (apply_af) { cv *= attn_factor; sv *= attn_factor; }
        c[d] = cv;
        s[d] = sv;
    }
}
static void rope_neox_head(float* h, const float* c, const float* s, int64_t half) {
    for (int64_t d = 0; d < half; ++d) {
        const float a = h[d], b = h[d + half];
        h[d] = fmaf(a, c[d], -(b * s[d]));
        h[d + half] = fmaf(a, s[d], b * c[d]);
    }
}
void po_rope_apply_neox(float* q, float* k, const float* c, const float* s,
                        int64_t n_heads, int64_t n_kv_heads, int64_t head_dim) {
    for (int64_t h = 0; h < n_heads; ++h) rope_neox_head(q + h * head_dim, c, s, head_dim / 2);
    for (int64_t h = 0; h < n_kv_heads; ++h) rope_neox_head(k + h * head_dim, c, s, head_dim / 2);
}

/* interleaved pairs (2d, 2d+1): the rotation of llama / mistral (reference: rope_apply_fused, hot_loops.cpp:1962-2030;
 * the reference build contracts x0*c - x1*s and x0*s + x1*c into one fused multiply-add each, as below) */
static void rope_norm_head(float* h, const float* c, const float* s, int64_t half) {
    for (int64_t d = 0; d < half; ++d) {
        const float a = h[2 * d], b = h[2 * d + 1];
        h[2 * d] = fmaf(a, c[d], -(b * s[d]));
        h[2 * d + 1] = fmaf(a, s[d], b * c[d]);
    }
}
void po_rope_apply_norm(float* q, float* k, const float* c, const float* s,
                        int64_t n_heads, int64_t n_kv_heads, int64_t head_dim) {
    for (int64_t h = 0; h < n_heads; ++h) rope_norm_head(q + h * head_dim, c, s, head_dim / 2);
    for (int64_t h = 0; h < n_kv_heads; ++h) rope_norm_head(k + h * head_dim, c, s, head_dim / 2);
}

/* ---- vector exp (reference: VectorizedOps.h:56-97; Cephes polynomial) ------------ */
static inline __m256 exp8(__m256 x) {
    x = _mm256_max_ps(_mm256_min_ps(x, _mm256_set1_ps(88.3762626647949f)), _mm256_set1_ps(-88.3762626647949f));
    const __m256 n = _mm256_round_ps(_mm256_mul_ps(x, _mm256_set1_ps(1.44269504088896341f)),
                                     _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
    /* the reference build fuses both "x - n*c" steps of the range reduction */
    x = _mm256_fnmadd_ps(n, _mm256_set1_ps(0.693359375f), x);
    x = _mm256_fnmadd_ps(n, _mm256_set1_ps(-2.12194440e-4f), x);
    static const float coef[5] = {1.3981999507E-3f, 8.3334519073E-3f, 4.1665795894E-2f,
                                  1.6666665459E-1f, 5.0000001201E-1f};
    __m256 y = _mm256_set1_ps(1.9875691500E-4f);
    for (int i = 0; i < 5; ++i) y = _mm256_fmadd_ps(y, x, _mm256_set1_ps(coef[i]));
    y = _mm256_fmadd_ps(y, _mm256_mul_ps(x, x), _mm256_add_ps(x, _mm256_set1_ps(1.0f)));
    const __m256i e = _mm256_slli_epi32(_mm256_add_epi32(_mm256_cvtps_epi32(n), _mm256_set1_epi32(127)), 23);
    return _mm256_mul_ps(y, _mm256_castsi256_ps(e));
}
void po_exp256(const float* in, float* out, int64_t n8) {
    for (int64_t i = 0; i < n8; ++i) _mm256_storeu_ps(out + 8 * i, exp8(_mm256_loadu_ps(in + 8 * i)));
}

/* ---- single-token attention for one head (reference: gguf_model.h:3510-3636) ----- */
void po_attn_head(const float* q, const float* k, const float* v, int64_t T, int64_t kv_dim,
                  int64_t head_dim, float scale, float* sc, float* out) {
    po_attn_head_window(q, k, v, T, 0, kv_dim, head_dim, scale, sc, out);
}
/* positions before t_start are masked the way the reference masks them (gguf_model.h:3528-3530): their scores are
 * -inf and every loop still runs over [0, T), so the 8-wide groups of the softmax keep their alignment */
void po_attn_head_window(const float* q, const float* k, const float* v, int64_t T, int64_t t_start, int64_t kv_dim,
                         int64_t head_dim, float scale, float* sc, float* out) {
    for (int64_t t = 0; t < t_start; ++t) sc[t] = -INFINITY;
    for (int64_t t = t_start; t < T; ++t) {
        const float* kt = k + t * kv_dim;
        __m256 a = _mm256_setzero_ps();
        int64_t d = 0;
        for (; d + 8 <= head_dim; d += 8) a = _mm256_fmadd_ps(_mm256_loadu_ps(q + d), _mm256_loadu_ps(kt + d), a);
        float dot = hsum8(a);
        for (; d < head_dim; ++d) dot = fmaf(q[d], kt[d], dot);
        sc[t] = dot * scale;
    }
    float mx = sc[0];
    for (int64_t t = 1; t < T; ++t) if (sc[t] > mx) mx = sc[t];
    __m256 vs = _mm256_setzero_ps();
    const __m256 vm = _mm256_set1_ps(mx);
    int64_t t = 0;
    for (; t + 8 <= T; t += 8) {
        const __m256 e = exp8(_mm256_sub_ps(_mm256_loadu_ps(sc + t), vm));
        _mm256_storeu_ps(sc + t, e);
        vs = _mm256_add_ps(vs, e);
    }
    float sum = hsum8(vs); /* same association as the reference's hsum_avx2 */
    for (; t < T; ++t) {
        sc[t] = expf(sc[t] - mx);
        sum += sc[t];
    }
    const float inv = 1.0f / (sum + 1e-10f);
    for (t = 0; t < T; ++t) sc[t] *= inv;
    for (int64_t d = 0; d < head_dim; ++d) out[d] = 0.0f;
    for (t = 0; t < T; ++t) {
        const float* vt = v + t * kv_dim;
        const float w = sc[t];
        for (int64_t d = 0; d < head_dim; ++d) out[d] = fmaf(w, vt[d], out[d]);
    }
}

/* ---- SiLU(gate)*up in place (reference: gguf_model.h:3728-3763) ------------------ */
/* tanh-approximated GELU times up (gguf_model.h:3730-3738): the expression as written there, libm tanhf */
void po_gelu_mul(float* gate, const float* up, int64_t n) {
    for (int64_t j = 0; j < n; ++j) {
        const float g = gate[j];
        const float c = 0.7978845608028654f;
        const float x3 = g * g * g;
        const float t = tanhf(c * (g + 0.044715f * x3));
        gate[j] = 0.5f * g * (1.0f + t) * up[j];
    }
}
void po_silu_mul(float* gate, const float* up, int64_t n) {
    int64_t j = 0;
    for (; j + 8 <= n; j += 8) {
        for (int i = 0; i < 8; ++i) {
            const float g = gate[j + i];
            float ng = 0.0f - g;
            ng = ng < -88.0f ? -88.0f : ng; /* max_ps(neg_g,-88) then min_ps(.,88) */
            ng = ng > 88.0f ? 88.0f : ng;
            const float sig = 1.0f / (1.0f + expf(ng));
            gate[j + i] = (g * sig) * up[j + i];
        }
    }
    for (; j < n; ++j) {
        const float g = gate[j];
        gate[j] = (g / (1.0f + expf(-g))) * up[j];
    }
}

/* ---- greedy argmax: strict '>', lowest index wins (reference: gguf_model.h:7662-7671) */
int64_t po_argmax(const float* x, int64_t n) {
    int64_t best = 0;
    float bv = x[0];
    for (int64_t j = 1; j < n; ++j)
        if (x[j] > bv) { bv = x[j]; best = j; }
    return best;
}

/* ---- one decode step (reference: gguf_model.h:3222-3893, Q4_K_M branch choices) -- */
static void qgemv(const po_qweight* w, const float* x, float* y) {
    po_cpu_quant_gemv(w->type, w->data, x, y, w->cols, w->rows, w->stride);
}

int64_t po_decode_step(po_model* m, int64_t token, float* logits, float* hidden_out) {
    return po_decode_step_trace(m, token, logits, hidden_out, NULL);
}

/* trace (optional): [n_layers][2][hidden], the residual stream after each layer's attention branch and after its
 * feed-forward branch (what the reference prints under PT_DUMP_HIDDEN, gguf_model.h:3268-3289) */
int64_t po_decode_step_trace(po_model* m, int64_t token, float* logits, float* hidden_out, float* trace) {
    const int64_t H = m->hidden, hd = m->head_dim, nh = m->n_heads, nkv = m->n_kv_heads;
    const int64_t qd = nh * hd, kvd = nkv * hd, inter = m->inter, past = m->seq_len, T = past + 1;
    float* buf = (float*)malloc(sizeof(float) * (4 * H + 2 * qd + 2 * kvd + 2 * inter));
    float *x = buf, *xn = x + H, *hb = xn + H, *x2 = hb + H, *qb = x2 + H, *ab = qb + qd,
          *kb = ab + qd, *vb = kb + kvd, *gb = vb + kvd, *ub = gb + inter;
    if (m->embedding) memcpy(x, m->embedding + token * H, sizeof(float) * H);
    else po_dequantize_q6_k((const uint8_t*)m->lm_head.data + token * m->lm_head.stride, x, H);

    if (m->scale_embeddings) { /* gguf_model.h:3252-3265 */
        const float es = sqrtf((float)H);
        for (int64_t j = 0; j < H; ++j) x[j] *= es;
    }

    float rc[256], rs[256];
    const float scale = 1.0f / sqrtf((float)hd);

    for (int64_t li = 0; li < m->n_layers; ++li) {
        po_layer* L = &m->layers[li];
        /* local (sliding-window) layers have their own rotation base and window start (gguf_model.h:265-302, :3490-3500) */
        const int global = m->swa_window <= 0 || m->swa_pattern <= 0 || ((li + 1) % m->swa_pattern) == 0;
        /* ModelConfig::rope_factors_for(past_len + 1), gguf_model.h:285-296: the short factors up to the original context */
        const float* factors = m->rope_orig_ctx <= 0 ? NULL : (past + 1 <= m->rope_orig_ctx ? m->rope_factors_short : m->rope_factors_long);
        po_rope_precompute_factors(rc, rs, past, hd, global ? m->rope_base : m->rope_swa_base, global ? m->rope_scale : 1.0f,
                                   factors, m->rope_attn_factor);
        const int64_t t_start = (!global && T > m->swa_window) ? T - m->swa_window : 0;
        const int fuse_qkv = L->q.type == L->k.type && L->q.type == L->v.type;
        if (fuse_qkv) po_rmsnorm_vec(x, L->attn_norm, m->eps, 0, H, xn);
        else po_rmsnorm_seq(x, L->attn_norm, m->eps, 0, H, xn);
        qgemv(&L->q, xn, qb);
        qgemv(&L->k, xn, kb);
        qgemv(&L->v, xn, vb);
        if (L->q_bias) { /* gguf_model.h:3413-3438: one fp32 add per element, before the per-head norm */
            for (int64_t j = 0; j < qd; ++j) qb[j] += L->q_bias[j];
            for (int64_t j = 0; j < kvd; ++j) { kb[j] += L->k_bias[j]; vb[j] += L->v_bias[j]; }
        }
        if (L->q_norm) { /* QK-norm only where the model has it (gguf_model.h:3441-3450) */
            for (int64_t h = 0; h < nh; ++h) po_rmsnorm_vec(qb + h * hd, L->q_norm, m->eps, 0, hd, qb + h * hd);
            for (int64_t h = 0; h < nkv; ++h) po_rmsnorm_vec(kb + h * hd, L->k_norm, m->eps, 0, hd, kb + h * hd);
        }
        if (m->rope_interleaved) po_rope_apply_norm(qb, kb, rc, rs, nh, nkv, hd); /* gguf_model.h:3464-3470 */
        else po_rope_apply_neox(qb, kb, rc, rs, nh, nkv, hd);
        float* kc = L->k_cache + past * kvd;
        float* vc = L->v_cache + past * kvd;
        for (int64_t j = 0; j < kvd; ++j) {
            kc[j] = m->kv_fp16 ? po_fp16_to_fp32(po_fp32_to_fp16(kb[j])) : kb[j];
            vc[j] = m->kv_fp16 ? po_fp16_to_fp32(po_fp32_to_fp16(vb[j])) : vb[j];
        }
#pragma omp parallel
        {
            float* sc = (float*)malloc(sizeof(float) * (T + 8));
#pragma omp for schedule(static)
            for (int64_t h = 0; h < nh; ++h) {
                const int64_t kvh = h / (nh / nkv);
                po_attn_head_window(qb + h * hd, L->k_cache + kvh * hd, L->v_cache + kvh * hd, T, t_start, kvd, hd,
                                    scale, sc, ab + h * hd);
            }
            free(sc);
        }
        qgemv(&L->o, ab, hb);
        if (L->post_attn_norm) po_rmsnorm_vec(hb, L->post_attn_norm, m->eps, 0, H, hb); /* gguf_model.h:3656-3663 */
        for (int64_t j = 0; j < H; ++j) x2[j] = x[j] + hb[j];
        if (trace) memcpy(trace + (2 * li) * H, x2, sizeof(float) * H);
        po_rmsnorm_vec(x2, L->ffn_norm, m->eps, 0, H, xn);
        qgemv(&L->gate, xn, gb);
        qgemv(&L->up, xn, ub);
        if (m->ffn_gelu) po_gelu_mul(gb, ub, inter);
        else po_silu_mul(gb, ub, inter);
        qgemv(&L->down, gb, hb);
        if (L->post_ffn_norm) po_rmsnorm_vec(hb, L->post_ffn_norm, m->eps, 0, H, hb); /* gguf_model.h:3787-3791 */
        for (int64_t j = 0; j < H; ++j) x[j] = x2[j] + hb[j];
        if (trace) memcpy(trace + (2 * li + 1) * H, x, sizeof(float) * H);
    }
    po_rmsnorm_vec(x, m->out_norm, m->eps, 0, H, xn);
    if (hidden_out) memcpy(hidden_out, xn, sizeof(float) * H);
    qgemv(&m->lm_head, xn, logits);
    m->seq_len += 1;
    const int64_t best = po_argmax(logits, m->vocab);
    free(buf);
    return best;
}

/* ================================================================================================
 * Sampling
 * ================================================================================================ */
/* mt19937 (Matsumoto & Nishimura), the engine behind std::mt19937; the reference's sampler owns a
 * function-local `static std::mt19937 rng(42)` (gguf_model.h:7740) */
void po_mt19937_seed(po_mt19937* g, uint32_t seed) {
    g->mt[0] = seed;
    for (int i = 1; i < 624; ++i) g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
    g->idx = 624;
}
uint32_t po_mt19937_next(po_mt19937* g) {
    if (g->idx >= 624) {
        for (int i = 0; i < 624; ++i) {
            const uint32_t y = (g->mt[i] & 0x80000000u) | (g->mt[(i + 1) % 624] & 0x7fffffffu);
            g->mt[i] = g->mt[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        g->idx = 0;
    }
    uint32_t y = g->mt[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}
/* libstdc++ generate_canonical<float, 24> over a 32-bit engine: one draw, float(draw) / float(2^32), and a
 * quotient that rounds up to 1 is replaced by the largest float below 1 (bits/random.tcc) */
float po_uniform01(po_mt19937* g) {
    const float sum = (float)po_mt19937_next(g);
    float r = sum / 4294967296.0f;
    if (r >= 1.0f) r = nextafterf(1.0f, 0.0f);
    return r;
}

/* gguf_model.h:4926-4938: once per generated token, duplicates included */
void po_repetition_penalty(float* logits, int64_t vocab, const int32_t* generated, int64_t n, float penalty) {
    if (!(penalty > 1.0f)) return;
    for (int64_t i = 0; i < n; ++i) {
        const int32_t t = generated[i];
        if (t >= 0 && t < vocab) {
            if (logits[t] > 0) logits[t] /= penalty;
            else logits[t] *= penalty;
        }
    }
}

typedef struct { float p; int32_t idx; } po_pi;
static int po_pi_desc(const void* a, const void* b) {
    const po_pi* x = (const po_pi*)a; const po_pi* y = (const po_pi*)b;
    if (x->p > y->p) return -1;
    if (x->p < y->p) return 1;
    return x->idx < y->idx ? -1 : (x->idx > y->idx ? 1 : 0); /* the reference's std::sort leaves ties unordered */
}
static int po_float_desc(const void* a, const void* b) {
    const float x = *(const float*)a, y = *(const float*)b;
    return x > y ? -1 : (x < y ? 1 : 0);
}

/* gguf_model.h:7658-7751 */
int32_t po_sample_token(const float* logits, int64_t vocab, float temperature, int top_k, float top_p, float r,
                        float* probs_out, float* gap_out) {
    if (gap_out) *gap_out = 1.0f;
    if (temperature < 1e-6f) { /* :7662-7673 greedy */
        const int32_t best = (int32_t)po_argmax(logits, vocab);
        if (probs_out) { memset(probs_out, 0, sizeof(float) * (size_t)vocab); probs_out[best] = 1.0f; }
        return best;
    }
    float* probs = (float*)malloc(sizeof(float) * (size_t)vocab);
    for (int64_t i = 0; i < vocab; ++i) probs[i] = logits[i] / temperature; /* :7677-7679 */
    if (top_k > 0 && top_k < vocab) { /* :7682-7691: below the k-th largest value -> -1e9 (ties at it stay) */
        float* sorted = (float*)malloc(sizeof(float) * (size_t)vocab);
        memcpy(sorted, probs, sizeof(float) * (size_t)vocab);
        qsort(sorted, (size_t)vocab, sizeof(float), po_float_desc);
        const float threshold = sorted[top_k - 1];
        free(sorted);
        for (int64_t i = 0; i < vocab; ++i)
            if (probs[i] < threshold) probs[i] = -1e9f;
    }
    float max_val = probs[0]; /* :7694-7703 softmax, sums in index order */
    for (int64_t i = 1; i < vocab; ++i) if (probs[i] > max_val) max_val = probs[i];
    float sum_exp = 0.0f;
    for (int64_t i = 0; i < vocab; ++i) { probs[i] = expf(probs[i] - max_val); sum_exp += probs[i]; }
    float inv_sum = 1.0f / sum_exp;
    for (int64_t i = 0; i < vocab; ++i) probs[i] *= inv_sum;
    if (top_p < 1.0f) { /* :7706-7736 nucleus: descending until the running sum reaches top_p, then renormalise */
        po_pi* sorted = (po_pi*)malloc(sizeof(po_pi) * (size_t)vocab);
        int64_t m = 0;
        for (int64_t i = 0; i < vocab; ++i)
            if (probs[i] > 1e-10f) { sorted[m].p = probs[i]; sorted[m].idx = (int32_t)i; ++m; }
        qsort(sorted, (size_t)m, sizeof(po_pi), po_pi_desc);
        uint8_t* keep = (uint8_t*)calloc((size_t)vocab, 1);
        float cumsum = 0.0f;
        for (int64_t j = 0; j < m; ++j) {
            keep[sorted[j].idx] = 1;
            cumsum += sorted[j].p;
            if (cumsum >= top_p) break;
        }
        for (int64_t i = 0; i < vocab; ++i) if (!keep[i]) probs[i] = 0.0f;
        sum_exp = 0.0f;
        for (int64_t i = 0; i < vocab; ++i) sum_exp += probs[i];
        if (sum_exp > 0) {
            inv_sum = 1.0f / sum_exp;
            for (int64_t i = 0; i < vocab; ++i) probs[i] *= inv_sum;
        }
        free(keep);
        free(sorted);
    }
    if (probs_out) memcpy(probs_out, probs, sizeof(float) * (size_t)vocab);
    int32_t chosen = (int32_t)(vocab - 1); /* :7739-7750 inverse CDF in index order */
    float cumsum = 0.0f, lo = 0.0f, gap = 1.0f;
    for (int64_t i = 0; i < vocab; ++i) {
        lo = cumsum;
        cumsum += probs[i];
        if (cumsum >= r) {
            chosen = (int32_t)i;
            gap = fminf(cumsum - r, r - lo);
            break;
        }
    }
    if (gap_out) *gap_out = gap;
    free(probs);
    return chosen;
}
