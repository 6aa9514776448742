// Token sampling on the device: repetition penalty, temperature, top-k, softmax, top-p, inverse-CDF draw.
//
// The reference samples on the host (GGUFModel::sample_token, torch/io/gguf_model.h:7658-7751; the penalty loop
// of generate(), :4926-4938; PromeServe's decode loop, promeserve/api_handlers.h:861-876) and so copies the whole
// logit row (608 KB for a 151 936-token vocabulary) to the host every token.  Here only the chosen id leaves the GPU.
//
// Semantics kept from the reference, in its order:
//   x_i = logit_i, divided (x > 0) or multiplied (x <= 0) by the penalty once per earlier occurrence of token i;
//   x_i /= temperature; everything below the k-th largest x (duplicates counted, ties at it kept) is dropped;
//   p = softmax(x) with sums taken in index order; top-p: tokens in descending p until the running sum reaches
//   top_p, renormalised; the token is the first index whose running sum of p (index order) reaches the uniform
//   draw r (index 0 when r <= 0, the last index when the sum never gets there).
//   temperature < 1e-6: argmax (strict '>', lowest index) of the penalised logits.
// Exact selection of the k-th largest x: a three-level radix select over the order-preserving integer image of x
// (11 + 11 + 10 bits: one histogram pass over the vocabulary per level), then a gather of everything at or above
// the threshold (<= SAMPLER_MAX_CAND, normally exactly k) and ONE workgroup that finishes on that short list,
// doing the reference's sequential fp32 sums in the reference's order (so results differ from the CPU's only
// through expf's last bit).
#include "ptm_common.h"

#include <random>

namespace ptm {

enum { SAMPLER_MAX_CAND = 2048, SAMPLER_MAX_TOPK = 1024, SAMPLER_ELEMS_PER_WG = 512 };

// workspace layout (uint32 words)
enum {
    SW_HIST0 = 0,                 // 2048 bins: key >> 21
    SW_HIST1 = 2048,              // 2048 bins: (key >> 10) & 0x7ff among keys of the level-0 bin
    SW_HIST2 = 4096,              // 1024 bins: key & 0x3ff among keys of the level-1 bin
    SW_COUNT = 5120,              // number of gathered candidates
    SW_CAND_KEY = 5128,           // [SAMPLER_MAX_CAND]
    SW_CAND_IDX = SW_CAND_KEY + SAMPLER_MAX_CAND,
    // the wide path (top-k off or beyond SAMPLER_MAX_TOPK): scalars, and a 2048-bin 64-bit mass histogram that shares the
    // candidate arrays (the two paths never run in the same call)
    SW_WIDE = SW_CAND_IDX + SAMPLER_MAX_CAND,
    SW_MASS_HIST = SW_CAND_KEY,
    SW_WORDS = SW_WIDE + 64,
    SW_CLEAR_WORDS = SW_COUNT + 8
};
// wide-path scalars (32-bit words from SW_WIDE): top-k threshold key, largest kept key, sum of exp (64-bit, 2^-32 units),
// probability mass above the current prefix (64-bit, 2^-40 units), key prefix chosen so far, 1 when every eligible token stays
// the narrow path's hand-over to its overflow kernel: 1 when more candidates tied at the threshold than the list holds, and the
// threshold key itself (outside the words the wide threshold kernel zeroes)
enum { WS_THR = 0, WS_MAXKEY = 1, WS_SUMEXP = 2, WS_MASS_ABOVE = 4, WS_PREFIX = 6, WS_KEEP_ALL = 7, WS_TSTAR = 8, WS_NTIE = 9,
       WS_OVERFLOW = 16, WS_THR_SAVE = 17 };

struct SamplerArgs {
    const float* logits;
    const int32_t* counts;          // occurrences of each token so far, or NULL
    int vocab;
    const ptm_sampling* d_params;   // device copy, or NULL: use `params`
    ptm_sampling params;
    uint32_t* ws;
};

__device__ __forceinline__ ptm_sampling sampler_params(const SamplerArgs& a) { return a.d_params ? *a.d_params : a.params; }

// float -> uint32 whose unsigned order is the float order
__device__ __forceinline__ uint32_t order_key(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// the value the selection runs on: penalised logit, over temperature unless greedy
__device__ __forceinline__ float sampler_value(const SamplerArgs& a, const ptm_sampling& p, int i) {
    float x = a.logits[i];
    if (a.counts && p.repeat_penalty > 1.0f) {
        const int c = a.counts[i];
        for (int n = 0; n < c; ++n) x = x > 0.0f ? x / p.repeat_penalty : x * p.repeat_penalty;
    }
    if (p.temperature >= 1e-6f) x = x / p.temperature;
    return x + 0.0f;  // -0 -> +0: the reference compares values, the radix select compares bit patterns
}
// value of lane i (i uniform over the wave): v_readlane, no LDS round trip
__device__ __forceinline__ float lane_f(float v, int i) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i)); }
__device__ __forceinline__ uint32_t lane_u(uint32_t v, int i) { return (uint32_t)__builtin_amdgcn_readlane((int)v, i); }

__device__ __forceinline__ int sampler_k(const ptm_sampling& p) { return p.temperature >= 1e-6f ? p.top_k : 1; }

// Which bin, counting from the top, holds the k-th largest key?  All 256 threads call it; returns the bin and how
// many keys are still wanted inside it.  s_scan: 8 words of LDS.  (Wave-level prefix sums: two barriers per call.)
__device__ void select_bin(const uint32_t* hist, int nbins, int k, int& bin, int& k_in_bin, uint32_t* s_scan) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, per = nbins / 256;
    uint32_t mine = 0;
    for (int j = 0; j < per; ++j) mine += hist[nbins - 1 - (tid * per + j)];
    uint32_t incl = mine;  // inclusive prefix sum over the wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t up = __shfl_up(incl, off, 64);
        if (lane >= off) incl += up;
    }
    __syncthreads();  // s_scan may still be read by the previous call
    if (lane == 63) s_scan[wave] = incl;
    __syncthreads();
    for (int w = 0; w < wave; ++w) incl += s_scan[w];
    const uint32_t excl = incl - mine;
    if (excl < (uint32_t)k && (uint32_t)k <= incl) {  // exactly one thread: the counts sum to at least k
        uint32_t above = excl;
        for (int j = 0; j < per; ++j) {
            const int b = nbins - 1 - (tid * per + j);
            const uint32_t h = hist[b];
            if (above + h >= (uint32_t)k) {
                s_scan[4] = (uint32_t)b;
                s_scan[5] = (uint32_t)k - above;
                break;
            }
            above += h;
        }
    }
    __syncthreads();
    bin = (int)s_scan[4];
    k_in_bin = (int)s_scan[5];
}

__global__ __launch_bounds__(256) void sampler_clear_kernel(uint32_t* ws) {
    for (int i = threadIdx.x + blockIdx.x * 256; i < SW_CLEAR_WORDS; i += 256 * gridDim.x) ws[i] = 0;
}

// LEVEL 0/1/2: histogram of the level's bits among the keys that share the prefix chosen by the levels above
template <int LEVEL>
__global__ __launch_bounds__(256) void sampler_hist_kernel(SamplerArgs a) {
    constexpr int NB = LEVEL == 2 ? 1024 : 2048;
    __shared__ uint32_t s_hist[NB];
    __shared__ uint32_t s_scan[8];
    const int tid = threadIdx.x;
    const ptm_sampling p = sampler_params(a);
    int b0 = 0, b1 = 0, k = sampler_k(p);
    if (LEVEL >= 1) select_bin(a.ws + SW_HIST0, 2048, k, b0, k, s_scan);
    if (LEVEL >= 2) select_bin(a.ws + SW_HIST1, 2048, k, b1, k, s_scan);
    for (int i = tid; i < NB; i += 256) s_hist[i] = 0;
    __syncthreads();
    const int base = blockIdx.x * SAMPLER_ELEMS_PER_WG;
#pragma unroll
    for (int u = 0; u < SAMPLER_ELEMS_PER_WG / 256; ++u) {
        const int i = base + tid + 256 * u;
        const bool in = i < a.vocab;
        const uint32_t key = in ? order_key(sampler_value(a, p, i)) : 0u;
        if (LEVEL == 0) {
            if (in) atomicAdd(&s_hist[key >> 21], 1u);
        } else if (in) {
            if (LEVEL == 1) { if ((int)(key >> 21) == b0) atomicAdd(&s_hist[(key >> 10) & 0x7ffu], 1u); }
            else { if ((key >> 10) == (((uint32_t)b0 << 11) | (uint32_t)b1)) atomicAdd(&s_hist[key & 0x3ffu], 1u); }
        }
    }
    __syncthreads();
    uint32_t* g = a.ws + (LEVEL == 0 ? SW_HIST0 : LEVEL == 1 ? SW_HIST1 : SW_HIST2);
    for (int i = tid; i < NB; i += 256)
        if (s_hist[i]) atomicAdd(&g[i], s_hist[i]);
}

// every key at or above the k-th largest goes to the candidate list (order of arrival; the finish kernel sorts)
__global__ __launch_bounds__(256) void sampler_gather_kernel(SamplerArgs a) {
    __shared__ uint32_t s_scan[8];
    const int tid = threadIdx.x;
    const ptm_sampling p = sampler_params(a);
    int b0, b1, b2, k = sampler_k(p);
    select_bin(a.ws + SW_HIST0, 2048, k, b0, k, s_scan);
    select_bin(a.ws + SW_HIST1, 2048, k, b1, k, s_scan);
    select_bin(a.ws + SW_HIST2, 1024, k, b2, k, s_scan);
    const uint32_t threshold = ((uint32_t)b0 << 21) | ((uint32_t)b1 << 10) | (uint32_t)b2;
    if (blockIdx.x == 0 && tid == 0) a.ws[SW_WIDE + WS_THR_SAVE] = threshold;   // for the overflow kernel
    const int base = blockIdx.x * SAMPLER_ELEMS_PER_WG;
#pragma unroll
    for (int u = 0; u < SAMPLER_ELEMS_PER_WG / 256; ++u) {
        const int i = base + tid + 256 * u;
        if (i < a.vocab) {
            const uint32_t key = order_key(sampler_value(a, p, i));
            if (key >= threshold) {
                const uint32_t slot = atomicAdd(&a.ws[SW_COUNT], 1u);
                if (slot < SAMPLER_MAX_CAND) {
                    a.ws[SW_CAND_KEY + slot] = key;
                    a.ws[SW_CAND_IDX + slot] = (uint32_t)i;
                }
            }
        }
    }
}

// in-LDS bitonic sort of n (power of two) 64-bit keys, ascending, by 1024 threads
__device__ void bitonic_sort_u64(unsigned long long* v, int n) {
    for (int size = 2; size <= n; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = threadIdx.x; t < n / 2; t += 1024) {
                const int lo = (t / stride) * 2 * stride + (t % stride), hi = lo + stride;
                const bool up = ((lo & size) == 0);
                const unsigned long long x = v[lo], y = v[hi];
                if ((x > y) == up) { v[lo] = y; v[hi] = x; }
            }
        }
    __syncthreads();
}

struct SamplerOut {
    int64_t* out_token;       // chosen id
    const float* uniforms;    // r of step s is uniforms[s]
    const int* d_step;        // NULL: s = 0
    int32_t* counts_rw;       // NULL, or the occurrence counts to bump for the chosen token
    ArgmaxAdvance adv;        // step bookkeeping of the decode loop (all NULL outside it)
    int leave_clean;          // zero the histograms and the candidate count for the next call (it then skips its clear launch)
};

// what the last thread of a draw does with the chosen id: result, occurrence count, the decode loop's step bookkeeping
__device__ __forceinline__ void sampler_publish(const SamplerOut& o, int token, int step, int64_t past_now) {
    if (o.out_token) *o.out_token = token;
    if (o.counts_rw) o.counts_rw[token] += 1;
    if (o.adv.d_step) {
        if (step < o.adv.cap) o.adv.tokens_out[step] = token;
        *o.adv.d_token = token;
        *o.adv.d_past = past_now + 1;
        *o.adv.d_step = step + 1;
    }
}

__global__ __launch_bounds__(1024) void sampler_finish_kernel(SamplerArgs a, SamplerOut o) {
    __shared__ unsigned long long s_sort[SAMPLER_MAX_CAND];   // 16 KB
    __shared__ float s_p[SAMPLER_MAX_CAND];                   // x, then p, in index order
    __shared__ uint32_t s_idx[SAMPLER_MAX_CAND];
    __shared__ uint8_t s_keep[SAMPLER_MAX_CAND];
    const int tid = threadIdx.x;
    // every load whose address is known goes out first, in one round trip; the draw follows as soon as the step is known
    const ptm_sampling p = sampler_params(a);
    const uint32_t total = a.ws[SW_COUNT];
    const uint32_t key0 = a.ws[SW_CAND_KEY + (tid & 63)], idx0 = a.ws[SW_CAND_IDX + (tid & 63)];
    const int step = o.d_step ? *o.d_step : 0;
    const int64_t past_now = o.adv.d_past ? *o.adv.d_past : 0;
    const float r_draw = o.uniforms[step];
    if (total > SAMPLER_MAX_CAND) {
        // more logits tie at the threshold than the candidate list holds: the kernel behind this one (sampler_overflow_kernel)
        // draws from the whole vocabulary instead and publishes the token
        if (tid == 0) a.ws[SW_WIDE + WS_OVERFLOW] = 1u;
        if (o.leave_clean) for (int i = tid; i < SW_CLEAR_WORDS; i += 1024) a.ws[i] = 0;
        return;
    }
    const int m = (int)total;
    if (m <= 64) {
        // The usual case (k candidates, k <= 64): one wave, one candidate per lane, no workgroup barrier.  Order by
        // counting, sequential sums by reading lane after lane -- the same additions in the same order as below.
        if (tid >= 64) {
            if (o.leave_clean) for (int i = tid - 64; i < SW_CLEAR_WORDS; i += 1024 - 64) if (i != SW_COUNT) a.ws[i] = 0;
            return;
        }
        const int lane = tid;
        const bool valid = lane < m;
        const uint32_t key = valid ? key0 : 0u, idx = valid ? idx0 : 0xffffffffu;
        int rank = 0;
        for (int j = 0; j < m; ++j) rank += lane_u(idx, j) < idx;
        if (valid) { s_idx[rank] = idx; s_p[rank] = key_value(key); }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t id = valid ? s_idx[lane] : 0u;   // index order from here on
        const float x = valid ? s_p[lane] : -INFINITY;
        const bool greedy = !(p.temperature >= 1e-6f);
        int token = a.vocab - 1;
        if (greedy) {
            token = (int)lane_u(id, 0);
        } else {
            const float mx = max64(x);
            const float e = valid ? expf(x - mx) : 0.0f;
            float sum = 0.0f;
            for (int i = 0; i < m; ++i) sum += lane_f(e, i);
            float pr = e * (1.0f / sum);
            if (p.top_p < 1.0f) {
                const bool elig = valid && pr > 1e-10f;
                int r2 = 0, n_elig = 0;
                for (int j = 0; j < m; ++j) {
                    const float pj = lane_f(pr, j);
                    const bool ej = pj > 1e-10f;
                    n_elig += ej;
                    r2 += ej && (pj > pr || (pj == pr && j < lane));
                }
                float* s_q = reinterpret_cast<float*>(s_sort);
                if (elig) s_q[r2] = pr;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const float q = lane < n_elig ? s_q[lane] : 0.0f;
                float cum = 0.0f;
                int n_keep = n_elig;
                for (int k = 0; k < n_elig; ++k) {
                    cum += lane_f(q, k);
                    if (cum >= p.top_p) { n_keep = k + 1; break; }
                }
                pr = (elig && r2 < n_keep) ? pr : 0.0f;
                float s2 = 0.0f;
                for (int i = 0; i < m; ++i) s2 += lane_f(pr, i);
                if (s2 > 0.0f) pr *= 1.0f / s2;
            }
            const float r = r_draw;
            if (r <= 0.0f) {
                token = 0;
            } else {
                float cum = 0.0f;
                for (int i = 0; i < m; ++i) {
                    cum += lane_f(pr, i);
                    if (cum >= r) { token = (int)lane_u(id, i); break; }
                }
            }
        }
        if (lane == 0) {
            if (o.out_token) *o.out_token = token;
            if (o.counts_rw) atomicAdd(&o.counts_rw[token], 1);  // no value needed back: nothing waits for it
            if (o.adv.d_step) {
                if (step < o.adv.cap) o.adv.tokens_out[step] = token;
                *o.adv.d_token = token;
                *o.adv.d_past = past_now + 1;
                *o.adv.d_step = step + 1;
            }
            if (o.leave_clean) a.ws[SW_COUNT] = 0;
            a.ws[SW_WIDE + WS_OVERFLOW] = 0u;
        }
        return;
    }
    int n = 1;
    while (n < m) n <<= 1;
    // ---- candidates in index order ----
    for (int i = tid; i < n; i += 1024)
        s_sort[i] = i < m ? (((unsigned long long)a.ws[SW_CAND_IDX + i] << 32) | a.ws[SW_CAND_KEY + i]) : ~0ull;
    bitonic_sort_u64(s_sort, n);
    for (int i = tid; i < m; i += 1024) {
        s_idx[i] = (uint32_t)(s_sort[i] >> 32);
        s_p[i] = key_value((uint32_t)s_sort[i]);
        s_keep[i] = 1;
    }
    __syncthreads();
    const bool greedy = !(p.temperature >= 1e-6f);
    if (!greedy) {
        // ---- softmax over the kept values; sums in index order, as the reference's loops over the vocabulary do
        // (dropped entries are exp(-1e9 - max) = 0 there and add nothing) ----
        if (tid == 0) {
            float mx = s_p[0];
            for (int i = 1; i < m; ++i) mx = s_p[i] > mx ? s_p[i] : mx;
            float sum = 0.0f;
            for (int i = 0; i < m; ++i) { const float e = expf(s_p[i] - mx); s_p[i] = e; sum += e; }
            const float inv = 1.0f / sum;
            for (int i = 0; i < m; ++i) s_p[i] *= inv;
        }
        __syncthreads();
        if (p.top_p < 1.0f) {
            // descending p (ties: lower index first; the reference's std::sort leaves ties unordered); payload = position
            for (int i = tid; i < n; i += 1024)
                s_sort[i] = (i < m && s_p[i] > 1e-10f) ? (((unsigned long long)(~__float_as_uint(s_p[i])) << 32) | (uint32_t)i) : ~0ull;
            bitonic_sort_u64(s_sort, n);
            for (int i = tid; i < m; i += 1024) s_keep[i] = 0;
            __syncthreads();
            if (tid == 0) {
                float cum = 0.0f;
                for (int j = 0; j < m; ++j) {
                    if (s_sort[j] == ~0ull) break;
                    const int pos = (int)(uint32_t)s_sort[j];
                    s_keep[pos] = 1;
                    cum += s_p[pos];
                    if (cum >= p.top_p) break;
                }
                float sum = 0.0f;
                for (int i = 0; i < m; ++i) { if (!s_keep[i]) s_p[i] = 0.0f; sum += s_p[i]; }
                if (sum > 0.0f) {
                    const float inv = 1.0f / sum;
                    for (int i = 0; i < m; ++i) s_p[i] *= inv;
                }
            }
            __syncthreads();
        }
    }
    if (tid == 0) {
        a.ws[SW_WIDE + WS_OVERFLOW] = 0u;
        int token;
        if (greedy) {
            token = (int)s_idx[0];  // every candidate equals the maximum; index order -> the lowest index
        } else {
            const float r = r_draw;
            token = a.vocab - 1;
            if (r <= 0.0f) {
                token = 0;  // the running sum reaches r at the very first index
            } else {
                float cum = 0.0f;
                for (int i = 0; i < m; ++i) {
                    cum += s_p[i];
                    if (cum >= r) { token = (int)s_idx[i]; break; }
                }
            }
        }
        sampler_publish(o, token, step, past_now);
    }
    if (o.leave_clean) {  // every thread read the candidate count long before (barriers above)
        for (int i = tid; i < SW_CLEAR_WORDS; i += 1024) a.ws[i] = 0;
    }
}


// ---------------------------------------------------------------------------------------------------------------------
// Wide path: top-k off (top_k <= 0 or >= vocab) or a top-k beyond the candidate list.  The distribution then spans (almost)
// the whole vocabulary, so nothing is gathered: every stage is a pass over the logits.  Sums that decide something (the
// softmax denominator, the nucleus mass) are accumulated in 64-bit fixed point with integer atomics, so that the result does
// not depend on the order in which workgroups arrive; they differ from the reference's sequential fp32 sums by rounding
// (~1e-7 relative), which moves a token's CDF interval by that much.
// ---------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float wide_inv_sum(const uint32_t* w) {
    const unsigned long long s = *reinterpret_cast<const unsigned long long*>(w + WS_SUMEXP);
    return 1.0f / ((float)s * 2.3283064365386963e-10f);  // 2^-32
}
__device__ __forceinline__ unsigned long long shfl_down_u64(unsigned long long v, int off) {
    const uint32_t lo = __shfl_down((uint32_t)v, off, 64), hi = __shfl_down((uint32_t)(v >> 32), off, 64);
    return ((unsigned long long)hi << 32) | lo;
}

// thr: key of the k-th largest value when a top-k beyond the candidate list is active (else 0: everything is kept)
__global__ __launch_bounds__(256) void sampler_wide_threshold_kernel(SamplerArgs a, int use_topk) {
    __shared__ uint32_t s_scan[8];
    uint32_t* w = a.ws + SW_WIDE;
    uint32_t thr = 0;
    if (use_topk) {
        const ptm_sampling p = sampler_params(a);
        int b0, b1, b2, k = sampler_k(p);
        select_bin(a.ws + SW_HIST0, 2048, k, b0, k, s_scan);
        select_bin(a.ws + SW_HIST1, 2048, k, b1, k, s_scan);
        select_bin(a.ws + SW_HIST2, 1024, k, b2, k, s_scan);
        thr = ((uint32_t)b0 << 21) | ((uint32_t)b1 << 10) | (uint32_t)b2;
    }
    if (threadIdx.x < 16) w[threadIdx.x] = threadIdx.x == WS_THR ? thr : 0u;
    // the mass histogram shares the candidate arrays of the narrow path, which leaves anything there
    for (int i = threadIdx.x; i < 2 * 2048; i += 256) a.ws[SW_MASS_HIST + i] = 0;
}

__global__ __launch_bounds__(256) void sampler_wide_max_kernel(SamplerArgs a) {
    const ptm_sampling p = sampler_params(a);
    uint32_t* w = a.ws + SW_WIDE;
    const uint32_t thr = w[WS_THR];
    uint32_t best = 0;
    const int base = blockIdx.x * SAMPLER_ELEMS_PER_WG;
#pragma unroll
    for (int u = 0; u < SAMPLER_ELEMS_PER_WG / 256; ++u) {
        const int i = base + threadIdx.x + 256 * u;
        if (i < a.vocab) {
            const uint32_t key = order_key(sampler_value(a, p, i));
            if (key >= thr && key > best) best = key;
        }
    }
    for (int off = 32; off > 0; off >>= 1) best = max(best, (uint32_t)__shfl_down(best, off, 64));
    if ((threadIdx.x & 63) == 0 && best) atomicMax(&w[WS_MAXKEY], best);
}

__global__ __launch_bounds__(256) void sampler_wide_sumexp_kernel(SamplerArgs a) {
    const ptm_sampling p = sampler_params(a);
    uint32_t* w = a.ws + SW_WIDE;
    const uint32_t thr = w[WS_THR];
    const float mx = key_value(w[WS_MAXKEY]);
    unsigned long long acc = 0;
    const int base = blockIdx.x * SAMPLER_ELEMS_PER_WG;
#pragma unroll
    for (int u = 0; u < SAMPLER_ELEMS_PER_WG / 256; ++u) {
        const int i = base + threadIdx.x + 256 * u;
        if (i < a.vocab) {
            const float x = sampler_value(a, p, i);
            if (order_key(x) >= thr) acc += (unsigned long long)(expf(x - mx) * 4294967296.0f);  // e <= 1
        }
    }
    for (int off = 32; off > 0; off >>= 1) acc += shfl_down_u64(acc, off);
    if ((threadIdx.x & 63) == 0 && acc) atomicAdd(reinterpret_cast<unsigned long long*>(w + WS_SUMEXP), acc);
}

// probability of a kept token as every wide kernel computes it
__device__ __forceinline__ float wide_prob(float x, float mx, float inv) { return expf(x - mx) * inv; }
__device__ __forceinline__ unsigned long long wide_mass(float pr) { return (unsigned long long)(pr * 1099511627776.0f); }  // 2^40

// LEVEL 0/1/2: probability mass (2^-40 units) per key bin among the kept, eligible (p > 1e-10) tokens under the prefix
template <int LEVEL>
__global__ __launch_bounds__(256) void sampler_wide_mass_hist_kernel(SamplerArgs a) {
    constexpr int NB = LEVEL == 2 ? 1024 : 2048;
    __shared__ unsigned long long s_hist[NB];
    const int tid = threadIdx.x;
    const ptm_sampling p = sampler_params(a);
    uint32_t* w = a.ws + SW_WIDE;
    if (w[WS_KEEP_ALL]) return;
    const uint32_t thr = w[WS_THR], prefix = w[WS_PREFIX];
    const float mx = key_value(w[WS_MAXKEY]), inv = wide_inv_sum(w);
    for (int i = tid; i < NB; i += 256) s_hist[i] = 0;
    __syncthreads();
    const int base = blockIdx.x * SAMPLER_ELEMS_PER_WG;
#pragma unroll
    for (int u = 0; u < SAMPLER_ELEMS_PER_WG / 256; ++u) {
        const int i = base + tid + 256 * u;
        if (i >= a.vocab) continue;
        const float x = sampler_value(a, p, i);
        const uint32_t key = order_key(x);
        if (key < thr) continue;
        const float pr = wide_prob(x, mx, inv);
        if (!(pr > 1e-10f)) continue;
        int bin;
        if (LEVEL == 0) bin = (int)(key >> 21);
        else if (LEVEL == 1) { if ((key >> 21) != prefix) continue; bin = (int)((key >> 10) & 0x7ffu); }
        else { if ((key >> 10) != prefix) continue; bin = (int)(key & 0x3ffu); }
        atomicAdd(&s_hist[bin], wide_mass(pr));
    }
    __syncthreads();
    unsigned long long* g = reinterpret_cast<unsigned long long*>(a.ws + SW_MASS_HIST);
    for (int i = tid; i < NB; i += 256)
        if (s_hist[i]) atomicAdd(&g[i], s_hist[i]);
}

// Walk the level's bins from the top: the bin in which the accumulated mass reaches top_p becomes part of the key prefix, the
// mass above it is carried on; the histogram is zeroed for the next level.  After level 2 the prefix is the key t* of the
// last token value that enters the nucleus, and the number of tokens of that value that enter is fixed (the reference adds
// tokens in descending order and stops as soon as the sum reaches top_p).
template <int LEVEL>
__global__ __launch_bounds__(256) void sampler_wide_select_kernel(SamplerArgs a) {
    constexpr int NB = LEVEL == 2 ? 1024 : 2048, PER = NB / 256;
    __shared__ unsigned long long s_wave[4];
    __shared__ uint32_t s_found[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const ptm_sampling p = sampler_params(a);
    uint32_t* w = a.ws + SW_WIDE;
    unsigned long long* g = reinterpret_cast<unsigned long long*>(a.ws + SW_MASS_HIST);
    if (w[WS_KEEP_ALL]) return;
    const unsigned long long target = (unsigned long long)((double)p.top_p * 1099511627776.0);
    const unsigned long long above0 = *reinterpret_cast<unsigned long long*>(w + WS_MASS_ABOVE);
    unsigned long long h[PER], mine = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) { h[j] = g[NB - 1 - (tid * PER + j)]; mine += h[j]; }
    unsigned long long incl = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t lo = __shfl_up((uint32_t)incl, off, 64), hi = __shfl_up((uint32_t)(incl >> 32), off, 64);
        if (lane >= off) incl += ((unsigned long long)hi << 32) | lo;
    }
    if (tid < 4) s_found[tid] = tid == 0 ? 0u : 0u;
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    for (int q = 0; q < wave; ++q) incl += s_wave[q];
    const unsigned long long excl = incl - mine;
    if (above0 + excl < target && above0 + incl >= target) {   // exactly one thread, if any
        unsigned long long above = above0 + excl;
        for (int j = 0; j < PER; ++j) {
            if (above + h[j] >= target) {
                const uint32_t bin = (uint32_t)(NB - 1 - (tid * PER + j));
                s_found[0] = 1;
                s_found[1] = bin;
                *reinterpret_cast<unsigned long long*>(w + WS_MASS_ABOVE) = above;
                break;
            }
            above += h[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) g[NB - 1 - (tid * PER + j)] = 0;   // clean for the next level / the next call
    if (tid == 0) {
        if (!s_found[0]) {
            w[WS_KEEP_ALL] = 1;   // the eligible tokens together do not reach top_p: all of them stay (the reference's loop runs out)
        } else {
            const uint32_t bin = s_found[1];
            const uint32_t prefix = LEVEL == 0 ? bin : LEVEL == 1 ? ((w[WS_PREFIX] << 11) | bin) : ((w[WS_PREFIX] << 10) | bin);
            w[WS_PREFIX] = prefix;
            if (LEVEL == 2) {
                const float pstar = wide_prob(key_value(prefix), key_value(w[WS_MAXKEY]), wide_inv_sum(w));
                const unsigned long long pf = wide_mass(pstar), above = *reinterpret_cast<unsigned long long*>(w + WS_MASS_ABOVE);
                unsigned long long n = pf ? (target - above + pf - 1) / pf : 1;
                w[WS_TSTAR] = prefix;
                w[WS_NTIE] = (uint32_t)(n < 1 ? 1 : (n > 0xffffffffull ? 0xffffffffull : n));
            }
        }
    }
}

// The draw: one workgroup, wave q walks the q-th sixteenth of the vocabulary in index order, 64 tokens at a time.
// Walk 0 counts the tokens of the nucleus' last value per wave (the first WS_NTIE of them in index order stay), walk 1 sums
// the kept probabilities per wave (the renormalisation of the reference's top-p step), walk 2 finds the first index whose
// running sum reaches the draw.
__device__ __forceinline__ void sampler_wide_draw_body(const SamplerArgs& a, const SamplerOut& o) {
    __shared__ uint32_t s_ties[16];
    __shared__ float s_sum[16];
    __shared__ int s_token[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const ptm_sampling p = sampler_params(a);
    uint32_t* w = a.ws + SW_WIDE;
    const int step = o.d_step ? *o.d_step : 0;
    const int64_t past_now = o.adv.d_past ? *o.adv.d_past : 0;
    const float r = o.uniforms[step];
    const uint32_t thr = w[WS_THR];
    const float mx = key_value(w[WS_MAXKEY]), inv = wide_inv_sum(w);
    const bool nucleus = p.top_p < 1.0f;
    const bool keep_all = w[WS_KEEP_ALL] != 0;
    const uint32_t tstar = w[WS_TSTAR], ntie = w[WS_NTIE];
    const int per_wave = ((a.vocab + 15) / 16 + 63) / 64 * 64;
    const int lo = wave * per_wave, hi = min(a.vocab, lo + per_wave);
    // walk 0: ties of the nucleus' last value in this wave's range
    uint32_t my_ties = 0;
    if (nucleus && !keep_all) {
        for (int b = lo; b < hi; b += 64) {
            const int i = b + lane;
            const bool tie = i < hi && order_key(sampler_value(a, p, i)) == tstar;
            my_ties += (uint32_t)__popcll(__ballot(tie));
        }
    }
    if (lane == 0) s_ties[wave] = my_ties;
    __syncthreads();
    uint32_t tie_base = 0;
    for (int q = 0; q < wave; ++q) tie_base += s_ties[q];
    // kept probability of token i (0 when dropped); tie_rank counts the ties seen so far in index order
    auto kept_prob = [&](int i, bool in, uint32_t& tie_seen) -> float {
        float pr = 0.0f;
        bool tie = false;
        if (in) {
            const float x = sampler_value(a, p, i);
            const uint32_t key = order_key(x);
            if (key >= thr) {
                pr = wide_prob(x, mx, inv);
                if (nucleus) {
                    if (!(pr > 1e-10f)) pr = 0.0f;
                    else if (!keep_all) {
                        tie = key == tstar;
                        if (key < tstar) pr = 0.0f;
                    }
                }
            }
        }
        const unsigned long long tb = __ballot(tie);
        if (tie) {
            const uint32_t rank = tie_seen + (uint32_t)__popcll(tb & ((1ull << lane) - 1ull));
            if (rank >= ntie) pr = 0.0f;
        }
        tie_seen += (uint32_t)__popcll(tb);
        return pr;
    };
    // walk 1: sum of the kept probabilities (only the nucleus step renormalises)
    float total = 1.0f;
    if (nucleus) {
        float acc = 0.0f;
        uint32_t seen = tie_base;
        for (int b = lo; b < hi; b += 64) acc += kept_prob(b + lane, b + lane < hi, seen);
        acc = sum64(acc);
        if (lane == 0) s_sum[wave] = acc;
        __syncthreads();
        total = 0.0f;
        for (int q = 0; q < 16; ++q) total += s_sum[q];
        __syncthreads();
    }
    const float scale = (nucleus && total > 0.0f) ? 1.0f / total : 1.0f;
    // walk 2: per-wave sums first (to know where each wave's running sum starts), then the crossing
    {
        float acc = 0.0f;
        uint32_t seen = tie_base;
        for (int b = lo; b < hi; b += 64) acc += kept_prob(b + lane, b + lane < hi, seen) * scale;
        acc = sum64(acc);
        if (lane == 0) s_sum[wave] = acc;
    }
    __syncthreads();
    float cum = 0.0f;
    for (int q = 0; q < wave; ++q) cum += s_sum[q];
    int found = 0x7fffffff;
    // Every wave adds the same per-wave sums in the same order, so exactly one wave (if any) sees the running sum pass the
    // draw inside its range; it looks for the index.  Its 64-wide scans round differently from the per-wave sum: should they
    // never reach the draw, the wave's last kept token is the one that tipped the sum.
    if (cum < r && cum + s_sum[wave] >= r) {
        uint32_t seen = tie_base;
        int last_kept = lo;
        for (int b = lo; b < hi && found == 0x7fffffff; b += 64) {
            const float v = kept_prob(b + lane, b + lane < hi, seen) * scale;
            float incl = v;   // inclusive prefix sum over the wave, lane order = index order
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const float up = __shfl_up(incl, off, 64);
                if (lane >= off) incl += up;
            }
            const unsigned long long hit = __ballot(b + lane < hi && cum + incl >= r);
            const unsigned long long any = __ballot(v > 0.0f);
            if (any) last_kept = b + 63 - (int)__builtin_clzll(any);
            if (hit) found = b + (int)__builtin_ctzll(hit);
            cum += lane_f(incl, 63);
        }
        if (found == 0x7fffffff) found = last_kept;
    }
    if (lane == 0) s_token[wave] = found;
    __syncthreads();
    if (tid == 0) {
        int token = a.vocab - 1;   // the running sum never reached the draw (rounding): the reference returns the last id
        for (int q = 0; q < 16; ++q) if (s_token[q] != 0x7fffffff) { token = s_token[q]; break; }
        if (r <= 0.0f) token = 0;
        sampler_publish(o, token, step, past_now);
    }
    __syncthreads();
    if (o.leave_clean) for (int i = tid; i < SW_CLEAR_WORDS; i += 1024) a.ws[i] = 0;
}

__global__ __launch_bounds__(1024) void sampler_wide_draw_kernel(SamplerArgs a, SamplerOut o) { sampler_wide_draw_body(a, o); }

// Behind the narrow path's finish kernel, always launched, one workgroup: returns at once unless that kernel found more
// logits tied at the top-k threshold than its candidate list holds (a flat or constant stretch of logits at the cut: the
// reference keeps every tie, gguf_model.h:7682-7691).  Then it does what the wide path does for a large top-k -- largest
// kept value, fixed-point softmax denominator, the nucleus' last value by a three-level walk over per-key-bin mass -- with
// loops of this one workgroup over the vocabulary (a rare case: no launch-level parallelism spent on it), and ends in the
// wide path's draw.  Greedy (k = 1 with the maximum tied that often): the lowest index among the maxima, as argmax gives.
__global__ __launch_bounds__(1024) void sampler_overflow_kernel(SamplerArgs a, SamplerOut o) {
    uint32_t* w = a.ws + SW_WIDE;
    if (w[WS_OVERFLOW] == 0u) return;
    __shared__ unsigned long long s_hist[2048];
    __shared__ unsigned long long s_red64[16];
    __shared__ uint32_t s_red32[16];
    __shared__ uint32_t s_sel[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const ptm_sampling p = sampler_params(a);
    const uint32_t thr = w[WS_THR_SAVE];
    // largest kept key (and, for greedy, the lowest index that holds it)
    uint32_t best = 0;
    for (int i = tid; i < a.vocab; i += 1024) {
        const uint32_t key = order_key(sampler_value(a, p, i));
        if (key >= thr && key > best) best = key;
    }
    for (int off = 32; off > 0; off >>= 1) best = max(best, (uint32_t)__shfl_down(best, off, 64));
    if (lane == 0) s_red32[wave] = best;
    __syncthreads();
    uint32_t mxkey = 0;
    for (int q = 0; q < 16; ++q) mxkey = max(mxkey, s_red32[q]);
    __syncthreads();
    if (!(p.temperature >= 1e-6f)) {
        uint32_t first = 0xffffffffu;
        for (int i = tid; i < a.vocab; i += 1024)
            if (order_key(sampler_value(a, p, i)) == mxkey) { first = (uint32_t)i; break; }
        for (int off = 32; off > 0; off >>= 1) first = min(first, (uint32_t)__shfl_down(first, off, 64));
        if (lane == 0) s_red32[wave] = first;
        __syncthreads();
        if (tid == 0) {
            for (int q = 1; q < 16; ++q) first = min(first, s_red32[q]);
            w[WS_OVERFLOW] = 0u;
            sampler_publish(o, (int)first, o.d_step ? *o.d_step : 0, o.adv.d_past ? *o.adv.d_past : 0);
        }
        return;
    }
    const float mx = key_value(mxkey);
    unsigned long long acc = 0;
    for (int i = tid; i < a.vocab; i += 1024) {
        const float x = sampler_value(a, p, i);
        if (order_key(x) >= thr) acc += (unsigned long long)(expf(x - mx) * 4294967296.0f);
    }
    for (int off = 32; off > 0; off >>= 1) acc += shfl_down_u64(acc, off);
    if (lane == 0) s_red64[wave] = acc;
    __syncthreads();
    unsigned long long sumexp = 0;
    for (int q = 0; q < 16; ++q) sumexp += s_red64[q];
    const float inv = 1.0f / ((float)sumexp * 2.3283064365386963e-10f);
    uint32_t keep_all = 0, prefix = 0, ntie = 0;
    if (p.top_p < 1.0f) {
        const unsigned long long target = (unsigned long long)((double)p.top_p * 1099511627776.0);
        unsigned long long above = 0;
        for (int level = 0; level < 3 && !keep_all; ++level) {
            const int nb = level == 2 ? 1024 : 2048;
            __syncthreads();
            for (int i = tid; i < nb; i += 1024) s_hist[i] = 0;
            __syncthreads();
            for (int i = tid; i < a.vocab; i += 1024) {
                const float x = sampler_value(a, p, i);
                const uint32_t key = order_key(x);
                if (key < thr) continue;
                const float pr = wide_prob(x, mx, inv);
                if (!(pr > 1e-10f)) continue;
                int bin;
                if (level == 0) bin = (int)(key >> 21);
                else if (level == 1) { if ((key >> 21) != prefix) continue; bin = (int)((key >> 10) & 0x7ffu); }
                else { if ((key >> 10) != prefix) continue; bin = (int)(key & 0x3ffu); }
                atomicAdd(&s_hist[bin], wide_mass(pr));
            }
            __syncthreads();
            if (tid == 0) {   // from the top: the bin in which the accumulated mass reaches top_p
                unsigned long long run = above;
                uint32_t found = 0, bin = 0;
                for (int b = nb - 1; b >= 0; --b) {
                    if (run + s_hist[b] >= target) { found = 1; bin = (uint32_t)b; break; }
                    run += s_hist[b];
                }
                s_sel[0] = found;
                s_sel[1] = bin;
                s_red64[0] = run;
            }
            __syncthreads();
            if (!s_sel[0]) { keep_all = 1; break; }   // the eligible tokens together do not reach top_p: all of them stay
            above = s_red64[0];
            prefix = level == 0 ? s_sel[1] : level == 1 ? ((prefix << 11) | s_sel[1]) : ((prefix << 10) | s_sel[1]);
        }
        if (!keep_all) {
            const unsigned long long pf = wide_mass(wide_prob(key_value(prefix), mx, inv));
            const unsigned long long n = pf ? (target - above + pf - 1) / pf : 1;
            ntie = (uint32_t)(n < 1 ? 1 : (n > 0xffffffffull ? 0xffffffffull : n));
        }
    }
    __syncthreads();
    if (tid == 0) {
        w[WS_THR] = thr;
        w[WS_MAXKEY] = mxkey;
        *reinterpret_cast<unsigned long long*>(w + WS_SUMEXP) = sumexp;
        w[WS_KEEP_ALL] = keep_all;
        w[WS_TSTAR] = prefix;
        w[WS_NTIE] = ntie;
        w[WS_OVERFLOW] = 0u;
    }
    __threadfence_block();
    __syncthreads();
    sampler_wide_draw_body(a, o);
}

static bool sampler_is_wide(const ptm_sampling& p, int vocab) {
    return p.temperature >= 1e-6f && (p.top_k <= 0 || p.top_k >= vocab || p.top_k > SAMPLER_MAX_TOPK);
}

static int sampler_check(const ptm_sampling& p, int vocab) {
    if (vocab <= 0) return PTM_E_SHAPE;
    if (!(p.temperature >= 1e-6f)) return PTM_OK;  // greedy: the other fields are not used
    if (!(p.top_p > 0.0f)) return PTM_E_SHAPE;
    return PTM_OK;
}

// Which launch sequence sampler_enqueue records for these parameters: 0 = candidate list (greedy included); otherwise the
// whole-vocabulary passes, bit 1 = with the top-k select, bit 2 = with the nucleus walk.  A captured graph of one key must
// not be replayed for parameters of another.
int sampler_launch_key(const ptm_sampling& p, int vocab) {
    if (!sampler_is_wide(p, vocab)) return 0;
    return 1 | ((p.top_k > 0 && p.top_k < vocab) ? 2 : 0) | (p.top_p < 1.0f ? 4 : 0);
}

// host_params are validated here; when d_params is given the kernels read the device copy (which must hold the same values)
int sampler_enqueue(const float* logits, int vocab, const int32_t* counts, const ptm_sampling& host_params,
                    const ptm_sampling* d_params, const float* d_uniforms, const int* d_step, void* workspace,
                    int64_t* out_token, int32_t* counts_rw, ArgmaxAdvance adv, bool ws_kept_clean, hipStream_t s) {
    // ws_kept_clean: the workspace was zeroed once by the caller and is only ever used through this function, whose last
    // kernel then leaves it zeroed again: the clear launch is skipped
    if (!logits || !workspace || !d_uniforms) return PTM_E_NULL;
    const int rc = sampler_check(host_params, vocab);
    if (rc != PTM_OK) return rc;
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return PTM_E_ALIGN;
    SamplerArgs a{logits, counts, vocab, d_params, host_params, static_cast<uint32_t*>(workspace)};
    SamplerOut o{out_token, d_uniforms, d_step, counts_rw, adv, ws_kept_clean ? 1 : 0};
    const dim3 grid((vocab + SAMPLER_ELEMS_PER_WG - 1) / SAMPLER_ELEMS_PER_WG);
    if (!ws_kept_clean) hipLaunchKernelGGL(sampler_clear_kernel, dim3(4), dim3(256), 0, s, a.ws);
    if (sampler_is_wide(host_params, vocab)) {
        // top-k off, or a top-k beyond the candidate list: passes over the whole vocabulary instead of a gathered list
        const int use_topk = host_params.top_k > 0 && host_params.top_k < vocab;
        if (use_topk) {
            hipLaunchKernelGGL(sampler_hist_kernel<0>, grid, dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_hist_kernel<1>, grid, dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_hist_kernel<2>, grid, dim3(256), 0, s, a);
        }
        hipLaunchKernelGGL(sampler_wide_threshold_kernel, dim3(1), dim3(256), 0, s, a, use_topk);
        hipLaunchKernelGGL(sampler_wide_max_kernel, grid, dim3(256), 0, s, a);
        hipLaunchKernelGGL(sampler_wide_sumexp_kernel, grid, dim3(256), 0, s, a);
        if (host_params.top_p < 1.0f) {
            hipLaunchKernelGGL(sampler_wide_mass_hist_kernel<0>, grid, dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_wide_select_kernel<0>, dim3(1), dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_wide_mass_hist_kernel<1>, grid, dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_wide_select_kernel<1>, dim3(1), dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_wide_mass_hist_kernel<2>, grid, dim3(256), 0, s, a);
            hipLaunchKernelGGL(sampler_wide_select_kernel<2>, dim3(1), dim3(256), 0, s, a);
        }
        hipLaunchKernelGGL(sampler_wide_draw_kernel, dim3(1), dim3(1024), 0, s, a, o);
        return launch_status();
    }
    hipLaunchKernelGGL(sampler_hist_kernel<0>, grid, dim3(256), 0, s, a);
    hipLaunchKernelGGL(sampler_hist_kernel<1>, grid, dim3(256), 0, s, a);
    hipLaunchKernelGGL(sampler_hist_kernel<2>, grid, dim3(256), 0, s, a);
    hipLaunchKernelGGL(sampler_gather_kernel, grid, dim3(256), 0, s, a);
    hipLaunchKernelGGL(sampler_finish_kernel, dim3(1), dim3(1024), 0, s, a, o);
    hipLaunchKernelGGL(sampler_overflow_kernel, dim3(1), dim3(1024), 0, s, a, o);   // returns at once in the usual case
    return launch_status();
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int64_t ptm_sampler_workspace_bytes(void) { return (int64_t)SW_WORDS * 4; }

int ptm_sample_token(const float* logits, int vocab, const int32_t* counts, const ptm_sampling* params, const float* d_uniform,
                     void* workspace, int64_t* out_token, ptm_stream_t stream) {
    if (!params || !out_token) return PTM_E_NULL;
    return sampler_enqueue(logits, vocab, counts, *params, nullptr, d_uniform, nullptr, workspace, out_token, nullptr,
                           ArgmaxAdvance{nullptr, nullptr, nullptr, nullptr, 0}, false, as_stream(stream));
}

// The reference's draws: `static std::mt19937 rng(42); std::uniform_real_distribution<float> dist(0.0f, 1.0f)`
// (gguf_model.h:7740-7742): the standard library itself is the definition, one 32-bit output per draw.
int ptm_mt19937_uniforms(uint32_t seed, int64_t skip, int64_t n, float* out_host) {
    if (!out_host) return PTM_E_NULL;
    if (skip < 0 || n < 0) return PTM_E_SHAPE;
    std::mt19937 rng(seed);
    rng.discard((unsigned long long)skip);
    std::uniform_real_distribution<float> dist(0.0f, 1.0f);
    for (int64_t i = 0; i < n; ++i) out_host[i] = dist(rng);
    return PTM_OK;
}

}  // extern "C"
