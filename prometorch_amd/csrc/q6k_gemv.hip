// Q6_K dequant-fused GEMV for gfx950 (wave64), fp32 activations as in the reference CPU
// kernel (torch/io/cpu_quant_gemv.h:883-1020): y = sum_k (d*scale*(q-32)) * x_k, fp32 accumulate.
//
// A row is swept by an aligned group of 8 lanes.  Per 210-byte super-block lane j fetches
//   ql[16j .. 16j+16)            16 low nibbles  -> group (j%4)/2   of half j/4
//                                16 high nibbles -> group (j%4)/2+2 of half j/4
//   qh[32*(j/4) + 16*(j%2) ..+16) the 2-bit planes of those 32 weights
//   its two scales (single signed bytes) and d
// with dword-aligned 128-bit loads: blocks are 210 bytes, so every other block starts 2 bytes off a dword, and
// 16-byte loads from such addresses run at a fraction of the aligned rate; the lane loads the aligned 16 bytes
// just below plus the piece's last two bytes and shifts them into place with v_alignbyte.
// Weights are assembled four at a time in a dword (q = nibble | twobits<<4, 0..63), converted
// with v_cvt_f32_ubyteN and multiplied with x from LDS; the "-32" offset is applied once per
// 16 weights through the per-16 sums of x kept in LDS:  sum (q-32) x = sum q x - 32 sum x.
// Every pass issues a fixed number of block loads (template NB) behind the activation loads, so the compiler can
// count the loads in flight and each block is consumed as soon as it has arrived.
#include "q6k_body.h"
#include "q6k_mfma_body.h"

#include <mutex>

namespace ptm {

template <bool ACC, bool ARGMAX, bool NORM, int XCH, int NB>
__global__ __launch_bounds__(Q6K_THREADS) void q6k_gemv_kernel(const Q6KArgs a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    q6k_gemv_body<ACC, ARGMAX, NORM, XCH, NB>(a, lds_raw, blockIdx.x);
}

// three waves per SIMD (at most 168 registers): with two the vector pipe idles while a wave waits for its staged block
template <bool ACC, bool ARGMAX, bool NORM, int XL, int NB>
__global__ __launch_bounds__(Q6K_THREADS) __attribute__((amdgpu_waves_per_eu(3, 3))) void q6k_mfma_gemv_kernel(const Q6KArgs a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    q6k_mfma_gemv_body<ACC, ARGMAX, NORM, XL, NB>(a, lds_raw);
}

// Few rows, long rows (a down projection: 2560 x 9728, 4096 x 14336): with 4 rows per workgroup every workgroup
// would stage the whole activation vector for 4 rows' worth of weights, and the staging traffic through L2 would
// exceed the weights'.  Here a workgroup is `waves` waves of 8 >> LOG2S rows each (a row's super-blocks strided over
// 1 << LOG2S lane groups), sized so that the launch is one workgroup per CU: x is staged once per CU.
// XL = float4 loads of x per thread.
enum { Q6K_TALL_MAX_WAVES = 16 };
// XMORE: rows of more than XL float4 per thread are staged in further rounds of loads (its own instantiation: the loop's
// wait for everything in flight would cost the ordinary shapes 7 % on 4096 x 14336).
// MAXW: the most waves a launch of the instantiation has (12, or 16 for the widest matrices: with the bound at 16 the 4096 x
// 14336 launch, 8 waves, measured 14.7 us against 13.8).
template <bool ACC, int NB, int XL, int LOG2S, bool XMORE = false, int MAXW = 12>
__global__ __launch_bounds__(64 * MAXW) void q6k_gemv_tall_kernel(const Q6KArgs a) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    constexpr int S = 1 << LOG2S, ROWS_PER_WAVE = 8 >> LOG2S;
    float* xf = reinterpret_cast<float*>(lds_raw);
    float* xsum16 = xf + q6k_x_floats(a.K);
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, j = lane & 7, grp = lane >> 3, sub = grp & (S - 1);
    const int r = (blockIdx.x * (nthr >> 6) + wave) * ROWS_PER_WAVE + (grp >> LOG2S);
    const bool live = r < a.N;
    const int rr = live ? r : a.N - 1;
    const int nblk = a.K / 256, n4 = a.K / 4;
    const int nb_max = (nblk + S - 1) >> LOG2S;
    const uint8_t* row = a.W + (int64_t)rr * a.stride;
    const int qh_off = 128 + 32 * (j >> 2) + 16 * (j & 1);
    const int sc_off = 192 + 8 * (j >> 2) + 2 * ((j & 3) >> 1) + (j & 1);

    // activation loads first (range-checked buffer loads: no predicate, zeros past the end), then the weights
    const __amdgpu_buffer_rsrc_t x4 = make_rsrc(a.x, a.K * 4);
    u32x4 xv[XL];
#pragma unroll
    for (int u = 0; u < XL; ++u) xv[u] = __builtin_amdgcn_raw_buffer_load_b128(x4, (tid + nthr * u) * 16, 0, 0);
    issue_order_fence();
    Q6Blk blk[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) blk[u] = q6k_load(row + (int64_t)min(sub + S * u, nblk - 1) * 210, j, qh_off, sc_off);
    issue_order_fence();
    // x and its per-16 sums to LDS: 4 consecutive lanes hold one group of 16 (n4 and nthr are multiples of 64, so
    // the range test is wave-uniform)
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int i = tid + nthr * u;
        if (i < n4) {
            const float4 v = make_float4(__uint_as_float(xv[u].x), __uint_as_float(xv[u].y), __uint_as_float(xv[u].z),
                                         __uint_as_float(xv[u].w));
            reinterpret_cast<float4*>(xf)[q6k_xslot(i)] = v;
            float sm = (v.x + v.y) + (v.z + v.w);
            sm += dpp_f<0xB1>(sm);
            sm += dpp_f<0x4E>(sm);
            if ((tid & 3) == 0) xsum16[i >> 2] = sm;
        }
    }
    // rows beyond XL float4 per thread (more than 16 K values with 8 waves): the rest in further rounds, fetched behind the
    // weights (a loop with loads: the compiler waits for everything in flight there, which these rare shapes can afford)
    if constexpr (XMORE)
    for (int base = XL * nthr; base < n4; base += XL * nthr) {
        u32x4 xw[XL];
#pragma unroll
        for (int u = 0; u < XL; ++u) xw[u] = __builtin_amdgcn_raw_buffer_load_b128(x4, (base + tid + nthr * u) * 16, 0, 0);
#pragma unroll
        for (int u = 0; u < XL; ++u) {
            const int i = base + tid + nthr * u;
            if (i < n4) {
                const float4 v = make_float4(__uint_as_float(xw[u].x), __uint_as_float(xw[u].y), __uint_as_float(xw[u].z),
                                             __uint_as_float(xw[u].w));
                reinterpret_cast<float4*>(xf)[q6k_xslot(i)] = v;
                float sm = (v.x + v.y) + (v.z + v.w);
                sm += dpp_f<0xB1>(sm);
                sm += dpp_f<0x4E>(sm);
                if ((tid & 3) == 0) xsum16[i >> 2] = sm;
            }
        }
    }
    __syncthreads();

    // rolling passes, as in q6k_gemv_body
    float acc = 0.0f;
    int i0 = 0;
    for (; i0 + NB < nb_max; i0 += NB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int b = sub + S * (i0 + u);
            const float t = q6k_block_term(blk[u], xf, xsum16, min(b, nblk - 1), j);
            acc += b < nblk ? t : 0.0f;
            blk[u] = q6k_load(row + (int64_t)min(sub + S * (i0 + NB + u), nblk - 1) * 210, j, qh_off, sc_off);
        }
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const int b = sub + S * (i0 + u);
        const float t = q6k_block_term(blk[u], xf, xsum16, min(b, nblk - 1), j);
        acc += b < nblk ? t : 0.0f;
    }
    // same reduction order as q6k_gemv_body
    float p = sum8(acc);
    p += dpp_f<0x128>(p);
    p += __shfl_xor(p, 16, 64);
    if (S >= 8) p += __shfl_xor(p, 32, 64);
    if (live && sub == 0 && j == 0) {
        if constexpr (ACC) a.y[rr] += p;
        else a.y[rr] = p;
    }
}

// Shape of a tall launch: waves per workgroup and lane groups per row, or waves = 0 when the shape is not one for
// it.  Rows that fill the chip once at one workgroup per CU: 8 lane groups per row while that needs at most 16 waves
// (2560 x 9728: 10 waves; 3584 x 18944, the down projection of a 7B model: 14 waves - on the four-row kernel, where 896
// workgroups each staged 76 KB of x, that launch took 33 us), else 4 groups per row and two rows per wave
// (4096 x 14336: 8 waves of 2 rows).
struct Q6KTall { int waves, log2S; };
inline Q6KTall q6k_tall_shape(int N, int K) {
    if (K < 4096 || K > 32768) return {0, 0};   // x and its sums in LDS: 4.4 bytes per value, at most 141 KB
    if (q6k_pick_log2S(N, K / 256) != 3) return {0, 0};   // only where the row tiles would be 4 rows anyway
    const int rows_per_wg = (N + 255) / 256;
    // 13 to 15 rows per workgroup, or 16 long ones: one row per wave beats 7 or 8 waves of two rows (3584 x 18944: 15.1 against
    // 16.6 us, 3200 x 16384: 12.7 against 14.2, 4096 x 28672: 22.4 against 23.6; 4096 x 11008 ... 14336: within 2 % either way)
    if (rows_per_wg >= 13 && rows_per_wg <= (int)Q6K_TALL_MAX_WAVES && (rows_per_wg < 16 || K >= 16384) &&
        K / 4 <= 16 * 64 * rows_per_wg)
        return {rows_per_wg, 3};
    // else up to 12 waves first (4096 x 14336 as 8 waves of two rows: 13.2 us; as 16 waves of one row: 13.0 - 13.5), then up to 16
    for (const int max_waves : {12, (int)Q6K_TALL_MAX_WAVES}) {
        for (int l = 3; l >= 2; --l) {
            const int rpw = 8 >> l;
            int waves = (rows_per_wg + rpw - 1) / rpw;
            if (waves < 2) waves = 2;
            if (waves > max_waves) continue;
            if (K / 4 > 16 * 64 * waves) continue;       // x in at most two rounds of 8 loads per thread
            return {waves, l};
        }
    }
    return {0, 0};
}

void q6k_init_attributes();
template <bool ACC, int NB, int LOG2S>
static int q6k_launch_tall_nb(const Q6KArgs& a, int waves, hipStream_t s) {
    const int rows_per_wg = waves * (8 >> LOG2S);
    const int grid = (a.N + rows_per_wg - 1) / rows_per_wg;
    const size_t lds = q6k_x_lds_bytes(a.K);
    if (lds > 64 * 1024) q6k_init_attributes();
    const int xl = (a.K / 4 + 64 * waves - 1) / (64 * waves);   // beyond 8: a second round of 8
    if (waves > 12) {
        if (xl <= 8) hipLaunchKernelGGL((q6k_gemv_tall_kernel<ACC, NB, 8, LOG2S, false, 16>), dim3(grid), dim3(64 * waves), lds, s, a);
        else hipLaunchKernelGGL((q6k_gemv_tall_kernel<ACC, NB, 8, LOG2S, true, 16>), dim3(grid), dim3(64 * waves), lds, s, a);
    } else if (xl <= 4) hipLaunchKernelGGL((q6k_gemv_tall_kernel<ACC, NB, 4, LOG2S>), dim3(grid), dim3(64 * waves), lds, s, a);
    else if (xl <= 8) hipLaunchKernelGGL((q6k_gemv_tall_kernel<ACC, NB, 8, LOG2S>), dim3(grid), dim3(64 * waves), lds, s, a);
    else hipLaunchKernelGGL((q6k_gemv_tall_kernel<ACC, NB, 8, LOG2S, true>), dim3(grid), dim3(64 * waves), lds, s, a);
    return launch_status();
}
template <bool ACC, int LOG2S>
static int q6k_launch_tall(const Q6KArgs& a, int waves, hipStream_t s) {
    // ONE block in flight per lane group.  The whole launch is resident at once, and a workgroup that requests all of its
    // blocks up front receives them in one burst, at a time set by its launch order, and only then starts its arithmetic:
    // the last workgroup served ends a full arithmetic phase behind the end of the stream.  With one block at a time the
    // requests of all workgroups interleave, every workgroup's arithmetic overlaps the stream, and the other waves of a
    // SIMD cover a wave's wait (2560 x 9728: 7.5 us against 10.4 with five blocks up front; 2, 3, 4 in flight: 9.6, 9.7, 11.4).
    // A second block in flight pays where the CU holds few blocks at a time - two rows per wave and many blocks per lane group
    // (4096 x 14336, 8 waves: 13.2 us against 14.9 with one, 13.7 with three), or fewer than ten waves of one row
    // (2048 x 16384: 9.2 against 10.0; 2048 x 11008: 7.6 against 8.1); with ten or more waves of one row it costs
    // (3072 x 14336: 11.7 against 10.7; 3584 x 18944, 14 waves: 15.8 against 15.1; 2560 x 10240: 9.4 against 7.8).
    const int nb = (a.K / 256 + (1 << LOG2S) - 1) >> LOG2S;
    if ((LOG2S == 2 && nb > 6) || (LOG2S == 3 && waves < 10 && nb >= 4)) return q6k_launch_tall_nb<ACC, 2, LOG2S>(a, waves, s);
    return q6k_launch_tall_nb<ACC, 1, LOG2S>(a, waves, s);
}

// Final argmax over the per-workgroup (value, index) pairs: one workgroup of 1024 threads; every thread issues its
// (up to 8 per round) loads before it compares, so a round costs one memory round trip.
__global__ __launch_bounds__(1024) void argmax_partials_kernel(const float* pv, const int* pi, int n, int64_t* out,
                                                               const ArgmaxAdvance adv) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    int step = 0;
    int64_t past = 0;
    if (threadIdx.x == 0 && adv.d_token) {  // fetched now so that the tail below does not wait on them
        step = *adv.d_step;
        past = *adv.d_past;
    }
    float v = -INFINITY;
    int idx = 0x7fffffff;
    for (int base = 0; base < n; base += 8 * 1024) {
        float tv[8];
        int ti[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = min(base + (int)threadIdx.x + 1024 * u, n - 1);  // clamped: a repeated pair changes nothing
            tv[u] = pv[i];
            ti[u] = pi[i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (tv[u] > v || (tv[u] == v && ti[u] < idx)) { v = tv[u]; idx = ti[u]; }
    }
    for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = v; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (bv[w] > v || (bv[w] == v && bi[w] < idx)) { v = bv[w]; idx = bi[w]; }
        // every comparison against NaN is false: with all-NaN logits no candidate ever replaces the start value.  Publish
        // row 0 then (as the standalone argmax does), never an index outside the table the next step's embedding reads.
        if (idx == 0x7fffffff) idx = 0;
        *out = (int64_t)idx;
        if (adv.d_token) {
            if (step < adv.cap) adv.tokens_out[step] = (int64_t)idx;
            *adv.d_token = idx;
            *adv.d_past = past + 1;
            *adv.d_step = step + 1;
        }
    }
}

static int q6k_check(const void* W, const void* x, int K, int N, int64_t stride) {
    if (!W || !x) return PTM_E_NULL;
    if (K <= 0 || N <= 0 || (K % 256) != 0) return PTM_E_SHAPE;
    if (K > 32768) return PTM_E_UNSUPPORTED;  // x + per-16 sums must fit LDS (K*4.25 bytes <= 136 KB)
    if (stride < (int64_t)(K / 256) * 210) return PTM_E_SHAPE;
    if ((stride & 1) != 0 || (reinterpret_cast<uintptr_t>(W) & 1u) || !aligned16(x)) return PTM_E_ALIGN;
    return PTM_OK;
}

template <bool ACC, bool ARGMAX, bool NORM, int XCH, int NB>
static void q6k_raise_lds_cap() {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_kernel<ACC, ARGMAX, NORM, XCH, NB>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
}
template <bool ACC, int LOG2S>
static void q6k_raise_lds_cap_tall() {
    const int cap = 144 * 1024;
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 1, 4, LOG2S>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 1, 8, LOG2S>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 2, 4, LOG2S>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 2, 8, LOG2S>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 1, 8, LOG2S, true>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 2, 8, LOG2S, true>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 1, 8, LOG2S, false, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 2, 8, LOG2S, false, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 1, 8, LOG2S, true, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&q6k_gemv_tall_kernel<ACC, 2, 8, LOG2S, true, 16>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
}
template <bool ACC, bool ARGMAX, bool NORM, int XCH>
static void q6k_raise_lds_cap_nb() {
    q6k_raise_lds_cap<ACC, ARGMAX, NORM, XCH, 2>();
    q6k_raise_lds_cap<ACC, ARGMAX, NORM, XCH, 3>();
    q6k_raise_lds_cap<ACC, ARGMAX, NORM, XCH, 5>();
}
// Raise the dynamic-LDS cap of every variant once (rows longer than 15K values need more than the default
// 64 KB); must happen outside stream capture, so the decoder calls it when it is created.
void q6k_init_attributes() {
    static std::once_flag done;  // callers on two host threads: the second returns only after the caps are raised
    std::call_once(done, [] {
    q6k_raise_lds_cap_nb<false, false, false, 1>();
    q6k_raise_lds_cap_nb<true, false, false, 1>();
    q6k_raise_lds_cap_nb<false, false, false, 3>();
    q6k_raise_lds_cap_nb<true, false, false, 3>();
    q6k_raise_lds_cap_nb<false, true, false, 1>();
    q6k_raise_lds_cap_nb<false, true, true, 1>();
    q6k_raise_lds_cap_nb<false, false, true, 1>();
    q6k_raise_lds_cap_tall<false, 2>();
    q6k_raise_lds_cap_tall<false, 3>();
    q6k_raise_lds_cap_tall<true, 2>();
    q6k_raise_lds_cap_tall<true, 3>();
    });
}

template <bool ACC, bool ARGMAX, bool NORM, int XCH, int NB>
static int q6k_launch_nb(const Q6KArgs& a, int grid, size_t lds, hipStream_t s) {
    if (lds > 64 * 1024) q6k_init_attributes();
    hipLaunchKernelGGL((q6k_gemv_kernel<ACC, ARGMAX, NORM, XCH, NB>), dim3(grid), dim3(Q6K_THREADS), lds, s, a);
    return launch_status();
}

template <bool ACC, bool ARGMAX, bool NORM, int XCH>
static int q6k_launch_xch(const Q6KArgs& a, int grid, size_t lds, hipStream_t s) {
    switch (q6k_blocks_per_pass(a.N, a.K)) {
        case 2: return q6k_launch_nb<ACC, ARGMAX, NORM, XCH, 2>(a, grid, lds, s);
        case 3: return q6k_launch_nb<ACC, ARGMAX, NORM, XCH, 3>(a, grid, lds, s);
        default: return q6k_launch_nb<ACC, ARGMAX, NORM, XCH, 5>(a, grid, lds, s);
    }
}

// many rows: the matrix-core kernel (64 rows per workgroup, a 16-row tile per wave)
template <bool ACC, bool ARGMAX, bool NORM>
static int q6k_launch_mfma(const Q6KArgs& a, hipStream_t s) {
    const int grid = q6k_mfma_workgroups(a.N);
    const size_t lds = 4 * (size_t)a.K + 4 * 16 * Q6M_PITCH;   // x as two fp16 terms + a tile of 16 row-blocks per wave
    const int nblk = a.K / 256;
    const int nb = nblk >= 4 ? 4 : 2;   // blocks in flight per lane (even: a slot's block parity is fixed); they roll
#define PTM_Q6M(XLV, NBV) hipLaunchKernelGGL((q6k_mfma_gemv_kernel<ACC, ARGMAX, NORM, XLV, NBV>), dim3(grid), dim3(Q6K_THREADS), lds, s, a)
    if (a.K <= 4096) {
        if (nb == 2) PTM_Q6M(4, 2);
        else PTM_Q6M(4, 4);
    } else {
        PTM_Q6M(8, 4);
    }
#undef PTM_Q6M
    return launch_status();
}

template <bool ACC, bool ARGMAX, bool NORM>
static int q6k_launch(Q6KArgs& a, hipStream_t s) {
    if (q6k_mfma_shape(a.N, a.K)) return q6k_launch_mfma<ACC, ARGMAX, NORM>(a, s);
    a.log2S = q6k_pick_log2S(a.N, a.K / 256);
    const int grid = q6k_workgroups(a.N, a.K);
    const size_t lds = q6k_x_lds_bytes(a.K);
    if constexpr (!ARGMAX && !NORM) {
        const Q6KTall tall = q6k_tall_shape(a.N, a.K);
        if (tall.waves > 0)
            return tall.log2S == 3 ? q6k_launch_tall<ACC, 3>(a, tall.waves, s) : q6k_launch_tall<ACC, 2>(a, tall.waves, s);
        // long rows (down projection): all of x is requested before the weights
        if (a.K > 4096 && a.K <= 3 * 4096) return q6k_launch_xch<ACC, false, false, 3>(a, grid, lds, s);
    }
    return q6k_launch_xch<ACC, ARGMAX, NORM, 1>(a, grid, lds, s);
}

int q6k_gemv_impl(const void* W, const float* x, float* y, int K, int N, int64_t stride, bool accumulate,
                  const float* gamma, float eps, int add_one, hipStream_t s) {
    const int rc = q6k_check(W, x, K, N, stride);
    if (rc != PTM_OK) return rc;
    if (!y) return PTM_E_NULL;
    Q6KArgs a{static_cast<const uint8_t*>(W), x, y, K, N, 0, stride, nullptr, nullptr, gamma, eps, add_one, nullptr};
    if (gamma) {
        if (accumulate) return PTM_E_UNSUPPORTED;
        if (!aligned16(gamma)) return PTM_E_ALIGN;
        return q6k_launch<false, false, true>(a, s);
    }
    return accumulate ? q6k_launch<true, false, false>(a, s) : q6k_launch<false, false, false>(a, s);
}

// lm_head of a decode step: optional RMSNorm of x in the prologue (gamma != NULL; the normalised vector is also
// stored to xn_out by one workgroup), logits, their argmax, and optionally the step bookkeeping.
int q6k_gemv_argmax_impl(const void* W, const float* x, const float* gamma, float eps, int add_one, float* xn_out,
                         float* logits, int K, int N, int64_t stride, int64_t* out_index, void* workspace,
                         const ArgmaxAdvance adv, hipStream_t s) {
    const int rc = q6k_check(W, x, K, N, stride);
    if (rc != PTM_OK) return rc;
    if (!out_index || !workspace) return PTM_E_NULL;
    if (gamma && !aligned16(gamma)) return PTM_E_ALIGN;
    if (xn_out && !aligned16(xn_out)) return PTM_E_ALIGN;
    const int grid = q6k_mfma_shape(N, K) ? q6k_mfma_workgroups(N) : q6k_workgroups(N, K);
    Q6KArgs a{static_cast<const uint8_t*>(W), x, logits, K, N, 0, stride, static_cast<float*>(workspace),
              reinterpret_cast<int*>(static_cast<float*>(workspace) + grid), gamma, eps, add_one, xn_out};
    const int rc2 = gamma ? q6k_launch<false, true, true>(a, s) : q6k_launch<false, true, false>(a, s);
    if (rc2 != PTM_OK) return rc2;
    hipLaunchKernelGGL(argmax_partials_kernel, dim3(1), dim3(1024), 0, s, a.part_val, a.part_idx, grid, out_index, adv);
    return launch_status();
}

}  // namespace ptm

using namespace ptm;

extern "C" {

int ptm_q6k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t stride, int accumulate,
                 ptm_stream_t stream) {
    return q6k_gemv_impl(W, x, y, K, N, stride, accumulate != 0, nullptr, 0.f, 0, as_stream(stream));
}

int64_t ptm_argmax_workspace_bytes(int N) {
    // one (value, index) pair per workgroup; the finest split uses 4 rows per workgroup
    return ((int64_t)N + 3) / 4 * 8;
}

int ptm_q6k_gemv_argmax(const void* W, const float* x, float* logits, int K, int N, int64_t stride,
                        int64_t* out_index, void* workspace, ptm_stream_t stream) {
    return q6k_gemv_argmax_impl(W, x, nullptr, 0.f, 0, nullptr, logits, K, N, stride, out_index, workspace,
                                ArgmaxAdvance{nullptr, nullptr, nullptr, nullptr, 0}, as_stream(stream));
}

}  // extern "C"

// ---- the same operator for callers that cannot allocate device memory ------------------------------------------
// The per-workgroup (value, index) pairs of the fused argmax live in a device array of this library instead of a
// caller-provided workspace.  Every GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends; host code only ever uses the address looked up below, never the array's name.
enum { PTM_NOALLOC_MAX_ROWS = 262144 };  // 8 bytes per 4 rows: 512 KiB
static __device__ __align__(256) unsigned char scratch[(PTM_NOALLOC_MAX_ROWS / 4) * 8];

namespace {
enum { MAX_DEVICES = 64 };
void* g_scratch_ptr[MAX_DEVICES];  // per device, filled on the first call with that device current
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (no allocation: a symbol lookup), or NULL with *rc set.
void* scratch_on_current_device(int* rc) {
    int dev = -1;
    *rc = hip_status(hipGetDevice(&dev));
    if (*rc != PTM_OK) return nullptr;
    if (dev < 0 || dev >= MAX_DEVICES) { *rc = PTM_E_UNSUPPORTED; return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        *rc = hip_status(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (*rc != PTM_OK) return nullptr;
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

int ptm_q6k_gemv_argmax_noalloc_max_rows(void) { return PTM_NOALLOC_MAX_ROWS; }

// One-time set-up for the current device, for callers that will call the entry point under stream capture: the symbol
// lookup and the kernel attributes are not capture-legal, everything the entry point does afterwards is.
int ptm_q6k_gemv_argmax_noalloc_init(void) {
    int rc = PTM_OK;
    if (!scratch_on_current_device(&rc)) return rc;
    q6k_init_attributes();
    return PTM_OK;
}

int ptm_q6k_gemv_argmax_noalloc(const void* W, const float* x, float* logits, int K, int N, int64_t stride,
                                int64_t* out_index, ptm_stream_t stream) {
    if (N > PTM_NOALLOC_MAX_ROWS) return PTM_E_RANGE;  // the array holds the partials of at most that many rows
    if (N > 0 && ptm_argmax_workspace_bytes(N) > (int64_t)sizeof(scratch)) return PTM_E_RANGE;
    int rc = PTM_OK;
    void* ws = scratch_on_current_device(&rc);
    if (!ws) return rc;
    // every workgroup of the GEMV overwrites its own pair and the finishing kernel reads exactly those: nothing in the
    // array has to start at zero, whatever an earlier call left there
    return q6k_gemv_argmax_impl(W, x, nullptr, 0.f, 0, nullptr, logits, K, N, stride, out_index, ws,
                                ArgmaxAdvance{nullptr, nullptr, nullptr, nullptr, 0}, as_stream(stream));
}

}  // extern "C"
