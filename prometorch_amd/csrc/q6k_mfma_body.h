// Q6_K dequant-fused GEMV on the matrix cores, for matrices of many rows (the vocabulary projection).
//
// The vector kernel (q6k_body.h) spends 4.9 vector instructions per weight - a conversion and an FMA per weight on top of
// the 6-bit assembly, because the reference multiplies fp32 activations - and the vocabulary projection is bound by their
// issue: 18 992 waves x 1554 instructions = 55 us of issue on 1024 SIMDs for a 49 us stream.  Here the multiply-accumulate
// goes to v_mfma_f32_16x16x32_f16 without leaving fp32 accuracy:
//   * a wave owns 16 rows.  It FETCHES a super-block of each row with 16 lanes x 16 bytes, contiguous and dword-aligned
//     (blocks are 210 bytes: every other one starts 2 bytes off a dword; a lane shifts its chunk into place with v_alignbyte,
//     taking the two missing bytes from its neighbour's chunk by DPP), and passes the aligned blocks through a wave-private
//     LDS tile.  Fetching per lane what that lane computes on - three 16-byte pieces, four single scale bytes, d, three
//     2-byte tails, from 16 rows 2100 bytes apart - costs an L1 access per lane and load: 68.9 M accesses per launch
//     (TCP_TOTAL_CACHE_ACCESSES), 1.2 per cycle and CU over the whole launch, and the launch took 80 us however little
//     arithmetic was left in it (the vector kernel has the same access count: that, not its 55 us of vector issue, is what
//     bounds it).  The cooperative fetch needs 13 accesses per row and block instead of 44;
//   * it COMPUTES with lane l on row l % 16 and the quarter kq = l / 16 of the block: 64 weights from three 16-byte pieces
//     (ql[64 h + 16 c ..], ql[64 h + 32 + 16 c ..], qh[32 h + 16 c ..], h = kq / 2, c = kq % 2), which are the groups
//     y[128 h + 16 c + {0, 32, 64, 96} .. +15] with scales sc[8 h + c + {0, 2, 4, 6}] (gguf_dequant.h:392-430);
//   * sc * (q - 32) is an integer of magnitude <= 1024, exact in fp16: the bytes of four assembled weights become the fp16
//     values 1024 + q by a byte permute (0x6400 | q), and one packed fp16 FMA, (1024 + q) * sc - 1056 * sc, rounds once to
//     the exact product - two instructions per pair of weights where the vector kernel needs four;
//   * the activation vector is the OTHER operand: x * 2^k (k puts max |x| near 2^13) split into two fp16 terms,
//     hi = fp16(x 2^k), lo = fp16((x 2^k - hi) 2^11) - 22 mantissa bits - as operand rows 0 and 1 (rows 2..15 are idle);
//     after the eight products of a super-block, lanes 0..15 hold sum(hi) and sum(lo) of their own row in the accumulator's
//     first two registers, and y += d * (sum_hi + 2^-11 sum_lo), scaled back by 2^-k at the end.
// Products are exact and accumulate in fp32, so the result differs from the vector kernel's by summation order and by the
// 2^-22 split of x (measured against the CPU oracle: ~1e-6 of rms(y), bar 1e-3).
#pragma once
#include "q6k_body.h"

namespace ptm {

typedef _Float16 q6m_h8 __attribute__((ext_vector_type(8)));
typedef _Float16 q6m_h2 __attribute__((ext_vector_type(2)));
typedef float q6m_f4 __attribute__((ext_vector_type(4)));

// One lane's share of the fetch of a super-block of the wave's 16 rows: four 16-byte chunks, chunk c = lane % 16 of rows
// lane / 16 + {0, 4, 8, 12}.  Chunks 0..12 are dword-aligned 16-byte loads from (block start - mis), mis = 0 or 2; chunk 13
// is the dword that holds d (fetched as the last of 16 bytes that end inside the dword the block ends in: never past the
// page); chunks 14, 15 repeat it.
struct Q6MFetch { uint4 v[4]; };
enum { Q6M_PITCH = 240 };  // LDS bytes per staged row-block: 16 B more than 14 chunks -> the 16 rows start 4 banks apart

// Per-lane addresses of the fetch.  Consecutive blocks of a row are 210 bytes apart, so their misalignment alternates:
// even[u] / odd[u] point at this lane's chunk of block 0 as it would lie for an even / odd block index (the row's block 0
// address minus that parity's misalignment; odd = even + 2 mis0 - 2); block b is at +210 b from the pointer of its parity.
struct Q6MAddr { const uint8_t* even[4]; uint32_t mis0[4]; };

template <int PARITY>
__device__ __forceinline__ Q6MFetch q6m_fetch(const Q6MAddr& ad, int b) {
    // every lane issues the same four loads (no load under a branch: the compiler must be able to count the loads in flight)
    Q6MFetch f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint8_t* base = PARITY ? ad.even[u] + 2 * (int)ad.mis0[u] - 2 : ad.even[u];
        const u128_a4 t = *reinterpret_cast<const u128_a4*>(base + (int64_t)b * 210);
        f.v[u] = make_uint4(t.v[0], t.v[1], t.v[2], t.v[3]);  // untouched until it is staged: nothing may wait for it here
    }
    return f;
}

// shift the fetched chunks into place (the two bytes a misaligned chunk lacks are the first two of the next lane's) and
// store the aligned blocks to the wave's LDS tile: row-block `lrow + 4 u` at stage + (lrow + 4 u) * Q6M_PITCH
template <int PARITY>
__device__ __forceinline__ void q6m_stage(const Q6MFetch& f, const Q6MAddr& ad, int chunk, uint8_t* stage_lane) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint32_t mis = PARITY ? ad.mis0[u] ^ 2u : ad.mis0[u];
        uint4 v = f.v[u];
        v.x = chunk < 13 ? v.x : v.w;   // chunks 13..15 fetched the 16 bytes that end with d's dword
        const uint32_t nxt = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v.x, 0x101, 0xF, 0xF, true);  // row_shl:1
        uint32_t o[4];
        realign16(v, nxt, mis, o);
        *reinterpret_cast<uint4*>(stage_lane + 4 * u * Q6M_PITCH) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// What a lane computes on, read back from the staged block of its row
struct Q6MBlk { uint4 qa, qb, qh; int sc[4]; uint32_t d; };

__device__ __forceinline__ Q6MBlk q6m_pieces(const uint8_t* rowblk, int off_a, int off_h, int h, int c) {
    Q6MBlk r;
    r.qa = *reinterpret_cast<const uint4*>(rowblk + off_a);
    r.qb = *reinterpret_cast<const uint4*>(rowblk + off_a + 32);
    r.qh = *reinterpret_cast<const uint4*>(rowblk + off_h);
    const uint2 s8 = *reinterpret_cast<const uint2*>(rowblk + 192 + 8 * h);   // sc[8 h .. 8 h + 7]
    r.sc[0] = __builtin_amdgcn_sbfe((int)s8.x, 8 * c, 8);
    r.sc[1] = __builtin_amdgcn_sbfe((int)s8.x, 8 * c + 16, 8);
    r.sc[2] = __builtin_amdgcn_sbfe((int)s8.y, 8 * c, 8);
    r.sc[3] = __builtin_amdgcn_sbfe((int)s8.y, 8 * c + 16, 8);
    r.d = *reinterpret_cast<const uint16_t*>(rowblk + 208);
    return r;
}

// four assembled weights (bytes 0..63) of one scale group -> sc * (q - 32) as two pairs of fp16
__device__ __forceinline__ void q6m_scale4(uint32_t q4, q6m_h2 sc2, q6m_h2 bias2, q6m_h2& lo, q6m_h2& hi) {
    const uint32_t b01 = __builtin_amdgcn_perm(0x64646464u, q4, 0x04010400u);  // halves 0x6400 | q = 1024 + q
    const uint32_t b23 = __builtin_amdgcn_perm(0x64646464u, q4, 0x04030402u);
    lo = __builtin_elementwise_fma(__builtin_bit_cast(q6m_h2, b01), sc2, bias2);
    hi = __builtin_elementwise_fma(__builtin_bit_cast(q6m_h2, b23), sc2, bias2);
}

// The eight products of one super-block: returns this lane's accumulator (lanes 0..15: [0] = sum over the block of
// w * x_hi, [1] = of w * x_lo, for row `lane` of the wave's tile).  xa: this lane's operand row in LDS at the block's first
// value plus the lane's quarter offset.  The x fragments are requested four at a time ahead of the unpacking arithmetic that
// covers their LDS round trip (read one by one in front of their products, each costs the wave a full LDS latency).
__device__ __forceinline__ q6m_f4 q6m_block(const Q6MBlk& k, const uint8_t* __restrict__ xa) {
    q6m_h8 a8[8];
#pragma unroll
    for (int s = 0; s < 4; ++s) a8[s] = *reinterpret_cast<const q6m_h8*>(xa + 64 * (s >> 1) + 16 * (s & 1));
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t qa[4] = {k.qa.x, k.qa.y, k.qa.z, k.qa.w}, qb[4] = {k.qb.x, k.qb.y, k.qb.z, k.qb.w},
                   qh[4] = {k.qh.x, k.qh.y, k.qh.z, k.qh.w};
    q6m_h2 sc2[4], bias2[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const _Float16 s = (_Float16)(float)k.sc[g];             // |sc| <= 32: exact
        const _Float16 b = (_Float16)(-1056.0f * (float)k.sc[g]);  // 33 * 32 * sc: at most 11 significant bits, exact
        sc2[g] = q6m_h2{s, s};
        bias2[g] = q6m_h2{b, b};
    }
    q6m_f4 c = {0.0f, 0.0f, 0.0f, 0.0f};
    // group g of the lane: 0 = low nibbles of piece a (y[l]), 1 = low nibbles of piece b (y[l + 32]), 2 = high nibbles of a
    // (y[l + 64]), 3 = high nibbles of b (y[l + 96]); its two bits are bits 2g, 2g + 1 of the qh bytes
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        if (g == 1) {   // the fragments of the last two groups are requested while the first two are worked on
#pragma unroll
            for (int s = 4; s < 8; ++s) a8[s] = *reinterpret_cast<const q6m_h8*>(xa + 64 * (s >> 1) + 16 * (s & 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        q6m_h2 w[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t nib = g == 0 ? (qa[i] & 0x0f0f0f0fu) : g == 1 ? (qb[i] & 0x0f0f0f0fu)
                               : g == 2 ? ((qa[i] >> 4) & 0x0f0f0f0fu) : ((qb[i] >> 4) & 0x0f0f0f0fu);
            const uint32_t two = g == 0 ? (qh[i] << 4) : g == 1 ? (qh[i] << 2) : g == 2 ? qh[i] : (qh[i] >> 2);
            q6m_scale4(nib | (two & 0x30303030u), sc2[g], bias2[g], w[2 * i], w[2 * i + 1]);
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const q6m_h8 b8 = {w[4 * e][0], w[4 * e][1], w[4 * e + 1][0], w[4 * e + 1][1],
                               w[4 * e + 2][0], w[4 * e + 2][1], w[4 * e + 3][0], w[4 * e + 3][1]};
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a8[2 * g + e], b8, c, 0, 0, 0);
        }
    }
    return c;
}

// XL: float4 loads of x per thread (K <= 1024 XL); NB: super-blocks in flight per lane.
template <bool ACC, bool ARGMAX, bool NORM, int XL, int NB>
__device__ __forceinline__ void q6k_mfma_gemv_body(const Q6KArgs a, uint8_t* lds_raw) {
    static_assert(NB % 2 == 0, "block parity is taken from the unrolled slot index");
    // LDS: x_hi[K] fp16 | x_lo[K] fp16
    uint8_t* s_hi = lds_raw;
    uint8_t* s_lo = lds_raw + 2 * (size_t)a.K;
    __shared__ float red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rl = lane & 15, kq = lane >> 4, h = kq >> 1, c = kq & 1;
    const int r0 = (blockIdx.x * 4 + wave) * 16;
    const int r = r0 + rl;
    const bool live = r < a.N;
    const int rr = live ? r : a.N - 1;
    const int nblk = a.K / 256, n4 = a.K / 4;
    const int off_a = 64 * h + 16 * c, off_h = 128 + 32 * h + 16 * c;
    // fetch role: chunk lane % 16 of rows lane / 16 + {0, 4, 8, 12} of the tile (rows past the end repeat the last row)
    const int chunk = lane & 15;
    Q6MAddr ad;
    {
        const int off = chunk < 13 ? 16 * chunk : 196;   // chunks 13..15: the 16 bytes that end with the dword holding d
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint8_t* rp = a.W + (int64_t)min(r0 + (lane >> 4) + 4 * u, a.N - 1) * a.stride;
            ad.mis0[u] = (uint32_t)reinterpret_cast<uintptr_t>(rp) & 2u;
            ad.even[u] = rp - ad.mis0[u] + off;
        }
    }
    // a block index past the row's end (prefetch of the last pass) is replaced by the last block of the same parity
    auto clampb = [nblk](int b) { return b < nblk ? b : (nblk - 1) - ((b - (nblk - 1)) & 1); };
    uint8_t* const stage = lds_raw + 4 * (size_t)a.K + (size_t)wave * 16 * Q6M_PITCH;   // this wave's tile of 16 row-blocks
    uint8_t* const stage_lane = stage + (lane >> 4) * Q6M_PITCH + 16 * min(chunk, 14);
    const uint8_t* const stage_row = stage + rl * Q6M_PITCH;

    // ---- activation loads first (range-checked buffer loads, zeros past the end), then the first blocks ----
    const __amdgpu_buffer_rsrc_t x4 = make_rsrc(a.x, a.K * 4);
    const __amdgpu_buffer_rsrc_t g4 = make_rsrc(NORM ? a.gamma : a.x, a.K * 4);
    u32x4 xv[XL], gv[NORM ? XL : 1];
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        xv[u] = __builtin_amdgcn_raw_buffer_load_b128(x4, (tid + 256 * u) * 16, 0, 0);
        if constexpr (NORM) gv[u] = __builtin_amdgcn_raw_buffer_load_b128(g4, (tid + 256 * u) * 16, 0, 0);
    }
    issue_order_fence();
    Q6MFetch ft[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) ft[u] = (u & 1) ? q6m_fetch<1>(ad, clampb(u)) : q6m_fetch<0>(ad, clampb(u));
    issue_order_fence();

    // ---- x (optionally RMS-normalised) -> power-of-two scale -> two fp16 terms in LDS ----
    float4 v[XL];
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        v[u] = make_float4(__uint_as_float(xv[u].x), __uint_as_float(xv[u].y), __uint_as_float(xv[u].z), __uint_as_float(xv[u].w));
        if constexpr (NORM) {
            ss = fmaf(v[u].x, v[u].x, ss);
            ss = fmaf(v[u].y, v[u].y, ss);
            ss = fmaf(v[u].z, v[u].z, ss);
            ss = fmaf(v[u].w, v[u].w, ss);
        }
    }
    if constexpr (NORM) {
        ss = block_sum256(ss, red);
        const float rs = 1.0f / sqrtf(ss / (float)a.K + a.eps);
        const float one = a.add_one ? 1.0f : 0.0f;
#pragma unroll
        for (int u = 0; u < XL; ++u) {
            const float4 g = make_float4(__uint_as_float(gv[u].x), __uint_as_float(gv[u].y), __uint_as_float(gv[u].z), __uint_as_float(gv[u].w));
            v[u] = norm4(v[u], g, rs, one);
            if (blockIdx.x == 0 && a.xn_out && tid + 256 * u < n4) reinterpret_cast<float4*>(a.xn_out)[tid + 256 * u] = v[u];
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int u = 0; u < XL; ++u)
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w))));
    amax = max64(amax);
    if (lane == 0) red[4 + wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
    // 2^k with max |x| 2^k in [2^13, 2^14); a zero or non-finite maximum leaves the scale at 1
    int ex = (int)((__float_as_uint(amax) >> 23) & 255u);
    if (ex == 0 || ex == 255) ex = 127 + 13;
    const int kexp = max(-120, min(120, 127 + 13 - ex));
    const float up = __uint_as_float((uint32_t)(127 + kexp) << 23);
    const float down = __uint_as_float((uint32_t)(127 - kexp) << 23);
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int i = tid + 256 * u;
        if (i < n4) {
            const float f[4] = {v[u].x * up, v[u].y * up, v[u].z * up, v[u].w * up};
            _Float16 hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                hi[e] = (_Float16)f[e];
                lo[e] = (_Float16)((f[e] - (float)hi[e]) * 2048.0f);
            }
            typedef _Float16 h4 __attribute__((ext_vector_type(4)));
            *reinterpret_cast<h4*>(s_hi + 8 * i) = h4{hi[0], hi[1], hi[2], hi[3]};
            *reinterpret_cast<h4*>(s_lo + 8 * i) = h4{lo[0], lo[1], lo[2], lo[3]};
        }
    }
    __syncthreads();

    // this lane's operand row of x: rows 0 and 1 of the 16-row operand are x_hi and x_lo; rows 2..15 only feed accumulator
    // rows that nobody reads, so their lanes fetch x_hi as well (no zero row, no per-lane address arithmetic)
    const uint8_t* xa = (rl == 1 ? s_lo : s_hi) + 2 * (128 * h + 16 * c);

    // Blocks roll through NB register sets: block b is shifted into place and staged, its successor NB blocks on is
    // requested into the same registers, then the lanes read their pieces of block b back and compute.  LDS operations of
    // a wave execute in order, so the tile needs no barrier and no second buffer.
    float acc = 0.0f;
    int b0 = 0;
    for (; b0 + NB < nblk; b0 += NB) {
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            // NB is even and b0 a multiple of it: the parity of block b0 + u is that of u
            if (u & 1) { q6m_stage<1>(ft[u], ad, chunk, stage_lane); ft[u] = q6m_fetch<1>(ad, clampb(b0 + NB + u)); }
            else { q6m_stage<0>(ft[u], ad, chunk, stage_lane); ft[u] = q6m_fetch<0>(ad, clampb(b0 + NB + u)); }
            const Q6MBlk k = q6m_pieces(stage_row, off_a, off_h, h, c);
            const q6m_f4 cc = q6m_block(k, xa + 512 * (b0 + u));
            acc = fmaf(h2f(k.d), fmaf(cc[1], 1.0f / 2048.0f, cc[0]), acc);
        }
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const int b = b0 + u;
        if (b < nblk) {  // wave-uniform
            if (u & 1) q6m_stage<1>(ft[u], ad, chunk, stage_lane);
            else q6m_stage<0>(ft[u], ad, chunk, stage_lane);
            const Q6MBlk k = q6m_pieces(stage_row, off_a, off_h, h, c);
            const q6m_f4 cc = q6m_block(k, xa + 512 * b);
            acc = fmaf(h2f(k.d), fmaf(cc[1], 1.0f / 2048.0f, cc[0]), acc);
        }
    }
    const float p = acc * down;   // lanes 0..15: row rl of the tile
    if (kq == 0 && live && a.y) {
        if constexpr (ACC) a.y[rr] += p;
        else a.y[rr] = p;
    }
    if constexpr (ARGMAX) {
        // best (value, lowest index) of this workgroup's 64 rows
        __shared__ float bv[4];
        __shared__ int bi[4];
        float bvv = (kq == 0 && live) ? p : -INFINITY;
        int idx = rr;
        for (int off = 1; off < 16; off <<= 1) {
            const float ov = __shfl_xor(bvv, off, 64);
            const int oi = __shfl_xor(idx, off, 64);
            if (ov > bvv || (ov == bvv && oi < idx)) { bvv = ov; idx = oi; }
        }
        if (lane == 0) { bv[wave] = bvv; bi[wave] = idx; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < 4; ++w)
                if (bv[w] > bvv || (bv[w] == bvv && bi[w] < idx)) { bvv = bv[w]; idx = bi[w]; }
            a.part_val[blockIdx.x] = bvv;
            a.part_idx[blockIdx.x] = idx;
        }
    }
}

inline int q6k_mfma_workgroups(int N) { return (N + 63) / 64; }
// shapes the matrix-core kernel takes: enough 16-row tiles to fill the chip several times over, x in at most 8 loads per thread
inline bool q6k_mfma_shape(int N, int K) { return N >= 16384 && K >= 512 && K <= 8192; }

}  // namespace ptm
