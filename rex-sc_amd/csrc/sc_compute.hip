// SC conv / linear compute: AND-multiply, popcount over the whole reduction of one stream
// slot, clamp to n_sat, sum over slots (sc_conv.cpp:204-299, sc_matmul.cpp:390-574).
//
// Mapping (wave64, no LDS, no MFMA -- the work is v_and_b32 + v_bcnt_u32_b32):
//   lane            = output pixel (PX pixels per lane), so activation words live in VGPRs;
//   weights         = wave-uniform, fetched with scalar loads into SGPRs and used directly
//                     as the scalar operand of v_and_b32;
//   register tile   = PX pixels x OT output channels per lane; per-slot counts for both
//                     polarities stay in VGPRs, per-output sums are packed u16|u16
//                     (positive | negative << 16), which also reproduces the reference's
//                     16-bit wrap-around of the running sum.
//   reduction order = slot (outer) -> kernel row ky -> channel chunk zg (runtime loops);
//                     inside a chunk everything is unrolled: OT x KW x ZC x PX (and+bcnt) x 2.
//   block           = NS waves that share one tile of 64*PX pixels x OT channels and split the
//                     stream slots among themselves; their partial sums meet in LDS, so the final
//                     int16 results are written once and no partial traffic reaches HBM.  Short
//                     waves (slots/NS each) keep the tail of the launch small: with ~1000 SIMDs
//                     and 3 resident waves each, whole-reduction waves would quantise badly.
//   grid            = pixel tiles x output-channel tiles x (optional) global slot splits, remapped
//                     so that the blocks sharing a pixel tile run on the same XCD (shared L2).
#include <stdlib.h>
#include <string>

#include "sc_compute.h"
#include "profile.h"

namespace rexsc {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b)
{
    u16x2 r = __builtin_elementwise_min(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_add_u16(uint32_t a, uint32_t b)
{
    u16x2 r = __builtin_bit_cast(u16x2, a) + __builtin_bit_cast(u16x2, b);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pk_sub_u16(uint32_t a, uint32_t b)
{
    u16x2 r = __builtin_bit_cast(u16x2, a) - __builtin_bit_cast(u16x2, b);
    return __builtin_bit_cast(uint32_t, r);
}

template <int ZC>
__device__ __forceinline__ void load_words(const uint32_t *__restrict__ p, uint32_t *dst)
{
    if constexpr (ZC == 1) {
        dst[0] = p[0];
    } else if constexpr (ZC == 2) {
        const uint2 v = *reinterpret_cast<const uint2 *>(p);
        dst[0] = v.x; dst[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < ZC; i += 4) {
            const uint4 v = *reinterpret_cast<const uint4 *>(p + i);
            dst[i] = v.x; dst[i + 1] = v.y; dst[i + 2] = v.z; dst[i + 3] = v.w;
        }
    }
}

// Output channels per weight batch: the largest power of two whose batch (G*2*KWZ dwords) fits 32
// SGPRs, at least 1 and at most OT/2 (so that a chunk holds an even number of batches).
constexpr int pick_group(int kwz, int ot)
{
    int g = 1;
    while (g * 2 <= ot / 2 && g * 2 * 2 * kwz <= 32) g *= 2;
    return g;
}

// count += popcount(a & w): v_and_b32 (weight word as the scalar operand) + v_bcnt_u32_b32 with its
// accumulate input.  The accumulate form is spelled out because the compiler otherwise reassociates
// chains of popcounts into popcount+popcount+add3, which costs 3 instructions per 2 words.
// The s_nop between the two is deliberate: measured on gfx950 (register-only loops, 2 to 8 waves per SIMD),
// a SIMD retires the pair in 6.2 cycles when the wave issues one scalar instruction per pair (v_and 2 cycles,
// v_bcnt 4) and in 8.2 cycles when the pairs follow each other with nothing in between, whatever the order
// of independent pairs; a two-cycle s_nop 1, or a nop after each of the two instructions, loses the gain again.
__device__ __forceinline__ void and_popc_acc(uint32_t &count, uint32_t a, uint32_t w)
{
    const uint32_t t = a & w;
#if defined(__HIP_DEVICE_COMPILE__) // the host pass of hipcc parses device functions too
    asm("s_nop 0\n\tv_bcnt_u32_b32 %0, %1, %0" : "+v"(count) : "v"(t));
#else
    count += __builtin_popcount(t);
#endif
}

// acc |= a & w as ONE v_and_or_b32 with the weight word as the scalar operand.  Spelled out because the
// compiler otherwise regroups chains of these into v_and + v_or3, about 1.3 instructions per word.
__device__ __forceinline__ void and_or_acc(uint32_t &acc, uint32_t a, uint32_t w)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm("v_and_or_b32 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "s"(w));
#else
    acc |= a & w;
#endif
}

// min(x, 1) as one v_min_u32 (the compiler's choice is a compare and a select)
__device__ __forceinline__ uint32_t min_one(uint32_t x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t r;
    asm("v_min_u32 %0, 1, %1" : "=v"(r) : "v"(x));
    return r;
#else
    return x < 1u ? x : 1u;
#endif
}

// One weight batch: G output channels starting at o0, both polarities, all KWZ words, PX pixels.
// wb holds [g][pol][j].
// OR1: the slot result is min(count, 1), i.e. "any product bit set": the AND results are OR-ed into
// the counter registers (one v_and_or_b32 per word) instead of being counted.
template <int PX, int OT, int KWZ, int G, bool OR1>
__device__ __forceinline__ void compute_batch(const uint32_t (&a)[PX][KWZ], const uint32_t (&wb)[G * 2 * KWZ],
                                              uint32_t (&cp)[PX][OT], uint32_t (&cn)[PX][OT], int o0)
{
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int j = 0; j < KWZ; j++) {
            const uint32_t wp = wb[(g * 2 + 0) * KWZ + j];
            const uint32_t wn = wb[(g * 2 + 1) * KWZ + j];
#pragma unroll
            for (int px = 0; px < PX; px++) {
                if (OR1) {
                    and_or_acc(cp[px][o0 + g], a[px][j], wp);
                    and_or_acc(cn[px][o0 + g], a[px][j], wn);
                } else {
                    and_popc_acc(cp[px][o0 + g], a[px][j], wp);
                    and_popc_acc(cn[px][o0 + g], a[px][j], wn);
                }
            }
        }
}

// The layer's float output from the packed 16-bit sums (pos | neg << 16): float(pos) / L - float(neg) / L with the
// sums read as int16, as the reference converts its int16 results (utils_functional.py:1181-1182, 1273-1274, 1317).
// inv_L is a power of two, so both products are exact.
__device__ __forceinline__ float counts_value(uint32_t packed, float inv_L)
{
    return (float)(int16_t)(packed & 0xffffu) * inv_L - (float)(int16_t)(packed >> 16) * inv_L;
}

constexpr int MAX_NS = 4; // waves per block (each takes a share of the stream slots)
// s_waitcnt immediate: lgkmcnt(0), vmcnt and expcnt left at their maxima (not waited for)
constexpr int WAIT_LGKM0 = 0xC07F;

// MODE 0: 16-bit packed sums; 1 (WIDE): 32-bit sums for the linear op's large saturation values;
// 2 (OR1): 16-bit packed sums with n_sat = 1, evaluated with and-or instead of and-popcount.
template <int KW, int ZC, int PX, int OT, int MODE>
__global__ __launch_bounds__(64 * MAX_NS) void sc_compute_kernel(const uint32_t *__restrict__ A,
                                                        const uint32_t *__restrict__ Wst, ComputeParams p,
                                                        uint32_t *__restrict__ part, int16_t *__restrict__ out_pos,
                                                        int16_t *__restrict__ out_neg, int16_t *__restrict__ out_diff,
                                                        float *__restrict__ out_value)
{
    constexpr bool WIDE = MODE == 1, OR1 = MODE == 2;
    constexpr int KWZ = KW * ZC;
    constexpr int BM = 64 * PX;            // pixels per block (every wave of the block covers all of them)
    __shared__ uint32_t s_red[MAX_NS][WIDE ? 2 : 1][PX * OT][64];

    // XCD-aware block remap: hardware deals consecutive block ids round-robin over 8 XCDs;
    // give each XCD a contiguous range of logical ids (o-tiles of one pixel tile are adjacent).
    const int per_xcd = gridDim.x >> 3;
    int bid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (bid >= p.m_tiles * p.o_tiles * p.splits) return;
    const int otile = bid % p.o_tiles; bid /= p.o_tiles;
    const int mtile = bid % p.m_tiles;
    const int split = bid / p.m_tiles;

    const int lane = threadIdx.x & 63, ns = blockDim.x >> 6;
    // wave index, made provably wave-uniform so that everything derived from it (slot range, weight
    // addresses) stays in SGPRs and the weight loads stay scalar
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int abase[PX]; // word offset of the lane's pixel inside one slot, for ky = 0, zg = 0
    int mpix[PX];
#pragma unroll
    for (int px = 0; px < PX; px++) {
        const int m = mtile * BM + px * 64 + lane;
        mpix[px] = m;
        const int mm = m < p.M ? m : p.M - 1;
        const int n = mm / p.HoWo, r = mm - n * p.HoWo;
        const int yo = r / p.Wo, xo = r - yo * p.Wo;
        abase[px] = (((n * p.ZG) * p.Hp + yo * p.s0) * p.Wp + xo * p.s1) * ZC;
    }

    uint32_t acc[PX][OT];
    uint32_t accw[WIDE ? PX : 1][WIDE ? OT : 1]; // negative sums when 16-bit packing could overflow
#pragma unroll
    for (int px = 0; px < PX; px++)
#pragma unroll
        for (int o = 0; o < OT; o++) { acc[px][o] = 0; if (WIDE) accw[px][o] = 0; }

    // slots of this block, then of this wave
    const int sb_begin = split * p.slots_per_split;
    const int sb_end = min(p.n_slots, sb_begin + p.slots_per_split);
    const int per_wave = (sb_end - sb_begin + ns - 1) / ns;
    const int s_begin = min(sb_end, sb_begin + wave * per_wave);
    const int s_end = min(sb_end, s_begin + per_wave);
    const int chunk_stride = p.Hp * p.Wp * ZC; // words between zg planes
    const int row_stride = p.Wp * ZC;          // words between kernel rows
    const long w_chunk_words = (long)p.O_pad * 2 * KWZ;

    // The reduction is walked chunk by chunk: chunk q = (slot, ky, zg) in that order, which is also
    // the order of the weight stream in memory.  Two software pipelines hide latency:
    //  * activations: the words of chunk q+1 are loaded into a second register set while chunk q
    //    is being computed;
    //  * weights: each chunk is consumed in batches of G output channels (BW dwords); the scalar
    //    loads of batch b+1 are issued before the VALU work of batch b.  Scalar loads return out of
    //    order, so a wave can only wait for all of them: issuing exactly one batch ahead keeps the
    //    wait at the top of every batch short.  The last batch of a chunk prefetches the first
    //    batch of the next chunk (the weight buffer is padded by one chunk for the final over-read).
    constexpr int G = pick_group(KWZ, OT);
    constexpr int BW = G * 2 * KWZ;  // dwords per weight batch
    constexpr int NB = OT / G;       // batches per chunk (even)
    static_assert(NB % 2 == 0, "the batch ping-pong needs an even number of batches per chunk");

    const int chunks_per_slot = p.KH * p.ZG;
    const int q_begin = s_begin * chunks_per_slot, q_end = s_end * chunks_per_slot;
    const uint32_t *w_q = Wst + (long)q_begin * w_chunk_words + (long)otile * OT * 2 * KWZ;

    uint32_t cp[PX][OT], cn[PX][OT];
#pragma unroll
    for (int px = 0; px < PX; px++)
#pragma unroll
        for (int o = 0; o < OT; o++) { cp[px][o] = 0; cn[px][o] = 0; }

    uint32_t a_cur[PX][KWZ], a_nxt[PX][KWZ];
    uint32_t wb0[BW], wb1[BW];
    int slot = s_begin, ky = 0, zg = 0;
    if (s_begin < s_end) { // wave-uniform
        const uint32_t *a_chunk = A + (long)slot * p.a_slot_stride;
#pragma unroll
        for (int px = 0; px < PX; px++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) load_words<ZC>(a_chunk + abase[px] + kx * ZC, &a_cur[px][kx * ZC]);
#pragma unroll
        for (int e = 0; e < BW; e++) wb0[e] = w_q[e];
    }

    for (int q = q_begin; q < q_end; q++) {
        // coordinates of the next chunk
        int zg_n = zg + 1, ky_n = ky, slot_n = slot;
        if (zg_n == p.ZG) { zg_n = 0; ky_n++; if (ky_n == p.KH) { ky_n = 0; slot_n++; } }
        const bool slot_done = (zg_n == 0 && ky_n == 0);
        {
            // prefetch its activation words (the last chunk re-reads itself: harmless)
            const bool has_next = q + 1 < q_end;
            const int sl = has_next ? slot_n : slot, kk = has_next ? ky_n : ky, zz = has_next ? zg_n : zg;
            const uint32_t *a_chunk = A + (long)sl * p.a_slot_stride + zz * chunk_stride + kk * row_stride;
#pragma unroll
            for (int px = 0; px < PX; px++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++) load_words<ZC>(a_chunk + abase[px] + kx * ZC, &a_nxt[px][kx * ZC]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < NB; b += 2) {
            // batch b lives in wb0, batch b+1 in wb1
            // Make sure the batch about to be used has landed BEFORE the next one is requested: the
            // compiler would otherwise place this wait after the request and wait for both.
            __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
            {
                const uint32_t *src = w_q + (b + 1) * BW;
#pragma unroll
                for (int e = 0; e < BW; e++) wb1[e] = src[e];
            }
            __builtin_amdgcn_sched_barrier(0); // keep the prefetch above the VALU work it overlaps with
            compute_batch<PX, OT, KWZ, G, OR1>(a_cur, wb0, cp, cn, b * G);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
            {
                const uint32_t *src = (b + 2 < NB) ? w_q + (b + 2) * BW : w_q + w_chunk_words;
#pragma unroll
                for (int e = 0; e < BW; e++) wb0[e] = src[e];
            }
            __builtin_amdgcn_sched_barrier(0);
            compute_batch<PX, OT, KWZ, G, OR1>(a_cur, wb1, cp, cn, (b + 1) * G);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (slot_done) {
            // per-slot saturation and accumulation
            if (OR1) { // [any bit set], both for min(count, 1) and for count >= 1
#pragma unroll
                for (int px = 0; px < PX; px++)
#pragma unroll
                    for (int o = 0; o < OT; o++)
                        acc[px][o] = pk_add_u16(acc[px][o], min_one(cp[px][o]) | (min_one(cn[px][o]) << 16));
            } else if (!WIDE) {
                // Only the linear op (a 1x1 problem) ever asks for the "count >= n" rule.  The empty asm keeps the
                // compiler from evaluating both rules and selecting (it did: two v_pk_min and a v_pk_sub per
                // output and slot on the common path).
                if (KW != 1 || p.mode == 0) {
#pragma unroll
                    for (int px = 0; px < PX; px++)
#pragma unroll
                        for (int o = 0; o < OT; o++) {
                            const uint32_t c = cp[px][o] | (cn[px][o] << 16);
                            acc[px][o] = pk_add_u16(acc[px][o], pk_min_u16(c, p.nn));
                        }
                } else { // [count >= n] = min(count, n) - min(count, n-1)
                    asm volatile("" ::: "memory");
#pragma unroll
                    for (int px = 0; px < PX; px++)
#pragma unroll
                        for (int o = 0; o < OT; o++) {
                            const uint32_t c = cp[px][o] | (cn[px][o] << 16);
                            const uint32_t d = pk_sub_u16(pk_min_u16(c, p.nn), pk_min_u16(c, p.nn - 0x00010001u));
                            acc[px][o] = pk_add_u16(acc[px][o], d);
                        }
                }
            } else {
                const uint32_t n = p.nn & 0xffffu;
#pragma unroll
                for (int px = 0; px < PX; px++)
#pragma unroll
                    for (int o = 0; o < OT; o++) {
                        if (p.mode == 0) {
                            acc[px][o] += min(cp[px][o], n);
                            accw[px][o] += min(cn[px][o], n);
                        } else {
                            acc[px][o] += cp[px][o] >= n;
                            accw[px][o] += cn[px][o] >= n;
                        }
                    }
            }
#pragma unroll
            for (int px = 0; px < PX; px++)
#pragma unroll
                for (int o = 0; o < OT; o++) { cp[px][o] = 0; cn[px][o] = 0; }
        }
#pragma unroll
        for (int px = 0; px < PX; px++)
#pragma unroll
            for (int j = 0; j < KWZ; j++) a_cur[px][j] = a_nxt[px][j];
        w_q += w_chunk_words;
        slot = slot_n; ky = ky_n; zg = zg_n;
    }

    // epilogue: sum the NS partial tiles in LDS
    if (ns > 1) {
#pragma unroll
        for (int px = 0; px < PX; px++)
#pragma unroll
            for (int o = 0; o < OT; o++) {
                s_red[wave][0][px * OT + o][lane] = acc[px][o];
                if (WIDE) s_red[wave][1][px * OT + o][lane] = accw[px][o];
            }
        __syncthreads();
    }
    // Each wave finishes a contiguous group of OT/ns output channels, four at a time: in channels-last
    // order the four values of a lane are adjacent in memory and leave as one 8- or 16-byte store.
    const long plane = (long)p.splits * p.O_pad * p.M;
    const int group = OT / ns; // output channels per wave: 16, 8 or 4
#pragma unroll
    for (int px = 0; px < PX; px++) {
        const int m = mpix[px];
        const int n = m / p.HoWo, r = m - n * p.HoWo;
#pragma unroll
        for (int q = 0; q < OT / 4; q++) {
            if ((q * 4) / group != wave) continue; // wave-uniform
            uint32_t v[4], vw[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int o = q * 4 + e;
                v[e] = acc[px][o]; vw[e] = WIDE ? accw[px][o] : 0;
                if (ns > 1) {
                    v[e] = 0; vw[e] = 0;
                    for (int w = 0; w < ns; w++) {
                        if (WIDE) { v[e] += s_red[w][0][px * OT + o][lane]; vw[e] += s_red[w][1][px * OT + o][lane]; }
                        else v[e] = pk_add_u16(v[e], s_red[w][0][px * OT + o][lane]);
                    }
                }
            }
            if (m >= p.M) continue;
            const int oo = otile * OT + q * 4;
            if (p.direct) {
                if (p.out_channels_last && p.vec_out && oo + 3 < p.O) {
                    const long idx = (long)m * p.O + oo;
                    const uint2 vp = make_uint2((v[0] & 0xffffu) | (v[1] << 16), (v[2] & 0xffffu) | (v[3] << 16));
                    const uint2 vn = make_uint2((v[0] >> 16) | (v[1] & 0xffff0000u), (v[2] >> 16) | (v[3] & 0xffff0000u));
                    if (out_pos) *reinterpret_cast<uint2 *>(out_pos + idx) = vp;
                    if (out_neg) *reinterpret_cast<uint2 *>(out_neg + idx) = vn;
                    if (out_diff) {
                        const uint32_t d0 = (v[0] - (v[0] >> 16)) & 0xffffu, d1 = (v[1] - (v[1] >> 16)) & 0xffffu;
                        const uint32_t d2 = (v[2] - (v[2] >> 16)) & 0xffffu, d3 = (v[3] - (v[3] >> 16)) & 0xffffu;
                        *reinterpret_cast<uint2 *>(out_diff + idx) = make_uint2(d0 | (d1 << 16), d2 | (d3 << 16));
                    }
                    if (out_value)
                        *reinterpret_cast<float4 *>(out_value + idx) = make_float4(counts_value(v[0], p.inv_L), counts_value(v[1], p.inv_L),
                                                                                   counts_value(v[2], p.inv_L), counts_value(v[3], p.inv_L));
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if (oo + e >= p.O) continue;
                    const long idx = p.out_channels_last ? (long)m * p.O + oo + e : ((long)n * p.O + oo + e) * p.HoWo + r;
                    const int16_t vp = (int16_t)(v[e] & 0xffffu), vn = (int16_t)(v[e] >> 16);
                    if (out_pos) out_pos[idx] = vp;
                    if (out_neg) out_neg[idx] = vn;
                    if (out_diff) out_diff[idx] = (int16_t)(vp - vn);
                    if (out_value) out_value[idx] = counts_value(v[e], p.inv_L);
                }
            } else if (p.out_channels_last) {
                // partial sums of a global slot split, laid out like the final tensor so that the
                // finalize pass is coalesced on both sides: part[plane][split][m][o] for NHWC,
                // part[plane][split][o][m] for NCHW; plane 1 only in WIDE mode
                const long idx = ((long)split * p.M + m) * p.O_pad + oo; // multiple of 4
                if (!WIDE && p.part_narrow) {
                    uint32_t h[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) h[e] = (v[e] & 0xffu) | ((v[e] >> 8) & 0xff00u);
                    *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(part) + idx) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                } else {
                    *reinterpret_cast<uint4 *>(part + idx) = make_uint4(v[0], v[1], v[2], v[3]);
                    if (WIDE) *reinterpret_cast<uint4 *>(part + plane + idx) = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const long idx = ((long)split * p.O_pad + oo + e) * p.M + m;
                    if (!WIDE && p.part_narrow) reinterpret_cast<uint16_t *>(part)[idx] = (uint16_t)((v[e] & 0xffu) | ((v[e] >> 8) & 0xff00u));
                    else part[idx] = v[e];
                    if (WIDE) part[plane + idx] = vw[e];
                }
            }
        }
    }
}

// Sum the slot-split partials and write the final tensors.
// conv:   int16 pos / neg / diff, NCHW or NHWC, sums wrap at 16 bits like the reference's.
// linear: int32 pos / neg [M][O].
// IdxT: unsigned when O*M fits 32 bits (64-bit divisions are slow), unsigned long otherwise.
template <bool WIDE, typename OutT, typename IdxT>
__global__ __launch_bounds__(256) void sc_finalize_kernel(const uint32_t *__restrict__ part, ComputeParams p,
                                                          OutT *__restrict__ out_pos, OutT *__restrict__ out_neg,
                                                          OutT *__restrict__ out_diff, float *__restrict__ out_value)
{
    const IdxT total = (IdxT)p.O * (IdxT)p.M;
    const long plane = (long)p.splits * p.O_pad * p.M;
    const long split_stride = (long)p.O_pad * p.M;
    const uint16_t *part16 = reinterpret_cast<const uint16_t *>(part);
    for (IdxT i = (IdxT)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (IdxT)gridDim.x * blockDim.x) {
        // i runs in output memory order
        IdxT o, m;
        if (p.out_channels_last) { m = i / (IdxT)p.O; o = i - m * (IdxT)p.O; }
        else {
            const IdxT no = i / (IdxT)p.HoWo; // n*O + o
            const IdxT r = i - no * (IdxT)p.HoWo, n = no / (IdxT)p.O;
            o = no - n * (IdxT)p.O; m = n * (IdxT)p.HoWo + r;
        }
        const long idx0 = p.out_channels_last ? (long)m * p.O_pad + o : (long)o * p.M + m;
        uint32_t sp = 0, sn = 0;
        // the loads of all splits (at most 8 at a time) are issued before the first sum
        for (int s0 = 0; s0 < p.splits; s0 += 8) {
            uint32_t v[8], vw[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                v[u] = 0; vw[u] = 0;
                if (s0 + u < p.splits) {
                    const long idx = idx0 + (long)(s0 + u) * split_stride;
                    if (WIDE) { v[u] = part[idx]; vw[u] = part[plane + idx]; }
                    else v[u] = p.part_narrow ? (uint32_t)part16[idx] : part[idx];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (WIDE) { sp += v[u]; sn += vw[u]; }
                else if (p.part_narrow) { sp += v[u] & 0xffu; sn += v[u] >> 8; }
                else { sp += v[u] & 0xffffu; sn += v[u] >> 16; }
            }
        }
        const OutT vp = (OutT)sp, vn = (OutT)sn; // int16: wraps
        if (out_pos) out_pos[i] = vp;
        if (out_neg) out_neg[i] = vn;
        if (out_diff) out_diff[i] = (OutT)(vp - vn);
        if (out_value) out_value[i] = (float)(int16_t)vp * p.inv_L - (float)(int16_t)vn * p.inv_L; // conv op only
    }
}

// Finalize for channels-last int16 results with narrow (uint16) partials and O % 4 == 0: a thread sums
// four adjacent output channels (one 8-byte load per split) and writes 8 bytes per tensor.
__global__ __launch_bounds__(256) void sc_finalize_nhwc4_kernel(const uint32_t *__restrict__ part, ComputeParams p,
                                                                int16_t *__restrict__ out_pos, int16_t *__restrict__ out_neg,
                                                                int16_t *__restrict__ out_diff, float *__restrict__ out_value)
{
    const unsigned o4 = (unsigned)p.O / 4;
    const unsigned total = (unsigned)p.M * o4;
    const long split_stride = (long)p.O_pad * p.M; // in uint16 elements
    const uint16_t *part16 = reinterpret_cast<const uint16_t *>(part);
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const unsigned m = i / o4, q = i - m * o4;
        const long idx0 = (long)m * p.O_pad + q * 4;
        uint32_t sp[4] = {0, 0, 0, 0}, sn[4] = {0, 0, 0, 0};
        for (int s0 = 0; s0 < p.splits; s0 += 8) {
            uint2 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                v[u] = make_uint2(0, 0);
                if (s0 + u < p.splits) v[u] = *reinterpret_cast<const uint2 *>(part16 + idx0 + (long)(s0 + u) * split_stride);
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                sp[0] += v[u].x & 0xffu; sn[0] += (v[u].x >> 8) & 0xffu;
                sp[1] += (v[u].x >> 16) & 0xffu; sn[1] += v[u].x >> 24;
                sp[2] += v[u].y & 0xffu; sn[2] += (v[u].y >> 8) & 0xffu;
                sp[3] += (v[u].y >> 16) & 0xffu; sn[3] += v[u].y >> 24;
            }
        }
        const long o_idx = (long)m * p.O + q * 4;
        if (out_pos) *reinterpret_cast<uint2 *>(out_pos + o_idx) = make_uint2((sp[0] & 0xffffu) | (sp[1] << 16), (sp[2] & 0xffffu) | (sp[3] << 16));
        if (out_neg) *reinterpret_cast<uint2 *>(out_neg + o_idx) = make_uint2((sn[0] & 0xffffu) | (sn[1] << 16), (sn[2] & 0xffffu) | (sn[3] << 16));
        if (out_diff) {
            uint32_t d[4];
#pragma unroll
            for (int e = 0; e < 4; e++) d[e] = (sp[e] - sn[e]) & 0xffffu;
            *reinterpret_cast<uint2 *>(out_diff + o_idx) = make_uint2(d[0] | (d[1] << 16), d[2] | (d[3] << 16));
        }
        if (out_value) {
            float f[4];
#pragma unroll
            for (int e = 0; e < 4; e++) f[e] = (float)(int16_t)sp[e] * p.inv_L - (float)(int16_t)sn[e] * p.inv_L;
            *reinterpret_cast<float4 *>(out_value + o_idx) = make_float4(f[0], f[1], f[2], f[3]);
        }
    }
}

// Generic fallback for kernel widths without a tuned instance: one output per thread, runtime loops.
__global__ __launch_bounds__(256) void sc_compute_generic_kernel(const uint32_t *__restrict__ A,
                                                                 const uint32_t *__restrict__ Wst, ComputeParams p,
                                                                 int KW, int ZC, int16_t *__restrict__ out_pos,
                                                                 int16_t *__restrict__ out_neg,
                                                                 int16_t *__restrict__ out_diff, float *__restrict__ out_value)
{
    const long total = (long)p.O * p.M;
    const int KWZ = KW * ZC;
    const uint32_t n_sat = p.nn & 0xffffu;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int o = (int)(i / p.M), m = (int)(i - (long)o * p.M);
        const int n = m / p.HoWo, r = m - n * p.HoWo;
        const int yo = r / p.Wo, xo = r - yo * p.Wo;
        const long abase = ((((long)n * p.ZG) * p.Hp + yo * p.s0) * p.Wp + xo * p.s1) * ZC;
        uint32_t sp = 0, sn = 0;
        for (int slot = 0; slot < p.n_slots; slot++) {
            uint32_t cp = 0, cn = 0;
            for (int ky = 0; ky < p.KH; ky++)
                for (int zg = 0; zg < p.ZG; zg++) {
                    const uint32_t *ap = A + (long)slot * p.a_slot_stride + abase + ((long)zg * p.Hp + ky) * p.Wp * ZC;
                    const uint32_t *wc = Wst + ((((long)slot * p.KH + ky) * p.ZG + zg) * p.O_pad + o) * 2 * KWZ;
                    for (int j = 0; j < KWZ; j++) {
                        cp += __builtin_popcount(ap[j] & wc[j]);
                        cn += __builtin_popcount(ap[j] & wc[KWZ + j]);
                    }
                }
            sp += min(cp, n_sat); sn += min(cn, n_sat);
        }
        const long idx = p.out_channels_last ? (long)m * p.O + o : ((long)n * p.O + o) * p.HoWo + r;
        const int16_t vp = (int16_t)sp, vn = (int16_t)sn;
        if (out_pos) out_pos[idx] = vp;
        if (out_neg) out_neg[idx] = vn;
        if (out_diff) out_diff[idx] = (int16_t)(vp - vn);
        if (out_value) out_value[idx] = (float)vp * p.inv_L - (float)vn * p.inv_L;
    }
}

// ---- host side ---------------------------------------------------------------------------------
template <int KW, int ZC, int PX, int OT, int MODE>
static int launch_compute(const uint32_t *A, const uint32_t *Wst, ComputeParams p, uint32_t *part, int16_t *out_pos,
                          int16_t *out_neg, int16_t *out_diff, float *out_value, hipStream_t stream)
{
    p.m_tiles = ceil_div(p.M, 64 * PX);
    p.o_tiles = p.O_pad / OT;
    // 8-byte stores of four adjacent int16 results need O % 4 == 0 and 8-byte aligned tensors
    p.vec_out = (p.O % 4 == 0 && ((uintptr_t)out_pos % 8) == 0 && ((uintptr_t)out_neg % 8) == 0 &&
                 ((uintptr_t)out_diff % 8) == 0 && ((uintptr_t)out_value % 16) == 0) ? 1 : 0;
    REXSC_CHECK_ARG(p.ns >= 1 && p.ns <= MAX_NS, "SC compute: %d waves per block not supported", p.ns);
    const long blocks = (long)p.m_tiles * p.o_tiles * p.splits;
    REXSC_CHECK_ARG(blocks < (1L << 30), "SC compute: grid too large (%ld blocks)", blocks);
    const int grid = (int)align_up((size_t)blocks, 8);
    // built once per instance; initialisation of a function-local static is thread-safe
    static const std::string name_str = [] {
        char b[64];
        snprintf(b, sizeof(b), "sc_compute<%d,%d,%d,%d,%d>", KW, ZC, PX, OT, MODE);
        return std::string(b);
    }();
    const char *name = name_str.c_str();
    // algorithmic lane-ops: (and + popcount-accumulate) x 2 polarities per 32-channel word
    ProfScope prof(name, 4.0 * p.M * p.O * p.KH * KW * p.Z * p.n_slots, stream);
    hipLaunchKernelGGL((sc_compute_kernel<KW, ZC, PX, OT, MODE>), dim3(grid), dim3(64 * p.ns), 0, stream, A, Wst, p, part,
                       out_pos, out_neg, out_diff, out_value);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sc_compute_tile_ot() { return 16; }

bool sc_compute_has_instance(int KW, int ZC)
{
    if (KW == 1) return ZC == 1 || ZC == 2 || ZC == 4 || ZC == 8;
    if (KW == 3) return ZC == 1 || ZC == 2 || ZC == 4;
    if (KW == 5 || KW == 7) return ZC == 1 || ZC == 2;
    return false;
}

int sc_compute(const uint32_t *A, const uint32_t *Wst, const ComputeParams &p, int KW, int ZC, bool wide,
               uint32_t *part, int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, float *out_value, hipStream_t stream)
{
    const int px = p.px;
    // saturation at one: the and-or instances (not in WIDE mode, whose sums are not packed)
    const bool or1 = !wide && (p.nn & 0xffffu) == 1u;
#define REXSC_INST_OT(KW_, ZC_, OT_)                                                                              \
    if (KW == KW_ && ZC == ZC_ && p.ot == OT_) {                                                                  \
        if (or1) {                                                                                                \
            if (px == 2) return launch_compute<KW_, ZC_, 2, OT_, 2>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream); \
            return launch_compute<KW_, ZC_, 1, OT_, 2>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream);     \
        }                                                                                                         \
        if (px == 2) return launch_compute<KW_, ZC_, 2, OT_, 0>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream); \
        return launch_compute<KW_, ZC_, 1, OT_, 0>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream);         \
    }
#define REXSC_INST(KW_, ZC_) REXSC_INST_OT(KW_, ZC_, 16)
    if (wide) {
        REXSC_CHECK_ARG(KW == 1 && (ZC == 4 || ZC == 8), "wide accumulation is only built for 1x1 / linear shapes");
        if (ZC == 4) return launch_compute<1, 4, 1, 16, 1>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream);
        return launch_compute<1, 8, 1, 16, 1>(A, Wst, p, part, out_pos, out_neg, out_diff, out_value, stream);
    }
    REXSC_INST(1, 1) REXSC_INST(1, 2) REXSC_INST(1, 4) REXSC_INST(1, 8)
    REXSC_INST(3, 1) REXSC_INST(3, 2) REXSC_INST(3, 4)
    REXSC_INST(5, 1) REXSC_INST(5, 2)
    REXSC_INST(7, 1) REXSC_INST(7, 2)
#undef REXSC_INST
#undef REXSC_INST_OT
    set_error("SC compute: no kernel instance for KW=%d ZC=%d", KW, ZC);
    return REXSC_ERR_INVALID;
}

int sc_compute_generic(const uint32_t *A, const uint32_t *Wst, const ComputeParams &p, int KW, int ZC,
                       int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, float *out_value, hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    ProfScope prof("sc_compute_generic", 4.0 * p.M * p.O * p.KH * KW * p.Z * p.n_slots, stream);
    hipLaunchKernelGGL(sc_compute_generic_kernel, dim3(grid), dim3(256), 0, stream, A, Wst, p, KW, ZC, out_pos,
                       out_neg, out_diff, out_value);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sc_finalize_i16(const uint32_t *part, const ComputeParams &p, int16_t *out_pos, int16_t *out_neg,
                    int16_t *out_diff, float *out_value, hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    const double out_bytes = (out_pos ? 2.0 : 0.0) + (out_neg ? 2.0 : 0.0) + (out_diff ? 2.0 : 0.0) + (out_value ? 4.0 : 0.0);
    ProfScope prof("sc_finalize_i16", (double)total * ((p.part_narrow ? 2.0 : 4.0) * p.splits + out_bytes), stream);
    const bool aligned8 = ((uintptr_t)out_pos % 8) == 0 && ((uintptr_t)out_neg % 8) == 0 && ((uintptr_t)out_diff % 8) == 0 &&
                          ((uintptr_t)out_value % 16) == 0;
    if (p.out_channels_last && p.part_narrow && p.O % 4 == 0 && aligned8 && total < (1L << 31)) {
        const long t4 = total / 4;
        const int grid4 = (int)((t4 + 255) / 256 < 16384 ? (t4 + 255) / 256 : 16384);
        hipLaunchKernelGGL(sc_finalize_nhwc4_kernel, dim3(grid4), dim3(256), 0, stream, part, p, out_pos, out_neg, out_diff,
                           out_value);
    } else if (total < (1L << 31))
        hipLaunchKernelGGL((sc_finalize_kernel<false, int16_t, unsigned>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                           out_neg, out_diff, out_value);
    else
        hipLaunchKernelGGL((sc_finalize_kernel<false, int16_t, unsigned long>), dim3(grid), dim3(256), 0, stream, part, p,
                           out_pos, out_neg, out_diff, out_value);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sc_finalize_i32(const uint32_t *part, const ComputeParams &p, bool wide, int32_t *out_pos, int32_t *out_neg,
                    hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    ProfScope prof("sc_finalize_i32", (double)total * (4.0 * p.splits * (wide ? 2 : 1) + 8.0), stream);
    REXSC_CHECK_ARG(total < (1L << 31), "linear: too many outputs (%ld)", total);
    if (wide)
        hipLaunchKernelGGL((sc_finalize_kernel<true, int32_t, unsigned>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                           out_neg, (int32_t *)nullptr, (float *)nullptr);
    else
        hipLaunchKernelGGL((sc_finalize_kernel<false, int32_t, unsigned>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                           out_neg, (int32_t *)nullptr, (float *)nullptr);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

} // namespace rexsc
