// Saturating fixed-point conv2d (fixed.cpp:56-238).
//
// Two paths:
//  * closed form (add_config 0): with non-negative products the saturating, rounding add of
//    fixed.cpp:56-64 does not depend on the order of the products:
//        d = max(0, 2*pin - pout) == 0:  sum_pol = min( sum(p + (p & 1)), max_value + 1 )
//        d > 0:                          sum_pol = min( sum(round_half_up_d(p)), max_value )
//    (every partial sum is a multiple of 2^d, so rounding distributes over the sum, and once the
//    clamp fires it keeps firing).  This path works on int8/int16 operands quantised once.
//  * sequential (add_config >= 1): the OR-style adders are order dependent and are evaluated
//    product by product in the reference's (c, ky, kx) order.
#include <stdlib.h>
#include <atomic>
#include "profile.h"
#include "rexsc_common.h"

namespace rexsc {

struct FixedParams {
    int N, C, H, W, O, KH, KW;
    int pad_h, pad_w, s0, s1;
    int Ho, Wo;
    int add_config, pin, d, max_value;
    float P2;
};

__device__ __forceinline__ int quant_round_pos(float v, float S)
{   // round(clamp(v*S, 0, S-1)), half to even (fixed.cpp:208-209)
    float t = v * S;
    t = fminf(fmaxf(t, 0.f), S - 1.f);
    return (int)rintf(t);
}
__device__ __forceinline__ int quant_round_neg(float v, float S)
{   // round(-clamp(v*S, 1-S, 0)) (fixed.cpp:210)
    float t = v * S;
    t = fminf(fmaxf(t, 1.f - S), 0.f);
    return (int)rintf(-t);
}

__device__ __forceinline__ int saturate_shift(int value, int max_value, int d)
{   // fixed.cpp:56-60
    const int vs = min(value, max_value);
    const int round_bit = (vs >> max(0, d - 1)) % 2;
    return ((vs >> d) + round_bit) << d;
}

// Quantise operands once: activations -> int32 [N][C][H][W] (unpadded), weights -> signed int32
// (positive part - negative part; at most one of them is non-zero).
__global__ __launch_bounds__(256) void fixed_quant_kernel(const float *__restrict__ x, int32_t *__restrict__ q, size_t n,
                                                          float S, int is_weight)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float v = x[i];
        q[i] = is_weight ? quant_round_pos(v, S) - quant_round_neg(v, S) : quant_round_pos(v, S);
    }
}

// One output per thread; lanes run along xo so activation loads coalesce and the weight is
// wave-uniform whenever a wave stays inside one (n, o) plane.
template <int ADD>
__global__ __launch_bounds__(256) void fixed_conv_kernel(const int32_t *__restrict__ xq, const int32_t *__restrict__ wq,
                                                         int32_t *__restrict__ out, FixedParams p)
{
    const long total = (long)p.N * p.O * p.Ho * p.Wo;
    const long stride = (long)gridDim.x * blockDim.x;
    const int KK = p.KH * p.KW;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int xo = (int)(i % p.Wo);
        const int yo = (int)((i / p.Wo) % p.Ho);
        const int o = (int)((i / ((long)p.Wo * p.Ho)) % p.O);
        const int n = (int)(i / ((long)p.Wo * p.Ho * p.O));
        const int32_t *xb = xq + (long)n * p.C * p.H * p.W;
        const int32_t *wb = wq + (long)o * p.C * KK;
        const int y0 = yo * p.s0 - p.pad_h, x0 = xo * p.s1 - p.pad_w;
        int result;
        if (ADD == 0) {
            // closed form, both polarities at once
            long sp = 0, sn = 0;
            const int half = p.d > 0 ? (1 << (p.d - 1)) : 0;
            for (int c = 0; c < p.C; c++)
                for (int ky = 0; ky < p.KH; ky++) {
                    const int yy = y0 + ky;
                    if (yy < 0 || yy >= p.H) continue;
                    for (int kx = 0; kx < p.KW; kx++) {
                        const int xx = x0 + kx;
                        if (xx < 0 || xx >= p.W) continue;
                        const int a = xb[((long)c * p.H + yy) * p.W + xx];
                        const int w = wb[(c * p.KH + ky) * p.KW + kx];
                        const int pr = a * (w < 0 ? -w : w);
                        const int r = p.d == 0 ? pr + (pr & 1) : (((pr + half) >> p.d) << p.d);
                        if (w < 0) sn += r; else sp += r;
                    }
                }
            const long cap = p.d == 0 ? (long)p.max_value + 1 : (long)p.max_value;
            result = (int)min(sp, cap) - (int)min(sn, cap);
        } else if (ADD == 1) {
            int sp = 0, sn = 0;
            for (int c = 0; c < p.C; c++)
                for (int ky = 0; ky < p.KH; ky++)
                    for (int kx = 0; kx < p.KW; kx++) {
                        const int yy = y0 + ky, xx = x0 + kx;
                        int a = 0;
                        if (yy >= 0 && yy < p.H && xx >= 0 && xx < p.W) a = xb[((long)c * p.H + yy) * p.W + xx];
                        const int w = wb[(c * p.KH + ky) * p.KW + kx];
                        const int pp = a * (w > 0 ? w : 0), pn = a * (w < 0 ? -w : 0);
                        // fixed_add_or, fixed.cpp:67-70
                        sp = saturate_shift(sp + pp - ((sp * pp) >> (p.pin * 2)), p.max_value, p.d);
                        sn = saturate_shift(sn + pn - ((sn * pn) >> (p.pin * 2)), p.max_value, p.d);
                    }
            result = sp - sn;
        } else {
            // pairwise OR2 model, fixed.cpp:71-78, 150-190
            int p1 = 0, p2 = 0, n1 = 0, n2 = 0;
            const int total_k = p.C * KK;
            const int sh4 = p.pin * 4, sh6 = p.pin * 6;
            for (int k = 0; k < total_k; k += 2) {
                int a[2] = {0, 0}, w[2] = {0, 0};
                for (int j = 0; j < 2; j++) {
                    const int kk = k + j;
                    if (kk >= total_k) break;
                    const int c = kk / KK, ky = (kk % KK) / p.KW, kx = kk % p.KW;
                    const int yy = y0 + ky, xx = x0 + kx;
                    if (yy >= 0 && yy < p.H && xx >= 0 && xx < p.W) a[j] = xb[((long)c * p.H + yy) * p.W + xx];
                    w[j] = wb[kk];
                }
                for (int pol = 0; pol < 2; pol++) {
                    const long b1 = pol == 0 ? a[0] * (w[0] > 0 ? w[0] : 0) : a[0] * (w[0] < 0 ? -w[0] : 0);
                    const long b2 = pol == 0 ? a[1] * (w[1] > 0 ? w[1] : 0) : a[1] * (w[1] < 0 ? -w[1] : 0);
                    const long a1 = pol == 0 ? p1 : n1, a2 = pol == 0 ? p2 : n2;
                    int o1 = (int)a1 + (int)b1 - (int)((a1 * a2 * b2) >> sh4) - (int)((a2 * b1 * b2) >> sh4) +
                             (int)((a1 * a2 * b1 * b2) >> sh6);
                    int o2 = (int)a2 + (int)b2 - (int)((a1 * a2 * b1) >> sh4) - (int)((a1 * b1 * b2) >> sh4) +
                             (int)((a1 * a2 * b1 * b2) >> sh6);
                    o1 = saturate_shift(o1, p.max_value, p.d);
                    o2 = saturate_shift(o2, p.max_value, p.d);
                    if (pol == 0) { p1 = o1; p2 = o2; } else { n1 = o1; n2 = o2; }
                }
            }
            result = p1 + p2 - n1 - n2;
        }
        out[i] = result;
    }
}


// ---- int8 MFMA path for the closed form ----------------------------------------------------------
// Valid when add_config = 0, d = 0, operands fit int8 (precision_in <= 7) and the clamp cannot fire
// (C*KH*KW*((2^pin-1)^2+1) < max_value+1).  Then pos - neg collapses to ONE signed contraction plus
// a parity term:   out = sum a*w  +  sum (a&1) * sgn(w)*(|w|&1).
//
// Operands are re-laid-out once, channel-blocked by 16 so that every MFMA operand fetch is one
// 16-byte load and adjacent lanes read adjacent memory:
//   xq16[n][cb][yp][xp][16]     int8 activations over the zero-padded plane
//   wq16[cb][ky][kx][o_pad][16] int8 signed weights;  wp16 (same shape) = sgn(w)*(|w|&1)
// The activation parities are not stored: a&1 is one v_and on the loaded bytes.
// GEMM orientation: MFMA rows = output channels (weights are the A operand), MFMA columns = pixels
// (activations are the B operand): the 32 lanes of a half-wave hold 32 consecutive pixels of one
// output channel, so the int32 NCHW stores are 128-byte runs.
// v_mfma_i32_32x32x32_i8: lane l feeds row/column l%32 with k = 16*(l/32) .. +15, i.e. the two
// half-waves take two consecutive 16-channel blocks; D[i][j] sits in lane (j + 32*((i/4)%2)),
// register 4*(i/8) + i%4.
typedef int v16i __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));

struct Fixed8Params {
    int N, C, H, W, O, O_pad, KH, KW;
    int pad_h, pad_w, s0, s1, Hp, Wp, Ho, Wo;
    int CB;      // 16-channel blocks, padded to an even count
    int M;       // N*Ho*Wo
    int ksplit;  // blocks of the reduction handled by different waves (results added atomically)
    float P2;
};

__device__ __forceinline__ void fixed_pack_act16(const float *__restrict__ x, int8_t *__restrict__ xq16,
                                                 const Fixed8Params &p, unsigned bid)
{
    // one thread per (n, cb, yp, xp), counted over the whole tensor so that small planes waste no lanes:
    // 16 channels -> 16 bytes.  Lanes of a wave are neighbouring pixels: each of the 16 loads is coalesced.
    const unsigned plane = (unsigned)p.Hp * p.Wp;
    const unsigned total = (unsigned)p.N * p.CB * plane; // the host checks that this fits 32 bits
    const unsigned t = bid * 256 + threadIdx.x;
    if (t >= total) return;
    const unsigned ncb = t / plane, i = t - ncb * plane;
    const unsigned n = ncb / (unsigned)p.CB, cb = ncb - n * (unsigned)p.CB;
    const long in_plane = (long)p.H * p.W;
    const unsigned yp = i / (unsigned)p.Wp, xp = i - yp * (unsigned)p.Wp;
    const int y = (int)yp - p.pad_h, xx = (int)xp - p.pad_w;
    const bool inb = y >= 0 && y < p.H && xx >= 0 && xx < p.W;
    const float *src = x + ((long)n * p.C + cb * 16) * in_plane + (long)y * p.W + xx;
    float f[16];
#pragma unroll
    for (int k = 0; k < 16; k++) f[k] = (inb && (int)(cb * 16 + k) < p.C) ? src[k * in_plane] : 0.f;
    uint32_t wds[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < 16; k++) wds[k >> 2] |= (uint32_t)(uint8_t)quant_round_pos(f[k], p.P2) << (8 * (k & 3));
    reinterpret_cast<uint4 *>(xq16)[t] = make_uint4(wds[0], wds[1], wds[2], wds[3]);
}

__device__ __forceinline__ void fixed_pack_w16(const float *__restrict__ w, int8_t *__restrict__ wq16,
                                               int8_t *__restrict__ wp16, const Fixed8Params &p, unsigned bid,
                                               unsigned n_blocks)
{
    // one thread per (cb, o, tap), tap fastest: the threads of one (cb, o) read one contiguous run of
    // the OIHW weights (16 channels x KH*KW taps) between them; each writes its 16-byte entries.
    const unsigned taps = (unsigned)(p.KH * p.KW);
    const unsigned total = (unsigned)p.CB * p.O_pad * taps;
    for (unsigned i = bid * 256 + threadIdx.x; i < total; i += n_blocks * 256) {
        const unsigned tap = i % taps, co = i / taps;
        const unsigned o = co % (unsigned)p.O_pad, cb = co / (unsigned)p.O_pad;
        uint32_t vals[4] = {0, 0, 0, 0}, pars[4] = {0, 0, 0, 0};
        if ((int)o < p.O) {
            const float *src = w + ((long)o * p.C + cb * 16) * taps + tap;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                if ((int)(cb * 16 + k) < p.C) {
                    const float f = src[(long)k * taps];
                    const int q = quant_round_pos(f, p.P2) - quant_round_neg(f, p.P2); // signed
                    const int par = (q & 1) ? (q < 0 ? -1 : 1) : 0;
                    vals[k >> 2] |= (uint32_t)(uint8_t)(int8_t)q << (8 * (k & 3));
                    pars[k >> 2] |= (uint32_t)(uint8_t)(int8_t)par << (8 * (k & 3));
                }
            }
        }
        const long dst = ((long)cb * taps + tap) * p.O_pad + o;
        reinterpret_cast<uint4 *>(wq16)[dst] = make_uint4(vals[0], vals[1], vals[2], vals[3]);
        reinterpret_cast<uint4 *>(wp16)[dst] = make_uint4(pars[0], pars[1], pars[2], pars[3]);
    }
}

// One launch prepares everything the MFMA kernel needs: the first w_blocks blocks pack the weights, the next
// act_blocks pack the activations, the last zero_blocks clear the output when the reduction is split
// over blocks that add their parts atomically.  (Three launches of this size cost more in launch
// latency than in work.)
__global__ __launch_bounds__(256) void fixed_prepare_kernel(const float *__restrict__ x, int8_t *__restrict__ xq16,
                                                            const float *__restrict__ w, int8_t *__restrict__ wq16,
                                                            int8_t *__restrict__ wp16, int32_t *__restrict__ out,
                                                            size_t n_out, Fixed8Params p, unsigned act_blocks,
                                                            unsigned w_blocks, unsigned zero_blocks)
{
    // the few weight blocks come first in the grid: their strided loads then run beside the activation blocks
    // instead of forming a round of their own at the end of the launch
    unsigned bid = blockIdx.x;
    if (bid < w_blocks) { fixed_pack_w16(w, wq16, wp16, p, bid, w_blocks); return; }
    bid -= w_blocks;
    if (bid < act_blocks) { fixed_pack_act16(x, xq16, p, bid); return; }
    bid -= act_blocks;
    if ((reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        uint4 *o4 = reinterpret_cast<uint4 *>(out);
        const size_t n4 = n_out / 4;
        for (size_t i = (size_t)bid * 256 + threadIdx.x; i < n4; i += (size_t)zero_blocks * 256) o4[i] = make_uint4(0, 0, 0, 0);
        if (bid == 0 && threadIdx.x < (n_out & 3)) out[n4 * 4 + threadIdx.x] = 0;
    } else {
        for (size_t i = (size_t)bid * 256 + threadIdx.x; i < n_out; i += (size_t)zero_blocks * 256) out[i] = 0;
    }
}

// A block of 4 waves computes a 64 (channels) x 256 (pixels) tile over its share of the channel-block
// pairs; each wave owns 64 pixels.  The weights of one pair (both half-wave blocks, all taps, values
// and parities) are staged in LDS once per block and read with ds_read_b128, so they cost L2
// bandwidth once per 256 pixels instead of once per 64.  Per kernel row all KW taps are loaded
// first, then the 8*KW MFMAs run: one exposed memory latency per row instead of one per tap.
// PB: 32-pixel blocks per wave.  Two blocks reuse every weight fetch twice; one block makes waves half
// as long and lighter on registers, which the launcher prefers when the pixel count leaves the
// last round of 64-pixel waves nearly empty.
constexpr int FT = 64;
template <int KW, int PB>
__global__ __launch_bounds__(256) void fixed_mfma_kernel(const int8_t *__restrict__ xq16, const int8_t *__restrict__ wq16,
                                                         const int8_t *__restrict__ wp16, int32_t *__restrict__ out,
                                                         Fixed8Params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t s_raw[];
    v4i *s_w = reinterpret_cast<v4i *>(s_raw); // [h][tap][val/par][o 0..63]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int o_tiles = p.O_pad / FT;
    constexpr int WPX = 32 * PB; // pixels per wave
    long blk = blockIdx.x;
    const int ks = (int)(blk % p.ksplit); blk /= p.ksplit;
    const int otile = (int)(blk % o_tiles);
    const long mtile = (blk / o_tiles) * 4 + wave;   // may be past the end: such a wave only helps staging
    const int j = lane & 31, h = lane >> 5;
    const long plane = (long)p.Hp * p.Wp;
    const int taps = p.KH * KW;

    long xoff[PB];
    int mm[PB];
#pragma unroll
    for (int pb = 0; pb < PB; pb++) {
        const long m = mtile * WPX + pb * 32 + j;
        mm[pb] = (int)(m < p.M ? m : p.M - 1);
        const int n = mm[pb] / (p.Ho * p.Wo), r = mm[pb] - n * (p.Ho * p.Wo);
        const int yo = r / p.Wo, xo = r - yo * p.Wo;
        xoff[pb] = (long)n * p.CB * plane + (long)(yo * p.s0) * p.Wp + xo * p.s1;
        if (m >= p.M) mm[pb] = -1;
    }
    const v4i *xb = reinterpret_cast<const v4i *>(xq16);
    const v4i *wb = reinterpret_cast<const v4i *>(wq16);
    const v4i *wpb = reinterpret_cast<const v4i *>(wp16);
    const long wkk = (long)taps * p.O_pad;

    v16i acc[2][PB]; // [channel block][pixel block]
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < PB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    const int pairs = p.CB / 2;
    const int per = (pairs + p.ksplit - 1) / p.ksplit;
    const int cbp_begin = ks * per, cbp_end = min(pairs, cbp_begin + per);
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    // Activation rows are software-pipelined: the KW taps of the next (pair, ky) row are requested
    // before the MFMAs of the current row are issued.
    v4i bc[PB][KW], bn[PB][KW];
    if (cbp_begin < cbp_end) {
        const v4i *xc = xb + (long)(2 * cbp_begin + h) * plane;
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int kx = 0; kx < KW; kx++) bc[pb][kx] = xc[xoff[pb] + kx];
    }
    for (int cbp = cbp_begin; cbp < cbp_end; cbp++) {
        // stage the pair's weights: 2 (h) x taps x 2 (val, par) x 64 (o) 16-byte entries
        __syncthreads();
        for (int e = threadIdx.x; e < 2 * taps * 2 * FT; e += 256) {
            const int o = e % FT, vp = (e / FT) % 2, tap = (e / (2 * FT)) % taps, hh = e / (2 * FT * taps);
            const long src = (long)(2 * cbp + hh) * wkk + (long)tap * p.O_pad + otile * FT + o;
            s_w[e] = vp ? wpb[src] : wb[src];
        }
        __syncthreads();
        const v4i *sw = s_w + (long)h * taps * 2 * FT + j;
        for (int ky = 0; ky < p.KH; ky++) {
            {
                // next row: (cbp, ky+1), or row 0 of the next pair; the very last row re-reads itself
                int cn = cbp, kn = ky + 1;
                if (kn == p.KH) { kn = 0; cn = cbp + 1; }
                if (cn >= cbp_end) { cn = cbp; kn = ky; }
                const v4i *xn = xb + (long)(2 * cn + h) * plane + (long)kn * p.Wp;
#pragma unroll
                for (int pb = 0; pb < PB; pb++)
#pragma unroll
                    for (int kx = 0; kx < KW; kx++) bn[pb][kx] = xn[xoff[pb] + kx];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kx = 0; kx < KW; kx++) {
                const v4i *wt = sw + (ky * KW + kx) * 2 * FT;
                const v4i a0 = wt[0], a1 = wt[32], q0 = wt[FT], q1 = wt[FT + 32];
#pragma unroll
                for (int pb = 0; pb < PB; pb++) {
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bc[pb][kx], acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bc[pb][kx], acc[1][pb], 0, 0, 0);
                }
#pragma unroll
                for (int pb = 0; pb < PB; pb++) {
                    const v4i par = bc[pb][kx] & ones; // activation parities
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q0, par, acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q1, par, acc[1][pb], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++) bc[pb][kx] = bn[pb][kx];
        }
    }
    const int HoWo = p.Ho * p.Wo;
#pragma unroll
    for (int pb = 0; pb < PB; pb++) {
        if (mm[pb] < 0) continue;
        const int n = mm[pb] / HoWo, r0 = mm[pb] - n * HoWo;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int o = otile * FT + a * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                if (o >= p.O) continue;
                int32_t *dst = out + ((long)n * p.O + o) * HoWo + r0;
                if (p.ksplit == 1) *dst = acc[a][pb][r];
                else atomicAdd(dst, acc[a][pb][r]); // integer adds commute: the split is exact
            }
    }
}

// Persistent variant for KH x KW known at compile time: a block walks over its work items
// (256-pixel group, 64-channel tile, share of the channel-block pairs) and over the pairs of each item
// with the weights double-buffered in LDS: the 16-byte entries of the next pair are requested from L2
// before the MFMAs of the current pair are issued and written to the other buffer after them, so a
// pair costs one barrier and no exposed staging latency.  A buffer that already holds the pair it is
// asked for is left alone: with one or two pairs and one channel tile (C <= 64, O <= 64) the weights
// stay resident for the whole launch.
template <int KH, int KW, int PB>
__global__ __launch_bounds__(256) void fixed_mfma_db_kernel(const int8_t *__restrict__ xq16, const int8_t *__restrict__ wq16,
                                                            const int8_t *__restrict__ wp16, int32_t *__restrict__ out,
                                                            Fixed8Params p, int n_items)
{
    constexpr int TAPS = KH * KW;
    constexpr int ENT = 2 * TAPS * 2 * FT; // 16-byte entries of one pair: [h][tap][val/par][o 0..63]
    static_assert(ENT % 256 == 0, "entries must divide among the threads");
    constexpr int EPT = ENT / 256;
    constexpr int WPX = 32 * PB;
    extern __shared__ __attribute__((aligned(16))) uint8_t s_raw[];
    v4i *s_w = reinterpret_cast<v4i *>(s_raw); // two buffers of ENT entries
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, h = lane >> 5;
    const int o_tiles = p.O_pad / FT;
    const long plane = (long)p.Hp * p.Wp;
    const int HoWo = p.Ho * p.Wo;
    const v4i *xb = reinterpret_cast<const v4i *>(xq16);
    const v4i *wb = reinterpret_cast<const v4i *>(wq16);
    const v4i *wpb = reinterpret_cast<const v4i *>(wp16);
    const long wkk = (long)TAPS * p.O_pad;
    const int pairs = p.CB / 2;
    const int per = (pairs + p.ksplit - 1) / p.ksplit;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

    // where thread t's e-th entry of pair (otile, cbp) comes from
    auto entry_src = [&](int e, int otile, int cbp, bool &is_par) -> long {
        const int o = e % FT, vp = (e / FT) % 2, tap = (e / (2 * FT)) % TAPS, hh = e / (2 * FT * TAPS);
        is_par = vp != 0;
        return (long)(2 * cbp + hh) * wkk + (long)tap * p.O_pad + otile * FT + o;
    };

    int held0 = -1, held1 = -1; // pair id (otile * pairs + cbp) in each buffer; block-uniform
    int step = 0;

    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        int t = item;
        const int ks = t % p.ksplit; t /= p.ksplit;
        const int otile = t % o_tiles;
        const long mtile = (long)(t / o_tiles) * 4 + wave;
        const int cbp_begin = ks * per, cbp_end = min(pairs, cbp_begin + per);
        // the next item's first pair, for the prefetch across the item boundary
        int n_otile = -1, n_cbp = -1;
        if (item + (int)gridDim.x < n_items) {
            int u = item + gridDim.x;
            const int nks = u % p.ksplit; u /= p.ksplit;
            n_otile = u % o_tiles; n_cbp = nks * per;
            if (n_cbp >= pairs) n_otile = -1;
        }

        long xoff[PB];
        int mm[PB];
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            const long m = mtile * WPX + pb * 32 + j;
            mm[pb] = (int)(m < p.M ? m : p.M - 1);
            const int n = mm[pb] / HoWo, r = mm[pb] - n * HoWo;
            const int yo = r / p.Wo, xo = r - yo * p.Wo;
            xoff[pb] = (long)n * p.CB * plane + (long)(yo * p.s0) * p.Wp + xo * p.s1;
            if (m >= p.M) mm[pb] = -1;
        }
        v16i acc[2][PB];
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < PB; b++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

        // Activation rows (one per (pair, ky)) run through a ring of KH register sets: row r lives in set
        // r % KH = ky, and the row two steps ahead is requested before the MFMAs of the current row, so a
        // load has two rows of MFMAs (and the other wave's) to arrive.
        static_assert(KH >= 3, "the ring holds the current row and two rows in flight");
        v4i rows[KH][PB][KW];
        const int n_rows = (cbp_end - cbp_begin) * KH;
        auto load_row = [&](int r, v4i (&dst)[PB][KW]) {
            r = r < n_rows ? r : n_rows - 1; // past the end: re-read the last row (harmless)
            const int cb = cbp_begin + r / KH, ky = r - (r / KH) * KH;
            const v4i *xr = xb + (long)(2 * cb + h) * plane + (long)ky * p.Wp;
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int kx = 0; kx < KW; kx++) dst[pb][kx] = xr[xoff[pb] + kx];
        };
        if (n_rows > 0) { load_row(0, rows[0]); load_row(1, rows[1]); }
        for (int cbp = cbp_begin; cbp < cbp_end; cbp++, step++) {
            const int buf = step & 1;
            const int id = otile * pairs + cbp;
            if ((buf ? held1 : held0) != id) {
                // not prefetched (first step of the block): stage it now
                v4i stage[EPT];
#pragma unroll
                for (int e = 0; e < EPT; e++) {
                    bool par;
                    const long src = entry_src(threadIdx.x + e * 256, otile, cbp, par);
                    stage[e] = par ? wpb[src] : wb[src];
                }
#pragma unroll
                for (int e = 0; e < EPT; e++) s_w[buf * ENT + threadIdx.x + e * 256] = stage[e];
                if (buf) held1 = id; else held0 = id;
                __syncthreads();
            }
            // the pair of the next step goes into the other buffer, a third of it per kernel row
            int p_otile = otile, p_cbp = cbp + 1;
            if (p_cbp >= cbp_end) { p_otile = n_otile; p_cbp = n_cbp; }
            const int nid = p_otile >= 0 ? p_otile * pairs + p_cbp : -1;
            const bool prefetch = nid >= 0 && (buf ? held0 : held1) != nid;
            constexpr int EPR = (EPT + KH - 1) / KH; // entries per thread and row
            const v4i *sw = s_w + buf * ENT + (long)h * TAPS * 2 * FT + j;
            const int r_base = (cbp - cbp_begin) * KH;
#pragma unroll
            for (int ky = 0; ky < KH; ky++) {
                v4i stage[EPR];
                if (prefetch) {
#pragma unroll
                    for (int e = 0; e < EPR; e++) {
                        if (ky * EPR + e < EPT) {
                            bool par;
                            const long src = entry_src(threadIdx.x + (ky * EPR + e) * 256, p_otile, p_cbp, par);
                            stage[e] = par ? wpb[src] : wb[src];
                        }
                    }
                }
                load_row(r_base + ky + 2, rows[(ky + 2) % KH]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kx = 0; kx < KW; kx++) {
                    const v4i *wt = sw + (ky * KW + kx) * 2 * FT;
                    const v4i a0 = wt[0], a1 = wt[32], q0 = wt[FT], q1 = wt[FT + 32];
#pragma unroll
                    for (int pb = 0; pb < PB; pb++) {
                        acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, rows[ky][pb][kx], acc[0][pb], 0, 0, 0);
                        acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, rows[ky][pb][kx], acc[1][pb], 0, 0, 0);
                    }
#pragma unroll
                    for (int pb = 0; pb < PB; pb++) {
                        const v4i par = rows[ky][pb][kx] & ones;
                        acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q0, par, acc[0][pb], 0, 0, 0);
                        acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q1, par, acc[1][pb], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (prefetch) {
#pragma unroll
                    for (int e = 0; e < EPR; e++)
                        if (ky * EPR + e < EPT) s_w[(buf ^ 1) * ENT + threadIdx.x + (ky * EPR + e) * 256] = stage[e];
                }
            }
            if (prefetch) { if (buf) held0 = nid; else held1 = nid; }
            // everyone is done reading this step's buffer (it is the next prefetch target) and the
            // other buffer is complete
            __syncthreads();
        }
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            if (mm[pb] < 0) continue;
            const int n = mm[pb] / HoWo, r0 = mm[pb] - n * HoWo;
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int o = otile * FT + a * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                    if (o >= p.O) continue;
                    int32_t *dst = out + ((long)n * p.O + o) * HoWo + r0;
                    if (p.ksplit == 1) *dst = acc[a][pb][r];
                    else atomicAdd(dst, acc[a][pb][r]);
                }
        }
    }
}

// ---- fused 3x3 / stride 1 / padding 1 kernel ---------------------------------------------------------
// The same contraction with the activation re-layout folded into the MFMA kernel: a block owns a tile of output
// pixels (NI images x TH rows x all columns, at most 256 pixels) and 64 output channels, and walks over the
// channel-block pairs.  Per pair it reads the float32 activations of the tile (with halo) straight from the NCHW
// tensor, rounds / clamps / packs them to int8 in registers and puts them into LDS as 16-byte vectors
// [half][padded pixel] -- the int8 copy never reaches HBM and the packing launch disappears -- and copies the
// pair's 36 KB of packed weights (values and parities, laid out by fixed_pack_w_tiles exactly as LDS wants them).
// Both MFMA operands then come from LDS.  One buffer per operand: several blocks share a CU, so one block's
// loads overlap another block's MFMAs.
struct FusedParams {
    int N, C, H, W, O, O_pad;
    int pairs;            // 32-channel groups, ceil(C / 32)
    int TH, NI;           // tile: NI images x TH output rows x W columns
    int tiles_y;          // tiles per image column (ceil(H / TH)); image groups: ceil(N / NI)
    int o_tiles, n_items;
    float P2;
};

// weights -> wpk[otile][pair][h][tap][val/par][o 0..63] 16-byte entries (one thread per entry pair)
__global__ __launch_bounds__(256) void fixed_pack_w_tiles(const float *__restrict__ w, int8_t *__restrict__ wpk, int O, int C,
                                                          int O_pad, int pairs, float P2)
{
    const unsigned total = (unsigned)O_pad * pairs * 2 * 9;
    for (unsigned i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
        const unsigned tap = i % 9, co = i / 9;                  // tap fastest: a thread group reads a contiguous run
        const unsigned o = co % (unsigned)O_pad, cb = co / (unsigned)O_pad; // cb = 2 * pair + h
        uint32_t vals[4] = {0, 0, 0, 0}, pars[4] = {0, 0, 0, 0};
        if ((int)o < O) {
            const float *src = w + ((long)o * C + cb * 16) * 9 + tap;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                if ((int)(cb * 16 + k) < C) {
                    const float f = src[(long)k * 9];
                    const int q = quant_round_pos(f, P2) - quant_round_neg(f, P2);
                    const int par = (q & 1) ? (q < 0 ? -1 : 1) : 0;
                    vals[k >> 2] |= (uint32_t)(uint8_t)(int8_t)q << (8 * (k & 3));
                    pars[k >> 2] |= (uint32_t)(uint8_t)(int8_t)par << (8 * (k & 3));
                }
            }
        }
        const unsigned otile = o / 64, ol = o % 64, pair = cb / 2, h = cb % 2;
        const long e = ((((long)otile * pairs + pair) * 2 + h) * 9 + tap) * 2 * 64 + ol;
        reinterpret_cast<uint4 *>(wpk)[e] = make_uint4(vals[0], vals[1], vals[2], vals[3]);
        reinterpret_cast<uint4 *>(wpk)[e + 64] = make_uint4(pars[0], pars[1], pars[2], pars[3]);
    }
}

constexpr int FUSED_W_ENTRIES = 2 * 9 * 2 * 64; // 16-byte entries of one (otile, pair): 36 KB

// Parity term of packed int8 weights: per byte, 0 for an even weight, +1 / -1 for an odd positive / negative one.
__device__ __forceinline__ v4i weight_parities(v4i a)
{
    v4i r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t w = (uint32_t)a[i];
        const uint32_t odd = w & 0x01010101u;         // 1 per odd byte
        const uint32_t neg_odd = (w >> 7) & odd;      // 1 per odd negative byte
        r[i] = (int)(((neg_odd << 8) - neg_odd) | odd); // 0xFF per odd negative byte, 0x01 per odd positive one
    }
    return r;
}

// PBW: 32-pixel blocks per wave; AR: rounds of 256 (padded pixel, half) entries that cover the tile.
// A block walks over its items (blockIdx.x, + gridDim.x, ...) and their pairs as one sequence of steps; the global
// loads of step s + 1 are issued before the MFMAs of step s and land in registers while those run.
// WS (weight-stationary; every weight of the layer fits 36 KB of int8, one output-channel tile): the block quantises
// the float32 weights itself once, keeps the int8 values of all pairs in LDS for all its items and derives the
// parities in registers -- no weight traffic per step and no separate weight-tiling launch; wpk is then the float32
// weight tensor [O][C][3][3].
// V4 (rows of a multiple of four pixels, 16-byte aligned tensor): a thread's entry is four neighbouring pixels of
// one row and 16-channel half, read as sixteen 16-byte loads (one per channel) instead of four times sixteen 4-byte
// loads -- vector-memory instruction issue, not bytes, was what the load phase of a step spent its time on.  The
// halo columns are then never loaded: they are zeroed once.
template <int PBW, int AR, bool WS, bool V4>
__global__ __launch_bounds__(256, 2) void fixed_fused_kernel(const float *__restrict__ x, const void *__restrict__ wpk,
                                                          int32_t *__restrict__ out, FusedParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t s_raw[];
    v4i *s_w = reinterpret_cast<v4i *>(s_raw);       // [h][tap][val/par][o 0..63]; WS: [pair][h][tap][o 0..63], values only
    v4i *s_a = s_w + (WS ? p.pairs * (FUSED_W_ENTRIES / 2) : FUSED_W_ENTRIES); // [h][padded pixel of the tile]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, h = lane >> 5;
    const int Wp = p.W + 2, RP = p.TH + 2;           // padded row length, padded rows per image of the tile
    const int NPP = p.NI * RP * Wp;                  // padded pixels of the tile
    const int TP = p.TH * p.W;                       // output pixels per image of the tile
    const long plane = (long)p.H * p.W;
    if ((int)blockIdx.x >= p.n_items) return;

    // this thread's entries of the activation tile: image and padded row inside the tile, and the entry's byte
    // offset from the tile's first halo element (first image, first channel of the pair, one row above and one
    // column left of the tile) -- never negative, and 32 bits are enough: the host checks the tensor's size
    int e_img[AR], e_row[AR];
    uint32_t e_off[AR];
    bool e_colok[AR];
    // V4: one entry per thread = (half, image, padded row, group of four pixels); GW groups per row
    const int GW = p.W / 4, NQ = p.NI * RP * GW;
    int q_img = 1 << 28, q_row = 0, q_half = 0, q_lds = 0;
    uint32_t q_off = 0;
    if (V4 && (int)threadIdx.x < 2 * NQ) {
        const int e = threadIdx.x;
        q_half = e >= NQ ? 1 : 0;
        const int pp = e - q_half * NQ;
        const int i = pp / (RP * GW), rem = pp - i * (RP * GW);
        q_row = rem / GW;
        const int g = rem - q_row * GW;
        q_img = i;
        q_off = (uint32_t)((((long)i * p.C + q_half * 16) * plane + (long)q_row * p.W + 4 * g) * 4);
        q_lds = q_half * NPP + (i * RP + q_row) * Wp + 4 * g + 1;
    }
#pragma unroll
    for (int a = 0; a < AR; a++) {
        const int e = a * 256 + threadIdx.x;
        const int hh = e >= NPP ? 1 : 0;
        const int pp = e - hh * NPP;
        const int i = pp / (RP * Wp), rem = pp - i * (RP * Wp);
        const int row = rem / Wp, col = rem - row * Wp;
        e_img[a] = e < 2 * NPP ? i : (1 << 28); // beyond the tile: never inside the batch
        e_row[a] = row;
        e_colok[a] = col >= 1 && col <= p.W;
        e_off[a] = (uint32_t)((((long)i * p.C + hh * 16) * plane + (long)row * p.W + col) * 4);
    }
    // this lane's output pixels (one per 32-pixel block of the wave)
    int l_img[PBW], l_row[PBW], l_col[PBW], abase[PBW];
#pragma unroll
    for (int pb = 0; pb < PBW; pb++) {
        const int t = (wave + 4 * pb) * 32 + j;
        const int i = t / TP, r = (t - i * TP) / p.W;
        l_img[pb] = i < p.NI ? i : (1 << 28);
        l_row[pb] = r;
        l_col[pb] = t - i * TP - r * p.W;
        abase[pb] = i < p.NI ? (i * RP + r) * Wp + l_col[pb] : 0;
    }

    v16i acc[2][PBW];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < PBW; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    constexpr int WR = WS ? 1 : FUSED_W_ENTRIES / 256;
    v4i wreg[WR];
    float freg[V4 ? 1 : AR][16];
    float4 qreg[V4 ? 16 : 1];

    auto issue = [&](int item, int pair) {
        const int otile = item % p.o_tiles, tile = item / p.o_tiles;
        const int ty = tile % p.tiles_y, tg = tile / p.tiles_y;
        const int n0 = tg * p.NI, y0 = ty * p.TH;
        if (!WS) {
            const v4i *src = reinterpret_cast<const v4i *>(wpk) + ((long)otile * p.pairs + pair) * FUSED_W_ENTRIES + threadIdx.x;
#pragma unroll
            for (int e = 0; e < WR; e++) wreg[e] = src[e * 256];
        }
        if (V4) {
            // (for the first tile this base lies one row before the tensor; those rows are never loaded)
            const char *xq = reinterpret_cast<const char *>(x) + (((long)n0 * p.C + pair * 32) * plane + (long)(y0 - 1) * p.W) * 4;
            const int n = n0 + q_img, y = y0 + q_row - 1;
            const bool inb = n < p.N && y >= 0 && y < p.H;
            const int kmax = inb ? p.C - pair * 32 - q_half * 16 : 0;
            if (kmax >= 16) {
#pragma unroll
                for (int k = 0; k < 16; k++) qreg[k] = *reinterpret_cast<const float4 *>(xq + k * plane * 4 + q_off);
            } else if (kmax > 0) {
#pragma unroll
                for (int k = 0; k < 16; k++)
                    qreg[k] = k < kmax ? *reinterpret_cast<const float4 *>(xq + k * plane * 4 + q_off) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
#pragma unroll
                for (int k = 0; k < 16; k++) qreg[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
            return;
        }
        // (for the first tile this base lies one row and one element before the tensor; those entries are never loaded)
        const char *xb = reinterpret_cast<const char *>(x) + (((long)n0 * p.C + pair * 32) * plane + (long)(y0 - 1) * p.W - 1) * 4;
#pragma unroll
        for (int a = 0; a < AR; a++) {
            const int n = n0 + e_img[a], y = y0 + e_row[a] - 1;
            const bool inb = e_colok[a] && n < p.N && y >= 0 && y < p.H;
            const int kmax = inb ? p.C - pair * 32 - (a * 256 + (int)threadIdx.x >= NPP ? 16 : 0) : 0;
            if (kmax >= 16) {
#pragma unroll
                for (int k = 0; k < 16; k++) freg[a][k] = *reinterpret_cast<const float *>(xb + k * plane * 4 + e_off[a]);
            } else if (kmax > 0) { // the channel tail of the last pair
#pragma unroll
                for (int k = 0; k < 16; k++)
                    freg[a][k] = k < kmax ? *reinterpret_cast<const float *>(xb + k * plane * 4 + e_off[a]) : 0.f;
            } else { // halo, or beyond the tile / the batch / the channels
#pragma unroll
                for (int k = 0; k < 16; k++) freg[a][k] = 0.f;
            }
        }
    };

    auto store_item = [&](int item) { // and clear the accumulators for the next item
        const int otile = item % p.o_tiles, tile = item / p.o_tiles;
        const int ty = tile % p.tiles_y, tg = tile / p.tiles_y;
        const int n0 = tg * p.NI, y0 = ty * p.TH;
        const bool whole = otile * 64 + 64 <= p.O;
#pragma unroll
        for (int pb = 0; pb < PBW; pb++) {
            const int n = n0 + l_img[pb], y = y0 + l_row[pb];
            if (n < p.N && y < p.H) {
                int32_t *o0 = out + (((long)n * p.O + otile * 64 + 4 * h) * plane + (long)y * p.W + l_col[pb]);
                if (whole) {
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int r = 0; r < 16; r++) o0[(long)(a * 32 + 8 * (r / 4) + (r % 4)) * plane] = acc[a][pb][r];
                } else {
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int ol = a * 32 + 8 * (r / 4) + (r % 4);
                            if (otile * 64 + 4 * h + ol < p.O) o0[(long)ol * plane] = acc[a][pb][r];
                        }
                }
            }
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[a][pb][r] = 0;
        }
    };

    // Consecutive items share their activation tile (they differ in the output-channel tile), and consecutive
    // block ids land on different XCDs: renumber so that the blocks of one XCD (ids b, b + 8, ...) take consecutive
    // items and the shared tile is served by that XCD's L2.  The host makes the grid a multiple of 8 when it can.
    const int G = gridDim.x;
    const int first = (G % 8 == 0) ? (int)(blockIdx.x % 8) * (G / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    int item = first, pair = 0, pending = -1;
    issue(item, pair); // the first activations are on their way while the weights are being prepared
    if (WS) {
        // All weights of the layer, once per block: a work item is four consecutive channels of one output channel
        // (36 contiguous floats); it yields one dword (bytes = the four channels) of the nine taps' LDS entries.
        const float *wf = reinterpret_cast<const float *>(wpk);
        const float hi = p.P2 - 1.f;
        uint32_t *s_wd = reinterpret_cast<uint32_t *>(s_w);
        const int n_quads = 64 * p.pairs * 8; // at most 1024: four work items per thread
        for (int it0 = 0; it0 < 4; it0 += 2) { // two batches of two work items: their loads are in flight together
        float4 v4[2][9];
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int qd = (it0 + it) * 256 + threadIdx.x;
            const int b = qd & 3, hh = (qd >> 2) & 1, rest = qd >> 3;
            const int pr = rest % p.pairs, o = rest / p.pairs;
            const int c0 = pr * 32 + hh * 16 + b * 4;
            if (qd < n_quads && o < p.O && c0 + 4 <= p.C) { // the host has checked C % 4 == 0 and the tensor's alignment
                const float4 *src = reinterpret_cast<const float4 *>(wf + ((long)o * p.C + c0) * 9);
#pragma unroll
                for (int e = 0; e < 9; e++) v4[it][e] = src[e];
            } else {
#pragma unroll
                for (int e = 0; e < 9; e++) v4[it][e] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int qd = (it0 + it) * 256 + threadIdx.x;
            if (qd >= n_quads) break;
            const int b = qd & 3, hh = (qd >> 2) & 1, rest = qd >> 3;
            const int pr = rest % p.pairs, o = rest / p.pairs;
            float v[36];
#pragma unroll
            for (int e = 0; e < 9; e++) {
                v[4 * e] = v4[it][e].x; v[4 * e + 1] = v4[it][e].y; v[4 * e + 2] = v4[it][e].z; v[4 * e + 3] = v4[it][e].w;
            }
            uint32_t *dst = s_wd + ((long)((pr * 2 + hh) * 9) * 64 + o) * 4 + b;
            // round(clamp(w * P2, 1 - P2, P2 - 1)), half to even (positive part minus negative part), as two instructions
            // per weight: w * P2 + 1.5 * 2^23 in one fma leaves the rounded integer in the low mantissa bits (two's
            // complement, exact for |w * P2| < 2^22), and clamping there equals clamping before the rounding because
            // the bounds are integers.  Larger magnitudes and infinities end at the bounds as well; v_perm_b32 gathers
            // the low bytes.
            const float magic = 12582912.f;
            uint32_t qb[36];
#pragma unroll
            for (int e = 0; e < 36; e++)
                qb[e] = __float_as_uint(__builtin_amdgcn_fmed3f(fmaf(v[e], p.P2, magic), magic - hi, magic + hi));
#pragma unroll
            for (int tap = 0; tap < 9; tap++) {
                // bytes 0 of the four channels' words -> one dword (selector bytes: 0..3 = second operand, 4..7 = first)
                const uint32_t lo = __builtin_amdgcn_perm(qb[9 + tap], qb[tap], 0x0c0c0400u);       // [k0, k1, 0, 0]
                const uint32_t hi2 = __builtin_amdgcn_perm(qb[27 + tap], qb[18 + tap], 0x04000c0cu); // [0, 0, k2, k3]
                dst[tap * 64 * 4] = lo | hi2;
            }
        }
        }
        // (no barrier here: the one behind the first step's LDS writes orders these writes before any MFMA as well)
    }
    if (V4) { // the halo columns of every padded row stay zero for the whole launch
        for (int e = threadIdx.x; e < 2 * p.NI * RP * 2; e += 256) {
            const int side = e & 1, rowi = e >> 1; // rowi counts (half, image, row)
            const int hh = rowi / (p.NI * RP), ir = rowi - hh * (p.NI * RP);
            s_a[hh * NPP + ir * Wp + (side ? Wp - 1 : 0)] = (v4i){0, 0, 0, 0};
        }
    }

    const float top = p.P2 - 1.f;
    while (true) {
        // operands of this step: registers -> LDS (activations rounded half to even and clamped to [0, P2 - 1] on the way:
        // v_cvt_pk_u8_f32 rounds to nearest even, clamps below at zero and drops the byte into place)
        if (!WS) {
#pragma unroll
            for (int e = 0; e < WR; e++) s_w[threadIdx.x + e * 256] = wreg[e];
        }
        if (V4) {
            if ((int)threadIdx.x < 2 * NQ) {
#pragma unroll
                for (int px = 0; px < 4; px++) {
                    uint32_t wds[4] = {0, 0, 0, 0};
#pragma unroll
                    for (int k = 0; k < 16; k++) {
                        const float f = px == 0 ? qreg[k].x : px == 1 ? qreg[k].y : px == 2 ? qreg[k].z : qreg[k].w;
                        wds[k >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(fminf(f * p.P2, top), k & 3, wds[k >> 2]);
                    }
                    s_a[q_lds + px] = (v4i){(int)wds[0], (int)wds[1], (int)wds[2], (int)wds[3]};
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < AR; a++) {
                uint32_t wds[4] = {0, 0, 0, 0};
#pragma unroll
                for (int k = 0; k < 16; k++)
                    wds[k >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(fminf(freg[a][k] * p.P2, top), k & 3, wds[k >> 2]);
                if (a * 256 + (int)threadIdx.x < 2 * NPP) s_a[a * 256 + threadIdx.x] = (v4i){(int)wds[0], (int)wds[1], (int)wds[2], (int)wds[3]};
            }
        }
        __syncthreads();
        // results of the item that ended with the previous step: stored here, before the next loads are issued, so
        // that waiting for those loads never means waiting for younger stores
        if (pending >= 0) store_item(pending);
        pending = -1;
        int nitem = item, npair = pair + 1;
        if (npair == p.pairs) { npair = 0; nitem = item + gridDim.x; }
        const bool more = nitem < p.n_items;
        if (more) issue(nitem, npair);

        const v4i *sw = WS ? s_w + (pair * 2 + h) * (9 * 64) + j : s_w + h * (9 * 2 * 64) + j;
        const v4i *sa = s_a + h * NPP;
#pragma unroll
        for (int ky = 0; ky < 3; ky++)
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const v4i *wt = sw + (ky * 3 + kx) * (WS ? 64 : 2 * 64);
                const v4i a0 = wt[0], a1 = wt[32];
                const v4i q0 = WS ? weight_parities(a0) : wt[64], q1 = WS ? weight_parities(a1) : wt[96];
#pragma unroll
                for (int pb = 0; pb < PBW; pb++) {
                    const v4i b = sa[abase[pb] + ky * Wp + kx];
                    const v4i par = b & ones;
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b, acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b, acc[1][pb], 0, 0, 0);
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q0, par, acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q1, par, acc[1][pb], 0, 0, 0);
                }
            }
        if (pair == p.pairs - 1) pending = item;
        if (!more) break;
        item = nitem; pair = npair;
        __syncthreads(); // all waves are done with this step's operands before the next ones overwrite them
    }
    if (pending >= 0) store_item(pending);
}

// ---- single pass for small planes: the reduction split over the waves of a block ---------------------------------
// 3x3 / stride 1 / padding 1 layers whose planes are small (14x14, 7x7) have many channels and few pixels: a block that
// walks the whole reduction is long, and there are too few of them to hide their load latency.  Here a block still owns a
// tile of output pixels (TH rows x W columns of one image, at most 64 pixels) and 64 output channels, but its four waves
// take a quarter of the 32-channel groups each and work on it independently of one another -- nothing is shared, so there
// is no barrier inside the reduction: a wave reads the float32 activations of its groups from the NCHW tensor, rounds /
// clamps / packs them to int8 into its own LDS region (halo included; LDS operations of one wave execute in order, so the
// wave may read what it has just written), and takes its weights -- int8 values tiled by fixed_pack_w_values in the MFMA
// operand order -- straight from L2 into registers, a kernel row at a time, two rows ahead of their use; the parity operand
// of the weights is derived in registers.  The four partial tiles meet in LDS at the end (two exchange rounds, after which
// every wave holds one quarter of the tile and stores it).  Blocks are four times shorter and four times more numerous than
// with the whole reduction per block, the int8 copy of the activations never reaches HBM and nothing is added atomically.
struct KsplitParams {
    int N, C, H, W, O, O_pad;
    int pairs;            // 32-channel groups, ceil(C / 32)
    int TH, tiles_y;      // tile: TH output rows x W columns; tiles per image
    int o_tiles, n_items; // one block per (image, tile, output-channel tile)
    float P2;
};

// weights -> wv[otile][pair][h][tap][o 0..63]: 16-byte entries (16 channels of one tap and output channel), values only.
// One thread per entry, tap fastest: the threads of one (o, 16-channel block) read one contiguous run of the OIHW tensor.
__global__ __launch_bounds__(256) void fixed_pack_w_values(const float *__restrict__ w, int8_t *__restrict__ wv, int O, int C,
                                                           int O_pad, int pairs, float P2)
{
    const unsigned total = (unsigned)O_pad * pairs * 2 * 9;
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const unsigned tap = i % 9, co = i / 9;
    const unsigned cb = co % (unsigned)(pairs * 2), o = co / (unsigned)(pairs * 2);
    float f[16];
    const float *src = w + ((long)o * C + cb * 16) * 9 + tap;
    if ((int)o < O && (int)(cb * 16 + 16) <= C) {
#pragma unroll
        for (int k = 0; k < 16; k++) f[k] = src[k * 9];
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) f[k] = ((int)o < O && (int)(cb * 16) + k < C) ? src[k * 9] : 0.f;
    }
    uint32_t vals[4] = {0, 0, 0, 0};
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int q = quant_round_pos(f[k], P2) - quant_round_neg(f[k], P2); // signed
        vals[k >> 2] |= (uint32_t)(uint8_t)(int8_t)q << (8 * (k & 3));
    }
    const unsigned otile = o / 64, ol = o % 64, pair = cb / 2, h = cb % 2;
    reinterpret_cast<uint4 *>(wv)[((((long)otile * pairs + pair) * 2 + h) * 9 + tap) * 64 + ol] = make_uint4(vals[0], vals[1], vals[2], vals[3]);
}

// A wave-uniform 64-bit offset the compiler has to materialise in scalar registers where it stands: it can then not be
// folded into loop-invariant per-lane address arithmetic (which would keep a 64-bit address pair alive per load).
__device__ __forceinline__ long opaque_uniform(long v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((unsigned long)v >> 32));
    asm volatile("" : "+s"(lo), "+s"(hi));
    return (long)(((unsigned long)hi << 32) | lo);
#else
    return v;
#endif
}

// AR: rounds of 64 (half, tile row incl. halo rows, column) entries that cover the wave's activation tile.
template <int AR>
__global__ __launch_bounds__(256, 2) void fixed_ksplit_kernel(const float *__restrict__ x, const v4i *__restrict__ wv,
                                                             int32_t *__restrict__ out, KsplitParams p)
{
    constexpr int PB = 2; // 32-pixel blocks per tile
    extern __shared__ __attribute__((aligned(16))) uint8_t s_raw[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, h = lane >> 5;
    const int Wp = p.W + 2, RP = p.TH + 2, NPP = RP * Wp; // padded tile
    v4i *s_a = reinterpret_cast<v4i *>(s_raw) + wave * (2 * NPP); // this wave's region: [half][padded pixel]
    // blocks of one XCD (ids b, b + 8, ...) take consecutive items: the output-channel tiles of one pixel tile
    const int G = gridDim.x;
    const int bid = (G % 8 == 0) ? (int)(blockIdx.x % 8) * (G / 8) + (int)(blockIdx.x / 8) : (int)blockIdx.x;
    const int otile = bid % p.o_tiles;
    const int tl = bid / p.o_tiles;
    const int ty = tl % p.tiles_y, n = tl / p.tiles_y;
    const int y0 = ty * p.TH;
    const long plane = (long)p.H * p.W;

    // the whole region starts as zeros: halo columns, rows outside the image and channels beyond C stay that way
    for (int e = lane; e < 2 * NPP; e += 64) s_a[e] = (v4i){0, 0, 0, 0};

    // this lane's entries of the tile: (half, padded row, column) -> element offset from x (32 bits: the host checks the
    // tensor's size), LDS index and half packed into one word (bit 31: half; negative offset: nothing to load)
    const int RW = RP * p.W;
    int e_off[AR], e_lds[AR];
#pragma unroll
    for (int a = 0; a < AR; a++) {
        const int e = a * 64 + lane;
        const int hh = e >= RW ? 1 : 0;
        const int rem = e - hh * RW;
        const int r = rem / p.W, c = rem - r * p.W;
        const int y = y0 - 1 + r;
        const bool ok = e < 2 * RW && y >= 0 && y < p.H;
        e_lds[a] = (hh * NPP + r * Wp + c + 1) | (hh << 30);
        e_off[a] = ok ? (int)(((long)n * p.C + hh * 16) * plane + (long)y * p.W + c) : -1;
    }
    // this lane's output pixels
    int abase[PB];
#pragma unroll
    for (int pb = 0; pb < PB; pb++) {
        const int t = pb * 32 + j;
        const int r = t / p.W, c = t - r * p.W;
        abase[pb] = (r < p.TH) ? r * Wp + c : 0;
    }

    const int per = (p.pairs + 3) / 4;
    const int g_begin = min(p.pairs, wave * per), g_end = min(p.pairs, g_begin + per);
    const int n_rows = (g_end - g_begin) * 3;

    v16i acc[2][PB];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < PB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    const float top = p.P2 - 1.f;

    // Rounds 0 .. PF-1 of a group's entries are requested one group ahead and wait in registers; a fourth round (tiles
    // with more than 192 entries) is loaded when the group is converted, reusing the same registers.
    constexpr int PF = AR < 3 ? AR : 3;
    float f[PF][16];
    auto load_round = [&](int g, int a, float (&dst)[16]) __attribute__((always_inline)) {
        // wave-uniform byte offset of (group, channel k) + this lane's 32-bit byte offset
        const char *xc = reinterpret_cast<const char *>(x);
        if (p.C - g * 32 >= 32) { // a whole group (wave-uniform): every lane loads, lanes without an entry re-read offset 0
            const uint32_t off = e_off[a] >= 0 ? (uint32_t)e_off[a] * 4u : 0u;
#pragma unroll
            for (int k = 0; k < 16; k++)
                dst[k] = *reinterpret_cast<const float *>(xc + opaque_uniform(((long)g * 32 + k) * plane * 4) + off);
        } else { // the channel tail of the last group
            const int kmax = e_off[a] >= 0 ? p.C - g * 32 - (e_lds[a] >> 30) * 16 : 0;
            const uint32_t off = (uint32_t)e_off[a] * 4u;
#pragma unroll
            for (int k = 0; k < 16; k++)
                dst[k] = k < kmax ? *reinterpret_cast<const float *>(xc + opaque_uniform(((long)g * 32 + k) * plane * 4) + off) : 0.f;
        }
    };
    auto convert_round = [&](int a, const float (&src)[16]) __attribute__((always_inline)) { // int8, round half to even, clamp to [0, P2 - 1] -> LDS
        uint32_t wds[4] = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 16; k++)
            wds[k >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(fminf(src[k] * p.P2, top), k & 3, wds[k >> 2]);
        if (e_off[a] >= 0) s_a[e_lds[a] & 0xffff] = (v4i){(int)wds[0], (int)wds[1], (int)wds[2], (int)wds[3]};
    };
    auto issue_acts = [&](int g) __attribute__((always_inline)) {
#pragma unroll
        for (int a = 0; a < PF; a++) load_round(g, a, f[a]);
    };
    // weight rows (group, ky) run through a ring of three register sets, two rows ahead of their use
    v4i wr[3][2][3]; // [slot][output-channel half][kx]
    const v4i *wbase = wv + ((long)otile * p.pairs * 2 + h) * (9 * 64) + j;
    auto load_row = [&](int r, v4i (&dst)[2][3]) __attribute__((always_inline)) {
        r = r < n_rows ? r : n_rows - 1; // past the end: re-read the last row (harmless)
        const int g = g_begin + r / 3, ky = r - (r / 3) * 3;
        const v4i *src = wbase + (long)g * (2 * 9 * 64) + ky * 3 * 64;
#pragma unroll
        for (int kx = 0; kx < 3; kx++) { dst[0][kx] = src[kx * 64]; dst[1][kx] = src[kx * 64 + 32]; }
    };
    if (n_rows > 0) {
        issue_acts(g_begin);
        load_row(0, wr[0]);
        load_row(1, wr[1]);
    }
    for (int g = g_begin; g < g_end; g++) {
        // activations of this group: registers -> int8 -> LDS
#pragma unroll
        for (int a0 = 0; a0 < AR; a0 += PF) {
            if (a0 > 0) {
                __builtin_amdgcn_sched_barrier(0); // not before the previous rounds have left these registers
#pragma unroll
                for (int a = 0; a < PF; a++) if (a0 + a < AR) load_round(g, a0 + a, f[a]);
            }
#pragma unroll
            for (int a = 0; a < PF; a++) if (a0 + a < AR) convert_round(a0 + a, f[a]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (g + 1 < g_end) issue_acts(g + 1);
        // other lanes of this wave read what this lane wrote: LDS executes a wave's operations in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int r_base = (g - g_begin) * 3;
        const v4i *sa = s_a + h * NPP;
#pragma unroll
        for (int ky = 0; ky < 3; ky++) {
            load_row(r_base + ky + 2, wr[(ky + 2) % 3]);
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const v4i a0 = wr[ky][0][kx], a1 = wr[ky][1][kx];
                const v4i q0 = weight_parities(a0), q1 = weight_parities(a1);
#pragma unroll
                for (int pb = 0; pb < PB; pb++) {
                    const v4i b = sa[abase[pb] + ky * Wp + kx];
                    const v4i par = b & ones;
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b, acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b, acc[1][pb], 0, 0, 0);
                    acc[0][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q0, par, acc[0][pb], 0, 0, 0);
                    acc[1][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(q1, par, acc[1][pb], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // The four partial tiles meet in LDS.  Round A: waves 0/1 and 2/3 exchange output-channel halves (even waves keep
    // half 0); round B: waves 0/2 and 1/3 exchange pixel blocks (waves 0, 1 keep block 0).  Afterwards wave w holds the
    // finished quarter (half w & 1, pixel block w >> 1).
    __syncthreads(); // every wave is done with its activation region, which the exchange buffers overlay
    int *s_red = reinterpret_cast<int *>(s_raw);
    v16i keep[PB];
    {
        int *mine = s_red + wave * (PB * 16 * 64) + lane;
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) mine[(pb * 16 + r) * 64] = (wave & 1) ? acc[0][pb][r] : acc[1][pb][r];
        __syncthreads();
        const int *theirs = s_red + (wave ^ 1) * (PB * 16 * 64) + lane;
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) keep[pb][r] = ((wave & 1) ? acc[1][pb][r] : acc[0][pb][r]) + theirs[(pb * 16 + r) * 64];
        __syncthreads();
    }
    v16i fin;
    {
        int *mine = s_red + wave * (16 * 64) + lane;
#pragma unroll
        for (int r = 0; r < 16; r++) mine[r * 64] = (wave & 2) ? keep[0][r] : keep[1][r];
        __syncthreads();
        const int *theirs = s_red + (wave ^ 2) * (16 * 64) + lane;
#pragma unroll
        for (int r = 0; r < 16; r++) fin[r] = ((wave & 2) ? keep[1][r] : keep[0][r]) + theirs[r * 64];
    }
    const int a_fin = wave & 1, pb_fin = wave >> 1;
    const int t = pb_fin * 32 + j;
    const int row = t / p.W, col = t - row * p.W;
    const int y = y0 + row;
    if (row < p.TH && y < p.H) {
        const int o_first = otile * 64 + a_fin * 32 + 4 * h;
        int32_t *o0 = out + ((long)n * p.O + o_first) * plane + (long)y * p.W + col;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int ol = 8 * (r / 4) + (r % 4);
            if (o_first + ol < p.O) o0[(long)ol * plane] = fin[r];
        }
    }
}

// Tile choice of the split-reduction kernel; false when the shape is not one it handles.
static bool ksplit_plan(const FixedParams &p, int O_pad, KsplitParams &k, int &AR)
{
    if (p.KH != 3 || p.KW != 3 || p.s0 != 1 || p.s1 != 1 || p.pad_h != 1 || p.pad_w != 1) return false;
    if (p.W > 64 || O_pad % 64 != 0) return false;
    k.N = p.N; k.C = p.C; k.H = p.H; k.W = p.W; k.O = p.O; k.O_pad = O_pad; k.P2 = p.P2;
    k.pairs = ceil_div(p.C, 32);
    k.o_tiles = O_pad / 64;
    int th = 64 / p.W;
    if (th > p.H) th = p.H;
    while (th > 1 && 2 * (th + 2) * p.W > 4 * 64) th--; // at most four rounds of tile entries per lane
    if (th < 1 || 2 * (th + 2) * p.W > 4 * 64) return false;
    k.TH = th;
    k.tiles_y = ceil_div(p.H, th);
    const long items = (long)p.N * k.tiles_y * k.o_tiles;
    if (items >= (1L << 31)) return false;
    if ((long)p.N * p.C * p.H * p.W >= (1L << 30)) return false; // 32-bit byte offsets inside the activation tensor
    k.n_items = (int)items;
    AR = ceil_div(2 * (th + 2) * p.W, 64);
    return true;
}

static int tune_flag(const char *name, int dflt)
{
    const char *e = getenv(name);
    return e && *e ? atoi(e) : dflt;
}

// The MFMA path is exact only where the per-product saturating add is provably inert.
static bool fixed_use_mfma(const FixedParams &p)
{
    if (p.add_config != 0 || p.d != 0 || p.pin > 7) return false;
    if (p.KW != 1 && p.KW != 3 && p.KW != 5) return false; // unrolled instances of the MFMA kernel
    if ((long)p.KH * p.KW * 4096 > 60 * 1024) return false;   // weight staging must fit the default LDS window
    const long pm = (1L << p.pin) - 1;
    const long bound = (long)p.C * p.KH * p.KW * (pm * pm + 1); // largest possible rounded sum of one polarity
    return bound < (long)p.max_value + 1 && (long)p.N * p.Ho * p.Wo < (1L << 31);
}

// Tile choice of the fused 3x3 kernel; false when the shape is not one it handles.
static bool fused_plan(const FixedParams &p, int O_pad, FusedParams &f)
{
    if (p.KH != 3 || p.KW != 3 || p.s0 != 1 || p.s1 != 1 || p.pad_h != 1 || p.pad_w != 1) return false;
    if (p.W > 256 || O_pad % 64 != 0) return false;
    if (((long)p.N * p.C * p.H * p.W + 2L * p.W + 2) * 4 >= (1L << 32)) return false; // 32-bit byte offsets inside the activation tensor
    f.N = p.N; f.C = p.C; f.H = p.H; f.W = p.W; f.O = p.O; f.O_pad = O_pad; f.P2 = p.P2;
    f.pairs = ceil_div(p.C, 32);
    f.o_tiles = O_pad / 64;
    const int plane = p.H * p.W;
    if (plane <= 128) {
        // small planes: whole images, as many as fit 256 pixels while every CU still gets a block
        f.TH = p.H;
        f.NI = 256 / plane;
        if (f.NI > p.N) f.NI = p.N;
        while (f.NI > 1 && (long)ceil_div(p.N, f.NI) * f.o_tiles < 256) f.NI--;
    } else {
        f.NI = 1;
        int th = 256 / p.W;
        if (th > p.H) th = p.H;
        if (th < 1) th = 1;
        f.TH = th;
        for (int t = th; 2 * t > th; t--) // a row count that divides the plane wastes no part of the last tile
            if (p.H % t == 0) { f.TH = t; break; }
    }
    f.tiles_y = ceil_div(p.H, f.TH);
    const long items = (long)ceil_div(p.N, f.NI) * f.tiles_y * f.o_tiles;
    if (items >= (1L << 31)) return false;
    f.n_items = (int)items;
    const int NPP = f.NI * (f.TH + 2) * (p.W + 2);
    if ((size_t)(FUSED_W_ENTRIES + 2 * NPP) * 16 > 64 * 1024) return false; // default LDS window
    if (2 * NPP > 3 * 256) return false;                                    // three rounds of tile entries per thread
    return ceil_div(f.NI * f.TH * p.W, 32) <= 8;
}

static int fixed_plan(const rexsc_fixed_desc *d, FixedParams &p, size_t &off_w, size_t &total)
{
    REXSC_CHECK_DESC(d, rexsc_fixed_desc);
    REXSC_CHECK_ARG(d->N > 0 && d->C > 0 && d->H > 0 && d->W > 0 && d->O > 0 && d->KH > 0 && d->KW > 0,
                    "non-positive dimension");
    REXSC_CHECK_ARG(d->pad_h >= 0 && d->pad_w >= 0 && d->stride_h > 0 && d->stride_w > 0, "bad padding/stride");
    REXSC_CHECK_ARG(d->precision_in >= 1 && d->precision_in <= 15, "precision_in must be 1..15 (got %d)", d->precision_in);
    REXSC_CHECK_ARG(d->precision_out >= 1, "precision_out must be positive (got %d)", d->precision_out);
    REXSC_CHECK_ARG(d->add_config >= 0, "add_config must be >= 0 (got %d)", d->add_config);
    p.N = d->N; p.C = d->C; p.H = d->H; p.W = d->W; p.O = d->O; p.KH = d->KH; p.KW = d->KW;
    p.pad_h = d->pad_h; p.pad_w = d->pad_w; p.s0 = d->stride_h; p.s1 = d->stride_w;
    const int Hp = p.H + 2 * p.pad_h, Wp = p.W + 2 * p.pad_w;
    REXSC_CHECK_ARG(Hp >= p.KH && Wp >= p.KW, "kernel larger than padded input");
    p.Ho = (Hp - p.KH) / p.s0 + 1; p.Wo = (Wp - p.KW) / p.s1 + 1;
    p.add_config = d->add_config; p.pin = d->precision_in;
    int pmax = 2 * d->precision_in > d->precision_out ? 2 * d->precision_in : d->precision_out;
    if (pmax > 31) pmax = 31;                                     // fixed.cpp:95
    p.d = 2 * d->precision_in - d->precision_out; if (p.d < 0) p.d = 0; // :97
    p.max_value = (int)(((((unsigned)1 << pmax) - 1u) >> p.d) << p.d);  // :96,:98
    p.P2 = (float)(1 << d->precision_in);
    size_t xbytes = (size_t)p.N * p.C * p.H * p.W * 4;
    size_t wbytes = (size_t)p.O * p.C * p.KH * p.KW * 4;
    if (fixed_use_mfma(p)) {
        const int CB = (int)align_up((size_t)ceil_div(p.C, 16), 2);
        const int O_pad = (int)align_up((size_t)p.O, FT);
        xbytes = (size_t)p.N * CB * (p.H + 2 * p.pad_h) * (p.W + 2 * p.pad_w) * 16;
        wbytes = 2 * (size_t)CB * p.KH * p.KW * O_pad * 16; // values + parities
    }
    off_w = align_up(xbytes, 256);
    total = off_w + align_up(wbytes, 256);
    return REXSC_OK;
}

} // namespace rexsc

using namespace rexsc;

extern "C" size_t rexsc_fixed_conv2d_workspace_bytes(const rexsc_fixed_desc *d)
{
    FixedParams p; size_t off_w, total;
    if (fixed_plan(d, p, off_w, total)) return 0;
    return total;
}

extern "C" int rexsc_fixed_conv2d(const rexsc_fixed_desc *d, const float *x, const float *w, int32_t *out,
                                  void *workspace, size_t workspace_bytes, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    FixedParams p; size_t off_w, total;
    int rc = fixed_plan(d, p, off_w, total);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && w && out, "null pointer");
    if (!workspace || workspace_bytes < total) {
        set_error("fixed conv2d: workspace of %zu bytes needed, %zu given", total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    if (fixed_use_mfma(p)) {
        Fixed8Params q;
        q.N = p.N; q.C = p.C; q.H = p.H; q.W = p.W; q.O = p.O; q.KH = p.KH; q.KW = p.KW;
        q.O_pad = (int)align_up((size_t)p.O, FT);
        q.pad_h = p.pad_h; q.pad_w = p.pad_w; q.s0 = p.s0; q.s1 = p.s1;
        q.Hp = p.H + 2 * p.pad_h; q.Wp = p.W + 2 * p.pad_w; q.Ho = p.Ho; q.Wo = p.Wo;
        q.CB = (int)align_up((size_t)ceil_div(p.C, 16), 2); q.M = p.N * p.Ho * p.Wo; q.P2 = p.P2;
        // split the channel-block pairs over waves until the launch has a few thousand of them
        int pb = 2;
        const bool db_shape = q.KH == 3 && q.KW == 3 && tune_flag("REXSC_TUNE_FIXED_DB", 1);
        // persistent kernel: 32-pixel waves when 64-pixel waves would leave SIMDs without any
        if (db_shape && (long)ceil_div(q.M, 64) * (q.O_pad / FT) < 1024) pb = 1;
        if (getenv("REXSC_TUNE_FIXED_PB")) pb = atoi(getenv("REXSC_TUNE_FIXED_PB")) == 1 ? 1 : 2;
        const int wpx = 32 * pb;
        const long tiles = (long)ceil_div(q.M, wpx) * (q.O_pad / FT);
        q.ksplit = 1;
        // (the atomic epilogue of a split costs about as much as the MFMA work of a wave: split only
        // while the launch has fewer wave tiles than about one per SIMD)
        if (db_shape) {
            // persistent kernel (staging overlapped, long blocks): split only while the work items would
            // not even give every CU one block
            const long items = (((long)ceil_div(q.M, wpx) + 3) / 4) * (q.O_pad / FT);
            while (items * q.ksplit * 2 <= 256 && q.ksplit * 2 <= q.CB / 2) q.ksplit *= 2;
        } else {
            while (tiles * q.ksplit < 1024 && q.ksplit * 2 <= q.CB / 2) q.ksplit *= 2;
        }
        if (getenv("REXSC_TUNE_FIXED_KSPLIT")) {
            q.ksplit = atoi(getenv("REXSC_TUNE_FIXED_KSPLIT"));
            if (q.ksplit < 1) q.ksplit = 1;
            if (q.ksplit > q.CB / 2) q.ksplit = q.CB / 2;
        }
        int8_t *xq16 = (int8_t *)workspace;
        int8_t *wq16 = (int8_t *)workspace + off_w;
        int8_t *wp16 = wq16 + (size_t)q.CB * q.KH * q.KW * q.O_pad * 16;
        auto gridf = [](long n) { long b = (n + 255) / 256; return (int)(b > 16384 ? 16384 : (b ? b : 1)); };
        const size_t nout = (size_t)p.N * p.O * p.Ho * p.Wo;
        const double io_bytes = 4.0 * p.N * p.C * p.H * p.W + 4.0 * p.O * p.C * p.KH * p.KW + 4.0 * nout;
        FusedParams fp;
        // The single-pass kernel wins where the planes are large (the int8 copy of the activations it avoids is what
        // the two-pass path spends its time on); on small planes with many channels its blocks are too few and too
        // long to hide their load latency, and the two-pass path stays ahead.  REXSC_TUNE_FIXED_FUSED: 0 never, 2 wherever it can.
        const int fused_mode = tune_flag("REXSC_TUNE_FIXED_FUSED", 1);
        // Planes that one 64-pixel tile covers (7x7) with at least eight 32-channel groups: the single pass whose waves split
        // the reduction (measured 39 us against 43 for the two passes on 512 x 7 x 7, batch 64; on 14 x 14 planes, four tiles
        // per image, it loses by 3 us).  REXSC_TUNE_FIXED_FUSED: 3 wherever it can run, 0 / 2 never.
        KsplitParams kp;
        int ks_ar = 0;
        if ((fused_mode == 1 || fused_mode == 3) && ksplit_plan(p, q.O_pad, kp, ks_ar) &&
            (fused_mode == 3 || (p.H * p.W <= 64 && kp.pairs >= 8))) {
            {
                ProfScope prof("fixed_pack_weights", 4.0 * p.O * p.C * 9 + 16.0 * q.O_pad * kp.pairs * 2 * 9, stream);
                const long threads = (long)q.O_pad * kp.pairs * 2 * 9;
                hipLaunchKernelGGL(fixed_pack_w_values, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, w, wq16,
                                   p.O, p.C, q.O_pad, kp.pairs, p.P2);
                REXSC_CHECK_HIP(hipGetLastError());
            }
            ProfScope prof("fixed_conv_ksplit", io_bytes, stream);
            const int NPP = (kp.TH + 2) * (kp.W + 2);
            size_t lds = (size_t)4 * 2 * NPP * 16;          // the waves' activation regions ...
            if (lds < 4 * 2 * 16 * 64 * 4) lds = 4 * 2 * 16 * 64 * 4; // ... overlaid by the exchange buffers (32 KB)
            const v4i *wvp = reinterpret_cast<const v4i *>(wq16);
            switch (ks_ar) {
            case 1: hipLaunchKernelGGL((fixed_ksplit_kernel<1>), dim3(kp.n_items), dim3(256), lds, stream, x, wvp, out, kp); break;
            case 2: hipLaunchKernelGGL((fixed_ksplit_kernel<2>), dim3(kp.n_items), dim3(256), lds, stream, x, wvp, out, kp); break;
            case 3: hipLaunchKernelGGL((fixed_ksplit_kernel<3>), dim3(kp.n_items), dim3(256), lds, stream, x, wvp, out, kp); break;
            default: hipLaunchKernelGGL((fixed_ksplit_kernel<4>), dim3(kp.n_items), dim3(256), lds, stream, x, wvp, out, kp); break;
            }
            REXSC_CHECK_HIP(hipGetLastError());
            return REXSC_OK;
        }
        if (fused_mode && fused_mode != 3 && fused_plan(p, q.O_pad, fp) && (fused_mode == 2 || p.H * p.W >= 512)) {
            const int NPP = fp.NI * (fp.TH + 2) * (fp.W + 2);
            const int PBT = ceil_div(fp.NI * fp.TH * fp.W, 32);
            const int AR = ceil_div(2 * NPP, 256);
            // weight-stationary: every weight of the layer as int8 in 36 KB of LDS, read as aligned float4 runs
            const bool ws = fp.o_tiles == 1 && fp.pairs <= 2 && p.C % 4 == 0 && ((uintptr_t)w % 16) == 0 &&
                            tune_flag("REXSC_TUNE_FIXED_WS", 1);
            // persistent blocks: two per CU stay resident (three measured a third slower: more blocks contending for the
            // same HBM time), then fewer until every block has the same number of items
            const int resident = 256 * 2;
            const int per_block = ceil_div(fp.n_items, resident);
            unsigned grid = (unsigned)ceil_div(fp.n_items, per_block);
            if (grid > 8 && grid % 8) grid += 8 - grid % 8;                  // XCD-aware item order needs a multiple of 8
            if (grid > (unsigned)fp.n_items) grid = (unsigned)fp.n_items;
            if (!ws) {
                ProfScope prof("fixed_pack_weights", 4.0 * p.O * p.C * 9 + 32.0 * q.O_pad * q.CB * 9, stream);
                const long entries = (long)q.O_pad * q.CB * 9;
                hipLaunchKernelGGL(fixed_pack_w_tiles, dim3((unsigned)gridf(entries)), dim3(256), 0, stream, w, wq16, p.O, p.C,
                                   q.O_pad, fp.pairs, p.P2);
                REXSC_CHECK_HIP(hipGetLastError());
            }
            ProfScope prof("fixed_conv_fused", io_bytes, stream);
            const size_t lds = (size_t)((ws ? fp.pairs * (FUSED_W_ENTRIES / 2) : FUSED_W_ENTRIES) + 2 * NPP) * 16;
            // float4 loads along the rows: rows of a multiple of four pixels, 16-byte aligned tensor
            const bool v4 = p.W % 4 == 0 && ((uintptr_t)x % 16) == 0 && 2 * fp.NI * (fp.TH + 2) * (p.W / 4) <= 256 &&
                            tune_flag("REXSC_TUNE_FIXED_V4", 1);
#define REXSC_FUSED2(PBW_, AR_, V4_)                                                                                                \
    do {                                                                                                                            \
        if (ws) hipLaunchKernelGGL((fixed_fused_kernel<PBW_, AR_, true, V4_>), dim3(grid), dim3(256), lds, stream, x, (const void *)w, out, fp); \
        else hipLaunchKernelGGL((fixed_fused_kernel<PBW_, AR_, false, V4_>), dim3(grid), dim3(256), lds, stream, x, (const void *)wq16, out, fp); \
    } while (0)
#define REXSC_FUSED(PBW_, AR_) REXSC_FUSED2(PBW_, AR_, false)
            if (v4) { if (PBT <= 4) REXSC_FUSED2(1, 1, true); else REXSC_FUSED2(2, 1, true); }
            else if (PBT <= 4) { if (AR <= 2) REXSC_FUSED(1, 2); else REXSC_FUSED(1, 3); }
            else { if (AR <= 2) REXSC_FUSED(2, 2); else REXSC_FUSED(2, 3); }
#undef REXSC_FUSED2
#undef REXSC_FUSED
            REXSC_CHECK_HIP(hipGetLastError());
            return REXSC_OK;
        }
        {
            ProfScope prof("fixed_pack", 4.0 * p.N * p.C * p.H * p.W + 16.0 * q.N * q.CB * q.Hp * q.Wp, stream);
            const long pack_threads = (long)q.Hp * q.Wp * q.N * q.CB;
            REXSC_CHECK_ARG(pack_threads < (1L << 32) - 256 && (long)q.CB * q.O_pad * q.KH * q.KW < (1L << 31), "fixed conv2d: problem too large");
            const long pack_blocks = (pack_threads + 255) / 256;
            const unsigned w_blocks = (unsigned)gridf((long)q.CB * q.O_pad * q.KH * q.KW);
            unsigned zero_blocks = 0;
            if (q.ksplit > 1) {
                zero_blocks = (unsigned)gridf((long)nout / 4 + 1);
                if (zero_blocks > 2048) zero_blocks = 2048;
            }
            REXSC_CHECK_ARG(pack_blocks + w_blocks + zero_blocks < (1L << 31), "fixed conv2d: problem too large");
            hipLaunchKernelGGL(fixed_prepare_kernel, dim3((unsigned)pack_blocks + w_blocks + zero_blocks), dim3(256), 0,
                               stream, x, xq16, w, wq16, wp16, out, nout, q, (unsigned)pack_blocks, w_blocks, zero_blocks);
        }
        REXSC_CHECK_HIP(hipGetLastError());
        const long m_groups = ((long)ceil_div(q.M, wpx) + 3) / 4;
        const unsigned grid = (unsigned)(m_groups * (q.O_pad / FT) * q.ksplit);
        const size_t lds = (size_t)2 * q.KH * q.KW * 2 * FT * 16;
        ProfScope prof("fixed_conv_mfma", io_bytes, stream);
        if (db_shape) {
            static std::atomic<bool> attr_set[64]; // zero-initialised; per device: the kernel needs more than the default 64 KB of LDS
            const size_t lds2 = 2 * lds;
            int dev = 0;
            REXSC_CHECK_HIP(hipGetDevice(&dev));
            if (dev < 0 || dev >= 64 || !attr_set[dev]) {
                REXSC_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&fixed_mfma_db_kernel<3, 3, 2>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2));
                REXSC_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&fixed_mfma_db_kernel<3, 3, 1>),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds2));
                if (dev >= 0 && dev < 64) attr_set[dev] = true;
            }
            const long n_items = (long)grid;
            const unsigned pgrid = (unsigned)(n_items < 512 ? n_items : 512); // two blocks per CU stay resident
            if (pb == 1)
                hipLaunchKernelGGL((fixed_mfma_db_kernel<3, 3, 1>), dim3(pgrid), dim3(256), lds2, stream, xq16, wq16, wp16,
                                   out, q, (int)n_items);
            else
                hipLaunchKernelGGL((fixed_mfma_db_kernel<3, 3, 2>), dim3(pgrid), dim3(256), lds2, stream, xq16, wq16, wp16,
                                   out, q, (int)n_items);
            REXSC_CHECK_HIP(hipGetLastError());
            return REXSC_OK;
        }
        switch (q.KW) {
        case 1:
            if (pb == 1) hipLaunchKernelGGL((fixed_mfma_kernel<1, 1>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            else hipLaunchKernelGGL((fixed_mfma_kernel<1, 2>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            break;
        case 3:
            if (pb == 1) hipLaunchKernelGGL((fixed_mfma_kernel<3, 1>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            else hipLaunchKernelGGL((fixed_mfma_kernel<3, 2>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            break;
        case 5:
            if (pb == 1) hipLaunchKernelGGL((fixed_mfma_kernel<5, 1>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            else hipLaunchKernelGGL((fixed_mfma_kernel<5, 2>), dim3(grid), dim3(256), lds, stream, xq16, wq16, wp16, out, q);
            break;
        default: break; // excluded by fixed_use_mfma
        }
        REXSC_CHECK_HIP(hipGetLastError());
        return REXSC_OK;
    }
    int32_t *xq = (int32_t *)workspace;
    int32_t *wq = (int32_t *)((uint8_t *)workspace + off_w);
    const size_t nx = (size_t)p.N * p.C * p.H * p.W, nw = (size_t)p.O * p.C * p.KH * p.KW;
    auto grid_for = [](size_t n) { size_t b = (n + 255) / 256; return (int)(b > 4096 ? 4096 : (b ? b : 1)); };
    hipLaunchKernelGGL(fixed_quant_kernel, dim3(grid_for(nx)), dim3(256), 0, stream, x, xq, nx, p.P2, 0);
    hipLaunchKernelGGL(fixed_quant_kernel, dim3(grid_for(nw)), dim3(256), 0, stream, w, wq, nw, p.P2, 1);
    REXSC_CHECK_HIP(hipGetLastError());
    const size_t nout = (size_t)p.N * p.O * p.Ho * p.Wo;
    const int grid = (int)((nout + 255) / 256 > 65536 ? 65536 : (nout + 255) / 256);
    ProfScope prof("fixed_conv", 4.0 * nx + 4.0 * nw + 4.0 * nout, stream);
    if (p.add_config == 0) hipLaunchKernelGGL(fixed_conv_kernel<0>, dim3(grid), dim3(256), 0, stream, xq, wq, out, p);
    else if (p.add_config == 1) hipLaunchKernelGGL(fixed_conv_kernel<1>, dim3(grid), dim3(256), 0, stream, xq, wq, out, p);
    else hipLaunchKernelGGL(fixed_conv_kernel<2>, dim3(grid), dim3(256), 0, stream, xq, wq, out, p);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}
