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
// (C*KH*KW*((2^pin-1)^2+1) < max_value+1).  Then pos - neg collapses to ONE signed contraction with
// the reduction doubled:  out = sum a*w  +  sum (a&1) * sgn(w)*(|w|&1).
//
// Operands are re-laid-out once, channel-blocked by 8 so that every MFMA operand fetch is an
// 8-byte load and adjacent lanes read adjacent memory:
//   xq8[n][cb][yp][xp][8]   int8, zero padded plane; blocks [0,CBV) values, [CBV,2*CBV) parities
//   wq8[cb][ky][kx][o_pad][8] int8, same block order
// GEMM orientation: MFMA rows = output channels (weights are the A operand), MFMA columns =
// pixels (activations are the B operand), so that the 32 lanes of a half-wave hold 32
// consecutive pixels of one output channel and the int32 NCHW stores are 128-byte runs.
typedef int v16i __attribute__((ext_vector_type(16)));

struct Fixed8Params {
    int N, C, H, W, O, O_pad, KH, KW;
    int pad_h, pad_w, s0, s1, Hp, Wp, Ho, Wo;
    int CBV, CB; // value blocks, total blocks (= 2*CBV)
    int M;       // N*Ho*Wo
    float P2;
};

__global__ __launch_bounds__(256) void fixed_pack_act8_kernel(const float *__restrict__ x, int8_t *__restrict__ xq8,
                                                              Fixed8Params p)
{
    // one thread per (n, cbv, yp, xp): 8 channels -> one value block and one parity block
    const long total = (long)p.N * p.CBV * p.Hp * p.Wp;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int xp = (int)(i % p.Wp);
        const int yp = (int)((i / p.Wp) % p.Hp);
        const int cbv = (int)((i / ((long)p.Wp * p.Hp)) % p.CBV);
        const int n = (int)(i / ((long)p.Wp * p.Hp * p.CBV));
        const int y = yp - p.pad_h, xx = xp - p.pad_w;
        const bool inb = y >= 0 && y < p.H && xx >= 0 && xx < p.W;
        uint64_t vals = 0, pars = 0;
        if (inb) {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int c = cbv * 8 + k;
                if (c < p.C) {
                    const int q = quant_round_pos(x[(((long)n * p.C + c) * p.H + y) * p.W + xx], p.P2);
                    vals |= (uint64_t)(uint8_t)q << (8 * k);
                    pars |= (uint64_t)(q & 1) << (8 * k);
                }
            }
        }
        const long plane = (long)p.Hp * p.Wp;
        uint64_t *dst = reinterpret_cast<uint64_t *>(xq8);
        dst[((long)n * p.CB + cbv) * plane + (long)yp * p.Wp + xp] = vals;
        dst[((long)n * p.CB + p.CBV + cbv) * plane + (long)yp * p.Wp + xp] = pars;
    }
}

__global__ __launch_bounds__(256) void fixed_pack_w8_kernel(const float *__restrict__ w, int8_t *__restrict__ wq8,
                                                            Fixed8Params p)
{
    const long total = (long)p.CBV * p.KH * p.KW * p.O_pad;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int o = (int)(i % p.O_pad);
        const int kx = (int)((i / p.O_pad) % p.KW);
        const int ky = (int)((i / ((long)p.O_pad * p.KW)) % p.KH);
        const int cbv = (int)(i / ((long)p.O_pad * p.KW * p.KH));
        uint64_t vals = 0, pars = 0;
        if (o < p.O) {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int c = cbv * 8 + k;
                if (c < p.C) {
                    const float f = w[(((long)o * p.C + c) * p.KH + ky) * p.KW + kx];
                    const int q = quant_round_pos(f, p.P2) - quant_round_neg(f, p.P2); // signed
                    const int par = (q & 1) ? (q < 0 ? -1 : 1) : 0;
                    vals |= (uint64_t)(uint8_t)(int8_t)q << (8 * k);
                    pars |= (uint64_t)(uint8_t)(int8_t)par << (8 * k);
                }
            }
        }
        uint64_t *dst = reinterpret_cast<uint64_t *>(wq8);
        const long kk = (long)p.KH * p.KW * p.O_pad;
        dst[(long)cbv * kk + ((long)ky * p.KW + kx) * p.O_pad + o] = vals;
        dst[(long)(p.CBV + cbv) * kk + ((long)ky * p.KW + kx) * p.O_pad + o] = pars;
    }
}

// One wave computes a 64 (channels) x 64 (pixels) tile with four 32x32x16 int8 MFMAs per step.
// A step covers 16 reduction entries: one (ky,kx) tap of a PAIR of 8-channel blocks; lanes 0..31
// feed block 2*cbp, lanes 32..63 block 2*cbp+1 (the MFMA's k = 8*(lane/32) + byte).
constexpr int FT = 64;
__global__ __launch_bounds__(256) void fixed_mfma_kernel(const int8_t *__restrict__ xq8, const int8_t *__restrict__ wq8,
                                                         int32_t *__restrict__ out, Fixed8Params p)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int o_tiles = p.O_pad / FT;
    const long tile = (long)blockIdx.x * 4 + wave;
    const long m_tiles = (p.M + FT - 1) / FT;
    if (tile >= m_tiles * o_tiles) return;
    const int otile = (int)(tile % o_tiles);
    const long mtile = tile / o_tiles;
    const int j = lane & 31, h = lane >> 5;
    const long plane = (long)p.Hp * p.Wp;

    // the two pixel columns of this lane (pixel blocks 0 and 1 of the tile)
    long xoff[2];
    int mm[2];
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
        long m = mtile * FT + pb * 32 + j;
        mm[pb] = (int)(m < p.M ? m : p.M - 1);
        const int n = mm[pb] / (p.Ho * p.Wo), r = mm[pb] - n * (p.Ho * p.Wo);
        const int yo = r / p.Wo, xo = r - yo * p.Wo;
        xoff[pb] = (long)n * p.CB * plane + (long)(yo * p.s0) * p.Wp + xo * p.s1;
        if (m >= p.M) mm[pb] = -1;
    }
    const uint64_t *xb = reinterpret_cast<const uint64_t *>(xq8);
    const uint64_t *wb = reinterpret_cast<const uint64_t *>(wq8);
    const long wkk = (long)p.KH * p.KW * p.O_pad;

    v16i acc[2][2]; // [channel block][pixel block]
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0;

    for (int cbp = 0; cbp < p.CB / 2; cbp++) {
        const int cb = 2 * cbp + h;
        const uint64_t *xc = xb + (long)cb * plane;
        const uint64_t *wc = wb + (long)cb * wkk + otile * FT + j;
        for (int ky = 0; ky < p.KH; ky++)
            for (int kx = 0; kx < p.KW; kx++) {
                const long tap = (long)ky * p.Wp + kx;
                const long b0 = (long)xc[xoff[0] + tap], b1 = (long)xc[xoff[1] + tap];
                const uint64_t *wt = wc + ((long)ky * p.KW + kx) * p.O_pad;
                const long a0 = (long)wt[0], a1 = (long)wt[32];
                acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(a0, b0, acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_i32_32x32x16_i8(a0, b1, acc[0][1], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(a1, b0, acc[1][0], 0, 0, 0);
                acc[1][1] = __builtin_amdgcn_mfma_i32_32x32x16_i8(a1, b1, acc[1][1], 0, 0, 0);
            }
    }
    // D[i][j]: column j = lane%32, row i = 8*(r/4) + 4*(lane/32) + r%4
    const int HoWo = p.Ho * p.Wo;
#pragma unroll
    for (int pb = 0; pb < 2; pb++) {
        if (mm[pb] < 0) continue;
        const int n = mm[pb] / HoWo, r0 = mm[pb] - n * HoWo;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int o = otile * FT + a * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                if (o < p.O) out[((long)n * p.O + o) * HoWo + r0] = acc[a][pb][r];
            }
    }
}

// The MFMA path is exact only where the per-product saturating add is provably inert.
static bool fixed_use_mfma(const FixedParams &p)
{
    if (p.add_config != 0 || p.d != 0 || p.pin > 7) return false;
    const long pm = (1L << p.pin) - 1;
    const long bound = (long)p.C * p.KH * p.KW * (pm * pm + 1); // largest possible rounded sum of one polarity
    return bound < (long)p.max_value + 1 && (long)p.N * p.Ho * p.Wo < (1L << 31);
}

static int fixed_plan(const rexsc_fixed_desc *d, FixedParams &p, size_t &off_w, size_t &total)
{
    REXSC_CHECK_ARG(d != nullptr, "null descriptor");
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
        const int CBV = ceil_div(p.C, 8);
        const int O_pad = (int)align_up((size_t)p.O, FT);
        xbytes = (size_t)p.N * 2 * CBV * (p.H + 2 * p.pad_h) * (p.W + 2 * p.pad_w) * 8;
        wbytes = (size_t)2 * CBV * p.KH * p.KW * O_pad * 8;
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
        q.CBV = ceil_div(p.C, 8); q.CB = 2 * q.CBV; q.M = p.N * p.Ho * p.Wo; q.P2 = p.P2;
        int8_t *xq8 = (int8_t *)workspace;
        int8_t *wq8 = (int8_t *)workspace + off_w;
        auto gridf = [](long n) { long b = (n + 255) / 256; return (int)(b > 8192 ? 8192 : (b ? b : 1)); };
        const double io_bytes = 4.0 * p.N * p.C * p.H * p.W + 4.0 * p.O * p.C * p.KH * p.KW + 4.0 * p.N * p.O * p.Ho * p.Wo;
        {
            ProfScope prof("fixed_pack", 4.0 * p.N * p.C * p.H * p.W + 8.0 * q.N * q.CB * q.Hp * q.Wp, stream);
            hipLaunchKernelGGL(fixed_pack_act8_kernel, dim3(gridf((long)q.N * q.CBV * q.Hp * q.Wp)), dim3(256), 0, stream,
                               x, xq8, q);
            hipLaunchKernelGGL(fixed_pack_w8_kernel, dim3(gridf((long)q.CBV * q.KH * q.KW * q.O_pad)), dim3(256), 0,
                               stream, w, wq8, q);
        }
        REXSC_CHECK_HIP(hipGetLastError());
        const long tiles = (long)ceil_div(q.M, FT) * (q.O_pad / FT);
        ProfScope prof("fixed_conv_mfma", io_bytes, stream);
        hipLaunchKernelGGL(fixed_mfma_kernel, dim3((unsigned)((tiles + 3) / 4)), dim3(256), 0, stream, xq8, wq8, out, q);
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
