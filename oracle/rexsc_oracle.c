/*
 * rexsc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU-only restatement of the stochastic-computing (SC) algorithms of the
 * reference CPU extension (torch_c/sc-extension/{sc_cpu.hpp,sc_conv.cpp,sc_matmul.cpp,
 * fixed.cpp}).  It exists so that tests, the smoke check and the benchmark's CPU-baseline
 * leg have something to compare the HIP kernels against.  Nothing in the shipped library
 * links, loads or calls this file.
 *
 * Every function names the reference lines it follows.  The loops are written for
 * clarity first (one output at a time, no blocking); OpenMP only parallelises over
 * independent outputs.
 *
 * Pinning status (what fixes each function besides this text):
 *   orc_lfsr_step            period / fixed-point invariants + golden outputs (indirect)
 *   orc_quantize_*           closed form on grids + golden outputs (indirect)
 *   orc_conv2d               golden outputs of the compiled reference + dense {0,1} conv
 *                            special case + OR-1 "any" special case
 *   orc_conv2d, xnor = 1     (generators of the reference's CUDA kernels; no CUDA build or fixture
 *                            exists) LFSR cycle / complement invariants + per-bit brute-force model
 *                            written from sc_cuda_conv.cu, tests/test_oracle_invariants.py
 *   orc_linear               golden outputs of the compiled reference + matmul special case
 *   orc_fixed_conv2d         golden outputs of the compiled reference + closed form
 *   orc_orn_* / orc_bias_*   analytic closed forms in float64 (forward and derivative)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_PACK 32 /* channels per stream word: COMPUTE_CINS, sc_cpu.hpp:13 */
#define ORC_WEIGHT_SEED 13 /* POS_SEED == NEG_SEED, sc_cpu.hpp:10-11 */

/* ------------------------------------------------------------------------------------
 * LFSR steps.  sc_cpu.hpp:49-190.  Fibonacci form: feedback = XOR of the tap bits,
 * next = feedback + 2*(state mod 2^(lb-1)).  Taps (bit positions, MSB = lb-1):
 *   3:{2,1} 4:{3,2} 5:{4,2} 6:{5,4} 7:{6,5} 8:{7,5,4,3}
 * Flavours (`acc`): 0 plain; 1 the "_acc" variant, which splices the all-zero state into
 * the cycle: 1 -> 0 -> 2; 2 the XNOR variant of the reference's CUDA kernels
 * (sc_device.cuh:108-286, d_lfsr_N_xnor): feedback = 1 - XOR of the tap bits.
 * ---------------------------------------------------------------------------------- */
int orc_lfsr_step(int lb, int acc, int v)
{
    if (acc == 1) {
        if (v == 1) return 0;
        if (v == 0) return 2;
    }
    int fb;
    switch (lb) {
    case 3: fb = ((v >> 2) ^ (v >> 1)) & 1; break;            /* sc_cpu.hpp:135-137 */
    case 4: fb = ((v >> 3) ^ (v >> 2)) & 1; break;            /* :117-120 */
    case 5: fb = ((v >> 4) ^ (v >> 2)) & 1; break;            /* :100-103 */
    case 6: fb = ((v >> 5) ^ (v >> 4)) & 1; break;            /* :83-86  */
    case 7: fb = ((v >> 6) ^ (v >> 5)) & 1; break;            /* :66-69  */
    case 8: fb = ((v >> 7) ^ (v >> 5) ^ (v >> 4) ^ (v >> 3)) & 1; break; /* :49-52 */
    default: return -1;
    }
    if (acc == 2) fb = 1 - fb;                                /* sc_device.cuh:108,147,172,197,224,244 */
    return fb + 2 * (v & ((1 << (lb - 1)) - 1));
}

/* log2(bit_length) with the reference's switch fall-through: 2, 4 and 8 all give 3.
 * sc_conv.cpp:335-360, sc_matmul.cpp:600-625.  Returns -1 for unsupported lengths
 * (the reference leaves its function pointer uninitialised there). */
int orc_lfsr_bits(int bit_length, int lfsr_length)
{
    if (lfsr_length > 0) return (lfsr_length >= 3 && lfsr_length <= 8) ? lfsr_length : -1;
    switch (bit_length) {
    case 2: case 4: case 8: return 3;
    case 16: return 4;
    case 32: return 5;
    case 64: return 6;
    case 128: return 7;
    case 256: return 8;
    default: return -1;
    }
}

/* ------------------------------------------------------------------------------------
 * Float -> integer operand quantisation done by the host wrappers.
 *   SC:    sc_conv.cpp:316-320, sc_matmul.cpp:586-590   (ceil)
 *   fixed: fixed.cpp:207-210                            (round half to even)
 * All arithmetic is float32, as ATen does it: multiply, clamp, (negate), ceil/round.
 * which: 0 = activation / positive weight part, 1 = negative weight part.
 * ---------------------------------------------------------------------------------- */
void orc_quantize_sc(const float *x, int32_t *q, long n, int scale, int which)
{
    const float S = (float)scale;
    for (long i = 0; i < n; i++) {
        float v = x[i] * S;
        if (which == 0) {
            v = fminf(fmaxf(v, 0.f), S - 1.f);
            q[i] = (int32_t)ceilf(v);
        } else {
            v = fminf(fmaxf(v, 1.f - S), 0.f);
            q[i] = (int32_t)ceilf(-v);
        }
    }
}

void orc_quantize_fixed(const float *x, int32_t *q, long n, int scale, int which)
{
    const float S = (float)scale;
    for (long i = 0; i < n; i++) {
        float v = x[i] * S;
        if (which == 0) {
            v = fminf(fmaxf(v, 0.f), S - 1.f);
            q[i] = (int32_t)nearbyintf(v); /* default rounding mode = half to even */
        } else {
            v = fminf(fmaxf(v, 1.f - S), 0.f);
            q[i] = (int32_t)nearbyintf(-v);
        }
    }
}

/* Progressive-loading truncation of an operand at stream cycle `bit`.
 * sc_conv.cpp:107-115 (same text at :183-189 and sc_matmul.cpp:127-138). */
static inline int orc_truncate(int v, int bit, int total_width, int load_width, int load_wait)
{
    int cur_width = (bit / load_wait + 1) * load_width - 1;
    if (cur_width > total_width) cur_width = total_width;
    int sh = total_width - cur_width;
    return (v >> sh) << sh;
}

/* One 32-channel group -> bit_length stream words (one word per cycle, bit c = channel c).
 * State is stepped BEFORE the compare (sc_conv.cpp:118-122).  Lanes with seed 0 / value 0
 * (channels past the end) never produce a one. */
static void orc_sng_group(const int *val, const int *seed, int lb, int acc, int bit_length,
                          int total_width, int load_width, int load_wait, uint32_t *words)
{
    int state[ORC_PACK];
    for (int c = 0; c < ORC_PACK; c++) state[c] = seed[c];
    for (int bit = 0; bit < bit_length; bit++) {
        uint32_t w = 0;
        for (int c = 0; c < ORC_PACK; c++) {
            int actual = orc_truncate(val[c], bit, total_width, load_width, load_wait);
            state[c] = orc_lfsr_step(lb, acc, state[c]);
            w += (uint32_t)(actual > state[c]) << c;
        }
        words[bit] = w;
    }
}

/* ------------------------------------------------------------------------------------
 * SC conv2d.  sc_conv.cpp:42-299 (generation :42-200, compute :204-299) and the
 * orchestration of conv2d_generic_general :301-489 minus the float quantisation
 * (callers pass already quantised, already padded int32 operands).
 *
 * xq    [N][C][H][W] (cl_act=0) or [N][H][W][C] (cl_act=1); H,W are PADDED sizes.
 * wpos/wneg [O][C][KH][KW] (cl_w=0) or [O][KH][KW][C] (cl_w=1).
 * out_pos/out_neg int16 [N][O][Ho][Wo] (cl_act=0) or [N][Ho][Wo][O] (cl_act=1),
 *        Ho=(H-KH)/s0+1, Wo=(W-KW)/s1+1.
 * Seeds: activation (c*H*W + y*W + x) % P + 1, weight (13 + c*KH*KW + ky*KW + kx) % P + 1,
 *        P = 2^lb - 1 (sc_conv.cpp:80,92-93,167,173).
 * Cycle interleave for gen_config g (T = bit_length*g slots): weight cycle t fills slots
 *        t*g + j; activation cycle t fills slots (t/g)*g*g + j*g + t%g, j<g (:127-130,:195-197).
 * Per output and polarity: sum over slots of min(popcount total of the slot, n_sat); the
 *        running sum lives in 16 bits and wraps (:25-33, :286-294).
 * n_sat = bin_config+1 if bin_config>=0 else 1-bin_config (:216-224).
 * xnor = 0: the CPU extension, which ignores its xnor argument.  xnor = 1: the stream generators
 *        of the reference's CUDA kernels called with xnor = true (sc_cuda_conv.cu:3-166): the
 *        XNOR LFSR for every gen_config (:28,139 -- the CUDA kernels have no "_acc" variant) and
 *        seeds lowered by one, (...) % P + 1 - 1 (:55-56,139).  No CUDA build or fixture of the
 *        reference exists to compare with; pinned by LFSR invariants and a per-bit brute-force
 *        model written from the CUDA source, tests/test_oracle_invariants.py.  8-bit LFSRs are refused: the CUDA
 *        kernels keep states and operands in int8 (:37-40).
 * Returns 0, or -1 for an unsupported stream length / generator.
 * ---------------------------------------------------------------------------------- */
int orc_conv2d(const int32_t *xq, const int32_t *wpos, const int32_t *wneg,
               int16_t *out_pos, int16_t *out_neg,
               int N, int C, int H, int W, int O, int KH, int KW, int s0, int s1,
               int bit_length, int lfsr_length, int gen_config,
               int total_width, int load_width, int load_wait,
               int bin_config, int cl_act, int cl_w, int xnor)
{
    const int lb = orc_lfsr_bits(bit_length, lfsr_length);
    if (lb < 0 || gen_config < 1 || gen_config > 2) return -1;
    if (xnor && lb == 8) return -1;
    const int acc = xnor ? 2 : (gen_config == 2);
    const int seed_off = xnor ? 0 : 1;
    const int P = (1 << lb) - 1;
    const int Z = (C + ORC_PACK - 1) / ORC_PACK;
    const int g = gen_config;
    const int T = bit_length * g;
    const int n_sat = bin_config >= 0 ? bin_config + 1 : 1 - bin_config;
    const int Ho = (H - KH) / s0 + 1, Wo = (W - KW) / s1 + 1;

    const long wsz = (long)O * KH * KW * Z;  /* words per weight slot */
    const long asz = (long)N * H * W * Z;    /* words per activation slot */
    uint32_t *ws_pos = (uint32_t *)malloc(sizeof(uint32_t) * wsz * T);
    uint32_t *ws_neg = (uint32_t *)malloc(sizeof(uint32_t) * wsz * T);
    uint32_t *as = (uint32_t *)malloc(sizeof(uint32_t) * asz * T);
    if (!ws_pos || !ws_neg || !as) { free(ws_pos); free(ws_neg); free(as); return -2; }

    /* weight streams, layout [slot][o][ky][kx][z] */
#pragma omp parallel for schedule(static)
    for (long i = 0; i < wsz; i++) {
        int z = (int)(i % Z), kx = (int)((i / Z) % KW), ky = (int)((i / ((long)Z * KW)) % KH);
        int o = (int)(i / ((long)Z * KW * KH));
        int vp[ORC_PACK], vn[ORC_PACK], seed[ORC_PACK];
        uint32_t words_p[256], words_n[256];
        for (int cc = 0; cc < ORC_PACK; cc++) {
            int c = z * ORC_PACK + cc;
            if (c < C) {
                long wi = cl_w ? (((long)o * KH + ky) * KW + kx) * C + c
                               : (((long)o * C + c) * KH + ky) * KW + kx;
                vp[cc] = wpos[wi]; vn[cc] = wneg[wi];
                seed[cc] = (ORC_WEIGHT_SEED + c * KH * KW + ky * KW + kx) % P + seed_off;
            } else { vp[cc] = vn[cc] = seed[cc] = 0; }
        }
        orc_sng_group(vp, seed, lb, acc, bit_length, total_width, load_width, load_wait, words_p);
        orc_sng_group(vn, seed, lb, acc, bit_length, total_width, load_width, load_wait, words_n);
        for (int t = 0; t < bit_length; t++)
            for (int j = 0; j < g; j++) {
                ws_pos[(long)(t * g + j) * wsz + i] = words_p[t];
                ws_neg[(long)(t * g + j) * wsz + i] = words_n[t];
            }
    }
    /* activation streams, layout [slot][n][y][x][z] */
#pragma omp parallel for schedule(static)
    for (long i = 0; i < asz; i++) {
        int z = (int)(i % Z), x = (int)((i / Z) % W), y = (int)((i / ((long)Z * W)) % H);
        int n = (int)(i / ((long)Z * W * H));
        int v[ORC_PACK], seed[ORC_PACK];
        uint32_t words[256];
        for (int cc = 0; cc < ORC_PACK; cc++) {
            int c = z * ORC_PACK + cc;
            if (c < C) {
                long xi = cl_act ? (((long)n * H + y) * W + x) * C + c
                                 : (((long)n * C + c) * H + y) * W + x;
                v[cc] = xq[xi];
                seed[cc] = (c * H * W + y * W + x) % P + seed_off;
            } else { v[cc] = seed[cc] = 0; }
        }
        orc_sng_group(v, seed, lb, acc, bit_length, total_width, load_width, load_wait, words);
        for (int t = 0; t < bit_length; t++)
            for (int j = 0; j < g; j++)
                as[(long)((t / g) * g * g + j * g + t % g) * asz + i] = words[t];
    }
    /* compute */
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int o = 0; o < O; o++)
            for (int yo = 0; yo < Ho; yo++)
                for (int xo = 0; xo < Wo; xo++) {
                    uint32_t sum_p = 0, sum_n = 0; /* 16-bit running sums */
                    for (int t = 0; t < T; t++) {
                        const uint32_t *a_t = as + (long)t * asz + (long)n * H * W * Z;
                        const uint32_t *wp_t = ws_pos + (long)t * wsz + (long)o * KH * KW * Z;
                        const uint32_t *wn_t = ws_neg + (long)t * wsz + (long)o * KH * KW * Z;
                        uint32_t cp = 0, cn = 0;
                        for (int ky = 0; ky < KH; ky++)
                            for (int kx = 0; kx < KW; kx++) {
                                const uint32_t *a = a_t + ((long)(yo * s0 + ky) * W + (xo * s1 + kx)) * Z;
                                const uint32_t *wp = wp_t + (long)(ky * KW + kx) * Z;
                                const uint32_t *wn = wn_t + (long)(ky * KW + kx) * Z;
                                for (int z = 0; z < Z; z++) {
                                    cp += (uint32_t)__builtin_popcount(a[z] & wp[z]);
                                    cn += (uint32_t)__builtin_popcount(a[z] & wn[z]);
                                }
                            }
                        cp &= 0xffffu; cn &= 0xffffu; /* count is read back from the low half */
                        sum_p = (sum_p + (cp < (uint32_t)n_sat ? cp : (uint32_t)n_sat)) & 0xffffu;
                        sum_n = (sum_n + (cn < (uint32_t)n_sat ? cn : (uint32_t)n_sat)) & 0xffffu;
                    }
                    long oi = cl_act ? (((long)n * Ho + yo) * Wo + xo) * O + o
                                     : (((long)n * O + o) * Ho + yo) * Wo + xo;
                    out_pos[oi] = (int16_t)sum_p;
                    out_neg[oi] = (int16_t)sum_n;
                }
    free(ws_pos); free(ws_neg); free(as);
    return 0;
}

/* ------------------------------------------------------------------------------------
 * SC linear.  sc_matmul.cpp:3-676 (AVX-512 indexing: weight_ind = o*C + z*32, :77,:287).
 * xq [B][C], wpos/wneg [O][C] quantised int32; out_pos/out_neg int32 [B][O].
 * Always the plain (non "_acc") LFSR (:21-45,:235-255).  Seeds: activation c % P + 1,
 * weight (13 + c) % P + 1 (:100-101,:302).  The compute loop visits only the first
 * bit_length slots although bit_length*gen_config are generated (:422,:667).
 * bin_config < 0 selects the "nth bit only" rule [count >= n_sat] (:531-538).
 * ---------------------------------------------------------------------------------- */
int orc_linear(const int32_t *xq, const int32_t *wpos, const int32_t *wneg,
               int32_t *out_pos, int32_t *out_neg,
               int B, int C, int O, int bit_length, int lfsr_length, int gen_config,
               int total_width, int load_width, int load_wait, int bin_config)
{
    const int lb = orc_lfsr_bits(bit_length, lfsr_length);
    if (lb < 0 || gen_config < 1) return -1;
    const int P = (1 << lb) - 1;
    const int Z = (C + ORC_PACK - 1) / ORC_PACK;
    const int g = gen_config;
    const int T = bit_length * g;
    const int or_no = bin_config < 0;
    const int n_sat = bin_config >= 0 ? bin_config + 1 : 1 - bin_config;
    const long wsz = (long)O * Z, asz = (long)B * Z;
    uint32_t *ws_pos = (uint32_t *)malloc(sizeof(uint32_t) * wsz * T);
    uint32_t *ws_neg = (uint32_t *)malloc(sizeof(uint32_t) * wsz * T);
    /* When gen_config does not divide bit_length the activation interleave below reaches slots
     * past bit_length*gen_config (the reference writes past its buffer there; those slots are
     * never read).  Size the buffer for the highest slot written so the restatement stays defined. */
    const int T_act = ((bit_length + g - 1) / g) * g * g;
    uint32_t *as = (uint32_t *)malloc(sizeof(uint32_t) * asz * (T_act > T ? T_act : T));
    if (!ws_pos || !ws_neg || !as) { free(ws_pos); free(ws_neg); free(as); return -2; }

#pragma omp parallel for schedule(static)
    for (long i = 0; i < wsz; i++) {
        int o = (int)(i / Z), z = (int)(i % Z);
        int vp[ORC_PACK], vn[ORC_PACK], seed[ORC_PACK];
        uint32_t words_p[256], words_n[256];
        for (int cc = 0; cc < ORC_PACK; cc++) {
            int c = z * ORC_PACK + cc;
            seed[cc] = (ORC_WEIGHT_SEED + c) % P + 1;
            vp[cc] = c < C ? wpos[(long)o * C + c] : 0;
            vn[cc] = c < C ? wneg[(long)o * C + c] : 0;
        }
        orc_sng_group(vp, seed, lb, 0, bit_length, total_width, load_width, load_wait, words_p);
        orc_sng_group(vn, seed, lb, 0, bit_length, total_width, load_width, load_wait, words_n);
        for (int t = 0; t < bit_length; t++)
            for (int j = 0; j < g; j++) {
                ws_pos[(long)(t * g + j) * wsz + i] = words_p[t];
                ws_neg[(long)(t * g + j) * wsz + i] = words_n[t];
            }
    }
#pragma omp parallel for schedule(static)
    for (long i = 0; i < asz; i++) {
        int b = (int)(i / Z), z = (int)(i % Z);
        int v[ORC_PACK], seed[ORC_PACK];
        uint32_t words[256];
        for (int cc = 0; cc < ORC_PACK; cc++) {
            int c = z * ORC_PACK + cc;
            seed[cc] = c % P + 1;
            v[cc] = c < C ? xq[(long)b * C + c] : 0;
        }
        orc_sng_group(v, seed, lb, 0, bit_length, total_width, load_width, load_wait, words);
        for (int t = 0; t < bit_length; t++)
            for (int j = 0; j < g; j++)
                as[(long)((t / g) * g * g + j * g + t % g) * asz + i] = words[t];
    }
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++)
        for (int o = 0; o < O; o++) {
            int32_t sp = 0, sn = 0;
            for (int t = 0; t < bit_length; t++) { /* NOT T: see header */
                const uint32_t *a = as + (long)t * asz + (long)b * Z;
                const uint32_t *wp = ws_pos + (long)t * wsz + (long)o * Z;
                const uint32_t *wn = ws_neg + (long)t * wsz + (long)o * Z;
                int cp = 0, cn = 0;
                for (int z = 0; z < Z; z++) {
                    cp += __builtin_popcount(a[z] & wp[z]);
                    cn += __builtin_popcount(a[z] & wn[z]);
                }
                if (or_no) { sp += cp >= n_sat; sn += cn >= n_sat; }
                else { sp += cp < n_sat ? cp : n_sat; sn += cn < n_sat ? cn : n_sat; }
            }
            out_pos[(long)b * O + o] = sp;
            out_neg[(long)b * O + o] = sn;
        }
    free(ws_pos); free(ws_neg); free(as);
    return 0;
}

/* ------------------------------------------------------------------------------------
 * Saturating fixed-point conv.  fixed.cpp:56-195.
 * xq [N][C][H][W] (padded), wpos/wneg [O][C][KH][KW], out int32 [N][O][Ho][Wo] = pos - neg.
 * Products are folded in one at a time in (c, ky, kx) order through the saturating,
 * rounding add selected by add_config (0 fixed_add :61-64, 1 fixed_add_or :67-70,
 * >=2 the pairwise OR2 model :71-78,:150-190).
 * ---------------------------------------------------------------------------------- */
static inline int orc_saturate_shift(int value, int max_value, int d)
{   /* fixed.cpp:56-60 */
    int vs = value < max_value ? value : max_value;
    int round_bit = (vs >> (d - 1 > 0 ? d - 1 : 0)) % 2;
    /* The OR adders can hand a negative sum in.  The reference shifts it left as it is (what its compiler makes of
     * that is a multiplication by 2^d); written as the multiplication here, which is defined for negative values. */
    return ((vs >> d) + round_bit) * (1 << d);
}

typedef struct { int v1, v2; } orc_or2_t;

static inline orc_or2_t orc_add_or2(orc_or2_t a, orc_or2_t b, int max_value, int pin, int d)
{   /* fixed.cpp:71-78 */
    int o1 = a.v1 + b.v1 - (int)(((long)a.v1 * (long)a.v2 * (long)b.v2) >> (pin * 4))
             - (int)(((long)a.v2 * (long)b.v1 * (long)b.v2) >> (pin * 4))
             + (int)(((long)a.v1 * (long)a.v2 * (long)b.v1 * (long)b.v2) >> (pin * 6));
    int o2 = a.v2 + b.v2 - (int)(((long)a.v1 * (long)a.v2 * (long)b.v1) >> (pin * 4))
             - (int)(((long)a.v1 * (long)b.v1 * (long)b.v2) >> (pin * 4))
             + (int)(((long)a.v1 * (long)a.v2 * (long)b.v1 * (long)b.v2) >> (pin * 6));
    orc_or2_t r = { orc_saturate_shift(o1, max_value, d), orc_saturate_shift(o2, max_value, d) };
    return r;
}

int orc_fixed_conv2d(const int32_t *xq, const int32_t *wpos, const int32_t *wneg, int32_t *out,
                     int N, int C, int H, int W, int O, int KH, int KW, int s0, int s1,
                     int add_config, int precision_in, int precision_out)
{
    int pmax = 2 * precision_in > precision_out ? 2 * precision_in : precision_out;
    if (pmax > 31) pmax = 31;                                  /* fixed.cpp:95 */
    int d = 2 * precision_in - precision_out; if (d < 0) d = 0; /* :97 */
    int max_value = (int)((((unsigned)1 << pmax) - 1u) >> d) << d; /* :96,:98 */
    const int Ho = (H - KH) / s0 + 1, Wo = (W - KW) / s1 + 1;
    const int pin = precision_in;
    if (add_config < 0) return -1;

#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int o = 0; o < O; o++)
            for (int yo = 0; yo < Ho; yo++)
                for (int xo = 0; xo < Wo; xo++) {
                    const int32_t *xb = xq + (long)n * C * H * W;
                    const int32_t *wp = wpos + (long)o * C * KH * KW;
                    const int32_t *wn = wneg + (long)o * C * KH * KW;
                    int result;
                    if (add_config < 2) {
                        int sp = 0, sn = 0;
                        for (int c = 0; c < C; c++)
                            for (int ky = 0; ky < KH; ky++)
                                for (int kx = 0; kx < KW; kx++) {
                                    int a = xb[((long)c * H + yo * s0 + ky) * W + xo * s1 + kx];
                                    int pp = a * wp[(c * KH + ky) * KW + kx];
                                    int pn = a * wn[(c * KH + ky) * KW + kx];
                                    if (add_config == 0) {
                                        sp = orc_saturate_shift(sp + pp, max_value, d);
                                        sn = orc_saturate_shift(sn + pn, max_value, d);
                                    } else {
                                        sp = orc_saturate_shift(sp + pp - (int)((sp * pp) >> (pin * 2)), max_value, d);
                                        sn = orc_saturate_shift(sn + pn - (int)((sn * pn) >> (pin * 2)), max_value, d);
                                    }
                                }
                        result = sp - sn;
                    } else {
                        orc_or2_t sp = {0, 0}, sn = {0, 0};
                        const int KK = KH * KW, total = C * KK;
                        int i = 0;
                        for (; i + 1 < total; i += 2) {
                            int a[2], pw[2], nw[2];
                            for (int j = 0; j < 2; j++) {
                                int c = (i + j) / KK, ky = ((i + j) % KK) / KW, kx = (i + j) % KW;
                                a[j] = xb[((long)c * H + yo * s0 + ky) * W + xo * s1 + kx];
                                pw[j] = wp[i + j]; nw[j] = wn[i + j];
                            }
                            orc_or2_t pp = { a[0] * pw[0], a[1] * pw[1] };
                            orc_or2_t pn = { a[0] * nw[0], a[1] * nw[1] };
                            sp = orc_add_or2(sp, pp, max_value, pin, d);
                            sn = orc_add_or2(sn, pn, max_value, pin, d);
                        }
                        if (i < total) {
                            int c = i / KK, ky = (i % KK) / KW, kx = i % KW;
                            int a = xb[((long)c * H + yo * s0 + ky) * W + xo * s1 + kx];
                            orc_or2_t pp = { a * wp[i], 0 }, pn = { a * wn[i], 0 };
                            sp = orc_add_or2(sp, pp, max_value, pin, d);
                            sn = orc_add_or2(sn, pn, max_value, pin, d);
                        }
                        result = sp.v1 + sp.v2 - sn.v1 - sn.v2;
                    }
                    out[(((long)n * O + o) * Ho + yo) * Wo + xo] = result;
                }
    return 0;
}

/* ------------------------------------------------------------------------------------
 * Pointwise closed forms, float32 with the reference's fmaf order.  sc_cpu.hpp:192-404.
 * ---------------------------------------------------------------------------------- */
float orc_orn_forward_s(float x, int n)
{
    float e = expf(-x);
    float x2 = x * x, x3 = x2 * x, r;
    switch (n) {
    case 1: return 1 - e;                                            /* :192-196 */
    case 2: r = fmaf(-2.f, e, 2.f); return fmaf(-x, e, r);            /* :198-203 */
    case 3: r = fmaf(-3.f, e, 3.f); r = fmaf(-2.f * x, e, r);         /* :205-213 */
            return fmaf(-0.5f * x2, e, r);
    case 4: r = fmaf(-4.f, e, 4.f); r = fmaf(-3.f * x, e, r);         /* :215-225 */
            r = fmaf(-x2, e, r); return fmaf((-1.f / 6.f) * x3, e, r);
    default: return NAN;
    }
}

float orc_orn_backward_s(float g, float x, int n)
{
    float e = expf(-x);
    float x2 = x * x, x3 = x2 * x, r;
    switch (n) {
    case 1: return e * g;                                             /* :227-232 */
    case 2: r = fmaf(x, e, e); return r * g;                          /* :234-240 */
    case 3: r = fmaf(x, e, e); r = fmaf(0.5f * x2, e, r); return r * g;        /* :242-250 */
    case 4: r = fmaf(x, e, e); r = fmaf(0.5f * x2, e, r);             /* :252-262 */
            r = fmaf((1.f / 6.f) * x3, e, r); return r * g;
    default: return NAN;
    }
}

float orc_bias_forward_s(float x, float xi, const float *b, const float *s)
{   /* sc_cpu.hpp:264-284 */
    float x2 = x * x, x3 = x2 * x, x4 = x3 * x, x5 = x4 * x;
    float xb = fmaf(b[1], x, b[0]);
    xb = fmaf(b[2], x2, xb); xb = fmaf(b[3], x3, xb); xb = fmaf(b[4], x4, xb); xb = fmaf(b[5], x5, xb);
    float xs = fmaf(s[1], x, s[0]);
    xs = fmaf(s[2], x2, xs); xs = fmaf(s[3], x3, xs); xs = fmaf(s[4], x4, xs); xs = fmaf(s[5], x5, xs);
    return x + xb + xs * xi;
}

float orc_bias_backward_s(float x, const float *b)
{   /* sc_cpu.hpp:286-297 */
    float x2 = x * x, x3 = x2 * x, x4 = x3 * x;
    float xd = fmaf(2.f * b[2], x, 1.f + b[1]);
    xd = fmaf(3.f * b[3], x2, xd); xd = fmaf(4.f * b[4], x3, xd); xd = fmaf(5.f * b[5], x4, xd);
    return xd;
}

/* Array drivers.  half_input != 0 rounds the saved pre-activation to IEEE binary16 first,
 * which is what the GPU host wrappers of the reference do on the backward pass
 * (sc_cuda_pw.cu:775,962-963); the rounding itself is done by the caller (numpy). */
void orc_orn_forward(const float *x, float *y, long n, int or_n)
{
    for (long i = 0; i < n; i++) y[i] = orc_orn_forward_s(x[i], or_n);
}

void orc_orn_backward(const float *g, const float *x, float *gx, long n, int or_n)
{
    for (long i = 0; i < n; i++) gx[i] = orc_orn_backward_s(g[i], x[i], or_n);
}

/* y = biasnoise(OR_n(x_pos), xi_pos) - biasnoise(OR_n(x_neg), xi_neg)
 * sc_cpu.hpp:299-333 composed as in sc_cuda_pw.cu:219-373 (noise supplied by the caller). */
void orc_orn_bias_std_both_forward(const float *xp, const float *xn, const float *xi_p,
                                   const float *xi_n, const float *b, const float *s,
                                   float *y, long n, int or_n)
{
    for (long i = 0; i < n; i++) {
        float p = orc_bias_forward_s(orc_orn_forward_s(xp[i], or_n), xi_p[i], b, s);
        float q = orc_bias_forward_s(orc_orn_forward_s(xn[i], or_n), xi_n[i], b, s);
        y[i] = p - q;
    }
}

/* sc_cpu.hpp:335-404 applied with +g to the positive and -g to the negative branch
 * (sc_cuda_pw.cu:541-547). */
void orc_orn_bias_std_both_backward(const float *g, const float *xp, const float *xn,
                                    const float *b, float *gp, float *gn, long n, int or_n)
{
    for (long i = 0; i < n; i++) {
        float yp = orc_orn_forward_s(xp[i], or_n), yn = orc_orn_forward_s(xn[i], or_n);
        gp[i] = orc_orn_backward_s(orc_bias_backward_s(yp, b) * g[i], xp[i], or_n);
        gn[i] = orc_orn_backward_s(orc_bias_backward_s(yn, b) * (-g[i]), xn[i], or_n);
    }
}

/* Number of OpenMP threads the parallel loops above will use (for reporting). */
#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
#else
int orc_num_threads(void) { return 1; }
#endif
