/*
 * rexsc.h -- C ABI of librexsc.so: the MI355X (gfx950) implementation of REX-SC's
 * stochastic-computing hot path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream; no torch types.
 * All return 0 on success and a negative code on failure; rexsc_last_error() returns the
 * message of the calling thread's last failure.  Nothing here allocates device memory:
 * ops that need scratch take a caller-owned workspace whose size the matching
 * *_workspace_bytes() call reports (rexsc_conv2d_orn_noalloc uses a static device array instead).  Inputs are never written.  Work is enqueued on
 * `stream` and the call returns without synchronising.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference tree, torch_c/sc-extension/ unless stated otherwise).
 */
#ifndef REXSC_H
#define REXSC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *rexsc_stream_t; /* hipStream_t */

enum {
    REXSC_OK = 0,
    REXSC_ERR_INVALID = -1,   /* bad argument / unsupported configuration */
    REXSC_ERR_WORKSPACE = -2, /* workspace missing or too small */
    REXSC_ERR_HIP = -3        /* a HIP runtime call failed */
};

const char *rexsc_last_error(void);

/* ABI version of the library.  It changes whenever a descriptor below changes its layout or an entry point its
 * signature; a caller built against another header must refuse to go on.  Every descriptor also starts with its own
 * size in bytes (struct_size = sizeof of the structure as the caller's header declares it): the library rejects a
 * descriptor whose size is not the one it was compiled with instead of reading past it. */
#define REXSC_ABI_VERSION 200
int rexsc_version(void);

/* One-time per-device set-up (LFSR sequence tables).  Called implicitly by the ops; exposed
 * so that a caller can pay for it outside a timed or captured region. */
int rexsc_init(rexsc_stream_t stream);

/* ---- SC conv2d -------------------------------------------------------------------------
 * Replaces sc_extension_cuda.conv2d_generic_general_split_acc / conv2d_generic_general_acc
 * (sc_cuda.cpp:73-99) and sc_extension.conv2d_generic_general (sc_conv.cpp:301-489), with
 * the arithmetic of the CPU extension: float operands are scaled by S (= bit_length, or
 * 2^lfsr_length when lfsr_length > 0), clamped and ceil'ed to integers, expanded to LFSR
 * bitstreams (XOR-feedback LFSR, seeds 1..2^lb-1), AND-multiplied, popcounted over the whole
 * Cin*KH*KW reduction per stream cycle, clamped to n_sat per cycle and summed over cycles.
 * desc.xnor = 1 switches the stream generators to those of the reference's CUDA kernels.
 */
typedef struct rexsc_conv_desc {
    int32_t struct_size;         /* sizeof(rexsc_conv_desc) */
    int32_t N, C, H, W;          /* activation dims, UNPADDED */
    int32_t O, KH, KW;           /* weight dims [O][C][KH][KW] */
    int32_t pad_h, pad_w;        /* zero padding of axis 2 / axis 3 (the reference's padding[1] / padding[0]) */
    int32_t stride_h, stride_w;  /* stride along axis 2 / axis 3 (the reference's stride[0] / stride[1]) */
    int32_t bit_length;          /* stream length L */
    int32_t lfsr_length;         /* <=0: derive from L (2,4,8->3; 16->4; ... 256->8) */
    int32_t gen_config;          /* 1 plain LFSR, 2 "and_2" generator (zero-including LFSR, 2x2 cycle interleave) */
    int32_t bin_config;          /* n_sat = bin_config+1 if >=0 else 1-bin_config */
    int32_t total_width, load_width, load_wait; /* progressive loading (7,8,1 = off) */
    int32_t act_channels_last;   /* memory order of x: 0 NCHW, 1 NHWC; outputs use the same order */
    int32_t weight_channels_last;/* memory order of w: 0 OIHW, 1 OHWI */
    int32_t xnor;                /* 0: the CPU extension's generator (it ignores its xnor argument, sc_conv.cpp:362-425);
                                  * 1: the generator of the reference's CUDA conv kernels called with xnor = true
                                  *    (sc_cuda_conv.cu:28,55-56,139; sc_device.cuh:108-286): XNOR-feedback LFSR,
                                  *    seeds (index % (2^lb-1)) + 0, the same LFSR for gen_config 2; lb <= 7 */
    int32_t act_fake_quant;      /* k > 0: x first goes through the layers' fake quantisation with prec = k - 1,   */
    int32_t weight_fake_quant;   /* clamp(round(v * 2^prec), +-(2^prec - 1)) / 2^prec (QuantizeGrad's forward,      */
                                 /* utils_functional.py:93-104, 117-123; utils_class.py:54,62); 0: operand as given */
} rexsc_conv_desc;

size_t rexsc_conv2d_workspace_bytes(const rexsc_conv_desc *d);

/* Planning decisions for a descriptor (no counterpart in the reference; for tests and tuning):
 * out[0..15] = {tuned kernel?, KW, words per chunk, chunks, O padded, pixels per lane, waves per
 * block, slot splits, slots per split, slots, direct store?, images per batch chunk, output pixels
 * per chunk, padded H, padded W, wide accumulators?}. */
int rexsc_conv2d_plan_info(const rexsc_conv_desc *d, int64_t *out);

/* x, w: float32 device arrays in the memory order the descriptor states.
 * out_pos, out_neg: int16 [N][O][Ho][Wo] (or NHWC), Ho=(H+2*pad_h-KH)/stride_h+1.
 * Either output pointer may be NULL together with out_diff != NULL to get pos-neg (int16,
 * wrapping) instead; all three may be given. */
int rexsc_conv2d_orn(const rexsc_conv_desc *d, const float *x, const float *w,
                     int16_t *out_pos, int16_t *out_neg, int16_t *out_diff,
                     void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* The same op with two optional extras for the caller conv2d_generic (utils_functional.py:1083-1317):
 *  - out_value: float32 pos / L - neg / L in the layout of the int16 outputs -- the int16 -> float, "/ bit_length"
 *    and "pos - neg" passes of :1181-1182, 1273-1274, 1317 done in the kernel that produces the sums (any of the
 *    three int16 outputs may then be NULL and is not written);
 *  - weight_streams: a caller-owned buffer of rexsc_conv2d_weight_streams_bytes() that receives the weight
 *    bitstreams, the generator table that goes with the descriptor and a copy of the weights they were made
 *    from: frozen weights (evaluation, utils_class.py:54 under no_grad) are expanded once, not per call.
 *    weight_streams_valid says what the buffer holds when the call starts:
 *      REXSC_WSTREAMS_FILL    nothing: generate, and keep the copy of w;
 *      REXSC_WSTREAMS_TRUST   the streams of this descriptor and of these weight values, on the caller's word:
 *                             generation is skipped and w may be NULL;
 *      REXSC_WSTREAMS_VERIFY  the streams of this descriptor, filled by an earlier call on the same device; whether
 *                             the weights are still the same is decided ON THE DEVICE: a small kernel compares w
 *                             bit for bit with the kept copy (updating it) and the generator's blocks return at
 *                             once when nothing differs.  No host synchronisation; in-place edits of w that no
 *                             host-side bookkeeping sees (the reference's own `p.weight.data.clamp_(-1, 0.999)`,
 *                             utils_own.py:187-190) are caught.  Under HIP graph capture the comparison is part
 *                             of the graph and repeats on every replay. */
enum { REXSC_WSTREAMS_FILL = 0, REXSC_WSTREAMS_TRUST = 1, REXSC_WSTREAMS_VERIFY = 2 };
size_t rexsc_conv2d_weight_streams_bytes(const rexsc_conv_desc *d);
int rexsc_conv2d_orn_ex(const rexsc_conv_desc *d, const float *x, const float *w,
                        int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, float *out_value,
                        void *weight_streams, size_t weight_streams_bytes, int weight_streams_valid,
                        void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* The weight half of rexsc_conv2d_orn_ex on its own (no counterpart in the reference, whose conv2d_generic_general
 * expands the weights inside every call, sc_conv.cpp:432-450): fills weight_streams as a call in mode
 * REXSC_WSTREAMS_FILL does and returns; the conv call proper follows in mode REXSC_WSTREAMS_TRUST on a stream ordered
 * after this one (or, when keep_weight_copy != 0 also stored the copy of w that mode compares with, in mode _VERIFY).
 * A layer's weight streams depend on its weights alone, so a caller can have them generated on a second stream while
 * the previous layer still computes. */
int rexsc_conv2d_prepare_weights(const rexsc_conv_desc *d, const float *w, void *weight_streams,
                                 size_t weight_streams_bytes, int keep_weight_copy, rexsc_stream_t stream);

/* The same op for callers that cannot allocate device memory or hand over a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  The workspace is a static device array inside the library
 * (REXSC_NOALLOC_SCRATCH_BYTES, held on every GPU the library runs on until the process ends); the
 * call makes no hipMalloc / hipFree and calls no allocating routine.  Problems whose workspace
 * (rexsc_conv2d_workspace_bytes) exceeds the array are rejected with REXSC_ERR_WORKSPACE.  All calls
 * on one GPU share the array: calls that overlap on one GPU (different streams or threads) race.
 * Call rexsc_init() once per device before the first call that runs under stream capture. */
#define REXSC_NOALLOC_SCRATCH_BYTES (32u << 20)
int rexsc_conv2d_orn_noalloc(const rexsc_conv_desc *d, const float *x, const float *w,
                             int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, rexsc_stream_t stream);

/* ---- SC linear -------------------------------------------------------------------------
 * Replaces sc_extension_cuda.linear_generic_general_acc (sc_cuda.cpp:101-120) and
 * sc_extension.linear_generic_general (sc_matmul.cpp:576-676).  x [B][C], w [O][C] float32
 * row-major; out_pos/out_neg int32 [B][O].  Only the first bit_length stream slots are
 * accumulated, and bin_config < 0 selects the "count >= n_sat" rule, as in the reference.
 */
typedef struct rexsc_linear_desc {
    int32_t struct_size;         /* sizeof(rexsc_linear_desc) */
    int32_t B, C, O;
    int32_t bit_length, lfsr_length, gen_config, bin_config;
    int32_t total_width, load_width, load_wait;
    int32_t act_fake_quant;      /* as in rexsc_conv_desc: k > 0 applies the layers' fake quantisation with       */
    int32_t weight_fake_quant;   /* prec = k - 1 to the operand inside the generator (utils_class.py:196-201)    */
} rexsc_linear_desc;

size_t rexsc_linear_workspace_bytes(const rexsc_linear_desc *d);
int rexsc_linear_orn(const rexsc_linear_desc *d, const float *x, const float *w,
                     int32_t *out_pos, int32_t *out_neg,
                     void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* rexsc_linear_orn with the weight bitstreams in a caller-owned buffer of rexsc_linear_weight_streams_bytes(d)
 * bytes, as rexsc_conv2d_orn_ex keeps them for the conv op (weight_streams_valid: REXSC_WSTREAMS_FILL / _TRUST /
 * _VERIFY with the same meaning; the batch size B is not part of what the buffer depends on as long as
 * rexsc_linear_weight_streams_bytes() returns the same value).  The reference regenerates them on every call
 * (sc_matmul.cpp:576-676) although its layers hold their weights fixed in evaluation (utils_class.py:54). */
size_t rexsc_linear_weight_streams_bytes(const rexsc_linear_desc *d);
int rexsc_linear_orn_ex(const rexsc_linear_desc *d, const float *x, const float *w,
                        int32_t *out_pos, int32_t *out_neg,
                        void *weight_streams, size_t weight_streams_bytes, int weight_streams_valid,
                        void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* The reference's legacy pure-torch simulation `linear_generic` (utils_functional.py:955-1081 with the
 * generators of :147-165, 254-272; generator 'lfsr', shared generators; what its Linear_Or layer runs,
 * utils_class.py:183-208) on the same kernels: operands q = ceil(float16(x * L)) with activations
 * unclamped and weight parts clamped to weight_clamp (the function's `prec - 1`: 127), seeds
 * (67 + c) % P + 1 / (37 + c) % P + 1 for the positive / negative weight part and c % P + 1 for
 * activations, P = L - 1; share = 0 is the function's share=False: one generator per element, the index c replaced
 * by the element's index in the whole tensor (o * C + c for weights, b * C + c for activations; :996-998).
 * bin_config 0 is its forward 'full_or' (per-cycle OR), 51200 its 'full_bin'.
 * bit_length 8..128, lfsr_length <= 0, gen_config 1, no progressive loading.  Outputs are the per-output
 * sums over the L cycles (the function returns them divided by L).  Workspace: rexsc_linear_workspace_bytes. */
int rexsc_linear_legacy(const rexsc_linear_desc *d, int weight_clamp, int share, const float *x, const float *w,
                        int32_t *out_pos, int32_t *out_neg,
                        void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* ---- OR-n pointwise activation ---------------------------------------------------------
 * y = n - exp(-x) * sum_{i<n} (n-i) x^i / i!  for n = 1..4, float32.
 * Replaces sc_extension_cuda.or_approx_n_forward_acc / _backward_acc (sc_cuda_pw.cu:708-811);
 * scalar math of sc_cpu.hpp:192-262.  half_input != 0 rounds the saved pre-activation to
 * IEEE binary16 before use, which is what the reference's backward wrapper does. */
int rexsc_orn_forward(const float *x, float *y, size_t n, int or_n, rexsc_stream_t stream);
int rexsc_orn_backward(const float *grad_out, const float *x, float *grad_in, size_t n, int or_n,
                       int half_input, rexsc_stream_t stream);

/* ---- fused OR-n + bias/noise error injection, both polarities --------------------------
 * y = f(OR_n(x_pos), xi1) - f(OR_n(x_neg), xi2),  f(v, xi) = v + poly5_bias(v) + poly5_std(v)*xi,
 * xi ~ N(0,1) from a counter-based Philox4x32-10 stream keyed by (seed, offset + element/4).
 * Replaces sc_extension_cuda.or_approx_n_forward_bias_std_both_acc / _backward_..._both_acc
 * (sc_cuda_pw.cu:863-927, 952-1011); scalar math of sc_cpu.hpp:264-404.
 * bias_coef / std_coef: 6 float32 coefficients each, device memory.
 * noise_out_pos / noise_out_neg: optional float32 [n] receiving the draws (NULL to skip).  When both are NULL
 * the kernel draws ONE normal per output and scales it by sqrt(poly5_std(v_pos)^2 + poly5_std(v_neg)^2): the
 * difference of the two independent noise terms has exactly that distribution and nothing else leaves the kernel.
 * offset_dev: optional device pointer to a uint64 added to `offset` when the kernel runs (NULL: none).
 * A call recorded into a HIP graph has its host arguments frozen; a caller that advances *offset_dev on
 * the stream after each call gets fresh noise on every replay. */
int rexsc_orn_bias_std_both_forward(const float *x_pos, const float *x_neg, const float *bias_coef,
                                    const float *std_coef, float *y, size_t n, int or_n,
                                    uint64_t seed, uint64_t offset, const uint64_t *offset_dev,
                                    float *noise_out_pos, float *noise_out_neg, rexsc_stream_t stream);
int rexsc_orn_bias_std_both_backward(const float *grad_out, const float *x_pos, const float *x_neg,
                                     const float *bias_coef, float *grad_pos, float *grad_neg, size_t n,
                                     int or_n, int half_input, rexsc_stream_t stream);

/* Single-polarity variants (sc_cuda_pw.cu:834-861, 929-950).  The forward reads and writes
 * binary16, as the reference's does. */
int rexsc_orn_bias_std_forward_f16(const uint16_t *x_half, const float *bias_coef, const float *std_coef,
                                   uint16_t *y_half, size_t n, int or_n, uint64_t seed, uint64_t offset,
                                   const uint64_t *offset_dev, rexsc_stream_t stream);
int rexsc_orn_bias_std_backward(const float *grad_out, const float *x, const float *bias_coef,
                                float *grad_in, size_t n, int or_n, int half_input, rexsc_stream_t stream);

/* ---- polarity-pair layout (merged surrogate convolution) ----------------------------------
 * conv2d_generic evaluates its float surrogate as two convolutions, with clamp(w, 0, 100) and with
 * -clamp(w, -100, 0) (utils_functional.py:1204-1211, 1249), and sends each sum through the OR-n
 * kernels.  Convolving once with the 2*O filters [w_pos ; w_neg] yields the same sums as one tensor
 * s2 laid out [outer][2][inner] float32 (channels-last: outer = N*Ho*Wo, inner = O; NCHW: outer = N,
 * inner = O*Ho*Wo; linear: outer = B, inner = O); y and grad_out are [outer][inner].  inner % 4 == 0.
 * rexsc_orn_pair_backward = two or_approx_n_backward_acc calls on (g, s_pos) and (-g, s_neg)
 * (sc_cuda_pw.cu:767-832); the bias_std_pair calls = the *_both_acc calls above on this layout, with
 * the same noise stream per element of y.  g2 has s2's layout (gradient of the merged convolution). */
int rexsc_orn_pair_backward(const float *grad_out, const float *s2, float *g2, size_t outer, size_t inner,
                            int or_n, int half_input, rexsc_stream_t stream);
/* The same with grad_out, s2 and g2 stored as binary16 (8-byte aligned), for callers inside a float16 autocast
 * region, where the convolutions on either side of this kernel produce and consume float16 (utils_own.py:127-131;
 * the wrappers of sc_cuda_pw.cu:767-832 take such tensors and widen them).  Arithmetic in float32, one rounding on
 * the store: equal to widening, rexsc_orn_pair_backward with half_input = 1, and a cast of g2 to float16. */
int rexsc_orn_pair_backward_f16(const uint16_t *grad_out, const uint16_t *s2, uint16_t *g2, size_t outer, size_t inner,
                                int or_n, rexsc_stream_t stream);
int rexsc_orn_bias_std_pair_forward(const float *s2, const float *bias_coef, const float *std_coef, float *y,
                                    size_t outer, size_t inner, int or_n, uint64_t seed, uint64_t offset,
                                    const uint64_t *offset_dev, rexsc_stream_t stream);
int rexsc_orn_bias_std_pair_backward(const float *grad_out, const float *s2, const float *bias_coef, float *g2,
                                     size_t outer, size_t inner, int or_n, int half_input,
                                     rexsc_stream_t stream);

/* y = float(pos) / bit_length - float(neg) / bit_length over n elements of any dense layout: the
 * int16 -> float, "/ bit_length" and "pos - neg" passes of utils_functional.py:1181-1182, 1273-1274
 * and 1317 in one. */
int rexsc_sc_counts_to_float(const int16_t *pos, const int16_t *neg, float *y, size_t n, int bit_length,
                             rexsc_stream_t stream);

/* w2 = [clamp(w, 0, 100) ; -clamp(w, -100, 0)] along the output-channel axis (utils_functional.py:1204-1205)
 * for w = [out_channels][in_channels][taps] (taps = KH*KW; 1 for a linear layer), and the gradient of that
 * split: dw = dw2[first half] * [0 <= w <= 100] - dw2[second half] * [-100 <= w <= 0].  Each tensor is
 * dense in one of two memory orders, named by its *_channels_last flag: [O][C][taps] (0) or [O][taps][C] (1);
 * w2 can so be produced directly in the order a channels-last convolution wants.  dw has w's order. */
int rexsc_split_weight(const float *w, float *w2, size_t out_channels, size_t in_channels, size_t taps,
                       int w_channels_last, int w2_channels_last, rexsc_stream_t stream);
int rexsc_merge_weight_grad(const float *dw2, const float *w, float *dw, size_t out_channels, size_t in_channels,
                            size_t taps, int dw2_channels_last, int w_channels_last, rexsc_stream_t stream);

/* Fake quantisation y = clamp(round(x * 2^prec), -(2^prec - 1), 2^prec - 1) / 2^prec, round half to even,
 * 0 <= prec <= 16: the mul / round / clamp / div passes of `quantize` (utils_functional.py:93-104, the
 * forward of QuantizeGrad :117-123) in one.  n float32 elements of any dense layout; y may alias x. */
int rexsc_quantize(const float *x, float *y, size_t n, int prec, rexsc_stream_t stream);
/* The same on binary16 tensors (8-byte aligned), prec 0..10: what QuantizeGrad sees inside a float16 autocast region
 * (utils_own.py:127-131); equal to the reference's four float16 tensor passes there. */
int rexsc_quantize_f16(const uint16_t *x, uint16_t *y, size_t n, int prec, rexsc_stream_t stream);

/* Philox4x32-10 block function on the host (for known-answer tests of the generator). */
void rexsc_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);

/* ---- saturating fixed-point conv -------------------------------------------------------
 * Replaces fixed_extension_cuda.conv2d_saturate_acc (fixed_cuda.cpp:24-34) and
 * fixed_extension.conv2d_saturate (fixed.cpp:197-238): operands scaled by 2^precision_in,
 * clamped, rounded half-to-even; products folded in (c, ky, kx) order through the saturating
 * rounding adder selected by add_config (0 fixed_add, 1 fixed_add_or, >=2 pairwise OR2).
 * x float32 NCHW [N][C][H][W], w float32 [O][C][KH][KW], out int32 NCHW = pos - neg. */
typedef struct rexsc_fixed_desc {
    int32_t struct_size;         /* sizeof(rexsc_fixed_desc) */
    int32_t N, C, H, W, O, KH, KW;
    int32_t pad_h, pad_w, stride_h, stride_w;
    int32_t add_config, precision_in, precision_out;
} rexsc_fixed_desc;

size_t rexsc_fixed_conv2d_workspace_bytes(const rexsc_fixed_desc *d);
int rexsc_fixed_conv2d(const rexsc_fixed_desc *d, const float *x, const float *w, int32_t *out,
                       void *workspace, size_t workspace_bytes, rexsc_stream_t stream);

/* ---- activation-calibration statistics -------------------------------------------------
 * One pass over (a_bit, a_act) producing, for each of n_win (<= 64) windows
 * win_lo[k] <= a_act < win_hi[k], the count, sum and sum of squares of err = a_bit - a_act
 * (float64).  Windows may overlap.  Replaces the 30 masked gathers of compute_bias_std_coef
 * (utils_functional.py:917-925).  win_lo / win_hi are HOST arrays; stats is float64
 * [n_win][3] in device memory, zeroed by the call. */
int rexsc_calib_stats(const float *a_bit, const float *a_act, size_t n, const float *win_lo_host,
                      const float *win_hi_host, int n_win, double *stats, rexsc_stream_t stream);

/* ---- per-kernel timing (no counterpart in the reference) --------------------------------
 * Between rexsc_profile_begin() and rexsc_profile_end() every kernel the library launches is
 * bracketed by two HIP events on its launch stream.  rexsc_profile_end() waits for them and
 * returns, per kernel name, the number of launches, their summed duration and their summed
 * algorithmic work (lane-ops for the AND/popcount kernels, bytes for the streaming kernels).
 * Returns the number of records written (<= max_records). */
typedef struct rexsc_profile_record {
    char name[64];
    int32_t calls;
    double total_ms;
    double total_work;
} rexsc_profile_record;
int rexsc_profile_begin(void);
int rexsc_profile_end(rexsc_profile_record *out, int max_records);

/* Integer VALU peak probe (no counterpart in the reference): runs a register-only kernel that issues the SC
 * compute kernel's instruction pair (mode 0: v_and_b32 + v_bcnt_u32_b32 accumulate; mode 1: v_and_or_b32)
 * with eight waves per SIMD and returns its duration and the lane-operations it executed, so that roofline
 * fractions can be quoted against a peak measured on the machine at hand.  Modes 2..4 time the pair without
 * the scalar instruction the kernel puts between its halves, v_and_b32 on vector registers alone and
 * v_bcnt_u32_b32 alone (the instruction costs the pair's roof is derived from).  Synchronises the stream. */
int rexsc_valu_probe(int mode, int iters, rexsc_stream_t stream, double *ms_out, double *lane_ops_out);

#ifdef __cplusplus
}
#endif
#endif /* REXSC_H */
