// extern "C" entry points for SC conv2d and SC linear: validation, planning (chunk widths,
// tiles, slot splits, workspace carving) and kernel sequencing.
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>

#include "sc_compute.h"
#include "sng.h"

namespace rexsc {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

namespace {

constexpr size_t WS_ALIGN = 256;
// Activation streams of one batch chunk are kept below this many MiB (REXSC_TUNE_ACT_CAP_MB);
// larger batches are processed chunk by chunk with the weight streams generated once.
constexpr int ACT_STREAM_CAP_MB = 1024;
constexpr int TARGET_WAVES = 3072; // 3 resident waves per SIMD on 256 CUs x 4 SIMDs

struct ScPlan {
    // generators
    GenParams gen_act, gen_w;
    ActGeom ag;
    WeightGeom wg;
    // compute
    ComputeParams cp;
    int KW, ZC;
    bool tuned, wide;
    int n_chunk;       // images per batch chunk
    int Ho, Wo;
    // workspace (bytes)
    size_t off_w, off_a, off_part, off_tab_a, total;
    size_t w_bytes;     // weight stream words incl. the over-read chunk
    // Tap folding (C*KH*KW <= 32): the whole receptive field of an output pixel fits one 32-bit word, so the
    // generated streams are regrouped (one word per output pixel and slot, bit (ky*KW+kx)*C + c) and the compute
    // kernel runs as a 1x1 layer with one word per pixel: the same popcounts from KH*KW times fewer AND/popcount pairs.
    bool fold;
    int fold_KH, fold_KW, fold_s0, fold_s1, fold_Hp, fold_Wp; // the generated (unfolded) geometry
    size_t off_w2, off_a2, w2_bytes;                          // folded streams in the workspace
    size_t wstream_off_w2;                                    // ... and in a separate weight-stream buffer
    size_t wstream_off_tab, wstream_total; // layout of a separate weight-stream buffer: [Wst][state-plane table]
    size_t wstream_off_snap, wstream_off_flag; // ... [folded streams][copy of the weights][change flag]
    size_t w_elems;                            // O*C*KH*KW
    size_t tab_a_words; // state-plane table of the bit-sliced activation generator (0: ballot generator)
};

// positive integer tuning knob from the environment
int tune_env(const char *name, int dflt)
{
    const char *e = getenv(name);
    const int v = e ? atoi(e) : dflt;
    return v > 0 ? v : dflt;
}

int choose_zc(int Z, int KW)
{
    int zc = Z >= 4 ? 4 : (Z >= 2 ? 2 : 1);
    if (KW == 1 && Z >= 8) zc = 8;
    if (KW >= 5 && zc > 2) zc = 2;
    return zc;
}

int fill_gen(GenParams &g, int lb, int acc, int scale, int n_slots, int div, int mul, int mod, int tw, int lw,
             int lwait, int bit_length)
{
    g.lb = lb; g.acc = acc;
    g.period = acc == LFSR_ACC ? (1 << lb) : (1 << lb) - 1;
    g.seed_mod = (1 << lb) - 1;
    g.seed_off = acc == LFSR_XNOR ? 0 : 1;
    g.scale = scale;
    g.n_slots = n_slots;
    g.slot_div = div; g.slot_mul = mul; g.slot_mod = mod;
    g.total_width = tw; g.load_width = lw; g.load_wait = lwait;
    g.prog = 0;
    g.seed_add = 0; g.legacy = 0; g.clamp_hi = (float)(scale - 1); g.sign = 1.f; g.fake_quant = 0;
    REXSC_CHECK_ARG(lwait >= 1, "prog_load: load_wait must be >= 1 (got %d)", lwait);
    for (int t = 0; t < bit_length; t++) {
        const int sh = prog_shift(g, t);
        REXSC_CHECK_ARG(sh >= 0 && sh < 31, "prog_load (%d,%d,%d) gives shift %d at cycle %d", tw, lw, lwait, sh, t);
        if (sh) g.prog = 1;
    }
    return REXSC_OK;
}

// Common planning for conv (N images of HxW, KHxKW kernel) and linear (one "image" whose row
// of B pixels is the batch, 1x1 kernel).
int make_plan(ScPlan &pl, int N, int C, int H, int W, int O, int KH, int KW, int pad_h, int pad_w, int s0, int s1,
              int bit_length, int lfsr_length, int gen_config, int bin_config, int tw, int lw, int lwait,
              int act_cl, int w_cl, bool linear, bool xnor, int act_fake_quant = 0, int weight_fake_quant = 0)
{
    memset(&pl, 0, sizeof(pl));
    REXSC_CHECK_ARG(N > 0 && C > 0 && H > 0 && W > 0 && O > 0 && KH > 0 && KW > 0, "non-positive dimension");
    REXSC_CHECK_ARG(pad_h >= 0 && pad_w >= 0 && s0 > 0 && s1 > 0, "bad padding/stride");
    REXSC_CHECK_ARG(bit_length > 0, "bit_length must be positive");
    const int lb = lfsr_bits(bit_length, lfsr_length);
    REXSC_CHECK_ARG(lb > 0, "unsupported stream length %d / lfsr_length %d (supported: 2,4,8,...,256 or lfsr_length 3..8)",
                    bit_length, lfsr_length);
    const int g = gen_config;
    if (linear) REXSC_CHECK_ARG(g >= 1 && g <= 4, "linear: gen_config must be 1..4 (got %d)", g);
    else REXSC_CHECK_ARG(g == 1 || g == 2, "conv2d: gen_config must be 1 (lfsr) or 2 (and_2), got %d", g);
    const int T = bit_length * g;
    REXSC_CHECK_ARG(bit_length <= MAX_CYCLES && T <= 4096, "stream too long (bit_length %d, gen_config %d)", bit_length, g);
    const int scale = lfsr_length > 0 ? (1 << lfsr_length) : bit_length;
    REXSC_CHECK_ARG(scale <= 256, "operand scale %d exceeds 8 bits", scale);
    const int Hp = H + 2 * pad_h, Wp = W + 2 * pad_w;
    REXSC_CHECK_ARG(Hp >= KH && Wp >= KW, "kernel larger than padded input");
    const int Ho = (Hp - KH) / s0 + 1, Wo = (Wp - KW) / s1 + 1;
    const int Z = ceil_div(C, 32);
    REXSC_CHECK_ARG((long)32 * KH * KW * Z < 65536, "reduction too large: 32*KH*KW*ceil(C/32) must stay below 65536");

    int n_sat = bin_config >= 0 ? bin_config + 1 : 1 - bin_config;
    if (bin_config >= 65535) n_sat = 65535;
    if (n_sat > 65535) n_sat = 65535;
    const int n_slots = linear ? bit_length : T; // the linear op never visits the replicated slots
    // 16-bit packed sums are exact for the linear op (int32 results) only while they cannot
    // overflow; the conv op's results wrap at 16 bits in the reference as well.
    const long per_slot_max = n_sat < 32L * KH * KW * Z ? n_sat : 32L * KH * KW * Z;
    pl.wide = linear && bin_config >= 0 && (per_slot_max * n_slots > 65535);

    pl.KW = KW; pl.Ho = Ho; pl.Wo = Wo;
    pl.ZC = choose_zc(Z, KW);
    if (pl.wide && pl.ZC < 4) pl.ZC = 4; // wide accumulation is built for chunk widths 4 and 8
    pl.tuned = sc_compute_has_instance(KW, pl.ZC);
    if (!pl.tuned) pl.ZC = Z >= 4 ? 4 : (Z >= 2 ? 2 : 1);
    const int ZC = pl.ZC, ZG = ceil_div(Z, ZC);
    const int OT = sc_compute_tile_ot();
    const int O_pad = (int)align_up((size_t)O, (size_t)16); // the weight generator works on groups of 16 output channels
    // CPU-extension rule: the and_2 generator steps the zero-including LFSR (sc_conv.cpp:365-425).  The CUDA
    // kernels have no such variant: with xnor they step the XNOR LFSR for every gen_config, seeds lowered by
    // one (sc_cuda_conv.cu:28,55-56,139), and keep seeds and operands in int8 (sc_cuda_conv.cu:37-40), which
    // leaves 8-bit LFSRs without a meaningful result.
    REXSC_CHECK_ARG(!(xnor && linear), "linear: the reference's linear kernels have no XNOR generator");
    REXSC_CHECK_ARG(!(xnor && lb == 8), "xnor generator: 8-bit LFSRs are not supported (the CUDA reference keeps states in int8)");
    const int acc = xnor ? LFSR_XNOR : ((!linear && g == 2) ? LFSR_ACC : LFSR_PLAIN);
    int rc = fill_gen(pl.gen_act, lb, acc, scale, n_slots, g * g, g, g, tw, lw, lwait, bit_length);
    if (rc) return rc;
    rc = fill_gen(pl.gen_w, lb, acc, scale, n_slots, g, 1, 1, tw, lw, lwait, bit_length);
    if (rc) return rc;
    pl.gen_w.seed_add = 13; // POS_SEED == NEG_SEED (sc_cpu.hpp:10-11)
    REXSC_CHECK_ARG(act_fake_quant >= 0 && act_fake_quant <= 17 && weight_fake_quant >= 0 && weight_fake_quant <= 17,
                    "fake quantisation precision out of range (0..16)");
    pl.gen_act.fake_quant = act_fake_quant;
    pl.gen_w.fake_quant = weight_fake_quant;

    // batch chunking
    const size_t words_per_image_slot = (size_t)ZG * Hp * Wp * ZC;
    const size_t bytes_per_image = words_per_image_slot * n_slots * 4;
    int n_chunk = N;
    const size_t act_cap = (size_t)tune_env("REXSC_TUNE_ACT_CAP_MB", ACT_STREAM_CAP_MB) << 20;
    if (bytes_per_image * (size_t)N > act_cap) {
        n_chunk = (int)(act_cap / bytes_per_image);
        if (n_chunk < 1) n_chunk = 1;
    }
    REXSC_CHECK_ARG(words_per_image_slot * n_chunk < ((size_t)1 << 31), "activation plane too large");
    REXSC_CHECK_ARG((long)n_chunk * Ho * Wo < (1L << 31), "too many output pixels per chunk");
    pl.n_chunk = n_chunk;

    ActGeom &ag = pl.ag;
    ag.N = n_chunk; ag.C = C; ag.H = H; ag.W = W; ag.Hp = Hp; ag.Wp = Wp; ag.pad_h = pad_h; ag.pad_w = pad_w;
    ag.channels_last = act_cl; ag.ZC = ZC; ag.ZG = ZG;
    ag.slot_stride = (long)(words_per_image_slot * n_chunk);
    if (linear) { ag.seed_cmul = 1; ag.seed_pmul = 0; }   // seed c % P + 1            (sc_matmul.cpp:302)
    else { ag.seed_cmul = Hp * Wp; ag.seed_pmul = 1; }     // seed (c*Hp*Wp + pp) % P+1 (sc_conv.cpp:167,173)

    WeightGeom &wg = pl.wg;
    wg.O = O; wg.C = C; wg.KH = KH; wg.KW = KW; wg.channels_last = w_cl; wg.ZC = ZC; wg.ZG = ZG; wg.O_pad = O_pad;

    // REXSC_FOLD_TAPS=0 switches tap folding off (tuning / tests)
    const char *fold_env = getenv("REXSC_FOLD_TAPS");
    pl.fold = !linear && C * KH * KW <= 32 && KH * KW > 1 && sc_compute_has_instance(1, 1) && !(fold_env && atoi(fold_env) == 0);
    if (pl.fold) pl.tuned = true; // the folded problem is a 1x1 layer with one word per pixel: always an instance
    pl.fold_KH = KH; pl.fold_KW = KW; pl.fold_s0 = s0; pl.fold_s1 = s1; pl.fold_Hp = Hp; pl.fold_Wp = Wp;
    // geometry the compute kernel sees
    const int cKH = pl.fold ? 1 : KH, cKW = pl.fold ? 1 : KW;
    const int cHp = pl.fold ? Ho : Hp, cWp = pl.fold ? Wo : Wp, cs0 = pl.fold ? 1 : s0, cs1 = pl.fold ? 1 : s1;
    const long c_slot_stride = pl.fold ? (long)n_chunk * Ho * Wo : ag.slot_stride;
    if (pl.fold) pl.KW = 1;

    ComputeParams &cp = pl.cp;
    cp.M = n_chunk * Ho * Wo; cp.HoWo = Ho * Wo; cp.Wo = Wo; cp.Hp = cHp; cp.Wp = cWp; cp.s0 = cs0; cp.s1 = cs1;
    cp.KH = cKH; cp.ZG = ZG; cp.Z = Z; cp.a_slot_stride = c_slot_stride; cp.O = O; cp.O_pad = O_pad; cp.n_slots = n_slots;
    cp.nn = (uint32_t)n_sat | ((uint32_t)n_sat << 16);
    cp.mode = (linear && bin_config < 0) ? 1 : 0;
    cp.out_channels_last = linear ? 1 : act_cl; // linear output is [B][O]
    cp.ot = OT;

    // tiling.  A block is NS waves sharing one tile of 64*px pixels x OT channels, each wave taking
    // 1/NS of the stream slots (partials meet in LDS).  Two pixels per lane halve the scalar weight
    // traffic per VALU instruction.  The launch should be several rounds of the ~3072 resident waves
    // (256 CUs x 4 SIMDs x 3) so that its tail is short; what the tiles and NS do not supply comes
    // from splitting the slots over blocks as well (partials merged by the finalize kernel).
    const int o_tiles = O_pad / OT;
    // Pixels per lane.  Two halve the scalar weight traffic per VALU instruction but need twice the registers
    // (3 resident waves per SIMD instead of 5-6).  Measured on the benchmark shapes: one pixel per lane wins by
    // 1-10 % once there are a few thousand output pixels to amortise the weights over, except for the and-or
    // (saturation at one) instances, whose single 4-cycle instruction per weight word leaves the scalar loads
    // exposed; few pixels (linear layers) want two.  REXSC_TUNE_PX forces 1 or 2;
    // REXSC_TUNE_PX_MIN_M (default 128): fewest output pixels for which a lane may take two of them.
    const bool or1_mode = !pl.wide && n_sat == 1;
    cp.px = (!pl.wide && cp.M >= tune_env("REXSC_TUNE_PX_MIN_M", 128) && (or1_mode || cp.M < 4096)) ? 2 : 1;
    {
        const int forced_px = tune_env("REXSC_TUNE_PX", 0);
        if (!pl.wide && (forced_px == 1 || (forced_px == 2 && cp.M >= 128))) cp.px = forced_px;
    }
    // waves resident at once: 3 per SIMD with two pixels per lane, 5 with one (register-limited)
    const long target_waves = tune_env("REXSC_TUNE_TARGET_WAVES", cp.px == 2 ? TARGET_WAVES : 5 * 1024);
    cp.ns = n_slots >= 8 ? 4 : (n_slots >= 2 ? 2 : 1);
    {
        const int forced_ns = tune_env("REXSC_TUNE_NS", 0); // 1, 2 or 4 waves per block (tuning only)
        if ((forced_ns == 1 || forced_ns == 2 || forced_ns == 4) && forced_ns <= n_slots) cp.ns = forced_ns;
    }
    const long waves = (long)ceil_div(cp.M, 64 * cp.px) * cp.ns * o_tiles;
    int splits = 1;
    if (pl.tuned) {
        // Cost model for splitting the slots over `s` blocks as well: the launch takes
        // ceil(waves*s / resident waves) rounds of waves, each lasting the wave's share of the work plus
        // a fixed cost per wave (prologue, LDS reduction, stores).  Powers of two keep the shares even.
        // REXSC_TUNE_WAVE_OVERHEAD: that fixed cost in VALU instructions; REXSC_TUNE_SPLITS forces s.
        const int max_splits = n_slots / cp.ns > 0 ? n_slots / cp.ns : 1;
        // saturation at one needs one and-or per word and polarity instead of and + popcount
        const double ops_per_word = (n_sat == 1 && !pl.wide) ? 2.0 : 4.0;
        const double work1 = (double)ceil_div(n_slots, cp.ns) * cKH * ZG * (ops_per_word * cp.px * OT * cKW * ZC);
        const double overhead = tune_env("REXSC_TUNE_WAVE_OVERHEAD", 1500);
        double best = 0;
        for (int s = 1; s <= max_splits && s <= 16; s *= 2) {
            const double rounds = (double)((waves * s + target_waves - 1) / target_waves);
            double cost = rounds * (work1 / s + overhead);
            if (s > 1) {
                // the finalize pass: launch (~8 us) + partial and output bytes at ~3 TB/s, converted to the
                // model's unit (one VALU instruction of a wave sharing its SIMD with two others ~ 5.1 ns)
                const bool narrow = (long)ceil_div(n_slots, s) * per_slot_max <= 255;
                const double bytes = (double)cp.M * O_pad * ((narrow ? 2.0 : 4.0) * s + 4.0);
                cost += (8e3 + bytes / 3e3) / 5.1;
            }
            if (s == 1 || cost < best) { best = cost; splits = s; }
        }
        const int forced = tune_env("REXSC_TUNE_SPLITS", 0);
        if (forced > 0) splits = forced < max_splits ? forced : max_splits;
    }
    cp.slots_per_split = ceil_div(n_slots, splits);
    cp.splits = ceil_div(n_slots, cp.slots_per_split);
    cp.direct = (!linear && cp.splits == 1 && !pl.wide) ? 1 : 0;
    // partial sums of one split: at most slots_per_split * (largest per-slot count)
    cp.part_narrow = (!pl.wide && (long)cp.slots_per_split * per_slot_max <= 255) ? 1 : 0;
    if (!pl.tuned) { cp.direct = 1; cp.splits = 1; cp.slots_per_split = n_slots; }

    // workspace
    // + one chunk: the compute kernel's weight prefetch reads one batch past the last chunk
    const size_t w_bytes = ((size_t)n_slots * KH * ZG + 1) * O_pad * 2 * KW * ZC * 4;
    const size_t a_bytes = (size_t)n_slots * ag.slot_stride * 4;
    const size_t part_bytes = cp.direct ? 0 : (size_t)(pl.wide ? 2 : 1) * cp.splits * O_pad * cp.M * 4;
    pl.off_w = 0;
    pl.off_a = align_up(w_bytes, WS_ALIGN);
    pl.off_part = pl.off_a + align_up(a_bytes, WS_ALIGN);
    pl.off_tab_a = pl.off_part + align_up(part_bytes, WS_ALIGN);
    pl.tab_a_words = sng_act_table_words(ag, pl.gen_act);
    pl.total = pl.off_tab_a + align_up(pl.tab_a_words * 4, WS_ALIGN);
    pl.w_bytes = w_bytes;
    pl.wstream_off_tab = align_up(w_bytes, WS_ALIGN);
    pl.wstream_total = pl.wstream_off_tab + align_up(pl.tab_a_words * 4, WS_ALIGN);
    if (pl.fold) {
        pl.w2_bytes = ((size_t)n_slots + 1) * O_pad * 2 * 4; // + one chunk for the prefetch over-read
        const size_t a2_bytes = (size_t)n_slots * c_slot_stride * 4;
        pl.off_w2 = pl.total;
        pl.off_a2 = pl.off_w2 + align_up(pl.w2_bytes, WS_ALIGN);
        pl.total = pl.off_a2 + align_up(a2_bytes, WS_ALIGN);
        pl.wstream_off_w2 = pl.wstream_total;
        pl.wstream_total += align_up(pl.w2_bytes, WS_ALIGN);
    }
    pl.w_elems = (size_t)O * C * KH * KW;
    pl.wstream_off_snap = pl.wstream_total;
    pl.wstream_off_flag = pl.wstream_off_snap + align_up(pl.w_elems * 4, WS_ALIGN);
    pl.wstream_total = pl.wstream_off_flag + WS_ALIGN;
    cp.inv_L = 1.0f / (float)bit_length;
    return REXSC_OK;
}

// Epochs of the weight-stream change flag: one per call that fills or verifies a kept buffer, never reused.
unsigned long long next_epoch()
{
    static std::atomic<unsigned long long> counter{0x5243000000000001ull};
    return counter.fetch_add(1);
}

int plan_conv(ScPlan &pl, const rexsc_conv_desc *d)
{
    REXSC_CHECK_DESC(d, rexsc_conv_desc);
    return make_plan(pl, d->N, d->C, d->H, d->W, d->O, d->KH, d->KW, d->pad_h, d->pad_w, d->stride_h, d->stride_w,
                     d->bit_length, d->lfsr_length, d->gen_config, d->bin_config, d->total_width, d->load_width,
                     d->load_wait, d->act_channels_last != 0, d->weight_channels_last != 0, false, d->xnor != 0,
                     d->act_fake_quant, d->weight_fake_quant);
}

int plan_linear(ScPlan &pl, const rexsc_linear_desc *d)
{
    REXSC_CHECK_DESC(d, rexsc_linear_desc);
    // batch rows become the pixels of a single 1 x B "image" in channels-last order
    int rc = make_plan(pl, 1, d->C, 1, d->B, d->O, 1, 1, 0, 0, 1, 1, d->bit_length, d->lfsr_length, d->gen_config,
                       d->bin_config, d->total_width, d->load_width, d->load_wait, 1, 0, true, false,
                       d->act_fake_quant, d->weight_fake_quant);
    if (rc) return rc;
    if (pl.wide && !(pl.ZC == 4 || pl.ZC == 8)) {
        set_error("linear: internal planning error (wide accumulation with chunk width %d)", pl.ZC);
        return REXSC_ERR_INVALID;
    }
    return REXSC_OK;
}

// ---- scratch of the entry point that allocates nothing ------------------------------------------
// rexsc_conv2d_orn_noalloc() carves its workspace (weight streams, activation streams, split
// partials, state-plane table) out of this array instead of a caller-owned buffer.  Every GPU the
// library runs on holds its own copy until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress: the address kernels may use is resolved once per device
// (static_scratch) and that pointer is what is carved up and passed to the kernels.
static __device__ __align__(256) unsigned char scratch[REXSC_NOALLOC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;

int static_scratch(void **out)
{
    static std::mutex mu;
    static void *dev_ptr[MAX_DEVICES] = {nullptr};
    int dev = 0;
    REXSC_CHECK_HIP(hipGetDevice(&dev));
    REXSC_CHECK_ARG(dev >= 0 && dev < MAX_DEVICES, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!dev_ptr[dev]) {
        void *p = nullptr;
        REXSC_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        REXSC_CHECK_ARG(p != nullptr && ((uintptr_t)p % WS_ALIGN) == 0, "static scratch has no usable device address");
        dev_ptr[dev] = p;
    }
    *out = dev_ptr[dev];
    return REXSC_OK;
}

// Kept weight streams (REXSC_WSTREAMS_FILL / _VERIFY): one small launch brings the buffer's copy of the weights up to
// date and stamps the buffer's flag with this call's epoch if anything differed (always, when filling).  The
// generator launches that follow carry (flag, epoch) and return at once when the stamp is an older one.
int kept_weights_changed(const ScPlan &pl, const float *w, void *wstreams, int mode, const unsigned long long **guard,
                         unsigned long long *epoch, hipStream_t stream)
{
    REXSC_CHECK_ARG(mode == REXSC_WSTREAMS_FILL || mode == REXSC_WSTREAMS_VERIFY, "weight_streams_valid must be 0, 1 or 2 (got %d)", mode);
    REXSC_CHECK_ARG(w != nullptr, "null weight pointer");
    uint8_t *base = (uint8_t *)wstreams;
    unsigned long long *flag = (unsigned long long *)(base + pl.wstream_off_flag);
    *epoch = next_epoch();
    *guard = mode == REXSC_WSTREAMS_VERIFY ? flag : nullptr;
    return weights_snapshot(w, (float *)(base + pl.wstream_off_snap), pl.w_elems, flag, *epoch,
                            mode == REXSC_WSTREAMS_FILL, stream);
}

// Weight streams (and the activation generator's table, and the folded streams) of a conv plan.  wstreams != nullptr: a
// kept buffer in mode REXSC_WSTREAMS_FILL or _VERIFY; nullptr: plain generation into the workspace.
int generate_weight_streams(const ScPlan &pl, int C, const float *w, uint32_t *Wst, uint32_t *tab_a, uint32_t *W2,
                            void *wstreams, int mode, hipStream_t stream)
{
    const unsigned long long *guard = nullptr;
    unsigned long long epoch = 0;
    int rc;
    if (wstreams) {
        rc = kept_weights_changed(pl, w, wstreams, mode, &guard, &epoch, stream);
        if (rc) return rc;
    }
    rc = sng_weights(w, Wst, pl.wg, pl.gen_w, tab_a, &pl.ag, &pl.gen_act, stream, guard, epoch);
    if (rc) return rc;
    if (pl.fold) {
        rc = fold_weight_streams(Wst, W2, pl.cp.n_slots, pl.fold_KH, pl.fold_KW, pl.wg.O_pad, C, stream, guard, epoch);
        if (rc) return rc;
    }
    return REXSC_OK;
}

// The conv op proper: generators, compute, finalize, batch chunk by batch chunk, in `workspace`
// (device memory of at least pl.total bytes).  wstreams != nullptr: the weight streams and the activation
// generator's state-plane table live there (pl.wstream_total bytes) instead of in the workspace;
// wstreams_valid is one of REXSC_WSTREAMS_*.
int run_conv(const ScPlan &pl, const rexsc_conv_desc *d, const float *x, const float *w, int16_t *out_pos,
             int16_t *out_neg, int16_t *out_diff, float *out_value, void *wstreams, int wstreams_valid, void *workspace,
             hipStream_t stream)
{
    uint8_t *ws = (uint8_t *)workspace;
    uint32_t *Wst = (uint32_t *)(ws + pl.off_w);
    uint32_t *A = (uint32_t *)(ws + pl.off_a);
    uint32_t *part = (uint32_t *)(ws + pl.off_part);
    uint32_t *tab_a = pl.tab_a_words ? (uint32_t *)(ws + pl.off_tab_a) : nullptr;
    uint32_t *W2 = pl.fold ? (uint32_t *)(ws + pl.off_w2) : nullptr;
    uint32_t *A2 = pl.fold ? (uint32_t *)(ws + pl.off_a2) : nullptr;
    if (wstreams) {
        Wst = (uint32_t *)wstreams;
        if (pl.tab_a_words) tab_a = (uint32_t *)((uint8_t *)wstreams + pl.wstream_off_tab);
        if (pl.fold) W2 = (uint32_t *)((uint8_t *)wstreams + pl.wstream_off_w2);
    }
    int rc;
    if (!wstreams || wstreams_valid != REXSC_WSTREAMS_TRUST) {
        rc = generate_weight_streams(pl, d->C, w, Wst, tab_a, W2, wstreams, wstreams_valid, stream);
        if (rc) return rc;
    }
    const size_t in_image = (size_t)d->C * d->H * d->W;
    const size_t out_image = (size_t)d->O * pl.Ho * pl.Wo;
    for (int n0 = 0; n0 < d->N; n0 += pl.n_chunk) {
        const int nc = d->N - n0 < pl.n_chunk ? d->N - n0 : pl.n_chunk;
        ActGeom ag = pl.ag;
        ComputeParams cp = pl.cp;
        ag.N = nc;
        cp.M = nc * pl.Ho * pl.Wo; // slot stride keeps the full-chunk value: the buffer is laid out for n_chunk images
        rc = sng_activations(x + n0 * in_image, A, tab_a, ag, pl.gen_act, stream);
        if (rc) return rc;
        if (pl.fold) {
            rc = fold_activation_streams(A, A2, cp.n_slots, pl.ag.slot_stride, cp.a_slot_stride, nc, pl.fold_Hp, pl.fold_Wp,
                                         pl.Ho, pl.Wo, pl.fold_KH, pl.fold_KW, pl.fold_s0, pl.fold_s1, d->C, stream);
            if (rc) return rc;
        }
        const uint32_t *Ac = pl.fold ? A2 : A, *Wc = pl.fold ? W2 : Wst;
        int16_t *op = out_pos ? out_pos + n0 * out_image : nullptr;
        int16_t *on = out_neg ? out_neg + n0 * out_image : nullptr;
        int16_t *od = out_diff ? out_diff + n0 * out_image : nullptr;
        float *ov = out_value ? out_value + n0 * out_image : nullptr;
        if (!pl.tuned) {
            rc = sc_compute_generic(Ac, Wc, cp, pl.KW, pl.ZC, op, on, od, ov, stream);
            if (rc) return rc;
            continue;
        }
        rc = sc_compute(Ac, Wc, cp, pl.KW, pl.ZC, false, part, op, on, od, ov, stream);
        if (rc) return rc;
        if (!cp.direct) {
            cp.m_tiles = cp.o_tiles = 0;
            rc = sc_finalize_i16(part, cp, op, on, od, ov, stream);
            if (rc) return rc;
        }
    }
    return REXSC_OK;
}

} // namespace
} // namespace rexsc

using namespace rexsc;

extern "C" const char *rexsc_last_error(void) { return g_error; }
extern "C" int rexsc_version(void) { return REXSC_ABI_VERSION; }

extern "C" int rexsc_init(rexsc_stream_t stream)
{
    const SeqTable *t = nullptr;
    int rc = get_seq_tables(&t, (hipStream_t)stream);
    if (rc) return rc;
    void *ws = nullptr;
    return static_scratch(&ws); // device address of the no-alloc entry point's scratch array
}

extern "C" size_t rexsc_conv2d_workspace_bytes(const rexsc_conv_desc *d)
{
    ScPlan pl;
    if (plan_conv(pl, d)) return 0;
    return pl.total;
}

// Planning decisions of the conv op, for tests and tuning: fills out[0..15] with
// {tuned, KW, ZC, ZG, O_pad, px, ns, splits, slots_per_split, n_slots, direct, n_chunk, M, Hp, Wp, wide}.
extern "C" int rexsc_conv2d_plan_info(const rexsc_conv_desc *d, int64_t *out)
{
    ScPlan pl;
    int rc = plan_conv(pl, d);
    if (rc) return rc;
    const int64_t v[16] = {pl.tuned, pl.KW, pl.ZC, pl.cp.ZG, pl.cp.O_pad, pl.cp.px, pl.cp.ns, pl.cp.splits,
                           pl.cp.slots_per_split, pl.cp.n_slots, pl.cp.direct, pl.n_chunk, pl.cp.M, pl.cp.Hp,
                           pl.cp.Wp, pl.wide};
    for (int i = 0; i < 16; i++) out[i] = v[i];
    return REXSC_OK;
}

extern "C" int rexsc_conv2d_orn(const rexsc_conv_desc *d, const float *x, const float *w, int16_t *out_pos,
                                int16_t *out_neg, int16_t *out_diff, void *workspace, size_t workspace_bytes,
                                rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_conv(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && w, "null operand pointer");
    REXSC_CHECK_ARG(out_pos || out_neg || out_diff, "no output pointer given");
    if (!workspace || workspace_bytes < pl.total) {
        set_error("conv2d: workspace of %zu bytes needed, %zu given", pl.total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    return run_conv(pl, d, x, w, out_pos, out_neg, out_diff, nullptr, nullptr, 0, workspace, stream);
}

extern "C" size_t rexsc_conv2d_weight_streams_bytes(const rexsc_conv_desc *d)
{
    ScPlan pl;
    if (plan_conv(pl, d)) return 0;
    return pl.wstream_total;
}

extern "C" int rexsc_conv2d_orn_ex(const rexsc_conv_desc *d, const float *x, const float *w, int16_t *out_pos,
                                   int16_t *out_neg, int16_t *out_diff, float *out_value, void *weight_streams,
                                   size_t weight_streams_bytes, int weight_streams_valid, void *workspace,
                                   size_t workspace_bytes, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_conv(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && (w || (weight_streams && weight_streams_valid == REXSC_WSTREAMS_TRUST)), "null operand pointer");
    REXSC_CHECK_ARG(weight_streams_valid >= 0 && weight_streams_valid <= 2, "weight_streams_valid must be 0, 1 or 2");
    REXSC_CHECK_ARG(out_pos || out_neg || out_diff || out_value, "no output pointer given");
    if (!workspace || workspace_bytes < pl.total) {
        set_error("conv2d: workspace of %zu bytes needed, %zu given", pl.total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    if (weight_streams && weight_streams_bytes < pl.wstream_total) {
        set_error("conv2d: weight-stream buffer of %zu bytes needed, %zu given", pl.wstream_total, weight_streams_bytes);
        return REXSC_ERR_WORKSPACE;
    }
    return run_conv(pl, d, x, w, out_pos, out_neg, out_diff, out_value, weight_streams, weight_streams_valid, workspace, stream);
}

// The weight half of rexsc_conv2d_orn_ex on its own: fills the kept buffer as a call in mode REXSC_WSTREAMS_FILL would
// (keep_weight_copy = 0: without the copy of the weights that a later VERIFY compares with), so that the conv call proper
// can follow in mode TRUST (or VERIFY).  The weight streams of a layer depend on nothing but its weights: a caller can
// issue this on another stream while the previous layer computes.
extern "C" int rexsc_conv2d_prepare_weights(const rexsc_conv_desc *d, const float *w, void *weight_streams,
                                            size_t weight_streams_bytes, int keep_weight_copy, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_conv(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(w && weight_streams, "null pointer");
    if (weight_streams_bytes < pl.wstream_total) {
        set_error("conv2d: weight-stream buffer of %zu bytes needed, %zu given", pl.wstream_total, weight_streams_bytes);
        return REXSC_ERR_WORKSPACE;
    }
    uint8_t *base = (uint8_t *)weight_streams;
    uint32_t *tab_a = pl.tab_a_words ? (uint32_t *)(base + pl.wstream_off_tab) : nullptr;
    uint32_t *W2 = pl.fold ? (uint32_t *)(base + pl.wstream_off_w2) : nullptr;
    // without the copy of the weights the buffer cannot be verified later: plain generation into it
    return generate_weight_streams(pl, d->C, w, (uint32_t *)weight_streams, tab_a, W2, keep_weight_copy ? weight_streams : nullptr,
                                   REXSC_WSTREAMS_FILL, stream);
}

// Same op with the workspace taken from the library's static device array: no allocation of any kind,
// for callers that cannot allocate (HIP graph capture, tight serving loops).  Calls that overlap on
// one GPU share that array and race.
extern "C" int rexsc_conv2d_orn_noalloc(const rexsc_conv_desc *d, const float *x, const float *w, int16_t *out_pos,
                                        int16_t *out_neg, int16_t *out_diff, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_conv(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && w, "null operand pointer");
    REXSC_CHECK_ARG(out_pos || out_neg || out_diff, "no output pointer given");
    if (pl.total > (size_t)REXSC_NOALLOC_SCRATCH_BYTES) {
        set_error("conv2d (no-alloc): this problem needs %zu bytes of scratch, the static array holds %zu; use "
                  "rexsc_conv2d_orn with a caller-owned workspace", pl.total, (size_t)REXSC_NOALLOC_SCRATCH_BYTES);
        return REXSC_ERR_WORKSPACE;
    }
    void *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc) return rc;
    // Nothing in the workspace has to start at zero: the generators write every word the compute
    // kernel uses, and the finalize pass reads only partials the compute kernel has just written.
    return run_conv(pl, d, x, w, out_pos, out_neg, out_diff, nullptr, nullptr, 0, ws, stream);
}

extern "C" size_t rexsc_linear_workspace_bytes(const rexsc_linear_desc *d)
{
    ScPlan pl;
    if (plan_linear(pl, d)) return 0;
    return pl.total;
}

static int run_linear(const ScPlan &pl, const float *x, const float *w, int32_t *out_pos, int32_t *out_neg,
                      void *wstreams, int wstreams_valid, void *workspace, hipStream_t stream)
{
    uint8_t *ws = (uint8_t *)workspace;
    uint32_t *Wst = (uint32_t *)(ws + pl.off_w);
    uint32_t *A = (uint32_t *)(ws + pl.off_a);
    uint32_t *part = (uint32_t *)(ws + pl.off_part);
    uint32_t *tab_a = pl.tab_a_words ? (uint32_t *)(ws + pl.off_tab_a) : nullptr;
    if (wstreams) {
        Wst = (uint32_t *)wstreams;
        if (pl.tab_a_words) tab_a = (uint32_t *)((uint8_t *)wstreams + pl.wstream_off_tab);
    }
    int rc;
    if (!wstreams || wstreams_valid != REXSC_WSTREAMS_TRUST) {
        const unsigned long long *guard = nullptr;
        unsigned long long epoch = 0;
        if (wstreams) {
            rc = kept_weights_changed(pl, w, wstreams, wstreams_valid, &guard, &epoch, stream);
            if (rc) return rc;
        }
        rc = sng_weights(w, Wst, pl.wg, pl.gen_w, tab_a, &pl.ag, &pl.gen_act, stream, guard, epoch);
        if (rc) return rc;
    }
    rc = sng_activations(x, A, tab_a, pl.ag, pl.gen_act, stream);
    if (rc) return rc;
    rc = sc_compute(A, Wst, pl.cp, 1, pl.ZC, pl.wide, part, nullptr, nullptr, nullptr, nullptr, stream);
    if (rc) return rc;
    return sc_finalize_i32(part, pl.cp, pl.wide, out_pos, out_neg, stream);
}

extern "C" int rexsc_linear_orn(const rexsc_linear_desc *d, const float *x, const float *w, int32_t *out_pos,
                                int32_t *out_neg, void *workspace, size_t workspace_bytes, rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_linear(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && w && out_pos && out_neg, "null pointer");
    if (!workspace || workspace_bytes < pl.total) {
        set_error("linear: workspace of %zu bytes needed, %zu given", pl.total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    REXSC_CHECK_ARG(pl.tuned, "linear: no kernel instance for chunk width %d", pl.ZC);
    return run_linear(pl, x, w, out_pos, out_neg, nullptr, 0, workspace, stream);
}

extern "C" size_t rexsc_linear_weight_streams_bytes(const rexsc_linear_desc *d)
{
    ScPlan pl;
    if (plan_linear(pl, d)) return 0;
    return pl.wstream_total;
}

extern "C" int rexsc_linear_orn_ex(const rexsc_linear_desc *d, const float *x, const float *w, int32_t *out_pos,
                                   int32_t *out_neg, void *weight_streams, size_t weight_streams_bytes,
                                   int weight_streams_valid, void *workspace, size_t workspace_bytes,
                                   rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_linear(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && out_pos && out_neg && (w || (weight_streams && weight_streams_valid == REXSC_WSTREAMS_TRUST)), "null pointer");
    REXSC_CHECK_ARG(weight_streams_valid >= 0 && weight_streams_valid <= 2, "weight_streams_valid must be 0, 1 or 2");
    if (!workspace || workspace_bytes < pl.total) {
        set_error("linear: workspace of %zu bytes needed, %zu given", pl.total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    if (weight_streams && weight_streams_bytes < pl.wstream_total) {
        set_error("linear: weight-stream buffer of %zu bytes needed, %zu given", pl.wstream_total, weight_streams_bytes);
        return REXSC_ERR_WORKSPACE;
    }
    REXSC_CHECK_ARG(pl.tuned, "linear: no kernel instance for chunk width %d", pl.ZC);
    return run_linear(pl, x, w, out_pos, out_neg, weight_streams, weight_streams_valid, workspace, stream);
}

// The reference's legacy pure-torch simulation `linear_generic` (utils_functional.py:955-1081; generator 'lfsr',
// shared generators): the same AND / popcount / per-cycle rule as the extension's linear op, with
//   * operands q = ceil(float16(x * L)), activations unclamped (anything >= L is "always one"), weight parts
//     clamped to weight_clamp (the function's `prec - 1`, 127 by default) -- the simulation compares the
//     float16 products with integer LFSR states, and v > s for an integer s is ceil(v) > s;
//   * seeds (67 + c) % P + 1 for the positive and (37 + c) % P + 1 for the negative weight part, c % P + 1
//     for activations (utils_functional.py:147-165); share == 0: the function's share=False, where c is replaced by
//     the element's index in the whole tensor (o * C + c, b * C + c).
// Two passes over one set of activation streams, one per weight polarity (each with its own seeds).
extern "C" int rexsc_linear_legacy(const rexsc_linear_desc *d, int weight_clamp, int share, const float *x, const float *w,
                                   int32_t *out_pos, int32_t *out_neg, void *workspace, size_t workspace_bytes,
                                   rexsc_stream_t stream_)
{
    hipStream_t stream = (hipStream_t)stream_;
    ScPlan pl;
    int rc = plan_linear(pl, d);
    if (rc) return rc;
    REXSC_CHECK_ARG(x && w && out_pos && out_neg, "null pointer");
    REXSC_CHECK_ARG(d->lfsr_length <= 0 && d->gen_config == 1 && d->bit_length >= 8 && d->bit_length <= 128,
                    "legacy linear: stream lengths 8..128 with the LFSR of that length and gen_config 1 only");
    REXSC_CHECK_ARG(d->total_width == 7 && d->load_width == 8 && d->load_wait == 1, "legacy linear: no progressive loading");
    REXSC_CHECK_ARG(weight_clamp >= 1, "legacy linear: weight_clamp must be positive");
    if (!workspace || workspace_bytes < pl.total) {
        set_error("legacy linear: workspace of %zu bytes needed, %zu given", pl.total, workspace ? workspace_bytes : (size_t)0);
        return REXSC_ERR_WORKSPACE;
    }
    REXSC_CHECK_ARG(pl.tuned, "linear: no kernel instance for chunk width %d", pl.ZC);
    uint8_t *ws = (uint8_t *)workspace;
    uint32_t *Wst = (uint32_t *)(ws + pl.off_w);
    uint32_t *A = (uint32_t *)(ws + pl.off_a);
    uint32_t *part = (uint32_t *)(ws + pl.off_part);
    uint32_t *tab_a = pl.tab_a_words ? (uint32_t *)(ws + pl.off_tab_a) : nullptr;
    const float L = (float)d->bit_length;
    pl.gen_act.legacy = 1; pl.gen_act.clamp_hi = L;
    pl.gen_w.legacy = 1; pl.gen_w.clamp_hi = weight_clamp < d->bit_length ? (float)weight_clamp : L;
    if (!share) {
        // one generator per element (utils_functional.py:996-998): the seed index runs over the whole weight tensor
        // (o * C + c) and the whole activation tensor (b * C + c).  The activation generator's table was planned for
        // seeds that do not depend on the row: the lane-ballot generator takes over.
        pl.wg.seed_omul = d->C;
        pl.ag.seed_pmul = d->C;
        tab_a = nullptr;
    }
    for (int pol = 0; pol < 2; pol++) {
        pl.gen_w.seed_add = pol == 0 ? 67 : 37;
        pl.gen_w.sign = pol == 0 ? 1.f : -1.f; // pass 1 streams -w: its positive part is w's negative part
        rc = sng_weights(w, Wst, pl.wg, pl.gen_w, pol == 0 ? tab_a : nullptr, &pl.ag, &pl.gen_act, stream);
        if (rc) return rc;
        if (pol == 0) {
            rc = sng_activations(x, A, tab_a, pl.ag, pl.gen_act, stream);
            if (rc) return rc;
        }
        rc = sc_compute(A, Wst, pl.cp, 1, pl.ZC, pl.wide, part, nullptr, nullptr, nullptr, nullptr, stream);
        if (rc) return rc;
        rc = sc_finalize_i32(part, pl.cp, pl.wide, pol == 0 ? out_pos : out_neg, nullptr, stream);
        if (rc) return rc;
    }
    return REXSC_OK;
}
