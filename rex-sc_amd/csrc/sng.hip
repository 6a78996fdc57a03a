// Stream-number generation (SNG): float operands -> quantised integers -> LFSR bitstreams,
// packed 32 channels per word.  One wave compares 64 channels against their LFSR states with
// a single v_cmp; the 64-bit lane mask that lands in an SGPR pair IS two stream words, so no
// shift/or bit packing is needed.  LFSR states are looked up in a per-width sequence table
// (any cycle of any seed is one LDS byte read), so slots can be produced in any order.
//
// Semantics follow the reference CPU extension: sc_conv.cpp:42-200 (conv), sc_matmul.cpp:3-383
// (linear); quantisation sc_conv.cpp:316-320.
#include <utility>

#include "sng.h"
#include "profile.h"

namespace rexsc {

// ---- sequence tables -------------------------------------------------------------------------
static __device__ SeqTable g_seq_tables[12];

__global__ void build_seq_tables_kernel()
{
    int idx = threadIdx.x;
    if (idx >= 12) return;
    int lb = idx / 2 + 3, acc = idx % 2;
    int period = acc ? (1 << lb) : (1 << lb) - 1;
    SeqTable &t = g_seq_tables[idx];
    int v = 1;
    for (int i = 0; i < 256; i++) t.inv[i] = 0;
    for (int i = 0; i < SEQ_LEN; i++) {
        t.seq[i] = (uint8_t)v;
        if (i < period) t.inv[v] = (uint8_t)i;
        v = lfsr_step(lb, acc, v);
    }
}

int get_seq_tables(const SeqTable **tables, hipStream_t stream)
{
    static SeqTable *dev_ptr[64] = {nullptr};
    int dev = 0;
    REXSC_CHECK_HIP(hipGetDevice(&dev));
    REXSC_CHECK_ARG(dev >= 0 && dev < 64, "device index %d out of range", dev);
    if (!dev_ptr[dev]) {
        SeqTable *p = nullptr;
        REXSC_CHECK_HIP(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(g_seq_tables)));
        hipLaunchKernelGGL(build_seq_tables_kernel, dim3(1), dim3(64), 0, stream);
        REXSC_CHECK_HIP(hipGetLastError());
        // Later launches may use other streams: make the tables visible to all of them.
        REXSC_CHECK_HIP(hipStreamSynchronize(stream));
        dev_ptr[dev] = p;
    }
    *tables = dev_ptr[dev];
    return REXSC_OK;
}

// ---- helpers -------------------------------------------------------------------------------
__device__ __forceinline__ int quant_ceil_pos(float v, float S)
{   // ceil(clamp(v*S, 0, S-1))
    float t = v * S;
    t = fminf(fmaxf(t, 0.f), S - 1.f);
    return (int)ceilf(t);
}
__device__ __forceinline__ int quant_ceil_neg(float v, float S)
{   // ceil(-clamp(v*S, 1-S, 0))
    float t = v * S;
    t = fminf(fmaxf(t, 1.f - S), 0.f);
    return (int)ceilf(-t);
}

__device__ __forceinline__ void load_tables_to_lds(const SeqTable *tab, uint8_t *seq, uint8_t *inv)
{
    const uint32_t *src = reinterpret_cast<const uint32_t *>(tab->seq);
    uint32_t *dst = reinterpret_cast<uint32_t *>(seq);
    for (int i = threadIdx.x; i < SEQ_LEN / 4; i += blockDim.x) dst[i] = src[i];
    const uint32_t *srci = reinterpret_cast<const uint32_t *>(tab->inv);
    uint32_t *dsti = reinterpret_cast<uint32_t *>(inv);
    for (int i = threadIdx.x; i < 64; i += blockDim.x) dsti[i] = srci[i];
}


// One 64-channel group, up to 32 consecutive slots [s0, s0+ns): lane = channel holds its quantised
// value v and its LFSR cycle position pos.  Each slot is one v_cmp whose 64-bit lane mask is the
// pair of stream words; the masks are deposited with v_writelane so that afterwards LANE s holds
// the two words of SLOT s0+s (lo = channels 0..31, hi = channels 32..63).
//
// v_writelane_b32 with an immediate lane select puts a wave-uniform value into lane LANE of a VGPR.
// Only one SGPR may feed a VALU instruction on this hardware, so the lane select cannot be a second
// SGPR.  The mask comes straight from a v_cmp: a VALU write of an SGPR needs two wait states before
// another VALU instruction reads it, and the compiler does not track hazards into inline asm, hence
// the s_nop.
template <int LANE>
__device__ __forceinline__ void write_lanes(uint32_t &lo, uint32_t &hi, unsigned long long mask)
{
#if defined(__HIP_DEVICE_COMPILE__) // the host pass of hipcc parses device functions too
    asm("s_nop 1\n\tv_writelane_b32 %0, %2, %4\n\tv_writelane_b32 %1, %3, %4"
        : "+v"(lo), "+v"(hi)
        : "s"((uint32_t)mask), "s"((uint32_t)(mask >> 32)), "n"(LANE));
#endif
}

template <int S>
__device__ __forceinline__ void gen_slot_fast(const uint8_t *p, int v, uint32_t &lo, uint32_t &hi)
{
    write_lanes<S>(lo, hi, __ballot(v > (int)p[S]));
}

template <int... S>
__device__ __forceinline__ void gen_slots_fast(const uint8_t *p, int v, uint32_t &lo, uint32_t &hi,
                                               std::integer_sequence<int, S...>)
{
    (gen_slot_fast<S>(p, v, lo, hi), ...);
}

__device__ __forceinline__ void gen_slots32(const uint8_t *s_seq, int pos, int v, const GenParams &gp, int s0, int ns,
                                            uint32_t &lo, uint32_t &hi)
{
    lo = 0; hi = 0;
    const bool ident = gp.slot_div == 1 && gp.slot_mul == 1 && gp.slot_mod == 1; // slot == cycle
    if (ident && !gp.prog && ns == 32) {
        gen_slots_fast(s_seq + pos + s0, v, lo, hi, std::make_integer_sequence<int, 32>{});
    } else {
        const int lane = threadIdx.x & 63;
        for (int s = 0; s < ns; s++) {
            const int t = slot_cycle(gp, s0 + s);
            const int st = s_seq[pos + t];
            int vv = v;
            if (gp.prog) { const int sh = prog_shift(gp, t); vv = (v >> sh) << sh; }
            const unsigned long long m = __ballot(vv > st);
            if (lane == s) { lo = (uint32_t)m; hi = (uint32_t)(m >> 32); }
        }
    }
}

// ---- activation SNG --------------------------------------------------------------------------
// Block: 256 threads.  Tile: 64 consecutive positions pp of the PADDED plane of image n,
// one channel chunk zg (32*ZC channels).
// Output layout (uint32 words): A[slot][n][zg][pp][zc], pp = yp*Wp + xp.
constexpr int ACT_TILE = 64;
constexpr int ACT_SLOT_GROUP = 32;
constexpr int QPITCH = ACT_TILE + 4; // bytes per channel row in LDS; 17 dwords -> conflict-free column reads
// dwords between the rows of two slots in the LDS staging buffer: +2 spreads the per-lane (= per-slot)
// 8-byte writes over the banks
template <int ZC> constexpr int act_pitch() { return ACT_TILE * ZC + 2; }

template <int ZC>
__global__ __launch_bounds__(256) void sng_act_kernel(const float *__restrict__ x, uint32_t *__restrict__ A,
                                                      const SeqTable *__restrict__ tables, ActGeom geo, GenParams gp)
{
    constexpr int CCH = 32 * ZC;           // channels per chunk
    constexpr int HALVES = (CCH + 63) / 64; // 64-channel compare passes
    __shared__ __attribute__((aligned(16))) uint8_t s_seq[SEQ_LEN];
    __shared__ __attribute__((aligned(16))) uint8_t s_inv[256];
    __shared__ __attribute__((aligned(16))) uint8_t s_q[CCH * QPITCH];
    constexpr int PITCH = act_pitch<ZC>();
    __shared__ __attribute__((aligned(16))) uint32_t s_stage[ACT_SLOT_GROUP * PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pp0 = blockIdx.x * ACT_TILE;
    const int zg = blockIdx.y;
    const int n = blockIdx.z;
    const int HpWp = geo.Hp * geo.Wp;
    const int npix = min(ACT_TILE, HpWp - pp0);
    const float S = (float)gp.scale;

    load_tables_to_lds(tables + seq_index(gp.lb, gp.acc), s_seq, s_inv);

    // phase 1: load + quantise -> s_q[channel][pixel].  All loads of a thread are issued before the
    // first one is consumed (fully unrolled into registers): the phase costs one memory latency,
    // not one per element.
    if (!geo.channels_last) {
        // lane = pixel, the block's waves interleave over the channels of the chunk
        const int pp = pp0 + lane;
        const int yp = pp / geo.Wp, xp = pp - yp * geo.Wp;
        const int y = yp - geo.pad_h, xx = xp - geo.pad_w;
        const bool inb = (lane < npix) && y >= 0 && y < geo.H && xx >= 0 && xx < geo.W;
        constexpr int PER = CCH / 4;
        float v[PER];
#pragma unroll
        for (int k = 0; k < PER; k++) {
            const int c = zg * CCH + wave + 4 * k;
            v[k] = (inb && c < geo.C) ? x[(((long)n * geo.C + c) * geo.H + y) * geo.W + xx] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < PER; k++) s_q[(wave + 4 * k) * QPITCH + lane] = (uint8_t)quant_ceil_pos(v[k], S);
    } else {
        // lane = channel, each wave takes 16 pixels
        constexpr int PIX = ACT_TILE / 4, PASS = (CCH + 63) / 64;
        float v[PIX][PASS];
#pragma unroll
        for (int k = 0; k < PIX; k++) {
            const int j = wave + 4 * k;
            const int pp = pp0 + j;
            const int yp = pp / geo.Wp, xp = pp - yp * geo.Wp;
            const int y = yp - geo.pad_h, xx = xp - geo.pad_w;
            const bool inb = (j < npix) && y >= 0 && y < geo.H && xx >= 0 && xx < geo.W;
#pragma unroll
            for (int h = 0; h < PASS; h++) {
                const int cl = h * 64 + lane;
                const int c = zg * CCH + cl;
                v[k][h] = (inb && cl < CCH && c < geo.C) ? x[(((long)n * geo.H + y) * geo.W + xx) * geo.C + c] : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < PIX; k++)
#pragma unroll
            for (int h = 0; h < PASS; h++) {
                const int cl = h * 64 + lane;
                if (cl < CCH) s_q[cl * QPITCH + wave + 4 * k] = (uint8_t)quant_ceil_pos(v[k][h], S);
            }
    }
    __syncthreads();

    // per-lane seed phase of channel (lane + 64*h): (c*cmul) mod seed_mod
    int cmod[HALVES];
#pragma unroll
    for (int h = 0; h < HALVES; h++) {
        const int c = zg * CCH + h * 64 + lane;
        cmod[h] = (int)(((long)c * geo.seed_cmul) % gp.seed_mod);
    }

    for (int s0 = 0; s0 < gp.n_slots; s0 += ACT_SLOT_GROUP) {
        const int ns = min(ACT_SLOT_GROUP, gp.n_slots - s0);
        // phase 2: each wave generates 16 pixels
        for (int jj = 0; jj < ACT_TILE / 4; jj++) {
            const int j = wave * (ACT_TILE / 4) + jj;
            if (j >= npix) break; // uniform per wave
            const int pmod = (int)(((long)(pp0 + j) * geo.seed_pmul) % gp.seed_mod);
#pragma unroll
            for (int h = 0; h < HALVES; h++) {
                const int cl = h * 64 + lane;
                int v = 0;
                if (cl < CCH) v = s_q[cl * QPITCH + j];
                int sd = cmod[h] + pmod;
                if (sd >= gp.seed_mod) sd -= gp.seed_mod;
                const int pos = s_inv[sd + 1] + 1; // state of cycle t is seq[pos + t]
                uint32_t lo, hi;
                gen_slots32(s_seq, pos, v, gp, s0, ns, lo, hi);
                if (lane < ns) {
                    uint32_t *dst = &s_stage[lane * PITCH + j * ZC + h * 2];
                    dst[0] = lo;
                    if (ZC > 1) dst[1] = hi;
                }
            }
        }
        __syncthreads();
        // phase 3: coalesced write-out, npix*ZC contiguous words per slot
        const int run = npix * ZC;
        for (int s = 0; s < ns; s++) {
            uint32_t *dst = A + (long)(s0 + s) * geo.slot_stride + (((long)n * geo.ZG + zg) * HpWp + pp0) * ZC;
            for (int i = tid; i < run; i += 256) dst[i] = s_stage[s * PITCH + i];
        }
        __syncthreads();
    }
}

// ---- weight SNG ------------------------------------------------------------------------------
// Output layout: Wst[slot][ky][zg][o][pol][kx][zc]  (o padded to O_pad; padded rows are zero).
// Block: 256 threads, one (group of `wog` output channels, ky, zg); wog is 16, 8, 4 or 2, the largest
// that still gives the launch a few thousand blocks.
constexpr int W_OG_MAX = 16;
constexpr int W_SLOT_GROUP = 32; // upper bound; the launcher shrinks it to fit the LDS budget

template <int ZC>
__global__ __launch_bounds__(256) void sng_weight_kernel(const float *__restrict__ w, uint32_t *__restrict__ Wst,
                                                         const SeqTable *__restrict__ tables, WeightGeom geo, GenParams gp,
                                                         int slot_group, int wog)
{
    constexpr int CCH = 32 * ZC;
    constexpr int HALVES = (CCH + 63) / 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
    uint8_t *s_seq = s_dyn;
    uint8_t *s_inv = s_dyn + SEQ_LEN;
    uint32_t *s_stage = reinterpret_cast<uint32_t *>(s_dyn + SEQ_LEN + 256);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int og = blockIdx.x, ky = blockIdx.y, zg = blockIdx.z;
    const int KW = geo.KW;
    const int row = wog * 2 * KW * ZC; // words per slot handled by this block
    const int pitch = row + 2;          // LDS row pitch (bank spreading for the per-slot writes)
    const float S = (float)gp.scale;

    load_tables_to_lds(tables + seq_index(gp.lb, gp.acc), s_seq, s_inv);
    __syncthreads();

    const int ntask = wog * KW * HALVES;
    auto task_weight = [&](int task) -> float {
        const int h = task % HALVES;
        const int kx = (task / HALVES) % KW;
        const int ol = task / (HALVES * KW);
        const int o = og * wog + ol;
        const int cl = h * 64 + lane;
        const int c = zg * CCH + cl;
        if (task < ntask && cl < CCH && c < geo.C && o < geo.O) {
            const long wi = geo.channels_last ? (((long)o * geo.KH + ky) * KW + kx) * geo.C + c
                                              : (((long)o * geo.C + c) * geo.KH + ky) * KW + kx;
            return w[wi];
        }
        return 0.f;
    };

    for (int s0 = 0; s0 < gp.n_slots; s0 += slot_group) {
        const int ns = min(slot_group, gp.n_slots - s0);
        float f = task_weight(wave);
        for (int task = wave; task < ntask; task += 4) {
            const float f_next = task_weight(task + 4); // in flight while this task's slots are generated
            const int h = task % HALVES;
            const int kx = (task / HALVES) % KW;
            const int ol = task / (HALVES * KW);
            const int cl = h * 64 + lane;
            const int c = zg * CCH + cl;
            const int vp = quant_ceil_pos(f, S);
            const int vn = quant_ceil_neg(f, S);
            // seed (13 + c*KH*KW + ky*KW + kx) % seed_mod + 1  (sc_conv.cpp:80,92-93)
            const int sd = (int)((13L + (long)c * geo.KH * KW + ky * KW + kx) % gp.seed_mod);
            const int pos = s_inv[sd + 1] + 1;
            uint32_t plo, phi, nlo, nhi;
            gen_slots32(s_seq, pos, vp, gp, s0, ns, plo, phi);
            gen_slots32(s_seq, pos, vn, gp, s0, ns, nlo, nhi);
            if (lane < ns) {
                uint32_t *dp = &s_stage[lane * pitch + ((ol * 2 + 0) * KW + kx) * ZC + h * 2];
                uint32_t *dn = &s_stage[lane * pitch + ((ol * 2 + 1) * KW + kx) * ZC + h * 2];
                dp[0] = plo; dn[0] = nlo;
                if (ZC > 1) { dp[1] = phi; dn[1] = nhi; }
            }
            f = f_next;
        }
        __syncthreads();
        for (int s = 0; s < ns; s++) {
            uint32_t *dst = Wst + ((((long)(s0 + s) * geo.KH + ky) * geo.ZG + zg) * geo.O_pad + og * wog) * 2 * KW * ZC;
            for (int i = tid; i < row; i += 256) dst[i] = s_stage[s * pitch + i];
        }
        __syncthreads();
    }
}

template <int ZC>
static int launch_act(const float *x, uint32_t *A, const SeqTable *tables, const ActGeom &geo, const GenParams &gp,
                      hipStream_t stream)
{
    dim3 grid(ceil_div(geo.Hp * geo.Wp, ACT_TILE), geo.ZG, geo.N);
    // algorithmic bytes: fp32 operands in, stream words out
    ProfScope prof("sng_act", 4.0 * geo.N * geo.C * geo.H * geo.W + 4.0 * gp.n_slots * geo.N * geo.ZG * geo.Hp * geo.Wp * ZC,
                   stream);
    hipLaunchKernelGGL(sng_act_kernel<ZC>, grid, dim3(256), 0, stream, x, A, tables, geo, gp);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sng_activations(const float *x, uint32_t *A, const ActGeom &geo, const GenParams &gp, hipStream_t stream)
{
    const SeqTable *tables = nullptr;
    int rc = get_seq_tables(&tables, stream);
    if (rc) return rc;
    REXSC_CHECK_ARG(geo.ZG <= 65535 && geo.N <= 65535, "activation SNG: grid too large (ZG=%d N=%d)", geo.ZG, geo.N);
    switch (geo.ZC) {
    case 1: return launch_act<1>(x, A, tables, geo, gp, stream);
    case 2: return launch_act<2>(x, A, tables, geo, gp, stream);
    case 4: return launch_act<4>(x, A, tables, geo, gp, stream);
    case 8: return launch_act<8>(x, A, tables, geo, gp, stream);
    default: set_error("activation SNG: unsupported chunk width %d", geo.ZC); return REXSC_ERR_INVALID;
    }
}

template <int ZC>
static int launch_weight(const float *w, uint32_t *Wst, const SeqTable *tables, const WeightGeom &geo,
                         const GenParams &gp, hipStream_t stream)
{
    int wog = W_OG_MAX;
    while (wog > 2 && (long)(geo.O_pad / wog) * geo.KH * geo.ZG < 2048) wog /= 2;
    dim3 grid(geo.O_pad / wog, geo.KH, geo.ZG);
    const size_t row_bytes = sizeof(uint32_t) * (wog * 2 * geo.KW * ZC + 2);
    int slot_group = (int)((60 * 1024 - SEQ_LEN - 256) / row_bytes);
    if (slot_group > W_SLOT_GROUP) slot_group = W_SLOT_GROUP;
    REXSC_CHECK_ARG(slot_group >= 1, "weight SNG: kernel width %d too large for LDS staging", geo.KW);
    const size_t lds = SEQ_LEN + 256 + row_bytes * slot_group;
    ProfScope prof("sng_weight", 4.0 * geo.O * geo.C * geo.KH * geo.KW +
                                     4.0 * gp.n_slots * geo.KH * geo.ZG * geo.O_pad * 2 * geo.KW * ZC, stream);
    hipLaunchKernelGGL(sng_weight_kernel<ZC>, grid, dim3(256), lds, stream, w, Wst, tables, geo, gp, slot_group, wog);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sng_weights(const float *w, uint32_t *Wst, const WeightGeom &geo, const GenParams &gp, hipStream_t stream)
{
    const SeqTable *tables = nullptr;
    int rc = get_seq_tables(&tables, stream);
    if (rc) return rc;
    REXSC_CHECK_ARG(geo.O_pad % W_OG_MAX == 0, "weight SNG: O_pad %d not a multiple of %d", geo.O_pad, W_OG_MAX);
    REXSC_CHECK_ARG(geo.KH <= 65535 && geo.ZG <= 65535, "weight SNG: grid too large");
    switch (geo.ZC) {
    case 1: return launch_weight<1>(w, Wst, tables, geo, gp, stream);
    case 2: return launch_weight<2>(w, Wst, tables, geo, gp, stream);
    case 4: return launch_weight<4>(w, Wst, tables, geo, gp, stream);
    case 8: return launch_weight<8>(w, Wst, tables, geo, gp, stream);
    default: set_error("weight SNG: unsupported chunk width %d", geo.ZC); return REXSC_ERR_INVALID;
    }
}

} // namespace rexsc
