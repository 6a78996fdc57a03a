// Stream-number generation (SNG): float operands -> quantised integers -> LFSR bitstreams,
// packed 32 channels per word.  LFSR states are looked up in a per-width sequence table (any cycle
// of any seed is one byte read), so slots can be produced in any order.  Three generators:
//  * sng_act_sliced_kernel: one thread per stream word, bit-plane ("bit-sliced") comparison of 32
//    channels at once against state planes from a small geometry-only table;
//  * sng_act_kernel: lane = channel, one v_cmp per slot whose 64-bit lane mask IS two stream
//    words (for problems too small to amortise the table);
//  * sng_weight_kernel: ballots for the weight bit planes, bit-sliced comparison per (word, slot)
//    lane, rows staged in LDS in the order the compute kernel reads them.
//
// Semantics follow the reference CPU extension: sc_conv.cpp:42-200 (conv), sc_matmul.cpp:3-383
// (linear); quantisation sc_conv.cpp:316-320.
#include <stdlib.h>
#include <string.h>
#include <mutex>
#include <type_traits>
#include <utility>

#include "sng.h"
#include "profile.h"

namespace rexsc {

// ---- sequence tables -------------------------------------------------------------------------
static __device__ SeqTable g_seq_tables[N_SEQ_TABLES];

__global__ void build_seq_tables_kernel()
{
    int idx = threadIdx.x;
    if (idx >= N_SEQ_TABLES) return;
    int lb = idx / 3 + 3, acc = idx % 3;
    int period = acc == LFSR_ACC ? (1 << lb) : (1 << lb) - 1;
    SeqTable &t = g_seq_tables[idx];
    int v = acc == LFSR_XNOR ? 0 : 1; // a state on the cycle (the plain LFSR never reaches 0, the XNOR one never all-ones)
    for (int i = 0; i < 256; i++) t.inv[i] = 0;
    for (int i = 0; i < SEQ_LEN; i++) {
        t.seq[i] = (uint8_t)v;
        if (i < period) t.inv[v] = (uint8_t)i;
        v = lfsr_step(lb, acc, v);
    }
}

int get_seq_tables(const SeqTable **tables, hipStream_t stream)
{
    static std::mutex mu;
    static SeqTable *dev_ptr[64] = {nullptr};
    int dev = 0;
    REXSC_CHECK_HIP(hipGetDevice(&dev));
    REXSC_CHECK_ARG(dev >= 0 && dev < 64, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!dev_ptr[dev]) {
        // The one-time build ends with a synchronisation, which a stream under capture cannot take.
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        REXSC_CHECK_HIP(hipStreamIsCapturing(stream, &cap));
        REXSC_CHECK_ARG(cap == hipStreamCaptureStatusNone,
                        "first use on this device while the stream is being captured: call rexsc_init() before the capture");
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
// The layers' fake quantisation (utils_functional.py:93-104), folded into the load stage on request:
// mul, round half to even, clamp, div by a power of two -- the same four float32 operations.
__device__ __forceinline__ float fake_quantize(float v, int k)
{
    if (k <= 0) return v;
    const float p2 = (float)(1 << (k - 1));
    const float t = fminf(fmaxf(rintf(v * p2), 1.f - p2), p2 - 1.f);
    return t / p2;
}

// x * S as the generator sees it: exact float32 product, rounded to binary16 in legacy mode
__device__ __forceinline__ float scaled_operand(float v, float S, int legacy)
{
    float t = v * S;
    if (legacy) t = (float)(_Float16)t; // round to nearest even, as a tensor cast to float16 does
    return t;
}
__device__ __forceinline__ int quant_ceil_pos(float v, float S, float hi, int legacy)
{   // ceil(clamp(v*S, 0, hi))
    float t = scaled_operand(v, S, legacy);
    t = fminf(fmaxf(t, 0.f), hi);
    return (int)ceilf(t);
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
        for (int k = 0; k < PER; k++) s_q[(wave + 4 * k) * QPITCH + lane] = (uint8_t)quant_ceil_pos(fake_quantize(v[k], gp.fake_quant), S, gp.clamp_hi, gp.legacy);
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
                if (cl < CCH) s_q[cl * QPITCH + wave + 4 * k] = (uint8_t)quant_ceil_pos(fake_quantize(v[k][h], gp.fake_quant), S, gp.clamp_hi, gp.legacy);
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
                const int pos = s_inv[sd + gp.seed_off] + 1; // state of cycle t is seq[pos + t]
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

// ---- bit-sliced activation SNG ---------------------------------------------------------------
// One thread produces one stream word per slot: the 32 channels of word z at padded pixel pp.
// The 32 quantised values are transposed once into LB bit planes (bit c of plane k = bit k of the
// value of channel c); the LFSR states of the same 32 channels at every slot come as bit planes
// from a table that depends only on the geometry (word, slot, pixel index mod seed_mod), and
// "value > state" for all 32 channels is 2*LB-1 bitwise operations.  Thread i of the grid writes
// word i of every slot plane, so stores are contiguous and nothing is staged through LDS.
//
// Table rows hold one word per pm = (pp * seed_pmul) mod seed_mod: 2^lb words (seed_mod entries and
// one of padding), or a single word when the seed does not depend on the pixel, as in the linear
// op.  Lanes of a wave are neighbouring pixels, so one load covers a few cache lines.
//  * full table T[z][slot][k][pm]: plane k of the states at that slot;
//  * shift table T[z][tau][pm], tau = cycle + lb - 1: plane 0 only.  A Fibonacci LFSR moves its
//    bits up by one place per step, so bit k of the state at cycle t is bit 0 of the state at
//    cycle t - k: consecutive slots share all but one plane, and the kernel slides a window of lb
//    words along the cycle axis, loading one new word per slot.  Valid when slot == cycle and the
//    LFSR has no spliced zero state.
struct ActTableJob {
    uint32_t *T; // nullptr: nothing to build
    GenParams gp;
    int n_words, PM, pitch, seed_cmul;
    int shift, n_tau;
};

// Half a wave per table entry (z, slot, pm): lane = channel, one ballot per bit plane.  Waves
// first_wave, first_wave + n_waves, ... of the caller's grid share the entries; s_seq / s_inv hold
// the sequence table of job.gp.
__device__ __forceinline__ void build_state_planes(const ActTableJob &job, const uint8_t *s_seq, const uint8_t *s_inv,
                                                   unsigned first_wave, unsigned n_waves)
{
    const GenParams &gp = job.gp;
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5, cc = lane & 31;
    const int rows = job.shift ? job.n_tau : gp.n_slots; // table rows per word: cycles or slots
    const unsigned entries = (unsigned)job.n_words * rows * job.PM;
    const unsigned pairs = (entries + 1) / 2;
    const int cmul = job.seed_cmul % gp.seed_mod;
    for (unsigned pair = first_wave; pair < pairs; pair += n_waves) {
        unsigned e = pair * 2 + half;
        const bool valid = e < entries;
        if (!valid) e = entries - 1;
        const int pm = (int)(e % job.PM);
        const unsigned sz = e / job.PM;
        const int s = (int)(sz % rows);
        const int z = (int)(sz / rows);
        const int ch = z * 32 + cc;
        int sd = ((ch % gp.seed_mod) * cmul) % gp.seed_mod + pm;
        if (sd >= gp.seed_mod) sd -= gp.seed_mod;
        const int pos = s_inv[sd + gp.seed_off] + 1;
        if (job.shift) {
            int idx = pos + s - (gp.lb - 1); // cycle s - (lb - 1); the sequence has period gp.period
            if (idx < 0) idx += gp.period;
            const unsigned long long m = __ballot(s_seq[idx] & 1u);
            if (valid && cc == 0) job.T[((long)z * rows + s) * job.pitch + pm] = half ? (uint32_t)(m >> 32) : (uint32_t)m;
            continue;
        }
        const uint32_t st = s_seq[pos + slot_cycle(gp, s)];
        uint32_t mine = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const unsigned long long m = __ballot((st >> k) & 1u);
            const uint32_t word = half ? (uint32_t)(m >> 32) : (uint32_t)m;
            if (cc == k) mine = word;
        }
        if (valid && cc < gp.lb) job.T[((long)(z * gp.n_slots + s) * gp.lb + cc) * job.pitch + pm] = mine;
    }
}

// all 32 channels of one word: value > state, from bit planes (least significant plane first):
// a higher plane decides wherever it differs, otherwise the result of the lower planes stands
template <int LB>
__device__ __forceinline__ uint32_t planes_greater(const uint32_t (&V)[LB], const uint32_t (&S)[LB], int first_plane)
{
    uint32_t gt = 0;
#pragma unroll
    for (int k = 0; k < LB; k++) {
        const uint32_t vk = k >= first_plane ? V[k] : 0u; // progressive loading truncates low bits
        const uint32_t d = vk ^ S[k];
        gt = (d & vk) | (~d & gt);
    }
    return gt;
}

// One round of the 8x8 bit-matrix transposition between register index and bit position inside
// every byte: exchanges index bit log2(D) with position bit log2(D).
template <int D, uint32_t MASK>
__device__ __forceinline__ void transpose_round(uint32_t &lo, uint32_t &hi)
{
    const uint32_t nlo = (lo & MASK) | ((hi << D) & ~MASK);
    const uint32_t nhi = ((lo >> D) & MASK) | (hi & ~MASK);
    lo = nlo; hi = nhi;
}

// 32 quantised values (at most 8 bits each), packed so that byte b of R[j] is the value of channel
// 8*b + j, become bit planes: afterwards bit c of R[k] is bit k of the value of channel c.
__device__ __forceinline__ void values_to_planes(uint32_t (&R)[8])
{
    transpose_round<1, 0x55555555u>(R[0], R[1]); transpose_round<1, 0x55555555u>(R[2], R[3]);
    transpose_round<1, 0x55555555u>(R[4], R[5]); transpose_round<1, 0x55555555u>(R[6], R[7]);
    transpose_round<2, 0x33333333u>(R[0], R[2]); transpose_round<2, 0x33333333u>(R[1], R[3]);
    transpose_round<2, 0x33333333u>(R[4], R[6]); transpose_round<2, 0x33333333u>(R[5], R[7]);
    transpose_round<4, 0x0f0f0f0fu>(R[0], R[4]); transpose_round<4, 0x0f0f0f0fu>(R[1], R[5]);
    transpose_round<4, 0x0f0f0f0fu>(R[2], R[6]); transpose_round<4, 0x0f0f0f0fu>(R[3], R[7]);
}

// ceil(clamp(v*S, 0, hi)) of channel c, deposited in its byte of the packed registers
template <int C>
__device__ __forceinline__ void pack_quantised(uint32_t (&R)[8], float v, float S, float hi, int legacy)
{
    float t = scaled_operand(v, S, legacy);
    t = ceilf(fminf(fmaxf(t, 0.f), hi));
    R[C & 7] = __builtin_amdgcn_cvt_pk_u8_f32(t, C >> 3, R[C & 7]);
}
template <int... C>
__device__ __forceinline__ void pack_quantised_all(uint32_t (&R)[8], const float (&v)[32], float S, float hi, int legacy,
                                                   std::integer_sequence<int, C...>)
{
    (pack_quantised<C>(R, v[C], S, hi, legacy), ...);
}

template <int LB, bool PIXSEED, bool SHIFT>
__global__ __launch_bounds__(256) void sng_act_sliced_kernel(const float *__restrict__ x, uint32_t *__restrict__ A,
                                                             const uint32_t *__restrict__ T, ActGeom geo, GenParams gp,
                                                             int slots_per_split, int vec4, int log2_zc,
                                                             int waves_per_plane, int n_waves)
{
    // wave-uniform part of the index: which (image, channel chunk) plane, which 64 words of it
    const int wg = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
    if (wg >= n_waves) return;
    const int q = wg / waves_per_plane;
    const int wb = wg - q * waves_per_plane;
    const int zg = q % geo.ZG, n = q / geo.ZG;
    const int HpWp = geo.Hp * geo.Wp;
    const int plane_words = HpWp << log2_zc;
    const int rem = wb * 64 + (threadIdx.x & 63);
    if (rem >= plane_words) return;
    const int zc = rem & ((1 << log2_zc) - 1);
    const int pp = rem >> log2_zc;
    const int z = (zg << log2_zc) + zc;
    const int c0 = z * 32;
    const int yp = pp / geo.Wp, xp = pp - yp * geo.Wp;
    const int y = yp - geo.pad_h, xx = xp - geo.pad_w;
    const bool inb = y >= 0 && y < geo.H && xx >= 0 && xx < geo.W && c0 < geo.C;
    const float S = (float)gp.scale;

    uint32_t R[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (inb) {
        float v[32];
        if (geo.channels_last) {
            const float *src = x + (((long)n * geo.H + y) * geo.W + xx) * geo.C + c0;
            if (vec4 && c0 + 32 <= geo.C) {
#pragma unroll
                for (int f4 = 0; f4 < 8; f4++) {
                    const float4 f = reinterpret_cast<const float4 *>(src)[f4];
                    v[4 * f4] = f.x; v[4 * f4 + 1] = f.y; v[4 * f4 + 2] = f.z; v[4 * f4 + 3] = f.w;
                }
            } else {
#pragma unroll
                for (int cc = 0; cc < 32; cc++) v[cc] = c0 + cc < geo.C ? src[cc] : 0.f;
            }
        } else {
            const long plane = (long)geo.H * geo.W;
            const float *src = x + ((long)n * geo.C + c0) * plane + (long)y * geo.W + xx;
#pragma unroll
            for (int cc = 0; cc < 32; cc++) v[cc] = c0 + cc < geo.C ? src[cc * plane] : 0.f;
        }
        if (gp.fake_quant) {
#pragma unroll
            for (int cc = 0; cc < 32; cc++) v[cc] = fake_quantize(v[cc], gp.fake_quant);
        }
        pack_quantised_all(R, v, S, gp.clamp_hi, gp.legacy, std::make_integer_sequence<int, 32>{});
        values_to_planes(R);
    }
    uint32_t V[LB];
#pragma unroll
    for (int k = 0; k < LB; k++) V[k] = R[k];
    // legacy quantisation can reach 2^LB, one more than any LFSR state: those channels are always one
    const uint32_t vtop = gp.legacy ? R[LB & 7] : 0u;

    constexpr int PITCH = PIXSEED ? (1 << LB) : 1; // words per table row
    const int pm = PIXSEED ? ((pp % gp.seed_mod) * (geo.seed_pmul % gp.seed_mod)) % gp.seed_mod : 0;
    const int s_begin = blockIdx.y * slots_per_split;
    const int s_end = min(gp.n_slots, s_begin + slots_per_split);
    uint32_t *dst = A + (long)q * plane_words + rem + (long)s_begin * geo.slot_stride;
    const int n_mine = s_end - s_begin;
    // Slots go in groups of U with the table words of the next group requested before the words of
    // the current one are stored: loads and stores complete in issue order on this hardware, so a
    // load issued after a store would have to wait for that store as well.
    constexpr int U = 4;
    if constexpr (SHIFT) {
        const int n_tau = gp.n_slots + LB - 1;
        // row r of T0: plane 0 at cycle s_begin + r - (LB - 1)
        const uint32_t *T0 = T + ((long)z * n_tau + s_begin) * PITCH + pm;
        uint32_t W[LB]; // W[k] = plane 0 at cycle (slot - k) = plane k at the current slot
#pragma unroll
        for (int k = 0; k < LB; k++) W[k] = T0[(LB - 1 - k) * PITCH];
        for (int g0 = 0; g0 < n_mine; g0 += U) {
            uint32_t nxt[U];
#pragma unroll
            for (int u = 0; u < U; u++) nxt[u] = T0[(long)(min(g0 + u + 1, n_mine - 1) + LB - 1) * PITCH];
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (g0 + u < n_mine) {
                    const int first = gp.prog ? prog_shift(gp, s_begin + g0 + u) : 0;
                    dst[(long)(g0 + u) * geo.slot_stride] = planes_greater<LB>(V, W, first) | vtop;
                }
#pragma unroll
                for (int k = LB - 1; k > 0; k--) W[k] = W[k - 1];
                W[0] = nxt[u];
            }
        }
    } else {
        const uint32_t *Ts = T + ((long)z * gp.n_slots + s_begin) * (LB * PITCH) + pm;
        constexpr int t_step = LB * PITCH;
        auto load_group = [&](uint32_t (&Sg)[U][LB], int g0) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int su = min(g0 + u, n_mine - 1); // past the end: re-read the last row (unused)
#pragma unroll
                for (int k = 0; k < LB; k++) Sg[u][k] = Ts[(long)su * t_step + k * PITCH];
            }
        };
        uint32_t Sa[U][LB];
        load_group(Sa, 0);
        for (int g0 = 0; g0 < n_mine; g0 += U) {
            uint32_t Sb[U][LB];
            load_group(Sb, g0 + U);
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (g0 + u < n_mine) {
                    const int first = gp.prog ? prog_shift(gp, slot_cycle(gp, s_begin + g0 + u)) : 0;
                    dst[(long)(g0 + u) * geo.slot_stride] = planes_greater<LB>(V, Sa[u], first) | vtop;
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int k = 0; k < LB; k++) Sa[u][k] = Sb[u][k];
        }
    }
}

// REXSC_SNG_MODE: 0/unset = choose per problem, 1 = always the ballot activation generator,
// 2 = always the bit-sliced one
static int sng_mode()
{
    const char *e = getenv("REXSC_SNG_MODE");
    return e ? atoi(e) : 0;
}

static ActTableJob act_table_job(uint32_t *T, const ActGeom &geo, const GenParams &gp)
{
    ActTableJob job;
    job.T = T;
    job.gp = gp;
    job.n_words = geo.ZG * geo.ZC;
    job.PM = geo.seed_pmul % gp.seed_mod == 0 ? 1 : gp.seed_mod;
    job.pitch = job.PM == 1 ? 1 : (1 << gp.lb);
    job.seed_cmul = geo.seed_cmul;
    job.shift = (gp.acc != LFSR_ACC && gp.slot_div == 1 && gp.slot_mul == 1 && gp.slot_mod == 1) ? 1 : 0;
    job.n_tau = gp.n_slots + gp.lb - 1;
    return job;
}

static size_t act_table_words_of(const ActTableJob &job)
{
    return (size_t)job.n_words * (job.shift ? (size_t)job.n_tau : (size_t)job.gp.n_slots * job.gp.lb) * job.pitch;
}

size_t sng_act_table_words(const ActGeom &geo, const GenParams &gp)
{
    const int mode = sng_mode();
    if (mode == 1) return 0;
    const size_t words = act_table_words_of(act_table_job(nullptr, geo, gp));
    // worth it only when the table is small against the streams it helps to produce
    if (mode != 2 && words * 8 > (size_t)gp.n_slots * (size_t)geo.slot_stride) return 0;
    return words;
}

template <int LB, bool PIXSEED, bool SHIFT>
static void launch_act_sliced(const float *x, uint32_t *A, const uint32_t *T, const ActGeom &geo, const GenParams &gp,
                              hipStream_t stream)
{
    int log2_zc = 0;
    while ((1 << log2_zc) < geo.ZC) log2_zc++;
    const int waves_per_plane = ceil_div(geo.Hp * geo.Wp * geo.ZC, 64);
    const long n_waves = (long)geo.N * geo.ZG * waves_per_plane;
    const long blocks = (n_waves + 3) / 4;
    // few words per slot plane: split the slots over blocks as well.  Every split repeats the plane
    // build, so only launches with less than two blocks per CU are split (REXSC_TUNE_SNG_BLOCKS).
    int splits = 1;
    const char *tune = getenv("REXSC_TUNE_SNG_BLOCKS");
    const long min_blocks = tune && atoi(tune) > 0 ? atoi(tune) : 512;
    while (blocks * splits < min_blocks && splits * 2 <= gp.n_slots) splits *= 2;
    const int sps = ceil_div(gp.n_slots, splits);
    const int vec4 = geo.channels_last && geo.C % 4 == 0 && ((uintptr_t)x % 16 == 0);
    hipLaunchKernelGGL((sng_act_sliced_kernel<LB, PIXSEED, SHIFT>), dim3((unsigned)blocks, ceil_div(gp.n_slots, sps)),
                       dim3(256), 0, stream, x, A, T, geo, gp, sps, vec4, log2_zc, waves_per_plane, (int)n_waves);
}

template <int LB>
static void launch_act_sliced_lb(const float *x, uint32_t *A, const uint32_t *T, const ActGeom &geo, const GenParams &gp,
                                 const ActTableJob &job, hipStream_t stream)
{
    if (job.PM == 1) {
        if (job.shift) launch_act_sliced<LB, false, true>(x, A, T, geo, gp, stream);
        else launch_act_sliced<LB, false, false>(x, A, T, geo, gp, stream);
    } else {
        if (job.shift) launch_act_sliced<LB, true, true>(x, A, T, geo, gp, stream);
        else launch_act_sliced<LB, true, false>(x, A, T, geo, gp, stream);
    }
}

// The table must have been built (by the weight generator's launch) for the same geo / gp.
static int sng_activations_sliced(const float *x, uint32_t *A, const uint32_t *T, const ActGeom &geo, const GenParams &gp,
                                  hipStream_t stream)
{
    const ActTableJob job = act_table_job(nullptr, geo, gp);
    REXSC_CHECK_ARG((long)geo.N * geo.ZG * ceil_div(geo.Hp * geo.Wp * geo.ZC, 64) < (1L << 31) &&
                    (geo.ZC & (geo.ZC - 1)) == 0, "activation SNG: problem too large");
    ProfScope prof("sng_act", 4.0 * geo.N * geo.C * geo.H * geo.W + 4.0 * gp.n_slots * geo.N * geo.ZG * geo.Hp * geo.Wp * geo.ZC,
                   stream);
    switch (gp.lb) {
    case 3: launch_act_sliced_lb<3>(x, A, T, geo, gp, job, stream); break;
    case 4: launch_act_sliced_lb<4>(x, A, T, geo, gp, job, stream); break;
    case 5: launch_act_sliced_lb<5>(x, A, T, geo, gp, job, stream); break;
    case 6: launch_act_sliced_lb<6>(x, A, T, geo, gp, job, stream); break;
    case 7: launch_act_sliced_lb<7>(x, A, T, geo, gp, job, stream); break;
    case 8: launch_act_sliced_lb<8>(x, A, T, geo, gp, job, stream); break;
    default: set_error("activation SNG: unsupported LFSR width %d", gp.lb); return REXSC_ERR_INVALID;
    }
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

// ---- weight SNG ------------------------------------------------------------------------------
// Output layout: Wst[slot][ky][zg][o][pol][kx][zc]  (o padded to O_pad; padded rows are zero).
// Block: 256 threads, one (group of `wog` output channels, ky, zg); wog is 16, 8, 4 or 2, the largest
// that still gives the launch several hundred blocks.
constexpr int W_OG_MAX = 16;
constexpr int W_SLOT_GROUP = 32; // upper bound (64 in the lane = slot variant); the launcher shrinks it to fit the LDS budget

// s_waitcnt immediate: vmcnt(0), expcnt and lgkmcnt left at their maxima (not waited for)
constexpr int WAIT_VM0 = 0x0F70;
constexpr int W_COMBO_CHUNK = 8; // (kx, 64-channel half) combinations whose state planes are held in LDS at a time

// Streams of one (kx, 64-channel half, output channel) triple for a group of up to 32 slots:
//  * lane = channel quantises its weight; one ballot per bit plane and polarity turns the 64 values
//    into value bit planes that sit in SGPR pairs (low word: channels 0..31, high word: 32..63);
//  * lane = (word w, slot t) holds the LFSR states of the word's 32 channels at slot t as bit planes
//    (computed once per block and slot group, shared by all output channels);
//  * "value > state" for the 32 channels of a word is then 2 bitwise operations per plane, and
//    the lane ends up with the finished stream word of (slot t, word w), which it puts into the
//    staging row of slot t.
// S64: a group is 64 slots and lane = slot; the two words of a 64-channel half are finished one after
// the other with the ballot halves as scalar operands (no per-lane select), and weights are loaded
// and balloted once per 64 slots.  Otherwise a group is 32 slots and lane = (word, slot).
template <int ZC, int LB, bool PROG, bool S64>
__global__ __launch_bounds__(256) void sng_weight_kernel(const float *__restrict__ w, uint32_t *__restrict__ Wst,
                                                         const SeqTable *__restrict__ tables, WeightGeom geo, GenParams gp,
                                                         int slot_group, int wog, ActTableJob job,
                                                         const unsigned long long *__restrict__ guard, unsigned long long epoch)
{
    constexpr int CCH = 32 * ZC;
    constexpr int HALVES = (CCH + 63) / 64;
    if (guard && *guard != epoch) return; // kept streams are still those of these weights (uniform over the grid)
    extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
    uint8_t *s_seq = s_dyn;
    uint8_t *s_inv = s_dyn + SEQ_LEN;
    uint8_t *s_pos = s_dyn + SEQ_LEN + 256;                                 // [combo in chunk][channel of the half]
    // [combo in chunk][word (S64 only)][plane 0..7][lane]: W_COMBO_CHUNK combinations, half as many for S64
    uint32_t *s_S = reinterpret_cast<uint32_t *>(s_pos + W_COMBO_CHUNK * 64);
    uint32_t *s_stage = s_S + W_COMBO_CHUNK * 8 * 64;
    constexpr int CCHUNK = S64 ? W_COMBO_CHUNK / 2 : W_COMBO_CHUNK;
    constexpr int NW = S64 ? 2 : 1;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wblock = blockIdx.x;
    const int n_og = geo.O_pad / wog;
    const int og = wblock % n_og;
    const int ky = (wblock / n_og) % geo.KH;
    const int zg = wblock / (n_og * geo.KH);
    const int KW = geo.KW;
    const int row = wog * 2 * KW * ZC; // words per slot handled by this block
    const int pitch = row + 2;          // LDS row pitch (bank spreading for the per-slot writes)
    const float S = (float)gp.scale;
    // this lane's word of the 64-channel half (both words in turn for S64), and its slot of the group
    const int wsel = S64 ? 0 : lane >> 5, t = S64 ? lane : lane & 31;
    const int ncombo = KW * HALVES;
    // weight element of (output channel o, channel c, ky, kx): o*o_stride + lane part + h*h_step + kx*kx_mul
    const long o_stride = (long)geo.C * geo.KH * KW;
    const long c_lane = (long)zg * CCH + lane;
    const long lane_off = geo.channels_last ? (long)ky * KW * geo.C + c_lane : (c_lane * geo.KH + ky) * KW;
    const int h_step = geo.channels_last ? 64 : 64 * geo.KH * KW;
    const int kx_mul = geo.channels_last ? geo.C : 1;

    load_tables_to_lds(tables + seq_index(gp.lb, gp.acc), s_seq, s_inv);
    __syncthreads();

    for (int s0 = 0; s0 < gp.n_slots; s0 += slot_group) {
        const int ns = min(slot_group, gp.n_slots - s0);
        const int cyc = slot_cycle(gp, s0 + min(t, ns - 1));
        const int first_plane = PROG ? prog_shift(gp, cyc) : 0;
        for (int combo0 = 0; combo0 < ncombo; combo0 += CCHUNK) {
            const int ncc = min(CCHUNK, ncombo - combo0);
            // cycle position of every channel's seed, lane = channel of the 64-channel half:
            // seed (seed_add + c*KH*KW + ky*KW + kx) % seed_mod + seed_off, seed_add = 13  (sc_conv.cpp:80,92-93)
            if (s0 == 0 || ncombo > CCHUNK) {
                for (int cl = wave; cl < ncc; cl += 4) {
                    const int combo = combo0 + cl;
                    const int h = combo % HALVES, kx = combo / HALVES;
                    const long c = (long)zg * CCH + h * 64 + lane;
                    // (+ o * seed_omul for generators that differ per output channel: blocks then hold one channel each)
                    const int sd = (int)(((long)gp.seed_add + (long)og * wog * geo.seed_omul + c * geo.KH * KW + ky * KW + kx) % gp.seed_mod);
                    s_pos[cl * 64 + lane] = s_inv[sd + gp.seed_off];
                }
                __syncthreads();
            }
            // state planes of this lane's (word, slot) for every combination of the chunk
            for (int cl = wave; cl < ncc; cl += 4) {
#pragma unroll
                for (int wq = 0; wq < NW; wq++) {
                    const uint8_t *pos = s_pos + cl * 64 + (S64 ? wq : wsel) * 32;
                    const uint8_t *seq = s_seq + 1 + cyc;
                    uint32_t R[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int cc = 0; cc < 32; cc++) {
                        const uint32_t st = seq[pos[cc]];
                        R[cc & 7] |= st << (8 * (cc >> 3));
                    }
                    values_to_planes(R);
#pragma unroll
                    for (int k = 0; k < LB; k++) s_S[((cl * NW + wq) * 8 + k) * 64 + lane] = R[k];
                }
            }
            __syncthreads();

            // tasks (output channel ol, combination cl) of this chunk, four apart per wave; all task
            // bookkeeping is wave-uniform (scalar) arithmetic
            const int ntask = wog * ncc;
            struct Task { int ol, cl; };
            auto advance = [&](Task &tk) {
                tk.cl += 4;
                while (tk.cl >= ncc) { tk.cl -= ncc; tk.ol++; }
            };
            auto task_weight = [&](const Task &tk) -> float {
                const int combo = combo0 + tk.cl;
                const int h = combo % HALVES, kx = combo / HALVES;
                const int o = og * wog + tk.ol;
                // channel of this lane: c = zg*CCH + h*64 + lane, inside the chunk and inside C
                const int lim = min(geo.C - zg * CCH - h * 64, CCH - h * 64);
                if (tk.ol < wog && lane < lim && o < geo.O)
                    return w[(long)o * o_stride + lane_off + (long)h * h_step + kx * kx_mul];
                return 0.f;
            };
            // The weights of Q tasks are requested together, one group ahead of their use.  Loads
            // complete in issue order, so the wait for the current group is placed before the next
            // group is requested; a wait after the request would cover the request as well.
            constexpr int Q = 4;
            Task cursor = {wave / ncc, wave % ncc};
            Task tq[Q], tq_next[Q];
            float cur[Q], nxt[Q];
#pragma unroll
            for (int i = 0; i < Q; i++) { tq[i] = cursor; advance(cursor); cur[i] = task_weight(tq[i]); }
            for (int base = wave; base < ntask; base += 4 * Q) {
                __builtin_amdgcn_s_waitcnt(WAIT_VM0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < Q; i++) { tq_next[i] = cursor; advance(cursor); nxt[i] = task_weight(tq_next[i]); }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < Q; i++) {
                    if (tq[i].ol >= wog) continue; // past the last task (wave-uniform)
                    const float f = fake_quantize(cur[i], gp.fake_quant) * gp.sign;
                    const int cl = tq[i].cl, ol = tq[i].ol;
                    const int combo = combo0 + cl;
                    const int h = combo % HALVES, kx = combo / HALVES;
                    // A weight feeds one polarity only (the other one quantises to 0): ballot the planes
                    // of the magnitude ceil(min(|f*S|, S-1)) and split them with the sign mask.  A NaN
                    // counts as negative, as it does in ceil(-clamp(f*S, 1-S, 0)).
                    const uint32_t mag = (uint32_t)(int)ceilf(fminf(fabsf(scaled_operand(f, S, gp.legacy)), gp.clamp_hi));
                    const unsigned long long neg = __ballot(!(f >= 0.f));
                    uint32_t gt_p[NW], gt_n[NW];
#pragma unroll
                    for (int wq = 0; wq < NW; wq++) { gt_p[wq] = 0; gt_n[wq] = 0; }
#pragma unroll
                    for (int k = 0; k < LB; k++) {
                        const unsigned long long m = __ballot((mag >> k) & 1u);
                        const unsigned long long mp = m & ~neg, mn = m & neg;
#pragma unroll
                        for (int wq = 0; wq < NW; wq++) {
                            const bool hi = S64 ? wq == 1 : wsel != 0;
                            uint32_t vkp = hi ? (uint32_t)(mp >> 32) : (uint32_t)mp;
                            uint32_t vkn = hi ? (uint32_t)(mn >> 32) : (uint32_t)mn;
                            if (PROG && k < first_plane) { vkp = 0; vkn = 0; } // progressive loading truncates low bits
                            const uint32_t sk = s_S[((cl * NW + wq) * 8 + k) * 64 + lane];
                            const uint32_t dp = vkp ^ sk, dn = vkn ^ sk;
                            gt_p[wq] = (dp & vkp) | (~dp & gt_p[wq]);
                            gt_n[wq] = (dn & vkn) | (~dn & gt_n[wq]);
                        }
                    }
                    if (gp.legacy) { // magnitudes of 2^LB (above every state): always one
                        const unsigned long long m = __ballot((mag >> LB) & 1u);
                        const unsigned long long mp = m & ~neg, mn = m & neg;
#pragma unroll
                        for (int wq = 0; wq < NW; wq++) {
                            const bool hi = S64 ? wq == 1 : wsel != 0;
                            gt_p[wq] |= hi ? (uint32_t)(mp >> 32) : (uint32_t)mp;
                            gt_n[wq] |= hi ? (uint32_t)(mn >> 32) : (uint32_t)mn;
                        }
                    }
#pragma unroll
                    for (int wq = 0; wq < NW; wq++) {
                        const int wd = S64 ? wq : wsel;
                        if (t < ns && h * 2 + wd < ZC) {
                            s_stage[t * pitch + ((ol * 2 + 0) * KW + kx) * ZC + h * 2 + wd] = gt_p[wq];
                            s_stage[t * pitch + ((ol * 2 + 1) * KW + kx) * ZC + h * 2 + wd] = gt_n[wq];
                        }
                    }
                }
#pragma unroll
                for (int i = 0; i < Q; i++) { cur[i] = nxt[i]; tq[i] = tq_next[i]; }
            }
            __syncthreads();
        }
        for (int s = wave; s < ns; s += 4) {
            uint32_t *dst = Wst + ((((long)(s0 + s) * geo.KH + ky) * geo.ZG + zg) * geo.O_pad + og * wog) * 2 * KW * ZC;
            for (int i = lane; i < row; i += 64) dst[i] = s_stage[s * pitch + i];
        }
        __syncthreads();
    }
    // every block also builds its share of the activation generator's state-plane table (same LFSR
    // width and flavour as the weights, so the sequence table in LDS serves both)
    if (job.T) build_state_planes(job, s_seq, s_inv, wblock * 4 + wave, gridDim.x * 4);
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

int sng_activations(const float *x, uint32_t *A, const uint32_t *table, const ActGeom &geo, const GenParams &gp,
                    hipStream_t stream)
{
    const SeqTable *tables = nullptr;
    int rc = get_seq_tables(&tables, stream);
    if (rc) return rc;
    if (table) return sng_activations_sliced(x, A, table, geo, gp, stream);
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
                         const GenParams &gp, const ActTableJob &job, hipStream_t stream, const unsigned long long *guard,
                         unsigned long long epoch)
{
    int wog = W_OG_MAX;
    // every block computes the state planes of its (ky, zg) once, so blocks should not be too small;
    // about three per CU keep the chip busy
    const char *tune = getenv("REXSC_TUNE_WSNG_BLOCKS");
    const long min_blocks = tune && atoi(tune) > 0 ? atoi(tune) : 768;
    while (wog > 2 && (long)(geo.O_pad / wog) * geo.KH * geo.ZG < min_blocks) wog /= 2;
    if (geo.seed_omul) wog = 1; // the state planes a block computes once serve one output channel only
    const long n_wblocks = (long)(geo.O_pad / wog) * geo.KH * geo.ZG;
    REXSC_CHECK_ARG(n_wblocks < (1L << 31), "weight SNG: grid too large");
    if (job.T) {
        const long entries = (long)(act_table_words_of(job) / job.pitch / (job.shift ? 1 : job.gp.lb)) * job.PM;
        REXSC_CHECK_ARG(entries < (1L << 31), "activation SNG: state table too large");
        REXSC_CHECK_ARG(job.gp.lb == gp.lb && job.gp.acc == gp.acc, "activation and weight generators use different LFSRs");
    }
    const size_t fixed = SEQ_LEN + 256 + W_COMBO_CHUNK * 64 + sizeof(uint32_t) * W_COMBO_CHUNK * 8 * 64;
    auto row_bytes_of = [&](int g) { return sizeof(uint32_t) * (g * 2 * geo.KW * ZC + 2); };
    // 64-slot groups (lane = slot) when the streams are long enough and 64 staging rows fit the LDS
    // budget, if need be with fewer output channels per block
    bool s64 = gp.n_slots >= 64;
    if (s64) {
        int g = wog;
        while (g > 2 && fixed + row_bytes_of(g) * 64 > 60 * 1024) g /= 2;
        if (fixed + row_bytes_of(g) * 64 <= 60 * 1024) wog = g; else s64 = false;
    }
    const long n_wblocks2 = (long)(geo.O_pad / wog) * geo.KH * geo.ZG; // wog may have shrunk
    REXSC_CHECK_ARG(n_wblocks2 < (1L << 31), "weight SNG: grid too large");
    const size_t row_bytes = row_bytes_of(wog);
    int slot_group = (int)((60 * 1024 - fixed) / row_bytes);
    const int group_cap = s64 ? 64 : W_SLOT_GROUP;
    if (slot_group > group_cap) slot_group = group_cap;
    REXSC_CHECK_ARG(slot_group >= 1, "weight SNG: kernel width %d too large for LDS staging", geo.KW);
    const size_t lds = fixed + row_bytes * slot_group;
    ProfScope prof("sng_weight", 4.0 * geo.O * geo.C * geo.KH * geo.KW +
                                     4.0 * gp.n_slots * geo.KH * geo.ZG * geo.O_pad * 2 * geo.KW * ZC, stream);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)n_wblocks2), dim3(256), lds, stream, w, Wst, tables, geo, gp, slot_group,
                           wog, job, guard, epoch);
    };
    auto launch_lb = [&](auto lb_tag) {
        constexpr int LB = decltype(lb_tag)::value;
        if (s64) {
            if (gp.prog) launch(sng_weight_kernel<ZC, LB, true, true>); else launch(sng_weight_kernel<ZC, LB, false, true>);
        } else {
            if (gp.prog) launch(sng_weight_kernel<ZC, LB, true, false>); else launch(sng_weight_kernel<ZC, LB, false, false>);
        }
    };
    switch (gp.lb) {
    case 3: launch_lb(std::integral_constant<int, 3>{}); break;
    case 4: launch_lb(std::integral_constant<int, 4>{}); break;
    case 5: launch_lb(std::integral_constant<int, 5>{}); break;
    case 6: launch_lb(std::integral_constant<int, 6>{}); break;
    case 7: launch_lb(std::integral_constant<int, 7>{}); break;
    case 8: launch_lb(std::integral_constant<int, 8>{}); break;
    default: set_error("weight SNG: unsupported LFSR width %d", gp.lb); return REXSC_ERR_INVALID;
    }
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sng_weights(const float *w, uint32_t *Wst, const WeightGeom &geo, const GenParams &gp, uint32_t *act_table,
                const ActGeom *act_geo, const GenParams *act_gp, hipStream_t stream, const unsigned long long *guard,
                unsigned long long epoch)
{
    const SeqTable *tables = nullptr;
    int rc = get_seq_tables(&tables, stream);
    if (rc) return rc;
    REXSC_CHECK_ARG(geo.O_pad % W_OG_MAX == 0, "weight SNG: O_pad %d not a multiple of %d", geo.O_pad, W_OG_MAX);
    ActTableJob job;
    memset(&job, 0, sizeof(job));
    if (act_table) {
        REXSC_CHECK_ARG(act_geo && act_gp, "weight SNG: activation table requested without its geometry");
        job = act_table_job(act_table, *act_geo, *act_gp);
    }
    switch (geo.ZC) {
    case 1: return launch_weight<1>(w, Wst, tables, geo, gp, job, stream, guard, epoch);
    case 2: return launch_weight<2>(w, Wst, tables, geo, gp, job, stream, guard, epoch);
    case 4: return launch_weight<4>(w, Wst, tables, geo, gp, job, stream, guard, epoch);
    case 8: return launch_weight<8>(w, Wst, tables, geo, gp, job, stream, guard, epoch);
    default: set_error("weight SNG: unsupported chunk width %d", geo.ZC); return REXSC_ERR_INVALID;
    }
}

// ---- change detection for kept weight streams -------------------------------------------------------
// Bitwise comparison (a NaN equals itself, -0 differs from +0: the streams are a function of the bit pattern's
// value class only, so this can regenerate needlessly but never miss a change).  Every thread repairs the
// snapshot elements it finds different; a wave that found any stores the epoch (all writers store the same value).
__global__ __launch_bounds__(256) void weights_snapshot_kernel(const uint32_t *__restrict__ w, uint32_t *__restrict__ snap,
                                                               size_t n, unsigned long long *__restrict__ flag,
                                                               unsigned long long epoch, int force, int vec4)
{
    bool diff = false;
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, nthreads = (size_t)gridDim.x * 256;
    if (vec4) {
        const size_t n4 = n / 4;
        const uint4 *w4 = reinterpret_cast<const uint4 *>(w);
        uint4 *s4 = reinterpret_cast<uint4 *>(snap);
        for (size_t i = tid; i < n4; i += nthreads) {
            const uint4 a = w4[i];
            bool d = true;
            if (!force) {
                const uint4 b = s4[i];
                d = (a.x != b.x) | (a.y != b.y) | (a.z != b.z) | (a.w != b.w);
            }
            if (d) { s4[i] = a; diff = true; }
        }
        for (size_t i = n4 * 4 + tid; i < n; i += nthreads) {
            const uint32_t a = w[i];
            if (force || a != snap[i]) { snap[i] = a; diff = true; }
        }
    } else {
        for (size_t i = tid; i < n; i += nthreads) {
            const uint32_t a = w[i];
            if (force || a != snap[i]) { snap[i] = a; diff = true; }
        }
    }
    if (force) diff = true;
    if (__ballot(diff) != 0ull && (threadIdx.x & 63) == 0) *flag = epoch;
}

int weights_snapshot(const float *w, float *snapshot, size_t n, unsigned long long *flag, unsigned long long epoch,
                     int force, hipStream_t stream)
{
    REXSC_CHECK_ARG(w && snapshot && flag && n > 0, "weight snapshot: null pointer");
    const int vec4 = ((uintptr_t)w % 16 == 0) && ((uintptr_t)snapshot % 16 == 0);
    const size_t per_block = 256 * 4 * 4; // four 16-byte vectors per thread
    size_t blocks = (n + per_block - 1) / per_block;
    if (blocks > 2048) blocks = 2048;
    ProfScope prof("weights_snapshot", 8.0 * n, stream); // w read, snapshot read or written
    hipLaunchKernelGGL(weights_snapshot_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint32_t *)w,
                       (uint32_t *)snapshot, n, flag, epoch, force, vec4);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

// ---- tap folding --------------------------------------------------------------------------------
// One thread per output pixel and group of FOLD_SLOTS slots: lanes are neighbouring output pixels, so every tap's
// load is coalesced.  KH, KW > 0: kernel size known at compile time, so that all loads of a thread are in flight
// together (with run-time bounds every tap waits for the one before it: a chain of KH*KW cache latencies); 0: any size.
constexpr int FOLD_SLOTS = 4;
template <int KH_T, int KW_T>
__global__ __launch_bounds__(256) void fold_act_kernel(const uint32_t *__restrict__ A, uint32_t *__restrict__ A2, long a_stride,
                                                       long a2_stride, unsigned M, int n_slots, int Hp, int Wp, int Ho, int Wo,
                                                       int KH_R, int KW_R, int s0, int s1, int C)
{
    const unsigned m = blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    const int KH = KH_T ? KH_T : KH_R, KW = KW_T ? KW_T : KW_R;
    const unsigned HoWo = (unsigned)Ho * Wo;
    const unsigned n = m / HoWo, r = m - n * HoWo;
    const unsigned yo = r / (unsigned)Wo, xo = r - yo * (unsigned)Wo;
    const int slot0 = blockIdx.y * FOLD_SLOTS;
    const uint32_t *src = A + (long)slot0 * a_stride + ((long)n * Hp + yo * s0) * Wp + xo * s1;
    uint32_t *dst = A2 + (long)slot0 * a2_stride + m;
    if (KH_T && slot0 + FOLD_SLOTS <= n_slots) {
        uint32_t v[FOLD_SLOTS][KH_T ? KH_T * KW_T : 1];
#pragma unroll
        for (int q = 0; q < FOLD_SLOTS; q++)
#pragma unroll
            for (int t = 0; t < KH_T * KW_T; t++) v[q][t] = src[q * a_stride + (t / KW_T) * Wp + (t % KW_T)];
#pragma unroll
        for (int q = 0; q < FOLD_SLOTS; q++) {
            uint32_t word = 0;
#pragma unroll
            for (int t = 0; t < KH_T * KW_T; t++) word |= v[q][t] << (t * C);
            dst[q * a2_stride] = word;
        }
        return;
    }
    for (int q = 0; q < FOLD_SLOTS && slot0 + q < n_slots; q++) {
        uint32_t word = 0;
        for (int ky = 0; ky < KH; ky++)
            for (int kx = 0; kx < KW; kx++) word |= src[q * a_stride + ky * Wp + kx] << ((ky * KW + kx) * C);
        dst[q * a2_stride] = word;
    }
}

__global__ __launch_bounds__(256) void fold_weight_kernel(const uint32_t *__restrict__ Wst, uint32_t *__restrict__ W2, int n_slots,
                                                          int KH, int KW, int O_pad, int C,
                                                          const unsigned long long *__restrict__ guard, unsigned long long epoch)
{
    if (guard && *guard != epoch) return;
    // one thread per (slot, o, pol); Wst[slot][ky][o][pol][kx] (one word per pixel and tap)
    const long total = (long)n_slots * O_pad * 2;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const int pol = (int)(i & 1);
        const long so = i >> 1;
        const int o = (int)(so % O_pad), slot = (int)(so / O_pad);
        uint32_t word = 0;
        for (int ky = 0; ky < KH; ky++)
            for (int kx = 0; kx < KW; kx++)
                word |= Wst[((((long)slot * KH + ky) * O_pad + o) * 2 + pol) * KW + kx] << ((ky * KW + kx) * C);
        W2[i] = word;
    }
}

int fold_activation_streams(const uint32_t *A, uint32_t *A2, int n_slots, long a_stride, long a2_stride, int N, int Hp, int Wp,
                            int Ho, int Wo, int KH, int KW, int s0, int s1, int C, hipStream_t stream)
{
    const long M = (long)N * Ho * Wo;
    REXSC_CHECK_ARG(C * KH * KW <= 32 && M > 0 && M < (1L << 31) && n_slots <= 65535, "tap folding: shape out of range");
    ProfScope prof("fold_act", 4.0 * n_slots * ((double)N * Hp * Wp + (double)M), stream);
    const dim3 grid((unsigned)((M + 255) / 256), (unsigned)ceil_div(n_slots, FOLD_SLOTS));
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, A, A2, a_stride, a2_stride, (unsigned)M, n_slots, Hp, Wp, Ho, Wo,
                           KH, KW, s0, s1, C);
    };
    if (KH == 3 && KW == 3) launch(fold_act_kernel<3, 3>);
    else if (KH == 5 && KW == 5) launch(fold_act_kernel<5, 5>);
    else if (KH == 2 && KW == 2) launch(fold_act_kernel<2, 2>);
    else launch(fold_act_kernel<0, 0>);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int fold_weight_streams(const uint32_t *Wst, uint32_t *W2, int n_slots, int KH, int KW, int O_pad, int C, hipStream_t stream,
                        const unsigned long long *guard, unsigned long long epoch)
{
    REXSC_CHECK_ARG(C * KH * KW <= 32, "tap folding: receptive field wider than one word");
    const long total = (long)n_slots * O_pad * 2;
    ProfScope prof("fold_weight", 4.0 * total * (KH * KW + 1), stream);
    const int grid = (int)((total + 255) / 256 < 2048 ? (total + 255) / 256 : 2048);
    hipLaunchKernelGGL(fold_weight_kernel, dim3(grid), dim3(256), 0, stream, Wst, W2, n_slots, KH, KW, O_pad, C, guard, epoch);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

} // namespace rexsc
