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
//   grid            = pixel tiles x output-channel tiles x slot splits, remapped so that the
//                     blocks sharing a pixel tile run on the same XCD (shared L2).
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

constexpr int CB = 256; // threads per block

template <int KW, int ZC, int PX, int OT, bool WIDE>
__global__ __launch_bounds__(CB) void sc_compute_kernel(const uint32_t *__restrict__ A,
                                                        const uint32_t *__restrict__ Wst, ComputeParams p,
                                                        uint32_t *__restrict__ part, int16_t *__restrict__ out_pos,
                                                        int16_t *__restrict__ out_neg, int16_t *__restrict__ out_diff)
{
    constexpr int KWZ = KW * ZC;
    constexpr int BM = CB * PX;

    // XCD-aware block remap: hardware deals consecutive block ids round-robin over 8 XCDs;
    // give each XCD a contiguous range of logical ids (o-tiles of one pixel tile are adjacent).
    const int per_xcd = gridDim.x >> 3;
    int bid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (bid >= p.m_tiles * p.o_tiles * p.splits) return;
    const int otile = bid % p.o_tiles; bid /= p.o_tiles;
    const int mtile = bid % p.m_tiles;
    const int split = bid / p.m_tiles;

    const int tid = threadIdx.x;
    int abase[PX]; // word offset of the lane's pixel inside one slot, for ky = 0, zg = 0
    int mpix[PX];
#pragma unroll
    for (int px = 0; px < PX; px++) {
        const int m = mtile * BM + px * CB + tid;
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

    const int s_begin = split * p.slots_per_split;
    const int s_end = min(p.n_slots, s_begin + p.slots_per_split);
    const int chunk_stride = p.Hp * p.Wp * ZC; // words between zg planes
    const long w_chunk_words = (long)p.O_pad * 2 * KWZ;

    for (int slot = s_begin; slot < s_end; slot++) {
        uint32_t cp[PX][OT], cn[PX][OT];
#pragma unroll
        for (int px = 0; px < PX; px++)
#pragma unroll
            for (int o = 0; o < OT; o++) { cp[px][o] = 0; cn[px][o] = 0; }

        const uint32_t *a_slot = A + (long)slot * p.a_slot_stride;
        const uint32_t *w_slot = Wst + (long)slot * p.KH * p.ZG * w_chunk_words + (long)otile * OT * 2 * KWZ;
        for (int ky = 0; ky < p.KH; ky++) {
            for (int zg = 0; zg < p.ZG; zg++) {
                uint32_t a[PX][KWZ];
#pragma unroll
                for (int px = 0; px < PX; px++) {
                    const uint32_t *ap = a_slot + abase[px] + zg * chunk_stride + ky * p.Wp * ZC;
#pragma unroll
                    for (int kx = 0; kx < KW; kx++) load_words<ZC>(ap + kx * ZC, &a[px][kx * ZC]);
                }
                const uint32_t *wc = w_slot + (long)(ky * p.ZG + zg) * w_chunk_words;
#pragma unroll
                for (int o = 0; o < OT; o++) {
#pragma unroll
                    for (int j = 0; j < KWZ; j++) {
                        const uint32_t wp = wc[(o * 2 + 0) * KWZ + j];
                        const uint32_t wn = wc[(o * 2 + 1) * KWZ + j];
#pragma unroll
                        for (int px = 0; px < PX; px++) {
                            cp[px][o] += __builtin_popcount(a[px][j] & wp);
                            cn[px][o] += __builtin_popcount(a[px][j] & wn);
                        }
                    }
                }
            }
        }
        // per-slot saturation and accumulation
        if (!WIDE) {
            if (p.mode == 0) {
#pragma unroll
                for (int px = 0; px < PX; px++)
#pragma unroll
                    for (int o = 0; o < OT; o++) {
                        const uint32_t c = cp[px][o] | (cn[px][o] << 16);
                        acc[px][o] = pk_add_u16(acc[px][o], pk_min_u16(c, p.nn));
                    }
            } else { // [count >= n] = min(count, n) - min(count, n-1)
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
    }

    // epilogue
    if (p.direct) {
#pragma unroll
        for (int px = 0; px < PX; px++) {
            const int m = mpix[px];
            if (m >= p.M) continue;
            const int n = m / p.HoWo, r = m - n * p.HoWo;
#pragma unroll
            for (int o = 0; o < OT; o++) {
                const int oo = otile * OT + o;
                if (oo >= p.O) continue;
                const long idx = p.out_channels_last ? (long)m * p.O + oo : ((long)n * p.O + oo) * p.HoWo + r;
                const int16_t vp = (int16_t)(acc[px][o] & 0xffffu), vn = (int16_t)(acc[px][o] >> 16);
                if (out_pos) out_pos[idx] = vp;
                if (out_neg) out_neg[idx] = vn;
                if (out_diff) out_diff[idx] = (int16_t)(vp - vn);
            }
        }
    } else {
        // partial sums: part[plane][split][o][m]; plane 1 only in WIDE mode
        const long plane = (long)p.splits * p.O_pad * p.M;
#pragma unroll
        for (int px = 0; px < PX; px++) {
            const int m = mpix[px];
            if (m >= p.M) continue;
#pragma unroll
            for (int o = 0; o < OT; o++) {
                const long idx = ((long)split * p.O_pad + otile * OT + o) * p.M + m;
                part[idx] = acc[px][o];
                if (WIDE) part[plane + idx] = accw[px][o];
            }
        }
    }
}

// Sum the slot-split partials and write the final tensors.
// conv:   int16 pos / neg / diff, NCHW or NHWC, sums wrap at 16 bits like the reference's.
// linear: int32 pos / neg [M][O].
template <bool WIDE, typename OutT>
__global__ __launch_bounds__(256) void sc_finalize_kernel(const uint32_t *__restrict__ part, ComputeParams p,
                                                          OutT *__restrict__ out_pos, OutT *__restrict__ out_neg,
                                                          OutT *__restrict__ out_diff)
{
    const long total = (long)p.O * p.M;
    const long plane = (long)p.splits * p.O_pad * p.M;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const int o = (int)(i / p.M), m = (int)(i - (long)o * p.M);
        uint32_t sp = 0, sn = 0;
        for (int s = 0; s < p.splits; s++) {
            const long idx = ((long)s * p.O_pad + o) * p.M + m;
            if (WIDE) { sp += part[idx]; sn += part[plane + idx]; }
            else { const uint32_t v = part[idx]; sp += v & 0xffffu; sn += v >> 16; }
        }
        long idx;
        if (p.out_channels_last) idx = (long)m * p.O + o;
        else { const int n = m / p.HoWo, r = m - n * p.HoWo; idx = ((long)n * p.O + o) * p.HoWo + r; }
        const OutT vp = (OutT)sp, vn = (OutT)sn; // int16: wraps
        if (out_pos) out_pos[idx] = vp;
        if (out_neg) out_neg[idx] = vn;
        if (out_diff) out_diff[idx] = (OutT)(vp - vn);
    }
}

// Generic fallback for kernel widths without a tuned instance: one output per thread, runtime loops.
__global__ __launch_bounds__(256) void sc_compute_generic_kernel(const uint32_t *__restrict__ A,
                                                                 const uint32_t *__restrict__ Wst, ComputeParams p,
                                                                 int KW, int ZC, int16_t *__restrict__ out_pos,
                                                                 int16_t *__restrict__ out_neg,
                                                                 int16_t *__restrict__ out_diff)
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
    }
}

// ---- host side ---------------------------------------------------------------------------------
template <int KW, int ZC, int PX, int OT, bool WIDE>
static int launch_compute(const uint32_t *A, const uint32_t *Wst, ComputeParams p, uint32_t *part, int16_t *out_pos,
                          int16_t *out_neg, int16_t *out_diff, hipStream_t stream)
{
    p.m_tiles = ceil_div(p.M, CB * PX);
    p.o_tiles = p.O_pad / OT;
    const long blocks = (long)p.m_tiles * p.o_tiles * p.splits;
    REXSC_CHECK_ARG(blocks < (1L << 30), "SC compute: grid too large (%ld blocks)", blocks);
    const int grid = (int)align_up((size_t)blocks, 8);
    static char name[64] = "";
    if (!name[0]) snprintf(name, sizeof(name), "sc_compute<%d,%d,%d,%d,%d>", KW, ZC, PX, OT, (int)WIDE);
    // algorithmic lane-ops: (and + popcount-accumulate) x 2 polarities per 32-channel word
    ProfScope prof(name, 4.0 * p.M * p.O * p.KH * KW * p.Z * p.n_slots, stream);
    hipLaunchKernelGGL((sc_compute_kernel<KW, ZC, PX, OT, WIDE>), dim3(grid), dim3(CB), 0, stream, A, Wst, p, part,
                       out_pos, out_neg, out_diff);
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
               uint32_t *part, int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, hipStream_t stream)
{
    const int px = p.px;
#define REXSC_INST(KW_, ZC_)                                                                                      \
    if (KW == KW_ && ZC == ZC_) {                                                                                 \
        if (px == 2) return launch_compute<KW_, ZC_, 2, 16, false>(A, Wst, p, part, out_pos, out_neg, out_diff, stream); \
        return launch_compute<KW_, ZC_, 1, 16, false>(A, Wst, p, part, out_pos, out_neg, out_diff, stream);      \
    }
    if (wide) {
        REXSC_CHECK_ARG(KW == 1 && (ZC == 4 || ZC == 8), "wide accumulation is only built for 1x1 / linear shapes");
        if (ZC == 4) return launch_compute<1, 4, 1, 16, true>(A, Wst, p, part, out_pos, out_neg, out_diff, stream);
        return launch_compute<1, 8, 1, 16, true>(A, Wst, p, part, out_pos, out_neg, out_diff, stream);
    }
    REXSC_INST(1, 1) REXSC_INST(1, 2) REXSC_INST(1, 4) REXSC_INST(1, 8)
    REXSC_INST(3, 1) REXSC_INST(3, 2) REXSC_INST(3, 4)
    REXSC_INST(5, 1) REXSC_INST(5, 2)
    REXSC_INST(7, 1) REXSC_INST(7, 2)
#undef REXSC_INST
    set_error("SC compute: no kernel instance for KW=%d ZC=%d", KW, ZC);
    return REXSC_ERR_INVALID;
}

int sc_compute_generic(const uint32_t *A, const uint32_t *Wst, const ComputeParams &p, int KW, int ZC,
                       int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
    ProfScope prof("sc_compute_generic", 4.0 * p.M * p.O * p.KH * KW * p.Z * p.n_slots, stream);
    hipLaunchKernelGGL(sc_compute_generic_kernel, dim3(grid), dim3(256), 0, stream, A, Wst, p, KW, ZC, out_pos,
                       out_neg, out_diff);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sc_finalize_i16(const uint32_t *part, const ComputeParams &p, int16_t *out_pos, int16_t *out_neg,
                    int16_t *out_diff, hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    ProfScope prof("sc_finalize_i16", (double)total * (4.0 * p.splits + 4.0), stream);
    hipLaunchKernelGGL((sc_finalize_kernel<false, int16_t>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                       out_neg, out_diff);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

int sc_finalize_i32(const uint32_t *part, const ComputeParams &p, bool wide, int32_t *out_pos, int32_t *out_neg,
                    hipStream_t stream)
{
    const long total = (long)p.O * p.M;
    const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    ProfScope prof("sc_finalize_i32", (double)total * (4.0 * p.splits * (wide ? 2 : 1) + 8.0), stream);
    if (wide)
        hipLaunchKernelGGL((sc_finalize_kernel<true, int32_t>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                           out_neg, (int32_t *)nullptr);
    else
        hipLaunchKernelGGL((sc_finalize_kernel<false, int32_t>), dim3(grid), dim3(256), 0, stream, part, p, out_pos,
                           out_neg, (int32_t *)nullptr);
    REXSC_CHECK_HIP(hipGetLastError());
    return REXSC_OK;
}

} // namespace rexsc
