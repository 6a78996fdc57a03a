// Stream generator interface (internal).
#pragma once
#include "rexsc_common.h"

namespace rexsc {

// Activations [N][C][H][W] (or NHWC) -> stream words A[slot][n][zg][pp][zc], where
// pp = yp*Wp + xp runs over the zero-PADDED plane and (zg, zc) split the channel words
// (32 channels per word, ZC words per chunk, ZG chunks).
struct ActGeom {
    int N, C, H, W;
    int Hp, Wp, pad_h, pad_w;
    int channels_last;
    int ZC, ZG;
    long slot_stride;         // words per slot: N*ZG*Hp*Wp*ZC
    int seed_cmul, seed_pmul; // seed index = c*seed_cmul + pp*seed_pmul
};

// Weights [O][C][KH][KW] (or OHWI) -> Wst[slot][ky][zg][o][pol][kx][zc], o padded to O_pad.
struct WeightGeom {
    int O, C, KH, KW;
    int channels_last;
    int ZC, ZG, O_pad;
    // seed index += o * seed_omul.  0 everywhere but in the reference's legacy linear simulation with one generator
    // per weight (utils_functional.py:996-998), where the index runs over the whole tensor: o * C + c.
    int seed_omul;
};

// Words of LFSR state-plane table the bit-sliced activation generator needs for this problem, or 0
// when the ballot generator is the better choice.  geo.N and geo.slot_stride must describe a full batch chunk.
size_t sng_act_table_words(const ActGeom &geo, const GenParams &gp);
// table != nullptr selects the bit-sliced generator; the table must have been built by sng_weights()
// for the same (geo, gp) earlier on the same stream.
int sng_activations(const float *x, uint32_t *A, const uint32_t *table, const ActGeom &geo, const GenParams &gp,
                    hipStream_t stream);
// act_table != nullptr: the launch also builds the activation generator's state-plane table
// (sng_act_table_words() words) for (*act_geo, *act_gp).
// guard != nullptr: every block first reads *guard and returns at once unless it equals `epoch`
// (weights_snapshot() writes it): streams and table of an earlier launch stay as they are.
int sng_weights(const float *w, uint32_t *Wst, const WeightGeom &geo, const GenParams &gp, uint32_t *act_table,
                const ActGeom *act_geo, const GenParams *act_gp, hipStream_t stream,
                const unsigned long long *guard = nullptr, unsigned long long epoch = 0);

// Device-side change detection for weight streams kept across calls: compares the n floats of w bit for bit with
// `snapshot`, copies what differs, and stores `epoch` into *flag when anything did (or when force != 0, which also
// makes the snapshot a plain copy).  *flag is left alone otherwise.
int weights_snapshot(const float *w, float *snapshot, size_t n, unsigned long long *flag, unsigned long long epoch,
                     int force, hipStream_t stream);

// Tap folding for layers whose whole receptive field fits one word (C*KH*KW <= 32, one 32-channel word per pixel):
//   A2[slot][m]      = OR over taps of A[slot][n][yo*s0+ky][xo*s1+kx] << ((ky*KW+kx)*C),  m = (n, yo, xo)
//   W2[slot][o][pol] = OR over taps of Wst[slot][ky][o][pol][kx]      << ((ky*KW+kx)*C)
// so that popcount(A2 & W2) is the sum over the taps of popcount(A & Wst).
int fold_activation_streams(const uint32_t *A, uint32_t *A2, int n_slots, long a_stride, long a2_stride, int N, int Hp, int Wp,
                            int Ho, int Wo, int KH, int KW, int s0, int s1, int C, hipStream_t stream);
int fold_weight_streams(const uint32_t *Wst, uint32_t *W2, int n_slots, int KH, int KW, int O_pad, int C, hipStream_t stream,
                        const unsigned long long *guard = nullptr, unsigned long long epoch = 0);

} // namespace rexsc
