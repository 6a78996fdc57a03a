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
};

int sng_activations(const float *x, uint32_t *A, const ActGeom &geo, const GenParams &gp, hipStream_t stream);
int sng_weights(const float *w, uint32_t *Wst, const WeightGeom &geo, const GenParams &gp, hipStream_t stream);

} // namespace rexsc
