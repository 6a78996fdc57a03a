// SC compute kernel interface (internal).
#pragma once
#include "rexsc_common.h"

namespace rexsc {

struct ComputeParams {
    int M;            // output pixels: N*Ho*Wo (linear: B)
    int HoWo, Wo;     // output plane geometry
    int Hp, Wp;       // padded input plane
    int s0, s1;       // stride along h / w
    int KH, ZG;       // kernel rows, channel chunks
    int Z;            // stream words per pixel actually carrying channels: ceil(C/32)
    long a_slot_stride; // activation words per slot
    int O, O_pad;
    int n_slots;      // slots accumulated
    int splits, slots_per_split;
    uint32_t nn;      // n_sat | n_sat << 16
    int mode;         // 0: min(count, n_sat); 1: count >= n_sat
    int direct;       // 1: the compute kernel writes the int16 outputs itself
    int part_narrow;  // 1: split partials are stored as uint16 (pos | neg << 8): both sums of a split fit 8 bits
    int out_channels_last;
    int px;           // pixels per lane (1 or 2)
    int ns;           // waves per block; they split the slots of the block among themselves
    int ot;           // output channels per block tile
    float inv_L;      // 1 / bit_length: scale of the optional float output
    int m_tiles, o_tiles; // filled by the launcher
    int vec_out;          // filled by the launcher: channels-last results may leave as 8-byte stores
};

int sc_compute_tile_ot();
bool sc_compute_has_instance(int KW, int ZC);
// out_value (optional, conv only): float32 pos / L - neg / L in the layout of the int16 outputs
int sc_compute(const uint32_t *A, const uint32_t *Wst, const ComputeParams &p, int KW, int ZC, bool wide,
               uint32_t *part, int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, float *out_value, hipStream_t stream);
int sc_compute_generic(const uint32_t *A, const uint32_t *Wst, const ComputeParams &p, int KW, int ZC,
                       int16_t *out_pos, int16_t *out_neg, int16_t *out_diff, float *out_value, hipStream_t stream);
int sc_finalize_i16(const uint32_t *part, const ComputeParams &p, int16_t *out_pos, int16_t *out_neg,
                    int16_t *out_diff, float *out_value, hipStream_t stream);
int sc_finalize_i32(const uint32_t *part, const ComputeParams &p, bool wide, int32_t *out_pos, int32_t *out_neg,
                    hipStream_t stream);

} // namespace rexsc
