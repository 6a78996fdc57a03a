// Shared host/device helpers of librexsc (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "rexsc.h"

namespace rexsc {

// ---- error reporting ---------------------------------------------------------------------
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define REXSC_CHECK_ARG(cond, ...)                 \
    do {                                           \
        if (!(cond)) {                             \
            ::rexsc::set_error(__VA_ARGS__);       \
            return REXSC_ERR_INVALID;              \
        }                                          \
    } while (0)

#define REXSC_CHECK_HIP(expr)                                                              \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            ::rexsc::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),      \
                               __FILE__, __LINE__);                                        \
            return REXSC_ERR_HIP;                                                          \
        }                                                                                  \
    } while (0)

// A descriptor carries the size its caller's header gives it: anything else was built against another ABI.
#define REXSC_CHECK_DESC(d, type)                                                                                       \
    do {                                                                                                                \
        REXSC_CHECK_ARG((d) != nullptr, "null descriptor");                                                             \
        REXSC_CHECK_ARG((d)->struct_size == (int32_t)sizeof(type),                                                      \
                        #type ": struct_size %d, this library (ABI %d) expects %zu -- caller and library were built "   \
                        "from different headers", (int)(d)->struct_size, REXSC_ABI_VERSION, sizeof(type));             \
    } while (0)

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ---- LFSR ------------------------------------------------------------------------------------
// Fibonacci LFSRs of 3..8 bits; taps per width as in the reference CPU extension
// (sc_cpu.hpp:49-137): 3:{2,1} 4:{3,2} 5:{4,2} 6:{5,4} 7:{6,5} 8:{7,5,4,3}.
// Flavours (the `acc` argument): 0 plain; 1 ("_acc") splices the zero state into the cycle
// (1 -> 0 -> 2), sc_cpu.hpp:54-64; 2 XNOR feedback, the generator the reference's CUDA conv kernels
// select with xnor = true (sc_device.cuh:108-286): the complemented feedback bit is shifted in, the
// cycle runs over 0 .. 2^lb-2 and the all-ones state is its fixed point.
enum { LFSR_PLAIN = 0, LFSR_ACC = 1, LFSR_XNOR = 2 };
__host__ __device__ inline int lfsr_step(int lb, int acc, int v)
{
    if (acc == LFSR_ACC) {
        if (v == 1) return 0;
        if (v == 0) return 2;
    }
    int fb;
    switch (lb) {
    case 3: fb = ((v >> 2) ^ (v >> 1)) & 1; break;
    case 4: fb = ((v >> 3) ^ (v >> 2)) & 1; break;
    case 5: fb = ((v >> 4) ^ (v >> 2)) & 1; break;
    case 6: fb = ((v >> 5) ^ (v >> 4)) & 1; break;
    case 7: fb = ((v >> 6) ^ (v >> 5)) & 1; break;
    default: fb = ((v >> 7) ^ (v >> 5) ^ (v >> 4) ^ (v >> 3)) & 1; break;
    }
    if (acc == LFSR_XNOR) fb = 1 - fb;
    return fb + 2 * (v & ((1 << (lb - 1)) - 1));
}

// Stream-length -> LFSR width, with the reference's fall-through for 2/4/8
// (sc_conv.cpp:335-360).  -1 if unsupported.
inline int lfsr_bits(int bit_length, int lfsr_length)
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

// The LFSR state sequence is a fixed cycle, so the state reached t steps after seed s is
// SEQ[(INV[s] + t) mod period].  SeqTable holds, for one (width, flavour):
//   seq[i]  = state at cycle position i, unrolled to SEQ_LEN entries (no modulo needed for
//             position + cycle < SEQ_LEN),
//   inv[s]  = cycle position of state s.
constexpr int SEQ_LEN = 1280; // >= 256 (max period) + 1024 (max stream cycles)
constexpr int MAX_CYCLES = 1024;
struct SeqTable {
    uint8_t seq[SEQ_LEN];
    uint8_t inv[256];
};
// table index for (lb in 3..8, flavour in 0..2)
constexpr int N_SEQ_TABLES = 18;
__host__ __device__ inline int seq_index(int lb, int acc) { return (lb - 3) * 3 + acc; }

// Device address of the per-device sequence tables (built on first use).
int get_seq_tables(const SeqTable **tables, hipStream_t stream);

// ---- stream-generation geometry --------------------------------------------------------------
// Parameters of one stream generator launch.  A stream "slot" s carries the operand's LFSR
// cycle cyc(s) = (s / slot_div) * slot_mul + (s % slot_mod): activations use
// (g*g, g, g) and weights (g, 1, 1) for gen_config g (sc_conv.cpp:127-130, 195-197).
struct GenParams {
    int lb, acc, period;             // LFSR width, flavour (LFSR_*), cycle length: 2^lb-1 (2^lb for LFSR_ACC)
    int seed_mod;                    // 2^lb - 1: seeds are (index % seed_mod) + seed_off
    int seed_off;                    // 1; 0 for LFSR_XNOR, whose cycle includes state 0 (sc_cuda_conv.cu:55-56,139)
    int scale;                       // S: float operands are multiplied by S
    int n_slots;                     // slots to generate
    int slot_div, slot_mul, slot_mod;
    int total_width, load_width, load_wait; // progressive loading
    int prog;                        // 0 when the truncation shift is 0 for every cycle
    int seed_add;                    // constant added to the seed index: 13 for weights (sc_cpu.hpp:10-11), 0 for activations
    // Operand quantisation: q = ceil(clamp(x * scale, 0, clamp_hi)), clamp_hi = scale - 1 (sc_conv.cpp:318-320).
    // legacy != 0 is the rule of the reference's pure-torch simulation `linear_generic`
    // (utils_functional.py:980-995, 1022-1024): the product is rounded to binary16 first, clamp_hi is set by the
    // caller and may reach `scale`, a value above every LFSR state ("always one").
    int legacy;
    float clamp_hi;
    float sign;                      // weights only: operand multiplied by +1 / -1 before the split into polarities
    // k > 0: the operand first goes through the layers' fake quantisation with prec = k - 1
    // (clamp(round(x * 2^prec), +-(2^prec - 1)) / 2^prec, utils_functional.py:93-104); 0: taken as it is
    int fake_quant;
};

__host__ __device__ inline int slot_cycle(const GenParams &g, int s)
{
    return (s / g.slot_div) * g.slot_mul + (s % g.slot_mod);
}

// Truncation shift of cycle t (sc_conv.cpp:107-115).
__host__ __device__ inline int prog_shift(const GenParams &g, int t)
{
    int cur = (t / g.load_wait + 1) * g.load_width - 1;
    if (cur > g.total_width) cur = g.total_width;
    return g.total_width - cur;
}

} // namespace rexsc
