#include "profile.h"

#include <mutex>
#include <string.h>
#include <vector>

namespace rexsc {
namespace {
struct Rec { const char *name; double work; hipEvent_t start, stop; };
std::mutex g_mu;
bool g_on = false;
std::vector<Rec> g_recs;
} // namespace

ProfScope::ProfScope(const char *name, double work, hipStream_t s) : slot(-1), stream(s)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_on) return;
    Rec r{name, work, nullptr, nullptr};
    if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
    (void)hipEventRecord(r.start, stream);
    g_recs.push_back(r);
    slot = (int)g_recs.size() - 1;
}

ProfScope::~ProfScope()
{
    if (slot < 0) return;
    std::lock_guard<std::mutex> lk(g_mu);
    if (slot < (int)g_recs.size()) (void)hipEventRecord(g_recs[slot].stop, stream);
}

} // namespace rexsc

using namespace rexsc;

extern "C" int rexsc_profile_begin(void)
{
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto &r : g_recs) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
    g_recs.clear();
    g_on = true;
    return REXSC_OK;
}

extern "C" int rexsc_profile_end(rexsc_profile_record *out, int max_records)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_on = false;
    int n = 0;
    for (auto &r : g_recs) {
        float ms = 0.f;
        if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            // aggregate by kernel name
            int k = 0;
            for (; k < n; k++) if (strcmp(out[k].name, r.name) == 0) break;
            if (k == n) {
                if (n >= max_records) continue;
                memset(&out[n], 0, sizeof(out[n]));
                strncpy(out[n].name, r.name, sizeof(out[n].name) - 1);
                n++;
            }
            out[k].calls += 1;
            out[k].total_ms += ms;
            out[k].total_work += r.work;
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    g_recs.clear();
    return n;
}

// ---- integer VALU peak probe ---------------------------------------------------------------------
// A register-only kernel issuing the instruction pair of the SC compute kernel exactly as that kernel issues
// it (v_and_b32 with a scalar operand, s_nop 0, v_bcnt_u32_b32 with its accumulate input; mode 1:
// v_and_or_b32, the OR-1 form) on 16 independent accumulators per lane, eight waves per SIMD, no memory
// traffic inside the timed loop.  What it sustains is the roof the AND/popcount kernels are measured against
// on the machine at hand.  Modes 2..4 document why the pair is issued that way: 2 is the pair without the
// scalar instruction between its halves, 3 a v_and_b32 on vector registers only, 4 a v_bcnt_u32_b32 alone.
namespace rexsc {
namespace {
static __device__ uint32_t g_probe_sink[64];

// operands: %0..%15 accumulators, %16 scratch, %17..%20 activation words, %21..%24 weight words (SGPRs)
#define REXSC_PROBE_PAIR(C, A, W) \
    "v_and_b32 %16, %" #W ", %" #A "\n\ts_nop 0\n\tv_bcnt_u32_b32 %" #C ", %16, %" #C "\n\t"
#define REXSC_PROBE_ANDOR(C, A, W) "v_and_or_b32 %" #C ", %" #A ", %" #W ", %" #C "\n\t"
#define REXSC_PROBE_PAIR_BARE(C, A, W) "v_and_b32 %16, %" #W ", %" #A "\n\tv_bcnt_u32_b32 %" #C ", %16, %" #C "\n\t"
#define REXSC_PROBE_AND(C, A, W) "v_and_b32 %" #C ", %" #A ", %" #C "\n\t"
#define REXSC_PROBE_BCNT(C, A, W) "v_bcnt_u32_b32 %" #C ", %" #A ", %" #C "\n\t"
#define REXSC_PROBE_ROW(OP, A0, A1, A2, A3)                                                        \
    OP(0, A0, 21) OP(1, A1, 22) OP(2, A2, 23) OP(3, A3, 24) OP(4, A0, 21) OP(5, A1, 22) OP(6, A2, 23) OP(7, A3, 24)       \
    OP(8, A0, 21) OP(9, A1, 22) OP(10, A2, 23) OP(11, A3, 24) OP(12, A0, 21) OP(13, A1, 22) OP(14, A2, 23) OP(15, A3, 24)
#define REXSC_PROBE_BODY(OP) \
    REXSC_PROBE_ROW(OP, 17, 18, 19, 20) REXSC_PROBE_ROW(OP, 18, 19, 20, 17) REXSC_PROBE_ROW(OP, 19, 20, 17, 18) REXSC_PROBE_ROW(OP, 20, 17, 18, 19)

template <int MODE>
__global__ __launch_bounds__(256) void valu_probe_kernel(int iters, uint32_t w0, uint32_t seed)
{
    uint32_t c[16], a[4];
#pragma unroll
    for (int i = 0; i < 16; i++) c[i] = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) a[i] = seed * (threadIdx.x + 1) + i * 0x9E3779B9u;
    const uint32_t w1 = w0 * 3u + 1u, w2 = w0 ^ 0x55555555u, w3 = ~w0;
    (void)w1; (void)w2; (void)w3; // only the device pass uses them
    for (int it = 0; it < iters; it++) {
        // 64 slots per iteration in ONE asm statement: between separate statements the compiler would put
        // scalar instructions of its own, and the pair's rate depends on exactly one scalar instruction per pair
#if defined(__HIP_DEVICE_COMPILE__)
        uint32_t t;
#define REXSC_PROBE_OPERANDS                                                                                          \
    : "+v"(c[0]), "+v"(c[1]), "+v"(c[2]), "+v"(c[3]), "+v"(c[4]), "+v"(c[5]), "+v"(c[6]), "+v"(c[7]), "+v"(c[8]), "+v"(c[9]), \
      "+v"(c[10]), "+v"(c[11]), "+v"(c[12]), "+v"(c[13]), "+v"(c[14]), "+v"(c[15]), "=&v"(t)                            \
    : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "s"(w0), "s"(w1), "s"(w2), "s"(w3)
        if (MODE == 0) asm volatile(REXSC_PROBE_BODY(REXSC_PROBE_PAIR) REXSC_PROBE_OPERANDS);
        else if (MODE == 1) asm volatile(REXSC_PROBE_BODY(REXSC_PROBE_ANDOR) REXSC_PROBE_OPERANDS);
        else if (MODE == 2) asm volatile(REXSC_PROBE_BODY(REXSC_PROBE_PAIR_BARE) REXSC_PROBE_OPERANDS);
        else if (MODE == 3) asm volatile(REXSC_PROBE_BODY(REXSC_PROBE_AND) REXSC_PROBE_OPERANDS);
        else asm volatile(REXSC_PROBE_BODY(REXSC_PROBE_BCNT) REXSC_PROBE_OPERANDS);
#endif
    }
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) s ^= c[i];
    if (s == 0xDEADBEEFu && iters < 0) g_probe_sink[threadIdx.x & 63] = s; // keeps the chain live; never taken
}
} // namespace
} // namespace rexsc

extern "C" int rexsc_valu_probe(int mode, int iters, rexsc_stream_t stream_, double *ms_out, double *lane_ops_out)
{
    hipStream_t stream = (hipStream_t)stream_;
    // 100000 iterations of 64 slots are about 20 ms per launch: long enough for any measurement
    REXSC_CHECK_ARG(mode >= 0 && mode <= 4 && iters > 0 && iters <= 100000 && ms_out && lane_ops_out,
                    "valu probe: mode 0..4, 1 <= iters <= 100000");
    hipDeviceProp_t prop;
    int dev = 0;
    REXSC_CHECK_HIP(hipGetDevice(&dev));
    REXSC_CHECK_HIP(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount * 8; // 4 waves per block: 8 waves per SIMD
    struct Events { // destroyed on every way out
        hipEvent_t a = nullptr, b = nullptr;
        ~Events() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
    } ev;
    REXSC_CHECK_HIP(hipEventCreate(&ev.a));
    REXSC_CHECK_HIP(hipEventCreate(&ev.b));
    const hipEvent_t e0 = ev.a, e1 = ev.b;
    for (int rep = 0; rep < 2; rep++) { // the first launch warms the clocks up
        REXSC_CHECK_HIP(hipEventRecord(e0, stream));
        switch (mode) {
        case 0: hipLaunchKernelGGL(valu_probe_kernel<0>, dim3(blocks), dim3(256), 0, stream, iters, 0x0F0F3355u, 12345u); break;
        case 1: hipLaunchKernelGGL(valu_probe_kernel<1>, dim3(blocks), dim3(256), 0, stream, iters, 0x0F0F3355u, 12345u); break;
        case 2: hipLaunchKernelGGL(valu_probe_kernel<2>, dim3(blocks), dim3(256), 0, stream, iters, 0x0F0F3355u, 12345u); break;
        case 3: hipLaunchKernelGGL(valu_probe_kernel<3>, dim3(blocks), dim3(256), 0, stream, iters, 0x0F0F3355u, 12345u); break;
        default: hipLaunchKernelGGL(valu_probe_kernel<4>, dim3(blocks), dim3(256), 0, stream, iters, 0x0F0F3355u, 12345u); break;
        }
        REXSC_CHECK_HIP(hipGetLastError());
        REXSC_CHECK_HIP(hipEventRecord(e1, stream));
        REXSC_CHECK_HIP(hipEventSynchronize(e1));
    }
    float ms = 0.f;
    REXSC_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
    *ms_out = ms;
    // VALU instructions per lane: 64 slots per iteration, two instructions each for the pairs, one otherwise
    *lane_ops_out = (double)blocks * 256.0 * (double)iters * 64.0 * (mode == 0 || mode == 2 ? 2.0 : 1.0);
    return REXSC_OK;
}
