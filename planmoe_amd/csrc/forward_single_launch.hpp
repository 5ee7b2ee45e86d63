// Host side of the one-launch forward kernel.  The kernel is instantiated for sixteen row lengths (NMMA =
// model_dim / 256 = 1 .. 16), two score dtypes, two expert bounds and one to four rounds of 16 tokens: 256
// kernels, most of the library's compile time.  So each row length is a translation unit of its own
// (forward_single_m.hip, compiled once per NMMA) that exports one function, fs_launch_m<NMMA>, and they
// compile side by side; forward.hip picks the function by model_dim.
#pragma once
#include "forward_single.hpp"

namespace pm {

struct FsLaunch {
    int rounds, groups;
    hipStream_t st;
    const void *x, *wg;
    const float *bias;
    int samples, experts, k, normalize, capacity;
    int32_t *indices, *locations;
    void *gates;
    int64_t stride;
    void *logits_out, *scores_out;
    float *l_aux;
    int32_t *counts;
    uint8_t *codes;
    void *bias_out, *scale_out, *ws;
    unsigned long long salt;
    int spin_limit;
    int32_t *gave_up;
    int fp32_gate;
    bool ask_only;          // do not launch: only say whether the launch would go ahead
};

// 0: launched (or, with ask_only, would be); 2: more work-groups than are resident at once (nothing was enqueued)
#define PM_FS_DECLARE(n) int fs_launch_m##n(const FsLaunch &a);
PM_FS_DECLARE(1) PM_FS_DECLARE(2) PM_FS_DECLARE(3) PM_FS_DECLARE(4) PM_FS_DECLARE(5) PM_FS_DECLARE(6) PM_FS_DECLARE(7) PM_FS_DECLARE(8)
PM_FS_DECLARE(9) PM_FS_DECLARE(10) PM_FS_DECLARE(11) PM_FS_DECLARE(12) PM_FS_DECLARE(13) PM_FS_DECLARE(14) PM_FS_DECLARE(15) PM_FS_DECLARE(16)
#undef PM_FS_DECLARE

// Whether every work-group of the launch is resident at once (asked of the runtime once per kernel and device).
template <int SDT, int CAP, int NMMA, int ROUNDS>
static bool single_fits(int groups)
{
    static int resident[STATIC_SCRATCH_DEVICES_MAX] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_SCRATCH_DEVICES_MAX) return false;
    if (resident[dev] == 0) {
        int per_cu = 0, cus = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, forward_single_kernel<SDT, CAP, NMMA, ROUNDS>,
                                                         FS_THREADS, 0) != hipSuccess) per_cu = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 0;
        resident[dev] = per_cu * cus > 0 ? per_cu * cus : -1;
    }
    return groups <= resident[dev];
}

template <int SDT, int CAP, int NMMA>
static int launch_single(const FsLaunch &a)
{
#define PM_FS(ROUNDS)                                                                                              \
    do {                                                                                                           \
        if (!single_fits<SDT, CAP, NMMA, ROUNDS>(a.groups)) return 2;                                              \
        if (a.ask_only) return 0;                                                                                  \
        forward_single_kernel<SDT, CAP, NMMA, ROUNDS><<<a.groups, FS_THREADS, 0, a.st>>>(                          \
            (const uint4 *)a.x, (const uint4 *)a.wg, a.bias, a.samples, a.experts, a.k, a.normalize, a.capacity,   \
            a.indices, a.locations, a.gates, a.stride, a.logits_out, a.scores_out, a.l_aux, a.counts, a.codes,     \
            a.bias_out, a.scale_out, a.ws, a.salt, a.spin_limit, a.gave_up);                                       \
    } while (0)
    switch (a.rounds) {
    case 1: PM_FS(1); break;
    case 2: PM_FS(2); break;
    case 3: PM_FS(3); break;
    default: PM_FS(4); break;
    }
#undef PM_FS
    return 0;
}

// the definition of fs_launch_m<NMMA>: scores in fp32 or bf16, expert bound 8 or 16
#define PM_FS_DEFINE(NMMA)                                                                                         \
    int fs_launch_m##NMMA(const FsLaunch &a)                                                                       \
    {                                                                                                              \
        if (a.fp32_gate) return a.experts <= 8 ? launch_single<PLANMOE_F32, 8, NMMA>(a)                            \
                                               : launch_single<PLANMOE_F32, 16, NMMA>(a);                          \
        return a.experts <= 8 ? launch_single<PLANMOE_BF16, 8, NMMA>(a) : launch_single<PLANMOE_BF16, 16, NMMA>(a); \
    }

} // namespace pm
