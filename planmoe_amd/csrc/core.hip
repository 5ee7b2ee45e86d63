// Error state, ABI version and the host-only capacity arithmetic.
#include "common.hpp"
#include <cmath>

namespace pm {

static thread_local std::string g_error;

void set_error(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
}

int fail(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
    return 1;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *p, size_t n, uint32_t value)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) p[i] = value;
}

void fill_u32(uint32_t *p, size_t n, uint32_t value, hipStream_t stream)
{
    if (n == 0) return;
    const unsigned grid = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    fill_u32_kernel<<<grid, 256, 0, stream>>>(p, n, value);
}

} // namespace pm

extern "C" int planmoe_abi_version(void) { return PLANMOE_ABI_VERSION; }

extern "C" const char *planmoe_last_error(void) { return pm::g_error.c_str(); }

// capacity = k * int(cf * ceil(T / E)), then rounded up to a multiple of `alignment`
extern "C" int planmoe_capacity(int samples, int experts, int top_k, double capacity_factor,
                                int alignment, int *capacity_host)
{
    PM_REQUIRE(capacity_host, "planmoe_capacity: capacity_host is NULL");
    PM_REQUIRE(samples >= 0 && experts >= 1 && top_k >= 1, "planmoe_capacity: bad shape");
    PM_REQUIRE(capacity_factor > 0, "planmoe_capacity: capacity_factor must be > 0 "
               "(the data-dependent capacity of capacity_factor <= 0 is computed by the caller)");
    PM_REQUIRE(alignment >= 1, "planmoe_capacity: alignment must be >= 1");
    const int k = top_k < experts ? top_k : experts;
    const int per_expert = (samples + experts - 1) / experts;
    long long cap = (long long)k * (long long)(capacity_factor * per_expert);
    const long long rem = cap % alignment;
    if (rem > 0) cap += alignment - rem;
    PM_REQUIRE(cap < (1ll << 31), "planmoe_capacity: capacity overflows int32");
    *capacity_host = (int)cap;
    return 0;
}
