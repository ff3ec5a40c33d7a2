// Library-level entry points of the C ABI: version, error strings, and which kernel families were taken.
#include <atomic>

#include "common.h"

namespace
{
std::atomic<uint64_t> g_routes{0};
static_assert(REPDL_ROUTE_COUNT <= 64, "one bit per route");
const char *const ROUTE_NAMES[REPDL_ROUTE_COUNT] = {
    "mm_128", "mm_128_tall", "mm_64_four_buffers", "mm_64_three_buffers", "mm_64_movers", "mm_64_wide_k", "mm_64_deep", "mm_64_quad", "mm_32", "mm_64x32",
    "mm_unaligned_128", "mm_unaligned_64_movers", "mm_unaligned_64", "mm_unaligned_quad", "mm_unaligned_32", "mm_fma",
    "conv_patch_16", "conv_patch_4", "conv_patch_16_wide", "conv_patch_4_wide", "conv_point", "conv_point_mm", "conv_padded_64_half", "conv_padded_64", "conv_padded_128",
    "conv_gather_64", "conv_gather_128", "conv_im2col", "dgrad_point_scatter", "dgrad_residues",
    "wgrad_point_gather", "wgrad_product", "wgrad_chain", "wgrad_fma",
    "sum_row_walk", "sum_chains", "sum_chains_rounds", "sum_column_walk", "sum_serial",
    "loss_onchip", "loss_row_per_wave"};
} // namespace

void repdl_route_note(int route)
{
    if (route >= 0 && route < REPDL_ROUTE_COUNT && !repdl_ws_dry())
        g_routes.fetch_or((uint64_t)1 << route, std::memory_order_relaxed);
}

REPDL_API uint64_t repdl_hip_routes_taken(int reset)
{
    return reset ? g_routes.exchange(0, std::memory_order_relaxed) : g_routes.load(std::memory_order_relaxed);
}

REPDL_API const char *repdl_hip_route_name(int route) { return route >= 0 && route < REPDL_ROUTE_COUNT ? ROUTE_NAMES[route] : nullptr; }

REPDL_API int repdl_hip_abi_version(void) { return 1; }

REPDL_API const char *repdl_hip_error_string(int code)
{
    switch (code)
    {
    case REPDL_OK:
        return "success";
    case REPDL_E_ARG:
        return "repdl_hip: invalid argument (null pointer, negative or oversized extent)";
    case REPDL_E_UNSUPPORTED:
        return "repdl_hip: unsupported combination of arguments";
    case REPDL_E_WORKSPACE:
        return "repdl_hip: workspace missing or too small";
    case REPDL_E_TOO_LARGE:
        return "repdl_hip: input exceeds the fixed capacity of this entry point (it allocates nothing; see its *_max_n)";
    default:
        break;
    }
    if (code > 0)
        return hipGetErrorString((hipError_t)code);
    return "repdl_hip: unknown error code";
}
