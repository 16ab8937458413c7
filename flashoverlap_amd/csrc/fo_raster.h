// Workgroup -> macro-tile rasterisation, shared by the GEMM kernels (device)
// and fo_raster_hint (host) so that both sides agree on the issue order.
//
// MI355X dispatches workgroup i of a grid to XCD i % 8, and every XCD has its
// own L2.  The map below first gives each XCD one contiguous range of
// "logical" tile ids, then walks that range in column strips of `kGroupM`
// macro-tile rows, so the 32 workgroups an XCD runs at a time cover a compact
// kGroupM x (32/kGroupM) block of the output and share A/B panels in that L2.
#pragma once

#if defined(__HIPCC__)
#define FO_HD __host__ __device__ inline
#else
#define FO_HD inline
#endif

namespace fo {

constexpr int kXcds = 8;
constexpr int kGroupM = 8;

struct TileCoord {
    int m, n;
};

// pid in [0, GM*GN) -> macro tile coordinate.
FO_HD TileCoord raster_map(int pid, int GM, int GN) {
    const int total = GM * GN;
    // XCD remap: pid -> logical id, XCD x owns a contiguous logical range.
    const int q = total / kXcds, r = total % kXcds;
    const int xcd = pid % kXcds, local = pid / kXcds;
    const int lid = (xcd < r) ? xcd * (q + 1) + local : r * (q + 1) + (xcd - r) * q + local;
    // Strips of kGroupM rows, column-major inside a strip.
    const int per_strip = kGroupM * GN;
    const int strip = lid / per_strip;
    const int first_m = strip * kGroupM;
    const int rows = (GM - first_m < kGroupM) ? (GM - first_m) : kGroupM;
    const int in_strip = lid - strip * per_strip;
    TileCoord c;
    c.m = first_m + in_strip % rows;
    c.n = in_strip / rows;
    return c;
}

}  // namespace fo
