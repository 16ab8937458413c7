// Workgroup -> macro-tile rasterisation, shared by the GEMM kernels (device)
// and fo_raster_hint (host) so that both sides agree on the issue order.
//
// MI355X dispatches workgroup i of a grid to XCD i % 8, and every XCD has its
// own L2.  The unit of the map is a block of kGroupM x 4 macro tiles: the 32
// workgroups one XCD runs at a time, which share their A and B panels in that
// L2.  Units are ordered band by band (a band = kGroupM rows of macro tiles,
// all columns), and the eight units of one hardware wave (256 workgroups) go to
// the eight XCDs.  So the XCDs of a wave work on the same A rows, which the
// memory-side cache then fetches from HBM once for all of them (with each XCD
// walking a strip of its own the same kernel ran 2 % longer on operands that
// were not cached), and a wave finishes whole rows of the output.
#pragma once

#if defined(__HIPCC__)
#define FO_HD __host__ __device__ inline
#else
#define FO_HD inline
#endif

namespace fo {

constexpr int kXcds = 8;
constexpr int kGroupM = 8;   // rows of a unit
constexpr int kUnitN = 4;    // columns of a unit: kGroupM * kUnitN = 32 workgroups, one XCD's share of a wave

struct TileCoord {
    int m, n;
};

// pid in [0, GM*GN) -> macro tile coordinate.
FO_HD TileCoord raster_map(int pid, int GM, int GN) {
    const int total = GM * GN;
    const int xcd = pid % kXcds, local = pid / kXcds;
    constexpr int kUnit = kGroupM * kUnitN, kWave = kXcds * kUnit;
    // Position in unit order: workgroup `local` of XCD `xcd` is workgroup local % 32 of that XCD's
    // unit in wave local / 32.  The workgroups behind the last whole wave keep their own number.
    const int whole = total / kWave * kWave;
    const int pos = pid < whole ? ((local / kUnit) * kXcds + xcd) * kUnit + local % kUnit : pid;
    // Position -> tile: bands of kGroupM rows (the last may be lower), in a band blocks of kUnitN
    // columns (the last may be narrower), in a block column by column.
    const int band_tiles = kGroupM * GN;
    const int band = pos / band_tiles;
    const int first_m = band * kGroupM;
    const int rows = (GM - first_m < kGroupM) ? (GM - first_m) : kGroupM;
    const int in_band = pos - band * band_tiles;
    const int block = in_band / (rows * kUnitN);
    const int in_block = in_band - block * rows * kUnitN;
    TileCoord c;
    c.m = first_m + in_block % rows;
    c.n = block * kUnitN + in_block / rows;
    return c;
}

}  // namespace fo
