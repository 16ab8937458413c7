// Workgroup -> macro-tile rasterisation, shared by the GEMM kernels (device)
// and fo_raster_hint (host) so that both sides agree on the issue order.
//
// MI355X dispatches workgroup i of a grid to XCD i % 8, and every XCD has its
// own L2.  The unit of the map is a block of kGroupM x 4 macro tiles: the 32
// workgroups one XCD runs at a time, which share their A and B panels in that
// L2 (numbered row by row inside the block).  Units are ordered band by band (a band = kGroupM rows of macro tiles,
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

// Division by the column count without a divide instruction (the kernel does this once per
// workgroup, in front of its first memory access): n / d == (n * magic) >> 32 with
// magic = 2^32 / d + 1, exact while n * d < 2^32 (tile counts are far below that).
// (d = 1 has no such 32-bit magic; it is stored as 0.)
FO_HD unsigned raster_magic(int d) { return d == 1 ? 0u : (unsigned)(0x100000000ull / (unsigned)d) + 1u; }
FO_HD int raster_div(int n, unsigned magic) {
    return magic ? (int)(((unsigned long long)(unsigned)n * magic) >> 32) : n;
}

// pid in [0, GM*GN) -> macro tile coordinate; gn_magic = raster_magic(GN).
FO_HD TileCoord raster_map(int pid, int GM, int GN, unsigned gn_magic) {
    const int total = GM * GN;
    const int xcd = pid % kXcds, local = pid / kXcds;
    constexpr int kUnit = kGroupM * kUnitN, kWave = kXcds * kUnit;
    // Position in unit order: workgroup `local` of XCD `xcd` is workgroup local % 32 of that XCD's
    // unit in wave local / 32.  The workgroups behind the last whole wave keep their own number.
    const int whole = total / kWave * kWave;
    const int pos = pid < whole ? ((local / kUnit) * kXcds + xcd) * kUnit + local % kUnit : pid;
    // Position -> tile: bands of kGroupM rows (the last may be lower), in a band blocks of kUnitN
    // columns (the last may be narrower), in a block row by row.  (Row by row, not column by
    // column: the slots of the tiles that one output row crosses are then a few slots apart
    // inside a block and one block apart between blocks, where column by column they were 256
    // slots = 8 MiB apart, a stride at which the segments that reorder+RMSNorm gathers for a row
    // fall into few memory channels: that kernel ran 5-7 % longer.)
    const int band = raster_div(pos / kGroupM, gn_magic);     // pos / (kGroupM * GN)
    const int first_m = band * kGroupM;
    const int in_band = pos - band * kGroupM * GN;
    const int rows = GM - first_m >= kGroupM ? kGroupM : GM - first_m;
    const int block = in_band / (rows * kUnitN);              // (only the band's last block can be narrower)
    const int in_block = in_band - block * rows * kUnitN;
    const int cols = GN - block * kUnitN >= kUnitN ? kUnitN : GN - block * kUnitN;
    const int r = cols == kUnitN ? in_block / kUnitN : in_block / cols;
    TileCoord c;
    c.m = first_m + r;
    c.n = block * kUnitN + (in_block - r * cols);
    return c;
}

}  // namespace fo
