// The map from workgroup ids to tiles that every tiled kernel of the library uses.  Plain C++ without HIP types, so that
// a host-only program can include it too (the CPU tests check the map exhaustively that way).
#pragma once

#if defined(__HIPCC__)
#define LCE_HOST_DEV __host__ __device__ __forceinline__
#else
#define LCE_HOST_DEV inline
#endif

namespace lce {

// XCD-aware decode of a flat workgroup id into a (row-tile, col-tile) pair.
// Hardware deals workgroup ids round-robin over the 8 XCDs (each with its own L2), so ids with the
// same (id % 8) share an L2.  The tiles are numbered block by block, a block being BR x (32/BR) tiles
// (narrower at the two far edges of the tile grid), and every XCD gets one contiguous eighth of that
// numbering: the 32 workgroups resident on an XCD then touch about BR row-tiles and 32/BR col-tiles of
// the operands, and every XCD has the same number of tiles (within one) whatever the shape.  (Numbering
// whole 32-slot blocks with empty slots at the edges instead left some XCDs with up to twice the tiles
// of others on ragged shapes: 12 token tiles x 20 splits of a forward took two rounds instead of one.)
struct TileMap {
  int nrow_tiles, ncol_tiles;  // tiles along the "row" operand (blocks of BR) and "col" operand
  int br, bc;                  // block shape, br * bc == 32
  int rows_fastest;            // 1: consecutive blocks walk the row dimension first
  int per;                     // tiles per XCD
  int total;                   // launched workgroups: 8 * per

  // shape of the 32-tile blocks that one XCD works on: up to 8 tiles along the row side
  LCE_HOST_DEV static int block_rows(int nrow_tiles) {
    int br = 1;
    while (br < 8 && br < nrow_tiles) br <<= 1;
    return br;
  }
  // the same map over fewer row tiles (a count that only the device knows): its workgroups are the
  // first `total` ids of the grid that was sized for the full map, the others have nothing to do
  LCE_HOST_DEV TileMap with_rows(int rows) const { return make(rows, ncol_tiles, rows >= br ? br : block_rows(rows), rows_fastest); }

  LCE_HOST_DEV static TileMap make(int nrow_tiles, int ncol_tiles, int br, int rows_fastest) {
    TileMap t;
    t.nrow_tiles = nrow_tiles;
    t.ncol_tiles = ncol_tiles;
    t.br = br;
    t.bc = 32 / br;
    t.rows_fastest = rows_fastest;
    t.per = (nrow_tiles * ncol_tiles + 7) >> 3;
    t.total = t.per * 8;
    return t;
  }
  // returns false when the slot is padding (no tile)
  LCE_HOST_DEV bool decode(int bid, int& rt, int& ct) const {
    if (bid >= total) return false;
    const int i = (bid & 7) * per + (bid >> 3);  // position in the block-by-block numbering
    if (i >= nrow_tiles * ncol_tiles) return false;
    // bands of blocks along the slow dimension; inside a band the blocks follow each other along the fast one
    const int n_fast = rows_fastest ? nrow_tiles : ncol_tiles, b_fast = rows_fastest ? br : bc;
    const int n_slow = rows_fastest ? ncol_tiles : nrow_tiles, b_slow = rows_fastest ? bc : br;
    const int band = i / (n_fast * b_slow);
    const int j = i - band * (n_fast * b_slow);
    const int w_slow = n_slow - band * b_slow < b_slow ? n_slow - band * b_slow : b_slow;  // the last band may be narrower
    const int blk = j / (b_fast * w_slow);
    const int k = j - blk * (b_fast * w_slow);
    const int w_fast = n_fast - blk * b_fast < b_fast ? n_fast - blk * b_fast : b_fast;    // and the last block of a band shorter
    // inside a block: columns fastest
    const int cols = rows_fastest ? w_slow : w_fast;
    const int r = k / cols, c = k - r * cols;
    rt = (rows_fastest ? blk * b_fast : band * b_slow) + r;
    ct = (rows_fastest ? band * b_slow : blk * b_fast) + c;
    return true;
  }
};

}  // namespace lce
