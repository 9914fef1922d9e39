// The two orders in which a weight matrix [rows, inner] (bfloat16) is laid out for the few-row products, so that
// a wave's load of an MFMA A operand (64 lanes x 8 elements) is 1 KB of consecutive memory.  Which one a matrix
// (or each row group of it) has follows from its number of rows alone, here and where the weights are packed.
//
//   16-row tiles   [ceil(rows/16)][ceil(inner/32)][64 lanes][8]: lane (r = l % 16, g = l / 16) of tile (o, j)
//                  holds W[o*16 + r][j*32 + g*8 .. +8].
//   pair layout    (few rows: 16 features per workgroup would leave compute units idle, workgroups take 8)
//                  [ceil(rows/16)*2][ceil(inner/64)][64 lanes][8]: lane (r8 = l % 8, half = l / 8 % 2, g = l / 16)
//                  of tile (o8, p) holds W[o8*8 + r8][p*64 + half*32 + g*8 .. +8]: the same 8 rows at two
//                  consecutive k tiles.
// Zeros beyond rows and inner.
#pragma once

constexpr int PAIR_LAYOUT_BELOW_TILES = 256;   // 16-row tiles (one per compute unit) below which the pair layout is used

inline bool pair_layout(long rows) { return (rows + 15) / 16 < PAIR_LAYOUT_BELOW_TILES; }
