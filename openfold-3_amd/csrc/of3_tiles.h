// Tiling of the N x N positions of a batch element into 128-position tiles for the position-wise passes.
// Plain C++ (no HIP types): the kernels and the host-side test of the scheme compile the same functions.
#pragma once

#if defined(__HIPCC__)
#define OF3_HD __host__ __device__
#else
#define OF3_HD
#endif

namespace of3 {

// The whole 128-wide pieces of every row come first (full_per_row per row), then the remaining N % 128
// columns in pieces of 2^tail_shift columns (the smallest power of two >= 2^min_shift that covers them)
// x (128 >> tail_shift) consecutive rows.
struct RaggedTiles {
  int full_per_row, tail_shift, per_batch;
};
inline RaggedTiles ragged_tiles(int N, int min_shift = 3) {
  RaggedTiles t;
  t.full_per_row = N / 128;
  const int r = N % 128;
  t.tail_shift = r ? min_shift : 7;
  while ((1 << t.tail_shift) < r) ++t.tail_shift;
  const int rows = 128 >> t.tail_shift;
  t.per_batch = N * t.full_per_row + (r ? (N + rows - 1) / rows : 0);
  return t;
}

// Where a tile lies: batch element, first row, first column, log2 of its width.  Position pos (0..127) of
// the tile is row i0 + (pos >> shift), column j0 + (pos & ((1 << shift) - 1)).
struct TilePlace {
  int b, i0, j0, shift;
};
// RAGGED = false: whole-row pieces only (full_per_row pieces per row, per_batch = rows * full_per_row).
// keep_rows_inside: the last piece of the ragged columns is moved up so that it ends at row N - 1 (its rows
// all exist, some of them belong to the piece before it as well; needs N >= 128 >> tail_shift); otherwise it
// runs past the last row and the caller leaves those positions out.
template <bool RAGGED>
OF3_HD inline TilePlace tile_place(int tile_id, int N, int full_per_row, int tail_shift, int per_batch,
                                   bool keep_rows_inside) {
  TilePlace t;
  t.b = tile_id / per_batch;
  const int rem = tile_id - t.b * per_batch;
  const int main_tiles = N * full_per_row;
  if (!RAGGED || rem < main_tiles) {
    t.i0 = rem / full_per_row;
    t.j0 = (rem - t.i0 * full_per_row) * 128;
    t.shift = 7;
  } else {
    const int rows = 128 >> tail_shift;
    t.i0 = (rem - main_tiles) * rows;
    if (keep_rows_inside && t.i0 + rows > N) t.i0 = N - rows;
    t.j0 = full_per_row * 128;
    t.shift = tail_shift;
  }
  return t;
}

}  // namespace of3
