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

// ---- tiles of 128 consecutive positions of the flattened [B][N][N] index space (triattn_out) -----------
// A tile starts at position p0 = 128 * tile_id = (b0, i0, j0).  MODE 0: N is a multiple of 128, a tile lies
// inside one row; 1: N >= 128, at most two rows, whose element offsets in the strided view are row0 and row1;
// 2: any N, the general walk.
struct FlatTile {
  int b0, i0, j0;
  long long row0, row1;
};
OF3_HD inline FlatTile flat_tile(int tile_id, int N, long long stride_b, long long stride_r) {
  FlatTile t;
  const unsigned p0 = (unsigned)tile_id * 128u, nn = (unsigned)N * (unsigned)N;
  t.b0 = (int)(p0 / nn);
  const unsigned rem = p0 - (unsigned)t.b0 * nn;
  t.i0 = (int)(rem / (unsigned)N);
  t.j0 = (int)(rem - (unsigned)t.i0 * (unsigned)N);
  const bool last = t.i0 + 1 == N;
  t.row0 = t.b0 * stride_b + t.i0 * stride_r;
  t.row1 = (t.b0 + (last ? 1 : 0)) * stride_b + (last ? 0 : t.i0 + 1) * stride_r;
  return t;
}
// element offset of position d (0..127) of the tile in the view; the position must exist
template <int MODE>
OF3_HD inline long long flat_offset(const FlatTile& t, int d, int N, long long stride_b, long long stride_r,
                                    long long stride_k) {
  int j = t.j0 + d;
  if (MODE == 0) {
    return t.row0 + j * stride_k;
  } else if (MODE == 1) {
    const bool wrapped = j >= N;
    j -= wrapped ? N : 0;
    return (wrapped ? t.row1 : t.row0) + j * stride_k;
  } else {
    int b = t.b0, i = t.i0;
    while (j >= N) j -= N, ++i;  // at most once when N >= 128
    while (i >= N) i -= N, ++b;
    return b * stride_b + i * stride_r + j * stride_k;
  }
}

// ---- order of the attention core's work-groups -----------------------------------------------------------
// Work items of one (batch element, head) are (query range qc < n_qc, row group rg < n_rg).  They are taken in
// blocks of RB row groups x QB query ranges; inside a block the query range runs fastest, then the row group.
struct FlashItem {
  int bh, qc, rg;
};
OF3_HD inline FlashItem flash_item(int logical, int n_qc, int n_rg, int RB, int QB) {
  FlashItem w;
  const int per_bh = n_qc * n_rg;
  w.bh = logical / per_bh;
  const int idx = logical - w.bh * per_bh;
  const int rb = idx / (RB * n_qc);
  const int within = idx - rb * (RB * n_qc);
  const int rows_here = n_rg - rb * RB < RB ? n_rg - rb * RB : RB;  // the last block of row groups may be short
  const int qb = within / (rows_here * QB);
  const int w2 = within - qb * (rows_here * QB);
  const int qw = n_qc - qb * QB < QB ? n_qc - qb * QB : QB;        // and so may the last block of query ranges
  const int rg_local = w2 / qw;
  w.qc = qb * QB + (w2 - rg_local * qw);
  w.rg = rb * RB + rg_local;
  return w;
}

// ---- contraction: rows a direct-to-LDS instruction brings in -------------------------------------------
// A tile's operand rows start at tile_first; an instruction covers the 16 rows from tile_first + rb on.  Rows
// from `token_rows` (the tokens, rounded up to whole 32-blocks) on are padding: such a block takes the last 16
// rows with tokens instead (lines the caches already hold), wherever the tile lies.  Returns the first row.
OF3_HD inline int contract_rows_first(int tile_first, int rb, int token_rows) {
  const int left = token_rows - tile_first;  // may be zero or less for a tile that lies in the padding
  return tile_first + (rb + 16 <= left ? rb : left - 16);
}

}  // namespace of3
