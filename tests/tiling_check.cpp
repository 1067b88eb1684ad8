// Host-side check of the tiling the position-wise passes use (openfold-3_amd/csrc/of3_tiles.h, the very
// functions the kernels compile): for a token count N and a batch of B it walks every tile as the kernels
// do and verifies that no position, row or column index leaves the tensors and that every position is
// covered.  Usage: tiling_check <N>...; prints "ok <N>" per count, or the first violation and exits 1.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "of3_tiles.h"

using namespace of3;

static int fail(const char* what, int N, int tile, int pos) {
  std::printf("FAIL %s: N=%d tile=%d pos=%d\n", what, N, tile, pos);
  return 1;
}

// trimul_out: pieces of >= 8 columns, the last ragged piece may run past the last row (positions left out);
// x is read in groups of 8 positions from planes padded to Np x Np
static int check_output_pass(int N, int B) {
  const int Np = (N + 127) / 128 * 128;
  const bool ragged = N % 128 != 0;
  const RaggedTiles t = ragged_tiles(N);
  std::vector<int> cover((size_t)B * N * N, 0);
  for (int tile = 0; tile < B * t.per_batch; ++tile) {
    const TilePlace p = ragged ? tile_place<true>(tile, N, t.full_per_row, t.tail_shift, t.per_batch, false)
                               : tile_place<false>(tile, N, t.full_per_row, t.tail_shift, t.per_batch, false);
    if (p.b < 0 || p.b >= B || p.i0 < 0 || p.i0 >= N || p.shift < 3 || p.shift > 7) return fail("origin", N, tile, 0);
    const int jmask = (1 << p.shift) - 1;
    for (int pos = 0; pos < 128; ++pos) {
      const int i = p.i0 + (pos >> p.shift), j = p.j0 + (pos & jmask);
      if (j < 0 || j >= Np) return fail("column beyond the padded row", N, tile, pos);
      if (i < N && j < N) ++cover[((size_t)p.b * N + i) * N + j];
    }
    for (int pg = 0; pg < 16; ++pg) {  // 16-byte groups of x
      int i = p.i0 + ((8 * pg) >> p.shift);
      const int j = p.j0 + ((8 * pg) & jmask);
      i = i < Np ? i : Np - 1;
      if (i < 0 || j < 0 || j + 7 >= Np || j % 8 != 0) return fail("x group", N, tile, pg);
      if (((8 * pg) >> p.shift) != ((8 * pg + 7) >> p.shift)) return fail("x group spans two rows", N, tile, pg);
    }
  }
  for (size_t k = 0; k < cover.size(); ++k)
    if (cover[k] != 1) return fail("position not covered exactly once", N, (int)k, cover[k]);
  return 0;
}

// triattn_proj: pieces of whole 32-key panels, every row of a tile exists (N >= 4), columns are written up to
// the end of the last token's panel inside rows padded to Jp
static int check_input_pass(int N, int B) {
  const int Jp = (N + 127) / 128 * 128;
  const bool ragged = N % 128 != 0 && N >= 4;
  RaggedTiles t = {Jp / 128, 7, N * (Jp / 128)};
  if (ragged) t = ragged_tiles(N, 5);
  std::vector<char> written((size_t)B * N * Jp, 0);
  for (int tile = 0; tile < B * t.per_batch; ++tile) {
    const TilePlace p = ragged ? tile_place<true>(tile, N, t.full_per_row, t.tail_shift, t.per_batch, true)
                               : tile_place<false>(tile, N, t.full_per_row, t.tail_shift, t.per_batch, true);
    if (p.b < 0 || p.b >= B || p.shift < 5 || p.shift > 7) return fail("origin", N, tile, 0);
    const int jmask = (1 << p.shift) - 1;
    for (int pos = 0; pos < 128; ++pos) {
      const int i = p.i0 + (pos >> p.shift), j = p.j0 + (pos & jmask);
      if (i < 0 || i >= N || j < 0 || j >= Jp) return fail("position outside the padded rows", N, tile, pos);
      written[((size_t)p.b * N + i) * Jp + j] = 1;
    }
    for (int tt = 0; tt < 4; ++tt) {  // 32-position tiles: one row, one key panel
      const int jt = p.j0 + ((32 * tt) & jmask);
      if (jt % 32 != 0 || jt + 31 >= Jp) return fail("panel", N, tile, tt);
      if (((32 * tt) >> p.shift) != ((32 * tt + 31) >> p.shift)) return fail("panel spans two rows", N, tile, tt);
    }
  }
  const int n32 = (N + 31) / 32 * 32;
  for (int b = 0; b < B; ++b)
    for (int i = 0; i < N; ++i)
      for (int j = 0; j < n32; ++j)
        if (!written[((size_t)b * N + i) * Jp + j]) return fail("column below the end of the last panel not written", N, i, j);
  return 0;
}

// triattn_out: tiles of 128 consecutive positions of the flattened [B][N][N] index space; the offset of a
// position in a strided view (plain and transposed) must be that of its (b, i, j)
static int check_flat_pass(int N, int B) {
  const long long C = 128;
  for (int transposed = 0; transposed < 2; ++transposed) {
    const long long sb = (long long)N * N * C, sr = transposed ? C : N * C, sk = transposed ? N * C : C;
    const long long total = (long long)B * N * N;
    const int tiles = (int)((total + 127) / 128);
    std::vector<char> seen((size_t)total, 0);
    for (int tile = 0; tile < tiles; ++tile) {
      const FlatTile t = flat_tile(tile, N, sb, sr);
      for (int d = 0; d < 128; ++d) {
        const long long p = (long long)tile * 128 + d;
        if (p >= total) continue;
        const int b = (int)(p / ((long long)N * N)), i = (int)(p / N % N), j = (int)(p % N);
        const long long want = b * sb + i * sr + j * sk;
        const long long got = N % 128 == 0 ? flat_offset<0>(t, d, N, sb, sr, sk)
                              : (N >= 128 ? flat_offset<1>(t, d, N, sb, sr, sk) : flat_offset<2>(t, d, N, sb, sr, sk));
        if (got != want || got < 0 || got + C > B * sb) return fail("flat offset", N, tile, d);
        seen[(size_t)p] = 1;
      }
    }
    for (long long p = 0; p < total; ++p)
      if (!seen[(size_t)p]) return fail("flat position not visited", N, (int)p, 0);
  }
  return 0;
}

// attention core: the order of the work-groups is a one-to-one map onto (head, query range, row group)
static int check_flash_order(int N) {
  const int n_qc = (N + 127) / 128, n_rg = (N + 3) / 4, BH = 3;
  std::vector<char> seen((size_t)BH * n_qc * n_rg, 0);
  for (int logical = 0; logical < BH * n_qc * n_rg; ++logical) {
    const FlashItem w = flash_item(logical, n_qc, n_rg, 8, 8);
    if (w.bh < 0 || w.bh >= BH || w.qc < 0 || w.qc >= n_qc || w.rg < 0 || w.rg >= n_rg) return fail("flash item", N, logical, 0);
    char& s = seen[((size_t)w.bh * n_qc + w.qc) * n_rg + w.rg];
    if (s) return fail("flash item taken twice", N, logical, 0);
    s = 1;
    // with eight query ranges or fewer the order is the plain one
    if (n_qc <= 8 && (w.qc != logical % n_qc || w.rg != logical / n_qc % n_rg)) return fail("flash plain order", N, logical, 0);
  }
  return 0;
}

// contraction: whatever the tile shape, every load instruction's 16 rows lie below the last row with tokens
static int check_contract_rows(int N) {
  const int Np = (N + 127) / 128 * 128, token_rows = (N + 31) / 32 * 32;
  const int shapes[4][2] = {{256, 192}, {256, 128}, {256, 256}, {384, 192}};
  for (const auto& sh : shapes)
    for (int side = 0; side < 2; ++side) {
      const int T = sh[side];
      for (int first = 0; first < Np; first += T)
        for (int rb = 0; rb < T; rb += 16) {
          const int row = contract_rows_first(first, rb, token_rows);
          if (row < 0 || row + 16 > token_rows || token_rows > Np) return fail("contraction rows", N, first, rb);
          if (first + rb + 16 <= token_rows && row != first + rb) return fail("contraction rows moved", N, first, rb);
        }
    }
  return 0;
}

int main(int argc, char** argv) {
  for (int a = 1; a < argc; ++a) {
    const int N = std::atoi(argv[a]);
    if (N < 1) return 2;
    if (check_output_pass(N, 2) || check_input_pass(N, 2) || check_flat_pass(N, 2) || check_flash_order(N) || check_contract_rows(N)) return 1;
    std::printf("ok %d\n", N);
  }
  return 0;
}
