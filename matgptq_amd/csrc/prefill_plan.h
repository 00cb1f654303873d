// Tile counts shared by the planner and the prefill launchers.
#pragma once

namespace matgptq {

// Prefill with two tile widths in one launch, sized so that the 512 resident slots (two workgroups
// per CU) are all taken in ONE round where neither width alone does that.  Widths in row blocks of 16
// weight rows: `wide` > `narrow`.  With s = 512 / m_tiles slots per column of activation tiles, the
// narrow tiles alone need row_blocks <= narrow * s, and the wide ones leave slots empty when
// row_blocks < wide * s.  Between the two, x wide tiles take the first wide * x row blocks and the
// rest goes to y narrow tiles, x + y <= s.  A CU then holds one wide and one narrow workgroup instead
// of two wide ones (or one), and the launch ends earlier.
// Returns x (0: the mix does not apply) and y in *narrow_tiles.
inline int prefill_mix_tiles(int row_blocks, int m_tiles, int wide, int narrow, int* narrow_tiles) {
  *narrow_tiles = 0;
  if (m_tiles <= 0 || m_tiles > 512) return 0;
  const int s = 512 / m_tiles;
  if (row_blocks <= narrow * s || row_blocks > wide * s) return 0;
  const int x = (row_blocks - narrow * s + (wide - narrow) - 1) / (wide - narrow);
  const int rest = row_blocks - wide * x;
  const int y = rest <= 0 ? 0 : (rest + narrow - 1) / narrow;
  if (x < 1 || y < 1 || x + y > s) return 0;
  *narrow_tiles = y;
  return x;
}

// 128 x 192 and 128 x 128 tiles
inline int prefill_mix_wide_tiles(int row_blocks, int m_tiles, int* narrow_tiles) {
  return prefill_mix_tiles(row_blocks, m_tiles, 12, 8, narrow_tiles);
}

// 128 x 256 and 128 x 192 tiles
inline int prefill_mix_widest_tiles(int row_blocks, int m_tiles, int* narrow_tiles) {
  return prefill_mix_tiles(row_blocks, m_tiles, 16, 12, narrow_tiles);
}

}  // namespace matgptq
