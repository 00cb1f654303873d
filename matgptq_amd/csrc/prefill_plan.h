// Tile counts shared by the planner and the prefill launchers.
#pragma once

namespace matgptq {

// Prefill with two tile widths in one launch (128 x 192 and 128 x 128), sized so that the 512 resident
// slots (two workgroups per CU) are all taken in ONE round where neither width alone does that: with
// s = 512 / m_tiles slots per column of activation tiles, 128 x 128 tiles need row_blocks <= 8 s and
// 128 x 192 tiles leave slots empty when row_blocks < 12 s.  Between the two, x tiles of 192 rows take
// the first 12 x row blocks and the rest goes to tiles of 128 rows, x + y <= s.  A CU then holds one
// wide and one narrow workgroup instead of two wide ones (or one), and the launch ends earlier.
// Returns x (0: the mix does not apply) and the number of narrow tiles per column in *narrow.
inline int prefill_mix_wide_tiles(int row_blocks, int m_tiles, int* narrow) {
  *narrow = 0;
  if (m_tiles <= 0 || m_tiles > 512) return 0;
  const int s = 512 / m_tiles;
  if (row_blocks <= 8 * s || row_blocks > 12 * s) return 0;
  const int x = (row_blocks - 8 * s + 3) / 4;
  const int rest = row_blocks - 12 * x;
  const int y = rest <= 0 ? 0 : (rest + 7) / 8;
  if (x < 1 || y < 1 || x + y > s) return 0;
  *narrow = y;
  return x;
}

}  // namespace matgptq
