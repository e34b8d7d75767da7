// Host-side check of retinags_amd/csrc/tile_order.h: for every grid up to the sizes below,
// the workgroups that get a tile cover each tile of the grid exactly once.  Prints "ok".
#include "tile_order.h"

#include <cstdio>
#include <vector>

int main()
{
	for (int gx = 1; gx <= 48; gx++)
		for (int gy = 1; gy <= 80; gy++) {
			const int n = gx * gy;
			std::vector<int> seen(n, 0);
			const int blocks = rgs::tile_order_blocks(gx, gy);
			if (blocks % rgs::kXcds != 0 || blocks < n) {
				std::printf("bad block count %d for %dx%d\n", blocks, gx, gy);
				return 1;
			}
			for (int b = 0; b < blocks; b++) {
				const int t = rgs::tile_of_block(b, gx, gy);
				if (t >= n) {
					std::printf("tile %d out of range for %dx%d\n", t, gx, gy);
					return 1;
				}
				if (t >= 0)
					seen[t]++;
			}
			for (int t = 0; t < n; t++)
				if (seen[t] != 1) {
					std::printf("%dx%d: tile %d taken %d times\n", gx, gy, t, seen[t]);
					return 1;
				}
		}
	// most neighbours along a row share an XCD: in a 100x65 grid, tiles (r, c) and (r, c+1)
	const int gx = 100, gy = 65, blocks = rgs::tile_order_blocks(gx, gy);
	std::vector<int> xcd(gx * gy, -1);
	for (int b = 0; b < blocks; b++) {
		const int t = rgs::tile_of_block(b, gx, gy);
		if (t >= 0)
			xcd[t] = b % rgs::kXcds;
	}
	int same = 0, pairs = 0;
	for (int r = 0; r < gy; r++)
		for (int c = 0; c + 1 < gx; c++, pairs++)
			same += xcd[r * gx + c] == xcd[r * gx + c + 1];
	if (same < pairs * (rgs::kPatchW - 1) / rgs::kPatchW - pairs / 50) {
		std::printf("only %d of %d row neighbours share an XCD\n", same, pairs);
		return 1;
	}
	std::puts("ok");
	return 0;
}
