// Order in which the blend kernels' workgroups take the tiles of the image.
//
// The chip hands consecutive workgroups to its 8 XCDs in turn (workgroup b runs on XCD b % 8)
// and every XCD has a second-level cache of its own.  A Gaussian's record is read by every
// tile it touches, typically a few neighbouring ones; with tile = b those neighbours sit on
// different XCDs and each of them fetches the record from memory again.  Here the image is
// cut into patches of kPatchW x kPatchH tiles; a patch belongs to one XCD, and 8 consecutive
// patches (row-major over the patches) are worked on at the same time, one per XCD.  Most
// neighbours of a tile then share its XCD, while the 8 XCDs always work on adjacent parts of
// the image, whose loads are alike: dealing out larger regions per XCD cuts the traffic
// further but was measured slower, because workgroups are placed in order and one XCD with
// heavier tiles holds up the others.
#pragma once

#if defined(__HIPCC__)
#define RGS_HOST_DEVICE __host__ __device__
#else
#define RGS_HOST_DEVICE
#endif

namespace rgs {

constexpr int kXcds = 8;
constexpr int kPatchW = 4, kPatchH = 4;
constexpr int kPatchTiles = kPatchW * kPatchH;

// Number of workgroups to launch for a grid of tiles; those without a tile return at once.
RGS_HOST_DEVICE inline int tile_order_blocks(int grid_x, int grid_y)
{
	const int patches = ((grid_x + kPatchW - 1) / kPatchW) * ((grid_y + kPatchH - 1) / kPatchH);
	return kXcds * kPatchTiles * ((patches + kXcds - 1) / kXcds);
}

// Tile (row-major index) of workgroup `b`, or -1 if it has none.  A bijection between the
// workgroups that return a tile and the tiles of the grid.
RGS_HOST_DEVICE inline int tile_of_block(int b, int grid_x, int grid_y)
{
	const int patches_x = (grid_x + kPatchW - 1) / kPatchW, patches_y = (grid_y + kPatchH - 1) / kPatchH;
	if (b < 0)
		return -1;
	const int xcd = b % kXcds, turn = b / kXcds;
	const int patch = (turn / kPatchTiles) * kXcds + xcd, k = turn % kPatchTiles;
	if (patch >= patches_x * patches_y)
		return -1;
	const int col = (patch % patches_x) * kPatchW + k % kPatchW;
	const int row = (patch / patches_x) * kPatchH + k / kPatchW;
	if (col >= grid_x || row >= grid_y)
		return -1;
	return row * grid_x + col;
}

}  // namespace rgs
