// Device-side helpers shared by the gfx950 kernels of the half-Gaussian rasterizer.
// Wave size is 64 everywhere; a tile is 16x16 pixels handled by 4 wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rgs {

constexpr int kTile = 16;         // K/cuda_rasterizer_hgs/config.h:16-17
constexpr int kTilePix = 256;
constexpr int kWave = 64;

// 3x3 matrix, c[column][row]; product and transpose keep the summation order of
// the reference's matrix library (K/third_party/glm/glm/detail/type_mat3x3.inl:509-517)
// because radii, tile rectangles and sort keys must come out bit-identical.
struct M3 {
	float c[3][3];
};

__device__ __forceinline__ M3 m3_cols(float x0, float y0, float z0, float x1, float y1, float z1, float x2, float y2,
                                      float z2)
{
	M3 r;
	r.c[0][0] = x0; r.c[0][1] = y0; r.c[0][2] = z0;
	r.c[1][0] = x1; r.c[1][1] = y1; r.c[1][2] = z1;
	r.c[2][0] = x2; r.c[2][1] = y2; r.c[2][2] = z2;
	return r;
}

__device__ __forceinline__ M3 m3_mul(const M3& a, const M3& b)
{
	M3 r;
#pragma unroll
	for (int col = 0; col < 3; col++)
#pragma unroll
		for (int row = 0; row < 3; row++)
			r.c[col][row] = a.c[0][row] * b.c[col][0] + a.c[1][row] * b.c[col][1] + a.c[2][row] * b.c[col][2];
	return r;
}

__device__ __forceinline__ M3 m3_transpose(const M3& a)
{
	M3 r;
#pragma unroll
	for (int col = 0; col < 3; col++)
#pragma unroll
		for (int row = 0; row < 3; row++)
			r.c[col][row] = a.c[row][col];
	return r;
}

// Column-major 4x4 affine map of a point (K/cuda_rasterizer_hgs/auxiliary.h:63-82).
__device__ __forceinline__ float3 xform_point_4x3(const float3 p, const float* __restrict__ m)
{
	float3 o;
	o.x = m[0] * p.x + m[4] * p.y + m[8] * p.z + m[12];
	o.y = m[1] * p.x + m[5] * p.y + m[9] * p.z + m[13];
	o.z = m[2] * p.x + m[6] * p.y + m[10] * p.z + m[14];
	return o;
}

__device__ __forceinline__ float4 xform_point_4x4(const float3 p, const float* __restrict__ m)
{
	float4 o;
	o.x = m[0] * p.x + m[4] * p.y + m[8] * p.z + m[12];
	o.y = m[1] * p.x + m[5] * p.y + m[9] * p.z + m[13];
	o.z = m[2] * p.x + m[6] * p.y + m[10] * p.z + m[14];
	o.w = m[3] * p.x + m[7] * p.y + m[11] * p.z + m[15];
	return o;
}

// NDC <-> pixel maps, evaluated in double and rounded once
// (K/cuda_rasterizer_hgs/auxiliary.h:41-49).
__device__ __forceinline__ float ndc_to_pix(float v, int S)
{
	return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5);
}

__device__ __forceinline__ float pix_to_ndc(float pix, int S)
{
	return (float)(((double)(2 * pix) + 1.0) / (double)S - 1.0);
}

struct TileRect {
	uint32_t x0, y0, x1, y1;
};

// Tile rectangle covered by a splat of integer radius (K/cuda_rasterizer_hgs/auxiliary.h:51-61).
// The float->int casts saturate on this hardware, like on the reference's.
__device__ __forceinline__ TileRect tile_rect(float px, float py, int radius, int gx, int gy)
{
	TileRect r;
	r.x0 = (uint32_t)min(gx, max(0, (int)((px - radius) / kTile)));
	r.y0 = (uint32_t)min(gy, max(0, (int)((py - radius) / kTile)));
	r.x1 = (uint32_t)min(gx, max(0, (int)((px + radius + kTile - 1) / kTile)));
	r.y1 = (uint32_t)min(gy, max(0, (int)((py + radius + kTile - 1) / kTile)));
	return r;
}

// ---- conservative bounds used to skip blend work without changing any result ---------------

// Lower bound on the exponent `power` below which alpha = min(0.99, opacity * exp(power)) is
// certainly under 1/255: alpha >= 1/255 needs power >= -ln(255 * opacity).  A NaN opacity
// makes alpha 0.99 in the exact evaluation (fminf drops the NaN), so it is never culled; a
// non-positive one can never reach 1/255.
__device__ __forceinline__ float exponent_floor(float opacity)
{
	if (opacity != opacity)
		return -INFINITY;
	if (!(opacity > 0.f))
		return INFINITY;
	return -logf(255.0f * opacity) - 1e-3f;
}

// power >= floor is the ellipse d^T Q d <= -2 floor around the Gaussian's centre (Q = conic).
// Half-widths of its bounding box, sqrt(-2 floor * Q^-1_xx) and sqrt(-2 floor * Q^-1_yy),
// inflated against rounding.  Infinite when the conic is not positive definite or the floor is
// -inf, so that nothing is culled; unused when floor > 0 (then no pixel can reach 1/255).
__device__ __forceinline__ float2 alpha_ellipse_half_extent(const float4 conic, float floor)
{
	const float det = conic.x * conic.z - conic.y * conic.y;
	if (!(det > 0.f) || !(floor <= 0.f))
		return float2{INFINITY, INFINITY};
	const float c = -2.f * floor;
	return float2{sqrtf(c * conic.z / det) * 1.0001f + 1e-2f, sqrtf(c * conic.x / det) * 1.0001f + 1e-2f};
}

// ---- wave64 cross-lane primitives (DPP) -----------------------------------------------

template <int Ctrl, int RowMask, int BankMask>
__device__ __forceinline__ float dpp_shift_add(float v)
{
	int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, RowMask, BankMask, true);
	return v + __builtin_bit_cast(float, moved);
}

// Sum over the 64 lanes; the total is valid in lane 63 only.
// The lanes for which `b` holds, as a mask.  (HIP's __ballot takes an int: a flag first becomes 0 or 1 in a vector
// register and is then compared with 0 again, two vector instructions per ballot; a comparison's result already is
// the mask.)
__device__ __forceinline__ uint64_t lanes_where(bool b)
{
	return __builtin_amdgcn_ballot_w64(b);
}

__device__ __forceinline__ float wave_sum_to_lane63(float v)
{
	v = dpp_shift_add<0x111, 0xF, 0xF>(v);  // row_shr:1
	v = dpp_shift_add<0x112, 0xF, 0xF>(v);  // row_shr:2
	v = dpp_shift_add<0x114, 0xF, 0xF>(v);  // row_shr:4
	v = dpp_shift_add<0x118, 0xF, 0xF>(v);  // row_shr:8  -> lane 15 of each row holds the row sum
	v = dpp_shift_add<0x142, 0xA, 0xF>(v);  // row_bcast:15 into rows 1 and 3
	v = dpp_shift_add<0x143, 0xC, 0xF>(v);  // row_bcast:31 into rows 2 and 3
	return v;
}

template <int Ctrl, int RowMask, int BankMask>
__device__ __forceinline__ uint32_t dpp_shift_add_u32(uint32_t v)
{
	int moved = __builtin_amdgcn_update_dpp(0, (int)v, Ctrl, RowMask, BankMask, true);
	return v + (uint32_t)moved;
}

// Inclusive prefix sum over the 64 lanes.
__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v)
{
	v = dpp_shift_add_u32<0x111, 0xF, 0xF>(v);
	v = dpp_shift_add_u32<0x112, 0xF, 0xF>(v);
	v = dpp_shift_add_u32<0x114, 0xF, 0xF>(v);
	v = dpp_shift_add_u32<0x118, 0xF, 0xF>(v);
	v = dpp_shift_add_u32<0x142, 0xA, 0xF>(v);
	v = dpp_shift_add_u32<0x143, 0xC, 0xF>(v);
	return v;
}

// The largest of the 64 lanes' values, the same in every lane (and in a scalar register): four exchanges inside each
// row of 16 lanes, then one lane of each row read out.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
	v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));   // quad_perm:[1,0,3,2]
	v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));   // quad_perm:[2,3,0,1]
	v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true));  // row_half_mirror
	v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, true));  // row_mirror
	const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16),
	               r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
	return max(max(r0, r1), max(r2, r3));
}

// Exclusive prefix sum of one u32 per thread over a 256-thread block.
// `lds` needs 5 words; returns the block total in `total`.
__device__ __forceinline__ uint32_t block256_exclusive_scan_u32(uint32_t v, uint32_t* lds, uint32_t& total)
{
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	uint32_t inc = wave_inclusive_scan_u32(v);
	if (lane == 63)
		lds[wave] = inc;
	__syncthreads();
	uint32_t base = 0;
#pragma unroll
	for (int w = 0; w < 4; w++) {
		uint32_t s = lds[w];
		if (w < wave)
			base += s;
	}
	total = lds[0] + lds[1] + lds[2] + lds[3];
	__syncthreads();
	return base + inc - v;
}

}  // namespace rgs
