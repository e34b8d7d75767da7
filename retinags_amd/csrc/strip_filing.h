// Which strips of a tile a list entry is filed for: shared by the kernel that emits the
// (Gaussian, tile) instances, which decides it, and the blend kernels, which rely on it.
//
// Most (pixel, Gaussian) visits of the reference loop (K/cuda_rasterizer_hgs/forward.cu:338-372,
// K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian) end at "alpha < 1/255" or at
// the half-Gaussian box test.  Three conservative tests remove such visits a whole 16x4 strip at a
// time without changing any result:
//  * alpha >= 1/255 needs power >= -ln(255 * opacity); with that floor (minus a margin) above
//    zero no pixel can pass;
//  * power >= floor is an ellipse around the Gaussian's centre; an entry whose ellipse (first its
//    bounding box, then the ellipse itself) misses the strip's rectangle is not filed;
//  * the world-space ray sample is affine in the pixel, so its range over a strip follows from the
//    strip's corner coordinates: an entry whose strip lies entirely outside the submodel box is not
//    filed, one whose strip lies entirely inside skips the per-pixel box test.
// All three only drop work that the exact evaluation would have skipped too.
#pragma once
#include "rgs_device.h"

namespace rgs {

__device__ __forceinline__ float wave_uniform(float v)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}

// What the half-Gaussian test needs besides the pixel: rows 0..2 of the inverse projection
// (column-major 4x4, m[c][r] = element (r, c)) and the submodel box.  Read once per wavefront
// into scalar registers; the test itself runs for every blended sample.
struct BoxFrame {
	float m[4][3];
	float3 lo, hi;
	float tanx, tany;
};

__device__ __forceinline__ BoxFrame load_box_frame(const float* __restrict__ projinv, const float* __restrict__ range_low,
                                                   const float* __restrict__ range_up, float tanx, float tany)
{
	BoxFrame b;
#pragma unroll
	for (int c = 0; c < 4; c++)
#pragma unroll
		for (int r = 0; r < 3; r++)
			b.m[c][r] = wave_uniform(projinv[4 * c + r]);
	b.lo = float3{wave_uniform(range_low[0]), wave_uniform(range_low[1]), wave_uniform(range_low[2])};
	b.hi = float3{wave_uniform(range_up[0]), wave_uniform(range_up[1]), wave_uniform(range_up[2])};
	b.tanx = tanx;
	b.tany = tany;
	return b;
}

// What the tests need of a Gaussian's 64-byte blend record: (pixel x, pixel y, exponent floor, clip w),
// the conic (xx, xy, yy) and the half extents of the alpha >= 1/255 ellipse's bounding box.
struct FiledGeometry {
	float4 geom;
	float4 conic;
	float2 half;
};

// NDC of the first and last pixel column of a tile and of the first and last row of each of its strips
// (pix_to_ndc with the division replaced by the reciprocal image size: these only feed the
// conservative range test, which has room for the last bit).
__device__ __forceinline__ float2 tile_column_ndc(int tile_x, int W)
{
	const double rw = 1.0 / (double)W;
	const float x0 = (float)(tile_x * kTile);
	return float2{(float)(((double)(2.f * x0) + 1.0) * rw - 1.0), (float)(((double)(2.f * (x0 + 15.f)) + 1.0) * rw - 1.0)};
}

__device__ __forceinline__ float2 strip_rows_ndc(int tile_y, int strip, int H)
{
	const double rh = 1.0 / (double)H;
	const float ya = (float)(tile_y * kTile + 4 * strip);
	return float2{(float)(((double)(2.f * ya) + 1.0) * rh - 1.0), (float)(((double)(2.f * (ya + 3.f)) + 1.0) * rh - 1.0)};
}

// The part of the tests that depends on the Gaussian and the frame but not on the tile, computed
// once per Gaussian.  The ray sample at the Gaussian's clip w is affine in the pixel's NDC
// coordinates, p_k = A_k nx + B_k ny + C_k per world coordinate k, so its range over a strip is the
// sum of the ranges of the two terms; the box tolerance is taken from the magnitudes of the terms, not
// of the result, so that it also covers the rounding of this regrouped evaluation when the terms
// cancel.  The rows an ellipse reaches are computed with the reciprocals of a and c.
struct StripTests {
	float gx, gy, hx, hy;
	float a, b, c, limit;   // conic; -2 floor
	float ra, rc;           // 1 / a, 1 / c
	float A[3], B[3], C[3], tol[3];
	uint32_t flags;         // bit 0: the conic is an ellipse; bit 1: no pixel can reach alpha >= 1/255
	uint32_t pad;
};

__device__ __forceinline__ StripTests prepare_strip_tests(const FiledGeometry& e, const BoxFrame& box)
{
#pragma clang fp contract(off)
	StripTests t;
	t.gx = e.geom.x; t.gy = e.geom.y; t.hx = e.half.x; t.hy = e.half.y;
	const float floor = e.geom.z, w = e.geom.w;
	t.a = e.conic.x; t.b = e.conic.y; t.c = e.conic.z;
	t.limit = -2.f * floor;
	// hardware reciprocals and square roots (one unit in the last place) here and below: these values only place the
	// bounds of conservative tests, whose margins are three orders of magnitude wider, and a correctly rounded division
	// or square root costs ten instructions where these cost one
	t.ra = __builtin_amdgcn_rcpf(t.a);
	t.rc = __builtin_amdgcn_rcpf(t.c);
	const bool ellipse = (t.a > 0.f) && (t.c > 0.f) && (t.a * t.c - t.b * t.b > 0.f);
	t.flags = (ellipse ? 1u : 0u) | ((floor > 0.f) ? 2u : 0u);  // floor > 0: even power = 0 gives alpha < 1/255
	t.pad = 0u;
	const float wp = w + 0.0000001f;
	const float sx = wp * box.tanx, sy = wp * box.tany;
#pragma unroll
	for (int k = 0; k < 3; k++) {
		const float m2w = box.m[2][k] * w;
		t.A[k] = box.m[0][k] * sx;
		t.B[k] = box.m[1][k] * sy;
		t.C[k] = m2w + box.m[3][k];
		t.tol[k] = 1e-4f * fmaxf(fabsf(t.A[k]) + fabsf(t.B[k]) + fabsf(m2w) + fabsf(box.m[3][k]), 1.f);
	}
	return t;
}

// The decisions for the four strips of the tile whose first pixel is (x0, y0): bit s of the result =
// the entry is filed for strip s, bit 4 + s = that strip lies inside the box.  nx = NDC of the tile's
// first and last pixel column, ny[2 s], ny[2 s + 1] = NDC of strip s's first and last row.
__device__ __forceinline__ uint32_t strips_filed_for(const StripTests& t, float x0, float y0, float2 nx, const float (&ny)[8],
                                                     const BoxFrame& box)
{
#pragma clang fp contract(off)
	if (t.flags & 2u)
		return 0u;
	if ((t.gx + t.hx < x0) || (t.gx - t.hx > x0 + 15.f))
		return 0u;
	const float a = t.a, b = t.b, c = t.c;
	const bool ellipse = (t.flags & 1u) != 0u;
	const float dxl = t.gx - (x0 + 15.f), dxh = t.gx - x0;

	// range of the ray sample's world coordinates over the tile's columns, per coordinate
	float xlo[3], xhi[3];
#pragma unroll
	for (int k = 0; k < 3; k++) {
		const float p0 = t.A[k] * nx.x, p1 = t.A[k] * nx.y;
		xlo[k] = fminf(p0, p1) + t.C[k];
		xhi[k] = fmaxf(p0, p1) + t.C[k];
	}
	const float lov[3] = {box.lo.x, box.lo.y, box.lo.z}, hiv[3] = {box.hi.x, box.hi.y, box.hi.z};

	// The same box test for the whole tile first (rows from the first of strip 0 to the last of strip 3): a product
	// with a constant is monotone in the row coordinate, so the tile's range contains every strip's, and a tile that
	// lies inside (outside) the box has all four strips inside (outside) by the very comparisons made below.  Most
	// Gaussians are far from their submodel's faces, and three of the four evaluations go.
	bool tile_inside = true, tile_outside = false;
#pragma unroll
	for (int k = 0; k < 3; k++) {
		const float q0 = t.B[k] * ny[0], q1 = t.B[k] * ny[7];
		const float pmin = xlo[k] + fminf(q0, q1), pmax = xhi[k] + fmaxf(q0, q1);
		tile_inside = tile_inside && (pmin > lov[k] + t.tol[k]) && (pmax < hiv[k] - t.tol[k]);
		tile_outside = tile_outside || (pmax < lov[k] - t.tol[k]) || (pmin > hiv[k] + t.tol[k]);
	}
	if (tile_outside)
		return 0u;

	// The rows the ellipse q(d) = a dx^2 + 2 b dx dy + c dy^2 <= limit reaches over the tile's 16 columns, once for the four
	// strips (d = centre - pixel, so dx runs over [dxl, dxh]).  For a given dx the ellipse holds the dy between
	// (-b dx -+ sqrt(c limit - det dx^2)) / c; the upper end is concave in dx and the lower convex, so over an interval
	// of dx each is extreme at the ellipse's own extreme point (dy = +-Y at dx = -+b Y / a, Y = sqrt(a limit / det)) if
	// that lies inside the interval, at one of its ends otherwise.  The limit gets room for the rounding
	// of q (relative to its largest terms over the tile), and the rows a margin of a hundredth of a pixel.
	float dy_low = -INFINITY, dy_high = INFINITY;
	if (ellipse) {
		const float dy_first = t.gy - y0, dy_last = t.gy - (y0 + 15.f);
		const float largest = a * fmaxf(dxl * dxl, dxh * dxh) + c * fmaxf(dy_first * dy_first, dy_last * dy_last);
		const float limit = t.limit + (1e-3f + 1e-4f * t.limit + 1e-5f * largest);
		const float det = a * c - b * b;
		const float rdet = __builtin_amdgcn_rcpf(det);
		const float X = __builtin_amdgcn_sqrtf(c * limit * rdet), Y = __builtin_amdgcn_sqrtf(a * limit * rdet);
		const float dl = fmaxf(dxl, -X), dh = fminf(dxh, X);
		if (dl > dh)
			return 0u;  // the columns lie beside the ellipse
		const float sl = __builtin_amdgcn_sqrtf(fmaxf(c * limit - det * dl * dl, 0.f)),
		            sh = __builtin_amdgcn_sqrtf(fmaxf(c * limit - det * dh * dh, 0.f));
		const float at_top = -b * Y * t.ra;  // dx of the ellipse's highest dy; that of its lowest is -at_top
		const float top = fmaxf((-b * dl + sl) * t.rc, (-b * dh + sh) * t.rc);
		const float bottom = fminf((-b * dl - sl) * t.rc, (-b * dh - sh) * t.rc);
		const float margin = 1e-2f + 1e-5f * Y;
		dy_high = ((!(at_top < dl) && !(at_top > dh)) ? Y : top) + margin;
		dy_low = ((!(-at_top < dl) && !(-at_top > dh)) ? -Y : bottom) - margin;
	}
	uint32_t bits = 0;
#pragma unroll
	for (int s = 0; s < 4; s++) {
		const float ya = y0 + (float)(4 * s);
		if ((t.gy + t.hy < ya) || (t.gy - t.hy > ya + 3.f))
			continue;
		const float dyl = t.gy - (ya + 3.f), dyh = t.gy - ya;
		if ((dyh < dy_low) || (dyl > dy_high))
			continue;
		bool inside = true, outside = false;
		if (!tile_inside) {
#pragma unroll
			for (int k = 0; k < 3; k++) {
				const float q0 = t.B[k] * ny[2 * s], q1 = t.B[k] * ny[2 * s + 1];
				const float pmin = xlo[k] + fminf(q0, q1), pmax = xhi[k] + fmaxf(q0, q1);
				inside = inside && (pmin > lov[k] + t.tol[k]) && (pmax < hiv[k] - t.tol[k]);
				outside = outside || (pmax < lov[k] - t.tol[k]) || (pmin > hiv[k] + t.tol[k]);
			}
		}
		// a NaN can set neither flag, which leaves the decision to the per-pixel test
		if (outside)
			continue;
		bits |= (1u << s) | (inside ? (16u << s) : 0u);
	}
	return bits;
}

}  // namespace rgs
