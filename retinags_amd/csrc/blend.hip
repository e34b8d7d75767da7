// Per-tile alpha blending, forward and backward.  One 16x16 tile per 256-thread block:
// 4 wavefronts of 64 lanes, wavefront w owns the strip of pixel rows 4w..4w+3 of the tile,
// one pixel per lane.  Tile lists are staged through LDS in batches of 256 entries.
//
// Compiled with -ffp-contract=off: every per-pixel decision (power > 0, alpha < 1/255,
// the half-Gaussian box test, T(1-alpha) < 1e-4) is evaluated with the unfused
// single-precision expressions of K/cuda_rasterizer_hgs/forward.cu:338-392
// (K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian), so a pixel
// can only differ from that evaluation through the last-bit behaviour of exp().
//
// Most (pixel, Gaussian) visits of the reference loop end at "alpha < 1/255".  Two
// conservative filters remove such visits without changing any result:
//  * alpha >= 1/255 needs power >= -ln(255 * opacity).  The staging thread stores that floor
//    (minus a margin) with the Gaussian, and a wavefront skips an entry with one ballot when
//    no live lane reaches it, before exp() is evaluated.
//  * power >= floor describes an ellipse around the Gaussian's centre.  The staging thread
//    intersects the ellipse's bounding box with the four 16x4 strips of the tile and files the
//    entry only in the lists of the strips it can reach; each wavefront walks its own list,
//    four entries at a time so that the LDS reads and the four exponent evaluations overlap.
// Both filters only drop visits that the exact evaluation would have skipped too.
#include "rgs_kernels.h"

namespace rgs {

struct PixelRay {
	float ndc_x, ndc_y;  // pixel centre in NDC
};

// World-space point of the pixel's ray at clip-w `w`, tested against the submodel box
// (low, up] (K/cuda_rasterizer_hgs/forward.cu:360-372).  True when the sample is clipped.
__device__ __forceinline__ bool clipped_by_box(const PixelRay& ray, float w, float tanx, float tany,
                                               const float* __restrict__ m, const float3 lo, const float3 hi)
{
	const float3 ph = {ray.ndc_x * (w + 0.0000001f) * tanx, ray.ndc_y * (w + 0.0000001f) * tany, w};
	const float wx = m[0] * ph.x + m[4] * ph.y + m[8] * ph.z + m[12];
	const float wy = m[1] * ph.x + m[5] * ph.y + m[9] * ph.z + m[13];
	const float wz = m[2] * ph.x + m[6] * ph.y + m[10] * ph.z + m[14];
	return (wx <= lo.x) || (wx > hi.x) || (wy <= lo.y) || (wy > hi.y) || (wz <= lo.z) || (wz > hi.z);
}

// exp(x) for the exponents of the blend (x <= 0, modest magnitude): 2^(x log2 e) on the
// hardware exp2 unit, with the rounding error of the product x * log2(e) folded back in, which
// keeps the relative error at about one unit in the last place.  Forward and backward use
// the same function, so they take the same per-pixel decisions.
__device__ __forceinline__ float exp_of_exponent(float x)
{
	const float kLog2eHi = 1.44269502e+0f, kLog2eLo = 1.92596303e-8f;
	const float t = x * kLog2eHi;
	float r = __builtin_fmaf(x, kLog2eHi, -t);
	r = __builtin_fmaf(x, kLog2eLo, r);
	const float e = __builtin_amdgcn_exp2f(t);
	return __builtin_fmaf(e, r * 0.693147182f, e);
}

// Bit w set: some pixel of strip w (rows 4w..4w+3 of the tile whose first pixel is
// (x0, y0)) may reach power >= floor, judged by the bounding box (half-widths hx, hy) of the
// ellipse power >= floor.  Every comparison is written so that NaN keeps the entry.
__device__ __forceinline__ uint32_t reachable_strips(float gx, float gy, float hx, float hy, float floor, float x0,
                                                     float y0)
{
	if (floor > 0.f)
		return 0u;  // even power = 0 gives alpha < 1/255
	if ((gx + hx < x0) || (gx - hx > x0 + 15.f))
		return 0u;
	uint32_t mask = 0u;
#pragma unroll
	for (int w = 0; w < 4; w++) {
		const float ya = y0 + 4.f * w;
		if (!((gy + hy < ya) || (gy - hy > ya + 3.f)))
			mask |= 1u << w;
	}
	return mask;
}

// Where the rays of a whole tile, sampled at clip-w `w`, fall relative to the submodel box.
// The world-space sample is affine in the pixel's NDC coordinates, so its extremes over the
// tile are attained at the tile's corner pixels.  With a tolerance far above the rounding error
// of that affine map: kBoxInside = every pixel's exact test passes, kBoxOutside = every
// pixel's exact test fails, kBoxMixed = decide per pixel.
enum { kBoxMixed = 0, kBoxInside = 1, kBoxOutside = 2 };

__device__ __forceinline__ int classify_tile_against_box(float w, float tile_x0, float tile_y0, const BlendArgs& a,
                                                         const float3 lo, const float3 hi)
{
	const float* __restrict__ m = a.projinv;
	float pmin[3] = {INFINITY, INFINITY, INFINITY}, pmax[3] = {-INFINITY, -INFINITY, -INFINITY};
#pragma unroll
	for (int c = 0; c < 4; c++) {
		const float nx = pix_to_ndc(tile_x0 + ((c & 1) ? 15.f : 0.f), a.W);
		const float ny = pix_to_ndc(tile_y0 + ((c & 2) ? 15.f : 0.f), a.H);
		const float3 ph = {nx * (w + 0.0000001f) * a.tanfovx, ny * (w + 0.0000001f) * a.tanfovy, w};
		const float q[3] = {m[0] * ph.x + m[4] * ph.y + m[8] * ph.z + m[12], m[1] * ph.x + m[5] * ph.y + m[9] * ph.z + m[13],
		                    m[2] * ph.x + m[6] * ph.y + m[10] * ph.z + m[14]};
#pragma unroll
		for (int k = 0; k < 3; k++) {
			pmin[k] = fminf(pmin[k], q[k]);
			pmax[k] = fmaxf(pmax[k], q[k]);
		}
	}
	const float lov[3] = {lo.x, lo.y, lo.z}, hiv[3] = {hi.x, hi.y, hi.z};
	bool inside = true, outside = false;
#pragma unroll
	for (int k = 0; k < 3; k++) {
		const float tol = 1e-4f * fmaxf(fmaxf(fabsf(pmin[k]), fabsf(pmax[k])), 1.f);
		inside = inside && (pmin[k] > lov[k] + tol) && (pmax[k] < hiv[k] - tol);
		outside = outside || (pmax[k] < lov[k] - tol) || (pmin[k] > hiv[k] + tol);
	}
	// NaN anywhere leaves both flags false except `outside`, which a NaN cannot set
	return outside ? kBoxOutside : (inside ? kBoxInside : kBoxMixed);
}

constexpr int kPadSlot = 256;  // staged slot that never passes the floor test; pads lists to a multiple of 4

// Files the staging thread's entry (slot `tid`, reachable strips `strips`) in the per-strip
// lists.  Each staging wavefront owns a 64-entry segment of every strip's list and fills it in
// slot order, so walking segments 0..3 visits a strip's entries in list order.
__device__ __forceinline__ void file_in_strip_lists(uint32_t strips, int tid, uint16_t (*s_list)[256],
                                                    uint32_t (*s_count)[4])
{
	const int lane = tid & 63, wave = tid >> 6;
	const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
	for (int w = 0; w < 4; w++) {
		const bool mine = (strips >> w) & 1u;
		const uint64_t m = __ballot(mine);
		const uint32_t n = (uint32_t)__popcll(m);
		if (mine)
			s_list[w][wave * 64 + __popcll(m & below)] = (uint16_t)tid;
		if ((uint32_t)lane < ((4u - (n & 3u)) & 3u))
			s_list[w][wave * 64 + n + lane] = (uint16_t)kPadSlot;
		if (lane == 0)
			s_count[wave][w] = n;
	}
}

__device__ __forceinline__ float exponent_of(const float4 g, const float4 co, const float2 pixf, float2& d)
{
	d = float2{g.x - pixf.x, g.y - pixf.y};
	return -0.5f * (co.x * d.x * d.x + co.z * d.y * d.y) - co.y * d.x * d.y;
}

// ---- forward (K/cuda_rasterizer_hgs/forward.cu:263-405) ---------------------------------------

struct ForwardPixel {
	bool done;
	float T, C0, C1, C2, weight, D;
	uint32_t last_contributor;
};

__device__ __forceinline__ void forward_visit(ForwardPixel& p, bool candidate, float power, const float4 g,
                                              const float4 co, const float4* s_cd, int slot, uint32_t position,
                                              const PixelRay& ray, const BlendArgs& a, const float3 lo, const float3 hi)
{
	candidate = candidate && !p.done;
	if (__ballot(candidate) == 0ull)
		return;
	if (candidate) {
		const float alpha = fminf(0.99f, co.w * exp_of_exponent(power));
		// a NaN clip-w marks an entry whose whole tile footprint lies inside the box
		if (!(alpha < 1.0f / 255.0f) &&
		    !((g.w == g.w) && clipped_by_box(ray, g.w, a.tanfovx, a.tanfovy, a.projinv, lo, hi))) {
			const float test_T = p.T * (1 - alpha);
			if (test_T < 0.0001f) {
				p.done = true;
			} else {
				const float4 cd = s_cd[slot];
				p.C0 += cd.x * alpha * p.T;
				p.C1 += cd.y * alpha * p.T;
				p.C2 += cd.z * alpha * p.T;
				p.weight += alpha * p.T;
				p.D += cd.w * alpha * p.T;
				p.T = test_T;
				p.last_contributor = position;
			}
		}
	}
}

__global__ __launch_bounds__(256) void blend_forward_kernel(BlendArgs a)
{
	__shared__ float4 s_geom[257];   // pixel x, pixel y, exponent floor, clip w
	__shared__ float4 s_conic[257];  // conic xx, xy, yy, opacity
	__shared__ float4 s_cd[256];     // r, g, b, view depth
	__shared__ __attribute__((aligned(8))) uint16_t s_list[4][256];
	__shared__ uint32_t s_count[4][4];  // [staging wave][strip]
	__shared__ int s_alive[2][4];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int tile = blockIdx.x;
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const uint32_t pix_id = (uint32_t)a.W * py + px;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const float3 lo = {a.range_low[0], a.range_low[1], a.range_low[2]};
	const float3 hi = {a.range_up[0], a.range_up[1], a.range_up[2]};
	const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);

	const uint2 range = a.ranges[tile];
	const int rounds = (int)((range.y - range.x + 255) / 256);

	ForwardPixel p = {!inside, 1.0f, 0.f, 0.f, 0.f, 0.f, 0.f, 0u};
	if (tid == 0) {
		s_geom[kPadSlot] = float4{0.f, 0.f, INFINITY, 0.f};
		s_conic[kPadSlot] = float4{0.f, 0.f, 0.f, 0.f};
	}

	for (int i = 0; i < rounds; i++) {
		uint64_t live = __ballot(!p.done);
		if (lane == 0)
			s_alive[i & 1][wave] = live != 0ull;
		const uint32_t src = range.x + (uint32_t)i * 256 + tid;
		uint32_t strips = 0u;
		if (src < range.y) {
			const uint32_t id = a.point_list[src];
			const float4* rec = a.record + 4 * (size_t)id;
			const float4 geom = rec[0], co = rec[1], cd = rec[2], half = rec[3];
			strips = reachable_strips(geom.x, geom.y, half.x, half.y, geom.z, tile_x0, tile_y0);
			float w = geom.w;
			if (strips) {
				const int where = classify_tile_against_box(w, tile_x0, tile_y0, a, lo, hi);
				if (where == kBoxOutside)
					strips = 0u;
				if (where == kBoxInside)
					w = __int_as_float(0x7FC00000);
			}
			s_geom[tid] = float4{geom.x, geom.y, geom.z, w};
			s_conic[tid] = co;
			s_cd[tid] = cd;
		}
		file_in_strip_lists(strips, tid, s_list, s_count);
		__syncthreads();
		if (!(s_alive[i & 1][0] | s_alive[i & 1][1] | s_alive[i & 1][2] | s_alive[i & 1][3]))
			break;

		for (int seg = 0; seg < 4 && live != 0ull; seg++) {
			const int n = (int)s_count[seg][wave];
			for (int k = 0; k < n && live != 0ull; k += 4) {
				const uint2 packed = *reinterpret_cast<const uint2*>(&s_list[wave][seg * 64 + k]);
				const int j0 = packed.x & 0xFFFFu, j1 = packed.x >> 16, j2 = packed.y & 0xFFFFu, j3 = packed.y >> 16;
				const float4 g0 = s_geom[j0], g1 = s_geom[j1], g2 = s_geom[j2], g3 = s_geom[j3];
				const float4 c0 = s_conic[j0], c1 = s_conic[j1], c2 = s_conic[j2], c3 = s_conic[j3];
				float2 d;
				const float w0 = exponent_of(g0, c0, pixf, d), w1 = exponent_of(g1, c1, pixf, d),
				            w2 = exponent_of(g2, c2, pixf, d), w3 = exponent_of(g3, c3, pixf, d);
				// written with negations so that a NaN exponent is kept, as in the exact loop
				const bool q0 = !(w0 > 0.0f) && !(w0 < g0.z), q1 = !(w1 > 0.0f) && !(w1 < g1.z),
				           q2 = !(w2 > 0.0f) && !(w2 < g2.z), q3 = !(w3 > 0.0f) && !(w3 < g3.z);
				if (__ballot((q0 | q1 | q2 | q3) && !p.done) == 0ull)
					continue;
				const uint32_t base = (uint32_t)i * 256 + 1;
				forward_visit(p, q0, w0, g0, c0, s_cd, j0, base + j0, ray, a, lo, hi);
				forward_visit(p, q1, w1, g1, c1, s_cd, j1, base + j1, ray, a, lo, hi);
				forward_visit(p, q2, w2, g2, c2, s_cd, j2, base + j2, ray, a, lo, hi);
				forward_visit(p, q3, w3, g3, c3, s_cd, j3, base + j3, ray, a, lo, hi);
				live = __ballot(!p.done);
			}
		}
		__syncthreads();
	}

	if (inside) {
		const size_t plane = (size_t)a.H * a.W;
		a.n_contrib[pix_id] = p.last_contributor;
		a.out_color[pix_id] = p.C0 + p.T * a.bg[0];
		a.out_color[plane + pix_id] = p.C1 + p.T * a.bg[1];
		a.out_color[2 * plane + pix_id] = p.C2 + p.T * a.bg[2];
		a.out_alpha[pix_id] = p.weight;
		a.out_depth[pix_id] = p.D;
	}
}

// Work accounting: the reference loop taken literally, one list entry at a time with no
// filter, counting over all pixels the entries visited by a live pixel (A), those with
// power <= 0 (B), with alpha >= 1/255 (C), inside the box (D), blended (E), and B and C
// restricted to entries up to each pixel's last blended one (the backward's share).
__global__ __launch_bounds__(256) void blend_count_kernel(BlendArgs a)
{
	__shared__ float4 s_geom[256];
	__shared__ float4 s_conic[256];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int tile = blockIdx.x;
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const float3 lo = {a.range_low[0], a.range_low[1], a.range_low[2]};
	const float3 hi = {a.range_up[0], a.range_up[1], a.range_up[2]};
	const uint2 range = a.ranges[tile];
	const int rounds = (int)((range.y - range.x + 255) / 256);
	int todo = (int)(range.y - range.x);

	bool done = !inside;
	float T = 1.0f;
	uint32_t nA = 0, nB = 0, nC = 0, nD = 0, nE = 0, nB_last = 0, nC_last = 0;
	for (int i = 0; i < rounds; i++, todo -= 256) {
		__syncthreads();
		const uint32_t src = range.x + (uint32_t)i * 256 + tid;
		if (src < range.y) {
			const uint32_t id = a.point_list[src];
			const float2 xy = a.xy[id];
			s_geom[tid] = float4{xy.x, xy.y, 0.f, a.clip_w[id]};
			s_conic[tid] = a.conic_opacity[id];
		}
		__syncthreads();
		const int count = todo < 256 ? todo : 256;
		for (int j = 0; !done && j < count; j++) {
			const float4 g = s_geom[j];
			const float4 co = s_conic[j];
			float2 d;
			const float power = exponent_of(g, co, pixf, d);
			nA++;
			if (power > 0.0f)
				continue;
			nB++;
			const float alpha = fminf(0.99f, co.w * expf(power));
			if (alpha < 1.0f / 255.0f)
				continue;
			nC++;
			if (clipped_by_box(ray, g.w, a.tanfovx, a.tanfovy, a.projinv, lo, hi))
				continue;
			nD++;
			const float test_T = T * (1 - alpha);
			if (test_T < 0.0001f) {
				done = true;
				continue;
			}
			nE++;
			nB_last = nB;
			nC_last = nC;
			T = test_T;
		}
	}
	const uint32_t c[7] = {nA, nB, nC, nD, nE, nB_last, nC_last};
#pragma unroll
	for (int q = 0; q < 7; q++) {
		const uint32_t tot = wave_inclusive_scan_u32(c[q]);
		if (lane == 63)
			atomicAdd(reinterpret_cast<unsigned long long*>(a.counters) + q, (unsigned long long)tot);
	}
}

// ---- backward (K/cuda_rasterizer_hgs/backward.cu:415-622) ---------------------------------------
// The tile list is walked back to front.  Each lane forms its pixel's ten partial
// derivatives for the staged Gaussian; they are summed over the wavefront with DPP,
// lane 63 adds the wave total to a per-batch LDS accumulator, and after the batch every
// thread flushes one Gaussian's ten sums with one global atomic each.

constexpr int kGradSlots = 10;  // mean2D x,y | conic xx,xy,yy | opacity | colour r,g,b | depth

struct BackwardPixel {
	float T, T_final;
	float accum_r, accum_g, accum_b, accum_depth, accum_alpha;
	float last_alpha, last_r, last_g, last_b, last_depth;
	float g_r, g_g, g_b, g_depth, g_alpha;
	float bg_dot_dpixel, ddelx_dx, ddely_dy;
};

__device__ __forceinline__ void backward_visit(BackwardPixel& p, bool candidate, float power, const float4 g,
                                               const float4 co, const float2 pixf, const float4* s_cd,
                                               float (*s_acc)[256], int slot, const PixelRay& ray, const BlendArgs& a,
                                               const float3 lo, const float3 hi, int lane)
{
	if (__ballot(candidate) == 0ull)
		return;
	float v[kGradSlots];
#pragma unroll
	for (int q = 0; q < kGradSlots; q++)
		v[q] = 0.f;
	bool valid = false;
	if (candidate) {
		const float2 d = {g.x - pixf.x, g.y - pixf.y};
		const float G = exp_of_exponent(power);
		const float alpha = fminf(0.99f, co.w * G);
		if (!(alpha < 1.0f / 255.0f) &&
		    !((g.w == g.w) && clipped_by_box(ray, g.w, a.tanfovx, a.tanfovy, a.projinv, lo, hi))) {
			valid = true;
			p.T = p.T / (1.f - alpha);
			const float aT = alpha * p.T;
			const float4 cd = s_cd[slot];
			float dL_dopa = 0.0f;
			p.accum_r = p.last_alpha * p.last_r + (1.f - p.last_alpha) * p.accum_r;
			p.last_r = cd.x;
			dL_dopa += (cd.x - p.accum_r) * p.g_r;
			p.accum_g = p.last_alpha * p.last_g + (1.f - p.last_alpha) * p.accum_g;
			p.last_g = cd.y;
			dL_dopa += (cd.y - p.accum_g) * p.g_g;
			p.accum_b = p.last_alpha * p.last_b + (1.f - p.last_alpha) * p.accum_b;
			p.last_b = cd.z;
			dL_dopa += (cd.z - p.accum_b) * p.g_b;
			p.accum_depth = p.last_alpha * p.last_depth + (1.f - p.last_alpha) * p.accum_depth;
			p.last_depth = cd.w;
			dL_dopa += (cd.w - p.accum_depth) * p.g_depth;
			p.accum_alpha = p.last_alpha + (1.f - p.last_alpha) * p.accum_alpha;
			dL_dopa += (1 - p.accum_alpha) * p.g_alpha;
			dL_dopa *= p.T;
			p.last_alpha = alpha;
			dL_dopa += (-p.T_final / (1.f - alpha)) * p.bg_dot_dpixel;

			const float dL_dG = co.w * dL_dopa;
			const float gdx = G * d.x;
			const float gdy = G * d.y;
			const float dG_ddelx = -gdx * co.x - gdy * co.y;
			const float dG_ddely = -gdy * co.z - gdx * co.y;
			v[0] = dL_dG * dG_ddelx * p.ddelx_dx;
			v[1] = dL_dG * dG_ddely * p.ddely_dy;
			v[2] = -0.5f * gdx * d.x * dL_dG;
			v[3] = -0.5f * gdx * d.y * dL_dG;
			v[4] = -0.5f * gdy * d.y * dL_dG;
			v[5] = G * dL_dopa;
			v[6] = aT * p.g_r;
			v[7] = aT * p.g_g;
			v[8] = aT * p.g_b;
			v[9] = aT * p.g_depth;
		}
	}
	if (__ballot(valid) == 0ull)
		return;
#pragma unroll
	for (int q = 0; q < kGradSlots; q++)
		v[q] = wave_sum_to_lane63(v[q]);
	if (lane == 63) {
#pragma unroll
		for (int q = 0; q < kGradSlots; q++)
			atomicAdd(&s_acc[q][slot], v[q]);
	}
}

__global__ __launch_bounds__(256) void blend_backward_kernel(BlendArgs a)
{
	__shared__ float4 s_geom[257];
	__shared__ float4 s_conic[257];
	__shared__ float4 s_cd[256];
	__shared__ uint32_t s_id[256];
	__shared__ float s_acc[kGradSlots][256];
	__shared__ __attribute__((aligned(8))) uint16_t s_list[4][256];
	__shared__ uint32_t s_count[4][4];
	__shared__ uint32_t s_max[4];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int tile = blockIdx.x;
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const uint32_t pix_id = (uint32_t)a.W * py + px;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const float3 lo = {a.range_low[0], a.range_low[1], a.range_low[2]};
	const float3 hi = {a.range_up[0], a.range_up[1], a.range_up[2]};
	const size_t plane = (size_t)a.H * a.W;
	const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);

	const uint2 range = a.ranges[tile];
	const uint32_t last_contributor = inside ? a.n_contrib[pix_id] : 0u;

	// Entries at or beyond the largest last_contributor of the tile are skipped by every
	// pixel, so the walk starts there instead of at the end of the list; likewise a strip's
	// list only takes entries below the largest last_contributor of that strip's 64 pixels.
	uint32_t wave_span = last_contributor;
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		wave_span = max(wave_span, (uint32_t)__shfl_xor((int)wave_span, off));
	if (lane == 0)
		s_max[wave] = wave_span;
#pragma unroll
	for (int q = 0; q < kGradSlots; q++)
		s_acc[q][tid] = 0.f;
	if (tid == 0) {
		s_geom[kPadSlot] = float4{0.f, 0.f, INFINITY, 0.f};
		s_conic[kPadSlot] = float4{0.f, 0.f, 0.f, 0.f};
	}
	__syncthreads();
	const uint32_t span0 = s_max[0], span1 = s_max[1], span2 = s_max[2], span3 = s_max[3];
	const uint32_t span = max(max(span0, span1), max(span2, span3));
	if (span == 0)
		return;
	const uint32_t back = range.x + span;  // one past the last entry any pixel uses
	const int rounds = (int)((span + 255) / 256);
	int todo = (int)span;

	BackwardPixel p;
	p.T_final = inside ? (1 - a.out_alpha[pix_id]) : 0.f;
	p.T = p.T_final;
	p.accum_r = p.accum_g = p.accum_b = p.accum_depth = p.accum_alpha = 0.f;
	p.last_alpha = p.last_r = p.last_g = p.last_b = p.last_depth = 0.f;
	p.g_r = p.g_g = p.g_b = p.g_depth = p.g_alpha = 0.f;
	if (inside) {
		p.g_r = a.dL_dpix[pix_id];
		p.g_g = a.dL_dpix[plane + pix_id];
		p.g_b = a.dL_dpix[2 * plane + pix_id];
		p.g_depth = a.dL_dpix_depth[pix_id];
		p.g_alpha = a.dL_dalpha[pix_id];
	}
	p.ddelx_dx = 0.5 * a.W;
	p.ddely_dy = 0.5 * a.H;
	p.bg_dot_dpixel = (0.f + a.bg[0] * p.g_r + a.bg[1] * p.g_g) + a.bg[2] * p.g_b;

	for (int i = 0; i < rounds; i++, todo -= 256) {
		const uint32_t progress = (uint32_t)i * 256 + tid;
		uint32_t strips = 0u;
		if (progress < span) {
			const uint32_t entry = span - 1 - progress;  // 0-based position in the tile list
			const uint32_t id = a.point_list[back - progress - 1];
			const float4* rec = a.record + 4 * (size_t)id;
			const float4 geom = rec[0], co = rec[1], cd = rec[2], half = rec[3];
			strips = reachable_strips(geom.x, geom.y, half.x, half.y, geom.z, tile_x0, tile_y0);
			strips &= (entry < span0 ? 1u : 0u) | (entry < span1 ? 2u : 0u) | (entry < span2 ? 4u : 0u) |
			          (entry < span3 ? 8u : 0u);
			float w = geom.w;
			if (strips) {
				const int where = classify_tile_against_box(w, tile_x0, tile_y0, a, lo, hi);
				if (where == kBoxOutside)
					strips = 0u;
				if (where == kBoxInside)
					w = __int_as_float(0x7FC00000);
			}
			s_id[tid] = id;
			s_geom[tid] = float4{geom.x, geom.y, geom.z, w};
			s_conic[tid] = co;
			s_cd[tid] = cd;
		}
		file_in_strip_lists(strips, tid, s_list, s_count);
		__syncthreads();

		for (int seg = 0; seg < 4; seg++) {
			const int n = (int)s_count[seg][wave];
			for (int k = 0; k < n; k += 4) {
				const uint2 packed = *reinterpret_cast<const uint2*>(&s_list[wave][seg * 64 + k]);
				const int j0 = packed.x & 0xFFFFu, j1 = packed.x >> 16, j2 = packed.y & 0xFFFFu, j3 = packed.y >> 16;
				const float4 g0 = s_geom[j0], g1 = s_geom[j1], g2 = s_geom[j2], g3 = s_geom[j3];
				const float4 c0 = s_conic[j0], c1 = s_conic[j1], c2 = s_conic[j2], c3 = s_conic[j3];
				float2 d;
				const float w0 = exponent_of(g0, c0, pixf, d), w1 = exponent_of(g1, c1, pixf, d),
				            w2 = exponent_of(g2, c2, pixf, d), w3 = exponent_of(g3, c3, pixf, d);
				// position of slot j in the tile list: span - 1 - (i * 256 + j)
				const uint32_t top = span - 1 - (uint32_t)i * 256;
				const bool q0 = (top - j0 < last_contributor) && !(w0 > 0.0f) && !(w0 < g0.z),
				           q1 = (top - j1 < last_contributor) && !(w1 > 0.0f) && !(w1 < g1.z),
				           q2 = (top - j2 < last_contributor) && !(w2 > 0.0f) && !(w2 < g2.z),
				           q3 = (top - j3 < last_contributor) && !(w3 > 0.0f) && !(w3 < g3.z);
				if (__ballot(q0 | q1 | q2 | q3) == 0ull)
					continue;
				backward_visit(p, q0, w0, g0, c0, pixf, s_cd, s_acc, j0, ray, a, lo, hi, lane);
				backward_visit(p, q1, w1, g1, c1, pixf, s_cd, s_acc, j1, ray, a, lo, hi, lane);
				backward_visit(p, q2, w2, g2, c2, pixf, s_cd, s_acc, j2, ray, a, lo, hi, lane);
				backward_visit(p, q3, w3, g3, c3, pixf, s_cd, s_acc, j3, ray, a, lo, hi, lane);
			}
		}
		__syncthreads();

		const int count = todo < 256 ? todo : 256;
		if (tid < count) {
			const size_t id = s_id[tid];
			float r[kGradSlots];
#pragma unroll
			for (int q = 0; q < kGradSlots; q++) {
				r[q] = s_acc[q][tid];
				s_acc[q][tid] = 0.f;
			}
			if (r[0] != 0.f) unsafeAtomicAdd(&a.dL_dmean2D[3 * id + 0], r[0]);
			if (r[1] != 0.f) unsafeAtomicAdd(&a.dL_dmean2D[3 * id + 1], r[1]);
			if (r[2] != 0.f) unsafeAtomicAdd(&a.dL_dconic[4 * id + 0], r[2]);
			if (r[3] != 0.f) unsafeAtomicAdd(&a.dL_dconic[4 * id + 1], r[3]);
			if (r[4] != 0.f) unsafeAtomicAdd(&a.dL_dconic[4 * id + 3], r[4]);
			if (r[5] != 0.f) unsafeAtomicAdd(&a.dL_dopacity[id], r[5]);
			if (r[6] != 0.f) unsafeAtomicAdd(&a.dL_dcolors[3 * id + 0], r[6]);
			if (r[7] != 0.f) unsafeAtomicAdd(&a.dL_dcolors[3 * id + 1], r[7]);
			if (r[8] != 0.f) unsafeAtomicAdd(&a.dL_dcolors[3 * id + 2], r[8]);
			if (r[9] != 0.f) unsafeAtomicAdd(&a.dL_ddepths[id], r[9]);
		}
	}
}

void launch_blend_forward(const BlendArgs& a, hipStream_t s)
{
	stage_mark(a.counters ? "blend_count" : "blend_forward", s);
	if (a.counters)
		hipLaunchKernelGGL(blend_count_kernel, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
	else
		hipLaunchKernelGGL(blend_forward_kernel, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
}

void launch_blend_backward(const BlendArgs& a, hipStream_t s)
{
	stage_mark("blend_backward", s);
	hipLaunchKernelGGL(blend_backward_kernel, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
}

}  // namespace rgs
