// Per-tile alpha blending, forward and backward.  One 16x16 tile per 256-thread block:
// 4 wavefronts of 64 lanes, wavefront w owns pixel rows 4w..4w+3 of the tile, one pixel
// per lane.  Tile lists are staged through LDS in batches of 256 entries.
//
// Compiled with -ffp-contract=off: every per-pixel decision (power > 0, alpha < 1/255,
// the half-Gaussian box test, T(1-alpha) < 1e-4) is evaluated with the unfused
// single-precision expressions of K/cuda_rasterizer_hgs/forward.cu:338-392
// (K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian), so a pixel
// can only differ from that evaluation through the last-bit behaviour of exp().
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

// ---- forward (K/cuda_rasterizer_hgs/forward.cu:263-405) ---------------------------------------

// kCount = true is the instrumented twin used for work accounting: it writes no image and
// instead adds, over all pixels, the number of list entries visited by a live pixel (A), those
// with power <= 0 (B), those with alpha >= 1/255 (C), those inside the box (D), those blended
// (E), and the B and C counts restricted to entries up to each pixel's last blended one (B', C'),
// which is what the backward pass re-evaluates.
template <bool kCount>
__global__ __launch_bounds__(256) void blend_forward_kernel(BlendArgs a)
{
	__shared__ float2 s_xy[256];
	__shared__ float4 s_co[256];
	__shared__ float4 s_cd[256];  // r, g, b, view depth
	__shared__ float s_w[256];
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

	const uint2 range = a.ranges[tile];
	const int rounds = (int)((range.y - range.x + 255) / 256);
	int todo = (int)(range.y - range.x);

	bool done = !inside;
	float T = 1.0f;
	uint32_t last_contributor = 0;
	float C0 = 0.f, C1 = 0.f, C2 = 0.f, weight = 0.f, D = 0.f;
	uint32_t nA = 0, nB = 0, nC = 0, nD = 0, nE = 0, nB_last = 0, nC_last = 0;

	for (int i = 0; i < rounds; i++, todo -= 256) {
		const int alive = __ballot(!done) != 0ull;
		if (lane == 0)
			s_alive[i & 1][wave] = alive;
		const uint32_t src = range.x + (uint32_t)i * 256 + tid;
		if (src < range.y) {
			const uint32_t id = a.point_list[src];
			s_xy[tid] = a.xy[id];
			s_co[tid] = a.conic_opacity[id];
			s_w[tid] = a.clip_w[id];
			s_cd[tid] = float4{a.colors[3 * (size_t)id], a.colors[3 * (size_t)id + 1], a.colors[3 * (size_t)id + 2],
			                   a.depths[id]};
		}
		__syncthreads();
		if (!(s_alive[i & 1][0] | s_alive[i & 1][1] | s_alive[i & 1][2] | s_alive[i & 1][3]))
			break;

		const int count = todo < 256 ? todo : 256;
		for (int j = 0; !done && j < count; j++) {
			const float2 xy = s_xy[j];
			const float2 d = {xy.x - pixf.x, xy.y - pixf.y};
			const float4 co = s_co[j];
			const float power = -0.5f * (co.x * d.x * d.x + co.z * d.y * d.y) - co.y * d.x * d.y;
			if (kCount) nA++;
			if (power > 0.0f)
				continue;
			if (kCount) nB++;
			const float alpha = fminf(0.99f, co.w * expf(power));
			if (alpha < 1.0f / 255.0f)
				continue;
			if (kCount) nC++;
			if (clipped_by_box(ray, s_w[j], a.tanfovx, a.tanfovy, a.projinv, lo, hi))
				continue;
			if (kCount) nD++;
			const float test_T = T * (1 - alpha);
			if (test_T < 0.0001f) {
				done = true;
				continue;
			}
			if (kCount) {
				nE++;
				nB_last = nB;
				nC_last = nC;
			}
			const float4 cd = s_cd[j];
			C0 += cd.x * alpha * T;
			C1 += cd.y * alpha * T;
			C2 += cd.z * alpha * T;
			weight += alpha * T;
			D += cd.w * alpha * T;
			T = test_T;
			last_contributor = (uint32_t)(i * 256 + j + 1);
		}
		__syncthreads();
	}

	if (kCount) {
		const uint32_t c[7] = {nA, nB, nC, nD, nE, nB_last, nC_last};
#pragma unroll
		for (int q = 0; q < 7; q++) {
			const uint32_t tot = wave_inclusive_scan_u32(c[q]);
			if (lane == 63)
				atomicAdd(reinterpret_cast<unsigned long long*>(a.counters) + q, (unsigned long long)tot);
		}
		return;
	}
	if (inside) {
		const size_t plane = (size_t)a.H * a.W;
		a.n_contrib[pix_id] = last_contributor;
		a.out_color[pix_id] = C0 + T * a.bg[0];
		a.out_color[plane + pix_id] = C1 + T * a.bg[1];
		a.out_color[2 * plane + pix_id] = C2 + T * a.bg[2];
		a.out_alpha[pix_id] = weight;
		a.out_depth[pix_id] = D;
	}
}

// ---- backward (K/cuda_rasterizer_hgs/backward.cu:415-622) ---------------------------------------
// The tile list is walked back to front.  Each lane forms its pixel's ten partial
// derivatives for the staged Gaussian; they are summed over the wavefront with DPP,
// lane 63 adds the wave total to a per-batch LDS accumulator, and after the batch every
// thread flushes one Gaussian's ten sums with one global atomic each.

constexpr int kGradSlots = 10;  // mean2D x,y | conic xx,xy,yy | opacity | colour r,g,b | depth

__global__ __launch_bounds__(256) void blend_backward_kernel(BlendArgs a)
{
	__shared__ float2 s_xy[256];
	__shared__ float4 s_co[256];
	__shared__ float4 s_cd[256];
	__shared__ float s_w[256];
	__shared__ uint32_t s_id[256];
	__shared__ float s_acc[kGradSlots][256];
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

	const uint2 range = a.ranges[tile];
	const uint32_t last_contributor = inside ? a.n_contrib[pix_id] : 0u;

	// Entries at or beyond the largest last_contributor of the tile are skipped by every
	// pixel, so the walk starts there instead of at the end of the list.
	uint32_t wmax = last_contributor;
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		wmax = max(wmax, (uint32_t)__shfl_xor((int)wmax, off));
	if (lane == 0)
		s_max[wave] = wmax;
#pragma unroll
	for (int q = 0; q < kGradSlots; q++)
		s_acc[q][tid] = 0.f;
	__syncthreads();
	const uint32_t span = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3]));
	if (span == 0)
		return;
	const uint32_t back = range.x + span;  // one past the last entry any pixel uses
	const int rounds = (int)((span + 255) / 256);
	int todo = (int)span;

	const float T_final = inside ? (1 - a.out_alpha[pix_id]) : 0.f;
	float T = T_final;
	float accum_r = 0.f, accum_g = 0.f, accum_b = 0.f, accum_depth = 0.f, accum_alpha = 0.f;
	float g_r = 0.f, g_g = 0.f, g_b = 0.f, g_depth = 0.f, g_alpha = 0.f;
	if (inside) {
		g_r = a.dL_dpix[pix_id];
		g_g = a.dL_dpix[plane + pix_id];
		g_b = a.dL_dpix[2 * plane + pix_id];
		g_depth = a.dL_dpix_depth[pix_id];
		g_alpha = a.dL_dalpha[pix_id];
	}
	float last_alpha = 0.f, last_r = 0.f, last_g = 0.f, last_b = 0.f, last_depth = 0.f;
	const float ddelx_dx = 0.5 * a.W;
	const float ddely_dy = 0.5 * a.H;
	const float bg_dot_dpixel = (0.f + a.bg[0] * g_r + a.bg[1] * g_g) + a.bg[2] * g_b;

	for (int i = 0; i < rounds; i++, todo -= 256) {
		const uint32_t progress = (uint32_t)i * 256 + tid;
		if (progress < span) {
			const uint32_t id = a.point_list[back - progress - 1];
			s_id[tid] = id;
			s_xy[tid] = a.xy[id];
			s_co[tid] = a.conic_opacity[id];
			s_w[tid] = a.clip_w[id];
			s_cd[tid] = float4{a.colors[3 * (size_t)id], a.colors[3 * (size_t)id + 1], a.colors[3 * (size_t)id + 2],
			                   a.depths[id]};
		}
		__syncthreads();

		const int count = todo < 256 ? todo : 256;
		for (int j = 0; j < count; j++) {
			// 0-based position of this entry in the tile list
			const uint32_t entry = span - 1 - ((uint32_t)i * 256 + j);
			float v[kGradSlots];
			bool valid = false;
			if (inside && entry < last_contributor) {
				const float2 xy = s_xy[j];
				const float2 d = {xy.x - pixf.x, xy.y - pixf.y};
				const float4 co = s_co[j];
				const float power = -0.5f * (co.x * d.x * d.x + co.z * d.y * d.y) - co.y * d.x * d.y;
				if (!(power > 0.0f)) {
					const float G = expf(power);
					const float alpha = fminf(0.99f, co.w * G);
					if (!(alpha < 1.0f / 255.0f) &&
					    !clipped_by_box(ray, s_w[j], a.tanfovx, a.tanfovy, a.projinv, lo, hi)) {
						valid = true;
						T = T / (1.f - alpha);
						const float aT = alpha * T;
						const float4 cd = s_cd[j];
						float dL_dopa = 0.0f;
						accum_r = last_alpha * last_r + (1.f - last_alpha) * accum_r;
						last_r = cd.x;
						dL_dopa += (cd.x - accum_r) * g_r;
						accum_g = last_alpha * last_g + (1.f - last_alpha) * accum_g;
						last_g = cd.y;
						dL_dopa += (cd.y - accum_g) * g_g;
						accum_b = last_alpha * last_b + (1.f - last_alpha) * accum_b;
						last_b = cd.z;
						dL_dopa += (cd.z - accum_b) * g_b;
						accum_depth = last_alpha * last_depth + (1.f - last_alpha) * accum_depth;
						last_depth = cd.w;
						dL_dopa += (cd.w - accum_depth) * g_depth;
						accum_alpha = last_alpha + (1.f - last_alpha) * accum_alpha;
						dL_dopa += (1 - accum_alpha) * g_alpha;
						dL_dopa *= T;
						last_alpha = alpha;
						dL_dopa += (-T_final / (1.f - alpha)) * bg_dot_dpixel;

						const float dL_dG = co.w * dL_dopa;
						const float gdx = G * d.x;
						const float gdy = G * d.y;
						const float dG_ddelx = -gdx * co.x - gdy * co.y;
						const float dG_ddely = -gdy * co.z - gdx * co.y;
						v[0] = dL_dG * dG_ddelx * ddelx_dx;
						v[1] = dL_dG * dG_ddely * ddely_dy;
						v[2] = -0.5f * gdx * d.x * dL_dG;
						v[3] = -0.5f * gdx * d.y * dL_dG;
						v[4] = -0.5f * gdy * d.y * dL_dG;
						v[5] = G * dL_dopa;
						v[6] = aT * g_r;
						v[7] = aT * g_g;
						v[8] = aT * g_b;
						v[9] = aT * g_depth;
					}
				}
			}
			if (__ballot(valid) == 0ull)
				continue;
			if (!valid) {
#pragma unroll
				for (int q = 0; q < kGradSlots; q++)
					v[q] = 0.f;
			}
#pragma unroll
			for (int q = 0; q < kGradSlots; q++)
				v[q] = wave_sum_to_lane63(v[q]);
			if (lane == 63) {
#pragma unroll
				for (int q = 0; q < kGradSlots; q++)
					atomicAdd(&s_acc[q][j], v[q]);
			}
		}
		__syncthreads();

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
		hipLaunchKernelGGL(blend_forward_kernel<true>, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
	else
		hipLaunchKernelGGL(blend_forward_kernel<false>, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
}

void launch_blend_backward(const BlendArgs& a, hipStream_t s)
{
	stage_mark("blend_backward", s);
	hipLaunchKernelGGL(blend_backward_kernel, dim3(a.grid_x * a.grid_y), dim3(256), 0, s, a);
}

}  // namespace rgs
