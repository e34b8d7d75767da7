// Per-Gaussian stages: visibility marking, forward preprocess (projection, EWA
// covariance, conic, radius, tile rectangle, SH colour) and the fused backward
// preprocess.  One thread per Gaussian (in the backward: per rendered Gaussian).
//
// This file is compiled with -ffp-contract=off: radii, tile counts, pixel
// centres and depth bits feed the integer stages and must equal the unfused
// single-precision evaluation of the reference's expressions
// (K/cuda_rasterizer_hgs/forward.cu:74-258 with
//  K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian).
#include "rgs_kernels.h"

namespace rgs {

__device__ const float kShC0 = 0.28209479177387814f;
__device__ const float kShC1 = 0.4886025119029199f;
__device__ const float kShC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                                   -1.0925484305920792f, 0.5462742152960396f};
__device__ const float kShC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                                   0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                                   -0.5900435899266435f};

// ---- visibility (K/cuda_rasterizer_hgs/rasterizer_impl.cu:54-66, auxiliary.h:155-180) ----

__global__ __launch_bounds__(256) void mark_visible_kernel(int P, const float* __restrict__ means,
                                                            const float* __restrict__ view, uint8_t* __restrict__ present)
{
	const int idx = blockIdx.x * 256 + threadIdx.x;
	if (idx >= P)
		return;
	const float3 p = {means[3 * (size_t)idx], means[3 * (size_t)idx + 1], means[3 * (size_t)idx + 2]};
	const float3 pv = xform_point_4x3(p, view);
	present[idx] = !(pv.z <= 0.2f);
}

// ---- shared pieces ------------------------------------------------------------------------

// World-space covariance from scale and the quaternion as given (r, x, y, z)
// (K/cuda_rasterizer_hgs/forward.cu:118-152): Sigma = (S R)^T (S R).
__device__ __forceinline__ M3 rotation_cols(const float4 q)
{
	const float r = q.x, x = q.y, y = q.z, z = q.w;
	return m3_cols(1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
	               2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
	               2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
}

__device__ __forceinline__ void covariance3d(const float3 scale, float mod, const float4 rot, float* cov6)
{
	M3 S = m3_cols(1.f, 0.f, 0.f, 0.f, 1.f, 0.f, 0.f, 0.f, 1.f);
	S.c[0][0] = mod * scale.x;
	S.c[1][1] = mod * scale.y;
	S.c[2][2] = mod * scale.z;
	const M3 R = rotation_cols(rot);
	const M3 M = m3_mul(S, R);
	const M3 Sigma = m3_mul(m3_transpose(M), M);
	cov6[0] = Sigma.c[0][0];
	cov6[1] = Sigma.c[0][1];
	cov6[2] = Sigma.c[0][2];
	cov6[3] = Sigma.c[1][1];
	cov6[4] = Sigma.c[1][2];
	cov6[5] = Sigma.c[2][2];
}

// EWA projection of the 3D covariance (K/cuda_rasterizer_hgs/forward.cu:74-113).
struct Ewa {
	float3 t;            // view-space mean, x and y clamped to the guard frustum
	float txtz, tytz, limx, limy;
	M3 W, T, Vrk, cov;   // cov before the 0.3 low-pass
};

__device__ __forceinline__ Ewa ewa_project(const float3 mean, float fx, float fy, float tanx, float tany,
                                           const float* cov6, const float* __restrict__ view)
{
	Ewa e;
	e.t = xform_point_4x3(mean, view);
	e.limx = 1.3f * tanx;
	e.limy = 1.3f * tany;
	e.txtz = e.t.x / e.t.z;
	e.tytz = e.t.y / e.t.z;
	e.t.x = fminf(e.limx, fmaxf(-e.limx, e.txtz)) * e.t.z;
	e.t.y = fminf(e.limy, fmaxf(-e.limy, e.tytz)) * e.t.z;
	const M3 J = m3_cols(fx / e.t.z, 0.0f, -(fx * e.t.x) / (e.t.z * e.t.z),
	                     0.0f, fy / e.t.z, -(fy * e.t.y) / (e.t.z * e.t.z),
	                     0.f, 0.f, 0.f);
	e.W = m3_cols(view[0], view[4], view[8], view[1], view[5], view[9], view[2], view[6], view[10]);
	e.T = m3_mul(e.W, J);
	e.Vrk = m3_cols(cov6[0], cov6[1], cov6[2], cov6[1], cov6[3], cov6[4], cov6[2], cov6[4], cov6[5]);
	e.cov = m3_mul(m3_mul(m3_transpose(e.T), m3_transpose(e.Vrk)), e.T);
	return e;
}

// SH (degree <= 3) to RGB for one colour channel (K/cuda_rasterizer_hgs/forward.cu:20-71).
// sh points at coefficient 0 of this channel; consecutive coefficients are 3 floats apart.
__device__ __forceinline__ float sh_channel(int deg, float x, float y, float z, const float* __restrict__ sh)
{
#define SHK(k) sh[3 * (k)]
	float result = kShC0 * SHK(0);
	if (deg > 0) {
		result = result - kShC1 * y * SHK(1) + kShC1 * z * SHK(2) - kShC1 * x * SHK(3);
		if (deg > 1) {
			const float xx = x * x, yy = y * y, zz = z * z;
			const float xy = x * y, yz = y * z, xz = x * z;
			result = result + kShC2[0] * xy * SHK(4) + kShC2[1] * yz * SHK(5) +
			         kShC2[2] * (2.0f * zz - xx - yy) * SHK(6) + kShC2[3] * xz * SHK(7) +
			         kShC2[4] * (xx - yy) * SHK(8);
			if (deg > 2) {
				result = result + kShC3[0] * y * (3.0f * xx - yy) * SHK(9) + kShC3[1] * xy * z * SHK(10) +
				         kShC3[2] * y * (4.0f * zz - xx - yy) * SHK(11) +
				         kShC3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * SHK(12) +
				         kShC3[4] * x * (4.0f * zz - xx - yy) * SHK(13) + kShC3[5] * z * (xx - yy) * SHK(14) +
				         kShC3[6] * x * (xx - 3.0f * yy) * SHK(15);
			}
		}
	}
#undef SHK
	return result + 0.5f;
}

// An SH row of up to 48 floats, read 16 bytes at a time into registers.  The evaluation reads
// coefficient k of channel c at float 3 k + c; done with one 4-byte load each, a wavefront's 48
// loads all touch 64 different cache lines and the address unit, not memory, sets the pace.
// Only the floats the active degree needs are read (3 (deg + 1)^2, rounded up to four).
constexpr int kShRegs = 48;

__device__ __forceinline__ void load_sh_row(const float* __restrict__ row, int deg, float (&out)[kShRegs])
{
	const int needed = 3 * (deg + 1) * (deg + 1);
#pragma unroll
	for (int k = 0; k < kShRegs; k += 4) {
		float4 v = {0.f, 0.f, 0.f, 0.f};
		if (k < needed)
			v = *reinterpret_cast<const float4*>(row + k);
		out[k] = v.x;
		out[k + 1] = v.y;
		out[k + 2] = v.z;
		out[k + 3] = v.w;
	}
}

// ---- forward preprocess (K/cuda_rasterizer_hgs/forward.cu:155-258) -------------------------

// SH rows through LDS: a wavefront reads the rows of its rendered Gaussians together, 16 lanes
// per row and 16 bytes per lane (a load instruction then covers four rows instead of one piece of
// 64), parks them in LDS and every lane picks up its own row.  32 rows at a time.
constexpr int kRecordStride = 5;  // float4 per parked record: 20 words, so 8 lanes' 16-byte writes meet no bank twice
static_assert(64 * kRecordStride <= 32 * 13, "the parked records share the rows' space");

__device__ __forceinline__ void wave_lds_fence()
{
	// orders the LDS traffic of one wavefront around a hand-over between its lanes
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
	__builtin_amdgcn_wave_barrier();
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kShRowStride = 13;  // float4 per parked row: 52 words, so 8 lanes' 16-byte reads meet no bank twice

__global__ __launch_bounds__(256) void preprocess_forward_kernel(Batch<PreprocessArgs> batch)
{
	__shared__ uint32_t s_scan[8];
	__shared__ float4 s_rows[4][32 * kShRowStride];
	__shared__ uint8_t s_listed[4][64];
	const PreprocessArgs& a = batch.job[blockIdx.y];  // one job per submodel of the frame
	const int idx = blockIdx.x * 256 + threadIdx.x;
	// the scratch of the depth sort that follows is cleared here, which saves a launch
	for (size_t w = (size_t)idx; w < a.clear_words; w += (size_t)gridDim.x * 256)
		a.clear[w] = 0u;
	if ((int)blockIdx.x * 256 >= a.P)
		return;  // the launch is sized for the job with the most Gaussians
	uint32_t touched = 0;
	bool rendered = false;
	float2 pix = {0.f, 0.f};
	float4 conic_o = {0.f, 0.f, 0.f, 0.f};
	float hom_w = 0.f, view_z = 0.f, my_radius = 0.f;
	float3 p = {0.f, 0.f, 0.f};

	if (idx < a.P) {
		do {
			p = float3{a.means[3 * (size_t)idx], a.means[3 * (size_t)idx + 1], a.means[3 * (size_t)idx + 2]};
			const float3 p_view = xform_point_4x3(p, a.view);
			if (p_view.z <= 0.2f)
				break;
			const float4 p_hom = xform_point_4x4(p, a.proj);
			const float p_w = 1.0f / (p_hom.w + 0.0000001f);
			const float2 p_proj = {p_hom.x * p_w, p_hom.y * p_w};

			float cov6[6];
			if (a.cov3D_precomp) {
#pragma unroll
				for (int i = 0; i < 6; i++)
					cov6[i] = a.cov3D_precomp[6 * (size_t)idx + i];
			} else {
				const float3 sc = {a.scales[3 * (size_t)idx], a.scales[3 * (size_t)idx + 1], a.scales[3 * (size_t)idx + 2]};
				const float4 q = reinterpret_cast<const float4*>(a.rotations)[idx];
				covariance3d(sc, a.scale_modifier, q, cov6);
			}
			Ewa e = ewa_project(p, a.focal_x, a.focal_y, a.tanfovx, a.tanfovy, cov6, a.view);
			const float cx = e.cov.c[0][0] + 0.3f, cy = e.cov.c[0][1], cz = e.cov.c[1][1] + 0.3f;

			const float det = (cx * cz - cy * cy);
			if (det == 0.0f)
				break;
			const float det_inv = 1.f / det;

			const float mid = 0.5f * (cx + cz);
			const float lambda1 = mid + sqrtf(fmaxf(0.1f, mid * mid - det));
			const float lambda2 = mid - sqrtf(fmaxf(0.1f, mid * mid - det));
			const float radius = ceilf(3.f * sqrtf(fmaxf(lambda1, lambda2)));
			const float2 at = {ndc_to_pix(p_proj.x, a.W), ndc_to_pix(p_proj.y, a.H)};
			const TileRect rc = tile_rect(at.x, at.y, (int)radius, a.grid_x, a.grid_y);
			const uint32_t ntiles = (rc.x1 - rc.x0) * (rc.y1 - rc.y0);
			if (ntiles == 0)
				break;
			conic_o = float4{cz * det_inv, -cy * det_inv, cx * det_inv, a.opacities[idx]};
			pix = at;
			hom_w = p_hom.w;
			view_z = p_view.z;
			my_radius = radius;
			touched = ntiles;
			rendered = true;
		} while (false);
	}

	// the rendered Gaussians of the wavefront, listed in lane order
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const uint64_t seen = lanes_where(rendered);
	const int n_seen = __popcll(seen);
	const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(seen >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)seen, 0u));
	float4* parked = s_rows[wave];
	uint8_t* listed = s_listed[wave];
	if (rendered)
		listed[rank] = (uint8_t)lane;
	wave_lds_fence();

	float3 col = {0.f, 0.f, 0.f};
	uint32_t clamp_bits = 0;
	if (a.colors_precomp) {
		if (rendered)
			col = float3{a.colors_precomp[3 * (size_t)idx], a.colors_precomp[3 * (size_t)idx + 1],
			             a.colors_precomp[3 * (size_t)idx + 2]};
	} else {
		const float3 cam = {a.campos[0], a.campos[1], a.campos[2]};
		const float3 dir = {p.x - cam.x, p.y - cam.y, p.z - cam.z};
		const float len = sqrtf(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
		const float dx = dir.x / len, dy = dir.y / len, dz = dir.z / len;
		float raw[3] = {0.f, 0.f, 0.f};
		if (a.sh_rows_by_16_bytes) {
			const int piece = lane & 15, sub = lane >> 4;
			const int row_pieces = a.M * 3 / 4;
			const int needed = 3 * (a.D + 1) * (a.D + 1);
			const float4* __restrict__ rows =
			    reinterpret_cast<const float4*>(a.shs) + (size_t)(idx - lane) * row_pieces;
			for (int base = 0; base < n_seen; base += 32) {
				float4 v[8];
#pragma unroll
				for (int r = 0; r < 8; r++) {
					const int slot = base + 4 * r + sub;
					v[r] = float4{0.f, 0.f, 0.f, 0.f};
					if (4 * piece < needed && slot < n_seen)
						v[r] = rows[(size_t)listed[slot] * row_pieces + piece];
				}
#pragma unroll
				for (int r = 0; r < 8; r++)
					if (piece < 12)
						parked[(4 * r + sub) * kShRowStride + piece] = v[r];
				wave_lds_fence();
				if (rendered && rank >= base && rank < base + 32) {
					float row[kShRegs];
					const float4* mine = parked + (rank - base) * kShRowStride;
#pragma unroll
					for (int k = 0; k < kShRegs; k += 4) {
						float4 q = {0.f, 0.f, 0.f, 0.f};
						if (k < needed)
							q = mine[k / 4];
						row[k] = q.x;
						row[k + 1] = q.y;
						row[k + 2] = q.z;
						row[k + 3] = q.w;
					}
#pragma unroll
					for (int ch = 0; ch < 3; ch++)
						raw[ch] = sh_channel(a.D, dx, dy, dz, row + ch);
				}
				wave_lds_fence();
			}
		} else if (rendered) {
			const float* sh = a.shs + (size_t)idx * a.M * 3;
#pragma unroll
			for (int ch = 0; ch < 3; ch++)
				raw[ch] = sh_channel(a.D, dx, dy, dz, sh + ch);
		}
		float rgb[3];
#pragma unroll
		for (int ch = 0; ch < 3; ch++) {
			const float v = raw[ch];
			clamp_bits |= (v < 0) ? (1u << ch) : 0u;
			rgb[ch] = fmaxf(v, 0.0f);
		}
		col = float3{rgb[0], rgb[1], rgb[2]};
	}

	if (idx < a.P) {
		if (rendered) {
			if (!a.colors_precomp)
				a.clamped[idx] = (uint8_t)clamp_bits;
		}
		a.radii[idx] = (int)my_radius;
		a.tiles_touched[idx] = touched;
		a.depths[idx] = view_z;  // 0 for a Gaussian that touches no tile: the depth order lists the others by this alone
	}
	{
		// Everything later stages read of a rendered Gaussian goes into one 64-byte record: a
		// gather by index then costs one cache line, and nothing is written a second time into
		// arrays of their own, where a rendered Gaussian among unrendered ones dirties a whole
		// line for a few bytes.  The 3D covariance is not kept: the backward computes it again.
		// The records leave through LDS, four lanes to a record, so that a store instruction
		// writes 16 whole records and not a quarter of 64.
		wave_lds_fence();
		if (rendered) {
			const float floor = exponent_floor(conic_o.w);
			const float2 half = alpha_ellipse_half_extent(conic_o, floor);
			float4* rec = parked + rank * kRecordStride;
			rec[0] = float4{pix.x, pix.y, floor, hom_w};
			rec[1] = conic_o;
			rec[2] = float4{col.x, col.y, col.z, view_z};
			// the third word is the integer radius (as bits): the key duplication reads the tile rectangle's inputs from here
			rec[3] = float4{half.x, half.y, __int_as_float((int)my_radius), 0.f};
		}
		wave_lds_fence();
		float4* records = a.blend_record + 4 * (size_t)(idx - lane);
		for (int base = 0; base < n_seen; base += 16) {
			const int slot = base + (lane >> 2);
			if (slot < n_seen)
				records[4 * (size_t)listed[slot] + (lane & 3)] = parked[slot * kRecordStride + (lane & 3)];
		}
	}

	// Per-block total of tiles_touched: the first level of the offset scan.
	uint32_t total;
	(void)block256_exclusive_scan_u32(touched, s_scan, total);
	if (threadIdx.x == 0)
		a.block_sums[blockIdx.x] = total;
	// ... and of the Gaussians that touch any tile: first level of the scan that compacts them
	__syncthreads();
	(void)block256_exclusive_scan_u32(touched != 0u ? 1u : 0u, s_scan, total);
	if (threadIdx.x == 0)
		a.block_visible[blockIdx.x] = total;
}

// ---- backward preprocess -------------------------------------------------------------------
// Fuses K/cuda_rasterizer_hgs/backward.cu:144-274 (conic -> 3D covariance and mean)
// with :346-412 (projection, depth, SH, scale/rotation).  Only Gaussians that were rendered
// have non-zero gradients; the kernel runs over the compacted list of those (in index order,
// every lane busy) and writes their rows.  The rows of all others must be zero beforehand:
// the caller says whether they already are, otherwise the launcher clears the arrays first.

__device__ __forceinline__ void sh_backward_channel(int deg, float x, float y, float z, const float* __restrict__ sh,
                                                    float g, float* __restrict__ dsh, float& ddx, float& ddy,
                                                    float& ddz)
{
#define SHK(k) sh[3 * (k)]
#define DSH(k) dsh[3 * (k)]
	float dRGBdx = 0.f, dRGBdy = 0.f, dRGBdz = 0.f;
	DSH(0) = kShC0 * g;
	if (deg > 0) {
		DSH(1) = (-kShC1 * y) * g;
		DSH(2) = (kShC1 * z) * g;
		DSH(3) = (-kShC1 * x) * g;
		dRGBdx = -kShC1 * SHK(3);
		dRGBdy = -kShC1 * SHK(1);
		dRGBdz = kShC1 * SHK(2);
		if (deg > 1) {
			const float xx = x * x, yy = y * y, zz = z * z;
			const float xy = x * y, yz = y * z, xz = x * z;
			DSH(4) = (kShC2[0] * xy) * g;
			DSH(5) = (kShC2[1] * yz) * g;
			DSH(6) = (kShC2[2] * (2.f * zz - xx - yy)) * g;
			DSH(7) = (kShC2[3] * xz) * g;
			DSH(8) = (kShC2[4] * (xx - yy)) * g;
			dRGBdx += kShC2[0] * y * SHK(4) + kShC2[2] * 2.f * -x * SHK(6) + kShC2[3] * z * SHK(7) +
			          kShC2[4] * 2.f * x * SHK(8);
			dRGBdy += kShC2[0] * x * SHK(4) + kShC2[1] * z * SHK(5) + kShC2[2] * 2.f * -y * SHK(6) +
			          kShC2[4] * 2.f * -y * SHK(8);
			dRGBdz += kShC2[1] * y * SHK(5) + kShC2[2] * 2.f * 2.f * z * SHK(6) + kShC2[3] * x * SHK(7);
			if (deg > 2) {
				DSH(9) = (kShC3[0] * y * (3.f * xx - yy)) * g;
				DSH(10) = (kShC3[1] * xy * z) * g;
				DSH(11) = (kShC3[2] * y * (4.f * zz - xx - yy)) * g;
				DSH(12) = (kShC3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy)) * g;
				DSH(13) = (kShC3[4] * x * (4.f * zz - xx - yy)) * g;
				DSH(14) = (kShC3[5] * z * (xx - yy)) * g;
				DSH(15) = (kShC3[6] * x * (xx - 3.f * yy)) * g;
				dRGBdx += (kShC3[0] * SHK(9) * 3.f * 2.f * xy + kShC3[1] * SHK(10) * yz +
				           kShC3[2] * SHK(11) * -2.f * xy + kShC3[3] * SHK(12) * -3.f * 2.f * xz +
				           kShC3[4] * SHK(13) * (-3.f * xx + 4.f * zz - yy) + kShC3[5] * SHK(14) * 2.f * xz +
				           kShC3[6] * SHK(15) * 3.f * (xx - yy));
				dRGBdy += (kShC3[0] * SHK(9) * 3.f * (xx - yy) + kShC3[1] * SHK(10) * xz +
				           kShC3[2] * SHK(11) * (-3.f * yy + 4.f * zz - xx) + kShC3[3] * SHK(12) * -3.f * 2.f * yz +
				           kShC3[4] * SHK(13) * -2.f * xy + kShC3[5] * SHK(14) * -2.f * yz +
				           kShC3[6] * SHK(15) * -3.f * 2.f * xy);
				dRGBdz += (kShC3[1] * SHK(10) * xy + kShC3[2] * SHK(11) * 4.f * 2.f * yz +
				           kShC3[3] * SHK(12) * 3.f * (2.f * zz - xx - yy) + kShC3[4] * SHK(13) * 4.f * 2.f * xz +
				           kShC3[5] * SHK(14) * (xx - yy));
			}
		}
	}
#undef SHK
#undef DSH
	ddx += dRGBdx * g;
	ddy += dRGBdy * g;
	ddz += dRGBdz * g;
}

// Built for 4 wavefronts per SIMD (left alone the compiler keeps both turns of the SH part in registers: 168
// of them, 3 wavefronts; 3, 4 and 5 measure the same: the kernel is bound by its stores).
__attribute__((amdgpu_waves_per_eu(4, 4)))
__global__ __launch_bounds__(128) void preprocess_backward_kernel(Batch<PreprocessBackwardArgs> batch)
{
	__shared__ float4 s_rows[2][32 * kShRowStride];
	__shared__ uint8_t s_listed[2][64];
	const PreprocessBackwardArgs& a = batch.job[blockIdx.y];
	if (blockIdx.x * 128u >= (uint32_t)a.P)
		return;  // the launch is sized for the job with the most Gaussians
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const size_t i = (size_t)blockIdx.x * 128 + threadIdx.x;
	const bool present = i < (size_t)a.P;
	const bool rendered = present && a.radii[i] > 0;  // backward.cu:357: the others get zeros
	const int n_sh = a.shs ? a.M * 3 : 0;
	float mean2d_x = 0.f, mean2d_y = 0.f, opacity_sum = 0.f, color_sum[3] = {0.f, 0.f, 0.f};
	float3 dmean = {0.f, 0.f, 0.f};
	float dcov[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
	float ds[3] = {0.f, 0.f, 0.f};
	float4 dq = {0.f, 0.f, 0.f, 0.f};

	const float* __restrict__ view = a.view;
	const float* __restrict__ proj = a.proj;
	float3 mean = {0.f, 0.f, 0.f};
	float4 sum0 = {0.f, 0.f, 0.f, 0.f}, sum1 = sum0, sum2v = sum0;
	uint32_t cl = 0;
	if (rendered) {
		mean = float3{a.means[3 * i], a.means[3 * i + 1], a.means[3 * i + 2]};
		const float4* sums = reinterpret_cast<const float4*>(a.sums + kSumCols * i);
		sum0 = sums[0];
		sum1 = sums[1];
		sum2v = sums[2];
		if (a.shs)
			cl = a.clamped[i];
	}
	const float3 dLc = {sum0.z, sum0.w, sum1.x};  // kSumConicXX, kSumConicXY, kSumConicYY
	const float sum_color[3] = {sum1.z, sum1.w, sum2v.x};
	mean2d_x = sum0.x;
	mean2d_y = sum0.y;
	opacity_sum = sum1.y;
	color_sum[0] = sum_color[0];
	color_sum[1] = sum_color[1];
	color_sum[2] = sum_color[2];

	// (ahead of the rest, while few other values are held)
	float3 sh_dmean = {0.f, 0.f, 0.f};
	// -- SH colour and the view direction's dependence on the mean (backward.cu:20-139)
	if (a.shs) {
		const float3 cam = {a.campos[0], a.campos[1], a.campos[2]};
		const float3 d0 = {mean.x - cam.x, mean.y - cam.y, mean.z - cam.z};
		const float len = sqrtf(d0.x * d0.x + d0.y * d0.y + d0.z * d0.z);
		const float x = d0.x / len, y = d0.y / len, z = d0.z / len;
		float ddx = 0.f, ddy = 0.f, ddz = 0.f;
		float g[3];
#pragma unroll
		for (int ch = 0; ch < 3; ch++)
			g[ch] = sum_color[ch] * (((cl >> ch) & 1u) ? 0.f : 1.f);
		if (a.sh_rows_by_16_bytes) {
			// The usual case.  The wavefront reads the SH rows of its rendered Gaussians together,
			// 16 lanes to a row and 16 bytes a lane, parks them in LDS (32 rows at a time) where
			// each lane picks up its own; the rows of dL_dsh, zeros for the others, leave the same way.
			const int piece = lane & 15, sub = lane >> 4;
			const int row_pieces = n_sh / 4;
			const int needed = 3 * (a.D + 1) * (a.D + 1);
			const int needed_pieces = (needed + 3) / 4;
			float4* parked = s_rows[wave];
			uint8_t* listed = s_listed[wave];
			const uint64_t seen = lanes_where(rendered);
			const int n_seen = __popcll(seen);
			const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(seen >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)seen, 0u));
			const size_t wave_first = i - (size_t)lane;
			const float4* __restrict__ rows = reinterpret_cast<const float4*>(a.shs) + wave_first * row_pieces;
			float4* __restrict__ grads = reinterpret_cast<float4*>(a.dL_dsh) + wave_first * row_pieces;
			if (rendered)
				listed[rank] = (uint8_t)lane;
			wave_lds_fence();
			for (int base = 0; base < n_seen; base += 32) {
				// (what a lane computes here does not depend on the turn; made opaque so that it is
				// computed in its turn and not kept in registers across both)
				float xo = x, yo = y, zo = z, go[3] = {g[0], g[1], g[2]};
				asm volatile("" : "+v"(xo), "+v"(yo), "+v"(zo), "+v"(go[0]), "+v"(go[1]), "+v"(go[2]));
				{
					float4 v[8];
#pragma unroll
					for (int r = 0; r < 8; r++) {
						const int slot = base + 4 * r + sub;
						v[r] = float4{0.f, 0.f, 0.f, 0.f};
						if (piece < needed_pieces && slot < n_seen)
							v[r] = rows[(size_t)listed[slot] * row_pieces + piece];
					}
#pragma unroll
					for (int r = 0; r < 8; r++)
						if (piece < 12)
							parked[(4 * r + sub) * kShRowStride + piece] = v[r];
				}
				wave_lds_fence();
				__builtin_amdgcn_sched_barrier(0);
				if (rendered && rank >= base && rank < base + 32) {
					// the coefficients' part in the gradient of the view direction
					const float4* mine = parked + (rank - base) * kShRowStride;
					float row[kShRegs], unused[kShRegs];
#pragma unroll
					for (int k = 0; k < kShRegs; k += 4) {
						float4 q = {0.f, 0.f, 0.f, 0.f};
						if (k < needed)
							q = mine[k / 4];
						row[k] = q.x;
						row[k + 1] = q.y;
						row[k + 2] = q.z;
						row[k + 3] = q.w;
					}
#pragma unroll
					for (int ch = 0; ch < 3; ch++)
						sh_backward_channel(a.D, xo, yo, zo, row + ch, go[ch], unused + ch, ddx, ddy, ddz);
				}
				wave_lds_fence();
				__builtin_amdgcn_sched_barrier(0);
			}
			for (int h = 0; h < 2; h++) {
				// the rows of dL_dsh of 32 neighbouring Gaussians; they do not depend on the coefficients
				if ((size_t)(32 * h) + wave_first >= (size_t)a.P)
					break;
				float xo = x, yo = y, zo = z, go[3] = {g[0], g[1], g[2]};
				asm volatile("" : "+v"(xo), "+v"(yo), "+v"(zo), "+v"(go[0]), "+v"(go[1]), "+v"(go[2]));
				if ((lane >> 5) == h) {
					float4* mine = parked + (lane & 31) * kShRowStride;
					float none[kShRegs], out[kShRegs];
#pragma unroll
					for (int k = 0; k < kShRegs; k++) {
						none[k] = 0.f;
						out[k] = 0.f;
					}
					if (rendered) {
						float t0 = 0.f, t1 = 0.f, t2 = 0.f;
#pragma unroll
						for (int ch = 0; ch < 3; ch++)
							sh_backward_channel(a.D, xo, yo, zo, none + ch, go[ch], out + ch, t0, t1, t2);
					}
#pragma unroll
					for (int k = 0; k < kShRegs; k += 4)
						if (k < n_sh)
							mine[k / 4] = float4{out[k], out[k + 1], out[k + 2], out[k + 3]};
				}
				wave_lds_fence();
				__builtin_amdgcn_sched_barrier(0);
#pragma unroll
				for (int r = 0; r < 8; r++) {
					const int row = 32 * h + 4 * r + sub;
					if (piece < row_pieces && wave_first + (size_t)row < (size_t)a.P)
						grads[(size_t)row * row_pieces + piece] = parked[(4 * r + sub) * kShRowStride + piece];
				}
				wave_lds_fence();
				__builtin_amdgcn_sched_barrier(0);
			}
		} else if (present) {
			float* dst = a.dL_dsh + i * n_sh;
			const int needed = 3 * (a.D + 1) * (a.D + 1);
			if (rendered) {
				const float* sh = a.shs + i * n_sh;
#pragma unroll
				for (int ch = 0; ch < 3; ch++)
					sh_backward_channel(a.D, x, y, z, sh + ch, g[ch], dst + ch, ddx, ddy, ddz);
			}
			for (int k = rendered ? needed : 0; k < n_sh; k++)
				dst[k] = 0.f;
		}
		// normalisation Jacobian (auxiliary.h:123-133)
		const float sum2 = d0.x * d0.x + d0.y * d0.y + d0.z * d0.z;
		const float invsum32 = 1.0f / sqrtf(sum2 * sum2 * sum2);
		sh_dmean.x = ((+sum2 - d0.x * d0.x) * ddx - d0.y * d0.x * ddy - d0.z * d0.x * ddz) * invsum32;
		sh_dmean.y = (-d0.x * d0.y * ddx + (sum2 - d0.y * d0.y) * ddy - d0.z * d0.y * ddz) * invsum32;
		sh_dmean.z = (-d0.x * d0.z * ddx - d0.y * d0.z * ddy + (sum2 - d0.z * d0.z) * ddz) * invsum32;
	}

	if (rendered) {
	// -- conic -> cov2D -> cov3D and mean (backward.cu:144-274)
	float cov6r[6];
	if (a.cov3D_precomp) {
#pragma unroll
		for (int k = 0; k < 6; k++)
			cov6r[k] = a.cov3D_precomp[6 * i + k];
	} else {
		// the same arithmetic as the forward's, which did not keep its result
		const float3 sc = {a.scales[3 * i], a.scales[3 * i + 1], a.scales[3 * i + 2]};
		covariance3d(sc, a.scale_modifier, reinterpret_cast<const float4*>(a.rotations)[i], cov6r);
	}
	Ewa e = ewa_project(mean, a.focal_x, a.focal_y, a.tanfovx, a.tanfovy, cov6r, view);
	const float x_grad_mul = (e.txtz < -e.limx || e.txtz > e.limx) ? 0.f : 1.f;
	const float y_grad_mul = (e.tytz < -e.limy || e.tytz > e.limy) ? 0.f : 1.f;
	const float ca = e.cov.c[0][0] + 0.3f, cb = e.cov.c[0][1], cc = e.cov.c[1][1] + 0.3f;
	const float denom = ca * cc - cb * cb;
	float dL_da = 0.f, dL_db = 0.f, dL_dc = 0.f;
	const float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
#define TM(i, j) e.T.c[i][j]
#define VM(i, j) e.Vrk.c[i][j]
	if (denom2inv != 0.f) {
		dL_da = denom2inv * (-cc * cc * dLc.x + 2 * cb * cc * dLc.y + (denom - ca * cc) * dLc.z);
		dL_dc = denom2inv * (-ca * ca * dLc.z + 2 * ca * cb * dLc.y + (denom - ca * cc) * dLc.x);
		dL_db = denom2inv * 2 * (cb * cc * dLc.x - (denom + 2 * cb * cb) * dLc.y + ca * cb * dLc.z);
		dcov[0] = (TM(0, 0) * TM(0, 0) * dL_da + TM(0, 0) * TM(1, 0) * dL_db + TM(1, 0) * TM(1, 0) * dL_dc);
		dcov[3] = (TM(0, 1) * TM(0, 1) * dL_da + TM(0, 1) * TM(1, 1) * dL_db + TM(1, 1) * TM(1, 1) * dL_dc);
		dcov[5] = (TM(0, 2) * TM(0, 2) * dL_da + TM(0, 2) * TM(1, 2) * dL_db + TM(1, 2) * TM(1, 2) * dL_dc);
		dcov[1] = 2 * TM(0, 0) * TM(0, 1) * dL_da + (TM(0, 0) * TM(1, 1) + TM(0, 1) * TM(1, 0)) * dL_db +
		          2 * TM(1, 0) * TM(1, 1) * dL_dc;
		dcov[2] = 2 * TM(0, 0) * TM(0, 2) * dL_da + (TM(0, 0) * TM(1, 2) + TM(0, 2) * TM(1, 0)) * dL_db +
		          2 * TM(1, 0) * TM(1, 2) * dL_dc;
		dcov[4] = 2 * TM(0, 2) * TM(0, 1) * dL_da + (TM(0, 1) * TM(1, 2) + TM(0, 2) * TM(1, 1)) * dL_db +
		          2 * TM(1, 1) * TM(1, 2) * dL_dc;
	} else {
#pragma unroll
		for (int k = 0; k < 6; k++)
			dcov[k] = 0.f;
	}
	const float dL_dT00 = 2 * (TM(0, 0) * VM(0, 0) + TM(0, 1) * VM(0, 1) + TM(0, 2) * VM(0, 2)) * dL_da +
	                      (TM(1, 0) * VM(0, 0) + TM(1, 1) * VM(0, 1) + TM(1, 2) * VM(0, 2)) * dL_db;
	const float dL_dT01 = 2 * (TM(0, 0) * VM(1, 0) + TM(0, 1) * VM(1, 1) + TM(0, 2) * VM(1, 2)) * dL_da +
	                      (TM(1, 0) * VM(1, 0) + TM(1, 1) * VM(1, 1) + TM(1, 2) * VM(1, 2)) * dL_db;
	const float dL_dT02 = 2 * (TM(0, 0) * VM(2, 0) + TM(0, 1) * VM(2, 1) + TM(0, 2) * VM(2, 2)) * dL_da +
	                      (TM(1, 0) * VM(2, 0) + TM(1, 1) * VM(2, 1) + TM(1, 2) * VM(2, 2)) * dL_db;
	const float dL_dT10 = 2 * (TM(1, 0) * VM(0, 0) + TM(1, 1) * VM(0, 1) + TM(1, 2) * VM(0, 2)) * dL_dc +
	                      (TM(0, 0) * VM(0, 0) + TM(0, 1) * VM(0, 1) + TM(0, 2) * VM(0, 2)) * dL_db;
	const float dL_dT11 = 2 * (TM(1, 0) * VM(1, 0) + TM(1, 1) * VM(1, 1) + TM(1, 2) * VM(1, 2)) * dL_dc +
	                      (TM(0, 0) * VM(1, 0) + TM(0, 1) * VM(1, 1) + TM(0, 2) * VM(1, 2)) * dL_db;
	const float dL_dT12 = 2 * (TM(1, 0) * VM(2, 0) + TM(1, 1) * VM(2, 1) + TM(1, 2) * VM(2, 2)) * dL_dc +
	                      (TM(0, 0) * VM(2, 0) + TM(0, 1) * VM(2, 1) + TM(0, 2) * VM(2, 2)) * dL_db;
#undef TM
#undef VM
	const float dL_dJ00 = e.W.c[0][0] * dL_dT00 + e.W.c[0][1] * dL_dT01 + e.W.c[0][2] * dL_dT02;
	const float dL_dJ02 = e.W.c[2][0] * dL_dT00 + e.W.c[2][1] * dL_dT01 + e.W.c[2][2] * dL_dT02;
	const float dL_dJ11 = e.W.c[1][0] * dL_dT10 + e.W.c[1][1] * dL_dT11 + e.W.c[1][2] * dL_dT12;
	const float dL_dJ12 = e.W.c[2][0] * dL_dT10 + e.W.c[2][1] * dL_dT11 + e.W.c[2][2] * dL_dT12;
	const float tz = 1.f / e.t.z;
	const float tz2 = tz * tz;
	const float tz3 = tz2 * tz;
	const float h_x = a.focal_x, h_y = a.focal_y;
	const float dL_dtx = x_grad_mul * -h_x * tz2 * dL_dJ02;
	const float dL_dty = y_grad_mul * -h_y * tz2 * dL_dJ12;
	const float dL_dtz = -h_x * tz2 * dL_dJ00 - h_y * tz2 * dL_dJ11 + (2 * h_x * e.t.x) * tz3 * dL_dJ02 +
	                     (2 * h_y * e.t.y) * tz3 * dL_dJ12;
	dmean.x = view[0] * dL_dtx + view[1] * dL_dty + view[2] * dL_dtz;
	dmean.y = view[4] * dL_dtx + view[5] * dL_dty + view[6] * dL_dtz;
	dmean.z = view[8] * dL_dtx + view[9] * dL_dty + view[10] * dL_dtz;

	// -- screen-space mean through the perspective divide (backward.cu:369-389)
	const float4 m_hom = xform_point_4x4(mean, proj);
	const float m_w = 1.0f / (m_hom.w + 0.0000001f);
	const float g2x = mean2d_x, g2y = mean2d_y;
	const float mul1 = (proj[0] * mean.x + proj[4] * mean.y + proj[8] * mean.z + proj[12]) * m_w * m_w;
	const float mul2 = (proj[1] * mean.x + proj[5] * mean.y + proj[9] * mean.z + proj[13]) * m_w * m_w;
	dmean.x += (proj[0] * m_w - proj[3] * mul1) * g2x + (proj[1] * m_w - proj[3] * mul2) * g2y;
	dmean.y += (proj[4] * m_w - proj[7] * mul1) * g2x + (proj[5] * m_w - proj[7] * mul2) * g2y;
	dmean.z += (proj[8] * m_w - proj[11] * mul1) * g2x + (proj[9] * m_w - proj[11] * mul2) * g2y;

	// -- per-Gaussian depth (backward.cu:391-403)
	const float gd = sum2v.y;  // kSumDepth
	const float mul3 = view[2] * mean.x + view[6] * mean.y + view[10] * mean.z + view[14];
	dmean.x += (view[2] - view[3] * mul3) * gd;
	dmean.y += (view[6] - view[7] * mul3) * gd;
	dmean.z += (view[10] - view[11] * mul3) * gd;

	dmean.x += sh_dmean.x;
	dmean.y += sh_dmean.y;
	dmean.z += sh_dmean.z;

	// -- 3D covariance -> scale and raw quaternion (backward.cu:278-341)
	if (a.scales) {
		const float3 sc = {a.scales[3 * i], a.scales[3 * i + 1], a.scales[3 * i + 2]};
		const float4 q = reinterpret_cast<const float4*>(a.rotations)[i];
		const float r = q.x, x = q.y, y = q.z, z = q.w;
		const M3 R = rotation_cols(q);
		const float s[3] = {a.scale_modifier * sc.x, a.scale_modifier * sc.y, a.scale_modifier * sc.z};
		M3 S = m3_cols(1.f, 0.f, 0.f, 0.f, 1.f, 0.f, 0.f, 0.f, 1.f);
		S.c[0][0] = s[0];
		S.c[1][1] = s[1];
		S.c[2][2] = s[2];
		const M3 M = m3_mul(S, R);
		const M3 dSigma = m3_cols(dcov[0], 0.5f * dcov[1], 0.5f * dcov[2], 0.5f * dcov[1], dcov[3], 0.5f * dcov[4],
		                          0.5f * dcov[2], 0.5f * dcov[4], dcov[5]);
		M3 M2;
#pragma unroll
		for (int c = 0; c < 3; c++)
#pragma unroll
			for (int rr = 0; rr < 3; rr++)
				M2.c[c][rr] = M.c[c][rr] * 2.0f;
		const M3 dM = m3_mul(M2, dSigma);
		const M3 Rt = m3_transpose(R);
		M3 dMt = m3_transpose(dM);
#pragma unroll
		for (int k = 0; k < 3; k++)
			ds[k] = Rt.c[k][0] * dMt.c[k][0] + Rt.c[k][1] * dMt.c[k][1] + Rt.c[k][2] * dMt.c[k][2];
#pragma unroll
		for (int k = 0; k < 3; k++)
#pragma unroll
			for (int rr = 0; rr < 3; rr++)
				dMt.c[k][rr] *= s[k];
#define DM(i, j) dMt.c[i][j]
		dq.x = 2 * z * (DM(0, 1) - DM(1, 0)) + 2 * y * (DM(2, 0) - DM(0, 2)) + 2 * x * (DM(1, 2) - DM(2, 1));
		dq.y = 2 * y * (DM(1, 0) + DM(0, 1)) + 2 * z * (DM(2, 0) + DM(0, 2)) + 2 * r * (DM(1, 2) - DM(2, 1)) -
		       4 * x * (DM(2, 2) + DM(1, 1));
		dq.z = 2 * x * (DM(1, 0) + DM(0, 1)) + 2 * r * (DM(2, 0) - DM(0, 2)) + 2 * z * (DM(1, 2) + DM(2, 1)) -
		       4 * y * (DM(2, 2) + DM(0, 0));
		dq.w = 2 * r * (DM(0, 1) - DM(1, 0)) + 2 * x * (DM(2, 0) + DM(0, 2)) + 2 * y * (DM(1, 2) + DM(2, 1)) -
		       4 * z * (DM(1, 1) + DM(0, 0));
#undef DM
	}
	}

	// Every Gaussian's rows are written, zeros for those that were not rendered: the arrays need no clearing.
	if (!present)
		return;
	a.dL_dmeans[3 * i + 0] = dmean.x;
	a.dL_dmeans[3 * i + 1] = dmean.y;
	a.dL_dmeans[3 * i + 2] = dmean.z;
	if (a.dL_dcov3D) {  // null when the covariance comes from scale and rotation and nobody asks for this intermediate
#pragma unroll
		for (int k = 0; k < 6; k++)
			a.dL_dcov3D[6 * i + k] = dcov[k];
	}
	if (a.dL_dscale) {
		a.dL_dscale[3 * i + 0] = ds[0];
		a.dL_dscale[3 * i + 1] = ds[1];
		a.dL_dscale[3 * i + 2] = ds[2];
	}
	if (a.dL_drot)
		reinterpret_cast<float4*>(a.dL_drot)[i] = dq;
	// the sums that are gradients as they stand
	a.dL_dmean2D[3 * i + 0] = mean2d_x;
	a.dL_dmean2D[3 * i + 1] = mean2d_y;
	a.dL_dmean2D[3 * i + 2] = 0.f;
	a.dL_dopacity[i] = opacity_sum;
	if (a.dL_dcolor) {  // null when the colours come from SH and nobody asks for this intermediate
		a.dL_dcolor[3 * i + 0] = color_sum[0];
		a.dL_dcolor[3 * i + 1] = color_sum[1];
		a.dL_dcolor[3 * i + 2] = color_sum[2];
	}
}

// ---- launchers -----------------------------------------------------------------------------

__global__ __launch_bounds__(256) void covariance3d_kernel(int P, const float* __restrict__ scales, float mod,
                                                            const float* __restrict__ rotations, float* __restrict__ cov3D)
{
	const int idx = blockIdx.x * 256 + threadIdx.x;
	if (idx >= P)
		return;
	const float3 sc = {scales[3 * (size_t)idx], scales[3 * (size_t)idx + 1], scales[3 * (size_t)idx + 2]};
	float cov6[6];
	covariance3d(sc, mod, reinterpret_cast<const float4*>(rotations)[idx], cov6);
#pragma unroll
	for (int i = 0; i < 6; i++)
		cov3D[6 * (size_t)idx + i] = cov6[i];
}

void launch_covariance3d(int P, const float* scales, float scale_modifier, const float* rotations, float* cov3D, hipStream_t s)
{
	hipLaunchKernelGGL(covariance3d_kernel, dim3((P + 255) / 256), dim3(256), 0, s, P, scales, scale_modifier, rotations, cov3D);
}

void launch_mark_visible(int P, const float* means, const float* view, uint8_t* present, hipStream_t s)
{
	stage_mark("mark_visible", s);
	hipLaunchKernelGGL(mark_visible_kernel, dim3((P + 255) / 256), dim3(256), 0, s, P, means, view, present);
}

void launch_preprocess_forward(const PreprocessArgs* jobs, int count, hipStream_t s)
{
	stage_mark("preprocess_forward", s);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<PreprocessArgs> b = {};
		int max_p = 0;
		for (int k = 0; k < nj; k++) {
			b.job[k] = jobs[at + k];
			max_p = b.job[k].P > max_p ? b.job[k].P : max_p;
		}
		hipLaunchKernelGGL(preprocess_forward_kernel, dim3((unsigned)((max_p + 255) / 256), (unsigned)nj), dim3(256), 0, s, b);
	}
}

void launch_preprocess_backward(const PreprocessBackwardArgs* jobs, int count, hipStream_t s)
{
	stage_mark("preprocess_backward", s);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<PreprocessBackwardArgs> b = {};
		int max_p = 0;
		for (int k = 0; k < nj; k++) {
			b.job[k] = jobs[at + k];
			max_p = b.job[k].P > max_p ? b.job[k].P : max_p;
		}
		hipLaunchKernelGGL(preprocess_backward_kernel, dim3((unsigned)((max_p + 127) / 128), (unsigned)nj), dim3(128), 0, s, b);
	}
}

}  // namespace rgs
