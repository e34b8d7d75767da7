/*
 * rgs_oracle.c -- CPU restatement of the half-Gaussian rasterizer (forward and
 * backward).  TEST INFRASTRUCTURE ONLY: nothing the library ships may link,
 * load or call this file.  It is the checker that the HIP kernels are compared
 * against and the host-CPU baseline that is timed beside them.
 *
 * Every function restates one routine of the reference, whose files are cited
 * as K/<file>:<lines> with
 *   K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian
 * All arithmetic is single precision, one rounding per operation, evaluated in
 * the reference's C++ left-to-right order (build with -ffp-contract=off and no
 * fast-math).  The two places where the reference computes in double
 * (ndc2Pix / pix2Ndc) are computed in double here too.  GLM's 3x3 product order
 * follows K/third_party/glm/glm/detail/type_mat3x3.inl:486-518.
 *
 * Pinning status (what checks each function independently of its own formula)
 * is listed in oracle/README.md; the tests that do it are tests/test_oracle_*.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TILE 16          /* K/cuda_rasterizer_hgs/config.h:15-17 */
#define TILE_PIX 256

static int g_threads = 1;

void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_threads(void) { return g_threads; }
int orc_max_threads(void)
{
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

/* ---- small helpers ------------------------------------------------------ */

/* 3x3 matrix stored like GLM: m[column][row]. */
typedef struct { float m[3][3]; } mat3;

/* GLM operator*(mat3, mat3): type_mat3x3.inl:509-517. */
static mat3 mat3_mul(const mat3 *A, const mat3 *B)
{
	mat3 R;
	for (int c = 0; c < 3; c++)
		for (int r = 0; r < 3; r++)
			R.m[c][r] = A->m[0][r] * B->m[c][0] + A->m[1][r] * B->m[c][1] + A->m[2][r] * B->m[c][2];
	return R;
}

/* GLM transpose: func_matrix.inl:119-137. */
static mat3 mat3_t(const mat3 *A)
{
	mat3 R;
	for (int c = 0; c < 3; c++)
		for (int r = 0; r < 3; r++)
			R.m[c][r] = A->m[r][c];
	return R;
}

/* Column-filling constructor mat3(x0,y0,z0, x1,y1,z1, x2,y2,z2). */
static mat3 mat3_cols(float x0, float y0, float z0, float x1, float y1, float z1, float x2, float y2, float z2)
{
	mat3 R;
	R.m[0][0] = x0; R.m[0][1] = y0; R.m[0][2] = z0;
	R.m[1][0] = x1; R.m[1][1] = y1; R.m[1][2] = z1;
	R.m[2][0] = x2; R.m[2][1] = y2; R.m[2][2] = z2;
	return R;
}

/* GPU float->int conversion truncates toward zero, saturates and maps NaN to 0;
 * x86 does none of the last two, so it is spelled out. */
static int f2i(float v)
{
	if (v != v) return 0;
	if (v >= 2147483648.0f) return 2147483647;
	if (v <= -2147483648.0f) return (-2147483647 - 1);
	return (int)v;
}

static int imin(int a, int b) { return a < b ? a : b; }
static int imax(int a, int b) { return a > b ? a : b; }

/* K/cuda_rasterizer_hgs/auxiliary.h:63-71 */
static void xform4x3(const float *p, const float *m, float *o)
{
	o[0] = m[0] * p[0] + m[4] * p[1] + m[8] * p[2] + m[12];
	o[1] = m[1] * p[0] + m[5] * p[1] + m[9] * p[2] + m[13];
	o[2] = m[2] * p[0] + m[6] * p[1] + m[10] * p[2] + m[14];
}

/* K/cuda_rasterizer_hgs/auxiliary.h:73-82 */
static void xform4x4(const float *p, const float *m, float *o)
{
	o[0] = m[0] * p[0] + m[4] * p[1] + m[8] * p[2] + m[12];
	o[1] = m[1] * p[0] + m[5] * p[1] + m[9] * p[2] + m[13];
	o[2] = m[2] * p[0] + m[6] * p[1] + m[10] * p[2] + m[14];
	o[3] = m[3] * p[0] + m[7] * p[1] + m[11] * p[2] + m[15];
}

/* K/cuda_rasterizer_hgs/auxiliary.h:41-44: evaluated in double, rounded once. */
static float ndc2pix(float v, int S)
{
	return (float)((((double)v + 1.0) * (double)S - 1.0) * 0.5);
}

/* K/cuda_rasterizer_hgs/auxiliary.h:46-49: 2*pix is a float product. */
static float pix2ndc(float pix, int S)
{
	return (float)(((double)(2 * pix) + 1.0) / (double)S - 1.0);
}

/* K/cuda_rasterizer_hgs/auxiliary.h:51-61.  rect = {minx, miny, maxx, maxy}. */
static void get_rect(float px, float py, int max_radius, int gx, int gy, uint32_t *rect)
{
	rect[0] = (uint32_t)imin(gx, imax(0, f2i((px - max_radius) / TILE)));
	rect[1] = (uint32_t)imin(gy, imax(0, f2i((py - max_radius) / TILE)));
	rect[2] = (uint32_t)imin(gx, imax(0, f2i((px + max_radius + TILE - 1) / TILE)));
	rect[3] = (uint32_t)imin(gy, imax(0, f2i((py + max_radius + TILE - 1) / TILE)));
}

/* K/cuda_rasterizer_hgs/rasterizer_impl.cu:35-50 */
uint32_t orc_get_higher_msb(uint32_t n)
{
	uint32_t msb = sizeof(n) * 4;
	uint32_t step = msb;
	while (step > 1) {
		step /= 2;
		if (n >> msb)
			msb += step;
		else
			msb -= step;
	}
	if (n >> msb)
		msb++;
	return msb;
}

/* ---- spherical harmonics -------------------------------------------------- */

/* K/cuda_rasterizer_hgs/auxiliary.h:22-39 */
static const float SH_C0 = 0.28209479177387814f;
static const float SH_C1 = 0.4886025119029199f;
static const float SH_C2[5] = { 1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
	-1.0925484305920792f, 0.5462742152960396f };
static const float SH_C3[7] = { -0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
	0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f, -0.5900435899266435f };

/* K/cuda_rasterizer_hgs/forward.cu:20-71.  sh points at this Gaussian's
 * (M,3) coefficient rows; rgb and clamped get 3 entries. */
static void sh_to_rgb(int deg, const float *mean, const float *campos, const float *sh, float *rgb, uint8_t *clamped)
{
	float dir[3] = { mean[0] - campos[0], mean[1] - campos[1], mean[2] - campos[2] };
	float len = sqrtf(dir[0] * dir[0] + dir[1] * dir[1] + dir[2] * dir[2]);
	float x = dir[0] / len, y = dir[1] / len, z = dir[2] / len;
	for (int c = 0; c < 3; c++) {
#define SH(k) sh[3 * (k) + c]
		float result = SH_C0 * SH(0);
		if (deg > 0) {
			result = result - SH_C1 * y * SH(1) + SH_C1 * z * SH(2) - SH_C1 * x * SH(3);
			if (deg > 1) {
				float xx = x * x, yy = y * y, zz = z * z;
				float xy = x * y, yz = y * z, xz = x * z;
				result = result +
					SH_C2[0] * xy * SH(4) +
					SH_C2[1] * yz * SH(5) +
					SH_C2[2] * (2.0f * zz - xx - yy) * SH(6) +
					SH_C2[3] * xz * SH(7) +
					SH_C2[4] * (xx - yy) * SH(8);
				if (deg > 2) {
					result = result +
						SH_C3[0] * y * (3.0f * xx - yy) * SH(9) +
						SH_C3[1] * xy * z * SH(10) +
						SH_C3[2] * y * (4.0f * zz - xx - yy) * SH(11) +
						SH_C3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * SH(12) +
						SH_C3[4] * x * (4.0f * zz - xx - yy) * SH(13) +
						SH_C3[5] * z * (xx - yy) * SH(14) +
						SH_C3[6] * x * (xx - 3.0f * yy) * SH(15);
				}
			}
		}
#undef SH
		result += 0.5f;
		clamped[c] = (result < 0);
		rgb[c] = fmaxf(result, 0.0f);
	}
}

/* ---- forward preprocess --------------------------------------------------- */

/* K/cuda_rasterizer_hgs/forward.cu:118-152.  rot = (r, x, y, z), used as given. */
static void cov3d_from_scale_rot(const float *scale, float mod, const float *rot, float *cov3D)
{
	mat3 S = mat3_cols(1, 0, 0, 0, 1, 0, 0, 0, 1);
	S.m[0][0] = mod * scale[0];
	S.m[1][1] = mod * scale[1];
	S.m[2][2] = mod * scale[2];
	float r = rot[0], x = rot[1], y = rot[2], z = rot[3];
	mat3 R = mat3_cols(
		1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
		2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
		2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
	mat3 M = mat3_mul(&S, &R);
	mat3 Mt = mat3_t(&M);
	mat3 Sigma = mat3_mul(&Mt, &M);
	cov3D[0] = Sigma.m[0][0];
	cov3D[1] = Sigma.m[0][1];
	cov3D[2] = Sigma.m[0][2];
	cov3D[3] = Sigma.m[1][1];
	cov3D[4] = Sigma.m[1][2];
	cov3D[5] = Sigma.m[2][2];
}

/* Pieces of the EWA projection shared by forward and backward
 * (K/cuda_rasterizer_hgs/forward.cu:74-113, backward.cu:166-198). */
typedef struct {
	float t[3];      /* view-space mean after the frustum clamp of x, y */
	float txtz, tytz, limx, limy;
	mat3 W, T, Vrk, cov;
} ewa_t;

static void ewa_project(const float *mean, float fx, float fy, float tanx, float tany, const float *cov3D,
	const float *view, ewa_t *e)
{
	xform4x3(mean, view, e->t);
	e->limx = 1.3f * tanx;
	e->limy = 1.3f * tany;
	e->txtz = e->t[0] / e->t[2];
	e->tytz = e->t[1] / e->t[2];
	e->t[0] = fminf(e->limx, fmaxf(-e->limx, e->txtz)) * e->t[2];
	e->t[1] = fminf(e->limy, fmaxf(-e->limy, e->tytz)) * e->t[2];
	const float *t = e->t;
	mat3 J = mat3_cols(
		fx / t[2], 0.0f, -(fx * t[0]) / (t[2] * t[2]),
		0.0f, fy / t[2], -(fy * t[1]) / (t[2] * t[2]),
		0, 0, 0);
	e->W = mat3_cols(view[0], view[4], view[8], view[1], view[5], view[9], view[2], view[6], view[10]);
	e->T = mat3_mul(&e->W, &J);
	e->Vrk = mat3_cols(cov3D[0], cov3D[1], cov3D[2], cov3D[1], cov3D[3], cov3D[4], cov3D[2], cov3D[4], cov3D[5]);
	mat3 Tt = mat3_t(&e->T);
	mat3 Vt = mat3_t(&e->Vrk);
	mat3 TtVt = mat3_mul(&Tt, &Vt);
	e->cov = mat3_mul(&TtVt, &e->T);
}

/* K/cuda_rasterizer_hgs/forward.cu:155-258 with in_frustum (auxiliary.h:155-180).
 * Pointers that the reference receives as nullptr may be NULL here as well:
 * cov3D_precomp (then scales/rots are used), colors_precomp (then shs are used).
 * Outputs for culled Gaussians are left untouched except radii/tiles_touched = 0,
 * exactly as the reference leaves them. */
void orc_preprocess(int P, int D, int M,
	const float *means, const float *scales, float mod, const float *rots, const float *opac,
	const float *shs, const float *cov3D_precomp, const float *colors_precomp,
	const float *view, const float *proj, const float *campos,
	int W, int H, float tanx, float tany,
	int *radii, float *xy, float *zw, float *depths, float *cov3Ds, float *rgb, float *conic_opacity,
	uint32_t *tiles_touched, uint8_t *clamped)
{
	/* K/cuda_rasterizer_hgs/rasterizer_impl.cu:227-228,239 */
	const float fy = H / (2.0f * tany);
	const float fx = W / (2.0f * tanx);
	const int gx = (W + TILE - 1) / TILE, gy = (H + TILE - 1) / TILE;

#pragma omp parallel for schedule(static) num_threads(g_threads)
	for (int idx = 0; idx < P; idx++) {
		radii[idx] = 0;
		tiles_touched[idx] = 0;
		const float *p = means + 3 * (size_t)idx;
		float p_hom[4], p_view[3];
		xform4x4(p, proj, p_hom);
		float p_w = 1.0f / (p_hom[3] + 0.0000001f);
		float p_proj[3] = { p_hom[0] * p_w, p_hom[1] * p_w, p_hom[2] * p_w };
		xform4x3(p, view, p_view);
		if (p_view[2] <= 0.2f)
			continue;

		const float *cov3D;
		if (cov3D_precomp) {
			cov3D = cov3D_precomp + 6 * (size_t)idx;
		} else {
			cov3d_from_scale_rot(scales + 3 * (size_t)idx, mod, rots + 4 * (size_t)idx, cov3Ds + 6 * (size_t)idx);
			cov3D = cov3Ds + 6 * (size_t)idx;
		}
		ewa_t e;
		ewa_project(p, fx, fy, tanx, tany, cov3D, view, &e);
		e.cov.m[0][0] += 0.3f;
		e.cov.m[1][1] += 0.3f;
		float cx = e.cov.m[0][0], cyy = e.cov.m[0][1], cz = e.cov.m[1][1];

		float det = (cx * cz - cyy * cyy);
		if (det == 0.0f)
			continue;
		float det_inv = 1.f / det;
		float conic[3] = { cz * det_inv, -cyy * det_inv, cx * det_inv };

		float mid = 0.5f * (cx + cz);
		float lambda1 = mid + sqrtf(fmaxf(0.1f, mid * mid - det));
		float lambda2 = mid - sqrtf(fmaxf(0.1f, mid * mid - det));
		float my_radius = ceilf(3.f * sqrtf(fmaxf(lambda1, lambda2)));
		float pix[2] = { ndc2pix(p_proj[0], W), ndc2pix(p_proj[1], H) };
		uint32_t rect[4];
		get_rect(pix[0], pix[1], f2i(my_radius), gx, gy, rect);
		if ((rect[2] - rect[0]) * (rect[3] - rect[1]) == 0)
			continue;

		if (!colors_precomp)
			sh_to_rgb(D, p, campos, shs + 3 * (size_t)M * idx, rgb + 3 * (size_t)idx, clamped + 3 * (size_t)idx);

		depths[idx] = p_view[2];
		radii[idx] = f2i(my_radius);
		xy[2 * (size_t)idx] = pix[0];
		xy[2 * (size_t)idx + 1] = pix[1];
		zw[2 * (size_t)idx] = p_hom[2];
		zw[2 * (size_t)idx + 1] = p_hom[3];
		conic_opacity[4 * (size_t)idx + 0] = conic[0];
		conic_opacity[4 * (size_t)idx + 1] = conic[1];
		conic_opacity[4 * (size_t)idx + 2] = conic[2];
		conic_opacity[4 * (size_t)idx + 3] = opac[idx];
		tiles_touched[idx] = (rect[3] - rect[1]) * (rect[2] - rect[0]);
	}
}

/* K/cuda_rasterizer_hgs/rasterizer_impl.cu:54-66 (checkFrustum via in_frustum). */
void orc_mark_visible(int P, const float *means, const float *view, const float *proj, uint8_t *present)
{
	(void)proj;
	for (int idx = 0; idx < P; idx++) {
		float p_view[3];
		xform4x3(means + 3 * (size_t)idx, view, p_view);
		present[idx] = !(p_view[2] <= 0.2f);
	}
}

/* ---- binning: scan, key duplication, sort, tile ranges --------------------- */

/* cub::DeviceScan::InclusiveSum as called at rasterizer_impl.cu:283: u32, wraps. */
void orc_inclusive_sum(int P, const uint32_t *in, uint32_t *out)
{
	uint32_t acc = 0;
	for (int i = 0; i < P; i++) {
		acc += in[i];
		out[i] = acc;
	}
}

/* K/cuda_rasterizer_hgs/rasterizer_impl.cu:70-111 */
void orc_duplicate_with_keys(int P, const float *xy, const float *depths, const uint32_t *offsets,
	uint64_t *keys, uint32_t *values, const int *radii, int gx, int gy)
{
	for (int idx = 0; idx < P; idx++) {
		if (radii[idx] > 0) {
			uint32_t off = (idx == 0) ? 0 : offsets[idx - 1];
			uint32_t rect[4];
			get_rect(xy[2 * (size_t)idx], xy[2 * (size_t)idx + 1], radii[idx], gx, gy, rect);
			uint32_t dbits;
			memcpy(&dbits, depths + idx, 4);
			for (uint32_t y = rect[1]; y < rect[3]; y++) {
				for (uint32_t x = rect[0]; x < rect[2]; x++) {
					uint64_t key = y * (uint32_t)gx + x;
					key <<= 32;
					key |= dbits;
					keys[off] = key;
					values[off] = (uint32_t)idx;
					off++;
				}
			}
		}
	}
}

/* cub::DeviceRadixSort::SortPairs as called at rasterizer_impl.cu:312-317:
 * a stable sort of (key, value) pairs that compares only key bits
 * [0, end_bit).  Restated as a least-significant-digit radix sort with 8-bit
 * digits, which is stable by construction.  tmp_* are scratch of n elements. */
void orc_sort_pairs(size_t n, const uint64_t *keys_in, uint64_t *keys_out, const uint32_t *vals_in, uint32_t *vals_out,
	int end_bit, uint64_t *tmp_k, uint32_t *tmp_v)
{
	memcpy(keys_out, keys_in, n * sizeof(uint64_t));
	memcpy(vals_out, vals_in, n * sizeof(uint32_t));
	uint64_t *src_k = keys_out, *dst_k = tmp_k;
	uint32_t *src_v = vals_out, *dst_v = tmp_v;
	for (int shift = 0; shift < end_bit; shift += 8) {
		int bits = end_bit - shift < 8 ? end_bit - shift : 8;
		uint32_t mask = (1u << bits) - 1u;
		size_t count[257];
		memset(count, 0, sizeof(count));
		for (size_t i = 0; i < n; i++)
			count[((src_k[i] >> shift) & mask) + 1]++;
		for (int d = 0; d < 256; d++)
			count[d + 1] += count[d];
		for (size_t i = 0; i < n; i++) {
			size_t pos = count[(src_k[i] >> shift) & mask]++;
			dst_k[pos] = src_k[i];
			dst_v[pos] = src_v[i];
		}
		uint64_t *tk = src_k; src_k = dst_k; dst_k = tk;
		uint32_t *tv = src_v; src_v = dst_v; dst_v = tv;
	}
	if (src_k != keys_out) {
		memcpy(keys_out, src_k, n * sizeof(uint64_t));
		memcpy(vals_out, src_v, n * sizeof(uint32_t));
	}
}

/* K/cuda_rasterizer_hgs/rasterizer_impl.cu:116-138 plus the memset at :319.
 * ranges holds T pairs (start, end). */
void orc_identify_tile_ranges(size_t L, const uint64_t *keys, uint32_t *ranges, int T)
{
	memset(ranges, 0, (size_t)T * 2 * sizeof(uint32_t));
	for (size_t idx = 0; idx < L; idx++) {
		uint32_t currtile = (uint32_t)(keys[idx] >> 32);
		if (idx == 0) {
			ranges[2 * currtile] = 0;
		} else {
			uint32_t prevtile = (uint32_t)(keys[idx - 1] >> 32);
			if (currtile != prevtile) {
				ranges[2 * prevtile + 1] = (uint32_t)idx;
				ranges[2 * currtile] = (uint32_t)idx;
			}
		}
		if (idx == L - 1)
			ranges[2 * currtile + 1] = (uint32_t)L;
	}
}

/* ---- forward blend ---------------------------------------------------------- */

/* The half-Gaussian test of K/cuda_rasterizer_hgs/forward.cu:360-372: the point
 * of the pixel's ray at the Gaussian's clip-w, taken to world space, must lie in
 * (low, up] on every axis.  Returns 1 when the Gaussian is clipped away. */
static int outside_box(float ndcx, float ndcy, float w, float tanx, float tany, const float *projinv,
	const float *low, const float *up)
{
	float p_hom[3] = { ndcx * (w + 0.0000001f) * tanx, ndcy * (w + 0.0000001f) * tany, w };
	float pw[4];
	xform4x4(p_hom, projinv, pw);
	return (pw[0] <= low[0]) || (pw[0] > up[0]) ||
		(pw[1] <= low[1]) || (pw[1] > up[1]) ||
		(pw[2] <= low[2]) || (pw[2] > up[2]);
}

/* K/cuda_rasterizer_hgs/forward.cu:263-405.  One pixel at a time; the block-wide
 * early exit of the reference (:321) changes no pixel's result.
 * counters (optional, 5 entries) count, over all pixels: every list entry
 * visited by a live pixel, those with power <= 0, those with alpha >= 1/255,
 * those inside the box, those blended.
 * margin (optional, H*W) receives, per pixel, the smallest relative distance
 * of any decision to its threshold: |alpha*255 - 1| and |T(1-alpha)/1e-4 - 1|;
 * a pixel with a tiny margin can legitimately differ between two exp()
 * implementations. */
void orc_render_forward(int W, int H, const uint32_t *ranges, const uint32_t *point_list,
	float tanx, float tany, const float *zw, const float *projinv, const float *low, const float *up,
	const float *xy, const float *features, const float *depths, const float *conic_opacity, const float *bg,
	float *out_color, float *out_depth, float *out_alpha, uint32_t *n_contrib,
	uint64_t *counters, float *margin)
{
	const int gx = (W + TILE - 1) / TILE, gy = (H + TILE - 1) / TILE;
	uint64_t nA = 0, nB = 0, nC = 0, nD = 0, nE = 0;
#pragma omp parallel for schedule(dynamic, 4) num_threads(g_threads) reduction(+ : nA, nB, nC, nD, nE)
	for (int tile = 0; tile < gx * gy; tile++) {
		const int tx = tile % gx, ty = tile / gx;
		const uint32_t r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
		for (int ly = 0; ly < TILE; ly++) {
			for (int lx = 0; lx < TILE; lx++) {
				const int pxi = tx * TILE + lx, pyi = ty * TILE + ly;
				if (!(pxi < W && pyi < H))
					continue;
				const size_t pix_id = (size_t)W * pyi + pxi;
				const float pixf[2] = { (float)pxi, (float)pyi };
				const float ndcx = pix2ndc(pixf[0], W), ndcy = pix2ndc(pixf[1], H);
				float T = 1.0f;
				uint32_t contributor = 0, last_contributor = 0;
				float C[3] = { 0, 0, 0 };
				float weight = 0, Dp = 0;
				float mg = INFINITY;
				for (uint32_t k = r0; k < r1; k++) {
					contributor++;
					nA++;
					const uint32_t id = point_list[k];
					const float dx = xy[2 * (size_t)id] - pixf[0], dy = xy[2 * (size_t)id + 1] - pixf[1];
					const float *co = conic_opacity + 4 * (size_t)id;
					float power = -0.5f * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
					if (power > 0.0f)
						continue;
					nB++;
					float alpha = fminf(0.99f, co[3] * expf(power));
					if (margin) {
						float m1 = fabsf(alpha * 255.0f - 1.0f);
						if (m1 < mg) mg = m1;
					}
					if (alpha < 1.0f / 255.0f)
						continue;
					nC++;
					if (outside_box(ndcx, ndcy, zw[2 * (size_t)id + 1], tanx, tany, projinv, low, up))
						continue;
					nD++;
					float test_T = T * (1 - alpha);
					if (margin) {
						float m2 = fabsf(test_T / 0.0001f - 1.0f);
						if (m2 < mg) mg = m2;
					}
					if (test_T < 0.0001f)
						break;  /* done = true: this pixel visits nothing more */
					nE++;
					for (int ch = 0; ch < 3; ch++)
						C[ch] += features[3 * (size_t)id + ch] * alpha * T;
					weight += alpha * T;
					Dp += depths[id] * alpha * T;
					T = test_T;
					last_contributor = contributor;
				}
				n_contrib[pix_id] = last_contributor;
				for (int ch = 0; ch < 3; ch++)
					out_color[(size_t)ch * H * W + pix_id] = C[ch] + T * bg[ch];
				out_alpha[pix_id] = weight;
				out_depth[pix_id] = Dp;
				if (margin)
					margin[pix_id] = mg;
			}
		}
	}
	if (counters) {
		counters[0] = nA; counters[1] = nB; counters[2] = nC; counters[3] = nD; counters[4] = nE;
	}
}

/* ---- backward blend --------------------------------------------------------- */

static void atomic_addf(float *p, float v)
{
	if (g_threads > 1) {
#pragma omp atomic
		*p += v;
	} else {
		*p += v;
	}
}

/* K/cuda_rasterizer_hgs/backward.cu:415-622.  Gradient buffers must arrive
 * zeroed (K/rasterize_points.cu:165-174); sums are accumulated in float like the
 * reference's atomicAdd.  With one thread the order is pixel-major within a
 * tile, tiles in index order.  dL_dmean2D is (P,3), dL_dconic (P,4). */
void orc_render_backward(int W, int H, const uint32_t *ranges, const uint32_t *point_list,
	float tanx, float tany, const float *projinv, const float *low, const float *up, const float *zw,
	const float *bg, const float *xy, const float *conic_opacity, const float *colors, const float *depths,
	const float *alphas, const uint32_t *n_contrib,
	const float *dL_dpixels, const float *dL_dpixel_depths, const float *dL_dalphas,
	float *dL_dmean2D, float *dL_dconic2D, float *dL_dopacity, float *dL_dcolors, float *dL_ddepths)
{
	const int gx = (W + TILE - 1) / TILE, gy = (H + TILE - 1) / TILE;
	const float ddelx_dx = 0.5 * W;
	const float ddely_dy = 0.5 * H;
#pragma omp parallel for schedule(dynamic, 4) num_threads(g_threads)
	for (int tile = 0; tile < gx * gy; tile++) {
		const int tx = tile % gx, ty = tile / gx;
		const uint32_t r0 = ranges[2 * tile];
		for (int ly = 0; ly < TILE; ly++) {
			for (int lx = 0; lx < TILE; lx++) {
				const int pxi = tx * TILE + lx, pyi = ty * TILE + ly;
				if (!(pxi < W && pyi < H))
					continue;
				const size_t pix_id = (size_t)W * pyi + pxi;
				const float pixf[2] = { (float)pxi, (float)pyi };
				const float ndcx = pix2ndc(pixf[0], W), ndcy = pix2ndc(pixf[1], H);
				const float T_final = 1 - alphas[pix_id];
				float T = T_final;
				const uint32_t last_contributor = n_contrib[pix_id];
				float accum_rec[3] = { 0, 0, 0 }, dL_dpixel[3];
				float accum_depth_rec = 0, accum_alpha_rec = 0;
				for (int i = 0; i < 3; i++)
					dL_dpixel[i] = dL_dpixels[(size_t)i * H * W + pix_id];
				const float dL_dpixel_depth = dL_dpixel_depths[pix_id];
				const float dL_dalpha = dL_dalphas[pix_id];
				float last_alpha = 0, last_color[3] = { 0, 0, 0 }, last_depth = 0;

				/* entries [r0, r0 + last_contributor) from the back */
				for (uint32_t k = r0 + last_contributor; k-- > r0;) {
					const uint32_t id = point_list[k];
					const float dx = xy[2 * (size_t)id] - pixf[0], dy = xy[2 * (size_t)id + 1] - pixf[1];
					const float *co = conic_opacity + 4 * (size_t)id;
					const float power = -0.5f * (co[0] * dx * dx + co[2] * dy * dy) - co[1] * dx * dy;
					if (power > 0.0f)
						continue;
					const float G = expf(power);
					const float alpha = fminf(0.99f, co[3] * G);
					if (alpha < 1.0f / 255.0f)
						continue;
					if (outside_box(ndcx, ndcy, zw[2 * (size_t)id + 1], tanx, tany, projinv, low, up))
						continue;

					T = T / (1.f - alpha);
					const float dchannel_dcolor = alpha * T;
					const float dpixel_depth_ddepth = alpha * T;
					float dL_dopa = 0.0f;
					for (int ch = 0; ch < 3; ch++) {
						const float c = colors[3 * (size_t)id + ch];
						accum_rec[ch] = last_alpha * last_color[ch] + (1.f - last_alpha) * accum_rec[ch];
						last_color[ch] = c;
						const float dL_dchannel = dL_dpixel[ch];
						dL_dopa += (c - accum_rec[ch]) * dL_dchannel;
						atomic_addf(&dL_dcolors[3 * (size_t)id + ch], dchannel_dcolor * dL_dchannel);
					}
					const float c_d = depths[id];
					accum_depth_rec = last_alpha * last_depth + (1.f - last_alpha) * accum_depth_rec;
					last_depth = c_d;
					dL_dopa += (c_d - accum_depth_rec) * dL_dpixel_depth;
					atomic_addf(&dL_ddepths[id], dpixel_depth_ddepth * dL_dpixel_depth);

					accum_alpha_rec = last_alpha + (1.f - last_alpha) * accum_alpha_rec;
					dL_dopa += (1 - accum_alpha_rec) * dL_dalpha;

					dL_dopa *= T;
					last_alpha = alpha;

					float bg_dot_dpixel = 0;
					for (int i = 0; i < 3; i++)
						bg_dot_dpixel += bg[i] * dL_dpixel[i];
					dL_dopa += (-T_final / (1.f - alpha)) * bg_dot_dpixel;

					const float dL_dG = co[3] * dL_dopa;
					const float gdx = G * dx;
					const float gdy = G * dy;
					const float dG_ddelx = -gdx * co[0] - gdy * co[1];
					const float dG_ddely = -gdy * co[2] - gdx * co[1];

					atomic_addf(&dL_dmean2D[3 * (size_t)id + 0], dL_dG * dG_ddelx * ddelx_dx);
					atomic_addf(&dL_dmean2D[3 * (size_t)id + 1], dL_dG * dG_ddely * ddely_dy);
					atomic_addf(&dL_dconic2D[4 * (size_t)id + 0], -0.5f * gdx * dx * dL_dG);
					atomic_addf(&dL_dconic2D[4 * (size_t)id + 1], -0.5f * gdx * dy * dL_dG);
					atomic_addf(&dL_dconic2D[4 * (size_t)id + 3], -0.5f * gdy * dy * dL_dG);
					atomic_addf(&dL_dopacity[id], G * dL_dopa);
				}
			}
		}
	}
}

/* ---- backward preprocess ---------------------------------------------------- */

/* K/cuda_rasterizer_hgs/backward.cu:144-274.  Writes dL_dcov[6*idx..] and
 * ASSIGNS dL_dmeans[3*idx..] for Gaussians with radii > 0. */
void orc_cov2d_backward(int P, const float *means, const int *radii, const float *cov3Ds,
	float h_x, float h_y, float tanx, float tany, const float *view, const float *dL_dconics,
	float *dL_dmeans, float *dL_dcov)
{
#pragma omp parallel for schedule(static) num_threads(g_threads)
	for (int idx = 0; idx < P; idx++) {
		if (!(radii[idx] > 0))
			continue;
		const float *cov3D = cov3Ds + 6 * (size_t)idx;
		const float *mean = means + 3 * (size_t)idx;
		const float dLc[3] = { dL_dconics[4 * (size_t)idx], dL_dconics[4 * (size_t)idx + 1], dL_dconics[4 * (size_t)idx + 3] };
		ewa_t e;
		ewa_project(mean, h_x, h_y, tanx, tany, cov3D, view, &e);
		const float *t = e.t;
		const float x_grad_mul = (e.txtz < -e.limx || e.txtz > e.limx) ? 0 : 1;
		const float y_grad_mul = (e.tytz < -e.limy || e.tytz > e.limy) ? 0 : 1;
		const mat3 *T = &e.T, *Vrk = &e.Vrk, *Wm = &e.W;
#define Tm(i, j) T->m[i][j]
#define Vm(i, j) Vrk->m[i][j]
		float a = e.cov.m[0][0] + 0.3f;
		float b = e.cov.m[0][1];
		float c = e.cov.m[1][1] + 0.3f;
		float denom = a * c - b * b;
		float dL_da = 0, dL_db = 0, dL_dc = 0;
		float denom2inv = 1.0f / ((denom * denom) + 0.0000001f);
		float *dcv = dL_dcov + 6 * (size_t)idx;
		if (denom2inv != 0) {
			dL_da = denom2inv * (-c * c * dLc[0] + 2 * b * c * dLc[1] + (denom - a * c) * dLc[2]);
			dL_dc = denom2inv * (-a * a * dLc[2] + 2 * a * b * dLc[1] + (denom - a * c) * dLc[0]);
			dL_db = denom2inv * 2 * (b * c * dLc[0] - (denom + 2 * b * b) * dLc[1] + a * b * dLc[2]);
			dcv[0] = (Tm(0, 0) * Tm(0, 0) * dL_da + Tm(0, 0) * Tm(1, 0) * dL_db + Tm(1, 0) * Tm(1, 0) * dL_dc);
			dcv[3] = (Tm(0, 1) * Tm(0, 1) * dL_da + Tm(0, 1) * Tm(1, 1) * dL_db + Tm(1, 1) * Tm(1, 1) * dL_dc);
			dcv[5] = (Tm(0, 2) * Tm(0, 2) * dL_da + Tm(0, 2) * Tm(1, 2) * dL_db + Tm(1, 2) * Tm(1, 2) * dL_dc);
			dcv[1] = 2 * Tm(0, 0) * Tm(0, 1) * dL_da + (Tm(0, 0) * Tm(1, 1) + Tm(0, 1) * Tm(1, 0)) * dL_db + 2 * Tm(1, 0) * Tm(1, 1) * dL_dc;
			dcv[2] = 2 * Tm(0, 0) * Tm(0, 2) * dL_da + (Tm(0, 0) * Tm(1, 2) + Tm(0, 2) * Tm(1, 0)) * dL_db + 2 * Tm(1, 0) * Tm(1, 2) * dL_dc;
			dcv[4] = 2 * Tm(0, 2) * Tm(0, 1) * dL_da + (Tm(0, 1) * Tm(1, 2) + Tm(0, 2) * Tm(1, 1)) * dL_db + 2 * Tm(1, 1) * Tm(1, 2) * dL_dc;
		} else {
			for (int i = 0; i < 6; i++)
				dcv[i] = 0;
		}
		float dL_dT00 = 2 * (Tm(0, 0) * Vm(0, 0) + Tm(0, 1) * Vm(0, 1) + Tm(0, 2) * Vm(0, 2)) * dL_da +
			(Tm(1, 0) * Vm(0, 0) + Tm(1, 1) * Vm(0, 1) + Tm(1, 2) * Vm(0, 2)) * dL_db;
		float dL_dT01 = 2 * (Tm(0, 0) * Vm(1, 0) + Tm(0, 1) * Vm(1, 1) + Tm(0, 2) * Vm(1, 2)) * dL_da +
			(Tm(1, 0) * Vm(1, 0) + Tm(1, 1) * Vm(1, 1) + Tm(1, 2) * Vm(1, 2)) * dL_db;
		float dL_dT02 = 2 * (Tm(0, 0) * Vm(2, 0) + Tm(0, 1) * Vm(2, 1) + Tm(0, 2) * Vm(2, 2)) * dL_da +
			(Tm(1, 0) * Vm(2, 0) + Tm(1, 1) * Vm(2, 1) + Tm(1, 2) * Vm(2, 2)) * dL_db;
		float dL_dT10 = 2 * (Tm(1, 0) * Vm(0, 0) + Tm(1, 1) * Vm(0, 1) + Tm(1, 2) * Vm(0, 2)) * dL_dc +
			(Tm(0, 0) * Vm(0, 0) + Tm(0, 1) * Vm(0, 1) + Tm(0, 2) * Vm(0, 2)) * dL_db;
		float dL_dT11 = 2 * (Tm(1, 0) * Vm(1, 0) + Tm(1, 1) * Vm(1, 1) + Tm(1, 2) * Vm(1, 2)) * dL_dc +
			(Tm(0, 0) * Vm(1, 0) + Tm(0, 1) * Vm(1, 1) + Tm(0, 2) * Vm(1, 2)) * dL_db;
		float dL_dT12 = 2 * (Tm(1, 0) * Vm(2, 0) + Tm(1, 1) * Vm(2, 1) + Tm(1, 2) * Vm(2, 2)) * dL_dc +
			(Tm(0, 0) * Vm(2, 0) + Tm(0, 1) * Vm(2, 1) + Tm(0, 2) * Vm(2, 2)) * dL_db;
#undef Tm
#undef Vm
		float dL_dJ00 = Wm->m[0][0] * dL_dT00 + Wm->m[0][1] * dL_dT01 + Wm->m[0][2] * dL_dT02;
		float dL_dJ02 = Wm->m[2][0] * dL_dT00 + Wm->m[2][1] * dL_dT01 + Wm->m[2][2] * dL_dT02;
		float dL_dJ11 = Wm->m[1][0] * dL_dT10 + Wm->m[1][1] * dL_dT11 + Wm->m[1][2] * dL_dT12;
		float dL_dJ12 = Wm->m[2][0] * dL_dT10 + Wm->m[2][1] * dL_dT11 + Wm->m[2][2] * dL_dT12;

		float tz = 1.f / t[2];
		float tz2 = tz * tz;
		float tz3 = tz2 * tz;
		float dL_dtx = x_grad_mul * -h_x * tz2 * dL_dJ02;
		float dL_dty = y_grad_mul * -h_y * tz2 * dL_dJ12;
		float dL_dtz = -h_x * tz2 * dL_dJ00 - h_y * tz2 * dL_dJ11 + (2 * h_x * t[0]) * tz3 * dL_dJ02 + (2 * h_y * t[1]) * tz3 * dL_dJ12;

		/* transformVec4x3Transpose, auxiliary.h:104-112 */
		float *dm = dL_dmeans + 3 * (size_t)idx;
		dm[0] = view[0] * dL_dtx + view[1] * dL_dty + view[2] * dL_dtz;
		dm[1] = view[4] * dL_dtx + view[5] * dL_dty + view[6] * dL_dtz;
		dm[2] = view[8] * dL_dtx + view[9] * dL_dty + view[10] * dL_dtz;
	}
}

/* K/cuda_rasterizer_hgs/backward.cu:20-139: SH backward for one Gaussian.
 * dL_dsh points at its (M,3) rows; adds the view-direction part into dL_dmean. */
static void sh_backward(int deg, const float *pos, const float *campos, const float *sh, const uint8_t *clamped,
	const float *dL_dcolor, float *dL_dmean, float *dL_dsh)
{
	float dir_orig[3] = { pos[0] - campos[0], pos[1] - campos[1], pos[2] - campos[2] };
	float len = sqrtf(dir_orig[0] * dir_orig[0] + dir_orig[1] * dir_orig[1] + dir_orig[2] * dir_orig[2]);
	float x = dir_orig[0] / len, y = dir_orig[1] / len, z = dir_orig[2] / len;
	float dL_dRGB[3];
	for (int c = 0; c < 3; c++)
		dL_dRGB[c] = dL_dcolor[c] * (clamped[c] ? 0 : 1);
	float dL_ddir[3];
	float ddx[3], ddy[3], ddz[3];  /* dRGB/dx, dRGB/dy, dRGB/dz per channel */
	for (int c = 0; c < 3; c++) {
#define SH(k) sh[3 * (k) + c]
#define DSH(k) dL_dsh[3 * (k) + c]
		float dRGBdx = 0, dRGBdy = 0, dRGBdz = 0;
		DSH(0) = SH_C0 * dL_dRGB[c];
		if (deg > 0) {
			float d1 = -SH_C1 * y, d2 = SH_C1 * z, d3 = -SH_C1 * x;
			DSH(1) = d1 * dL_dRGB[c];
			DSH(2) = d2 * dL_dRGB[c];
			DSH(3) = d3 * dL_dRGB[c];
			dRGBdx = -SH_C1 * SH(3);
			dRGBdy = -SH_C1 * SH(1);
			dRGBdz = SH_C1 * SH(2);
			if (deg > 1) {
				float xx = x * x, yy = y * y, zz = z * z;
				float xy = x * y, yz = y * z, xz = x * z;
				DSH(4) = (SH_C2[0] * xy) * dL_dRGB[c];
				DSH(5) = (SH_C2[1] * yz) * dL_dRGB[c];
				DSH(6) = (SH_C2[2] * (2.f * zz - xx - yy)) * dL_dRGB[c];
				DSH(7) = (SH_C2[3] * xz) * dL_dRGB[c];
				DSH(8) = (SH_C2[4] * (xx - yy)) * dL_dRGB[c];
				dRGBdx += SH_C2[0] * y * SH(4) + SH_C2[2] * 2.f * -x * SH(6) + SH_C2[3] * z * SH(7) + SH_C2[4] * 2.f * x * SH(8);
				dRGBdy += SH_C2[0] * x * SH(4) + SH_C2[1] * z * SH(5) + SH_C2[2] * 2.f * -y * SH(6) + SH_C2[4] * 2.f * -y * SH(8);
				dRGBdz += SH_C2[1] * y * SH(5) + SH_C2[2] * 2.f * 2.f * z * SH(6) + SH_C2[3] * x * SH(7);
				if (deg > 2) {
					DSH(9) = (SH_C3[0] * y * (3.f * xx - yy)) * dL_dRGB[c];
					DSH(10) = (SH_C3[1] * xy * z) * dL_dRGB[c];
					DSH(11) = (SH_C3[2] * y * (4.f * zz - xx - yy)) * dL_dRGB[c];
					DSH(12) = (SH_C3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy)) * dL_dRGB[c];
					DSH(13) = (SH_C3[4] * x * (4.f * zz - xx - yy)) * dL_dRGB[c];
					DSH(14) = (SH_C3[5] * z * (xx - yy)) * dL_dRGB[c];
					DSH(15) = (SH_C3[6] * x * (xx - 3.f * yy)) * dL_dRGB[c];
					dRGBdx += (
						SH_C3[0] * SH(9) * 3.f * 2.f * xy +
						SH_C3[1] * SH(10) * yz +
						SH_C3[2] * SH(11) * -2.f * xy +
						SH_C3[3] * SH(12) * -3.f * 2.f * xz +
						SH_C3[4] * SH(13) * (-3.f * xx + 4.f * zz - yy) +
						SH_C3[5] * SH(14) * 2.f * xz +
						SH_C3[6] * SH(15) * 3.f * (xx - yy));
					dRGBdy += (
						SH_C3[0] * SH(9) * 3.f * (xx - yy) +
						SH_C3[1] * SH(10) * xz +
						SH_C3[2] * SH(11) * (-3.f * yy + 4.f * zz - xx) +
						SH_C3[3] * SH(12) * -3.f * 2.f * yz +
						SH_C3[4] * SH(13) * -2.f * xy +
						SH_C3[5] * SH(14) * -2.f * yz +
						SH_C3[6] * SH(15) * -3.f * 2.f * xy);
					dRGBdz += (
						SH_C3[1] * SH(10) * xy +
						SH_C3[2] * SH(11) * 4.f * 2.f * yz +
						SH_C3[3] * SH(12) * 3.f * (2.f * zz - xx - yy) +
						SH_C3[4] * SH(13) * 4.f * 2.f * xz +
						SH_C3[5] * SH(14) * (xx - yy));
				}
			}
		}
#undef SH
#undef DSH
		ddx[c] = dRGBdx; ddy[c] = dRGBdy; ddz[c] = dRGBdz;
	}
	dL_ddir[0] = ddx[0] * dL_dRGB[0] + ddx[1] * dL_dRGB[1] + ddx[2] * dL_dRGB[2];
	dL_ddir[1] = ddy[0] * dL_dRGB[0] + ddy[1] * dL_dRGB[1] + ddy[2] * dL_dRGB[2];
	dL_ddir[2] = ddz[0] * dL_dRGB[0] + ddz[1] * dL_dRGB[1] + ddz[2] * dL_dRGB[2];

	/* dnormvdv, auxiliary.h:123-133 */
	const float *v = dir_orig, *dv = dL_ddir;
	float sum2 = v[0] * v[0] + v[1] * v[1] + v[2] * v[2];
	float invsum32 = 1.0f / sqrtf(sum2 * sum2 * sum2);
	float g0 = ((+sum2 - v[0] * v[0]) * dv[0] - v[1] * v[0] * dv[1] - v[2] * v[0] * dv[2]) * invsum32;
	float g1 = (-v[0] * v[1] * dv[0] + (sum2 - v[1] * v[1]) * dv[1] - v[2] * v[1] * dv[2]) * invsum32;
	float g2 = (-v[0] * v[2] * dv[0] - v[1] * v[2] * dv[1] + (sum2 - v[2] * v[2]) * dv[2]) * invsum32;
	dL_dmean[0] += g0;
	dL_dmean[1] += g1;
	dL_dmean[2] += g2;
}

/* K/cuda_rasterizer_hgs/backward.cu:278-341: cov3D gradient to scale and the
 * raw (r,x,y,z) quaternion; no normalisation Jacobian (:340). */
static void cov3d_backward(const float *scale, float mod, const float *rot, const float *dL_dcov3D, float *dL_dscale, float *dL_drot)
{
	float r = rot[0], x = rot[1], y = rot[2], z = rot[3];
	mat3 R = mat3_cols(
		1.f - 2.f * (y * y + z * z), 2.f * (x * y - r * z), 2.f * (x * z + r * y),
		2.f * (x * y + r * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - r * x),
		2.f * (x * z - r * y), 2.f * (y * z + r * x), 1.f - 2.f * (x * x + y * y));
	mat3 S = mat3_cols(1, 0, 0, 0, 1, 0, 0, 0, 1);
	float s[3] = { mod * scale[0], mod * scale[1], mod * scale[2] };
	S.m[0][0] = s[0];
	S.m[1][1] = s[1];
	S.m[2][2] = s[2];
	mat3 M = mat3_mul(&S, &R);
	const float *d = dL_dcov3D;
	mat3 dL_dSigma = mat3_cols(
		d[0], 0.5f * d[1], 0.5f * d[2],
		0.5f * d[1], d[3], 0.5f * d[4],
		0.5f * d[2], 0.5f * d[4], d[5]);
	mat3 M2;
	for (int c = 0; c < 3; c++)
		for (int rr = 0; rr < 3; rr++)
			M2.m[c][rr] = M.m[c][rr] * 2.0f;
	mat3 dL_dM = mat3_mul(&M2, &dL_dSigma);
	mat3 Rt = mat3_t(&R);
	mat3 dL_dMt = mat3_t(&dL_dM);
	for (int k = 0; k < 3; k++)
		dL_dscale[k] = Rt.m[k][0] * dL_dMt.m[k][0] + Rt.m[k][1] * dL_dMt.m[k][1] + Rt.m[k][2] * dL_dMt.m[k][2];
	for (int k = 0; k < 3; k++)
		for (int rr = 0; rr < 3; rr++)
			dL_dMt.m[k][rr] *= s[k];
#define D(i, j) dL_dMt.m[i][j]
	dL_drot[0] = 2 * z * (D(0, 1) - D(1, 0)) + 2 * y * (D(2, 0) - D(0, 2)) + 2 * x * (D(1, 2) - D(2, 1));
	dL_drot[1] = 2 * y * (D(1, 0) + D(0, 1)) + 2 * z * (D(2, 0) + D(0, 2)) + 2 * r * (D(1, 2) - D(2, 1)) - 4 * x * (D(2, 2) + D(1, 1));
	dL_drot[2] = 2 * x * (D(1, 0) + D(0, 1)) + 2 * r * (D(2, 0) - D(0, 2)) + 2 * z * (D(1, 2) + D(2, 1)) - 4 * y * (D(2, 2) + D(0, 0));
	dL_drot[3] = 2 * r * (D(0, 1) - D(1, 0)) + 2 * x * (D(2, 0) + D(0, 2)) + 2 * y * (D(1, 2) + D(2, 1)) - 4 * z * (D(1, 1) + D(0, 0));
#undef D
}

/* K/cuda_rasterizer_hgs/backward.cu:346-412.  shs / scales may be NULL like in
 * the reference (then those parts are skipped).  dL_dmeans is accumulated into
 * (it holds the covariance part written by orc_cov2d_backward). */
void orc_preprocess_backward(int P, int D, int M, const float *means, const int *radii, const float *shs,
	const uint8_t *clamped, const float *scales, const float *rots, float mod,
	const float *view, const float *proj, const float *campos,
	const float *dL_dmean2D, float *dL_dmeans, const float *dL_dcolor, const float *dL_ddepth,
	const float *dL_dcov3D, float *dL_dsh, float *dL_dscale, float *dL_drot)
{
#pragma omp parallel for schedule(static) num_threads(g_threads)
	for (int idx = 0; idx < P; idx++) {
		if (!(radii[idx] > 0))
			continue;
		const float *m = means + 3 * (size_t)idx;
		float m_hom[4];
		xform4x4(m, proj, m_hom);
		float m_w = 1.0f / (m_hom[3] + 0.0000001f);
		const float *g2 = dL_dmean2D + 3 * (size_t)idx;
		float mul1 = (proj[0] * m[0] + proj[4] * m[1] + proj[8] * m[2] + proj[12]) * m_w * m_w;
		float mul2 = (proj[1] * m[0] + proj[5] * m[1] + proj[9] * m[2] + proj[13]) * m_w * m_w;
		float dm[3];
		dm[0] = (proj[0] * m_w - proj[3] * mul1) * g2[0] + (proj[1] * m_w - proj[3] * mul2) * g2[1];
		dm[1] = (proj[4] * m_w - proj[7] * mul1) * g2[0] + (proj[5] * m_w - proj[7] * mul2) * g2[1];
		dm[2] = (proj[8] * m_w - proj[11] * mul1) * g2[0] + (proj[9] * m_w - proj[11] * mul2) * g2[1];
		float *out = dL_dmeans + 3 * (size_t)idx;
		out[0] += dm[0];
		out[1] += dm[1];
		out[2] += dm[2];

		float mul3 = view[2] * m[0] + view[6] * m[1] + view[10] * m[2] + view[14];
		float dm2[3];
		dm2[0] = (view[2] - view[3] * mul3) * dL_ddepth[idx];
		dm2[1] = (view[6] - view[7] * mul3) * dL_ddepth[idx];
		dm2[2] = (view[10] - view[11] * mul3) * dL_ddepth[idx];
		out[0] += dm2[0];
		out[1] += dm2[1];
		out[2] += dm2[2];

		if (shs)
			sh_backward(D, m, campos, shs + 3 * (size_t)M * idx, clamped + 3 * (size_t)idx,
				dL_dcolor + 3 * (size_t)idx, out, dL_dsh + 3 * (size_t)M * idx);
		if (scales)
			cov3d_backward(scales + 3 * (size_t)idx, mod, rots + 4 * (size_t)idx, dL_dcov3D + 6 * (size_t)idx,
				dL_dscale + 3 * (size_t)idx, dL_drot + 4 * (size_t)idx);
	}
}
