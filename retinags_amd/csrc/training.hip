// The two steps either side of the renderer in a training iteration: the image loss
// (1 - lambda) L1 + lambda (1 - SSIM) with its gradient, and the Adam update of the parameters.
//
// SSIM (utils/loss_utils.py:39-63): five zero-padded 11x11 Gaussian-window (sigma 1.5) means per
// pixel and channel, of x, y, x^2, y^2 and xy, then
//   f = (2 mu1 mu2 + C1)(2 s12 + C2) / ((mu1^2 + mu2^2 + C1)(s11 + s22 + C2)),  C1 = 0.01^2, C2 = 0.03^2.
// The window is an outer product, so each mean is a row pass followed by a column pass.  A
// workgroup produces a 32x16 tile of one channel: the 42x26 pixels it needs go to LDS once, the
// row pass leaves 5 x 26 x 32 partial means in LDS, the column pass finishes them, and the
// per-pixel SSIM and |x - y| are summed per workgroup (a second kernel adds the partial sums in a
// fixed order, so the loss is reproducible).  For the backward the same kernel stores three
// derivative maps per pixel,
//   a = df/dmu1,  b = df/dE[x^2] = -f / B2,  c = df/dE[xy] = 2 A1 / (B1 B2),
// and the gradient is their windowed means: dL/dx(q) = W*a (q) + 2 x(q) W*b (q) + y(q) W*c (q),
// which the backward kernel computes with the same two passes.  Bound by HBM (44 bytes per pixel
// and channel over both kernels) and by LDS reads.
//
// Activation (scene/gaussian_nn_module.py:373-394): what a submodel's renderer and neighbours see
// is exp of the stored scales, sigmoid of the stored opacities, the normalised quaternions and the
// two SH parameter tensors joined: one flat pass forward and one backward.
//
// Adam (torch.optim.Adam as the reference configures it, scene/gaussian_nn_module.py:429-444:
// eps 1e-15, no weight decay, no amsgrad): one pass over parameter, gradient and both moments.
#include "rgs_device.h"
#include "rgs_kernels.h"

namespace rgs {

namespace {

constexpr int kLossTileW = 32, kLossTileH = 16;
constexpr int kHalo = 5, kTaps = 11;
constexpr int kRegionW = kLossTileW + 2 * kHalo, kRegionH = kLossTileH + 2 * kHalo;
constexpr int kRowRun = 4;   // columns a thread takes in the row pass (26 x 8 runs for 256 threads)
constexpr int kColRun = 2;   // rows a thread takes in the column pass (8 x 32 runs)
static_assert(kRegionH * (kLossTileW / kRowRun) <= 256 && (kLossTileH / kColRun) * kLossTileW == 256, "pass shapes");

__device__ __forceinline__ float block256_sum(float v, float* lds)
{
	v = wave_sum_to_lane63(v);
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	if (lane == 63)
		lds[wave] = v;
	__syncthreads();
	const float total = lds[0] + lds[1] + lds[2] + lds[3];
	__syncthreads();
	return total;
}

// Workgroups are dealt to the 8 XCDs in turn, and each XCD has its own L2.  Workgroup b therefore
// takes tile (b % 8) * ceil(tiles / 8) + b / 8 of the row-major (channel, tile row, tile column)
// order: an XCD gets a contiguous band of tiles, and the halo a tile shares with its neighbours is
// fetched from memory once per band instead of once per tile.
struct LossTile {
	int channel, tx, ty;
	uint32_t linear;
	bool valid;
};

__device__ __forceinline__ LossTile loss_tile_of_block(const LossArgs& a)
{
	const uint32_t tiles_x = (a.W + kLossTileW - 1) / kLossTileW, tiles_y = (a.H + kLossTileH - 1) / kLossTileH;
	const uint32_t total = tiles_x * tiles_y * (uint32_t)a.C;
	const uint32_t per_xcd = (total + 7) / 8;
	LossTile t;
	t.linear = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
	t.valid = blockIdx.x / 8 < per_xcd && t.linear < total;
	const uint32_t in_plane = t.linear % (tiles_x * tiles_y);
	t.channel = (int)(t.linear / (tiles_x * tiles_y));
	t.ty = (int)(in_plane / tiles_x);
	t.tx = (int)(in_plane % tiles_x);
	return t;
}

__global__ __launch_bounds__(256) void ssim_forward_kernel(LossArgs a)
{
	__shared__ float sx[kRegionH][kRegionW + 1];
	__shared__ float sy[kRegionH][kRegionW + 1];
	__shared__ float rows[5][kRegionH][kLossTileW + 1];
	__shared__ float red[4];
	const int tid = threadIdx.x;
	const LossTile tile = loss_tile_of_block(a);
	if (!tile.valid)
		return;
	const size_t plane = (size_t)tile.channel * a.H * a.W;
	const int x0 = tile.tx * kLossTileW - kHalo, y0 = tile.ty * kLossTileH - kHalo;
	for (int i = tid; i < kRegionH * kRegionW; i += 256) {
		const int r = i / kRegionW, c = i % kRegionW;
		const int gx = x0 + c, gy = y0 + r;
		const bool inside = gx >= 0 && gx < a.W && gy >= 0 && gy < a.H;
		const size_t at = plane + (size_t)gy * a.W + gx;
		sx[r][c] = inside ? a.x[at] : 0.f;
		sy[r][c] = inside ? a.y[at] : 0.f;
	}
	__syncthreads();
	// row pass: a thread takes 4 neighbouring columns of one row, so 14 pixels of each image
	// feed 4 x 5 sums (28 LDS reads instead of 88)
	if (tid < kRegionH * (kLossTileW / kRowRun)) {
		const int r = tid / (kLossTileW / kRowRun), c0 = kRowRun * (tid % (kLossTileW / kRowRun));
		float u[kTaps + kRowRun - 1], v[kTaps + kRowRun - 1];
#pragma unroll
		for (int k = 0; k < kTaps + kRowRun - 1; k++) {
			u[k] = sx[r][c0 + k];
			v[k] = sy[r][c0 + k];
		}
#pragma unroll
		for (int o = 0; o < kRowRun; o++) {
			float m1 = 0.f, m2 = 0.f, xx = 0.f, yy = 0.f, xy = 0.f;
#pragma unroll
			for (int k = 0; k < kTaps; k++) {
				const float w = a.w[k];
				m1 += w * u[o + k];
				m2 += w * v[o + k];
				xx += w * (u[o + k] * u[o + k]);
				yy += w * (v[o + k] * v[o + k]);
				xy += w * (u[o + k] * v[o + k]);
			}
			rows[0][r][c0 + o] = m1; rows[1][r][c0 + o] = m2; rows[2][r][c0 + o] = xx; rows[3][r][c0 + o] = yy;
			rows[4][r][c0 + o] = xy;
		}
	}
	__syncthreads();
	float ssim_sum = 0.f, l1_sum = 0.f;
	// column pass: a thread takes kColRun rows of one column
	float part[5][kTaps + kColRun - 1];
	const int col = tid % kLossTileW, row0 = kColRun * (tid / kLossTileW);
#pragma unroll
	for (int q = 0; q < 5; q++)
#pragma unroll
		for (int k = 0; k < kTaps + kColRun - 1; k++)
			part[q][k] = rows[q][row0 + k][col];
#pragma unroll
	for (int o = 0; o < kColRun; o++) {
		const int r = row0 + o, c = col;
		const int gx = x0 + kHalo + c, gy = y0 + kHalo + r;
		if (gx >= a.W || gy >= a.H)
			continue;
		float m1 = 0.f, m2 = 0.f, xx = 0.f, yy = 0.f, xy = 0.f;
#pragma unroll
		for (int k = 0; k < kTaps; k++) {
			const float w = a.w[k];
			m1 += w * part[0][o + k];
			m2 += w * part[1][o + k];
			xx += w * part[2][o + k];
			yy += w * part[3][o + k];
			xy += w * part[4][o + k];
		}
		const float C1 = 0.01f * 0.01f, C2 = 0.03f * 0.03f;
		const float m11 = m1 * m1, m22 = m2 * m2, m12 = m1 * m2;
		const float s11 = xx - m11, s22 = yy - m22, s12 = xy - m12;
		const float A1 = 2.f * m12 + C1, A2 = 2.f * s12 + C2, B1 = m11 + m22 + C1, B2 = s11 + s22 + C2;
		const float inv = 1.f / (B1 * B2);
		const float f = A1 * A2 * inv;
		ssim_sum += f;
		l1_sum += fabsf(sx[r + kHalo][c + kHalo] - sy[r + kHalo][c + kHalo]);
		if (a.maps) {
			const size_t n = (size_t)a.C * a.H * a.W;
			const size_t at = plane + (size_t)gy * a.W + gx;
			a.maps[at] = 2.f * m2 * (A2 - A1) * inv - 2.f * m1 * f * (1.f / B1 - 1.f / B2);
			a.maps[n + at] = -f / B2;
			a.maps[2 * n + at] = 2.f * A1 * inv;
		}
	}
	ssim_sum = block256_sum(ssim_sum, red);
	l1_sum = block256_sum(l1_sum, red);
	if (tid == 0) {
		a.partial[2 * (size_t)tile.linear] = ssim_sum;
		a.partial[2 * (size_t)tile.linear + 1] = l1_sum;
	}
}

// One workgroup: the partial sums in index order (double accumulators), then the three results.
__global__ __launch_bounds__(256) void loss_finish_kernel(LossArgs a, uint32_t blocks)
{
	__shared__ double red[2][256];
	double s = 0.0, l = 0.0;
	for (uint32_t i = threadIdx.x; i < blocks; i += 256) {
		s += (double)a.partial[2 * i];
		l += (double)a.partial[2 * i + 1];
	}
	red[0][threadIdx.x] = s;
	red[1][threadIdx.x] = l;
	__syncthreads();
	for (int step = 128; step > 0; step >>= 1) {
		if ((int)threadIdx.x < step) {
			red[0][threadIdx.x] += red[0][threadIdx.x + step];
			red[1][threadIdx.x] += red[1][threadIdx.x + step];
		}
		__syncthreads();
	}
	if (threadIdx.x == 0) {
		const double n = (double)a.C * a.H * a.W;
		const float ssim = (float)(red[0][0] / n), l1 = (float)(red[1][0] / n);
		a.out[0] = (1.0f - a.lambda) * l1 + a.lambda * (1.0f - ssim);
		a.out[1] = l1;
		a.out[2] = ssim;
	}
}

__global__ __launch_bounds__(256) void ssim_backward_kernel(LossArgs a)
{
	__shared__ float sm[3][kRegionH][kRegionW + 1];
	__shared__ float rows[3][kRegionH][kLossTileW + 1];
	const int tid = threadIdx.x;
	const size_t n = (size_t)a.C * a.H * a.W;
	const LossTile tile = loss_tile_of_block(a);
	if (!tile.valid)
		return;
	const size_t plane = (size_t)tile.channel * a.H * a.W;
	const int x0 = tile.tx * kLossTileW - kHalo, y0 = tile.ty * kLossTileH - kHalo;
	for (int i = tid; i < kRegionH * kRegionW; i += 256) {
		const int r = i / kRegionW, c = i % kRegionW;
		const int gx = x0 + c, gy = y0 + r;
		const bool inside = gx >= 0 && gx < a.W && gy >= 0 && gy < a.H;
		const size_t at = plane + (size_t)gy * a.W + gx;
		sm[0][r][c] = inside ? a.maps[at] : 0.f;
		sm[1][r][c] = inside ? a.maps[n + at] : 0.f;
		sm[2][r][c] = inside ? a.maps[2 * n + at] : 0.f;
	}
	__syncthreads();
	if (tid < kRegionH * (kLossTileW / kRowRun)) {
		const int r = tid / (kLossTileW / kRowRun), c0 = kRowRun * (tid % (kLossTileW / kRowRun));
#pragma unroll
		for (int q = 0; q < 3; q++) {
			float u[kTaps + kRowRun - 1];
#pragma unroll
			for (int k = 0; k < kTaps + kRowRun - 1; k++)
				u[k] = sm[q][r][c0 + k];
#pragma unroll
			for (int o = 0; o < kRowRun; o++) {
				float acc = 0.f;
#pragma unroll
				for (int k = 0; k < kTaps; k++)
					acc += a.w[k] * u[o + k];
				rows[q][r][c0 + o] = acc;
			}
		}
	}
	__syncthreads();
	const float upstream = a.grad_loss ? a.grad_loss[0] : 1.0f;
	const float l1_scale = upstream * (1.0f - a.lambda) / (float)n, ssim_scale = -upstream * a.lambda / (float)n;
	float part[3][kTaps + kColRun - 1];
	const int col = tid % kLossTileW, row0 = kColRun * (tid / kLossTileW);
#pragma unroll
	for (int q = 0; q < 3; q++)
#pragma unroll
		for (int k = 0; k < kTaps + kColRun - 1; k++)
			part[q][k] = rows[q][row0 + k][col];
#pragma unroll
	for (int o = 0; o < kColRun; o++) {
		const int r = row0 + o, c = col;
		const int gx = x0 + kHalo + c, gy = y0 + kHalo + r;
		if (gx >= a.W || gy >= a.H)
			continue;
		float ca = 0.f, cb = 0.f, cc = 0.f;
#pragma unroll
		for (int k = 0; k < kTaps; k++) {
			const float w = a.w[k];
			ca += w * part[0][o + k];
			cb += w * part[1][o + k];
			cc += w * part[2][o + k];
		}
		const size_t at = plane + (size_t)gy * a.W + gx;
		const float x = a.x[at], y = a.y[at];
		const float d = x - y;
		const float sign = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
		a.d_image[at] = l1_scale * sign + ssim_scale * (ca + 2.f * x * cb + y * cc);
	}
}

// torch.optim.Adam's single-tensor update, in its order of operations:
//   m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g g;
//   p = p - (lr / (1 - b1^t)) * m / (sqrt(v) / sqrt(1 - b2^t) + eps)
// One launch updates every tensor of a parameter-group list; a workgroup takes kAdamBlock
// consecutive elements of one tensor.
constexpr int kAdamBlock = 4096;

__device__ __forceinline__ void adam_one(float& p, float g, float& m, float& v, const AdamTensor& t, const AdamArgs& a)
{
	m = m * a.beta1 + g * a.one_minus_beta1;
	v = v * a.beta2 + (g * g) * a.one_minus_beta2;
	const float denom = sqrtf(v) / t.bias2_sqrt + a.eps;
	p = p - t.step_size * (m / denom);
}

__global__ __launch_bounds__(256) void adam_step_kernel(AdamArgs a)
{
	int k = 0;
	while (k + 1 < a.tensors && blockIdx.x >= a.t[k + 1].block0)
		k++;
	const AdamTensor& t = a.t[k];
	const size_t base = (size_t)(blockIdx.x - t.block0) * kAdamBlock;
#pragma unroll
	for (int it = 0; it < kAdamBlock / 1024; it++) {
		const size_t i = base + (size_t)it * 1024 + threadIdx.x * 4;
		if (i >= t.n)
			break;
		if (i + 4 <= t.n && t.by_16_bytes) {
			float4 p = *reinterpret_cast<float4*>(t.param + i);
			const float4 g = *reinterpret_cast<const float4*>(t.grad + i);
			float4 m = *reinterpret_cast<float4*>(t.exp_avg + i);
			float4 v = *reinterpret_cast<float4*>(t.exp_avg_sq + i);
			adam_one(p.x, g.x, m.x, v.x, t, a);
			adam_one(p.y, g.y, m.y, v.y, t, a);
			adam_one(p.z, g.z, m.z, v.z, t, a);
			adam_one(p.w, g.w, m.w, v.w, t, a);
			*reinterpret_cast<float4*>(t.param + i) = p;
			*reinterpret_cast<float4*>(t.exp_avg + i) = m;
			*reinterpret_cast<float4*>(t.exp_avg_sq + i) = v;
		} else {
			for (size_t j = i; j < t.n && j < i + 4; j++) {
				float p = t.param[j], m = t.exp_avg[j], v = t.exp_avg_sq[j];
				adam_one(p, t.grad[j], m, v, t, a);
				t.param[j] = p;
				t.exp_avg[j] = m;
				t.exp_avg_sq[j] = v;
			}
		}
	}
}

// Both activation kernels are flat passes over four arrays; a workgroup works on one of them
// (its part is the same for all its threads), 1024 sixteen-byte units per workgroup, so every
// store is a full 16 bytes to consecutive addresses.  The SH rows are the one place where that
// takes care: a row of the joined tensor is 3 floats of one source followed by 3 * rest of the
// other, so the 16-byte units of the output (or of its gradient) straddle the two sources and
// are put together from 4-byte accesses on the source side.
constexpr int kActUnits = 1024;   // 16-byte units per workgroup: 4 per thread

struct ActParts {
	uint32_t sh_blocks, rot_blocks, scale_blocks, opacity_blocks;
};

__host__ __device__ inline ActParts act_parts(int n, int rest)
{
	const size_t sh_floats = 3 * (size_t)(1 + rest);
	auto blocks = [](size_t units) { return (uint32_t)((units + kActUnits - 1) / kActUnits); };
	ActParts p;
	p.sh_blocks = blocks(((size_t)n * sh_floats + 3) / 4);
	p.rot_blocks = blocks((size_t)n);
	p.scale_blocks = blocks(((size_t)n * 3 + 3) / 4);
	p.opacity_blocks = blocks(((size_t)n + 3) / 4);
	return p;
}

// floats [4u, 4u+4) of a flat array of `total` floats, element by element where the array ends
template <typename F>
__device__ __forceinline__ void flat_unit(size_t u, size_t total, const float* __restrict__ in, float* __restrict__ out, F f)
{
	if (4 * u + 4 <= total) {
		const float4 v = reinterpret_cast<const float4*>(in)[u];
		reinterpret_cast<float4*>(out)[u] = float4{f(v.x, 4 * u), f(v.y, 4 * u + 1), f(v.z, 4 * u + 2), f(v.w, 4 * u + 3)};
	} else {
		for (size_t k = 4 * u; k < total; k++)
			out[k] = f(in[k], k);
	}
}

__global__ __launch_bounds__(256) void activate_forward_kernel(ActivateArgs a, ActParts parts)
{
	uint32_t block = blockIdx.x;
	const size_t n = (size_t)a.n;
	if (block < parts.sh_blocks) {
		const size_t sh_floats = 3 * (size_t)(1 + a.rest), rest_floats = 3 * (size_t)a.rest, total = n * sh_floats;
		for (int it = 0; it < kActUnits / 256; it++) {
			const size_t u = (size_t)block * kActUnits + it * 256 + threadIdx.x;
			if (4 * u >= total)
				break;
			float v[4];
#pragma unroll
			for (int k = 0; k < 4; k++) {
				const size_t at = 4 * u + k;
				if (at < total) {
					const size_t row = at / sh_floats, col = at - row * sh_floats;
					v[k] = col < 3 ? a.features_dc[3 * row + col] : a.features_rest[rest_floats * row + (col - 3)];
				} else {
					v[k] = 0.f;
				}
			}
			if (4 * u + 4 <= total)
				reinterpret_cast<float4*>(a.shs)[u] = float4{v[0], v[1], v[2], v[3]};
			else
				for (size_t k = 4 * u; k < total; k++)
					a.shs[k] = v[k - 4 * u];
		}
		return;
	}
	block -= parts.sh_blocks;
	if (block < parts.rot_blocks) {
		for (int it = 0; it < kActUnits / 256; it++) {
			const size_t i = (size_t)block * kActUnits + it * 256 + threadIdx.x;
			if (i >= n)
				break;
			const float4 q = reinterpret_cast<const float4*>(a.rotation)[i];
			const float len = fmaxf(sqrtf(q.x * q.x + q.y * q.y + q.z * q.z + q.w * q.w), 1e-12f);  // torch.nn.functional.normalize
			reinterpret_cast<float4*>(a.rotations)[i] = float4{q.x / len, q.y / len, q.z / len, q.w / len};
		}
		return;
	}
	block -= parts.rot_blocks;
	if (block < parts.scale_blocks) {
		for (int it = 0; it < kActUnits / 256; it++)
			flat_unit((size_t)block * kActUnits + it * 256 + threadIdx.x, 3 * n, a.scaling, a.scales,
			          [](float v, size_t) { return expf(v); });
		return;
	}
	block -= parts.scale_blocks;
	for (int it = 0; it < kActUnits / 256; it++)
		flat_unit((size_t)block * kActUnits + it * 256 + threadIdx.x, n, a.opacity, a.opacities,
		          [](float v, size_t) { return 1.0f / (1.0f + expf(-v)); });
}

__global__ __launch_bounds__(256) void activate_backward_kernel(ActivateBackwardArgs a, ActParts parts)
{
	uint32_t block = blockIdx.x;
	const size_t n = (size_t)a.n;
	if (block < parts.sh_blocks) {
		if (!a.g_shs)
			return;
		const size_t sh_floats = 3 * (size_t)(1 + a.rest), rest_floats = 3 * (size_t)a.rest, total = n * sh_floats;
		for (int it = 0; it < kActUnits / 256; it++) {
			const size_t u = (size_t)block * kActUnits + it * 256 + threadIdx.x;
			if (4 * u >= total)
				break;
			float v[4] = {0.f, 0.f, 0.f, 0.f};
			if (4 * u + 4 <= total) {
				const float4 g = reinterpret_cast<const float4*>(a.g_shs)[u];
				v[0] = g.x; v[1] = g.y; v[2] = g.z; v[3] = g.w;
			} else {
				for (size_t k = 4 * u; k < total; k++)
					v[k - 4 * u] = a.g_shs[k];
			}
#pragma unroll
			for (int k = 0; k < 4; k++) {
				const size_t at = 4 * u + k;
				if (at < total) {
					const size_t row = at / sh_floats, col = at - row * sh_floats;
					if (col < 3)
						a.d_features_dc[3 * row + col] = v[k];
					else
						a.d_features_rest[rest_floats * row + (col - 3)] = v[k];
				}
			}
		}
		return;
	}
	block -= parts.sh_blocks;
	if (block < parts.rot_blocks) {
		if (!a.g_rotations)
			return;
		for (int it = 0; it < kActUnits / 256; it++) {
			const size_t i = (size_t)block * kActUnits + it * 256 + threadIdx.x;
			if (i >= n)
				break;
			// d/dq of q / |q|: (g - u (u . g)) / |q| with u = q / |q|
			const float4 q = reinterpret_cast<const float4*>(a.rotation)[i];
			const float4 g = reinterpret_cast<const float4*>(a.g_rotations)[i];
			const float len = fmaxf(sqrtf(q.x * q.x + q.y * q.y + q.z * q.z + q.w * q.w), 1e-12f);
			const float u0 = q.x / len, u1 = q.y / len, u2 = q.z / len, u3 = q.w / len;
			const float along = u0 * g.x + u1 * g.y + u2 * g.z + u3 * g.w;
			reinterpret_cast<float4*>(a.d_rotation)[i] =
			    float4{(g.x - u0 * along) / len, (g.y - u1 * along) / len, (g.z - u2 * along) / len, (g.w - u3 * along) / len};
		}
		return;
	}
	block -= parts.rot_blocks;
	if (block < parts.scale_blocks) {
		if (!a.g_scales)
			return;
		const float* scales = a.scales;
		for (int it = 0; it < kActUnits / 256; it++)
			flat_unit((size_t)block * kActUnits + it * 256 + threadIdx.x, 3 * n, a.g_scales, a.d_scaling,
			          [scales](float g, size_t k) { return g * scales[k]; });
		return;
	}
	block -= parts.scale_blocks;
	if (!a.g_opacities)
		return;
	const float* opacities = a.opacities;
	for (int it = 0; it < kActUnits / 256; it++)
		flat_unit((size_t)block * kActUnits + it * 256 + threadIdx.x, n, a.g_opacities, a.d_opacity, [opacities](float g, size_t k) {
			const float o = opacities[k];
			return g * (o * (1.0f - o));
		});
}

}  // namespace

void launch_activate_forward(const ActivateArgs& a, hipStream_t s)
{
	stage_mark("activate_forward", s);
	if (a.n <= 0)
		return;
	const ActParts p = act_parts(a.n, a.rest);
	hipLaunchKernelGGL(activate_forward_kernel, dim3(p.sh_blocks + p.rot_blocks + p.scale_blocks + p.opacity_blocks), dim3(256),
	                   0, s, a, p);
}

void launch_activate_backward(const ActivateBackwardArgs& a, hipStream_t s)
{
	stage_mark("activate_backward", s);
	if (a.n <= 0)
		return;
	const ActParts p = act_parts(a.n, a.rest);
	hipLaunchKernelGGL(activate_backward_kernel, dim3(p.sh_blocks + p.rot_blocks + p.scale_blocks + p.opacity_blocks), dim3(256),
	                   0, s, a, p);
}

uint32_t loss_blocks(int C, int H, int W)
{
	return (uint32_t)(((W + kLossTileW - 1) / kLossTileW) * ((H + kLossTileH - 1) / kLossTileH) * C);
}

void launch_l1_ssim_forward(const LossArgs& a, hipStream_t s)
{
	stage_mark("l1_ssim_forward", s);
	const uint32_t grid = 8 * ((loss_blocks(a.C, a.H, a.W) + 7) / 8);
	hipLaunchKernelGGL(ssim_forward_kernel, dim3(grid), dim3(256), 0, s, a);
	hipLaunchKernelGGL(loss_finish_kernel, dim3(1), dim3(256), 0, s, a, loss_blocks(a.C, a.H, a.W));
}

void launch_l1_ssim_backward(const LossArgs& a, hipStream_t s)
{
	stage_mark("l1_ssim_backward", s);
	const uint32_t grid = 8 * ((loss_blocks(a.C, a.H, a.W) + 7) / 8);
	hipLaunchKernelGGL(ssim_backward_kernel, dim3(grid), dim3(256), 0, s, a);
}

uint32_t adam_blocks_for(size_t n)
{
	return (uint32_t)((n + kAdamBlock - 1) / kAdamBlock);
}

void launch_adam_step(const AdamArgs& a, uint32_t blocks, hipStream_t s)
{
	stage_mark("adam_step", s);
	if (blocks)
		hipLaunchKernelGGL(adam_step_kernel, dim3(blocks), dim3(256), 0, s, a);
}

}  // namespace rgs
