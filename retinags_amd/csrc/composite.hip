// Front-to-back compositing of K partial images (RGB, depth, accumulated alpha), forward
// and backward, one pixel per thread, one pass over every input plane.
// Restates parallel_utils/basic_parallel_trainer/result_aggregator.py:244-259:
//   T_0 = 1, T_k = prod_{j<k} (1 - alpha_j)
//   image = sum_k T_k image_k + bg T_K,  depth = sum_k T_k depth_k,  alpha = 1 - T_K
// The inputs arrive already in compositing order.
#include "rgs_kernels.h"

namespace rgs {

__global__ __launch_bounds__(256) void composite_forward_kernel(CompositeArgs a)
{
	const size_t n = (size_t)a.H * a.W;
	const size_t p = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (p >= n)
		return;
	float T = 1.f, r = 0.f, g = 0.f, b = 0.f, d = 0.f;
	for (int k = 0; k < a.K; k++) {
		const float* img = a.images[k];
		r += T * img[p];
		g += T * img[n + p];
		b += T * img[2 * n + p];
		d += T * a.depths[k][p];
		T = T * (1.f - a.alphas[k][p]);
	}
	float bg0 = 0.f, bg1 = 0.f, bg2 = 0.f;
	if (a.bg) {
		bg0 = a.bg[0];
		bg1 = a.bg[1];
		bg2 = a.bg[2];
	}
	a.out_image[p] = r + bg0 * T;
	a.out_image[n + p] = g + bg1 * T;
	a.out_image[2 * n + p] = b + bg2 * T;
	a.out_depth[p] = d;
	a.out_alpha[p] = 1.f - T;
}

// dL/dimage_k = T_k g, dL/ddepth_k = T_k g_d, dL/dalpha_k = -T_k R_k with
// R_{K-1} = <bg, g> - g_a and R_{k-1} = <image_k, g> + depth_k g_d + (1 - alpha_k) R_k.
// No division, so alpha_k = 1 is handled exactly.  T_k and alpha_k are kept per thread for the
// back-to-front sweep: in registers when the number of layers is at most kLayers (the loops are unrolled over kLayers
// and guarded by K, so the arrays are indexed by constants), otherwise (kLayers = 0) in an array indexed at run time,
// which the compiler places in scratch memory: every value then goes out to memory and comes back.
template <int kLayers>
__global__ __launch_bounds__(256) void composite_backward_kernel(CompositeArgs a)
{
	const size_t n = (size_t)a.H * a.W;
	const size_t p = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (p >= n)
		return;
	constexpr int kHeld = kLayers > 0 ? kLayers : kMaxComposite;
	float Tk[kHeld], alpha[kHeld];
	float T = 1.f;
	if (kLayers > 0) {
#pragma unroll
		for (int k = 0; k < kLayers; k++)
			if (k < a.K) {
				alpha[k] = a.alphas[k][p];
				Tk[k] = T;
				T = T * (1.f - alpha[k]);
			}
	} else {
		for (int k = 0; k < a.K; k++) {
			alpha[k] = a.alphas[k][p];
			Tk[k] = T;
			T = T * (1.f - alpha[k]);
		}
	}
	const float gr = a.g_image[p], gg = a.g_image[n + p], gb = a.g_image[2 * n + p];
	const float gd = a.g_depth ? a.g_depth[p] : 0.f;
	const float ga = a.g_alpha ? a.g_alpha[p] : 0.f;
	float R = -ga;
	if (a.bg)
		R += a.bg[0] * gr + a.bg[1] * gg + a.bg[2] * gb;
	auto layer = [&](int k, float t, float alpha_k) {
		float* di = a.d_images[k];
		di[p] = t * gr;
		di[n + p] = t * gg;
		di[2 * n + p] = t * gb;
		a.d_depths[k][p] = t * gd;
		a.d_alphas[k][p] = -(t * R);
		const float* img = a.images[k];
		R = img[p] * gr + img[n + p] * gg + img[2 * n + p] * gb + a.depths[k][p] * gd + (1.f - alpha_k) * R;
	};
	if (kLayers > 0) {
#pragma unroll
		for (int k = kLayers - 1; k >= 0; k--)
			if (k < a.K)
				layer(k, Tk[k], alpha[k]);
	} else {
		for (int k = a.K - 1; k >= 0; k--)
			layer(k, Tk[k], alpha[k]);
	}
}

void launch_composite_forward(const CompositeArgs& a, hipStream_t s)
{
	const size_t n = (size_t)a.H * a.W;
	stage_mark("composite_forward", s);
	hipLaunchKernelGGL(composite_forward_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a);
}

void launch_composite_backward(const CompositeArgs& a, hipStream_t s)
{
	const size_t n = (size_t)a.H * a.W;
	stage_mark("composite_backward", s);
	const dim3 grid((unsigned)((n + 255) / 256));
	if (a.K <= 4)
		hipLaunchKernelGGL(composite_backward_kernel<4>, grid, dim3(256), 0, s, a);
	else if (a.K <= 16)
		hipLaunchKernelGGL(composite_backward_kernel<16>, grid, dim3(256), 0, s, a);
	else
		hipLaunchKernelGGL(composite_backward_kernel<0>, grid, dim3(256), 0, s, a);
}

}  // namespace rgs
