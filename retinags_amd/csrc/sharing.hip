// Boundary straddlers: which Gaussians of a submodel are lent to which neighbours, and the
// merge of the lent rows behind a submodel's own rows (forward: gather; backward: the
// gradients of lent rows go back to the rows they were read from).
//
// Selection (parallel_utils/basic_parallel_trainer/result_aggregator.py:76-106).  A Gaussian
// reaches 3 x its largest activated scale (never less than 0) along every axis.  It is a
// candidate when that cube touches or crosses a face of its own submodel's box, and it is lent
// to a destination whose box the cube meets on all three axes.  Row lists come out in ascending
// row order (what boolean-mask indexing gives), so three short kernels: per-block counts per
// destination, one scan per destination over the blocks, then the ordered emission.  Every
// comparison is a single float32 operation on float32 sums, so the lists are exact.
//
// Merge (result_aggregator.py:263-288).  A row is 59 floats in five arrays of widths 3, 1, 3, 4
// and 3M.  Sixteen lanes take one row: twelve move the SH coefficients 16 bytes at a time, one
// the quaternion, and the last three the narrow arrays; a wavefront moves four rows.  Nothing
// here is reused, so there is no LDS staging; the kernel is bound by HBM bandwidth and by the
// 12-byte rows that cannot be moved as one aligned access.
#include "rgs_device.h"
#include "rgs_kernels.h"

namespace rgs {

namespace {

constexpr int kSelectThreads = 256;
constexpr int kSelectItems = 4;
constexpr int kSelectBlock = kSelectThreads * kSelectItems;   // Gaussians per workgroup
constexpr int kSelectWaves = kSelectThreads / kWave;
constexpr int kSelectCells = kSelectItems * kSelectWaves;     // (item, wave) cells of a workgroup, in row order

__device__ __forceinline__ uint64_t lend_mask(const StraddlerSelectArgs& a, uint32_t i)
{
	const float* m = a.means3D + 3 * (size_t)i;
	const float* s = a.scales + 3 * (size_t)i;
	const float mx = m[0], my = m[1], mz = m[2];
	const float largest = fmaxf(fmaxf(s[0], s[1]), s[2]);
	const float reach = fmaxf(largest * 3.0f, 0.0f);
	const float hx = mx + reach, hy = my + reach, hz = mz + reach;
	const float lx = mx - reach, ly = my - reach, lz = mz - reach;
	const bool candidate = hx >= a.src_up[0] || hy >= a.src_up[1] || hz >= a.src_up[2] ||
	                       lx <= a.src_low[0] || ly <= a.src_low[1] || lz <= a.src_low[2];
	if (!candidate)
		return 0;
	uint64_t mask = 0;
	for (int d = 0; d < a.boxes.count; d++) {
		if (d == a.skip)
			continue;
		const bool meets = hx >= a.boxes.low[d][0] && hy >= a.boxes.low[d][1] && hz >= a.boxes.low[d][2] &&
		                   lx <= a.boxes.up[d][0] && ly <= a.boxes.up[d][1] && lz <= a.boxes.up[d][2];
		mask |= (uint64_t)meets << d;
	}
	return mask;
}

__global__ __launch_bounds__(kSelectThreads) void straddler_count_kernel(StraddlerSelectArgs a, uint32_t blocks)
{
	__shared__ uint32_t total[kMaxShareBoxes];
	const int tid = threadIdx.x;
	if (tid < kMaxShareBoxes)
		total[tid] = 0;
	__syncthreads();
	const uint32_t base = blockIdx.x * kSelectBlock;
#pragma unroll
	for (int j = 0; j < kSelectItems; j++) {
		const uint32_t i = base + j * kSelectThreads + tid;
		const uint64_t m = i < (uint32_t)a.n ? lend_mask(a, i) : 0;
		if (__ballot(m != 0) == 0)
			continue;
		for (int d = 0; d < a.boxes.count; d++) {
			const uint64_t lent = __ballot((m >> d) & 1);
			if (lent && (tid & (kWave - 1)) == 0)
				atomicAdd(&total[d], (uint32_t)__popcll(lent));
		}
	}
	__syncthreads();
	if (tid < a.boxes.count)
		a.block_counts[(size_t)tid * blocks + blockIdx.x] = total[tid];
}

// One workgroup per destination: exclusive scan of that destination's per-block counts, in place.
__global__ __launch_bounds__(256) void straddler_scan_kernel(uint32_t* block_counts, uint32_t blocks, uint32_t* counts)
{
	__shared__ uint32_t lds[8];
	uint32_t* row = block_counts + (size_t)blockIdx.x * blocks;
	uint32_t carry = 0;
	for (uint32_t at = 0; at < blocks; at += 256) {
		const uint32_t i = at + threadIdx.x;
		const uint32_t v = i < blocks ? row[i] : 0;
		uint32_t sum;
		const uint32_t before = block256_exclusive_scan_u32(v, lds, sum);
		if (i < blocks)
			row[i] = carry + before;
		carry += sum;
		__syncthreads();
	}
	if (threadIdx.x == 0)
		counts[blockIdx.x] = carry;
}

__global__ __launch_bounds__(kSelectThreads) void straddler_emit_kernel(StraddlerSelectArgs a, uint32_t blocks)
{
	__shared__ uint32_t cell[kSelectCells][kMaxShareBoxes];
	const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
	for (int c = tid; c < kSelectCells * kMaxShareBoxes; c += kSelectThreads)
		(&cell[0][0])[c] = 0;
	__syncthreads();
	const uint32_t base = blockIdx.x * kSelectBlock;
	uint64_t masks[kSelectItems];
#pragma unroll
	for (int j = 0; j < kSelectItems; j++) {
		const uint32_t i = base + j * kSelectThreads + tid;
		masks[j] = i < (uint32_t)a.n ? lend_mask(a, i) : 0;
		if (__ballot(masks[j] != 0) == 0)
			continue;
		for (int d = 0; d < a.boxes.count; d++) {
			const uint64_t lent = __ballot((masks[j] >> d) & 1);
			if (lent && lane == 0)
				cell[j * kSelectWaves + wave][d] = (uint32_t)__popcll(lent);
		}
	}
	__syncthreads();
#pragma unroll
	for (int j = 0; j < kSelectItems; j++) {
		if (__ballot(masks[j] != 0) == 0)
			continue;
		const uint32_t i = base + j * kSelectThreads + tid;
		const int mine = j * kSelectWaves + wave;
		for (int d = 0; d < a.boxes.count; d++) {
			const bool bit = (masks[j] >> d) & 1;
			const uint64_t lent = __ballot(bit);
			if (!lent)
				continue;
			uint32_t at = a.block_counts[(size_t)d * blocks + blockIdx.x];
			for (int c = 0; c < mine; c++)
				at += cell[c][d];
			at += (uint32_t)__popcll(lent & ((1ull << lane) - 1));
			if (bit && at < a.capacity)
				a.rows[(size_t)d * a.capacity + at] = i;
		}
	}
}

// ---- merge ----------------------------------------------------------------------------------

constexpr int kRowLanes = 16;
constexpr int kRowsPerBlock = 256 / kRowLanes;

template <bool kVector>
__device__ __forceinline__ void copy_wide(const float* __restrict__ from, float* __restrict__ to, int floats, int part, int parts)
{
	if (kVector) {
		for (int c = part; c * 4 < floats; c += parts)
			reinterpret_cast<float4*>(to)[c] = reinterpret_cast<const float4*>(from)[c];
	} else {
		for (int c = part; c < floats; c += parts)
			to[c] = from[c];
	}
}

template <bool kVector>
__global__ __launch_bounds__(256) void merge_rows_kernel(MergeArgs a)
{
	// segments start at workgroup boundaries, so the segment of a workgroup is a scalar
	int s = 0;
	while (s + 1 < a.segments && blockIdx.x >= a.seg[s + 1].block0)
		s++;
	const MergeSegment& seg = a.seg[s];
	const uint32_t j = (blockIdx.x - seg.block0) * kRowsPerBlock + threadIdx.x / kRowLanes;
	if (j >= seg.count)
		return;
	const size_t from = seg.rows ? seg.rows[j] : j;
	const size_t to = (size_t)seg.dst_row0 + j;
	const int part = threadIdx.x % kRowLanes;
	if (part < 12) {
		copy_wide<kVector>(seg.shs + from * a.sh_floats, a.shs + to * a.sh_floats, a.sh_floats, part, 12);
	} else if (part == 12) {
		copy_wide<kVector>(seg.rotations + from * 4, a.rotations + to * 4, 4, 0, 1);
	} else if (part == 13) {
		for (int c = 0; c < 3; c++)
			a.means3D[to * 3 + c] = seg.means3D[from * 3 + c];
	} else if (part == 14) {
		for (int c = 0; c < 3; c++)
			a.scales[to * 3 + c] = seg.scales[from * 3 + c];
	} else {
		a.opacity[to] = seg.opacity[from];
	}
}

template <bool kVector>
__device__ __forceinline__ void add_wide(const float* __restrict__ g, float* __restrict__ into, int floats, int part, int parts)
{
	if (kVector) {
		for (int c = part; c * 4 < floats; c += parts) {
			const float4 v = reinterpret_cast<const float4*>(g)[c];
			float4 t = reinterpret_cast<float4*>(into)[c];
			t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
			reinterpret_cast<float4*>(into)[c] = t;
		}
	} else {
		for (int c = part; c < floats; c += parts)
			into[c] += g[c];
	}
}

// Rows of one launch are distinct within a segment and segments of one launch belong to
// different sources, so the read-modify-write needs no atomics; launches for different
// destinations are ordered by the stream.
template <bool kVector>
__global__ __launch_bounds__(256) void merge_rows_backward_kernel(MergeBackwardArgs a)
{
	int s = 0;
	while (s + 1 < a.segments && blockIdx.x >= a.seg[s + 1].block0)
		s++;
	const MergeBackwardSegment& seg = a.seg[s];
	const uint32_t j = (blockIdx.x - seg.block0) * kRowsPerBlock + threadIdx.x / kRowLanes;
	if (j >= seg.count)
		return;
	const size_t into = seg.rows[j];
	const size_t g = (size_t)seg.dst_row0 + j;
	const int part = threadIdx.x % kRowLanes;
	if (part < 12) {
		if (a.shs && seg.shs)
			add_wide<kVector>(a.shs + g * a.sh_floats, seg.shs + into * a.sh_floats, a.sh_floats, part, 12);
	} else if (part == 12) {
		if (a.rotations && seg.rotations)
			add_wide<kVector>(a.rotations + g * 4, seg.rotations + into * 4, 4, 0, 1);
	} else if (part == 13) {
		if (a.means3D && seg.means3D)
			for (int c = 0; c < 3; c++)
				seg.means3D[into * 3 + c] += a.means3D[g * 3 + c];
	} else if (part == 14) {
		if (a.scales && seg.scales)
			for (int c = 0; c < 3; c++)
				seg.scales[into * 3 + c] += a.scales[g * 3 + c];
		if (a.opacity && seg.opacity)
			seg.opacity[into] += a.opacity[g];
	} else {
		if (a.means2D && seg.means2D)
			for (int c = 0; c < 3; c++)
				seg.means2D[into * 3 + c] += a.means2D[g * 3 + c];
	}
}

}  // namespace

uint32_t straddler_select_blocks(int n)
{
	return (uint32_t)((n + kSelectBlock - 1) / kSelectBlock);
}

void launch_straddler_select(const StraddlerSelectArgs& a, hipStream_t s)
{
	const uint32_t blocks = straddler_select_blocks(a.n);
	stage_mark("straddler_select", s);
	if (blocks) {
		hipLaunchKernelGGL(straddler_count_kernel, dim3(blocks), dim3(kSelectThreads), 0, s, a, blocks);
		hipLaunchKernelGGL(straddler_scan_kernel, dim3(a.boxes.count), dim3(256), 0, s, a.block_counts, blocks, a.counts);
		hipLaunchKernelGGL(straddler_emit_kernel, dim3(blocks), dim3(kSelectThreads), 0, s, a, blocks);
	} else {
		launch_fill_u32(a.counts, 0, a.boxes.count, s);
	}
}

uint32_t merge_blocks_for(uint32_t rows)
{
	return (rows + kRowsPerBlock - 1) / kRowsPerBlock;
}

void launch_merge_rows(const MergeArgs& a, uint32_t blocks, bool by_16_bytes, hipStream_t s)
{
	stage_mark("merge_rows", s);
	if (!blocks)
		return;
	if (by_16_bytes)
		hipLaunchKernelGGL(merge_rows_kernel<true>, dim3(blocks), dim3(256), 0, s, a);
	else
		hipLaunchKernelGGL(merge_rows_kernel<false>, dim3(blocks), dim3(256), 0, s, a);
}

void launch_merge_rows_backward(const MergeBackwardArgs& a, uint32_t blocks, bool by_16_bytes, hipStream_t s)
{
	stage_mark("merge_rows_backward", s);
	if (!blocks)
		return;
	if (by_16_bytes)
		hipLaunchKernelGGL(merge_rows_backward_kernel<true>, dim3(blocks), dim3(256), 0, s, a);
	else
		hipLaunchKernelGGL(merge_rows_backward_kernel<false>, dim3(blocks), dim3(256), 0, s, a);
}

}  // namespace rgs
