// Binning stages: offset scans, depth order of the Gaussians, tile-key duplication, stable
// radix sorts and per-tile range extraction.  All integer work; results are bit-exact by
// construction.  K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian.
//
// The reference sorts R (Gaussian, tile) instances by the 64-bit key (tile << 32) | depth bits
// with a stable sort (K/cuda_rasterizer_hgs/rasterizer_impl.cu:300-317): 6 passes over 12-byte
// pairs at 6 500 tiles.  The same permutation is produced here in two cheaper steps:
//   1. the P Gaussians are sorted by their depth bits (stable, so equal depths stay in index
//      order), 4 passes over P 8-byte pairs;
//   2. instances are emitted in that order with the tile as a 32-bit key and sorted by it
//      (stable, so every tile keeps depth order, ties in index order), ceil(log2(tiles)/8)
//      passes over R 8-byte pairs.
// A stable sort by (tile, depth) of instances emitted in index order and a stable sort by tile
// of instances emitted in (depth, index) order give the same list: within a tile both order by
// depth and break ties by Gaussian index (a Gaussian touches a tile at most once).
#include "rgs_kernels.h"

#include <atomic>

namespace rgs {

// ---- prefix sums ---------------------------------------------------------------------------
// Replaces cub::DeviceScan::InclusiveSum at K/cuda_rasterizer_hgs/rasterizer_impl.cu:283
// with three small kernels: per-256 block totals, one single-block scan of those totals,
// and a per-block scan that adds the block's base.  On the rasterizer path the block totals
// come from the kernel that produces the values (the forward preprocess, the gather of the
// depth order), so only the last two run there.

// In all three kernels a non-null n_device overrides n (the launch is then sized for an upper bound).
__global__ __launch_bounds__(256) void block_totals_kernel(const uint32_t* __restrict__ in, size_t n,
                                                            const uint32_t* __restrict__ n_device,
                                                            uint32_t* __restrict__ totals)
{
	__shared__ uint32_t lds[8];
	if (n_device)
		n = *n_device;
	const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
	const uint32_t v = i < n ? in[i] : 0u;
	uint32_t total;
	(void)block256_exclusive_scan_u32(v, lds, total);
	if (threadIdx.x == 0)
		totals[blockIdx.x] = total;
}

// In-place exclusive scan of `data[0..n)` by one block of 1024 threads; the grand total goes
// to *total_out (if non-null).
// Block 1, if launched, does the same for a second array of the same length.
__global__ __launch_bounds__(1024) void single_block_exclusive_scan_kernel(uint32_t* __restrict__ data, size_t n,
                                                                            const uint32_t* __restrict__ n_device,
                                                                            uint32_t* __restrict__ total_out,
                                                                            uint32_t* __restrict__ data_b,
                                                                            uint32_t* __restrict__ total_out_b)
{
	__shared__ uint32_t wave_tot[16];
	if (blockIdx.x == 1) {
		data = data_b;
		total_out = total_out_b;
	}
	if (n_device)
		n = ((size_t)*n_device + 255) / 256;  // one entry per 256 elements
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const size_t chunk = (n + 1023) / 1024;
	const size_t lo = (size_t)tid * chunk;
	const size_t hi = lo + chunk < n ? lo + chunk : n;
	uint32_t sum = 0;
	for (size_t i = lo; i < hi; i++)
		sum += data[i];
	const uint32_t inc = wave_inclusive_scan_u32(sum);
	if (lane == 63)
		wave_tot[wave] = inc;
	__syncthreads();
	uint32_t base = 0, total = 0;
#pragma unroll
	for (int w = 0; w < 16; w++) {
		const uint32_t s = wave_tot[w];
		if (w < wave)
			base += s;
		total += s;
	}
	uint32_t run = base + inc - sum;
	for (size_t i = lo; i < hi; i++) {
		const uint32_t v = data[i];
		data[i] = run;
		run += v;
	}
	if (tid == 0 && total_out)
		*total_out = total;
}

__global__ __launch_bounds__(256) void block_inclusive_scan_kernel(const uint32_t* __restrict__ in,
                                                                    const uint32_t* __restrict__ block_base, size_t n,
                                                                    const uint32_t* __restrict__ n_device,
                                                                    uint32_t* __restrict__ out)
{
	__shared__ uint32_t lds[8];
	if (n_device)
		n = *n_device;
	const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
	const uint32_t v = i < n ? in[i] : 0u;
	uint32_t total;
	const uint32_t ex = block256_exclusive_scan_u32(v, lds, total);
	if (i < n)
		out[i] = block_base[blockIdx.x] + ex + v;
}

size_t scan_temp_words(size_t n)
{
	return (n + 255) / 256 + 1;
}

static void inclusive_sum(const uint32_t* in, uint32_t* out, size_t n, const uint32_t* n_device, uint32_t* temp,
                          hipStream_t s)
{
	const size_t nb = (n + 255) / 256;
	hipLaunchKernelGGL(block_totals_kernel, dim3((unsigned)nb), dim3(256), 0, s, in, n, n_device, temp);
	hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(1), dim3(1024), 0, s, temp, nb, n_device,
	                   (uint32_t*)nullptr, (uint32_t*)nullptr, (uint32_t*)nullptr);
	hipLaunchKernelGGL(block_inclusive_scan_kernel, dim3((unsigned)nb), dim3(256), 0, s, in, temp, n, n_device, out);
}

void launch_inclusive_sum(const uint32_t* in, uint32_t* out, size_t n, uint32_t* temp, const char* stage,
                          hipStream_t s)
{
	if (n == 0)
		return;
	if (stage)
		stage_mark(stage, s);
	inclusive_sum(in, out, n, nullptr, temp, s);
}

void launch_totals_from_block_sums(uint32_t* block_sums, uint32_t* block_visible, int P, uint32_t* total_out,
                                   uint32_t* visible_count, hipStream_t s)
{
	const size_t nb = ((size_t)P + 255) / 256;
	stage_mark("offset_scan", s);
	hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(2), dim3(1024), 0, s, block_sums, nb,
	                   (const uint32_t*)nullptr, total_out, block_visible, visible_count);
}

// ---- depth order and key duplication (K/cuda_rasterizer_hgs/rasterizer_impl.cu:70-111) -------

// (depth bits, index) pairs of the Gaussians that touch a tile, compacted in index order:
// block b of 256 Gaussians writes from visible_base[b] on.  Depths of rendered Gaussians are
// positive floats (> 0.2), whose bit patterns order like the values.
__global__ __launch_bounds__(256) void depth_pairs_kernel(int P, const float* __restrict__ depths,
                                                           const uint32_t* __restrict__ tiles_touched,
                                                           const uint32_t* __restrict__ visible_base,
                                                           uint32_t* __restrict__ keys, uint32_t* __restrict__ values,
                                                           uint32_t* __restrict__ visible_list)
{
	__shared__ uint32_t lds[8];
	const int idx = blockIdx.x * 256 + threadIdx.x;
	const bool visible = idx < P && tiles_touched[idx] != 0u;
	uint32_t total;
	const uint32_t rank = block256_exclusive_scan_u32(visible ? 1u : 0u, lds, total);
	if (visible) {
		const uint32_t at = visible_base[blockIdx.x] + rank;
		keys[at] = __float_as_uint(depths[idx]);
		values[at] = (uint32_t)idx;
		visible_list[at] = (uint32_t)idx;  // the sort reorders `values`; this copy stays in index order
	}
}

// out[k] = in[index[k]] for k below the count on the device, and the sum of every 256 of them
// (the first level of the scan that follows).  `in` has in_size entries; an index beyond it (only
// possible in what a sort that gave up left behind) reads the last entry instead.
__global__ __launch_bounds__(256) void gather_u32_kernel(const uint32_t* __restrict__ n_device,
                                                          const uint32_t* __restrict__ index,
                                                          const uint32_t* __restrict__ in, uint32_t in_size,
                                                          uint32_t* __restrict__ out,
                                                          uint32_t* __restrict__ block_totals)
{
	__shared__ uint32_t lds[8];
	const uint32_t k = blockIdx.x * 256 + threadIdx.x;
	uint32_t v = 0;
	if (k < *n_device) {
		v = in[min(index[k], in_size - 1u)];
		out[k] = v;
	}
	uint32_t total;
	(void)block256_exclusive_scan_u32(v, lds, total);
	if (threadIdx.x == 0)
		block_totals[blockIdx.x] = total;
}

// Instances of the Gaussians in depth order, tiles row by row like the reference, at the offsets
// of the scan taken in that same order.  A wavefront takes 64 Gaussians; their instances form one
// contiguous run of the output, which the wavefront writes 64 consecutive entries at a time:
// each lane finds the Gaussian its output position belongs to by a binary search over the 64
// inclusive offsets, then the tile from the position inside that Gaussian's rectangle.  (With
// one thread per Gaussian every store touched 64 different cache lines, and a Gaussian that
// covers hundreds of tiles kept its wavefront busy alone.)
// `order` is the output of a sort: should that sort ever have given up, its entries may be anything, so
// they are clamped to the P Gaussians there are (the tile ranges then stay empty and nothing reads the result).
__global__ __launch_bounds__(256) void duplicate_with_keys_kernel(uint32_t P, const uint32_t* __restrict__ visible_count,
                                                                   const uint32_t* __restrict__ order,
                                                                   const uint32_t* __restrict__ offsets,
                                                                   const float2* __restrict__ xy,
                                                                   const int* __restrict__ radii, int gx, int gy,
                                                                   uint32_t* __restrict__ keys,
                                                                   uint32_t* __restrict__ values, uint32_t capacity,
                                                                   uint32_t* __restrict__ clear, size_t clear_words)
{
	__shared__ uint32_t s_end[4][64];     // inclusive offset of each of the wavefront's Gaussians
	__shared__ uint32_t s_origin[4][64];  // first tile of its rectangle
	__shared__ uint32_t s_width[4][64];   // tiles per row of its rectangle
	__shared__ uint32_t s_index[4][64];
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const uint32_t k = blockIdx.x * 256 + threadIdx.x;
	// the scratch of the sort that follows is cleared here, which saves a launch
	for (size_t w = k; w < clear_words; w += (size_t)gridDim.x * 256)
		clear[w] = 0u;
	const uint32_t n = min(*visible_count, P);
	const uint32_t k0 = k - (uint32_t)lane;  // the wavefront's first Gaussian
	if (k0 >= n)
		return;
	const uint32_t run_begin = k0 == 0u ? 0u : offsets[k0 - 1];
	uint32_t end = 0, origin = 0, width = 1, idx = 0;
	if (k < n) {
		idx = min(order[k], P - 1u);
		end = offsets[k];
		const float2 p = xy[idx];
		const TileRect rc = tile_rect(p.x, p.y, radii[idx], gx, gy);
		origin = rc.y0 * (uint32_t)gx + rc.x0;
		width = rc.x1 - rc.x0;
	} else {
		end = offsets[n - 1];  // no instances of its own
	}
	s_end[wave][lane] = end;
	s_origin[wave][lane] = origin;
	s_width[wave][lane] = width;
	s_index[wave][lane] = idx;
	__builtin_amdgcn_wave_barrier();
	const uint32_t run_end = s_end[wave][63];
	for (uint32_t base = run_begin; base < run_end; base += 64) {
		const uint32_t pos = base + (uint32_t)lane;
		if (pos < run_end && pos < capacity) {  // positions beyond the room the caller gave are dropped
			// the first Gaussian whose inclusive offset exceeds pos
			int lo = 0;
#pragma unroll
			for (int step = 32; step > 0; step >>= 1)
				if (s_end[wave][lo + step - 1] <= pos)
					lo += step;
			const uint32_t first = lo == 0 ? run_begin : s_end[wave][lo - 1];
			const uint32_t t = pos - first, w = s_width[wave][lo];
			const uint32_t row = t / w;
			keys[pos] = s_origin[wave][lo] + row * (uint32_t)gx + (t - row * w);
			values[pos] = s_index[wave][lo];
		}
	}
}

void launch_depth_order(int P, const float* depths, const uint32_t* tiles_touched, uint32_t* block_visible,
                        uint32_t* visible_count, uint32_t* visible_list, uint32_t* keys_a, uint32_t* keys_b, uint32_t* order, uint32_t* vals_b,
                        uint32_t* tiles_in_order, uint32_t* offsets_in_order, uint32_t* sort_temp, uint32_t* scan_temp,
                        hipStream_t s)
{
	const unsigned nb = (unsigned)((P + 255) / 256);
	stage_mark("depth_order", s);
	hipLaunchKernelGGL(depth_pairs_kernel, dim3(nb), dim3(256), 0, s, P, depths, tiles_touched, block_visible, keys_a,
	                   order, visible_list);
	// 4 passes: the sorted pairs end up in the first buffer pair again
	launch_sort_pairs_u32(keys_a, keys_b, order, vals_b, (size_t)P, visible_count, 32, sort_temp, true, nullptr, 0, nullptr,
	                      s);
	hipLaunchKernelGGL(gather_u32_kernel, dim3(nb), dim3(256), 0, s, visible_count, order, tiles_touched, (uint32_t)P,
	                   tiles_in_order, scan_temp);
	hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(1), dim3(1024), 0, s, scan_temp, (size_t)nb,
	                   visible_count, (uint32_t*)nullptr, (uint32_t*)nullptr, (uint32_t*)nullptr);
	hipLaunchKernelGGL(block_inclusive_scan_kernel, dim3(nb), dim3(256), 0, s, tiles_in_order, scan_temp, (size_t)P,
	                   visible_count, offsets_in_order);
}

void launch_duplicate_with_keys(int P, const uint32_t* visible_count, const uint32_t* order,
                                const uint32_t* offsets_in_order, const float2* xy, const int* radii, int grid_x,
                                int grid_y, uint32_t* keys, uint32_t* values, uint32_t capacity, uint32_t* clear,
                                size_t clear_words, hipStream_t s)
{
	stage_mark("duplicate_with_keys", s);
	hipLaunchKernelGGL(duplicate_with_keys_kernel, dim3((P + 255) / 256), dim3(256), 0, s, (uint32_t)P, visible_count, order,
	                   offsets_in_order, xy, radii, grid_x, grid_y, keys, values, capacity, clear, clear_words);
}

// ---- radix sort -------------------------------------------------------------------------------
// Replaces cub::DeviceRadixSort::SortPairs at K/cuda_rasterizer_hgs/rasterizer_impl.cu:312-317:
// a stable least-significant-digit sort of (u64 key, u32 value) on key bits [0, end_bit),
// 8 bits per pass, in the one-sweep form: one kernel reads the keys once and builds the digit
// histogram of every pass, then each pass is a single kernel whose blocks take tiles of
// kSortBlock pairs in arrival order, rank them in LDS, obtain their global digit offsets from
// the blocks before them through a chained look-back over per-tile status words, and scatter.
// Element order inside a tile is (wave, round, lane); ranking preserves it, and tiles are
// ordered by their id, so every pass is stable.
//
// Scratch layout (u32 words):
//   [0, 2048)      digit histograms of up to 8 passes (every block of a pass scans its 256 counts itself)
//   [2048, 2056)   tile counter of each pass
//   [2056]         status: non-zero if a look-back ever gave up waiting (never expected)
//   [kSortHeader + pass * 256 * tiles + tile * 256 + digit]  look-back words

constexpr uint32_t kSortCounters = 2048;
constexpr uint32_t kSortStatus = 2056;
constexpr uint32_t kFlagAggregate = 1u << 30;  // word holds this tile's own digit count
constexpr uint32_t kFlagInclusive = 2u << 30;  // word holds the count of this and all earlier tiles
constexpr uint32_t kValueMask = (1u << 30) - 1u;
constexpr int kLookbackSpinLimit = 1 << 18;

// How many times a look-back polls a word that has not been published yet before it gives up.
// A negative value makes every look-back give up at once: the way a test drives the give-up
// path from the host (every kernel still runs to its end).
static std::atomic<int> g_lookback_spin_limit{kLookbackSpinLimit};

void set_lookback_spin_limit(int polls)
{
	g_lookback_spin_limit.store(polls == 0 ? kLookbackSpinLimit : polls);
}

template <typename KeyT>
__device__ __forceinline__ uint32_t digit_of(KeyT key, int shift, uint32_t mask)
{
	return (uint32_t)(key >> shift) & mask;
}

template <typename KeyT>
__global__ __launch_bounds__(256) void sort_digit_histogram_kernel(const KeyT* __restrict__ keys, size_t n,
                                                                    const uint32_t* __restrict__ n_device,
                                                                    int passes, int end_bit,
                                                                    uint32_t* __restrict__ hist,
                                                                    uint32_t* __restrict__ clear, size_t clear_words)
{
	__shared__ uint32_t s_hist[kSortMaxPasses][256];
	for (size_t w = (size_t)blockIdx.x * 256 + threadIdx.x; w < clear_words; w += (size_t)gridDim.x * 256)
		clear[w] = 0u;  // an array that a later kernel of the same stream wants cleared
	if (n_device)
		n = min(n, (size_t)*n_device);
#pragma unroll
	for (int p = 0; p < kSortMaxPasses; p++)
		s_hist[p][threadIdx.x] = 0;
	__syncthreads();
	for (size_t k = (size_t)blockIdx.x * 256 + threadIdx.x; k < n; k += (size_t)gridDim.x * 256) {
		const KeyT key = keys[k];
		for (int p = 0; p < passes; p++) {
			const int shift = 8 * p;
			const int bits = end_bit - shift < 8 ? end_bit - shift : 8;
			atomicAdd(&s_hist[p][digit_of(key, shift, (1u << bits) - 1u)], 1u);
		}
	}
	__syncthreads();
	for (int p = 0; p < passes; p++) {
		const uint32_t c = s_hist[p][threadIdx.x];
		if (c)
			atomicAdd(&hist[p * 256 + threadIdx.x], c);
	}
}

template <typename KeyT>
__global__ __launch_bounds__(256) void sort_onesweep_kernel(const KeyT* __restrict__ keys_in,
                                                             const uint32_t* __restrict__ vals_in,
                                                             KeyT* __restrict__ keys_out,
                                                             uint32_t* __restrict__ vals_out, size_t n,
                                                             const uint32_t* __restrict__ n_device, int shift,
                                                             uint32_t mask, const uint32_t* __restrict__ digit_count,
                                                             uint32_t* __restrict__ lookback,
                                                             uint32_t* __restrict__ tile_counter,
                                                             uint32_t* __restrict__ status, int spin_limit)
{
	__shared__ KeyT s_keys[kSortBlock];
	__shared__ uint32_t s_vals[kSortBlock];
	__shared__ uint32_t s_wave_hist[4][256];  // per-wave digit counts, then exclusive prefix over waves
	__shared__ uint32_t s_digit_base[256];    // exclusive prefix over digits within the tile
	__shared__ uint32_t s_global_base[256];   // where this tile's run of each digit starts globally
	__shared__ uint32_t s_scan[8];
	__shared__ uint32_t s_tile;

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	// Tiles are handed out in arrival order, so every tile a block waits for below belongs to
	// a block that is already running.
	if (tid == 0)
		s_tile = atomicAdd(tile_counter, 1u);
#pragma unroll
	for (int w = 0; w < 4; w++)
		s_wave_hist[w][tid] = 0;
	__syncthreads();
	const uint32_t tile = s_tile;
	const size_t block_base = (size_t)tile * kSortBlock;
	if (n_device)
		n = min(n, (size_t)*n_device);
	// launched for an upper bound of n: tiles beyond the data leave, and no tile waits for them
	if (block_base >= n)
		return;
	const size_t wave_base = block_base + (size_t)wave * (kSortItems * 64);

	KeyT key[kSortItems];
	uint32_t val[kSortItems];
	uint32_t rank[kSortItems];
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const size_t k = wave_base + (size_t)i * 64 + lane;
		const bool ok = k < n;
		key[i] = ok ? keys_in[k] : (KeyT)~(KeyT)0;
		val[i] = ok ? vals_in[k] : 0u;
	}

	const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const size_t k = wave_base + (size_t)i * 64 + lane;
		// Padding elements rank as digit 255 after every real element, so they never disturb one.
		const uint32_t d = (k < n) ? digit_of(key[i], shift, mask) : 255u;
		uint64_t same = ~0ull;
#pragma unroll
		for (int b = 0; b < 8; b++) {
			const bool bit = (d >> b) & 1u;
			const uint64_t vote = __ballot(bit);
			same &= bit ? vote : ~vote;
		}
		const uint32_t below = (uint32_t)__popcll(same & lanes_below);
		const uint32_t count = (uint32_t)__popcll(same);
		const int leader = __ffsll((unsigned long long)same) - 1;
		uint32_t prior = 0;
		if (lane == leader) {
			prior = s_wave_hist[wave][d];
			s_wave_hist[wave][d] = prior + count;
		}
		prior = __shfl(prior, leader);
		rank[i] = prior + below;
		__builtin_amdgcn_wave_barrier();
	}
	__syncthreads();

	// Thread d owns digit d: prefix over the 4 waves, publish the tile's count, look back.
	{
		const size_t remaining = n - block_base;
		const uint32_t valid = remaining < (size_t)kSortBlock ? (uint32_t)remaining : (uint32_t)kSortBlock;
		const uint32_t c0 = s_wave_hist[0][tid], c1 = s_wave_hist[1][tid], c2 = s_wave_hist[2][tid],
		               c3 = s_wave_hist[3][tid];
		s_wave_hist[0][tid] = 0;
		s_wave_hist[1][tid] = c0;
		s_wave_hist[2][tid] = c0 + c1;
		s_wave_hist[3][tid] = c0 + c1 + c2;
		uint32_t count = c0 + c1 + c2 + c3;
		uint32_t total;
		const uint32_t ex = block256_exclusive_scan_u32(count, s_scan, total);
		s_digit_base[tid] = ex;
		if (tid == 255)
			count -= (uint32_t)kSortBlock - valid;  // padding is not published

		uint32_t* my_word = lookback + (size_t)tile * 256 + tid;
		uint32_t exclusive = 0;
		if (tile == 0) {
			__hip_atomic_store(my_word, count | kFlagInclusive, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		} else {
			__hip_atomic_store(my_word, count | kFlagAggregate, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			uint32_t t = tile;
			bool gave_up = spin_limit < 0;
			while (!gave_up) {
				t--;
				const uint32_t* word = lookback + (size_t)t * 256 + tid;
				uint32_t v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				for (int spins = 0; (v >> 30) == 0u; spins++) {
					// give up after a bounded wait, or as soon as any other look-back has
					if (spins >= spin_limit ||
					    ((spins & 255) == 255 &&
					     __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
						gave_up = true;
						break;
					}
					__builtin_amdgcn_s_sleep(1);
					v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
				}
				if (gave_up)
					break;
				exclusive += v & kValueMask;
				if ((v & kFlagInclusive) || t == 0)
					break;
			}
			if (gave_up)
				atomicOr(status, 1u);
			// On the (never expected) give-up path `exclusive` is too small, which keeps every
			// scatter address inside the array; the status word tells the consumer to discard it.
			__hip_atomic_store(my_word, ((exclusive + count) & kValueMask) | kFlagInclusive, __ATOMIC_RELAXED,
			                   __HIP_MEMORY_SCOPE_AGENT);
		}
		// where the digit's run starts in the whole array: the exclusive scan of the digit counts
		uint32_t all;
		const uint32_t digit_start = block256_exclusive_scan_u32(digit_count[tid], s_scan, all);
		s_global_base[tid] = digit_start + exclusive;
	}
	__syncthreads();

#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const size_t k = wave_base + (size_t)i * 64 + lane;
		const uint32_t d = (k < n) ? digit_of(key[i], shift, mask) : 255u;
		const uint32_t pos = s_digit_base[d] + s_wave_hist[wave][d] + rank[i];
		s_keys[pos] = key[i];
		s_vals[pos] = val[i];
	}
	__syncthreads();

	const size_t remaining = n - block_base;
	const uint32_t valid = remaining < (size_t)kSortBlock ? (uint32_t)remaining : (uint32_t)kSortBlock;
#pragma unroll 4
	for (int i = 0; i < kSortItems; i++) {
		const uint32_t p = (uint32_t)i * 256 + tid;
		if (p < valid) {
			const KeyT kk = s_keys[p];
			const uint32_t d = digit_of(kk, shift, mask);
			const size_t dst = (size_t)s_global_base[d] + (p - s_digit_base[d]);
			if (dst < n) {
				keys_out[dst] = kk;
				vals_out[dst] = s_vals[p];
			}
		}
	}
}

size_t sort_temp_words(size_t n)
{
	return sort_temp_words_for(n);
}

const uint32_t* sort_status_word(const uint32_t* temp)
{
	return temp + kSortStatus;
}

size_t sort_clear_words(size_t n, int end_bit)
{
	const size_t tiles = (n + kSortBlock - 1) / kSortBlock;
	return kSortHeader + (size_t)((end_bit + 7) / 8) * 256 * tiles;
}

template <typename KeyT>
static void sort_pairs(KeyT* keys_in, KeyT* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                       const uint32_t* n_device, int end_bit, uint32_t* temp, bool temp_cleared, bool mark_stages,
                       uint32_t* also_clear, size_t also_clear_words, hipStream_t s)
{
	if (n == 0)
		return;
	const uint32_t tiles = (uint32_t)((n + kSortBlock - 1) / kSortBlock);
	const int passes = (end_bit + 7) / 8;
	if (mark_stages)
		stage_mark("sort_setup", s);
	if (!temp_cleared)
		launch_fill_u32(temp, 0u, sort_clear_words(n, end_bit), s);
	const uint32_t hist_blocks = tiles < 2048u ? tiles : 2048u;
	hipLaunchKernelGGL(sort_digit_histogram_kernel<KeyT>, dim3(hist_blocks), dim3(256), 0, s, keys_in, n, n_device, passes,
	                   end_bit, temp, also_clear, also_clear_words);
	KeyT *ksrc = keys_in, *kdst = keys_out;
	uint32_t *vsrc = vals_in, *vdst = vals_out;
	for (int p = 0; p < passes; p++) {
		const int shift = 8 * p;
		const int bits = end_bit - shift < 8 ? end_bit - shift : 8;
		const uint32_t mask = (1u << bits) - 1u;
		if (mark_stages)
			stage_mark("sort_onesweep", s);
		hipLaunchKernelGGL(sort_onesweep_kernel<KeyT>, dim3(tiles), dim3(256), 0, s, ksrc, vsrc, kdst, vdst, n, n_device, shift,
		                   mask,
		                   temp + p * 256, temp + kSortHeader + (size_t)p * 256 * tiles, temp + kSortCounters + p,
		                   temp + kSortStatus, g_lookback_spin_limit.load());
		KeyT* tk = ksrc; ksrc = kdst; kdst = tk;
		uint32_t* tv = vsrc; vsrc = vdst; vdst = tv;
	}
}

void launch_sort_pairs(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                       int end_bit, uint32_t* temp, hipStream_t s)
{
	sort_pairs<uint64_t>(keys_in, keys_out, vals_in, vals_out, n, nullptr, end_bit, temp, false, true, nullptr, 0, s);
}

void launch_sort_pairs_u32(uint32_t* keys_in, uint32_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                           const uint32_t* n_device, int end_bit, uint32_t* temp, bool temp_cleared, uint32_t* also_clear,
                           size_t also_clear_words, const char* stage, hipStream_t s)
{
	sort_pairs<uint32_t>(keys_in, keys_out, vals_in, vals_out, n, n_device, end_bit, temp, temp_cleared, stage != nullptr,
	                     also_clear, also_clear_words, s);
}

// ---- tile ranges (K/cuda_rasterizer_hgs/rasterizer_impl.cu:116-138 and the memset at :319) ----

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t v, size_t n)
{
	const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (i < n)
		p[i] = v;
}

void launch_fill_u32(uint32_t* p, uint32_t v, size_t n, hipStream_t s)
{
	if (n == 0)
		return;
	hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, v, n);
}

// The status words (may be null) are those of the two sorts: if either reported a failure the
// ranges stay empty, so no later stage walks an unsorted list, and *fault (host memory that the
// device can write, may be null) is set for the host to find.
__global__ __launch_bounds__(256) void tile_ranges_kernel(const uint32_t* __restrict__ keys, size_t n,
                                                           const uint32_t* __restrict__ n_device,
                                                           uint2* __restrict__ ranges,
                                                           const uint32_t* __restrict__ sort_status,
                                                           const uint32_t* __restrict__ order_status,
                                                           uint32_t* __restrict__ fault)
{
	const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
	if ((sort_status && *sort_status != 0u) || (order_status && *order_status != 0u)) {
		if (idx == 0 && fault)
			__hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		return;
	}
	if (n_device)
		n = min(n, (size_t)*n_device);  // launched for an upper bound
	if (idx >= n)
		return;
	const uint32_t cur = keys[idx];
	if (idx == 0) {
		ranges[cur].x = 0;
	} else {
		const uint32_t prev = keys[idx - 1];
		if (cur != prev) {
			ranges[prev].y = (uint32_t)idx;
			ranges[cur].x = (uint32_t)idx;
		}
	}
	if (idx == n - 1)
		ranges[cur].y = (uint32_t)n;
}

__global__ void report_sort_status_kernel(const uint32_t* __restrict__ status, uint32_t* __restrict__ fault)
{
	if (threadIdx.x == 0 && *status != 0u)
		__hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

void launch_report_sort_status(const uint32_t* temp, uint32_t* fault, hipStream_t s)
{
	if (fault)
		hipLaunchKernelGGL(report_sort_status_kernel, dim3(1), dim3(64), 0, s, temp + kSortStatus, fault);
}

void launch_tile_ranges(const uint32_t* keys, size_t n, const uint32_t* n_device, uint2* ranges, int tiles,
                        const uint32_t* sort_status, const uint32_t* order_status, uint32_t* fault, bool ranges_cleared,
                        hipStream_t s)
{
	stage_mark("tile_ranges", s);
	if (!ranges_cleared)
		launch_fill_u32(reinterpret_cast<uint32_t*>(ranges), 0u, (size_t)tiles * 2 + kRangeTailWords, s);
	if (n == 0)
		return;
	hipLaunchKernelGGL(tile_ranges_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, keys, n, n_device,
	                   ranges, sort_status, order_status, fault);
}

}  // namespace rgs
