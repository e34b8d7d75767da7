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
#include "strip_filing.h"

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
// to *total_out and *total_copy (if non-null).  Block 1, if launched, does the same for a second
// array of the same length.  blockIdx.y selects the job.
struct BlockScanJob {
	uint32_t* data;
	size_t n;
	const uint32_t* n_device;  // if non-null: the number of elements behind the entries, `per_entry` of them to an entry
	uint32_t per_entry;
	uint32_t* total_out;
	uint32_t* total_copy;
	uint32_t* data_b;
	uint32_t* total_out_b;
};

__global__ __launch_bounds__(1024) void single_block_exclusive_scan_kernel(Batch<BlockScanJob> batch)
{
	__shared__ uint32_t wave_tot[16];
	const BlockScanJob& j = batch.job[blockIdx.y];
	uint32_t* data = j.data;
	size_t n = j.n;
	const uint32_t* n_device = j.n_device;
	uint32_t* total_out = j.total_out;
	uint32_t* total_copy = j.total_copy;
	if (blockIdx.x == 1) {
		data = j.data_b;
		total_out = j.total_out_b;
		total_copy = nullptr;
	}
	if (!data)
		return;
	if (n_device)
		n = ((size_t)*n_device + j.per_entry - 1) / j.per_entry;
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
	if (tid == 0 && total_copy)
		*total_copy = total;
}

struct BlockInclusiveJob {
	const uint32_t* in;
	const uint32_t* block_base;
	size_t n;
	const uint32_t* n_device;
	uint32_t* out;
	uint32_t* first_of_block;  // may be null; see DuplicateJob
	uint32_t first_of_block_words;
	// non-zero: block_base holds the totals of the workgroups' elements, not yet scanned: a workgroup adds up those
	// ahead of its own itself (for a few thousand workgroups at most, which saves the launch that scans them)
	uint32_t base_from_totals;
};

// kPer consecutive elements per thread; with kPer = 4 `in` and `out` are 16-byte aligned and moved 16 bytes at a time.
constexpr int kScanGroup = 1024;  // elements per workgroup of the four-per-thread kernels of the depth order
template <int kPer>
__global__ __launch_bounds__(256) void block_inclusive_scan_kernel(Batch<BlockInclusiveJob> batch)
{
	__shared__ uint32_t lds[8];
	constexpr size_t kGroup = 256 * (size_t)kPer;
	const BlockInclusiveJob& j = batch.job[blockIdx.y];
	const uint32_t* __restrict__ in = j.in;
	const uint32_t* __restrict__ block_base = j.block_base;
	uint32_t* __restrict__ out = j.out;
	size_t n = j.n;
	if (j.n_device)
		n = *j.n_device;
	if ((size_t)blockIdx.x * kGroup >= n)
		return;
	const size_t i0 = (size_t)blockIdx.x * kGroup + (size_t)kPer * threadIdx.x;
	uint32_t v[kPer];
	const bool whole = i0 + kPer <= n;
	bool loaded = false;
	if constexpr (kPer == 4) {
		if (whole) {
			const uint4 v4 = *reinterpret_cast<const uint4*>(in + i0);
			v[0] = v4.x; v[1] = v4.y; v[2] = v4.z; v[3] = v4.w;
			loaded = true;
		}
	}
	if (!loaded) {
#pragma unroll
		for (int q = 0; q < kPer; q++)
			v[q] = i0 + q < n ? in[i0 + q] : 0u;
	}
	uint32_t sum = 0;
#pragma unroll
	for (int q = 0; q < kPer; q++)
		sum += v[q];
	uint32_t total;
	uint32_t base = 0;
	if (j.base_from_totals) {
		uint32_t ahead = 0;
		for (uint32_t b = threadIdx.x; b < blockIdx.x; b += 256)
			ahead += block_base[b];
		(void)block256_exclusive_scan_u32(ahead, lds, base);
	} else {
		base = block_base[blockIdx.x];
	}
	uint32_t run = base + block256_exclusive_scan_u32(sum, lds, total);
	uint32_t end[kPer];
#pragma unroll
	for (int q = 0; q < kPer; q++) {
		const uint32_t begin = run;
		run += v[q];
		end[q] = run;
		if (j.first_of_block && i0 + q < n) {
			// element i covers positions [begin, end): it is where every workgroup of the key duplication starts whose
			// first position, a multiple of kDupPositions, lies among them
			for (uint32_t b = (begin + (uint32_t)kDupPositions - 1u) / (uint32_t)kDupPositions;
			     b < j.first_of_block_words && (uint64_t)b * (uint64_t)kDupPositions < (uint64_t)run; b++)
				j.first_of_block[b] = (uint32_t)(i0 + q);
		}
	}
	bool stored = false;
	if constexpr (kPer == 4) {
		if (whole) {
			*reinterpret_cast<uint4*>(out + i0) = uint4{end[0], end[1], end[2], end[3]};
			stored = true;
		}
	}
	if (!stored) {
#pragma unroll
		for (int q = 0; q < kPer; q++)
			if (i0 + q < n)
				out[i0 + q] = end[q];
	}
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
	Batch<BlockScanJob> scan = {};
	scan.job[0] = BlockScanJob{temp, nb, n_device, 256u, nullptr, nullptr, nullptr, nullptr};
	hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(1), dim3(1024), 0, s, scan);
	Batch<BlockInclusiveJob> inc = {};
	inc.job[0] = BlockInclusiveJob{in, temp, n, n_device, out, nullptr, 0u, 0u};
	hipLaunchKernelGGL(block_inclusive_scan_kernel<1>, dim3((unsigned)nb), dim3(256), 0, s, inc);
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

void launch_totals_from_block_sums(const TotalsJob* jobs, int count, hipStream_t s)
{
	stage_mark("offset_scan", s);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<BlockScanJob> b = {};
		for (int k = 0; k < nj; k++) {
			const TotalsJob& t = jobs[at + k];
			b.job[k] = BlockScanJob{t.block_sums, ((size_t)t.P + 255) / 256, nullptr, 256u, t.total_out, t.total_copy, t.block_visible,
			                        t.visible_count};
		}
		hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(2, (unsigned)nj), dim3(1024), 0, s, b);
	}
}

// ---- depth order and key duplication (K/cuda_rasterizer_hgs/rasterizer_impl.cu:70-111) -------

// Keys of the depth sort.  A rendered Gaussian's depth exceeds 0.2, so its bit pattern, which orders like the value,
// lies above that of 0.125: the sort looks at bits - kDepthKeyBase, whose low kDepthKeyBits bits (three 9-bit digits)
// tell every depth below 8192 apart.  Should a key have bits above those (a depth of 8192 or more), the kernel that
// writes the keys says so in the sort's scratch and a fourth pass over the remaining bits runs; otherwise that pass
// returns at once.  Either way the order is that of the full 32 bits.
constexpr uint32_t kDepthKeyBase = 0x3E000000u;
constexpr int kDepthKeyBits = 27;
constexpr int kDepthPasses = 3;                 // of 9 bits each, plus the one on demand
constexpr uint32_t kSortExtraPass = 2057;       // word of the sort scratch's header: non-zero = the fourth pass is needed

// The values of the depth sort carry the Gaussian's tile count above its index, so that the pass that ends the sort
// can write the counts in depth order itself (a gather of its own over the sorted indices cost as much as a pass).
// A count that does not fit is stored as all ones and looked up by that pass.
__host__ __device__ inline uint32_t depth_index_bits(uint32_t P)
{
	uint32_t bits = 1;
	while (bits < 31u && (P - 1u) >> bits)
		bits++;
	return bits;
}

// (depth key, index and tile count) pairs of the Gaussians that touch a tile, compacted in index order: the
// group of Gaussians [kScanGroup b, kScanGroup (b + 1)), four neighbouring ones per thread, is written
// from visible_base[4 b] on (the bases are per 256 Gaussians).  A workgroup takes every gridDim.x-th group and
// counts the digits of the keys it writes on the way: at the end it adds its counts to the digit histograms
// the sort of these pairs starts from (cleared beforehand), which saves that sort its own pass over the keys.
__global__ __launch_bounds__(256) void depth_pairs_kernel(Batch<DepthOrderJob> batch)
{
	__shared__ uint32_t lds[8];
	__shared__ uint32_t s_hist[kDepthPasses][512];
	__shared__ uint32_t s_top[32];   // digit of the pass on demand; value 0 is not counted here but derived
	const DepthOrderJob& j = batch.job[blockIdx.y];
	const size_t P = (size_t)j.P;
	if ((size_t)blockIdx.x * kScanGroup >= P)
		return;
	const float* __restrict__ depths = j.depths;
	const uint32_t* __restrict__ tiles_touched = j.tiles_touched;
	const uint32_t* __restrict__ visible_base = j.block_visible;
	uint32_t* __restrict__ keys = j.keys_a;
	uint32_t* __restrict__ values = j.vals_a;
	const uint32_t index_bits = depth_index_bits((uint32_t)j.P), cap = 0xFFFFFFFFu >> index_bits;
#pragma unroll
	for (int p = 0; p < kDepthPasses; p++) {
		s_hist[p][threadIdx.x] = 0u;
		s_hist[p][256 + threadIdx.x] = 0u;
	}
	if (threadIdx.x < 32)
		s_top[threadIdx.x] = 0u;
	__syncthreads();
	uint32_t written = 0;
	for (size_t group = blockIdx.x; group * kScanGroup < P; group += gridDim.x) {
		const size_t idx0 = group * kScanGroup + 4 * (size_t)threadIdx.x;
		// the depth of a Gaussian that touches no tile is stored as 0, that of one that does exceeds 0.2: the
		// depths alone say which ones are listed
		float depth[4] = {0.f, 0.f, 0.f, 0.f};
		uint32_t count[4] = {0u, 0u, 0u, 0u};
		if (idx0 + 4 <= P) {
			const float4 d4 = *reinterpret_cast<const float4*>(depths + idx0);
			const uint4 c4 = *reinterpret_cast<const uint4*>(tiles_touched + idx0);
			depth[0] = d4.x; depth[1] = d4.y; depth[2] = d4.z; depth[3] = d4.w;
			count[0] = c4.x; count[1] = c4.y; count[2] = c4.z; count[3] = c4.w;
		} else {
#pragma unroll
			for (int q = 0; q < 4; q++)
				if (idx0 + q < P) {
					depth[q] = depths[idx0 + q];
					count[q] = tiles_touched[idx0 + q];
				}
		}
		uint32_t mine = 0;
#pragma unroll
		for (int q = 0; q < 4; q++)
			mine += __float_as_uint(depth[q]) != 0u ? 1u : 0u;
		uint32_t total;
		uint32_t at = visible_base[4 * group] + block256_exclusive_scan_u32(mine, lds, total);
		written += mine;
#pragma unroll
		for (int q = 0; q < 4; q++)
			if (__float_as_uint(depth[q]) != 0u) {
				const uint32_t key = __float_as_uint(depth[q]) - kDepthKeyBase;
				keys[at] = key;
				values[at] = (uint32_t)(idx0 + q) | (min(count[q], cap) << index_bits);
				at++;
#pragma unroll
				for (int p = 0; p < kDepthPasses; p++)
					atomicAdd(&s_hist[p][(key >> (9 * p)) & 511u], 1u);
				if (key >> kDepthKeyBits)
					atomicAdd(&s_top[key >> kDepthKeyBits], 1u);
			}
	}
	__syncthreads();
#pragma unroll
	for (int p = 0; p < kDepthPasses; p++)
#pragma unroll
		for (int h = 0; h < 2; h++) {
			const uint32_t c = s_hist[p][256 * h + threadIdx.x];
			if (c)
				atomicAdd(&j.sort_temp[512 * p + 256 * h + threadIdx.x], c);
		}
	// the digit of the pass on demand: value 0 takes every key that was not counted under another value
	uint32_t all_written;
	(void)block256_exclusive_scan_u32(written, lds, all_written);
	if (threadIdx.x < 32) {
		uint32_t c = s_top[threadIdx.x];
		if (threadIdx.x == 0) {
			uint32_t others = 0;
			for (int v = 1; v < 32; v++)
				others += s_top[v];
			c = all_written - others;
			if (others)
				atomicOr(&j.sort_temp[kSortExtraPass], 1u);
		}
		if (c)
			atomicAdd(&j.sort_temp[512 * kDepthPasses + threadIdx.x], c);
	}
}

// The sum of every kScanGroup of the tile counts in depth order (the first level of the scan that follows),
// four neighbouring ones per thread; the count of them is on the device.
__global__ __launch_bounds__(256) void order_totals_kernel(Batch<DepthOrderJob> batch)
{
	__shared__ uint32_t lds[8];
	const DepthOrderJob& j = batch.job[blockIdx.y];
	if (blockIdx.x == 0)  // what the key duplication will count the digits of its tiles into
		for (int w = threadIdx.x; w < kTileDigitWords; w += 256)
			j.tile_digits[w] = 0u;
	const size_t n = min((size_t)*j.visible_count, (size_t)j.P);
	if ((size_t)blockIdx.x * kScanGroup >= n)
		return;
	const uint32_t* __restrict__ in = j.tiles_in_order;
	const size_t k0 = (size_t)blockIdx.x * kScanGroup + 4 * (size_t)threadIdx.x;
	uint32_t sum = 0;
	if (k0 + 4 <= n) {
		const uint4 v = *reinterpret_cast<const uint4*>(in + k0);
		sum = v.x + v.y + v.z + v.w;
	} else {
#pragma unroll
		for (int q = 0; q < 4; q++)
			if (k0 + q < n)
				sum += in[k0 + q];
	}
	uint32_t total;
	(void)block256_exclusive_scan_u32(sum, lds, total);
	if (threadIdx.x == 0)
		j.scan_temp[blockIdx.x] = total;
}

// Instances of the Gaussians in depth order, tiles row by row like the reference, at the offsets
// of the scan taken in that same order.  The work is dealt out by output position, not by Gaussian:
// a workgroup writes runs of kDupPositions consecutive instances, whichever Gaussians they belong to (one
// that covers thousands of tiles is shared by several runs, a thousand that cover one tile
// each are taken by one).  It takes the first Gaussian of a run from the table the offset scan has filled
// (beyond that table, from a 64-ary search over the inclusive offsets), stages the offsets and indices of
// the Gaussians of the run in LDS 256 at a time
// and lets every thread find the Gaussian of its output position by a binary search over those 256
// offsets, read that Gaussian's 64-byte record, and take the tile from the position inside the
// record's rectangle; stores are contiguous.  The thread also decides which of the
// tile's four strips the instance can matter to (strip_filing.h) and puts those bits above the
// tile in the key: the sort only looks at the tile bits, so they travel with the instance for free.
// On the way the workgroup counts the digits of the tiles it writes (what the sort's passes start from:
// the sort then has no pass of its own over the keys) and it clears the sort's scratch and the tile ranges.
// `order` is the output of a sort: should that sort ever have given up, its entries may be anything, so
// they are clamped to the P Gaussians there are (the tile ranges then stay empty and nothing reads the result).
struct DuplicateStage {
	uint32_t end[256];     // inclusive offset of each staged Gaussian
	uint32_t index[256];
};

// Floats of LDS for the NDC tables of a grid of tiles: 2 per tile column (rounded up to a multiple of 4), 8 per tile row.
static inline size_t ndc_table_floats(int gx, int gy)
{
	return (size_t)((2 * gx + 3) & ~3) + 8 * (size_t)gy;
}
constexpr size_t kNdcTableMaxFloats = 8192;  // larger grids compute the coordinates per instance

__global__ __launch_bounds__(256) void duplicate_with_keys_kernel(Batch<DuplicateJob> batch, int gx, int gy, int ndc_in_lds)
{
	__shared__ DuplicateStage st;
	__shared__ uint32_t s_first;
	__shared__ uint32_t s_digits[kTileDigitWords];  // digit counts of the tiles this workgroup writes
	extern __shared__ __align__(16) float s_ndc[];  // NDC of every tile column's first and last pixel, then of every strip's first and last row
	const DuplicateJob& job = batch.job[blockIdx.y];
	const uint32_t P = (uint32_t)job.P;
	const uint32_t* __restrict__ visible_count = job.visible_count;
	const uint32_t* __restrict__ order = job.order;
	const uint32_t* __restrict__ offsets = job.offsets;
	const FilingArgs& filing = job.filing;
	uint32_t* __restrict__ keys = job.keys;
	uint32_t* __restrict__ values = job.values;
	const uint32_t capacity = job.capacity;
	uint32_t* __restrict__ clear = job.clear;
	const size_t clear_words = job.clear_words;
	const int tid = threadIdx.x, lane = tid & 63;
	// the scratch of the sort that follows is cleared here, which saves a launch
	for (size_t w = (size_t)blockIdx.x * 256 + tid; w < clear_words; w += (size_t)gridDim.x * 256)
		clear[w] = 0u;
	for (size_t w = (size_t)blockIdx.x * 256 + tid; w < job.also_clear_words; w += (size_t)gridDim.x * 256)
		job.also_clear[w] = 0u;
	const uint32_t n = min(*visible_count, P);
	const uint32_t total = *job.total;
	if (n == 0u)
		return;
	const uint32_t limit = min(total, capacity);  // positions beyond the room the caller gave are dropped
	if (blockIdx.x * (uint32_t)kDupPositions >= limit)
		return;
	const int digit_bits = sort_max_digit_bits_u32(job.end_bit);
	const int passes = sort_passes(job.end_bit, digit_bits);
	for (int w = tid; w < kTileDigitWords; w += 256)
		s_digits[w] = 0u;

	const int rows_at = (2 * gx + 3) & ~3;
	if (ndc_in_lds) {
		for (int c = tid; c < gx; c += 256) {
			const float2 v = tile_column_ndc(c, filing.W);
			s_ndc[2 * c] = v.x;
			s_ndc[2 * c + 1] = v.y;
		}
		for (int r = tid; r < 4 * gy; r += 256) {
			const float2 v = strip_rows_ndc(r >> 2, r & 3, filing.H);
			s_ndc[rows_at + 2 * r] = v.x;
			s_ndc[rows_at + 2 * r + 1] = v.y;
		}
	}
	const BoxFrame box = load_box_frame(filing.projinv, filing.range_low, filing.range_up, filing.tanfovx, filing.tanfovy);

	// A workgroup takes every gridDim.x-th run of kDupPositions positions: the tables above are set up once, and the
	// digit counts of many runs leave with one atomic add per digit.  What a run needs first (the Gaussian its
	// positions begin at, from the table the offset scan has filled, and the offsets and indices of the 256 Gaussians
	// from there on: a run of 256 positions cannot span more, every listed Gaussian having an instance) is asked for
	// one run ahead, so that these two dependent reads are under way while the previous run is worked on.
	const uint32_t table_runs = (uint32_t)dup_first_words((size_t)P);
	uint32_t ahead_end = 0, ahead_index = 0, ahead_begin = 0;
	bool ahead = false;  // the same for every thread of the workgroup
	auto ask_for = [&](uint32_t r) {
		const uint32_t f = min(job.first_of_block[r], n - 1u);
		const uint32_t g = f + (uint32_t)tid;
		ahead_end = g < n ? offsets[g] : total;
		ahead_index = g < n ? min(order[g], P - 1u) : 0u;
		ahead_begin = f == 0u ? 0u : offsets[f - 1];
		ahead = true;
	};
	if (blockIdx.x < table_runs)
		ask_for(blockIdx.x);
	for (uint32_t run = blockIdx.x; (uint64_t)run * kDupPositions < (uint64_t)limit; run += gridDim.x) {
	const uint32_t start = run * (uint32_t)kDupPositions;
	const uint32_t stop = min(start + (uint32_t)kDupPositions, limit);
	__syncthreads();  // the previous run is done with s_first and the staged Gaussians; the tables are written
	uint32_t staged_begin;
	if (ahead) {
		st.end[tid] = ahead_end;
		st.index[tid] = ahead_index;
		staged_begin = ahead_begin;
	} else {
		// beyond the table (more than 16 instances per Gaussian on average): the first Gaussian whose inclusive offset
		// exceeds `start` by a 64-ary search of the first wavefront
		if (tid < 64) {
			uint32_t lo = 0, hi = n;  // the answer lies in [lo, hi]
			while (lo < hi) {
				const uint32_t step = (hi - lo + 63u) / 64u;
				const uint32_t probe = lo + (uint32_t)lane * step;
				const bool below = probe < hi && offsets[probe] <= start;
				const uint32_t c = (uint32_t)__popcll(lanes_where(below));  // the predicate is monotone: the first c probes hold
				if (c == 0u) {
					hi = lo;
				} else {
					const uint32_t last_true = lo + (c - 1u) * step;
					lo = last_true + 1u;
					hi = min(last_true + step, hi);
				}
			}
			if (lane == 0)
				s_first = min(lo, n - 1u);
		}
		__syncthreads();
		const uint32_t g0 = s_first, g = g0 + (uint32_t)tid;
		st.end[tid] = g < n ? offsets[g] : total;
		st.index[tid] = g < n ? min(order[g], P - 1u) : 0u;
		staged_begin = g0 == 0u ? 0u : offsets[g0 - 1];
	}
	__syncthreads();
	ahead = false;
	if ((uint64_t)(run + gridDim.x) * kDupPositions < (uint64_t)limit && run + gridDim.x < table_runs)
		ask_for(run + gridDim.x);

	{
		const uint32_t staged_end = st.end[255];
		const uint32_t from = max(start, staged_begin), to = min(stop, staged_end);
		// Up to kDupPositions / 256 positions per thread.  First all of them find their Gaussian and ask for its
		// record (pixel centre, conic, extents, radius: everything else follows from those), then each is finished:
		// the records of a thread arrive together, not one wait after another.
		constexpr int kPerThread = kDupPositions / 256;
		uint32_t first[kPerThread], index[kPerThread];
		float4 r0[kPerThread], r1[kPerThread], r3[kPerThread];
#pragma unroll
		for (int q = 0; q < kPerThread; q++) {
			const uint32_t pos = from + (uint32_t)tid + 256u * (uint32_t)q;
			first[q] = 0u;
			index[q] = 0u;
			if (pos < to) {
				// the first staged Gaussian whose inclusive offset exceeds pos
				int lo = 0;
#pragma unroll
				for (int step = 128; step > 0; step >>= 1)
					if (st.end[lo + step - 1] <= pos)
						lo += step;
				first[q] = lo == 0 ? staged_begin : st.end[lo - 1];
				index[q] = st.index[lo];
				const float4* rec = filing.record + 4 * (size_t)index[q];
				r0[q] = rec[0];
				r1[q] = rec[1];
				r3[q] = rec[3];
			}
		}
		uint32_t tile_of[kPerThread];
#pragma unroll
		for (int q = 0; q < kPerThread; q++) {
			const uint32_t pos = from + (uint32_t)tid + 256u * (uint32_t)q;
			tile_of[q] = 0xFFFFFFFFu;
			if (pos >= to)
				continue;
			const TileRect rc = tile_rect(r0[q].x, r0[q].y, __float_as_int(r3[q].z), gx, gy);
			const uint32_t t = pos - first[q], w = max(rc.x1 - rc.x0, 1u);
			// t / w through the reciprocal in single precision (both are below 2^24, so exact as floats; the quotient
			// is off by one at most, which the remainder shows): a third of the instructions of the integer division
			uint32_t row = (uint32_t)((float)t * __builtin_amdgcn_rcpf((float)w));
			int col = (int)(t - row * w);
			if (col < 0) {
				row--;
				col += (int)w;
			} else if (col >= (int)w) {
				row++;
				col -= (int)w;
			}
			const int tx = (int)rc.x0 + col, ty = (int)(rc.y0 + row);
			const uint32_t tile = (uint32_t)ty * (uint32_t)gx + (uint32_t)tx;
			float2 nx;
			float ny[8];
			if (ndc_in_lds) {
				nx = float2{s_ndc[2 * tx], s_ndc[2 * tx + 1]};
				const float4 y0 = *reinterpret_cast<const float4*>(s_ndc + rows_at + 8 * ty);
				const float4 y1 = *reinterpret_cast<const float4*>(s_ndc + rows_at + 8 * ty + 4);
				ny[0] = y0.x; ny[1] = y0.y; ny[2] = y0.z; ny[3] = y0.w;
				ny[4] = y1.x; ny[5] = y1.y; ny[6] = y1.z; ny[7] = y1.w;
			} else {
				nx = tile_column_ndc(tx, filing.W);
#pragma unroll
				for (int h = 0; h < 4; h++) {
					const float2 v = strip_rows_ndc(ty, h, filing.H);
					ny[2 * h] = v.x;
					ny[2 * h + 1] = v.y;
				}
			}
			const StripTests tests = prepare_strip_tests(FiledGeometry{r0[q], r1[q], float2{r3[q].x, r3[q].y}}, box);
			const uint32_t strips = strips_filed_for(tests, (float)(tx * kTile), (float)(ty * kTile), nx, ny, box);
			keys[pos] = tile | (strips << kKeyTileBits);
			values[pos] = index[q];
			tile_of[q] = tile;
		}
		// the digits of the tiles just written, for the sort (every lane comes here: the narrow digits are counted by ballot)
#pragma unroll
		for (int q = 0; q < kPerThread; q++) {
			const bool have = tile_of[q] != 0xFFFFFFFFu;
			for (int p = 0; p < passes; p++) {
				const int shift = sort_digit_shift(job.end_bit, p, digit_bits);
				const int bits = sort_digit_bits(job.end_bit, p, digit_bits);
				const uint32_t d = (tile_of[q] >> shift) & ((1u << bits) - 1u);
				if (bits <= 2) {
					// a digit of one or two bits: every lane would add to one of a few words, one after the other
					for (uint32_t v = 0; v < (1u << bits); v++) {
						const uint32_t c = (uint32_t)__popcll(lanes_where(have && d == v));
						if (lane == 0 && c != 0u)
							atomicAdd(&s_digits[512 * p + v], c);
					}
				} else if (have) {
					atomicAdd(&s_digits[512 * p + d], 1u);
				}
			}
		}
	}
	}
	__syncthreads();
	for (int w = tid; w < 512 * passes; w += 256) {
		const uint32_t c = s_digits[w];
		if (c)
			atomicAdd(&job.tile_digits[w], c);
	}
}

void launch_duplicate_with_keys(const DuplicateJob* jobs, int count, int grid_x, int grid_y, hipStream_t s)
{
	stage_mark("duplicate_with_keys", s);
	const size_t table = ndc_table_floats(grid_x, grid_y);
	const int ndc_in_lds = table <= kNdcTableMaxFloats ? 1 : 0;
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<DuplicateJob> b = {};
		size_t blocks = 1;
		for (int k = 0; k < nj; k++) {
			b.job[k] = jobs[at + k];
			// sized for the positions there is room for; at least enough workgroups to clear the sort's scratch at a decent rate
			const size_t need = max((size_t)(b.job[k].capacity + kDupPositions - 1) / kDupPositions,
			                        min((b.job[k].clear_words + 4095) / 4096, (size_t)1024));
			blocks = need > blocks ? need : blocks;
		}
		// every workgroup ends with an atomic add per digit into its job's counts: enough of them to fill the GPU several
		// times over, each over many runs of positions, rather than one per run
		const size_t most = nj >= 8 ? 512 : nj >= 4 ? 4096 / (size_t)nj : 1024;  // twice and four times as many were measured slower
		blocks = blocks < most ? blocks : most;
		hipLaunchKernelGGL(duplicate_with_keys_kernel, dim3((unsigned)blocks, (unsigned)nj), dim3(256),
		                   ndc_in_lds ? table * sizeof(float) : 0, s, b, grid_x, grid_y, ndc_in_lds);
	}
}

// ---- radix sort -------------------------------------------------------------------------------
// Replaces cub::DeviceRadixSort::SortPairs at K/cuda_rasterizer_hgs/rasterizer_impl.cu:312-317:
// a stable least-significant-digit sort of (key, u32 value) pairs on key bits [0, end_bit), in the one-sweep form:
// the digit histogram of every pass is built while the keys are written (or, for the stand-alone entry points, by one
// kernel that reads them once), then each pass is a single kernel whose blocks take tiles of
// kSortBlock pairs in arrival order, rank them in LDS, obtain their global digit offsets from
// the blocks before them through a chained look-back over per-tile status words, and scatter.
// Element order inside a tile is (wave, round, lane); ranking preserves it, and tiles are
// ordered by their id, so every pass is stable.  A digit has up to kBits bits (template parameter): 9 for 32-bit
// keys, which sorts 17 or 18 tile bits in two passes and 27 depth bits in three, 8 for 64-bit keys, whose tiles of
// pairs fill the LDS.
//
// Scratch layout (u32 words), B = 2^kBits:
//   [0, 2048)      digit histograms, B words per pass (every block of a pass scans its counts itself)
//   [2048, 2056)   tile counter of each pass
//   [2056]         status: non-zero if a look-back ever gave up waiting (never expected)
//   [2057]         depth sort only: non-zero if its pass on demand is needed (kSortExtraPass)
//   [kSortHeader + pass * B * tiles + tile * B + digit]  look-back words

constexpr uint32_t kSortCounters = 2048;
constexpr uint32_t kSortStatus = 2056;
constexpr uint32_t kFlagAggregate = 1u << 30;  // word holds this tile's own digit count
constexpr uint32_t kFlagInclusive = 2u << 30;  // word holds the count of this and all earlier tiles
constexpr uint32_t kValueMask = (1u << 30) - 1u;
constexpr int kLookbackSpinLimit = 1 << 18;
constexpr int kLookBatch = 4;  // earlier tiles a look-back reads at once (1, 2 and 8 to 32 were measured slower)

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

// Only the stand-alone sort entry points run this (64-bit keys, digits of kDigitBitsU64 bits).
template <typename KeyT>
__global__ __launch_bounds__(256) void sort_digit_histogram_kernel(Batch<SortJob<KeyT>> batch, int passes, int end_bit)
{
	constexpr int kMaxPasses = 8;
	__shared__ uint32_t s_hist[kMaxPasses][256];
	const SortJob<KeyT>& j = batch.job[blockIdx.y];
	const KeyT* __restrict__ keys = j.keys_in;
	size_t n = j.n;
	const uint32_t* __restrict__ n_device = j.n_device;
	uint32_t* __restrict__ hist = j.temp;
	uint32_t* __restrict__ clear = j.also_clear;
	const size_t clear_words = j.also_clear_words;
	for (size_t w = (size_t)blockIdx.x * 256 + threadIdx.x; w < clear_words; w += (size_t)gridDim.x * 256)
		clear[w] = 0u;  // an array that a later kernel of the same stream wants cleared
	if (n_device)
		n = min(n, (size_t)*n_device);
#pragma unroll
	for (int p = 0; p < kMaxPasses; p++)
		s_hist[p][threadIdx.x] = 0;
	__syncthreads();
	// four keys per thread and round, requested together: one key at a time the loop waits for
	// memory once per key and the kernel takes as long as a pass of the sort
	const size_t threads = (size_t)gridDim.x * 256;
	for (size_t k = (size_t)blockIdx.x * 256 + threadIdx.x; k < n; k += 4 * threads) {
		KeyT key[4];
#pragma unroll
		for (int q = 0; q < 4; q++)
			key[q] = k + q * threads < n ? keys[k + q * threads] : (KeyT)0;
#pragma unroll
		for (int q = 0; q < 4; q++) {
			if (k + q * threads >= n)
				break;
			for (int p = 0; p < passes; p++) {
				const int shift = sort_digit_shift(end_bit, p, kDigitBitsU64);
				const int bits = sort_digit_bits(end_bit, p, kDigitBitsU64);
				const uint32_t d = digit_of(key[q], shift, (1u << bits) - 1u);
				if (bits <= 2) {
					// a digit of one or two bits: every lane would add to one of a few words, one after the
					// other; count the lanes of each value instead
					for (uint32_t v = 0; v < (1u << bits); v++) {
						const uint32_t c = (uint32_t)__popcll(lanes_where(d == v));
						if ((threadIdx.x & 63) == 0 && c != 0u)
							atomicAdd(&s_hist[p][v], c);
					}
				} else {
					atomicAdd(&s_hist[p][d], 1u);
				}
			}
		}
	}
	__syncthreads();
	for (int p = 0; p < passes; p++) {
		const uint32_t c = s_hist[p][threadIdx.x];
		if (c)
			atomicAdd(&hist[p * 256 + threadIdx.x], c);
	}
}

// What a pass does with its output:
//   kPassPlain        keys and values to the other buffer pair;
//   kPassEndsUnless   depth sort, third pass: if the scratch says that a fourth pass is needed, as kPassPlain; otherwise the
//                     sort ends here and the values are taken apart (Gaussian index to final_index, its tile count to
//                     final_count, see SortJob);
//   kPassOnDemand     depth sort, fourth pass: returns at once unless the scratch says it is needed; ends the sort.
enum SortPassKind { kPassPlain = 0, kPassEndsUnless = 1, kPassOnDemand = 2 };

// Per-wave digit counts fit 16 bits (a wavefront ranks kSortItems * 64 keys), and so does a digit's place inside a tile.
template <int kBits>
struct SortCounts {
	uint16_t wave_hist[4][1 << kBits];  // per-wave digit counts, then exclusive prefix over waves
	uint16_t digit_base[1 << kBits];    // exclusive prefix over digits within the tile
	uint32_t global_base[1 << kBits];   // where this tile's run of each digit starts globally
};

template <typename KeyT, int kBits, int kKind>
__global__ __launch_bounds__(256) void sort_onesweep_kernel(Batch<SortJob<KeyT>> batch, int pass, int shift, uint32_t mask,
                                                             int spin_limit)
{
	constexpr int kBins = 1 << kBits;
	constexpr int kOwn = kBins / 256;  // digit values a thread owns: kOwn * tid .. kOwn * tid + kOwn - 1
	static_assert(kOwn == 1 || kOwn == 2, "256 threads own one or two digit values each");
	const SortJob<KeyT>& j = batch.job[blockIdx.y];
	// the passes ping-pong between the two buffer pairs, starting in -> out
	const KeyT* __restrict__ keys_in = (pass & 1) ? j.keys_out : j.keys_in;
	const uint32_t* __restrict__ vals_in = (pass & 1) ? j.vals_out : j.vals_in;
	KeyT* __restrict__ keys_out = (pass & 1) ? j.keys_in : j.keys_out;
	uint32_t* __restrict__ vals_out = (pass & 1) ? j.vals_in : j.vals_out;
	size_t n = j.n;
	const uint32_t* __restrict__ n_device = j.n_device;
	const size_t job_tiles = (j.n + kSortBlock - 1) / kSortBlock;
	if (blockIdx.x >= job_tiles)
		return;  // the launch is sized for the job with the most tiles
	bool ends_here = false;
	if (kKind != kPassPlain) {
		const bool extra = j.temp[kSortExtraPass] != 0u;
		if (kKind == kPassOnDemand && !extra)
			return;
		ends_here = kKind == kPassOnDemand || !extra;
	}
	// the digit counts of a pass: 512 words apart for 32-bit keys whatever the digit width, 256 for 64-bit keys
	constexpr int kCountStride = sizeof(KeyT) == 4 ? 512 : 256;
	const uint32_t* __restrict__ digit_count = (j.digit_counts ? j.digit_counts : j.temp) + pass * kCountStride;
	uint32_t* __restrict__ lookback = j.temp + kSortHeader + (size_t)pass * kBins * job_tiles;
	uint32_t* __restrict__ tile_counter = j.temp + kSortCounters + pass;
	uint32_t* __restrict__ status = j.temp + kSortStatus;
	__shared__ KeyT s_keys[kSortBlock];
	__shared__ uint32_t s_vals[kSortBlock];
	__shared__ SortCounts<kBits> sc;
	__shared__ uint32_t s_scan[8];
	__shared__ uint32_t s_tile;

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	// asked for before anything else: needed only after the look-back, by when it has long arrived
	uint32_t digit_total[kOwn];
#pragma unroll
	for (int o = 0; o < kOwn; o++)
		digit_total[o] = digit_count[kOwn * tid + o];
	// Tiles are handed out in arrival order, so every tile a block waits for below belongs to
	// a block that is already running.
	if (tid == 0)
		s_tile = atomicAdd(tile_counter, 1u);
#pragma unroll
	for (int w = 0; w < 4; w++)
#pragma unroll
		for (int o = 0; o < kOwn; o++)
			sc.wave_hist[w][kOwn * tid + o] = 0;
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
		// Padding elements rank as the last digit value after every real element, so they never disturb one.
		const uint32_t d = (k < n) ? digit_of(key[i], shift, mask) : (uint32_t)(kBins - 1);
		uint64_t same = ~0ull;
#pragma unroll
		for (int b = 0; b < kBits; b++) {
			const bool bit = (d >> b) & 1u;
			const uint64_t vote = lanes_where(bit);
			same &= bit ? vote : ~vote;
		}
		const uint32_t below = (uint32_t)__popcll(same & lanes_below);
		const uint32_t count = (uint32_t)__popcll(same);
		const int leader = __ffsll((unsigned long long)same) - 1;
		uint32_t prior = 0;
		if (lane == leader) {
			prior = sc.wave_hist[wave][d];
			sc.wave_hist[wave][d] = (uint16_t)(prior + count);
		}
		prior = __shfl(prior, leader);
		rank[i] = prior + below;
		__builtin_amdgcn_wave_barrier();
	}
	__syncthreads();

	// A thread owns kOwn neighbouring digit values: prefix over the 4 waves, publish the tile's counts.
	const size_t remaining = n - block_base;
	const uint32_t valid = remaining < (size_t)kSortBlock ? (uint32_t)remaining : (uint32_t)kSortBlock;
	uint32_t* const my_word = lookback + (size_t)tile * kBins + kOwn * tid;
	uint32_t count[kOwn], digit_start[kOwn];
	{
		uint32_t mine = 0;
#pragma unroll
		for (int o = 0; o < kOwn; o++) {
			const int d = kOwn * tid + o;
			const uint32_t c0 = sc.wave_hist[0][d], c1 = sc.wave_hist[1][d], c2 = sc.wave_hist[2][d], c3 = sc.wave_hist[3][d];
			sc.wave_hist[0][d] = 0;
			sc.wave_hist[1][d] = (uint16_t)c0;
			sc.wave_hist[2][d] = (uint16_t)(c0 + c1);
			sc.wave_hist[3][d] = (uint16_t)(c0 + c1 + c2);
			count[o] = c0 + c1 + c2 + c3;
			mine += count[o];
		}
		uint32_t total;
		uint32_t ex = block256_exclusive_scan_u32(mine, s_scan, total);
#pragma unroll
		for (int o = 0; o < kOwn; o++) {
			sc.digit_base[kOwn * tid + o] = (uint16_t)ex;
			ex += count[o];
		}
		if (tid == 255)
			count[kOwn - 1] -= (uint32_t)kSortBlock - valid;  // padding is not published
		const uint32_t flag = tile == 0 ? kFlagInclusive : kFlagAggregate;
		if (kOwn == 1) {
			__hip_atomic_store(my_word, count[0] | flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		} else {
			// both counts in one 8-byte store: a reader sees the pair published or not, never one of the two
			__hip_atomic_store(reinterpret_cast<uint64_t*>(my_word),
			                   (uint64_t)(count[0] | flag) | ((uint64_t)(count[kOwn - 1] | flag) << 32), __ATOMIC_RELAXED,
			                   __HIP_MEMORY_SCOPE_AGENT);
		}
		// where the digit's run starts in the whole array: the exclusive scan of the digit counts
		uint32_t all, totals = 0;
#pragma unroll
		for (int o = 0; o < kOwn; o++)
			totals += digit_total[o];
		uint32_t start = block256_exclusive_scan_u32(totals, s_scan, all);
#pragma unroll
		for (int o = 0; o < kOwn; o++) {
			digit_start[o] = start;
			start += digit_total[o];
		}
	}

	// The tile's pairs in digit order, through LDS.  None of this needs the tiles before this one: by the time
	// the look-back below starts, more of them have finished theirs and it has fewer words to read.
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const size_t k = wave_base + (size_t)i * 64 + lane;
		const uint32_t d = (k < n) ? digit_of(key[i], shift, mask) : (uint32_t)(kBins - 1);
		const uint32_t pos = (uint32_t)sc.digit_base[d] + (uint32_t)sc.wave_hist[wave][d] + rank[i];
		s_keys[pos] = key[i];
		s_vals[pos] = val[i];
	}
	__syncthreads();
	// every LDS read of the thread is asked for before anything needs one
	KeyT out_key[kSortItems];
	uint32_t out_val[kSortItems];
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const uint32_t p = (uint32_t)i * 256 + tid;
		const uint32_t q = p < valid ? p : 0u;
		out_key[i] = s_keys[q];
		out_val[i] = s_vals[q];
	}

	// Look back: the pairs of this thread's digit values in all earlier tiles.
	{
		uint32_t exclusive[kOwn];
#pragma unroll
		for (int o = 0; o < kOwn; o++)
			exclusive[o] = 0;
		if (tile != 0) {
			// Words of the tiles below t are still to be added.  Up to kLookBatch of them are requested
			// together: walked one load at a time, the chain of tiles and not memory sets the pace of a pass.
			uint32_t t = tile;
			bool gave_up = spin_limit < 0, done = false;
			while (!gave_up && !done) {
				uint32_t v[kLookBatch][kOwn];
#pragma unroll
				for (int q = 0; q < kLookBatch; q++) {
					const uint32_t* word = lookback + (size_t)(t - 1u - (uint32_t)q) * kBins + kOwn * tid;
					if ((uint32_t)q < t) {
						if (kOwn == 1) {
							v[q][0] = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
						} else {
							const uint64_t both = __hip_atomic_load(reinterpret_cast<const uint64_t*>(word), __ATOMIC_RELAXED,
							                                        __HIP_MEMORY_SCOPE_AGENT);
							v[q][0] = (uint32_t)both;
							v[q][kOwn - 1] = (uint32_t)(both >> 32);
						}
					} else {
#pragma unroll
						for (int o = 0; o < kOwn; o++)
							v[q][o] = kFlagInclusive;  // below the first tile there is nothing
					}
				}
				uint32_t used = 0;
#pragma unroll
				for (int q = 0; q < kLookBatch; q++) {
					// a word counts once every nearer one has been published and none of them closed the sum (a tile's
					// words are published together and carry the same flag, so the first tells for all)
					if (!done && used == (uint32_t)q && (v[q][0] >> 30) != 0u) {
#pragma unroll
						for (int o = 0; o < kOwn; o++)
							exclusive[o] += v[q][o] & kValueMask;
						used = (uint32_t)q + 1u;
						done = (v[q][0] & kFlagInclusive) != 0u;
					}
				}
				t -= used < t ? used : t;
				if (t == 0u)
					done = true;
				if (!done && used < (uint32_t)kLookBatch) {
					// tile t - 1 has not published yet: wait for its word, then look again from there
					const uint32_t* word = lookback + (size_t)(t - 1u) * kBins + kOwn * tid;
					uint32_t w = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					for (int spins = 0; (w >> 30) == 0u; spins++) {
						// give up after a bounded wait, or as soon as any other look-back has
						if (spins >= spin_limit ||
						    ((spins & 255) == 255 &&
						     __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)) {
							gave_up = true;
							break;
						}
						__builtin_amdgcn_s_sleep(1);
						w = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
					}
				}
			}
			if (gave_up)
				atomicOr(status, 1u);
			// On the (never expected) give-up path `exclusive` is too small, which keeps every
			// scatter address inside the array; the status word tells the consumer to discard it.
			if (kOwn == 1) {
				__hip_atomic_store(my_word, ((exclusive[0] + count[0]) & kValueMask) | kFlagInclusive, __ATOMIC_RELAXED,
				                   __HIP_MEMORY_SCOPE_AGENT);
			} else {
				__hip_atomic_store(reinterpret_cast<uint64_t*>(my_word),
				                   (uint64_t)(((exclusive[0] + count[0]) & kValueMask) | kFlagInclusive) |
				                       ((uint64_t)(((exclusive[kOwn - 1] + count[kOwn - 1]) & kValueMask) | kFlagInclusive) << 32),
				                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
#pragma unroll
		for (int o = 0; o < kOwn; o++)
			sc.global_base[kOwn * tid + o] = digit_start[o] + exclusive[o];
	}
	__syncthreads();

	size_t out_at[kSortItems];
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		const uint32_t p = (uint32_t)i * 256 + tid;
		const uint32_t d = digit_of(out_key[i], shift, mask);
		out_at[i] = p < valid ? (size_t)sc.global_base[d] + (p - (uint32_t)sc.digit_base[d]) : n;
	}
	if (kKind != kPassPlain && ends_here) {
		// the sort ends here: a value's index and tile count go to arrays of their own (a count stored as all ones did
		// not fit and is looked up; an index that a sort which gave up left behind may be anything and is clamped)
		const uint32_t index_bits = j.index_bits, cap = 0xFFFFFFFFu >> index_bits, index_mask = (1u << index_bits) - 1u;
#pragma unroll
		for (int i = 0; i < kSortItems; i++) {
			if (out_at[i] < n) {
				const uint32_t index = out_val[i] & index_mask;
				uint32_t c = out_val[i] >> index_bits;
				if (c == cap)
					c = j.count_of[min(index, j.in_size - 1u)];
				j.final_index[out_at[i]] = index;
				j.final_count[out_at[i]] = c;
			}
		}
		return;
	}
#pragma unroll
	for (int i = 0; i < kSortItems; i++) {
		if (out_at[i] < n) {
			keys_out[out_at[i]] = out_key[i];
			vals_out[out_at[i]] = out_val[i];
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

size_t sort_clear_words(size_t n, int end_bit, int max_bits)
{
	const size_t tiles = (n + kSortBlock - 1) / kSortBlock;
	return kSortHeader + (size_t)sort_passes(end_bit, max_bits) * ((size_t)1 << max_bits) * tiles;
}

size_t depth_sort_clear_words(size_t n)
{
	const size_t tiles = (n + kSortBlock - 1) / kSortBlock;
	return kSortHeader + (size_t)(kDepthPasses + 1) * 512 * tiles;
}

template <typename KeyT, int kBits>
static void sort_pairs(const SortJob<KeyT>* jobs, int count, int end_bit, bool temp_cleared, bool histograms_done, bool mark_stages,
                       hipStream_t s)
{
	const int passes = sort_passes(end_bit, kBits);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<SortJob<KeyT>> b = {};
		uint32_t max_tiles = 0;
		int live = 0;
		for (int k = 0; k < nj; k++) {
			const SortJob<KeyT>& j = jobs[at + k];
			if (j.n == 0)
				continue;
			b.job[live++] = j;
			const uint32_t tiles = (uint32_t)((j.n + kSortBlock - 1) / kSortBlock);
			max_tiles = tiles > max_tiles ? tiles : max_tiles;
			if (!temp_cleared)
				launch_fill_u32(j.temp, 0u, sort_clear_words(j.n, end_bit, kBits), s);
		}
		if (live == 0)
			continue;
		if (mark_stages && !histograms_done)
			stage_mark("sort_setup", s);
		// every block ends with an atomic add per digit and pass into its job's counts: a few hundred blocks per
		// job read the keys as fast as thousands would, and queue far fewer adds on the same words
		const uint32_t most_blocks = live >= 8 ? 256u : 2048u / (uint32_t)live;
		const uint32_t hist_blocks = max_tiles < most_blocks ? max_tiles : most_blocks;
		if (!histograms_done) {
			if constexpr (sizeof(KeyT) == 8)
				hipLaunchKernelGGL(sort_digit_histogram_kernel<KeyT>, dim3(hist_blocks, (unsigned)live), dim3(256), 0, s, b, passes, end_bit);
		}
		for (int p = 0; p < passes; p++) {
			const int shift = sort_digit_shift(end_bit, p, kBits);
			const int bits = sort_digit_bits(end_bit, p, kBits);
			const uint32_t mask = (1u << bits) - 1u;
			if (mark_stages)
				stage_mark("sort_onesweep", s);
			hipLaunchKernelGGL((sort_onesweep_kernel<KeyT, kBits, kPassPlain>), dim3(max_tiles, (unsigned)live), dim3(256), 0, s, b, p, shift,
			                   mask, g_lookback_spin_limit.load());
		}
	}
}

void launch_sort_pairs(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                       int end_bit, uint32_t* temp, hipStream_t s)
{
	SortJob<uint64_t> job = {};
	job.keys_in = keys_in; job.keys_out = keys_out; job.vals_in = vals_in; job.vals_out = vals_out;
	job.n = n; job.temp = temp;
	sort_pairs<uint64_t, kDigitBitsU64>(&job, 1, end_bit, false, false, true, s);
}

// The digit counts must come from the kernel that wrote the keys (histograms_done): nothing here reads 32-bit keys for them.
void launch_sort_pairs_u32(const SortJob<uint32_t>* jobs, int count, int end_bit, bool temp_cleared, bool histograms_done,
                           const char* stage, hipStream_t s)
{
	if (sort_max_digit_bits_u32(end_bit) == 9)
		sort_pairs<uint32_t, 9>(jobs, count, end_bit, temp_cleared, histograms_done, stage != nullptr, s);
	else
		sort_pairs<uint32_t, 8>(jobs, count, end_bit, temp_cleared, histograms_done, stage != nullptr, s);
}

void launch_depth_order(const DepthOrderJob* jobs, int count, hipStream_t s)
{
	stage_mark("depth_order", s);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<DepthOrderJob> b = {};
		Batch<BlockScanJob> scan = {};
		Batch<BlockInclusiveJob> inc = {};
		Batch<SortJob<uint32_t>> sorts = {};
		int max_p = 0;
		for (int k = 0; k < nj; k++)
			max_p = jobs[at + k].P > max_p ? jobs[at + k].P : max_p;
		const bool few_groups = ((size_t)max_p + kScanGroup - 1) / kScanGroup <= 4096;
		for (int k = 0; k < nj; k++) {
			const DepthOrderJob& j = jobs[at + k];
			b.job[k] = j;
			SortJob<uint32_t>& sj = sorts.job[k];
			sj.keys_in = j.keys_a; sj.keys_out = j.keys_b; sj.vals_in = j.vals_a; sj.vals_out = j.vals_b;
			sj.n = (size_t)j.P; sj.n_device = j.visible_count; sj.temp = j.sort_temp;
			sj.final_index = j.order; sj.final_count = j.tiles_in_order; sj.count_of = j.tiles_touched;
			sj.index_bits = depth_index_bits((uint32_t)j.P); sj.in_size = (uint32_t)j.P;
			scan.job[k] = BlockScanJob{j.scan_temp, ((size_t)j.P + kScanGroup - 1) / kScanGroup, j.visible_count, (uint32_t)kScanGroup, nullptr, nullptr,
			                           nullptr, nullptr};
			inc.job[k] = BlockInclusiveJob{j.tiles_in_order, j.scan_temp, (size_t)j.P, j.visible_count, j.offsets_in_order, j.dup_first,
			                               (uint32_t)dup_first_words((size_t)j.P), few_groups ? 1u : 0u};
		}
		const dim3 grid((unsigned)((max_p + kScanGroup - 1) / kScanGroup), (unsigned)nj);
		// few workgroups per job, each over many groups: every one ends with an atomic add per digit into its job's counts
		const unsigned most = nj >= 8 ? 256u : 2048u / (unsigned)nj;
		hipLaunchKernelGGL(depth_pairs_kernel, dim3(grid.x < most ? grid.x : most, (unsigned)nj), dim3(256), 0, s, b);
		// three passes of nine bits (a -> b -> a -> the order and the tile counts in that order), and the pass on demand
		const dim3 tiles((unsigned)((max_p + kSortBlock - 1) / kSortBlock), (unsigned)nj);
		const int spin = g_lookback_spin_limit.load();
		hipLaunchKernelGGL((sort_onesweep_kernel<uint32_t, 9, kPassPlain>), tiles, dim3(256), 0, s, sorts, 0, 0, 511u, spin);
		hipLaunchKernelGGL((sort_onesweep_kernel<uint32_t, 9, kPassPlain>), tiles, dim3(256), 0, s, sorts, 1, 9, 511u, spin);
		hipLaunchKernelGGL((sort_onesweep_kernel<uint32_t, 9, kPassEndsUnless>), tiles, dim3(256), 0, s, sorts, 2, 18, 511u, spin);
		hipLaunchKernelGGL((sort_onesweep_kernel<uint32_t, 9, kPassOnDemand>), tiles, dim3(256), 0, s, sorts, 3, kDepthKeyBits, 31u, spin);
		hipLaunchKernelGGL(order_totals_kernel, grid, dim3(256), 0, s, b);
		if (!few_groups)
			hipLaunchKernelGGL(single_block_exclusive_scan_kernel, dim3(1, (unsigned)nj), dim3(1024), 0, s, scan);
		hipLaunchKernelGGL(block_inclusive_scan_kernel<4>, grid, dim3(256), 0, s, inc);
	}
}

// Sets n words to v, 16 bytes per store where the address allows; a capped grid walks the array.
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t v, size_t n)
{
	const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, threads = (size_t)gridDim.x * 256;
	// words up to the first 16-byte boundary, whole 16-byte groups, the rest
	const size_t head = min(n, (size_t)((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / 4);
	const size_t groups = (n - head) / 4;
	if (tid < head)
		p[tid] = v;
	uint4* q = reinterpret_cast<uint4*>(p + head);
	const uint4 vv = {v, v, v, v};
	for (size_t g = tid; g < groups; g += threads)
		q[g] = vv;
	const size_t done = head + 4 * groups;
	if (tid < n - done)
		p[done + tid] = v;
}

// The same for several arrays in one launch (the array in blockIdx.y).
__global__ __launch_bounds__(256) void fill_many_kernel(Batch<FillJob> batch, uint32_t v)
{
	uint32_t* __restrict__ p = batch.job[blockIdx.y].p;
	const size_t n = batch.job[blockIdx.y].n;
	const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, threads = (size_t)gridDim.x * 256;
	const size_t head = min(n, (size_t)((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / 4);
	const size_t groups = (n - head) / 4;
	if (tid < head)
		p[tid] = v;
	uint4* q = reinterpret_cast<uint4*>(p + head);
	const uint4 vv = {v, v, v, v};
	for (size_t g = tid; g < groups; g += threads)
		q[g] = vv;
	const size_t done = head + 4 * groups;
	if (tid < n - done)
		p[done + tid] = v;
}

void launch_fill_many(const FillJob* jobs, int count, uint32_t v, hipStream_t s)
{
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<FillJob> b = {};
		size_t most = 0;
		for (int k = 0; k < nj; k++) {
			b.job[k] = jobs[at + k];
			most = b.job[k].n > most ? b.job[k].n : most;
		}
		if (most == 0)
			continue;
		const size_t blocks = (most / 4 + 255) / 256 + 1, cap = 4096 / (size_t)nj + 1;
		hipLaunchKernelGGL(fill_many_kernel, dim3((unsigned)(blocks < cap ? blocks : cap), (unsigned)nj), dim3(256), 0, s, b, v);
	}
}

void launch_fill_u32(uint32_t* p, uint32_t v, size_t n, hipStream_t s)
{
	if (n == 0)
		return;
	const size_t blocks = (n / 4 + 255) / 256 + 1;
	hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0, s, p, v, n);
}

// The status words (may be null) are those of the two sorts: if either reported a failure the
// ranges stay empty, so no later stage walks an unsorted list, and *fault (host memory that the
// device can write, may be null) is set for the host to find.  The keys carry strip bits above the
// tile (key_strips); per workgroup of kFileGroup keys (four neighbouring keys per thread), file_tail
// (may be null) receives how many keys of the tile of its last key have each of the four "filed" bits
// set, which is what the kernel that places the entries in their strips' lists needs from the
// workgroups ahead of its own.
__global__ __launch_bounds__(kFileBlock) void tile_ranges_kernel(Batch<TileRangesJob> batch)
{
	__shared__ uint2 s_tail[4];  // per wave, the four strips' counts packed 16 bits each
	__shared__ uint32_t s_last_tile;
	const TileRangesJob& j = batch.job[blockIdx.y];
	const uint32_t* __restrict__ keys = j.keys;
	size_t n = j.n;
	const uint32_t* __restrict__ n_device = j.n_device;
	uint2* __restrict__ ranges = j.ranges;
	const uint32_t* __restrict__ sort_status = j.sort_status;
	const uint32_t* __restrict__ order_status = j.order_status;
	uint32_t* __restrict__ fault = j.fault;
	uint4* __restrict__ file_tail = j.file_tail;
	const size_t first = (size_t)blockIdx.x * kFileGroup;
	if (first >= j.n)
		return;  // the launch is sized for the job with the most keys
	if (blockIdx.x == 0 && j.rezero)  // the sort has read its digit counts: zero again for the next to count into them
		for (int w = threadIdx.x; w < kTileDigitWords; w += kFileBlock)
			j.rezero[w] = 0u;
	if ((sort_status && *sort_status != 0u) || (order_status && *order_status != 0u)) {
		if (blockIdx.x == 0 && threadIdx.x == 0 && fault)
			__hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		return;
	}
	if (n_device)
		n = min(n, (size_t)*n_device);  // launched for an upper bound
	if (first >= n)
		return;
	const size_t idx0 = first + 4 * (size_t)threadIdx.x;
	uint32_t key[4] = {0u, 0u, 0u, 0u};
	if (idx0 + 3 < n) {
		const uint4 k4 = *reinterpret_cast<const uint4*>(keys + idx0);
		key[0] = k4.x; key[1] = k4.y; key[2] = k4.z; key[3] = k4.w;
	} else {
#pragma unroll
		for (int q = 0; q < 4; q++)
			if (idx0 + q < n)
				key[q] = keys[idx0 + q];
	}
	uint32_t prev = (idx0 > 0 && idx0 < n) ? key_tile(keys[idx0 - 1]) : 0u;
	const size_t last = min(n, first + kFileGroup) - 1;
#pragma unroll
	for (int q = 0; q < 4; q++) {
		const size_t idx = idx0 + q;
		const uint32_t cur = key_tile(key[q]);
		if (idx < n) {
			if (idx == 0) {
				ranges[cur].x = 0;
			} else if (cur != prev) {
				ranges[prev].y = (uint32_t)idx;
				ranges[cur].x = (uint32_t)idx;
			}
			if (idx == n - 1)
				ranges[cur].y = (uint32_t)n;
			if (idx == last)
				s_last_tile = cur;
		}
		prev = cur;
	}
	if (!file_tail)
		return;
	__syncthreads();
	const uint32_t last_tile = s_last_tile;
	uint2 own = {0u, 0u};
#pragma unroll
	for (int q = 0; q < 4; q++)
		if (idx0 + q < n && key_tile(key[q]) == last_tile) {  // sorted: these are the workgroup's last keys
			const uint32_t bits = key_strips(key[q]);
			own.x += (bits & 1u) | ((bits & 2u) << 15);
			own.y += ((bits >> 2) & 1u) | ((bits & 8u) << 13);
		}
	const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
	const uint2 inc = {wave_inclusive_scan_u32(own.x), wave_inclusive_scan_u32(own.y)};
	if (lane == 63)
		s_tail[wave] = inc;
	__syncthreads();
	if (threadIdx.x == 0) {
		const uint32_t x = s_tail[0].x + s_tail[1].x + s_tail[2].x + s_tail[3].x;
		const uint32_t y = s_tail[0].y + s_tail[1].y + s_tail[2].y + s_tail[3].y;
		file_tail[blockIdx.x] = uint4{x & 0xFFFFu, x >> 16, y & 0xFFFFu, y >> 16};
	}
}

__global__ void report_sort_status_kernel(const uint32_t* __restrict__ status, uint32_t* __restrict__ fault,
                                          uint32_t* __restrict__ device_fault)
{
	if (threadIdx.x == 0 && *status != 0u) {
		if (fault)
			__hip_atomic_store(fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		if (device_fault)
			*device_fault = 1u;
	}
}

void launch_report_sort_status(const uint32_t* temp, uint32_t* fault, uint32_t* device_fault, hipStream_t s)
{
	if (fault || device_fault)
		hipLaunchKernelGGL(report_sort_status_kernel, dim3(1), dim3(64), 0, s, temp + kSortStatus, fault, device_fault);
}

void launch_tile_ranges(const TileRangesJob* jobs, int count, hipStream_t s)
{
	stage_mark("tile_ranges", s);
	for (int at = 0; at < count; at += kMaxBatch) {
		const int nj = count - at < kMaxBatch ? count - at : kMaxBatch;
		Batch<TileRangesJob> b = {};
		size_t max_n = 0;
		int live = 0;
		for (int k = 0; k < nj; k++) {
			if (jobs[at + k].n == 0)
				continue;
			b.job[live++] = jobs[at + k];
			max_n = jobs[at + k].n > max_n ? jobs[at + k].n : max_n;
		}
		if (live)
			hipLaunchKernelGGL(tile_ranges_kernel, dim3((unsigned)((max_n + kFileGroup - 1) / kFileGroup), (unsigned)live),
			                   dim3(kFileBlock), 0, s, b);
	}
}

}  // namespace rgs
