// Argument blocks and launcher prototypes shared between the kernel files and the
// C-ABI layer.  All pointers are device pointers unless a comment says otherwise.
#pragma once
#include "rgs_device.h"

namespace rgs {

constexpr int kMaxComposite = 64;  // most partial images one composite call can take

// Jobs of one launch: kernels that run once per submodel take the submodels of a frame together, the job in
// blockIdx.y; the arguments travel by value.  More jobs than kMaxBatch take several launches.  16 of the largest
// job (248 bytes) stay inside the 4096 bytes a launch can carry.
constexpr int kMaxBatch = 16;
template <typename T>
struct Batch {
	T job[kMaxBatch];
};

struct PreprocessArgs {
	int P, D, M;
	const float* means;
	const float* scales;
	float scale_modifier;
	const float* rotations;
	const float* opacities;
	const float* shs;
	const float* cov3D_precomp;   // may be null
	const float* colors_precomp;  // may be null
	const float* view;
	const float* proj;
	const float* campos;
	int W, H;
	float tanfovx, tanfovy, focal_x, focal_y;
	int grid_x, grid_y;
	// outputs
	int* radii;
	float* depths;
	uint32_t* tiles_touched;
	uint8_t* clamped;
	uint32_t* block_sums;  // one per 256 Gaussians
	uint32_t* block_visible;  // one per 256 Gaussians: how many of them touch a tile
	bool sh_rows_by_16_bytes; // SH rows are 16-byte aligned, a multiple of 16 bytes long and at most 48 floats
	uint32_t* clear;          // clear_words words that the kernel sets to zero for a later stage
	size_t clear_words;
	float4* blend_record;  // 4 float4 per Gaussian, see blend.hip
};

struct PreprocessBackwardArgs {
	int P, D, M;
	const float* means;
	const int* radii;
	const float* shs;      // may be null
	const uint8_t* clamped;
	const float* scales;   // may be null
	const float* rotations;
	float scale_modifier;
	const float* cov3D_precomp;  // may be null: then the 3D covariance is computed from scale and rotation, as the forward did
	const float* view;
	const float* proj;
	const float* campos;
	float focal_x, focal_y, tanfovx, tanfovy;
	const float* sums;  // (P, kSumCols): what the backward blend accumulated, see SumCol
	bool sh_rows_by_16_bytes;       // SH rows are 16-byte aligned, a multiple of 16 bytes long and at most 48 floats
	// outputs: every row is written, zeros where radii[i] <= 0
	float* dL_dmean2D;  // (P,3), third column 0
	float* dL_dopacity; // (P)
	float* dL_dcolor;   // (P,3)
	float* dL_dmeans;   // (P,3)
	float* dL_dcov3D;   // (P,6)
	float* dL_dsh;      // (P,M,3)
	float* dL_dscale;   // (P,3)
	float* dL_drot;     // (P,4)
};

struct BlendArgs {
	const uint2* ranges;
	const uint32_t* point_list;
	int W, H, grid_x, grid_y;
	float tanfovx, tanfovy;
	const float* projinv;
	const float* range_low;
	const float* range_up;
	const float* bg;
	const float4* record;  // 4 float4 per Gaussian: everything the blend reads of it
	// forward outputs / backward inputs
	float* out_color;
	float* out_depth;
	float* out_alpha;
	uint32_t* n_contrib;
	uint32_t* strip_lists;  // 4 R words: for strip s of a tile whose list is [x, x + n), the entries filed
	                        // for it, at 4 x + s n: list position, bit 31 = strip inside the box
	uint32_t* strip_total;  // per 16x4 strip (tile * 4 + strip): how many entries are filed for it; zero before the filing
	uint32_t* strip_filed;  // per strip: how many of them the backward walks, i.e. up to the last one blended
	const uint32_t* tile_keys;    // the sorted key of every list position: tile and strip bits (key_tile, key_strips)
	const uint32_t* count_device; // non-null: the number of instances is min(capacity, *count_device)
	uint32_t capacity;      // instances the launch is sized for
	uint32_t gaussians;     // P: the records there are
	const uint4* file_tail; // per kFileGroup list positions: entries filed per strip for the tile of the last of them
	const uint32_t* sort_status;   // status words of the two sorts (may be null): non-zero = the sort gave up
	const uint32_t* order_status;
	uint32_t* strip_order;  // strips by decreasing strip_filed, written behind the forward blend
	uint32_t* strip_order_forward;  // strips by decreasing strip_total, written ahead of the forward blend
	uint32_t* strip_classes;  // 4 x 256 words, zero before the forward blend: strips per class and placement cursors,
	                          // for strip_order and then for strip_order_forward
	uint64_t* counters;  // non-null selects the work-accounting twin of the forward blend (7 sums)
	// backward
	const float* dL_dpix;
	const float* dL_dpix_depth;
	const float* dL_dalpha;
	float* sums;  // (P, kSumCols), cleared by the caller; the blend adds into it atomically
};

// Columns of a Gaussian's row of gradient sums.  One row is 48 bytes, so the (up to) ten atomic
// adds that a wavefront issues for a Gaussian fall into one or two cache lines.
enum SumCol {
	kSumMeanX = 0, kSumMeanY = 1, kSumConicXX = 2, kSumConicXY = 3,
	kSumConicYY = 4, kSumOpacity = 5, kSumR = 6, kSumG = 7,
	kSumB = 8, kSumDepth = 9, kSumCols = 12
};

struct CompositeArgs {
	int K, H, W;
	const float* bg;  // may be null (black)
	const float* images[kMaxComposite];
	const float* depths[kMaxComposite];
	const float* alphas[kMaxComposite];
	float* out_image;
	float* out_depth;
	float* out_alpha;
	// backward
	const float* g_image;
	const float* g_depth;  // may be null
	const float* g_alpha;  // may be null
	float* d_images[kMaxComposite];
	float* d_depths[kMaxComposite];
	float* d_alphas[kMaxComposite];
};

// Boundary straddlers (sharing.hip).  Boxes are passed by value: at most kMaxShareBoxes per launch.
constexpr int kMaxShareBoxes = 64;
struct ShareBoxes {
	float low[kMaxShareBoxes][3];
	float up[kMaxShareBoxes][3];
	int count;
};
struct StraddlerSelectArgs {
	int n;
	const float* means3D;   // (n,3)
	const float* scales;    // (n,3) activated
	float src_low[3], src_up[3];
	ShareBoxes boxes;       // destinations
	int skip;               // index of a destination that is never lent to (the source itself), or -1
	uint32_t* block_counts; // boxes.count x straddler_select_blocks(n) words of scratch
	uint32_t* counts;       // boxes.count
	uint32_t* rows;         // boxes.count x capacity; rows beyond capacity are counted, not stored
	uint32_t capacity;
};
constexpr int kMaxMergeSegments = 32;
struct MergeSegment {
	const float* means3D;
	const float* opacity;
	const float* scales;
	const float* rotations;
	const float* shs;
	const uint32_t* rows;   // null: rows 0..count-1 of the source
	uint32_t count, dst_row0, block0;
};
struct MergeArgs {
	MergeSegment seg[kMaxMergeSegments];
	int segments;
	int sh_floats;
	float* means3D;
	float* opacity;
	float* scales;
	float* rotations;
	float* shs;
};
struct MergeBackwardSegment {
	float* means3D;
	float* means2D;
	float* opacity;
	float* scales;
	float* rotations;
	float* shs;
	const uint32_t* rows;
	uint32_t count, dst_row0, block0;
};
struct MergeBackwardArgs {
	MergeBackwardSegment seg[kMaxMergeSegments];
	int segments;
	int sh_floats;
	const float* means3D;   // gradients of the merged arrays; any may be null
	const float* means2D;
	const float* opacity;
	const float* scales;
	const float* rotations;
	const float* shs;
};

// Image loss and optimiser step (training.hip).
struct LossArgs {
	int C, H, W;
	const float* x;          // rendered image (C,H,W)
	const float* y;          // ground truth
	float w[11];             // normalised 1-D Gaussian window
	float lambda;            // weight of (1 - SSIM)
	float* maps;             // 3 x C x H x W derivative maps (may be null in the forward: no backward will follow)
	float* partial;          // 2 floats per workgroup
	float* out;              // loss, L1, SSIM
	const float* grad_loss;  // backward: upstream gradient of the loss (device scalar) or null for 1
	float* d_image;          // backward: gradient of the loss with respect to x
};
struct ActivateArgs {
	int n, rest;                 // Gaussians; SH coefficients beyond the first (15 at degree 3)
	const float* features_dc;    // (n,1,3)
	const float* features_rest;  // (n,rest,3)
	const float* scaling;        // (n,3) log of the scales
	const float* rotation;       // (n,4) as stored
	const float* opacity;        // (n,1) logit
	float* shs;                  // (n,1+rest,3)
	float* scales;
	float* rotations;
	float* opacities;
};
struct ActivateBackwardArgs {
	int n, rest;
	const float* rotation;       // stored quaternions
	const float* scales;         // activated values, as the forward wrote them
	const float* opacities;
	const float* g_shs;          // gradients of the activated tensors; any may be null (that output is left alone)
	const float* g_scales;
	const float* g_rotations;
	const float* g_opacities;
	float* d_features_dc;
	float* d_features_rest;
	float* d_scaling;
	float* d_rotation;
	float* d_opacity;
};
constexpr int kMaxAdamTensors = 16;
struct AdamTensor {
	float* param;
	const float* grad;
	float* exp_avg;
	float* exp_avg_sq;
	size_t n;
	float step_size;         // lr / (1 - beta1^t)
	float bias2_sqrt;        // sqrt(1 - beta2^t)
	uint32_t block0;
	int by_16_bytes;
};
struct AdamArgs {
	AdamTensor t[kMaxAdamTensors];
	int tensors;
	float beta1, beta2, eps;
	float one_minus_beta1, one_minus_beta2;   // formed in double by the host
};

// An instance's sort key: the tile in the low kKeyTileBits bits (all the sort looks at) and above them
// what strip_filing.h decides for the four strips of that tile: bits 0-3 filed, bits 4-7 inside the box.
constexpr int kKeyTileBits = 24;
__host__ __device__ inline uint32_t key_tile(uint32_t key) { return key & ((1u << kKeyTileBits) - 1u); }
__host__ __device__ inline uint32_t key_strips(uint32_t key) { return key >> kKeyTileBits; }
constexpr int kFileBlock = 256;   // threads of a workgroup of the kernels that file entries for strips
constexpr int kFileGroup = 1024;  // list positions such a workgroup takes, four neighbouring ones per thread

// What the key duplication needs to decide the strips: the packed records and the submodel box test's frame.
struct FilingArgs {
	const float4* record;      // 4 float4 per Gaussian: pixel centre, conic, ellipse extents and the integer radius among them
	const float* projinv;
	const float* range_low;
	const float* range_up;
	float tanfovx, tanfovy;
	int W, H;
};

// preprocess.hip
void launch_mark_visible(int P, const float* means, const float* view, uint8_t* present, hipStream_t s);
void launch_covariance3d(int P, const float* scales, float scale_modifier, const float* rotations, float* cov3D, hipStream_t s);
// `jobs` are host arrays: the submodels of a frame in one launch (kMaxBatch of them at a time).
void launch_preprocess_forward(const PreprocessArgs* jobs, int count, hipStream_t s);
// Writes every row of the output arrays (zeros for Gaussians that were not rendered).
void launch_preprocess_backward(const PreprocessBackwardArgs* jobs, int count, hipStream_t s);

// binning.hip
// A sort on the lowest end_bit bits of its keys takes ceil(end_bit / max_bits) passes, max_bits being the widest digit
// its kernel handles (kDigitBitsU32 for 32-bit keys, kDigitBitsU64 for 64-bit ones); the bits are shared out evenly
// between the passes, the wider digits first (13 bits: 7 then 6, not 9 then 4: the fewer values a digit has, the longer
// the runs of neighbouring keys a pass writes).
constexpr int kDigitBitsU32 = 9;   // 512 digit values: the 17 tile bits of a 5185x3359 image in two passes, 27 depth bits in three
constexpr int kDigitBitsU64 = 8;
// The widest digit the sort of 32-bit keys on end_bit bits uses: 9 bits where that saves a pass, 8 otherwise (a pass
// over 512 digit values writes shorter runs and was measured 14 % slower than one over 256).
__host__ __device__ inline int sort_max_digit_bits_u32(int end_bit)
{
	return (end_bit + 8) / 9 < (end_bit + 7) / 8 ? 9 : 8;
}
__host__ __device__ inline int sort_passes(int end_bit, int max_bits)
{
	return (end_bit + max_bits - 1) / max_bits;
}
__host__ __device__ inline int sort_digit_bits(int end_bit, int p, int max_bits)
{
	const int n = sort_passes(end_bit, max_bits);
	return end_bit / n + (p < end_bit % n ? 1 : 0);
}
__host__ __device__ inline int sort_digit_shift(int end_bit, int p, int max_bits)
{
	const int n = sort_passes(end_bit, max_bits);
	return p * (end_bit / n) + (p < end_bit % n ? p : end_bit % n);
}
constexpr int kSortItems = 16;                    // keys per thread in one sort block
constexpr int kSortBlock = 256 * kSortItems;      // keys per sort block
size_t scan_temp_words(size_t n);                 // u32 words of scratch for launch_inclusive_sum
// `stage` (may be null) names the stage for the timing aid.
void launch_inclusive_sum(const uint32_t* in, uint32_t* out, size_t n, uint32_t* temp, const char* stage,
                          hipStream_t s);
// Scans the per-256 block sums of the tile counts and of the visible flags in place;
// *total_out (and *total_copy, if non-null) = number of instances, *visible_count = number of Gaussians that touch a tile.
struct TotalsJob {
	uint32_t* block_sums;
	uint32_t* block_visible;
	int P;
	uint32_t* total_out;
	uint32_t* total_copy;
	uint32_t* visible_count;
};
void launch_totals_from_block_sums(const TotalsJob* jobs, int count, hipStream_t s);
// Depth order of the Gaussians that touch a tile.  block_visible holds the exclusive scan of
// their count per 256 Gaussians and *visible_count the total; sort_temp has been cleared
// (sort_clear_words(P, 32) words).  On return order[0..count)
// lists them by increasing depth, ties by index, and offsets_in_order is the inclusive scan of
// their tile counts in that order.  The count stays on the device: every kernel is launched
// for P elements and reads it.
struct DepthOrderJob {
	int P;
	const float* depths;
	const uint32_t* tiles_touched;
	uint32_t* block_visible;
	uint32_t* visible_count;
	uint32_t* keys_a;
	uint32_t* keys_b;
	uint32_t* vals_a;
	uint32_t* order;
	uint32_t* vals_b;
	uint32_t* tiles_in_order;
	uint32_t* offsets_in_order;
	uint32_t* sort_temp;
	uint32_t* scan_temp;
	uint32_t* dup_first;       // dup_first_words(P) words: see launch_duplicate_with_keys
	uint32_t* tile_digits;     // kTileDigitWords words, left zero: see DuplicateJob
};
void launch_depth_order(const DepthOrderJob* jobs, int count, hipStream_t s);
// Also sets clear[0..clear_words) to zero (the scratch of the sort that follows).  Instances whose
// position is `capacity` or more are not written.
// Output positions a workgroup of the key duplication writes, and the table that tells each such workgroup at
// which Gaussian (of the depth order) its positions begin: entry b = the Gaussian whose instances include position
// b * kDupPositions.  The scan that produces the offsets fills it; it has room for dup_first_words(P) workgroups,
// those beyond (more than 16 instances per Gaussian on average) search the offsets instead.  One position per thread:
// with 1 024 positions (four per thread) the kernel held 117 registers and 4 wavefronts per SIMD; with 256 it holds
// 79 and 6, and is 22 % faster where the Gaussians are small.
constexpr int kDupPositions = 256;
constexpr size_t dup_first_words(size_t P) { return P / 16 + 2; }
// The key duplication also counts the digits of the tiles it writes, which is what the sort of its keys starts
// from: counts[512 p + d] = keys whose digit p of the tile bits (sort_digit_shift / sort_digit_bits with
// sort_max_digit_bits_u32(end_bit)) is d, in kTileDigitWords words that are zero when it starts (the depth order leaves them so, and so does the
// tile-range kernel, the last to run after they were read).
constexpr int kTileDigitWords = 3 * 512;  // tiles have at most 24 bits: three passes at most
struct DuplicateJob {
	int P;
	const uint32_t* visible_count;
	const uint32_t* order;
	const uint32_t* offsets;   // inclusive, in depth order
	const uint32_t* total;     // the last of them
	const uint32_t* first_of_block;  // dup_first_words(P) words
	uint32_t* tile_digits;     // kTileDigitWords words, zero beforehand
	int end_bit;               // bits of the tile the sort will look at
	uint32_t* also_clear;      // a second array to clear (the tile ranges and what lies behind them)
	size_t also_clear_words;
	FilingArgs filing;
	uint32_t* keys;
	uint32_t* values;
	uint32_t capacity;
	uint32_t* clear;
	size_t clear_words;
};
void launch_duplicate_with_keys(const DuplicateJob* jobs, int count, int grid_x, int grid_y, hipStream_t s);
// words of the sort scratch that must be zero before a sort on end_bit bits with digits of at most max_bits bits
size_t sort_clear_words(size_t n, int end_bit, int max_bits);
size_t depth_sort_clear_words(size_t n);          // the same for the depth sort of launch_depth_order
// The scratch has room for 2048 digit counts and as many look-back words per tile of kSortBlock pairs: 8 passes of 256
// digit values (64-bit keys) or 4 passes of 512 (32-bit keys).
constexpr uint32_t kSortScratchPerTile = 2048;
constexpr uint32_t kSortHeader = 2112;            // words ahead of the look-back words: histograms, counters, status
constexpr size_t sort_temp_words_for(size_t n)
{
	return kSortHeader + (size_t)kSortScratchPerTile * ((n + kSortBlock - 1) / kSortBlock > 0 ? (n + kSortBlock - 1) / kSortBlock : 1);
}
size_t sort_temp_words(size_t n);                 // u32 words of scratch for launch_sort_pairs* (= sort_temp_words_for)
// Stable LSD radix sort on key bits [0, end_bit), sort_passes(end_bit, kDigitBitsU64) passes that ping-pong between
// the two buffer pairs starting in -> out: an odd pass count leaves the result in
// keys_out/vals_out, an even one in keys_in/vals_in.
void launch_sort_pairs(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                       int end_bit, uint32_t* temp, hipStream_t s);
// One sort of a batch.  With a non-null n_device the number of pairs is min(n, *n_device), read by the kernels, and
// `n` is only its upper bound (grids and scratch are sized for it).  also_clear: an array the first kernel sets to
// zero on the way (for a later stage), or null.
template <typename KeyT>
struct SortJob {
	KeyT* keys_in;
	KeyT* keys_out;
	uint32_t* vals_in;
	uint32_t* vals_out;
	size_t n;
	const uint32_t* n_device;
	uint32_t* temp;
	uint32_t* also_clear;
	size_t also_clear_words;
	const uint32_t* digit_counts;  // null: the counts are at the start of temp
	// Only for the passes that end the depth sort (launch_depth_order): the values are a Gaussian's index in the low
	// index_bits bits and above them its tile count (all ones: too large to fit, look it up in count_of); the last pass
	// writes index and count apart, to final_index and final_count, instead of keys and values.
	uint32_t* final_index;
	uint32_t* final_count;
	const uint32_t* count_of;      // tile count of every Gaussian, in_size of them
	uint32_t index_bits, in_size;
};
// The same for 32-bit keys (sort_passes(end_bit, sort_max_digit_bits_u32(end_bit)) passes), every job in one launch per
// kernel; with a null `stage` its kernels are not marked for the timing aid.  temp_cleared: the caller has cleared
// sort_clear_words(n, end_bit, sort_max_digit_bits_u32(end_bit)) words of every temp already.  histograms_done: the kernel that wrote keys_in
// has also added every key's digits to the counts (counts[512 p + d] = keys whose digit p is d), so the sort need not
// read the keys for that.
void launch_sort_pairs_u32(const SortJob<uint32_t>* jobs, int count, int end_bit, bool temp_cleared, bool histograms_done,
                           const char* stage, hipStream_t s);
const uint32_t* sort_status_word(const uint32_t* temp);  // non-zero after a failed sort (never expected)
// Polls a look-back allows before it gives up (0 restores the default; negative: give up at once,
// which is how a test exercises the give-up path with every kernel still running to its end).
void set_lookback_spin_limit(int polls);
// Sets *fault (host memory the device can write, may be null) and *device_fault (device memory, may be null) if the sort
// that used `temp` gave up; with both null nothing is launched.
void launch_report_sort_status(const uint32_t* temp, uint32_t* fault, uint32_t* device_fault, hipStream_t s);
// The tile ranges from the sorted keys.  Either status word (may be null) being non-zero leaves every range empty
// and sets *fault (host memory the device can write, may be null).  The caller has cleared `ranges`.  With a non-null
// n_device the number of keys is min(n, *n_device) and the launch is sized for n.  file_tail (may be null)
// receives, per kFileGroup keys, how many entries of the tile of the last of them have each strip bit set.
constexpr int kRangeTailWords = 1024;   // words behind the ranges: the strip class counters of the blend
struct TileRangesJob {
	const uint32_t* keys;
	size_t n;
	const uint32_t* n_device;
	uint2* ranges;
	const uint32_t* sort_status;
	const uint32_t* order_status;
	uint32_t* fault;
	uint4* file_tail;
	uint32_t* rezero;  // may be null: kTileDigitWords words set to zero (the digit counts the sort has read)
};
void launch_tile_ranges(const TileRangesJob* jobs, int count, hipStream_t s);

// blend.hip
constexpr int kMaxBlendBatch = 16;   // jobs one launch of a blend kernel can take (their arguments travel by value)
struct BlendBatch {
	BlendArgs job[kMaxBlendBatch];
	int count;
};
void launch_strip_filing(const BlendArgs* jobs, int count, hipStream_t s);   // the per-strip lists, from the sorted keys' strip bits
// `jobs` (host array) share one image size; more than kMaxBlendBatch take several launches.
void launch_blend_forward(const BlendArgs* jobs, int count, hipStream_t s);
void launch_blend_backward(const BlendArgs* jobs, int count, hipStream_t s);
void launch_blend_count(const BlendArgs& a, hipStream_t s);    // the work-accounting twin of the forward (a.counters)

// composite.hip
void launch_composite_forward(const CompositeArgs& a, hipStream_t s);
void launch_composite_backward(const CompositeArgs& a, hipStream_t s);
void launch_fill_u32(uint32_t* p, uint32_t v, size_t n, hipStream_t s);
struct FillJob {
	uint32_t* p;
	size_t n;  // words
};
void launch_fill_many(const FillJob* jobs, int count, uint32_t v, hipStream_t s);  // every array in one launch

// sharing.hip
uint32_t straddler_select_blocks(int n);
void launch_straddler_select(const StraddlerSelectArgs& a, hipStream_t s);
uint32_t merge_blocks_for(uint32_t rows);   // workgroups one segment of that many rows takes
void launch_merge_rows(const MergeArgs& a, uint32_t blocks, bool by_16_bytes, hipStream_t s);
void launch_merge_rows_backward(const MergeBackwardArgs& a, uint32_t blocks, bool by_16_bytes, hipStream_t s);

// training.hip
uint32_t loss_blocks(int C, int H, int W);   // workgroups of the loss kernels = pairs of partial sums
void launch_l1_ssim_forward(const LossArgs& a, hipStream_t s);
void launch_l1_ssim_backward(const LossArgs& a, hipStream_t s);
void launch_activate_forward(const ActivateArgs& a, hipStream_t s);
void launch_activate_backward(const ActivateBackwardArgs& a, hipStream_t s);
uint32_t adam_blocks_for(size_t n);
void launch_adam_step(const AdamArgs& a, uint32_t blocks, hipStream_t s);

// api.hip: optional stage timing.  A mark names the work launched after it.
void stage_mark(const char* name, hipStream_t s);

}  // namespace rgs
