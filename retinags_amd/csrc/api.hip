// extern "C" surface of librgs_gfx950.so: argument checks, workspace carving, stage
// sequencing and error reporting.  The declarations and the reference interfaces they
// replace are in include/rgs.h.
#include "../../include/rgs.h"
#include "rgs_kernels.h"

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

// Scratch of rgs_sort_pairs_static, the entry point that allocates nothing: digit histograms, tile
// counters and look-back words of a sort of up to RGS_STATIC_SORT_MAX_PAIRS pairs.  Every device the
// library runs on holds its own copy until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress; the address the kernels get is looked up once per device (static_sort_scratch).
constexpr size_t kStaticSortWords = rgs::sort_temp_words_for(RGS_STATIC_SORT_MAX_PAIRS);
static __device__ __align__(256) uint32_t scratch[kStaticSortWords];
// Set (and left set until rgs_sort_fault has read it) when a sort of rgs_sort_pairs_static gave up: that entry point may
// not allocate the pinned word the other sorts report through, so its report lives in device memory like its scratch.
static __device__ __align__(256) uint32_t scratch_sort_gave_up[64];

namespace {

thread_local char g_error[512] = "";

int fail(const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
	return 1;
}

#define RGS_REQUIRE(cond, ...)          \
	do {                                \
		if (!(cond))                    \
			return fail(__VA_ARGS__);   \
	} while (0)

// Launch errors are cheap to poll; in debug mode every stage is also synchronised, which
// is where the reference's CHECK_CUDA does its cudaDeviceSynchronize.
int check_stage(const char* stage, hipStream_t s, int debug)
{
	hipError_t e = hipGetLastError();
	if (e == hipSuccess && debug)
		e = hipStreamSynchronize(s);
	if (e != hipSuccess)
		return fail("%s: %s", stage, hipGetErrorString(e));
	return 0;
}

#define RGS_STAGE(name)                               \
	do {                                              \
		if (int rc_ = check_stage(name, s, debug))    \
			return rc_;                               \
	} while (0)

// ---- optional stage timing -------------------------------------------------------------
// While enabled, every launcher records a HIP event on the caller's stream before its kernel
// (rgs::stage_mark) and every entry point records one when it has queued its last kernel.
// The time between two consecutive events is charged to the earlier event's stage.
// The record is one per process.  Entry points may be called from several host threads: the switch is atomic (it is all
// a call looks at while recording is off) and the record itself is taken under a lock, so concurrent calls cannot
// corrupt it; what they record still interleaves, which is why measurements are made from one thread.
struct StageTimer {
	std::atomic<bool> on{false};
	std::mutex lock;
	std::vector<hipEvent_t> pool;
	std::vector<const char*> tags;  // tag of event i; nullptr closes an entry point
	size_t used = 0;
};
StageTimer g_timer;
constexpr size_t kMaxTimerEvents = 1 << 16;

void timer_record(const char* tag, hipStream_t s)
{
	if (!g_timer.on.load(std::memory_order_relaxed))
		return;
	std::lock_guard<std::mutex> hold(g_timer.lock);
	if (g_timer.used >= kMaxTimerEvents)
		return;
	if (g_timer.used == g_timer.pool.size()) {
		hipEvent_t e;
		if (hipEventCreate(&e) != hipSuccess)
			return;
		g_timer.pool.push_back(e);
		g_timer.tags.push_back(nullptr);
	}
	g_timer.tags[g_timer.used] = tag;
	if (hipEventRecord(g_timer.pool[g_timer.used], s) == hipSuccess)
		g_timer.used++;
}

struct EntryScope {
	hipStream_t s;
	explicit EntryScope(hipStream_t stream) : s(stream) {}
	~EntryScope() { timer_record(nullptr, s); }
};

// ---- sticky report of a sort that gave up ------------------------------------------------------
// One word of pinned host memory per device, which the device can write: the kernel that reads the
// sorts' status words sets it, and every rasterizer entry point looks at it (a plain host read) when
// it is called, so a give-up surfaces as an error of the next call on that device without any
// additional synchronisation.
constexpr int kMaxDevices = 64;
std::mutex g_device_mutex;
uint32_t* g_fault_word[kMaxDevices] = {};
uint32_t* g_static_scratch[kMaxDevices] = {};
uint32_t* g_static_gave_up[kMaxDevices] = {};

int current_device()
{
	int dev = 0;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
		return -1;
	return dev;
}

// The current device's word; allocated on first use unless `allocate` is false (then null if absent).
uint32_t* fault_word(bool allocate)
{
	const int dev = current_device();
	if (dev < 0)
		return nullptr;
	std::lock_guard<std::mutex> lock(g_device_mutex);
	if (!g_fault_word[dev] && allocate) {
		void* p = nullptr;
		if (hipHostMalloc(&p, 64, hipHostMallocDefault) == hipSuccess && p) {
			memset(p, 0, 64);
			g_fault_word[dev] = static_cast<uint32_t*>(p);
		} else {
			(void)hipGetLastError();
		}
	}
	return g_fault_word[dev];
}

// Non-zero (with the error set) if a sort of an earlier call on this device gave up; clears the report.
int take_sort_fault(const char* who)
{
	uint32_t* w = fault_word(false);
	if (!w || __atomic_load_n(w, __ATOMIC_RELAXED) == 0u)
		return 0;
	__atomic_store_n(w, 0u, __ATOMIC_RELAXED);
	return fail("%s: a radix sort of an earlier call on this device gave up waiting for a neighbouring workgroup; "
	            "that call left empty tile lists (background-only images, zero gradients) and must be repeated", who);
}

#define RGS_TAKE_SORT_FAULT(who)                   \
	do {                                           \
		if (int rc_ = take_sort_fault(who))        \
			return rc_;                            \
	} while (0)

// Device addresses of this device's copies of `scratch` and of its give-up word, looked up once per device with that
// device current.
int static_sort_scratch(uint32_t** out, uint32_t** gave_up)
{
	const int dev = current_device();
	if (dev < 0)
		return fail("rgs_sort_pairs_static: no current device");
	std::lock_guard<std::mutex> lock(g_device_mutex);
	if (!g_static_scratch[dev] || !g_static_gave_up[dev]) {
		void* p = nullptr;
		void* q = nullptr;
		hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
		if (e == hipSuccess)
			e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch_sort_gave_up));
		if (e != hipSuccess || !p || !q)
			return fail("rgs_sort_pairs_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
		g_static_scratch[dev] = static_cast<uint32_t*>(p);
		g_static_gave_up[dev] = static_cast<uint32_t*>(q);
	}
	*out = g_static_scratch[dev];
	*gave_up = g_static_gave_up[dev];
	return 0;
}

// Non-zero (with the error set) if a sort of rgs_sort_pairs_static on this device gave up; clears the report.  The
// caller has waited for the stream that sort ran on.
int take_static_sort_fault(const char* who)
{
	const int dev = current_device();
	uint32_t* word = nullptr;
	{
		std::lock_guard<std::mutex> lock(g_device_mutex);
		word = dev >= 0 ? g_static_gave_up[dev] : nullptr;
	}
	if (!word)
		return 0;  // no such sort has run on this device
	uint32_t seen = 0;
	hipError_t e = hipMemcpy(&seen, word, sizeof(seen), hipMemcpyDeviceToHost);
	if (e == hipSuccess && seen != 0u)
		e = hipMemset(word, 0, sizeof(seen));
	if (e != hipSuccess)
		return fail("%s: reading the report of rgs_sort_pairs_static failed: %s", who, hipGetErrorString(e));
	if (seen == 0u)
		return 0;
	return fail("%s: a radix sort of an earlier rgs_sort_pairs_static call on this device gave up waiting for a neighbouring "
	            "workgroup; its output is not sorted and the call must be repeated", who);
}

constexpr size_t kAlign = 256;

size_t align_up(size_t v)
{
	return (v + kAlign - 1) & ~(kAlign - 1);
}

struct Carver {
	size_t cursor = 0;
	size_t take(size_t bytes)
	{
		const size_t at = cursor;
		cursor = align_up(cursor + bytes);
		return at;
	}
};

// Scratch of the depth sort of the Gaussians, inside the geometry workspace.
struct OrderScratch {
	size_t keys_a, keys_b, vals_a, vals_b, tiles_in_order, sort_temp, scan_temp, dup_first, tile_digits, total;
};

OrderScratch order_scratch(size_t P)
{
	Carver c;
	OrderScratch o;
	o.keys_a = c.take(4 * P);
	o.keys_b = c.take(4 * P);
	o.vals_a = c.take(4 * P);
	o.vals_b = c.take(4 * P);
	o.tiles_in_order = c.take(4 * P);
	o.sort_temp = c.take(4 * rgs::sort_temp_words(P));
	o.scan_temp = c.take(4 * rgs::scan_temp_words(P));
	o.dup_first = c.take(4 * rgs::dup_first_words(P));
	o.tile_digits = c.take(4 * rgs::kTileDigitWords);
	o.total = c.cursor;
	return o;
}

size_t geom_layout(size_t P, size_t* off)
{
	Carver c;
	off[RGS_GEOM_DEPTHS] = c.take(4 * P);
	off[RGS_GEOM_TILES_TOUCHED] = c.take(4 * P);
	off[RGS_GEOM_POINT_OFFSETS] = c.take(4 * P);
	off[RGS_GEOM_CLAMPED] = c.take(P);
	off[RGS_GEOM_BLOCK_SUMS] = c.take(4 * ((P + 255) / 256 + 1));
	off[RGS_GEOM_TOTAL] = c.take(4 * (1 + RGS_MAX_FRAME_LAYERS));  // + where the first layer of a frame gathers every layer's count
	off[RGS_GEOM_BLEND_RECORD] = c.take(64 * P);
	off[RGS_GEOM_DEPTH_ORDER] = c.take(4 * P);
	off[RGS_GEOM_BLOCK_VISIBLE] = c.take(4 * ((P + 255) / 256 + 1));
	off[RGS_GEOM_VISIBLE_COUNT] = c.take(4);
	off[RGS_GEOM_ORDER_SCRATCH] = c.take(order_scratch(P).total);
	return c.cursor;
}

// Bits of the tile key that the instance sort looks at.
int tile_key_bits(int width, int height)
{
	const uint32_t tiles = (uint32_t)((width + rgs::kTile - 1) / rgs::kTile) * (uint32_t)((height + rgs::kTile - 1) / rgs::kTile);
	return (int)rgs_get_higher_msb(tiles);
}

// Passes of the instance sort on the tile bits.
int tile_sort_passes(int width, int height)
{
	const int bits = tile_key_bits(width, height);
	return rgs::sort_passes(bits, rgs::sort_max_digit_bits_u32(bits));
}

// Physical buffers: A receives the duplicated keys, B is its ping-pong partner.
struct BinningPhysical {
	size_t keys_a, keys_b, vals_a, vals_b, temp, strip_lists, file_tail, total;
};

BinningPhysical binning_physical(size_t R)
{
	Carver c;
	BinningPhysical b;
	b.keys_a = c.take(4 * R);
	b.keys_b = c.take(4 * R);
	b.vals_a = c.take(4 * R);
	b.vals_b = c.take(4 * R);
	b.temp = c.take(4 * rgs::sort_temp_words(R));
	b.strip_lists = c.take(16 * R);
	b.file_tail = c.take(16 * ((R + rgs::kFileGroup - 1) / rgs::kFileGroup));
	b.total = c.cursor;
	return b;
}

size_t image_layout(int width, int height, size_t* off)
{
	const size_t tiles = (size_t)((width + rgs::kTile - 1) / rgs::kTile) * (size_t)((height + rgs::kTile - 1) / rgs::kTile);
	Carver c;
	// the ranges, the strip class counters and the strips' totals lie one behind the other: they are cleared together
	off[RGS_IMG_RANGES] = c.take(8 * tiles + 4 * rgs::kRangeTailWords + 4 * 4 * tiles);
	off[RGS_IMG_STRIP_TOTAL] = off[RGS_IMG_RANGES] + 8 * tiles + 4 * rgs::kRangeTailWords;
	off[RGS_IMG_N_CONTRIB] = c.take(4 * (size_t)width * height);
	off[RGS_IMG_STRIP_FILED] = c.take(4 * 4 * tiles);
	off[RGS_IMG_STRIP_ORDER] = c.take(4 * 4 * tiles);
	off[RGS_IMG_STRIP_ORDER_FORWARD] = c.take(4 * 4 * tiles);
	return c.cursor;
}

template <typename T>
T* at(void* base, size_t off)
{
	return reinterpret_cast<T*>(static_cast<char*>(base) + off);
}
template <typename T>
const T* at(const void* base, size_t off)
{
	return reinterpret_cast<const T*>(static_cast<const char*>(base) + off);
}

}  // namespace

namespace rgs {
void stage_mark(const char* name, hipStream_t s)
{
	timer_record(name, s);
}
}  // namespace rgs

extern "C" {

int rgs_stage_timing(int enable)
{
	std::lock_guard<std::mutex> hold(g_timer.lock);
	g_timer.on.store(enable != 0, std::memory_order_relaxed);
	g_timer.used = 0;
	return 0;
}

int rgs_stage_timing_read(int max_stages, const char** names, float* total_ms, int* launches)
{
	RGS_REQUIRE(max_stages >= 0 && (max_stages == 0 || (names && total_ms && launches)), "rgs_stage_timing_read: bad arguments");
	int n = 0;
	std::lock_guard<std::mutex> hold(g_timer.lock);
	if (g_timer.used > 0) {
		hipError_t e = hipEventSynchronize(g_timer.pool[g_timer.used - 1]);
		if (e != hipSuccess)
			return -fail("rgs_stage_timing_read: %s", hipGetErrorString(e));
	}
	for (size_t i = 0; i + 1 < g_timer.used; i++) {
		const char* tag = g_timer.tags[i];
		if (!tag)
			continue;
		float ms = 0.f;
		if (hipEventElapsedTime(&ms, g_timer.pool[i], g_timer.pool[i + 1]) != hipSuccess)
			continue;
		int k = 0;
		while (k < n && strcmp(names[k], tag) != 0)
			k++;
		if (k == n) {
			if (n == max_stages)
				continue;
			names[n] = tag;
			total_ms[n] = 0.f;
			launches[n] = 0;
			n++;
		}
		total_ms[k] += ms;
		launches[k] += 1;
	}
	g_timer.used = 0;
	return n;
}

int rgs_version(void)
{
	return 100;
}

const char* rgs_last_error(void)
{
	return g_error;
}

uint32_t rgs_get_higher_msb(uint32_t n)
{
	// Smallest b with (n >> b) == 0, found by the reference's halving search
	// (K/cuda_rasterizer_hgs/rasterizer_impl.cu:35-50); both agree for every n.
	uint32_t msb = 16, step = 16;
	while (step > 1) {
		step >>= 1;
		msb = (n >> msb) ? msb + step : msb - step;
	}
	return (n >> msb) ? msb + 1 : msb;
}

size_t rgs_geom_bytes(int P)
{
	size_t off[RGS_GEOM_FIELDS];
	return geom_layout(P > 0 ? (size_t)P : 0, off) + kAlign;
}

size_t rgs_binning_bytes(int R)
{
	return binning_physical(R > 0 ? (size_t)R : 0).total + kAlign;
}

size_t rgs_image_bytes(int width, int height)
{
	size_t off[RGS_IMG_FIELDS];
	return image_layout(width, height, off) + kAlign;
}

int rgs_geom_layout(int P, size_t offsets[RGS_GEOM_FIELDS])
{
	RGS_REQUIRE(P >= 0 && offsets, "rgs_geom_layout: bad arguments");
	geom_layout((size_t)P, offsets);
	return 0;
}

int rgs_binning_layout(int R, int width, int height, size_t offsets[RGS_BIN_FIELDS])
{
	RGS_REQUIRE(R >= 0 && width > 0 && height > 0 && offsets, "rgs_binning_layout: bad arguments");
	const BinningPhysical b = binning_physical((size_t)R);
	const bool sorted_in_a = (tile_sort_passes(width, height) % 2) == 0;
	offsets[RGS_BIN_KEYS_UNSORTED] = sorted_in_a ? b.keys_b : b.keys_a;
	offsets[RGS_BIN_KEYS_SORTED] = sorted_in_a ? b.keys_a : b.keys_b;
	offsets[RGS_BIN_VALUES_UNSORTED] = sorted_in_a ? b.vals_b : b.vals_a;
	offsets[RGS_BIN_VALUES_SORTED] = sorted_in_a ? b.vals_a : b.vals_b;
	offsets[RGS_BIN_SORT_TEMP] = b.temp;
	offsets[RGS_BIN_STRIP_LISTS] = b.strip_lists;
	return 0;
}

int rgs_image_layout(int width, int height, size_t offsets[RGS_IMG_FIELDS])
{
	RGS_REQUIRE(width > 0 && height > 0 && offsets, "rgs_image_layout: bad arguments");
	image_layout(width, height, offsets);
	return 0;
}

int rgs_mark_visible(int P, const float* means3D, const float* viewmatrix, const float* projmatrix,
                     uint8_t* present, void* stream)
{
	(void)projmatrix;
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(P >= 0, "rgs_mark_visible: negative P");
	if (P == 0)
		return 0;
	RGS_REQUIRE(means3D && viewmatrix && present, "rgs_mark_visible: null pointer");
	rgs::launch_mark_visible(P, means3D, viewmatrix, present, s);
	RGS_STAGE("mark_visible");
	return 0;
}

int rgs_covariance3d(int P, const float* scales, float scale_modifier, const float* rotations, float* cov3D, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(P >= 0, "rgs_covariance3d: negative P");
	if (P == 0)
		return 0;
	RGS_REQUIRE(scales && rotations && cov3D, "rgs_covariance3d: null pointer");
	RGS_REQUIRE((reinterpret_cast<uintptr_t>(rotations) & 15) == 0, "rgs_covariance3d: rotations must be 16-byte aligned");
	rgs::launch_covariance3d(P, scales, scale_modifier, rotations, cov3D, s);
	RGS_STAGE("covariance3d");
	return 0;
}

// Whether SH rows can be moved 16 bytes at a time: aligned base, row length a multiple of four
// floats, at most 48 of them, and enough of them for the degree's rounded-up count.
static bool sh_rows_by_16_bytes(const float* shs, int M, int D)
{
	const int n = 3 * M, needed = (3 * (D + 1) * (D + 1) + 3) & ~3;
	return shs && (reinterpret_cast<uintptr_t>(shs) & 15) == 0 && (n & 3) == 0 && n <= 48 && needed <= n;
}

// One event per host thread and device, for waiting on the copy of the instance count alone.
static hipEvent_t count_event_of_this_thread()
{
	constexpr int kMaxDevices = 64;
	static thread_local hipEvent_t events[kMaxDevices] = {};
	int dev = 0;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
		return nullptr;
	if (!events[dev] && hipEventCreateWithFlags(&events[dev], hipEventDisableTiming) != hipSuccess)
		events[dev] = nullptr;
	return events[dev];
}

// One layer's arguments of the geometry stage.
struct GeomCall {
	int P, D, M;
	const float* means3D;
	const float* shs;
	const float* colors_precomp;
	const float* opacities;
	const float* scales;
	float scale_modifier;
	const float* rotations;
	const float* cov3D_precomp;
	int* radii;
	void* geom_ws;
	size_t geom_bytes;
};

// The geometry stage of `K` layers that share a camera, every kernel launched once for all of them: preprocess,
// the instance counts (one copy to counts_host[0..K)), and, behind that copy, the depth order.
static int forward_geom(bool wait_for_count, void* count_ready_event, const char* who, int K, const GeomCall* calls,
                        int width, int height, const float* viewmatrix, const float* projmatrix, const float* cam_pos,
                        float tan_fovx, float tan_fovy, uint32_t* counts_host, void* stream, int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT(who);
	RGS_REQUIRE(width > 0 && height > 0, "%s: bad image size %dx%d", who, width, height);
	RGS_REQUIRE(viewmatrix && projmatrix && cam_pos && counts_host, "%s: null pointer", who);
	std::vector<rgs::PreprocessArgs> pre((size_t)K);
	std::vector<rgs::TotalsJob> totals((size_t)K);
	std::vector<rgs::DepthOrderJob> orders((size_t)K);
	uint32_t* frame_counts = nullptr;  // K words in the first layer's workspace, so that one copy brings all counts
	for (int k = 0; k < K; k++) {
		const GeomCall& c = calls[k];
		RGS_REQUIRE(c.P > 0, "%s: P must be positive (the caller short-circuits P == 0)", who);
		RGS_REQUIRE(c.means3D && c.opacities && c.radii && c.geom_ws, "%s: null pointer", who);
		RGS_REQUIRE((c.shs != nullptr) != (c.colors_precomp != nullptr),
		            "%s: provide exactly one of SHs or precomputed colours", who);
		RGS_REQUIRE(((c.scales != nullptr) && (c.rotations != nullptr)) != (c.cov3D_precomp != nullptr) &&
		                ((c.scales != nullptr) == (c.rotations != nullptr)),
		            "%s: provide exactly one of scale/rotation or precomputed 3D covariance", who);
		RGS_REQUIRE(c.D >= 0 && c.D <= 3, "%s: SH degree %d out of range", who, c.D);
		RGS_REQUIRE(!c.shs || c.M >= (c.D + 1) * (c.D + 1), "%s: %d SH coefficients cannot hold degree %d", who, c.M, c.D);
		RGS_REQUIRE(c.geom_bytes >= rgs_geom_bytes(c.P), "%s: geometry workspace too small", who);
		RGS_REQUIRE((reinterpret_cast<uintptr_t>(c.geom_ws) & 15) == 0, "%s: workspace must be 16-byte aligned", who);

		size_t off[RGS_GEOM_FIELDS];
		geom_layout((size_t)c.P, off);
		void* ws = c.geom_ws;
		if (k == 0)
			frame_counts = at<uint32_t>(ws, off[RGS_GEOM_TOTAL]) + 1;
		rgs::PreprocessArgs& a = pre[(size_t)k];
		a.P = c.P; a.D = c.D; a.M = c.M;
		a.means = c.means3D; a.scales = c.scales; a.scale_modifier = c.scale_modifier; a.rotations = c.rotations;
		a.opacities = c.opacities; a.shs = c.shs; a.cov3D_precomp = c.cov3D_precomp; a.colors_precomp = c.colors_precomp;
		a.view = viewmatrix; a.proj = projmatrix; a.campos = cam_pos;
		a.W = width; a.H = height;
		a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
		// K/cuda_rasterizer_hgs/rasterizer_impl.cu:227-228
		a.focal_y = height / (2.0f * tan_fovy);
		a.focal_x = width / (2.0f * tan_fovx);
		a.grid_x = (width + rgs::kTile - 1) / rgs::kTile;
		a.grid_y = (height + rgs::kTile - 1) / rgs::kTile;
		a.radii = c.radii;
		a.depths = at<float>(ws, off[RGS_GEOM_DEPTHS]);
		a.tiles_touched = at<uint32_t>(ws, off[RGS_GEOM_TILES_TOUCHED]);
		a.clamped = at<uint8_t>(ws, off[RGS_GEOM_CLAMPED]);
		a.block_sums = at<uint32_t>(ws, off[RGS_GEOM_BLOCK_SUMS]);
		a.blend_record = at<float4>(ws, off[RGS_GEOM_BLEND_RECORD]);
		a.block_visible = at<uint32_t>(ws, off[RGS_GEOM_BLOCK_VISIBLE]);
		a.sh_rows_by_16_bytes = sh_rows_by_16_bytes(c.shs, c.M, c.D);
		const OrderScratch o = order_scratch((size_t)c.P);
		char* scratch = at<char>(ws, off[RGS_GEOM_ORDER_SCRATCH]);
		a.clear = at<uint32_t>(scratch, o.sort_temp);
		a.clear_words = rgs::depth_sort_clear_words((size_t)c.P);

		totals[(size_t)k] = rgs::TotalsJob{a.block_sums, a.block_visible, c.P, at<uint32_t>(ws, off[RGS_GEOM_TOTAL]),
		                                   frame_counts + k, at<uint32_t>(ws, off[RGS_GEOM_VISIBLE_COUNT])};
		rgs::DepthOrderJob& d = orders[(size_t)k];
		d.P = c.P;
		d.depths = a.depths; d.tiles_touched = a.tiles_touched; d.block_visible = a.block_visible;
		d.visible_count = at<uint32_t>(ws, off[RGS_GEOM_VISIBLE_COUNT]);
		d.keys_a = at<uint32_t>(scratch, o.keys_a); d.keys_b = at<uint32_t>(scratch, o.keys_b);
		d.order = at<uint32_t>(ws, off[RGS_GEOM_DEPTH_ORDER]); d.vals_a = at<uint32_t>(scratch, o.vals_a);
		d.vals_b = at<uint32_t>(scratch, o.vals_b);
		d.tiles_in_order = at<uint32_t>(scratch, o.tiles_in_order);
		d.offsets_in_order = at<uint32_t>(ws, off[RGS_GEOM_POINT_OFFSETS]);
		d.sort_temp = at<uint32_t>(scratch, o.sort_temp); d.scan_temp = at<uint32_t>(scratch, o.scan_temp);
		d.dup_first = at<uint32_t>(scratch, o.dup_first);
		d.tile_digits = at<uint32_t>(scratch, o.tile_digits);
	}
	rgs::launch_preprocess_forward(pre.data(), K, s);
	RGS_STAGE("preprocess");
	rgs::launch_totals_from_block_sums(totals.data(), K, s);
	RGS_STAGE("instance count");
	hipError_t e = hipMemcpyAsync(counts_host, frame_counts, sizeof(uint32_t) * (size_t)K, hipMemcpyDeviceToHost, s);
	// the host only needs the counts: it waits for this event, not for the kernels queued below
	hipEvent_t ready = wait_for_count ? count_event_of_this_thread() : static_cast<hipEvent_t>(count_ready_event);
	if (e == hipSuccess && ready)
		e = hipEventRecord(ready, s);
	// depth order of the Gaussians and the offsets of their instances in that order: needs
	// nothing from the host, so it is queued behind the counts' copy
	rgs::launch_depth_order(orders.data(), K, s);
	RGS_STAGE("depth order");
	if (e == hipSuccess && wait_for_count)
		e = ready ? hipEventSynchronize(ready) : hipStreamSynchronize(s);
	if (e != hipSuccess)
		return fail("%s: reading the instance count failed: %s", who, hipGetErrorString(e));
	if (wait_for_count)
		for (int k = 0; k < K; k++)
			RGS_REQUIRE(counts_host[k] < 0x40000000u, "%s: %u (Gaussian, tile) instances exceed the 2^30 limit of the sort", who,
			            counts_host[k]);
	return 0;
}

int rgs_forward_geom(int P, int D, int M, int width, int height,
                     const float* means3D, const float* shs, const float* colors_precomp, const float* opacities,
                     const float* scales, float scale_modifier, const float* rotations, const float* cov3D_precomp,
                     const float* viewmatrix, const float* projmatrix, const float* cam_pos,
                     float tan_fovx, float tan_fovy, int prefiltered,
                     int* radii, void* geom_ws, size_t geom_bytes,
                     uint32_t* num_rendered_host, void* stream, int debug)
{
	// `prefiltered` promises that no Gaussian is culled; the reference traps the device when
	// the promise is broken (K/cuda_rasterizer_hgs/auxiliary.h:172-176).  Here a culled
	// Gaussian is simply skipped.
	(void)prefiltered;
	RGS_REQUIRE(P > 0, "rgs_forward_geom: P must be positive (the caller short-circuits P == 0)");
	RGS_REQUIRE(num_rendered_host, "rgs_forward_geom: null pointer");
	const GeomCall c = {P, D, M, means3D, shs, colors_precomp, opacities, scales, scale_modifier, rotations, cov3D_precomp, radii,
	                    geom_ws, geom_bytes};
	return forward_geom(true, nullptr, "rgs_forward_geom", 1, &c, width, height, viewmatrix, projmatrix, cam_pos, tan_fovx,
	                    tan_fovy, num_rendered_host, stream, debug);
}

int rgs_forward_geom_enqueue(int P, int D, int M, int width, int height,
                             const float* means3D, const float* shs, const float* colors_precomp,
                             const float* opacities, const float* scales, float scale_modifier, const float* rotations,
                             const float* cov3D_precomp, const float* viewmatrix, const float* projmatrix,
                             const float* cam_pos, float tan_fovx, float tan_fovy, int prefiltered,
                             int* radii, void* geom_ws, size_t geom_bytes,
                             uint32_t* num_rendered_pinned, void* count_ready_event, void* stream, int debug)
{
	(void)prefiltered;
	RGS_REQUIRE(P > 0, "rgs_forward_geom_enqueue: P must be positive (the caller short-circuits P == 0)");
	RGS_REQUIRE(num_rendered_pinned, "rgs_forward_geom_enqueue: null pointer");
	const GeomCall c = {P, D, M, means3D, shs, colors_precomp, opacities, scales, scale_modifier, rotations, cov3D_precomp, radii,
	                    geom_ws, geom_bytes};
	return forward_geom(false, count_ready_event, "rgs_forward_geom_enqueue", 1, &c, width, height, viewmatrix, projmatrix, cam_pos,
	                    tan_fovx, tan_fovy, num_rendered_pinned, stream, debug);
}


}  // extern "C"

namespace {

// The blend kernels' view of one call's workspaces (everything but the outputs and the gradients).
void fill_blend_args(rgs::BlendArgs& a, int P, int R, int width, int height, float tan_fovx, float tan_fovy,
                     const float* background, const float* projmatrix_inv, const float* range_low, const float* range_up,
                     const float* colors_precomp, const void* geom_ws, const void* binning_ws, const void* image_ws)
{
	size_t goff[RGS_GEOM_FIELDS], ioff[RGS_IMG_FIELDS];
	geom_layout((size_t)P, goff);
	image_layout(width, height, ioff);
	const int gx = (width + rgs::kTile - 1) / rgs::kTile, gy = (height + rgs::kTile - 1) / rgs::kTile;
	memset(&a, 0, sizeof(a));
	void* img = const_cast<void*>(image_ws);
	a.ranges = at<uint2>(image_ws, ioff[RGS_IMG_RANGES]);
	a.W = width; a.H = height; a.grid_x = gx; a.grid_y = gy;
	a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
	a.projinv = projmatrix_inv; a.range_low = range_low; a.range_up = range_up; a.bg = background;
	a.record = at<float4>(geom_ws, goff[RGS_GEOM_BLEND_RECORD]);
	a.n_contrib = at<uint32_t>(img, ioff[RGS_IMG_N_CONTRIB]);
	a.strip_filed = at<uint32_t>(img, ioff[RGS_IMG_STRIP_FILED]);
	a.strip_order = at<uint32_t>(img, ioff[RGS_IMG_STRIP_ORDER]);
	a.strip_order_forward = at<uint32_t>(img, ioff[RGS_IMG_STRIP_ORDER_FORWARD]);
	a.strip_total = at<uint32_t>(img, ioff[RGS_IMG_STRIP_TOTAL]);
	a.strip_classes = reinterpret_cast<uint32_t*>(at<uint2>(img, ioff[RGS_IMG_RANGES])) + 2 * (size_t)gx * gy;
	a.capacity = (uint32_t)R;
	a.gaussians = (uint32_t)P;
	if (R > 0) {
		const BinningPhysical b = binning_physical((size_t)R);
		const bool sorted_in_a = (tile_sort_passes(width, height) % 2) == 0;
		void* bin = const_cast<void*>(binning_ws);
		a.point_list = at<uint32_t>(binning_ws, sorted_in_a ? b.vals_a : b.vals_b);
		a.tile_keys = at<uint32_t>(binning_ws, sorted_in_a ? b.keys_a : b.keys_b);
		a.strip_lists = at<uint32_t>(bin, b.strip_lists);
		a.file_tail = at<uint4>(binning_ws, b.file_tail);
		a.sort_status = rgs::sort_status_word(at<uint32_t>(binning_ws, b.temp));
		a.order_status = rgs::sort_status_word(at<uint32_t>(at<char>(geom_ws, goff[RGS_GEOM_ORDER_SCRATCH]), order_scratch((size_t)P).sort_temp));
	}
}

// One layer's arguments of the second half of the forward.
struct RasterCall {
	int P, R;
	const float* background;
	const float* range_low;
	const float* range_up;
	const float* colors_precomp;
	void* geom_ws;
	size_t geom_bytes;
	void* binning_ws;
	size_t binning_bytes;
	void* image_ws;
	size_t image_bytes;
};

// Second half of the forward up to the blend, for `K` layers that share a camera, every kernel launched once for
// all of them: key duplication, the instance sort, tile ranges, the strips' lists.  A layer's R sizes its binning
// workspace and its share of the launches.  With count_on_device the number of instances is the smaller of R and
// the count the geometry stage left in the layer's workspace, read by the kernels.  Fills jobs[k] for the blend.
int forward_binning(const char* who, bool count_on_device, int K, const RasterCall* calls, int width, int height,
                    float tan_fovx, float tan_fovy, const float* projmatrix_inv, rgs::BlendArgs* jobs, hipStream_t s, int debug)
{
	RGS_TAKE_SORT_FAULT(who);
	RGS_REQUIRE(width > 0 && height > 0, "%s: bad image size %dx%d", who, width, height);
	RGS_REQUIRE((uint64_t)((width + rgs::kTile - 1) / rgs::kTile) * (uint64_t)((height + rgs::kTile - 1) / rgs::kTile) <
	                (1ull << rgs::kKeyTileBits),
	            "%s: a %dx%d image has 2^%d tiles or more", who, width, height, rgs::kKeyTileBits);
	RGS_REQUIRE(projmatrix_inv, "%s: null pointer", who);
	const int gx = (width + rgs::kTile - 1) / rgs::kTile, gy = (height + rgs::kTile - 1) / rgs::kTile;
	const int end_bit = tile_key_bits(width, height);
	// the tile ranges, the strip class counters and the strips' totals, cleared together
	const size_t clear_words = (size_t)gx * gy * 2 + rgs::kRangeTailWords + (size_t)gx * gy * 4;
	std::vector<rgs::DuplicateJob> dups;
	std::vector<rgs::SortJob<uint32_t>> sorts;
	std::vector<rgs::TileRangesJob> ranges_jobs;
	std::vector<int> with_instances;
	uint32_t* fault = fault_word(true);
	for (int k = 0; k < K; k++) {
		const RasterCall& c = calls[k];
		const int P = c.P, R = c.R;
		RGS_REQUIRE(P > 0 && R >= 0, "%s: bad sizes P=%d R=%d", who, P, R);
		RGS_REQUIRE(R < 0x40000000, "%s: %d (Gaussian, tile) instances exceed the 2^30 limit of the sort", who, R);
		RGS_REQUIRE(c.background && c.range_low && c.range_up && c.geom_ws && c.image_ws, "%s: null pointer", who);
		RGS_REQUIRE(R == 0 || c.binning_ws, "%s: null binning workspace", who);
		RGS_REQUIRE((reinterpret_cast<uintptr_t>(c.binning_ws) & 15) == 0 && (reinterpret_cast<uintptr_t>(c.image_ws) & 15) == 0,
		            "%s: workspaces must be 16-byte aligned", who);
		RGS_REQUIRE(c.geom_bytes >= rgs_geom_bytes(P), "%s: geometry workspace too small", who);
		RGS_REQUIRE(R == 0 || c.binning_bytes >= rgs_binning_bytes(R), "%s: binning workspace too small", who);
		RGS_REQUIRE(c.image_bytes >= rgs_image_bytes(width, height), "%s: image workspace too small", who);
		rgs::BlendArgs& a = jobs[k];
		fill_blend_args(a, P, R, width, height, tan_fovx, tan_fovy, c.background, projmatrix_inv, c.range_low, c.range_up,
		                c.colors_precomp, c.geom_ws, c.binning_ws, c.image_ws);
		uint2* ranges = const_cast<uint2*>(a.ranges);
		if (R == 0) {
			rgs::launch_fill_u32(reinterpret_cast<uint32_t*>(ranges), 0u, clear_words, s);
			RGS_STAGE("tile_ranges");
			continue;
		}
		size_t goff[RGS_GEOM_FIELDS];
		geom_layout((size_t)P, goff);
		const BinningPhysical b = binning_physical((size_t)R);
		uint32_t* keys_a = at<uint32_t>(c.binning_ws, b.keys_a);
		uint32_t* keys_b = at<uint32_t>(c.binning_ws, b.keys_b);
		uint32_t* vals_a = at<uint32_t>(c.binning_ws, b.vals_a);
		uint32_t* vals_b = at<uint32_t>(c.binning_ws, b.vals_b);
		uint32_t* temp = at<uint32_t>(c.binning_ws, b.temp);
		const uint32_t* count = count_on_device ? at<uint32_t>(c.geom_ws, goff[RGS_GEOM_TOTAL]) : nullptr;
		a.count_device = count;
		rgs::DuplicateJob d;
		d.P = P;
		d.visible_count = at<uint32_t>(c.geom_ws, goff[RGS_GEOM_VISIBLE_COUNT]);
		d.order = at<uint32_t>(c.geom_ws, goff[RGS_GEOM_DEPTH_ORDER]);
		d.offsets = at<uint32_t>(c.geom_ws, goff[RGS_GEOM_POINT_OFFSETS]);
		d.total = at<uint32_t>(c.geom_ws, goff[RGS_GEOM_TOTAL]);
		d.first_of_block = at<uint32_t>(at<char>(c.geom_ws, goff[RGS_GEOM_ORDER_SCRATCH]), order_scratch((size_t)P).dup_first);
		d.filing.record = a.record;
		d.filing.projinv = projmatrix_inv; d.filing.range_low = c.range_low; d.filing.range_up = c.range_up;
		d.filing.tanfovx = tan_fovx; d.filing.tanfovy = tan_fovy;
		d.filing.W = width; d.filing.H = height;
		d.keys = keys_a; d.values = vals_a; d.capacity = (uint32_t)R;
		d.clear = temp; d.clear_words = rgs::sort_clear_words((size_t)R, end_bit, rgs::sort_max_digit_bits_u32(end_bit));
		// it also clears the tile ranges (and the counters and totals behind them) and counts the digits of the tiles
		// it writes, so the sort starts with its passes
		uint32_t* tile_digits = at<uint32_t>(at<char>(c.geom_ws, goff[RGS_GEOM_ORDER_SCRATCH]), order_scratch((size_t)P).tile_digits);
		d.tile_digits = tile_digits; d.end_bit = end_bit;
		d.also_clear = reinterpret_cast<uint32_t*>(ranges); d.also_clear_words = clear_words;
		dups.push_back(d);
		rgs::SortJob<uint32_t> sj = {};
		sj.keys_in = keys_a; sj.keys_out = keys_b; sj.vals_in = vals_a; sj.vals_out = vals_b;
		sj.n = (size_t)R; sj.n_device = count; sj.temp = temp; sj.digit_counts = tile_digits;
		sorts.push_back(sj);
		ranges_jobs.push_back(rgs::TileRangesJob{a.tile_keys, (size_t)R, count, ranges, a.sort_status, a.order_status, fault,
		                                         at<uint4>(c.binning_ws, b.file_tail), tile_digits});
		with_instances.push_back(k);
	}
	if (with_instances.empty())
		return 0;
	const int n = (int)with_instances.size();
	rgs::launch_duplicate_with_keys(dups.data(), n, gx, gy, s);
	RGS_STAGE("duplicate_with_keys");
	rgs::launch_sort_pairs_u32(sorts.data(), n, end_bit, true, true, "sort", s);
	RGS_STAGE("sort_pairs");
	if (debug)
		for (int k : with_instances) {
			uint32_t status = 0, status2 = 0;
			hipError_t e = hipMemcpy(&status, jobs[k].sort_status, sizeof(status), hipMemcpyDeviceToHost);
			if (e == hipSuccess)
				e = hipMemcpy(&status2, jobs[k].order_status, sizeof(status2), hipMemcpyDeviceToHost);
			status |= status2;
			if (e != hipSuccess || status != 0)
				return fail("sort_pairs: %s", e != hipSuccess ? hipGetErrorString(e) : "a look-back wait timed out");
		}
	rgs::launch_tile_ranges(ranges_jobs.data(), n, s);
	RGS_STAGE("tile_ranges");
	std::vector<rgs::BlendArgs> filing((size_t)n);
	for (int i = 0; i < n; i++)
		filing[(size_t)i] = jobs[with_instances[(size_t)i]];
	rgs::launch_strip_filing(filing.data(), n, s);
	RGS_STAGE("strip_filing");
	return 0;
}

int forward_raster(bool count_on_device, int P, int R, int width, int height,
                   const float* background, float tan_fovx, float tan_fovy,
                   const float* projmatrix_inv, const float* range_low, const float* range_up,
                   const float* colors_precomp, const int* radii,
                   void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                   void* image_ws, size_t image_bytes,
                   float* out_color, float* out_depth, float* out_alpha, void* stream, int debug)
{
	(void)radii;  // the key duplication reads the radius from the Gaussian's packed record
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_REQUIRE(out_color && out_depth && out_alpha, "rgs_forward_raster: null pointer");
	rgs::BlendArgs a;
	const RasterCall c = {P, R, background, range_low, range_up, colors_precomp, geom_ws, geom_bytes, binning_ws, binning_bytes,
	                      image_ws, image_bytes};
	if (int rc = forward_binning("rgs_forward_raster", count_on_device, 1, &c, width, height, tan_fovx, tan_fovy, projmatrix_inv,
	                             &a, s, debug))
		return rc;
	a.out_color = out_color; a.out_depth = out_depth; a.out_alpha = out_alpha;
	rgs::launch_blend_forward(&a, 1, s);
	RGS_STAGE("blend_forward");
	return 0;
}

// The per-Gaussian half of the backward: fused cov2D / preprocess backward over the rendered Gaussians.
void fill_backward_geometry(rgs::PreprocessBackwardArgs& p, int P, int D, int M, int width, int height, const float* means3D,
                            const float* shs, const float* scales, float scale_modifier, const float* rotations,
                            const float* cov3D_precomp, const float* viewmatrix, const float* projmatrix, const float* cam_pos,
                            float tan_fovx, float tan_fovy, const int* radii, const void* geom_ws, const float* grad_accum,
                            float* dL_dmean2D, float* dL_dopacity, float* dL_dcolor, float* dL_dmean3D, float* dL_dcov3D,
                            float* dL_dsh, float* dL_dscale, float* dL_drot)
{
	size_t goff[RGS_GEOM_FIELDS];
	geom_layout((size_t)P, goff);
	memset(&p, 0, sizeof(p));
	p.P = P; p.D = D; p.M = M;
	p.means = means3D; p.radii = radii; p.shs = shs;
	p.clamped = at<uint8_t>(geom_ws, goff[RGS_GEOM_CLAMPED]);
	p.scales = scales; p.rotations = rotations; p.scale_modifier = scale_modifier;
	p.cov3D_precomp = cov3D_precomp;
	p.view = viewmatrix; p.proj = projmatrix; p.campos = cam_pos;
	p.focal_y = height / (2.0f * tan_fovy);
	p.focal_x = width / (2.0f * tan_fovx);
	p.tanfovx = tan_fovx; p.tanfovy = tan_fovy;
	p.sums = grad_accum;
	p.dL_dmean2D = dL_dmean2D; p.dL_dopacity = dL_dopacity; p.dL_dcolor = dL_dcolor;
	p.dL_dmeans = dL_dmean3D; p.dL_dcov3D = dL_dcov3D; p.dL_dsh = dL_dsh; p.dL_dscale = dL_dscale; p.dL_drot = dL_drot;
	p.sh_rows_by_16_bytes = sh_rows_by_16_bytes(shs, M, D) && (reinterpret_cast<uintptr_t>(dL_dsh) & 15) == 0;
}

// Events for ordering a frame's stream against its layers' own streams: a few per host thread and device, reused.
hipEvent_t frame_event(size_t i)
{
	static thread_local std::vector<hipEvent_t> events[kMaxDevices];
	const int dev = current_device();
	if (dev < 0)
		return nullptr;
	std::vector<hipEvent_t>& v = events[dev];
	while (v.size() <= i) {
		hipEvent_t e = nullptr;
		if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess)
			return nullptr;
		v.push_back(e);
	}
	return v[i];
}

// The distinct streams among the layers' own that are not the frame's.
std::vector<hipStream_t> side_streams(int K, const rgs_frame_layer* layers, hipStream_t frame)
{
	std::vector<hipStream_t> out;
	for (int k = 0; k < K; k++) {
		hipStream_t ls = static_cast<hipStream_t>(layers[k].stream);
		if (!ls || ls == frame)
			continue;
		bool seen = false;
		for (hipStream_t o : out)
			seen = seen || o == ls;
		if (!seen)
			out.push_back(ls);
	}
	return out;
}

int check_backward_pointers(const char* who, int P, int R, int width, int height, const float* background,
                            const float* means3D, const float* shs, const float* colors_precomp, const float* alphas,
                            const float* scales, const float* rotations, const float* cov3D_precomp, const float* viewmatrix,
                            const float* projmatrix, const float* projmatrix_inv, const float* range_low,
                            const float* range_up, const float* cam_pos, const int* radii, const void* geom_ws,
                            const void* binning_ws, const void* image_ws, const float* dL_dpix, const float* grad_accum,
                            const float* dL_dmean2D, const float* dL_dopacity, const float* dL_dcolor, const float* dL_dmean3D,
                            const float* dL_dcov3D, const float* dL_dsh, const float* dL_dscale, const float* dL_drot)
{
	RGS_REQUIRE(P > 0 && R >= 0, "%s: bad sizes P=%d R=%d", who, P, R);
	RGS_REQUIRE(width > 0 && height > 0, "%s: bad image size %dx%d", who, width, height);
	RGS_REQUIRE(background && means3D && alphas && viewmatrix && projmatrix && projmatrix_inv && range_low && range_up &&
	                cam_pos && radii && geom_ws && image_ws && dL_dpix && grad_accum &&
	                dL_dmean2D && dL_dopacity && dL_dmean3D,
	            "%s: null pointer", who);
	RGS_REQUIRE(!colors_precomp || dL_dcolor, "%s: dL_dcolor is required with precomputed colours", who);
	RGS_REQUIRE(!cov3D_precomp || dL_dcov3D, "%s: dL_dcov3D is required with a precomputed covariance", who);
	RGS_REQUIRE(R == 0 || binning_ws, "%s: null binning workspace", who);
	RGS_REQUIRE((shs != nullptr) != (colors_precomp != nullptr), "%s: provide exactly one of SHs or colours", who);
	RGS_REQUIRE(!shs || dL_dsh, "%s: dL_dsh is required with SHs", who);
	RGS_REQUIRE(!scales || (rotations && dL_dscale && dL_drot), "%s: scale/rotation outputs missing", who);
	RGS_REQUIRE(scales || cov3D_precomp, "%s: neither scales nor precomputed covariance", who);
	return 0;
}

}  // namespace

extern "C" {

int rgs_forward_raster(int P, int R, int width, int height,
                       const float* background, float tan_fovx, float tan_fovy,
                       const float* projmatrix_inv, const float* range_low, const float* range_up,
                       const float* colors_precomp, const int* radii,
                       void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                       void* image_ws, size_t image_bytes,
                       float* out_color, float* out_depth, float* out_alpha, void* stream, int debug)
{
	return forward_raster(false, P, R, width, height, background, tan_fovx, tan_fovy, projmatrix_inv, range_low, range_up,
	                      colors_precomp, radii, geom_ws, geom_bytes, binning_ws, binning_bytes, image_ws, image_bytes,
	                      out_color, out_depth, out_alpha, stream, debug);
}

int rgs_forward_raster_bounded(int P, int R_bound, int width, int height,
                               const float* background, float tan_fovx, float tan_fovy,
                               const float* projmatrix_inv, const float* range_low, const float* range_up,
                               const float* colors_precomp, const int* radii,
                               void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                               void* image_ws, size_t image_bytes,
                               float* out_color, float* out_depth, float* out_alpha, void* stream, int debug)
{
	return forward_raster(true, P, R_bound, width, height, background, tan_fovx, tan_fovy, projmatrix_inv, range_low,
	                      range_up, colors_precomp, radii, geom_ws, geom_bytes, binning_ws, binning_bytes, image_ws,
	                      image_bytes, out_color, out_depth, out_alpha, stream, debug);
}

int rgs_backward(int P, int D, int M, int R, int width, int height,
                 const float* background, const float* means3D, const float* shs, const float* colors_precomp,
                 const float* alphas, const float* scales, float scale_modifier, const float* rotations,
                 const float* cov3D_precomp, const float* viewmatrix, const float* projmatrix,
                 const float* projmatrix_inv, const float* range_low, const float* range_up, const float* cam_pos,
                 float tan_fovx, float tan_fovy, const int* radii,
                 const void* geom_ws, const void* binning_ws, const void* image_ws,
                 const float* dL_dpix, const float* dL_dpix_depth, const float* dL_dalphas,
                 float* grad_accum, float* dL_dmean2D, float* dL_dopacity, float* dL_dcolor, float* dL_dmean3D,
                 float* dL_dcov3D, float* dL_dsh, float* dL_dscale, float* dL_drot, int accum_zeroed, void* stream,
                 int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT("rgs_backward");
	if (int rc = check_backward_pointers("rgs_backward", P, R, width, height, background, means3D, shs, colors_precomp, alphas,
	                                     scales, rotations, cov3D_precomp, viewmatrix, projmatrix, projmatrix_inv, range_low,
	                                     range_up, cam_pos, radii, geom_ws, binning_ws, image_ws, dL_dpix, grad_accum, dL_dmean2D,
	                                     dL_dopacity, dL_dcolor, dL_dmean3D, dL_dcov3D, dL_dsh, dL_dscale, dL_drot))
		return rc;
	if (!accum_zeroed) {
		rgs::launch_fill_u32(reinterpret_cast<uint32_t*>(grad_accum), 0u, (size_t)RGS_ACC_FLOATS * (size_t)P, s);
		RGS_STAGE("clear gradient sums");
	}
	if (R > 0) {
		rgs::BlendArgs a;
		fill_blend_args(a, P, R, width, height, tan_fovx, tan_fovy, background, projmatrix_inv, range_low, range_up, colors_precomp,
		                geom_ws, binning_ws, image_ws);
		a.out_alpha = const_cast<float*>(alphas);
		a.dL_dpix = dL_dpix; a.dL_dpix_depth = dL_dpix_depth; a.dL_dalpha = dL_dalphas;
		a.sums = grad_accum;
		rgs::launch_blend_backward(&a, 1, s);
		RGS_STAGE("blend_backward");
	}
	rgs::PreprocessBackwardArgs p;
	fill_backward_geometry(p, P, D, M, width, height, means3D, shs, scales, scale_modifier, rotations, cov3D_precomp, viewmatrix,
	                       projmatrix, cam_pos, tan_fovx, tan_fovy, radii, geom_ws, grad_accum, dL_dmean2D, dL_dopacity,
	                       dL_dcolor, dL_dmean3D, dL_dcov3D, dL_dsh, dL_dscale, dL_drot);
	rgs::launch_preprocess_backward(&p, 1, s);
	RGS_STAGE("preprocess_backward");
	return 0;
}

int rgs_frame_forward_geom(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, uint32_t* counts_pinned,
                           void* stream, int debug)
{
	RGS_REQUIRE(K >= 1 && K <= RGS_MAX_FRAME_LAYERS && layers && view && counts_pinned,
	            "rgs_frame_forward_geom: K = %d outside 1..%d, or null", K, RGS_MAX_FRAME_LAYERS);
	std::vector<GeomCall> calls((size_t)K);
	for (int k = 0; k < K; k++) {
		const rgs_frame_layer& l = layers[k];
		calls[(size_t)k] = GeomCall{l.P, l.D, l.M, l.means3D, l.shs, l.colors_precomp, l.opacities, l.scales, l.scale_modifier,
		                            l.rotations, l.cov3D_precomp, const_cast<int*>(l.radii), l.geom_ws, l.geom_bytes};
	}
	return forward_geom(true, nullptr, "rgs_frame_forward_geom", K, calls.data(), view->width, view->height, view->viewmatrix,
	                    view->projmatrix, view->cam_pos, view->tan_fovx, view->tan_fovy, counts_pinned, stream, debug);
}

int rgs_frame_forward_raster(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, void* stream, int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_REQUIRE(K >= 1 && K <= RGS_MAX_FRAME_LAYERS && layers && view, "rgs_frame_forward_raster: K = %d outside 1..%d, or null", K,
	            RGS_MAX_FRAME_LAYERS);
	std::vector<rgs::BlendArgs> jobs((size_t)K);
	std::vector<RasterCall> calls((size_t)K);
	for (int k = 0; k < K; k++) {
		const rgs_frame_layer& l = layers[k];
		RGS_REQUIRE(l.out_color && l.out_depth && l.out_alpha, "rgs_frame_forward_raster: layer %d has a null output", k);
		calls[(size_t)k] = RasterCall{l.P, l.R, l.background, l.range_low, l.range_up, l.colors_precomp, l.geom_ws, l.geom_bytes,
		                              l.binning_ws, l.binning_bytes, l.image_ws, l.image_bytes};
	}
	if (int rc = forward_binning("rgs_frame_forward_raster", false, K, calls.data(), view->width, view->height, view->tan_fovx,
	                             view->tan_fovy, view->projmatrix_inv, jobs.data(), s, debug))
		return rc;
	for (int k = 0; k < K; k++) {
		jobs[(size_t)k].out_color = layers[k].out_color;
		jobs[(size_t)k].out_depth = layers[k].out_depth;
		jobs[(size_t)k].out_alpha = layers[k].out_alpha;
	}
	rgs::launch_blend_forward(jobs.data(), K, s);
	RGS_STAGE("blend_forward");
	return 0;
}

int rgs_frame_backward(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, void* stream, int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT("rgs_frame_backward");
	RGS_REQUIRE(K >= 1 && K <= RGS_MAX_FRAME_LAYERS && layers && view, "rgs_frame_backward: K = %d outside 1..%d, or null", K,
	            RGS_MAX_FRAME_LAYERS);
	const std::vector<hipStream_t> sides = side_streams(K, layers, s);
	// where the bandwidth-bound work goes; the stage timing charges the time between consecutive events of one stream,
	// so while it is on everything stays on the frame's stream
	hipStream_t beside = (sides.empty() || g_timer.on.load(std::memory_order_relaxed)) ? s : sides[0];
	std::vector<rgs::BlendArgs> jobs;
	std::vector<int> job_layer;
	std::vector<rgs::PreprocessBackwardArgs> geometry((size_t)K);
	std::vector<rgs::FillJob> sums_to_clear;
	for (int k = 0; k < K; k++) {
		const rgs_frame_layer& l = layers[k];
		if (int rc = check_backward_pointers("rgs_frame_backward", l.P, l.R, view->width, view->height, l.background, l.means3D,
		                                     l.shs, l.colors_precomp, l.out_alpha, l.scales, l.rotations, l.cov3D_precomp,
		                                     view->viewmatrix, view->projmatrix, view->projmatrix_inv, l.range_low, l.range_up,
		                                     view->cam_pos, l.radii, l.geom_ws, l.binning_ws, l.image_ws, l.dL_dpix, l.grad_accum,
		                                     l.dL_dmean2D, l.dL_dopacity, l.dL_dcolor, l.dL_dmean3D, l.dL_dcov3D, l.dL_dsh,
		                                     l.dL_dscale, l.dL_drot))
			return rc;
		if (!l.accum_zeroed)  // the blend adds into the rows of sums: they come first, on the frame's stream
			sums_to_clear.push_back(rgs::FillJob{reinterpret_cast<uint32_t*>(l.grad_accum), (size_t)RGS_ACC_FLOATS * (size_t)l.P});
		if (l.R > 0) {
			rgs::BlendArgs a;
			fill_blend_args(a, l.P, l.R, view->width, view->height, view->tan_fovx, view->tan_fovy, l.background,
			                view->projmatrix_inv, l.range_low, l.range_up, l.colors_precomp, l.geom_ws, l.binning_ws, l.image_ws);
			a.out_alpha = l.out_alpha;
			a.dL_dpix = l.dL_dpix; a.dL_dpix_depth = l.dL_dpix_depth; a.dL_dalpha = l.dL_dalphas;
			a.sums = l.grad_accum;
			jobs.push_back(a);
			job_layer.push_back(k);
		}
		fill_backward_geometry(geometry[(size_t)k], l.P, l.D, l.M, view->width, view->height, l.means3D, l.shs, l.scales,
		                       l.scale_modifier, l.rotations, l.cov3D_precomp, view->viewmatrix, view->projmatrix, view->cam_pos,
		                       view->tan_fovx, view->tan_fovy, l.radii, l.geom_ws, l.grad_accum, l.dL_dmean2D, l.dL_dopacity,
		                       l.dL_dcolor, l.dL_dmean3D, l.dL_dcov3D, l.dL_dsh, l.dL_dscale, l.dL_drot);
	}
	if (!sums_to_clear.empty()) {
		rgs::stage_mark("clear_gradients", s);
		rgs::launch_fill_many(sums_to_clear.data(), (int)sums_to_clear.size(), 0u, s);
		RGS_STAGE("clear gradient sums");
	}
	hipError_t e = hipSuccess;
	if (beside != s) {
		hipEvent_t begun = frame_event(0);
		e = begun ? hipEventRecord(begun, s) : hipErrorUnknown;
		if (e == hipSuccess)
			e = hipStreamWaitEvent(beside, begun, 0);
		if (e != hipSuccess)
			return fail("rgs_frame_backward: ordering the streams failed: %s", hipGetErrorString(e));
	}
	// With a second stream the blend goes in two halves, so that the per-Gaussian backward of the first half's layers
	// (memory bandwidth) runs beside the blend of the second half.  Layers without instances go with the last half.
	const int n_jobs = (int)jobs.size();
	const int halves = (beside != s && n_jobs >= 2) ? 2 : 1;
	const int first_half = halves == 2 ? (n_jobs + 1) / 2 : n_jobs;
	std::vector<char> in_first((size_t)K, 0);
	for (int i = 0; i < first_half; i++)
		in_first[(size_t)job_layer[(size_t)i]] = 1;
	for (int half = 0; half < halves; half++) {
		const int from = half == 0 ? 0 : first_half, to = half == 0 ? first_half : n_jobs;
		if (to > from) {
			rgs::launch_blend_backward(jobs.data() + from, to - from, s);
			RGS_STAGE("blend_backward");
		}
		std::vector<rgs::PreprocessBackwardArgs> part;
		for (int k = 0; k < K; k++)
			if (halves == 1 || (in_first[(size_t)k] != 0) == (half == 0))
				part.push_back(geometry[(size_t)k]);
		if (part.empty())
			continue;
		if (beside != s) {
			hipEvent_t blended = frame_event((size_t)(1 + half));
			e = blended ? hipEventRecord(blended, s) : hipErrorUnknown;
			if (e == hipSuccess)
				e = hipStreamWaitEvent(beside, blended, 0);
			if (e != hipSuccess)
				return fail("rgs_frame_backward: ordering the streams failed: %s", hipGetErrorString(e));
		}
		rgs::launch_preprocess_backward(part.data(), (int)part.size(), beside);
		RGS_STAGE("preprocess_backward");
	}
	if (beside != s) {
		hipEvent_t done = frame_event(3);
		e = done ? hipEventRecord(done, beside) : hipErrorUnknown;
		if (e == hipSuccess)
			e = hipStreamWaitEvent(s, done, 0);
		if (e != hipSuccess)
			return fail("rgs_frame_backward: ordering the streams failed: %s", hipGetErrorString(e));
	}
	return 0;
}

int rgs_blend_work_counters(int P, int R, int width, int height, float tan_fovx, float tan_fovy,
                            const float* projmatrix_inv, const float* range_low, const float* range_up,
                            const float* colors_precomp, const void* geom_ws, const void* binning_ws,
                            const void* image_ws, uint64_t* counters, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(P > 0 && R >= 0 && width > 0 && height > 0, "rgs_blend_work_counters: bad sizes");
	RGS_REQUIRE(projmatrix_inv && range_low && range_up && geom_ws && image_ws && counters && (R == 0 || binning_ws),
	            "rgs_blend_work_counters: null pointer");
	rgs::launch_fill_u32(reinterpret_cast<uint32_t*>(counters), 0u, 2 * RGS_WORK_COUNTERS, s);
	if (R == 0)
		return 0;
	rgs::BlendArgs a;
	fill_blend_args(a, P, R, width, height, tan_fovx, tan_fovy, range_low /* unused by the counting kernel */, projmatrix_inv,
	                range_low, range_up, colors_precomp, geom_ws, binning_ws, image_ws);
	a.counters = counters;
	rgs::launch_blend_count(a, s);
	RGS_STAGE("blend_count");
	return 0;
}

size_t rgs_scan_temp_bytes(size_t n)
{
	return 4 * rgs::scan_temp_words(n);
}

int rgs_inclusive_sum(const uint32_t* in, uint32_t* out, size_t n, void* temp, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	if (n == 0)
		return 0;
	RGS_REQUIRE(in && out && temp, "rgs_inclusive_sum: null pointer");
	RGS_REQUIRE(n < ((size_t)1 << 38), "rgs_inclusive_sum: n too large");
	rgs::launch_inclusive_sum(in, out, n, static_cast<uint32_t*>(temp), "inclusive_sum", s);
	RGS_STAGE("inclusive_sum");
	return 0;
}

size_t rgs_sort_temp_bytes(size_t n)
{
	return 4 * rgs::sort_temp_words(n);
}

// fault: pinned host word (may be null); device_fault: a word of device memory (may be null).  A sort that gave up sets both.
static int sort_pairs_u64(const char* who, uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                          size_t n, int end_bit, uint32_t* temp, uint32_t* fault, uint32_t* device_fault, hipStream_t s)
{
	const int debug = 0;
	rgs::launch_sort_pairs(keys_in, keys_out, vals_in, vals_out, n, end_bit, temp, s);
	RGS_STAGE("sort_pairs");
	rgs::launch_report_sort_status(temp, fault, device_fault, s);
	if ((rgs::sort_passes(end_bit, rgs::kDigitBitsU64) % 2) == 0) {
		// An even number of passes leaves the result in the input buffers; hand it over.
		hipError_t e = hipMemcpyAsync(keys_out, keys_in, n * sizeof(uint64_t), hipMemcpyDeviceToDevice, s);
		if (e == hipSuccess)
			e = hipMemcpyAsync(vals_out, vals_in, n * sizeof(uint32_t), hipMemcpyDeviceToDevice, s);
		if (e != hipSuccess)
			return fail("%s: copy failed: %s", who, hipGetErrorString(e));
	}
	return 0;
}

int rgs_sort_pairs(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                   int end_bit, void* temp, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_REQUIRE(end_bit >= 1 && end_bit <= 64, "rgs_sort_pairs: end_bit %d out of range", end_bit);
	if (n == 0)
		return 0;
	RGS_REQUIRE(keys_in && keys_out && vals_in && vals_out && temp, "rgs_sort_pairs: null pointer");
	RGS_REQUIRE(n < 0x40000000ull, "rgs_sort_pairs: 2^30 pairs or more");
	return sort_pairs_u64("rgs_sort_pairs", keys_in, keys_out, vals_in, vals_out, n, end_bit, static_cast<uint32_t*>(temp),
	                      fault_word(true), nullptr, s);
}

int rgs_sort_pairs_static(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                          int end_bit, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_REQUIRE(end_bit >= 1 && end_bit <= 64, "rgs_sort_pairs_static: end_bit %d out of range", end_bit);
	RGS_REQUIRE(n <= (size_t)RGS_STATIC_SORT_MAX_PAIRS,
	            "rgs_sort_pairs_static: %zu pairs exceed the %d the library's own scratch has room for (use rgs_sort_pairs "
	            "with a workspace)", n, RGS_STATIC_SORT_MAX_PAIRS);
	if (n == 0)
		return 0;
	RGS_REQUIRE(keys_in && keys_out && vals_in && vals_out, "rgs_sort_pairs_static: null pointer");
	RGS_REQUIRE(rgs::sort_temp_words(n) <= kStaticSortWords, "rgs_sort_pairs_static: scratch layout mismatch");
	uint32_t* temp = nullptr;
	uint32_t* gave_up = nullptr;
	if (int rc = static_sort_scratch(&temp, &gave_up))
		return rc;
	// Nothing is allocated here: a give-up is reported in a word of device memory beside the scratch, which
	// rgs_sort_fault reads, and also in the pinned word of the other entry points if an earlier call has set that up.
	return sort_pairs_u64("rgs_sort_pairs_static", keys_in, keys_out, vals_in, vals_out, n, end_bit, temp, fault_word(false), gave_up,
	                      s);
}

int rgs_set_lookback_spin_limit(int polls)
{
	rgs::set_lookback_spin_limit(polls);
	return 0;
}

int rgs_sort_fault(void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	const hipError_t e = hipStreamSynchronize(s);
	if (e != hipSuccess)
		return fail("rgs_sort_fault: %s", hipGetErrorString(e));
	const int pinned = take_sort_fault("rgs_sort_fault");
	const int in_device_memory = take_static_sort_fault("rgs_sort_fault");  // read (and cleared) either way
	return pinned ? pinned : in_device_memory;
}

static int fill_composite(rgs::CompositeArgs& a, int K, int height, int width, const float* const* images,
                          const float* const* depths, const float* const* alphas, const float* background)
{
	RGS_REQUIRE(K >= 1 && K <= RGS_MAX_COMPOSITE, "composite: K=%d outside 1..%d", K, RGS_MAX_COMPOSITE);
	RGS_REQUIRE(height > 0 && width > 0, "composite: bad image size %dx%d", width, height);
	RGS_REQUIRE(images && depths && alphas, "composite: null pointer table");
	memset(&a, 0, sizeof(a));
	a.K = K; a.H = height; a.W = width; a.bg = background;
	for (int k = 0; k < K; k++) {
		RGS_REQUIRE(images[k] && depths[k] && alphas[k], "composite: null input plane at k=%d", k);
		a.images[k] = images[k];
		a.depths[k] = depths[k];
		a.alphas[k] = alphas[k];
	}
	return 0;
}

int rgs_composite_forward(int K, int height, int width,
                          const float* const* images, const float* const* depths, const float* const* alphas,
                          const float* background, float* out_image, float* out_depth, float* out_alpha,
                          void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	rgs::CompositeArgs a;
	if (int rc = fill_composite(a, K, height, width, images, depths, alphas, background))
		return rc;
	RGS_REQUIRE(out_image && out_depth && out_alpha, "rgs_composite_forward: null output");
	a.out_image = out_image; a.out_depth = out_depth; a.out_alpha = out_alpha;
	rgs::launch_composite_forward(a, s);
	RGS_STAGE("composite_forward");
	return 0;
}

int rgs_composite_backward(int K, int height, int width,
                           const float* const* images, const float* const* depths, const float* const* alphas,
                           const float* background, const float* g_image, const float* g_depth,
                           const float* g_alpha, float* const* d_images, float* const* d_depths,
                           float* const* d_alphas, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	rgs::CompositeArgs a;
	if (int rc = fill_composite(a, K, height, width, images, depths, alphas, background))
		return rc;
	RGS_REQUIRE(g_image && d_images && d_depths && d_alphas, "rgs_composite_backward: null pointer");
	a.g_image = g_image; a.g_depth = g_depth; a.g_alpha = g_alpha;
	for (int k = 0; k < K; k++) {
		RGS_REQUIRE(d_images[k] && d_depths[k] && d_alphas[k], "rgs_composite_backward: null output plane at k=%d", k);
		a.d_images[k] = d_images[k];
		a.d_depths[k] = d_depths[k];
		a.d_alphas[k] = d_alphas[k];
	}
	rgs::launch_composite_backward(a, s);
	RGS_STAGE("composite_backward");
	return 0;
}

size_t rgs_straddler_scratch_bytes(int n, int n_boxes)
{
	if (n < 0 || n_boxes < 0)
		return 0;
	return sizeof(uint32_t) * (size_t)n_boxes * (rgs::straddler_select_blocks(n) + 1);
}

int rgs_straddler_select(int n, const float* means3D, const float* scales, const float* src_low, const float* src_up,
                         int n_boxes, const float* boxes_low, const float* boxes_up, int skip, uint32_t* counts,
                         uint32_t* rows, uint32_t capacity, void* scratch, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n >= 0, "rgs_straddler_select: negative n");
	RGS_REQUIRE(n_boxes >= 1 && n_boxes <= rgs::kMaxShareBoxes, "rgs_straddler_select: n_boxes = %d, must be 1..%d", n_boxes,
	            rgs::kMaxShareBoxes);
	RGS_REQUIRE(skip >= -1 && skip < n_boxes, "rgs_straddler_select: skip = %d is not a box", skip);
	RGS_REQUIRE(src_low && src_up && boxes_low && boxes_up, "rgs_straddler_select: null box");
	RGS_REQUIRE(counts && scratch, "rgs_straddler_select: null counts or scratch");
	RGS_REQUIRE(n == 0 || (means3D && scales), "rgs_straddler_select: null input");
	RGS_REQUIRE(capacity == 0 || rows, "rgs_straddler_select: null rows");
	rgs::StraddlerSelectArgs a;
	a.n = n;
	a.means3D = means3D;
	a.scales = scales;
	for (int c = 0; c < 3; c++) {
		a.src_low[c] = src_low[c];
		a.src_up[c] = src_up[c];
	}
	a.boxes.count = n_boxes;
	for (int b = 0; b < n_boxes; b++)
		for (int c = 0; c < 3; c++) {
			a.boxes.low[b][c] = boxes_low[3 * b + c];
			a.boxes.up[b][c] = boxes_up[3 * b + c];
		}
	a.skip = skip;
	a.block_counts = static_cast<uint32_t*>(scratch);
	a.counts = counts;
	a.rows = rows;
	a.capacity = capacity;
	rgs::launch_straddler_select(a, s);
	RGS_STAGE("straddler_select");
	return 0;
}

namespace {
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
}

int rgs_merge_rows(int n_segments, const rgs_shared_rows* segments, uint32_t dst_row0, int sh_floats, float* means3D,
                   float* opacity, float* scales, float* rotations, float* shs, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n_segments >= 0 && (n_segments == 0 || segments), "rgs_merge_rows: bad segment list");
	RGS_REQUIRE(sh_floats >= 0, "rgs_merge_rows: negative sh_floats");
	uint64_t total = dst_row0;
	for (int i = 0; i < n_segments; i++) {
		const rgs_shared_rows& g = segments[i];
		RGS_REQUIRE(g.count == 0 || (g.means3D && g.opacity && g.scales && g.rotations && (g.shs || sh_floats == 0)),
		            "rgs_merge_rows: null field in segment %d", i);
		total += g.count;
	}
	RGS_REQUIRE(total <= 0xffffffffull, "rgs_merge_rows: more than 2^32 rows");
	if (total == dst_row0)
		return 0;
	RGS_REQUIRE(means3D && opacity && scales && rotations && (shs || sh_floats == 0), "rgs_merge_rows: null destination");
	uint32_t row0 = dst_row0;
	int i = 0;
	while (i < n_segments) {
		rgs::MergeArgs a;
		a.segments = 0;
		a.sh_floats = sh_floats;
		a.means3D = means3D; a.opacity = opacity; a.scales = scales; a.rotations = rotations; a.shs = shs;
		bool wide = sh_floats % 4 == 0 && aligned16(shs) && aligned16(rotations);
		uint32_t blocks = 0;
		for (; i < n_segments && a.segments < rgs::kMaxMergeSegments; i++) {
			const rgs_shared_rows& g = segments[i];
			if (g.count == 0)
				continue;
			rgs::MergeSegment& m = a.seg[a.segments++];
			m.means3D = g.means3D; m.opacity = g.opacity; m.scales = g.scales; m.rotations = g.rotations; m.shs = g.shs;
			m.rows = g.rows;
			m.count = g.count;
			m.dst_row0 = row0;
			m.block0 = blocks;
			wide = wide && aligned16(g.shs) && aligned16(g.rotations);
			row0 += g.count;
			blocks += rgs::merge_blocks_for(g.count);
		}
		rgs::launch_merge_rows(a, blocks, wide, s);
		RGS_STAGE("merge_rows");
	}
	return 0;
}

int rgs_merge_rows_backward(int n_segments, const rgs_shared_grads* segments, uint32_t dst_row0, int sh_floats,
                            const float* g_means3D, const float* g_means2D, const float* g_opacity, const float* g_scales,
                            const float* g_rotations, const float* g_shs, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n_segments >= 0 && (n_segments == 0 || segments), "rgs_merge_rows_backward: bad segment list");
	RGS_REQUIRE(sh_floats >= 0, "rgs_merge_rows_backward: negative sh_floats");
	uint64_t total = dst_row0;
	for (int i = 0; i < n_segments; i++) {
		RGS_REQUIRE(segments[i].count == 0 || segments[i].rows, "rgs_merge_rows_backward: segment %d has no row list", i);
		total += segments[i].count;
	}
	RGS_REQUIRE(total <= 0xffffffffull, "rgs_merge_rows_backward: more than 2^32 rows");
	uint32_t row0 = dst_row0;
	int i = 0;
	while (i < n_segments) {
		rgs::MergeBackwardArgs a;
		a.segments = 0;
		a.sh_floats = sh_floats;
		a.means3D = g_means3D; a.means2D = g_means2D; a.opacity = g_opacity; a.scales = g_scales;
		a.rotations = g_rotations; a.shs = g_shs;
		bool wide = sh_floats % 4 == 0 && aligned16(g_shs) && aligned16(g_rotations);
		uint32_t blocks = 0;
		for (; i < n_segments && a.segments < rgs::kMaxMergeSegments; i++) {
			const rgs_shared_grads& g = segments[i];
			if (g.count == 0)
				continue;
			rgs::MergeBackwardSegment& m = a.seg[a.segments++];
			m.means3D = g.means3D; m.means2D = g.means2D; m.opacity = g.opacity; m.scales = g.scales;
			m.rotations = g.rotations; m.shs = g.shs;
			m.rows = g.rows;
			m.count = g.count;
			m.dst_row0 = row0;
			m.block0 = blocks;
			wide = wide && aligned16(g.shs) && aligned16(g.rotations);
			row0 += g.count;
			blocks += rgs::merge_blocks_for(g.count);
		}
		rgs::launch_merge_rows_backward(a, blocks, wide, s);
		RGS_STAGE("merge_rows_backward");
	}
	return 0;
}

namespace {

size_t loss_map_floats(int C, int H, int W) { return (size_t)3 * C * H * W; }

int fill_loss(rgs::LossArgs& a, const char* who, int C, int H, int W, const float* image, const float* gt, float lambda,
              const void* workspace)
{
	RGS_REQUIRE(C >= 1 && H >= 1 && W >= 1, "%s: bad image size %dx%dx%d", who, C, H, W);
	RGS_REQUIRE((size_t)C * H * W < (1ull << 31), "%s: image too large", who);
	RGS_REQUIRE(image && gt && workspace, "%s: null pointer", who);
	a.C = C; a.H = H; a.W = W;
	a.x = image;
	a.y = gt;
	a.lambda = lambda;
	// utils/loss_utils.py:23-25: exp in double, stored as float, normalised in float
	float g[11], sum = 0.f;
	for (int i = 0; i < 11; i++) {
		g[i] = (float)exp(-(double)((i - 5) * (i - 5)) / (2.0 * 1.5 * 1.5));
		sum += g[i];
	}
	for (int i = 0; i < 11; i++)
		a.w[i] = g[i] / sum;
	float* ws = static_cast<float*>(const_cast<void*>(workspace));
	a.maps = ws;
	a.partial = ws + loss_map_floats(C, H, W);
	a.out = nullptr;
	a.grad_loss = nullptr;
	a.d_image = nullptr;
	return 0;
}

}  // namespace

size_t rgs_loss_workspace_bytes(int channels, int height, int width)
{
	if (channels < 1 || height < 1 || width < 1)
		return 0;
	return sizeof(float) * (loss_map_floats(channels, height, width) + 2 * (size_t)rgs::loss_blocks(channels, height, width));
}

int rgs_l1_ssim_forward(int channels, int height, int width, const float* image, const float* gt, float lambda_dssim,
                        float* out, void* workspace, int keep_for_backward, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	rgs::LossArgs a;
	if (int rc = fill_loss(a, "rgs_l1_ssim_forward", channels, height, width, image, gt, lambda_dssim, workspace))
		return rc;
	RGS_REQUIRE(out, "rgs_l1_ssim_forward: null output");
	a.out = out;
	if (!keep_for_backward)
		a.maps = nullptr;
	rgs::launch_l1_ssim_forward(a, s);
	RGS_STAGE("l1_ssim_forward");
	return 0;
}

int rgs_l1_ssim_backward(int channels, int height, int width, const float* image, const float* gt, float lambda_dssim,
                         const float* grad_loss, const void* workspace, float* d_image, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	rgs::LossArgs a;
	if (int rc = fill_loss(a, "rgs_l1_ssim_backward", channels, height, width, image, gt, lambda_dssim, workspace))
		return rc;
	RGS_REQUIRE(d_image, "rgs_l1_ssim_backward: null output");
	a.grad_loss = grad_loss;
	a.d_image = d_image;
	rgs::launch_l1_ssim_backward(a, s);
	RGS_STAGE("l1_ssim_backward");
	return 0;
}

int rgs_activate_forward(int n, int rest, const float* features_dc, const float* features_rest, const float* scaling,
                         const float* rotation, const float* opacity, float* shs, float* scales, float* rotations,
                         float* opacities, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n >= 0 && rest >= 0, "rgs_activate_forward: bad sizes n=%d rest=%d", n, rest);
	if (n == 0)
		return 0;
	RGS_REQUIRE(features_dc && (features_rest || rest == 0) && scaling && rotation && opacity && shs && scales && rotations &&
	                opacities,
	            "rgs_activate_forward: null pointer");
	RGS_REQUIRE(aligned16(scaling) && aligned16(rotation) && aligned16(opacity) && aligned16(shs) && aligned16(scales) &&
	                aligned16(rotations) && aligned16(opacities),
	            "rgs_activate_forward: arrays must start at multiples of 16 bytes");
	rgs::ActivateArgs a;
	a.n = n; a.rest = rest;
	a.features_dc = features_dc; a.features_rest = features_rest; a.scaling = scaling; a.rotation = rotation;
	a.opacity = opacity;
	a.shs = shs; a.scales = scales; a.rotations = rotations; a.opacities = opacities;
	rgs::launch_activate_forward(a, s);
	RGS_STAGE("activate_forward");
	return 0;
}

int rgs_activate_backward(int n, int rest, const float* rotation, const float* scales, const float* opacities,
                          const float* g_shs, const float* g_scales, const float* g_rotations, const float* g_opacities,
                          float* d_features_dc, float* d_features_rest, float* d_scaling, float* d_rotation,
                          float* d_opacity, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n >= 0 && rest >= 0, "rgs_activate_backward: bad sizes n=%d rest=%d", n, rest);
	if (n == 0)
		return 0;
	RGS_REQUIRE(!g_shs || (d_features_dc && (d_features_rest || rest == 0)), "rgs_activate_backward: no room for the SH gradients");
	RGS_REQUIRE(!g_scales || (scales && d_scaling), "rgs_activate_backward: scales or their gradient missing");
	RGS_REQUIRE(!g_rotations || (rotation && d_rotation), "rgs_activate_backward: rotation or its gradient missing");
	RGS_REQUIRE(!g_opacities || (opacities && d_opacity), "rgs_activate_backward: opacities or their gradient missing");
	RGS_REQUIRE(aligned16(rotation) && aligned16(scales) && aligned16(opacities) && aligned16(g_shs) && aligned16(g_scales) &&
	                aligned16(g_rotations) && aligned16(g_opacities) && aligned16(d_scaling) && aligned16(d_rotation) &&
	                aligned16(d_opacity),
	            "rgs_activate_backward: arrays must start at multiples of 16 bytes");
	rgs::ActivateBackwardArgs a;
	a.n = n; a.rest = rest;
	a.rotation = rotation; a.scales = scales; a.opacities = opacities;
	a.g_shs = g_shs; a.g_scales = g_scales; a.g_rotations = g_rotations; a.g_opacities = g_opacities;
	a.d_features_dc = d_features_dc; a.d_features_rest = d_features_rest; a.d_scaling = d_scaling;
	a.d_rotation = d_rotation; a.d_opacity = d_opacity;
	rgs::launch_activate_backward(a, s);
	RGS_STAGE("activate_backward");
	return 0;
}

int rgs_adam_step(int n_tensors, const rgs_adam_tensor* tensors, double beta1, double beta2, double eps, void* stream)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	const int debug = 0;
	RGS_REQUIRE(n_tensors >= 0 && (n_tensors == 0 || tensors), "rgs_adam_step: bad tensor list");
	for (int i = 0; i < n_tensors; i++) {
		const rgs_adam_tensor& t = tensors[i];
		RGS_REQUIRE(t.n == 0 || (t.param && t.grad && t.exp_avg && t.exp_avg_sq), "rgs_adam_step: null array in tensor %d", i);
		RGS_REQUIRE(t.step >= 1, "rgs_adam_step: tensor %d has step %d; the count includes this update", i, t.step);
	}
	int i = 0;
	while (i < n_tensors) {
		rgs::AdamArgs a;
		a.tensors = 0;
		a.beta1 = (float)beta1; a.beta2 = (float)beta2; a.eps = (float)eps;
		a.one_minus_beta1 = (float)(1.0 - beta1); a.one_minus_beta2 = (float)(1.0 - beta2);
		uint32_t blocks = 0;
		for (; i < n_tensors && a.tensors < rgs::kMaxAdamTensors; i++) {
			const rgs_adam_tensor& t = tensors[i];
			if (t.n == 0)
				continue;
			rgs::AdamTensor& k = a.t[a.tensors++];
			k.param = t.param; k.grad = t.grad; k.exp_avg = t.exp_avg; k.exp_avg_sq = t.exp_avg_sq;
			k.n = t.n;
			// torch/optim/adam.py: bias corrections and step size in double, applied as floats
			const double c1 = 1.0 - pow(beta1, (double)t.step), c2 = 1.0 - pow(beta2, (double)t.step);
			k.step_size = (float)(t.lr / c1);
			k.bias2_sqrt = (float)sqrt(c2);
			k.block0 = blocks;
			k.by_16_bytes = aligned16(t.param) && aligned16(t.grad) && aligned16(t.exp_avg) && aligned16(t.exp_avg_sq);
			blocks += rgs::adam_blocks_for(t.n);
		}
		rgs::launch_adam_step(a, blocks, s);
		RGS_STAGE("adam_step");
	}
	return 0;
}

}  // extern "C"
