// extern "C" surface of librgs_gfx950.so: argument checks, workspace carving, stage
// sequencing and error reporting.  The declarations and the reference interfaces they
// replace are in include/rgs.h.
#include "../../include/rgs.h"
#include "rgs_kernels.h"

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
struct StageTimer {
	bool on = false;
	std::vector<hipEvent_t> pool;
	std::vector<const char*> tags;  // tag of event i; nullptr closes an entry point
	size_t used = 0;
};
StageTimer g_timer;
constexpr size_t kMaxTimerEvents = 1 << 16;

void timer_record(const char* tag, hipStream_t s)
{
	if (!g_timer.on || g_timer.used >= kMaxTimerEvents)
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

// Device address of this device's copy of `scratch`, looked up once per device with that device current.
int static_sort_scratch(uint32_t** out)
{
	const int dev = current_device();
	if (dev < 0)
		return fail("rgs_sort_pairs_static: no current device");
	std::lock_guard<std::mutex> lock(g_device_mutex);
	if (!g_static_scratch[dev]) {
		void* p = nullptr;
		const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
		if (e != hipSuccess || !p)
			return fail("rgs_sort_pairs_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
		g_static_scratch[dev] = static_cast<uint32_t*>(p);
	}
	*out = g_static_scratch[dev];
	return 0;
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
	size_t keys_a, keys_b, vals_b, tiles_in_order, sort_temp, scan_temp, total;
};

OrderScratch order_scratch(size_t P)
{
	Carver c;
	OrderScratch o;
	o.keys_a = c.take(4 * P);
	o.keys_b = c.take(4 * P);
	o.vals_b = c.take(4 * P);
	o.tiles_in_order = c.take(4 * P);
	o.sort_temp = c.take(4 * rgs::sort_temp_words(P));
	o.scan_temp = c.take(4 * rgs::scan_temp_words(P));
	o.total = c.cursor;
	return o;
}

size_t geom_layout(size_t P, size_t* off)
{
	Carver c;
	off[RGS_GEOM_DEPTHS] = c.take(4 * P);
	off[RGS_GEOM_XY] = c.take(8 * P);
	off[RGS_GEOM_CLIP_W] = c.take(4 * P);
	off[RGS_GEOM_COV3D] = c.take(24 * P);
	off[RGS_GEOM_CONIC_OPACITY] = c.take(16 * P);
	off[RGS_GEOM_RGB] = c.take(12 * P);
	off[RGS_GEOM_TILES_TOUCHED] = c.take(4 * P);
	off[RGS_GEOM_POINT_OFFSETS] = c.take(4 * P);
	off[RGS_GEOM_CLAMPED] = c.take(P);
	off[RGS_GEOM_BLOCK_SUMS] = c.take(4 * ((P + 255) / 256 + 1));
	off[RGS_GEOM_TOTAL] = c.take(4);
	off[RGS_GEOM_BLEND_RECORD] = c.take(64 * P);
	off[RGS_GEOM_DEPTH_ORDER] = c.take(4 * P);
	off[RGS_GEOM_BLOCK_VISIBLE] = c.take(4 * ((P + 255) / 256 + 1));
	off[RGS_GEOM_VISIBLE_COUNT] = c.take(4);
	off[RGS_GEOM_VISIBLE_LIST] = c.take(4 * P);
	off[RGS_GEOM_ORDER_SCRATCH] = c.take(order_scratch(P).total);
	return c.cursor;
}

// Bits of the tile key that the instance sort looks at.
int tile_key_bits(int width, int height)
{
	const uint32_t tiles = (uint32_t)((width + rgs::kTile - 1) / rgs::kTile) * (uint32_t)((height + rgs::kTile - 1) / rgs::kTile);
	return (int)rgs_get_higher_msb(tiles);
}

// Physical buffers: A receives the duplicated keys, B is its ping-pong partner.
struct BinningPhysical {
	size_t keys_a, keys_b, vals_a, vals_b, temp, strip_lists, total;
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
	b.total = c.cursor;
	return b;
}

size_t image_layout(int width, int height, size_t* off)
{
	const size_t tiles = (size_t)((width + rgs::kTile - 1) / rgs::kTile) * (size_t)((height + rgs::kTile - 1) / rgs::kTile);
	Carver c;
	off[RGS_IMG_RANGES] = c.take(8 * tiles + 4 * rgs::kRangeTailWords);  // + the strip class counters, cleared with it
	off[RGS_IMG_N_CONTRIB] = c.take(4 * (size_t)width * height);
	off[RGS_IMG_STRIP_FILED] = c.take(4 * 4 * tiles);
	off[RGS_IMG_STRIP_ORDER] = c.take(4 * 4 * tiles);
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
	g_timer.on = enable != 0;
	g_timer.used = 0;
	return 0;
}

int rgs_stage_timing_read(int max_stages, const char** names, float* total_ms, int* launches)
{
	RGS_REQUIRE(max_stages >= 0 && (max_stages == 0 || (names && total_ms && launches)), "rgs_stage_timing_read: bad arguments");
	int n = 0;
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
	const bool sorted_in_a = (((tile_key_bits(width, height) + 7) / 8) % 2) == 0;
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

static int forward_geom(bool wait_for_count, void* count_ready_event, const char* who, int P, int D, int M, int width, int height,
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
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT(who);
	RGS_REQUIRE(P > 0, "%s: P must be positive (the caller short-circuits P == 0)", who);
	RGS_REQUIRE(width > 0 && height > 0, "%s: bad image size %dx%d", who, width, height);
	RGS_REQUIRE(means3D && opacities && viewmatrix && projmatrix && cam_pos && radii && geom_ws && num_rendered_host,
	            "%s: null pointer", who);
	RGS_REQUIRE((shs != nullptr) != (colors_precomp != nullptr),
	            "%s: provide exactly one of SHs or precomputed colours", who);
	RGS_REQUIRE(((scales != nullptr) && (rotations != nullptr)) != (cov3D_precomp != nullptr) &&
	                ((scales != nullptr) == (rotations != nullptr)),
	            "%s: provide exactly one of scale/rotation or precomputed 3D covariance", who);
	RGS_REQUIRE(D >= 0 && D <= 3, "%s: SH degree %d out of range", who, D);
	RGS_REQUIRE(!shs || M >= (D + 1) * (D + 1), "%s: %d SH coefficients cannot hold degree %d", who, M, D);
	RGS_REQUIRE(geom_bytes >= rgs_geom_bytes(P), "%s: geometry workspace too small", who);
	RGS_REQUIRE((reinterpret_cast<uintptr_t>(geom_ws) & 15) == 0, "%s: workspace must be 16-byte aligned", who);

	size_t off[RGS_GEOM_FIELDS];
	geom_layout((size_t)P, off);

	rgs::PreprocessArgs a;
	a.P = P; a.D = D; a.M = M;
	a.means = means3D; a.scales = scales; a.scale_modifier = scale_modifier; a.rotations = rotations;
	a.opacities = opacities; a.shs = shs; a.cov3D_precomp = cov3D_precomp; a.colors_precomp = colors_precomp;
	a.view = viewmatrix; a.proj = projmatrix; a.campos = cam_pos;
	a.W = width; a.H = height;
	a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
	// K/cuda_rasterizer_hgs/rasterizer_impl.cu:227-228
	a.focal_y = height / (2.0f * tan_fovy);
	a.focal_x = width / (2.0f * tan_fovx);
	a.grid_x = (width + rgs::kTile - 1) / rgs::kTile;
	a.grid_y = (height + rgs::kTile - 1) / rgs::kTile;
	a.radii = radii;
	a.xy = at<float2>(geom_ws, off[RGS_GEOM_XY]);
	a.clip_w = at<float>(geom_ws, off[RGS_GEOM_CLIP_W]);
	a.depths = at<float>(geom_ws, off[RGS_GEOM_DEPTHS]);
	a.cov3D = at<float>(geom_ws, off[RGS_GEOM_COV3D]);
	a.rgb = at<float>(geom_ws, off[RGS_GEOM_RGB]);
	a.conic_opacity = at<float4>(geom_ws, off[RGS_GEOM_CONIC_OPACITY]);
	a.tiles_touched = at<uint32_t>(geom_ws, off[RGS_GEOM_TILES_TOUCHED]);
	a.clamped = at<uint8_t>(geom_ws, off[RGS_GEOM_CLAMPED]);
	a.block_sums = at<uint32_t>(geom_ws, off[RGS_GEOM_BLOCK_SUMS]);
	a.blend_record = at<float4>(geom_ws, off[RGS_GEOM_BLEND_RECORD]);
	a.block_visible = at<uint32_t>(geom_ws, off[RGS_GEOM_BLOCK_VISIBLE]);
	a.sh_rows_by_16_bytes = sh_rows_by_16_bytes(shs, M, D);

	const OrderScratch order = order_scratch((size_t)P);
	a.clear = at<uint32_t>(at<char>(geom_ws, off[RGS_GEOM_ORDER_SCRATCH]), order.sort_temp);
	a.clear_words = rgs::sort_clear_words((size_t)P, 32);
	rgs::launch_preprocess_forward(a, s);
	RGS_STAGE("preprocess");
	rgs::launch_totals_from_block_sums(a.block_sums, a.block_visible, P, at<uint32_t>(geom_ws, off[RGS_GEOM_TOTAL]),
	                                   at<uint32_t>(geom_ws, off[RGS_GEOM_VISIBLE_COUNT]), s);
	RGS_STAGE("instance count");
	hipError_t e = hipMemcpyAsync(num_rendered_host, at<uint32_t>(geom_ws, off[RGS_GEOM_TOTAL]), sizeof(uint32_t),
	                              hipMemcpyDeviceToHost, s);
	// the host only needs the count: it waits for this event, not for the kernels queued below
	hipEvent_t ready = wait_for_count ? count_event_of_this_thread() : static_cast<hipEvent_t>(count_ready_event);
	if (e == hipSuccess && ready)
		e = hipEventRecord(ready, s);
	{
		// depth order of the Gaussians and the offsets of their instances in that order: needs
		// nothing from the host, so it is queued behind the count's copy
		const OrderScratch& o = order;
		char* scratch = at<char>(geom_ws, off[RGS_GEOM_ORDER_SCRATCH]);
		rgs::launch_depth_order(P, a.depths, a.tiles_touched, a.block_visible, at<uint32_t>(geom_ws, off[RGS_GEOM_VISIBLE_COUNT]),
		                        at<uint32_t>(geom_ws, off[RGS_GEOM_VISIBLE_LIST]),
		                        at<uint32_t>(scratch, o.keys_a), at<uint32_t>(scratch, o.keys_b),
		                        at<uint32_t>(geom_ws, off[RGS_GEOM_DEPTH_ORDER]), at<uint32_t>(scratch, o.vals_b),
		                        at<uint32_t>(scratch, o.tiles_in_order), at<uint32_t>(geom_ws, off[RGS_GEOM_POINT_OFFSETS]),
		                        at<uint32_t>(scratch, o.sort_temp), at<uint32_t>(scratch, o.scan_temp), s);
		RGS_STAGE("depth order");
	}
	if (e == hipSuccess && wait_for_count)
		e = ready ? hipEventSynchronize(ready) : hipStreamSynchronize(s);
	if (e != hipSuccess)
		return fail("%s: reading the instance count failed: %s", who, hipGetErrorString(e));
	if (wait_for_count)
		RGS_REQUIRE(*num_rendered_host < 0x40000000u,
		            "%s: %u (Gaussian, tile) instances exceed the 2^30 limit of the sort", who, *num_rendered_host);
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
	return forward_geom(true, nullptr, "rgs_forward_geom", P, D, M, width, height, means3D, shs, colors_precomp, opacities, scales,
	                    scale_modifier, rotations, cov3D_precomp, viewmatrix, projmatrix, cam_pos, tan_fovx, tan_fovy,
	                    prefiltered, radii, geom_ws, geom_bytes, num_rendered_host, stream, debug);
}

int rgs_forward_geom_enqueue(int P, int D, int M, int width, int height,
                             const float* means3D, const float* shs, const float* colors_precomp,
                             const float* opacities, const float* scales, float scale_modifier, const float* rotations,
                             const float* cov3D_precomp, const float* viewmatrix, const float* projmatrix,
                             const float* cam_pos, float tan_fovx, float tan_fovy, int prefiltered,
                             int* radii, void* geom_ws, size_t geom_bytes,
                             uint32_t* num_rendered_pinned, void* count_ready_event, void* stream, int debug)
{
	return forward_geom(false, count_ready_event, "rgs_forward_geom_enqueue", P, D, M, width, height, means3D, shs, colors_precomp, opacities,
	                    scales, scale_modifier, rotations, cov3D_precomp, viewmatrix, projmatrix, cam_pos, tan_fovx,
	                    tan_fovy, prefiltered, radii, geom_ws, geom_bytes, num_rendered_pinned, stream, debug);
}


}  // extern "C"

namespace {

// `R` sizes the binning workspace and the launches.  With count_on_device the number of instances
// is the smaller of R and the count the geometry stage left in its workspace, read by the kernels.
int forward_raster(bool count_on_device, int P, int R, int width, int height,
                   const float* background, float tan_fovx, float tan_fovy,
                   const float* projmatrix_inv, const float* range_low, const float* range_up,
                   const float* colors_precomp, const int* radii,
                   void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                   void* image_ws, size_t image_bytes,
                   float* out_color, float* out_depth, float* out_alpha, void* stream, int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT("rgs_forward_raster");
	RGS_REQUIRE(P > 0 && R >= 0, "rgs_forward_raster: bad sizes P=%d R=%d", P, R);
	RGS_REQUIRE(R < 0x40000000, "rgs_forward_raster: %d (Gaussian, tile) instances exceed the 2^30 limit of the sort", R);
	RGS_REQUIRE(width > 0 && height > 0, "rgs_forward_raster: bad image size %dx%d", width, height);
	RGS_REQUIRE(background && projmatrix_inv && range_low && range_up && radii && geom_ws && image_ws && out_color &&
	                out_depth && out_alpha,
	            "rgs_forward_raster: null pointer");
	RGS_REQUIRE(R == 0 || binning_ws, "rgs_forward_raster: null binning workspace");
	RGS_REQUIRE(geom_bytes >= rgs_geom_bytes(P), "rgs_forward_raster: geometry workspace too small");
	RGS_REQUIRE(R == 0 || binning_bytes >= rgs_binning_bytes(R), "rgs_forward_raster: binning workspace too small");
	RGS_REQUIRE(image_bytes >= rgs_image_bytes(width, height), "rgs_forward_raster: image workspace too small");

	size_t goff[RGS_GEOM_FIELDS], ioff[RGS_IMG_FIELDS];
	geom_layout((size_t)P, goff);
	image_layout(width, height, ioff);
	const int gx = (width + rgs::kTile - 1) / rgs::kTile, gy = (height + rgs::kTile - 1) / rgs::kTile;
	uint2* ranges = at<uint2>(image_ws, ioff[RGS_IMG_RANGES]);
	const uint32_t* point_list = nullptr;

	if (R > 0) {
		const BinningPhysical b = binning_physical((size_t)R);
		uint32_t* keys_a = at<uint32_t>(binning_ws, b.keys_a);
		uint32_t* keys_b = at<uint32_t>(binning_ws, b.keys_b);
		uint32_t* vals_a = at<uint32_t>(binning_ws, b.vals_a);
		uint32_t* vals_b = at<uint32_t>(binning_ws, b.vals_b);
		const uint32_t* order_status =
		    rgs::sort_status_word(at<uint32_t>(at<char>(geom_ws, goff[RGS_GEOM_ORDER_SCRATCH]), order_scratch((size_t)P).sort_temp));
		const uint32_t* count = count_on_device ? at<uint32_t>(geom_ws, goff[RGS_GEOM_TOTAL]) : nullptr;
		rgs::launch_duplicate_with_keys(P, at<uint32_t>(geom_ws, goff[RGS_GEOM_VISIBLE_COUNT]),
		                                at<uint32_t>(geom_ws, goff[RGS_GEOM_DEPTH_ORDER]),
		                                at<uint32_t>(geom_ws, goff[RGS_GEOM_POINT_OFFSETS]), at<float2>(geom_ws, goff[RGS_GEOM_XY]),
		                                radii, gx, gy, keys_a, vals_a, (uint32_t)R, at<uint32_t>(binning_ws, b.temp),
		                                rgs::sort_clear_words((size_t)R, tile_key_bits(width, height)), s);
		RGS_STAGE("duplicate_with_keys");
		const int end_bit = tile_key_bits(width, height);
		// the first kernel of the sort also clears the tile ranges (and the counters behind them)
		rgs::launch_sort_pairs_u32(keys_a, keys_b, vals_a, vals_b, (size_t)R, count, end_bit, at<uint32_t>(binning_ws, b.temp),
		                           true, reinterpret_cast<uint32_t*>(ranges), (size_t)gx * gy * 2 + rgs::kRangeTailWords,
		                           "sort", s);
		RGS_STAGE("sort_pairs");
		const bool sorted_in_a = (((end_bit + 7) / 8) % 2) == 0;
		if (debug) {
			uint32_t status = 0, status2 = 0;
			hipError_t e = hipMemcpy(&status, rgs::sort_status_word(at<uint32_t>(binning_ws, b.temp)), sizeof(status),
			                         hipMemcpyDeviceToHost);
			if (e == hipSuccess)
				e = hipMemcpy(&status2, order_status, sizeof(status2), hipMemcpyDeviceToHost);
			status |= status2;
			if (e != hipSuccess || status != 0)
				return fail("sort_pairs: %s", e != hipSuccess ? hipGetErrorString(e) : "a look-back wait timed out");
		}
		rgs::launch_tile_ranges(sorted_in_a ? keys_a : keys_b, (size_t)R, count, ranges, gx * gy,
		                        rgs::sort_status_word(at<uint32_t>(binning_ws, b.temp)), order_status, fault_word(true), true, s);
		RGS_STAGE("tile_ranges");
		point_list = sorted_in_a ? vals_a : vals_b;
	} else {
		rgs::launch_tile_ranges(nullptr, 0, nullptr, ranges, gx * gy, nullptr, nullptr, nullptr, false, s);
		RGS_STAGE("tile_ranges");
	}

	rgs::BlendArgs a;
	memset(&a, 0, sizeof(a));
	a.ranges = ranges;
	a.point_list = point_list;
	a.W = width; a.H = height; a.grid_x = gx; a.grid_y = gy;
	a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
	a.projinv = projmatrix_inv; a.range_low = range_low; a.range_up = range_up; a.bg = background;
	a.xy = at<float2>(geom_ws, goff[RGS_GEOM_XY]);
	a.clip_w = at<float>(geom_ws, goff[RGS_GEOM_CLIP_W]);
	a.conic_opacity = at<float4>(geom_ws, goff[RGS_GEOM_CONIC_OPACITY]);
	a.colors = colors_precomp ? colors_precomp : at<float>(geom_ws, goff[RGS_GEOM_RGB]);
	a.depths = at<float>(geom_ws, goff[RGS_GEOM_DEPTHS]);
	a.record = at<float4>(geom_ws, goff[RGS_GEOM_BLEND_RECORD]);
	a.out_color = out_color; a.out_depth = out_depth; a.out_alpha = out_alpha;
	a.n_contrib = at<uint32_t>(image_ws, ioff[RGS_IMG_N_CONTRIB]);
	a.strip_filed = at<uint32_t>(image_ws, ioff[RGS_IMG_STRIP_FILED]);
	a.strip_order = at<uint32_t>(image_ws, ioff[RGS_IMG_STRIP_ORDER]);
	a.strip_lists = R > 0 ? at<uint32_t>(binning_ws, binning_physical((size_t)R).strip_lists) : nullptr;
	a.strip_classes = reinterpret_cast<uint32_t*>(ranges) + 2 * (size_t)gx * gy;
	rgs::launch_blend_forward(a, s);
	RGS_STAGE("blend_forward");
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
                 float* dL_dcov3D, float* dL_dsh, float* dL_dscale, float* dL_drot, int outputs_zeroed, void* stream,
                 int debug)
{
	hipStream_t s = static_cast<hipStream_t>(stream);
	EntryScope scope_(s);
	RGS_TAKE_SORT_FAULT("rgs_backward");
	RGS_REQUIRE(P > 0 && R >= 0, "rgs_backward: bad sizes P=%d R=%d", P, R);
	RGS_REQUIRE(width > 0 && height > 0, "rgs_backward: bad image size %dx%d", width, height);
	RGS_REQUIRE(background && means3D && alphas && viewmatrix && projmatrix && projmatrix_inv && range_low && range_up &&
	                cam_pos && radii && geom_ws && image_ws && dL_dpix && grad_accum &&
	                dL_dmean2D && dL_dopacity && dL_dcolor && dL_dmean3D && dL_dcov3D,
	            "rgs_backward: null pointer");
	RGS_REQUIRE(R == 0 || binning_ws, "rgs_backward: null binning workspace");
	RGS_REQUIRE((shs != nullptr) != (colors_precomp != nullptr), "rgs_backward: provide exactly one of SHs or colours");
	RGS_REQUIRE(!shs || dL_dsh, "rgs_backward: dL_dsh is required with SHs");
	RGS_REQUIRE(!scales || (rotations && dL_dscale && dL_drot), "rgs_backward: scale/rotation outputs missing");
	RGS_REQUIRE(scales || cov3D_precomp, "rgs_backward: neither scales nor precomputed covariance");

	size_t goff[RGS_GEOM_FIELDS], ioff[RGS_IMG_FIELDS];
	geom_layout((size_t)P, goff);
	image_layout(width, height, ioff);
	const int gx = (width + rgs::kTile - 1) / rgs::kTile, gy = (height + rgs::kTile - 1) / rgs::kTile;
	const size_t n = (size_t)P;

	if (!outputs_zeroed) {
		rgs::launch_fill_u32(reinterpret_cast<uint32_t*>(grad_accum), 0u, (size_t)RGS_ACC_FLOATS * n, s);
		RGS_STAGE("clear gradient sums");
	}

	const float* colors = colors_precomp ? colors_precomp : at<float>(geom_ws, goff[RGS_GEOM_RGB]);
	if (R > 0) {
		const BinningPhysical b = binning_physical((size_t)R);
		const bool sorted_in_a = (((tile_key_bits(width, height) + 7) / 8) % 2) == 0;
		rgs::BlendArgs a;
		memset(&a, 0, sizeof(a));
		a.ranges = at<uint2>(image_ws, ioff[RGS_IMG_RANGES]);
		a.point_list = at<uint32_t>(binning_ws, sorted_in_a ? b.vals_a : b.vals_b);
		a.W = width; a.H = height; a.grid_x = gx; a.grid_y = gy;
		a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
		a.projinv = projmatrix_inv; a.range_low = range_low; a.range_up = range_up; a.bg = background;
		a.xy = at<float2>(geom_ws, goff[RGS_GEOM_XY]);
		a.clip_w = at<float>(geom_ws, goff[RGS_GEOM_CLIP_W]);
		a.conic_opacity = at<float4>(geom_ws, goff[RGS_GEOM_CONIC_OPACITY]);
		a.colors = colors;
		a.depths = at<float>(geom_ws, goff[RGS_GEOM_DEPTHS]);
		a.record = at<float4>(geom_ws, goff[RGS_GEOM_BLEND_RECORD]);
		a.out_alpha = const_cast<float*>(alphas);
		a.n_contrib = const_cast<uint32_t*>(at<uint32_t>(image_ws, ioff[RGS_IMG_N_CONTRIB]));
		a.strip_filed = const_cast<uint32_t*>(at<uint32_t>(image_ws, ioff[RGS_IMG_STRIP_FILED]));
		a.strip_order = const_cast<uint32_t*>(at<uint32_t>(image_ws, ioff[RGS_IMG_STRIP_ORDER]));
		a.strip_lists = const_cast<uint32_t*>(at<uint32_t>(binning_ws, b.strip_lists));
		a.dL_dpix = dL_dpix; a.dL_dpix_depth = dL_dpix_depth; a.dL_dalpha = dL_dalphas;
		a.sums = grad_accum;
		rgs::launch_blend_backward(a, s);
		RGS_STAGE("blend_backward");
	}

	rgs::PreprocessBackwardArgs p;
	memset(&p, 0, sizeof(p));
	p.P = P; p.D = D; p.M = M;
	p.means = means3D; p.radii = radii; p.shs = shs;
	p.clamped = at<uint8_t>(geom_ws, goff[RGS_GEOM_CLAMPED]);
	p.scales = scales; p.rotations = rotations; p.scale_modifier = scale_modifier;
	p.cov3D = cov3D_precomp ? cov3D_precomp : at<float>(geom_ws, goff[RGS_GEOM_COV3D]);
	p.view = viewmatrix; p.proj = projmatrix; p.campos = cam_pos;
	p.focal_y = height / (2.0f * tan_fovy);
	p.focal_x = width / (2.0f * tan_fovx);
	p.tanfovx = tan_fovx; p.tanfovy = tan_fovy;
	p.sums = grad_accum;
	p.dL_dmean2D = dL_dmean2D; p.dL_dopacity = dL_dopacity; p.dL_dcolor = dL_dcolor;
	p.dL_dmeans = dL_dmean3D; p.dL_dcov3D = dL_dcov3D; p.dL_dsh = dL_dsh; p.dL_dscale = dL_dscale; p.dL_drot = dL_drot;
	p.visible_list = at<uint32_t>(geom_ws, goff[RGS_GEOM_VISIBLE_LIST]);
	p.sh_rows_by_16_bytes = sh_rows_by_16_bytes(shs, M, D) && (reinterpret_cast<uintptr_t>(dL_dsh) & 15) == 0;
	p.visible_count = at<uint32_t>(geom_ws, goff[RGS_GEOM_VISIBLE_COUNT]);
	rgs::launch_preprocess_backward(p, outputs_zeroed != 0, s);
	RGS_STAGE("preprocess_backward");
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
	size_t goff[RGS_GEOM_FIELDS], ioff[RGS_IMG_FIELDS];
	geom_layout((size_t)P, goff);
	image_layout(width, height, ioff);
	rgs::launch_fill_u32(reinterpret_cast<uint32_t*>(counters), 0u, 2 * RGS_WORK_COUNTERS, s);
	if (R == 0)
		return 0;
	const BinningPhysical b = binning_physical((size_t)R);
	const bool sorted_in_a = (((tile_key_bits(width, height) + 7) / 8) % 2) == 0;
	rgs::BlendArgs a;
	memset(&a, 0, sizeof(a));
	a.ranges = at<uint2>(image_ws, ioff[RGS_IMG_RANGES]);
	a.point_list = at<uint32_t>(binning_ws, sorted_in_a ? b.vals_a : b.vals_b);
	a.W = width; a.H = height;
	a.grid_x = (width + rgs::kTile - 1) / rgs::kTile;
	a.grid_y = (height + rgs::kTile - 1) / rgs::kTile;
	a.tanfovx = tan_fovx; a.tanfovy = tan_fovy;
	a.projinv = projmatrix_inv; a.range_low = range_low; a.range_up = range_up;
	a.bg = range_low;  // unused by the counting kernel
	a.xy = at<float2>(geom_ws, goff[RGS_GEOM_XY]);
	a.clip_w = at<float>(geom_ws, goff[RGS_GEOM_CLIP_W]);
	a.conic_opacity = at<float4>(geom_ws, goff[RGS_GEOM_CONIC_OPACITY]);
	a.colors = colors_precomp ? colors_precomp : at<float>(geom_ws, goff[RGS_GEOM_RGB]);
	a.depths = at<float>(geom_ws, goff[RGS_GEOM_DEPTHS]);
	a.record = at<float4>(geom_ws, goff[RGS_GEOM_BLEND_RECORD]);
	a.counters = counters;
	rgs::launch_blend_forward(a, s);
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

static int sort_pairs_u64(const char* who, uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out,
                          size_t n, int end_bit, uint32_t* temp, uint32_t* fault, hipStream_t s)
{
	const int debug = 0;
	rgs::launch_sort_pairs(keys_in, keys_out, vals_in, vals_out, n, end_bit, temp, s);
	RGS_STAGE("sort_pairs");
	rgs::launch_report_sort_status(temp, fault, s);
	if ((((end_bit + 7) / 8) % 2) == 0) {
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
	                      fault_word(true), s);
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
	if (int rc = static_sort_scratch(&temp))
		return rc;
	// the report word is only used if an earlier call has set it up: nothing is allocated here
	return sort_pairs_u64("rgs_sort_pairs_static", keys_in, keys_out, vals_in, vals_out, n, end_bit, temp, fault_word(false), s);
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
	return take_sort_fault("rgs_sort_fault");
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
