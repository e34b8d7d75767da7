// Per-tile alpha blending, forward and backward.  A 16x16 tile is four strips of 16x4 pixels;
// a wavefront owns one strip, one pixel per lane, and every strip is a workgroup of its own
// (strips end at very different times, and a wave slot should not idle until its tile's longest
// strip is done); the backward takes the longest strips first.
//
// Compiled with -ffp-contract=off: every per-pixel decision (power > 0, alpha < 1/255,
// the half-Gaussian box test, T(1-alpha) < 1e-4) is evaluated with the unfused
// single-precision expressions of K/cuda_rasterizer_hgs/forward.cu:338-392
// (K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian), so a pixel
// can only differ from that evaluation through the last bits of exp() (exp_of_exponent below).
//
// Blending front to back gives a strip no parallelism beyond its 64 pixels, but deciding which
// entries of a tile's list can matter to a strip needs no order at all.  So the work is split:
// the kernel that emits the (Gaussian, tile) instances decides for each of them which of the
// tile's four strips it can matter to (strip_filing.h) and sends that along with the tile key
// through the sort; a placing kernel turns the sorted bits into one list per strip (the list
// positions that matter to it, in list order); the blend kernels then walk only those, in chunks
// of 64 (lane l takes entry l of the chunk; the next chunk's records, the ids of the one after and
// the positions of the one after that are already in flight while the current chunk is
// processed).  With many small Gaussians a tile's list runs to tens of thousands of entries of
// which a strip needs a few thousand at most.  The backward walks the same filed lists, up to the
// last entry any pixel blended.  The forward narrows a step further: of each chunk it packs, per
// 8-pixel-wide half of the strip, the entries whose ellipse reaches that half, and the lanes of
// each half walk their own packed entries side by side (as many steps as the longer of the two).
//
// Inside the walk, alpha >= 1/255 needs power >= -ln(255 * opacity); that floor (minus a margin) is
// stored with the Gaussian, and a group of four entries is skipped with one ballot when no live
// lane reaches it, before exp() is evaluated.
#include "rgs_kernels.h"
#include "strip_filing.h"
#include "tile_order.h"

namespace rgs {

struct PixelRay {
	float ndc_x, ndc_y;  // pixel centre in NDC
};

__device__ __forceinline__ BoxFrame load_box_frame(const BlendArgs& a)
{
	return load_box_frame(a.projinv, a.range_low, a.range_up, a.tanfovx, a.tanfovy);
}

// World-space point of the pixel's ray at clip-w `w`, tested against the submodel box
// (low, up] (K/cuda_rasterizer_hgs/forward.cu:360-372).  True when the sample is clipped.
__device__ __forceinline__ bool clipped_by_box(const PixelRay& ray, float w, const BoxFrame& b)
{
	const float3 ph = {ray.ndc_x * (w + 0.0000001f) * b.tanx, ray.ndc_y * (w + 0.0000001f) * b.tany, w};
	const float wx = b.m[0][0] * ph.x + b.m[1][0] * ph.y + b.m[2][0] * ph.z + b.m[3][0];
	const float wy = b.m[0][1] * ph.x + b.m[1][1] * ph.y + b.m[2][1] * ph.z + b.m[3][1];
	const float wz = b.m[0][2] * ph.x + b.m[1][2] * ph.y + b.m[2][2] * ph.z + b.m[3][2];
	return (wx <= b.lo.x) || (wx > b.hi.x) || (wy <= b.lo.y) || (wy > b.hi.y) || (wz <= b.lo.z) || (wz > b.hi.z);
}

// exp(x) for the exponents of the blend (-6 < x <= 0 where the result is used): 2^(x log2 e) on the hardware exp2 unit.
// The product's rounding (half a unit in the last place of a number below 8) and the unit's own leave the result within
// four units in the last place, the class of a library expf; the decisions taken on it (alpha against 1/255, the
// transmittance against 1e-4) agree with an exact evaluation except within a few 1e-7 of their thresholds.  Forward
// and backward use the same function, so they take the same per-pixel decisions.
__device__ __forceinline__ float exp_of_exponent(float x)
{
	return __builtin_amdgcn_exp2f(x * 1.44269502e+0f);
}

// Launch-order classes of the backward's strips, by the number of entries they have to walk.
constexpr int kStripClasses = 256;
__device__ __forceinline__ uint32_t strip_class(uint32_t filed) { return 255u - min(filed >> 3, 255u); }

constexpr uint32_t kLongList = 2048;    // filed entries from which a strip's wavefront takes the highest issue priority
constexpr int kPerLane = 1;             // list entries per lane and step (2 was measured slower)
constexpr int kChunk = 64 * kPerLane;   // list entries a wavefront takes per step

// What the backward reads of a record: it takes the forward's word for which entries matter.
struct LoadedRecord {
	float4 geom, conic, cd;
	uint32_t id;
};

__device__ __forceinline__ LoadedRecord load_record(const BlendArgs& a, uint32_t id, bool in_range)
{
	LoadedRecord e;
	id = min(id, a.gaussians - 1u);  // (a list that is not this frame's must not lead outside the records)
	e.id = id;
	if (in_range) {
		const float4* rec = a.record + 4 * (size_t)id;
		e.geom = rec[0];
		e.conic = rec[1];
		e.cd = rec[2];
	} else {
		e.geom = float4{0.f, 0.f, INFINITY, 0.f};
		e.conic = float4{0.f, 0.f, 0.f, 0.f};
		e.cd = float4{0.f, 0.f, 0.f, 0.f};
	}
	return e;
}

__device__ __forceinline__ float exponent_of(const float4 g, const float4 co, const float2 pixf, float2& d)
{
	d = float2{g.x - pixf.x, g.y - pixf.y};
	return -0.5f * (co.x * d.x * d.x + co.z * d.y * d.y) - co.y * d.x * d.y;
}

// The blend kernels stage a conic as (-xx / 2, -xy, -yy / 2, opacity): scaling by a power of two and negation commute
// with rounding, so the exponent below has the very bits of exponent_of() on the conic as stored, one multiplication less
// per pixel and entry.
__device__ __forceinline__ float4 staged_conic(const float4 co) { return float4{-0.5f * co.x, -co.y, -0.5f * co.z, co.w}; }
__device__ __forceinline__ float exponent_of_staged(const float4 g, const float4 sc, const float2 pixf)
{
	const float dx = g.x - pixf.x, dy = g.y - pixf.y;
	return (sc.x * dx * dx + sc.z * dy * dy) + sc.y * dx * dy;
}

// ---- filing ------------------------------------------------------------------------------------
// The sorted keys carry, above the tile, one bit per strip the entry is filed for and one per strip
// that lies inside the box (key_strips).  A workgroup takes kFileGroup consecutive positions of the
// sorted list, whichever tiles they belong to, four neighbouring positions per thread.  An entry's rank
// in its strip's list is the number of filed entries of its tile before it: those inside the workgroup
// follow from a prefix count over the workgroup (per thread in LDS, four strips packed 16 bits each),
// taken at the entry and at the place where its tile begins; those in earlier workgroups (only the
// tile of the workgroup's first entry can have any) are the sum, over the workgroups since that tile
// began, of what each filed for the tile of its LAST entry, which the tile-range kernel has left in
// file_tail.  The thread that holds a tile's last entry also writes the strips' totals.

// Counts of the four strips packed in two words, 16 bits each (a workgroup files at most kFileGroup per strip).
__device__ __forceinline__ uint2 packed_strip_bits(uint32_t bits)
{
	return uint2{(bits & 1u) | ((bits & 2u) << 15), ((bits >> 2) & 1u) | ((bits & 8u) << 13)};
}

struct FileStage {
	uint2 before[kFileBlock];   // entries filed by the threads before this one
	uint16_t bits[kFileBlock];  // the filed bits of the thread's four positions, four bits each
	uint2 wave_total[4];
	uint32_t carry[4][4];       // [wave][strip] partial sums of the earlier workgroups' counts
};

// Entries filed at positions [0, i) of the workgroup.
__device__ __forceinline__ uint2 filed_before(const FileStage& st, uint32_t i)
{
	const uint32_t t = i >> 2, q = i & 3u;
	uint2 n = st.before[t];
	const uint32_t bits = st.bits[t];
#pragma unroll
	for (uint32_t k = 0; k < 3; k++)
		if (k < q) {
			const uint2 c = packed_strip_bits((bits >> (4 * k)) & 0xFu);
			n.x += c.x;
			n.y += c.y;
		}
	return n;
}

__global__ __launch_bounds__(kFileBlock) void strip_file_place_kernel(BlendBatch batch)
{
	__shared__ FileStage st;
	const BlendArgs& a = batch.job[blockIdx.y];
	const uint32_t capacity = a.capacity;
	const uint32_t R = a.count_device ? min(capacity, *a.count_device) : capacity;
	const uint32_t first = blockIdx.x * (uint32_t)kFileGroup;
	// after a sort that gave up the list is not sorted and the tile ranges are empty: nothing to place
	if (first >= R || (a.sort_status && *a.sort_status != 0u) || (a.order_status && *a.order_status != 0u))
		return;
	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const uint32_t pos0 = first + 4u * (uint32_t)tid;
	uint32_t key[4] = {0u, 0u, 0u, 0u};
	if (pos0 + 3u < R) {
		const uint4 k4 = *reinterpret_cast<const uint4*>(a.tile_keys + pos0);
		key[0] = k4.x; key[1] = k4.y; key[2] = k4.z; key[3] = k4.w;
	} else {
#pragma unroll
		for (int q = 0; q < 4; q++)
			if (pos0 + (uint32_t)q < R)
				key[q] = a.tile_keys[pos0 + q];
	}
	uint2 range[4];
	uint32_t filed[4];
	uint2 own = {0u, 0u};
	uint32_t all = 0;
#pragma unroll
	for (int q = 0; q < 4; q++) {
		const bool valid = pos0 + (uint32_t)q < R;
		range[q] = valid ? a.ranges[key_tile(key[q])] : uint2{0u, 0u};
		filed[q] = valid ? (key_strips(key[q]) & 0xFu) : 0u;
		const uint2 c = packed_strip_bits(filed[q]);
		own.x += c.x;
		own.y += c.y;
		all |= filed[q] << (4 * q);
	}
	const uint2 inc = {wave_inclusive_scan_u32(own.x), wave_inclusive_scan_u32(own.y)};
	if (lane == 63)
		st.wave_total[wave] = inc;
	st.bits[tid] = (uint16_t)all;
	// what the tile of this workgroup's first entry filed in the workgroups before this one
	{
		const uint32_t begin0 = a.ranges[key_tile(a.tile_keys[first])].x;
		uint4 sum = {0u, 0u, 0u, 0u};
		if (begin0 < first)
			for (uint32_t g = begin0 / (uint32_t)kFileGroup + (uint32_t)tid; g < blockIdx.x; g += kFileBlock) {
				const uint4 t = a.file_tail[g];
				sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
			}
		uint32_t v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
		for (int s = 0; s < 4; s++) {
			const uint32_t tot = wave_inclusive_scan_u32(v[s]);
			if (lane == 63)
				st.carry[wave][s] = tot;
		}
	}
	__syncthreads();
	uint2 mine = {inc.x - own.x, inc.y - own.y};  // filed before this thread's first position
#pragma unroll
	for (int w = 0; w < 3; w++)
		if (w < wave) {
			mine.x += st.wave_total[w].x;
			mine.y += st.wave_total[w].y;
		}
	st.before[tid] = mine;
	__syncthreads();
	uint32_t carry[4];
#pragma unroll
	for (int s = 0; s < 4; s++)
		carry[s] = st.carry[0][s] + st.carry[1][s] + st.carry[2][s] + st.carry[3][s];

	uint32_t begin_of = 0xFFFFFFFFu;  // the tile start the last `from` was taken at
	uint2 from = {0u, 0u};
#pragma unroll
	for (int q = 0; q < 4; q++) {
		const uint32_t pos = pos0 + (uint32_t)q;
		if (pos < R) {
			const uint2 r = range[q];
			const bool continues = r.x < first;  // the tile began in an earlier workgroup
			const uint32_t begin = max(r.x, first) - first;
			if (begin != begin_of) {
				from = begin == 0u ? uint2{0u, 0u} : filed_before(st, begin);
				begin_of = begin;
			}
			const uint32_t n = r.y - r.x, e = pos - r.x, bits = key_strips(key[q]);
			uint32_t* lists = a.strip_lists + 4 * (size_t)r.x;
			const uint32_t at[4] = {mine.x & 0xFFFFu, mine.x >> 16, mine.y & 0xFFFFu, mine.y >> 16};
			const uint32_t base[4] = {from.x & 0xFFFFu, from.x >> 16, from.y & 0xFFFFu, from.y >> 16};
			uint32_t rank[4];
#pragma unroll
			for (int s = 0; s < 4; s++) {
				rank[s] = (continues ? carry[s] : 0u) + at[s] - base[s];
				if ((bits >> s) & 1u)
					lists[(size_t)s * n + rank[s]] = e | (((bits >> (4 + s)) & 1u) ? 0x80000000u : 0u);
			}
			if (pos + 1u == r.y) {  // the tile's last entry: its ranks plus itself are the strips' totals
				uint4 total = {rank[0] + (bits & 1u), rank[1] + ((bits >> 1) & 1u), rank[2] + ((bits >> 2) & 1u),
				               rank[3] + ((bits >> 3) & 1u)};
				reinterpret_cast<uint4*>(a.strip_total)[key_tile(key[q])] = total;
			}
		}
		const uint2 c = packed_strip_bits(filed[q]);
		mine.x += c.x;
		mine.y += c.y;
	}
}

// ---- forward (K/cuda_rasterizer_hgs/forward.cu:263-405) ---------------------------------------

struct ForwardPixel {
	float T, C0, C1, C2, weight, D;
	uint32_t last_filed;  // the last entry blended, counted in entries filed for the strip (1-based; 0: none)
};

struct ForwardStage {  // one per workgroup (a single wavefront)
	// The chunk's entries once per 8-pixel-wide half of the strip they can reach, each half's packed to the front, so
	// that a step's reads are at addresses known when the step begins:
	float4 geom[2][kChunk + 3];   // pixel x, pixel y, exponent floor, clip w (NaN: strip inside the box)
	float4 conic[2][kChunk + 3];  // staged_conic(): -xx / 2, -xy, -yy / 2, opacity
	float4 cd[2][kChunk];         // r, g, b, view depth: what only a blended sample uses
	uint8_t entry[2][kChunk + 4]; // which entry of the chunk a packed slot holds
};

// `first` is the number of entries filed for the strip ahead of the chunk; `slot` is the packed slot in the
// pixel's half.
// `done` holds a bit per pixel (lane) that takes no further entries: kept as a lane mask in scalar registers,
// so that "a candidate that is not done" is two scalar instructions and not a flag byte per lane to test and set.
__device__ __forceinline__ void forward_visit(ForwardPixel& p, uint64_t& done, uint64_t candidates, float power, const float4 g,
                                              const float4 co, const ForwardStage& st, int half, int slot, uint32_t first,
                                              const PixelRay& ray, const BoxFrame& box)
{
	const uint64_t taking = candidates & ~done;
	if (taking == 0ull)
		return;
	// Every lane evaluates alpha and the transmittance behind the entry (an instruction costs the wavefront the same
	// whatever its lanes), and the decisions are kept as lane masks: no branch, and no flag in a register, per decision.
	// (the entry's colour is asked for ahead of its use in the masked region: the wait falls behind the exp)
	const float4 cd = st.cd[half][slot];
	const uint32_t entry = st.entry[half][slot];
	const float alpha = fminf(0.99f, co.w * exp_of_exponent(power));
	const float test_T = p.T * (1 - alpha);
	uint64_t ok = taking & lanes_where(!(alpha < 1.0f / 255.0f));
	const float clip_w = g.w;  // the same for every lane; NaN: the whole strip is inside the box
	if (lanes_where(clip_w == clip_w) != 0ull)
		ok &= lanes_where(!clipped_by_box(ray, clip_w, box));
	const uint64_t finished = ok & lanes_where(test_T < 0.0001f);
	done |= finished;
	const uint64_t blending = ok & ~finished;
	if (blending == 0ull)
		return;
	if (__builtin_amdgcn_inverse_ballot_w64(blending)) {
		// The sums feed no decision (the images are compared by tolerance): one product alpha T and a fused
		// multiply-add per channel instead of the reference's two products and an add each (forward.cu:378-385).
		const float weight = alpha * p.T;
		p.C0 = __builtin_fmaf(cd.x, weight, p.C0);
		p.C1 = __builtin_fmaf(cd.y, weight, p.C1);
		p.C2 = __builtin_fmaf(cd.z, weight, p.C2);
		p.weight += weight;
		p.D = __builtin_fmaf(cd.w, weight, p.D);
		p.T = test_T;
		p.last_filed = first + entry + 1u;
	}
}

// Number of set bits of a ballot below the calling lane.
__device__ __forceinline__ uint32_t lanes_below(uint64_t ballot)
{
	return __builtin_amdgcn_mbcnt_hi((uint32_t)(ballot >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)ballot, 0u));
}

// Whether the ellipse power >= floor of a filed entry can reach pixel columns [xa, xa + 7] (x relative to the
// Gaussian's centre: dxa = centre - xa).  `reach` is the ellipse's half extent in x, with room for rounding.
__device__ __forceinline__ bool reaches_columns(float dxa, float reach)
{
	return !(dxa + reach < 0.f) && !(dxa - reach > 7.f);
}

__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(6, 6))) void blend_forward_kernel(BlendBatch batch)
{
	__shared__ ForwardStage st;

	const int lane = threadIdx.x;
	// The jobs of a batch (the submodels of a frame) take turns, each handing out its strips longest
	// list first: a long strip that starts late is what a launch waits for, and with several jobs in one
	// launch there is other work to run beside the longest strips of each.
	const BlendArgs& a = batch.job[blockIdx.x % (uint32_t)batch.count];
	const uint32_t strip_id = a.strip_order_forward[blockIdx.x / (uint32_t)batch.count];
	const int tile = (int)(strip_id >> 2), wave = (int)(strip_id & 3u);  // wave: which strip of the tile
	const uint2 range = a.ranges[tile];
	const uint32_t n = range.y - range.x;
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const BoxFrame box = load_box_frame(a);

	ForwardPixel p = {1.0f, 0.f, 0.f, 0.f, 0.f, 0.f, 0u};
	uint64_t done = lanes_where(!inside);
	uint64_t live = ~done;
	// the entries filed for this strip, in list order: list position, bit 31 = strip inside the box
	const uint32_t filed = a.strip_total[strip_id];
	// A long list is a long chain of dependent steps: its wavefront goes first where it shares a SIMD with
	// wavefronts of short lists, which lose little by waiting and would otherwise stretch the launch's longest walk.
	if (filed > kLongList)
		__builtin_amdgcn_s_setprio(3);
	else if (filed > kLongList / 4)
		__builtin_amdgcn_s_setprio(2);

	if (filed != 0u && live != 0ull) {
		const uint32_t* list = a.point_list + range.x;
		const uint32_t* filed_list = a.strip_lists + 4 * (size_t)range.x + (size_t)wave * n;
		constexpr uint32_t kNone = 0xFFFFFFFFu, kPosition = 0x7FFFFFFFu;
		// Lane l of the chunk that starts at filed entry `first` takes entry first + l: its list
		// position (and box flag), through that the Gaussian's index, through that its record.
		// Three chunks are in flight: the records of the next one, the indices of the one after,
		// the positions of the one after that.
		uint32_t pos_cur = (uint32_t)lane < filed ? filed_list[lane] : kNone;
		uint32_t pos_next = (uint32_t)(64 + lane) < filed ? filed_list[64 + lane] : kNone;
		uint32_t pos_after = (uint32_t)(128 + lane) < filed ? filed_list[128 + lane] : kNone;
		LoadedRecord cur = load_record(a, pos_cur != kNone ? list[pos_cur & kPosition] : 0u, pos_cur != kNone);
		uint32_t id_next = pos_next != kNone ? list[pos_next & kPosition] : 0u;

		const int half = (lane >> 3) & 1;
		const float x0 = (float)(tx * kTile), ya = (float)(ty * kTile + wave * 4);
		for (uint32_t first = 0; first < filed && live != 0ull; first += 64) {
			const int count = (int)min(filed - first, 64u);
			// Which 8-pixel-wide halves of the strip the entry's ellipse power >= floor can reach: its half extent
			// in x is sqrt(limit c / (a c - b^2)) with limit = -2 floor, here with room for the rounding of the
			// exponent the pixels evaluate (relative to its largest terms over the strip) and of the determinant.
			// A half that cannot be reached holds no pixel that would pass the floor test below, so leaving the
			// entry out of that half's walk changes no result.
			bool left = false, right = false;
			if (lane < count) {
				const float ca = cur.conic.x, cb = cur.conic.y, cc = cur.conic.z;
				const float dxa = cur.geom.x - x0, dya = cur.geom.y - ya;
				const float limit = -2.f * cur.geom.z;
				const float far_x = fmaxf(fabsf(dxa), fabsf(dxa - 15.f)), far_y = fmaxf(fabsf(dya), fabsf(dya - 3.f));
				const float allowed = limit + (1e-3f + 1e-4f * limit + 1e-5f * (ca * far_x * far_x + cc * far_y * far_y));
				const float det = ca * cc - cb * cb - 1e-6f * ca * cc;
				float reach = INFINITY;
				if ((ca > 0.f) && (cc > 0.f) && (det > 0.f))
					reach = __builtin_sqrtf(allowed * cc / det) * 1.001f + 0.01f;
				if (!(reach == reach))
					reach = INFINITY;
				left = reaches_columns(dxa, reach);
				right = reaches_columns(dxa - 8.f, reach);
			}
			const uint64_t in_left = lanes_where(left), in_right = lanes_where(right);
			const int n_left = __popcll(in_left), n_right = __popcll(in_right);
			const int steps = max(n_left, n_right), padded = (steps + 3) & ~3;
			if (lane < count) {
				float4 g = cur.geom;
				if (pos_cur & 0x80000000u)
					g.w = __int_as_float(0x7FC00000);  // the strip lies inside the box: no per-pixel test
				if (left) {
					const uint32_t r = lanes_below(in_left);
					st.geom[0][r] = g;
					st.conic[0][r] = staged_conic(cur.conic);
					st.cd[0][r] = cur.cd;
					st.entry[0][r] = (uint8_t)lane;
				}
				if (right) {
					const uint32_t r = lanes_below(in_right);
					st.geom[1][r] = g;
					st.conic[1][r] = staged_conic(cur.conic);
					st.cd[1][r] = cur.cd;
					st.entry[1][r] = (uint8_t)lane;
				}
			}
			// both halves are walked for `padded` slots: the rest get entries that never pass the floor test (an
			// infinite floor; their conic may be any finite one, and the lane's own record is at hand: a real one or zeros)
			if (lane >= n_left && lane < padded) {
				st.geom[0][lane] = float4{0.f, 0.f, INFINITY, 0.f};
				st.conic[0][lane] = cur.conic;
			}
			if (lane >= n_right && lane < padded) {
				st.geom[1][lane] = float4{0.f, 0.f, INFINITY, 0.f};
				st.conic[1][lane] = cur.conic;
			}
			__builtin_amdgcn_wave_barrier();
			// the chunk is in LDS now: its registers take the next chunk's records, loaded during the walk
			cur = load_record(a, id_next, pos_next != kNone);
			pos_cur = pos_next;
			pos_next = pos_after;
			id_next = pos_next != kNone ? list[pos_next & kPosition] : 0u;
			const uint32_t e3 = first + 192 + (uint32_t)lane;
			pos_after = e3 < filed ? filed_list[e3] : kNone;

			const float4* geom = st.geom[half];
			const float4* conic = st.conic[half];
			for (int k = 0; k < steps && live != 0ull; k += 4) {
				const float4 g0 = geom[k], g1 = geom[k + 1], g2 = geom[k + 2], g3 = geom[k + 3];
				const float4 c0 = conic[k], c1 = conic[k + 1], c2 = conic[k + 2], c3 = conic[k + 3];
				const float w0 = exponent_of_staged(g0, c0, pixf), w1 = exponent_of_staged(g1, c1, pixf),
				            w2 = exponent_of_staged(g2, c2, pixf), w3 = exponent_of_staged(g3, c3, pixf);
				// written with negations so that a NaN exponent is kept, as in the exact loop; each mask from single
				// comparisons (a comparison's result is the mask; that of a combined flag is formed through a register)
				const uint64_t q0 = lanes_where(!(w0 > 0.0f)) & lanes_where(!(w0 < g0.z)),
				               q1 = lanes_where(!(w1 > 0.0f)) & lanes_where(!(w1 < g1.z)),
				               q2 = lanes_where(!(w2 > 0.0f)) & lanes_where(!(w2 < g2.z)),
				               q3 = lanes_where(!(w3 > 0.0f)) & lanes_where(!(w3 < g3.z));
				if (((q0 | q1 | q2 | q3) & ~done) == 0ull)
					continue;
				forward_visit(p, done, q0, w0, g0, c0, st, half, k, first, ray, box);
				forward_visit(p, done, q1, w1, g1, c1, st, half, k + 1, first, ray, box);
				forward_visit(p, done, q2, w2, g2, c2, st, half, k + 2, first, ray, box);
				forward_visit(p, done, q3, w3, g3, c3, st, half, k + 3, first, ray, box);
				live = ~done;
			}
			__builtin_amdgcn_wave_barrier();
		}
	}

	{
		// how many of the filed entries the backward has to walk: up to the last one some pixel blended
		const uint32_t upto = filed != 0u ? wave_max_u32(p.last_filed) : 0u;  // (zero for a pixel outside the image)
		if (lane == 0)
			a.strip_filed[strip_id] = upto;
	}
	// (the pixel's place is worked out again from the lane, made opaque: kept from the start it would hold a register
	// through the whole walk, one more than the kernel's wavefronts per SIMD leave it)
	int lane_again = lane;
	asm volatile("" : "+v"(lane_again));
	const uint32_t out_x = tx * kTile + (lane_again & 15), out_y = ty * kTile + wave * 4 + (lane_again >> 4);
	if (out_x < (uint32_t)a.W && out_y < (uint32_t)a.H) {
		const uint32_t pix_id = (uint32_t)a.W * out_y + out_x;
		const size_t plane = (size_t)a.H * a.W;
		// the reference's n_contrib: the 1-based position in the tile's list of the last entry the pixel blended
		uint32_t last_contributor = 0u;
		if (p.last_filed != 0u) {
			const uint32_t* filed_list = a.strip_lists + 4 * (size_t)range.x + (size_t)wave * n;
			last_contributor = (filed_list[p.last_filed - 1u] & 0x7FFFFFFFu) + 1u;
		}
		a.n_contrib[pix_id] = last_contributor;
		a.out_color[pix_id] = p.C0 + p.T * a.bg[0];
		a.out_color[plane + pix_id] = p.C1 + p.T * a.bg[1];
		a.out_color[2 * plane + pix_id] = p.C2 + p.T * a.bg[2];
		a.out_alpha[pix_id] = p.weight;
		a.out_depth[pix_id] = p.D;
	}
}

// Work accounting: the reference loop taken literally, one list entry at a time with no
// filter, counting over all pixels the entries visited by a live pixel (A), those with
// power <= 0 (B), with alpha >= 1/255 (C), inside the box (D), blended (E), and B, C and A
// restricted to entries up to each pixel's last blended one (the backward's share).
__global__ __launch_bounds__(256) void blend_count_kernel(BlendArgs a)
{
	__shared__ float4 s_geom[256];
	__shared__ float4 s_conic[256];

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int tile = tile_of_block((int)blockIdx.x, a.grid_x, a.grid_y);
	if (tile < 0)
		return;
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const BoxFrame box = load_box_frame(a);
	const uint2 range = a.ranges[tile];
	const int rounds = (int)((range.y - range.x + 255) / 256);
	int todo = (int)(range.y - range.x);

	bool done = !inside;
	float T = 1.0f;
	uint32_t nA = 0, nB = 0, nC = 0, nD = 0, nE = 0, nA_last = 0, nB_last = 0, nC_last = 0;
	for (int i = 0; i < rounds; i++, todo -= 256) {
		__syncthreads();
		const uint32_t src = range.x + (uint32_t)i * 256 + tid;
		if (src < range.y) {
			const uint32_t id = a.point_list[src];
			const float4 r0 = a.record[4 * (size_t)id];
			s_geom[tid] = float4{r0.x, r0.y, 0.f, r0.w};
			s_conic[tid] = a.record[4 * (size_t)id + 1];
		}
		__syncthreads();
		const int count = todo < 256 ? todo : 256;
		for (int j = 0; !done && j < count; j++) {
			const float4 g = s_geom[j];
			const float4 co = s_conic[j];
			float2 d;
			const float power = exponent_of(g, co, pixf, d);
			nA++;
			if (power > 0.0f)
				continue;
			nB++;
			const float alpha = fminf(0.99f, co.w * expf(power));
			if (alpha < 1.0f / 255.0f)
				continue;
			nC++;
			if (clipped_by_box(ray, g.w, box))
				continue;
			nD++;
			const float test_T = T * (1 - alpha);
			if (test_T < 0.0001f) {
				done = true;
				continue;
			}
			nE++;
			nA_last = nA;
			nB_last = nB;
			nC_last = nC;
			T = test_T;
		}
	}
	const uint32_t c[8] = {nA, nB, nC, nD, nE, nB_last, nC_last, nA_last};
#pragma unroll
	for (int q = 0; q < 8; q++) {
		const uint32_t tot = wave_inclusive_scan_u32(c[q]);
		if (lane == 63)
			atomicAdd(reinterpret_cast<unsigned long long*>(a.counters) + q, (unsigned long long)tot);
	}
}

// ---- backward (K/cuda_rasterizer_hgs/backward.cu:415-622) ---------------------------------------
// Each wavefront walks, back to front, the entries the forward filed for its strip, starting at
// the last one that any of its 64 pixels blended.  The pass is split in two so that no
// cross-lane reduction is needed per entry:
//  * pixel-parallel part (lane = pixel, as in the forward): the per-pixel recurrences of the
//    reference loop give, for an entry, two numbers per pixel: u = G dL/dalpha-term and
//    aT = alpha T.  They are parked in one LDS row per entry.
//  * entry-parallel part, run whenever 8 rows are full (lane = (entry, strip row, half of the row)):
//    each lane sweeps 8 pixels and accumulates sum u, sum u dx, sum u dx^2 and
//    sum aT g_{r,g,b,depth}; dy is constant along a strip row, so the y moments follow from
//    those; three exchanges inside each group of eight lanes finish the sums, and the group adds its
//    entry's ten sums into the Gaussian's row of `sums`, eight neighbouring columns in one atomic
//    instruction and the last two in another.  Eight rows rather than sixteen keep the wavefront's
//    LDS under 10 KB, which is what lets sixteen of them share a CU.
// All ten sums of the reference (mean2D x/y, conic xx/xy/yy, opacity, colour r/g/b, depth)
// are linear in u and aT, which is what makes the split possible.

constexpr int kRows = 8;      // entries gathered before the entry-parallel part runs
// Pixel p of the strip sits in column p + (p >> 4) of a row of kRowStride (u, alpha T) pairs, and its four upstream
// gradients in element p + (p >> 3) of their array: the LDS has 32 banks of 4 bytes, an 8-byte access is served 16
// lanes at a time and a 16-byte access 8 lanes at a time, and with these numbers neither the per-pixel writes nor
// the per-(entry, strip row, half row) reads below hit a bank twice within such a group.
constexpr int kRowStride = 68;
__device__ __forceinline__ int row_column(int pixel) { return pixel + (pixel >> 4); }
__device__ __forceinline__ int upstream_column(int pixel) { return pixel + (pixel >> 3); }

struct BackwardPixel {
	float T;
	float behind;  // what lies behind the entry being visited, weighted with the upstream gradient: see backward_visit
	float g_r, g_g, g_b, g_depth, g_alpha;
};

struct BackwardStage {  // wave-private
	float4 geom[kChunk + 3];  // + padding up to a multiple of four entries
	float4 conic[kChunk + 3];  // staged_conic(): -xx / 2, -xy, -yy / 2, opacity
	float4 cd[kChunk];
	uint32_t entry[kChunk + 3];  // 0-based position in the tile list
	uint32_t id[kChunk];
	float2 u_at[kRows * kRowStride];  // [row][row_column(pixel)]: (u, alpha T)
	float4 upstream[72];              // dL/dpixel r, g, b, depth of the strip's 64 pixels, by upstream_column
};

struct StripFrame {
	float x0, y0;            // first pixel of the strip
	float ddelx_dx, ddely_dy;
};

template <int DppCtrl>
__device__ __forceinline__ float dpp_exchange_add(float v)
{
	const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), DppCtrl, 0xF, 0xF, true);
	return v + __builtin_bit_cast(float, moved);
}

// Entry-parallel part for the first `rows` rows.  A 16-lane row of the wavefront serves two entries, e in its low
// eight lanes and e + 4 in its high eight; lane (h = (lane >> 1) & 3, half = lane & 1) of the eight
// sums the entry's row over the 8 pixels of one half of strip row h; the eight lanes of an entry then add up what
// they hold (three exchanges inside their group of eight) and the entry's ten sums go into the Gaussian's
// row of `sums` with one atomic instruction: the entry's own lanes add columns 0-7, two lanes of the other eight of
// the 16-lane row add columns 8 and 9, so a first instruction serves entries 0-3 and a second one entries 4-7.
// (Adding columns 0-7 of all eight entries first and columns 8-9 after them, which needs no exchange between the
// groups, had every request of the second instruction hit a cache line that one of the first was still at work on:
// measured, that second instruction cost eight times what the first did, a fifth of the kernel's time.)
// `row_slots` holds, one byte per row, which staged entry of the current chunk the row belongs to: the entry's centre,
// conic and Gaussian are read from where the chunk was staged (so the rows are flushed before the next chunk is).
// kDepth: a gradient arrived for the depth image (without one, the usual case of a loss on the colour image alone, the
// terms it multiplies are left out: the depth column of `sums` stays zero).
template <bool kDepth>
__device__ __forceinline__ void flush_rows(const BackwardStage& st, int rows, uint64_t row_slots, const StripFrame& f,
                                           const BlendArgs& a, int lane)
{
#pragma clang fp contract(fast)
	__builtin_amdgcn_wave_barrier();
	const int upper = (lane >> 3) & 1;  // which eight of the 16-lane row
	const int e = (lane >> 4) + 4 * upper, h = (lane >> 1) & 3, half = lane & 1, j = lane & 7;
	const int slot = (int)((row_slots >> (8 * e)) & 0xFFull);
	const float4 centre = st.geom[slot];
	const float2 xy = {centre.x, centre.y};
	const float dy = xy.y - (f.y0 + (float)h);
	const float x_first = f.x0 + (float)(8 * half);
	float s0 = 0.f, sx = 0.f, sxx = 0.f, cr = 0.f, cg = 0.f, cb = 0.f, cdp = 0.f;
	const int col0 = row_column(h * 16 + 8 * half);
	const float2* row = st.u_at + e * kRowStride + col0;
	const float4* upstream = st.upstream + upstream_column(h * 16 + 8 * half);
#pragma unroll
	for (int step = 0; step < 8; step++) {
		const float2 ua = row[step];
		const float4 g = upstream[step];
		const float uu = ua.x, tt = ua.y;
		const float dx = xy.x - (x_first + (float)step);
		const float t = uu * dx;
		s0 += uu;
		sx += t;
		sxx += t * dx;
		cr += tt * g.x;
		cg += tt * g.y;
		cb += tt * g.z;
		if (kDepth)
			cdp += tt * g.w;
	}
	// the two halves of the strip row first (dy is theirs in common), then the four strip rows
	float w[7] = {s0, sx, sxx, cr, cg, cb, cdp};
#pragma unroll
	for (int q = 0; q < (kDepth ? 7 : 6); q++)
		w[q] = dpp_exchange_add<0xB1>(w[q]);  // quad_perm:[1,0,3,2]
	float v[10] = {w[0], w[1], dy * w[0], w[2], dy * w[1], dy * dy * w[0], w[3], w[4], w[5], w[6]};
#pragma unroll
	for (int q = 0; q < (kDepth ? 10 : 9); q++) {
		v[q] = dpp_exchange_add<0x4E>(v[q]);   // quad_perm:[2,3,0,1]
		v[q] = dpp_exchange_add<0x141>(v[q]);  // row_half_mirror: the other quad of the eight
	}
	// (every lane forms all five products and then picks its own: a handful of multiplications more than the one or
	// two a lane needs, but no branch per column and no wait for the conic inside one)
	const float4 co = st.conic[slot];  // the staged conic: -xx / 2, -xy, -yy / 2, opacity
	const uint32_t id = e < rows ? st.id[slot] : 0u;
	const float S0 = v[0], Sx = v[1], Sy = v[2], Sxx = v[3], Sxy = v[4], Syy = v[5];
	const float m0 = co.w * f.ddelx_dx * (2.f * co.x * Sx + co.y * Sy);
	const float m1 = co.w * f.ddely_dy * (2.f * co.z * Sy + co.y * Sx);
	const float half_w = -0.5f * co.w;
	const float k0 = half_w * Sxx, k1 = half_w * Sxy, k3 = half_w * Syy;
	// lane j of the eight holds column j of the row, lanes 0 and 1 also columns 8 and 9: see SumCol
	float first = j == 0 ? m0 : j == 1 ? m1 : j == 2 ? k0 : j == 3 ? k1 : j == 4 ? k3 : j == 5 ? S0 : j == 6 ? v[6] : v[7];
	float second = j == 0 ? v[8] : j == 1 ? v[9] : 0.f;
	if (!(e < rows)) {
		first = 0.f;
		second = 0.f;
	}
	// columns 8 and 9 and the Gaussian's index go to the same lanes of the other eight of the 16-lane row (row_ror:8)
	const float second_there = __builtin_bit_cast(
		float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, second), 0x128, 0xF, 0xF, true));
	const uint32_t id_there = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)id, 0x128, 0xF, 0xF, true);
	{
		// entries 0-3: their own (lower) lanes add columns 0-7, the upper lanes columns 8 and 9 for them
		const float value = upper ? second_there : first;
		float* at = a.sums + (size_t)kSumCols * (upper ? id_there : id) + (upper ? 8 + j : j);
		if (value != 0.f) unsafeAtomicAdd(at, value);
	}
	{
		// entries 4-7: the other way round
		const float value = upper ? first : second_there;
		float* at = a.sums + (size_t)kSumCols * (upper ? id : id_there) + (upper ? j : 8 + j);
		if (value != 0.f) unsafeAtomicAdd(at, value);
	}
	__builtin_amdgcn_wave_barrier();
}

// Pixel-parallel part for one entry; `rows` (wave-uniform) counts the LDS rows in use.
template <bool kDepth>
__device__ __forceinline__ void backward_visit(BackwardPixel& p, uint64_t candidates, float power, const float4 g,
                                               const float4 co, BackwardStage& st, int slot, int& rows, uint64_t& row_slots,
                                               const StripFrame& f, const PixelRay& ray, const BlendArgs& a, int lane)
{
	if (candidates == 0ull)
		return;
	// Every lane evaluates alpha (an instruction costs the wavefront the same whatever its lanes); the decisions are
	// lane masks, and one masked region holds what only a blended sample computes.
	const float4 cd = st.cd[slot];  // asked for ahead of its use in the masked region: the wait falls behind the exp
	const float G = exp_of_exponent(power);
	const float alpha = fminf(0.99f, co.w * G);
	uint64_t blended = candidates & lanes_where(!(alpha < 1.0f / 255.0f));
	// the box and the inverse projection are read where they are needed (few strips straddle a face of their
	// box): kept in scalar registers for the whole walk they crowd out the candidate masks of a step
	const float clip_w = g.w;  // the same for every lane; NaN: the whole strip is inside the box
	if (lanes_where(clip_w == clip_w) != 0ull)
		blended &= lanes_where(!clipped_by_box(ray, clip_w, load_box_frame(a)));
	if (blended == 0ull)
		return;
	float u = 0.f, aT = 0.f;
	if (__builtin_amdgcn_inverse_ballot_w64(blended)) {
		// From here on nothing feeds a decision: gradients are compared by tolerance, so the
		// compiler may contract multiply-adds and the divisions use the hardware reciprocal.
#pragma clang fp contract(fast)
		const float inv_one_minus_alpha = __builtin_amdgcn_rcpf(1.f - alpha);
		p.T = p.T * inv_one_minus_alpha;
		aT = alpha * p.T;
		// The pixel's outputs are sums over its blended entries j of w_j (colour_j, depth_j, 1) with w_j = alpha_j T_j,
		// T_j the product of (1 - alpha_k) over the entries in front, plus T_final times the background.  Their
		// derivative with respect to alpha_i is T_i (colour_i, depth_i, 1) minus (the sum over the entries behind i +
		// T_final background) / (1 - alpha_i).  The reference carries that sum per channel and per unit of transmittance
		// (K/cuda_rasterizer_hgs/backward.cu:568-599: accum_rec = last_alpha * last_color + (1 - last_alpha) * accum_rec,
		// and the background term apart); only its product with the upstream gradient is needed, so one number per
		// pixel does for all channels: `behind` = sum over the entries behind of w_j <g, (colour_j, depth_j, 1)> +
		// T_final <g, background>, started with the latter.  Same quantity, a third of the arithmetic.
		float weighted = __builtin_fmaf(cd.x, p.g_r, __builtin_fmaf(cd.y, p.g_g, __builtin_fmaf(cd.z, p.g_b, p.g_alpha)));
		if (kDepth)
			weighted = __builtin_fmaf(cd.w, p.g_depth, weighted);
		const float dL_dopa = weighted * p.T - p.behind * inv_one_minus_alpha;
		p.behind = __builtin_fmaf(aT, weighted, p.behind);
		u = G * dL_dopa;
	}
	st.u_at[rows * kRowStride + row_column(lane)] = float2{u, aT};
	row_slots |= (uint64_t)slot << (8 * rows);
	rows++;
	if (rows == kRows) {
		flush_rows<kDepth>(st, kRows, row_slots, f, a, lane);
		rows = 0;
		row_slots = 0ull;
	}
}

// 128 registers and under 10 KB of LDS: four wavefronts per SIMD (three, as the compiler chooses by itself, were
// measured 19 % slower; five spill)
template <bool kDepth>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 4))) void blend_backward_kernel(BlendBatch batch)
{
	__shared__ BackwardStage s_stage;

	const int lane = threadIdx.x;
	// the jobs of the batch take turns; each hands out its strips with the most entries first: a long
	// strip that starts late is what the whole launch waits for
	const BlendArgs& a = batch.job[blockIdx.x % (uint32_t)batch.count];
	// What the forward left in the workspaces (the strips' order, the tiles' ranges, the lists, the walk lengths) comes
	// back through the caller's hands: every index taken from it is held inside the arrays' bounds, so that a
	// workspace that is not the forward's (stale, or another frame's) gives wrong gradients and no stray access.
	const uint32_t strip_id = min(a.strip_order[blockIdx.x / (uint32_t)batch.count], 4u * (uint32_t)(a.grid_x * a.grid_y) - 1u);
	const int tile = (int)(strip_id >> 2), wave = (int)(strip_id & 3u);  // wave: which strip of the tile
	uint2 range = a.ranges[tile];
	range.y = min(range.y, a.capacity);
	range.x = min(range.x, range.y);
	const int tx = tile % a.grid_x, ty = tile / a.grid_x;
	const uint32_t px = tx * kTile + (lane & 15), py = ty * kTile + wave * 4 + (lane >> 4);
	const bool inside = px < (uint32_t)a.W && py < (uint32_t)a.H;
	const uint32_t pix_id = (uint32_t)a.W * py + px;
	const float2 pixf = {(float)px, (float)py};
	const PixelRay ray = {pix_to_ndc(pixf.x, a.W), pix_to_ndc(pixf.y, a.H)};
	const size_t plane = (size_t)a.H * a.W;
	const float strip_x0 = (float)(tx * kTile), strip_y0 = (float)(ty * kTile + wave * 4);
	const StripFrame frame = {strip_x0, strip_y0, (float)(0.5 * a.W), (float)(0.5 * a.H)};
	BackwardStage& st = s_stage;

	// The forward blend has written down which entries of the tile's list matter to this strip
	// (its conservative filters, not repeated here), up to the last one that any pixel blended.
	const uint32_t n = range.y - range.x;
	const uint32_t filed = min(a.strip_filed[strip_id], n);
	if (filed == 0u)
		return;
	const uint32_t last_contributor = inside ? a.n_contrib[pix_id] : 0u;

	BackwardPixel p;
	const float T_final = inside ? (1 - a.out_alpha[pix_id]) : 0.f;
	p.T = T_final;
	p.g_r = p.g_g = p.g_b = p.g_depth = p.g_alpha = 0.f;
	if (inside) {
		p.g_r = a.dL_dpix[pix_id];
		p.g_g = a.dL_dpix[plane + pix_id];
		p.g_b = a.dL_dpix[2 * plane + pix_id];
		p.g_depth = a.dL_dpix_depth ? a.dL_dpix_depth[pix_id] : 0.f;  // absent: no gradient came in
		p.g_alpha = a.dL_dalpha ? a.dL_dalpha[pix_id] : 0.f;
	}
	p.behind = T_final * ((0.f + a.bg[0] * p.g_r + a.bg[1] * p.g_g) + a.bg[2] * p.g_b);
	st.upstream[upstream_column(lane)] = float4{p.g_r, p.g_g, p.g_b, p.g_depth};
	int rows = 0;
	uint64_t row_slots = 0ull;

	// Lane l of the chunk that starts `first` entries from the back takes filed entry
	// filed-1-first-l: its list position (and box flag), through that the Gaussian's index,
	// through that its record.  Three chunks are in flight: the records of the next one, the
	// indices of the one after, the positions of the one after that.
	const uint32_t* list = a.point_list + range.x;
	const uint32_t* filed_list = a.strip_lists + 4 * (size_t)range.x + (size_t)wave * n;
	constexpr uint32_t kNone = 0xFFFFFFFFu, kPosition = 0x7FFFFFFFu;
	uint32_t pos_cur = (uint32_t)lane < filed ? filed_list[filed - 1 - lane] : kNone;
	uint32_t pos_next = (uint32_t)(64 + lane) < filed ? filed_list[filed - 1 - (64 + lane)] : kNone;
	uint32_t pos_after = (uint32_t)(128 + lane) < filed ? filed_list[filed - 1 - (128 + lane)] : kNone;
	LoadedRecord cur = load_record(a, pos_cur != kNone ? list[min(pos_cur & kPosition, n - 1u)] : 0u, pos_cur != kNone);
	uint32_t id_next = pos_next != kNone ? list[min(pos_next & kPosition, n - 1u)] : 0u;

	for (uint32_t first = 0; first < filed; first += 64) {
		const int count = (int)min(filed - first, 64u);
		if (lane < count) {
			float4 g = cur.geom;
			if (pos_cur & 0x80000000u)
				g.w = __int_as_float(0x7FC00000);  // the strip lies inside the box: no per-pixel test
			st.geom[lane] = g;
			st.conic[lane] = staged_conic(cur.conic);
			st.cd[lane] = cur.cd;
			st.entry[lane] = pos_cur & kPosition;
			st.id[lane] = cur.id;
		}
		if (lane < 3) {  // pad to a multiple of four with entries that never pass the floor test
			st.geom[count + lane] = float4{0.f, 0.f, INFINITY, 0.f};
			st.conic[count + lane] = float4{0.f, 0.f, 0.f, 0.f};
			st.entry[count + lane] = 0xFFFFFFFFu;
		}
		__builtin_amdgcn_wave_barrier();
		// the chunk is in LDS now: its registers take the next chunk's records, loaded during the walk
		cur = load_record(a, id_next, pos_next != kNone);
		pos_cur = pos_next;
		pos_next = pos_after;
		id_next = pos_next != kNone ? list[min(pos_next & kPosition, n - 1u)] : 0u;
		const uint32_t e3 = first + 192 + (uint32_t)lane;
		pos_after = e3 < filed ? filed_list[filed - 1 - e3] : kNone;

		for (int k = 0; k < count; k += 4) {
			const float4 g0 = st.geom[k], g1 = st.geom[k + 1], g2 = st.geom[k + 2], g3 = st.geom[k + 3];
			const float4 c0 = st.conic[k], c1 = st.conic[k + 1], c2 = st.conic[k + 2], c3 = st.conic[k + 3];
			const uint32_t p0 = st.entry[k], p1 = st.entry[k + 1], p2 = st.entry[k + 2], p3 = st.entry[k + 3];
			const float w0 = exponent_of_staged(g0, c0, pixf), w1 = exponent_of_staged(g1, c1, pixf),
			            w2 = exponent_of_staged(g2, c2, pixf), w3 = exponent_of_staged(g3, c3, pixf);
			// Each entry's candidates are formed right where its visit looks at them: nearly every walked entry has
			// some, so a test for the four together would save little.  Each mask comes from single comparisons (a
			// comparison's result is the mask; that of a combined flag is formed through a register).
			backward_visit<kDepth>(p, lanes_where(p0 < last_contributor) & lanes_where(!(w0 > 0.0f)) & lanes_where(!(w0 < g0.z)), w0,
			                       g0, c0, st, k, rows, row_slots, frame, ray, a, lane);
			backward_visit<kDepth>(p, lanes_where(p1 < last_contributor) & lanes_where(!(w1 > 0.0f)) & lanes_where(!(w1 < g1.z)), w1,
			                       g1, c1, st, k + 1, rows, row_slots, frame, ray, a, lane);
			backward_visit<kDepth>(p, lanes_where(p2 < last_contributor) & lanes_where(!(w2 > 0.0f)) & lanes_where(!(w2 < g2.z)), w2,
			                       g2, c2, st, k + 2, rows, row_slots, frame, ray, a, lane);
			backward_visit<kDepth>(p, lanes_where(p3 < last_contributor) & lanes_where(!(w3 > 0.0f)) & lanes_where(!(w3 < g3.z)), w3,
			                       g3, c3, st, k + 3, rows, row_slots, frame, ray, a, lane);
		}
		// the rows point into this chunk's staged entries: they go before the next chunk takes their place
		if (rows > 0) {
			flush_rows<kDepth>(st, rows, row_slots, frame, a, lane);
			rows = 0;
			row_slots = 0ull;
		}
		__builtin_amdgcn_wave_barrier();
	}
}

// Strips by decreasing number of entries to walk, in kStripClasses classes of 8 (longer ones share
// the first class); the order inside a class is whatever the atomics give, which is all a
// launch order needs.  Two small kernels: count the strips of every class, then place them; one
// launch of each serves every job of a batch (blockIdx.y).  Both aggregate in LDS first: most
// strips fall into one class (nothing to walk), and thousands of global atomics on one word would
// take longer than the blend itself.
struct StripOrderJob {
	const uint32_t* length;  // per strip
	uint32_t* classes;       // kStripClasses counters and as many placement cursors, zero beforehand
	uint32_t* order;
};
struct StripOrderBatch {
	StripOrderJob job[kMaxBlendBatch];
	uint32_t strips;
};

__global__ __launch_bounds__(256) void strip_count_kernel(StripOrderBatch batch)
{
	__shared__ uint32_t s_count[kStripClasses];
	const StripOrderJob& j = batch.job[blockIdx.y];
	s_count[threadIdx.x] = 0;
	__syncthreads();
	const uint32_t k = blockIdx.x * 256 + threadIdx.x;
	if (k < batch.strips)
		atomicAdd(&s_count[strip_class(j.length[k])], 1u);
	__syncthreads();
	if (s_count[threadIdx.x] != 0u)
		atomicAdd(&j.classes[threadIdx.x], s_count[threadIdx.x]);
}

__global__ __launch_bounds__(256) void strip_place_kernel(StripOrderBatch batch)
{
	__shared__ uint32_t s_count[kStripClasses];  // strips of this block per class, then where they go
	__shared__ uint32_t s_scan[8];
	const StripOrderJob& j = batch.job[blockIdx.y];
	s_count[threadIdx.x] = 0;
	__syncthreads();
	const uint32_t k = blockIdx.x * 256 + threadIdx.x;
	uint32_t c = 0, rank = 0;
	if (k < batch.strips) {
		c = strip_class(j.length[k]);
		rank = atomicAdd(&s_count[c], 1u);
	}
	__syncthreads();
	uint32_t total;
	const uint32_t start = block256_exclusive_scan_u32(j.classes[threadIdx.x], s_scan, total);
	const uint32_t mine = s_count[threadIdx.x];
	__syncthreads();
	s_count[threadIdx.x] = start + (mine != 0u ? atomicAdd(&j.classes[kStripClasses + threadIdx.x], mine) : 0u);
	__syncthreads();
	if (k < batch.strips)
		j.order[s_count[c] + rank] = k;
}

// which: 0 = the forward's order (by the entries filed), 1 = the backward's (by the entries up to the last one blended)
static void launch_strip_order(const BlendArgs* jobs, int count, int which, hipStream_t s)
{
	StripOrderBatch b;
	b.strips = (uint32_t)(4 * jobs[0].grid_x * jobs[0].grid_y);
	for (int k = 0; k < count; k++) {
		b.job[k].length = which == 0 ? jobs[k].strip_total : jobs[k].strip_filed;
		b.job[k].classes = jobs[k].strip_classes + (which == 0 ? 2 * kStripClasses : 0);
		b.job[k].order = which == 0 ? jobs[k].strip_order_forward : jobs[k].strip_order;
	}
	const dim3 grid((b.strips + 255) / 256, (unsigned)count);
	hipLaunchKernelGGL(strip_count_kernel, grid, dim3(256), 0, s, b);
	hipLaunchKernelGGL(strip_place_kernel, grid, dim3(256), 0, s, b);
}

void launch_blend_count(const BlendArgs& a, hipStream_t s)
{
	stage_mark("blend_count", s);
	hipLaunchKernelGGL(blend_count_kernel, dim3(tile_order_blocks(a.grid_x, a.grid_y)), dim3(256), 0, s, a);
}

void launch_strip_filing(const BlendArgs* jobs, int count, hipStream_t s)
{
	stage_mark("strip_filing", s);
	for (int at = 0; at < count; at += kMaxBlendBatch) {
		BlendBatch batch;
		batch.count = 0;
		uint32_t most = 0;
		for (int k = at; k < count && k < at + kMaxBlendBatch; k++)
			if (jobs[k].capacity != 0u) {
				batch.job[batch.count++] = jobs[k];
				most = jobs[k].capacity > most ? jobs[k].capacity : most;
			}
		if (batch.count)
			hipLaunchKernelGGL(strip_file_place_kernel, dim3((most + kFileGroup - 1) / kFileGroup, (unsigned)batch.count),
			                   dim3(kFileBlock), 0, s, batch);
	}
}

// All jobs share the image size (they are the submodels of one frame, or a single call).
void launch_blend_forward(const BlendArgs* jobs, int count, hipStream_t s)
{
	const unsigned strips = (unsigned)(4 * jobs[0].grid_x * jobs[0].grid_y);
	for (int at = 0; at < count; at += kMaxBlendBatch) {
		BlendBatch batch;
		batch.count = count - at < kMaxBlendBatch ? count - at : kMaxBlendBatch;
		for (int k = 0; k < batch.count; k++)
			batch.job[k] = jobs[at + k];
		stage_mark("strip_order", s);
		launch_strip_order(jobs + at, batch.count, 0, s);
		stage_mark("blend_forward", s);
		hipLaunchKernelGGL(blend_forward_kernel, dim3(strips * (unsigned)batch.count), dim3(64), 0, s, batch);
		// the order in which the backward will take the strips
		stage_mark("strip_order", s);
		launch_strip_order(jobs + at, batch.count, 1, s);
	}
}

void launch_blend_backward(const BlendArgs* jobs, int count, hipStream_t s)
{
	const unsigned strips = (unsigned)(4 * jobs[0].grid_x * jobs[0].grid_y);
	stage_mark("blend_backward", s);
	for (int at = 0; at < count; at += kMaxBlendBatch) {
		BlendBatch batch;
		batch.count = count - at < kMaxBlendBatch ? count - at : kMaxBlendBatch;
		for (int k = 0; k < batch.count; k++)
			batch.job[k] = jobs[at + k];
		bool depth = false;  // does any job of the batch bring a gradient of the depth image?
		for (int k = 0; k < batch.count; k++)
			depth = depth || batch.job[k].dL_dpix_depth != nullptr;
		if (depth)
			hipLaunchKernelGGL(blend_backward_kernel<true>, dim3(strips * (unsigned)batch.count), dim3(64), 0, s, batch);
		else
			hipLaunchKernelGGL(blend_backward_kernel<false>, dim3(strips * (unsigned)batch.count), dim3(64), 0, s, batch);
	}
}

}  // namespace rgs
