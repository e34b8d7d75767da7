/*
 * rgs.h -- C ABI of librgs_gfx950.so, the MI355X (gfx950) half-Gaussian rasterizer.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream (as void*;
 * NULL = the default stream).  The library never allocates or frees device memory:
 * the caller sizes the three workspaces with the rgs_*_bytes() functions and owns
 * them; a workspace starts at a multiple of 16 bytes.  All float data is fp32, contiguous, on the device the stream belongs to.
 * Matrices are 16 floats in the reference's layout (row-vector convention, i.e.
 * element [4*c + r] is row r, column c of the usual column-vector matrix).
 *
 * Functions return 0 on success; on failure they return non-zero and
 * rgs_last_error() gives the reason for the calling thread.
 *
 * Limits: a call handles fewer than 2^30 (Gaussian, tile) instances (the radix sorts pack a
 * count and two flag bits into one word); rgs_forward_geom reports a larger count as an error.
 * An image has fewer than 2^24 tiles of 16x16 pixels (the tile shares its 32-bit sort key with
 * eight strip bits); rgs_forward_raster refuses a larger one.
 *
 * A sort that gives up: the radix sorts wait for neighbouring workgroups with a bounded number
 * of polls.  Should such a wait ever run out (never observed), every later kernel of that call
 * still runs to its end inside its buffers, the call's tile lists are left empty (the images show
 * the background only, the gradients are zero) and a word of pinned host memory is set, which
 * rgs_forward_geom*, rgs_forward_raster*, rgs_backward and rgs_sort_fault look at when they are
 * called: the next of these calls on that device then fails with a message that says so, without
 * doing its work, and clears the report.  A caller that wants to know before its next call asks
 * rgs_sort_fault, which waits for the stream first.  The reference's cub::DeviceRadixSort has no
 * such state (K/cuda_rasterizer_hgs/rasterizer_impl.cu:312-317).
 *
 * Citations name the interface of the reference that each entry point replaces,
 * with K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian.
 */
#ifndef RGS_H_INCLUDED
#define RGS_H_INCLUDED

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Library version (major*10000 + minor*100 + patch). */
int rgs_version(void);

/* Message for the last failure on the calling thread ("" if none).
 * Replaces the exceptions thrown through CHECK_CUDA (K/cuda_rasterizer_hgs/auxiliary.h:182-189)
 * and AT_ERROR (K/rasterize_points.cu:60-62). */
const char* rgs_last_error(void);

/* The reference's sort-key width helper: number of bits needed for n tile ids
 * (getHigherMsb, K/cuda_rasterizer_hgs/rasterizer_impl.cu:35-50). */
uint32_t rgs_get_higher_msb(uint32_t n);

/* ---- workspace sizing -------------------------------------------------------------
 * Replace required<GeometryState>/<BinningState>/<ImageState>
 * (K/cuda_rasterizer_hgs/rasterizer_impl.h:65-72, rasterizer_impl.cu:155-194). */
size_t rgs_geom_bytes(int P);
size_t rgs_binning_bytes(int R);
size_t rgs_image_bytes(int width, int height);

/* Byte offsets of the arrays inside the workspaces, for tests and tools that want to
 * look at intermediate results.  The workspaces are otherwise opaque. */
enum {
	RGS_GEOM_DEPTHS = 0,        /* float[P]   view-space z of the Gaussians that touch a tile (> 0.2), 0 for the others */
	RGS_GEOM_TILES_TOUCHED,     /* uint32[P] */
	RGS_GEOM_POINT_OFFSETS,     /* uint32[P]  inclusive prefix sum of the tile counts of the Gaussians in
	                               RGS_GEOM_DEPTH_ORDER (as many entries as that has) */
	RGS_GEOM_CLAMPED,           /* uint8[P]   bit c set: colour channel c was clamped at 0 */
	RGS_GEOM_BLOCK_SUMS,        /* uint32[ceil(P/256)+1] */
	RGS_GEOM_TOTAL,             /* uint32     number of (Gaussian, tile) instances */
	RGS_GEOM_BLEND_RECORD,      /* float[16P] one 64-byte record per Gaussian with everything the blend reads:
	                               x, y, exponent floor, clip w | conic xx, xy, yy, opacity | r, g, b, depth |
	                               half-width, half-height of the alpha >= 1/255 ellipse's bounding box, the radius (int32 bits), 0.
	                               The pixel centre, clip w, conic, opacity and colour of a Gaussian are kept here only; its
	                               3D covariance is not kept at all (the backward computes it again from scale and rotation) */
	RGS_GEOM_DEPTH_ORDER,       /* uint32[P]  the Gaussians that touch a tile by increasing depth, ties by index;
	                               entries from RGS_GEOM_VISIBLE_COUNT on are unused */
	RGS_GEOM_BLOCK_VISIBLE,     /* uint32[ceil(P/256)+1] */
	RGS_GEOM_VISIBLE_COUNT,     /* uint32     number of Gaussians that touch a tile */
	RGS_GEOM_ORDER_SCRATCH,     /* scratch of the depth sort */
	RGS_GEOM_FIELDS
};
enum {
	RGS_BIN_KEYS_UNSORTED = 0,  /* uint32[R]  key of each instance, emitted Gaussian after Gaussian in depth order: the tile in
	                               the low 24 bits; above it, per 16x4 strip s of the tile, bit 24+s = the instance can
	                               matter to the strip, bit 28+s = that strip lies inside the submodel box */
	RGS_BIN_KEYS_SORTED,        /* uint32[R]  the same after the stable sort by tile */
	RGS_BIN_VALUES_UNSORTED,    /* uint32[R]  Gaussian index */
	RGS_BIN_VALUES_SORTED,      /* uint32[R]  the per-tile Gaussian lists, tile after tile */
	RGS_BIN_SORT_TEMP,          /* uint32[..] */
	RGS_BIN_STRIP_LISTS,        /* uint32[4R] written ahead of the forward blend: for strip s of a tile with list [x, x+n), from
	                               4x + s*n on, the list positions that can matter to the strip (bit 31: strip inside the box) */
	RGS_BIN_FIELDS
};
enum {
	RGS_IMG_RANGES = 0,         /* uint2[tiles]  [start, end) of each tile in the sorted list */
	RGS_IMG_N_CONTRIB,          /* uint32[H*W]   list position of the last blended Gaussian */
	RGS_IMG_STRIP_FILED,        /* uint32[4*tiles] per 16x4 strip (tile * 4 + strip): entries of RGS_BIN_STRIP_LISTS the backward walks */
	RGS_IMG_STRIP_ORDER,        /* uint32[4*tiles] the strips by decreasing RGS_IMG_STRIP_FILED: the order the backward blend takes them in */
	RGS_IMG_STRIP_TOTAL,        /* uint32[4*tiles] per strip: entries of RGS_BIN_STRIP_LISTS in all */
	RGS_IMG_STRIP_ORDER_FORWARD,/* uint32[4*tiles] the strips by decreasing RGS_IMG_STRIP_TOTAL: the order the forward blend takes them in */
	RGS_IMG_FIELDS
};
int rgs_geom_layout(int P, size_t offsets[RGS_GEOM_FIELDS]);
/* After rgs_forward_raster the *_UNSORTED arrays have been used as sort scratch.  Which
 * physical buffer ends up holding the sorted data depends on the number of radix
 * passes, so the layout is reported for a given image size. */
int rgs_binning_layout(int R, int width, int height, size_t offsets[RGS_BIN_FIELDS]);
int rgs_image_layout(int width, int height, size_t offsets[RGS_IMG_FIELDS]);

/* ---- rasterizer ---------------------------------------------------------------------- */

/* Frustum mask: present[i] = (view-space z of means3D[i] > 0.2).
 * Replaces Rasterizer::markVisible (K/cuda_rasterizer_hgs/rasterizer.h:22-27,
 * rasterizer_impl.cu:141-153) behind _C.mark_visible (K/ext.cpp:18). */
int rgs_mark_visible(int P, const float* means3D, const float* viewmatrix, const float* projmatrix,
                     uint8_t* present, void* stream);

/* cov3D[6 i .. 6 i + 5] = the upper triangle of R S S^T R^T of Gaussian i (S = scale_modifier * scales, R from the
 * quaternion), exactly as the forward and the backward compute it for themselves: neither keeps it in a workspace.
 * Restates computeCov3D (K/cuda_rasterizer_hgs/forward.cu:117-152), which the reference reaches only from inside
 * preprocessCUDA; offered for callers and tests that want the values. */
int rgs_covariance3d(int P, const float* scales, float scale_modifier, const float* rotations, float* cov3D, void* stream);

/* First half of Rasterizer::forward (K/cuda_rasterizer_hgs/rasterizer.h:29-58,
 * rasterizer_impl.cu:198-287): per-Gaussian preprocess and the prefix sum of the tile
 * counts.  Writes radii[P], fills the geometry workspace and stores the number of
 * (Gaussian, tile) instances R to *num_rendered_host (host memory, preferably
 * pinned); the call returns when that copy has completed, which is where the reference
 * blocks too (rasterizer_impl.cu:287); kernels that prepare the sort may still be running
 * on the stream.
 * Exactly one of shs / colors_precomp and one of (scales, rotations) / cov3D_precomp
 * is non-NULL.  D = active SH degree (0..3), M = SH coefficients per Gaussian. */
int rgs_forward_geom(int P, int D, int M, int width, int height,
                     const float* means3D, const float* shs, const float* colors_precomp, const float* opacities,
                     const float* scales, float scale_modifier, const float* rotations, const float* cov3D_precomp,
                     const float* viewmatrix, const float* projmatrix, const float* cam_pos,
                     float tan_fovx, float tan_fovy, int prefiltered,
                     int* radii, void* geom_ws, size_t geom_bytes,
                     uint32_t* num_rendered_host, void* stream, int debug);

/* rgs_forward_geom without the wait: enqueues the same work and the copy of R to
 * *num_rendered_pinned, which must be pinned host memory, and returns.  count_ready_event
 * (a hipEvent_t, or NULL) is recorded right behind that copy, ahead of the kernels that
 * do not concern the host; the caller reads R once that event (or the whole stream) has
 * completed.  The reference has no counterpart (it always blocks, rasterizer_impl.cu:287);
 * this is for a caller that renders several submodels of a frame on separate streams and
 * wants every geometry stage in flight before it waits for the first count. */
int rgs_forward_geom_enqueue(int P, int D, int M, int width, int height,
                     const float* means3D, const float* shs, const float* colors_precomp, const float* opacities,
                     const float* scales, float scale_modifier, const float* rotations, const float* cov3D_precomp,
                     const float* viewmatrix, const float* projmatrix, const float* cam_pos,
                     float tan_fovx, float tan_fovy, int prefiltered,
                     int* radii, void* geom_ws, size_t geom_bytes,
                     uint32_t* num_rendered_pinned, void* count_ready_event, void* stream, int debug);

/* Second half of Rasterizer::forward (rasterizer_impl.cu:289-351): key duplication,
 * stable sort of the (tile | depth) keys, tile ranges and the per-tile blend with the
 * per-pixel submodel-box test.  R is the value rgs_forward_geom reported.
 * Writes out_color (3,H,W), out_depth (1,H,W), out_alpha (1,H,W). */
int rgs_forward_raster(int P, int R, int width, int height,
                       const float* background, float tan_fovx, float tan_fovy,
                       const float* projmatrix_inv, const float* range_low, const float* range_up,
                       const float* colors_precomp, const int* radii,
                       void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                       void* image_ws, size_t image_bytes,
                       float* out_color, float* out_depth, float* out_alpha, void* stream, int debug);

/* rgs_forward_raster for a caller that does not wait for the instance count: R_bound sizes the
 * binning workspace (rgs_binning_bytes(R_bound)) and the launches, and the kernels take the
 * count the geometry stage left on the device.  The host never learns R before launching, so
 * a frame's forward needs no round trip; the price is a check afterwards: if the count that
 * rgs_forward_geom_enqueue delivered exceeds R_bound, instances beyond it were dropped, the images
 * are wrong and the call must be repeated with a larger bound (nothing is written out of bounds).
 * rgs_backward is then given R_bound as its R.  The reference has no counterpart: it sizes its
 * buffers after a blocking read of the count (rasterizer_impl.cu:287-292), through callbacks that
 * grow them (K/rasterize_points.cu:27-33). */
int rgs_forward_raster_bounded(int P, int R_bound, int width, int height,
                       const float* background, float tan_fovx, float tan_fovy,
                       const float* projmatrix_inv, const float* range_low, const float* range_up,
                       const float* colors_precomp, const int* radii,
                       void* geom_ws, size_t geom_bytes, void* binning_ws, size_t binning_bytes,
                       void* image_ws, size_t image_bytes,
                       float* out_color, float* out_depth, float* out_alpha, void* stream, int debug);

/* grad_accum is scratch for the backward pass: RGS_ACC_FLOATS floats per Gaussian in which
 * the backward blend accumulates its per-Gaussian sums atomically (one 48-byte row per
 * Gaussian, so that the adds a wavefront issues for one Gaussian share a cache line).  The
 * library clears it and the fused preprocess backward consumes it; its contents are not
 * part of the interface. */
enum { RGS_ACC_FLOATS = 12 };

/* Rasterizer::backward (K/cuda_rasterizer_hgs/rasterizer.h:60-96, rasterizer_impl.cu:355-466)
 * together with the zero-initialisation done by its torch shim
 * (K/rasterize_points.cu:165-174).  grad_accum is RGS_ACC_FLOATS*P floats.  dL_dmean2D (P,3; third column 0), dL_dopacity (P), dL_dcolor (P,3),
 * dL_dmean3D (P,3), dL_dcov3D (P,6), dL_dsh (P,M,3), dL_dscale (P,3), dL_drot (P,4) are
 * complete when the call has run: every row is written, those of Gaussians that were not
 * rendered as zeros, so the arrays may arrive uninitialised (the reference's shim clears them
 * first and writes the rendered rows).  Only grad_accum has to be zero when the blend starts:
 * with accum_zeroed = 0 the library clears it, a caller that hands it over cleared (say, while
 * the forward pass was still running) passes 1.  dL_dsh / dL_dscale / dL_drot may be NULL when
 * shs / scales are NULL (given without scales, dL_dscale and dL_drot are filled with zeros);
 * dL_dcolor may be NULL when shs are given and dL_dcov3D when scales are (they are
 * intermediates then: the reference fills them, a caller that hands them to nobody saves their
 * traffic); dL_dpix_depth / dL_dalphas may be NULL when no gradient arrived for the depth /
 * alpha image (taken as zero). */
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
                 int debug);

/* ---- the submodels of a frame in one go ----------------------------------------------------------
 * The reference renders the submodels that a camera sees one call after the other
 * (gather_RenderResult_pool, parallel_utils/basic_parallel_trainer/result_aggregator.py:22-38) and hands
 * each its gradient in turn (trainer4tree_partition.py:505-514).  These two entry points take all of them
 * ("layers": same camera, same image size) so that the per-tile blends, whose launches end with a few
 * long tiles each, run as one launch per frame in which the layers' tails overlap.  A layer's fields are
 * the arguments of rgs_forward_raster / rgs_backward with the same meaning; the geometry stage of every
 * layer (rgs_forward_geom or rgs_forward_geom_enqueue) comes first and supplies R.  Results are those of
 * the per-layer calls, bit for bit in the forward. */
#define RGS_MAX_FRAME_LAYERS 64
typedef struct rgs_frame_view {
	int width, height;
	float tan_fovx, tan_fovy;
	const float* viewmatrix;
	const float* projmatrix;
	const float* projmatrix_inv;
	const float* cam_pos;
} rgs_frame_view;
typedef struct rgs_frame_layer {
	int P, D, M, R;
	const float* means3D;
	const float* shs;
	const float* colors_precomp;
	const float* opacities;
	const float* scales;
	const float* rotations;
	const float* cov3D_precomp;
	float scale_modifier;
	const float* background;
	const float* range_low;
	const float* range_up;
	const int* radii;
	void* geom_ws;
	void* binning_ws;
	void* image_ws;
	size_t geom_bytes, binning_bytes, image_bytes;
	float* out_color;          /* forward outputs; the backward reads out_alpha */
	float* out_depth;
	float* out_alpha;
	const float* dL_dpix;      /* backward inputs; depth / alpha may be NULL */
	const float* dL_dpix_depth;
	const float* dL_dalphas;
	float* grad_accum;         /* backward scratch and outputs, as in rgs_backward */
	float* dL_dmean2D;
	float* dL_dopacity;
	float* dL_dcolor;
	float* dL_dmean3D;
	float* dL_dcov3D;
	float* dL_dsh;
	float* dL_dscale;
	float* dL_drot;
	int accum_zeroed;          /* as in rgs_backward: grad_accum arrives cleared */
	void* stream;              /* NULL, or a second HIP stream for rgs_frame_backward (the forward calls ignore it): work that is
	                              bound by memory bandwidth (the per-Gaussian backward of the layers whose blend is done) then
	                              runs on it beside the blend, which is bound by instruction issue; the frame's stream waits for it */
} rgs_frame_layer;
/* rgs_forward_geom for every layer (P > 0 each): every geometry stage of every layer is queued on `stream` (one
 * launch per stage for all layers; rgs_frame_layer.stream is not looked at by the forward) before the host waits for
 * the instance counts; returns when all counts have arrived in counts_pinned[0..K) (pinned host memory), which is
 * also where the layers' R for the next call is read from. */
int rgs_frame_forward_geom(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, uint32_t* counts_pinned,
                           void* stream, int debug);
/* rgs_forward_raster for every layer (P > 0 each): the key duplication, sort, ranges and strip lists, each one
 * launch for all layers, then one blend launch for all, everything on `stream`.  `layers` and `view` are HOST
 * structures. */
int rgs_frame_forward_raster(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, void* stream, int debug);
/* rgs_backward for every layer: the blend backward of all layers in one launch (two, one behind the other, when a
 * layer names a second stream, so that the first half's per-Gaussian backward runs beside the second half's blend),
 * then each layer's per-Gaussian backward.  Only the first stream among the layers' that differs from `stream` is
 * used; `stream` waits for it before the call's work counts as done.  While rgs_stage_timing is on, everything runs
 * on `stream`. */
int rgs_frame_backward(int K, const rgs_frame_layer* layers, const rgs_frame_view* view, void* stream, int debug);

/* ---- measurement aids (no counterpart in the reference, which times whole iterations
 * with CUDA events: parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:590-643) -- */

/* Per-stage timing with HIP events on the caller's stream.  rgs_stage_timing(1) clears and
 * starts recording, rgs_stage_timing(0) stops.  rgs_stage_timing_read waits for the recorded
 * work, fills up to max_stages (name, total milliseconds, launches) triples, clears the record
 * and returns the number of stages (negative on error).  The names are static strings.
 * Recording is process-wide: calls from several host threads are safe but land in one record, interleaved, so
 * measure from one thread and leave it off otherwise.  The time between two
 * consecutive events is charged to the earlier one's stage, which takes a single stream: while recording is on,
 * rgs_frame_backward does not use a second stream. */
int rgs_stage_timing(int enable);
int rgs_stage_timing_read(int max_stages, const char** names, float* total_ms, int* launches);

/* Work accounting of the blend for the frame held in the workspaces after rgs_forward_raster:
 * re-walks every tile exactly like the forward blend and writes RGS_WORK_COUNTERS uint64 sums
 * to `counters` (device memory): [0] list entries visited by a live pixel, [1] of those with
 * power <= 0, [2] with alpha >= 1/255, [3] inside the submodel box, [4] blended; [5], [6] are
 * [1], [2] restricted to entries up to each pixel's last blended one (the backward's share), and
 * [7] is [0] restricted the same way. */
#define RGS_WORK_COUNTERS 8
int rgs_blend_work_counters(int P, int R, int width, int height, float tan_fovx, float tan_fovy,
                            const float* projmatrix_inv, const float* range_low, const float* range_up,
                            const float* colors_precomp, const void* geom_ws, const void* binning_ws,
                            const void* image_ws, uint64_t* counters, void* stream);

/* ---- stand-alone binning primitives ---------------------------------------------------- */

/* Inclusive uint32 prefix sum; replaces the cub::DeviceScan::InclusiveSum call at
 * K/cuda_rasterizer_hgs/rasterizer_impl.cu:283.  temp: rgs_scan_temp_bytes(n) bytes. */
size_t rgs_scan_temp_bytes(size_t n);
int rgs_inclusive_sum(const uint32_t* in, uint32_t* out, size_t n, void* temp, void* stream);

/* Stable sort of (uint64 key, uint32 value) pairs on key bits [0, end_bit); replaces the
 * cub::DeviceRadixSort::SortPairs call at K/cuda_rasterizer_hgs/rasterizer_impl.cu:312-317.
 * keys_in / vals_in are overwritten (used as scratch).  temp: rgs_sort_temp_bytes(n) bytes. */
size_t rgs_sort_temp_bytes(size_t n);
int rgs_sort_pairs(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                   int end_bit, void* temp, void* stream);

/* Waits for `stream`, then returns non-zero (and clears the report) if a sort of an earlier call on
 * the current device gave up; see the note at the top.  That includes rgs_sort_pairs_static, whose report is a word
 * of device memory beside its scratch (read here with a 4-byte copy; nothing is allocated for it). */
int rgs_sort_fault(void* stream);

/* Test hook: the number of polls a look-back of the sorts allows before it gives up (0 restores
 * the default of 2^18; a negative value makes every look-back give up at once, which drives the
 * give-up path from the host while every kernel still runs to its end).  Process-wide. */
int rgs_set_lookback_spin_limit(int polls);

/* rgs_sort_pairs for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it): the same sort with the same results, whose
 * scratch is an array the library itself holds on every device it runs on (about 8.4 MB, until
 * the process ends), so no workspace is passed.  No counterpart in the reference, whose
 * cub::DeviceRadixSort::SortPairs always works in a buffer the caller grows
 * (K/cuda_rasterizer_hgs/rasterizer_impl.cu:188-194, 312-317).  n <= RGS_STATIC_SORT_MAX_PAIRS, else the
 * call fails.  It calls no allocation routine; all calls on one device share the one array, so
 * calls that overlap on a device (two streams, two threads) race: issue them on one stream. */
#define RGS_STATIC_SORT_MAX_PAIRS (1 << 22)
int rgs_sort_pairs_static(uint64_t* keys_in, uint64_t* keys_out, uint32_t* vals_in, uint32_t* vals_out, size_t n,
                          int end_bit, void* stream);

/* ---- partial-image compositor ------------------------------------------------------------
 * Replaces the tensor expression in blender_render_result
 * (parallel_utils/basic_parallel_trainer/result_aggregator.py:244-259) and its autograd
 * backward.  images[k] (3,H,W), depths[k] (1,H,W), alphas[k] (1,H,W) are HOST arrays of
 * K device pointers, already in front-to-back order; K <= RGS_MAX_COMPOSITE.
 * background: 3 floats on the device, or NULL for black. */
#define RGS_MAX_COMPOSITE 64
int rgs_composite_forward(int K, int height, int width,
                          const float* const* images, const float* const* depths, const float* const* alphas,
                          const float* background, float* out_image, float* out_depth, float* out_alpha,
                          void* stream);
/* g_depth / g_alpha may be NULL (treated as zero).  d_images[k], d_depths[k], d_alphas[k]
 * receive the gradients and are fully written. */
int rgs_composite_backward(int K, int height, int width,
                           const float* const* images, const float* const* depths, const float* const* alphas,
                           const float* background, const float* g_image, const float* g_depth,
                           const float* g_alpha, float* const* d_images, float* const* d_depths,
                           float* const* d_alphas, void* stream);

/* ---- boundary straddlers: what a submodel lends to its neighbours ---------------------------
 * The reference picks, per source submodel, the Gaussians whose 3-sigma cube reaches a face of
 * the source's box, then per destination those whose cube meets the destination's box, with
 * boolean-mask indexing of six tensors each time (gather_SharedGSInfo_with_boxes,
 * parallel_utils/basic_parallel_trainer/result_aggregator.py:55-121), and concatenates a
 * destination's own rows with what every other submodel lends it (merge_SharedGSInfo,
 * result_aggregator.py:263-288).  Here the selection yields row lists and the merge reads the
 * sources through them, once.
 *
 * rgs_straddler_select: means3D (n,3), scales (n,3; activated) on the device.  src_low/src_up
 * (3 floats) and boxes_low/boxes_up (n_boxes x 3) are HOST arrays in world units;
 * n_boxes <= RGS_MAX_SHARE_BOXES.  Box `skip` (the source itself; -1 for none) is lent nothing.
 * counts[b] (device) receives the number of rows lent to box b and rows[b*capacity + j] their
 * row numbers in ascending order; a count above `capacity` means the list was truncated and
 * the call must be repeated with more room.  scratch: rgs_straddler_scratch_bytes(n, n_boxes). */
#define RGS_MAX_SHARE_BOXES 64
size_t rgs_straddler_scratch_bytes(int n, int n_boxes);
int rgs_straddler_select(int n, const float* means3D, const float* scales,
                         const float* src_low, const float* src_up,
                         int n_boxes, const float* boxes_low, const float* boxes_up, int skip,
                         uint32_t* counts, uint32_t* rows, uint32_t capacity, void* scratch, void* stream);

/* One source's share of a destination: the five forward fields of the reference's SharedGSInfo
 * (parallel_utils/basic_parallel_trainer/task_utils.py:230-247; its means2D is all zero in the
 * forward direction, render_half_gs.py:7-14), device arrays of widths 3, 1, 3, 4, sh_floats,
 * and the rows to take (device; NULL takes rows 0..count-1, which is how a destination's own
 * rows are passed). */
typedef struct rgs_shared_rows {
	const float* means3D;
	const float* opacity;
	const float* scales;
	const float* rotations;
	const float* shs;
	const uint32_t* rows;
	uint32_t count;
} rgs_shared_rows;
/* Writes the segments one behind the other into the destination's arrays from row dst_row0 on
 * (torch.cat of the picked rows, result_aggregator.py:279-286).  `segments` is a HOST array. */
int rgs_merge_rows(int n_segments, const rgs_shared_rows* segments, uint32_t dst_row0, int sh_floats,
                   float* means3D, float* opacity, float* scales, float* rotations, float* shs, void* stream);

/* The adjoint (what autograd does for indexing followed by torch.cat): the gradient rows
 * dst_row0.. of the merged arrays are ADDED to the rows they were read from.  A segment names
 * the source's six gradient arrays (means2D included: its gradient is what densification reads,
 * render_half_gs.py:16-18) and the same row list as in the forward, which must not be NULL.
 * Any array pointer may be NULL on either side (that field is skipped). */
typedef struct rgs_shared_grads {
	float* means3D;
	float* means2D;
	float* opacity;
	float* scales;
	float* rotations;
	float* shs;
	const uint32_t* rows;
	uint32_t count;
} rgs_shared_grads;
int rgs_merge_rows_backward(int n_segments, const rgs_shared_grads* segments, uint32_t dst_row0, int sh_floats,
                            const float* g_means3D, const float* g_means2D, const float* g_opacity,
                            const float* g_scales, const float* g_rotations, const float* g_shs, void* stream);

/* ---- image loss ------------------------------------------------------------------------------
 * loss = (1 - lambda_dssim) * mean|image - gt| + lambda_dssim * (1 - SSIM(image, gt)), what
 * loss_local computes per camera (parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:
 * 436-455) from l1_loss and ssim (utils/loss_utils.py:17-18, 39-63: 11x11 Gaussian window, sigma
 * 1.5, zero padding, mean over all pixels and channels).  image, gt: (channels, height, width)
 * on the device.  out receives 3 floats on the device: the loss, the L1 term, the SSIM.
 * workspace: rgs_loss_workspace_bytes() bytes; with keep_for_backward it keeps what
 * rgs_l1_ssim_backward needs until that call.  The backward writes d loss / d image scaled by
 * *grad_loss (a device scalar; NULL means 1); image, gt and lambda_dssim must be the forward's. */
size_t rgs_loss_workspace_bytes(int channels, int height, int width);
int rgs_l1_ssim_forward(int channels, int height, int width, const float* image, const float* gt,
                        float lambda_dssim, float* out, void* workspace, int keep_for_backward, void* stream);
int rgs_l1_ssim_backward(int channels, int height, int width, const float* image, const float* gt,
                         float lambda_dssim, const float* grad_loss, const void* workspace, float* d_image,
                         void* stream);

/* ---- activation ------------------------------------------------------------------------------
 * From a submodel's stored parameters to the tensors its renderer and its neighbours see
 * (scene/gaussian_nn_module.py:373-394: get_scaling = exp, get_opacity = sigmoid, get_rotation =
 * torch.nn.functional.normalize, get_features = cat(features_dc, features_rest); get_xyz is the
 * stored tensor itself and has no part here).  features_dc (n,1,3), features_rest (n,rest,3),
 * scaling (n,3), rotation (n,4), opacity (n,1) in; shs (n,1+rest,3), scales, rotations, opacities
 * out; all on the device.  The backward turns the gradients of the four outputs (any may be NULL:
 * that parameter's gradient is then not written) into gradients of the five stored tensors; it
 * reads the stored rotation and the activated scales and opacities the forward wrote.  Every array
 * except features_dc / features_rest and their gradients must start at a multiple of 16 bytes. */
int rgs_activate_forward(int n, int rest, const float* features_dc, const float* features_rest, const float* scaling,
                         const float* rotation, const float* opacity, float* shs, float* scales, float* rotations,
                         float* opacities, void* stream);
int rgs_activate_backward(int n, int rest, const float* rotation, const float* scales, const float* opacities,
                          const float* g_shs, const float* g_scales, const float* g_rotations, const float* g_opacities,
                          float* d_features_dc, float* d_features_rest, float* d_scaling, float* d_rotation,
                          float* d_opacity, void* stream);

/* ---- optimiser step ---------------------------------------------------------------------------
 * torch.optim.Adam without weight decay or amsgrad, as the reference sets it up per submodel
 * (scene/gaussian_nn_module.py:429-444) and steps it once per iteration
 * (trainer4tree_partition.py:662-666): for every tensor, with t = step (>= 1, the count
 * including this update),
 *   exp_avg = beta1 exp_avg + (1 - beta1) grad;  exp_avg_sq = beta2 exp_avg_sq + (1 - beta2) grad^2;
 *   param -= lr / (1 - beta1^t) * exp_avg / (sqrt(exp_avg_sq) / sqrt(1 - beta2^t) + eps).
 * `tensors` is a HOST array (one entry per parameter group member); all arrays on the device,
 * n floats each.  Hyper-parameters are doubles, as torch holds them: 1 - beta and the bias
 * corrections are formed in double and rounded to float once.  One launch per 16 tensors. */
typedef struct rgs_adam_tensor {
	float* param;
	const float* grad;
	float* exp_avg;
	float* exp_avg_sq;
	size_t n;
	double lr;
	int step;
} rgs_adam_tensor;
int rgs_adam_step(int n_tensors, const rgs_adam_tensor* tensors, double beta1, double beta2, double eps, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RGS_H_INCLUDED */
