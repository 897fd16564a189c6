/* trigrad_hip.h -- C ABI of libtrigrad_hip.so, the MI355X (gfx950) implementation of
 * trigrad's differentiable tile rasterizer.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - the library allocates nothing and keeps no state between calls: the
 *     caller owns every buffer, including workspaces, whose size the
 *     *_workspace_bytes functions report (one entry point,
 *     tg_scan_exclusive_u32_noalloc, works in a device array of its own
 *     instead of a workspace);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all
 *     work is enqueued on it and no entry point synchronises;
 *   - the return value is 0 on success, a negative TG_E_* code for rejected
 *     arguments, or a positive hipError_t; tg_last_error() describes the last
 *     failure on the calling thread;
 *   - data layout is the reference's: vertices (V,4) tg_real
 *     (x/w, y/w, z/w, 1/w), indices (M,3) int32, colors (V,3), opacities (V),
 *     image (H,W,4) with remaining transmittance in channel 3, row 0 at
 *     y = -1 (reference src/trigrad/wrapper.py:131-141, render.cu:557-562).
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the reference tree).
 */
#ifndef TRIGRAD_HIP_H
#define TRIGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TG_ABI_VERSION 1

/* The scalar type of the build, like the reference's `scalar` (util.h:5-20):
 * libtrigrad_hip.so is built with float, libtrigrad_hip_f64.so with
 * -DTG_DOUBLE_PRECISION (the reference's DOUBLE_PRECISION switch, which lets
 * its gradcheck tests run).  tg_precision_bits() tells which one a library is. */
#ifdef TG_DOUBLE_PRECISION
typedef double tg_real;
#else
typedef float tg_real;
#endif

#define TG_E_ARG (-1)       /* null pointer, negative size, unsupported tile size */
#define TG_E_WORKSPACE (-2) /* workspace too small */

#define TG_MAX_SAVED_LAYERS 32 /* largest max_layers for which the forward pass can save the blend order */

/* Status word values written by the kernels that wait on other workgroups
 * (the scans' and the sweeps' decoupled look-back).  Their waits are bounded: a
 * wait that expires sets TG_STATUS_LOOKBACK_TIMEOUT and the kernel carries on,
 * so every wave exits; the results of that call are then invalid and the
 * caller must look at the word before it trusts them.  A grid that fits the
 * device whole numbers its tiles by workgroup id (every workgroup it waits
 * for is resident by then); that presumes the kernel has the device to itself.
 * With other streams or processes on the GPU a wait can expire. */
#define TG_STATUS_OK 0u
#define TG_STATUS_LOOKBACK_TIMEOUT 1u

int tg_version(void);
int tg_precision_bits(void); /* 32 or 64 */

/* on != 0: every kernel that waits on other workgroups numbers its tiles by an
 * atomic ticket, whatever the size of its grid, so that it only ever waits
 * for workgroups that already run.  Slower (the tickets are same-address
 * atomics), and safe when the device is shared; for a caller that has seen
 * TG_STATUS_LOOKBACK_TIMEOUT.  Process-wide, like tg_profile_enable. */
void tg_force_tickets(int on);
const char *tg_last_error(void);

/* Number of tiles of a W x H image (reference render.cu:105-106). */
int tg_num_tiles(int width, int height, int tile_w, int tile_h);

/* Per-kernel timing, the counterpart of the reference's CudaTimer
 * (render.cu:11-49).  While enabled, every kernel launch of the library is
 * bracketed by events on its stream.  tg_profile_report waits for them, writes
 * one line "kernel_name launches total_milliseconds" per kernel into buffer
 * (host, NUL-terminated, truncated to capacity), forgets them, and returns the
 * length of the full text. */
void tg_profile_enable(int on);
int tg_profile_report(char *buffer, size_t capacity);

/* ---- (1) tile binning ------------------------------------------------------- */

/* Per-triangle screen bounds and tile-overlap count: tri_counts[i] = number of
 * tiles in the clamped tile AABB of triangle i, 0 for a degenerate triangle or
 * one with a vertex index outside [0, n_vertices).
 * Replaces count_per_tile / count_per_tile_kernel / touched_tiles
 * (render.cu:51-76, 90-139); the per-tile histogram of the reference is not
 * needed by the key pipeline (the tile ranges come out of the sort). */
int tg_bin_count(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width, int height, int tile_w,
                 int tile_h, uint32_t *tri_counts, void *stream);

/* Exclusive prefix sum of n uint32 (single pass, decoupled look-back).
 * out[i] = sum(in[0..i)), *total = sum(in[0..n)).  Replaces the
 * sum().item() / cumsum_out sequence of per_tile_lists (render.cu:290-295).
 * `status` (1 uint32, may be NULL) receives TG_STATUS_*; in and out may alias.
 * Optional (heads may be NULL): for every h < head_capacity with
 * h * head_stride < total, heads[h] = the index i whose output range
 * [out[i], out[i] + in[i]) contains position h * head_stride.  tg_bin_emit uses
 * it (head_stride 256) to find the triangle that owns a key without searching. */
size_t tg_scan_workspace_bytes(int64_t n);
int tg_scan_exclusive_u32(const uint32_t *in, uint32_t *out, int64_t n, uint32_t *total, void *workspace,
                          size_t workspace_bytes, uint32_t *status, uint32_t head_stride, uint32_t head_capacity,
                          uint32_t *heads, void *stream);

/* The same scan with nothing to allocate.  It has no counterpart in the
 * reference: it is for callers that cannot allocate device memory or pass a
 * workspace (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  The look-back state lives in a device array inside
 * the library (65 600 bytes per GPU: 64 for the ticket, 8 for each of 8192 tiles
 * of 2048 elements; held until the process ends) instead of a
 * workspace; the call allocates and frees nothing.  n may not exceed
 * TG_SCAN_NOALLOC_MAX_N = tg_scan_noalloc_max_n() (TG_E_ARG otherwise).  All
 * calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are safe.  Otherwise as
 * tg_scan_exclusive_u32, result for result. */
#define TG_SCAN_NOALLOC_MAX_N (1 << 24)
int64_t tg_scan_noalloc_max_n(void);
int tg_scan_exclusive_u32_noalloc(const uint32_t *in, uint32_t *out, int64_t n, uint32_t *total, uint32_t *status,
                                  uint32_t head_stride, uint32_t head_capacity, uint32_t *heads, void *stream);

/* Key emission: for triangle i and each tile of its AABB (tile x outer, tile y
 * inner, render.cu:235-236), at position tri_offsets[i] + local:
 *   keys[pos]    = (tile_id << 32) | orderable(depth_key)
 *   payload[pos] = i
 * where depth_key is the minimum of the triangle's z plane over the triangle
 * clipped to the tile (1e30 when the clip is empty) and orderable() is the
 * order-preserving map of tg_real bits to uint32.  Replaces
 * fill_per_tile_lists_kernel, compute_plane, clip_polygon_to_halfspace
 * (render.cu:140-270).  n_keys = total of the scan.  owner_heads (may be NULL)
 * is the scan's `heads` output for head_stride = 256 with owner_capacity
 * entries; without it the owners are found by binary search.
 * Double-precision build: a depth key needs all 64 bits, so keys holds
 * 2 * n_keys words, keys[pos] = orderable(depth_key) and
 * keys[n_keys + pos] = tile_id; the caller sorts by depth, then stably by tile
 * (two calls of tg_sort_pairs_u64_u32). */
int tg_bin_emit(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width, int height, int tile_w,
                int tile_h, const uint32_t *tri_offsets, int64_t n_keys, const uint32_t *owner_heads,
                uint32_t owner_capacity, uint64_t *keys, uint32_t *payload, void *stream);

/* ---- (2) radix sort --------------------------------------------------------- */

/* Stable LSD radix sort of (uint64 key, uint32 value) pairs on key bits
 * [0, end_bit).  Replaces cub::DeviceSegmentedSort::StableSortPairs as called
 * by sort_depth_ranges (render.cu:272-284): with the tile id in the high word
 * one global stable sort yields every tile segment sorted by depth with ties
 * in input order.  Both buffer pairs are used as ping-pong storage;
 * *result_in_alt (host) is set to 0 when the sorted data ends in
 * (keys, values), 1 when it ends in (keys_alt, values_alt). */
size_t tg_sort_workspace_bytes(int64_t n);
int tg_sort_pairs_u64_u32(uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int64_t n,
                          int end_bit, void *workspace, size_t workspace_bytes, uint32_t *status,
                          int *result_in_alt, void *stream);

/* ---- (3) tile ranges -------------------------------------------------------- */

/* offsets[t] = first position in sorted_keys whose tile id (key >> 32) is >= t,
 * for t in [0, n_tiles]; offsets[n_tiles] = n_keys.  Produces the offsets
 * array that per_tile_lists builds by cumsum (render.cu:292-295). */
int tg_tile_ranges(const uint64_t *sorted_keys, int64_t n_keys, int n_tiles, int32_t *offsets, void *stream);

/* ---- (2)+(3) for the frame: the tile lists in one call --------------------- */

/* Sorts (tile << 32 | depth bits, triangle) pairs like tg_sort_pairs_u64_u32 on
 * key bits [0, 32 + bits of n_tiles - 1) and writes the tile ranges like
 * tg_tile_ranges: same sorted keys, values and offsets, bit for bit.  Replaces
 * sort_depth_ranges and the offsets of per_tile_lists (render.cu:272-308) for
 * keys whose high word is a tile number below n_tiles.  It moves the pairs
 * through memory for the tile bits only (LSD passes of at most 8 bits with
 * decoupled look-back); the stable passes over the 32 depth bits then run per
 * tile inside one workgroup, pairs in registers and LDS (a tile list longer
 * than 8192 entries is sorted by its workgroup through memory instead).
 * *result_in_alt (host): 0 = sorted data in (keys, values), 1 = in the _alt
 * pair.  offsets: n_tiles + 1 entries. */
size_t tg_tile_list_sort_workspace_bytes(int64_t n, int n_tiles);
int tg_sort_tile_lists(uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int64_t n,
                       int n_tiles, int32_t *offsets, void *workspace, size_t workspace_bytes, uint32_t *status,
                       int *result_in_alt, void *stream);

/* ---- (1)-(3) as the frame runs them: two calls --------------------------------- */

/* tg_bin_setup = tg_bin_count + tg_scan_exclusive_u32 in one pass over the
 * triangles (count_per_tile and the cumsum of per_tile_lists, render.cu:90-139,
 * 290-295): tri_offsets[i] = number of keys of the triangles before i,
 * total_and_status[0] = K, [1] = TG_STATUS_*.  It also leaves per triangle a
 * record of TG_RECORD_SCALARS scalars (depth plane of compute_plane,
 * render.cu:140-152; first tile and rows of the tile rectangle of
 * touched_tiles, :51-76; the corners) from which tg_build_tile_lists emits the
 * keys, and in `frame` (tg_bin_setup_workspace_bytes, 256-byte aligned, the
 * caller's; both calls of a frame get the same one) the state the two calls
 * share.  heads as in tg_scan_exclusive_u32 with head_stride 256.
 *
 * tg_build_tile_lists = tg_bin_emit + tg_sort_tile_lists: emits the K keys from
 * the records (fill_per_tile_lists_kernel, render.cu:202-270), sorts them and
 * writes the tile ranges; results as those two calls give them, bit for bit.
 * While emitting it adds up the digits of the tile passes, so the sort reads
 * the keys for no histogram.  emit_only != 0: stop after the emission (keys and
 * values in emission order, as tg_bin_emit leaves them; the double build, whose
 * depth keys take 64 bits, has this mode only). */
#define TG_RECORD_SCALARS 12
size_t tg_bin_setup_workspace_bytes(int32_t n_triangles, int width, int height, int tile_w, int tile_h);
int tg_bin_setup(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width,
                 int height, int tile_w, int tile_h, uint32_t *tri_offsets, tg_real *records, uint32_t *total_and_status,
                 uint32_t head_capacity, uint32_t *heads, void *frame, size_t frame_bytes, void *stream);
size_t tg_build_tile_lists_workspace_bytes(int64_t n_keys, int n_tiles);
int tg_build_tile_lists(const tg_real *records, const uint32_t *tri_offsets, int32_t n_triangles, int64_t n_keys,
                        uint32_t head_capacity, const uint32_t *heads, void *frame, int width, int height, int tile_w,
                        int tile_h, uint64_t *keys, uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt,
                        int32_t *offsets, void *workspace, size_t workspace_bytes, uint32_t *status, int emit_only,
                        int *result_in_alt, void *stream);

/* ---- (1)-(3) as the frame runs them now: no wait for the host inside the binning ---- */

/* tg_bin_frame = tg_bin_count + tg_scan_exclusive_u32 + tg_bin_emit in one call
 * and two launches (count_per_tile, the cumsum of per_tile_lists and
 * fill_per_tile_lists_kernel, render.cu:90-139, 202-270, 290-308): keys and
 * values in tg_bin_emit's order with tg_bin_emit's depth word,
 * total_and_status[0] = K.  The high word of a key is the tile id only when the
 * frame has more than 256 tile columns or rows; otherwise it is
 * (tile row << column_bits) | tile column, column_bits = the bits that tell the
 * frame's tile columns apart (7 for 120 columns): tg_build_frame_lists sorts by
 * column, then by row, and its last pass writes the tile id, so the sorted keys
 * are those of tg_sort_tile_lists either way.  The emission
 * reads K on the device, so the host does not have to know it in between: the
 * key buffers are the caller's guess, a key whose position is key_capacity or
 * more is not written, K is exact either way, and a caller who finds
 * K > key_capacity calls again with larger buffers.  Float build only, up to
 * 2^21 tiles (tg_bin_frame_supported; tg_bin_setup + tg_build_tile_lists take
 * the rest).
 *
 * frame: tg_bin_frame_workspace_bytes() bytes, 256-byte aligned, ZERO before the
 * first call that uses it; every call leaves it ready for the next.  It holds
 * what the two launches hand each other (per-triangle records as tg_bin_setup
 * makes them) and what calls share.  epoch: its low 30 bits must not be 0,
 * must differ from those of every earlier call on this frame state since it
 * was zeroed, and its lowest bit must differ from the previous call's (count
 * up by one).  The scan marks what it publishes with the epoch, so nothing is
 * cleared between calls.  One call at a time per frame state.  A wait for
 * another workgroup that expires (see TG_STATUS_*) writes `epoch` to
 * total_and_status[1], which is not written otherwise: pass a word that holds
 * something else.
 *
 * On the side the first launch zeroes zero_bytes bytes at `zero` (pass the
 * workspace of the tg_build_frame_lists call that follows, sized for
 * key_capacity keys) and *clear_word (its status word); both may be NULL / 0.
 *
 * tg_build_frame_lists = tg_sort_tile_lists on the keys tg_bin_frame emitted
 * (sort_depth_ranges and the offsets of per_tile_lists, render.cu:272-308),
 * same results bit for bit.  It takes the digit totals of the tile passes from
 * the frame state (tg_bin_frame counted them for `epoch`), so it reads the keys
 * for no histogram.  workspace: tg_build_frame_lists_workspace_bytes(), zeroed
 * by the tg_bin_frame call; status: cleared by that call. */
int tg_bin_frame_supported(int width, int height, int tile_w, int tile_h);
size_t tg_bin_frame_workspace_bytes(int32_t n_triangles, int64_t key_capacity, int width, int height, int tile_w, int tile_h);
int tg_bin_frame(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, int width,
                 int height, int tile_w, int tile_h, uint64_t *keys, uint32_t *values, int64_t key_capacity,
                 uint32_t *total_and_status, void *frame, size_t frame_bytes, uint32_t epoch, void *zero,
                 size_t zero_bytes, uint32_t *clear_word, void *stream);
size_t tg_build_frame_lists_workspace_bytes(int64_t n_keys, int tiles_x, int tiles_y);
int tg_build_frame_lists(void *frame, uint32_t epoch, int64_t n_keys, int tiles_x, int tiles_y, uint64_t *keys,
                         uint32_t *values, uint64_t *keys_alt, uint32_t *values_alt, int32_t *offsets, void *workspace,
                         size_t workspace_bytes, uint32_t *status, int *result_in_alt, void *stream);

/* ---- bary matrices ---------------------------------------------------------- */

/* Row-major 3x3 cartesian-to-barycentric matrix per triangle, out is (M,3,3).
 * Replaces cartesian_to_bary / cartesian_to_bary_kernel (render.cu:310-337,
 * 697-711), also exported by the reference as _C.cartesian_to_bary. */
int tg_bary(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles, tg_real *out,
            void *stream);

/* ---- depth bounds of the lists (optional) ------------------------------------- */

/* bounds (tg_list_bound_words() scalars): for every tile and every 256 entries
 * of its list a lower bound of the per-pixel depth (render.cu:404) of the
 * entries from there to far_start[tile]; far_start (n_tiles int32): the list
 * position from which on the entries have the sort key 1e30 (empty clipped
 * polygon, render.cu:259: they sit at the end whatever their depth).  With
 * both, the per_pixel_sort selection of tg_render_forward
 * (select_next_k_in_tile, render.cu:375-415, which always scans the whole list)
 * skips from the point where every pixel's 32 candidates are nearer than
 * anything the bounds cover to far_start: same result, and lists of thousands
 * of entries are not scanned to the end.  triangle_low: n_triangles scalars of
 * working memory (every triangle's own bound). */
size_t tg_list_bound_words(int64_t n_keys, int n_tiles);
int tg_list_bounds(const tg_real *vertices, int32_t n_vertices, const int32_t *indices, int32_t n_triangles,
                   const uint64_t *sorted_keys, const int32_t *sorted_ids, const int32_t *offsets, int n_tiles,
                   tg_real *triangle_low, tg_real *bounds, int32_t *far_start, void *stream);

/* ---- (4) forward blend ------------------------------------------------------ */

/* One workgroup per tile composites the tile's sorted list.  Replaces
 * render_forward_kernel and its helpers (render.cu:338-453, 540-619).
 * Outputs: image (H,W,4), depthmap (H,W), final_weights (H,W), ends (H,W) =
 * number of blended fragments (the reference's `ends`), and last (H,W) = one
 * past the tile-list position, relative to the tile's start, of the last
 * blended entry, and last_depth (H,W) = that entry's pixel depth when
 * per_pixel_sort is on (render.cu:605-606 lastJ / lastDepth).  last and
 * last_depth may be NULL; the backward pass needs them.
 * fragments (2*max_layers,H,W) uint16, or NULL: with per_pixel_sort and
 * max_layers <= TG_MAX_SAVED_LAYERS the kernel also writes, for every pixel,
 * the list positions (relative to the tile's start) of its blended fragments
 * in blend order: the low 16 bits of layer k of pixel p at fragments[k*H*W + p],
 * k < ends[p], and, only in tiles whose list holds more than 65535 entries, the
 * high 16 bits at fragments[(max_layers + k)*H*W + p] (elsewhere that half is
 * left as it was).  tg_render_backward then walks them backwards instead of
 * selecting the fragments again (the reference re-selects, render.cu:667-693).
 * hit_masks (tg_hit_mask_words() uint64 words), or NULL: without per_pixel_sort
 * the kernel also writes, for every pixel and every 64 consecutive entries of
 * its tile's list that it looked at, which of them cover the pixel, and per
 * workgroup how far into the list its pixels got; tg_render_backward then
 * reads them back instead of repeating the inside tests.  The buffer is
 * private to the two calls: its layout is theirs to change.
 * batch_bounds, far_start: tg_list_bounds' outputs, or NULL (used with per_pixel_sort only).
 * list_status (may be NULL): the status word of the call that made the lists.  If it
 * is not TG_STATUS_OK when the kernel runs, the lists are not read: image and depthmap
 * are filled with NaN (ends, last 0), so that an invalid frame shows in the frame itself.
 * max_layers must be > 0 (the Python layer maps <= 0 to M+1, wrapper.py:35). */
size_t tg_hit_mask_words(int64_t n_keys, int width, int height, int tile_w, int tile_h);
int tg_render_forward(const tg_real *vertices, const int32_t *indices, const tg_real *colors, const tg_real *opacities,
                      const int32_t *sorted_ids, const int32_t *offsets, const tg_real *bary, int width, int height,
                      int tile_w, int tile_h, tg_real early_stopping_threshold, int per_pixel_sort, int max_layers,
                      tg_real *image, tg_real *depthmap, tg_real *final_weights, int32_t *ends, int32_t *last,
                      tg_real *last_depth, uint16_t *fragments, uint64_t *hit_masks,
                      const tg_real *batch_bounds, const int32_t *far_start, const uint32_t *list_status, void *stream);

/* ---- (5) backward ----------------------------------------------------------- */

/* Accumulates into grad_vertices (V,4), grad_colors (V,3), grad_opacities (V),
 * which the caller zero-initialises.  Replaces render_backward_kernel /
 * process_backward (render.cu:455-538, 621-695).  Fragments are visited in
 * exact reverse blend order.  grad_depthmap may be NULL (= all zero: the depth
 * map took no part in the loss).  fragments, hit_masks: what tg_render_forward
 * saved, or NULL (then the fragments are selected, the inside tests made again).
 * vertex_stride, color_stride, opacity_stride: scalars from one vertex to the
 * next in the three gradient arrays, (4, 3, 1) for dense arrays.  (8, 8, 8)
 * with the pointers 0, 4 and 7 scalars into one (V,8) block keeps a vertex's
 * eight gradients in one 32-byte sector, which the atomics of the per-pixel
 * order then hit together (measured 19 % faster there). */
int tg_render_backward(const tg_real *grad_image, const tg_real *grad_depthmap, const tg_real *vertices,
                       const int32_t *indices, const tg_real *colors, const tg_real *opacities,
                       const int32_t *sorted_ids, const int32_t *offsets, const tg_real *bary, const tg_real *image,
                       const tg_real *depthmap, const tg_real *final_weights, const int32_t *ends, const int32_t *last,
                       const tg_real *last_depth, const uint16_t *fragments, const uint64_t *hit_masks, int width, int height,
                       int tile_w, int tile_h,
                       tg_real early_stopping_threshold, int per_pixel_sort, int max_layers, tg_real *grad_vertices,
                       tg_real *grad_colors, tg_real *grad_opacities, int vertex_stride, int color_stride,
                       int opacity_stride, void *stream);

/* The (V,8) block that tg_render_backward accumulates into with strides
 * (8, 8, 8) -> the three dense arrays the reference's render_backward returns
 * (render.cu:765-804: grad_vertices (V,4), grad_colors (V,3), grad_opacities
 * (V)): scalars 0..3 of a vertex's row, 4..6 and 7.  One pass over the block. */
int tg_split_gradient_block(const tg_real *block, int64_t n_vertices, tg_real *grad_vertices, tg_real *grad_colors,
                            tg_real *grad_opacities, void *stream);

/* ---- host-side component hooks ---------------------------------------------- */

/* HOST pointers, run on the CPU.  The reference exports the same six functions
 * from its extension for its component tests (tests.cu:43-76: barycentric_torch,
 * barycentric_backward_torch, interpolate3_scalar_torch, ..._backward_torch,
 * interpolate3_vector_torch, ..._backward_torch around util.h:232-250, 299-355,
 * 395-455).  2-vectors and 3-vectors are plain tg_real arrays. */
void tg_barycentric(const tg_real *v0, const tg_real *v1, const tg_real *v2, const tg_real *p, tg_real *out3);
void tg_barycentric_backward(const tg_real *g3, const tg_real *a, const tg_real *b, const tg_real *c, const tg_real *p,
                             tg_real *grads_4x2);
tg_real tg_interpolate3_scalar(const tg_real *bary, tg_real a, tg_real b, tg_real c, const tg_real *w);
void tg_interpolate3_scalar_backward(tg_real g, const tg_real *bary, tg_real a, tg_real b, tg_real c, const tg_real *w,
                                     tg_real *grad_bary, tg_real *grad_values, tg_real *grad_w);
void tg_interpolate3_vector(const tg_real *bary, const tg_real *a, const tg_real *b, const tg_real *c, const tg_real *w, tg_real *out3);
void tg_interpolate3_vector_backward(const tg_real *g3, const tg_real *bary, const tg_real *a, const tg_real *b, const tg_real *c,
                                     const tg_real *w, tg_real *grad_bary, tg_real *grad_a, tg_real *grad_b, tg_real *grad_c,
                                     tg_real *grad_w);

#ifdef __cplusplus
}
#endif
#endif /* TRIGRAD_HIP_H */
