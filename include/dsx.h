/*
 * dsx — C ABI of the MI355X (gfx950) 3D-Gaussian-Splatting rasterizer.
 *
 * Plain pointers and sizes only; no torch types.  Every pointer is DEVICE memory unless it
 * is marked "host".  `stream` is a hipStream_t passed as void* (NULL = the null stream).
 * The library allocates nothing on the device: outputs and workspace are the caller's.
 * All functions return 0 on success or a negative dsx_status; dsx_error_string() explains it.
 * Functions are re-entrant: different streams / devices may be driven concurrently by different
 * host threads (each call uses the current HIP device), and nothing that a call computes depends on
 * a process-wide setting: the bin size of the tile lists travels in dsx_camera::list_bin and, on the
 * device, in the header word of the `ranges` buffer.  What the process does share, all of it behind
 * locks or atomics: (1) the optional per-kernel timing trace (dsx_trace_enable / dsx_trace_read),
 * a list behind a mutex, off by default; (2) one helper stream per device, created on first use
 * and kept until the process ends: dsx_depth_order / dsx_forward_project fork onto it and join
 * before they return, so that the tile counting runs beside the depth sort; callers on
 * different streams of one device share it and their forked parts serialise there; (3) the
 * blend-kernel form override of dsx_set_blend_pixels_per_lane, a diagnostic that changes no result
 * of the forward and only the order of the backward's sums; (4) the device address of the
 * built-in scratch of dsx_backward_static, looked up once per device.
 *
 * What each entry point replaces in the reference (deepsense-ai/ds-splat) is cited as
 * file:line next to it.  Matrices are row-major, math convention (translation in elements
 * 3, 7, 11): what the reference's native code receives after ds_splat/rasterizer.py:147-148
 * transposed the user's matrices.
 */
#ifndef DSX_H_
#define DSX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSX_TILE 16            /* cpp/rasterizer_kernels.cuh:6 */
#define DSX_SPLAT_FLOATS 12    /* projected record, 48 bytes (3 x float4) */
#define DSX_GRAD_FLOATS 12     /* screen-space gradient accumulator record, 48 bytes */
#define DSX_PROJ_BLOCK 256     /* Gaussians per workgroup in the per-Gaussian kernels */
#define DSX_STATIC_MAX_GAUSSIANS 524288 /* largest n of dsx_backward_static (24 MiB of built-in scratch) */

typedef enum dsx_status
{
    DSX_OK = 0,
    DSX_ERR_BAD_ARG = -1,      /* NULL where data is required, negative size, bad degree ... */
    DSX_ERR_LAUNCH = -2,       /* hipGetLastError() after a launch reported a failure       */
    DSX_ERR_RUNTIME = -3,      /* a HIP runtime call (memcpy, sync, event) failed           */
    DSX_ERR_TOO_LARGE = -4,    /* 2^30 pairs or more in the lists that are built, or 2^31   */
                               /* or more in the per-tile lists (the reference's K)         */
    DSX_ERR_WORKSPACE = -5,    /* workspace smaller than dsx_workspace_bytes() asks for     */
    DSX_ERR_STATIC_LIMIT = -6  /* n beyond DSX_STATIC_MAX_GAUSSIANS (dsx_backward_static)   */
} dsx_status;

/* Mirrors TorchRasterizationSettings, cpp/ds_cuda_rasterizer/rasterizer_torch.hpp:7-22.
 * `prefiltered` and `debug` are carried by the reference but never read; they are omitted.
 * list_bin has no counterpart there: the tile lists are built per BIN of list_bin x list_bin tiles
 * (1, 2, 4 or 8; 0 = the library's choice for the image size, see dsx_list_bin).  Every call that
 * belongs to one forward and its backward must be given the same value. */
typedef struct dsx_camera
{
    int32_t image_height;
    int32_t image_width;
    float tanfovx;
    float tanfovy;
    float scale_modifier;
    int32_t sh_degree;      /* active degree, 0..3                                  */
    int32_t max_sh_degree;  /* row stride of shs is (max_sh_degree+1)^2 * 3 floats  */
    const float* view;      /* device float[16], row-major world->view              */
    const float* proj;      /* device float[16], row-major world->clip              */
    const float* campos;    /* device float[3]                                      */
    const float* bg;        /* device float[3]                                      */
    int32_t list_bin;       /* tiles per side of a list's bin: 0 (automatic), 1, 2, 4, 8 */
} dsx_camera;

/*
 * Projected record ("splat"), one per Gaussian, DSX_SPLAT_FLOATS floats:
 *   [0] pixel x   [1] pixel y   [2] view depth   [3] radius (int32 bits)
 *   [4] conic a   [5] conic b   [6] conic c      [7] opacity
 *   [8] red       [9] green     [10] blue        [11] tiles touched (int32 bits)
 * It plays the role of the reference's 48-byte `Gaussian` (cpp/rasterizer_kernels.cuh:18-26).
 *
 * Gradient accumulator record, DSX_GRAD_FLOATS floats:
 *   [0] v_x [1] v_y [2] v_conic_a [3] v_conic_b [4] v_conic_c [5] v_opacity
 *   [6] v_red [7] v_green [8] v_blue [9..11] unused (the conic, once dsx_forward_finish has prepared it)
 * The accumulator of the whole backward (dsx_forward_finish's grads_to_prepare, dsx_backward's
 * grads) is a buffer of dsx_grads_bytes(n) bytes, 16-byte aligned: the n records and, behind
 * them, one byte per Gaussian that the blend backward sets when it adds a term to the record.
 * The stage entry points dsx_blend_bwd / dsx_gaussian_bwd take the n records alone.
 */

const char* dsx_error_string(int status);
/* 100 * major + minor.  300: the bin size of the tile lists is an argument (dsx_camera::list_bin and
 * the size helpers) instead of a process-wide setting; the `ranges` buffer carries it in a header word;
 * the blend entry points and the backward are told n and k and follow no id or list position beyond
 * them; dsx_forward_project returns both pair counts.  (200 had dsx_set_list_bin.) */
int dsx_version(void);
/* bytes of the accumulator that dsx_forward_finish prepares and dsx_backward uses:
 * n * DSX_GRAD_FLOATS * 4 for the records + n bytes rounded up to 16 */
size_t dsx_grads_bytes(int64_t n);

/* number of workgroups of the per-Gaussian kernels = entries of `block_sums` */
int64_t dsx_num_blocks(int64_t n);
/* tiles of an image, and radix passes the sort runs for that many tiles */
int32_t dsx_num_tiles(int32_t width, int32_t height);
int32_t dsx_sort_passes(int32_t num_tiles);
/* The tile lists of the whole forward (dsx_forward_project / dsx_forward_finish / dsx_backward,
 * dsx_depth_order / dsx_tile_lists / dsx_blend_fwd / dsx_blend_bwd) are built per BIN of b x b tiles,
 * b = 1, 2, 4 or 8: a Gaussian enters the list of every bin that its tile rectangle touches, and a
 * blend tile walks its bin's list and keeps the entries whose rectangle contains the tile.  With
 * b = 1 the lists are the reference's own (sorted_ids is the value array of its sorted keys, bit for
 * bit); with b > 1 the same entries reach every pixel in the same order, final_idx holds the same
 * indices, and emission and partition handle a fraction of the pairs.  b is dsx_camera::list_bin, or,
 * when that is 0, the library's choice for the image size: 1 below 2048 tiles; above, 8 where that
 * brings the lists down to the 256 slots of a single partition pass and 4 does not, else 4 (and
 * never more than 65534 bins: an image of hundreds of megapixels gets 8, or per-tile lists).
 * dsx_list_bin(width, height, list_bin) returns the b that a call with this list_bin uses (0 for a
 * list_bin that is none of 0, 1, 2, 4, 8).
 * dsx_ranges_count: int32 words of the `ranges` buffer of those entry points: tiles + 1 words of
 * per-tile ranges as the reference defines them (cpp/rasterizer_torch.cu:23-42), one header word
 * (log2 of b: the blend kernels walk nothing when it is not the b they were launched for) and, for
 * b > 1, the highest occupied tile, the bins' ranges and 8 words per tile that the blend forward
 * leaves for the backward.  No counterpart in the reference. */
int32_t dsx_list_bin(int32_t width, int32_t height, int32_t list_bin);
int64_t dsx_ranges_count(int32_t width, int32_t height, int32_t list_bin);
/* int32 words of the `sorted_ids` buffer for k pairs: k ids and, for b > 1, behind them one word per
 * pair whose high half says which tiles of the bin the pair's Gaussian covers (the blend kernels pick
 * a tile's entries out of its bin's list by it): 2 k words.  Wherever this header says sorted_ids[k],
 * the buffer has this many words and k is still the number of pairs. */
int64_t dsx_sorted_ids_count(int64_t k, int32_t width, int32_t height, int32_t list_bin);
/* bytes of `workspace` dsx_forward_finish / dsx_tile_lists need for k keys */
size_t dsx_workspace_bytes(int64_t n, int64_t k, int32_t width, int32_t height, int32_t list_bin);
/* bytes of `workspace` dsx_sort_pairs needs for k keys, and dsx_sort_pairs_u32 for count pairs */
size_t dsx_sort_workspace_bytes(int64_t k, int32_t num_tiles);
size_t dsx_sort_u32_workspace_bytes(int64_t count, int32_t key_bits);
/* bytes of the per-Gaussian `order` buffer that carries the depth order from the projection
 * (dsx_project_fwd / dsx_forward_project) to the tile lists (dsx_tile_lists / dsx_forward_finish) */
size_t dsx_order_bytes(int64_t n, int32_t width, int32_t height, int32_t list_bin);

/* ------------------------------------------------------------------------------------ */
/* Per-stage entry points (each one individually parity-tested and timed)                */
/* ------------------------------------------------------------------------------------ */

/* Stage 1 — replaces rasterizer_preprocessing_kernel, cpp/rasterizer_kernels.cu:57-161 and
 * its launcher cpp/rasterizer_torch.cu:115-168.  Writes splats[n*12], radii[n], cov3d[n*6]
 * and block_sums[dsx_num_blocks(n)] (tile count of each 256-Gaussian block; the last
 * Gaussian counts as zero, cpp/rasterizer_torch.cu:99-104).  shs may be NULL iff
 * colors_precomp is given; scales/quats may be NULL iff cov3d_precomp is given (then cov3d
 * receives a copy).  cov3d may be NULL: it is then not stored (the reference keeps it for its
 * backward, cpp/rasterizer_torch.cu:207; dsx_gaussian_bwd can do without).  order (may be NULL):
 * buffer of dsx_order_bytes(n, W, H, cam->list_bin) that also receives each Gaussian's depth bits and
 * packed tile rectangle, the input of dsx_depth_order. */
int dsx_project_fwd(const dsx_camera* cam, int64_t n, const float* means3d, const float* scales,
                    const float* quats, const float* opacities, const float* shs,
                    const float* cov3d_precomp, const float* colors_precomp, float* splats,
                    int32_t* radii, float* cov3d, uint32_t* block_sums, void* order,
                    size_t order_bytes, void* stream);

/* Exclusive prefix of `count` uint32 values in place, total written to *total (device).
 * Replaces the in-block Hillis-Steele scan of cpp/rasterizer_kernels.cu:131-142 together
 * with thrust::exclusive_scan, cpp/rasterizer_torch.cu:95.  The prefixes are modulo 2^32; the
 * total saturates at 0xffffffff, so a key count that does not fit is seen as too large
 * (DSX_ERR_TOO_LARGE from dsx_forward_project) and never as a small wrapped number. */
int dsx_scan_u32(int64_t count, uint32_t* data, uint32_t* total, void* stream);

/* Stage 2a — replaces calculate_keys_and_indices_kernel, cpp/rasterizer_kernels.cu:252-306.
 * block_offsets = scanned block_sums.  keys[k] = (tile << 32) | sign-extended depth bits,
 * values[k] = Gaussian index, in emission order. */
int dsx_emit_keys(const dsx_camera* cam, int64_t n, int64_t k, const float* splats,
                  const uint32_t* block_offsets, int64_t* keys, int32_t* values, void* stream);

/* Stage 2b — replaces thrust::sort_by_key, cpp/rasterizer_torch.cu:70-76: stable ascending
 * sort of (int64 key, int32 value) pairs where every key is (tile << 32 | depth bits) with
 * tile in [0, num_tiles) or a negative key (tile field all ones).  keys/values are sorted
 * in place; workspace needs dsx_sort_workspace_bytes(k, num_tiles) bytes. */
int dsx_sort_pairs(int64_t k, int32_t num_tiles, int64_t* keys, int32_t* values, void* workspace,
                   size_t workspace_bytes, void* stream);

/* Stage 3 — replaces identify_tile_ranges + identify_tile_ranges_kernel +
 * thrust::inclusive_scan(max), cpp/rasterizer_torch.cu:23-42, cpp/rasterizer_kernels.cu:308-323.
 * ranges has num_tiles+1 entries. */
int dsx_tile_ranges(int64_t k, const int64_t* sorted_keys, int32_t num_tiles, int32_t* ranges,
                    void* stream);

/* Stages 2+3, fast route — with cam->list_bin = 1 the same sorted_ids[k] and ranges[T+1] as
 * dsx_emit_keys + dsx_sort_pairs + dsx_tile_ranges (i.e. as calculate_keys_and_indices_kernel,
 * thrust::sort_by_key and identify_tile_ranges, cpp/rasterizer_torch.cu:70-104) without sorting K
 * 64-bit keys; with larger bins the same per-tile ranges and the lists per bin (see dsx_list_bin),
 * which dsx_blend_fwd / dsx_blend_bwd walk when they are given the same cam->list_bin.  The
 * order (tile, depth bits, Gaussian index) is produced by (1) a stable sort of the n Gaussians by
 * their 32 depth bits, (2) emission of (tile slot, Gaussian) pairs in that order, (3) a stable
 * partition of the k pairs by tile slot.
 *
 * dsx_sort_pairs_u32: stable ascending sort of (uint32 key, uint32 value) pairs by the low
 * key_bits bits of the key, in place (the building block of both (1) and (3)).
 * dsx_depth_order: step (1) on an `order` buffer the projection has filled; it also leaves the
 * scanned tile counts of the depth-ordered 256-Gaussian blocks, the number of pairs of every
 * tile and the digit histograms of the tile slots (from the rectangles by a 2-D prefix sum of
 * their corners: no pair is enumerated) in the buffer.  The number of pairs k of the lists that
 * dsx_tile_lists will build is the last entry of the block offsets (dsx_order_view).
 * dsx_order_view: device pointers into the buffer (depth order uint32[n], block offsets
 * uint32[dsx_num_blocks(n)+1] whose last entry is K), for inspection.
 * dsx_tile_lists: steps (2) and (3) and the ranges: sorted_ids[k], ranges[dsx_ranges_count(W, H,
 * cam->list_bin)] (everything but the part that the blend forward writes). */
int dsx_sort_pairs_u32(int64_t count, int32_t key_bits, uint32_t* keys, uint32_t* values,
                       void* workspace, size_t workspace_bytes, void* stream);
int dsx_depth_order(const dsx_camera* cam, int64_t n, void* order, size_t order_bytes, void* stream);
int dsx_order_view(int64_t n, const void* order, const uint32_t** depth_order,
                   const uint32_t** block_offsets);
/* The chained scan of a sort pass waits for its predecessor tile with a BOUNDED spin; a tile that
 * gives up (it never should: tiles take their numbers in start order) sets a flag instead of
 * hanging the GPU, and the result of that sort is then wrong.  This returns the device
 * addresses of the two flags (uint32, non-zero = gave up) inside an `order` buffer after
 * dsx_depth_order / dsx_forward_project and inside a `workspace` after dsx_tile_lists /
 * dsx_forward_finish, for callers that want to check after synchronising.  Either output may
 * be NULL; an address is NULL when its buffer is NULL or empty.  No counterpart in the
 * reference (thrust's sort has no such wait). */
int dsx_sort_flags(int64_t n, int64_t k, int32_t width, int32_t height, int32_t list_bin,
                   const void* order, const void* workspace, const uint32_t** depth_sort_flag,
                   const uint32_t** partition_flag);
int dsx_tile_lists(const dsx_camera* cam, int64_t n, int64_t k, const void* order,
                   int32_t* sorted_ids, int32_t* ranges, void* workspace, size_t workspace_bytes,
                   void* stream);

/* Stage 4 — replaces rasterizer_cuda_forward + render_image_kernel,
 * cpp/rasterizer_torch.cu:44-68, cpp/rasterizer_kernels.cu:341-431.
 * image[H*W*3] (HWC, background not composited), final_T[H*W], final_idx[H*W].
 * ranges / sorted_ids[k]: what dsx_tile_lists wrote for the same cam->list_bin (the kernel adds the
 * part of `ranges` that the backward reads when the lists are per bin); with cam->list_bin = 1 (or 0
 * on an image below 2048 tiles) ranges may also be the num_tiles + 1 words of dsx_tile_ranges and
 * sorted_ids the values of dsx_sort_pairs.  n: Gaussians behind `splats`.  An id of the lists is
 * taken only up to n - 1 and a list position only inside [0, k): lists in disorder give a wrong
 * image, not a fetch outside the arrays; a `ranges` buffer whose header names another bin size
 * than this call's gives a NaN image. */
int dsx_blend_fwd(const dsx_camera* cam, int64_t n, int64_t k, int32_t* ranges, const int32_t* sorted_ids,
                  const float* splats, float* image, float* final_T, int32_t* final_idx, void* stream);

/* Stage 5a — replaces rasterize_backward_tensor + rasterize_backward_kernel,
 * cpp/gsplat/bindings.cu:140-194, cpp/gsplat/backward.cu:25-202.  grads[n*12] is zeroed by
 * the call and then accumulated with float atomics.  v_image[H*W*3].  ranges, sorted_ids, n, k: as
 * for dsx_blend_fwd, after it has run on them. */
int dsx_blend_bwd(const dsx_camera* cam, int64_t n, int64_t k, const int32_t* ranges,
                  const int32_t* sorted_ids, const float* splats, const float* final_T,
                  const int32_t* final_idx, const float* v_image, float* grads, void* stream);

/* Stage 5b+5c — replaces compute_sh_backward_tensor/kernel (cpp/gsplat/bindings.cu:22-51,
 * cpp/gsplat/sh.cuh:95-203), project_gaussians_backward_tensor/kernel
 * (cpp/gsplat/bindings.cu:61-131, cpp/gsplat/backward.cu:216-393) and the ATen glue of
 * rasterizer_backward_deepsense, cpp/rasterizer_torch.cu:291-313.
 * Outputs: v_mean3d[n*3], v_means2d[n*3] (xy gradient in pixels, z = 0), v_shs[n*num_bases*3]
 * (may be NULL), v_colors[n*3], v_opacity[n], v_scale[n*3], v_quat[n*4], v_cov3d[n*6].
 * Any output may be NULL: that gradient is then not written (the reference computes all of them
 * and lets autograd drop those of inputs that were not given, cpp/rasterizer_torch.cu:315;
 * here an unwanted one costs no store).  v_quat must be 16-byte aligned and v_cov3d 8-byte aligned;
 * the others need only the alignment of a float.
 * Every output is linear in the nine sums of the Gaussian's accumulator record, so the call first
 * clears the outputs with a fill and then works on the Gaussians that have a non-zero sum only
 * (a NaN counts as one); a Gaussian without one gets +0 everywhere, where the reference would
 * compute a signed zero, or NaN for a non-finite input of that Gaussian.
 * scales/quats may be NULL when the forward used cov3d_precomp (v_scale, v_quat zeroed).
 * cov3d is what the forward stored, or cov3d_precomp itself, or NULL when scales/quats are
 * given: the kernel then rebuilds it with the forward's own routine (bit-identical). */
int dsx_gaussian_bwd(const dsx_camera* cam, int64_t n, int32_t num_bases, const float* means3d,
                     const float* scales, const float* quats, const float* splats,
                     const float* cov3d, const int32_t* radii, const float* grads, float* v_mean3d,
                     float* v_means2d, float* v_shs, float* v_colors, float* v_opacity,
                     float* v_scale, float* v_quat, float* v_cov3d, void* stream);

/* ------------------------------------------------------------------------------------ */
/* Whole forward / backward — what the PyTorch extension calls                           */
/* ------------------------------------------------------------------------------------ */

/* First half of rasterizer_forward_deepsense (cpp/rasterizer_torch.cu:170-208): projection,
 * the read-back of K (the one host wait of the forward, in place of the reference's block scan
 * and two device drains at cpp/rasterizer_torch.cu:95-104; K is summed from the tile rectangles
 * by the first kernel that runs beside the depth sort) and, overlapping that read-back, the depth
 * order.  block_sums[dsx_num_blocks(n)] receives the tile count of each 256-Gaussian block
 * (not scanned).  order: device buffer of dsx_order_bytes(n, W, H, cam->list_bin).  num_keys (host,
 * TWO entries; pinned memory lets the copy overlap): [0] receives k, the number of pairs of the lists
 * that dsx_forward_finish will build (entries of sorted_ids); [1] the number of pairs of the per-tile
 * lists, the reference's K (equal to [0] when the lists are per tile), which the per-tile ranges and
 * final_idx index.  DSX_ERR_TOO_LARGE when [0] >= 2^30 or [1] >= 2^31. */
int dsx_forward_project(const dsx_camera* cam, int64_t n, const float* means3d,
                        const float* scales, const float* quats, const float* opacities,
                        const float* shs, const float* cov3d_precomp, const float* colors_precomp,
                        float* splats, int32_t* radii, float* cov3d, uint32_t* block_sums,
                        void* order, size_t order_bytes, int64_t* num_keys /* host */,
                        void* stream);

/* Second half: tile lists (dsx_tile_lists) and blend.  sorted_ids[k] and ranges[T+1] are
 * outputs that backward needs; workspace as dsx_workspace_bytes(n, k, W, H).  If one of the two
 * sorts gave up a bounded wait (see dsx_sort_flags) the image is written as NaN: a failure
 * shows without a read-back of the flags.
 * The blend kernels take an id from the lists only up to n - 1 (larger or negative ones read as
 * n - 1) and a list position only inside [0, k): lists in disorder give a wrong image or gradient,
 * not a fetch outside the splat records or sorted_ids.
 * grads_to_prepare (may be NULL; 16-byte aligned, dsx_grads_bytes(n) bytes): the accumulator that
 * a dsx_backward of this forward will use.  The blend kernel, which leaves the memory system idle,
 * prepares it on the side (the nine sums zeroed, each Gaussian's conic in the three spare places,
 * the byte per Gaussian behind the records cleared), and that
 * dsx_backward is then called with grads_prepared = 1: it needs no fill of its own and its
 * per-Gaussian kernel does not fetch the splat records for the conic. */
int dsx_forward_finish(const dsx_camera* cam, int64_t n, int64_t k, const float* splats,
                       const void* order, int32_t* sorted_ids, int32_t* ranges, float* image,
                       float* final_T, int32_t* final_idx, void* workspace,
                       size_t workspace_bytes, float* grads_to_prepare, void* stream);

/* rasterizer_backward_deepsense, cpp/rasterizer_torch.cu:263-316.  k: entries of sorted_ids (the k
 * of the forward); ranges: the buffer that dsx_forward_finish filled, for the same cam->list_bin (a
 * buffer whose header names another bin size is not walked: the gradients are then zero).  grads is scratch of
 * dsx_grads_bytes(n) bytes, 16-byte aligned; grads_prepared != 0 says that dsx_forward_finish has
 * prepared it (true for one call: this one leaves sums in it).  The outputs are as for
 * dsx_gaussian_bwd: zero wherever the blend backward added no term to a Gaussian's record (most
 * of a dense scene), written by the blend kernel's wavefronts on their way out; the per-Gaussian
 * kernel then works on the marked Gaussians only. */
int dsx_backward(const dsx_camera* cam, int64_t n, int64_t k, int32_t num_bases, const float* means3d,
                 const float* scales, const float* quats, const float* splats, const float* cov3d,
                 const int32_t* radii, const int32_t* ranges, const int32_t* sorted_ids,
                 const float* final_T, const int32_t* final_idx, const float* v_image,
                 float* grads, int32_t grads_prepared, float* v_mean3d, float* v_means2d,
                 float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                 float* v_cov3d, void* stream);

/* dsx_backward for callers that cannot allocate or bring device scratch: code under HIP graph
 * capture, tight serving or training loops, harnesses that forbid hipMalloc.  No counterpart in
 * the reference (its backward allocates every temporary through torch).  The same computation and
 * the same arguments as dsx_backward, except that the gradient accumulator is not an
 * argument: it is a device array built into the library, dsx_grads_bytes(DSX_STATIC_MAX_GAUSSIANS) =
 * 24.5 MiB, which every GPU the library runs on holds until the process ends.  The call allocates
 * and frees nothing, on the device or through any library; it returns DSX_ERR_STATIC_LIMIT for
 * n > DSX_STATIC_MAX_GAUSSIANS.  The array keeps the previous call's sums; each call clears the
 * n records it uses with a fill kernel (plain stores) before accumulating.  All calls on one GPU
 * share the one array: calls that overlap on a GPU (two streams, two host threads) race — keep
 * them on one stream or serialise them.  The array's device address is looked up on the first
 * call on each device: make that first call outside a graph capture. */
int dsx_backward_static(const dsx_camera* cam, int64_t n, int64_t k, int32_t num_bases,
                        const float* means3d, const float* scales, const float* quats, const float* splats,
                        const float* cov3d, const int32_t* radii, const int32_t* ranges,
                        const int32_t* sorted_ids, const float* final_T, const int32_t* final_idx,
                        const float* v_image, float* v_mean3d, float* v_means2d, float* v_shs,
                        float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                        float* v_cov3d, void* stream);

/* Raw-pointer forward-only render, the role of rasterizer_forward_core_deepsense
 * (cpp/ds_cuda_rasterizer/rasterizer_cuda.hpp:4-9, cpp/rasterizer_cuda.cu:128-158) without
 * its truncation of the sort to the first n keys.  Unlike every other entry point this one
 * allocates its temporaries itself (hipMallocAsync on `stream`) as the reference's does with
 * thrust::device_vector.  All pointers are device pointers. */
int dsx_forward_core(const float* means3d, const float* shs, const float* opacities,
                     const float* scales, const float* quats, int64_t n, const float* view,
                     const float* proj, const float* campos, int32_t image_width,
                     int32_t image_height, float tanfovx, float tanfovy, float scale_modifier,
                     int32_t max_sh_degree, int32_t sh_degree, float* image, void* stream);

/* ------------------------------------------------------------------------------------ */
/* Diagnostics: per-kernel timing with events on the launch stream.  No counterpart in the  */
/* reference (its test harness times whole calls on the host, tests/rasterizer_test.cpp:    */
/* 112-143).  While enabled, every kernel launch of the library records a start/stop event  */
/* pair; dsx_trace_read waits for them, returns up to max_entries (name, ms) records in     */
/* launch order and clears the trace (process-wide, like the rest of the list at the top).  */
/* ------------------------------------------------------------------------------------ */
typedef struct dsx_trace_entry
{
    char name[48];
    float milliseconds;
} dsx_trace_entry;

int dsx_trace_enable(int on);
int dsx_trace_read(dsx_trace_entry* out /* host */, int max_entries);

/* The two blend kernels exist in two forms: one wavefront per tile with four pixels per lane
 * (images with enough tiles to fill the chip) and four wavefronts per tile with one pixel per
 * lane.  The library picks by tile count; this forces one form for the whole process (pixels =
 * 1 or 4) or returns the choice to the library (0).  Results of the forward are bit-identical in
 * both forms.  For tests, which run both forms at every size.  No counterpart in the reference. */
int dsx_set_blend_pixels_per_lane(int pixels);

#ifdef __cplusplus
}
#endif
#endif
