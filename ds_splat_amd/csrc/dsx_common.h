// Internal declarations shared by the HIP translation units of libdsx (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dsx.h"

#define DSX_WAVE 64
#define DSX_LAUNCH_CHECK()                                                                         \
    do                                                                                             \
    {                                                                                              \
        if(hipGetLastError() != hipSuccess)                                                        \
            return DSX_ERR_LAUNCH;                                                                 \
    } while(0)

namespace dsx
{

constexpr int kTile = DSX_TILE;
constexpr int kTilePixels = DSX_TILE * DSX_TILE;
constexpr int kProjBlock = DSX_PROJ_BLOCK;

// Radix sort geometry: digits of up to 9 bits (512 bins), kSortThreads x kSortItems keys per tile.
constexpr int kRadixBitsMax = 9;
constexpr int kRadix = 1 << kRadixBitsMax;
#ifndef DSX_SORT_THREADS
#define DSX_SORT_THREADS 768
#endif
#ifndef DSX_SORT_ITEMS
#define DSX_SORT_ITEMS 8
#endif
constexpr int kSortThreads = DSX_SORT_THREADS;
constexpr int kSortItems = DSX_SORT_ITEMS;
constexpr int kSortTile = kSortThreads * kSortItems;
constexpr int kMaxPasses = 8;

inline int tiles_x(int w)
{
    return (w + kTile - 1) / kTile;
}
inline int tiles_y(int h)
{
    return (h + kTile - 1) / kTile;
}

// Bits of the sortable image of a key: 32 depth bits + enough for tile ids 0..num_tiles
// (tile + 1; slot 0 holds the negative keys).
inline int sort_key_bits(int num_tiles)
{
    int b = 0;
    while((1ll << b) < (long long)num_tiles + 1)
        ++b;
    return 32 + b;
}

// Digit plan: the fewest passes with digits of at most 9 bits, bits spread evenly.
struct SortPlan
{
    int passes;
    int shift[kMaxPasses];
    int bits[kMaxPasses];
};
inline SortPlan sort_plan(int num_tiles)
{
    SortPlan pl;
    const int total = sort_key_bits(num_tiles);
    pl.passes = (total + kRadixBitsMax - 1) / kRadixBitsMax;
    const int base = total / pl.passes, rem = total % pl.passes;
    int shift = 0;
    for(int p = 0; p < kMaxPasses; ++p)
    {
        pl.shift[p] = shift;
        pl.bits[p] = p < pl.passes ? base + (p < rem ? 1 : 0) : 0;
        shift += pl.bits[p];
    }
    return pl;
}
inline int sort_passes(int num_tiles)
{
    return sort_plan(num_tiles).passes;
}

// Workspace layout of the sort for k keys (all offsets 256-byte aligned).
struct SortWorkspace
{
    size_t keys_alt;    // int64[k]
    size_t values_alt;  // int32[k]
    size_t global_hist; // uint32[passes * 256]
    size_t status;      // uint32[passes * tiles * 256]
    size_t counters;    // uint32[passes + 1]: dynamic tile ids per pass, [passes] = error flag
    size_t bytes;
    int passes;
    int64_t tiles;
};
SortWorkspace sort_workspace(int64_t k, int num_tiles);

// ---- 32-bit radix sort (depth order of the Gaussians, tile partition of the tile lists) ----
constexpr int kBits32 = 8;
constexpr int kBins32 = 1 << kBits32;
// One pass kernel, workgroups of 1024 threads, and a family of tile sizes: 1, 2, 3, 4, 6, 8 or 12 keys
// per thread.  A pass is a chained scan over its tiles, all resident at once, and takes about as long as
// one tile's own serial work (every thread ranks its keys one after the other) plus the chain: the
// fastest tile size is the smallest that still leaves at most one tile per compute unit (measured at
// 16 K to 3 M keys: 1 M keys take 0.094 ms in 8192-key tiles of 512 threads, 0.075 in 4096-key ones of
// 1024, 0.125 in 1024-key ones; 16 K keys 0.074 against 0.034).  Beyond 12 keys per thread registers
// run out, so larger inputs get more tiles than compute units.  A tile must stay below 65536 keys
// (positions inside a tile are kept as 16 bits).
constexpr int kSortThreads32 = 1024;
constexpr int kSortItemsMax32 = 12;
constexpr int kSortTilesWanted32 = 256; // compute units of an MI355X
inline int sort32_items(int64_t count)
{
    const int64_t want = (count + (int64_t)kSortThreads32 * kSortTilesWanted32 - 1) / ((int64_t)kSortThreads32 * kSortTilesWanted32);
    const int family[] = {1, 2, 3, 4, 6, 8, kSortItemsMax32};
    for(int items : family)
        if(items >= want)
            return items;
    return kSortItemsMax32;
}
constexpr int kMaxPasses32 = 4;
inline int sort32_tile_keys(int64_t count)
{
    return kSortThreads32 * sort32_items(count);
}
// depth key of a Gaussian that emits no (tile, Gaussian) pair; as a float it is a NaN, which no
// emitting Gaussian has (a NaN depth fails the frustum test)
constexpr uint32_t kNoPairsKey = 0xffffffffu;

// Digits of a key whose low `key_bits` bits are significant: fewest passes with digits of at
// most 8 bits, bits spread evenly.
struct Digits32
{
    int passes;
    int shift[kMaxPasses32];
    uint32_t mask[kMaxPasses32];
};
inline Digits32 digits32(int key_bits)
{
    Digits32 d;
    if(key_bits < 1)
        key_bits = 1;
    if(key_bits > 32)
        key_bits = 32;
    d.passes = (key_bits + kBits32 - 1) / kBits32;
    const int base = key_bits / d.passes, rem = key_bits % d.passes;
    int shift = 0;
    for(int p = 0; p < kMaxPasses32; ++p)
    {
        const int bits = p < d.passes ? base + (p < rem ? 1 : 0) : 0;
        d.shift[p] = shift;
        d.mask[p] = bits ? (1u << bits) - 1u : 0u;
        shift += bits;
    }
    return d;
}
// bits needed for tile slots 0..num_tiles (slot 0 = keys with a negative depth, slot t+1 = tile t)
inline int slot_bits(int num_tiles)
{
    int b = 1;
    while((1ll << b) < (long long)num_tiles + 1)
        ++b;
    return b;
}

// The tile lists are built per BIN of (1 << shift) x (1 << shift) tiles: a Gaussian enters the list
// of every bin that its tile rectangle touches, once, and a blend tile walks its bin's list and
// keeps the entries whose rectangle contains the tile itself.  shift = 0: one list per tile, the
// reference's own lists.  Larger bins mean fewer pairs to emit and to partition (a Gaussian that
// covers 11 tiles touches 2 or 3 bins of 4 x 4) and longer lists to filter in the blend.
struct ListGrid
{
    int shift;    // log2 of the bin's side in tiles
    int ntx, nty; // tiles of the image
    int nbx, nby; // bins of the image
    int tiles() const { return ntx * nty; }
    int bins() const { return nbx * nby; }
    // what the partition sorts by: bins when the lists are binned, tiles when they are not
    int lists() const { return shift ? bins() : tiles(); }
};
// list_bin: 0: choose by image size; 1, 2, 4, 8: bins of that many tiles a side (dsx_camera::list_bin)
ListGrid list_grid(int image_width, int image_height, int list_bin);
inline ListGrid list_grid(const dsx_camera& cam)
{
    return list_grid(cam.image_width, cam.image_height, cam.list_bin);
}
inline bool valid_list_bin(int b)
{
    return b == 0 || b == 1 || b == 2 || b == 4 || b == 8;
}

// Layout of the `ranges` buffer of the forward (int32 words):
//   fine[tiles + 1]   ranges of the per-tile lists as the reference defines them (the index of a
//                     tile's first pair in the fully sorted key array; the last word is the
//                     number of pairs)
//   shift[1]          log2 of the bin side that the lists were built for (0: one list per tile): the
//                     blend kernels compare it with the bin size they are launched for and walk
//                     nothing when the two differ
// and, when the lists are binned,
//   last_tile[1]      highest tile that holds a pair of non-negative depth, -1 if none
//   bins[bins + 1]    ranges of the bin lists inside sorted_ids
//   walk[tiles * 8]   written by the blend forward for the backward: per tile and band of four
//                     rows, the position in the bin's list where the forward's scan stopped and
//                     the number of the tile's own entries it had met by then
struct RangesLayout
{
    int fine, header, last_tile, bins, walk, count;
    int ready; // words that exist before the blend forward runs (everything but `walk`)
};
inline RangesLayout ranges_layout(const ListGrid& g)
{
    RangesLayout r;
    r.fine = 0;
    r.header = g.tiles() + 1;
    r.last_tile = r.header + 1;
    r.bins = r.last_tile + 1;
    r.walk = r.bins + g.bins() + 1;
    r.count = g.shift ? r.walk + g.tiles() * 8 : r.header + 1;
    r.ready = g.shift ? r.walk : r.count;
    return r;
}

// Workspace of one 32-bit sort of `count` pairs (offsets relative to its base, 256-byte aligned).
struct Sort32Workspace
{
    size_t hist;     // uint32[passes * 256]
    size_t counters; // uint32[passes + 1]: dynamic tile ids per pass, [passes] = error flag
    size_t status;   // uint32[passes * tiles * 256]
    size_t bytes;
    int passes;
    int64_t tiles;
};
Sort32Workspace sort32_workspace(int64_t count, int key_bits, int tile_keys);

// Per-Gaussian buffer that carries the depth order from the projection to the tile lists.
struct OrderLayout
{
    size_t depth_keys; // uint32[n]  depth bits (written by the projection)
    size_t keys_alt;   // uint32[n]
    size_t ids_a;      // uint32[n]  the depth order ends here
    size_t ids_b;      // uint32[n]
    size_t rects;      // uint2[n]   packed tile rectangle (written by the projection)
    size_t rects_sorted; // uint2[n] the same in depth order
    size_t rects32;    // uint32[n]  packed rectangles on their way through the depth sort
    size_t block_sums; // uint32[blocks + 1] tile counts of 256 consecutive Gaussians IN DEPTH ORDER, scanned
    size_t slot_hist;  // uint32[kMaxPasses32 * 256] digit histograms of the tile slots of all pairs
    size_t cover;      // int32[(ntx + 1) * (nty + 1) + 1] pairs per tile (corner grid, then its 2-D prefix sum)
    size_t bin_cover;  // int32[(nbx + 1) * (nby + 1) + 1] the same per bin (binned lists only)
    size_t key_count;  // uint64[2]  pairs of the per-tile lists, pairs of the bin lists (summed by the corner-grid kernel)
    size_t ranges;     // int32[...] ranges_layout() without its `walk` part, ready before the pairs exist
    size_t sort;       // Sort32Workspace
    size_t bytes;
};
// the grid is the last member, so every other offset depends on n alone
OrderLayout order_layout(int64_t n, int image_width = 0, int image_height = 0, int list_bin = 0);

// Workspace of the tile lists for k keys.
struct ListsWorkspace
{
    size_t slots_a; // uint16 / uint32[k]
    size_t slots_b; // the same (per-tile lists only)
    size_t ids_alt; // int32[k]
    size_t sort;    // Sort32Workspace
    size_t bytes;
    int passes;
};
// binned: lists per bin (32-bit slot words that carry the tile masks and end in the caller's buffer)
ListsWorkspace lists_workspace(int64_t k, int num_tiles, bool binned);

// launchers (each returns a dsx_status)
int launch_sort32(int64_t count, int key_bits, uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b,
                  uint32_t* vals_b, bool iota_values, bool keep_keys, void* sort_ws, hipStream_t stream,
                  uint32_t** keys_out, uint32_t** vals_out, const uint2* gather_src = nullptr,
                  uint2* gather_dst = nullptr, bool already_cleared = false, uint32_t* carry_a = nullptr,
                  uint32_t* carry_b = nullptr);
// already_cleared: the words of depth_order_clear_region are zero already (the projection did it)
int launch_depth_order(const dsx_camera& cam, int64_t n, void* order, hipStream_t stream,
                       bool already_cleared = false, void* k_host = nullptr, hipEvent_t k_copied = nullptr);
// the part of an `order` buffer that must be zero when launch_depth_order starts
void depth_order_clear_region(const dsx_camera& cam, int64_t n, void* order, uint32_t** words, int64_t* count);
int launch_tile_lists(const dsx_camera& cam, int64_t n, int64_t k, const void* order, int32_t* sorted_ids,
                      int32_t* ranges, void* workspace, hipStream_t stream);
int launch_project_fwd(const dsx_camera& cam, int64_t n, const float* means3d, const float* scales,
                       const float* quats, const float* opacities, const float* shs,
                       const float* cov3d_precomp, const float* colors_precomp, float* splats,
                       int32_t* radii, float* cov3d, uint32_t* block_sums, uint32_t* depth_keys,
                       uint2* rects, hipStream_t stream, uint32_t* clear = nullptr, int64_t clear_words = 0);
int launch_scan_u32(int64_t count, uint32_t* data, uint32_t* total, hipStream_t stream);
int launch_emit_keys(const dsx_camera& cam, int64_t n, int64_t k, const float* splats,
                     const uint32_t* block_offsets, int64_t* keys, int32_t* values,
                     hipStream_t stream);
// Sorts (keys_a, values_a); the result lands in (keys_a, values_a) when `passes` is even and
// in the workspace's alternate buffers when odd, unless want_in_place (then it is copied).
int launch_sort_pairs(int64_t k, int num_tiles, int64_t* keys_a, int32_t* values_a, int64_t* keys_b,
                      int32_t* values_b, void* sort_ws, hipStream_t stream, int64_t** keys_out,
                      int32_t** values_out);
int launch_tile_ranges(int64_t k, const int64_t* sorted_keys, int num_tiles, int32_t* ranges,
                       hipStream_t stream);
// sort_flag_*: error words of the sorts that built the lists (null: none); the image becomes NaN if one is set
// The accumulator of the whole backward (dsx_backward and what prepares it): n records of
// DSX_GRAD_FLOATS floats, then one byte per Gaussian that the blend backward sets when it adds a
// term to the record (the per-Gaussian kernel then reads 1 byte instead of 48 to learn that a
// Gaussian has nothing to propagate), padded to 16 bytes.
constexpr size_t grads_bytes(int64_t n)
{
    return (size_t)n * DSX_GRAD_FLOATS * 4 + (((size_t)n + 15) & ~(size_t)15);
}
inline uint8_t* grad_marks(float* grads, int64_t n)
{
    return reinterpret_cast<uint8_t*>(grads + n * DSX_GRAD_FLOATS);
}
// The zeros of the per-Gaussian backward's outputs: up to eight arrays.  Their 16-byte-aligned middles
// form one range of 16-byte stores that the parts of a launch share evenly (v_shs alone is three
// quarters of it); the few floats in front of and behind a middle are stored one by one.
struct ZeroJobs
{
    float* ptr[8];     // null: not wanted
    int64_t floats[8]; // length of the array
    int64_t end[8];    // 16-byte stores of this and all earlier arrays
    int any;           // is there anything to store?
};
inline ZeroJobs make_zero_jobs(int64_t n, int num_bases, float* v_mean3d, float* v_means2d, float* v_shs,
                               float* v_colors, float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d)
{
    ZeroJobs jobs;
    float* ptrs[8] = {v_mean3d, v_means2d, num_bases > 0 ? v_shs : nullptr, v_colors, v_opacity, v_scale, v_quat, v_cov3d};
    const int64_t per[8] = {3, 3, 3 * (int64_t)num_bases, 3, 1, 3, 4, 6};
    int64_t stores = 0;
    jobs.any = 0;
    for(int j = 0; j < 8; ++j)
    {
        jobs.ptr[j] = n > 0 ? ptrs[j] : nullptr;
        jobs.floats[j] = jobs.ptr[j] ? n * per[j] : 0;
        if(jobs.ptr[j])
        {
            jobs.any = 1;
            const int64_t head = (int64_t)(((16 - ((uintptr_t)ptrs[j] & 15)) & 15) / 4);
            stores += jobs.floats[j] > head ? (jobs.floats[j] - head) / 4 : 0;
        }
        jobs.end[j] = stores;
    }
    return jobs;
}

int launch_blend_fwd(const dsx_camera& cam, int64_t n, int64_t k, int32_t* ranges, const int32_t* sorted_ids,
                     const float* splats, float* image, float* final_T, int32_t* final_idx, hipStream_t stream,
                     bool check_header, const uint32_t* sort_flag_a = nullptr, const uint32_t* sort_flag_b = nullptr,
                     float* prepare_grads = nullptr, bool prepare_marks = false);
int launch_blend_bwd(const dsx_camera& cam, int64_t n, int64_t k, const int32_t* ranges, const int32_t* sorted_ids,
                     const float* splats, const float* final_T, const int32_t* final_idx, const float* v_image,
                     float* grads, hipStream_t stream, bool check_header, bool grads_prepared = false,
                     bool with_marks = false, const ZeroJobs* zeros = nullptr);
int launch_gaussian_bwd(const dsx_camera& cam, int64_t n, int num_bases, const float* means3d,
                        const float* scales, const float* quats, const float* splats,
                        const float* cov3d, const int32_t* radii, const float* grads,
                        float* v_mean3d, float* v_means2d, float* v_shs, float* v_colors,
                        float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d,
                        hipStream_t stream, bool conic_in_grads = false, bool outputs_cleared = false,
                        bool with_marks = false);
// zeros in every output of launch_gaussian_bwd that is not null (it writes only the Gaussians that
// have something to propagate; outputs_cleared tells it that this has been done)
int launch_zero_outputs(const ZeroJobs& jobs, hipStream_t stream);
int launch_fill_u32(uint32_t* p, int64_t count, uint32_t value, hipStream_t stream);
// 1 or 4: force that form of both blend kernels for the whole process; 0: choose by image size
int set_blend_pixels_per_lane(int pixels);

// Optional per-kernel timing (diagnostics for benchmarks): when switched on through
// dsx_trace_enable(), every launch is bracketed by two events on the launch stream.
struct KernelTimer
{
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
    int slot;
    hipStream_t stream;
    hipEvent_t stop;
};
#define DSX_TIMED(name, stream) dsx::KernelTimer dsx_timer_##__LINE__(name, stream)

#ifdef __HIPCC__
// ---- device helpers -------------------------------------------------------------------
__device__ __forceinline__ int lane_id()
{
    return __lane_id();
}

// Sum of the first `wave` entries of a 16-byte aligned LDS array of kWaves per-wavefront totals
// (kWaves a multiple of four): 16-byte reads and selects on the wavefront's index.  A loop
// `for(w = 0; w < wave; ++w)` compiles to dependent 4-byte reads under an exec mask.
template <int kWaves>
__device__ __forceinline__ uint32_t sum_of_waves_before(const uint32_t* totals, int wave)
{
    static_assert(kWaves % 4 == 0, "whole 16-byte words");
    uint32_t s = 0;
#pragma unroll
    for(int q = 0; q < kWaves / 4; ++q)
    {
        const uint4 v = reinterpret_cast<const uint4*>(totals)[q];
        s += (4 * q < wave ? v.x : 0u) + (4 * q + 1 < wave ? v.y : 0u) + (4 * q + 2 < wave ? v.z : 0u) +
             (4 * q + 3 < wave ? v.w : 0u);
    }
    return s;
}

// cov3D = (R S)(R S)^T from scale and (w,x,y,z) quaternion; cpp/rasterizer_kernels.cu:615-659
__device__ __forceinline__ void cov3d_from_scale_rot(const float* sc, float4 q, float mod, float* out)
{
#pragma clang fp contract(off) // same bits in every translation unit (radii and tile counts derive from them)
    float r = q.x, x = q.y, y = q.z, z = q.w;
    const float inv_norm = 1.0f / sqrtf(r * r + x * x + y * y + z * z);
    r = r * inv_norm;
    x = x * inv_norm;
    y = y * inv_norm;
    z = z * inv_norm;
    const float s0 = sc[0] * mod, s1 = sc[1] * mod, s2 = sc[2] * mod;
    const float r00 = 1.0f - 2.0f * (y * y + z * z);
    const float r01 = 2.0f * (x * y - r * z);
    const float r02 = 2.0f * (x * z + r * y);
    const float r10 = 2.0f * (x * y + r * z);
    const float r11 = 1.0f - 2.0f * (x * x + z * z);
    const float r12 = 2.0f * (y * z - r * x);
    const float r20 = 2.0f * (x * z - r * y);
    const float r21 = 2.0f * (y * z + r * x);
    const float r22 = 1.0f - 2.0f * (x * x + y * y);
    const float m00 = s0 * r00, m01 = s1 * r01, m02 = s2 * r02;
    const float m10 = s0 * r10, m11 = s1 * r11, m12 = s2 * r12;
    const float m20 = s0 * r20, m21 = s1 * r21, m22 = s2 * r22;
    out[0] = m00 * m00 + m01 * m01 + m02 * m02;
    out[1] = m00 * m10 + m01 * m11 + m02 * m12;
    out[2] = m00 * m20 + m01 * m21 + m02 * m22;
    out[3] = m10 * m10 + m11 * m11 + m12 * m12;
    out[4] = m10 * m20 + m11 * m21 + m12 * m22;
    out[5] = m20 * m20 + m21 * m21 + m22 * m22;
}

// float -> int32 with the hardware conversion's semantics made explicit (saturate, NaN -> 0).
__device__ __forceinline__ int f2i_sat(float x)
{
    if(x != x)
        return 0;
    if(x >= 2147483648.0f)
        return 0x7fffffff;
    if(x <= -2147483648.0f)
        return (int)0x80000000;
    return (int)x;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, DSX_WAVE);
    return v;
}

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves only: four shifts
// inside each row of 16 (lanes without a source add 0), then the row totals are broadcast into
// the rows behind them.  (A shuffle goes through the LDS crossbar and takes a round trip per step.)
template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_add_u32(uint32_t v)
{
    return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, 0xf, false);
}

__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t v)
{
    v = dpp_add_u32<0x111, 0xf>(v); // row_shr:1
    v = dpp_add_u32<0x112, 0xf>(v); // row_shr:2
    v = dpp_add_u32<0x114, 0xf>(v); // row_shr:4
    v = dpp_add_u32<0x118, 0xf>(v); // row_shr:8
    v = dpp_add_u32<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v = dpp_add_u32<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

typedef float dsx_v4f __attribute__((ext_vector_type(4)));

// streaming (non-temporal) 16-byte load / store: data that is touched once
__device__ __forceinline__ float4 nt_load_f4(const float4* p)
{
    const dsx_v4f v = __builtin_nontemporal_load(reinterpret_cast<const dsx_v4f*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void nt_store_f4(float4* p, float4 v)
{
    dsx_v4f t;
    t.x = v.x;
    t.y = v.y;
    t.z = v.z;
    t.w = v.w;
    __builtin_nontemporal_store(t, reinterpret_cast<dsx_v4f*>(p));
}

// the 16-byte stores [lo, hi) of the arrays' middles, by `threads` threads (this one: tid)
__device__ __forceinline__ void zero_range(const ZeroJobs& jobs, int64_t lo, int64_t hi, int tid, int threads)
{
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for(int j = 0; j < 8; ++j)
    {
        float* ptr = jobs.ptr[j];
        if(ptr == nullptr)
            continue;
        const int64_t start = j ? jobs.end[j - 1] : 0;
        const int head = (int)(((16 - ((uintptr_t)ptr & 15)) & 15) / 4);
        float4* q = reinterpret_cast<float4*>(ptr + head) - start;
        for(int64_t i = max(lo, start) + tid; i < min(hi, jobs.end[j]); i += threads)
            nt_store_f4(q + i, zero);
    }
}
// the floats in front of and behind the middles (threads 0..3 of one part of the launch)
__device__ __forceinline__ void zero_edges(const ZeroJobs& jobs, int tid)
{
    if(tid >= 4)
        return;
#pragma unroll
    for(int j = 0; j < 8; ++j)
    {
        float* ptr = jobs.ptr[j];
        if(ptr == nullptr)
            continue;
        const int64_t start = j ? jobs.end[j - 1] : 0;
        const int head = (int)(((16 - ((uintptr_t)ptr & 15)) & 15) / 4);
        const int64_t n = jobs.floats[j];
        if(tid < head && (int64_t)tid < n)
            ptr[tid] = 0.f;
        const int64_t t = head + (jobs.end[j] - start) * 4 + tid;
        if(t < n)
            ptr[t] = 0.f;
    }
}
// part `part` of `parts` stores its share of the zeros
__device__ __forceinline__ void zero_share(const ZeroJobs& jobs, int64_t part, int64_t parts, int tid, int threads)
{
    const int64_t total = jobs.end[7];
    const int64_t share = (total + parts - 1) / parts;
    zero_range(jobs, part * share, min((part + 1) * share, total), tid, threads);
    if(part == 0)
        zero_edges(jobs, tid);
}

struct TileRect
{
    int sx, ex, sy, ey;
};

// Tile rectangle of a splat: truncation toward zero, +1 on the upper bound, clamped to the
// tile grid.  Pure IEEE ops on powers of two, so it is exact on any target.
__device__ __forceinline__ TileRect tile_rect(float px, float py, int radius, int ntx, int nty)
{
    const float cx = px / 16.0f;
    const float cy = py / 16.0f;
    const float d = (float)radius / 16.0f;
    TileRect r;
    r.sx = min(max(0, f2i_sat(cx - d)), ntx);
    r.ex = min(max(0, f2i_sat((cx + d) + 1.0f)), ntx);
    r.sy = min(max(0, f2i_sat(cy - d)), nty);
    r.ey = min(max(0, f2i_sat((cy + d) + 1.0f)), nty);
    return r;
}
#endif

} // namespace dsx
