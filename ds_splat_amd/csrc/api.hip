// extern "C" surface of libdsx: argument checks, stage sequencing, the one host
// synchronisation of the forward (read-back of the key count) and error strings.
#include "dsx_common.h"

#include <mutex>
#include <string.h>
#include <vector>

using namespace dsx;

// ---- optional per-kernel timing -----------------------------------------------------------
namespace
{
struct TraceSlot
{
    const char* name;
    hipEvent_t start, stop;
};
bool g_trace_on = false;
std::mutex g_trace_mutex;
std::vector<TraceSlot> g_trace;
} // namespace

dsx::KernelTimer::KernelTimer(const char* name, hipStream_t s) : slot(-1), stream(s), stop(nullptr)
{
    if(!g_trace_on)
        return;
    TraceSlot t;
    t.name = name;
    if(hipEventCreate(&t.start) != hipSuccess)
        return;
    if(hipEventCreate(&t.stop) != hipSuccess)
    {
        (void)hipEventDestroy(t.start);
        return;
    }
    (void)hipEventRecord(t.start, s);
    std::lock_guard<std::mutex> lock(g_trace_mutex);
    slot = (int)g_trace.size();
    stop = t.stop;
    g_trace.push_back(t);
}

dsx::KernelTimer::~KernelTimer()
{
    if(slot < 0)
        return;
    std::lock_guard<std::mutex> lock(g_trace_mutex);
    // a dsx_trace_read from another thread may have emptied the list since the constructor ran
    if((size_t)slot < g_trace.size() && g_trace[slot].stop == stop)
        (void)hipEventRecord(stop, stream);
}

extern "C" int dsx_trace_enable(int on)
{
    std::lock_guard<std::mutex> lock(g_trace_mutex);
    g_trace_on = on != 0;
    return DSX_OK;
}

extern "C" int dsx_trace_read(dsx_trace_entry* out, int max_entries)
{
    std::lock_guard<std::mutex> lock(g_trace_mutex);
    int count = 0;
    for(const TraceSlot& t : g_trace)
    {
        float ms = 0.f;
        const bool ok = hipEventSynchronize(t.stop) == hipSuccess && hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess;
        if(ok && out && count < max_entries)
        {
            strncpy(out[count].name, t.name, sizeof(out[count].name) - 1);
            out[count].name[sizeof(out[count].name) - 1] = 0;
            out[count].milliseconds = ms;
            ++count;
        }
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    g_trace.clear();
    return count;
}

namespace
{

inline hipStream_t as_stream(void* s)
{
    return static_cast<hipStream_t>(s);
}

int check_camera(const dsx_camera* cam)
{
    if(cam == nullptr)
        return DSX_ERR_BAD_ARG;
    if(cam->image_width <= 0 || cam->image_height <= 0)
        return DSX_ERR_BAD_ARG;
    if(cam->view == nullptr || cam->proj == nullptr || cam->campos == nullptr || cam->bg == nullptr)
        return DSX_ERR_BAD_ARG;
    // the reference asserts 0 <= sh_degree <= 4 and max_sh_degree == 3
    // (cpp/rasterizer_torch.cu:124-129); degree 4 has no forward there, so 0..3 it is
    if(cam->sh_degree < 0 || cam->sh_degree > 3 || cam->max_sh_degree < cam->sh_degree || cam->max_sh_degree > 3)
        return DSX_ERR_BAD_ARG;
    if(!valid_list_bin(cam->list_bin))
        return DSX_ERR_BAD_ARG;
    return DSX_OK;
}

} // namespace

extern "C" const char* dsx_error_string(int status)
{
    switch(status)
    {
        case DSX_OK: return "ok";
        case DSX_ERR_BAD_ARG: return "dsx: bad argument (null pointer, negative size or unsupported SH degree)";
        case DSX_ERR_LAUNCH: return "dsx: kernel launch failed";
        case DSX_ERR_RUNTIME: return "dsx: HIP runtime call failed";
        case DSX_ERR_TOO_LARGE:
            return "dsx: too many (tile, Gaussian) pairs for 32-bit indexing (2^30 pairs of the lists that are built, "
                   "or 2^31 pairs of the per-tile lists that the ranges and final_idx index)";
        case DSX_ERR_WORKSPACE: return "dsx: workspace too small (see dsx_workspace_bytes)";
        case DSX_ERR_STATIC_LIMIT:
            return "dsx: more Gaussians than the built-in scratch of dsx_backward_static holds "
                   "(DSX_STATIC_MAX_GAUSSIANS = 524288); use dsx_backward with a caller-provided accumulator";
        default: return "dsx: unknown status";
    }
}

extern "C" int dsx_version(void)
{
    return 300;
}

extern "C" int64_t dsx_num_blocks(int64_t n)
{
    return n <= 0 ? 0 : (n + kProjBlock - 1) / kProjBlock;
}

extern "C" int32_t dsx_num_tiles(int32_t width, int32_t height)
{
    return tiles_x(width) * tiles_y(height);
}

extern "C" int32_t dsx_sort_passes(int32_t num_tiles)
{
    return sort_passes(num_tiles);
}

extern "C" size_t dsx_workspace_bytes(int64_t n, int64_t k, int32_t width, int32_t height, int32_t list_bin)
{
    (void)n;
    if(!valid_list_bin(list_bin))
        return 0;
    const ListGrid lg = list_grid(width, height, list_bin);
    return lists_workspace(k < 0 ? 0 : k, lg.lists(), lg.shift != 0).bytes;
}

extern "C" int32_t dsx_list_bin(int32_t width, int32_t height, int32_t list_bin)
{
    if(!valid_list_bin(list_bin))
        return 0;
    return 1 << list_grid(width < 0 ? 0 : width, height < 0 ? 0 : height, list_bin).shift;
}

extern "C" int64_t dsx_sorted_ids_count(int64_t k, int32_t width, int32_t height, int32_t list_bin)
{
    if(!valid_list_bin(list_bin) || k < 0)
        return 0;
    return list_grid(width < 0 ? 0 : width, height < 0 ? 0 : height, list_bin).shift ? 2 * k : k;
}

extern "C" size_t dsx_grads_bytes(int64_t n)
{
    return grads_bytes(n < 0 ? 0 : n);
}

extern "C" int64_t dsx_ranges_count(int32_t width, int32_t height, int32_t list_bin)
{
    if(!valid_list_bin(list_bin))
        return 0;
    return ranges_layout(list_grid(width < 0 ? 0 : width, height < 0 ? 0 : height, list_bin)).count;
}

extern "C" size_t dsx_sort_workspace_bytes(int64_t k, int32_t num_tiles)
{
    return sort_workspace(k < 0 ? 0 : k, num_tiles < 0 ? 0 : num_tiles).bytes;
}

extern "C" size_t dsx_order_bytes(int64_t n, int32_t width, int32_t height, int32_t list_bin)
{
    if(!valid_list_bin(list_bin))
        return 0;
    return order_layout(n < 0 ? 0 : n, width < 0 ? 0 : width, height < 0 ? 0 : height, list_bin).bytes;
}

namespace
{
// keys_alt | values_alt | Sort32Workspace
struct SortU32Layout
{
    size_t keys_alt, values_alt, sort, bytes;
};
SortU32Layout sort_u32_layout(int64_t count, int key_bits)
{
    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    SortU32Layout l;
    l.keys_alt = 0;
    l.values_alt = align((size_t)count * 4);
    l.sort = align(l.values_alt + (size_t)count * 4);
    l.bytes = l.sort + sort32_workspace(count, key_bits, sort32_tile_keys(count)).bytes;
    return l;
}
} // namespace

extern "C" size_t dsx_sort_u32_workspace_bytes(int64_t count, int32_t key_bits)
{
    return sort_u32_layout(count < 0 ? 0 : count, key_bits).bytes;
}

// clear_for_depth_order: the kernel also zeroes what launch_depth_order needs zeroed in `order`
static int project_fwd_checked(const dsx_camera* cam, int64_t n, const float* means3d, const float* scales,
                               const float* quats, const float* opacities, const float* shs,
                               const float* cov3d_precomp, const float* colors_precomp, float* splats,
                               int32_t* radii, float* cov3d, uint32_t* block_sums, void* order, size_t order_bytes,
                               void* stream, bool clear_for_depth_order)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0)
        return DSX_ERR_BAD_ARG;
    if(n == 0)
        return DSX_OK;
    if(!means3d || !opacities || !splats || !radii || !block_sums)
        return DSX_ERR_BAD_ARG; // cov3d may be null: not stored
    uint32_t* depth_keys = nullptr;
    uint2* rects = nullptr;
    if(order)
    {
        const OrderLayout o = order_layout(n, cam->image_width, cam->image_height, cam->list_bin);
        if(order_bytes < o.bytes)
            return DSX_ERR_WORKSPACE;
        depth_keys = reinterpret_cast<uint32_t*>(static_cast<char*>(order) + o.depth_keys);
        rects = reinterpret_cast<uint2*>(static_cast<char*>(order) + o.rects);
    }
    if(!cov3d_precomp && (!scales || !quats))
        return DSX_ERR_BAD_ARG;
    if(!colors_precomp && !shs)
        return DSX_ERR_BAD_ARG;
    uint32_t* clear = nullptr;
    int64_t clear_words = 0;
    if(order && clear_for_depth_order)
        depth_order_clear_region(*cam, n, order, &clear, &clear_words);
    return launch_project_fwd(*cam, n, means3d, scales, quats, opacities, shs, cov3d_precomp, colors_precomp, splats,
                              radii, cov3d, block_sums, depth_keys, rects, as_stream(stream), clear, clear_words);
}

extern "C" int dsx_project_fwd(const dsx_camera* cam, int64_t n, const float* means3d, const float* scales,
                               const float* quats, const float* opacities, const float* shs,
                               const float* cov3d_precomp, const float* colors_precomp, float* splats,
                               int32_t* radii, float* cov3d, uint32_t* block_sums, void* order, size_t order_bytes,
                               void* stream)
{
    return project_fwd_checked(cam, n, means3d, scales, quats, opacities, shs, cov3d_precomp, colors_precomp, splats,
                               radii, cov3d, block_sums, order, order_bytes, stream, false);
}

extern "C" int dsx_scan_u32(int64_t count, uint32_t* data, uint32_t* total, void* stream)
{
    if(count < 0 || !total || (count > 0 && !data))
        return DSX_ERR_BAD_ARG;
    return launch_scan_u32(count, data, total, as_stream(stream));
}

extern "C" int dsx_emit_keys(const dsx_camera* cam, int64_t n, int64_t k, const float* splats,
                             const uint32_t* block_offsets, int64_t* keys, int32_t* values, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || k < 0)
        return DSX_ERR_BAD_ARG;
    if(n == 0 || k == 0)
        return DSX_OK;
    if(!splats || !block_offsets || !keys || !values)
        return DSX_ERR_BAD_ARG;
    return launch_emit_keys(*cam, n, k, splats, block_offsets, keys, values, as_stream(stream));
}

extern "C" int dsx_sort_pairs(int64_t k, int32_t num_tiles, int64_t* keys, int32_t* values, void* workspace,
                              size_t workspace_bytes, void* stream)
{
    if(k < 0 || num_tiles < 0)
        return DSX_ERR_BAD_ARG;
    if(k <= 1)
        return DSX_OK;
    if(!keys || !values || !workspace)
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    const SortWorkspace w = sort_workspace(k, num_tiles);
    if(workspace_bytes < w.bytes)
        return DSX_ERR_WORKSPACE;
    char* base = static_cast<char*>(workspace);
    int64_t* keys_b = reinterpret_cast<int64_t*>(base + w.keys_alt);
    int32_t* values_b = reinterpret_cast<int32_t*>(base + w.values_alt);
    int64_t* ko;
    int32_t* vo;
    int rc = launch_sort_pairs(k, num_tiles, keys, values, keys_b, values_b, workspace, as_stream(stream), &ko, &vo);
    if(rc)
        return rc;
    if(ko != keys)
    {
        if(hipMemcpyAsync(keys, ko, (size_t)k * 8, hipMemcpyDeviceToDevice, as_stream(stream)) != hipSuccess ||
           hipMemcpyAsync(values, vo, (size_t)k * 4, hipMemcpyDeviceToDevice, as_stream(stream)) != hipSuccess)
            return DSX_ERR_RUNTIME;
    }
    return DSX_OK;
}

extern "C" int dsx_tile_ranges(int64_t k, const int64_t* sorted_keys, int32_t num_tiles, int32_t* ranges,
                               void* stream)
{
    if(k < 0 || num_tiles < 0 || !ranges || (k > 0 && !sorted_keys))
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    return launch_tile_ranges(k, sorted_keys, num_tiles, ranges, as_stream(stream));
}

extern "C" int dsx_sort_pairs_u32(int64_t count, int32_t key_bits, uint32_t* keys, uint32_t* values, void* workspace,
                                  size_t workspace_bytes, void* stream)
{
    if(count < 0 || key_bits < 1 || key_bits > 32)
        return DSX_ERR_BAD_ARG;
    if(count <= 1)
        return DSX_OK;
    if(!keys || !values || !workspace)
        return DSX_ERR_BAD_ARG;
    if(count >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    const SortU32Layout l = sort_u32_layout(count, key_bits);
    if(workspace_bytes < l.bytes)
        return DSX_ERR_WORKSPACE;
    char* base = static_cast<char*>(workspace);
    uint32_t *ko, *vo;
    int rc = launch_sort32(count, key_bits, keys, values, reinterpret_cast<uint32_t*>(base + l.keys_alt),
                           reinterpret_cast<uint32_t*>(base + l.values_alt), false, true, base + l.sort,
                           as_stream(stream), &ko, &vo);
    if(rc)
        return rc;
    if(ko != keys)
    {
        if(hipMemcpyAsync(keys, ko, (size_t)count * 4, hipMemcpyDeviceToDevice, as_stream(stream)) != hipSuccess ||
           hipMemcpyAsync(values, vo, (size_t)count * 4, hipMemcpyDeviceToDevice, as_stream(stream)) != hipSuccess)
            return DSX_ERR_RUNTIME;
    }
    return DSX_OK;
}

extern "C" int dsx_depth_order(const dsx_camera* cam, int64_t n, void* order, size_t order_bytes, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0)
        return DSX_ERR_BAD_ARG;
    if(n == 0)
        return DSX_OK;
    if(!order)
        return DSX_ERR_BAD_ARG;
    if(order_bytes < order_layout(n, cam->image_width, cam->image_height, cam->list_bin).bytes)
        return DSX_ERR_WORKSPACE;
    return launch_depth_order(*cam, n, order, as_stream(stream));
}

extern "C" int dsx_order_view(int64_t n, const void* order, const uint32_t** depth_order,
                              const uint32_t** block_offsets)
{
    if(n < 0 || !order)
        return DSX_ERR_BAD_ARG;
    const OrderLayout o = order_layout(n);
    if(depth_order)
        *depth_order = reinterpret_cast<const uint32_t*>(static_cast<const char*>(order) + o.ids_a);
    if(block_offsets)
        *block_offsets = reinterpret_cast<const uint32_t*>(static_cast<const char*>(order) + o.block_sums);
    return DSX_OK;
}

extern "C" int dsx_sort_flags(int64_t n, int64_t k, int32_t width, int32_t height, int32_t list_bin,
                              const void* order, const void* workspace, const uint32_t** depth_sort_flag,
                              const uint32_t** partition_flag)
{
    if(n < 0 || k < 0 || width <= 0 || height <= 0 || !valid_list_bin(list_bin))
        return DSX_ERR_BAD_ARG;
    if(depth_sort_flag)
    {
        *depth_sort_flag = nullptr;
        if(order && n > 0)
        {
            const OrderLayout o = order_layout(n);
            const Sort32Workspace w = sort32_workspace(n, 32, sort32_tile_keys(n));
            *depth_sort_flag =
                reinterpret_cast<const uint32_t*>(static_cast<const char*>(order) + o.sort + w.counters) + w.passes;
        }
    }
    if(partition_flag)
    {
        *partition_flag = nullptr;
        if(workspace && k > 0)
        {
            const ListGrid lg = list_grid(width, height, list_bin);
            const int tiles = lg.lists();
            const ListsWorkspace lw = lists_workspace(k, tiles, lg.shift != 0);
            const Sort32Workspace w = sort32_workspace(k, slot_bits(tiles), sort32_tile_keys(k));
            *partition_flag =
                reinterpret_cast<const uint32_t*>(static_cast<const char*>(workspace) + lw.sort + w.counters) + w.passes;
        }
    }
    return DSX_OK;
}

extern "C" int dsx_tile_lists(const dsx_camera* cam, int64_t n, int64_t k, const void* order, int32_t* sorted_ids,
                              int32_t* ranges, void* workspace, size_t workspace_bytes, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || k < 0 || !ranges)
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    if(k > 0 && n > 0)
    {
        if(!order || !sorted_ids || !workspace)
            return DSX_ERR_BAD_ARG;
        if(workspace_bytes < lists_workspace(k, list_grid(*cam).lists(), list_grid(*cam).shift != 0).bytes)
            return DSX_ERR_WORKSPACE;
    }
    return launch_tile_lists(*cam, n, k, order, sorted_ids, ranges, workspace, as_stream(stream));
}

extern "C" int dsx_blend_fwd(const dsx_camera* cam, int64_t n, int64_t k, int32_t* ranges,
                             const int32_t* sorted_ids, const float* splats, float* image, float* final_T,
                             int32_t* final_idx, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || k < 0 || !ranges || !image || !final_T || !final_idx)
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 31))
        return DSX_ERR_TOO_LARGE;
    return launch_blend_fwd(*cam, n, k, ranges, sorted_ids, splats, image, final_T, final_idx, as_stream(stream),
                            false);
}

extern "C" int dsx_blend_bwd(const dsx_camera* cam, int64_t n, int64_t k, const int32_t* ranges,
                             const int32_t* sorted_ids, const float* splats, const float* final_T,
                             const int32_t* final_idx, const float* v_image, float* grads, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || k < 0)
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 31))
        return DSX_ERR_TOO_LARGE;
    if(n == 0)
        return DSX_OK;
    if(!ranges || !final_T || !final_idx || !v_image || !grads || !splats)
        return DSX_ERR_BAD_ARG;
    return launch_blend_bwd(*cam, n, k, ranges, sorted_ids, splats, final_T, final_idx, v_image, grads,
                            as_stream(stream), false);
}

// conic_in_grads: places 9..11 of every accumulator record hold the conic (dsx_forward_finish put it there)
static int gaussian_bwd_checked(const dsx_camera* cam, int64_t n, int32_t num_bases, const float* means3d,
                                const float* scales, const float* quats, const float* splats, const float* cov3d,
                                const int32_t* radii, const float* grads, float* v_mean3d, float* v_means2d,
                                float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                                float* v_cov3d, void* stream, bool conic_in_grads, bool outputs_cleared = false,
                                bool with_marks = false)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || num_bases < 0 || num_bases > 16)
        return DSX_ERR_BAD_ARG;
    if(n == 0)
        return DSX_OK;
    if(!means3d || !splats || !radii || !grads)
        return DSX_ERR_BAD_ARG; // any of the outputs may be null: that gradient is not wanted
    if((scales == nullptr) != (quats == nullptr))
        return DSX_ERR_BAD_ARG;
    if(!cov3d && !scales)
        return DSX_ERR_BAD_ARG; // without the stored covariance the kernel rebuilds it from scale and rotation
    return launch_gaussian_bwd(*cam, n, num_bases, means3d, scales, quats, splats, cov3d, radii, grads, v_mean3d,
                               v_means2d, num_bases > 0 ? v_shs : nullptr, v_colors, v_opacity, v_scale, v_quat,
                               v_cov3d, as_stream(stream), conic_in_grads, outputs_cleared, with_marks);
}

extern "C" int dsx_gaussian_bwd(const dsx_camera* cam, int64_t n, int32_t num_bases, const float* means3d,
                                const float* scales, const float* quats, const float* splats, const float* cov3d,
                                const int32_t* radii, const float* grads, float* v_mean3d, float* v_means2d,
                                float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                                float* v_cov3d, void* stream)
{
    return gaussian_bwd_checked(cam, n, num_bases, means3d, scales, quats, splats, cov3d, radii, grads, v_mean3d,
                                v_means2d, v_shs, v_colors, v_opacity, v_scale, v_quat, v_cov3d, stream, false);
}

// The pair counts a forward can index: the lists that are built are sorted with 30-bit counters, and
// the per-tile pairs (the reference's K) are what the fine ranges, final_idx and the walk records
// index as int32.  With binned lists the first is a fraction of the second, so both are checked.
static int check_pair_counts(int64_t list_pairs, int64_t tile_pairs)
{
    if(list_pairs < 0 || tile_pairs < 0 || list_pairs >= (1ll << 30) || tile_pairs >= (1ll << 31))
        return DSX_ERR_TOO_LARGE;
    return DSX_OK;
}

extern "C" int dsx_forward_project(const dsx_camera* cam, int64_t n, const float* means3d, const float* scales,
                                   const float* quats, const float* opacities, const float* shs,
                                   const float* cov3d_precomp, const float* colors_precomp, float* splats,
                                   int32_t* radii, float* cov3d, uint32_t* block_sums, void* order, size_t order_bytes,
                                   int64_t* num_keys, void* stream)
{
    if(!num_keys || (n > 0 && !order))
        return DSX_ERR_BAD_ARG;
    num_keys[0] = num_keys[1] = 0;
    hipStream_t s = as_stream(stream);
    int rc = project_fwd_checked(cam, n, means3d, scales, quats, opacities, shs, cov3d_precomp, colors_precomp,
                                 splats, radii, cov3d, block_sums, order, order_bytes, stream, true);
    if(rc || n == 0)
        return rc;
    // The pair counts are sums over the rectangles: the corner-grid kernel, first thing beside the
    // depth sort, adds them up, and they travel to the host while the depth order is computed.  The
    // wait below is for that copy only (it overlaps when num_keys is pinned host memory; with
    // pageable memory the copy is synchronous and nothing is lost).
    hipEvent_t copied;
    if(hipEventCreateWithFlags(&copied, hipEventDisableTiming) != hipSuccess)
        return DSX_ERR_RUNTIME;
    rc = launch_depth_order(*cam, n, order, s, true, num_keys, copied);
    // (an event that was never recorded counts as complete: no wait after a failed launch)
    const bool ok = hipEventSynchronize(copied) == hipSuccess;
    (void)hipEventDestroy(copied);
    if(rc)
        return rc;
    if(!ok)
        return DSX_ERR_RUNTIME;
    // the device wrote (per-tile pairs, bin pairs); the caller gets (pairs of the lists, per-tile pairs)
    const int64_t tile_pairs = num_keys[0], bin_pairs = num_keys[1];
    num_keys[0] = list_grid(*cam).shift ? bin_pairs : tile_pairs;
    num_keys[1] = tile_pairs;
    return check_pair_counts(num_keys[0], num_keys[1]);
}

extern "C" int dsx_forward_finish(const dsx_camera* cam, int64_t n, int64_t k, const float* splats,
                                  const void* order, int32_t* sorted_ids, int32_t* ranges, float* image,
                                  float* final_T, int32_t* final_idx, void* workspace, size_t workspace_bytes,
                                  float* grads_to_prepare, void* stream)
{
    if(!image || !final_T || !final_idx)
        return DSX_ERR_BAD_ARG;
    int rc = dsx_tile_lists(cam, n, k, order, sorted_ids, ranges, workspace, workspace_bytes, stream);
    if(rc)
        return rc;
    const uint32_t *depth_flag = nullptr, *partition_flag = nullptr;
    rc = dsx_sort_flags(n, k, cam->image_width, cam->image_height, cam->list_bin, order, workspace, &depth_flag,
                        &partition_flag);
    if(rc)
        return rc;
    return launch_blend_fwd(*cam, n, n > 0 ? k : 0, ranges, sorted_ids, splats, image, final_T, final_idx,
                            as_stream(stream), true, depth_flag, partition_flag, n > 0 ? grads_to_prepare : nullptr,
                            true);
}

static int backward_impl(const dsx_camera* cam, int64_t n, int64_t k, int32_t num_bases, const float* means3d,
                         const float* scales, const float* quats, const float* splats, const float* cov3d,
                         const int32_t* radii, const int32_t* ranges, const int32_t* sorted_ids,
                         const float* final_T, const int32_t* final_idx, const float* v_image, float* grads,
                         int32_t grads_prepared, float* v_mean3d, float* v_means2d, float* v_shs, float* v_colors,
                         float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d, void* stream)
{
    if(int rc = check_camera(cam))
        return rc;
    if(n < 0 || k < 0 || num_bases < 0 || num_bases > 16)
        return DSX_ERR_BAD_ARG;
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    if(n == 0)
        return DSX_OK;
    if(!ranges || !final_T || !final_idx || !v_image || !grads || !splats || (k > 0 && !sorted_ids))
        return DSX_ERR_BAD_ARG;
    // The per-Gaussian kernel writes only the Gaussians that received a gradient term; everything
    // else in its outputs is zero: 260 bytes per Gaussian of plain stores, which the wavefronts of the
    // blend kernel (bound by its arithmetic, the memory system idle) issue on their way out.
    const ZeroJobs zeros = make_zero_jobs(n, num_bases, v_mean3d, v_means2d, v_shs, v_colors, v_opacity, v_scale,
                                          v_quat, v_cov3d);
    int rc = launch_blend_bwd(*cam, n, k, ranges, sorted_ids, splats, final_T, final_idx, v_image, grads,
                              as_stream(stream), true, grads_prepared != 0, true, &zeros);
    if(rc)
        return rc;
    return gaussian_bwd_checked(cam, n, num_bases, means3d, scales, quats, splats, cov3d, radii, grads, v_mean3d,
                                v_means2d, v_shs, v_colors, v_opacity, v_scale, v_quat, v_cov3d, stream,
                                grads_prepared != 0, true, true);
}

extern "C" int dsx_backward(const dsx_camera* cam, int64_t n, int64_t k, int32_t num_bases, const float* means3d,
                            const float* scales, const float* quats, const float* splats, const float* cov3d,
                            const int32_t* radii, const int32_t* ranges, const int32_t* sorted_ids,
                            const float* final_T, const int32_t* final_idx, const float* v_image, float* grads,
                            int32_t grads_prepared, float* v_mean3d, float* v_means2d, float* v_shs, float* v_colors,
                            float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d, void* stream)
{
    return backward_impl(cam, n, k, num_bases, means3d, scales, quats, splats, cov3d, radii, ranges, sorted_ids,
                         final_T, final_idx, v_image, grads, grads_prepared, v_mean3d, v_means2d, v_shs, v_colors,
                         v_opacity, v_scale, v_quat, v_cov3d, stream);
}

extern "C" int dsx_forward_core(const float* means3d, const float* shs, const float* opacities, const float* scales,
                                const float* quats, int64_t n, const float* view, const float* proj,
                                const float* campos, int32_t image_width, int32_t image_height, float tanfovx,
                                float tanfovy, float scale_modifier, int32_t max_sh_degree, int32_t sh_degree,
                                float* image, void* stream)
{
    hipStream_t s = as_stream(stream);
    dsx_camera cam;
    cam.image_height = image_height;
    cam.image_width = image_width;
    cam.tanfovx = tanfovx;
    cam.tanfovy = tanfovy;
    cam.scale_modifier = scale_modifier;
    cam.sh_degree = sh_degree;
    cam.max_sh_degree = max_sh_degree;
    cam.view = view;
    cam.proj = proj;
    cam.campos = campos;
    cam.bg = campos; // unused by the forward
    cam.list_bin = 0;
    if(int rc = check_camera(&cam))
        return rc;
    if(n < 0 || !image)
        return DSX_ERR_BAD_ARG;
    const int64_t P = (int64_t)image_width * image_height;
    const int64_t nb = dsx_num_blocks(n);

    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    size_t o_splats = 0, o_radii, o_cov3d, o_bs, o_ranges, o_T, o_idx, o_order, stage1;
    o_radii = align(o_splats + (size_t)n * 48);
    o_cov3d = align(o_radii + (size_t)n * 4);
    o_bs = align(o_cov3d + (size_t)n * 24);
    o_ranges = align(o_bs + (size_t)nb * 4);
    o_T = align(o_ranges + (size_t)dsx_ranges_count(image_width, image_height, 0) * 4);
    o_idx = align(o_T + (size_t)P * 4);
    o_order = align(o_idx + (size_t)P * 4);
    const size_t order_bytes = order_layout(n, image_width, image_height, 0).bytes;
    stage1 = align(o_order + order_bytes);
    char* buf = nullptr;
    if(hipMallocAsync(reinterpret_cast<void**>(&buf), stage1 + 256, s) != hipSuccess)
        return DSX_ERR_RUNTIME;
    int64_t counts[2] = {0, 0};
    int rc = dsx_forward_project(&cam, n, means3d, scales, quats, opacities, shs, nullptr, nullptr,
                                 reinterpret_cast<float*>(buf + o_splats), reinterpret_cast<int32_t*>(buf + o_radii),
                                 reinterpret_cast<float*>(buf + o_cov3d), reinterpret_cast<uint32_t*>(buf + o_bs),
                                 buf + o_order, order_bytes, counts, stream);
    const int64_t k = counts[0];
    char* buf2 = nullptr;
    if(rc == DSX_OK)
    {
        const size_t ws = lists_workspace(k, list_grid(cam).lists(), list_grid(cam).shift != 0).bytes;
        const size_t o_ids = align(ws);
        if(hipMallocAsync(reinterpret_cast<void**>(&buf2), o_ids + (size_t)dsx_sorted_ids_count(k, image_width, image_height, 0) * 4 + 256, s) != hipSuccess)
            rc = DSX_ERR_RUNTIME;
        else
            rc = dsx_forward_finish(&cam, n, k, reinterpret_cast<float*>(buf + o_splats), buf + o_order,
                                    reinterpret_cast<int32_t*>(buf2 + o_ids),
                                    reinterpret_cast<int32_t*>(buf + o_ranges), image,
                                    reinterpret_cast<float*>(buf + o_T), reinterpret_cast<int32_t*>(buf + o_idx),
                                    buf2, ws, nullptr, stream);
    }
    if(buf2)
        (void)hipFreeAsync(buf2, s);
    (void)hipFreeAsync(buf, s);
    return rc;
}

// ---- backward without a caller-provided accumulator ---------------------------------------
// The gradient accumulator of dsx_backward ([n * 12] floats of scratch) lives in a file-scope
// device array here.  In host code the array's NAME is only a stand-in: each device holds its own
// copy at its own address, which hipGetSymbolAddress returns; that address is what the kernels get.
namespace
{
constexpr int64_t kStaticMaxGaussians = DSX_STATIC_MAX_GAUSSIANS;
// (the accumulator records and, behind them, the byte per Gaussian: grads_bytes(kStaticMaxGaussians))
static __device__ __align__(256) float scratch[kStaticMaxGaussians * DSX_GRAD_FLOATS + kStaticMaxGaussians / 4];
static_assert(sizeof(scratch) >= grads_bytes(kStaticMaxGaussians), "records and marks of the largest call");

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device (looked up once per device), or null
float* static_scratch()
{
    int device = -1;
    if(hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
        return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if(g_scratch_ptr[device] == nullptr)
    {
        void* p = nullptr;
        if(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess)
            return nullptr;
        g_scratch_ptr[device] = static_cast<float*>(p);
    }
    return g_scratch_ptr[device];
}
} // namespace

extern "C" int dsx_backward_static(const dsx_camera* cam, int64_t n, int64_t k, int32_t num_bases,
                                   const float* means3d,
                                   const float* scales, const float* quats, const float* splats,
                                   const float* cov3d, const int32_t* radii, const int32_t* ranges,
                                   const int32_t* sorted_ids, const float* final_T, const int32_t* final_idx,
                                   const float* v_image, float* v_mean3d, float* v_means2d, float* v_shs,
                                   float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                                   float* v_cov3d, void* stream)
{
    if(n > kStaticMaxGaussians)
        return DSX_ERR_STATIC_LIMIT;
    // (n <= 0 touches no memory: dsx_backward rejects a negative n and returns at n == 0)
    float* grads = n > 0 ? static_scratch() : nullptr;
    if(n > 0 && grads == nullptr)
        return DSX_ERR_RUNTIME;
    // grads_prepared = 0: the array keeps the last call's sums, so this call clears its n records
    // itself (a fill kernel with plain stores, which a caller may capture in a graph)
    return backward_impl(cam, n, k, num_bases, means3d, scales, quats, splats, cov3d, radii, ranges, sorted_ids,
                         final_T, final_idx, v_image, grads, 0, v_mean3d, v_means2d, v_shs, v_colors, v_opacity, v_scale,
                         v_quat, v_cov3d, stream);
}

extern "C" int dsx_set_blend_pixels_per_lane(int pixels)
{
    return set_blend_pixels_per_lane(pixels);
}
