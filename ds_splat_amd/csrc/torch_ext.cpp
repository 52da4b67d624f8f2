// Thin PyTorch binding over the C ABI of libdsx (include/dsx.h): it owns no kernels and no
// HIP calls.  It plays the role of the reference's pybind module ds_splat_cuda
// (cpp/rasterizer_python.cpp:3-23) and of the tensor plumbing in cpp/rasterizer_torch.cu:170-316:
// allocate the outputs as torch tensors, hand raw device pointers and the caller's stream to
// the library, return the tensors the autograd function keeps for the backward.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>

#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "dsx.h"

namespace
{

void check(int status)
{
    if(status != DSX_OK)
        throw std::runtime_error(dsx_error_string(status));
}

const float* fptr(const c10::optional<at::Tensor>& t)
{
    return (t.has_value() && t->defined() && t->numel() > 0) ? t->data_ptr<float>() : nullptr;
}

struct Camera
{
    at::Tensor view, proj, campos, bg; // float32, contiguous, on the device: kept alive for the call
    dsx_camera c;
};

Camera make_camera(int64_t height, int64_t width, double tanfovx, double tanfovy, double scale_modifier,
                   int64_t sh_degree, int64_t max_sh_degree, const at::Tensor& view, const at::Tensor& proj,
                   const at::Tensor& campos, const at::Tensor& bg, int64_t list_bin, const at::Device& dev)
{
    Camera cam;
    auto prep = [&](const at::Tensor& t) { return t.to(dev, at::kFloat).contiguous(); };
    cam.view = prep(view);
    cam.proj = prep(proj);
    cam.campos = prep(campos);
    cam.bg = prep(bg);
    TORCH_CHECK(cam.view.numel() == 16 && cam.proj.numel() == 16 && cam.campos.numel() >= 3 && cam.bg.numel() >= 3,
                "camera tensors must be 4x4, 4x4, [3], [3]");
    cam.c.image_height = (int32_t)height;
    cam.c.image_width = (int32_t)width;
    cam.c.tanfovx = (float)tanfovx;
    cam.c.tanfovy = (float)tanfovy;
    cam.c.scale_modifier = (float)scale_modifier;
    cam.c.sh_degree = (int32_t)sh_degree;
    cam.c.max_sh_degree = (int32_t)max_sh_degree;
    cam.c.view = cam.view.data_ptr<float>();
    cam.c.proj = cam.proj.data_ptr<float>();
    cam.c.campos = cam.campos.data_ptr<float>();
    cam.c.bg = cam.bg.data_ptr<float>();
    TORCH_CHECK(list_bin == 0 || list_bin == 1 || list_bin == 2 || list_bin == 4 || list_bin == 8,
                "list_bin must be 0 (the library's choice), 1, 2, 4 or 8 tiles a side");
    cam.c.list_bin = (int32_t)list_bin;
    return cam;
}

at::Tensor& pinned_key_count()
{
    // two pinned int64 per host thread: the landing place of the two pair counts
    thread_local at::Tensor slot = at::zeros({2}, at::TensorOptions().dtype(at::kLong).pinned_memory(true));
    return slot;
}

} // namespace

// list_bin: tiles per side of the bins that the tile lists are built for (0: the library's choice);
// the backward of this forward must be given the same value.
// image[H,W,3], radii[N], splats[N,12], sorted_ids[dsx_sorted_ids_count(K)], ranges[dsx_ranges_count], final_T[H,W], final_idx[H,W]
// (the 3-D covariances are not kept: the backward rebuilds them from scales and rotations, or
// reads cov3d_precomp) and, when prepare_backward is set, the backward's gradient accumulator
// (dsx_grads_bytes(N) bytes as float32), which the blend kernel prepares on the side: sums zeroed,
// conics in the spare places, the byte per Gaussian behind the records cleared (undefined otherwise)
std::vector<at::Tensor> forward(int64_t height, int64_t width, double tanfovx, double tanfovy, double scale_modifier,
                                int64_t sh_degree, int64_t max_sh_degree, const at::Tensor& view,
                                const at::Tensor& proj, const at::Tensor& campos, const at::Tensor& bg,
                                int64_t list_bin, const at::Tensor& means3d, const c10::optional<at::Tensor>& scales,
                                const c10::optional<at::Tensor>& quats, const at::Tensor& opacities,
                                const c10::optional<at::Tensor>& shs, const c10::optional<at::Tensor>& cov3d_precomp,
                                const c10::optional<at::Tensor>& colors_precomp, bool prepare_backward,
                                int64_t stream)
{
    const at::Device dev = means3d.device();
    c10::DeviceGuard guard(dev);
    Camera cam = make_camera(height, width, tanfovx, tanfovy, scale_modifier, sh_degree, max_sh_degree, view, proj,
                             campos, bg, list_bin, dev);
    const int64_t n = means3d.numel() / 3;
    const auto f32 = at::TensorOptions().dtype(at::kFloat).device(dev);
    const auto i32 = at::TensorOptions().dtype(at::kInt).device(dev);
    const auto u8 = at::TensorOptions().dtype(at::kByte).device(dev);
    void* s = reinterpret_cast<void*>(stream);

    at::Tensor splats = at::empty({n, DSX_SPLAT_FLOATS}, f32);
    at::Tensor radii = at::empty({n}, i32);
    at::Tensor block_sums = at::empty({std::max<int64_t>(dsx_num_blocks(n), 1)}, i32);
    const size_t order_bytes = dsx_order_bytes(n, (int32_t)width, (int32_t)height, cam.c.list_bin);
    at::Tensor order = at::empty({(int64_t)std::max<size_t>(order_bytes, 1)}, u8);
    at::Tensor& k_host = pinned_key_count();
    uint32_t* bs = reinterpret_cast<uint32_t*>(block_sums.data_ptr<int32_t>());
    check(dsx_forward_project(&cam.c, n, means3d.data_ptr<float>(), fptr(scales), fptr(quats),
                              opacities.data_ptr<float>(), fptr(shs), fptr(cov3d_precomp), fptr(colors_precomp),
                              splats.data_ptr<float>(), radii.data_ptr<int32_t>(), nullptr, bs, order.data_ptr(),
                              order_bytes, k_host.data_ptr<int64_t>(), s));
    const int64_t k = *k_host.data_ptr<int64_t>();
    at::Tensor sorted_ids = at::empty({dsx_sorted_ids_count(k, (int32_t)width, (int32_t)height, cam.c.list_bin)}, i32);
    at::Tensor ranges = at::empty({dsx_ranges_count((int32_t)width, (int32_t)height, cam.c.list_bin)}, i32);
    at::Tensor image = at::empty({height, width, 3}, f32);
    at::Tensor final_T = at::empty({height, width}, f32);
    at::Tensor final_idx = at::empty({height, width}, i32);
    const size_t ws_bytes = dsx_workspace_bytes(n, k, (int32_t)width, (int32_t)height, cam.c.list_bin);
    at::Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 1)}, u8);
    at::Tensor grads = prepare_backward && n > 0 ? at::empty({(int64_t)(dsx_grads_bytes(n) / 4)}, f32) : at::Tensor();
    check(dsx_forward_finish(&cam.c, n, k, splats.data_ptr<float>(), order.data_ptr(), sorted_ids.data_ptr<int32_t>(),
                             ranges.data_ptr<int32_t>(), image.data_ptr<float>(), final_T.data_ptr<float>(),
                             final_idx.data_ptr<int32_t>(), ws.data_ptr(), ws_bytes,
                             grads.defined() ? grads.data_ptr<float>() : nullptr, s));
    return {image, radii, splats, sorted_ids, ranges, final_T, final_idx, grads};
}

// v_mean3d[N,3], v_means2d[N,3], v_shs[N,B,3] (undefined when num_bases == 0), v_colors[N,3],
// v_opacity[N,1], v_scale[N,3], v_quat[N,4], v_cov3d[N,6].  Bit i of `wanted` asks for the i-th
// of them; the others are neither allocated nor written and come back undefined (None).
std::vector<at::Tensor> backward(int64_t height, int64_t width, double tanfovx, double tanfovy, double scale_modifier,
                                 int64_t sh_degree, int64_t max_sh_degree, const at::Tensor& view,
                                 const at::Tensor& proj, const at::Tensor& campos, const at::Tensor& bg,
                                 int64_t list_bin, int64_t num_bases, const at::Tensor& means3d, const c10::optional<at::Tensor>& scales,
                                 const c10::optional<at::Tensor>& quats, const at::Tensor& splats,
                                 const c10::optional<at::Tensor>& cov3d_precomp, const at::Tensor& radii,
                                 const at::Tensor& ranges,
                                 const at::Tensor& sorted_ids, const at::Tensor& final_T, const at::Tensor& final_idx,
                                 const at::Tensor& v_image, const c10::optional<at::Tensor>& prepared_grads,
                                 int64_t wanted, int64_t stream)
{
    const at::Device dev = means3d.device();
    c10::DeviceGuard guard(dev);
    Camera cam = make_camera(height, width, tanfovx, tanfovy, scale_modifier, sh_degree, max_sh_degree, view, proj,
                             campos, bg, list_bin, dev);
    const int64_t n = means3d.numel() / 3;
    const auto f32 = at::TensorOptions().dtype(at::kFloat).device(dev);
    TORCH_CHECK(v_image.is_contiguous() && v_image.scalar_type() == at::kFloat && v_image.numel() == height * width * 3,
                "v_image must be a contiguous float32 [H, W, 3] tensor");
    // The lists that `ranges` and `sorted_ids` describe are per tile or per bin of tiles, as the forward was
    // told (list_bin); the library compares the buffer's header word with this call's bin size on the device.
    TORCH_CHECK(ranges.is_contiguous() && ranges.scalar_type() == at::kInt &&
                    ranges.numel() == dsx_ranges_count((int32_t)width, (int32_t)height, cam.c.list_bin),
                "ranges does not have the layout of this image size and bin size (the backward must be given the "
                "list_bin of its forward)");
    TORCH_CHECK(sorted_ids.is_contiguous() && sorted_ids.scalar_type() == at::kInt, "sorted_ids must be int32");
    // pairs in sorted_ids: the buffer holds k ids and, for lists per bin, k more words
    const int64_t words_per_pair = dsx_sorted_ids_count(1, (int32_t)width, (int32_t)height, cam.c.list_bin);
    TORCH_CHECK(words_per_pair > 0 && sorted_ids.numel() % words_per_pair == 0, "sorted_ids has the wrong size");
    const int64_t k = sorted_ids.numel() / words_per_pair;
    auto out = [&](int bit, std::initializer_list<int64_t> shape) {
        return (wanted >> bit) & 1 ? at::empty(shape, f32) : at::Tensor();
    };
    auto ptr = [](const at::Tensor& t) { return t.defined() ? t.data_ptr<float>() : nullptr; };
    if(num_bases <= 0 || !((wanted >> 2) & 1))
        num_bases = 0;
    at::Tensor v_mean3d = out(0, {n, 3}), v_means2d = out(1, {n, 3});
    at::Tensor v_shs = num_bases > 0 ? at::empty({n, num_bases, 3}, f32) : at::Tensor();
    at::Tensor v_colors = out(3, {n, 3}), v_opacity = out(4, {n, 1});
    at::Tensor v_scale = out(5, {n, 3}), v_quat = out(6, {n, 4}), v_cov3d = out(7, {n, 6});
    // the accumulator that the forward prepared (sums zeroed, conics in place; good for one
    // backward), or a new one that the call fills
    const bool prepared = prepared_grads.has_value() && prepared_grads->defined();
    if(prepared)
        TORCH_CHECK(prepared_grads->is_contiguous() && prepared_grads->scalar_type() == at::kFloat &&
                        prepared_grads->numel() == (int64_t)(dsx_grads_bytes(n) / 4) && prepared_grads->device() == dev,
                    "prepared_grads must be the float32 accumulator of this forward (dsx_grads_bytes(N) bytes)");
    at::Tensor grads = prepared ? *prepared_grads : at::empty({(int64_t)(dsx_grads_bytes(n) / 4)}, f32);
    check(dsx_backward(&cam.c, n, k, (int32_t)num_bases, means3d.data_ptr<float>(), fptr(scales),
                       fptr(quats),
                       splats.data_ptr<float>(), fptr(cov3d_precomp), radii.data_ptr<int32_t>(),
                       ranges.data_ptr<int32_t>(), sorted_ids.numel() ? sorted_ids.data_ptr<int32_t>() : nullptr,
                       final_T.data_ptr<float>(), final_idx.data_ptr<int32_t>(), v_image.data_ptr<float>(),
                       grads.data_ptr<float>(), prepared ? 1 : 0, ptr(v_mean3d), ptr(v_means2d), ptr(v_shs), ptr(v_colors),
                       ptr(v_opacity), ptr(v_scale), ptr(v_quat), ptr(v_cov3d), reinterpret_cast<void*>(stream)));
    return {v_mean3d, v_means2d, v_shs, v_colors, v_opacity, v_scale, v_quat, v_cov3d};
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "torch binding of libdsx (gfx950 3D-Gaussian-Splatting rasterizer)";
    m.def("forward", &forward, "projection, tile lists and blend; returns the tensors the backward needs");
    m.def("backward", &backward, "blend backward and per-Gaussian backward");
    m.def("version", []() { return dsx_version(); });
}
