// Python module `flash_gaussian_splatting` with submodule `ops`: the op surface of FlashGS
// (csrc/pybind.cpp:122-271 of the reference) on top of the C ABI of libflashgs_hip.so.
//
// Names, positional argument order, tensor layouts and dtypes are the reference's, so a caller
// written like its example.py:47-94 runs unchanged.  Differences, all on the strict side:
//  * inputs are validated (device, dtype, contiguity, sizes) and a RuntimeError is raised
//    instead of reading garbage; output tensors must be contiguous because they are written in
//    place (the reference calls .contiguous() on outputs, which would silently write to a copy);
//  * work is enqueued on torch's current HIP stream of the tensors' device, not on stream 0;
//  * preprocess never writes past the end of the key/value tensors.
// This file is host-only C++ (g++); it contains no device code.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <fstream>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "flashgs_hip.h"
#include "ply_reader.h"

namespace {

void fgs_check(int rc, const char* op)
{
    if (rc != FGS_OK) throw std::runtime_error(std::string(op) + ": " + fgs_last_error());
}

void need(bool ok, const std::string& msg)
{
    if (!ok) throw std::runtime_error(msg);
}

void need_device(const torch::Tensor& t, const char* name, torch::ScalarType dt, int64_t min_numel, const torch::Tensor& like)
{
    need(t.is_cuda(), std::string(name) + " must be a GPU tensor");
    need(t.scalar_type() == dt, std::string(name) + " has the wrong dtype");
    need(t.is_contiguous(), std::string(name) + " must be contiguous");
    need(t.numel() >= min_numel, std::string(name) + " is too small");
    need(t.device() == like.device(), std::string(name) + " is on a different device");
}

// host tensor of n floats (pybind.cpp:131-132,177 read such tensors with data_ptr<float>())
std::vector<float> host_floats(const torch::Tensor& t, const char* name, int64_t n)
{
    need(!t.is_cuda(), std::string(name) + " must be a CPU tensor");
    need(t.scalar_type() == torch::kFloat32, std::string(name) + " must be float32");
    need(t.numel() == n, std::string(name) + " has the wrong number of elements");
    torch::Tensor c = t.contiguous();
    const float* p = c.data_ptr<float>();
    return std::vector<float>(p, p + n);
}

// Makes the tensors' device current for the duration of a call (the C ABI works on the current
// device) and restores the previous one afterwards.
struct DeviceScope {
    int previous = -1;
    explicit DeviceScope(const torch::Tensor& on)
    {
        const int want = on.device().index();
        if (hipGetDevice(&previous) != hipSuccess) throw std::runtime_error("hipGetDevice failed");
        if (want >= 0 && want != previous && hipSetDevice(want) != hipSuccess)
            throw std::runtime_error("hipSetDevice failed");
    }
    ~DeviceScope()
    {
        int now = -1;
        if (hipGetDevice(&now) == hipSuccess && now != previous && previous >= 0) (void)hipSetDevice(previous);
    }
};

void* current_stream(const torch::Tensor& on)
{
    return (void*)c10::hip::getCurrentHIPStream(on.device().index()).stream();
}

// ---- ops -----------------------------------------------------------------------------------------

// pybind.cpp:122-150
void preprocess_to(torch::Tensor& orig_points, torch::Tensor& shs, torch::Tensor& opacities, torch::Tensor& cov3Ds,
                   int width, int height, int block_x, int block_y,
                   torch::Tensor& position, torch::Tensor& rotation,
                   float focal_x, float focal_y, float zFar, float zNear,
                   torch::Tensor& points_xy, torch::Tensor& rgb_depth, torch::Tensor& conic_opacity,
                   torch::Tensor& gaussian_keys_unsorted, torch::Tensor& gaussian_values_unsorted,
                   torch::Tensor& curr_offset, int* count_mirror)
{
    need(opacities.dim() >= 1, "opacities must have at least one dimension");
    const int64_t P = opacities.size(0);
    need(P <= INT32_MAX, "too many Gaussians");
    need_device(opacities, "opacities", torch::kFloat32, P, opacities);
    need_device(orig_points, "orig_points", torch::kFloat32, 3 * P, opacities);
    need_device(shs, "shs", torch::kFloat32, 48 * P, opacities);
    need_device(cov3Ds, "cov3Ds", torch::kFloat32, 6 * P, opacities);
    need_device(points_xy, "points_xy", torch::kFloat32, 2 * P, opacities);
    need_device(rgb_depth, "rgb_depth", torch::kFloat32, 4 * P, opacities);
    need_device(conic_opacity, "conic_opacity", torch::kFloat32, 4 * P, opacities);
    need_device(gaussian_keys_unsorted, "gaussian_keys_unsorted", torch::kInt64, 0, opacities);
    need_device(gaussian_values_unsorted, "gaussian_values_unsorted", torch::kInt32, 0, opacities);
    need_device(curr_offset, "curr_offset", torch::kInt32, 1, opacities);
    const std::vector<float> pos = host_floats(position, "position", 3);
    const std::vector<float> rot = host_floats(rotation, "rotation", 9);
    const int64_t capacity = std::min(gaussian_keys_unsorted.numel(), gaussian_values_unsorted.numel());
    need(capacity > 0, "gaussian_keys_unsorted / gaussian_values_unsorted are empty");

    DeviceScope scope(opacities);
    if (count_mirror) {
        *count_mirror = FGS_COUNT_PENDING;
        fgs_check(fgs_preprocess_mirrored((int)P,
                                          orig_points.data_ptr<float>(), shs.data_ptr<float>(), opacities.data_ptr<float>(),
                                          cov3Ds.data_ptr<float>(), width, height, block_x, block_y, pos.data(), rot.data(),
                                          focal_x, focal_y, zFar, zNear,
                                          points_xy.data_ptr<float>(), rgb_depth.data_ptr<float>(), conic_opacity.data_ptr<float>(),
                                          (uint64_t*)gaussian_keys_unsorted.data_ptr<int64_t>(),
                                          (uint32_t*)gaussian_values_unsorted.data_ptr<int>(),
                                          curr_offset.data_ptr<int>(), capacity, count_mirror, current_stream(opacities)),
                  "preprocess_mirrored");
        return;
    }
    fgs_check(fgs_preprocess((int)P,
                             orig_points.data_ptr<float>(), shs.data_ptr<float>(), opacities.data_ptr<float>(),
                             cov3Ds.data_ptr<float>(), width, height, block_x, block_y, pos.data(), rot.data(),
                             focal_x, focal_y, zFar, zNear,
                             points_xy.data_ptr<float>(), rgb_depth.data_ptr<float>(), conic_opacity.data_ptr<float>(),
                             (uint64_t*)gaussian_keys_unsorted.data_ptr<int64_t>(),
                             (uint32_t*)gaussian_values_unsorted.data_ptr<int>(),
                             curr_offset.data_ptr<int>(), capacity, current_stream(opacities)),
              "preprocess");
}

// pybind.cpp:122-150
void preprocess(torch::Tensor& orig_points, torch::Tensor& shs, torch::Tensor& opacities, torch::Tensor& cov3Ds,
                int width, int height, int block_x, int block_y,
                torch::Tensor& position, torch::Tensor& rotation,
                float focal_x, float focal_y, float zFar, float zNear,
                torch::Tensor& points_xy, torch::Tensor& rgb_depth, torch::Tensor& conic_opacity,
                torch::Tensor& gaussian_keys_unsorted, torch::Tensor& gaussian_values_unsorted,
                torch::Tensor& curr_offset)
{
    preprocess_to(orig_points, shs, opacities, cov3Ds, width, height, block_x, block_y, position, rotation,
                  focal_x, focal_y, zFar, zNear, points_xy, rgb_depth, conic_opacity,
                  gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset, nullptr);
}

int* mirror_word(torch::Tensor& count_mirror)
{
    need(!count_mirror.is_cuda() && count_mirror.is_pinned() && count_mirror.scalar_type() == torch::kInt32 &&
             count_mirror.numel() >= 1 && count_mirror.is_contiguous(),
         "count_mirror must be a pinned int32 host tensor (torch.zeros(1, dtype=torch.int32, pin_memory=True))");
    return count_mirror.data_ptr<int>();
}

// No counterpart in the reference: preprocess that also stores the pair count into `count_mirror`,
// pinned host memory, as soon as the launch knows it (fgs_preprocess_mirrored); wait_count polls it.
void preprocess_mirrored(torch::Tensor& orig_points, torch::Tensor& shs, torch::Tensor& opacities, torch::Tensor& cov3Ds,
                         int width, int height, int block_x, int block_y,
                         torch::Tensor& position, torch::Tensor& rotation,
                         float focal_x, float focal_y, float zFar, float zNear,
                         torch::Tensor& points_xy, torch::Tensor& rgb_depth, torch::Tensor& conic_opacity,
                         torch::Tensor& gaussian_keys_unsorted, torch::Tensor& gaussian_values_unsorted,
                         torch::Tensor& curr_offset, torch::Tensor& count_mirror)
{
    preprocess_to(orig_points, shs, opacities, cov3Ds, width, height, block_x, block_y, position, rotation,
                  focal_x, focal_y, zFar, zNear, points_xy, rgb_depth, conic_opacity,
                  gaussian_keys_unsorted, gaussian_values_unsorted, curr_offset, mirror_word(count_mirror));
}

int wait_count(torch::Tensor& count_mirror, double timeout_seconds)
{
    int count = 0;
    const int* const word = mirror_word(count_mirror);
    py::gil_scoped_release release;
    fgs_check(fgs_wait_count(word, timeout_seconds, &count), "wait_count");
    return count;
}

// pybind.cpp:152-163
void sort_gaussian(int num_rendered, int width, int height, int block_x, int block_y,
                   torch::Tensor& list_sorting_space,
                   torch::Tensor& gaussian_keys_unsorted, torch::Tensor& gaussian_values_unsorted,
                   torch::Tensor& gaussian_keys_sorted, torch::Tensor& gaussian_values_sorted)
{
    need(num_rendered >= 0, "num_rendered is negative");
    need(list_sorting_space.is_cuda() && list_sorting_space.is_contiguous() && list_sorting_space.element_size() == 1,
         "list_sorting_space must be a contiguous 1-byte GPU tensor");
    need_device(gaussian_keys_unsorted, "gaussian_keys_unsorted", torch::kInt64, num_rendered, list_sorting_space);
    need_device(gaussian_values_unsorted, "gaussian_values_unsorted", torch::kInt32, num_rendered, list_sorting_space);
    need_device(gaussian_keys_sorted, "gaussian_keys_sorted", torch::kInt64, num_rendered, list_sorting_space);
    need_device(gaussian_values_sorted, "gaussian_values_sorted", torch::kInt32, num_rendered, list_sorting_space);

    DeviceScope scope(list_sorting_space);
    fgs_check(fgs_sort_gaussian(num_rendered, width, height, block_x, block_y,
                                (char*)list_sorting_space.data_ptr(), (size_t)list_sorting_space.numel(),
                                (const uint64_t*)gaussian_keys_unsorted.data_ptr<int64_t>(),
                                (const uint32_t*)gaussian_values_unsorted.data_ptr<int>(),
                                (uint64_t*)gaussian_keys_sorted.data_ptr<int64_t>(),
                                (uint32_t*)gaussian_values_sorted.data_ptr<int>(),
                                current_stream(list_sorting_space)),
              "sort_gaussian");
}

// pybind.cpp:165-168
size_t get_sort_buffer_size(int num_rendered)
{
    need(num_rendered >= 0 && num_rendered <= FGS_MAX_RENDERED, "num_rendered out of range");
    return fgs_get_sort_buffer_size(num_rendered);
}

// pybind.cpp:170-228
template <int BX, int BY>
void render(int num_rendered, int width, int height,
            torch::Tensor& points_xy, torch::Tensor& rgb_depth, torch::Tensor& conic_opacity,
            torch::Tensor& gaussian_keys_sorted, torch::Tensor& gaussian_values_sorted,
            torch::Tensor& ranges, torch::Tensor& bg_color, torch::Tensor& out_color)
{
    need(num_rendered >= 0, "num_rendered is negative");
    need(width > 0 && height > 0, "width and height must be positive");
    const int64_t tiles = (int64_t)((width + BX - 1) / BX) * ((height + BY - 1) / BY);
    need(out_color.is_cuda() && out_color.is_contiguous() && out_color.element_size() == 1,
         "out_color must be a contiguous 1-byte GPU tensor");
    need(out_color.numel() >= (int64_t)width * height * 3, "out_color is too small");
    need_device(points_xy, "points_xy", torch::kFloat32, 0, out_color);
    need_device(rgb_depth, "rgb_depth", torch::kFloat32, 0, out_color);
    need_device(conic_opacity, "conic_opacity", torch::kFloat32, 0, out_color);
    need(rgb_depth.numel() >= 2 * points_xy.numel() && conic_opacity.numel() >= 2 * points_xy.numel(),
         "points_xy, rgb_depth and conic_opacity disagree on the number of Gaussians");
    need_device(gaussian_keys_sorted, "gaussian_keys_sorted", torch::kInt64, num_rendered, out_color);
    need_device(gaussian_values_sorted, "gaussian_values_sorted", torch::kInt32, num_rendered, out_color);
    need_device(ranges, "ranges", torch::kInt32, 2 * tiles, out_color);
    const std::vector<float> bg = host_floats(bg_color, "bg_color", 3);

    DeviceScope scope(out_color);
    auto fn = BX == 16 ? fgs_render_16x16 : (BY == 16 ? fgs_render_32x16 : fgs_render_32x32);
    fgs_check(fn(num_rendered, width, height,
                 points_xy.data_ptr<float>(), rgb_depth.data_ptr<float>(), conic_opacity.data_ptr<float>(),
                 (const uint64_t*)gaussian_keys_sorted.data_ptr<int64_t>(),
                 (const uint32_t*)gaussian_values_sorted.data_ptr<int>(),
                 ranges.data_ptr<int>(), bg.data(), (uint8_t*)out_color.data_ptr(), current_stream(out_color)),
              "render");
}

// ---- loadPly (pybind.cpp:12-120) --------------------------------------------------------------------
//
// The parsing lives in ply_reader.h (no torch in it).  Returns CPU tensors
// (n, position[n,3], shs[n,48] interleaved per coefficient, opacity[n] after sigmoid,
// cov3d[n,6] = upper triangle of R S^2 R^T).
std::tuple<int, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> loadPly(const std::string& name)
{
    std::ifstream file(name, std::ios::binary);
    if (!file.is_open()) throw std::runtime_error(std::string("Failed to open file: ") + name);
    file.seekg(0, std::ios::end);
    const std::streamoff size = file.tellg();
    file.seekg(0, std::ios::beg);
    if (size < 0) throw std::runtime_error(std::string("Failed to open file: ") + name);
    // the count is bounded by the file's size before anything is allocated for it
    const int n = fgs_ply::read_header(file, (uint64_t)size);

    auto opt = torch::TensorOptions().dtype(torch::kFloat32).device(torch::kCPU);
    torch::Tensor position = torch::empty({n, 3}, opt), shs = torch::empty({n, 48}, opt);
    torch::Tensor opacity = torch::empty({n}, opt), cov3d = torch::empty({n, 6}, opt);
    fgs_ply::read_records(file, n, position.data_ptr<float>(), shs.data_ptr<float>(), opacity.data_ptr<float>(),
                          cov3d.data_ptr<float>());
    return std::make_tuple(n, position, shs, opacity, cov3d);
}

// No counterpart in the reference: clears the scan status that preprocess keeps for the current
// stream of `like`'s device (fgs_reset_scan), the way back after a preprocess reported a negative
// pair count.
void reset_scan(torch::Tensor& like)
{
    need(like.is_cuda(), "reset_scan takes a GPU tensor that names the device");
    DeviceScope scope(like);
    fgs_check(fgs_reset_scan(current_stream(like)), "reset_scan");
}

} // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "MI355X-native drop-in for FlashGS's flash_gaussian_splatting extension";
    auto ops = m.def_submodule("ops", "3DGS forward rasterizer operators");
    ops.def("loadPly", &loadPly, "load .ply file and return gaussian model data");
    ops.def("preprocess", &preprocess, "preprocess gaussian model data and generate key-value pairs");
    ops.def("sort_gaussian", &sort_gaussian, "sort gaussian key-value pairs");
    ops.def("get_sort_buffer_size", &get_sort_buffer_size, "get sort buffer size");
    ops.def("render_16x16", &render<16, 16>, "tile ranges and alpha blending, 16x16 tiles");
    ops.def("render_32x16", &render<32, 16>, "tile ranges and alpha blending, 32x16 tiles");
    ops.def("render_32x32", &render<32, 32>, "tile ranges and alpha blending, 32x32 tiles");
    ops.def("preprocess_mirrored", &preprocess_mirrored,
            "preprocess that also stores the pair count into a pinned host tensor as soon as it is known");
    ops.def("wait_count", &wait_count, "poll the pinned host tensor of preprocess_mirrored for the pair count");
    ops.def("reset_scan", &reset_scan, "clear preprocess's scan status on the tensor's device and current stream");
}
