// flashbevpool_ext: the torch-facing native module of the fused camera->BEV pooling
// operator.  It exports the two entry points of the reference's extension with the same
// names and positional order (flashbev/flashbevpool/src/flash_bevpool.cpp:79-101,168-183,
// 243-246) and does nothing but validate tensors, select the device and PyTorch's current
// HIP stream, and call the C ABI of libflashbev_hip.so.  Unlike the reference it checks
// every argument and raises (c10::Error -> RuntimeError) instead of launching on bad input.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <string>
#include <vector>

#include "flashbev_hip.h"

namespace {

struct DeviceScope {
    int prev = -1;
    explicit DeviceScope(int dev) {
        TORCH_CHECK(hipGetDevice(&prev) == hipSuccess, "flashbevpool_ext: hipGetDevice failed");
        if (prev != dev) {
            TORCH_CHECK(hipSetDevice(dev) == hipSuccess, "flashbevpool_ext: hipSetDevice failed");
        } else {
            prev = -1;
        }
    }
    ~DeviceScope() { if (prev >= 0) (void)hipSetDevice(prev); }
};

int dtype_code(const at::Tensor &t, const char *name) {
    switch (t.scalar_type()) {
        case at::kFloat: return FBEV_F32;
        case at::kHalf: return FBEV_F16;
        case at::kBFloat16: return FBEV_BF16;
        default: TORCH_CHECK(false, "flashbevpool_ext: ", name, " must be float32, float16 or bfloat16, got ",
                             t.scalar_type());
    }
    return -1;
}

// Small integer / float tensors (sizes, ranges) may live on either side; a device tensor
// costs one synchronous copy, as in the reference (flash_bevpool.cpp:118-124).
std::vector<int64_t> host_ints(const at::Tensor &t, int64_t n, const char *name) {
    TORCH_CHECK(t.numel() == n, "flashbevpool_ext: ", name, " must have ", n, " elements, got ", t.numel());
    // host tensors in their usual types are read in place (no temporary tensor per call)
    if (t.device().is_cpu() && t.is_contiguous()) {
        if (t.scalar_type() == at::kInt) {
            const int32_t *v = t.data_ptr<int32_t>();
            return std::vector<int64_t>(v, v + n);
        }
        if (t.scalar_type() == at::kLong) {
            const int64_t *v = t.data_ptr<int64_t>();
            return std::vector<int64_t>(v, v + n);
        }
    }
    at::Tensor h = t.to(at::kCPU, at::kLong).contiguous();
    return std::vector<int64_t>(h.data_ptr<int64_t>(), h.data_ptr<int64_t>() + n);
}

std::vector<float> host_floats(const at::Tensor &t, int64_t n, const char *name) {
    TORCH_CHECK(t.numel() == n, "flashbevpool_ext: ", name, " must have ", n, " elements, got ", t.numel());
    if (t.device().is_cpu() && t.is_contiguous() && t.scalar_type() == at::kFloat) {
        const float *v = t.data_ptr<float>();
        return std::vector<float>(v, v + n);
    }
    at::Tensor h = t.to(at::kCPU, at::kFloat).contiguous();
    return std::vector<float>(h.data_ptr<float>(), h.data_ptr<float>() + n);
}

void check_dev(const at::Tensor &t, const at::Tensor &ref, const char *name) {
    TORCH_CHECK(t.is_cuda(), "flashbevpool_ext: ", name, " must be a GPU tensor");
    TORCH_CHECK(t.device() == ref.device(), "flashbevpool_ext: ", name, " is on ", t.device(), " but depth_params is on ",
                ref.device());
    TORCH_CHECK(t.is_contiguous(), "flashbevpool_ext: ", name, " must be contiguous");
}

// Shapes and dtypes shared by forward and backward.
fbev_problem describe(const at::Tensor &depth, const at::Tensor &feats, const at::Tensor &proj,
                      const at::Tensor &feature_size, const at::Tensor &image_size, const at::Tensor &grid_size,
                      int depth_distribution, float epsilon, float threshold, float depth_min, float depth_step,
                      int reduction) {
    TORCH_CHECK(depth.is_cuda(), "flashbevpool_ext: depth_params must be a GPU tensor");
    TORCH_CHECK(depth.is_contiguous(), "flashbevpool_ext: depth_params must be contiguous");
    check_dev(feats, depth, "image_feats");
    check_dev(proj, depth, "projection_matrices");
    TORCH_CHECK(depth.dim() == 5 && feats.dim() == 5,
                "flashbevpool_ext: depth_params and image_feats must be [B,N,H,W,*], got ", depth.sizes(), " and ",
                feats.sizes());
    for (int d = 0; d < 4; ++d)
        TORCH_CHECK(depth.size(d) == feats.size(d), "flashbevpool_ext: depth_params ", depth.sizes(),
                    " and image_feats ", feats.sizes(), " disagree in dimension ", d);
    TORCH_CHECK(depth.scalar_type() == feats.scalar_type(),
                "flashbevpool_ext: depth_params and image_feats must share a dtype");
    TORCH_CHECK(proj.scalar_type() == at::kFloat, "flashbevpool_ext: projection_matrices must be float32");
    TORCH_CHECK(proj.dim() == 4 && proj.size(0) == depth.size(0) && proj.size(1) == depth.size(1) &&
                    (proj.size(2) == 3 || proj.size(2) == 4) && proj.size(3) == 4,
                "flashbevpool_ext: projection_matrices must be [B,N,3,4] or [B,N,4,4], got ", proj.sizes());
    TORCH_CHECK(depth_distribution >= 0 && depth_distribution <= 2,
                "flashbevpool_ext: depth_distribution must be 0 (gaussian), 1 (laplace) or 2 (categorical), got ",
                depth_distribution);
    if (depth_distribution != FBEV_CATEGORICAL)
        TORCH_CHECK(depth.size(4) == 2, "flashbevpool_ext: depth_params must be [B,N,H,W,2] (mean, sigma), got ",
                    depth.sizes());

    fbev_problem p{};
    p.batch = (int32_t)depth.size(0);
    p.num_cams = (int32_t)depth.size(1);
    p.feat_h = (int32_t)depth.size(2);
    p.feat_w = (int32_t)depth.size(3);
    p.channels = (int32_t)feats.size(4);
    p.depth_bins = (int32_t)depth.size(4);
    p.in_dtype = dtype_code(feats, "image_feats");

    // feature_size [B,N,2] must repeat (H, W) of the feature tensor for every camera.  The reference
    // kernel reads it per camera (flash_bevpool_cuda.cu:134-135); valid sizes smaller than a padded
    // tensor are not supported here, so it is always checked (a device tensor costs one synchronous
    // copy, like the reference's read of grid_size; the Python operator passes a host table).
    TORCH_CHECK(feature_size.numel() == (int64_t)p.batch * p.num_cams * 2,
                "flashbevpool_ext: feature_size must be [B,N,2], got ", feature_size.sizes());
    {
        auto fs = host_ints(feature_size, feature_size.numel(), "feature_size");
        for (size_t i = 0; i < fs.size(); i += 2)
            TORCH_CHECK(fs[i] == p.feat_h && fs[i + 1] == p.feat_w, "flashbevpool_ext: feature_size entry (",
                        fs[i], ",", fs[i + 1], ") differs from the feature tensor's (", p.feat_h, ",", p.feat_w,
                        "); per-camera valid sizes are not supported");
    }
    auto im = host_ints(image_size, 2, "image_size");
    auto gs = host_ints(grid_size, 3, "grid_size");
    TORCH_CHECK(im[0] > 0 && im[1] > 0, "flashbevpool_ext: image_size must be positive");
    TORCH_CHECK(gs[0] > 0 && gs[1] > 0 && gs[2] > 0, "flashbevpool_ext: grid_size must be positive");
    p.image_h = (int32_t)im[0];
    p.image_w = (int32_t)im[1];
    p.grid_x = (int32_t)gs[0];
    p.grid_y = (int32_t)gs[1];
    p.grid_z = (int32_t)gs[2];
    p.epsilon = epsilon;
    p.depth_weight_threshold = threshold;
    p.depth_distribution = depth_distribution;
    p.depth_min = depth_min;
    p.depth_step = depth_step;
    p.reduction = reduction;
    p.proj_stride = (int32_t)(proj.size(2) * 4);
    return p;
}

void raise_on(int rc, const char *what) {
    TORCH_CHECK(rc == FBEV_OK, "flashbevpool_ext: ", what, " failed: ", fbev_status_string(rc), " (", rc, ")");
}

}  // namespace

// Same positional order as the reference's flash_bevpool_forward
// (flashbev/flashbevpool/src/flash_bevpool.cpp:79-101).  The four kernel-variant booleans
// select nothing here (one kernel serves all); the trailing arguments are extensions.  The six voxel
// scalars are float64 (the reference takes them as float): cell centres are evaluated in float64.
void flash_bevpool_forward(const at::Tensor &depth_params, const at::Tensor &image_feats,
                           const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                           const at::Tensor &image_size, const at::Tensor &grid_size, double voxel_size_x,
                           double voxel_size_y, double voxel_size_z, double voxel_x_min, double voxel_y_min,
                           double voxel_z_min, at::Tensor out, int64_t total_threads, int depth_distribution,
                           bool use_shared_memory, bool optimize_z_precompute, bool use_warp_kernel,
                           bool use_vectorized_load, float epsilon, float depth_weight_threshold,
                           float depth_min, float depth_step, int reduction, std::optional<at::Tensor> count_out,
                           std::optional<at::Tensor> geometry_cache, std::optional<at::Tensor> sample_store) {
    (void)use_shared_memory; (void)optimize_z_precompute; (void)use_warp_kernel; (void)use_vectorized_load;
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, epsilon, depth_weight_threshold, depth_min, depth_step, reduction);
    p.voxel_min[0] = voxel_x_min; p.voxel_min[1] = voxel_y_min; p.voxel_min[2] = voxel_z_min;
    p.voxel_size[0] = voxel_size_x; p.voxel_size[1] = voxel_size_y; p.voxel_size[2] = voxel_size_z;
    check_dev(out, depth_params, "out");
    TORCH_CHECK(out.scalar_type() == at::kFloat, "flashbevpool_ext: out must be float32");
    TORCH_CHECK(out.dim() == 4 && out.size(0) == p.batch && out.size(1) == p.grid_y && out.size(2) == p.grid_x &&
                    out.size(3) == p.channels,
                "flashbevpool_ext: out must be [B,grid_y,grid_x,C] = [", p.batch, ",", p.grid_y, ",", p.grid_x, ",",
                p.channels, "], got ", out.sizes());
    TORCH_CHECK(total_threads == out.numel(), "flashbevpool_ext: total_threads (", total_threads,
                ") must equal out.numel() (", out.numel(), ")");
    float *cnt = nullptr;
    if (count_out.has_value() && count_out->defined()) {
        check_dev(*count_out, depth_params, "count_out");
        TORCH_CHECK(count_out->scalar_type() == at::kFloat && count_out->numel() == (int64_t)p.batch * p.grid_y * p.grid_x,
                    "flashbevpool_ext: count_out must be float32 [B,grid_y,grid_x]");
        cnt = count_out->data_ptr<float>();
    }
    DeviceScope scope(depth_params.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(depth_params.get_device()).stream();
    if (geometry_cache.has_value() && geometry_cache->defined()) {
        // lists built by build_geometry_cache for these matrices and this grid: same result, less work
        check_dev(*geometry_cache, depth_params, "geometry_cache");
        TORCH_CHECK(geometry_cache->scalar_type() == at::kByte, "flashbevpool_ext: geometry_cache must be a uint8 tensor");
        raise_on(fbev_forward_cached(&p, depth_params.data_ptr(), image_feats.data_ptr(), geometry_cache->data_ptr(),
                                     (size_t)geometry_cache->numel(), out.data_ptr<float>(), cnt, st),
                 "fbev_forward_cached");
        return;
    }
    if (sample_store.has_value() && sample_store->defined()) {
        // a forward that will be differentiated: the kept samples' records stay behind for flash_bevpool_backward
        check_dev(*sample_store, depth_params, "sample_store");
        TORCH_CHECK(sample_store->scalar_type() == at::kByte, "flashbevpool_ext: sample_store must be a uint8 tensor");
        TORCH_CHECK(cnt != nullptr, "flashbevpool_ext: sample_store needs count_out");
        raise_on(fbev_forward_store(&p, depth_params.data_ptr(), image_feats.data_ptr(), projection_matrices.data_ptr<float>(),
                                    out.data_ptr<float>(), cnt, sample_store->data_ptr(), (size_t)sample_store->numel(), st),
                 "fbev_forward_store");
        return;
    }
    raise_on(fbev_forward(&p, depth_params.data_ptr(), image_feats.data_ptr(), projection_matrices.data_ptr<float>(),
                          out.data_ptr<float>(), cnt, st),
             "fbev_forward");
}

// Bytes of the sample store flash_bevpool_forward(..., sample_store=...) fills for these tensors (0: none).
int64_t sample_store_bytes(const at::Tensor &depth_params, const at::Tensor &image_feats,
                           const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                           const at::Tensor &image_size, const at::Tensor &grid_size, int depth_distribution) {
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, 1e-6f, 0.0f, 1.0f, 1.0f, 0);
    return (int64_t)fbev_sample_store_bytes(&p);
}

// The per-cell lists of samples in view for these matrices and this grid (fbev_geometry_cache_build),
// as a uint8 tensor to hand to flash_bevpool_forward while calibration and grid stay the same.
at::Tensor build_geometry_cache(const at::Tensor &projection_matrices, int64_t feat_h, int64_t feat_w, int64_t image_h,
                                int64_t image_w, std::vector<int64_t> grid_size, std::vector<double> voxel_min,
                                std::vector<double> voxel_size, float epsilon) {
    TORCH_CHECK(projection_matrices.is_cuda() && projection_matrices.is_contiguous() &&
                    projection_matrices.scalar_type() == at::kFloat && projection_matrices.dim() == 4 &&
                    (projection_matrices.size(2) == 3 || projection_matrices.size(2) == 4) &&
                    projection_matrices.size(3) == 4,
                "flashbevpool_ext: projection_matrices must be a contiguous float32 GPU tensor [B,N,3|4,4]");
    TORCH_CHECK(grid_size.size() == 3 && voxel_min.size() == 3 && voxel_size.size() == 3,
                "flashbevpool_ext: grid_size, voxel_min and voxel_size need 3 entries each");
    fbev_problem p{};
    p.batch = (int32_t)projection_matrices.size(0);
    p.num_cams = (int32_t)projection_matrices.size(1);
    p.feat_h = (int32_t)feat_h; p.feat_w = (int32_t)feat_w;
    p.image_h = (int32_t)image_h; p.image_w = (int32_t)image_w;
    p.grid_x = (int32_t)grid_size[0]; p.grid_y = (int32_t)grid_size[1]; p.grid_z = (int32_t)grid_size[2];
    for (int a = 0; a < 3; ++a) { p.voxel_min[a] = voxel_min[a]; p.voxel_size[a] = voxel_size[a]; }
    p.epsilon = epsilon;
    p.channels = 1; p.depth_bins = 2;
    p.proj_stride = (int32_t)(projection_matrices.size(2) * 4);
    const size_t bytes = fbev_geometry_cache_bytes(&p);
    TORCH_CHECK(bytes > 0, "flashbevpool_ext: no geometry cache for this problem (sizes must be positive and "
                           "B*N*H*W below 2^29)");
    at::Tensor cache = at::empty({(int64_t)bytes}, projection_matrices.options().dtype(at::kByte));
    DeviceScope scope(projection_matrices.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(projection_matrices.get_device()).stream();
    raise_on(fbev_geometry_cache_build(&p, projection_matrices.data_ptr<float>(), cache.data_ptr(), bytes, st),
             "fbev_geometry_cache_build");
    return cache;
}

// Same positional order as the reference's flash_bevpool_backward
// (flashbev/flashbevpool/src/flash_bevpool.cpp:168-183).  Gradient buffers are float32 and
// zero-filled by the caller; an undefined (None) gradient tensor skips that gradient.
void flash_bevpool_backward(const at::Tensor &out_grad, const at::Tensor &depth_params, const at::Tensor &image_feats,
                            const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                            const at::Tensor &image_size, const at::Tensor &roi_range, const at::Tensor &grid_size,
                            std::optional<at::Tensor> depth_params_grad, std::optional<at::Tensor> image_feats_grad,
                            int64_t total_threads, int depth_distribution, float epsilon, float depth_weight_threshold,
                            float depth_min, float depth_step, int reduction, int backward_mode,
                            int64_t pair_capacity, std::optional<at::Tensor> cell_count, bool accumulate,
                            std::optional<at::Tensor> workspace, std::optional<at::Tensor> sample_store,
                            std::optional<std::vector<double>> voxel_size, int workspace_layout) {
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, epsilon, depth_weight_threshold, depth_min, depth_step, reduction);
    auto roi = host_floats(roi_range, 6, "roi_range");
    const int32_t g[3] = {p.grid_x, p.grid_y, p.grid_z};
    TORCH_CHECK(!voxel_size.has_value() || voxel_size->size() == 3, "flashbevpool_ext: voxel_size needs 3 entries");
    for (int a = 0; a < 3; ++a) {
        p.voxel_min[a] = (double)roi[2 * a];
        // The cell size must be the one the forward was given, or forward and backward would disagree on
        // samples that sit within rounding of a border.  A caller that names it (the Python operator passes the
        // float64 quotient of the fp32 bounds to both) is taken at its word.  The reference's 14 positional
        // arguments carry no size: its Python forms fp32((max - min) / grid) on the fp32 tensor and hands that
        // to the forward (flash_bevpool.py:62-64), so that is what an unnamed size means here.
        p.voxel_size[a] = voxel_size.has_value() ? (*voxel_size)[a]
                                                 : (double)((float)(roi[2 * a + 1] - roi[2 * a]) / (float)g[a]);
    }
    check_dev(out_grad, depth_params, "out_grad");
    TORCH_CHECK(out_grad.scalar_type() == at::kFloat, "flashbevpool_ext: out_grad must be float32");
    TORCH_CHECK(out_grad.dim() == 4 && out_grad.size(0) == p.batch && out_grad.size(1) == p.grid_y &&
                    out_grad.size(2) == p.grid_x && out_grad.size(3) == p.channels,
                "flashbevpool_ext: out_grad must be [B,grid_y,grid_x,C], got ", out_grad.sizes());
    TORCH_CHECK(total_threads == out_grad.numel(), "flashbevpool_ext: total_threads (", total_threads,
                ") must equal out_grad.numel() (", out_grad.numel(), ")");
    float *dd = nullptr, *df = nullptr;
    if (depth_params_grad.has_value() && depth_params_grad->defined()) {
        check_dev(*depth_params_grad, depth_params, "depth_params_grad");
        TORCH_CHECK(depth_params_grad->scalar_type() == at::kFloat && depth_params_grad->sizes() == depth_params.sizes(),
                    "flashbevpool_ext: depth_params_grad must be float32 with the shape of depth_params");
        dd = depth_params_grad->data_ptr<float>();
    }
    if (image_feats_grad.has_value() && image_feats_grad->defined()) {
        check_dev(*image_feats_grad, depth_params, "image_feats_grad");
        TORCH_CHECK(image_feats_grad->scalar_type() == at::kFloat && image_feats_grad->sizes() == image_feats.sizes(),
                    "flashbevpool_ext: image_feats_grad must be float32 with the shape of image_feats");
        df = image_feats_grad->data_ptr<float>();
    }
    DeviceScope scope(depth_params.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(depth_params.get_device()).stream();
    TORCH_CHECK(backward_mode >= 0 && backward_mode <= 3,
                "flashbevpool_ext: backward_mode must be 0 (auto), 1 (atomic scatter), 2 (inverse-map gather) or "
                "3 (column owner)");
    // the records and counts the forward left (flash_bevpool_forward(..., count_out, sample_store)), if any
    const float *stored_count = nullptr;
    const void *store = nullptr;
    size_t store_bytes = 0;
    if (sample_store.has_value() && sample_store->defined()) {
        check_dev(*sample_store, depth_params, "sample_store");
        TORCH_CHECK(sample_store->scalar_type() == at::kByte, "flashbevpool_ext: sample_store must be a uint8 tensor");
        TORCH_CHECK(cell_count.has_value() && cell_count->defined(), "flashbevpool_ext: sample_store needs cell_count");
        check_dev(*cell_count, depth_params, "cell_count");
        TORCH_CHECK(cell_count->scalar_type() == at::kFloat && cell_count->numel() == (int64_t)p.batch * p.grid_y * p.grid_x,
                    "flashbevpool_ext: cell_count must be float32 [B,grid_y,grid_x]");
        TORCH_CHECK(backward_mode == 0 || backward_mode == 2,
                    "flashbevpool_ext: a sample store goes with backward_mode 0 (auto) or 2 (gather)");
        stored_count = cell_count->data_ptr<float>();
        store = sample_store->data_ptr();
        store_bytes = (size_t)sample_store->numel();
    }
    auto run_columns = [&]() -> int {
        const float *cnt = nullptr;
        at::Tensor ws;
        size_t ws_bytes = 0;
        if (cell_count.has_value() && cell_count->defined()) {
            check_dev(*cell_count, depth_params, "cell_count");
            TORCH_CHECK(cell_count->scalar_type() == at::kFloat &&
                            cell_count->numel() == (int64_t)p.batch * p.grid_y * p.grid_x,
                        "flashbevpool_ext: cell_count must be float32 [B,grid_y,grid_x]");
            cnt = cell_count->data_ptr<float>();
        } else {
            ws_bytes = fbev_backward_columns_workspace_bytes(&p);
            ws = at::empty({(int64_t)ws_bytes}, at::TensorOptions().device(depth_params.device()).dtype(at::kByte));
        }
        return fbev_backward_columns(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                                     projection_matrices.data_ptr<float>(), cnt, dd, df, accumulate ? 1 : 0,
                                     ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, st);
    };
    // Inverse-map gather.  The pair array comes from PyTorch's caching allocator (no device
    // allocation in steady state).  By default it has room for every sample, which lets
    // the library use fixed per-texel segments and skip its counting pass; a smaller
    // pair_capacity selects the exactly packed layout (what does not fit is applied with atomics).
    auto run_gather = [&]() -> int {
        const uint64_t max_pairs = fbev_backward_max_pairs(&p);
        // pair positions and claim counters are 32-bit in the library: say so before any allocation
        // (what fbev_backward_gather itself would answer), so that "auto" can still take the column owner
        const uint64_t texels = (uint64_t)p.batch * p.num_cams * p.feat_h * p.feat_w;
        if (max_pairs == 0 || max_pairs >= (1ull << 31) || texels * 32 >= (1ull << 31)) return FBEV_ERR_TOO_LARGE;
        uint64_t cap = pair_capacity >= 0 ? (uint64_t)pair_capacity : max_pairs;
        if (cap > max_pairs) cap = max_pairs;
        const size_t bytes = fbev_backward_workspace_bytes(&p, cap);
        at::Tensor ws = at::empty({(int64_t)bytes}, at::TensorOptions().device(depth_params.device()).dtype(at::kByte));
        if (store != nullptr)
            return fbev_backward_gather_stored(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                                               projection_matrices.data_ptr<float>(), stored_count, store, store_bytes, dd, df,
                                               accumulate ? 1 : 0, ws.data_ptr(), bytes, 0, st);
        return fbev_backward_gather(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                                    projection_matrices.data_ptr<float>(), dd, df, accumulate ? 1 : 0, ws.data_ptr(),
                                    bytes, st);
    };
    if (workspace.has_value() && workspace->defined()) {
        // a workspace from prepare_backward_workspace: the inverse map in two launches, nothing allocated
        TORCH_CHECK(backward_mode == 0 || backward_mode == 2,
                    "flashbevpool_ext: a persistent workspace goes with backward_mode 0 (auto) or 2 (gather)");
        check_dev(*workspace, depth_params, "workspace");
        TORCH_CHECK(workspace->scalar_type() == at::kByte, "flashbevpool_ext: workspace must be a uint8 tensor");
        TORCH_CHECK(workspace_layout == 1 || workspace_layout == 2,
                    "flashbevpool_ext: workspace_layout must be 1 (segments of one capacity) or 2 (sized by the geometry)");
        if (store != nullptr)
            raise_on(fbev_backward_gather_stored(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                                                 projection_matrices.data_ptr<float>(), stored_count, store, store_bytes, dd, df,
                                                 accumulate ? 1 : 0, workspace->data_ptr(), (size_t)workspace->numel(),
                                                 workspace_layout, st),
                     "fbev_backward_gather_stored");
        else if (workspace_layout == 2)
            raise_on(fbev_backward_gather_sized(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                                                projection_matrices.data_ptr<float>(), dd, df, accumulate ? 1 : 0,
                                                workspace->data_ptr(), (size_t)workspace->numel(), st),
                     "fbev_backward_gather_sized");
        else
            raise_on(fbev_backward_gather_persistent(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(),
                                                     image_feats.data_ptr(), projection_matrices.data_ptr<float>(), dd, df,
                                                     accumulate ? 1 : 0, workspace->data_ptr(), (size_t)workspace->numel(), st),
                     "fbev_backward_gather_persistent");
    } else if (backward_mode == 1) {
        raise_on(fbev_backward(&p, out_grad.data_ptr<float>(), depth_params.data_ptr(), image_feats.data_ptr(),
                               projection_matrices.data_ptr<float>(), dd, df, accumulate ? 1 : 0, st),
                 "fbev_backward");
    } else if (backward_mode == 2) {
        raise_on(run_gather(), "fbev_backward_gather");
    } else if (backward_mode == 3) {
        raise_on(run_columns(), "fbev_backward_columns");
    } else {
        // auto: the inverse map; problems beyond its 32-bit pair positions go to the column owner
        int rc = run_gather();
        if (rc == FBEV_ERR_TOO_LARGE) raise_on(run_columns(), "fbev_backward_columns");
        else raise_on(rc, "fbev_backward_gather");
    }
}

// Bytes of a persistent inverse-map workspace for these tensors (0: the problem is beyond the
// inverse map's 32-bit positions), and a workspace allocated and prepared on the current stream.
int64_t backward_workspace_bytes(const at::Tensor &depth_params, const at::Tensor &image_feats,
                                 const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                                 const at::Tensor &image_size, const at::Tensor &grid_size, int depth_distribution) {
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, 1e-6f, 0.0f, 1.0f, 1.0f, 0);
    const uint64_t max_pairs = fbev_backward_max_pairs(&p);
    const uint64_t texels = (uint64_t)p.batch * p.num_cams * p.feat_h * p.feat_w;
    if (max_pairs == 0 || max_pairs >= (1ull << 31) || texels * 32 >= (1ull << 31)) return 0;
    return (int64_t)fbev_backward_persistent_workspace_bytes(&p);
}

// A persistent workspace whose segments are sized by the geometry (fbev_backward_workspace_init_sized): counted for
// these matrices, this grid, region of interest, image size and epsilon; one device-to-host copy (the number of
// samples in view) decides its size.  For flash_bevpool_backward(..., workspace_layout=2).
at::Tensor prepare_sized_backward_workspace(const at::Tensor &depth_params, const at::Tensor &image_feats,
                                            const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                                            const at::Tensor &image_size, const at::Tensor &grid_size,
                                            int depth_distribution, std::vector<double> voxel_min,
                                            std::vector<double> voxel_size, float epsilon) {
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, epsilon, 0.0f, 1.0f, 1.0f, 0);
    TORCH_CHECK(voxel_min.size() == 3 && voxel_size.size() == 3, "flashbevpool_ext: voxel_min and voxel_size need 3 entries each");
    for (int a = 0; a < 3; ++a) { p.voxel_min[a] = voxel_min[a]; p.voxel_size[a] = voxel_size[a]; }
    const size_t head = fbev_backward_sized_workspace_bytes(&p, 0), at_total = fbev_backward_sized_total_offset(&p);
    TORCH_CHECK(head > 0 && at_total + sizeof(int32_t) <= head, "flashbevpool_ext: no sized workspace for this problem");
    auto bytes_on = at::TensorOptions().device(depth_params.device()).dtype(at::kByte);
    at::Tensor tables = at::empty({(int64_t)head}, bytes_on);
    DeviceScope scope(depth_params.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(depth_params.get_device()).stream();
    raise_on(fbev_backward_workspace_init_sized(&p, projection_matrices.data_ptr<float>(), tables.data_ptr(), head, st),
             "fbev_backward_workspace_init_sized");
    const int64_t total = tables.narrow(0, (int64_t)at_total, 4).view(at::kInt).item<int32_t>();
    TORCH_CHECK(total >= 0, "flashbevpool_ext: sized workspace: negative sample count");
    at::Tensor ws = at::empty({(int64_t)fbev_backward_sized_workspace_bytes(&p, (uint64_t)total)}, bytes_on);
    ws.narrow(0, 0, (int64_t)head).copy_(tables);      // what lies in front of the pairs does not depend on their number
    return ws;
}

at::Tensor prepare_backward_workspace(const at::Tensor &depth_params, const at::Tensor &image_feats,
                                      const at::Tensor &projection_matrices, const at::Tensor &feature_size,
                                      const at::Tensor &image_size, const at::Tensor &grid_size,
                                      int depth_distribution) {
    fbev_problem p = describe(depth_params, image_feats, projection_matrices, feature_size, image_size, grid_size,
                              depth_distribution, 1e-6f, 0.0f, 1.0f, 1.0f, 0);
    const size_t bytes = fbev_backward_persistent_workspace_bytes(&p);
    TORCH_CHECK(bytes > 0, "flashbevpool_ext: no persistent workspace for this problem");
    at::Tensor ws = at::empty({(int64_t)bytes}, at::TensorOptions().device(depth_params.device()).dtype(at::kByte));
    DeviceScope scope(depth_params.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(depth_params.get_device()).stream();
    raise_on(fbev_backward_workspace_init(&p, ws.data_ptr(), bytes, st), "fbev_backward_workspace_init");
    return ws;
}

// Parity hook: per-sample validity mask and bilinear corner indices, [B,gy,gx,N,gz(,4|2)].
std::vector<at::Tensor> sample_geometry(const at::Tensor &projection_matrices, int64_t feat_h, int64_t feat_w,
                                        int64_t image_h, int64_t image_w, std::vector<int64_t> grid_size,
                                        std::vector<double> voxel_min, std::vector<double> voxel_size, float epsilon) {
    TORCH_CHECK(projection_matrices.is_cuda() && projection_matrices.is_contiguous() &&
                    projection_matrices.scalar_type() == at::kFloat && projection_matrices.dim() == 4 &&
                    (projection_matrices.size(2) == 3 || projection_matrices.size(2) == 4) &&
                    projection_matrices.size(3) == 4,
                "flashbevpool_ext: projection_matrices must be a contiguous float32 GPU tensor [B,N,3|4,4]");
    TORCH_CHECK(grid_size.size() == 3 && voxel_min.size() == 3 && voxel_size.size() == 3,
                "flashbevpool_ext: grid_size, voxel_min and voxel_size need 3 entries each");
    fbev_problem p{};
    p.batch = (int32_t)projection_matrices.size(0);
    p.num_cams = (int32_t)projection_matrices.size(1);
    p.feat_h = (int32_t)feat_h; p.feat_w = (int32_t)feat_w;
    p.image_h = (int32_t)image_h; p.image_w = (int32_t)image_w;
    p.grid_x = (int32_t)grid_size[0]; p.grid_y = (int32_t)grid_size[1]; p.grid_z = (int32_t)grid_size[2];
    for (int a = 0; a < 3; ++a) { p.voxel_min[a] = voxel_min[a]; p.voxel_size[a] = voxel_size[a]; }
    p.epsilon = epsilon;
    p.channels = 1; p.depth_bins = 2;
    p.proj_stride = (int32_t)(projection_matrices.size(2) * 4);
    TORCH_CHECK(p.grid_x > 0 && p.grid_y > 0 && p.grid_z > 0, "flashbevpool_ext: grid_size must be positive");
    auto dev = projection_matrices.device();
    std::vector<int64_t> shp = {p.batch, p.grid_y, p.grid_x, p.num_cams, p.grid_z};
    at::Tensor mask = at::empty(shp, at::TensorOptions().device(dev).dtype(at::kByte));
    shp.push_back(4);
    at::Tensor idx = at::empty(shp, at::TensorOptions().device(dev).dtype(at::kInt));
    shp.back() = 2;
    at::Tensor frac = at::empty(shp, at::TensorOptions().device(dev).dtype(at::kFloat));
    DeviceScope scope(projection_matrices.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(projection_matrices.get_device()).stream();
    raise_on(fbev_sample_geometry(&p, projection_matrices.data_ptr<float>(), mask.data_ptr<uint8_t>(),
                                  idx.data_ptr<int32_t>(), frac.data_ptr<float>(), st),
             "fbev_sample_geometry");
    return {mask, idx, frac};
}

// create_projection_matrix of the reference's module (flashbev/flashbevpool/sampling_vt.py:21-33) as one launch.
at::Tensor create_projection_matrix(const at::Tensor &sensor2ego, const at::Tensor &camera2imgs,
                                    const at::Tensor &post_rots, const at::Tensor &post_trans) {
    TORCH_CHECK(camera2imgs.is_cuda() && camera2imgs.dim() == 4 && camera2imgs.size(2) == 3 && camera2imgs.size(3) == 3,
                "create_projection_matrix: camera2imgs must be a GPU tensor [B,N,3,3], got ", camera2imgs.sizes());
    const int64_t B = camera2imgs.size(0), N = camera2imgs.size(1);
    TORCH_CHECK(sensor2ego.sizes() == at::IntArrayRef({B, N, 4, 4}), "create_projection_matrix: sensor2ego must be [B,N,4,4], got ",
                sensor2ego.sizes());
    TORCH_CHECK(post_rots.sizes() == at::IntArrayRef({B, N, 3, 3}), "create_projection_matrix: post_rots must be [B,N,3,3], got ",
                post_rots.sizes());
    TORCH_CHECK(post_trans.sizes() == at::IntArrayRef({B, N, 3}), "create_projection_matrix: post_trans must be [B,N,3], got ",
                post_trans.sizes());
    for (const at::Tensor *t : {&sensor2ego, &post_rots, &post_trans}) check_dev(*t, camera2imgs, "a calibration tensor");
    TORCH_CHECK(B * N < (1ll << 31), "create_projection_matrix: too many cameras");
    auto f32 = [](const at::Tensor &t) { return t.to(at::kFloat).contiguous(); };
    const at::Tensor e = f32(sensor2ego), k = f32(camera2imgs), r = f32(post_rots), t = f32(post_trans);
    at::Tensor proj = at::empty({B, N, 3, 4}, camera2imgs.options().dtype(at::kFloat));
    DeviceScope scope(camera2imgs.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(camera2imgs.get_device()).stream();
    raise_on(fbev_projection_matrices(e.data_ptr<float>(), k.data_ptr<float>(), r.data_ptr<float>(), t.data_ptr<float>(),
                                      proj.data_ptr<float>(), (int32_t)(B * N), st),
             "fbev_projection_matrices");
    return proj;
}

// Same positional order as the reference's sampling_vt_pillarpool_fused_forward
// (flashbev/flashbevpool/src/sampling_vt.cpp:13-52): note interval_lengths before
// interval_starts.  All tensors on one device, contiguous; float32 / int32 as in the reference.
void sampling_vt_pillarpool_fused_forward(const at::Tensor &depth, const at::Tensor &feat, const at::Tensor &u_coords,
                                          const at::Tensor &v_coords, const at::Tensor &z_coords,
                                          const at::Tensor &batch_camera_indices, const at::Tensor &ranks_bev,
                                          const at::Tensor &interval_lengths, const at::Tensor &interval_starts,
                                          at::Tensor out, int batch_size, int num_cameras, int feat_h, int feat_w,
                                          float epsilon, int depth_distribution) {
    TORCH_CHECK(feat.is_cuda(), "sampling_vt_pillarpool_fused_forward: feat must be on a ROCm GPU");
    const at::Tensor *all[] = {&depth, &u_coords, &v_coords, &z_coords, &batch_camera_indices, &ranks_bev,
                               &interval_lengths, &interval_starts, &out};
    for (const at::Tensor *t : all) check_dev(*t, feat, "an argument");
    for (const at::Tensor *t : {&depth, &feat, &u_coords, &v_coords, &z_coords, (const at::Tensor *)&out})
        TORCH_CHECK(t->scalar_type() == at::kFloat && t->is_contiguous(),
                    "sampling_vt_pillarpool_fused_forward: float tensors must be contiguous float32");
    for (const at::Tensor *t : {&batch_camera_indices, &ranks_bev, &interval_lengths, &interval_starts})
        TORCH_CHECK(t->scalar_type() == at::kInt && t->is_contiguous(),
                    "sampling_vt_pillarpool_fused_forward: index tensors must be contiguous int32");
    TORCH_CHECK(feat.dim() == 5 && feat.size(0) == batch_size && feat.size(1) == num_cameras && feat.size(2) == feat_h &&
                    feat.size(3) == feat_w,
                "sampling_vt_pillarpool_fused_forward: feat must be [B,N,H,W,C], got ", feat.sizes());
    TORCH_CHECK(depth.numel() == (int64_t)batch_size * num_cameras * feat_h * feat_w * 2,
                "sampling_vt_pillarpool_fused_forward: depth must be [B,N,H,W,2], got ", depth.sizes());
    const int64_t n = u_coords.numel();
    TORCH_CHECK(v_coords.numel() == n && z_coords.numel() == n && batch_camera_indices.numel() == n &&
                    ranks_bev.numel() == n,
                "sampling_vt_pillarpool_fused_forward: per-sample tensors must have the same length");
    TORCH_CHECK(interval_starts.numel() == interval_lengths.numel(),
                "sampling_vt_pillarpool_fused_forward: interval_starts and interval_lengths differ in length");
    TORCH_CHECK(out.size(-1) == feat.size(4), "sampling_vt_pillarpool_fused_forward: out's last dimension must be C");
    fbev_pillar_problem p = {};
    p.channels = (int32_t)feat.size(4);
    p.n_intervals = (int32_t)interval_lengths.numel();
    p.batch = batch_size; p.num_cams = num_cameras; p.feat_h = feat_h; p.feat_w = feat_w;
    p.epsilon = epsilon; p.depth_distribution = depth_distribution;
    DeviceScope scope(feat.get_device());
    hipStream_t st = c10::hip::getCurrentHIPStream(feat.get_device()).stream();
    raise_on(fbev_pillarpool_forward(&p, depth.data_ptr<float>(), feat.data_ptr<float>(), u_coords.data_ptr<float>(),
                                     v_coords.data_ptr<float>(), z_coords.data_ptr<float>(),
                                     batch_camera_indices.data_ptr<int>(), ranks_bev.data_ptr<int>(),
                                     interval_starts.data_ptr<int>(), interval_lengths.data_ptr<int>(),
                                     out.data_ptr<float>(), st),
             "fbev_pillarpool_forward");
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    namespace py = pybind11;
    m.def("flash_bevpool_forward", &flash_bevpool_forward, "fused camera->BEV pooling, forward",
          py::arg("depth_params"), py::arg("image_feats"), py::arg("projection_matrices"), py::arg("feature_size"),
          py::arg("image_size"), py::arg("grid_size"), py::arg("voxel_size_x"), py::arg("voxel_size_y"),
          py::arg("voxel_size_z"), py::arg("voxel_x_min"), py::arg("voxel_y_min"), py::arg("voxel_z_min"),
          py::arg("out"), py::arg("total_threads"), py::arg("depth_distribution"), py::arg("use_shared_memory"),
          py::arg("optimize_z_precompute"), py::arg("use_warp_kernel"), py::arg("use_vectorized_load"),
          py::arg("epsilon") = 1e-6f, py::arg("depth_weight_threshold") = 1e-6f, py::arg("depth_min") = 1.0f,
          py::arg("depth_step") = 1.0f, py::arg("reduction") = 0, py::arg("count_out") = py::none(),
          py::arg("geometry_cache") = py::none(), py::arg("sample_store") = py::none());
    m.def("sample_store_bytes", &sample_store_bytes,
          "bytes of the sample store a differentiated forward may fill for the backward (0: none for this problem)");
    m.def("build_geometry_cache", &build_geometry_cache,
          "per-cell lists of the samples in view, for flash_bevpool_forward(..., geometry_cache=...)",
          py::arg("projection_matrices"), py::arg("feat_h"), py::arg("feat_w"), py::arg("image_h"), py::arg("image_w"),
          py::arg("grid_size"), py::arg("voxel_min"), py::arg("voxel_size"), py::arg("epsilon") = 1e-6f);
    m.def("flash_bevpool_backward", &flash_bevpool_backward, "fused camera->BEV pooling, backward",
          py::arg("out_grad"), py::arg("depth_params"), py::arg("image_feats"), py::arg("projection_matrices"),
          py::arg("feature_size"), py::arg("image_size"), py::arg("roi_range"), py::arg("grid_size"),
          py::arg("depth_params_grad"), py::arg("image_feats_grad"), py::arg("total_threads"),
          py::arg("depth_distribution"), py::arg("epsilon") = 1e-6f, py::arg("depth_weight_threshold") = 1e-6f,
          py::arg("depth_min") = 1.0f, py::arg("depth_step") = 1.0f, py::arg("reduction") = 0,
          py::arg("backward_mode") = 0, py::arg("pair_capacity") = -1, py::arg("cell_count") = py::none(),
          py::arg("accumulate") = true, py::arg("workspace") = py::none(), py::arg("sample_store") = py::none(),
          py::arg("voxel_size") = py::none(), py::arg("workspace_layout") = 1);
    m.def("backward_workspace_bytes", &backward_workspace_bytes,
          "bytes of a persistent inverse-map workspace (0 when the problem is beyond the inverse map)");
    m.def("prepare_backward_workspace", &prepare_backward_workspace,
          "a persistent inverse-map workspace, allocated and prepared on the current stream");
    m.def("prepare_sized_backward_workspace", &prepare_sized_backward_workspace,
          "a persistent inverse-map workspace with segments sized by the geometry, prepared on the current stream",
          py::arg("depth_params"), py::arg("image_feats"), py::arg("projection_matrices"), py::arg("feature_size"),
          py::arg("image_size"), py::arg("grid_size"), py::arg("depth_distribution"), py::arg("voxel_min"),
          py::arg("voxel_size"), py::arg("epsilon") = 1e-6f);
    m.def("sample_geometry", &sample_geometry, "per-sample validity mask and corner indices (parity hook)",
          py::arg("projection_matrices"), py::arg("feat_h"), py::arg("feat_w"), py::arg("image_h"), py::arg("image_w"),
          py::arg("grid_size"), py::arg("voxel_min"), py::arg("voxel_size"), py::arg("epsilon") = 1e-6f);
    m.def("sampling_vt_pillarpool_fused_forward", &sampling_vt_pillarpool_fused_forward,
          "interval pooling over precomputed sample lists (the reference's PillarPool baseline)");
    m.def("create_projection_matrix", &create_projection_matrix,
          "[B,N,3,4] projection matrices from sensor2ego, camera2imgs, post_rots, post_trans", py::arg("sensor2ego"),
          py::arg("camera2imgs"), py::arg("post_rots"), py::arg("post_trans"));
    m.def("abi_version", []() { return fbev_abi_version(); });
}
