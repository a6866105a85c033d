/*
 * flashbev_hip.h -- C ABI of libflashbev_hip.so: fused camera->BEV pooling for gfx950.
 *
 * Plain pointers and sizes only; no torch types.  All data pointers are DEVICE pointers
 * valid on the device that is current when the call is made; `stream` is a hipStream_t
 * passed as void* (NULL = the null stream).  Every call is asynchronous with respect to
 * the host and allocates nothing.  Return value: FBEV_OK or a negative fbev_status.
 *
 * Tensor layouts (all dense, row-major, innermost index last):
 *   feats  [B, N, H, W, C]   fp32 / fp16 / bf16 (in_dtype), channels last
 *   depth  [B, N, H, W, Dd]  same dtype as feats; Dd = 2 (mean, sigma) for the Gaussian /
 *                            Laplace models, Dd = depth_bins for the categorical model
 *   proj   [B, N, proj_stride] fp32; the first 12 floats of each block are a row-major
 *                            3x4 projection matrix (proj_stride = 12 for [B,N,3,4],
 *                            16 for [B,N,4,4])
 *   out / grad_out [B, grid_y, grid_x, C] fp32
 *   d_feats [B, N, H, W, C] fp32,  d_depth [B, N, H, W, Dd] fp32
 */
#ifndef FLASHBEV_HIP_H
#define FLASHBEV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FBEV_ABI_VERSION 9

typedef enum fbev_status {
    FBEV_OK = 0,
    FBEV_ERR_NULL = -1,        /* a required pointer is NULL */
    FBEV_ERR_SHAPE = -2,       /* a size is <= 0 or inconsistent */
    FBEV_ERR_UNSUPPORTED = -3, /* unknown dtype / depth model / reduction */
    FBEV_ERR_TOO_LARGE = -4,   /* an element count does not fit the 32-bit indices used */
    FBEV_ERR_ALIGNMENT = -5,   /* a pointer is not aligned to its element type */
    FBEV_ERR_LAUNCH = -6       /* the HIP runtime reported a launch error */
} fbev_status;

enum { FBEV_F32 = 0, FBEV_F16 = 1, FBEV_BF16 = 2 };
enum { FBEV_GAUSSIAN = 0, FBEV_LAPLACE = 1, FBEV_CATEGORICAL = 2 };
enum { FBEV_REDUCE_MEAN = 0, FBEV_REDUCE_SUM = 1 };

/*
 * Problem description.  It gathers, by value, what the reference passes as scalars and
 * small tensors to flash_bevpool_forward / flash_bevpool_backward
 * (flashbev/flashbevpool/src/flash_bevpool.cpp:79-101,168-183).
 */
typedef struct fbev_problem {
    int32_t batch;       /* B */
    int32_t num_cams;    /* N */
    int32_t feat_h;      /* H: rows of every camera's feature map */
    int32_t feat_w;      /* W */
    int32_t channels;    /* C */
    int32_t image_h;     /* Hi: image rows the projection matrices refer to */
    int32_t image_w;     /* Wi */
    int32_t grid_x;      /* BEV cells along x */
    int32_t grid_y;
    int32_t grid_z;      /* height bins reduced per cell */
    double voxel_min[3];  /* lower edge of the region of interest along x, y, z (the reference's
                             voxel_x_min .. voxel_z_min, flash_bevpool.py:65-67, widened) */
    double voxel_size[3]; /* cell size along x, y, z: (max - min) / grid in float64 (the reference's
                             voxel_size_x .. voxel_size_z, flash_bevpool.py:62-64, widened).  Cell i has
                             its centre at fp32(min + (i + 0.5) * size), evaluated in float64 and
                             rounded once: the correctly rounded centre, within an ulp of the dense
                             path's linspace(min, max, grid + 1)[:-1] + size / 2
                             (sampling_vt.py:364-378).  An fp32 size would carry its rounding error
                             i times along the axis. */
    float epsilon;       /* added to sigma; lower clamp of the perspective divisor */
    float depth_weight_threshold; /* samples with weight < threshold are dropped */
    int32_t depth_distribution;   /* FBEV_GAUSSIAN / FBEV_LAPLACE / FBEV_CATEGORICAL */
    int32_t depth_bins;  /* Dd: 2 for the parametric models */
    float depth_min;     /* categorical: depth of bin 0 */
    float depth_step;    /* categorical: spacing of the bins */
    int32_t in_dtype;    /* FBEV_F32 / FBEV_F16 / FBEV_BF16 for feats and depth */
    int32_t reduction;   /* FBEV_REDUCE_MEAN (the reference's) / FBEV_REDUCE_SUM */
    int32_t proj_stride; /* 12 or 16 */
} fbev_problem;

/*
 * Forward: out[b,y,x,:] = mean (or sum) over the valid (camera, height-bin) samples of
 * depth_weight * bilinear(feats).  Every element of `out` is written (cells that no
 * camera sees get 0), so `out` need not be zeroed.  If `count_out` is not NULL it receives,
 * as float [B, grid_y, grid_x], the number of samples that entered each cell's mean (what the
 * reference keeps in `valid_count`, flash_bevpool_cuda.cu:198-216); fbev_backward_columns can
 * reuse it.
 * Replaces the launcher flash_bevpool(...) (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:757-865)
 * as bound by flash_bevpool_forward (flashbev/flashbevpool/src/flash_bevpool.cpp:79-166).
 */
int fbev_forward(const fbev_problem *p, const void *depth, const void *feats, const float *proj,
                 float *out, float *count_out, void *stream);

/*
 * Forward on cached geometry.  Which samples are in view, and their bilinear corners and fractions,
 * depend only on the projection matrices, the feature-map and image sizes and the grid: when those
 * repeat from call to call (a fixed rig at inference) the lists can be built once and every later
 * forward starts from them, skipping the column cull, the projection and its divisions (about a
 * third of the forward at the large configurations).  The cache is caller-owned device memory of
 * fbev_geometry_cache_bytes(p) bytes (0: outside the limits, B*N*H*W >= 2^29), 16-byte aligned:
 * per BEV cell the number of samples in view and up to N * grid_z 16-byte records (du, dv, first
 * corner texel with the two clamp flags, depth along the optical axis), i.e.
 * B * ceil(gx/8) * ceil(gy/8) * 64 * (4 + 16 * N * grid_z) bytes.  fbev_geometry_cache_build fills it
 * (p->channels, in_dtype and the depth fields are ignored); fbev_forward_cached is fbev_forward with
 * the cache in place of the matrices and gives the same result bit for bit.  The caller rebuilds
 * the cache whenever proj, the sizes, the grid, the region of interest or epsilon change.  The cache
 * records the sizes and a hash of image size, region of interest, cell size and epsilon; the kernel of
 * fbev_forward_cached compares them with its own problem and, when they differ (or the memory is no
 * cache at all), reads none of it and fills out and count_out with NaN: the call still returns
 * FBEV_OK, since the host never reads device memory.  A change of proj alone cannot be seen.  The optional cached workspace keyed by geometry has no counterpart in the reference,
 * which recomputes the projection per channel thread (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:102-159).
 */
size_t fbev_geometry_cache_bytes(const fbev_problem *p);
int fbev_geometry_cache_build(const fbev_problem *p, const float *proj, void *cache, size_t cache_bytes,
                              void *stream);
int fbev_forward_cached(const fbev_problem *p, const void *depth, const void *feats, const void *cache,
                        size_t cache_bytes, float *out, float *count_out, void *stream);

/*
 * Backward: the exact gradients of fbev_forward.  With accumulate != 0 they are ADDED to
 * d_depth and d_feats, which the caller has zero-filled (the reference's ownership rule,
 * flashbev/flashbevpool/flash_bevpool.py:115-116); with accumulate == 0 the library defines
 * every element itself (the zero-fill is folded into its first launch) and the buffers may
 * hold anything.  Either gradient pointer may be NULL to skip that gradient.
 * Replaces flash_bevpool_grad(...) (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:867-937) as bound by
 * flash_bevpool_backward (flashbev/flashbevpool/src/flash_bevpool.cpp:168-241).  The depth gradient is
 * the true derivative of the forward, not the reference kernel's expression at
 * flash_bevpool_cuda.cu:665-674.
 */
int fbev_backward(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                  const float *proj, float *d_depth, float *d_feats, int accumulate, void *stream);

/*
 * Backward through an inverse map (texel -> contributing samples): the same gradients as
 * fbev_backward, formed without floating-point atomics on the feature gradient.  The cell
 * pass writes one 32-byte record ("pair": cell, coefficient, bilinear fractions, depth-gradient
 * terms) per kept sample into the workspace segment of the sample's first corner texel; the
 * texel pass of a texel gathers from the segments of the four texels whose samples reach it.
 * `accumulate` as in fbev_backward.
 * `workspace` is caller-owned device memory, 16-byte aligned, of at least
 * fbev_backward_workspace_bytes(p, 0) bytes, and carries no state between calls.  Its pair
 * capacity selects the layout:
 *   - room for fbev_backward_max_pairs(p) pairs or more: every texel owns fixed segments
 *     (capacity / texels pair slots, in four replicas) and the call is three launches;
 *   - anything smaller: the call first counts the samples per first-corner texel and prefix-sums
 *     the counts, so that the pairs are packed exactly (two more passes over the samples).
 * Pairs that find no room (a full segment, or a packed array shorter than the number of
 * pairs) are applied with atomics instead, so any capacity gives correct results.
 * It is the deterministic-gather alternative to the atomic scatter of
 * flash_bevpool_grad_kernel (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:570-681); the sorted
 * (cell -> sample) intervals of flashbev/flashbevpool/sampling_vt.py:296-311 are the same idea
 * applied to the forward pass.
 */
int fbev_backward_gather(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                         const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                         size_t workspace_bytes, void *stream);

/*
 * fbev_backward_gather on a workspace that persists between calls: two launches (cell pass, texel
 * pass) instead of three, because nothing has to be cleared at the start of a call.  The workspace
 * holds two sets of claim counters (a call claims in one, its texel pass clears the other for the
 * next call; a call counter kept in the workspace selects the set, so a call captured into a HIP
 * graph can be replayed) and gradient buffers of its own for what the cell pass cannot file under
 * a texel (a full segment), which the texel pass takes over and clears again.  Every element of
 * d_depth and d_feats is stored (accumulate == 0) or added to (accumulate != 0) by the texel pass.
 * Contract: `workspace` has at least fbev_backward_persistent_workspace_bytes(p) bytes (room for
 * every sample: fixed segments), is 16-byte aligned, was prepared by fbev_backward_workspace_init
 * for the same p once (again whenever batch, cameras, feature-map size, channels or depth bins
 * change, or after anything else wrote to it), and is used by one call at a time (calls on one
 * stream are ordered; calls that overlap in time race).  A call that fails, or is not followed by
 * its own completion, leaves the workspace undefined: prepare it again.  Same results as
 * fbev_backward_gather.  No counterpart in the reference, whose backward allocates nothing and
 * scatters with atomics (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:867-937).
 */
size_t fbev_backward_persistent_workspace_bytes(const fbev_problem *p);
int fbev_backward_workspace_init(const fbev_problem *p, void *workspace, size_t workspace_bytes, void *stream);
int fbev_backward_gather_persistent(const fbev_problem *p, const float *grad_out, const void *depth,
                                    const void *feats, const float *proj, float *d_depth, float *d_feats,
                                    int accumulate, void *workspace, size_t workspace_bytes, void *stream);

/*
 * A persistent workspace whose segments are sized by the geometry.  fbev_backward_gather_persistent keeps room for
 * every (cell, camera, height) sample, in segments of one common capacity: 32 bytes x B x gy x gx x N x gz
 * (0.98 GB for 8 x 200 x 200 cells x 6 cameras x 16 bins) of which a call fills under a tenth, because only one
 * sample in six is in view and the texels on the horizon collect ten times the average.  Which samples are in view
 * depends on the projection matrices and the grid only, so a workspace prepared for one set of matrices can give
 * each (texel, replica) segment exactly the room its samples in view need:
 *   fbev_backward_workspace_init_sized   zero-fills everything but the pairs, counts the samples in view per
 *       segment and prefix-sums the counts (one pass over the samples, once); `workspace` needs at least
 *       fbev_backward_sized_workspace_bytes(p, 0) bytes for that.  The total number of pairs the segments hold is
 *       then the int32 at byte offset fbev_backward_sized_total_offset(p) of the workspace: the caller reads it
 *       (the one device-to-host copy of this interface), allocates fbev_backward_sized_workspace_bytes(p, total)
 *       bytes and either prepares that memory the same way or copies the first
 *       fbev_backward_sized_workspace_bytes(p, 0) bytes over: what lies in front of the pairs does not depend on
 *       their number.
 *   fbev_backward_gather_sized   is fbev_backward_gather_persistent on such a workspace: two launches, same
 *       results, same contract (one call at a time, prepared again after a failed call or a change of batch,
 *       cameras, feature-map size, channels or depth bins), and in addition: prepared again whenever proj, the
 *       grid, the image size, the region of interest or epsilon change.  Nothing breaks if they change without
 *       that: a sample that finds its segment full (or a pair array shorter than the total) is added with atomics,
 *       as everywhere; it only costs time.
 * No counterpart in the reference, whose backward keeps no workspace (flash_bevpool_cuda.cu:867-937).
 */
size_t fbev_backward_sized_workspace_bytes(const fbev_problem *p, uint64_t pair_capacity);
size_t fbev_backward_sized_total_offset(const fbev_problem *p);
int fbev_backward_workspace_init_sized(const fbev_problem *p, const float *proj, void *workspace, size_t workspace_bytes,
                                       void *stream);
int fbev_backward_gather_sized(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                               const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                               size_t workspace_bytes, void *stream);

/*
 * Forward and backward of one differentiated call sharing the sample evaluation.  fbev_forward_store is
 * fbev_forward (same `out`, same `count_out`, which is required here) that also leaves, for every kept
 * sample, a 32-byte record (bilinear fractions, first corner texel with the two clamp flags, depth weight
 * and its two derivative terms, depth bins) in `store`: caller-owned device memory of
 * fbev_sample_store_bytes(p) bytes, 16-byte aligned, one slot of N * grid_z records per BEV cell, i.e.
 * B * ceil(gx/8) * ceil(gy/8) * 64 * N * grid_z * 32 bytes (0: outside the limits, B*N*H*W >= 2^29); only the
 * records of kept samples are written.  fbev_backward_gather_stored is fbev_backward_gather (persistent == 0),
 * fbev_backward_gather_persistent (persistent == 1) or fbev_backward_gather_sized (persistent == 2), with
 * `workspace` prepared as described there, whose cell
 * pass copies those records instead of projecting and weighting every sample again; `cell_count` and `store`
 * are what fbev_forward_store wrote for the same p, depth, feats and proj.  Same gradients as
 * fbev_backward_gather, to rounding.  It pays where a call is bound by latency rather than throughput (small
 * grids); the store is per-call state, like a tensor saved for the backward, and nothing checks that it
 * belongs to these inputs: records that cannot have come from this problem are clamped, so a wrong buffer
 * gives wrong numbers, never an access out of bounds.  No counterpart in the reference, whose backward
 * recomputes every sample per channel thread (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:448-568).
 */
size_t fbev_sample_store_bytes(const fbev_problem *p);
int fbev_forward_store(const fbev_problem *p, const void *depth, const void *feats, const float *proj, float *out,
                       float *count_out, void *store, size_t store_bytes, void *stream);
int fbev_backward_gather_stored(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                                const float *proj, const float *cell_count, const void *store, size_t store_bytes,
                                float *d_depth, float *d_feats, int accumulate, void *workspace, size_t workspace_bytes,
                                int persistent, void *stream);

/*
 * fbev_backward_gather without a workspace argument and without any allocation: the inverse map
 * lives in a scratch array of FBEV_STATIC_SCRATCH_BYTES that the library itself holds in device
 * memory (one copy per GPU, from the moment the library is loaded until the process ends).  It has
 * no counterpart in the reference; it is for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call makes no
 * hipMalloc / hipFree and calls no allocating library routine; inputs and outputs are the caller's,
 * as in fbev_backward_gather, and the results are the same (fixed segments and three launches where a
 * (texel, replica) segment of the worst-case layout holds four pairs or more, the counted layout otherwise).
 * The first call on a device also asks the runtime for the array's address on that device and for the
 * kernels' register counts (hipGetSymbolAddress, hipFuncGetAttributes): make that call outside a graph capture.
 * Limits: the worst-case workspace, fbev_backward_workspace_bytes(p, fbev_backward_max_pairs(p)),
 * must fit the scratch array, else FBEV_ERR_TOO_LARGE (128x128x8 cells x 6 cameras on a 16x44 map
 * needs 25.8 MB); with the per-kernel timers enabled (fbev_profile_enable), which create events,
 * it returns FBEV_ERR_UNSUPPORTED.  The device of `stream` must be the current device.  All calls
 * on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and each clears what it needs at its start.
 */
#define FBEV_STATIC_SCRATCH_BYTES (32u << 20)
int fbev_backward_gather_static(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                                const float *proj, float *d_depth, float *d_feats, int accumulate, void *stream);

/* FBEV_STATIC_SCRATCH_BYTES as the loaded library was built. */
size_t fbev_static_scratch_bytes(void);

/*
 * Backward by column ownership: the same gradients again, one launch, no global atomics and
 * no pair lists.  One workgroup owns one feature-map column (b, camera, u), finds the BEV
 * tiles whose samples can reach it, re-projects those samples, gathers the grad_out rows and
 * accumulates the column's gradient in LDS, then stores it.  Every element of d_depth and
 * d_feats is written by exactly one workgroup: with accumulate = 0 the buffers need not be
 * zero-filled (they are overwritten), with accumulate != 0 the result is added to them as in
 * fbev_backward.  `cell_count` is the count_out of fbev_forward for the same inputs; if it is
 * NULL the counts are recomputed into `workspace` (at least
 * fbev_backward_columns_workspace_bytes(p) bytes, 16-byte aligned), which is otherwise unused
 * and may be NULL.  Limits: feat_h * (channels + depth_bins) * 4 bytes must fit LDS beside the
 * sample buffer (about 80 KiB), feat_h <= 65535.
 * Replaces flash_bevpool_grad(...) (flashbev/flashbevpool/src/flash_bevpool_cuda.cu:867-937) like
 * fbev_backward does.
 */
int fbev_backward_columns(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                          const float *proj, const float *cell_count, float *d_depth, float *d_feats,
                          int accumulate, void *workspace, size_t workspace_bytes, void *stream);

size_t fbev_backward_columns_workspace_bytes(const fbev_problem *p);

/* Upper bound of the pairs one backward call can produce: one per (cell, camera, height) sample. */
uint64_t fbev_backward_max_pairs(const fbev_problem *p);

/* Bytes of a workspace holding the per-texel index plus `pair_capacity` pairs. */
size_t fbev_backward_workspace_bytes(const fbev_problem *p, uint64_t pair_capacity);

/*
 * The reference's baseline method "Sampling-VT + PillarPool": pooling over precomputed,
 * cell-sorted sample lists.  The caller has projected every (cell, camera, height) sample,
 * kept those in view and sorted them by BEV cell; sample s has feature-map coordinates
 * (u_coords[s], v_coords[s]) in texels, depth z_coords[s] and camera
 * batch_camera[s] = b * num_cams + n; interval i covers samples
 * [interval_starts[i], interval_starts[i] + interval_lengths[i]) of one cell, whose output row
 * is out[ranks_bev[interval_starts[i]] * channels ...].  Each row receives the mean over its
 * in-view samples of the bilinearly sampled features times the Gaussian / Laplace depth
 * likelihood (no weight threshold); rows no interval names are left untouched (the caller
 * zero-fills `out`).  fp32 only: depth [B,N,H,W,2], feats [B,N,H,W,C] channels-last.
 * Replaces sampling_vt_pillarpool_fused(...)
 * (flashbev/flashbevpool/src/sampling_vt_cuda.cu:131-148, kernel :24-129).
 */
typedef struct fbev_pillar_problem {
    int32_t channels;    /* C */
    int32_t n_intervals; /* touched cells */
    int32_t batch;       /* B */
    int32_t num_cams;    /* N */
    int32_t feat_h;      /* H */
    int32_t feat_w;      /* W */
    float epsilon;       /* added to sigma */
    int32_t depth_distribution; /* FBEV_GAUSSIAN / FBEV_LAPLACE */
} fbev_pillar_problem;

int fbev_pillarpool_forward(const fbev_pillar_problem *p, const float *depth, const float *feats,
                            const float *u_coords, const float *v_coords, const float *z_coords,
                            const int32_t *batch_camera, const int32_t *ranks_bev, const int32_t *interval_starts,
                            const int32_t *interval_lengths, float *out, void *stream);

/*
 * Inspection hook for parity tests: per (b, y, x, camera, height-bin) sample, in that
 * order, the projection validity and the bilinear corner indices the kernels use.
 *   mask  uint8  [B,gy,gx,N,gz]      1 = depth > 0 and inside the feature map
 *   idx   int32  [B,gy,gx,N,gz,4]    (u0,u1,v0,v1), -1 where mask is 0
 *   frac  float  [B,gy,gx,N,gz,2]    (du,dv), 0 where mask is 0
 * Any of the three may be NULL.  p->channels, in_dtype and the depth fields are ignored.
 * Restates flashbev/flashbevpool/src/flash_bevpool_cuda.cu:102-159; the reference exports no such call.
 */
int fbev_sample_geometry(const fbev_problem *p, const float *proj, uint8_t *mask, int32_t *idx,
                         float *frac, void *stream);

/*
 * Projection matrices from calibration tensors, count = B*N cameras:
 *   sensor2ego [count,4,4], camera2imgs [count,3,3], post_rots [count,3,3], post_trans [count,3]
 *   -> proj [count,3,4] = rows 0..2 of [post_rots*camera2imgs (+post_trans on column 2), 0; 0, 1] * inverse(sensor2ego)
 * Evaluated in double and rounded once to float32.  A singular sensor2ego yields non-finite entries
 * (the reference's torch.inverse raises instead, after a device synchronisation).
 * Replaces create_projection_matrix, flashbev/flashbevpool/sampling_vt.py:21-33 (about twenty
 * small PyTorch launches per call there).
 */
int fbev_projection_matrices(const float *sensor2ego, const float *camera2imgs, const float *post_rots,
                             const float *post_trans, float *proj, int32_t count, void *stream);

/* Compulsory bytes moved by one call: every operand tensor once (backward != 0 selects the backward). */
uint64_t fbev_algorithmic_bytes(const fbev_problem *p, int backward);

/*
 * Opt-in per-kernel timing for benchmarks.  While enabled, every kernel this library launches
 * is bracketed by a pair of HIP events on the launch stream (so enabling it makes calls
 * allocate events).  fbev_profile_collect waits for all recorded events, writes the summed
 * duration (ms) and launch count of each of the fbev_profile_kernel_count() kernels, and
 * clears the record.  No counterpart in the reference, which times whole calls with
 * time.perf_counter (tools/utils/benchmark_utils.py:44-69).
 */
int fbev_profile_enable(int on);
int fbev_profile_kernel_count(void);
const char *fbev_profile_kernel_name(int kernel);
int fbev_profile_collect(double *total_ms, int64_t *calls);

const char *fbev_status_string(int status);
int fbev_abi_version(void);
size_t fbev_problem_size(void);

#ifdef __cplusplus
}
#endif
#endif /* FLASHBEV_HIP_H */
