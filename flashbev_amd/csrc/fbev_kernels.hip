// Fused camera->BEV pooling for gfx950 (MI355X): the host side and the C ABI declared in
// include/flashbev_hip.h.  One translation unit; the kernels live in the headers included below:
//   fbev_common.hpp            timers, tuning constants, KParams, element access, sample geometry, depth models
//   fbev_phase_a.hpp           the sample phase shared by the cell-centric kernels
//   fbev_forward.hpp           forward kernel
//   fbev_backward_cells.hpp    pair record, zero-fill / count / scan kernels, backward cell pass
//   fbev_backward_texel.hpp    backward texel pass of the inverse map
//   fbev_backward_columns.hpp  backward with one block per feature-map column
//   fbev_aux_kernels.hpp       interval pooling (baseline method), projection matrices, geometry dump
//
// Structure of the cell-centric kernels.  A wavefront (64 lanes) owns S consecutive BEV cells
// ("slots") of one batch element and works in two phases:
//   phase A  the samples (slot, camera, height bin) of its cells: whole (cell, camera) columns
//            are culled first, then single samples with a cheap test; what is left is projected
//            through the camera's 3x4 matrix (held in LDS) in the canonical arithmetic, tested
//            against the field of view, and gets its depth weight -- once per sample, not once
//            per channel.  Kept samples are compacted, in (camera, height) order, into a
//            per-slot list in LDS.
//   phase B  lanes = (slot, channel vector).  Each slot walks its list; every entry is four
//            128-bit gathers per lane from the channels-last feature map, coalesced across the
//            lanes of the slot, accumulated in registers.
// The frustum volume never exists in memory.  The backward's cell pass repeats phase A with the
// derivative terms added to each entry and reduces the per-sample inner product
// <grad_out, sampled feature> across the slot; the feature gradient is then either scattered
// with hardware fp32 atomics, or (default) gathered per texel from 32-byte records the cell pass
// files under each sample's first corner texel (the inverse map).
//
// Arithmetic contract: this file is compiled with -ffp-contract=off.  The geometry
// (projection, mask, indices, bilinear fractions) uses individually rounded fp32
// operations in a fixed order so that masks and indices are reproducible bit for bit;
// fused multiply-adds appear only where written explicitly (the channel accumulation).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <type_traits>
#include <vector>

#include "flashbev_hip.h"

#include "fbev_common.hpp"
#include "fbev_phase_a.hpp"
#include "fbev_forward.hpp"
#include "fbev_backward_cells.hpp"
#include "fbev_backward_texel.hpp"
#include "fbev_backward_columns.hpp"
#include "fbev_aux_kernels.hpp"

namespace {

// ---------------------------------------------------------------- host side
struct Plan {
    KParams k;
    int vec;        // elements per 16-byte load, or 1
    int cpl;        // channel vectors per lane per pass
    size_t lds_fwd, lds_bwd, lds_fill, lds_count;
};

int elem_size(int dtype) { return dtype == FBEV_F32 ? 4 : 2; }

int validate(const fbev_problem *p, bool need_channels) {
    if (p == nullptr) return FBEV_ERR_NULL;
    if (p->batch <= 0 || p->num_cams <= 0 || p->feat_h <= 0 || p->feat_w <= 0 || p->image_h <= 0 ||
        p->image_w <= 0 || p->grid_x <= 0 || p->grid_y <= 0 || p->grid_z <= 0)
        return FBEV_ERR_SHAPE;
    if (need_channels && p->channels <= 0) return FBEV_ERR_SHAPE;
    if (p->proj_stride != 12 && p->proj_stride != 16) return FBEV_ERR_SHAPE;
    if (need_channels) {
        if (p->in_dtype != FBEV_F32 && p->in_dtype != FBEV_F16 && p->in_dtype != FBEV_BF16)
            return FBEV_ERR_UNSUPPORTED;
        if (p->depth_distribution < FBEV_GAUSSIAN || p->depth_distribution > FBEV_CATEGORICAL)
            return FBEV_ERR_UNSUPPORTED;
        if (p->reduction != FBEV_REDUCE_MEAN && p->reduction != FBEV_REDUCE_SUM) return FBEV_ERR_UNSUPPORTED;
        if (p->depth_distribution == FBEV_CATEGORICAL) {
            if (p->depth_bins < 1 || p->depth_bins > 0xffff || !(p->depth_step > 0.0f)) return FBEV_ERR_SHAPE;
        } else if (p->depth_bins != 2) {
            return FBEV_ERR_SHAPE;
        }
    }
    // texel indices, cell counts and sample counts are 32-bit in the kernels
    const long long texels = (long long)p->batch * p->num_cams * p->feat_h * p->feat_w;
    const long long nz = (long long)p->num_cams * p->grid_z;
    const long long tiles = (long long)((p->grid_x + kTile - 1) / kTile) * ((p->grid_y + kTile - 1) / kTile);
    if (texels >= (1ll << 31) || nz >= (1 << 20) || tiles * 64 >= (1ll << 30)) return FBEV_ERR_TOO_LARGE;
    // the sample decode table packs the camera into 12 bits and the height bin into 16
    if (p->num_cams > 0xfff || p->grid_z > 0xffff) return FBEV_ERR_TOO_LARGE;
    return FBEV_OK;
}

int make_plan(const fbev_problem *p, bool allow_vec, Plan *plan, int waves = kWavesPerBlock, int max_rounds = 3,
              int slot_budget = kMaxSlotLdsBytes, int max_batch = 4) {
    const int entry_bytes = 32 + 4;      // an entry (two float4 in every kernel) and its candidate index
    KParams &k = plan->k;
    k.B = p->batch; k.N = p->num_cams; k.H = p->feat_h; k.W = p->feat_w; k.C = p->channels;
    k.gx = p->grid_x; k.gy = p->grid_y; k.gz = p->grid_z;
    k.NZ = k.N * k.gz;
    k.tiles_x = (k.gx + kTile - 1) / kTile;
    k.tiles_y = (k.gy + kTile - 1) / kTile;
    k.padded_cells = k.tiles_x * k.tiles_y * 64;
    k.Wi_f = (float)p->image_w; k.Hi_f = (float)p->image_h;
    k.W_f = (float)p->feat_w; k.H_f = (float)p->feat_h;
    k.xmin = p->voxel_min[0]; k.ymin = p->voxel_min[1]; k.zmin = p->voxel_min[2];
    k.vx = p->voxel_size[0]; k.vy = p->voxel_size[1]; k.vz = p->voxel_size[2];
    k.eps = p->epsilon; k.thr = p->depth_weight_threshold;
    {
        // FNV-1a over the bytes of the values a geometry cache was built from
        uint64_t h = 1469598103934665603ull;
        auto mix = [&h](const void *v, size_t n) {
            const unsigned char *c = static_cast<const unsigned char *>(v);
            for (size_t i = 0; i < n; ++i) h = (h ^ c[i]) * 1099511628211ull;
        };
        mix(&p->image_h, sizeof p->image_h); mix(&p->image_w, sizeof p->image_w);
        mix(p->voxel_min, sizeof p->voxel_min); mix(p->voxel_size, sizeof p->voxel_size);
        mix(&p->epsilon, sizeof p->epsilon);
        k.geo_lo = (unsigned)h; k.geo_hi = (unsigned)(h >> 32);
    }
    k.dist = p->depth_distribution; k.Dd = p->depth_bins;
    k.dmin = p->depth_min; k.dstep = p->depth_step;
    k.reduce_sum = p->reduction == FBEV_REDUCE_SUM;
    k.proj_stride = p->proj_stride;
    {
        int bits = 0;
        if (k.dist == FBEV_CATEGORICAL) while ((1 << bits) < k.Dd) ++bits;
        const long long cells = (long long)k.B * p->grid_y * p->grid_x;
        k.bin_bits = (cells << bits) < (1ll << 31) ? bits : -1;
    }

    const int es = elem_size(p->in_dtype);
    const int full_vec = 16 / es;
    plan->vec = (allow_vec && k.C % full_vec == 0) ? full_vec : 1;
    {
        // feature rows are addressed by 32-bit byte offsets from the tensor's base (the gather loops then
        // form an address with one 32-bit add): the feature tensor stays below 4 GiB
        if ((long long)k.B * k.N * k.H * k.W * k.C * es >= (1ll << 32)) return FBEV_ERR_TOO_LARGE;
        k.row_units = k.C * es;
        // exact division of a tile index by tiles_x: umulhi(tile, ceil(2^32 / tiles_x)) is the quotient for
        // every tile with tile * tiles_x < 2^32
        const long long tiles = (long long)k.tiles_x * k.tiles_y;
        if (tiles * k.tiles_x >= (1ll << 32)) return FBEV_ERR_TOO_LARGE;
        // (a divisor of 1 has no 32-bit magic; the kernels test for it)
        k.tiles_x_magic = k.tiles_x > 1 ? (unsigned)(((1ull << 32) + k.tiles_x - 1) / k.tiles_x) : 0u;
        k.cams_magic = k.N > 1 ? (unsigned)(((1ull << 32) + k.N - 1) / k.N) : 0u;
    }
    const int cq = (k.C + plan->vec - 1) / plan->vec;      // channel vectors per texel
    int lps = cq < kWave ? cq : kWave;
    int cpl = (cq + lps - 1) / lps;
    cpl = cpl <= 1 ? 1 : (cpl <= 2 ? 2 : 4);               // more than 4*lps vectors: extra passes
    plan->cpl = cpl;
    k.lanes_per_slot = lps;
    int slots = kWave / lps;
    // the lists must fit the per-wave LDS budget
    while (slots > 1 && (long long)slots * k.NZ * entry_bytes > slot_budget) --slots;
    if (slots > 16) slots = 16;
    {
        // The lane groups (kWave / lps of them) are shared out among the slots in equal numbers, and
        // groups left over idle through phase B: take fewer slots when that leaves more than a fifth of
        // the groups without work (four groups and room for three cells: two cells with two groups each;
        // 400x400 grid, 64 channels: cell pass 329 -> 268 us at 20 height bins, forward 235 -> 173 us at 24).
        const int groups_all = kWave / lps;
        while (slots > 1 && (groups_all / slots) * slots * 5 < groups_all * 4) --slots;
    }
    k.slots = slots;
    k.groups_per_slot = (kWave / lps) / slots;     // >= 1: slots <= kWave / lps
    k.lps_magic = 65535u / (unsigned)lps + 1u;
    k.gps_magic = 65535u / (unsigned)k.groups_per_slot + 1u;
    k.list_cap = k.NZ;
    k.pool_cap = slots * k.NZ;       // what one group of `slots` cells can keep at most
    // enough wavefronts to fill 256 CUs several times over before a wavefront takes more rounds,
    // and never many rounds: cells differ widely in their number of samples, and short wavefronts
    // even that out (training-size cell pass: 439 / 406 / 399 / 404 / 439 us with at most
    // 8 / 4 / 3 / 2 / 1 rounds; the forward does not care)
    const long long groups = ((long long)k.padded_cells + slots - 1) / slots * k.B;
    int rounds = (int)(groups / (256ll * 4 * 8 * 2));
    rounds = rounds < 1 ? 1 : (rounds > max_rounds ? max_rounds : rounds);
    // Groups of one batch: the sample phase runs over `batch` groups of `slots` cells together, so that
    // its 64-lane passes are filled (about one sample in six is in view: a group with fewer than some
    // forty in-view samples leaves stage 2 half empty).  Never more groups than the wavefront has rounds
    // (a small problem keeps its many short wavefronts), at most four, at most 16 cells.
    int batch = 1;
    if (max_batch > 1 && plan->vec > 1) {
        const int expect = (slots * k.NZ + 5) / 6;          // candidates of one group, roughly
        batch = expect > 0 ? (64 + expect / 2) / expect : 1;      // as many groups as fill one pass, rounded
        if (batch > max_batch) batch = max_batch;
        if (batch > rounds) batch = rounds;
        while (batch > 1 && (slots * batch > 16 || (long long)slots * batch * k.NZ >= 4096)) --batch;
        if (batch < 1) batch = 1;
    }
    k.batch_groups = batch;
    k.slots_a = slots * batch;
    k.rounds = (rounds + batch - 1) / batch;          // batches per wavefront
    k.waves = waves;
    const int cells_per_block = waves * k.slots_a * k.rounds;
    k.blocks_per_batch = (k.padded_cells + cells_per_block - 1) / cells_per_block;
    k.n_blocks = k.blocks_per_batch * k.B;
    // exact for every block index when n_blocks * blocks_per_batch < 2^32; otherwise the kernels divide
    k.bpb_magic = (k.blocks_per_batch > 1 && (long long)k.n_blocks * k.blocks_per_batch < (1ll << 32))
                      ? (unsigned)(((1ull << 32) + k.blocks_per_batch - 1) / k.blocks_per_batch) : 0u;
    const size_t p_f4 = (size_t)(k.N * 12 + 3) / 4;
    const size_t cols = (size_t)k.slots_a * k.N, dec_f4 = (cols + 3) / 4;
    const size_t cand_f4 = ((size_t)k.slots_a * k.NZ + 3) / 4, z_f4 = ((size_t)k.gz + 3) / 4;
    auto block_lds = [&](int entry_f4) {
        return (p_f4 + dec_f4 + z_f4 +
                (size_t)waves * ((2 * (size_t)k.slots_a + 8 + 3) / 4 + k.slots_a + cols + dec_f4 + cand_f4 +
                                 (size_t)k.pool_cap * entry_f4)) * 16;
    };
    {
        // exact division of a sample index below 4096 by gz: multiply and shift
        if ((long long)k.slots_a * k.NZ >= 4096) return FBEV_ERR_TOO_LARGE;
        int l = 0;
        while ((1 << l) < k.gz) ++l;
        k.gz_shift = 12 + l;
        k.gz_magic = (int)((((long long)1 << k.gz_shift) + k.gz - 1) / k.gz);
    }
    plan->lds_fwd = block_lds(2);
    plan->lds_bwd = block_lds(2);
    plan->lds_fill = block_lds(2);
    plan->lds_count = block_lds(0);
    if (plan->lds_fill > (size_t)kLdsLimitBytes) return FBEV_ERR_TOO_LARGE;
    return FBEV_OK;
}

// More than 64 KiB of dynamic LDS has to be opted into per kernel; only long sample lists
// (many cameras x height bins) or wide columns get there.
template <typename Kernel>
bool lds_opt_in(Kernel kernel, size_t lds) {
    if (lds <= (size_t)kMaxBlockLdsBytes) return true;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds) == hipSuccess;
}

template <typename T, int VEC>
int launch_forward(const Plan &pl, const void *depth, const void *feats, const float *proj, float *out,
                   float *cnt, hipStream_t st, float4 *store = nullptr) {
    dim3 grid(pl.k.n_blocks), block(kWave * pl.k.waves);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    prof::Scope timer(out != nullptr ? prof::kForward : prof::kCellCount, st);
    // (a forward that stores its samples writes its output with ordinary stores: the problems it serves are small)
    const bool stream = store == nullptr && VEC > 1 && (long long)pl.k.B * pl.k.gy * pl.k.gx * pl.k.C * 4 > kStreamOutputFrom;
    auto launch = [&](auto kernel) {
        if (!lds_opt_in(kernel, pl.lds_fwd)) return false;
        hipLaunchKernelGGL(kernel, grid, block, pl.lds_fwd, st, pl.k, d, f, proj, out, cnt, store);
        return true;
    };
    // (batches of several groups and streamed output exist on the vector paths only; the plan asks for
    // neither elsewhere)
    constexpr bool V = VEC > 1;
    const bool batched = V && pl.k.batch_groups > 1;
    if (!V && pl.k.batch_groups > 1) return FBEV_ERR_LAUNCH;
    auto pick = [&](auto cpl_tag) {
        constexpr int CPL = decltype(cpl_tag)::value;
        if (store != nullptr)
            return batched ? launch(fbev_forward_kernel<T, VEC, CPL, false, V, true>) : launch(fbev_forward_kernel<T, VEC, CPL, false, false, true>);
        if (stream) return batched ? launch(fbev_forward_kernel<T, VEC, CPL, V, V>) : launch(fbev_forward_kernel<T, VEC, CPL, V, false>);
        return batched ? launch(fbev_forward_kernel<T, VEC, CPL, false, V>) : launch(fbev_forward_kernel<T, VEC, CPL, false, false>);
    };
    const bool ok = pl.cpl == 1 ? pick(std::integral_constant<int, 1>{})
                                : (pl.cpl == 2 ? pick(std::integral_constant<int, 2>{}) : pick(std::integral_constant<int, 4>{}));
    if (!ok) return FBEV_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int dispatch_forward(const fbev_problem *p, const Plan &pl, const void *depth, const void *feats, const float *proj,
                     float *out, float *cnt, hipStream_t st, float4 *store = nullptr) {
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_forward<float, 4>(pl, depth, feats, proj, out, cnt, st, store)
                               : launch_forward<float, 1>(pl, depth, feats, proj, out, cnt, st, store);
        case FBEV_F16:
            return pl.vec == 8 ? launch_forward<__half, 8>(pl, depth, feats, proj, out, cnt, st, store)
                               : launch_forward<__half, 1>(pl, depth, feats, proj, out, cnt, st, store);
        default:
            return pl.vec == 8 ? launch_forward<bf16_raw, 8>(pl, depth, feats, proj, out, cnt, st, store)
                               : launch_forward<bf16_raw, 1>(pl, depth, feats, proj, out, cnt, st, store);
    }
}

// Bytes of a sample store: per cell of the tiled walk a slot of N * gz records of 32 bytes.
size_t sample_store_bytes(const fbev_problem *p) {
    const long long tiles = (long long)((p->grid_x + kTile - 1) / kTile) * ((p->grid_y + kTile - 1) / kTile);
    // a stored first-corner texel shares its word with the two clamp flags
    if ((long long)p->batch * p->num_cams * p->feat_h * p->feat_w >= (1ll << 29)) return 0;
    return (size_t)p->batch * (size_t)tiles * 64 * (size_t)p->num_cams * (size_t)p->grid_z * 2 * sizeof(float4);
}

template <typename T, int VEC>
int launch_forward_cached(const Plan &pl, const void *depth, const void *feats, const void *cache, float *out,
                          float *cnt, hipStream_t st) {
    dim3 grid(pl.k.n_blocks), block(kWave * pl.k.waves);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    prof::Scope timer(prof::kForwardCached, st);
    const bool stream = VEC > 1 && (long long)pl.k.B * pl.k.gy * pl.k.gx * pl.k.C * 4 > kStreamOutputFrom;
    auto launch = [&](auto kernel) {
        if (!lds_opt_in(kernel, pl.lds_fwd)) return false;
        hipLaunchKernelGGL(kernel, grid, block, pl.lds_fwd, st, pl.k, d, f, cache, out, cnt);
        return true;
    };
    bool ok;
    if (stream) {
        constexpr bool S = VEC > 1;
        ok = pl.cpl == 1 ? launch(fbev_forward_cached_kernel<T, VEC, 1, S>)
                         : (pl.cpl == 2 ? launch(fbev_forward_cached_kernel<T, VEC, 2, S>)
                                        : launch(fbev_forward_cached_kernel<T, VEC, 4, S>));
    } else {
        ok = pl.cpl == 1 ? launch(fbev_forward_cached_kernel<T, VEC, 1, false>)
                         : (pl.cpl == 2 ? launch(fbev_forward_cached_kernel<T, VEC, 2, false>)
                                        : launch(fbev_forward_cached_kernel<T, VEC, 4, false>));
    }
    if (!ok) return FBEV_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

// bytes of a geometry cache; 0 when the problem is outside its limits
size_t geometry_cache_bytes(const fbev_problem *p) {
    const long long tiles = (long long)((p->grid_x + kTile - 1) / kTile) * ((p->grid_y + kTile - 1) / kTile);
    const long long cells = (long long)p->batch * tiles * 64;
    // a cached first-corner texel shares its word with the two clamp flags
    if ((long long)p->batch * p->num_cams * p->feat_h * p->feat_w >= (1ll << 29)) return 0;
    return cache_entries_offset(cells) + (size_t)cells * p->num_cams * p->grid_z * sizeof(float4);
}

template <typename T, int VEC>
int launch_columns(const Plan &pl, const ColParams &cp, size_t lds, const float *go, const void *depth,
                   const void *feats, const float *proj, const float *count, float *dd, float *df, hipStream_t st) {
    auto kernel = fbev_backward_column_kernel<T, VEC>;
    if (!lds_opt_in(kernel, lds)) return FBEV_ERR_LAUNCH;
    prof::Scope timer(prof::kBackwardColumn, st);
    hipLaunchKernelGGL(kernel, dim3(cp.n_blocks), dim3(kColThreads), lds, st, pl.k, cp, go,
                       static_cast<const T *>(depth), static_cast<const T *>(feats), proj, count, dd, df);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

template <typename T, int VEC, int FILL>
int launch_cells(const Plan &pl, const float *go, const void *depth, const void *feats, const float *proj,
                 float *dd, float *df, const int *prefix, int *cursor, Pair *pairs, int cap, hipStream_t st,
                 int *epoch = nullptr, int set_stride = 0, const float *count = nullptr, const float4 *store = nullptr,
                 SegTable segs = SegTable{nullptr}) {
    dim3 grid(pl.k.n_blocks), block(kWave * pl.k.waves);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    const size_t lds = FILL ? pl.lds_fill : pl.lds_bwd;
    prof::Scope timer(FILL ? prof::kBackwardCells : prof::kBackwardScatter, st);
    constexpr bool V = VEC > 1;
    const bool batched = V && pl.k.batch_groups > 1;
    if (!V && pl.k.batch_groups > 1) return FBEV_ERR_LAUNCH;
    auto launch = [&](auto kernel) {
        if (!lds_opt_in(kernel, lds)) return false;
        hipLaunchKernelGGL(kernel, grid, block, lds, st, pl.k, go, d, f, proj, dd, df, prefix, cursor, pairs, cap, epoch, set_stride,
                           count, store, segs);
        return true;
    };
    auto pick = [&](auto cpl_tag) {
        constexpr int CPL = decltype(cpl_tag)::value;
        if constexpr (FILL == 3) {
            // stored samples go through a batch in one piece: the plan has one group per batch
            return !batched && launch(fbev_backward_cells_kernel<T, VEC, CPL, FILL, false>);
        } else {
            return batched ? launch(fbev_backward_cells_kernel<T, VEC, CPL, FILL, V>) : launch(fbev_backward_cells_kernel<T, VEC, CPL, FILL, false>);
        }
    };
    const bool ok = pl.cpl == 1 ? pick(std::integral_constant<int, 1>{})
                                : (pl.cpl == 2 ? pick(std::integral_constant<int, 2>{}) : pick(std::integral_constant<int, 4>{}));
    if (!ok) return FBEV_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

// Whether the batched cell pass pays for this instantiation: it holds a few more registers than the
// plain one, and where those cost a wavefront per SIMD (512 registers per lane, allocated in eights)
// the plain kernel is the faster one (training size, fp16: 101 against 91 registers, 4 against 5
// wavefronts per SIMD, 397 against 385 us).  Asked of the runtime once per instantiation.
int kernel_registers(const void *kernel) {
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, kernel) != hipSuccess) return 0;
    return attr.numRegs;
}

template <typename T, int VEC, int FILL>
bool cells_batch_pays_for(int cpl) {
    static std::atomic<int> cache[3] = {{-1}, {-1}, {-1}};
    const int idx = cpl == 1 ? 0 : (cpl == 2 ? 1 : 2);
    int got = cache[idx].load(std::memory_order_relaxed);
    if (got < 0) {
        auto waves = [](int regs) { return regs > 0 ? 512 / ((regs + 7) / 8 * 8) : 0; };
        auto both = [&](auto cpl_tag) {
            constexpr int CPL = decltype(cpl_tag)::value;
            const int with = kernel_registers(reinterpret_cast<const void *>(fbev_backward_cells_kernel<T, VEC, CPL, FILL, true>));
            const int without = kernel_registers(reinterpret_cast<const void *>(fbev_backward_cells_kernel<T, VEC, CPL, FILL, false>));
            return (with > 0 && without > 0 && waves(with) >= waves(without)) ? 1 : 0;
        };
        got = cpl == 1 ? both(std::integral_constant<int, 1>{})
                       : (cpl == 2 ? both(std::integral_constant<int, 2>{}) : both(std::integral_constant<int, 4>{}));
        cache[idx].store(got, std::memory_order_relaxed);
    }
    return got != 0;
}

template <int FILL>
bool cells_batch_pays(const fbev_problem *p, const Plan &pl) {
    if (pl.vec == 1) return false;
    switch (p->in_dtype) {
        case FBEV_F32: return cells_batch_pays_for<float, 4, FILL>(pl.cpl);
        case FBEV_F16: return cells_batch_pays_for<__half, 8, FILL>(pl.cpl);
        default: return cells_batch_pays_for<bf16_raw, 8, FILL>(pl.cpl);
    }
}

template <int FILL>
int dispatch_cells(const fbev_problem *p, const Plan &pl, const float *go, const void *depth, const void *feats,
                   const float *proj, float *dd, float *df, const int *prefix, int *cursor, Pair *pairs, int cap,
                   hipStream_t st, int *epoch = nullptr, int set_stride = 0, const float *count = nullptr,
                   const float4 *store = nullptr, SegTable segs = SegTable{nullptr}) {
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_cells<float, 4, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs)
                               : launch_cells<float, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs);
        case FBEV_F16:
            return pl.vec == 8 ? launch_cells<__half, 8, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs)
                               : launch_cells<__half, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs);
        default:
            return pl.vec == 8 ? launch_cells<bf16_raw, 8, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs)
                               : launch_cells<bf16_raw, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st, epoch, set_stride, count, store, segs);
    }
}

template <typename T, bool VIEW = false>
int launch_count(const Plan &pl, const void *depth, const float *proj, int *counts, hipStream_t st) {
    if (!lds_opt_in(fbev_count_kernel<T, VIEW>, pl.lds_count)) return FBEV_ERR_LAUNCH;
    prof::Scope timer(prof::kCount, st);
    hipLaunchKernelGGL((fbev_count_kernel<T, VIEW>), dim3(pl.k.n_blocks), dim3(kWave * pl.k.waves), pl.lds_count, st, pl.k,
                       static_cast<const T *>(depth), proj, counts);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

long long texel_count(const fbev_problem *p) {
    return (long long)p->batch * p->num_cams * p->feat_h * p->feat_w;
}

long long sample_count(const fbev_problem *p) {
    return (long long)p->batch * p->grid_y * p->grid_x * p->num_cams * p->grid_z;
}

// Workspace layout: [texels * kReplicas int32 segment cursors][chunk prefix sums], padded to
// 256 bytes, then the pairs.
long long counter_count(const fbev_problem *p) { return texel_count(p) * kReplicas; }
long long chunk_count(const fbev_problem *p) {
    return (counter_count(p) + (1ll << kScanChunkBits) - 1) >> kScanChunkBits;
}
size_t ws_index_bytes(const fbev_problem *p) {
    return ((size_t)(counter_count(p) + chunk_count(p) + 1) * sizeof(int) + 255) / 256 * 256;
}

// A persistent workspace (fixed segments only) starts with
//   [256 bytes: the two call counters][two sets of texels * kFixedReplicas claim counters]
//   [a depth-gradient and a feature-gradient buffer of the workspace's own], each padded to 256 bytes,
// then the pairs.  fbev_backward_workspace_init zero-fills all of it but the pairs, once.
// A workspace whose segments are sized by the geometry (fbev_backward_workspace_init_sized) holds, between the
// gradient buffers and the pairs, the table the kernels read (per segment its start in the pair array and its
// capacity, the samples in view that claim there) and what it was made from: the capacities, their prefix sums
// within scan chunks of 4096 segments, and per chunk the pairs before it, with the total behind the last chunk.
struct PersistLayout {
    size_t sets, ovf_depth, ovf_feats, pairs;      // byte offsets
    long long segments;                            // (texel, replica) segments = claim counters per set
    long long set_stride;                          // ints between the two sets (sized segments: 64-bit counters)
    size_t seg_tab, seg_cap, seg_off, seg_prefix;  // byte offsets of the tables (sized segments only)
    long long seg_chunks;                          // scan chunks of the segment tables
};
PersistLayout persist_layout(const fbev_problem *p, bool sized = false) {
    auto pad = [](size_t n) { return (n + 255) / 256 * 256; };
    const size_t texels = (size_t)texel_count(p);
    PersistLayout l;
    l.segments = (long long)texels * kFixedReplicas;
    l.set_stride = sized ? 2 * l.segments : l.segments;
    l.sets = 256;
    l.ovf_depth = l.sets + pad(2 * (size_t)l.set_stride * sizeof(int));
    l.ovf_feats = l.ovf_depth + pad(texels * p->depth_bins * sizeof(float));
    l.pairs = l.ovf_feats + pad(texels * p->channels * sizeof(float));
    l.seg_tab = l.seg_cap = l.seg_off = l.seg_prefix = 0;
    l.seg_chunks = (l.segments + (1ll << kScanChunkBits) - 1) >> kScanChunkBits;
    if (sized) {
        l.seg_tab = l.pairs;
        l.seg_cap = l.seg_tab + pad((size_t)l.segments * sizeof(int2));
        l.seg_off = l.seg_cap + pad((size_t)l.segments * sizeof(int));
        l.seg_prefix = l.seg_off + pad((size_t)l.segments * sizeof(int));
        l.pairs = l.seg_prefix + pad((size_t)(l.seg_chunks + 1) * sizeof(int));
    }
    return l;
}

int launch_zero(int *a, long long na, float *b, long long nb, float *c, long long nc, hipStream_t st) {
    if (!a) na = 0;
    if (!b) nb = 0;
    if (!c) nc = 0;
    const long long n = zero_units(na) + zero_units(nb) + zero_units(nc);
    if (n == 0) return FBEV_OK;
    prof::Scope timer(prof::kZero, st);
    hipLaunchKernelGGL(fbev_fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, na,
                       reinterpret_cast<int *>(b), nb, reinterpret_cast<int *>(c), nc);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int check_backward_args(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                        const float *proj, const float *d_depth, const float *d_feats) {
    if (!grad_out || !depth || !feats || !proj) return FBEV_ERR_NULL;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)proj % 4 || (uintptr_t)grad_out % 4 ||
        (uintptr_t)d_depth % 4 || (uintptr_t)d_feats % 4)
        return FBEV_ERR_ALIGNMENT;
    return FBEV_OK;
}


// ---------------------------------------------------------------- library-owned scratch
// Workspace of fbev_backward_gather_static, for callers that cannot allocate: one array per
// GPU, held from the moment the library is loaded there until the process ends.  In host code
// the array's name is a stand-in, not a device address; the address on each device comes from
// hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[FBEV_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex scratch_mu;
void *scratch_ptr[kMaxDevices] = {};

int scratch_of_current_device(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FBEV_ERR_LAUNCH;
    std::lock_guard<std::mutex> g(scratch_mu);
    if (scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return FBEV_ERR_LAUNCH;
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return FBEV_OK;
}

int backward_gather_impl(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                         const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                         size_t workspace_bytes, void *stream, int ws_kind = 0, const float *cell_count = nullptr,
                         const void *store = nullptr, size_t store_bytes = 0) {
    // ws_kind: 0 a per-call workspace, 1 a persistent one with segments of one common capacity, 2 a persistent
    // one whose segments were sized by the geometry
    if (ws_kind < 0 || ws_kind > 2) return FBEV_ERR_UNSUPPORTED;
    const bool persistent = ws_kind != 0, sized = ws_kind == 2;
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    rc = check_backward_args(p, grad_out, depth, feats, proj, d_depth, d_feats);
    if (rc != FBEV_OK) return rc;
    if (!d_depth && !d_feats) return FBEV_OK;
    if (!workspace) return FBEV_ERR_NULL;
    if ((uintptr_t)workspace % 16) return FBEV_ERR_ALIGNMENT;
    const PersistLayout lay = persist_layout(p, sized);
    const size_t index_bytes = persistent ? lay.pairs : ws_index_bytes(p);
    if (workspace_bytes < index_bytes) return FBEV_ERR_SHAPE;
    // pair positions are 32-bit: every sample must be countable
    if (sample_count(p) >= (1ll << 31) || counter_count(p) >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
    // the texel pass addresses grad_out rows in 32-bit units (16 bytes, or one float off the vector path)
    const bool rows_vec4 = p->channels % 4 == 0 && (uintptr_t)grad_out % 16 == 0;
    if ((long long)p->batch * p->grid_y * p->grid_x * (rows_vec4 ? p->channels / 4 : p->channels) >= (1ll << 32))
        return FBEV_ERR_TOO_LARGE;
    size_t cap64 = (workspace_bytes - index_bytes) / sizeof(Pair);
    const int cap = cap64 > 0x7fffffffull ? 0x7fffffff : (int)cap64;
    Plan pl;
    const bool allow_vec = (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0;
    // the samples the forward stored serve where claims are made one by one (the only kind phase_a_stored makes)
    bool stored = store != nullptr;
    if (stored) {
        // (where a claim counter may get hundreds of samples the claims go per run, which the stored samples do
        // not: such problems evaluate their samples again)
        const long long tx = texel_count(p);
        const bool fixed_layout = sized || ((uint64_t)cap >= fbev_backward_max_pairs(p) && cap / (tx * kFixedReplicas) >= kFixedMinSegment);
        if (sample_count(p) / (fixed_layout ? tx * kFixedReplicas : counter_count(p)) >= kClaimRunsFrom) stored = false;
    }
    if (stored) {
        if (!cell_count) return FBEV_ERR_NULL;
        if ((uintptr_t)store % 16 || (uintptr_t)cell_count % 4) return FBEV_ERR_ALIGNMENT;
        const size_t need = sample_store_bytes(p);
        if (need == 0) return FBEV_ERR_TOO_LARGE;
        if (store_bytes < need) return FBEV_ERR_SHAPE;
    }
    rc = make_plan(p, allow_vec, &pl, kCellPassWaves, 3, kMaxSlotLdsBytes, stored ? 1 : 4);
    if (rc != FBEV_OK) return rc;
    if (!stored) {
        // the cell pass in batches of several groups only where that does not cost occupancy
        const long long tx = texel_count(p);
        const bool fixed_layout = sized || ((uint64_t)cap >= fbev_backward_max_pairs(p) && cap / (tx * kFixedReplicas) >= kFixedMinSegment);
        const bool runs = sample_count(p) / (fixed_layout ? tx * kFixedReplicas : counter_count(p)) >= kClaimRunsFrom;
        if (pl.k.batch_groups > 1 && !(runs ? cells_batch_pays<2>(p, pl) : cells_batch_pays<1>(p, pl))) {
            rc = make_plan(p, allow_vec, &pl, kCellPassWaves, 3, kMaxSlotLdsBytes, 1);
            if (rc != FBEV_OK) return rc;
        }
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    char *base = static_cast<char *>(workspace);
    int *cursor = persistent ? reinterpret_cast<int *>(base + lay.sets) : static_cast<int *>(workspace);
    Pair *pairs = reinterpret_cast<Pair *>(base + index_bytes);
    const long long texels = texel_count(p);
    const long long counters = counter_count(p), chunks = chunk_count(p);
    int *chunk_prefix = cursor + counters;

    // A workspace with room for every sample gets fixed segments: each (texel, replica)
    // owns cap / (texels * kFixedReplicas) pair slots, and the counting pass and the prefix sums
    // are not needed.  (A texel that outgrows its segments falls back to atomics, like a full
    // pair array does.)  Smaller workspaces are packed exactly: count, scan, fill.
    const bool fixed = sized || ((uint64_t)cap >= fbev_backward_max_pairs(p) && cap / (texels * kFixedReplicas) >= kFixedMinSegment);
    if (persistent && !fixed) return FBEV_ERR_SHAPE;      // a persistent workspace holds the worst case, or sized segments
    // (with sized segments the kernels compare positions with the whole array's capacity)
    const int seg_cap = sized ? cap : (fixed ? (int)(cap / (texels * kFixedReplicas)) : 0);
    // what the two kernels get when the workspace is persistent: no zero-fill launch then
    Persist ps = {nullptr, nullptr, 0, nullptr, nullptr, SegTable{nullptr}};
    if (sized)
        ps.segs = SegTable{reinterpret_cast<const int2 *>(base + lay.seg_tab)};
    float *cells_dd = d_depth, *cells_df = d_feats;
    if (persistent) {
        ps.epoch = reinterpret_cast<int *>(base);
        ps.sets = cursor;
        ps.set_stride = (int)lay.set_stride;
        ps.ovf_depth = reinterpret_cast<float *>(base + lay.ovf_depth);
        ps.ovf_feats = reinterpret_cast<float *>(base + lay.ovf_feats);
        // the cell pass adds what it cannot file to the workspace's own gradient buffers
        if (d_depth) cells_dd = ps.ovf_depth;
        if (d_feats) cells_df = ps.ovf_feats;
    } else {
        rc = launch_zero(cursor, fixed ? texels * kFixedReplicas : counters, accumulate ? nullptr : d_depth,
                         texels * p->depth_bins, accumulate ? nullptr : d_feats, texels * p->channels, st);
        if (rc != FBEV_OK) return rc;
    }
    if (!fixed) {
        switch (p->in_dtype) {
            case FBEV_F32: rc = launch_count<float>(pl, depth, proj, cursor, st); break;
            case FBEV_F16: rc = launch_count<__half>(pl, depth, proj, cursor, st); break;
            default: rc = launch_count<bf16_raw>(pl, depth, proj, cursor, st); break;
        }
        if (rc != FBEV_OK) return rc;
        {
            prof::Scope timer(prof::kScanChunks, st);
            hipLaunchKernelGGL(fbev_scan_chunks_kernel, dim3((unsigned)chunks), dim3(1024), 0, st, cursor, counters,
                               chunk_prefix);
        }
        if (hipGetLastError() != hipSuccess) return FBEV_ERR_LAUNCH;
        {
            prof::Scope timer(prof::kScanSums, st);
            hipLaunchKernelGGL(fbev_scan_sums_kernel, dim3(1), dim3(1024), 0, st, chunk_prefix, (int)chunks);
        }
        if (hipGetLastError() != hipSuccess) return FBEV_ERR_LAUNCH;
    }
    const int *prefix_arg = fixed ? nullptr : chunk_prefix;
    const int cap_arg = fixed ? seg_cap : cap;
    // samples a claim counter gets if every sample is kept
    const bool claim_runs = sample_count(p) / (fixed ? texels * kFixedReplicas : counters) >= kClaimRunsFrom;
    if (stored)
        rc = dispatch_cells<3>(p, pl, grad_out, depth, feats, proj, cells_dd, cells_df, prefix_arg, cursor, pairs, cap_arg, st,
                               ps.epoch, ps.set_stride, cell_count, static_cast<const float4 *>(store), ps.segs);
    else
    rc = claim_runs ? dispatch_cells<2>(p, pl, grad_out, depth, feats, proj, cells_dd, cells_df, prefix_arg, cursor, pairs,
                                        cap_arg, st, ps.epoch, ps.set_stride, nullptr, nullptr, ps.segs)
                    : dispatch_cells<1>(p, pl, grad_out, depth, feats, proj, cells_dd, cells_df, prefix_arg, cursor, pairs,
                                        cap_arg, st, ps.epoch, ps.set_stride, nullptr, nullptr, ps.segs);
    if (rc != FBEV_OK) return rc;

    // texel pass: rows of grad_out are fp32, so 128-bit gathers need C % 4 == 0 and aligned rows
    const bool vec4 = p->channels % 4 == 0 && (uintptr_t)grad_out % 16 == 0;
    const int vec = vec4 ? 4 : 1;
    const int cq = (p->channels + vec - 1) / vec;
    const int lpr = cq < kWave ? cq : kWave;
    // One, two or four wavefronts per texel.  A texel's block is a chain of dependent loads (list bounds,
    // pairs, grad_out rows); small blocks fit the machine in fewer generations, large ones shorten the
    // chain of a long list.  What is known here is only how many samples a texel could get if every one were
    // kept, and that the categorical model, or a threshold of zero, keeps about twice as many as the parametric
    // models under a threshold.  Measured (us for 1 / 2 / 4 wavefronts; Laplace, then the categorical model):
    // 23 possible samples per texel 8.2 / 8.9 / 10.4 and 8.2 / 8.7 / 10.1; 186 per texel and 4224 texels
    // 17.3 / 18.2 / 23.5 and 32.6 / 26.1 / 30.4; 227: 21.6 / 20.5 / 24.8 and 41.0 / 33.5 / 34.5; 454: 33.0 / 26.1 / 28.2
    // and 64.9 / 49.4 / 46.8; 681: 39.7 / 30.9 / 31.5 and 90.2 / 65.9 / 59.5; 909: 44.5 / 33.8 / 33.6 and
    // 114.5 / 82.4 / 71.2; 1818: 102.8 / 70.0 / 53.3 and 287.2 / 204.4 / 133.5.  With more texels: 186 per texel on
    // 33 792 texels 56.8 / 80.3 / 135.1 and 94.0 / 113.2 / 163.6, on 67 584 texels 111.9 / 160.4 / 266.4 and
    // 210.6 / 247.6 / 349.0; 909 per texel on 8448 texels 124.7 / 92.0 / 88.1 and 218.9 / 160.2 / 152.3, on 33 792
    // texels 390.6 / 337.6 / 344.1 and 655.5 / 554.4 / 567.4.
    const uint64_t per_texel = fbev_backward_max_pairs(p) / (uint64_t)texels;
    const bool keeps_most = p->depth_distribution == FBEV_CATEGORICAL || !(p->depth_weight_threshold > 0.0f);
    const uint64_t expected = per_texel * (keeps_most ? 2 : 1);
    int texel_waves = expected < kTexelOneWaveBelow ? 1 : (expected < kTexelTwoWavesBelow ? 2 : kWavesPerBlock);
    if (texel_waves == 2 && texels * texel_waves > kTexelWavesAtOnce) texel_waves = 1;
    const int nw = (kWave / lpr) * texel_waves;
    // the depth gradient rides on the pairs exactly when the cell pass folds it in (one channel pass
    // and room for the depth bin in a pair's first word)
    const int from_pairs =
        (d_depth != nullptr && pl.k.C <= pl.k.lanes_per_slot * pl.vec * pl.cpl && pl.k.bin_bits >= 0) ? 1 : 0;
    const size_t lds = ((size_t)texel_waves * kWave * 2 + (size_t)nw * (lpr * vec + 2) +
                        (p->depth_distribution == FBEV_CATEGORICAL ? p->depth_bins : 0)) * sizeof(float);
    // (the blocks of a split texel add their shares with atomics, which needs cleared buffers: a
    // persistent workspace, whose calls clear nothing, keeps one block per texel)
    long long want_split = persistent ? 1 : kTexelSplitBelow / texels;
    const unsigned n_split = (unsigned)(want_split < 1 ? 1 : (want_split > kTexelMaxSplit ? kTexelMaxSplit : want_split));
    prof::Scope timer(prof::kBackwardTexel, st);
    const dim3 tgrid((unsigned)texels, n_split), tblock(kWave * texel_waves);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, tgrid, tblock, lds, st, pl.k, grad_out, prefix_arg, cursor, pairs, cap_arg, d_depth, d_feats,
                           lpr, from_pairs, accumulate ? 0 : 1, ps);
    };
    // (rows of a grad_out below 4 GiB are addressed with 32-bit byte offsets)
    const bool narrow = (uint64_t)p->batch * p->grid_y * p->grid_x * p->channels * sizeof(float) < (1ull << 32);
    auto launch_waves = [&](auto vec_tag, auto narrow_tag) {
        constexpr int V = decltype(vec_tag)::value;
        constexpr bool N = decltype(narrow_tag)::value;
        if (texel_waves == 1) launch(fbev_backward_texel_kernel<V, 1, N>);
        else if (texel_waves == 2) launch(fbev_backward_texel_kernel<V, 2, N>);
        else launch(fbev_backward_texel_kernel<V, kWavesPerBlock, N>);
    };
    using std::integral_constant;
    if (vec4) {
        if (narrow) launch_waves(integral_constant<int, 4>{}, integral_constant<bool, true>{});
        else launch_waves(integral_constant<int, 4>{}, integral_constant<bool, false>{});
    } else {
        if (narrow) launch_waves(integral_constant<int, 1>{}, integral_constant<bool, true>{});
        else launch_waves(integral_constant<int, 1>{}, integral_constant<bool, false>{});
    }
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

// Zero-fill everything of a persistent workspace but its pairs.
int workspace_init_impl(const fbev_problem *p, void *workspace, size_t workspace_bytes, hipStream_t st) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!workspace) return FBEV_ERR_NULL;
    if ((uintptr_t)workspace % 16) return FBEV_ERR_ALIGNMENT;
    const PersistLayout lay = persist_layout(p);
    if (workspace_bytes < lay.pairs) return FBEV_ERR_SHAPE;
    return launch_zero(static_cast<int *>(workspace), (long long)(lay.pairs / sizeof(int)), nullptr, 0, nullptr, 0, st);
}

// Prepare a persistent workspace whose segments are sized by the geometry: zero-fill everything but the pairs,
// count the samples in view per segment (no depth model: an upper bound of what any depth tensor and threshold
// keep), and prefix-sum the counts into the segments' starts.
int workspace_init_sized_impl(const fbev_problem *p, const float *proj, void *workspace, size_t workspace_bytes,
                              hipStream_t st) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!workspace || !proj) return FBEV_ERR_NULL;
    if ((uintptr_t)workspace % 16 || (uintptr_t)proj % 4) return FBEV_ERR_ALIGNMENT;
    if (sample_count(p) >= (1ll << 31) || counter_count(p) >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
    const PersistLayout lay = persist_layout(p, true);
    if (workspace_bytes < lay.pairs) return FBEV_ERR_SHAPE;
    rc = launch_zero(static_cast<int *>(workspace), (long long)(lay.pairs / sizeof(int)), nullptr, 0, nullptr, 0, st);
    if (rc != FBEV_OK) return rc;
    fbev_problem q = *p;      // the samples in view depend on the geometry only
    q.channels = 4; q.in_dtype = FBEV_F32; q.depth_distribution = FBEV_GAUSSIAN; q.depth_bins = 2;
    q.reduction = FBEV_REDUCE_MEAN;
    Plan pl;
    rc = make_plan(&q, true, &pl, kCellPassWaves);
    if (rc != FBEV_OK) return rc;
    char *base = static_cast<char *>(workspace);
    int *seg_cap = reinterpret_cast<int *>(base + lay.seg_cap), *seg_off = reinterpret_cast<int *>(base + lay.seg_off);
    int *seg_prefix = reinterpret_cast<int *>(base + lay.seg_prefix);
    rc = launch_count<float, true>(pl, nullptr, proj, seg_cap, st);
    if (rc != FBEV_OK) return rc;
    if (hipMemcpyAsync(seg_off, seg_cap, (size_t)lay.segments * sizeof(int), hipMemcpyDeviceToDevice, st) != hipSuccess)
        return FBEV_ERR_LAUNCH;
    {
        prof::Scope timer(prof::kScanChunks, st);
        hipLaunchKernelGGL(fbev_scan_chunks_kernel, dim3((unsigned)lay.seg_chunks), dim3(1024), 0, st, seg_off,
                           lay.segments, seg_prefix);
    }
    if (hipGetLastError() != hipSuccess) return FBEV_ERR_LAUNCH;
    {
        // (one entry more than there are chunks, zero so far: it receives the total)
        prof::Scope timer(prof::kScanSums, st);
        hipLaunchKernelGGL(fbev_scan_sums_kernel, dim3(1), dim3(1024), 0, st, seg_prefix, (int)lay.seg_chunks + 1);
    }
    if (hipGetLastError() != hipSuccess) return FBEV_ERR_LAUNCH;
    hipLaunchKernelGGL(fbev_segment_table_kernel, dim3((unsigned)((lay.segments + 255) / 256)), dim3(256), 0, st,
                       lay.segments, seg_cap, seg_off, seg_prefix, reinterpret_cast<int2 *>(base + lay.seg_tab),
                       reinterpret_cast<int *>(base + lay.sets), lay.set_stride);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int fbev_forward(const fbev_problem *p, const void *depth, const void *feats, const float *proj, float *out,
                 float *count_out, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!depth || !feats || !proj || !out) return FBEV_ERR_NULL;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)proj % 4 || (uintptr_t)out % 4 ||
        (uintptr_t)count_out % 4)
        return FBEV_ERR_ALIGNMENT;
    Plan pl;
    // 128-bit gathers and stores need 16-byte aligned feature and result tensors
    // measured: the forward is fastest with at most 4 rounds per wavefront, the backward's cell pass with 8
    // More cells per round pay for the LDS here (measured with 64 channels on a 400x400 grid: 20 height bins
    // 185 -> 166 us, 40 bins 785 -> 476 us); the cell pass of the backward is better off with the smaller budget.
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)out % 16 == 0, &pl, kCellPassWaves, 4);
    if (rc != FBEV_OK) return rc;
    return dispatch_forward(p, pl, depth, feats, proj, out, count_out, static_cast<hipStream_t>(stream));
}

size_t fbev_sample_store_bytes(const fbev_problem *p) {
    if (validate(p, true) != FBEV_OK) return 0;
    return sample_store_bytes(p);
}

int fbev_forward_store(const fbev_problem *p, const void *depth, const void *feats, const float *proj, float *out,
                       float *count_out, void *store, size_t store_bytes, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!depth || !feats || !proj || !out || !count_out || !store) return FBEV_ERR_NULL;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)proj % 4 || (uintptr_t)out % 4 ||
        (uintptr_t)count_out % 4 || (uintptr_t)store % 16)
        return FBEV_ERR_ALIGNMENT;
    const size_t need = sample_store_bytes(p);
    if (need == 0) return FBEV_ERR_TOO_LARGE;
    if (store_bytes < need) return FBEV_ERR_SHAPE;
    Plan pl;
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)out % 16 == 0, &pl, kCellPassWaves, 4);
    if (rc != FBEV_OK) return rc;
    return dispatch_forward(p, pl, depth, feats, proj, out, count_out, static_cast<hipStream_t>(stream),
                            static_cast<float4 *>(store));
}

size_t fbev_geometry_cache_bytes(const fbev_problem *p) {
    if (validate(p, false) != FBEV_OK) return 0;
    return geometry_cache_bytes(p);
}

int fbev_geometry_cache_build(const fbev_problem *p, const float *proj, void *cache, size_t cache_bytes, void *stream) {
    int rc = validate(p, false);
    if (rc != FBEV_OK) return rc;
    if (!proj || !cache) return FBEV_ERR_NULL;
    if ((uintptr_t)proj % 4 || (uintptr_t)cache % 16) return FBEV_ERR_ALIGNMENT;
    const size_t need = geometry_cache_bytes(p);
    if (need == 0) return FBEV_ERR_TOO_LARGE;
    if (cache_bytes < need) return FBEV_ERR_SHAPE;
    fbev_problem q = *p;      // the lists depend on the geometry only
    q.channels = 4; q.in_dtype = FBEV_F32; q.depth_distribution = FBEV_GAUSSIAN; q.depth_bins = 2;
    q.reduction = FBEV_REDUCE_MEAN;
    Plan pl;
    rc = make_plan(&q, true, &pl, kCellPassWaves, 4);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t lds = pl.lds_fwd;         // sized for two-word entries: more than the one-word lists need
    if (!lds_opt_in(fbev_geometry_cache_kernel, lds)) return FBEV_ERR_LAUNCH;
    prof::Scope timer(prof::kGeometryCache, st);
    hipLaunchKernelGGL(fbev_geometry_cache_kernel, dim3(pl.k.n_blocks), dim3(kWave * pl.k.waves), lds, st, pl.k, proj,
                       cache);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int fbev_forward_cached(const fbev_problem *p, const void *depth, const void *feats, const void *cache,
                        size_t cache_bytes, float *out, float *count_out, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!depth || !feats || !cache || !out) return FBEV_ERR_NULL;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)cache % 16 || (uintptr_t)out % 4 ||
        (uintptr_t)count_out % 4)
        return FBEV_ERR_ALIGNMENT;
    const size_t need = geometry_cache_bytes(p);
    if (need == 0) return FBEV_ERR_TOO_LARGE;
    if (cache_bytes < need) return FBEV_ERR_SHAPE;
    Plan pl;
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)out % 16 == 0, &pl, kCellPassWaves, 4);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_forward_cached<float, 4>(pl, depth, feats, cache, out, count_out, st)
                               : launch_forward_cached<float, 1>(pl, depth, feats, cache, out, count_out, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_forward_cached<__half, 8>(pl, depth, feats, cache, out, count_out, st)
                               : launch_forward_cached<__half, 1>(pl, depth, feats, cache, out, count_out, st);
        default:
            return pl.vec == 8 ? launch_forward_cached<bf16_raw, 8>(pl, depth, feats, cache, out, count_out, st)
                               : launch_forward_cached<bf16_raw, 1>(pl, depth, feats, cache, out, count_out, st);
    }
}

int fbev_backward(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                  const float *proj, float *d_depth, float *d_feats, int accumulate, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    rc = check_backward_args(p, grad_out, depth, feats, proj, d_depth, d_feats);
    if (rc != FBEV_OK) return rc;
    if (!d_depth && !d_feats) return FBEV_OK;
    Plan pl;
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0, &pl, kCellPassWaves);
    if (rc == FBEV_OK && pl.k.batch_groups > 1 && !cells_batch_pays<0>(p, pl))
        rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0, &pl, kCellPassWaves, 3,
                       kMaxSlotLdsBytes, 1);
    if (rc != FBEV_OK) return rc;
    if (!accumulate) {
        rc = launch_zero(nullptr, 0, d_depth, texel_count(p) * p->depth_bins, d_feats, texel_count(p) * p->channels,
                         static_cast<hipStream_t>(stream));
        if (rc != FBEV_OK) return rc;
    }
    return dispatch_cells<0>(p, pl, grad_out, depth, feats, proj, d_depth, d_feats, nullptr, nullptr, nullptr, 0,
                                 static_cast<hipStream_t>(stream));
}

size_t fbev_backward_columns_workspace_bytes(const fbev_problem *p) {
    if (validate(p, true) != FBEV_OK) return 0;
    return ((size_t)p->batch * p->grid_y * p->grid_x * sizeof(float) + 255) / 256 * 256;
}

int fbev_backward_columns(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                          const float *proj, const float *cell_count, float *d_depth, float *d_feats,
                          int accumulate, void *workspace, size_t workspace_bytes, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    rc = check_backward_args(p, grad_out, depth, feats, proj, d_depth, d_feats);
    if (rc != FBEV_OK) return rc;
    if ((uintptr_t)cell_count % 4 || (uintptr_t)workspace % 16) return FBEV_ERR_ALIGNMENT;
    if (!d_depth && !d_feats) return FBEV_OK;
    if (p->feat_h > 0xffff || (long long)p->batch * p->grid_y * p->grid_x >= (1ll << 30)) return FBEV_ERR_TOO_LARGE;
    Plan pl;
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0, &pl);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (cell_count == nullptr) {
        // recount: the forward's sample phase alone, counts into the workspace
        if (!workspace) return FBEV_ERR_NULL;
        if (workspace_bytes < fbev_backward_columns_workspace_bytes(p)) return FBEV_ERR_SHAPE;
        rc = dispatch_forward(p, pl, depth, feats, proj, nullptr, static_cast<float *>(workspace), st);
        if (rc != FBEV_OK) return rc;
        cell_count = static_cast<const float *>(workspace);
    }
    ColParams cp;
    cp.n_tiles = pl.k.tiles_x * pl.k.tiles_y;
    const int cq = (p->channels + pl.vec - 1) / pl.vec;
    cp.lanes_per_slot = cq < kWave ? cq : kWave;
    cp.slots = kWave / cp.lanes_per_slot;
    if (cp.slots * kColWaves > 64) cp.slots = 64 / kColWaves;
    cp.part_stride = (cp.lanes_per_slot * pl.vec + 2 + 3) / 4 * 4;
    cp.accumulate = accumulate != 0;
    cp.n_blocks = p->batch * p->num_cams * p->feat_w;
    if (p->feat_h > kColMaxRows || p->grid_x > 0xffff || p->grid_y > 0x7fff) return FBEV_ERR_TOO_LARGE;
    const size_t ints = (size_t)kColThreads + kColCells + 2 * kColEntries + 3 * kColMaxRows + 4 + 3 * 64 + kColEntries;
    const size_t lds = 8 * sizeof(float4) + (size_t)kColEntries * 32 + ints * sizeof(int) +
                       (size_t)kColWaves * cp.slots * cp.part_stride * sizeof(float);
    if (lds > (size_t)kLdsLimitBytes) return FBEV_ERR_TOO_LARGE;
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_columns<float, 4>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st)
                               : launch_columns<float, 1>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_columns<__half, 8>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st)
                               : launch_columns<__half, 1>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st);
        default:
            return pl.vec == 8 ? launch_columns<bf16_raw, 8>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st)
                               : launch_columns<bf16_raw, 1>(pl, cp, lds, grad_out, depth, feats, proj, cell_count, d_depth, d_feats, st);
    }
}

uint64_t fbev_backward_max_pairs(const fbev_problem *p) {
    if (validate(p, true) != FBEV_OK) return 0;
    return (uint64_t)sample_count(p);        // one pair per sample
}

size_t fbev_backward_workspace_bytes(const fbev_problem *p, uint64_t pair_capacity) {
    if (validate(p, true) != FBEV_OK) return 0;
    return ws_index_bytes(p) + (size_t)pair_capacity * sizeof(Pair);
}

int fbev_backward_gather(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                         const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                         size_t workspace_bytes, void *stream) {
    return backward_gather_impl(p, grad_out, depth, feats, proj, d_depth, d_feats, accumulate, workspace,
                                workspace_bytes, stream);
}

size_t fbev_backward_persistent_workspace_bytes(const fbev_problem *p) {
    if (validate(p, true) != FBEV_OK) return 0;
    // room for every sample, and never less than the shortest segment the fixed layout works with
    const uint64_t least = (uint64_t)texel_count(p) * kFixedReplicas * kFixedMinSegment;
    const uint64_t pairs = fbev_backward_max_pairs(p) > least ? fbev_backward_max_pairs(p) : least;
    return persist_layout(p).pairs + (size_t)pairs * sizeof(Pair);
}

int fbev_backward_workspace_init(const fbev_problem *p, void *workspace, size_t workspace_bytes, void *stream) {
    return workspace_init_impl(p, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int fbev_backward_gather_persistent(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                                    const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    return backward_gather_impl(p, grad_out, depth, feats, proj, d_depth, d_feats, accumulate, workspace,
                                workspace_bytes, stream, 1);
}

size_t fbev_backward_sized_workspace_bytes(const fbev_problem *p, uint64_t pair_capacity) {
    if (validate(p, true) != FBEV_OK) return 0;
    return persist_layout(p, true).pairs + (size_t)pair_capacity * sizeof(Pair);
}

size_t fbev_backward_sized_total_offset(const fbev_problem *p) {
    if (validate(p, true) != FBEV_OK) return 0;
    const PersistLayout lay = persist_layout(p, true);
    return lay.seg_prefix + (size_t)lay.seg_chunks * sizeof(int);
}

int fbev_backward_workspace_init_sized(const fbev_problem *p, const float *proj, void *workspace, size_t workspace_bytes,
                                       void *stream) {
    return workspace_init_sized_impl(p, proj, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int fbev_backward_gather_sized(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                               const float *proj, float *d_depth, float *d_feats, int accumulate, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return backward_gather_impl(p, grad_out, depth, feats, proj, d_depth, d_feats, accumulate, workspace,
                                workspace_bytes, stream, 2);
}

int fbev_backward_gather_stored(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                                const float *proj, const float *cell_count, const void *store, size_t store_bytes,
                                float *d_depth, float *d_feats, int accumulate, void *workspace, size_t workspace_bytes,
                                int persistent, void *stream) {
    if (!store) return FBEV_ERR_NULL;
    return backward_gather_impl(p, grad_out, depth, feats, proj, d_depth, d_feats, accumulate, workspace,
                                workspace_bytes, stream, persistent, cell_count, store, store_bytes);
}

int fbev_backward_gather_static(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                                const float *proj, float *d_depth, float *d_feats, int accumulate, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    // the per-kernel timers create HIP events: not in a call that promises to allocate nothing
    if (prof::enabled.load(std::memory_order_relaxed)) return FBEV_ERR_UNSUPPORTED;
    // the scratch array must hold the worst case of one pair per sample (fixed segments, three launches, where a
    // segment then has room for four pairs or more; the counted layout, which allocates nothing either, otherwise)
    const uint64_t max_pairs = fbev_backward_max_pairs(p);
    if (max_pairs >= (1ull << 31) || ws_index_bytes(p) + (size_t)max_pairs * sizeof(Pair) > (size_t)FBEV_STATIC_SCRATCH_BYTES)
        return FBEV_ERR_TOO_LARGE;
    void *ws = nullptr;
    rc = scratch_of_current_device(&ws);
    if (rc != FBEV_OK) return rc;
    return backward_gather_impl(p, grad_out, depth, feats, proj, d_depth, d_feats, accumulate, ws, (size_t)FBEV_STATIC_SCRATCH_BYTES,
                                stream);
}

size_t fbev_static_scratch_bytes(void) { return (size_t)FBEV_STATIC_SCRATCH_BYTES; }

int fbev_pillarpool_forward(const fbev_pillar_problem *p, const float *depth, const float *feats,
                            const float *u_coords, const float *v_coords, const float *z_coords,
                            const int32_t *batch_camera, const int32_t *ranks_bev, const int32_t *interval_starts,
                            const int32_t *interval_lengths, float *out, void *stream) {
    if (!p) return FBEV_ERR_NULL;
    if (p->channels <= 0 || p->n_intervals < 0 || p->batch <= 0 || p->num_cams <= 0 || p->feat_h <= 0 || p->feat_w <= 0)
        return FBEV_ERR_SHAPE;
    if (p->depth_distribution != FBEV_GAUSSIAN && p->depth_distribution != FBEV_LAPLACE) return FBEV_ERR_UNSUPPORTED;
    if (p->n_intervals == 0) return FBEV_OK;
    if (!depth || !feats || !u_coords || !v_coords || !z_coords || !batch_camera || !ranks_bev || !interval_starts ||
        !interval_lengths || !out)
        return FBEV_ERR_NULL;
    if ((uintptr_t)depth % 8 || (uintptr_t)feats % 4 || (uintptr_t)u_coords % 4 || (uintptr_t)v_coords % 4 ||
        (uintptr_t)z_coords % 4 || (uintptr_t)batch_camera % 4 || (uintptr_t)ranks_bev % 4 ||
        (uintptr_t)interval_starts % 4 || (uintptr_t)interval_lengths % 4 || (uintptr_t)out % 4)
        return FBEV_ERR_ALIGNMENT;
    if ((long long)p->batch * p->num_cams * p->feat_h * p->feat_w >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
    const bool vec4 = p->channels % 4 == 0 && (uintptr_t)feats % 16 == 0;
    const int vec = vec4 ? 4 : 1;
    const int cq = (p->channels + vec - 1) / vec;
    const int lps = cq < kWave ? cq : kWave;
    const int per_block = (kWave / lps) * kWavesPerBlock;
    const long long blocks = ((long long)p->n_intervals + per_block - 1) / per_block;
    if (blocks >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
    hipStream_t st = static_cast<hipStream_t>(stream);
    prof::Scope timer(prof::kPillar, st);
    if (vec4)
        hipLaunchKernelGGL((fbev_pillar_kernel<4>), dim3((unsigned)blocks), dim3(kWave * kWavesPerBlock), 0, st,
                           p->channels, p->n_intervals, p->feat_h, p->feat_w, lps, p->epsilon,
                           p->depth_distribution == FBEV_LAPLACE ? 1 : 0, depth, feats, u_coords, v_coords, z_coords,
                           batch_camera, ranks_bev, interval_starts, interval_lengths, out);
    else
        hipLaunchKernelGGL((fbev_pillar_kernel<1>), dim3((unsigned)blocks), dim3(kWave * kWavesPerBlock), 0, st,
                           p->channels, p->n_intervals, p->feat_h, p->feat_w, lps, p->epsilon,
                           p->depth_distribution == FBEV_LAPLACE ? 1 : 0, depth, feats, u_coords, v_coords, z_coords,
                           batch_camera, ranks_bev, interval_starts, interval_lengths, out);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int fbev_sample_geometry(const fbev_problem *p, const float *proj, uint8_t *mask, int32_t *idx, float *frac,
                         void *stream) {
    int rc = validate(p, false);
    if (rc != FBEV_OK) return rc;
    if (!proj) return FBEV_ERR_NULL;
    if ((uintptr_t)proj % 4 || (uintptr_t)idx % 4 || (uintptr_t)frac % 4) return FBEV_ERR_ALIGNMENT;
    fbev_problem q = *p;
    q.channels = 1; q.in_dtype = FBEV_F32; q.depth_distribution = FBEV_GAUSSIAN; q.depth_bins = 2;
    q.reduction = FBEV_REDUCE_MEAN;
    Plan pl;
    rc = make_plan(&q, false, &pl);
    if (rc != FBEV_OK) return rc;
    const long long total = (long long)p->batch * p->grid_y * p->grid_x * p->num_cams * p->grid_z;
    const long long blocks = (total + 255) / 256;
    if (blocks >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
    prof::Scope timer(prof::kGeometry, static_cast<hipStream_t>(stream));
    hipLaunchKernelGGL(fbev_geometry_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), pl.k, proj, mask, idx, frac, total);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int fbev_projection_matrices(const float *sensor2ego, const float *camera2imgs, const float *post_rots,
                             const float *post_trans, float *proj, int32_t count, void *stream) {
    if (count < 0) return FBEV_ERR_SHAPE;
    if (count == 0) return FBEV_OK;
    if (!sensor2ego || !camera2imgs || !post_rots || !post_trans || !proj) return FBEV_ERR_NULL;
    if ((uintptr_t)sensor2ego % 4 || (uintptr_t)camera2imgs % 4 || (uintptr_t)post_rots % 4 || (uintptr_t)post_trans % 4 ||
        (uintptr_t)proj % 4)
        return FBEV_ERR_ALIGNMENT;
    hipStream_t st = static_cast<hipStream_t>(stream);
    prof::Scope timer(prof::kProjection, st);
    hipLaunchKernelGGL(fbev_projection_kernel, dim3((unsigned)((count + 63) / 64)), dim3(64), 0, st, (int)count,
                       sensor2ego, camera2imgs, post_rots, post_trans, proj);
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

uint64_t fbev_algorithmic_bytes(const fbev_problem *p, int backward) {
    if (validate(p, true) != FBEV_OK) return 0;
    const uint64_t es = (uint64_t)elem_size(p->in_dtype);
    const uint64_t texels = (uint64_t)p->batch * p->num_cams * p->feat_h * p->feat_w;
    const uint64_t feats = texels * p->channels * es;
    const uint64_t depth = texels * p->depth_bins * es;
    const uint64_t mats = (uint64_t)p->batch * p->num_cams * 48;
    const uint64_t bev = (uint64_t)p->batch * p->grid_y * p->grid_x * p->channels * 4;
    if (!backward) return feats + depth + mats + bev;
    return bev + feats + depth + mats + texels * p->channels * 4 + texels * p->depth_bins * 4;
}

const char *fbev_status_string(int status) {
    switch (status) {
        case FBEV_OK: return "ok";
        case FBEV_ERR_NULL: return "a required pointer is NULL";
        case FBEV_ERR_SHAPE: return "a size is non-positive or inconsistent";
        case FBEV_ERR_UNSUPPORTED: return "unsupported dtype, depth model or reduction";
        case FBEV_ERR_TOO_LARGE: return "problem too large for the 32-bit indices / LDS lists used";
        case FBEV_ERR_ALIGNMENT: return "a pointer is not aligned to its element type";
        case FBEV_ERR_LAUNCH: return "HIP reported a kernel launch error";
        default: return "unknown status";
    }
}

int fbev_profile_enable(int on) {
    std::lock_guard<std::mutex> g(prof::mu);
    for (auto &r : prof::recs) { (void)hipEventDestroy(r.a); (void)hipEventDestroy(r.b); }
    prof::recs.clear();
    prof::enabled.store(on != 0);
    return FBEV_OK;
}

int fbev_profile_kernel_count(void) { return prof::kNum; }

const char *fbev_profile_kernel_name(int kernel) {
    return (kernel >= 0 && kernel < prof::kNum) ? prof::kNames[kernel] : "";
}

int fbev_profile_collect(double *total_ms, int64_t *calls) {
    if (!total_ms || !calls) return FBEV_ERR_NULL;
    std::lock_guard<std::mutex> g(prof::mu);
    for (int i = 0; i < prof::kNum; ++i) { total_ms[i] = 0.0; calls[i] = 0; }
    int rc = FBEV_OK;
    for (auto &r : prof::recs) {
        float ms = 0.0f;
        if (hipEventSynchronize(r.b) != hipSuccess || hipEventElapsedTime(&ms, r.a, r.b) != hipSuccess) rc = FBEV_ERR_LAUNCH;
        total_ms[r.kid] += ms;
        calls[r.kid] += 1;
        (void)hipEventDestroy(r.a);
        (void)hipEventDestroy(r.b);
    }
    prof::recs.clear();
    return rc;
}

int fbev_abi_version(void) { return FBEV_ABI_VERSION; }
size_t fbev_problem_size(void) { return sizeof(fbev_problem); }

}  // extern "C"
