// The forward kernel.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// ---------------------------------------------------------------- forward
// How the lanes of a wavefront share the slots in phase B.
struct LaneRole {
    int gps;        // lane groups per slot
    int slot, sub;  // this lane's slot and its group's index among the slot's groups
    int lis;        // lane within the group
    bool carrier;   // the lane belongs to a slot
    int span;       // channels covered per pass
};

template <int VEC, int CPL>
__device__ __forceinline__ LaneRole lane_role(const KParams &k, int lane) {
    LaneRole r;
    // a lane group covers the channels of one cell; when long lists leave room for few slots,
    // several groups share a slot and take its entries in turn
    r.gps = k.groups_per_slot;
    const int group = (int)(((unsigned)lane * k.lps_magic) >> 16);       // lane / lanes_per_slot
    r.slot = (int)(((unsigned)group * k.gps_magic) >> 16);              // group / groups per slot
    r.sub = group - r.slot * r.gps;
    r.lis = lane - group * k.lanes_per_slot;
    r.carrier = r.slot < k.slots;
    r.span = k.lanes_per_slot * VEC * CPL;
    return r;
}

// Phase B of one group of a batch: every slot walks its cell's list of kept samples (the sample phase
// left the entries, where each cell's start, their number and the cells in LDS) and stores its
// cell's row of the output.
// STREAM: the output is stored with non-temporal stores (a template parameter: as a run-time
// choice between two stores the compiler merges them into one ordinary store).
template <typename T, int VEC, int CPL, bool STREAM>
__device__ __forceinline__ void forward_phase_b(const KParams &k, const WaveLds &L, const LaneRole &role, int b,
                                                int group, const T *__restrict__ feats, float *__restrict__ out,
                                                float *__restrict__ count_out) {
    lds_counter *cnt = L.cnt;
    const float4 *lst = L.lst;
    const int gps = role.gps, sub = role.sub, lis = role.lis, span = role.span;
    const bool carrier = role.carrier;
    const int slot = carrier ? group * k.slots + role.slot : 0;      // the lane's cell within the batch
    // a feature row starts at a 32-bit byte offset from the tensor's base: uniform base + 32-bit lane offset
    const char *fbytes = reinterpret_cast<const char *>(feats);
    auto row_at = [&](unsigned byte_offset) { return reinterpret_cast<const T *>(fbytes + byte_offset); };
    {
        // phase A left the slot's cell in LDS: valid flag and ix | iy << 16
        const float4 mycell = L.cell[slot];
        const int ix = __float_as_int(mycell.w) & 0xffff, iy = __float_as_int(mycell.w) >> 16;
        const bool mine = carrier && mycell.z != 0.0f;
        const int n = mine ? cnt[slot] : 0;
        const float4 *my = lst + (size_t)L.start[slot] * 2;
        // (the count: the number of samples that enter the mean; the backward pass can reuse it)
        const unsigned cell_index = (unsigned)((b * k.gy + iy) * k.gx + ix);       // fits: the plan checks B * gy * gx
        if (count_out != nullptr && mine && lis == 0 && sub == 0) count_out[cell_index] = (float)n;
        float *o = out + (size_t)cell_index * k.C;
        for (int c0 = 0; out != nullptr && c0 < k.C; c0 += span) {
            float acc[CPL][VEC];
#pragma unroll
            for (int j = 0; j < CPL; ++j)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[j][v] = 0.0f;
            // one entry: four row loads per channel vector, then the weighted sum
            auto gather = [&](int e) {
                float4 w = my[2 * e];
                float4 tf = my[2 * e + 1];
                const unsigned o00 = (unsigned)__float_as_int(tf.x), o01 = (unsigned)__float_as_int(tf.y);
                const unsigned o10 = (unsigned)__float_as_int(tf.z), o11 = (unsigned)__float_as_int(tf.w);
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        const unsigned chb = (unsigned)ch * (unsigned)sizeof(T);
                        float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                        VecLoad<T, VEC>::ld(row_at(o00 + chb), f00);
                        VecLoad<T, VEC>::ld(row_at(o01 + chb), f01);
                        VecLoad<T, VEC>::ld(row_at(o10 + chb), f10);
                        VecLoad<T, VEC>::ld(row_at(o11 + chb), f11);
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            float a = acc[j][v];
                            a = __builtin_fmaf(w.x, f00[v], a);
                            a = __builtin_fmaf(w.y, f01[v], a);
                            a = __builtin_fmaf(w.z, f10[v], a);
                            a = __builtin_fmaf(w.w, f11[v], a);
                            acc[j][v] = a;
                        }
                    }
                }
            };
            // two entries per trip where the registers allow, all eight row loads issued before the
            // first is used (the loop is a chain of gather latencies, not of arithmetic)
            // (group `sub` of the slot takes the entry pairs sub, sub + gps, ...)
            if (CPL == 1) {
                const int ch = c0 + lis * VEC;
                const unsigned chb = (unsigned)ch * (unsigned)sizeof(T);
                int e = 2 * sub;
                for (; ch < k.C && e + 1 < n; e += 2 * gps) {
                    const float4 wa = my[2 * e], ta = my[2 * e + 1], wb = my[2 * e + 2], tb = my[2 * e + 3];
                    const int off[8] = {__float_as_int(ta.x), __float_as_int(ta.y), __float_as_int(ta.z), __float_as_int(ta.w),
                                        __float_as_int(tb.x), __float_as_int(tb.y), __float_as_int(tb.z), __float_as_int(tb.w)};
                    const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
                    float f[8][VEC];
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        VecLoad<T, VEC>::ld(row_at((unsigned)off[c] + chb), f[c]);
#pragma unroll
                    for (int c = 0; c < 8; ++c)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) acc[0][v] = __builtin_fmaf(wv[c], f[c][v], acc[0][v]);
                }
                if (e < n) gather(e);       // the odd entry at the end falls to one group
            } else {
                for (int e = sub; e < n; e += gps) gather(e);
            }
            // the groups of a slot add up in its first group
            if (gps > 1) {
#pragma unroll
                for (int jj = 0; jj < CPL; ++jj)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        const float part = acc[jj][v];
                        float sum = part;
                        for (int j = 1; j < gps; ++j) sum += __shfl_down(part, j * k.lanes_per_slot, kWave);
                        acc[jj][v] = sum;
                    }
            }
            if (mine && sub == 0) {
                // the mean as a product with 1/n (one division per cell instead of one per channel;
                // it can differ from the quotient in the last place)
                const float scale = k.reduce_sum ? 1.0f : (n > 0 ? 1.0f / (float)n : 0.0f);
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        float res[VEC];
#pragma unroll
                        for (int v = 0; v < VEC; ++v) res[v] = acc[j][v] * scale;
                        if (VEC == 1) {
                            o[ch] = res[0];
                        } else {
#pragma unroll
                            for (int v = 0; v < VEC; v += 4) {
                                // an output too large for the L2s is streamed past them: it is written
                                // once, and what the next kernel reads stays cached instead
                                typedef float float4v __attribute__((ext_vector_type(4)));
                                const float4v row = {res[v], res[v + 1], res[v + 2], res[v + 3]};
                                if (STREAM) __builtin_nontemporal_store(row, reinterpret_cast<float4v *>(o + ch + v));
                                else *reinterpret_cast<float4v *>(o + ch + v) = row;
                            }
                        }
                    }
                }
            }
        }
    }
}

// STORE: the forward of a call that will be differentiated also leaves every kept sample's record in
// `store` (see kModeForwardStore), so that the backward's cell pass need not evaluate the samples again.
template <typename T, int VEC, int CPL, bool STREAM, bool BATCHED, bool STORE = false>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_forward_kernel(
    KParams k, const T *__restrict__ depth, const T *__restrict__ feats, const float *__restrict__ proj,
    float *__restrict__ out, float *__restrict__ count_out, float4 *__restrict__ store = nullptr) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = batch_of(k, bid);
    const int blk = bid - b * k.blocks_per_batch;

    const WaveLds L = block_lds_setup(k, smem, proj, b, 2);
    const LaneRole role = lane_role<VEC, CPL>(k, lane);
    const int cells_per_wave = k.slots_a * k.rounds;
    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots_a;
        if (q0 >= k.padded_cells) break;
        const int n_cand = phase_a_candidates<BATCHED>(k, L, q0, lane);
        // all groups of the batch through stage 2 together when the pool is sure to hold what they keep
        const int n_groups = BATCHED ? k.batch_groups : 1;
        const int step = n_cand <= k.pool_cap ? n_groups : 1;
        for (int g = 0; g < n_groups; g += step) {
            phase_a_samples<2, T, STORE ? kModeForwardStore : kModeForward>(
                k, L, depth, b, lane, BATCHED ? L.gcand[g] : 0, BATCHED ? L.gcand[g + step] : n_cand, nullptr, nullptr, 0,
                STORE ? store + ((size_t)b * k.padded_cells + q0) * k.NZ * 2 : nullptr);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            for (int j = g; j < g + step; ++j) forward_phase_b<T, VEC, CPL, STREAM>(k, L, role, b, j, feats, out, count_out);
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// ---------------------------------------------------------------- forward on cached geometry
// The samples in view depend on the calibration and the grid only.  When those repeat from call to
// call (a fixed rig at inference), fbev_geometry_cache_build keeps, per cell, the compacted list of
// its samples in view -- 16 bytes each: the bilinear fractions, the first corner texel with the two
// clamp flags below it, and the sample's depth along the optical axis, exactly the values the sample
// phase computes -- and this kernel starts from those lists: no matrices, no column cull, no
// projection, no divisions; the depth model, the weight threshold and phase B are the same code, on
// the same values in the same order, so the results are the same bit for bit.
// Cache layout: [256 bytes: header][B * padded_cells int32: samples in view per cell, cells in the
// order of the tiled walk][B * padded_cells * NZ entries].
constexpr int kCacheHeaderBytes = 256;
constexpr int kCacheMagic = 0x46424743;      // "FBGC"

__device__ __forceinline__ const int *cache_counts(const void *cache) {
    return reinterpret_cast<const int *>(static_cast<const char *>(cache) + kCacheHeaderBytes);
}
__host__ __device__ inline size_t cache_entries_offset(long long cells) {
    return (size_t)kCacheHeaderBytes + ((size_t)cells * sizeof(int) + 255) / 256 * 256;
}

// Sample phase on cached geometry: lanes = the cached samples of the round's cells, densely packed.
template <typename T>
__device__ __forceinline__ void phase_a_cached(const KParams &k, const WaveLds &L, const T *__restrict__ depth,
                                               const int *__restrict__ counts, const float4 *__restrict__ entries,
                                               int b, int q0, int lane) {
    if (lane < k.slots) {
        L.cnt[lane] = 0;
        L.start[lane] = lane * k.NZ;      // a cell's entries start at its own stretch of the pool here
    }
    // lane s < slots: its cell, the number of cached samples, and where they start among the round's
    int mine_n = 0;
    if (lane < k.slots) {
        int ix = 0, iy = 0;
        const bool ok = cell_of(k, q0 + lane, ix, iy);
        mine_n = ok ? counts[(size_t)b * k.padded_cells + q0 + lane] : 0;
        L.cell[lane] = make_float4(0.0f, 0.0f, ok ? 1.0f : 0.0f, __int_as_float(ix | (iy << 16)));
    }
    int incl = mine_n;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        const int other = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += other;
    }
    const int total = __shfl(incl, 15, kWave);        // slots <= 16; lanes past the slots carry 0
    const int my_start = incl - mine_n;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const float4 *base = entries + ((size_t)b * k.padded_cells + q0) * k.NZ;
    for (int jb = 0; jb < total; jb += kWave) {
        const int j = jb + lane;
        const bool active = j < total;
        // the slot whose range holds j: the last one that starts at or before j (empty slots start
        // where the next one does, so later ones win)
        int slot = 0;
        for (int s = 1; s < k.slots; ++s) slot = (__shfl(my_start, s, kWave) <= j) ? s : slot;
        const int first = __shfl(my_start, slot, kWave);
        float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f);
        int4 tx = make_int4(0, 0, 0, 0);
        bool keep = false;
        if (active) {
            const float4 c = base[(size_t)slot * k.NZ + (j - first)];
            const float du = c.x, dv = c.y;
            const int code = __float_as_int(c.z), t00 = code >> 2;
            const float w00 = (1.0f - du) * (1.0f - dv);
            const float w01 = (1.0f - du) * dv;
            const float w10 = du * (1.0f - dv);
            const float w11 = du * dv;
            const int t01 = t00 + ((code & 2) ? k.W : 0), t10 = t00 + (code & 1), t11 = t01 + (code & 1);
            DepthEval e = eval_depth<T>(k, depth, t00, t01, t10, t11, w00, w01, w10, w11, c.w);
            keep = e.keep;
            tx = make_int4(t00, t01, t10, t11);
            w0 = make_float4(w00 * e.wgt, w01 * e.wgt, w10 * e.wgt, w11 * e.wgt);
        }
        const int slot_eff = active ? slot : 16 + (lane & 1);       // idle lanes: no real slot
        const int prev_slot = __shfl_up(slot_eff, 1, kWave);
        // the lanes of one slot are contiguous: [lo, hi)
        const unsigned long long bm = __ballot(lane == 0 || slot_eff != prev_slot);
        const unsigned long long m = __ballot(keep);
        const int lo = 63 - __clzll(bm & lanemask_le(lane));
        const unsigned long long above = lane == 63 ? 0ull : (bm & ~lanemask_le(lane));
        const int hi = above ? __ffsll((long long)above) - 1 : kWave;
        const unsigned long long seg = (~0ull << lo) & (hi >= 64 ? ~0ull : ((1ull << hi) - 1ull));
        const int prefix = __popcll(m & seg & lanemask_lt(lane));
        const int old = active ? L.cnt[slot] : 0;
        if (keep) {
            float4 *e = L.lst + (size_t)(slot * k.NZ + old + prefix) * 2;
            e[0] = w0;
            e[1] = make_float4(__int_as_float(tx.x * k.row_units), __int_as_float(tx.y * k.row_units),
                               __int_as_float(tx.z * k.row_units), __int_as_float(tx.w * k.row_units));
        }
        if (active && lane == lo) L.cnt[slot] = old + __popcll(m & seg);
    }
}

template <typename T, int VEC, int CPL, bool STREAM>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_forward_cached_kernel(
    KParams k, const T *__restrict__ depth, const T *__restrict__ feats, const void *__restrict__ cache,
    float *__restrict__ out, float *__restrict__ count_out) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = batch_of(k, bid);
    const int blk = bid - b * k.blocks_per_batch;
    const WaveLds L = wave_lds_view(k, smem, 2);
    const LaneRole role = lane_role<VEC, CPL>(k, lane);
    const int *counts = cache_counts(cache);
    const float4 *entries = reinterpret_cast<const float4 *>(static_cast<const char *>(cache) +
                                                             cache_entries_offset((long long)k.B * k.padded_cells));
    // (the cached lists are walked one group of `slots` cells at a time: their lengths are known, and
    // each cell's entries go to its own stretch of the pool)
    const int cells_per_wave = k.slots_a * k.rounds;
    // A cache built for other sizes would send the gathers out of bounds, and one built for another region
    // of interest or image size would pool the wrong texels: such a cache is not read at all, and the output
    // (and the counts) are filled with NaN instead.  (The matrices themselves cannot be checked.)
    const int *h = static_cast<const int *>(cache);
    const bool cache_fits = h[0] == kCacheMagic && h[1] == k.B && h[2] == k.N && h[3] == k.H && h[4] == k.W && h[5] == k.gx &&
                            h[6] == k.gy && h[7] == k.gz && h[8] == k.padded_cells && h[9] == k.NZ &&
                            h[10] == (int)k.geo_lo && h[11] == (int)k.geo_hi;
    for (int r = 0; r < k.rounds * k.batch_groups; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        if (!cache_fits) {
            const float nan = __int_as_float(0x7fc00000);
            for (int s = 0; s < k.slots; ++s) {
                int ix = 0, iy = 0;
                if (!cell_of(k, q0 + s, ix, iy)) continue;
                const size_t cell = (size_t)((b * k.gy + iy) * k.gx + ix);
                for (int c = lane; out != nullptr && c < k.C; c += kWave) out[cell * k.C + c] = nan;
                if (count_out != nullptr && lane == 0) count_out[cell] = nan;
            }
            continue;
        }
        phase_a_cached<T>(k, L, depth, counts, entries, b, q0, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        forward_phase_b<T, VEC, CPL, STREAM>(k, L, role, b, 0, feats, out, count_out);
        __builtin_amdgcn_wave_barrier();
    }
}

// Builds the cache: the sample phase with the depth model left out (every sample in view is
// listed), then each slot's list is copied out behind its cell's count.
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_geometry_cache_kernel(KParams k, const float *__restrict__ proj,
                                                                                   void *__restrict__ cache) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = batch_of(k, bid);
    const int blk = bid - b * k.blocks_per_batch;
    const WaveLds L = block_lds_setup(k, smem, proj, b, 1);
    int *counts = reinterpret_cast<int *>(static_cast<char *>(cache) + kCacheHeaderBytes);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        // what the lists were built for: the forward on cached geometry compares it with its own problem
        int *h = static_cast<int *>(cache);
        h[0] = kCacheMagic; h[1] = k.B; h[2] = k.N; h[3] = k.H; h[4] = k.W; h[5] = k.gx; h[6] = k.gy; h[7] = k.gz;
        h[8] = k.padded_cells; h[9] = k.NZ; h[10] = (int)k.geo_lo; h[11] = (int)k.geo_hi;
    }
    float4 *entries = reinterpret_cast<float4 *>(static_cast<char *>(cache) +
                                                 cache_entries_offset((long long)k.B * k.padded_cells));
    const int cells_per_wave = k.slots_a * k.rounds;
    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots_a;
        if (q0 >= k.padded_cells) break;
        const int n_cand = phase_a_candidates<true>(k, L, q0, lane);
        const int step = n_cand <= k.pool_cap ? k.batch_groups : 1;
        for (int g = 0; g < k.batch_groups; g += step) {
            phase_a_samples<1, float, kModeCache>(k, L, nullptr, b, lane, L.gcand[g], L.gcand[g + step]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            for (int s = g * k.slots; s < (g + step) * k.slots && q0 + s < k.padded_cells; ++s) {
                const size_t cell = (size_t)b * k.padded_cells + q0 + s;
                const int n = L.cnt[s], first = L.start[s];
                if (lane == 0) counts[cell] = n;
                for (int i = lane; i < n; i += kWave) entries[cell * k.NZ + i] = L.lst[first + i];
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

}  // namespace
