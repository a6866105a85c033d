// Backward, cell side: the pair record, the zero-fill, count and scan kernels, and the cell pass
// (atomic scatter, or the inverse map's pair writer).
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// ---------------------------------------------------------------- backward
// Two ways to form the feature gradient, which is a sum over all samples that touch a texel:
//   scatter      fbev_backward_cells_kernel<.., 0>: one hardware fp32 atomic per (sample,
//                corner, channel).  Needs no workspace; slow under contention.
//   inverse map  let the cell pass (fbev_backward_cells_kernel<.., 1 or 2>) drop one 32-byte record
//                per kept sample into the segment of the sample's first corner texel (segments
//                of fixed capacity, or packed after a counting pass and a prefix sum), then
//                gather per texel from the segments of the four texels whose samples reach it
//                (fbev_backward_texel_kernel): the same coalesced row reads as the forward
//                pass, no floating-point atomics, each gradient row written once.
__device__ __forceinline__ void atomic_add_f32(float *p, float v) { unsafeAtomicAdd(p, v); }

// One record per kept sample, filed under the sample's first corner texel (v0, u0): the texel
// pass of a texel reads the lists of the (up to) four texels whose samples can reach it.
struct Pair {       // 32 bytes
    int cell;       // row of grad_out: (b * gy + iy) * gx + ix, shifted left by bin_bits with the depth bin below
    float coef;     // depth weight (/ count for the mean): d out[cell, c] / d feats[corner, c] is coef * corner weight
    float du, dv;   // bilinear fractions
    float ga, gb;   // <grad_out, sampled feature> * (d weight / d depth parameter); times the corner weight it is
                    // the sample's contribution to d_depth[corner, 0 / 1] (parametric) or [corner, k0 / k1]
    int flags;      // bit 0: u1 != u0, bit 1: v1 != v0 (clamped at the last column / row otherwise)
    int pad;
};
static_assert(sizeof(Pair) == 32, "a pair is written as two 16-byte words");

// Zero up to three regions of 32-bit words in one launch (segment counters and, when the
// library is asked to, the two gradient buffers).  A kernel rather than hipMemsetAsync, so the
// call can be captured in a HIP graph.
// One thread clears one 16-byte unit of a region (its ragged head and tail word by word), so
// the regions only have to be 4-byte aligned.
__device__ __forceinline__ void zero_unit(int *p, long long n, long long unit) {
    // units are counted from the first 16-byte boundary at or after p; unit 0 also takes the head
    const long long head = (4 - (((uintptr_t)p >> 2) & 3)) & 3;      // words before the boundary
    const long long first = unit * 4 + head;
    if (unit == 0)
        for (long long i = 0; i < head && i < n; ++i) p[i] = 0;
    if (first + 4 <= n) {
        *reinterpret_cast<int4 *>(p + first) = make_int4(0, 0, 0, 0);
    } else {
        for (long long i = first; i < n; ++i) p[i] = 0;
    }
}
__host__ __device__ inline long long zero_units(long long n) { return n > 0 ? (n + 3) / 4 + 1 : 0; }

__global__ __launch_bounds__(256) void fbev_fill_zero_kernel(int *a, long long na, int *b, long long nb, int *c,
                                                             long long nc) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long ua = zero_units(na), ub = zero_units(nb), uc = zero_units(nc);
    if (i < ua) zero_unit(a, na, i);
    else if (i < ua + ub) zero_unit(b, nb, i - ua);
    else if (i < ua + ub + uc) zero_unit(c, nc, i - ua - ub);
}

// Count, per (first-corner texel, replica), the samples that will contribute: phase A alone, with
// exactly the decisions the cell pass takes later (same code, same inputs).
// VIEW: count the samples in view (no depth model, no threshold) per fixed segment instead: the capacities of
// segments sized by the geometry.
template <typename T, bool VIEW = false>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_count_kernel(KParams k, const T *__restrict__ depth,
                                                                         const float *__restrict__ proj,
                                                                         int *__restrict__ counts) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = batch_of(k, bid);
    const int blk = bid - b * k.blocks_per_batch;
    const WaveLds L = block_lds_setup(k, smem, proj, b, 0);
    const int cells_per_wave = k.slots_a * k.rounds;
    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots_a;
        if (q0 >= k.padded_cells) break;
        const int n_cand = phase_a_candidates<false>(k, L, q0, lane);     // group boundaries are not needed
        phase_a_samples<0, T, VIEW ? kModeCountView : kModeCount>(k, L, depth, b, lane, 0, n_cand, nullptr, counts, 0);      // no entries: no pool
        __builtin_amdgcn_wave_barrier();
    }
}

// Prefix sum of the counters in two launches.  (1) Every block turns its chunk of 4096
// counters into exclusive prefix sums within the chunk and records the chunk total.
// (2) One block turns the chunk totals into exclusive prefix sums.  A counter's global
// position is chunk_prefix[i >> 12] + v[i]; nobody needs it materialised.
// (One launch with a last-block-done ticket was measured: the device-scope release every block
// then needs costs more than the second launch.)

// Inclusive scan of one value per thread of a 1024-thread block: shuffles inside a wavefront,
// LDS (32 ints) across the 16 wavefronts.
__device__ __forceinline__ int block_scan_1024(int *part, int tid, int sum) {
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    int incl = sum;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int other = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += other;
    }
    if (lane == kWave - 1) part[wave] = incl;
    __syncthreads();
    if (tid < 16) {
        int t = part[tid];
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            const int other = __shfl_up(t, off, kWave);
            if (tid >= off) t += other;
        }
        part[16 + tid] = t;
    }
    __syncthreads();
    return incl + (wave == 0 ? 0 : part[16 + wave - 1]);
}

__global__ __launch_bounds__(1024) void fbev_scan_chunks_kernel(int *__restrict__ v, long long n,
                                                                int *__restrict__ chunk_sums) {
    __shared__ int part[32];
    const int tid = threadIdx.x;
    const long long base = ((long long)blockIdx.x << kScanChunkBits) + tid * 4;
    int4 c = make_int4(0, 0, 0, 0);
    if (base + 3 < n) {
        c = *reinterpret_cast<const int4 *>(v + base);
    } else {
        if (base < n) c.x = v[base];
        if (base + 1 < n) c.y = v[base + 1];
        if (base + 2 < n) c.z = v[base + 2];
    }
    const int sum = c.x + c.y + c.z + c.w;
    const int incl = block_scan_1024(part, tid, sum);
    const int run = incl - sum;
    const int4 o = make_int4(run, run + c.x, run + c.x + c.y, run + c.x + c.y + c.z);
    if (base + 3 < n) {
        *reinterpret_cast<int4 *>(v + base) = o;
    } else {
        if (base < n) v[base] = o.x;
        if (base + 1 < n) v[base + 1] = o.y;
        if (base + 2 < n) v[base + 2] = o.z;
    }
    if (tid == 1023) chunk_sums[blockIdx.x] = incl;
}

__global__ __launch_bounds__(1024) void fbev_scan_sums_kernel(int *v, int n) {
    __shared__ int part[32];
    const int tid = threadIdx.x;
    const int per = (n + 1023) / 1024;
    const int lo = min(tid * per, n), hi = min(lo + per, n);
    int sum = 0;
    for (int i = lo; i < hi; ++i) sum += v[i];
    int run = block_scan_1024(part, tid, sum) - sum;
    for (int i = lo; i < hi; ++i) {
        const int c = v[i];
        v[i] = run;
        run += c;
    }
}

// The table of segments sized by the geometry: absolute start and capacity of every segment, from the
// capacities, their prefix sums within chunks of 4096 and the chunks' prefix sums; and the segments' packed
// claim counters in their initial state, in both sets (set_stride 32-bit words apart).
__global__ __launch_bounds__(256) void fbev_segment_table_kernel(long long n, const int *__restrict__ cap,
                                                                 const int *__restrict__ off,
                                                                 const int *__restrict__ prefix, int2 *__restrict__ tab,
                                                                 int *__restrict__ sets, long long set_stride) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int start = prefix[i >> kScanChunkBits] + off[i];
    tab[i] = make_int2(start, cap[i]);
    const unsigned long long word = packed_counter(start, cap[i]);
    reinterpret_cast<unsigned long long *>(sets)[i] = word;
    reinterpret_cast<unsigned long long *>(sets + set_stride)[i] = word;
}

// Cell pass of the backward.  FILL = 0: scatter with atomics.  FILL = 1: write pairs (inverse
// map); FILL = 2: the same with one claim per run of samples on one texel; FILL = 3: write pairs for the
// samples the forward stored (`store`, with the forward's per-cell counts in `count`) instead of
// evaluating the samples again.
// `cursor` holds, on entry, the start (within its scan chunk) of every (texel, replica)
// segment; phase A advances it, so on exit cursor[i] is the END of segment i.
template <typename T, int VEC, int CPL, int FILL, bool BATCHED>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_backward_cells_kernel(
    KParams k, const float *__restrict__ grad_out, const T *__restrict__ depth, const T *__restrict__ feats,
    const float *__restrict__ proj, float *__restrict__ d_depth, float *__restrict__ d_feats,
    const int *__restrict__ chunk_prefix, int *__restrict__ cursor, Pair *__restrict__ pairs, int pair_cap,
    int *epoch, int set_stride, const float *__restrict__ count = nullptr, const float4 *__restrict__ store = nullptr,
    const SegTable segs = SegTable{nullptr}) {
    extern __shared__ float4 smem[];
    constexpr int EF4 = 2;
    constexpr bool STORED = FILL == 3;
    static_assert(!(STORED && BATCHED), "the stored samples of a batch go through in one piece");
    if (FILL && epoch != nullptr) {
        // persistent workspace: the call counter's low bit selects the set of claim counters, and the
        // texel pass finds the counter where no block of its own writes (see struct Persist)
        const int e = epoch[1];
        cursor += (size_t)(e & 1) * set_stride;
        if (blockIdx.x == 0 && threadIdx.x == 0) epoch[0] = e;
    }
    // first corner texel and clamp flags of an entry
    auto entry_texel = [](const float4 &geo) { return FILL ? __float_as_int(geo.z) >> 2 : __float_as_int(geo.z); };
    auto entry_flags = [](const float4 &geo) { return FILL ? __float_as_int(geo.z) & 3 : __float_as_int(geo.w); };
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = batch_of(k, bid);
    const int blk = bid - b * k.blocks_per_batch;

    // (nothing is projected when the samples come from the store: no matrices, no tables)
    const WaveLds L = STORED ? wave_lds_view(k, smem, EF4) : block_lds_setup(k, smem, proj, b, EF4);
    lds_counter *cnt = L.cnt;
    float4 *lst = L.lst;

    const int cells_per_wave = k.slots_a * k.rounds;
    // lane groups of lanes_per_slot lanes; the groups_per_slot groups of a slot take its entries in turn
    const int gps = k.groups_per_slot;
    const int group = (int)(((unsigned)lane * k.lps_magic) >> 16);       // lane / lanes_per_slot
    const int slot = (int)(((unsigned)group * k.gps_magic) >> 16), sub = group - slot * gps;
    const int lis = lane - group * k.lanes_per_slot;
    const bool carrier = slot < k.slots;
    const int span = k.lanes_per_slot * VEC * CPL;
    const int Dd = k.Dd;
    const bool parametric = k.dist != FBEV_CATEGORICAL;
    // the inner product <grad_out, sampled feature> is only needed for the depth gradient
    const bool need_G = d_depth != nullptr;

    // G of four entries is summed over the lanes of a slot at a time when the slots start on
    // multiples of four lanes (always, on the 128-bit path)
    const bool grouped = (k.lanes_per_slot & 3) == 0;
    // first step of the sum over a slot's lanes: the largest power of two below the slot's width
    int red_first = 32;
    while (red_first >= k.lanes_per_slot && red_first > 1) red_first >>= 1;
    // The depth gradient travels with the pairs when one channel pass sees the whole of G and
    // the pair's first word has room for the depth bin; otherwise it is added with atomics here.
    const bool fold = FILL && need_G && k.C <= span && k.bin_bits >= 0;
    // a feature row starts at a 32-bit byte offset from the tensor's base: uniform base + 32-bit lane offset
    const char *fbytes = reinterpret_cast<const char *>(feats);
    auto row_at = [&](unsigned byte_offset) { return reinterpret_cast<const T *>(fbytes + byte_offset); };
    const unsigned row_step_v = (unsigned)(k.W * k.row_units);      // one feature-map row down

    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots_a;
        if (q0 >= k.padded_cells) break;
        // the lane's cell in the group of the batch it is working on
        bool mine = false;
        int cell = 0;
        const float *go = grad_out;
        auto enter_group = [&](int j) {
            int ix = 0, iy = 0;
            mine = carrier && cell_of(k, q0 + j * k.slots + slot, ix, iy);
            cell = (b * k.gy + iy) * k.gx + ix;
            go = grad_out + (size_t)cell * k.C;
        };
        // the grad_out row of the cell (first channel pass) of the first group that goes through stage 2
        // is requested before the sample phase and arrives while the samples are evaluated; the
        // groups behind it in a batch ask for theirs when their turn comes
        float g[CPL][VEC];
        auto load_g = [&](int c0) {
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
#pragma unroll
                for (int v = 0; v < VEC; ++v) g[j][v] = 0.0f;
                if (mine && ch < k.C) {
                    if (VEC == 1) {
                        g[j][0] = go[ch];
                    } else {
#pragma unroll
                        for (int v = 0; v < VEC; v += 4) {
                            const float4 t = *reinterpret_cast<const float4 *>(go + ch + v);
                            g[j][v] = t.x; g[j][v + 1] = t.y; g[j][v + 2] = t.z; g[j][v + 3] = t.w;
                        }
                    }
                }
            }
        };
        enter_group(0);
        load_g(0);
        const int n_cand = STORED ? 0 : phase_a_candidates<BATCHED>(k, L, q0, lane);
        // all groups of the batch through stage 2 together when the pool is sure to hold what they keep
        const int n_groups = BATCHED ? k.batch_groups : 1;
        const int step = n_cand <= k.pool_cap ? n_groups : 1;
        for (int g0 = 0; g0 < n_groups; g0 += step) {
        if (BATCHED && g0 > 0) {
            enter_group(g0);
            load_g(0);
        }
        if (STORED)
            phase_a_stored(k, L, count, store + ((size_t)b * k.padded_cells + q0) * k.NZ * 2, b, q0, lane, chunk_prefix,
                           cursor, pair_cap, segs);
        else
            phase_a_samples<EF4, T, FILL == 2 ? kModeFillRuns : (FILL ? kModeFill : kModeScatter)>(
                k, L, depth, b, lane, BATCHED ? L.gcand[g0] : 0, BATCHED ? L.gcand[g0 + step] : n_cand, chunk_prefix, cursor,
                pair_cap, nullptr, segs);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (int grp = g0; grp < g0 + step; ++grp) {
        if (BATCHED && grp > g0) {
            enter_group(grp);
            load_g(0);
        }
        const int slot_a = carrier ? grp * k.slots + slot : 0;

        const int n = mine ? cnt[slot_a] : 0;
        // every lane of the wavefront takes part in the shuffles below, so all lanes run
        // the longest list of the wavefront and idle past their own.
        int n_max = n;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) n_max = max(n_max, __shfl_xor(n_max, off, kWave));
        float4 *my = lst + (size_t)L.start[slot_a] * EF4;
        const float inv = (k.reduce_sum || n == 0) ? 1.0f : 1.0f / (float)n;

        for (int c0 = 0; c0 < k.C; c0 += span) {
            const bool first_pass = c0 == 0;
            if (!first_pass) load_g(c0);
#pragma unroll
            for (int j = 0; j < CPL; ++j)
#pragma unroll
                for (int v = 0; v < VEC; ++v) g[j][v] = n > 0 ? g[j][v] * inv : 0.0f;

            // this lane's share of <grad_out, sampled feature> of entry e (e < n); on the scatter
            // path (and for corners without room in the pair array) also the feature-gradient atomics
            auto entry_share = [&](int e) -> float {
                float G = 0.0f;
                const float4 geo = my[EF4 * e];
                const float wgt = my[EF4 * e + 1].x;
                const float du = geo.x, dv = geo.y;
                const float w00 = (1.0f - du) * (1.0f - dv), w01 = (1.0f - du) * dv, w10 = du * (1.0f - dv), w11 = du * dv;
                const int t00 = entry_texel(geo), fl = entry_flags(geo);
                const int su = fl & 1, sv = (fl & 2) ? k.W : 0;
                // feature rows as byte offsets: one 32-bit multiply and three adds, then one add each
                const unsigned r00 = (unsigned)t00 * (unsigned)k.row_units;
                const unsigned r01 = r00 + ((fl & 2) ? row_step_v : 0u);
                const unsigned r10 = r00 + ((fl & 1) ? (unsigned)k.row_units : 0u), r11 = r01 + (r10 - r00);
                // scatter path, or a sample without room in the pair array: atomics for all four corners
                const bool spill = FILL ? __float_as_int(geo.w) < 0 : true;
                const bool s00 = spill, s01 = spill, s10 = spill, s11 = spill;
                const float a00 = w00 * wgt, a01 = w01 * wgt, a10 = w10 * wgt, a11 = w11 * wgt;
                // <grad_out, sampled feature> = sum over the corners of w_ij * <grad_out, row_ij>: the four inner
                // products take the rows as they come (half-precision rows enter the multiply-adds unconverted),
                // and the bilinear weights are applied once per entry instead of once per channel
                float d00 = 0.0f, d01 = 0.0f, d10 = 0.0f, d11 = 0.0f;
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        if (need_G) {
                            const unsigned chb = (unsigned)ch * (unsigned)sizeof(T);
                            float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                            VecLoad<T, VEC>::ld(row_at(r00 + chb), f00);
                            VecLoad<T, VEC>::ld(row_at(r01 + chb), f01);
                            VecLoad<T, VEC>::ld(row_at(r10 + chb), f10);
                            VecLoad<T, VEC>::ld(row_at(r11 + chb), f11);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) {
                                d00 = __builtin_fmaf(g[j][v], f00[v], d00);
                                d01 = __builtin_fmaf(g[j][v], f01[v], d01);
                                d10 = __builtin_fmaf(g[j][v], f10[v], d10);
                                d11 = __builtin_fmaf(g[j][v], f11[v], d11);
                            }
                        }
                        if (d_feats != nullptr && (s00 || s01 || s10 || s11)) {
                            const size_t o00 = (size_t)t00 * k.C, o01 = (size_t)(t00 + sv) * k.C;
                            const size_t o10 = (size_t)(t00 + su) * k.C, o11 = (size_t)(t00 + sv + su) * k.C;
#pragma unroll
                            for (int v = 0; v < VEC; ++v) {
                                if (s00) atomic_add_f32(d_feats + o00 + ch + v, g[j][v] * a00);
                                if (s01) atomic_add_f32(d_feats + o01 + ch + v, g[j][v] * a01);
                                if (s10) atomic_add_f32(d_feats + o10 + ch + v, g[j][v] * a10);
                                if (s11) atomic_add_f32(d_feats + o11 + ch + v, g[j][v] * a11);
                            }
                        }
                    }
                }
                if (need_G) G = __builtin_fmaf(w11, d11, __builtin_fmaf(w10, d10, __builtin_fmaf(w01, d01, w00 * d00)));
                return G;
            };
            // what one lane does with the complete G of entry e
            auto entry_done = [&](int e, float G) {
                if (fold) {
                    // the pairs are written after the loop, 64 at a time; keep G * (a, b) with the
                    // entry in place of (a, b)
                    my[EF4 * e + 1].y *= G;
                    my[EF4 * e + 1].z *= G;
                } else {
                    // scatter path, or G arrives in several channel passes
                    const float4 geo = my[EF4 * e], dw = my[EF4 * e + 1];
                    const float du = geo.x, dv = geo.y;
                    const float wc[4] = {(1.0f - du) * (1.0f - dv), (1.0f - du) * dv, du * (1.0f - dv), du * dv};
                    const int t00 = entry_texel(geo), fl = entry_flags(geo);
                    const int su = fl & 1, sv = (fl & 2) ? k.W : 0;
                    const int t[4] = {t00, t00 + sv, t00 + su, t00 + sv + su};
                    const int kk = __float_as_int(dw.w);
                    const int k0 = parametric ? 0 : (kk & 0xffff), k1 = parametric ? 1 : (kk >> 16);
                    const float ga = G * dw.y, gb = G * dw.z;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        atomic_add_f32(d_depth + (size_t)t[c] * Dd + k0, ga * wc[c]);
                        atomic_add_f32(d_depth + (size_t)t[c] * Dd + k1, gb * wc[c]);
                    }
                }
            };

            if (grouped) {
                for (int t0 = 0; t0 < n_max; t0 += 4 * gps) {
                    const int e0 = t0 + 4 * sub;
                    float G0 = e0 < n ? entry_share(e0) : 0.0f;
                    float G1 = e0 + 1 < n ? entry_share(e0 + 1) : 0.0f;
                    float G2 = e0 + 2 < n ? entry_share(e0 + 2) : 0.0f;
                    float G3 = e0 + 3 < n ? entry_share(e0 + 3) : 0.0f;
                    if (need_G) {
                        // two exchange steps inside every group of four lanes leave lane q of the
                        // group with the group's sum for entry (q & 1) * 2 + (q >> 1) ...
                        const bool b0 = lane & 1, b1 = lane & 2;
                        const float ra = quad_xor1(b0 ? G0 : G2), rb = quad_xor1(b0 ? G1 : G3);
                        const float ka = (b0 ? G2 : G0) + ra, kb = (b0 ? G3 : G1) + rb;
                        float Gq = (b1 ? kb : ka) + quad_xor2(b1 ? ka : kb);
                        // ... and four more add up the groups of the slot
                        for (int off = red_first; off >= 4; off >>= 1) {
                            const float other = __shfl_down(Gq, off, kWave);
                            if (lis + off < k.lanes_per_slot) Gq += other;
                        }
                        const int e = e0 + ((lis & 1) << 1) + ((lis >> 1) & 1);
                        if (lis < 4 && e < n) entry_done(e, Gq);
                    }
                }
            } else {
                for (int t0 = 0; t0 < n_max; t0 += gps) {
                    const int e = t0 + sub;
                    float G = e < n ? entry_share(e) : 0.0f;
                    if (need_G) {
                        for (int off = red_first; off > 0; off >>= 1) {
                            const float other = __shfl_down(G, off, kWave);
                            if (lis + off < k.lanes_per_slot) G += other;
                        }
                        if (e < n && lis == 0) entry_done(e, G);
                    }
                }
            }
            if (FILL && first_pass) {
                // ---- the pairs of this round: the lanes of a slot's groups take the slot's entries in turn
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                {
                    const int pcell = cell;
                    const float pinv = inv;
                    const float4 *lst_s = my;
                    for (int pe = sub * k.lanes_per_slot + lis; pe < n; pe += gps * k.lanes_per_slot) {
                        const float4 geo = lst_s[EF4 * pe], dwp = lst_s[EF4 * pe + 1];
                        const int posp = __float_as_int(geo.w);
                        const int kk = __float_as_int(dwp.w);
                        const int k0 = parametric ? 0 : (kk & 0xffff), k1 = parametric ? 1 : (kk >> 16);
                        // G * a and G * b (G already carries 1/count)
                        const float ga = fold ? dwp.y : 0.0f, gb = fold ? dwp.z : 0.0f;
                        if (posp >= 0) {
                            const int word = fold ? ((pcell << k.bin_bits) | k0) : pcell;
                            float4 *dst = reinterpret_cast<float4 *>(pairs + posp);
                            dst[0] = make_float4(__int_as_float(word), dwp.x * pinv, geo.x, geo.y);
                            dst[1] = make_float4(ga, gb, __int_as_float(entry_flags(geo)), 0.0f);
                        } else if (fold) {
                            const float du = geo.x, dv = geo.y;
                            const int fl = entry_flags(geo), t00 = entry_texel(geo);
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                // corner c: 0 (v0,u0) 1 (v1,u0) 2 (v0,u1) 3 (v1,u1); same products as phase A
                                const float wcc = ((c & 2) ? du : 1.0f - du) * ((c & 1) ? dv : 1.0f - dv);
                                const int tt = t00 + ((c & 1) && (fl & 2) ? k.W : 0) + ((c & 2) ? (fl & 1) : 0);
                                atomic_add_f32(d_depth + (size_t)tt * Dd + k0, ga * wcc);
                                atomic_add_f32(d_depth + (size_t)tt * Dd + k1, gb * wcc);
                            }
                        }
                    }
                }
            }
        }
        }      // the groups of this pass through stage 2
        __builtin_amdgcn_wave_barrier();
        }      // the passes of the batch through stage 2
    }
}

}  // namespace
