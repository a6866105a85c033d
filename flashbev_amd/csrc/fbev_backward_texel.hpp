// Backward, texel side of the inverse map.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// Texel pass of the inverse-map backward.  The samples that reach texel t are filed under their
// first corner: t itself, its left neighbour, the texel above, and the one above-left (a sample's
// corners are (v0|v1, u0|u1) with u1 = u0 + 1 and v1 = v0 + 1 unless clamped).  Those four lists
// are handled by one block, or, when the grid has a second dimension and a list is longer than
// kTexelPart, by up to gridDim.y blocks that each take an equal share of every list.  Every block
// of a texel first has to read the lists' bounds, so idle blocks are not free: the host splits
// only when there are too few texels to fill the machine otherwise (kTexelSplitBelow).  A block's
// WAVES * (64 / lanes_per_row) workers stride over the pairs, each gathering grad_out rows with
// 128-bit loads; partial rows meet in LDS.  A texel handled by one block is updated with plain
// loads and stores; the shares of a split texel are combined with fp32 atomics (at most
// gridDim.y per address).
constexpr int kTexelMaxSplit = 8;
constexpr int kTexelSplitBelow = 16384;     // texels * blocks per texel stay below this (400x400x12 grid on 4224 texels: 1 / 3 / 7 blocks per texel 107 / 101 / 127 us)
constexpr int kTexelPart = 128;
// Wavefronts per texel block, chosen from the samples a texel could get if every one were kept ("possible"), counted
// twice where about twice as many are kept (categorical depth, or no weight threshold):
constexpr int kTexelOneWaveBelow = 200;      // one wavefront below this,
constexpr int kTexelTwoWavesBelow = 800;     // two below this, four from there on;
// and one instead of two when two would make more wavefronts than eight times what the machine holds at once
// (256 CUs x 4 SIMDs x 6): the blocks then run in many generations anyway, and what a second wavefront per block adds
// is its share of the set-up, not a shorter chain.  (Four are kept: at the training size two per texel are 3 % faster
// but put twice the texels in flight per die, more than its L2 holds grad_out rows for: 541 instead of 382 MB from HBM.)
constexpr long long kTexelWavesAtOnce = 8ll * 256 * 4 * 6;
constexpr int kTexelSegs = 4 * kFixedReplicas;   // lists of a texel with fixed segments: 4 first corners x replicas

// What a persistent workspace adds to the fixed-segment layout, so that a call needs no zero-fill
// launch (all null / 0 otherwise):
//   epoch      two call counters.  The cell pass reads epoch[1] and copies it to epoch[0]; the texel
//              pass reads epoch[0] and stores epoch[0] + 1 to epoch[1]: neither kernel reads a word
//              that one of its own blocks writes.  The low bit selects the set of claim counters.
//   sets       two sets of claim counters, set_stride ints apart.  A call claims in one set; its
//              texel pass clears the other, which the previous call left behind and the next will use.
//   ovf_*      gradient buffers of the workspace's own, all zero between calls.  What the cell pass
//              cannot file (a full segment) or does not file (a depth gradient that does not ride on
//              the pairs) it adds here with atomics; the texel pass of a texel that sees a full
//              segment, the only texels such samples reach, takes its rows from here and clears them.
//   segs       segments sized by the geometry (see SegTable), or all null for segments of one common capacity.
struct Persist {
    int *epoch;
    int *sets;
    int set_stride;
    float *ovf_depth, *ovf_feats;
    SegTable segs;
};

// NARROW: grad_out is smaller than 4 GiB, so a row is addressed by a 32-bit byte offset from the tensor's uniform base
// (one add per gather instead of a 64-bit shift-add: a sixth of the pass's vector instructions).
template <int VEC, int WAVES, bool NARROW>
__global__ __launch_bounds__(kWave *WAVES) void fbev_backward_texel_kernel(
    KParams k, const float *__restrict__ grad_out, const int *__restrict__ chunk_prefix,
    const int *__restrict__ seg_end, const Pair *__restrict__ pairs, int pair_cap, float *__restrict__ d_depth,
    float *__restrict__ d_feats, int lanes_per_row, int depth_from_pairs, int fresh, Persist ps) {
    extern __shared__ float4 smem[];
    // per wavefront 64 (grad_out row, coefficient) records of the chunk in hand, then the partial rows
    float2 *stage = reinterpret_cast<float2 *>(smem) + (threadIdx.x >> 6) * kWave;
    float *part = reinterpret_cast<float *>(smem) + WAVES * kWave * 2;
    // Blocks are dealt to the accelerator dies in turn; let each die walk a contiguous range of
    // texels, column by column: the texels of a feature-map column gather the cells along one
    // wedge of rays (a cell's height bins land on neighbouring rows), so their grad_out rows meet
    // in one L2 while they are still there.
    // (Measured: 10 % faster at 33 792 texels with 1 KiB rows; at 4224 texels no faster, but the pass
    // reads 3.7 times less from HBM.)
    int t = blockIdx.x;
    if (gridDim.x >= 1024) {
        const int j = xcd_swizzle(blockIdx.x, gridDim.x), hw = k.H * k.W;
        const int img = j / hw, rem = j - img * hw, u = rem / k.H, v = rem - u * k.H;
        t = (img * k.H + v) * k.W + u;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    constexpr int n_waves = WAVES;
    const bool counted = chunk_prefix != nullptr;
    const bool persistent = ps.epoch != nullptr;
    // (persistent: which set of counters this call claimed in; the lists' bounds are requested
    // from both sets before the answer is needed)
    const int epoch = persistent ? ps.epoch[0] : 0, set = epoch & 1;
    // List e of the texel: first corner (e & 3 with fixed segments, e when counted): bit 0 = one
    // texel to the left, bit 1 = one row up; replica e >> 2 with fixed segments.  A cell's samples
    // on neighbouring height bins sit in different lists of the same replica, at about the same
    // relative position (they were claimed together): replica-major order keeps them close in
    // time, so the second gather of the cell's grad_out row finds it in cache.
    // Every wavefront builds the table for itself in its first kTexelSegs lanes (lane e holds list
    // e): no LDS, no barrier before the first pair is requested.
    const int tu = t % k.W, tv = (t / k.W) % k.H;
    int my_lo = 0, my_len = 0;
    bool spilled = false;      // a list of this texel was full: the cell pass added the rest with atomics
    unsigned long long own_word = 0;   // (packed counters) the initial state of the counter of an own segment
    if (lane < kTexelSegs) {
        const int e = lane;
        const int o = counted ? e : e & 3;
        const bool exists = (counted ? e < 4 : true) && (!(o & 1) || tu > 0) && (!(o & 2) || tv > 0);
        const int q = t - (o & 1) - ((o & 2) ? k.W : 0);
        if (exists && counted) {
            // counted segments, one after the other: from the end of the previous texel's last
            // replica to the end of this texel's
            const long long first = (long long)q * kReplicas - 1, last = (long long)q * kReplicas + kReplicas - 1;
            my_lo = q == 0 ? 0 : chunk_prefix[first >> kScanChunkBits] + seg_end[first];
            const int list_end = chunk_prefix[last >> kScanChunkBits] + seg_end[last];
            spilled = list_end > pair_cap;
            my_len = max(min(list_end, pair_cap) - my_lo, 0);
        } else if (exists) {
            // fixed segments of pair_cap pairs; seg_end holds how many were claimed
            const int i = q * kFixedReplicas + (e >> 2);
            my_lo = i * pair_cap;
            int room = pair_cap, seg_cap = 0;
            if (ps.segs.tab != nullptr) {
                // (a segment that would reach past the pair array holds what fits: the rest was added with atomics)
                const int2 seg = ps.segs.tab[i];
                my_lo = seg.x;
                seg_cap = seg.y;
                room = max(min(seg.y, pair_cap - my_lo), 0);
            }
            int claimed;
            if (ps.segs.tab != nullptr) {
                // packed counters: the low word started at kSegBias - capacity
                const int in_first = ps.sets[2 * i], in_second = ps.sets[ps.set_stride + 2 * i];
                claimed = (int)((unsigned)(set ? in_second : in_first) - (kSegBias - (unsigned)seg_cap));
            } else if (persistent) {
                const int in_first = ps.sets[i], in_second = ps.sets[ps.set_stride + i];
                claimed = set ? in_second : in_first;
            } else {
                claimed = seg_end[i];
            }
            spilled = claimed > room;
            my_len = max(min(claimed, room), 0);
            if (o == 0) own_word = packed_counter(my_lo, seg_cap);
        }
    }
    if (persistent && blockIdx.y == 0) {
        // the counters of this texel in the set the next call claims in: zero, or, packed, their initial state
        // (lists 0, 4, 8, 12 are the texel's own segments, one per replica)
        int *next = ps.sets + (size_t)(set ^ 1) * ps.set_stride;
        if (ps.segs.tab != nullptr) {
            if (threadIdx.x < kTexelSegs && (threadIdx.x & 3) == 0)
                reinterpret_cast<unsigned long long *>(next)[(size_t)t * kFixedReplicas + (threadIdx.x >> 2)] = own_word;
        } else if (threadIdx.x == 0) {
            *reinterpret_cast<int4 *>(next + (size_t)t * kFixedReplicas) = make_int4(0, 0, 0, 0);
        }
        if (blockIdx.x == 0 && threadIdx.x == 0) ps.epoch[1] = epoch + 1;
    }
    // the lists one after the other form one sequence of pairs; list e starts at my_pre of lane e
    int my_pre = my_len;
#pragma unroll
    for (int off = 1; off < kTexelSegs; off <<= 1) {
        const int other = __shfl_up(my_pre, off, kWave);
        if (lane >= off) my_pre += other;
    }
    my_pre -= my_len;                              // exclusive
    int list_start[kTexelSegs];                    // wave-uniform copies of the starts of lists 1 ..
#pragma unroll
    for (int j = 1; j < kTexelSegs; ++j) list_start[j] = __builtin_amdgcn_readlane(my_pre, j);
    const int n_all = __builtin_amdgcn_readlane(my_pre, kTexelSegs - 1) + __builtin_amdgcn_readlane(my_len, kTexelSegs - 1);
    // (a texel nothing was claimed for has no part at all, unless the workspace is persistent: then
    // nobody has cleared the gradient buffers and its block stores the zeros)
    const int n_parts = max(min((int)gridDim.y, (n_all + 4 * kTexelPart - 1) / (4 * kTexelPart)), persistent ? 1 : 0);
    if ((int)blockIdx.y >= n_parts) return;      // uniform for the block
    const bool shared_texel = n_parts > 1;
    // The gradient buffers were cleared by this call (fresh) and nothing but this block touches the
    // texel unless a list spilled: then its rows are stored, not added, and the pass ends without a
    // dependent load.
    const bool any_spill = __ballot(spilled) != 0ull;
    const bool store_only = fresh != 0 && !shared_texel && !any_spill;
    const int part_lo = (int)(((long long)n_all * blockIdx.y) / n_parts);
    const int part_hi = (int)(((long long)n_all * (blockIdx.y + 1)) / n_parts);
    // the wavefronts take chunks of the sequence in turn: 64 pairs, fewer when that leaves a wavefront idle
    const int chunk = min(kWave, max(1, (part_hi - part_lo + n_waves - 1) / n_waves));
    const unsigned n_cells = (unsigned)(k.B * k.gy * k.gx);
    const int wpw = kWave / lanes_per_row;            // workers per wavefront
    const int nw = wpw * n_waves;
    const int wslot = lane / lanes_per_row;
    const int lir = lane - wslot * lanes_per_row;
    const bool worker_lane = wslot < wpw;
    const int worker = wave * wpw + wslot;
    const int span = lanes_per_row * VEC;
    const int stride = span + 2;                      // partial row + the two depth sums
    // categorical depth gradient: one LDS accumulator per depth bin of this texel
    const bool bin_sums = depth_from_pairs && k.dist == FBEV_CATEGORICAL;
    float *bins = part + nw * stride;
    const int bin_bits = depth_from_pairs ? k.bin_bits : 0, bin_mask = (1 << bin_bits) - 1;
    if (bin_sums) {
        for (int i = threadIdx.x; i < k.Dd; i += blockDim.x) bins[i] = 0.0f;
        __syncthreads();
    }
    constexpr int kOutShift = VEC > 1 ? 4 : 2;
    const unsigned out_units = NARROW ? (unsigned)k.C * 4u : (unsigned)(VEC > 1 ? k.C / 4 : k.C);
    const char *gbytes = reinterpret_cast<const char *>(grad_out);
    unsigned ch_bytes = 0;      // (set per channel pass: where the lane's channels start in a row)
    auto row_at = [&](unsigned row) {
        return NARROW ? reinterpret_cast<const float *>(gbytes + (row + ch_bytes))
                      : reinterpret_cast<const float *>(gbytes + ((size_t)row << kOutShift)) + (ch_bytes >> 2);
    };
    for (int c0 = 0; c0 < k.C; c0 += span) {
        const int ch = c0 + lir * VEC;
        const bool on = worker_lane && ch < k.C;
        const int wslot_eff = min(wslot, wpw - 1);
        ch_bytes = on ? (unsigned)ch * 4u : 0u;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
        float sa = 0.0f, sb = 0.0f;
        // A wavefront takes 64 consecutive pairs at a time, one per lane in a single coalesced
        // load, and hands them to its workers through 512 bytes of LDS; four grad_out rows per
        // worker are in flight before the first is used.  The loop is bound by load latency:
        // without this the pair load and the row load it addresses form a dependent chain.
        for (int bstart = part_lo + wave * chunk; bstart < part_hi; bstart += n_waves * chunk) {
            const int nb = min(chunk, part_hi - bstart);
            float4 pr = make_float4(__int_as_float(-1), 0.f, 0.f, 0.f), pd = make_float4(0.f, 0.f, 0.f, 0.f);
            // which list position bstart + lane falls into (all lanes take part in the shuffles;
            // positions past the chunk fall into some list and are not loaded)
            const int vi = bstart + lane;
            int e = 0;
#pragma unroll
            for (int j = 1; j < kTexelSegs; ++j) e += vi >= list_start[j] ? 1 : 0;
            const int o = counted ? e : e & 3;
            // lane e of the wavefront knows where list e lies in the pair array
            const int src_pos = __shfl(my_lo, e, kWave) + (vi - __shfl(my_pre, e, kWave));
            if (lane < nb) {
                const float4 *src = reinterpret_cast<const float4 *>(pairs + src_pos);
                pr = src[0];
                pd = src[1];
            }
            const int word = __float_as_int(pr.x);
            // a pair is written by the cell pass before this kernel starts; the range check only
            // keeps a logic error from turning into a wild read (such a pair counts as cell 0
            // with coefficient 0)
            const bool valid = (unsigned)(word >> bin_bits) < n_cells;
            // the sample's bilinear weight on this texel: the corners that land here (a clamped
            // corner stays on the first corner's column / row)
            const float du = pr.z, dv = pr.w;
            const bool fu = __float_as_int(pd.z) & 1, fv = __float_as_int(pd.z) & 2;
            const float w00 = (1.0f - du) * (1.0f - dv), w01 = (1.0f - du) * dv, w10 = du * (1.0f - dv), w11 = du * dv;
            float cw;
            if (o == 0) cw = w00 + (fu ? 0.0f : w10) + (fv ? 0.0f : w01) + ((fu || fv) ? 0.0f : w11);
            else if (o == 1) cw = fu ? w10 + (fv ? 0.0f : w11) : 0.0f;
            else if (o == 2) cw = fv ? w01 + (fu ? 0.0f : w11) : 0.0f;
            else cw = (fu && fv) ? w11 : 0.0f;
            // where the pair's grad_out row starts: in bytes, or (a tensor of 4 GiB and more) in units of 16 bytes
            // (one float off the vector path)
            const unsigned my_row = valid ? (unsigned)(word >> bin_bits) * out_units : 0u;
            const float my_coef = valid ? pr.y * cw : 0.0f;
            if (c0 == 0 && valid) {
                if (bin_sums) {
                    const int k0 = word & bin_mask;
                    __hip_atomic_fetch_add(bins + k0, pd.x * cw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(bins + min(k0 + 1, k.Dd - 1), pd.y * cw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                } else {
                    sa += pd.x * cw;
                    sb += pd.y * cw;
                }
            }
            // Pairs that follow each other in a list and come from one cell (its samples on
            // neighbouring height bins that share a first corner claimed neighbouring positions)
            // gather the same grad_out row: their coefficients are added up and the row is
            // gathered once.  A run gets a new leader every eight lanes, so that three steps of a
            // suffix sum inside the runs leave every leader with its run's coefficient.
            const unsigned prev_row = (unsigned)__shfl_up((int)my_row, 1, kWave);
            const bool in_chunk = lane < nb;
            const unsigned long long cm = __ballot(in_chunk && lane > 0 && my_row == prev_row);
            const int run_lead = 63 - __clzll(~cm & lanemask_le(lane));
            const unsigned long long lm = __ballot(in_chunk && ((lane - run_lead) & 7) == 0);
            const unsigned long long later = lane == 63 ? 0ull : (lm >> (lane + 1));      // leaders after me
            const int followers = later ? __ffsll((long long)later) - 1 : 63 - lane;    // lanes past the chunk carry 0
            float run_coef = my_coef;
#pragma unroll
            for (int off = 1; off <= 4; off <<= 1) {
                const float other = __shfl_down(run_coef, off, kWave);
                if (off <= followers) run_coef += other;
            }
            const int n_lead = __popcll(lm);
            if ((lm >> lane) & 1ull) stage[__popcll(lm & lanemask_lt(lane))] = make_float2(__int_as_float((int)my_row), run_coef);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            // Full groups of UNR rows per worker run without predicates (lanes that carry no
            // channel gather channel 0 of some row and drop the result); the remainder goes one
            // row per worker.
            constexpr int UNR = 4;
            const int group = wpw * UNR, full = n_lead - n_lead % group;
            for (int i = 0; i < full; i += group) {
                float coefs[UNR];
                float g[UNR][VEC];
#pragma unroll
                for (int q = 0; q < UNR; ++q) {
                    const float2 rc = stage[i + q * wpw + wslot_eff];
                    coefs[q] = rc.y;
                    VecLoad<float, VEC>::ld(row_at((unsigned)__float_as_int(rc.x)), g[q]);
                }
#pragma unroll
                for (int q = 0; q < UNR; ++q)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(coefs[q], g[q][v], acc[v]);
            }
            if (full < n_lead) {
                // the rest as one more group, its gathers in flight together: a worker past the last row takes
                // the last row again with a coefficient of zero
                float coefs[UNR];
                float g[UNR][VEC];
#pragma unroll
                for (int q = 0; q < UNR; ++q) {
                    const int want = full + q * wpw + wslot_eff;
                    const float2 rc = stage[min(want, n_lead - 1)];
                    coefs[q] = want < n_lead ? rc.y : 0.0f;
                    VecLoad<float, VEC>::ld(row_at((unsigned)__float_as_int(rc.x)), g[q]);
                }
#pragma unroll
                for (int q = 0; q < UNR; ++q)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(coefs[q], g[q][v], acc[v]);
            }
            __builtin_amdgcn_wave_barrier();      // the records are read before the next chunk overwrites them
        }
        // the depth sums sit in the lanes that loaded the pairs: fold them into lane 0
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            sa += __shfl_xor(sa, off, kWave);
            sb += __shfl_xor(sb, off, kWave);
        }
        __syncthreads();   // previous pass has been read
        if (worker_lane) {
            if (ch < k.C) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) part[worker * stride + lir * VEC + v] = acc[v];
            }
            if (lir == 0) {
                part[worker * stride + span] = wslot == 0 ? sa : 0.0f;
                part[worker * stride + span + 1] = wslot == 0 ? sb : 0.0f;
            }
        }
        __syncthreads();
        for (int c = threadIdx.x; c < span && c0 + c < k.C; c += blockDim.x) {
            float sum = 0.0f;
            for (int w = 0; w < nw; ++w) sum += part[w * stride + c];
            if (d_feats != nullptr) {
                float *dst = d_feats + (size_t)t * k.C + c0 + c;
                if (persistent) {
                    if (any_spill) {
                        float *o = ps.ovf_feats + (size_t)t * k.C + c0 + c;
                        sum += *o;
                        *o = 0.0f;
                    }
                    if (fresh) *dst = sum;
                    else *dst += sum;
                } else if (shared_texel) atomic_add_f32(dst, sum);
                else if (store_only) *dst = sum;
                else *dst += sum;
            }
        }
        if (c0 == 0 && bin_sums) {
            for (int i = threadIdx.x; i < k.Dd; i += blockDim.x) {
                float sum = bins[i];
                float *dst = d_depth + (size_t)t * k.Dd + i;
                if (persistent) {
                    if (any_spill) {
                        float *o = ps.ovf_depth + (size_t)t * k.Dd + i;
                        sum += *o;
                        *o = 0.0f;
                    }
                    if (fresh) *dst = sum;
                    else *dst += sum;
                } else if (sum != 0.0f) {
                    if (shared_texel) atomic_add_f32(dst, sum);
                    else if (store_only) *dst = sum;
                    else *dst += sum;
                }
            }
        } else if (c0 == 0 && depth_from_pairs && threadIdx.x < 2) {
            float sum = 0.0f;
            for (int w = 0; w < nw; ++w) sum += part[w * stride + span + threadIdx.x];
            float *dst = d_depth + (size_t)t * 2 + threadIdx.x;
            if (persistent) {
                if (any_spill) {
                    float *o = ps.ovf_depth + (size_t)t * 2 + threadIdx.x;
                    sum += *o;
                    *o = 0.0f;
                }
                if (fresh) *dst = sum;
                else *dst += sum;
            } else if (shared_texel) atomic_add_f32(dst, sum);
            else if (store_only) *dst = sum;
            else *dst += sum;
        } else if (c0 == 0 && persistent && d_depth != nullptr && !depth_from_pairs) {
            // the cell pass added the whole depth gradient of this texel to the workspace's buffer
            for (int i = threadIdx.x; i < k.Dd; i += blockDim.x) {
                float *o = ps.ovf_depth + (size_t)t * k.Dd + i;
                const float sum = *o;
                *o = 0.0f;
                float *dst = d_depth + (size_t)t * k.Dd + i;
                if (fresh) *dst = sum;
                else *dst += sum;
            }
        }
    }
}

}  // namespace
