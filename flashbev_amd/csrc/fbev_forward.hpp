// The forward kernel.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// ---------------------------------------------------------------- forward
// STREAM: the output is stored with non-temporal stores (a template parameter: as a run-time
// choice between two stores the compiler merges them into one ordinary store).
template <typename T, int VEC, int CPL, bool STREAM>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_forward_kernel(
    KParams k, const T *__restrict__ depth, const T *__restrict__ feats, const float *__restrict__ proj,
    float *__restrict__ out, float *__restrict__ count_out) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = bid / k.blocks_per_batch;
    const int blk = bid - b * k.blocks_per_batch;

    const WaveLds L = block_lds_setup(k, smem, proj, b, 2);
    lds_counter *cnt = L.cnt;
    float4 *lst = L.lst;

    const int cells_per_wave = k.slots * k.rounds;
    // a lane group covers the channels of one cell; when long lists leave room for few slots,
    // several groups share a slot and take its entries in turn
    const int gps = k.groups_per_slot;
    const int group = lane / k.lanes_per_slot;
    const int slot = group / gps, sub = group - slot * gps;
    const int lis = lane - group * k.lanes_per_slot;
    const bool carrier = slot < k.slots;
    const int span = k.lanes_per_slot * VEC * CPL;   // channels covered per pass
    constexpr int kUnitShift = VEC > 1 ? 4 : (sizeof(T) == 4 ? 2 : 1);
    const char *fbytes = reinterpret_cast<const char *>(feats);

    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        phase_a<2, T, kModeForward>(k, L, depth, b, q0, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // phase A left the slot's cell in LDS: valid flag and ix | iy << 16
        const float4 mycell = L.cell[carrier ? slot : 0];
        const int ix = __float_as_int(mycell.w) & 0xffff, iy = __float_as_int(mycell.w) >> 16;
        const bool mine = carrier && mycell.z != 0.0f;
        const int n = mine ? cnt[slot] : 0;
        const float4 *my = lst + (size_t)(carrier ? slot : 0) * k.list_cap * 2;
        // the number of samples that enter the mean; the backward pass can reuse it
        if (count_out != nullptr && mine && lis == 0 && sub == 0) count_out[((size_t)b * k.gy + iy) * k.gx + ix] = (float)n;
        float *o = out + (((size_t)b * k.gy + iy) * k.gx + ix) * k.C;
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
                const T *p00 = reinterpret_cast<const T *>(fbytes + ((size_t)(unsigned)__float_as_int(tf.x) << kUnitShift));
                const T *p01 = reinterpret_cast<const T *>(fbytes + ((size_t)(unsigned)__float_as_int(tf.y) << kUnitShift));
                const T *p10 = reinterpret_cast<const T *>(fbytes + ((size_t)(unsigned)__float_as_int(tf.z) << kUnitShift));
                const T *p11 = reinterpret_cast<const T *>(fbytes + ((size_t)(unsigned)__float_as_int(tf.w) << kUnitShift));
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                        VecLoad<T, VEC>::ld(p00 + ch, f00);
                        VecLoad<T, VEC>::ld(p01 + ch, f01);
                        VecLoad<T, VEC>::ld(p10 + ch, f10);
                        VecLoad<T, VEC>::ld(p11 + ch, f11);
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
                int e = 2 * sub;
                for (; ch < k.C && e + 1 < n; e += 2 * gps) {
                    const float4 wa = my[2 * e], ta = my[2 * e + 1], wb = my[2 * e + 2], tb = my[2 * e + 3];
                    const int off[8] = {__float_as_int(ta.x), __float_as_int(ta.y), __float_as_int(ta.z), __float_as_int(ta.w),
                                        __float_as_int(tb.x), __float_as_int(tb.y), __float_as_int(tb.z), __float_as_int(tb.w)};
                    const float wv[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
                    float f[8][VEC];
#pragma unroll
                    for (int c = 0; c < 8; ++c)
                        VecLoad<T, VEC>::ld(reinterpret_cast<const T *>(fbytes + ((size_t)(unsigned)off[c] << kUnitShift)) + ch, f[c]);
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
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace
