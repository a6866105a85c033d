// Fused camera->BEV pooling for gfx950 (MI355X): kernels and the C ABI declared in
// include/flashbev_hip.h.
//
// Structure of both hot kernels.  A wavefront (64 lanes) owns S consecutive BEV cells
// ("slots") of one batch element and works in two phases:
//   phase A  lanes = (slot, camera, height-bin) samples.  Each lane projects one voxel
//            centre through the camera's 3x4 matrix (held in LDS), tests the field of
//            view, interpolates the depth model at the sample and evaluates the depth
//            weight -- once per sample, not once per channel.  Surviving samples are
//            compacted, in (camera, height) order, into a per-slot list in LDS.
//   phase B  lanes = (slot, channel vector).  Each slot walks its list; every entry is
//            four 128-bit gathers per lane from the channels-last feature map, coalesced
//            across the lanes of the slot, accumulated in registers.
// The frustum volume never exists in memory.  The backward kernel repeats phase A with the
// derivative terms added to each entry; its phase B scatters feature gradients with
// hardware fp32 atomics (one per channel and corner) and reduces the per-sample inner
// product <grad_out, sampled feature> across the slot before issuing the depth atomics
// (8 per sample instead of 8 per sample and channel).
//
// Arithmetic contract: this file is compiled with -ffp-contract=off.  The geometry
// (projection, mask, indices, bilinear fractions) uses individually rounded fp32
// operations in a fixed order so that masks and indices are reproducible bit for bit;
// fused multiply-adds appear only where written explicitly (the channel accumulation).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "flashbev_hip.h"

namespace {

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kTile = 8;            // BEV cells are walked in 8x8 tiles for gather locality
constexpr int kMaxSlotLdsBytes = 12 * 1024;  // per-wave budget for the compacted lists
constexpr int kMaxBlockLdsBytes = 64 * 1024; // dynamic LDS a block may ask for without opting in

struct KParams {
    int B, N, H, W, C;
    int gx, gy, gz;
    int NZ;              // N * gz samples per cell
    int tiles_x, tiles_y;
    int padded_cells;    // tiles_x * tiles_y * 64
    int blocks_per_batch;
    int slots;           // S: cells per wavefront per round
    int rounds;          // rounds per wavefront
    int lanes_per_slot;  // lanes that carry channels in phase B
    int list_cap;        // entries per slot list (= NZ)
    float Wi_f, Hi_f, W_f, H_f;
    float xmin, ymin, zmin, vx, vy, vz;
    float eps, thr;
    int dist, Dd;
    float dmin, dstep;
    int reduce_sum;
    int proj_stride;
    int n_blocks;
};

// ---------------------------------------------------------------- element access
struct bf16_raw { uint16_t v; };

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }
template <> __device__ __forceinline__ float to_f32<bf16_raw>(bf16_raw v) {
    return __uint_as_float(((uint32_t)v.v) << 16);
}

// Load VEC consecutive elements (16 bytes when VEC > 1) and widen to fp32.
template <typename T, int VEC> struct VecLoad;
template <> struct VecLoad<float, 4> {
    static __device__ __forceinline__ void ld(const float *p, float (&o)[4]) {
        float4 v = *reinterpret_cast<const float4 *>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct VecLoad<float, 1> {
    static __device__ __forceinline__ void ld(const float *p, float (&o)[1]) { o[0] = *p; }
};
template <> struct VecLoad<__half, 8> {
    static __device__ __forceinline__ void ld(const __half *p, float (&o)[8]) {
        uint4 v = *reinterpret_cast<const uint4 *>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __half2 h = *reinterpret_cast<const __half2 *>(&w[i]);
            float2 f = __half22float2(h);
            o[2 * i] = f.x; o[2 * i + 1] = f.y;
        }
    }
};
template <> struct VecLoad<__half, 1> {
    static __device__ __forceinline__ void ld(const __half *p, float (&o)[1]) { o[0] = __half2float(*p); }
};
template <> struct VecLoad<bf16_raw, 8> {
    static __device__ __forceinline__ void ld(const bf16_raw *p, float (&o)[8]) {
        uint4 v = *reinterpret_cast<const uint4 *>(p);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = __uint_as_float(w[i] << 16);
            o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};
template <> struct VecLoad<bf16_raw, 1> {
    static __device__ __forceinline__ void ld(const bf16_raw *p, float (&o)[1]) { o[0] = to_f32(*p); }
};

// ---------------------------------------------------------------- geometry
struct Geom {
    bool valid;
    int u0, u1, v0, v1;
    float du, dv;
    float depth;
};

// One sample in the canonical operation order (each line is one rounded fp32 operation
// sequence, left to right; no contraction).  P points at 12 floats.
__device__ __forceinline__ Geom project_sample(const KParams &k, const float *P, float x, float y, float z) {
    Geom g;
    g.valid = false;
    g.u0 = g.u1 = g.v0 = g.v1 = 0;
    g.du = g.dv = 0.0f;
    float U = ((P[0] * x + P[1] * y) + P[2] * z) + P[3];
    float V = ((P[4] * x + P[5] * y) + P[6] * z) + P[7];
    float D = ((P[8] * x + P[9] * y) + P[10] * z) + P[11];
    g.depth = D;
    if (!(D > 0.0f)) return g;
    float dc = fmaxf(D, k.eps);
    float ui = U / dc;
    float vi = V / dc;
    float fu = (ui / k.Wi_f) * k.W_f;
    float fv = (vi / k.Hi_f) * k.H_f;
    if (!(fu >= 0.0f && fu < k.W_f && fv >= 0.0f && fv < k.H_f)) return g;
    float u0f = floorf(fu), v0f = floorf(fv);
    g.du = fu - u0f;
    g.dv = fv - v0f;
    g.u0 = min(max((int)u0f, 0), k.W - 1);
    g.u1 = min(max(g.u0 + 1, 0), k.W - 1);
    g.v0 = min(max((int)v0f, 0), k.H - 1);
    g.v1 = min(max(g.v0 + 1, 0), k.H - 1);
    g.valid = true;
    return g;
}

__device__ __forceinline__ float voxel_coord(float lo, int i, float step) {
    return lo + ((float)i + 0.5f) * step;
}

__device__ __forceinline__ float bilerp(float w00, float w01, float w10, float w11,
                                        float a00, float a01, float a10, float a11) {
    return ((w00 * a00 + w01 * a01) + w10 * a10) + w11 * a11;
}

// Depth weight of one sample and, for the backward pass, what its gradient needs.
struct DepthEval {
    float wgt;
    float a, b;   // parametric: d wgt/d mean, d wgt/d sigma.  categorical: (1-r), r
    int k0, k1;   // categorical bins (0, 1 for the parametric models)
    bool keep;
};

template <typename T>
__device__ __forceinline__ DepthEval eval_depth(const KParams &k, const T *__restrict__ depth,
                                                long long t00, long long t01, long long t10, long long t11,
                                                float w00, float w01, float w10, float w11, float D) {
    DepthEval e;
    e.wgt = 0.0f; e.a = 0.0f; e.b = 0.0f; e.k0 = 0; e.k1 = 1; e.keep = false;
    const int Dd = k.Dd;
    if (k.dist == FBEV_CATEGORICAL) {
        float t = (D - k.dmin) / k.dstep;
        if (!(t >= 0.0f && t <= (float)(Dd - 1))) return e;
        float k0f = floorf(t);
        e.k0 = min(max((int)k0f, 0), Dd - 1);
        e.k1 = min(e.k0 + 1, Dd - 1);
        float r = t - k0f;
        float p0 = bilerp(w00, w01, w10, w11, to_f32(depth[t00 * Dd + e.k0]), to_f32(depth[t01 * Dd + e.k0]),
                          to_f32(depth[t10 * Dd + e.k0]), to_f32(depth[t11 * Dd + e.k0]));
        float p1 = bilerp(w00, w01, w10, w11, to_f32(depth[t00 * Dd + e.k1]), to_f32(depth[t01 * Dd + e.k1]),
                          to_f32(depth[t10 * Dd + e.k1]), to_f32(depth[t11 * Dd + e.k1]));
        e.a = 1.0f - r;
        e.b = r;
        e.wgt = e.a * p0 + r * p1;
    } else {
        float mu = bilerp(w00, w01, w10, w11, to_f32(depth[t00 * 2]), to_f32(depth[t01 * 2]),
                          to_f32(depth[t10 * 2]), to_f32(depth[t11 * 2]));
        float sg = bilerp(w00, w01, w10, w11, to_f32(depth[t00 * 2 + 1]), to_f32(depth[t01 * 2 + 1]),
                          to_f32(depth[t10 * 2 + 1]), to_f32(depth[t11 * 2 + 1]));
        float s = sg + k.eps;
        float zs = (D - mu) / s;
        if (k.dist == FBEV_GAUSSIAN) {
            e.wgt = expf((-0.5f * zs) * zs) / s;
            e.a = e.wgt * zs / s;
            e.b = e.wgt * (zs * zs - 1.0f) / s;
        } else {
            e.wgt = (0.5f * expf(-fabsf(zs))) / s;
            float sgn = (zs > 0.0f) ? 1.0f : ((zs < 0.0f) ? -1.0f : 0.0f);
            e.a = e.wgt * sgn / s;
            e.b = e.wgt * (fabsf(zs) - 1.0f) / s;
        }
    }
    e.keep = !(e.wgt < k.thr);
    return e;
}

// Cell index inside one batch element's padded 8x8-tiled walk -> (ix, iy).
__device__ __forceinline__ bool cell_of(const KParams &k, int q, int &ix, int &iy) {
    int tile = q >> 6, l = q & 63;
    int ty = tile / k.tiles_x, tx = tile - ty * k.tiles_x;
    ix = tx * kTile + (l & 7);
    iy = ty * kTile + (l >> 3);
    return q < k.padded_cells && ix < k.gx && iy < k.gy;
}

// Blocks are dealt round-robin to the 8 XCDs; renumber them so that each XCD walks one
// contiguous range of (batch, tile) space and its L2 keeps one batch element's maps.
__device__ __forceinline__ int xcd_swizzle(int bid, int n_blocks) {
    constexpr int kXcd = 8;
    int per = n_blocks / kXcd;
    int main = per * kXcd;
    if (bid >= main) return bid;
    return (bid % kXcd) * per + bid / kXcd;
}

__device__ __forceinline__ unsigned long long lanemask_lt(int lane) {
    return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

// Entry of a compacted list: ENTRY_F4 float4 words.
//   word 0: forward: corner weights already multiplied by the depth weight
//           backward: raw bilinear corner weights (w00, w01, w10, w11)
//   word 1: four texel indices ((b*N+n)*H + v)*W + u as int bits (t00, t01, t10, t11)
//   word 2 (backward only): wgt, a, b, (k0 | k1 << 16)
template <int ENTRY_F4, typename T, bool BACKWARD>
__device__ __forceinline__ void phase_a(const KParams &k, const float *Pm, const T *__restrict__ depth,
                                        int b, int q0, int lane, float4 *lst, volatile int *cnt) {
    const int total = k.slots * k.NZ;
    for (int base = 0; base < total; base += kWave) {
        int idx = base + lane;
        bool active = idx < total;
        int slot = active ? idx / k.NZ : k.slots - 1;
        int s = idx - slot * k.NZ;
        int cam = s / k.gz;
        int iz = s - cam * k.gz;
        int ix, iy;
        bool ok = active && cell_of(k, q0 + slot, ix, iy);
        float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w2 = w0;
        int4 tx = make_int4(0, 0, 0, 0);
        bool keep = false;
        if (ok) {
            float x = voxel_coord(k.xmin, ix, k.vx);
            float y = voxel_coord(k.ymin, iy, k.vy);
            float z = voxel_coord(k.zmin, iz, k.vz);
            Geom g = project_sample(k, Pm + cam * 12, x, y, z);
            if (g.valid) {
                float w00 = (1.0f - g.du) * (1.0f - g.dv);
                float w01 = (1.0f - g.du) * g.dv;
                float w10 = g.du * (1.0f - g.dv);
                float w11 = g.du * g.dv;
                int rowbase = (b * k.N + cam) * k.H;
                int t00 = (rowbase + g.v0) * k.W + g.u0;
                int t01 = (rowbase + g.v1) * k.W + g.u0;
                int t10 = (rowbase + g.v0) * k.W + g.u1;
                int t11 = (rowbase + g.v1) * k.W + g.u1;
                DepthEval e = eval_depth<T>(k, depth, t00, t01, t10, t11, w00, w01, w10, w11, g.depth);
                keep = e.keep;
                tx = make_int4(t00, t01, t10, t11);
                if (BACKWARD) {
                    w0 = make_float4(w00, w01, w10, w11);
                    w2 = make_float4(e.wgt, e.a, e.b, __int_as_float(e.k0 | (e.k1 << 16)));
                } else {
                    w0 = make_float4(w00 * e.wgt, w01 * e.wgt, w10 * e.wgt, w11 * e.wgt);
                }
            }
        }
        unsigned long long m = __ballot(keep);
        int lo = max(slot * k.NZ - base, 0);            // first lane of my slot this iteration
        int hi = min((slot + 1) * k.NZ - base, kWave);   // one past its last lane
        unsigned long long seg = (~0ull << lo) & (hi >= 64 ? ~0ull : ((1ull << hi) - 1ull));
        int prefix = __popcll(m & seg & lanemask_lt(lane));
        int old = cnt[slot];
        if (keep) {
            float4 *e = lst + (size_t)(slot * k.list_cap + old + prefix) * ENTRY_F4;
            e[0] = w0;
            e[1] = make_float4(__int_as_float(tx.x), __int_as_float(tx.y), __int_as_float(tx.z),
                               __int_as_float(tx.w));
            if (ENTRY_F4 > 2) e[2] = w2;
        }
        if (active && lane == lo) cnt[slot] = old + __popcll(m & seg);
    }
}

// ---------------------------------------------------------------- forward
template <typename T, int VEC, int CPL>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_forward_kernel(
    KParams k, const T *__restrict__ depth, const T *__restrict__ feats, const float *__restrict__ proj,
    float *__restrict__ out) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = bid / k.blocks_per_batch;
    const int blk = bid - b * k.blocks_per_batch;

    // LDS: [N*12 floats of matrices, padded to float4][per wave: 16 ints of counts][lists]
    float *Pm = reinterpret_cast<float *>(smem);
    const int p_f4 = (k.N * 12 + 3) / 4;
    const int per_wave_f4 = 4 + k.slots * k.list_cap * 2;
    float4 *wbase = smem + p_f4 + wave * per_wave_f4;
    volatile int *cnt = reinterpret_cast<volatile int *>(wbase);
    float4 *lst = wbase + 4;

    for (int i = threadIdx.x; i < k.N * 12; i += blockDim.x)
        Pm[i] = proj[(size_t)(b * k.N + i / 12) * k.proj_stride + (i % 12)];
    __syncthreads();

    const int cells_per_wave = k.slots * k.rounds;
    const int slot = lane / k.lanes_per_slot;
    const int lis = lane - slot * k.lanes_per_slot;
    const bool carrier = slot < k.slots;
    const int span = k.lanes_per_slot * VEC * CPL;   // channels covered per pass

    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * kWavesPerBlock + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        if (lane < 16) cnt[lane] = 0;
        phase_a<2, T, false>(k, Pm, depth, b, q0, lane, lst, cnt);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        int ix = 0, iy = 0;
        bool mine = carrier && cell_of(k, q0 + slot, ix, iy);
        const int n = mine ? cnt[slot] : 0;
        const float4 *my = lst + (size_t)(carrier ? slot : 0) * k.list_cap * 2;
        float *o = out + (((size_t)b * k.gy + iy) * k.gx + ix) * k.C;
        for (int c0 = 0; c0 < k.C; c0 += span) {
            float acc[CPL][VEC];
#pragma unroll
            for (int j = 0; j < CPL; ++j)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[j][v] = 0.0f;
            for (int e = 0; e < n; ++e) {
                float4 w = my[2 * e];
                float4 tf = my[2 * e + 1];
                const T *p00 = feats + (size_t)__float_as_int(tf.x) * k.C;
                const T *p01 = feats + (size_t)__float_as_int(tf.y) * k.C;
                const T *p10 = feats + (size_t)__float_as_int(tf.z) * k.C;
                const T *p11 = feats + (size_t)__float_as_int(tf.w) * k.C;
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
            }
            if (mine) {
                const float nf = (float)n;
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        float res[VEC];
#pragma unroll
                        for (int v = 0; v < VEC; ++v)
                            res[v] = k.reduce_sum ? acc[j][v] : (n > 0 ? acc[j][v] / nf : 0.0f);
                        if (VEC == 1) {
                            o[ch] = res[0];
                        } else {
#pragma unroll
                            for (int v = 0; v < VEC; v += 4)
                                *reinterpret_cast<float4 *>(o + ch + v) =
                                    make_float4(res[v], res[v + 1], res[v + 2], res[v + 3]);
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ---------------------------------------------------------------- backward
__device__ __forceinline__ void atomic_add_f32(float *p, float v) { unsafeAtomicAdd(p, v); }

template <typename T, int VEC, int CPL>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_backward_kernel(
    KParams k, const float *__restrict__ grad_out, const T *__restrict__ depth, const T *__restrict__ feats,
    const float *__restrict__ proj, float *__restrict__ d_depth, float *__restrict__ d_feats) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = bid / k.blocks_per_batch;
    const int blk = bid - b * k.blocks_per_batch;

    float *Pm = reinterpret_cast<float *>(smem);
    const int p_f4 = (k.N * 12 + 3) / 4;
    const int per_wave_f4 = 4 + k.slots * k.list_cap * 3;
    float4 *wbase = smem + p_f4 + wave * per_wave_f4;
    volatile int *cnt = reinterpret_cast<volatile int *>(wbase);
    float4 *lst = wbase + 4;

    for (int i = threadIdx.x; i < k.N * 12; i += blockDim.x)
        Pm[i] = proj[(size_t)(b * k.N + i / 12) * k.proj_stride + (i % 12)];
    __syncthreads();

    const int cells_per_wave = k.slots * k.rounds;
    const int slot = lane / k.lanes_per_slot;
    const int lis = lane - slot * k.lanes_per_slot;
    const bool carrier = slot < k.slots;
    const int span = k.lanes_per_slot * VEC * CPL;
    const int Dd = k.Dd;

    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * kWavesPerBlock + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        if (lane < 16) cnt[lane] = 0;
        phase_a<3, T, true>(k, Pm, depth, b, q0, lane, lst, cnt);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        int ix = 0, iy = 0;
        bool mine = carrier && cell_of(k, q0 + slot, ix, iy);
        const int n = mine ? cnt[slot] : 0;
        // every lane of the wavefront takes part in the shuffles below, so all lanes run
        // the longest list of the wavefront and idle past their own.
        int n_max = n;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) n_max = max(n_max, __shfl_xor(n_max, off, kWave));
        const float4 *my = lst + (size_t)(carrier ? slot : 0) * k.list_cap * 3;
        const float *go = grad_out + (((size_t)b * k.gy + iy) * k.gx + ix) * k.C;
        const float inv = (k.reduce_sum || n == 0) ? 1.0f : 1.0f / (float)n;

        for (int c0 = 0; c0 < k.C; c0 += span) {
            float g[CPL][VEC];
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
#pragma unroll
                for (int v = 0; v < VEC; ++v) g[j][v] = 0.0f;
                if (mine && n > 0 && ch < k.C) {
                    if (VEC == 1) {
                        g[j][0] = go[ch] * inv;
                    } else {
#pragma unroll
                        for (int v = 0; v < VEC; v += 4) {
                            float4 t = *reinterpret_cast<const float4 *>(go + ch + v);
                            g[j][v] = t.x * inv; g[j][v + 1] = t.y * inv;
                            g[j][v + 2] = t.z * inv; g[j][v + 3] = t.w * inv;
                        }
                    }
                }
            }
            for (int e = 0; e < n_max; ++e) {
                const bool live = e < n;
                float G = 0.0f;
                float4 w = make_float4(0.f, 0.f, 0.f, 0.f), tf = w, dw = w;
                if (live) {
                    w = my[3 * e];
                    tf = my[3 * e + 1];
                    dw = my[3 * e + 2];
                    const size_t o00 = (size_t)__float_as_int(tf.x) * k.C;
                    const size_t o01 = (size_t)__float_as_int(tf.y) * k.C;
                    const size_t o10 = (size_t)__float_as_int(tf.z) * k.C;
                    const size_t o11 = (size_t)__float_as_int(tf.w) * k.C;
                    const float a00 = w.x * dw.x, a01 = w.y * dw.x, a10 = w.z * dw.x, a11 = w.w * dw.x;
#pragma unroll
                    for (int j = 0; j < CPL; ++j) {
                        int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                        if (ch < k.C) {
                            if (d_depth != nullptr) {
                                float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                                VecLoad<T, VEC>::ld(feats + o00 + ch, f00);
                                VecLoad<T, VEC>::ld(feats + o01 + ch, f01);
                                VecLoad<T, VEC>::ld(feats + o10 + ch, f10);
                                VecLoad<T, VEC>::ld(feats + o11 + ch, f11);
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    float f = bilerp(w.x, w.y, w.z, w.w, f00[v], f01[v], f10[v], f11[v]);
                                    G = __builtin_fmaf(g[j][v], f, G);
                                }
                            }
                            if (d_feats != nullptr) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) {
                                    atomic_add_f32(d_feats + o00 + ch + v, g[j][v] * a00);
                                    atomic_add_f32(d_feats + o01 + ch + v, g[j][v] * a01);
                                    atomic_add_f32(d_feats + o10 + ch + v, g[j][v] * a10);
                                    atomic_add_f32(d_feats + o11 + ch + v, g[j][v] * a11);
                                }
                            }
                        }
                    }
                }
                if (d_depth != nullptr) {
                    // sum G over the lanes of the slot: lane `lis` adds lane `lis + off`
#pragma unroll
                    for (int off = 32; off > 0; off >>= 1) {
                        float other = __shfl_down(G, off, kWave);
                        if (lis + off < k.lanes_per_slot) G += other;
                    }
                    if (live && lis == 0) {
                        const int kk = __float_as_int(dw.w);
                        const int k0 = kk & 0xffff, k1 = kk >> 16;
                        const float ga = G * dw.y, gb = G * dw.z;
                        const size_t t00 = (size_t)__float_as_int(tf.x) * Dd, t01 = (size_t)__float_as_int(tf.y) * Dd;
                        const size_t t10 = (size_t)__float_as_int(tf.z) * Dd, t11 = (size_t)__float_as_int(tf.w) * Dd;
                        atomic_add_f32(d_depth + t00 + k0, ga * w.x);
                        atomic_add_f32(d_depth + t00 + k1, gb * w.x);
                        atomic_add_f32(d_depth + t01 + k0, ga * w.y);
                        atomic_add_f32(d_depth + t01 + k1, gb * w.y);
                        atomic_add_f32(d_depth + t10 + k0, ga * w.z);
                        atomic_add_f32(d_depth + t10 + k1, gb * w.z);
                        atomic_add_f32(d_depth + t11 + k0, ga * w.w);
                        atomic_add_f32(d_depth + t11 + k1, gb * w.w);
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

// ---------------------------------------------------------------- geometry inspection
__global__ __launch_bounds__(256) void fbev_geometry_kernel(KParams k, const float *__restrict__ proj,
                                                            uint8_t *mask, int32_t *idx, float *frac,
                                                            long long total) {
    long long s = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= total) return;
    int iz = (int)(s % k.gz);
    long long r = s / k.gz;
    int n = (int)(r % k.N); r /= k.N;
    int ix = (int)(r % k.gx); r /= k.gx;
    int iy = (int)(r % k.gy);
    int b = (int)(r / k.gy);
    const float *P = proj + (size_t)(b * k.N + n) * k.proj_stride;
    float Pl[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) Pl[i] = P[i];
    Geom g = project_sample(k, Pl, voxel_coord(k.xmin, ix, k.vx), voxel_coord(k.ymin, iy, k.vy),
                            voxel_coord(k.zmin, iz, k.vz));
    if (mask) mask[s] = g.valid ? 1 : 0;
    if (idx) {
        idx[4 * s + 0] = g.valid ? g.u0 : -1;
        idx[4 * s + 1] = g.valid ? g.u1 : -1;
        idx[4 * s + 2] = g.valid ? g.v0 : -1;
        idx[4 * s + 3] = g.valid ? g.v1 : -1;
    }
    if (frac) {
        frac[2 * s + 0] = g.valid ? g.du : 0.0f;
        frac[2 * s + 1] = g.valid ? g.dv : 0.0f;
    }
}

// ---------------------------------------------------------------- host side
struct Plan {
    KParams k;
    int vec;        // elements per 16-byte load, or 1
    int cpl;        // channel vectors per lane per pass
    size_t lds_fwd, lds_bwd;
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
    return FBEV_OK;
}

int make_plan(const fbev_problem *p, bool allow_vec, Plan *plan) {
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
    k.dist = p->depth_distribution; k.Dd = p->depth_bins;
    k.dmin = p->depth_min; k.dstep = p->depth_step;
    k.reduce_sum = p->reduction == FBEV_REDUCE_SUM;
    k.proj_stride = p->proj_stride;

    const int es = elem_size(p->in_dtype);
    const int full_vec = 16 / es;
    plan->vec = (allow_vec && k.C % full_vec == 0) ? full_vec : 1;
    const int cq = (k.C + plan->vec - 1) / plan->vec;      // channel vectors per texel
    int lps = cq < kWave ? cq : kWave;
    int cpl = (cq + lps - 1) / lps;
    cpl = cpl <= 1 ? 1 : (cpl <= 2 ? 2 : 4);               // more than 4*lps vectors: extra passes
    plan->cpl = cpl;
    k.lanes_per_slot = lps;
    int slots = kWave / lps;
    // lists of both kernels must fit the per-wave LDS budget (3 float4 per entry in backward)
    const int entry_bytes = 48;
    while (slots > 1 && (long long)slots * k.NZ * entry_bytes > kMaxSlotLdsBytes) --slots;
    if (slots > 16) slots = 16;
    k.slots = slots;
    k.list_cap = k.NZ;
    // enough wavefronts to fill 256 CUs several times over before a wavefront takes more rounds
    const long long groups = ((long long)k.padded_cells + slots - 1) / slots * k.B;
    int rounds = (int)(groups / (256ll * 4 * 8 * 2));
    k.rounds = rounds < 1 ? 1 : (rounds > 8 ? 8 : rounds);
    const int cells_per_block = kWavesPerBlock * k.slots * k.rounds;
    k.blocks_per_batch = (k.padded_cells + cells_per_block - 1) / cells_per_block;
    k.n_blocks = k.blocks_per_batch * k.B;
    const size_t p_f4 = (size_t)(k.N * 12 + 3) / 4;
    plan->lds_fwd = (p_f4 + (size_t)kWavesPerBlock * (4 + (size_t)k.slots * k.list_cap * 2)) * 16;
    plan->lds_bwd = (p_f4 + (size_t)kWavesPerBlock * (4 + (size_t)k.slots * k.list_cap * 3)) * 16;
    if (plan->lds_bwd > (size_t)kMaxBlockLdsBytes) return FBEV_ERR_TOO_LARGE;
    return FBEV_OK;
}

template <typename T, int VEC>
int launch_forward(const Plan &pl, const void *depth, const void *feats, const float *proj, float *out,
                   hipStream_t st) {
    dim3 grid(pl.k.n_blocks), block(kWave * kWavesPerBlock);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    switch (pl.cpl) {
        case 1: hipLaunchKernelGGL((fbev_forward_kernel<T, VEC, 1>), grid, block, pl.lds_fwd, st, pl.k, d, f, proj, out); break;
        case 2: hipLaunchKernelGGL((fbev_forward_kernel<T, VEC, 2>), grid, block, pl.lds_fwd, st, pl.k, d, f, proj, out); break;
        default: hipLaunchKernelGGL((fbev_forward_kernel<T, VEC, 4>), grid, block, pl.lds_fwd, st, pl.k, d, f, proj, out); break;
    }
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

template <typename T, int VEC>
int launch_backward(const Plan &pl, const float *go, const void *depth, const void *feats, const float *proj,
                    float *dd, float *df, hipStream_t st) {
    dim3 grid(pl.k.n_blocks), block(kWave * kWavesPerBlock);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    switch (pl.cpl) {
        case 1: hipLaunchKernelGGL((fbev_backward_kernel<T, VEC, 1>), grid, block, pl.lds_bwd, st, pl.k, go, d, f, proj, dd, df); break;
        case 2: hipLaunchKernelGGL((fbev_backward_kernel<T, VEC, 2>), grid, block, pl.lds_bwd, st, pl.k, go, d, f, proj, dd, df); break;
        default: hipLaunchKernelGGL((fbev_backward_kernel<T, VEC, 4>), grid, block, pl.lds_bwd, st, pl.k, go, d, f, proj, dd, df); break;
    }
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int fbev_forward(const fbev_problem *p, const void *depth, const void *feats, const float *proj, float *out,
                 void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!depth || !feats || !proj || !out) return FBEV_ERR_NULL;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)proj % 4 || (uintptr_t)out % 4)
        return FBEV_ERR_ALIGNMENT;
    Plan pl;
    // 128-bit gathers and stores need 16-byte aligned feature and result tensors
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)out % 16 == 0, &pl);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_forward<float, 4>(pl, depth, feats, proj, out, st)
                               : launch_forward<float, 1>(pl, depth, feats, proj, out, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_forward<__half, 8>(pl, depth, feats, proj, out, st)
                               : launch_forward<__half, 1>(pl, depth, feats, proj, out, st);
        default:
            return pl.vec == 8 ? launch_forward<bf16_raw, 8>(pl, depth, feats, proj, out, st)
                               : launch_forward<bf16_raw, 1>(pl, depth, feats, proj, out, st);
    }
}

int fbev_backward(const fbev_problem *p, const float *grad_out, const void *depth, const void *feats,
                  const float *proj, float *d_depth, float *d_feats, void *stream) {
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    if (!grad_out || !depth || !feats || !proj) return FBEV_ERR_NULL;
    if (!d_depth && !d_feats) return FBEV_OK;
    const int es = elem_size(p->in_dtype);
    if ((uintptr_t)depth % es || (uintptr_t)feats % es || (uintptr_t)proj % 4 || (uintptr_t)grad_out % 4 ||
        (uintptr_t)d_depth % 4 || (uintptr_t)d_feats % 4)
        return FBEV_ERR_ALIGNMENT;
    Plan pl;
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0, &pl);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_backward<float, 4>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st)
                               : launch_backward<float, 1>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_backward<__half, 8>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st)
                               : launch_backward<__half, 1>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st);
        default:
            return pl.vec == 8 ? launch_backward<bf16_raw, 8>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st)
                               : launch_backward<bf16_raw, 1>(pl, grad_out, depth, feats, proj, d_depth, d_feats, st);
    }
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
    hipLaunchKernelGGL(fbev_geometry_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       static_cast<hipStream_t>(stream), pl.k, proj, mask, idx, frac, total);
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

int fbev_abi_version(void) { return FBEV_ABI_VERSION; }
size_t fbev_problem_size(void) { return sizeof(fbev_problem); }

}  // extern "C"
