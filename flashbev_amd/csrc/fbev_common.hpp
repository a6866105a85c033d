// Shared by every kernel of the library: per-kernel timers, tuning constants, the kernel
// parameter block, element access for the three input types, the canonical sample geometry and the
// depth models, and small wavefront helpers.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// ---------------------------------------------------------------- per-kernel timing (opt-in)
// While enabled, every kernel launch of this library is bracketed by a pair of HIP events
// on the launch stream; fbev_profile_collect() waits for them and returns total time and
// call count per kernel.  Disabled (the default) it costs one relaxed atomic load per launch.
namespace prof {
enum Kid { kForward, kBackwardScatter, kZero, kCount, kScanChunks, kScanSums, kBackwardCells, kBackwardTexel,
           kGeometry, kBackwardColumn, kCellCount, kPillar, kProjection, kForwardCached, kGeometryCache, kNum };
const char *const kNames[kNum] = {"fbev_forward_kernel", "fbev_backward_cells_kernel<scatter>",
                                  "fbev_fill_zero_kernel", "fbev_count_kernel", "fbev_scan_chunks_kernel",
                                  "fbev_scan_sums_kernel", "fbev_backward_cells_kernel<fill>",
                                  "fbev_backward_texel_kernel", "fbev_geometry_kernel",
                                  "fbev_backward_column_kernel", "fbev_forward_kernel<count only>",
                                  "fbev_pillar_kernel", "fbev_projection_kernel", "fbev_forward_cached_kernel",
                                  "fbev_geometry_cache_kernel"};
struct Rec { hipEvent_t a, b; int kid; };
std::atomic<bool> enabled{false};
std::mutex mu;
std::vector<Rec> recs;

struct Scope {
    hipStream_t st;
    Rec r;
    bool live;
    Scope(int kid, hipStream_t s) : st(s), live(enabled.load(std::memory_order_relaxed)) {
        if (!live) return;
        r.kid = kid;
        if (hipEventCreate(&r.a) != hipSuccess || hipEventCreate(&r.b) != hipSuccess) { live = false; return; }
        (void)hipEventRecord(r.a, st);
    }
    ~Scope() {
        if (!live) return;
        (void)hipEventRecord(r.b, st);
        std::lock_guard<std::mutex> g(mu);
        recs.push_back(r);
    }
};
}  // namespace prof

constexpr int kWave = 64;
constexpr int kWavesPerBlock = 4;
// The cell-centric kernels (forward, backward cell pass) hold several KB of LDS per wavefront:
// small blocks pack a CU's LDS better and are scheduled more evenly (measured: 2 wavefronts per
// block instead of 4, cell pass 6 % faster at the large configurations; forward 8 % faster on a
// 400x400x12 grid, 3 % at 128x128x8, equal at the largest).
constexpr int kCellPassWaves = 2;
constexpr int kTile = 8;            // BEV cells are walked in 8x8 tiles for gather locality
// Per-wavefront LDS budget for the compacted lists (sized for the worst case of N * gz entries per
// cell).  It leaves LDS for three wavefronts per SIMD: idle lane groups share a cell's list, so fewer
// cells per round cost less than the occupancy that longer lists would (400x400 grid, 64 channels,
// 16 height bins: forward 131 -> 117 us and cell pass 218 -> 186 us against budgets of 20 and 14 KB).
constexpr int kMaxSlotLdsBytes = 11500;
constexpr int kMaxBlockLdsBytes = 64 * 1024; // dynamic LDS a block may ask for without opting in
constexpr int kLdsLimitBytes = 150 * 1024;   // what a block may ask for at all (160 KiB per CU)
constexpr int kXcdCount = 8;                 // accelerator complex dies, each with its own L2
// The inverse map counts the samples per first-corner texel with integer atomics.  Atomics on
// one address execute one after the other, and the texels on the horizon collect thousands of
// samples, so every texel owns kReplicas counters and a sample picks one from its cell.
constexpr int kReplicaBits = 5;
constexpr int kReplicas = 1 << kReplicaBits;
// With fixed-capacity segments (no counting pass) a texel has four segments, again chosen by cell.
constexpr int kFixedReplicas = 4;
constexpr int kFixedMinSegment = 4;           // shorter segments would mostly overflow: count instead
constexpr long long kStreamOutputFrom = 32ll << 20;   // bytes of forward output beyond what the eight L2s hold
constexpr int kClaimRunsFrom = 300;           // possible samples per claim counter from which runs claim together
static_assert(kFixedReplicas == 4, "the texel pass numbers a texel's lists first corner + 4 * replica");
constexpr int kScanChunkBits = 12;           // counters are prefix-summed in chunks of 4096

struct KParams {
    int B, N, H, W, C;
    int gx, gy, gz;
    int NZ;              // N * gz samples per cell
    int tiles_x, tiles_y;
    int padded_cells;    // tiles_x * tiles_y * 64
    int blocks_per_batch;
    int slots;           // S: cells per group (phase B works on one group: its lane groups cover S cells)
    int batch_groups;    // groups that go through the sample phase together (1 to 4)
    int slots_a;         // cells per batch = slots * batch_groups (at most 16)
    int pool_cap;        // entries the pool of a wavefront holds (= slots * NZ)
    int rounds;          // batches per wavefront
    int lanes_per_slot;  // lanes that carry channels in phase B (one lane group)
    int groups_per_slot; // lane groups that share a slot's list (more than one when long lists leave few slots)
    int list_cap;        // entries per slot list (= NZ)
    float Wi_f, Hi_f, W_f, H_f;
    double xmin, ymin, zmin, vx, vy, vz;   // region of interest and cell size in float64 (see voxel_coord)
    float eps, thr;
    int dist, Dd;
    float dmin, dstep;
    int reduce_sum;
    int proj_stride;
    int n_blocks;
    int waves;           // wavefronts per block of the cell-centric kernels
    int bin_bits;        // a pair's first word is cell << bin_bits | depth bin; -1: the word cannot hold both
    int row_units;       // bytes of a texel's feature row (C * element size): rows are addressed by 32-bit byte offsets
    unsigned tiles_x_magic;   // tile / tiles_x == umulhi(tile, tiles_x_magic) for every tile of the walk
    unsigned lps_magic, gps_magic;   // lane / lanes_per_slot and group / groups_per_slot: (x * magic) >> 16 for x < 64
    unsigned cams_magic;      // i / N == umulhi(i, cams_magic) for i < 2^16
    unsigned bpb_magic;       // block / blocks_per_batch == umulhi(block, bpb_magic); 0: divide
    int gz_magic, gz_shift;   // i / gz == (i * gz_magic) >> gz_shift for 0 <= i < 4096
    unsigned geo_lo, geo_hi;  // hash of what a geometry cache depends on besides the matrices and the sizes above it:
                              // image size, region of interest, cell size, epsilon
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
// The (x, y) part of the three dot products is shared by all height bins of a (cell, camera)
// column: au = P[0] * x + P[1] * y, av and ad likewise.
__device__ __forceinline__ Geom project_column(const KParams &k, const float *P, float au, float av, float ad, float z) {
    Geom g;
    g.valid = false;
    g.u0 = g.u1 = g.v0 = g.v1 = 0;
    g.du = g.dv = 0.0f;
    float U = (au + P[2] * z) + P[3];
    float V = (av + P[6] * z) + P[7];
    float D = (ad + P[10] * z) + P[11];
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

// The same sample, evaluated without branches (the sample phase runs it on lanes that passed a cheap
// test, nearly all of which are in view): every operation is the one project_column performs, in the
// same order, so a sample in view gets the same bits; a sample out of view gets clamped indices and
// fractions nobody uses.
__device__ __forceinline__ Geom project_column_flat(const KParams &k, const float *P, float au, float av, float ad, float z) {
    Geom g;
    const float U = (au + P[2] * z) + P[3];
    const float V = (av + P[6] * z) + P[7];
    const float D = (ad + P[10] * z) + P[11];
    g.depth = D;
    const float dc = fmaxf(D, k.eps);
    const float ui = U / dc;
    const float vi = V / dc;
    const float fu = (ui / k.Wi_f) * k.W_f;
    const float fv = (vi / k.Hi_f) * k.H_f;
    g.valid = D > 0.0f && fu >= 0.0f && fu < k.W_f && fv >= 0.0f && fv < k.H_f;
    const float u0f = floorf(fu), v0f = floorf(fv);
    g.du = fu - u0f;
    g.dv = fv - v0f;
    g.u0 = min(max((int)u0f, 0), k.W - 1);
    g.u1 = min(g.u0 + 1, k.W - 1);
    g.v0 = min(max((int)v0f, 0), k.H - 1);
    g.v1 = min(g.v0 + 1, k.H - 1);
    return g;
}

__device__ __forceinline__ Geom project_sample(const KParams &k, const float *P, float x, float y, float z) {
    return project_column(k, P, P[0] * x + P[1] * y, P[4] * x + P[5] * y, P[8] * x + P[9] * y, z);
}

// Centre of cell i along one axis: evaluated in float64 and rounded once to fp32, so that it is the
// correctly rounded value of lo + (i + 0.5) * (hi - lo) / n.  An fp32 step would carry its rounding
// error i times along the axis (0.8 m is not an fp32 number), and a Gaussian tail weight multiplies
// that by z^2.  One float64 multiply-add per cell (x, y) and per height bin of a block (z, kept in
// an LDS table); nothing per sample.
__device__ __forceinline__ float voxel_coord(double lo, int i, double step) {
    return (float)(lo + ((double)i + 0.5) * step);
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
    int ty = k.tiles_x == 1 ? tile : (int)__umulhi((unsigned)tile, k.tiles_x_magic), tx = tile - ty * k.tiles_x;
    ix = tx * kTile + (l & 7);
    iy = ty * kTile + (l >> 3);
    return q < k.padded_cells && ix < k.gx && iy < k.gy;
}

// Blocks are dealt round-robin to the 8 XCDs; renumber them so that each XCD walks one
// contiguous range of (batch, tile) space and its L2 keeps one batch element's maps.
__device__ __forceinline__ int xcd_swizzle(int bid, int n_blocks) {
    constexpr int kXcd = kXcdCount;
    int per = n_blocks / kXcd;
    int main = per * kXcd;
    if (bid >= main) return bid;
    return (bid % kXcd) * per + bid / kXcd;
}

// Batch element of a (renumbered) block of the cell-centric kernels.
__device__ __forceinline__ int batch_of(const KParams &k, int bid) {
    if (k.B == 1) return 0;
    return k.bpb_magic ? (int)__umulhi((unsigned)bid, k.bpb_magic) : bid / k.blocks_per_batch;
}

__device__ __forceinline__ int replica_of(int ix, int iy) { return (ix + 5 * iy) & (kReplicas - 1); }

// Value of the lane whose index differs in bit 0 (bit 1) inside every group of four lanes.
// All 64 lanes must be active.
__device__ __forceinline__ float quad_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float quad_xor2(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
}

__device__ __forceinline__ unsigned long long lanemask_lt(int lane) {
    return lane == 0 ? 0ull : (~0ull >> (64 - lane));
}

__device__ __forceinline__ unsigned long long lanemask_le(int lane) { return ~0ull >> (63 - lane); }

}  // namespace
