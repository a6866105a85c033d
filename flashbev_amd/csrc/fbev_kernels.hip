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

#include <atomic>
#include <mutex>
#include <vector>

#include "flashbev_hip.h"

namespace {

// ---------------------------------------------------------------- per-kernel timing (opt-in)
// While enabled, every kernel launch of this library is bracketed by a pair of HIP events
// on the launch stream; fbev_profile_collect() waits for them and returns total time and
// call count per kernel.  Disabled (the default) it costs one relaxed atomic load per launch.
namespace prof {
enum Kid { kForward, kBackwardScatter, kZero, kCount, kScanChunks, kScanSums, kBackwardCells, kBackwardTexel,
           kGeometry, kBackwardColumn, kCellCount, kPillar, kProjection, kNum };
const char *const kNames[kNum] = {"fbev_forward_kernel", "fbev_backward_cells_kernel<scatter>",
                                  "fbev_fill_zero_kernel", "fbev_count_kernel", "fbev_scan_chunks_kernel",
                                  "fbev_scan_sums_kernel", "fbev_backward_cells_kernel<fill>",
                                  "fbev_backward_texel_kernel", "fbev_geometry_kernel",
                                  "fbev_backward_column_kernel", "fbev_forward_kernel<count only>",
                                  "fbev_pillar_kernel", "fbev_projection_kernel"};
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
// The backward's cell pass keeps three float4 per entry in LDS and about 100 VGPRs: smaller blocks
// pack the CU's LDS better (measured: 2 wavefronts per block 6 % faster than 4 at the large
// configurations; the forward prefers 4).
constexpr int kCellPassWaves = 2;
constexpr int kTile = 8;            // BEV cells are walked in 8x8 tiles for gather locality
constexpr int kMaxSlotLdsBytes = 14 * 1024;  // per-wave budget for the compacted lists
constexpr int kForwardSlotLdsBytes = 20000;  // the same for the forward kernel
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
    int slots;           // S: cells per wavefront per round
    int rounds;          // rounds per wavefront
    int lanes_per_slot;  // lanes that carry channels in phase B (one lane group)
    int groups_per_slot; // lane groups that share a slot's list (more than one when long lists leave few slots)
    int list_cap;        // entries per slot list (= NZ)
    float Wi_f, Hi_f, W_f, H_f;
    float xmin, ymin, zmin, vx, vy, vz;
    float eps, thr;
    int dist, Dd;
    float dmin, dstep;
    int reduce_sum;
    int proj_stride;
    int n_blocks;
    int waves;           // wavefronts per block of the cell-centric kernels
    int bin_bits;        // a pair's first word is cell << bin_bits | depth bin; -1: the word cannot hold both
    int row_units;       // a texel's feature row in address units: 16 bytes on the vector paths, else one element
    int gz_magic, gz_shift;   // i / gz == (i * gz_magic) >> gz_shift for 0 <= i < 4096
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

__device__ __forceinline__ Geom project_sample(const KParams &k, const float *P, float x, float y, float z) {
    return project_column(k, P, P[0] * x + P[1] * y, P[4] * x + P[5] * y, P[8] * x + P[9] * y, z);
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
    constexpr int kXcd = kXcdCount;
    int per = n_blocks / kXcd;
    int main = per * kXcd;
    if (bid >= main) return bid;
    return (bid % kXcd) * per + bid / kXcd;
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

// LDS of one block of the cell-centric kernels (float4 units):
//   [matrices: N*12 floats][column table: slots*N ints]
//   per wavefront: [16 ints of list lengths][16 float4 of cell centres][slots*N column records]
//   [slots*N ints: columns in view][slots*NZ ints of candidates][slots * list_cap entries]
// Counters that several lanes of a wavefront update in turn live in LDS and are read as
// volatile.  The pointer carries the LDS address space: a volatile access through a generic
// pointer becomes a system-coherent flat load that first waits for every outstanding global
// store and atomic of the wavefront.
using lds_counter = volatile __attribute__((address_space(3))) int;

struct WaveLds {
    const float *Pm;
    const int *dec;       // column index within the wavefront's round -> slot << 28 | camera << 16
    lds_counter *cnt;     // entries per slot
    float4 *cell;         // per slot: x, y, valid flag, ix | iy << 16
    float4 *col;          // per column: the (x, y) part of U, V, D, and its dec word
    int *alive;           // columns with a height bin that may be in view
    unsigned *cand;       // samples that survive the cheap test: column << 16 | height bin
    float4 *lst;
};

__device__ __forceinline__ int lds_p_f4(const KParams &k) { return (k.N * 12 + 3) / 4; }
__device__ __forceinline__ int lds_dec_f4(const KParams &k) { return (k.slots * k.N + 3) / 4; }
__device__ __forceinline__ int lds_cand_f4(const KParams &k) { return (k.slots * k.NZ + 3) / 4; }

// Stage the block's matrices and the column table; returns the wavefront's view.  Ends with a
// barrier.
__device__ __forceinline__ WaveLds block_lds_setup(const KParams &k, float4 *smem, const float *__restrict__ proj,
                                                   int b, int entry_f4) {
    WaveLds L;
    float *Pm = reinterpret_cast<float *>(smem);
    int *dec = reinterpret_cast<int *>(smem + lds_p_f4(k));
    const int dec_f4 = lds_dec_f4(k), cand_f4 = lds_cand_f4(k), cols = k.slots * k.N;
    const int per_wave_f4 = 4 + 16 + cols + dec_f4 + cand_f4 + k.slots * k.list_cap * entry_f4;
    float4 *wbase = smem + lds_p_f4(k) + dec_f4 + (threadIdx.x >> 6) * per_wave_f4;
    L.Pm = Pm;
    L.dec = dec;
    L.cnt = (lds_counter *)reinterpret_cast<int *>(wbase);
    L.cell = wbase + 4;
    L.col = wbase + 20;
    L.alive = reinterpret_cast<int *>(wbase + 20 + cols);
    L.cand = reinterpret_cast<unsigned *>(wbase + 20 + cols + dec_f4);
    L.lst = wbase + 20 + cols + dec_f4 + cand_f4;
    for (int i = threadIdx.x; i < k.N * 12; i += blockDim.x)
        Pm[i] = proj[(size_t)(b * k.N + i / 12) * k.proj_stride + (i % 12)];
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const int slot = i / k.N, cam = i - slot * k.N;
        dec[i] = (slot << 28) | (cam << 16);
    }
    __syncthreads();
    return L;
}

// Entry of a compacted list: ENTRY_F4 float4 words.
//   forward   word 0: corner weights already multiplied by the depth weight
//             word 1: where the four texels' feature rows start, in address units (texel index
//                     ((b*N+n)*H + v)*W + u times KParams::row_units) as int bits (t00, t01, t10, t11):
//                     the gather loop then forms an address with one shift-add, not a 64-bit multiply
//   backward  word 0: du, dv, t00, (u1 != u0) | (v1 != v0) << 1 -- the four weights and texels
//                     follow from these exactly as phase A computed them.  Inverse map: t00 << 2 with
//                     the two flags below it, and in the fourth place the position of the sample's
//                     pair in the pair array (sorted by first corner texel), or -1 if the array is full
//             word 1: wgt, a, b, (k0 | k1 << 16)
enum { kModeForward = 0, kModeScatter = 1, kModeFill = 2, kModeCount = 3, kModeFillRuns = 4 };

// Relative slack of the cheap field-of-view test.  A sample is dropped early only if its
// pixel coordinate misses the image by more than this fraction, far beyond any rounding of
// the exact test it would otherwise take (and fail).
constexpr float kEarlySlack = 1.0e-3f;

// Phase A of one round of a wavefront: the samples of its `slots` cells, in three stages.
//   stage 0  lanes = (cell, camera) columns: the (x, y) part of the three dot products, shared by
//            the column's height bins, and a test of the column's two end bins.  U, V and D are
//            monotone in the height bin (every rounded operation is), so a column whose end bins
//            both miss the image on the same side, or both lie behind the camera, holds no sample
//            that stage 1 could pass.  About three columns in four end here.
//   stage 1  lanes = height bins of the remaining columns: the rest of the dot products and a
//            division-free test that can only reject samples the exact test rejects too (behind
//            the camera, or outside the image by more than kEarlySlack).  Survivors are compacted,
//            in order, into the candidate list.
//   stage 2  lanes = candidates, densely packed: the canonical arithmetic (divisions, floor,
//            bilinear weights), the depth model, the weight threshold; what is kept goes, still
//            in (camera, height) order, into its slot's entry list.
// kModeCount writes no entries; it only counts the kept samples per (first-corner texel, replica).
template <int ENTRY_F4, typename T, int MODE>
__device__ __forceinline__ void phase_a(const KParams &k, const WaveLds &L, const T *__restrict__ depth, int b, int q0,
                                        int lane, const int *__restrict__ chunk_prefix = nullptr,
                                        int *__restrict__ cursor = nullptr, int pair_cap = 0) {
    constexpr bool FILLING = MODE == kModeFill || MODE == kModeFillRuns;   // the latter claims per run
    constexpr bool BACKWARD = MODE == kModeScatter || FILLING;
    const int n_cols = k.slots * k.N;
    if (lane < 16) L.cnt[lane] = 0;
    if (lane < k.slots) {
        int ix = 0, iy = 0;
        const bool ok = cell_of(k, q0 + lane, ix, iy);
        L.cell[lane] = make_float4(voxel_coord(k.xmin, ix, k.vx), voxel_coord(k.ymin, iy, k.vy), ok ? 1.0f : 0.0f,
                                   __int_as_float(ix | (iy << 16)));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    const float u_max = k.Wi_f * (1.0f + kEarlySlack), v_max = k.Hi_f * (1.0f + kEarlySlack);
    // ---- stage 0
    int n_alive = 0;
    const float z_first = voxel_coord(k.zmin, 0, k.vz), z_last = voxel_coord(k.zmin, k.gz - 1, k.vz);
    for (int base = 0; base < n_cols; base += kWave) {
        const int cc = base + lane;
        bool alive = false;
        if (cc < n_cols) {
            const int code = L.dec[cc];
            const float4 c = L.cell[(code >> 28) & 15];
            if (c.z != 0.0f) {
                const float *P = L.Pm + ((code >> 16) & 0xfff) * 12;
                const float au = P[0] * c.x + P[1] * c.y, av = P[4] * c.x + P[5] * c.y, ad = P[8] * c.x + P[9] * c.y;
                L.col[cc] = make_float4(au, av, ad, __int_as_float(code));
                const float d0 = (ad + P[10] * z_first) + P[11], d1 = (ad + P[10] * z_last) + P[11];
                const float d_hi = fmaxf(d0, d1);
                if (d_hi > 0.0f) {
                    const float u0 = (au + P[2] * z_first) + P[3], u1 = (au + P[2] * z_last) + P[3];
                    const float v0 = (av + P[6] * z_first) + P[7], v1 = (av + P[6] * z_last) + P[7];
                    // stage 1 compares every bin with bounds that grow with its clamped depth
                    const float dc = fmaxf(d_hi, k.eps), lo = -kEarlySlack * dc;
                    alive = fmaxf(u0, u1) >= lo && fminf(u0, u1) <= u_max * dc && fmaxf(v0, v1) >= lo &&
                            fminf(v0, v1) <= v_max * dc;
                }
            }
        }
        const unsigned long long m = __ballot(alive);
        if (alive) L.alive[n_alive + __popcll(m & lanemask_lt(lane))] = cc;
        n_alive += __popcll(m);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- stage 1
    int n_cand = 0;
    const int total = n_alive * k.gz;
    for (int base = 0; base < total; base += kWave) {
        const int idx = base + lane;
        bool pass = false;
        unsigned key = 0;
        if (idx < total) {
            const int a = (int)(__umul24((unsigned)idx, (unsigned)k.gz_magic) >> k.gz_shift);
            const int iz = idx - a * k.gz;
            const int cc = L.alive[a];
            const float4 col = L.col[cc];
            const float *P = L.Pm + ((__float_as_int(col.w) >> 16) & 0xfff) * 12;
            const float z = voxel_coord(k.zmin, iz, k.vz);
            const float D = (col.z + P[10] * z) + P[11];
            key = ((unsigned)cc << 16) | (unsigned)iz;
            if (D > 0.0f) {
                const float U = (col.x + P[2] * z) + P[3];
                const float V = (col.y + P[6] * z) + P[7];
                const float dc = fmaxf(D, k.eps), lo = -kEarlySlack * dc;
                pass = U >= lo && U <= u_max * dc && V >= lo && V <= v_max * dc;
            }
        }
        const unsigned long long m = __ballot(pass);
        if (pass) L.cand[n_cand + __popcll(m & lanemask_lt(lane))] = key;
        n_cand += __popcll(m);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- stage 2
    for (int base = 0; base < n_cand; base += kWave) {
        const int j = base + lane;
        const bool active = j < n_cand;
        const unsigned key = active ? L.cand[j] : 0u;
        const float4 col = active ? L.col[key >> 16] : make_float4(0.f, 0.f, 0.f, 0.f);
        const int d = __float_as_int(col.w);
        const int slot = active ? (d >> 28) & 15 : 16 + (lane & 1);   // idle lanes: no real slot
        const int cam = (d >> 16) & 0xfff;
        float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w2 = w0;
        int4 tx = make_int4(0, 0, 0, 0);
        int cellxy = 0;
        bool keep = false;
        if (active) {
            const float4 c = L.cell[slot];
            cellxy = __float_as_int(c.w);
            Geom g = project_column(k, L.Pm + cam * 12, col.x, col.y, col.z, voxel_coord(k.zmin, key & 0xffffu, k.vz));
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
                    const int fl = (g.u1 != g.u0 ? 1 : 0) | (g.v1 != g.v0 ? 2 : 0);
                    w0 = FILLING ? make_float4(g.du, g.dv, __int_as_float((t00 << 2) | fl), __int_as_float(-1))
                                           : make_float4(g.du, g.dv, __int_as_float(t00), __int_as_float(fl));
                    w2 = make_float4(e.wgt, e.a, e.b, __int_as_float(e.k0 | (e.k1 << 16)));
                } else {
                    w0 = make_float4(w00 * e.wgt, w01 * e.wgt, w10 * e.wgt, w11 * e.wgt);
                }
            }
        }
        const int prev_slot = __shfl_up(slot, 1, kWave);
        // Consecutive height bins of one (cell, camera) often fall on the same texel (far cells
        // compress onto the horizon rows).  Samples that repeat the first corner of the previous
        // kept sample of the same cell form a run; when counting, the run's first lane adds the
        // whole run with ONE atomic.  Positions are claimed per run as well where a claim counter
        // may get hundreds of samples (kModeFillRuns): claims on one address are served one
        // after the other, and a 400 x 400 x 12 grid on 4224 texels spent half of the cell pass
        // waiting for them.  Elsewhere the shuffles cost more than the saved returning atomics.
        int run_lead = lane, run_len = 1;
        if (MODE == kModeCount || MODE == kModeFillRuns) {
            const int prev_keep = __shfl_up((int)keep, 1, kWave);
            const int prev_texel = __shfl_up(tx.x, 1, kWave);      // every lane takes part in the exchange
            const bool cont = keep && lane > 0 && prev_keep != 0 && prev_slot == slot && prev_texel == tx.x;
            const unsigned long long cm = __ballot(cont);
            // first lane of my run: the highest lane at or below me that does not continue
            run_lead = 63 - __clzll(~cm & lanemask_le(lane));
            // lanes after me that continue without a gap
            const unsigned long long after = lane == 63 ? 0ull : (cm >> (lane + 1));
            run_len = 1 + (~after == 0ull ? 63 - lane : __ffsll((long long)~after) - 1);
        }
        if (MODE == kModeCount) {
            if (keep && run_lead == lane)
                atomicAdd(cursor + tx.x * kReplicas + replica_of(cellxy & 0xffff, cellxy >> 16), run_len);
            continue;
        }
        // candidates are in sample order, so the lanes of one slot are contiguous: [lo, hi)
        const unsigned long long bm = __ballot(lane == 0 || slot != prev_slot);
        const unsigned long long m = __ballot(keep);
        const int lo = 63 - __clzll(bm & lanemask_le(lane));
        const unsigned long long above = lane == 63 ? 0ull : (bm & ~lanemask_le(lane));
        const int hi = above ? __ffsll((long long)above) - 1 : kWave;
        const unsigned long long seg = (~0ull << lo) & (hi >= 64 ? ~0ull : ((1ull << hi) - 1ull));
        const int prefix = __popcll(m & seg & lanemask_lt(lane));
        const int old = active ? L.cnt[slot] : 0;
        if (keep) {
            float4 *e = L.lst + (size_t)(slot * k.list_cap + old + prefix) * ENTRY_F4;
            e[0] = w0;
            e[1] = BACKWARD ? w2
                            : make_float4(__int_as_float(tx.x * k.row_units), __int_as_float(tx.y * k.row_units),
                                          __int_as_float(tx.z * k.row_units), __int_as_float(tx.w * k.row_units));
        }
        if (MODE == kModeFill && keep) {
            // claim the sample's position in the list of its first corner texel
            int pos;
            if (chunk_prefix != nullptr) {
                // counted segments: cursor holds each segment's start within its scan chunk
                const int i0 = tx.x * kReplicas + replica_of(cellxy & 0xffff, cellxy >> 16);
                pos = atomicAdd(cursor + i0, 1) + chunk_prefix[i0 >> kScanChunkBits];
                pos = pos < pair_cap ? pos : -1;
            } else {
                // fixed segments of pair_cap pairs per (texel, replica): cursor counts from zero
                const int i0 = tx.x * kFixedReplicas + (replica_of(cellxy & 0xffff, cellxy >> 16) & (kFixedReplicas - 1));
                pos = atomicAdd(cursor + i0, 1);
                pos = pos < pair_cap ? i0 * pair_cap + pos : -1;
            }
            reinterpret_cast<int *>(L.lst + (size_t)(slot * k.list_cap + old + prefix) * ENTRY_F4)[3] = pos;
        }
        if (MODE == kModeFillRuns) {
            // the same, but the run's first lane claims for the whole run (same cell and texel: same
            // counter) and hands the positions out; every lane takes part in the exchange
            const int rep = replica_of(cellxy & 0xffff, cellxy >> 16);
            const bool counted = chunk_prefix != nullptr;
            const int i0 = counted ? tx.x * kReplicas + rep : tx.x * kFixedReplicas + (rep & (kFixedReplicas - 1));
            int pos = 0;
            if (keep && run_lead == lane) pos = atomicAdd(cursor + i0, run_len);
            pos = __shfl(pos, run_lead, kWave) + (lane - run_lead);
            if (keep) {
                if (counted) {
                    pos += chunk_prefix[i0 >> kScanChunkBits];
                    pos = pos < pair_cap ? pos : -1;
                } else {
                    pos = pos < pair_cap ? i0 * pair_cap + pos : -1;
                }
                reinterpret_cast<int *>(L.lst + (size_t)(slot * k.list_cap + old + prefix) * ENTRY_F4)[3] = pos;
            }
        }
        if (active && lane == lo) L.cnt[slot] = old + __popcll(m & seg);
    }
}

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
template <typename T>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_count_kernel(KParams k, const T *__restrict__ depth,
                                                                         const float *__restrict__ proj,
                                                                         int *__restrict__ counts) {
    extern __shared__ float4 smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = bid / k.blocks_per_batch;
    const int blk = bid - b * k.blocks_per_batch;
    const WaveLds L = block_lds_setup(k, smem, proj, b, 0);
    const int cells_per_wave = k.slots * k.rounds;
    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        phase_a<0, T, kModeCount>(k, L, depth, b, q0, lane, nullptr, counts, 0);
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

// Cell pass of the backward.  FILL = 0: scatter with atomics.  FILL = 1: write pairs (inverse
// map); FILL = 2: the same with one claim per run of samples on one texel.
// `cursor` holds, on entry, the start (within its scan chunk) of every (texel, replica)
// segment; phase A advances it, so on exit cursor[i] is the END of segment i.
template <typename T, int VEC, int CPL, int FILL>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_backward_cells_kernel(
    KParams k, const float *__restrict__ grad_out, const T *__restrict__ depth, const T *__restrict__ feats,
    const float *__restrict__ proj, float *__restrict__ d_depth, float *__restrict__ d_feats,
    const int *__restrict__ chunk_prefix, int *__restrict__ cursor, Pair *__restrict__ pairs, int pair_cap) {
    extern __shared__ float4 smem[];
    constexpr int EF4 = 2;
    // first corner texel and clamp flags of an entry
    auto entry_texel = [](const float4 &geo) { return FILL ? __float_as_int(geo.z) >> 2 : __float_as_int(geo.z); };
    auto entry_flags = [](const float4 &geo) { return FILL ? __float_as_int(geo.z) & 3 : __float_as_int(geo.w); };
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int bid = xcd_swizzle(blockIdx.x, k.n_blocks);
    const int b = bid / k.blocks_per_batch;
    const int blk = bid - b * k.blocks_per_batch;

    const WaveLds L = block_lds_setup(k, smem, proj, b, EF4);
    lds_counter *cnt = L.cnt;
    float4 *lst = L.lst;

    const int cells_per_wave = k.slots * k.rounds;
    // lane groups of lanes_per_slot lanes; the groups_per_slot groups of a slot take its entries in turn
    const int gps = k.groups_per_slot;
    const int group = lane / k.lanes_per_slot;
    const int slot = group / gps, sub = group - slot * gps;
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
    constexpr int kUnitShift = VEC > 1 ? 4 : (sizeof(T) == 4 ? 2 : 1);
    const char *fbytes = reinterpret_cast<const char *>(feats);
    const unsigned row_step_v = (unsigned)(k.W * k.row_units);      // one feature-map row down

    for (int r = 0; r < k.rounds; ++r) {
        const int q0 = (blk * k.waves + wave) * cells_per_wave + r * k.slots;
        if (q0 >= k.padded_cells) break;
        int ix = 0, iy = 0;
        const bool mine = carrier && cell_of(k, q0 + slot, ix, iy);
        const int cell = (b * k.gy + iy) * k.gx + ix;
        const float *go = grad_out + (size_t)cell * k.C;
        // the cell's grad_out row (first channel pass) is requested before phase A and arrives
        // while the samples are evaluated
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
        load_g(0);
        phase_a<EF4, T, FILL == 2 ? kModeFillRuns : (FILL ? kModeFill : kModeScatter)>(k, L, depth, b, q0, lane, chunk_prefix, cursor, pair_cap);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        const int n = mine ? cnt[slot] : 0;
        // every lane of the wavefront takes part in the shuffles below, so all lanes run
        // the longest list of the wavefront and idle past their own.
        int n_max = n;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) n_max = max(n_max, __shfl_xor(n_max, off, kWave));
        float4 *my = lst + (size_t)(carrier ? slot : 0) * k.list_cap * EF4;
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
                // feature rows in address units: one 32-bit multiply and three adds, then a shift-add each
                const unsigned r00 = (unsigned)t00 * (unsigned)k.row_units;
                const unsigned r01 = r00 + ((fl & 2) ? row_step_v : 0u);
                const unsigned r10 = r00 + ((fl & 1) ? (unsigned)k.row_units : 0u), r11 = r01 + (r10 - r00);
                // scatter path, or a sample without room in the pair array: atomics for all four corners
                const bool spill = FILL ? __float_as_int(geo.w) < 0 : true;
                const bool s00 = spill, s01 = spill, s10 = spill, s11 = spill;
                const float a00 = w00 * wgt, a01 = w01 * wgt, a10 = w10 * wgt, a11 = w11 * wgt;
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const int ch = c0 + (j * k.lanes_per_slot + lis) * VEC;
                    if (ch < k.C) {
                        if (need_G) {
                            float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                            VecLoad<T, VEC>::ld(reinterpret_cast<const T *>(fbytes + ((size_t)r00 << kUnitShift)) + ch, f00);
                            VecLoad<T, VEC>::ld(reinterpret_cast<const T *>(fbytes + ((size_t)r01 << kUnitShift)) + ch, f01);
                            VecLoad<T, VEC>::ld(reinterpret_cast<const T *>(fbytes + ((size_t)r10 << kUnitShift)) + ch, f10);
                            VecLoad<T, VEC>::ld(reinterpret_cast<const T *>(fbytes + ((size_t)r11 << kUnitShift)) + ch, f11);
#pragma unroll
                            for (int v = 0; v < VEC; ++v) {
                                const float f = __builtin_fmaf(w11, f11[v], __builtin_fmaf(w10, f10[v],
                                                __builtin_fmaf(w01, f01[v], w00 * f00[v])));
                                G = __builtin_fmaf(g[j][v], f, G);
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
        __builtin_amdgcn_wave_barrier();
    }
}

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
constexpr int kTexelSplitBelow = 8192;
constexpr int kTexelPart = 128;
constexpr int kTexelOneWaveBelow = 100;      // possible samples per texel below which a block is one wavefront ...
constexpr int kTexelManyTexels = 50000;      // ... or three times that when there are this many texels
constexpr int kTexelTwoWavesBelow = 450;     // below which it is two wavefronts; four from there on
constexpr int kTexelSegs = 4 * kFixedReplicas;   // lists of a texel with fixed segments: 4 first corners x replicas
template <int VEC, int WAVES>
__global__ __launch_bounds__(kWave *WAVES) void fbev_backward_texel_kernel(
    KParams k, const float *__restrict__ grad_out, const int *__restrict__ chunk_prefix,
    const int *__restrict__ seg_end, const Pair *__restrict__ pairs, int pair_cap, float *__restrict__ d_depth,
    float *__restrict__ d_feats, int lanes_per_row, int depth_from_pairs, int fresh) {
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
            const int claimed = seg_end[i];
            spilled = claimed > pair_cap;
            my_len = max(min(claimed, pair_cap), 0);
        }
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
    const int n_parts = min((int)gridDim.y, (n_all + 4 * kTexelPart - 1) / (4 * kTexelPart));
    if ((int)blockIdx.y >= n_parts) return;      // uniform for the block (also when nothing was claimed)
    const bool shared_texel = n_parts > 1;
    // The gradient buffers were cleared by this call (fresh) and nothing but this block touches the
    // texel unless a list spilled: then its rows are stored, not added, and the pass ends without a
    // dependent load.
    const bool store_only = fresh != 0 && !shared_texel && __ballot(spilled) == 0ull;
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
    const unsigned out_units = (unsigned)(VEC > 1 ? k.C / 4 : k.C);
    const char *gbytes = reinterpret_cast<const char *>(grad_out);
    for (int c0 = 0; c0 < k.C; c0 += span) {
        const int ch = c0 + lir * VEC;
        const bool on = worker_lane && ch < k.C;
        const int ch_eff = on ? ch : 0, wslot_eff = min(wslot, wpw - 1);
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
            // where the pair's grad_out row starts, in units of 16 bytes (one float off the vector path)
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
                    VecLoad<float, VEC>::ld(reinterpret_cast<const float *>(gbytes + ((size_t)(unsigned)__float_as_int(rc.x) << kOutShift)) + ch_eff, g[q]);
                }
#pragma unroll
                for (int q = 0; q < UNR; ++q)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(coefs[q], g[q][v], acc[v]);
            }
            for (int i = full; i < n_lead; i += wpw) {
                const int j = i + wslot_eff;
                if (j < n_lead) {
                    const float2 rc = stage[j];
                    float g[VEC];
                    VecLoad<float, VEC>::ld(reinterpret_cast<const float *>(gbytes + ((size_t)(unsigned)__float_as_int(rc.x) << kOutShift)) + ch_eff, g);
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(rc.y, g[v], acc[v]);
                }
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
                if (shared_texel) atomic_add_f32(dst, sum);
                else if (store_only) *dst = sum;
                else *dst += sum;
            }
        }
        if (c0 == 0 && bin_sums) {
            for (int i = threadIdx.x; i < k.Dd; i += blockDim.x) {
                const float sum = bins[i];
                if (sum != 0.0f) {
                    float *dst = d_depth + (size_t)t * k.Dd + i;
                    if (shared_texel) atomic_add_f32(dst, sum);
                    else if (store_only) *dst = sum;
                    else *dst += sum;
                }
            }
        } else if (c0 == 0 && depth_from_pairs && threadIdx.x < 2) {
            float sum = 0.0f;
            for (int w = 0; w < nw; ++w) sum += part[w * stride + span + threadIdx.x];
            float *dst = d_depth + (size_t)t * 2 + threadIdx.x;
            if (shared_texel) atomic_add_f32(dst, sum);
            else if (store_only) *dst = sum;
            else *dst += sum;
        }
    }
}

// ---------------------------------------------------------------- backward, column owner
// One block owns one column (b, camera, u) of the feature map: all H texels of that column,
// all channels.  Every sample that touches the column lies in a thin wedge of the BEV grid.
//   (1) cull   keep the 8x8-cell tiles, then the cells, whose projected u-range can reach the
//              column.  For a perspective map u = U/D is monotone along every segment in
//              front of the camera, so its extremes over a box (tile footprint x height range)
//              or a segment (one cell, all heights) sit at the vertices / end points; whatever
//              comes near the camera plane is kept unconditionally.  Culling only discards:
//              every kept sample is decided by the canonical arithmetic.
//   (2) sample re-project the kept cells' samples; those with a corner in the column become
//              32-byte entries in LDS.
//   (3) G      per entry, <grad_out / count, sampled feature> (needed by the depth gradient).
//   (4) rows   bucket the entries' row contributions by row (LDS integer atomics), share the
//              slots of the block among the rows in proportion to their length, let every slot
//              gather grad_out rows into registers, and add the partial rows in a fixed order.
//   (5) store  every d_feats / d_depth element of the column is written by this block alone.
// No floating-point atomics on the feature gradient (LDS float atomics cost about two clocks
// per lane on this machine, global ones serialise per address), no workspace, one launch.
// The per-cell sample count that the mean divides by comes from the forward pass or from a
// recount launch.
constexpr int kColThreads = 512;
constexpr int kColWaves = kColThreads / kWave;
constexpr int kColCells = 2048;          // candidate cells per batch (32 tiles)
constexpr int kColEntries = 1024;        // entries buffered before they are consumed
constexpr int kColMaxRows = 256;
constexpr float kCullMargin = 0.05f;     // texels; fp32 error of u is < 1e-2 once D > kCullNear
constexpr float kCullNear = 0.25f;       // metres in front of the camera plane

struct ColParams {
    int n_tiles;          // tiles per batch element
    int lanes_per_slot;   // lanes that carry one grad_out row
    int slots;            // rows in flight per wavefront
    int part_stride;      // floats per slot in the partial-row buffer (C + 2, padded)
    int accumulate;       // add to the gradient buffers instead of overwriting them
    int n_blocks;
};

struct ColLds {
    float *Pm;
    lds_counter *ctrl;     // 0: tiles kept, 1: cells kept, 2: entries
    int *tiles, *cells, *contrib, *rowcnt, *rowstart, *rowfill, *wk_row, *wk_first, *wk_n;
    float4 *entries;
    float *G, *part;
};

// Append `keep` lanes' values to a list with one LDS atomic per wavefront.
__device__ __forceinline__ int wave_append(lds_counter *counter, bool keep, int lane) {
    const unsigned long long m = __ballot(keep);
    int base = 0;
    if (lane == 0 && m != 0ull) base = __hip_atomic_fetch_add((__attribute__((address_space(3))) int *)counter, __popcll(m), __ATOMIC_RELAXED,
                                                                __HIP_MEMORY_SCOPE_WORKGROUP);
    base = __shfl(base, 0, kWave);
    return base + __popcll(m & lanemask_lt(lane));
}

template <typename T, int VEC>
__device__ __forceinline__ void column_consume(const KParams &k, const ColParams &cp, const ColLds &L, int n_ent,
                                               int u, int rowbase, bool first_flush,
                                               const float *__restrict__ grad_out, const T *__restrict__ feats,
                                               float *__restrict__ d_depth, float *__restrict__ d_feats) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int slot = lane / cp.lanes_per_slot, lis = lane - slot * cp.lanes_per_slot;
    const bool carrier = slot < cp.slots;
    const int worker = wave * cp.slots + slot, n_workers = kColWaves * cp.slots;
    const int span = cp.lanes_per_slot * VEC;
    const bool need_f = d_feats != nullptr, need_d = d_depth != nullptr;
    const bool parametric = k.dist != FBEV_CATEGORICAL;
    const int Dd = k.Dd;

    // ---- (3) G per entry.  UNR entries per slot could be kept in flight; measured, a deeper
    // pipeline costs more in occupancy than it hides in latency, so it stays at one.
    if (need_d) {
        constexpr int UNR = 1;
        const int iters = (n_ent + n_workers - 1) / n_workers;
        for (int it = 0; it < iters; it += UNR) {
            bool live[UNR];
            float G[UNR], w00[UNR], w01[UNR], w10[UNR], w11[UNR];
            const float *go[UNR];
            const T *p00[UNR], *p01[UNR], *p10[UNR], *p11[UNR];
#pragma unroll
            for (int q = 0; q < UNR; ++q) {
                const int e = (it + q) * n_workers + worker;
                live[q] = carrier && it + q < iters && e < n_ent;
                G[q] = 0.0f;
                const float4 e0 = L.entries[2 * (live[q] ? e : 0)];
                const int word = __float_as_int(e0.x);
                const bool c0 = (word >> 30) & 1, c1 = (word >> 31) & 1;
                const int v0 = __float_as_int(e0.y) & 0xffff, v1 = (__float_as_int(e0.y) >> 16) & 0xffff;
                const float du = e0.z, dv = e0.w;
                w00[q] = (1.0f - du) * (1.0f - dv); w01[q] = (1.0f - du) * dv;
                w10[q] = du * (1.0f - dv); w11[q] = du * dv;
                const int u0 = c0 ? u : u - 1;
                const int u1 = c0 ? (c1 ? u : min(u + 1, k.W - 1)) : u;
                go[q] = grad_out + (size_t)(word & 0x3fffffff) * k.C;
                p00[q] = feats + (size_t)((rowbase + v0) * k.W + u0) * k.C;
                p01[q] = feats + (size_t)((rowbase + v1) * k.W + u0) * k.C;
                p10[q] = feats + (size_t)((rowbase + v0) * k.W + u1) * k.C;
                p11[q] = feats + (size_t)((rowbase + v1) * k.W + u1) * k.C;
            }
            for (int ch = lis * VEC; ch < k.C; ch += span) {
                float g[UNR][VEC], f00[UNR][VEC], f01[UNR][VEC], f10[UNR][VEC], f11[UNR][VEC];
#pragma unroll
                for (int q = 0; q < UNR; ++q) {
                    if (live[q]) {
                        VecLoad<float, VEC == 1 ? 1 : 4>::ld(go[q] + ch, *reinterpret_cast<float(*)[VEC == 1 ? 1 : 4]>(&g[q][0]));
                        if (VEC == 8) VecLoad<float, 4>::ld(go[q] + ch + 4, *reinterpret_cast<float(*)[4]>(&g[q][VEC == 8 ? 4 : 0]));
                        VecLoad<T, VEC>::ld(p00[q] + ch, f00[q]);
                        VecLoad<T, VEC>::ld(p01[q] + ch, f01[q]);
                        VecLoad<T, VEC>::ld(p10[q] + ch, f10[q]);
                        VecLoad<T, VEC>::ld(p11[q] + ch, f11[q]);
                    }
                }
#pragma unroll
                for (int q = 0; q < UNR; ++q) {
                    if (live[q]) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v)
                            G[q] = __builtin_fmaf(g[q][v], bilerp(w00[q], w01[q], w10[q], w11[q], f00[q][v], f01[q][v], f10[q][v], f11[q][v]), G[q]);
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < UNR; ++q) {
                float Gq = G[q];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) {
                    const float other = __shfl_down(Gq, off, kWave);
                    if (lis + off < cp.lanes_per_slot) Gq += other;
                }
                if (live[q] && lis == 0) L.G[(it + q) * n_workers + worker] = Gq;
            }
        }
    }

    // ---- (4) rows, in groups of at most n_workers rows
    for (int row_base = 0; row_base < k.H; row_base += n_workers) {
        const int rows_here = min(n_workers, k.H - row_base);
        for (int i = tid; i < rows_here; i += kColThreads) { L.rowcnt[i] = 0; L.rowfill[i] = 0; }
        __syncthreads();
        for (int e = tid; e < n_ent; e += kColThreads) {
            const int vv = __float_as_int(L.entries[2 * e].y);
            const int r0 = (vv & 0xffff) - row_base, r1 = ((vv >> 16) & 0xffff) - row_base;
            if (r0 >= 0 && r0 < rows_here) atomicAdd(L.rowcnt + r0, 1);
            if (r1 >= 0 && r1 < rows_here) atomicAdd(L.rowcnt + r1, 1);
        }
        __syncthreads();
        if (tid == 0) {
            // prefix sum of the row lengths and slots per row: one each, the spare ones in proportion
            int total = 0, nonempty = 0;
            for (int r = 0; r < rows_here; ++r) { L.rowstart[r] = total; total += L.rowcnt[r]; nonempty += L.rowcnt[r] > 0; }
            L.rowstart[rows_here] = total;
            const int spare = n_workers - nonempty;
            int w = 0;
            for (int r = 0; r < rows_here; ++r) {
                const int c = L.rowcnt[r];
                if (c == 0) continue;
                int n = 1 + (int)(((long long)spare * c) / total);
                if (n > c) n = c;
                for (int i = 0; i < n; ++i) { L.wk_row[w + i] = r; L.wk_first[w + i] = w; L.wk_n[w + i] = n; }
                w += n;
            }
            for (; w < n_workers; ++w) L.wk_row[w] = -1;
        }
        __syncthreads();
        for (int e = tid; e < n_ent; e += kColThreads) {
            const int vv = __float_as_int(L.entries[2 * e].y);
            const int r0 = (vv & 0xffff) - row_base, r1 = ((vv >> 16) & 0xffff) - row_base;
            if (r0 >= 0 && r0 < rows_here) L.contrib[L.rowstart[r0] + atomicAdd(L.rowfill + r0, 1)] = e;
            if (r1 >= 0 && r1 < rows_here) L.contrib[L.rowstart[r1] + atomicAdd(L.rowfill + r1, 1)] = e | (1 << 30);
        }
        __syncthreads();

        // every slot gathers its share of one row into registers
        const int my_row = carrier ? L.wk_row[worker] : -1;
        float sa = 0.0f, sb = 0.0f;
        for (int cb = 0; cb < k.C; cb += span) {
            const int ch = cb + lis * VEC;
            float acc[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
            if (my_row >= 0) {
                const int part = worker - L.wk_first[worker], np = L.wk_n[worker];
                const int lo = L.rowstart[my_row], hi = L.rowstart[my_row + 1];
                constexpr int UNR = 1;
                for (int j0 = lo + part; j0 < hi; j0 += np * UNR) {
                    bool on[UNR];
                    float coef[UNR], g[UNR][VEC];
#pragma unroll
                    for (int q = 0; q < UNR; ++q) {
                        const int j = j0 + q * np;
                        on[q] = j < hi;
                        const int ce = L.contrib[on[q] ? j : lo];
                        const int e = ce & 0x3fffffff;
                        const bool second = (ce >> 30) & 1;             // this is the entry's v1 row
                        const float4 e0 = L.entries[2 * e];
                        const float4 e1 = L.entries[2 * e + 1];
                        const int word = __float_as_int(e0.x);
                        const bool c0 = (word >> 30) & 1, c1 = (word >> 31) & 1;
                        const float du = e0.z, dv = e0.w;
                        const float wv = second ? dv : 1.0f - dv;
                        // my column's bilinear weight in this row, same products as the forward
                        const float wc = (c0 ? (1.0f - du) * wv : 0.0f) + (c1 ? du * wv : 0.0f);
                        coef[q] = e1.x * wc;
                        if (on[q] && need_f && ch < k.C) {
                            const float *go = grad_out + (size_t)(word & 0x3fffffff) * k.C + ch;
                            VecLoad<float, VEC == 1 ? 1 : 4>::ld(go, *reinterpret_cast<float(*)[VEC == 1 ? 1 : 4]>(&g[q][0]));
                            if (VEC == 8) VecLoad<float, 4>::ld(go + 4, *reinterpret_cast<float(*)[4]>(&g[q][VEC == 8 ? 4 : 0]));
                        }
                        if (on[q] && need_d && cb == 0 && lis == 0) {
                            const float Gw = L.G[e] * wc;
                            if (parametric) {
                                sa = __builtin_fmaf(Gw, e1.y, sa);
                                sb = __builtin_fmaf(Gw, e1.z, sb);
                            } else {
                                // two bins per contribution: the column is owned, the adds only meet
                                // adds of this block
                                const int kk = __float_as_int(e1.w);
                                float *dst = d_depth + (size_t)((rowbase + row_base + my_row) * k.W + u) * Dd;
                                atomic_add_f32(dst + (kk & 0xffff), Gw * e1.y);
                                atomic_add_f32(dst + (kk >> 16), Gw * e1.z);
                            }
                        }
                    }
                    if (need_f && ch < k.C) {
#pragma unroll
                        for (int q = 0; q < UNR; ++q) {
                            if (on[q]) {
#pragma unroll
                                for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(coef[q], g[q][v], acc[v]);
                            }
                        }
                    }
                }
            }
            if (cb > 0) __syncthreads();         // the previous channel block has been read
            if (my_row >= 0) {
                float *pw = L.part + (size_t)worker * cp.part_stride;
                if (ch < k.C) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) pw[lis * VEC + v] = acc[v];
                }
                if (cb == 0 && lis == 0) { pw[span] = sa; pw[span + 1] = sb; }
            }
            __syncthreads();
            // fixed-order sum of the partial rows; rows without contributions are written as
            // zeros by the first flush so that the whole column is defined
            const int width = min(span, k.C - cb);
            for (int i = tid; i < rows_here * width; i += kColThreads) {
                const int r = i / width, c = i - r * width;
                float sum = 0.0f;
                bool any = false;
                for (int w = 0; w < n_workers; ++w) {
                    if (L.wk_row[w] == r) { sum += L.part[(size_t)w * cp.part_stride + c]; any = true; }
                }
                if (need_f && (any || first_flush)) {
                    float *dst = d_feats + (size_t)((rowbase + row_base + r) * k.W + u) * k.C + cb + c;
                    *dst = (first_flush && !cp.accumulate) ? sum : *dst + sum;
                }
            }
            if (cb == 0 && need_d && parametric) {
                for (int i = tid; i < rows_here * 2; i += kColThreads) {
                    const int r = i >> 1, c = i & 1;
                    float sum = 0.0f;
                    bool any = false;
                    for (int w = 0; w < n_workers; ++w) {
                        if (L.wk_row[w] == r) { sum += L.part[(size_t)w * cp.part_stride + span + c]; any = true; }
                    }
                    if (any || first_flush) {
                        float *dst = d_depth + (size_t)((rowbase + row_base + r) * k.W + u) * 2 + c;
                        *dst = (first_flush && !cp.accumulate) ? sum : *dst + sum;
                    }
                }
            }
        }
        __syncthreads();
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kColThreads) void fbev_backward_column_kernel(
    KParams k, ColParams cp, const float *__restrict__ grad_out, const T *__restrict__ depth,
    const T *__restrict__ feats, const float *__restrict__ proj, const float *__restrict__ count,
    float *__restrict__ d_depth, float *__restrict__ d_feats) {
    extern __shared__ float4 smem[];
    const int n_workers = kColWaves * cp.slots;
    ColLds L;
    L.Pm = reinterpret_cast<float *>(smem);
    L.ctrl = (lds_counter *)reinterpret_cast<int *>(smem + 4);
    L.entries = smem + 8;
    int *ip = reinterpret_cast<int *>(L.entries + 2 * kColEntries);
    L.tiles = ip; ip += kColThreads;
    L.cells = ip; ip += kColCells;
    L.contrib = ip; ip += 2 * kColEntries;
    L.rowcnt = ip; ip += kColMaxRows;
    L.rowstart = ip; ip += kColMaxRows + 4;
    L.rowfill = ip; ip += kColMaxRows;
    L.wk_row = ip; ip += 64;
    L.wk_first = ip; ip += 64;
    L.wk_n = ip; ip += 64;
    L.G = reinterpret_cast<float *>(ip); ip += kColEntries;
    L.part = reinterpret_cast<float *>(ip);
    (void)n_workers;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int bid = xcd_swizzle(blockIdx.x, cp.n_blocks);
    const int u = bid % k.W;
    const int cam = (bid / k.W) % k.N;
    const int b = bid / (k.W * k.N);
    const int Dd = k.Dd;
    const int rowbase = (b * k.N + cam) * k.H;

    if (tid < 12) L.Pm[tid] = proj[(size_t)(b * k.N + cam) * k.proj_stride + tid];
    if (tid < 4) L.ctrl[tid] = 0;
    // the categorical depth gradient is added with atomics below: define the owned region first
    if (d_depth != nullptr && k.dist == FBEV_CATEGORICAL && !cp.accumulate) {
        for (int i = tid; i < k.H * Dd; i += kColThreads)
            d_depth[(size_t)((rowbase + i / Dd) * k.W + u) * Dd + (i % Dd)] = 0.0f;
        __threadfence();
    }
    __syncthreads();
    const float *Pm = L.Pm;

    const float z_lo = voxel_coord(k.zmin, 0, k.vz), z_hi = voxel_coord(k.zmin, k.gz - 1, k.vz);
    const float u_lo = (float)(u - 1) - kCullMargin, u_hi = (float)(u + 1) + kCullMargin;
    bool first_flush = true;

    for (int tile_base = 0; tile_base < cp.n_tiles; tile_base += kColThreads) {
        // ---- (1a) tiles: one per thread
        {
            const int tile = tile_base + tid;
            bool keep = false;
            if (tile < cp.n_tiles) {
                const int ty = tile / k.tiles_x, tx = tile - ty * k.tiles_x;
                const int ix0 = tx * kTile, ix1 = min(ix0 + kTile, k.gx) - 1;
                const int iy0 = ty * kTile, iy1 = min(iy0 + kTile, k.gy) - 1;
                const float xs[2] = {voxel_coord(k.xmin, ix0, k.vx), voxel_coord(k.xmin, ix1, k.vx)};
                const float ys[2] = {voxel_coord(k.ymin, iy0, k.vy), voxel_coord(k.ymin, iy1, k.vy)};
                const float zs[2] = {z_lo, z_hi};
                float fu_min = 3.0e38f, fu_max = -3.0e38f, fv_min = 3.0e38f, fv_max = -3.0e38f, d_min = 3.0e38f,
                      d_max = -3.0e38f;
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const float x = xs[c & 1], y = ys[(c >> 1) & 1], z = zs[c >> 2];
                    const float U = ((Pm[0] * x + Pm[1] * y) + Pm[2] * z) + Pm[3];
                    const float V = ((Pm[4] * x + Pm[5] * y) + Pm[6] * z) + Pm[7];
                    const float D = ((Pm[8] * x + Pm[9] * y) + Pm[10] * z) + Pm[11];
                    d_min = fminf(d_min, D);
                    d_max = fmaxf(d_max, D);
                    const float dc = fmaxf(D, kCullNear);
                    const float fu = ((U / dc) / k.Wi_f) * k.W_f, fv = ((V / dc) / k.Hi_f) * k.H_f;
                    fu_min = fminf(fu_min, fu); fu_max = fmaxf(fu_max, fu);
                    fv_min = fminf(fv_min, fv); fv_max = fmaxf(fv_max, fv);
                }
                if (!(d_max > -1.0e-3f)) keep = false;                 // the whole box is behind the camera
                else if (!(d_min > kCullNear)) keep = true;            // too close to the camera plane to bound u
                else keep = fu_max >= u_lo && fu_min < u_hi && fv_max >= -kCullMargin &&
                            fv_min < k.H_f + kCullMargin;
            }
            const int pos = wave_append(&L.ctrl[0], keep, lane);
            if (keep) L.tiles[pos] = tile_base + tid;
        }
        __syncthreads();
        const int n_tiles_kept = L.ctrl[0];

        for (int tb = 0; tb < n_tiles_kept; tb += kColCells / 64) {
            // ---- (1b) cells of up to 32 kept tiles: u-range over the cell's height segment
            const int n_cell_tests = min(kColCells / 64, n_tiles_kept - tb) * 64;
            for (int c0 = 0; c0 < n_cell_tests; c0 += kColThreads) {
                const int ci = c0 + tid;
                bool keep = false;
                int packed = 0;
                if (ci < n_cell_tests) {
                    const int tile = L.tiles[tb + (ci >> 6)];
                    const int ty = tile / k.tiles_x, tx = tile - ty * k.tiles_x;
                    const int ix = tx * kTile + (ci & 7), iy = ty * kTile + ((ci >> 3) & 7);
                    if (ix < k.gx && iy < k.gy) {
                        const float x = voxel_coord(k.xmin, ix, k.vx), y = voxel_coord(k.ymin, iy, k.vy);
                        const float Uxy = Pm[0] * x + Pm[1] * y, Dxy = Pm[8] * x + Pm[9] * y;
                        const float Ua = (Uxy + Pm[2] * z_lo) + Pm[3], Da = (Dxy + Pm[10] * z_lo) + Pm[11];
                        const float Ub = (Uxy + Pm[2] * z_hi) + Pm[3], Db = (Dxy + Pm[10] * z_hi) + Pm[11];
                        const float dmin = fminf(Da, Db), dmax = fmaxf(Da, Db);
                        if (!(dmax > -1.0e-3f)) keep = false;
                        else if (!(dmin > kCullNear)) keep = true;
                        else {
                            const float fa = ((Ua / Da) / k.Wi_f) * k.W_f, fb = ((Ub / Db) / k.Wi_f) * k.W_f;
                            keep = fmaxf(fa, fb) >= u_lo && fminf(fa, fb) < u_hi;
                        }
                        packed = ix | (iy << 16);
                    }
                }
                const int pos = wave_append(&L.ctrl[1], keep, lane);
                if (keep) L.cells[pos] = packed;
            }
            __syncthreads();
            const int n_cells = L.ctrl[1];
            const int n_samples = n_cells * k.gz;

            // ---- (2) samples of the kept cells, one per thread and round
            for (int s0 = 0; s0 < n_samples; s0 += kColThreads) {
                {
                    const int idx = s0 + tid;
                    bool keep = false;
                    float4 e0 = make_float4(0.f, 0.f, 0.f, 0.f), e1 = e0;
                    if (idx < n_samples) {
                        const int ci = idx / k.gz, iz = idx - ci * k.gz;
                        const int packed = L.cells[ci];
                        const int ix = packed & 0xffff, iy = packed >> 16;
                        Geom g = project_sample(k, Pm, voxel_coord(k.xmin, ix, k.vx), voxel_coord(k.ymin, iy, k.vy),
                                                voxel_coord(k.zmin, iz, k.vz));
                        const bool c0 = g.u0 == u, c1 = g.u1 == u;
                        if (g.valid && (c0 || c1)) {
                            const float w00 = (1.0f - g.du) * (1.0f - g.dv), w01 = (1.0f - g.du) * g.dv;
                            const float w10 = g.du * (1.0f - g.dv), w11 = g.du * g.dv;
                            const int t00 = (rowbase + g.v0) * k.W + g.u0, t01 = (rowbase + g.v1) * k.W + g.u0;
                            const int t10 = (rowbase + g.v0) * k.W + g.u1, t11 = (rowbase + g.v1) * k.W + g.u1;
                            DepthEval e = eval_depth<T>(k, depth, t00, t01, t10, t11, w00, w01, w10, w11, g.depth);
                            if (e.keep) {
                                const int cell = (b * k.gy + iy) * k.gx + ix;
                                const float n = count[cell];
                                const float inv = k.reduce_sum ? 1.0f : (n > 0.0f ? 1.0f / n : 0.0f);
                                keep = true;
                                e0 = make_float4(__int_as_float(cell | (c0 ? (1 << 30) : 0) | (c1 ? (1 << 31) : 0)),
                                                 __int_as_float(g.v0 | (g.v1 << 16)), g.du, g.dv);
                                e1 = make_float4(e.wgt * inv, e.a * inv, e.b * inv, __int_as_float(e.k0 | (e.k1 << 16)));
                            }
                        }
                    }
                    const int pos = wave_append(&L.ctrl[2], keep, lane);
                    if (keep) {
                        L.entries[2 * pos] = e0;
                        L.entries[2 * pos + 1] = e1;
                    }
                }
                __syncthreads();
                const int n_ent = L.ctrl[2];
                if (n_ent + kColThreads > kColEntries) {
                    column_consume<T, VEC>(k, cp, L, n_ent, u, rowbase, first_flush, grad_out, feats, d_depth, d_feats);
                    first_flush = false;
                    __syncthreads();
                    if (tid == 0) L.ctrl[2] = 0;
                    __syncthreads();
                }
            }
            __syncthreads();
            if (tid == 0) L.ctrl[1] = 0;
            __syncthreads();
        }
        __syncthreads();
        if (tid == 0) L.ctrl[0] = 0;
        __syncthreads();
    }
    // whatever is left, and in any case one flush so that every element of the column is written
    const int n_ent = L.ctrl[2];
    if (n_ent > 0 || first_flush)
        column_consume<T, VEC>(k, cp, L, n_ent, u, rowbase, first_flush, grad_out, feats, d_depth, d_feats);
}

// ---------------------------------------------------------------- interval pooling (baseline)
// The reference's second method ("Sampling-VT + PillarPool"): the host projects every sample,
// keeps those in view, sorts them by BEV cell and hands over per-sample feature-map coordinates
// plus one (start, length) interval per touched cell.  Lanes = (interval, channel vector): the
// lanes of a slot walk their interval together; bilinear weights and the depth likelihood are
// evaluated by every lane of the slot (cheap beside the four row gathers).  No weight threshold;
// the mean runs over the samples that pass the kernel's own in-view test.
template <int VEC>
__global__ __launch_bounds__(kWave *kWavesPerBlock) void fbev_pillar_kernel(
    int C, int n_intervals, int H, int W, int lanes_per_slot, float eps, int laplace,
    const float *__restrict__ depth, const float *__restrict__ feats, const float *__restrict__ u_coords,
    const float *__restrict__ v_coords, const float *__restrict__ z_coords, const int *__restrict__ batch_camera,
    const int *__restrict__ ranks_bev, const int *__restrict__ interval_starts,
    const int *__restrict__ interval_lengths, float *__restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int slots = kWave / lanes_per_slot;
    const int slot = lane / lanes_per_slot, lis = lane - slot * lanes_per_slot;
    const long long interval = ((long long)blockIdx.x * kWavesPerBlock + wave) * slots + slot;
    if (slot >= slots || interval >= n_intervals) return;
    const int start = interval_starts[interval], len = interval_lengths[interval];
    const float Wf = (float)W, Hf = (float)H;
    const int span = lanes_per_slot * VEC;
    float *o = out + (size_t)ranks_bev[start] * C;
    for (int c0 = 0; c0 < C; c0 += span) {
        const int ch = c0 + lis * VEC;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
        int count = 0;
        for (int i = 0; i < len; ++i) {
            const float fu = u_coords[start + i], fv = v_coords[start + i], d = z_coords[start + i];
            if (!(fu >= 0.0f && fu < Wf && fv >= 0.0f && fv < Hf && d > 0.0f)) continue;
            const float u0f = floorf(fu), v0f = floorf(fv);
            const int u0 = (int)u0f, v0 = (int)v0f;
            const int u1 = min(u0 + 1, W - 1), v1 = min(v0 + 1, H - 1);
            const float du = fu - u0f, dv = fv - v0f;
            const float w00 = (1.0f - du) * (1.0f - dv), w01 = (1.0f - du) * dv, w10 = du * (1.0f - dv), w11 = du * dv;
            const size_t base = (size_t)batch_camera[start + i] * H * W;
            const size_t t00 = base + (size_t)v0 * W + u0, t01 = base + (size_t)v1 * W + u0;
            const size_t t10 = base + (size_t)v0 * W + u1, t11 = base + (size_t)v1 * W + u1;
            const float2 p00 = *reinterpret_cast<const float2 *>(depth + t00 * 2);
            const float2 p01 = *reinterpret_cast<const float2 *>(depth + t01 * 2);
            const float2 p10 = *reinterpret_cast<const float2 *>(depth + t10 * 2);
            const float2 p11 = *reinterpret_cast<const float2 *>(depth + t11 * 2);
            const float mu = bilerp(w00, w01, w10, w11, p00.x, p01.x, p10.x, p11.x);
            const float s = bilerp(w00, w01, w10, w11, p00.y, p01.y, p10.y, p11.y) + eps;
            const float zs = (d - mu) / s;
            const float wgt = laplace ? (0.5f * expf(-fabsf(zs))) / s : expf((-0.5f * zs) * zs) / s;
            ++count;
            if (ch < C) {
                float f00[VEC], f01[VEC], f10[VEC], f11[VEC];
                VecLoad<float, VEC>::ld(feats + t00 * C + ch, f00);
                VecLoad<float, VEC>::ld(feats + t01 * C + ch, f01);
                VecLoad<float, VEC>::ld(feats + t10 * C + ch, f10);
                VecLoad<float, VEC>::ld(feats + t11 * C + ch, f11);
                const float a00 = w00 * wgt, a01 = w01 * wgt, a10 = w10 * wgt, a11 = w11 * wgt;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    float a = acc[v];
                    a = __builtin_fmaf(a00, f00[v], a);
                    a = __builtin_fmaf(a01, f01[v], a);
                    a = __builtin_fmaf(a10, f10[v], a);
                    a = __builtin_fmaf(a11, f11[v], a);
                    acc[v] = a;
                }
            }
        }
        if (ch < C) {
            const float nf = (float)count;
#pragma unroll
            for (int v = 0; v < VEC; ++v) o[ch + v] = count > 0 ? acc[v] / nf : 0.0f;
        }
    }
}

// Projection matrices from calibration, one thread per camera (flashbev/flashbevpool/sampling_vt.py:21-33):
// K = post_rots * camera2imgs with post_trans added to its third column, E = inverse(sensor2ego),
// P = rows 0..2 of [K 0; 0 1] * E.  Everything is evaluated in double and rounded once; the inverse is
// the adjugate over the determinant from 2x2 minors, so a singular sensor2ego gives non-finite
// entries rather than an error.
__global__ __launch_bounds__(64) void fbev_projection_kernel(int count, const float *__restrict__ sensor2ego,
                                                            const float *__restrict__ camera2imgs,
                                                            const float *__restrict__ post_rots,
                                                            const float *__restrict__ post_trans,
                                                            float *__restrict__ proj) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    double a[16], r[9], c[9], kk[9];
    for (int j = 0; j < 16; ++j) a[j] = (double)sensor2ego[(size_t)i * 16 + j];
    for (int j = 0; j < 9; ++j) { r[j] = (double)post_rots[(size_t)i * 9 + j]; c[j] = (double)camera2imgs[(size_t)i * 9 + j]; }
    for (int row = 0; row < 3; ++row)
        for (int col = 0; col < 3; ++col)
            kk[row * 3 + col] = (r[row * 3] * c[col] + r[row * 3 + 1] * c[3 + col]) + r[row * 3 + 2] * c[6 + col];
    for (int row = 0; row < 3; ++row) kk[row * 3 + 2] += (double)post_trans[(size_t)i * 3 + row];
    const double s0 = a[0] * a[5] - a[4] * a[1], s1 = a[0] * a[6] - a[4] * a[2], s2 = a[0] * a[7] - a[4] * a[3];
    const double s3 = a[1] * a[6] - a[5] * a[2], s4 = a[1] * a[7] - a[5] * a[3], s5 = a[2] * a[7] - a[6] * a[3];
    const double c5 = a[10] * a[15] - a[14] * a[11], c4 = a[9] * a[15] - a[13] * a[11], c3 = a[9] * a[14] - a[13] * a[10];
    const double c2 = a[8] * a[15] - a[12] * a[11], c1 = a[8] * a[14] - a[12] * a[10], c0 = a[8] * a[13] - a[12] * a[9];
    const double inv_det = 1.0 / (s0 * c5 - s1 * c4 + s2 * c3 + s3 * c2 - s4 * c1 + s5 * c0);
    double e[12];   // rows 0..2 of the inverse (row 3 only meets the zero column of [K 0; 0 1])
    e[0] = (a[5] * c5 - a[6] * c4 + a[7] * c3) * inv_det;
    e[1] = (-a[1] * c5 + a[2] * c4 - a[3] * c3) * inv_det;
    e[2] = (a[13] * s5 - a[14] * s4 + a[15] * s3) * inv_det;
    e[3] = (-a[9] * s5 + a[10] * s4 - a[11] * s3) * inv_det;
    e[4] = (-a[4] * c5 + a[6] * c2 - a[7] * c1) * inv_det;
    e[5] = (a[0] * c5 - a[2] * c2 + a[3] * c1) * inv_det;
    e[6] = (-a[12] * s5 + a[14] * s2 - a[15] * s1) * inv_det;
    e[7] = (a[8] * s5 - a[10] * s2 + a[11] * s1) * inv_det;
    e[8] = (a[4] * c4 - a[5] * c2 + a[7] * c0) * inv_det;
    e[9] = (-a[0] * c4 + a[1] * c2 - a[3] * c0) * inv_det;
    e[10] = (a[12] * s4 - a[13] * s2 + a[15] * s0) * inv_det;
    e[11] = (-a[8] * s4 + a[9] * s2 - a[11] * s0) * inv_det;
    for (int row = 0; row < 3; ++row)
        for (int col = 0; col < 4; ++col)
            proj[(size_t)i * 12 + row * 4 + col] =
                (float)((kk[row * 3] * e[col] + kk[row * 3 + 1] * e[4 + col]) + kk[row * 3 + 2] * e[8 + col]);
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
              int slot_budget = kMaxSlotLdsBytes) {
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
        // feature rows are addressed in 32-bit units (16 bytes, or one element off the vector paths)
        const long long units = plan->vec > 1 ? (long long)k.C * es / 16 : k.C;
        if ((long long)k.B * k.N * k.H * k.W * units >= (1ll << 31)) return FBEV_ERR_TOO_LARGE;
        k.row_units = (int)units;
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
    k.slots = slots;
    k.groups_per_slot = (kWave / lps) / slots;     // >= 1: slots <= kWave / lps
    k.list_cap = k.NZ;
    // enough wavefronts to fill 256 CUs several times over before a wavefront takes more rounds,
    // and never many rounds: cells differ widely in their number of samples, and short wavefronts
    // even that out (training-size cell pass: 439 / 406 / 399 / 404 / 439 us with at most
    // 8 / 4 / 3 / 2 / 1 rounds; the forward does not care)
    const long long groups = ((long long)k.padded_cells + slots - 1) / slots * k.B;
    int rounds = (int)(groups / (256ll * 4 * 8 * 2));
    k.rounds = rounds < 1 ? 1 : (rounds > max_rounds ? max_rounds : rounds);
    k.waves = waves;
    const int cells_per_block = waves * k.slots * k.rounds;
    k.blocks_per_batch = (k.padded_cells + cells_per_block - 1) / cells_per_block;
    k.n_blocks = k.blocks_per_batch * k.B;
    const size_t p_f4 = (size_t)(k.N * 12 + 3) / 4;
    const size_t cols = (size_t)k.slots * k.N, dec_f4 = (cols + 3) / 4;
    const size_t cand_f4 = ((size_t)k.slots * k.NZ + 3) / 4;
    auto block_lds = [&](int entry_f4) {
        return (p_f4 + dec_f4 +
                (size_t)waves * (20 + cols + dec_f4 + cand_f4 + (size_t)k.slots * k.list_cap * entry_f4)) * 16;
    };
    {
        // exact division of a sample index below 4096 by gz: multiply and shift
        if ((long long)k.slots * k.NZ >= 4096) return FBEV_ERR_TOO_LARGE;
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
                   float *cnt, hipStream_t st) {
    dim3 grid(pl.k.n_blocks), block(kWave * pl.k.waves);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    prof::Scope timer(out != nullptr ? prof::kForward : prof::kCellCount, st);
    const bool stream = VEC > 1 && (long long)pl.k.B * pl.k.gy * pl.k.gx * pl.k.C * 4 > kStreamOutputFrom;
    auto launch = [&](auto kernel) {
        if (!lds_opt_in(kernel, pl.lds_fwd)) return false;
        hipLaunchKernelGGL(kernel, grid, block, pl.lds_fwd, st, pl.k, d, f, proj, out, cnt);
        return true;
    };
    bool ok;
    if (stream) {
        constexpr bool S = VEC > 1;      // no streaming instantiations off the vector paths
        ok = pl.cpl == 1 ? launch(fbev_forward_kernel<T, VEC, 1, S>)
                         : (pl.cpl == 2 ? launch(fbev_forward_kernel<T, VEC, 2, S>) : launch(fbev_forward_kernel<T, VEC, 4, S>));
    } else {
        ok = pl.cpl == 1 ? launch(fbev_forward_kernel<T, VEC, 1, false>)
                         : (pl.cpl == 2 ? launch(fbev_forward_kernel<T, VEC, 2, false>)
                                        : launch(fbev_forward_kernel<T, VEC, 4, false>));
    }
    if (!ok) return FBEV_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

int dispatch_forward(const fbev_problem *p, const Plan &pl, const void *depth, const void *feats, const float *proj,
                     float *out, float *cnt, hipStream_t st) {
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_forward<float, 4>(pl, depth, feats, proj, out, cnt, st)
                               : launch_forward<float, 1>(pl, depth, feats, proj, out, cnt, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_forward<__half, 8>(pl, depth, feats, proj, out, cnt, st)
                               : launch_forward<__half, 1>(pl, depth, feats, proj, out, cnt, st);
        default:
            return pl.vec == 8 ? launch_forward<bf16_raw, 8>(pl, depth, feats, proj, out, cnt, st)
                               : launch_forward<bf16_raw, 1>(pl, depth, feats, proj, out, cnt, st);
    }
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
                 float *dd, float *df, const int *prefix, int *cursor, Pair *pairs, int cap, hipStream_t st) {
    dim3 grid(pl.k.n_blocks), block(kWave * pl.k.waves);
    const T *d = static_cast<const T *>(depth);
    const T *f = static_cast<const T *>(feats);
    const size_t lds = FILL ? pl.lds_fill : pl.lds_bwd;
    prof::Scope timer(FILL ? prof::kBackwardCells : prof::kBackwardScatter, st);
    switch (pl.cpl) {
        case 1: if (!lds_opt_in(fbev_backward_cells_kernel<T, VEC, 1, FILL>, lds)) return FBEV_ERR_LAUNCH;
                hipLaunchKernelGGL((fbev_backward_cells_kernel<T, VEC, 1, FILL>), grid, block, lds, st, pl.k, go, d, f, proj, dd, df, prefix, cursor, pairs, cap); break;
        case 2: if (!lds_opt_in(fbev_backward_cells_kernel<T, VEC, 2, FILL>, lds)) return FBEV_ERR_LAUNCH;
                hipLaunchKernelGGL((fbev_backward_cells_kernel<T, VEC, 2, FILL>), grid, block, lds, st, pl.k, go, d, f, proj, dd, df, prefix, cursor, pairs, cap); break;
        default: if (!lds_opt_in(fbev_backward_cells_kernel<T, VEC, 4, FILL>, lds)) return FBEV_ERR_LAUNCH;
                hipLaunchKernelGGL((fbev_backward_cells_kernel<T, VEC, 4, FILL>), grid, block, lds, st, pl.k, go, d, f, proj, dd, df, prefix, cursor, pairs, cap); break;
    }
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

template <int FILL>
int dispatch_cells(const fbev_problem *p, const Plan &pl, const float *go, const void *depth, const void *feats,
                   const float *proj, float *dd, float *df, const int *prefix, int *cursor, Pair *pairs, int cap,
                   hipStream_t st) {
    switch (p->in_dtype) {
        case FBEV_F32:
            return pl.vec == 4 ? launch_cells<float, 4, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st)
                               : launch_cells<float, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st);
        case FBEV_F16:
            return pl.vec == 8 ? launch_cells<__half, 8, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st)
                               : launch_cells<__half, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st);
        default:
            return pl.vec == 8 ? launch_cells<bf16_raw, 8, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st)
                               : launch_cells<bf16_raw, 1, FILL>(pl, go, depth, feats, proj, dd, df, prefix, cursor, pairs, cap, st);
    }
}

template <typename T>
int launch_count(const Plan &pl, const void *depth, const float *proj, int *counts, hipStream_t st) {
    if (!lds_opt_in(fbev_count_kernel<T>, pl.lds_count)) return FBEV_ERR_LAUNCH;
    prof::Scope timer(prof::kCount, st);
    hipLaunchKernelGGL((fbev_count_kernel<T>), dim3(pl.k.n_blocks), dim3(kWave * pl.k.waves), pl.lds_count, st, pl.k,
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
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)out % 16 == 0, &pl, kWavesPerBlock, 4, kForwardSlotLdsBytes);
    if (rc != FBEV_OK) return rc;
    return dispatch_forward(p, pl, depth, feats, proj, out, count_out, static_cast<hipStream_t>(stream));
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
    int rc = validate(p, true);
    if (rc != FBEV_OK) return rc;
    rc = check_backward_args(p, grad_out, depth, feats, proj, d_depth, d_feats);
    if (rc != FBEV_OK) return rc;
    if (!d_depth && !d_feats) return FBEV_OK;
    if (!workspace) return FBEV_ERR_NULL;
    if ((uintptr_t)workspace % 16) return FBEV_ERR_ALIGNMENT;
    const size_t index_bytes = ws_index_bytes(p);
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
    rc = make_plan(p, (uintptr_t)feats % 16 == 0 && (uintptr_t)grad_out % 16 == 0, &pl, kCellPassWaves);
    if (rc != FBEV_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int *cursor = static_cast<int *>(workspace);
    Pair *pairs = reinterpret_cast<Pair *>(static_cast<char *>(workspace) + index_bytes);
    const long long texels = texel_count(p);
    const long long counters = counter_count(p), chunks = chunk_count(p);
    int *chunk_prefix = cursor + counters;

    // A workspace with room for every sample gets fixed segments: each (texel, replica)
    // owns cap / (texels * kFixedReplicas) pair slots, and the counting pass and the prefix sums
    // are not needed.  (A texel that outgrows its segments falls back to atomics, like a full
    // pair array does.)  Smaller workspaces are packed exactly: count, scan, fill.
    const bool fixed = (uint64_t)cap >= fbev_backward_max_pairs(p) && cap / (texels * kFixedReplicas) >= kFixedMinSegment;
    const int seg_cap = fixed ? (int)(cap / (texels * kFixedReplicas)) : 0;
    rc = launch_zero(cursor, fixed ? texels * kFixedReplicas : counters, accumulate ? nullptr : d_depth,
                     texels * p->depth_bins, accumulate ? nullptr : d_feats, texels * p->channels, st);
    if (rc != FBEV_OK) return rc;
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
    rc = claim_runs ? dispatch_cells<2>(p, pl, grad_out, depth, feats, proj, d_depth, d_feats, prefix_arg, cursor, pairs,
                                        cap_arg, st)
                    : dispatch_cells<1>(p, pl, grad_out, depth, feats, proj, d_depth, d_feats, prefix_arg, cursor, pairs,
                                        cap_arg, st);
    if (rc != FBEV_OK) return rc;

    // texel pass: rows of grad_out are fp32, so 128-bit gathers need C % 4 == 0 and aligned rows
    const bool vec4 = p->channels % 4 == 0 && (uintptr_t)grad_out % 16 == 0;
    const int vec = vec4 ? 4 : 1;
    const int cq = (p->channels + vec - 1) / vec;
    const int lpr = cq < kWave ? cq : kWave;
    // One, two or four wavefronts per texel.  A texel's block is a chain of dependent loads (list bounds,
    // pairs, grad_out rows); small blocks fit the machine in fewer generations, large ones shorten the
    // chain of a long list.  What is known here is only how many samples a texel could get if every one were
    // kept.  Measured (us for 1 / 2 / 4 wavefronts; Laplace, then the categorical model, which keeps twice
    // as many): 23 possible samples per texel 8 / 9 / 11; 186 per texel and 4224 texels 20 / 19 / 23 and
    // 39 / 30 / 31; 186 per texel and 67 584 texels 125 / 154 / 239 and 256 / 274 / 365; 454 per texel
    // 38 / 29 / 29 and 80 / 60 / 52; 909 per texel 493 / 426 / 431; 2727 per texel 352 / 209 / 124.
    const uint64_t per_texel = fbev_backward_max_pairs(p) / (uint64_t)texels;
    const int texel_waves = (per_texel < kTexelOneWaveBelow || (texels >= kTexelManyTexels && per_texel < 3 * kTexelOneWaveBelow)) ? 1
                            : (per_texel < kTexelTwoWavesBelow ? 2 : kWavesPerBlock);
    const int nw = (kWave / lpr) * texel_waves;
    // the depth gradient rides on the pairs exactly when the cell pass folds it in (one channel pass
    // and room for the depth bin in a pair's first word)
    const int from_pairs =
        (d_depth != nullptr && pl.k.C <= pl.k.lanes_per_slot * pl.vec * pl.cpl && pl.k.bin_bits >= 0) ? 1 : 0;
    const size_t lds = ((size_t)texel_waves * kWave * 2 + (size_t)nw * (lpr * vec + 2) +
                        (p->depth_distribution == FBEV_CATEGORICAL ? p->depth_bins : 0)) * sizeof(float);
    long long want_split = kTexelSplitBelow / texels;
    const unsigned n_split = (unsigned)(want_split < 1 ? 1 : (want_split > kTexelMaxSplit ? kTexelMaxSplit : want_split));
    prof::Scope timer(prof::kBackwardTexel, st);
    const dim3 tgrid((unsigned)texels, n_split), tblock(kWave * texel_waves);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, tgrid, tblock, lds, st, pl.k, grad_out, prefix_arg, cursor, pairs, cap_arg, d_depth, d_feats,
                           lpr, from_pairs, accumulate ? 0 : 1);
    };
    if (vec4) {
        if (texel_waves == 1) launch(fbev_backward_texel_kernel<4, 1>);
        else if (texel_waves == 2) launch(fbev_backward_texel_kernel<4, 2>);
        else launch(fbev_backward_texel_kernel<4, kWavesPerBlock>);
    } else {
        if (texel_waves == 1) launch(fbev_backward_texel_kernel<1, 1>);
        else if (texel_waves == 2) launch(fbev_backward_texel_kernel<1, 2>);
        else launch(fbev_backward_texel_kernel<1, kWavesPerBlock>);
    }
    return hipGetLastError() == hipSuccess ? FBEV_OK : FBEV_ERR_LAUNCH;
}

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
