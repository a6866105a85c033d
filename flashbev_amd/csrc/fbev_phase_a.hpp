// The sample phase of the cell-centric kernels (forward, backward cell pass, count): a
// wavefront's LDS view and the three-stage evaluation of the samples of its cells.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

// LDS of one block of the cell-centric kernels (float4 units):
//   [matrices: N*12 floats][column table: batch*N ints][height table: gz floats]
//   per wavefront: [batch ints: entries per cell][batch ints: where a cell's entries start][8 ints: candidates
//   before each group][batch float4 of cell centres][batch*N column records][batch*N ints: columns in view]
//   [batch*NZ ints of candidates][pool of pool_cap entries]
// where batch = KParams::slots_a cells go through the sample phase together and their kept samples
// share one pool of entries, each cell's entries in one contiguous stretch.
// Counters that several lanes of a wavefront update in turn live in LDS and are read as
// volatile.  The pointer carries the LDS address space: a volatile access through a generic
// pointer becomes a system-coherent flat load that first waits for every outstanding global
// store and atomic of the wavefront.
using lds_counter = volatile __attribute__((address_space(3))) int;

struct WaveLds {
    const float *Pm;
    const int *dec;       // column index within the wavefront's batch -> cell << 28 | camera << 16
    const float *zt;      // height bin -> z of the bin's centre
    lds_counter *cnt;     // entries per cell of the batch
    lds_counter *start;   // first entry of each cell in the pool
    lds_counter *gcand;   // candidates that come before each group of the batch (groups + 1 values)
    float4 *cell;         // per cell: x, y, valid flag, ix | iy << 16
    float4 *col;          // per column: the (x, y) part of U, V, D, and its dec word
    int *alive;           // columns with a height bin that may be in view
    unsigned *cand;       // samples that survive the cheap test: column << 16 | height bin
    float4 *lst;          // the pool
};

__device__ __forceinline__ int lds_p_f4(const KParams &k) { return (k.N * 12 + 3) / 4; }
__device__ __forceinline__ int lds_dec_f4(const KParams &k) { return (k.slots_a * k.N + 3) / 4; }
__device__ __forceinline__ int lds_cand_f4(const KParams &k) { return (k.slots_a * k.NZ + 3) / 4; }
__device__ __forceinline__ int lds_z_f4(const KParams &k) { return (k.gz + 3) / 4; }
// the three small tables and the cell records (LDS is granted in large granules: a few hundred bytes
// per wavefront decide whether a tenth block fits a CU at the training size)
__device__ __forceinline__ int lds_tables_f4(const KParams &k) { return (2 * k.slots_a + 8 + 3) / 4; }
__device__ __forceinline__ int lds_head_f4(const KParams &k) { return lds_tables_f4(k) + k.slots_a; }

// The wavefront's view of the block's LDS (pointers only).
__device__ __forceinline__ WaveLds wave_lds_view(const KParams &k, float4 *smem, int entry_f4) {
    WaveLds L;
    const int dec_f4 = lds_dec_f4(k), cand_f4 = lds_cand_f4(k), cols = k.slots_a * k.N;
    const int head_f4 = lds_head_f4(k);
    const int per_wave_f4 = head_f4 + cols + dec_f4 + cand_f4 + k.pool_cap * entry_f4;
    float4 *wbase = smem + lds_p_f4(k) + dec_f4 + lds_z_f4(k) + (threadIdx.x >> 6) * per_wave_f4;
    L.Pm = reinterpret_cast<float *>(smem);
    L.dec = reinterpret_cast<int *>(smem + lds_p_f4(k));
    L.zt = reinterpret_cast<float *>(smem + lds_p_f4(k) + dec_f4);
    L.cnt = (lds_counter *)reinterpret_cast<int *>(wbase);
    L.start = L.cnt + k.slots_a;
    L.gcand = L.cnt + 2 * k.slots_a;
    L.cell = wbase + lds_tables_f4(k);
    L.col = wbase + head_f4;
    L.alive = reinterpret_cast<int *>(wbase + head_f4 + cols);
    L.cand = reinterpret_cast<unsigned *>(wbase + head_f4 + cols + dec_f4);
    L.lst = wbase + head_f4 + cols + dec_f4 + cand_f4;
    return L;
}

// Stage the block's matrices, the column table and the height table; returns the wavefront's view.  Ends with a
// barrier.
__device__ __forceinline__ WaveLds block_lds_setup(const KParams &k, float4 *smem, const float *__restrict__ proj,
                                                   int b, int entry_f4) {
    const WaveLds L = wave_lds_view(k, smem, entry_f4);
    float *Pm = reinterpret_cast<float *>(smem);
    int *dec = reinterpret_cast<int *>(smem + lds_p_f4(k));
    float *zt = reinterpret_cast<float *>(smem + lds_p_f4(k) + lds_dec_f4(k));
    const int cols = k.slots_a * k.N;
    for (int i = threadIdx.x; i < k.N * 12; i += blockDim.x)
        Pm[i] = proj[(size_t)(b * k.N + i / 12) * k.proj_stride + (i % 12)];
    for (int i = threadIdx.x; i < cols; i += blockDim.x) {
        const int slot = k.N == 1 ? i : (int)__umulhi((unsigned)i, k.cams_magic), cam = i - slot * k.N;
        dec[i] = (slot << 28) | (cam << 16);
    }
    for (int i = threadIdx.x; i < k.gz; i += blockDim.x) zt[i] = voxel_coord(k.zmin, i, k.vz);
    __syncthreads();
    return L;
}

// Entry of a compacted list: ENTRY_F4 float4 words.
//   forward   word 0: corner weights already multiplied by the depth weight
//             word 1: where the four texels' feature rows start, in address units (texel index
//                     ((b*N+n)*H + v)*W + u times KParams::row_units) as unsigned bits (t00, t01, t10, t11):
//                     the gather loop then forms an address with one shift-add, not a 64-bit multiply
//   cache     one word: du, dv, t00 << 2 | (u1 != u0) | (v1 != v0) << 1, depth along the optical axis
//   backward  word 0: du, dv, t00, (u1 != u0) | (v1 != v0) << 1 -- the four weights and texels
//                     follow from these exactly as phase A computed them.  Inverse map: t00 << 2 with
//                     the two flags below it, and in the fourth place the position of the sample's
//                     pair in the pair array (sorted by first corner texel), or -1 if the array is full
//             word 1: wgt, a, b, (k0 | k1 << 16)
//   store     what a forward that is going to be differentiated leaves behind for the backward's cell pass, two
//             words per kept sample in the slot of its cell (cells in the order of the tiled walk, N * gz entries
//             per cell): the backward entry above with -1 in the fourth place (no pair position yet)
enum { kModeForward = 0, kModeScatter = 1, kModeFill = 2, kModeCount = 3, kModeFillRuns = 4, kModeCache = 5,
       kModeForwardStore = 6, kModeCountView = 7 };

// Segments sized by the geometry (a persistent workspace prepared for one set of matrices): segment i =
// (texel, replica) starts at tab[i].x in the pair array and has room for tab[i].y pairs, the number of samples in
// view that can claim there.  Null: segments of one common capacity.
// The claim counter of such a segment is a 64-bit word that carries the segment along, so that the one returning
// atomic of a claim brings back all a claim needs:
//   low word   kSegBias - capacity + claims so far: the sign bit comes on with the first claim that does not fit
//   high word  start + capacity - kSegBias:         low + high (mod 2^32) = start + claims so far, the position
// (fewer than 2^31 samples exist, so the low word never carries into the high one).
struct SegTable {
    const int2 *tab;
};
constexpr unsigned kSegBias = 0x80000000u;
__host__ __device__ __forceinline__ unsigned long long packed_counter(int start, int cap) {
    return ((unsigned long long)((unsigned)start + (unsigned)cap - kSegBias) << 32) | (kSegBias - (unsigned)cap);
}
// The addend of a single claim on a packed counter, made where it is used: as a constant the compiler would hold
// the pair of registers from the kernel's start to its end, and the cell pass's fp16 instantiation has none to spare.
__device__ __forceinline__ unsigned long long fresh_one() {
    unsigned long long one = 1ull;
    asm volatile("" : "+v"(one));
    return one;
}
// Position in the pair array of the claim that read (lo, hi) from a packed counter, or -1 if the segment (or the
// array) is full.  (Counters that were not prepared for this problem may hold anything: whatever comes out is
// either -1 or inside the array.)
__device__ __forceinline__ int packed_position(unsigned lo, unsigned hi, int pair_cap) {
    const unsigned at = hi + lo;
    return ((int)lo >= 0 && at < (unsigned)pair_cap) ? (int)at : -1;
}

// Where claim number `pos` of segment i0 lies when every segment holds pair_cap pairs, or -1 if the segment is full
// (compared as unsigned: counters that were not prepared for this problem may hold anything, and a negative
// position must not become an address).
__device__ __forceinline__ int fixed_position(int pair_cap, int i0, int pos) {
    return (unsigned)pos < (unsigned)pair_cap ? i0 * pair_cap + pos : -1;
}

// Position of a kept sample's pair in the list of its first corner texel: one returning integer atomic
// on the counter the sample's cell selects among the texel's replicas.  -1: the list is full (compared
// as unsigned: counters that were not prepared for this problem may hold anything, and a negative
// position must not become an address).
__device__ __forceinline__ int claim_pair(const int *__restrict__ chunk_prefix, int *__restrict__ cursor, int pair_cap,
                                          int texel, int cellxy, const SegTable &segs) {
    const int rep = replica_of(cellxy & 0xffff, cellxy >> 16);
    if (chunk_prefix != nullptr) {
        // counted segments: cursor holds each segment's start within its scan chunk
        const int i0 = texel * kReplicas + rep;
        const int pos = atomicAdd(cursor + i0, 1) + chunk_prefix[i0 >> kScanChunkBits];
        return (unsigned)pos < (unsigned)pair_cap ? pos : -1;
    }
    const int i0 = texel * kFixedReplicas + (rep & (kFixedReplicas - 1));
    if (segs.tab != nullptr) {
        // segments sized by the geometry: packed counters
        const unsigned long long old = atomicAdd(reinterpret_cast<unsigned long long *>(cursor) + i0, fresh_one());
        return packed_position((unsigned)old, (unsigned)(old >> 32), pair_cap);
    }
    // fixed segments per (texel, replica) of pair_cap pairs each: cursor counts from zero
    return fixed_position(pair_cap, i0, atomicAdd(cursor + i0, 1));
}

// Relative slack of the cheap field-of-view test.  A sample is dropped early only if its
// pixel coordinate misses the image by more than this fraction, far beyond any rounding of
// the exact test it would otherwise take (and fail).
constexpr float kEarlySlack = 1.0e-3f;

// The sample phase of one batch of a wavefront: the samples of its `slots_a` cells, in three stages.
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
//            in (cell, camera, height) order, into the pool of entries.
// A batch is `batch_groups` groups of `slots` cells: phase B works on one group at a time (its lane
// groups cover `slots` cells), while stages 0 to 2 run over the whole batch, so that their passes
// of 64 lanes are filled by more than one group's samples (a group of two cells has about thirty
// candidates: stage 2, a third of the forward's instructions, ran at half its lanes).  The pool holds
// slots * NZ entries, what one group can keep at most; when a batch has more candidates than that
// (rare: about one sample in six is in view), its groups go through stage 2 one at a time.

// Stages 0 and 1 of the batch that starts at cell q0.  Returns the number of candidates; the number
// of candidates before each group is left in L.gcand.
// BATCHED = false is the batch of one group, with the bookkeeping of several compiled away.
template <bool BATCHED>
__device__ __forceinline__ int phase_a_candidates(const KParams &k, const WaveLds &L, int q0, int lane) {
    const int n_groups = BATCHED ? k.batch_groups : 1;
    const int n_cols = k.slots_a * k.N;
    if (lane < k.slots_a) {
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
    const float z_first = L.zt[0], z_last = L.zt[k.gz - 1];
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
    int before1 = 0, before2 = 0, before3 = 0;      // candidates of groups below 1, 2, 3 (at most four groups)
    const int total = n_alive * k.gz;
    for (int base = 0; base < total; base += kWave) {
        const int idx = base + lane;
        bool pass = false;
        unsigned key = 0;
        int cell = 0;
        if (idx < total) {
            const int a = (int)(__umul24((unsigned)idx, (unsigned)k.gz_magic) >> k.gz_shift);
            const int iz = idx - a * k.gz;
            const int cc = L.alive[a];
            const float4 col = L.col[cc];
            cell = (__float_as_int(col.w) >> 28) & 15;
            const float *P = L.Pm + ((__float_as_int(col.w) >> 16) & 0xfff) * 12;
            const float z = L.zt[iz];
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
        if (BATCHED) {
            before1 += __popcll(__ballot(pass && cell < k.slots));
            before2 += __popcll(__ballot(pass && cell < 2 * k.slots));
            before3 += __popcll(__ballot(pass && cell < 3 * k.slots));
        }
    }
    if (BATCHED && lane == 0) {
        L.gcand[0] = 0;
        L.gcand[1] = before1;
        L.gcand[2] = before2;
        L.gcand[3] = before3;
        L.gcand[n_groups] = n_cand;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    return n_cand;
}

// Stage 2 over the candidates [c_lo, c_hi) of the batch (whole groups).  Entries are appended to the
// pool from its start; on return L.cnt holds the entries of every cell (0 for the cells of other
// groups) and L.start where they begin.
// kModeCount writes no entries; it only counts the kept samples per (first-corner texel, replica).
template <int ENTRY_F4, typename T, int MODE>
__device__ __forceinline__ void phase_a_samples(const KParams &k, const WaveLds &L, const T *__restrict__ depth, int b,
                                                int lane, int c_lo, int c_hi,
                                                const int *__restrict__ chunk_prefix = nullptr,
                                                int *__restrict__ cursor = nullptr, int pair_cap = 0,
                                                float4 *__restrict__ store = nullptr,
                                                const SegTable segs = SegTable{nullptr}) {
    constexpr bool FILLING = MODE == kModeFill || MODE == kModeFillRuns;   // the latter claims per run
    constexpr bool COUNTING = MODE == kModeCount || MODE == kModeCountView;
    constexpr bool BACKWARD = MODE == kModeScatter || FILLING;
    constexpr bool STORING = MODE == kModeForwardStore;      // `store`: the slot of the batch's first cell
    if (lane < k.slots_a) L.cnt[lane] = 0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int n_pool = 0;       // entries in the pool so far
    for (int base = c_lo; base < c_hi; base += kWave) {
        const int j = base + lane;
        const bool active = j < c_hi;
        const unsigned key = active ? L.cand[j] : 0u;
        const float4 col = active ? L.col[key >> 16] : make_float4(0.f, 0.f, 0.f, 0.f);
        const int d = __float_as_int(col.w);
        const int slot = active ? (d >> 28) & 15 : 16 + (lane & 1);   // idle lanes: no real cell
        const int cam = (d >> 16) & 0xfff;
        float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w2 = w0, rec = w0;
        int4 tx = make_int4(0, 0, 0, 0);
        int cellxy = 0;
        bool keep = false;
        if (active) {
            const float4 c = L.cell[slot];
            cellxy = __float_as_int(c.w);
            // no branch on the outcome of the exact test: nearly every candidate passes it, and the joins
            // of a branch here cost more moves than the arithmetic it skips (indices are clamped, so the
            // depth loads of a sample out of view read valid memory and their result is dropped)
            const Geom g = project_column_flat(k, L.Pm + cam * 12, col.x, col.y, col.z, L.zt[key & 0xffffu]);
            const float w00 = (1.0f - g.du) * (1.0f - g.dv);
            const float w01 = (1.0f - g.du) * g.dv;
            const float w10 = g.du * (1.0f - g.dv);
            const float w11 = g.du * g.dv;
            const int rowbase = (b * k.N + cam) * k.H;
            const int t00 = (rowbase + g.v0) * k.W + g.u0;
            const int t01 = (rowbase + g.v1) * k.W + g.u0;
            const int t10 = (rowbase + g.v0) * k.W + g.u1;
            const int t11 = (rowbase + g.v1) * k.W + g.u1;
            DepthEval e;
            if (MODE == kModeCache || MODE == kModeCountView) {
                e.keep = true;       // every sample in view is listed / counted; the depth model comes later
                e.wgt = e.a = e.b = 0.0f;
                e.k0 = e.k1 = 0;
            } else {
                e = eval_depth<T>(k, depth, t00, t01, t10, t11, w00, w01, w10, w11, g.depth);
            }
            keep = g.valid && e.keep;
            tx = make_int4(t00, t01, t10, t11);
            if (MODE == kModeCache) {
                const int fl = (g.u1 != g.u0 ? 1 : 0) | (g.v1 != g.v0 ? 2 : 0);
                w0 = make_float4(g.du, g.dv, __int_as_float((t00 << 2) | fl), g.depth);
            } else if (BACKWARD) {
                const int fl = (g.u1 != g.u0 ? 1 : 0) | (g.v1 != g.v0 ? 2 : 0);
                w0 = FILLING ? make_float4(g.du, g.dv, __int_as_float((t00 << 2) | fl), __int_as_float(-1))
                                       : make_float4(g.du, g.dv, __int_as_float(t00), __int_as_float(fl));
                w2 = make_float4(e.wgt, e.a, e.b, __int_as_float(e.k0 | (e.k1 << 16)));
            } else {
                w0 = make_float4(w00 * e.wgt, w01 * e.wgt, w10 * e.wgt, w11 * e.wgt);
                if (STORING) {
                    const int fl = (g.u1 != g.u0 ? 1 : 0) | (g.v1 != g.v0 ? 2 : 0);
                    rec = make_float4(g.du, g.dv, __int_as_float((t00 << 2) | fl), __int_as_float(-1));
                    w2 = make_float4(e.wgt, e.a, e.b, __int_as_float(e.k0 | (e.k1 << 16)));
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
        if (COUNTING || MODE == kModeFillRuns) {
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
        if (MODE == kModeCountView) {
            // the samples in view per fixed segment: what a segment sized by the geometry has to hold
            if (keep && run_lead == lane)
                atomicAdd(cursor + tx.x * kFixedReplicas + (replica_of(cellxy & 0xffff, cellxy >> 16) & (kFixedReplicas - 1)), run_len);
            continue;
        }
        // candidates are in sample order, so the lanes of one slot are contiguous: [lo, hi)
        const unsigned long long bm = __ballot(lane == 0 || slot != prev_slot);
        const unsigned long long m = __ballot(keep);
        const int lo = 63 - __clzll(bm & lanemask_le(lane));
        const unsigned long long above = lane == 63 ? 0ull : (bm & ~lanemask_le(lane));
        const int hi = above ? __ffsll((long long)above) - 1 : kWave;
        const unsigned long long seg = (~0ull << lo) & (hi >= 64 ? ~0ull : ((1ull << hi) - 1ull));
        const int old = active ? L.cnt[slot] : 0;
        // kept samples are appended to the pool in order: a cell's entries end up next to each other
        // (`at` of a lane that keeps nothing is where the next kept sample after it goes)
        const int at = n_pool + __popcll(m & lanemask_lt(lane));
        n_pool += __popcll(m);
        if (keep && ENTRY_F4 > 0) {
            float4 *e = L.lst + (size_t)at * ENTRY_F4;
            e[0] = w0;
            if (ENTRY_F4 > 1)
                e[1] = BACKWARD ? w2
                                : make_float4(__int_as_float(tx.x * k.row_units), __int_as_float(tx.y * k.row_units),
                                              __int_as_float(tx.z * k.row_units), __int_as_float(tx.w * k.row_units));
        }
        if (STORING && keep) {
            // the sample's record for the backward, at its place among the kept samples of its cell
            float4 *dst = store + ((size_t)slot * k.NZ + old + __popcll(m & seg & lanemask_lt(lane))) * 2;
            dst[0] = rec;
            dst[1] = w2;
        }
        if (MODE == kModeFill && keep)
            reinterpret_cast<int *>(L.lst + (size_t)at * ENTRY_F4)[3] = claim_pair(chunk_prefix, cursor, pair_cap, tx.x, cellxy, segs);
        if (MODE == kModeFillRuns) {
            // the same, but the run's first lane claims for the whole run (same cell and texel: same
            // counter) and hands the positions out; every lane takes part in the exchange
            const int rep = replica_of(cellxy & 0xffff, cellxy >> 16);
            const bool counted = chunk_prefix != nullptr;
            const int i0 = counted ? tx.x * kReplicas + rep : tx.x * kFixedReplicas + (rep & (kFixedReplicas - 1));
            if (segs.tab != nullptr) {
                // packed counters: both words of the lead's answer go round
                unsigned long long word = 0;
                if (keep && run_lead == lane)
                    word = atomicAdd(reinterpret_cast<unsigned long long *>(cursor) + i0, (unsigned long long)run_len);
                const unsigned lo_w = (unsigned)__shfl((int)(unsigned)word, run_lead, kWave) + (unsigned)(lane - run_lead);
                const unsigned hi_w = (unsigned)__shfl((int)(unsigned)(word >> 32), run_lead, kWave);
                if (keep) reinterpret_cast<int *>(L.lst + (size_t)at * ENTRY_F4)[3] = packed_position(lo_w, hi_w, pair_cap);
            } else {
                int pos = 0;
                if (keep && run_lead == lane) pos = atomicAdd(cursor + i0, run_len);
                pos = __shfl(pos, run_lead, kWave) + (lane - run_lead);
                if (keep) {
                    if (counted) {
                        pos += chunk_prefix[i0 >> kScanChunkBits];
                        pos = (unsigned)pos < (unsigned)pair_cap ? pos : -1;
                    } else {
                        pos = fixed_position(pair_cap, i0, pos);
                    }
                    reinterpret_cast<int *>(L.lst + (size_t)at * ENTRY_F4)[3] = pos;
                }
            }
        }
        if (active && lane == lo) {
            // the first lane of a cell's stretch of lanes keeps the cell's books: its entries so far, and,
            // when these are its first, where they start in the pool (a cell without entries has no start)
            L.cnt[slot] = old + __popcll(m & seg);
            if (old == 0) L.start[slot] = at;
        }
    }
}

// The sample phase of the backward's cell pass when the forward left its kept samples behind (kModeForwardStore):
// lanes = the stored samples of the batch's cells, densely packed; each is copied into the pool and claims
// its pair position.  No matrices, no projection, no depth model.  `count` holds the forward's per-cell
// counts, [B, gy, gx]; `store` points at the slot of the batch's first cell.  Values that cannot have come
// from a forward of this problem (a count beyond N * gz, a texel beyond the feature maps) are clamped and
// zeroed, so that a wrong buffer gives wrong numbers but no access out of bounds.
__device__ __forceinline__ void phase_a_stored(const KParams &k, const WaveLds &L, const float *__restrict__ count,
                                               const float4 *__restrict__ store, int b, int q0, int lane,
                                               const int *__restrict__ chunk_prefix, int *__restrict__ cursor,
                                               int pair_cap, const SegTable &segs) {
    int mine_n = 0, mine_xy = 0;
    if (lane < k.slots_a) {
        int ix = 0, iy = 0;
        if (cell_of(k, q0 + lane, ix, iy)) {
            mine_n = min(max((int)count[(size_t)(b * k.gy + iy) * k.gx + ix], 0), k.NZ);
            mine_xy = ix | (iy << 16);
        }
    }
    int incl = mine_n;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        const int other = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += other;
    }
    const int total = __shfl(incl, 15, kWave);        // slots_a <= 16; lanes past the cells carry 0
    const int my_start = incl - mine_n;
    if (lane < k.slots_a) {
        L.cnt[lane] = mine_n;
        L.start[lane] = my_start;
    }
    const unsigned n_texels = (unsigned)(k.B * k.N * k.H * k.W);
    for (int jb = 0; jb < total; jb += kWave) {
        const int j = jb + lane;
        // the cell whose stretch holds j: the last one that starts at or before j (empty cells start
        // where the next one does, so later ones win)
        int slot = 0;
        for (int s = 1; s < k.slots_a; ++s) slot = (__shfl(my_start, s, kWave) <= j) ? s : slot;
        const int first = __shfl(my_start, slot, kWave);
        const int cellxy = __shfl(mine_xy, slot, kWave);
        if (j < total) {
            // (only cells of the walk have a count above zero, so the slot exists)
            const float4 *src = store + ((size_t)slot * k.NZ + (j - first)) * 2;
            float4 geo = src[0], dw = src[1];
            if ((unsigned)(__float_as_int(geo.z) >> 2) >= n_texels) {
                geo = make_float4(0.f, 0.f, __int_as_float(0), 0.f);
                dw = make_float4(0.f, 0.f, 0.f, __int_as_float(1 << 16));
            }
            geo.w = __int_as_float(claim_pair(chunk_prefix, cursor, pair_cap, __float_as_int(geo.z) >> 2, cellxy, segs));
            L.lst[2 * j] = geo;
            L.lst[2 * j + 1] = dw;
        }
    }
}

}  // namespace
