// Backward with one block per feature-map column (no workspace, no atomics on the feature gradient).
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

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

}  // namespace
