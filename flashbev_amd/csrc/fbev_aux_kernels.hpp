// Interval pooling over host-prepared sample lists (the reference's baseline method), the
// projection-matrix builder and the per-sample geometry dump.
// Part of the single translation unit fbev_kernels.hip; not meant to be compiled on its own.
#pragma once

namespace {

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

}  // namespace
