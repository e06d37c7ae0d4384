// Windowed bilinear lookup of the correlation pyramid without the 4D volume (gfx950).
//
// What the caller's corr_fn(coords) returns on the stored-volume path (core/corr.py:193-248), for the block that
// never stores the volume (core/corr.py:479-510, where the reference raises NotImplementedError because its native
// part is missing).  For image-1 pixel p = (i,j) with target (x,y) = coords[b,:,i,j] / 2^l in level l:
//   out[b, l*n*n + a*n + c, i, j] = scale * bilinear(S_l[p,:,:])(x + a - r, y + c - r),   n = 2r+1,
// corners outside the level's image counting as zero (grid_sample, align_corners=True, zero padding,
// core/utils/utils.py:110-118).  The x offset runs with the first window index, as in the reference
// (meshgrid(dy, dx) stacked onto (x, y) coordinates, core/corr.py:213-226).
//
// Bilinear sampling is linear in S and all n*n samples of a pixel share one fractional part, so a pixel needs the
// (n+1)^2 dot products <f1[p], f2_l[y0-r+gy, x0-r+gx]> and four weights.  The kernel is a gather: 2*C flops per
// 4*C bytes fetched through the vector cache, far below the matrix-core ridge, so it runs on the vector lanes and is
// bound by cache bandwidth; there is no contraction tile to put on MFMA.
//
// Mapping: workgroup = TP consecutive pixels of one image-1 row at one level, 4 waves, each wave takes one pixel at a
// time.  Inside a wave the four 16-lane rows each take one grid point per step: lane k of a row loads float4s at
// channels 4k + 64m (256 contiguous bytes per row and load), multiplies with f1[p] held in registers, and the row is
// summed with DPP row shifts.  Dot products go to a per-wave LDS grid, the n*n samples are combined from it and staged
// in an LDS tile so that the workgroup writes every output channel as one contiguous run of TP floats.
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

constexpr int TP = 32;          // pixels per workgroup
constexpr int MAXL = 8;         // pyramid levels per launch
constexpr int MAXR = 8;         // window radius

struct LookupArgs {
    const float *f1;            // (B,H1,W1,C)
    const float *coords;        // (B,2,H1,W1): x then y, level-0 pixels
    float *out;                 // (B, L*n*n, H1, W1)
    const float *f2[MAXL];      // level l: (B,H2[l],W2[l],C)
    int H2[MAXL], W2[MAXL];
    int B, H1, W1, C, L, r;
    float scale;
};

__device__ __forceinline__ float row16_sum_to_last(float x) {
    // after the four steps lane 15 of every row of 16 holds the row's sum
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xe, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xc, true));
    return x;
}

// Integer cell and fractional part of a sampling coordinate.  Coordinates far outside any image (or NaN) are moved to
// a cell whose whole window is outside, so the int conversion is defined; the samples are then 0 (NaN stays NaN
// through the weights only if the caller passed NaN, as with grid_sample).
__device__ __forceinline__ void split_coord(float x, int &x0, float &fx) {
    const float fl = floorf(x);
    fx = x - fl;
    const float cl = fminf(fmaxf(fl, -1048576.f), 1048576.f);
    x0 = (int)cl;
    if (!(fx >= 0.f && fx <= 1.f)) fx = x - x;   // inf - inf = NaN for infinite x; finite x never gets here
}

// M = float4 loads per lane and grid point (covers 64*M channels), RT = radius known at compile time (0: runtime),
// VEC = C is a multiple of 4 (float4 loads); otherwise scalar loads, lane k taking channels k, k+16, ...
template <int M, int RT, bool VEC>
__global__ void __launch_bounds__(256) lookup_forward_kernel(const LookupArgs a) {
    extern __shared__ float lds[];
    const int r = RT ? RT : a.r;
    const int n = 2 * r + 1, G = n + 1, GG = G * G, NN = n * n;
    float *otile = lds;                                   // [NN][TP+1]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index as a scalar
    float *dgrid = lds + NN * (TP + 1) + wave * GG;        // [G][G] dot products of this wave's pixel
    const int row = lane >> 4, k = lane & 15;
    const int lvl = blockIdx.z % a.L, b = blockIdx.z / a.L;
    const int i = blockIdx.y, j0 = blockIdx.x * TP;
    const int H2 = a.H2[lvl], W2 = a.W2[lvl], C = a.C;
    const float *f2 = a.f2[lvl] + (size_t)b * H2 * W2 * C;
    const float lscale = 1.f / (float)(1 << lvl);
    const size_t plane = (size_t)a.H1 * a.W1;

    for (int t = 0; t < TP / 4; ++t) {
        const int jj = t * 4 + wave, j = j0 + jj;
        const bool live = j < a.W1;                        // uniform per wave
        int x0 = 0, y0 = 0;
        float fx = 0.f, fy = 0.f;
        if (live) {
            const float *cp = a.coords + (size_t)b * 2 * plane + (size_t)i * a.W1 + j;
            split_coord(cp[0] * lscale, x0, fx);
            split_coord(cp[plane] * lscale, y0, fy);
            const float *p1 = a.f1 + (((size_t)b * a.H1 + i) * a.W1 + j) * C;
            if constexpr (VEC) {
                float4 q[M];
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const int ch = (m * 16 + k) * 4;
                    q[m] = ch < C ? *reinterpret_cast<const float4 *>(p1 + ch) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
                for (int it = 0; it < (GG + 3) / 4; ++it) {    // same trip count in all rows (DPP needs them in step)
                    const int g = it * 4 + row;
                    const int gy = g / G, gx = g - gy * G;
                    const int yy = y0 - r + gy, xx = x0 - r + gx;
                    const bool ok = g < GG && yy >= 0 && yy < H2 && xx >= 0 && xx < W2;
                    float acc = 0.f;
                    if (ok) {
                        const float *p2 = f2 + ((size_t)yy * W2 + xx) * C;
#pragma unroll
                        for (int m = 0; m < M; ++m) {
                            const int ch = (m * 16 + k) * 4;
                            if (ch < C) {
                                const float4 v = *reinterpret_cast<const float4 *>(p2 + ch);
                                acc = fmaf(q[m].x, v.x, acc);
                                acc = fmaf(q[m].y, v.y, acc);
                                acc = fmaf(q[m].z, v.z, acc);
                                acc = fmaf(q[m].w, v.w, acc);
                            }
                        }
                    }
                    acc = row16_sum_to_last(acc);
                    if (k == 15 && g < GG) dgrid[g] = acc;
                }
            } else {
                for (int it = 0; it < (GG + 3) / 4; ++it) {
                    const int g = it * 4 + row;
                    const int gy = g / G, gx = g - gy * G;
                    const int yy = y0 - r + gy, xx = x0 - r + gx;
                    const bool ok = g < GG && yy >= 0 && yy < H2 && xx >= 0 && xx < W2;
                    float acc = 0.f;
                    if (ok) {
                        const float *p2 = f2 + ((size_t)yy * W2 + xx) * C;
                        for (int ch = k; ch < C; ch += 16) acc = fmaf(p1[ch], p2[ch], acc);
                    }
                    acc = row16_sum_to_last(acc);
                    if (k == 15 && g < GG) dgrid[g] = acc;
                }
            }
        }
        __syncthreads();
        if (live) {
            const float w00 = (1.f - fx) * (1.f - fy), w01 = fx * (1.f - fy), w10 = (1.f - fx) * fy, w11 = fx * fy;
            for (int o = lane; o < NN; o += 64) {
                const int ax = o / n, cy = o - ax * n;       // ax: x offset index, cy: y offset index
                const float *d = dgrid + cy * G + ax;
                otile[o * (TP + 1) + jj] = w00 * d[0] + w01 * d[1] + w10 * d[G] + w11 * d[G + 1];
            }
        }
        __syncthreads();
    }
    const int nj = min(TP, a.W1 - j0);
    float *o0 = a.out + (((size_t)b * a.L + lvl) * NN) * plane + (size_t)i * a.W1 + j0;
    for (int t = threadIdx.x; t < NN * TP; t += 256) {
        const int c = t / TP, jj = t % TP;
        if (jj < nj) o0[(size_t)c * plane + jj] = a.scale * otile[c * (TP + 1) + jj];
    }
}



// Forward for C <= 256 (a multiple of 4): a wave takes NPX consecutive pixels of the row at once.  Neighbouring
// pixels of a smooth flow field read almost the same fmap2 positions (their windows are shifted by about one
// column), so the wave walks the bounding box of the NPX windows once, multiplies every fetched fmap2 row with the
// NPX pixels' f1 held in registers, and each pixel then picks its own window out of the box of dot products.  At a
// uniform flow the box has (G+NPX-1)*G points for NPX*G*G window points: 3.1 times fewer fetches for NPX = 4, G = 10.
// Where the windows are scattered (box above BOXMAX points) the pixels are taken one by one, each with its own window
// as the box.
constexpr int NPX = 4;
constexpr int TPG = 16;         // pixels per workgroup of the grouped kernel: one group of NPX per wave
constexpr int BOXMAX = 324;      // (2*8+2)^2: one window at the largest radius always fits

// Fetch of one box point's channels for this lane.  Always a valid address: positions outside the level (or past the
// box) are clamped into it and their dot products are discarded by the caller; channel slots past C re-read channel
// 0 and meet zeros in q.
template <int M>
__device__ __forceinline__ void box_fetch(const float *f2, int H2, int W2, int C, int k, int yy, int xx, float4 (&v)[M]) {
    const int yc = min(max(yy, 0), H2 - 1), xc = min(max(xx, 0), W2 - 1);
    const float *p2 = f2 + ((size_t)yc * W2 + xc) * C;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int ch = (m * 16 + k) * 4;
        v[m] = *reinterpret_cast<const float4 *>(p2 + (ch < C ? ch : 0));
    }
}

template <int M, int NP>
__device__ __forceinline__ void box_point(const float4 (&q)[NPX][M], int k0, const float4 (&v)[M], bool keep, bool store,
                                          float *dst) {
    float acc[NP];
#pragma unroll
    for (int t = 0; t < NP; ++t) acc[t] = 0.f;
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int t = 0; t < NP; ++t) {
            acc[t] = fmaf(q[k0 + t][m].x, v[m].x, acc[t]);
            acc[t] = fmaf(q[k0 + t][m].y, v[m].y, acc[t]);
            acc[t] = fmaf(q[k0 + t][m].z, v[m].z, acc[t]);
            acc[t] = fmaf(q[k0 + t][m].w, v[m].w, acc[t]);
        }
#pragma unroll
    for (int t = 0; t < NP; ++t) {
        const float sum = row16_sum_to_last(acc[t]);
        if (store) dst[t * BOXMAX] = keep ? sum : 0.f;
    }
}

// Dot products of NP pixels' f1 (q[k0..k0+NP)) with every fmap2 position of the box [bx0,bx0+BW) x [by0,by0+BH);
// positions outside the level count as zero.  The four 16-lane rows take box points bp = 4*it + row; the fetch of the
// next point is issued before the arithmetic of the current one (two points per trip, registers ping-pong).
template <int M, int NP>
__device__ __forceinline__ void box_dots(const float *f2, int H2, int W2, int C, int k, int row, const float4 (&q)[NPX][M],
                                         int k0, int bx0, int by0, int BW, int BH, float *dbox) {
    const int npts = BW * BH;
    int bx = row, by = 0;                                   // BW >= 4 > row
    float4 va[M], vb[M];
    box_fetch<M>(f2, H2, W2, C, k, by0, bx0 + bx, va);
    for (int bp = row; bp - row < npts; bp += 8) {          // same trip count in all rows (DPP needs them in step)
        const int ya = by0 + by, xa = bx0 + bx;
        bx += 4;
        if (bx >= BW) { bx -= BW; ++by; }
        const int yb = by0 + by, xb = bx0 + bx;
        box_fetch<M>(f2, H2, W2, C, k, yb, xb, vb);
        box_point<M, NP>(q, k0, va, ya >= 0 && ya < H2 && xa >= 0 && xa < W2, k == 15 && bp < npts, dbox + bp);
        bx += 4;
        if (bx >= BW) { bx -= BW; ++by; }
        box_fetch<M>(f2, H2, W2, C, k, by0 + by, bx0 + bx, va);
        box_point<M, NP>(q, k0, vb, yb >= 0 && yb < H2 && xb >= 0 && xb < W2, k == 15 && bp + 4 < npts, dbox + bp + 4);
    }
}

template <int M>
__global__ void __launch_bounds__(256) lookup_forward_group_kernel(const LookupArgs a) {
    extern __shared__ float lds[];
    const int r = a.r, n = 2 * r + 1, G = n + 1, NN = n * n;
    float *otile = lds;                                   // [NN][TPG+1]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index as a scalar
    float *dbox = lds + NN * (TPG + 1) + wave * (NPX * BOXMAX);   // [NPX][BOXMAX] dot products of this wave's box
    const int row = lane >> 4, k = lane & 15;
    const int lvl = blockIdx.z % a.L, b = blockIdx.z / a.L;
    const int i = blockIdx.y, j0 = blockIdx.x * TPG;
    const int H2 = a.H2[lvl], W2 = a.W2[lvl], C = a.C;
    const float *f2 = a.f2[lvl] + (size_t)b * H2 * W2 * C;
    const float lscale = 1.f / (float)(1 << lvl);
    const size_t plane = (size_t)a.H1 * a.W1;

    for (int t = 0; t < TPG / (4 * NPX); ++t) {
        const int jj0 = (t * 4 + wave) * NPX;
        if (j0 + jj0 >= a.W1) break;                       // uniform per wave; no workgroup barrier inside the loop
        int ox[NPX], oy[NPX];
        float fx[NPX], fy[NPX];
        float4 q[NPX][M];
        int bx0 = 0, bx1 = 0, by0 = 0, by1 = 0;
#pragma unroll
        for (int e = 0; e < NPX; ++e) {
            const int j = min(j0 + jj0 + e, a.W1 - 1);     // pixels past the row's end repeat the last one (not stored)
            const float *cp = a.coords + (size_t)b * 2 * plane + (size_t)i * a.W1 + j;
            int x0, y0;
            split_coord(cp[0] * lscale, x0, fx[e]);
            split_coord(cp[plane] * lscale, y0, fy[e]);
            ox[e] = x0 - r;
            oy[e] = y0 - r;
            bx0 = e ? min(bx0, ox[e]) : ox[e];
            bx1 = e ? max(bx1, ox[e]) : ox[e];
            by0 = e ? min(by0, oy[e]) : oy[e];
            by1 = e ? max(by1, oy[e]) : oy[e];
            const float *p1 = a.f1 + (((size_t)b * a.H1 + i) * a.W1 + j) * C;
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const int ch = (m * 16 + k) * 4;
                q[e][m] = ch < C ? *reinterpret_cast<const float4 *>(p1 + ch) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
        const long BWl = (long)bx1 - bx0 + G, BHl = (long)by1 - by0 + G;
        const bool joint = BWl * BHl <= BOXMAX;
        if (joint) box_dots<M, NPX>(f2, H2, W2, C, k, row, q, 0, bx0, by0, (int)BWl, (int)BHl, dbox);
#pragma unroll
        for (int e = 0; e < NPX; ++e) {
            if (!joint) box_dots<M, 1>(f2, H2, W2, C, k, row, q, e, ox[e], oy[e], G, G, dbox);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const int BW = joint ? (int)BWl : G;
            const float *dp = dbox + (joint ? e * BOXMAX + (oy[e] - by0) * BW + (ox[e] - bx0) : 0);
            const float w00 = (1.f - fx[e]) * (1.f - fy[e]), w01 = fx[e] * (1.f - fy[e]);
            const float w10 = (1.f - fx[e]) * fy[e], w11 = fx[e] * fy[e];
            if (j0 + jj0 + e < a.W1)
                for (int o = lane; o < NN; o += 64) {
                    const int ax = o / n, cy = o - ax * n;
                    const float *d = dp + cy * BW + ax;
                    otile[o * (TPG + 1) + jj0 + e] = w00 * d[0] + w01 * d[1] + w10 * d[BW] + w11 * d[BW + 1];
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads();
    const int nj = min(TPG, a.W1 - j0);
    float *o0 = a.out + (((size_t)b * a.L + lvl) * NN) * plane + (size_t)i * a.W1 + j0;
    for (int t = threadIdx.x; t < NN * TPG; t += 256) {
        const int c = t / TPG, jj = t % TPG;
        if (jj < nj) o0[(size_t)c * plane + jj] = a.scale * otile[c * (TPG + 1) + jj];
    }
}

// ------------------------------------------------------------------------------------------------------------
// Backward: gradients of the lookup w.r.t. both feature maps (coords get none: the flow iterations detach them,
// core/sepflow.py:194).  With W[p,l][gy][gx] = scale * sum over the samples (a,c) and corners (dy,dx) that read grid
// point (gy,gx) = (c+dy, a+dx) of weight(dy,dx) * grad_out[b,l,a,c,p]:
//   d_f1[p]        = sum_l sum_g W[p,l][g] * f2_l[origin_p + g]           (gather, same reads as the forward)
//   d_f2_l[q]      = sum_p W[p,l][q - origin_p] * f1[p]                   (scatter, done by the owner of q)
// Three kernels: W and the window origins go to scratch once; d_f1 is one thread per (pixel, channel); d_f2 is
// owned by tiles of fmap2 positions that scan the pixels for windows touching the tile, in ascending pixel order,
// so no atomics are used and sums are run-to-run identical.  Coarse levels have few positions but as many
// (pixel, grid point) pairs as level 0: their pixel range is cut into S_l slices, each slice writes a partial
// result, and a last kernel adds the slices in order.
// ------------------------------------------------------------------------------------------------------------

constexpr int TQX = 8, TQY = 4;                     // fmap2 positions per d_f2 wave: the 32 rows of one MFMA tile
constexpr int NCH = 128;                            // channels per d_f2 wave
constexpr int NPR = 2;                              // pixel pairs fetched before their MFMAs are issued
static_assert(TQX * TQY == 32, "one tile position per MFMA row");

struct LookupBwdArgs {
    const float *f1, *coords, *gout;
    float *d_f1;
    const float *f2[MAXL];
    float *d_f2[MAXL];
    float *part[MAXL];          // S[l] partial results of d_f2[l] (unused when S[l] == 1)
    float *wg;                  // (B,L,H1*W1,G*G)
    int *org;                   // (B,L,H1*W1,2): x then y of the window's first grid point
    int H2[MAXL], W2[MAXL], S[MAXL], tile0[MAXL + 1];
    int B, H1, W1, C, L, r;
    float scale;
};

__global__ void __launch_bounds__(256) lookup_grid_grad_kernel(const LookupBwdArgs a) {
    extern __shared__ float lds[];
    const int r = a.r, n = 2 * r + 1, G = n + 1, GG = G * G, NN = n * n;
    float *gtile = lds;                                   // [NN][TP+1]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // wave index as a scalar
    const int lvl = blockIdx.z % a.L, b = blockIdx.z / a.L;
    const int i = blockIdx.y, j0 = blockIdx.x * TP;
    const size_t plane = (size_t)a.H1 * a.W1;
    const int nj = min(TP, a.W1 - j0);
    const float *g0 = a.gout + (((size_t)b * a.L + lvl) * NN) * plane + (size_t)i * a.W1 + j0;
    for (int t = threadIdx.x; t < NN * TP; t += 256) {
        const int c = t / TP, jj = t % TP;
        gtile[c * (TP + 1) + jj] = jj < nj ? g0[(size_t)c * plane + jj] : 0.f;
    }
    __syncthreads();
    const float lscale = 1.f / (float)(1 << lvl);
    for (int jj = wave; jj < nj; jj += 4) {
        const int j = j0 + jj;
        const float *cp = a.coords + (size_t)b * 2 * plane + (size_t)i * a.W1 + j;
        int x0, y0;
        float fx, fy;
        split_coord(cp[0] * lscale, x0, fx);
        split_coord(cp[plane] * lscale, y0, fy);
        const float w[2][2] = {{(1.f - fx) * (1.f - fy), fx * (1.f - fy)}, {(1.f - fx) * fy, fx * fy}};   // [dy][dx]
        const size_t pl = ((size_t)b * a.L + lvl) * plane + (size_t)i * a.W1 + j;
        for (int g = lane; g < GG; g += 64) {
            const int gy = g / G, gx = g - gy * G;
            float sum = 0.f;
#pragma unroll
            for (int dy = 0; dy < 2; ++dy)
#pragma unroll
                for (int dx = 0; dx < 2; ++dx) {
                    const int c = gy - dy, ax = gx - dx;
                    if (c >= 0 && c < n && ax >= 0 && ax < n) sum = fmaf(w[dy][dx], gtile[(ax * n + c) * (TP + 1) + jj], sum);
                }
            a.wg[pl * GG + g] = a.scale * sum;
        }
        if (lane == 0) {
            a.org[pl * 2] = x0 - r;
            a.org[pl * 2 + 1] = y0 - r;
        }
    }
}

// one workgroup per image-1 pixel, thread = channel (channels beyond 256 in further passes)
__global__ void __launch_bounds__(256) lookup_df1_kernel(const LookupBwdArgs a) {
    const int G = 2 * a.r + 2, GG = G * G, C = a.C;
    const size_t plane = (size_t)a.H1 * a.W1;
    const size_t p = blockIdx.x % plane;
    const int b = blockIdx.x / plane;
    for (int c = threadIdx.x; c < C; c += 256) {
        float acc0 = 0.f, acc1 = 0.f;
        for (int l = 0; l < a.L; ++l) {
            const int H2 = a.H2[l], W2 = a.W2[l];
            const size_t pl = ((size_t)b * a.L + l) * plane + p;
            const int ox = a.org[pl * 2], oy = a.org[pl * 2 + 1];
            const float *w = a.wg + pl * GG;
            const float *f2 = a.f2[l] + (size_t)b * H2 * W2 * C + c;
            const int gy0 = max(0, -oy), gy1 = min(G, H2 - oy);       // rows and columns of the window inside the level
            const int gx0 = max(0, -ox), gx1 = min(G, W2 - ox);
            for (int gy = gy0; gy < gy1; ++gy) {
                const float *rowp = f2 + ((size_t)(oy + gy) * W2 + ox) * C;
                const float *wr = w + gy * G;
                int gx = gx0;
                for (; gx + 1 < gx1; gx += 2) {
                    acc0 = fmaf(wr[gx], rowp[(size_t)gx * C], acc0);
                    acc1 = fmaf(wr[gx + 1], rowp[(size_t)(gx + 1) * C], acc1);
                }
                if (gx < gx1) acc0 = fmaf(wr[gx], rowp[(size_t)gx * C], acc0);
            }
        }
        a.d_f1[((size_t)b * plane + p) * C + c] = acc0 + acc1;
    }
}

// d_f1 for C a multiple of 4: a wave takes NPX consecutive pixels and, level by level, walks the bounding box of their
// windows once.  Lane = 4 channels (float4 fetch of a whole fmap2 row per wave and box point); the NPX weights of a box
// point (zero outside a pixel's own window or outside the level) sit in a per-wave LDS table and arrive as one
// broadcast read.  Scattered windows (box above BOXMAX points) are walked pixel by pixel with the same code.
__global__ void __launch_bounds__(256) lookup_df1_group_kernel(const LookupBwdArgs a) {
    __shared__ __attribute__((aligned(16))) float wtab[4][BOXMAX][NPX];
    const int G = 2 * a.r + 2, GG = G * G, C = a.C;
    // (the wave index stays a vector value here: with it as a scalar the walk measured slower, 0.137 against 0.127 ms)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int b = blockIdx.z, i = blockIdx.y, j0 = blockIdx.x * TPG + wave * NPX;
    if (j0 >= a.W1) return;                                 // whole wave; the kernel has no workgroup barrier
    const size_t plane = (size_t)a.H1 * a.W1;
    float (*wt)[NPX] = wtab[wave];
    for (int c0 = 0; c0 < C; c0 += 256) {
        const int ch = c0 + lane * 4;
        const int chl = ch < C ? ch : 0;                    // idle lanes re-read channel 0 and store nothing
        float4 acc[NPX];
#pragma unroll
        for (int e = 0; e < NPX; ++e) acc[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int l = 0; l < a.L; ++l) {
            const int H2 = a.H2[l], W2 = a.W2[l];
            const float *f2 = a.f2[l] + (size_t)b * H2 * W2 * C + chl;
            int ox[NPX], oy[NPX];
            size_t pl[NPX];
            int bx0 = 0, bx1 = 0, by0 = 0, by1 = 0;
#pragma unroll
            for (int e = 0; e < NPX; ++e) {
                const int j = min(j0 + e, a.W1 - 1);
                pl[e] = ((size_t)b * a.L + l) * plane + (size_t)i * a.W1 + j;
                ox[e] = a.org[pl[e] * 2];
                oy[e] = a.org[pl[e] * 2 + 1];
                bx0 = e ? min(bx0, ox[e]) : ox[e];
                bx1 = e ? max(bx1, ox[e]) : ox[e];
                by0 = e ? min(by0, oy[e]) : oy[e];
                by1 = e ? max(by1, oy[e]) : oy[e];
            }
            const long BWl = (long)bx1 - bx0 + G, BHl = (long)by1 - by0 + G;
            const bool joint = BWl * BHl <= BOXMAX;
            for (int sub = 0; sub < (joint ? 1 : NPX); ++sub) {
                int qx0 = bx0, qy0 = by0, BW = (int)(joint ? BWl : G), BH = (int)(joint ? BHl : G);
                if (!joint) {
#pragma unroll
                    for (int e = 0; e < NPX; ++e)
                        if (e == sub) { qx0 = ox[e]; qy0 = oy[e]; }
                }
                const int npts = BW * BH;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                for (int bp = lane; bp < npts; bp += 64) {
                    const int by = bp / BW, bx = bp - by * BW;
                    const int yy = qy0 + by, xx = qx0 + bx;
                    const bool inside = yy >= 0 && yy < H2 && xx >= 0 && xx < W2;
                    float w[NPX];
#pragma unroll
                    for (int e = 0; e < NPX; ++e) {
                        const int gy = yy - oy[e], gx = xx - ox[e];
                        const bool use = inside && (joint || e == sub) && j0 + e < a.W1 && gy >= 0 && gy < G && gx >= 0 && gx < G;
                        w[e] = use ? a.wg[pl[e] * GG + gy * G + gx] : 0.f;
                    }
                    *reinterpret_cast<float4 *>(wt[bp]) = make_float4(w[0], w[1], w[2], w[3]);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                int bx = 0, by = 0;
#pragma unroll 4
                for (int bp = 0; bp < npts; ++bp) {
                    const int yc = min(max(qy0 + by, 0), H2 - 1), xc = min(max(qx0 + bx, 0), W2 - 1);
                    const float4 v = *reinterpret_cast<const float4 *>(f2 + ((size_t)yc * W2 + xc) * C);
                    const float4 w = *reinterpret_cast<const float4 *>(wt[bp]);
                    const float ws[NPX] = {w.x, w.y, w.z, w.w};
#pragma unroll
                    for (int e = 0; e < NPX; ++e) {
                        acc[e].x = fmaf(ws[e], v.x, acc[e].x);
                        acc[e].y = fmaf(ws[e], v.y, acc[e].y);
                        acc[e].z = fmaf(ws[e], v.z, acc[e].z);
                        acc[e].w = fmaf(ws[e], v.w, acc[e].w);
                    }
                    if (++bx == BW) { bx = 0; ++by; }
                }
            }
        }
        if (ch < C) {
#pragma unroll
            for (int e = 0; e < NPX; ++e)
                if (j0 + e < a.W1)
                    *reinterpret_cast<float4 *>(a.d_f1 + (((size_t)b * a.H1 + i) * a.W1 + j0 + e) * C + ch) = acc[e];
        }
    }
}

// One wave = (tile of TQY x TQX positions of one level, slice of the pixel range, block of NCH channels).  For the
// tile, d_f2[pos, ch] = sum over pixels of W[pos, pixel] * f1[pixel, ch] is a small matrix product whose inner index
// runs over the pixels whose window touches the tile.  The wave scans its pixels 64 at a time (origins stay in the
// lanes' registers), takes the touching ones in ascending order, two per v_mfma_f32_32x32x2_f32: operand A = the two
// pixels' window entries at the tile's positions (zero outside the window), operand B = their f1 channels, fetched as
// contiguous runs.  Four pixels are fetched before their MFMAs are issued (measured: 2 pixels 0.147, 4 0.137, 8 0.142 ms).
// No LDS, no barrier, no atomics.
typedef float lk_v16f __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(64) lookup_df2_kernel(const LookupBwdArgs a) {
    constexpr int NB = NCH / 32;                               // operand-B registers (32 channels each) per pixel pair
    const int G = 2 * a.r + 2, GG = G * G, C = a.C;
    const int lane = threadIdx.x, half = lane >> 5, l32 = lane & 31;
    int l = 0;
    while (l + 1 < a.L && (int)blockIdx.x >= a.tile0[l + 1]) ++l;
    const int H2 = a.H2[l], W2 = a.W2[l], S = a.S[l];
    const int tx_n = (W2 + TQX - 1) / TQX, ty_n = (H2 + TQY - 1) / TQY;
    int t = blockIdx.x - a.tile0[l];
    const int slice = t / (tx_n * ty_n);
    t -= slice * tx_n * ty_n;
    const int ty0 = (t / tx_n) * TQY, tx0 = (t % tx_n) * TQX;
    const int b = blockIdx.z, c0 = blockIdx.y * NCH;
    const int P = a.H1 * a.W1;
    const int per = (P + S - 1) / S, p_begin = slice * per, p_end = min(P, p_begin + per);
    const size_t pl0 = ((size_t)b * a.L + l) * P;
    const int *__restrict__ org = a.org + pl0 * 2;
    const float *__restrict__ wg = a.wg + pl0 * GG;
    const float *__restrict__ f1 = a.f1 + (size_t)b * P * C;
    // operand A row of this lane: tile position l32; operand B columns: channels c0 + 32*cb + l32
    const int qy = ty0 + l32 / TQX, qx = tx0 + l32 % TQX;

    lk_v16f acc[NB];
#pragma unroll
    for (int cb = 0; cb < NB; ++cb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[cb][v] = 0.f;

    // origins of the next 64 pixels are fetched while the current ones are worked on
    int2 nxt = make_int2(0, 0);
    if (p_begin + lane < p_end) nxt = *reinterpret_cast<const int2 *>(org + (size_t)(p_begin + lane) * 2);
    for (int pc = p_begin; pc < p_end; pc += 64) {
        const int p = pc + lane;
        const int ox = nxt.x, oy = nxt.y;
        if (p + 64 < p_end) nxt = *reinterpret_cast<const int2 *>(org + (size_t)(p + 64) * 2);
        const bool hit = p < p_end && ox < tx0 + TQX && ox + G > tx0 && oy < ty0 + TQY && oy + G > ty0;
        unsigned long long m = __ballot(hit);
        while (m) {
            float wa[NPR], fb[NPR][NB];
            bool any[NPR];
#pragma unroll
            for (int pr = 0; pr < NPR; ++pr) {
                any[pr] = m != 0;                              // wave-uniform
                if (!any[pr]) {                                // nothing left in these 64 pixels: skip the slot
                    wa[pr] = 0.f;
#pragma unroll
                    for (int cb = 0; cb < NB; ++cb) fb[pr][cb] = 0.f;
                    continue;
                }
                const int cn0 = m ? __builtin_ctzll(m) : 0;
                m &= m - 1;
                const bool two = m != 0;
                const int cn1 = two ? __builtin_ctzll(m) : cn0;
                m &= m - 1;
                const bool mine = any[pr] && (half == 0 || two);
                const int cn = half ? cn1 : cn0;
                const int oxc = __shfl(ox, cn), oyc = __shfl(oy, cn);
                const size_t pp = (size_t)(pc + cn);
                const int gx = qx - oxc, gy = qy - oyc;
                wa[pr] = mine && gx >= 0 && gx < G && gy >= 0 && gy < G ? wg[pp * GG + gy * G + gx] : 0.f;
#pragma unroll
                for (int cb = 0; cb < NB; ++cb) {
                    const int c = c0 + 32 * cb + l32;
                    fb[pr][cb] = mine && c < C ? f1[pp * C + c] : 0.f;
                }
            }
#pragma unroll
            for (int pr = 0; pr < NPR; ++pr)
                if (any[pr]) {
#pragma unroll
                    for (int cb = 0; cb < NB; ++cb)
                        acc[cb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[pr], fb[pr][cb], acc[cb], 0, 0, 0);
                }
        }
    }
    // register v of lane (half, l32) holds tile position 8*(v/4) + 4*half + v%4, channel c0 + 32*cb + l32
    const size_t lvl_elems = (size_t)a.B * H2 * W2 * C;
    float *dst = (S == 1 ? a.d_f2[l] : a.part[l] + (size_t)slice * lvl_elems) + (size_t)b * H2 * W2 * C;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int pos = 8 * (v / 4) + 4 * half + v % 4;
        const int y = ty0 + pos / TQX, x = tx0 + pos % TQX;
        if (y < H2 && x < W2) {
            float *d = dst + ((size_t)y * W2 + x) * C;
#pragma unroll
            for (int cb = 0; cb < NB; ++cb) {
                const int c = c0 + 32 * cb + l32;
                if (c < C) d[c] = acc[cb][v];
            }
        }
    }
}

// d_f2[l] = sum over the S[l] slices, in slice order; blockIdx.y = level
__global__ void __launch_bounds__(256) lookup_df2_reduce_kernel(const LookupBwdArgs a) {
    const int l = blockIdx.y;
    const int S = a.S[l];
    if (S == 1) return;
    const size_t n = (size_t)a.B * a.H2[l] * a.W2[l] * a.C;
    const float *__restrict__ part = a.part[l];
    float *__restrict__ dst = a.d_f2[l];
    const size_t stride = (size_t)gridDim.x * 256;
    if (n % 4 == 0 && (uintptr_t)dst % 16 == 0) {
        for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n / 4; e += stride) {
            float4 s = reinterpret_cast<const float4 *>(part)[e];
#pragma unroll 8
            for (int k = 1; k < S; ++k) {
                const float4 v = reinterpret_cast<const float4 *>(part + (size_t)k * n)[e];
                s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
            }
            reinterpret_cast<float4 *>(dst)[e] = s;
        }
    } else {
        for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
            float s = part[e];
            for (int k = 1; k < S; ++k) s += part[(size_t)k * n + e];
            dst[e] = s;
        }
    }
}

int bad(const char *msg) { return sepcorr_set_error(SEPCORR_EINVAL, msg); }

template <int M, int RT, bool VEC>
void launch(const LookupArgs &a, dim3 grid, size_t lds, hipStream_t s) {
    hipLaunchKernelGGL((lookup_forward_kernel<M, RT, VEC>), grid, dim3(256), lds, s, a);
}

template <int RT>
void launch_c(const LookupArgs &a, dim3 grid, size_t lds, hipStream_t s) {
    const int C = a.C;
    bool vec = C % 4 == 0 && (uintptr_t)a.f1 % 16 == 0;
    for (int l = 0; l < a.L; ++l) vec = vec && (uintptr_t)a.f2[l] % 16 == 0;
    if (!vec) launch<1, RT, false>(a, grid, lds, s);
    else if (C <= 64) launch<1, RT, true>(a, grid, lds, s);
    else if (C <= 128) launch<2, RT, true>(a, grid, lds, s);
    else if (C <= 256) launch<4, RT, true>(a, grid, lds, s);
    else if (C <= 512) launch<8, RT, true>(a, grid, lds, s);
    else launch<16, RT, true>(a, grid, lds, s);
}


// slices of the pixel range for level l: twice as many as level 0 has more positions than level l, at most 128
// (measured: with one slice per unit of positions the waves run too long for the launch to balance)
int level_slices(const int *h2, const int *w2, int l) {
    const long n0 = (long)h2[0] * w2[0], nl = (long)h2[l] * w2[l];
    long s = nl > 0 ? 2 * n0 / nl : 2;
    if (s < 2) s = 2;
    return (int)(s > 128 ? 128 : s);
}

int check_common(const void *f1, const float *const *f2_levels, const int *h2, const int *w2, const void *coords,
                 int B, int H1, int W1, int C, int L, int radius) {
    if (!f1 || !f2_levels || !h2 || !w2 || !coords) return bad("sepcorr: lookup: NULL pointer");
    if (B < 1 || H1 < 1 || W1 < 1 || C < 1) return bad("sepcorr: lookup: sizes must be positive");
    if (C > 1024) return bad("sepcorr: lookup: C above 1024 is not supported");
    if (L < 1 || L > MAXL) return bad("sepcorr: lookup: 1 to 8 pyramid levels are supported");
    if (radius < 1 || radius > MAXR) return bad("sepcorr: lookup: radius must be 1..8");
    const int n = 2 * radius + 1;
    if ((double)B * L * n * n * H1 * W1 > 2147483647.0 || (double)B * H1 * W1 * C > 2147483647.0)
        return bad("sepcorr: a tensor would have 2^31 or more elements");
    if ((long)B * L > 65535 || H1 > 65535) return bad("sepcorr: lookup: B*L and H1 must be below 65536");
    for (int l = 0; l < L; ++l) {
        if (!f2_levels[l]) return bad("sepcorr: lookup: NULL level pointer");
        if (h2[l] < 1 || w2[l] < 1) return bad("sepcorr: lookup: level sizes must be positive");
        if ((double)B * h2[l] * w2[l] * C > 2147483647.0) return bad("sepcorr: a tensor would have 2^31 or more elements");
    }
    return SEPCORR_OK;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

int launch_error(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return SEPCORR_OK;
    char msg[160];
    snprintf(msg, sizeof(msg), "sepcorr: %s: %s", what, hipGetErrorString(e));
    return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
}

}  // namespace

extern "C" {

int sepcorr_lookup_forward(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                           const float *coords, float *out, int B, int H1, int W1, int C, int L, int radius,
                           float scale, void *stream) {
    const int rc = check_common(f1, f2_levels, h2, w2, coords, B, H1, W1, C, L, radius);
    if (rc != SEPCORR_OK) return rc;
    if (!out) return bad("sepcorr: lookup: NULL pointer");
    const int n = 2 * radius + 1;
    LookupArgs a = {};
    a.f1 = f1; a.coords = coords; a.out = out;
    for (int l = 0; l < L; ++l) {
        a.f2[l] = f2_levels[l]; a.H2[l] = h2[l]; a.W2[l] = w2[l];
    }
    a.B = B; a.H1 = H1; a.W1 = W1; a.C = C; a.L = L; a.r = radius; a.scale = scale;
    const size_t lds = ((size_t)n * n * (TP + 1) + 4 * (size_t)(n + 1) * (n + 1)) * sizeof(float);
    const dim3 grid((W1 + TP - 1) / TP, H1, B * L);
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool vec = C % 4 == 0 && (uintptr_t)f1 % 16 == 0;
    for (int l = 0; l < L; ++l) vec = vec && (uintptr_t)a.f2[l] % 16 == 0;
    if (vec && C <= 256) {
        const size_t glds = ((size_t)n * n * (TPG + 1) + 4 * (size_t)NPX * BOXMAX) * sizeof(float);
        const dim3 ggrid((W1 + TPG - 1) / TPG, H1, B * L);
        if (C <= 64) hipLaunchKernelGGL(lookup_forward_group_kernel<1>, ggrid, dim3(256), glds, s, a);
        else if (C <= 128) hipLaunchKernelGGL(lookup_forward_group_kernel<2>, ggrid, dim3(256), glds, s, a);
        else hipLaunchKernelGGL(lookup_forward_group_kernel<4>, ggrid, dim3(256), glds, s, a);
    } else if (radius == 4) launch_c<4>(a, grid, lds, s);
    else launch_c<0>(a, grid, lds, s);
    return launch_error("lookup kernel");
}

size_t sepcorr_lookup_backward_workspace_bytes(const int *h2, const int *w2, int B, int H1, int W1, int C, int L,
                                               int radius) {
    if (!h2 || !w2 || B < 1 || H1 < 1 || W1 < 1 || C < 1 || L < 1 || L > MAXL || radius < 1 || radius > MAXR) return 0;
    const size_t G = 2 * (size_t)radius + 2, pix = (size_t)B * L * H1 * W1;
    size_t n = align256(pix * G * G * sizeof(float)) + align256(pix * 2 * sizeof(int));
    for (int l = 0; l < L; ++l) {
        if (h2[l] < 1 || w2[l] < 1) return 0;
        const int S = level_slices(h2, w2, l);
        if (S > 1) n += align256((size_t)S * B * h2[l] * w2[l] * C * sizeof(float));
    }
    return n;
}

int sepcorr_lookup_backward(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                            const float *coords, const float *grad_out, float *d_f1, float *const *d_f2_levels,
                            int B, int H1, int W1, int C, int L, int radius, float scale,
                            void *workspace, size_t workspace_bytes, void *stream) {
    const int rc = check_common(f1, f2_levels, h2, w2, coords, B, H1, W1, C, L, radius);
    if (rc != SEPCORR_OK) return rc;
    if (!grad_out || !d_f1 || !d_f2_levels) return bad("sepcorr: lookup: NULL pointer");
    const size_t need = sepcorr_lookup_backward_workspace_bytes(h2, w2, B, H1, W1, C, L, radius);
    if (!workspace || workspace_bytes < need)
        return sepcorr_set_error(SEPCORR_EWORKSPACE, "sepcorr: lookup backward: workspace missing or too small");
    if ((uintptr_t)workspace % 256) return bad("sepcorr: lookup backward: workspace must be 256-byte aligned");
    const int n = 2 * radius + 1, G = n + 1;
    const size_t pix = (size_t)B * L * H1 * W1;
    LookupBwdArgs a = {};
    a.f1 = f1; a.coords = coords; a.gout = grad_out; a.d_f1 = d_f1;
    char *ws = static_cast<char *>(workspace);
    a.wg = reinterpret_cast<float *>(ws); ws += align256(pix * G * G * sizeof(float));
    a.org = reinterpret_cast<int *>(ws); ws += align256(pix * 2 * sizeof(int));
    long tiles = 0;
    for (int l = 0; l < L; ++l) {
        if (!d_f2_levels[l]) return bad("sepcorr: lookup: NULL level pointer");
        a.f2[l] = f2_levels[l]; a.d_f2[l] = d_f2_levels[l]; a.H2[l] = h2[l]; a.W2[l] = w2[l];
        a.S[l] = level_slices(h2, w2, l);
        if (a.S[l] > 1) {
            a.part[l] = reinterpret_cast<float *>(ws);
            ws += align256((size_t)a.S[l] * B * h2[l] * w2[l] * C * sizeof(float));
        }
        a.tile0[l] = (int)tiles;
        tiles += (long)((w2[l] + TQX - 1) / TQX) * ((h2[l] + TQY - 1) / TQY) * a.S[l];
        if (tiles > 2147483647L) return bad("sepcorr: lookup backward: too many tiles");
    }
    a.tile0[L] = (int)tiles;
    a.B = B; a.H1 = H1; a.W1 = W1; a.C = C; a.L = L; a.r = radius; a.scale = scale;
    if (B > 65535) return bad("sepcorr: lookup backward: B must be below 65536");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t lds = (size_t)n * n * (TP + 1) * sizeof(float);
    hipLaunchKernelGGL(lookup_grid_grad_kernel, dim3((W1 + TP - 1) / TP, H1, B * L), dim3(256), lds, s, a);
    if (int e = launch_error("lookup grid-gradient kernel")) return e;
    // d_f1 and d_f2 only read the window gradients: they run side by side on the library's side streams
    void *va = nullptr, *vb = nullptr;
    void *token = sepcorr_fork(s, &va, &vb);
    hipStream_t sa = static_cast<hipStream_t>(va), sb = static_cast<hipStream_t>(vb);
    bool vec = C % 4 == 0 && (uintptr_t)d_f1 % 16 == 0;
    for (int l = 0; l < L; ++l) vec = vec && (uintptr_t)a.f2[l] % 16 == 0;
    if (vec) hipLaunchKernelGGL(lookup_df1_group_kernel, dim3((W1 + TPG - 1) / TPG, H1, B), dim3(256), 0, sa, a);
    else hipLaunchKernelGGL(lookup_df1_kernel, dim3((unsigned)((size_t)B * H1 * W1)), dim3(256), 0, sa, a);
    int rl = launch_error("lookup d_f1 kernel");
    if (rl == SEPCORR_OK) {
        hipLaunchKernelGGL(lookup_df2_kernel, dim3((unsigned)tiles, (C + NCH - 1) / NCH, B), dim3(64), 0, sb, a);
        rl = launch_error("lookup d_f2 kernel");
    }
    if (rl == SEPCORR_OK) {
        hipLaunchKernelGGL(lookup_df2_reduce_kernel, dim3(1024, L), dim3(256), 0, sb, a);
        rl = launch_error("lookup d_f2 reduction");
    }
    const int rj = sepcorr_join(token);
    return rl ? rl : rj;
}

}  // extern "C"
