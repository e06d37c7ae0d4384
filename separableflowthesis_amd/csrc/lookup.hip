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
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
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

}  // namespace

extern "C" {

int sepcorr_lookup_forward(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                           const float *coords, float *out, int B, int H1, int W1, int C, int L, int radius,
                           float scale, void *stream) {
    if (!f1 || !f2_levels || !h2 || !w2 || !coords || !out) return bad("sepcorr: lookup: NULL pointer");
    if (B < 1 || H1 < 1 || W1 < 1 || C < 1) return bad("sepcorr: lookup: sizes must be positive");
    if (C > 1024) return bad("sepcorr: lookup: C above 1024 is not supported");
    if (L < 1 || L > MAXL) return bad("sepcorr: lookup: 1 to 8 pyramid levels are supported");
    if (radius < 1 || radius > MAXR) return bad("sepcorr: lookup: radius must be 1..8");
    const int n = 2 * radius + 1;
    if ((double)B * L * n * n * H1 * W1 > 2147483647.0 || (double)B * H1 * W1 * C > 2147483647.0)
        return bad("sepcorr: a tensor would have 2^31 or more elements");
    if ((long)B * L > 65535 || H1 > 65535) return bad("sepcorr: lookup: B*L and H1 must be below 65536");
    LookupArgs a = {};
    a.f1 = f1; a.coords = coords; a.out = out;
    for (int l = 0; l < L; ++l) {
        if (!f2_levels[l]) return bad("sepcorr: lookup: NULL level pointer");
        if (h2[l] < 1 || w2[l] < 1) return bad("sepcorr: lookup: level sizes must be positive");
        if ((double)B * h2[l] * w2[l] * C > 2147483647.0) return bad("sepcorr: a tensor would have 2^31 or more elements");
        a.f2[l] = f2_levels[l]; a.H2[l] = h2[l]; a.W2[l] = w2[l];
    }
    a.B = B; a.H1 = H1; a.W1 = W1; a.C = C; a.L = L; a.r = radius; a.scale = scale;
    const size_t lds = ((size_t)n * n * (TP + 1) + 4 * (size_t)(n + 1) * (n + 1)) * sizeof(float);
    const dim3 grid((W1 + TP - 1) / TP, H1, B * L);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (radius == 4) launch_c<4>(a, grid, lds, s);
    else launch_c<0>(a, grid, lds, s);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: lookup kernel: %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}

}  // extern "C"
