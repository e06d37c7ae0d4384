// Lookup in one separated 3D correlation volume: the consumer of the volumes that separate() produces (gfx950).
//
// What the reference's CorrBlock1D does for one of its two volumes (core/corr.py:513-624): the volume
// corr (B,dim,L,H1,W1) is pooled by two along the displacement axis L into a pyramid (avg_pool2d [1,2],
// core/corr.py:546-550) and every level l is sampled linearly (grid_sample on a one-row image, align_corners=True,
// zero padding) at x/2^l + k - r, k = 0..2r, where x = coords[b, coord_channel, i, j]:
//   out[b, l*dim*n + d*n + k, i, j],  n = 2r+1.
// For its first volume the reference clamps the sampling positions to [-1, 1] before sampling
// (core/corr.py:593); `clamp_unit` reproduces that.
//
// The pyramid is not stored: entry m of level l is the mean of level-0 entries [m*2^l, (m+1)*2^l).  One thread per (b, d, i, j): neighbouring threads are
// neighbouring image-1 pixels, whose reads of corr[b,d,w,i,j] sit side by side whenever their w agree (smooth flow).
// HBM/L2-bound gather, no matrix work.  The backward pass is its exact adjoint in gather form: one thread per entry
// of d_corr collects what the samples around it passed on, so there are no atomics and the order of the sums is fixed.
#include <hip/hip_runtime.h>
#include <climits>
#include <cstdint>
#include <cstdio>
#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

struct L1dArgs {
    const float *corr;      // forward: (B,dim,L,H1,W1)
    const float *coords;    // (B,2,H1,W1)
    const float *gout;      // backward: (B, levels*dim*n, H1, W1)
    float *out;             // forward: (B, levels*dim*n, H1, W1); backward: d_corr (B,dim,L,H1,W1)
    int B, dim, L, H1, W1, coord_channel, clamp_unit, levels, r;
};

// entry m of level l: the mean of the 2^l level-0 entries under it (the chain of pair means, summed in one go;
// the scaling by 2^-l is exact)
__device__ __forceinline__ float pooled_any(const float *col, size_t plane, int m, int l) {
    const int base = m << l;
    float s = 0.f;
    for (int t = 0; t < (1 << l); ++t) s += col[(size_t)(base + t) * plane];
    return s / (float)(1 << l);
}

__device__ __forceinline__ void sample_pos(float x, int k, int r, bool clamp_unit, int &p0, float &f) {
    float pos = x + (float)(k - r);
    if (clamp_unit) pos = fminf(fmaxf(pos, -1.f), 1.f);
    const float fl = floorf(pos);
    f = pos - fl;
    p0 = (int)fminf(fmaxf(fl, -1048576.f), 1048576.f);
    if (!(f >= 0.f && f <= 1.f)) f = pos - pos;     // NaN for infinite positions, as in the sampler
}

// grid.x covers (b, d, pixel), grid.y = pyramid level
__global__ void __launch_bounds__(256) lookup1d_forward_kernel(const L1dArgs a) {
    const size_t plane = (size_t)a.H1 * a.W1;
    const size_t total = (size_t)a.B * a.dim * plane;
    const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const size_t pix = e % plane;
    const int d = (int)((e / plane) % a.dim), b = (int)(e / (plane * a.dim));
    const int n = 2 * a.r + 1, l = blockIdx.y, Ll = a.L >> l;
    const float xl = a.coords[((size_t)b * 2 + a.coord_channel) * plane + pix] / (float)(1 << l);
    const float *col = a.corr + ((size_t)b * a.dim + d) * a.L * plane + pix;
    float *o = a.out + ((size_t)b * a.levels * a.dim + (size_t)l * a.dim + d) * n * plane + pix;
    // neighbouring samples share an entry (the right one of sample k is the left one of k+1 unless the positions
    // were clamped): it is formed once
    int have = INT_MIN;
    float hv = 0.f;
    for (int k = 0; k < n; ++k) {
        int p0;
        float f;
        sample_pos(xl, k, a.r, a.clamp_unit != 0, p0, f);
        float v0 = 0.f, v1 = 0.f;
        if (p0 >= 0 && p0 < Ll) v0 = p0 == have ? hv : pooled_any(col, plane, p0, l);
        if (p0 + 1 >= 0 && p0 + 1 < Ll) v1 = pooled_any(col, plane, p0 + 1, l);
        have = p0 + 1;
        hv = v1;
        o[(size_t)k * plane] = fmaf(f, v1, (1.f - f) * v0);
    }
}

// adds g / 2^l to the 2^l level-0 entries under entry m of level l
__device__ __forceinline__ void spread(float *col, size_t plane, int m, int l, float g) {
    const float gs = g / (float)(1 << l);
    const int base = m << l;
    for (int t = 0; t < (1 << l); ++t) col[(size_t)(base + t) * plane] += gs;
}

// Adjoint in scatter form: one thread per column (b, d, pixel), which it alone reads and writes (no atomics).  Fewer
// position computations per entry than the gather form below; needs enough columns to fill the chip.
__global__ void __launch_bounds__(256) lookup1d_backward_columns_kernel(const L1dArgs a) {
    const size_t plane = (size_t)a.H1 * a.W1;
    const size_t total = (size_t)a.B * a.dim * plane;
    const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const size_t pix = e % plane;
    const int d = (int)((e / plane) % a.dim), b = (int)(e / (plane * a.dim));
    const int n = 2 * a.r + 1;
    const float x = a.coords[((size_t)b * 2 + a.coord_channel) * plane + pix];
    float *col = a.out + ((size_t)b * a.dim + d) * a.L * plane + pix;      // this thread's own column of d_corr
    for (int w = 0; w < a.L; ++w) col[(size_t)w * plane] = 0.f;
    const float *g = a.gout + (size_t)b * a.levels * a.dim * n * plane + pix;
    int Ll = a.L;
    for (int l = 0; l < a.levels; ++l) {
        const float xl = x / (float)(1 << l);
        for (int k = 0; k < n; ++k) {
            int p0;
            float f;
            sample_pos(xl, k, a.r, a.clamp_unit != 0, p0, f);
            const float gv = g[((size_t)(l * a.dim + d) * n + k) * plane];
            if (p0 >= 0 && p0 < Ll) spread(col, plane, p0, l, (1.f - f) * gv);
            if (p0 + 1 >= 0 && p0 + 1 < Ll) spread(col, plane, p0 + 1, l, f * gv);
        }
        Ll >>= 1;
    }
}

// Adjoint in gather form: one thread per entry (b, d, w, pixel) of d_corr.  Entry w lies under entry m = w >> l of
// level l (if that level has one), which sample k reads with weight (1-f) when it is its left entry and f when it is
// its right one; each level passes 2^-l of that on.  Without the clamp only the two samples around m can read it.
__global__ void __launch_bounds__(256) lookup1d_backward_kernel(const L1dArgs a) {
    // grid: x = pixels, y = entry w, z = (b, d)
    const size_t plane = (size_t)a.H1 * a.W1;
    const size_t pix = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (pix >= plane) return;
    const int w = blockIdx.y, d = blockIdx.z % a.dim, b = blockIdx.z / a.dim;
    const size_t e = (((size_t)b * a.dim + d) * a.L + w) * plane + pix;
    const int n = 2 * a.r + 1;
    const float x = a.coords[((size_t)b * 2 + a.coord_channel) * plane + pix];
    const float *g = a.gout + (size_t)b * a.levels * a.dim * n * plane + pix;
    float sum = 0.f;
    for (int l = 0; l < a.levels; ++l) {
        const int Ll = a.L >> l, m = w >> l;
        if (m >= Ll) break;                                  // dropped by the pooling (odd length); so at coarser levels
        const float xl = x / (float)(1 << l);
        int k0 = 0, k1 = n - 1;
        if (a.clamp_unit) {
            if (m > 1) continue;                             // clamped positions read entries -1..1 only
        } else {
            const float fl = fminf(fmaxf(floorf(xl), -1048576.f), 1048576.f);
            const int base = (int)fl - a.r;                  // left entry of sample k is base + k, give or take the
            k0 = max(0, m - 2 - base);                       // rounding of x + (k - r): one more sample on each side
            k1 = min(n - 1, m + 1 - base);
        }
        float s = 0.f;
        for (int k = k0; k <= k1; ++k) {
            int p0;
            float f;
            sample_pos(xl, k, a.r, a.clamp_unit != 0, p0, f);
            if (p0 != m && p0 + 1 != m) continue;
            const float gv = g[((size_t)(l * a.dim + d) * n + k) * plane];
            s += p0 == m ? (1.f - f) * gv : f * gv;
        }
        sum += s / (float)(1 << l);
    }
    a.out[e] = sum;
}

int bad(const char *msg) { return sepcorr_set_error(SEPCORR_EINVAL, msg); }

int run(bool backward, const float *corr, const float *coords, const float *gout, float *out, int B, int dim, int L,
        int H1, int W1, int coord_channel, int clamp_unit, int levels, int radius, void *stream) {
    if ((!backward && !corr) || !coords || !out || (backward && !gout)) return bad("sepcorr: lookup1d: NULL pointer");
    if (B < 1 || dim < 1 || L < 1 || H1 < 1 || W1 < 1) return bad("sepcorr: lookup1d: sizes must be positive");
    if (coord_channel < 0 || coord_channel > 1) return bad("sepcorr: lookup1d: coord_channel must be 0 or 1");
    if (levels < 1 || levels > 8) return bad("sepcorr: lookup1d: 1 to 8 pyramid levels are supported");
    if (radius < 1 || radius > 16) return bad("sepcorr: lookup1d: radius must be 1..16");
    if ((L >> (levels - 1)) < 1) return bad("sepcorr: lookup1d: the displacement axis is too short for that many levels");
    const int n = 2 * radius + 1;
    if ((double)B * dim * L * H1 * W1 > 2147483647.0 || (double)B * levels * dim * n * H1 * W1 > 2147483647.0)
        return bad("sepcorr: a tensor would have 2^31 or more elements");
    L1dArgs a = {corr, coords, gout, out, B, dim, L, H1, W1, coord_channel, clamp_unit, levels, radius};
    const size_t total = (size_t)B * dim * H1 * W1;
    const dim3 block(256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (backward) {
        // columns as units fill the chip from about four waves per SIMD on (measured at 55x128: 1 channel 0.10 ms by
        // columns, 0.026 ms by entries; 24 channels 0.25 against 0.38 ms)
        const bool fits_grid = L <= 65535 && (long)B * dim <= 65535;
        const bool by_entries = fits_grid && total < (size_t)256 * 1024;
        if (by_entries)
            hipLaunchKernelGGL(lookup1d_backward_kernel, dim3((unsigned)(((size_t)H1 * W1 + 255) / 256), L, B * dim), block, 0, s, a);
        else
            hipLaunchKernelGGL(lookup1d_backward_columns_kernel, dim3((unsigned)((total + 255) / 256)), block, 0, s, a);
    }
    else hipLaunchKernelGGL(lookup1d_forward_kernel, dim3((unsigned)((total + 255) / 256), levels), block, 0, s, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: lookup1d kernel: %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}

}  // namespace

extern "C" {

int sepcorr_lookup1d_forward(const float *corr, const float *coords, float *out, int B, int dim, int L, int H1, int W1,
                             int coord_channel, int clamp_unit, int levels, int radius, void *stream) {
    return run(false, corr, coords, nullptr, out, B, dim, L, H1, W1, coord_channel, clamp_unit, levels, radius, stream);
}

int sepcorr_lookup1d_backward(const float *coords, const float *grad_out, float *d_corr, int B, int dim, int L, int H1,
                              int W1, int coord_channel, int clamp_unit, int levels, int radius, void *stream) {
    return run(true, nullptr, coords, grad_out, d_corr, B, dim, L, H1, W1, coord_channel, clamp_unit, levels, radius, stream);
}

}  // extern "C"
