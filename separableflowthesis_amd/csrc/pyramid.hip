// The caller's preparation of the feature maps, fused for gfx950.  AlternateCorrBlockSepflow holds fmap1 and fmap2 as
// (B,C,H,W), builds the image-2 pyramid with F.avg_pool2d(fmap2, 2, stride=2) level after level
// (core/corr.py:376-382) and hands every level to the operator as permute(0,2,3,1).contiguous(), fmap1 also divided
// by sqrt(C) (core/corr.py:419-422).  Here one pass reads a feature map in (B,C,H,W) and writes all of that in the
// operator's (B,H,W,C) layout: level 0 and the pooled levels from the same LDS tile.  The backward pass is the
// adjoint: the gradients of all levels, in (B,H_l,W_l,C), folded into one gradient in (B,C,H,W).
// HBM-bound: every byte is read once and written once; tiles go through LDS so that reads (along W in the source,
// along C in the destination) and writes are both whole cache lines.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

constexpr int TY = 8, TX = 32, TC = 32;   // tile: 8 rows x 32 columns of level 0 (one 8 x 8 block per level-3 pixel) x 32 channels
constexpr int CS = TC + 1;                // channel stride in LDS (odd: column-wise reads hit distinct banks)
constexpr int MAXLEV = 4;

struct PyrArgs {
    const float *src;            // forward: (B,C,H,W); backward: unused
    float *dst;                  // backward: gradient in (B,C,H,W); forward: unused
    float *lev[MAXLEV];          // forward: level l in (B,H>>l,W>>l,C)
    const float *glev[MAXLEV];   // backward: gradient of level l
    int B, C, H, W, nlev;
    float divisor;               // level 0 is divided by this (sqrt(C) for fmap1, 1 for fmap2)
};

__device__ __forceinline__ int lds_at(int l, int y, int x) {
    // levels one after the other: [y][x][CS] each, level l has (TY >> l) x (TX >> l) pixels
    int base = 0;
    for (int k = 0; k < l; ++k) base += (TY >> k) * (TX >> k);
    return (base + y * (TX >> l) + x) * CS;
}
constexpr int LDS_PIXELS = TY * TX + (TY / 2) * (TX / 2) + (TY / 4) * (TX / 4) + (TY / 8) * (TX / 8);

typedef float v4f __attribute__((ext_vector_type(4)));

// grid: (ceil(W/TX), ceil(H/TY), B * ceil(C/TC)), 256 threads.  VEC: W and C are multiples of 4 and all pointers are
// 16-byte aligned: 16-byte accesses on both sides, all loads of a thread in flight before its first LDS write.
template <bool VEC>
__global__ void __launch_bounds__(256) pyramid_forward_kernel(const PyrArgs a) {
    __shared__ float t[LDS_PIXELS * CS];
    const int ncb = (a.C + TC - 1) / TC;
    const int b = blockIdx.z / ncb, c0 = (blockIdx.z % ncb) * TC;
    const int y0 = blockIdx.y * TY, x0 = blockIdx.x * TX;
    const int H = a.H, W = a.W, C = a.C;
    const float inv = 1.f / a.divisor;
    // read: for a channel and a row, TX consecutive floats of the source
    if constexpr (VEC) {
        constexpr int N = TC * TY * (TX / 4) / 256;
        v4f v[N];
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int i = threadIdx.x + 256 * k;
            const int x4 = i % (TX / 4), y = (i / (TX / 4)) % TY, c = i / ((TX / 4) * TY);
            v[k] = v4f{0.f, 0.f, 0.f, 0.f};
            if (c0 + c < C && y0 + y < H && x0 + 4 * x4 < W)
                v[k] = *reinterpret_cast<const v4f *>(a.src + (((size_t)b * C + c0 + c) * H + y0 + y) * W + x0 + 4 * x4);
        }
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const int i = threadIdx.x + 256 * k;
            const int x4 = i % (TX / 4), y = (i / (TX / 4)) % TY, c = i / ((TX / 4) * TY);
#pragma unroll
            for (int e = 0; e < 4; ++e) t[lds_at(0, y, 4 * x4 + e) + c] = v[k][e];
        }
    } else {
        for (int i = threadIdx.x; i < TC * TY * TX; i += blockDim.x) {
            const int x = i % TX, y = (i / TX) % TY, c = i / (TX * TY);
            float v = 0.f;
            if (c0 + c < C && y0 + y < H && x0 + x < W) v = a.src[(((size_t)b * C + c0 + c) * H + y0 + y) * W + x0 + x];
            t[lds_at(0, y, x) + c] = v;
        }
    }
    __syncthreads();
    // pooled levels, each from the one below: the four values are added row by row, left to right, and the sum is
    // divided by 4, the order of torch's avg_pool2d
    for (int l = 1; l < a.nlev; ++l) {
        const int ny = TY >> l, nx = TX >> l;
        for (int i = threadIdx.x; i < ny * nx * TC; i += blockDim.x) {
            const int c = i % TC, x = (i / TC) % nx, y = i / (TC * nx);
            const float s = ((t[lds_at(l - 1, 2 * y, 2 * x) + c] + t[lds_at(l - 1, 2 * y, 2 * x + 1) + c]) +
                             t[lds_at(l - 1, 2 * y + 1, 2 * x) + c]) + t[lds_at(l - 1, 2 * y + 1, 2 * x + 1) + c];
            t[lds_at(l, y, x) + c] = s / 4.f;
        }
        __syncthreads();
    }
    // write: for a pixel, TC consecutive channels; a pooled pixel exists where all its sources do (sizes round down)
    for (int l = 0; l < a.nlev; ++l) {
        const int ny = TY >> l, nx = TX >> l, Hl = H >> l, Wl = W >> l;
        const int yl0 = y0 >> l, xl0 = x0 >> l;
        if constexpr (VEC) {
            for (int i = threadIdx.x; i < ny * nx * (TC / 4); i += blockDim.x) {
                const int c4 = i % (TC / 4), x = (i / (TC / 4)) % nx, y = i / ((TC / 4) * nx);
                if (c0 + 4 * c4 < C && yl0 + y < Hl && xl0 + x < Wl) {
                    const float *p = t + lds_at(l, y, x) + 4 * c4;
                    v4f v = {p[0], p[1], p[2], p[3]};
                    if (l == 0) v = v * inv;
                    *reinterpret_cast<v4f *>(a.lev[l] + (((size_t)b * Hl + yl0 + y) * Wl + xl0 + x) * C + c0 + 4 * c4) = v;
                }
            }
            continue;
        }
        for (int i = threadIdx.x; i < ny * nx * TC; i += blockDim.x) {
            const int c = i % TC, x = (i / TC) % nx, y = i / (TC * nx);
            if (c0 + c < C && yl0 + y < Hl && xl0 + x < Wl) {
                float v = t[lds_at(l, y, x) + c];
                if (l == 0) v = v * inv;   // (torch divides by a host scalar by multiplying with its reciprocal)
                a.lev[l][(((size_t)b * Hl + yl0 + y) * Wl + xl0 + x) * C + c0 + c] = v;
            }
        }
    }
}

template <bool VEC>
__global__ void __launch_bounds__(256) pyramid_backward_kernel(const PyrArgs a) {
    __shared__ float t[LDS_PIXELS * CS];
    const int ncb = (a.C + TC - 1) / TC;
    const int b = blockIdx.z / ncb, c0 = (blockIdx.z % ncb) * TC;
    const int y0 = blockIdx.y * TY, x0 = blockIdx.x * TX;
    const int H = a.H, W = a.W, C = a.C;
    const float inv = 1.f / a.divisor;
    for (int l = 0; l < a.nlev; ++l) {
        const int ny = TY >> l, nx = TX >> l, Hl = H >> l, Wl = W >> l;
        const int yl0 = y0 >> l, xl0 = x0 >> l;
        if constexpr (VEC) {
            for (int i = threadIdx.x; i < ny * nx * (TC / 4); i += blockDim.x) {
                const int c4 = i % (TC / 4), x = (i / (TC / 4)) % nx, y = i / ((TC / 4) * nx);
                v4f v = {0.f, 0.f, 0.f, 0.f};
                if (c0 + 4 * c4 < C && yl0 + y < Hl && xl0 + x < Wl)
                    v = *reinterpret_cast<const v4f *>(a.glev[l] + (((size_t)b * Hl + yl0 + y) * Wl + xl0 + x) * C + c0 + 4 * c4);
                if (l == 0) v = v * inv;
                float *p = t + lds_at(l, y, x) + 4 * c4;
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e] = v[e];
            }
            continue;
        }
        for (int i = threadIdx.x; i < ny * nx * TC; i += blockDim.x) {
            const int c = i % TC, x = (i / TC) % nx, y = i / (TC * nx);
            float v = 0.f;
            if (c0 + c < C && yl0 + y < Hl && xl0 + x < Wl)
                v = a.glev[l][(((size_t)b * Hl + yl0 + y) * Wl + xl0 + x) * C + c0 + c];
            if (l == 0) v = v * inv;
            t[lds_at(l, y, x) + c] = v;
        }
    }
    __syncthreads();
    // from the coarsest level down: a pixel's gradient is its own plus a quarter of its parent's
    // (what autograd does through the chain of avg_pool2d calls)
    for (int l = a.nlev - 2; l >= 0; --l) {
        const int ny = TY >> l, nx = TX >> l;
        for (int i = threadIdx.x; i < ny * nx * TC; i += blockDim.x) {
            const int c = i % TC, x = (i / TC) % nx, y = i / (TC * nx);
            t[lds_at(l, y, x) + c] += t[lds_at(l + 1, y >> 1, x >> 1) + c] / 4.f;
        }
        __syncthreads();
    }
    if constexpr (VEC) {
        for (int i = threadIdx.x; i < TC * TY * (TX / 4); i += blockDim.x) {
            const int x4 = i % (TX / 4), y = (i / (TX / 4)) % TY, c = i / ((TX / 4) * TY);
            if (c0 + c < C && y0 + y < H && x0 + 4 * x4 < W) {
                v4f v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = t[lds_at(0, y, 4 * x4 + e) + c];
                *reinterpret_cast<v4f *>(a.dst + (((size_t)b * C + c0 + c) * H + y0 + y) * W + x0 + 4 * x4) = v;
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < TC * TY * TX; i += blockDim.x) {
        const int x = i % TX, y = (i / TX) % TY, c = i / (TX * TY);
        if (c0 + c < C && y0 + y < H && x0 + x < W)
            a.dst[(((size_t)b * C + c0 + c) * H + y0 + y) * W + x0 + x] = t[lds_at(0, y, x) + c];
    }
}

int bad(const char *msg) { return sepcorr_set_error(SEPCORR_EINVAL, msg); }

int run(bool backward, PyrArgs a, void *stream) {
    if (a.B < 1 || a.C < 1 || a.H < 1 || a.W < 1) return bad("sepcorr: feature pyramid: sizes must be positive");
    if (a.nlev < 1 || a.nlev > MAXLEV) return bad("sepcorr: feature pyramid: 1 to 4 levels");
    if ((a.H >> (a.nlev - 1)) < 1 || (a.W >> (a.nlev - 1)) < 1) return bad("sepcorr: feature pyramid: the coarsest level would be empty");
    if ((size_t)a.B * a.C * a.H * a.W >= ((size_t)1 << 31)) return bad("sepcorr: feature pyramid: tensor too large");
    const long nz = (long)a.B * ((a.C + TC - 1) / TC);
    if (nz > 65535) return bad("sepcorr: feature pyramid: B * C / 32 must stay below 65536");
    const dim3 grid((a.W + TX - 1) / TX, (a.H + TY - 1) / TY, (unsigned)nz);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uintptr_t align = reinterpret_cast<uintptr_t>(a.src) | reinterpret_cast<uintptr_t>(a.dst);
    for (int l = 0; l < a.nlev; ++l) align |= reinterpret_cast<uintptr_t>(a.lev[l]) | reinterpret_cast<uintptr_t>(a.glev[l]);
    const bool vec = a.W % 4 == 0 && a.C % 4 == 0 && align % 16 == 0;
    if (backward) {
        if (vec) hipLaunchKernelGGL(pyramid_backward_kernel<true>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(pyramid_backward_kernel<false>, grid, dim3(256), 0, s, a);
    } else {
        if (vec) hipLaunchKernelGGL(pyramid_forward_kernel<true>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(pyramid_forward_kernel<false>, grid, dim3(256), 0, s, a);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: feature pyramid launch failed: %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}

}  // namespace

extern "C" {

int sepcorr_feature_pyramid_forward(const float *fmap, float *const *levels, int B, int C, int H, int W, int nlev,
                                    float divisor, void *stream) {
    if (!fmap || !levels) return bad("sepcorr: feature pyramid: NULL pointer");
    if (!(divisor > 0.f)) return bad("sepcorr: feature pyramid: divisor must be positive");
    PyrArgs a = {};
    a.src = fmap;
    for (int l = 0; l < nlev && l < MAXLEV; ++l) {
        if (!levels[l]) return bad("sepcorr: feature pyramid: NULL level pointer");
        a.lev[l] = levels[l];
    }
    a.B = B; a.C = C; a.H = H; a.W = W; a.nlev = nlev; a.divisor = divisor;
    return run(false, a, stream);
}

int sepcorr_feature_pyramid_backward(const float *const *grad_levels, float *grad_fmap, int B, int C, int H, int W, int nlev,
                                     float divisor, void *stream) {
    if (!grad_fmap || !grad_levels) return bad("sepcorr: feature pyramid: NULL pointer");
    if (!(divisor > 0.f)) return bad("sepcorr: feature pyramid: divisor must be positive");
    PyrArgs a = {};
    a.dst = grad_fmap;
    for (int l = 0; l < nlev && l < MAXLEV; ++l) {
        if (!grad_levels[l]) return bad("sepcorr: feature pyramid: NULL level pointer");
        a.glev[l] = grad_levels[l];
    }
    a.B = B; a.C = C; a.H = H; a.W = W; a.nlev = nlev; a.divisor = divisor;
    return run(true, a, stream);
}

}  // extern "C"
