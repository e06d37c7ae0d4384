// Assembly of the module-level volumes from operator-level outputs, fused for gfx950.
// For one operator output src (B,H1,W1,ch,Li) this writes channels [c0, c0+ch) of dst (B,CT,L0,H1,W1):
//   dst[b, c0+c, l0, i, j] = linear interpolation along L (align_corners=True) of src[b,i,j,c,:] at l0
// which is what the caller does per level with permute(0,3,4,1,2), torch.cat over channels,
// F.interpolate(..., [L0,h1,w1], mode='trilinear', align_corners=True) (H1 and W1 keep their size, so the
// trilinear interpolation is linear along L only) and the final torch.cat over levels
// (core/corr.py:428-429, 451-475).  HBM-bound transpose: tiles of 32 pixels go through LDS so that both
// the reads (along l) and the writes (along j) are coalesced.  The backward kernel is the exact adjoint,
// evaluated in gather form (fixed order, no atomics).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

constexpr int TJ = 32;   // pixels (consecutive j of one image row) per workgroup

// Source position of output index l0 (torch's align_corners=True rule, float arithmetic).
__device__ __forceinline__ void src_pos(int l0, float scale, int Li, int &x0, int &x1, float &lam) {
    const float pos = scale * (float)l0;
    x0 = (int)pos;
    if (x0 > Li - 1) x0 = Li - 1;
    x1 = x0 + (x0 < Li - 1 ? 1 : 0);
    lam = pos - (float)x0;
}

struct AsmArgs {
    const float *src;   // forward: (B,H1,W1,ch,Li); backward: grad of dst (B,CT,L0,H1,W1)
    float *dst;         // forward: (B,CT,L0,H1,W1);  backward: grad of src (B,H1,W1,ch,Li)
    int B, H1, W1, ch, Li, CT, c0, L0;
    float scale;        // (Li-1)/(L0-1), 0 when L0 == 1
};

// grid: (ceil(W1/TJ), H1, B*ch); LDS tile [TJ][Li+1]
__global__ void __launch_bounds__(256) assemble_forward_kernel(const AsmArgs a) {
    extern __shared__ float tile[];
    const int Li = a.Li, L0 = a.L0, W1 = a.W1, H1 = a.H1;
    const int LS = Li + 1;
    const int j0 = blockIdx.x * TJ, i = blockIdx.y, c = blockIdx.z % a.ch, b = blockIdx.z / a.ch;
    const int nj = min(TJ, W1 - j0);
    for (int t = threadIdx.x; t < nj * Li; t += blockDim.x) {
        const int jj = t / Li, l = t - jj * Li;
        tile[jj * LS + l] = a.src[((((size_t)b * H1 + i) * W1 + j0 + jj) * a.ch + c) * Li + l];
    }
    __syncthreads();
    float *out = a.dst + (((size_t)b * a.CT + a.c0 + c) * L0) * H1 * W1 + (size_t)i * W1 + j0;
    for (int t = threadIdx.x; t < L0 * TJ; t += blockDim.x) {
        const int l0 = t / TJ, jj = t % TJ;
        if (jj < nj) {
            int x0, x1; float lam;
            src_pos(l0, a.scale, Li, x0, x1, lam);
            out[(size_t)l0 * H1 * W1 + jj] = (1.f - lam) * tile[jj * LS + x0] + lam * tile[jj * LS + x1];
        }
    }
}

// grid as above; LDS tile [L0][TJ+1] of the output gradient
__global__ void __launch_bounds__(256) assemble_backward_kernel(const AsmArgs a) {
    extern __shared__ float tile[];
    const int Li = a.Li, L0 = a.L0, W1 = a.W1, H1 = a.H1;
    constexpr int GS = TJ + 1;
    const int j0 = blockIdx.x * TJ, i = blockIdx.y, c = blockIdx.z % a.ch, b = blockIdx.z / a.ch;
    const int nj = min(TJ, W1 - j0);
    const float *g = a.src + (((size_t)b * a.CT + a.c0 + c) * L0) * H1 * W1 + (size_t)i * W1 + j0;
    for (int t = threadIdx.x; t < L0 * TJ; t += blockDim.x) {
        const int l0 = t / TJ, jj = t % TJ;
        tile[l0 * GS + jj] = jj < nj ? g[(size_t)l0 * H1 * W1 + jj] : 0.f;
    }
    __syncthreads();
    // d_src[l] = sum over l0 of (1-lam)[x0==l] + lam[x1==l, x1!=x0]; candidates around l/scale
    const float inv = a.scale > 0.f ? 1.f / a.scale : 0.f;
    for (int t = threadIdx.x; t < nj * Li; t += blockDim.x) {
        const int jj = t / Li, l = t - jj * Li;
        int lo = 0, hi = L0 - 1;
        if (a.scale > 0.f) {
            lo = max(0, (int)floorf((float)(l - 1) * inv) - 1);
            hi = min(L0 - 1, (int)ceilf((float)(l + 1) * inv) + 1);
        }
        float s = 0.f;
        for (int l0 = lo; l0 <= hi; ++l0) {
            int x0, x1; float lam;
            src_pos(l0, a.scale, Li, x0, x1, lam);
            const float gv = tile[l0 * GS + jj];
            if (x0 == l) s += (1.f - lam) * gv;
            if (x1 == l) s += lam * gv;     // when x1 == x0 the two weights add up to 1, as in the forward
        }
        a.dst[((((size_t)b * H1 + i) * W1 + j0 + jj) * a.ch + c) * Li + l] = s;
    }
}

int bad(const char *msg) { return sepcorr_set_error(SEPCORR_EINVAL, msg); }

int run(bool backward, const float *src, float *dst, int B, int H1, int W1, int ch, int Li, int CT, int c0, int L0, void *stream) {
    if (!src || !dst) return bad("sepcorr: assemble: NULL pointer");
    if (B < 1 || H1 < 1 || W1 < 1 || ch < 1 || Li < 1 || CT < 1 || L0 < 1 || c0 < 0 || c0 + ch > CT)
        return bad("sepcorr: assemble: sizes out of range");
    if ((double)B * CT * L0 * H1 * W1 > 2147483647.0 || (double)B * H1 * W1 * ch * Li > 2147483647.0)
        return bad("sepcorr: a tensor would have 2^31 or more elements");
    if ((long)B * ch > 65535 || H1 > 65535) return bad("sepcorr: assemble: B*ch and H1 must be below 65536");
    const size_t lds = backward ? (size_t)L0 * (TJ + 1) * sizeof(float) : (size_t)TJ * (Li + 1) * sizeof(float);
    if (lds > 64 * 1024) return bad("sepcorr: assemble: displacement axis too long for the LDS tile");
    AsmArgs a = {src, dst, B, H1, W1, ch, Li, CT, c0, L0, L0 > 1 ? (float)(Li - 1) / (float)(L0 - 1) : 0.f};
    const dim3 grid((W1 + TJ - 1) / TJ, H1, B * ch), block(256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (backward) hipLaunchKernelGGL(assemble_backward_kernel, grid, block, lds, s, a);
    else hipLaunchKernelGGL(assemble_forward_kernel, grid, block, lds, s, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: assemble kernel: %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}

}  // namespace

extern "C" {

int sepcorr_assemble_forward(const float *src, float *dst, int B, int H1, int W1, int ch, int Li, int CT, int c0, int L0,
                             void *stream) {
    return run(false, src, dst, B, H1, W1, ch, Li, CT, c0, L0, stream);
}

int sepcorr_assemble_backward(const float *grad_dst, float *grad_src, int B, int H1, int W1, int ch, int Li, int CT, int c0,
                              int L0, void *stream) {
    return run(true, grad_dst, grad_src, B, H1, W1, ch, Li, CT, c0, L0, stream);
}

}  // extern "C"
