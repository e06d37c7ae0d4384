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

constexpr int MAXSRC = 8;   // sources per launch (4 pyramid levels x 2 operator outputs)

struct AsmArgs {
    const float *src[MAXSRC];   // forward: (B,H1,W1,ch,Li) each; backward: unused
    float *gsrc[MAXSRC];        // backward: gradients of the sources, (B,H1,W1,ch,Li) each
    const float *gdst;          // backward: gradient of dst (B,CT,L0,H1,W1)
    float *dst;                 // forward: (B,CT,L0,H1,W1)
    int ch[MAXSRC], Li[MAXSRC], c0[MAXSRC];
    int z0[MAXSRC + 1];         // first blockIdx.z of each source (B*ch[s] blocks each)
    float scale[MAXSRC];        // (Li-1)/(L0-1), 0 when L0 == 1
    int nsrc, B, H1, W1, CT, L0;
    int vl[MAXSRC];             // rows of this source are accessed 16 bytes per lane (Li % 4 == 0, aligned)
    int vj;                     // the volume is accessed 16 bytes per lane (W1 % 4 == 0, aligned)
};

// source that owns blockIdx.z
__device__ __forceinline__ int find_src(const AsmArgs &a) {
    int s = 0;
    while (s + 1 < a.nsrc && (int)blockIdx.z >= a.z0[s + 1]) ++s;
    return s;
}

// Rows of a [rows][n] block dealt to the 4 waves of a workgroup with lanes along the row, VL entries per lane:
// a wave takes 64 / lpr rows at a time, lpr = lanes per row (power of two, at least ceil(n / VL), at most 64).
struct RowLanes {
    int lpr, rpw, row, pos;   // lanes per row, rows per wave and step, this lane's row within the step, its position
};
__device__ __forceinline__ RowLanes row_lanes(int n, int VL) {
    RowLanes r;
    const int need = (n + VL - 1) / VL;
    r.lpr = need <= 1 ? 1 : need >= 33 ? 64 : 1 << (32 - __builtin_clz(need - 1));
    r.rpw = 64 / r.lpr;
    const int lane = threadIdx.x & 63;
    r.row = lane / r.lpr;
    r.pos = lane & (r.lpr - 1);
    return r;
}

// grid: (ceil(W1/TJ), H1, B*ch); LDS tile [TJ][Li+1].  vl: source rows are read 4 entries per lane (Li % 4 == 0,
// aligned); vj: the volume is written 4 pixels per lane (W1 % 4 == 0, aligned).
__global__ void __launch_bounds__(256) assemble_forward_kernel(const AsmArgs a) {
    extern __shared__ float tile[];
    const int sI = find_src(a), z = blockIdx.z - a.z0[sI], nch = a.ch[sI];
    const int Li = a.Li[sI], L0 = a.L0, W1 = a.W1, H1 = a.H1;
    const int LS = Li + 1;
    const int j0 = blockIdx.x * TJ, i = blockIdx.y, c = z % nch, b = z / nch;
    const int nj = min(TJ, W1 - j0);
    const float *src = a.src[sI] + ((((size_t)b * H1 + i) * W1 + j0) * nch + c) * Li;   // pixel jj: + jj * nch * Li
    const float scale = a.scale[sI];
    const int wave = threadIdx.x >> 6;
    {
        const int VL = a.vl[sI] ? 4 : 1;
        const RowLanes rl = row_lanes(Li, VL);
        for (int jj = wave * rl.rpw + rl.row; jj < nj; jj += 4 * rl.rpw) {
            const float *row = src + (size_t)jj * nch * Li;
            float *trow = tile + jj * LS;
            if (VL == 4) {
                for (int l = 4 * rl.pos; l < Li; l += 4 * rl.lpr) {
                    const float4 v = *reinterpret_cast<const float4 *>(row + l);
                    trow[l] = v.x; trow[l + 1] = v.y; trow[l + 2] = v.z; trow[l + 3] = v.w;
                }
            } else {
                for (int l = rl.pos; l < Li; l += rl.lpr) trow[l] = row[l];
            }
        }
    }
    __syncthreads();
    float *out = a.dst + (((size_t)b * a.CT + a.c0[sI] + c) * L0) * H1 * W1 + (size_t)i * W1 + j0;
    if (a.vj) {   // 8 lanes x 4 pixels per output row
        const int q = threadIdx.x & 7;
        if (4 * q < nj)   // (nj is a multiple of 4 here)
            for (int l0 = threadIdx.x >> 3; l0 < L0; l0 += 32) {
                int x0, x1; float lam;
                src_pos(l0, scale, Li, x0, x1, lam);
                const float *t0 = tile + (4 * q) * LS + x0, *t1 = tile + (4 * q) * LS + x1;
                float4 o;
                o.x = (1.f - lam) * t0[0] + lam * t1[0];
                o.y = (1.f - lam) * t0[LS] + lam * t1[LS];
                o.z = (1.f - lam) * t0[2 * LS] + lam * t1[2 * LS];
                o.w = (1.f - lam) * t0[3 * LS] + lam * t1[3 * LS];
                *reinterpret_cast<float4 *>(out + (size_t)l0 * H1 * W1 + 4 * q) = o;
            }
    } else {
        const int jj = threadIdx.x & (TJ - 1);
        if (jj < nj)
            for (int l0 = threadIdx.x / TJ; l0 < L0; l0 += 256 / TJ) {
                int x0, x1; float lam;
                src_pos(l0, scale, Li, x0, x1, lam);
                out[(size_t)l0 * H1 * W1 + jj] = (1.f - lam) * tile[jj * LS + x0] + lam * tile[jj * LS + x1];
            }
    }
}

// d_src[l] of one pixel from the column of the gradient tile under it: sum over l0 of (1-lam)[x0==l] + lam[x1==l];
// candidates around l / scale.
__device__ __forceinline__ float gather_adjoint(const float *col, int GS, int l, int Li, int L0, float scale, float inv) {
    if (Li == L0) return col[l * GS];   // the finest level: the interpolation is the identity (scale 1, every weight 1 or 0)
    int lo = 0, hi = L0 - 1;
    if (scale > 0.f) {
        lo = max(0, (int)floorf((float)(l - 1) * inv) - 1);
        hi = min(L0 - 1, (int)ceilf((float)(l + 1) * inv) + 1);
    }
    float s = 0.f;
    for (int l0 = lo; l0 <= hi; ++l0) {
        int x0, x1; float lam;
        src_pos(l0, scale, Li, x0, x1, lam);
        const float gv = col[l0 * GS];
        if (x0 == l) s += (1.f - lam) * gv;
        if (x1 == l) s += lam * gv;     // when x1 == x0 the two weights add up to 1, as in the forward
    }
    return s;
}

// grid as above; LDS tile [L0][TJ+1] of the output gradient
__global__ void __launch_bounds__(256) assemble_backward_kernel(const AsmArgs a) {
    extern __shared__ float tile[];
    const int sI = find_src(a), z = blockIdx.z - a.z0[sI], nch = a.ch[sI];
    const int Li = a.Li[sI], L0 = a.L0, W1 = a.W1, H1 = a.H1;
    constexpr int GS = TJ + 1;
    const int j0 = blockIdx.x * TJ, i = blockIdx.y, c = z % nch, b = z / nch;
    const int nj = min(TJ, W1 - j0);
    const float scale = a.scale[sI];
    const float *g = a.gdst + (((size_t)b * a.CT + a.c0[sI] + c) * L0) * H1 * W1 + (size_t)i * W1 + j0;
    if (a.vj) {
        const int q = threadIdx.x & 7;
        for (int l0 = threadIdx.x >> 3; l0 < L0; l0 += 32) {
            const float4 v = 4 * q < nj ? *reinterpret_cast<const float4 *>(g + (size_t)l0 * H1 * W1 + 4 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
            float *t = tile + l0 * GS + 4 * q;
            t[0] = v.x; t[1] = v.y; t[2] = v.z; t[3] = v.w;
        }
    } else {
        const int jj = threadIdx.x & (TJ - 1);
        for (int l0 = threadIdx.x / TJ; l0 < L0; l0 += 256 / TJ) tile[l0 * GS + jj] = jj < nj ? g[(size_t)l0 * H1 * W1 + jj] : 0.f;
    }
    __syncthreads();
    const float inv = scale > 0.f ? 1.f / scale : 0.f;
    float *gsrc = a.gsrc[sI] + ((((size_t)b * H1 + i) * W1 + j0) * nch + c) * Li;
    const int wave = threadIdx.x >> 6;
    const int VL = a.vl[sI] ? 4 : 1;
    const RowLanes rl = row_lanes(Li, VL);
    for (int jj = wave * rl.rpw + rl.row; jj < nj; jj += 4 * rl.rpw) {
        float *row = gsrc + (size_t)jj * nch * Li;
        const float *col = tile + jj;
        if (VL == 4) {
            for (int l = 4 * rl.pos; l < Li; l += 4 * rl.lpr) {
                float4 o;
                o.x = gather_adjoint(col, GS, l, Li, L0, scale, inv);
                o.y = gather_adjoint(col, GS, l + 1, Li, L0, scale, inv);
                o.z = gather_adjoint(col, GS, l + 2, Li, L0, scale, inv);
                o.w = gather_adjoint(col, GS, l + 3, Li, L0, scale, inv);
                *reinterpret_cast<float4 *>(row + l) = o;
            }
        } else {
            for (int l = rl.pos; l < Li; l += rl.lpr) row[l] = gather_adjoint(col, GS, l, Li, L0, scale, inv);
        }
    }
}

int bad(const char *msg) { return sepcorr_set_error(SEPCORR_EINVAL, msg); }

// One launch for up to MAXSRC sources that share dst (forward) or grad_dst (backward); channel offsets follow the
// order of the sources, starting at c0.
int run(bool backward, const float *const *srcs, float *const *gsrcs, const float *gdst, float *dst, const int *ch,
        const int *Li, int nsrc, int B, int H1, int W1, int CT, int c0, int L0, void *stream) {
    if (nsrc < 1 || nsrc > MAXSRC) return bad("sepcorr: assemble: 1 to 8 sources per call");
    if ((backward ? (const void *)gdst : (const void *)dst) == nullptr || !ch || !Li) return bad("sepcorr: assemble: NULL pointer");
    if (B < 1 || H1 < 1 || W1 < 1 || CT < 1 || L0 < 1 || c0 < 0) return bad("sepcorr: assemble: sizes out of range");
    if ((double)B * CT * L0 * H1 * W1 > 2147483647.0) return bad("sepcorr: a tensor would have 2^31 or more elements");
    if (H1 > 65535) return bad("sepcorr: assemble: B*ch and H1 must be below 65536");
    AsmArgs a = {};
    a.gdst = gdst; a.dst = dst; a.nsrc = nsrc; a.B = B; a.H1 = H1; a.W1 = W1; a.CT = CT; a.L0 = L0;
    size_t lds = 0;
    long z = 0;
    int c = c0;
    for (int s = 0; s < nsrc; ++s) {
        if (!(backward ? (const void *)gsrcs[s] : (const void *)srcs[s])) return bad("sepcorr: assemble: NULL pointer");
        if (ch[s] < 1 || Li[s] < 1 || c + ch[s] > CT) return bad("sepcorr: assemble: sizes out of range");
        if ((double)B * H1 * W1 * ch[s] * Li[s] > 2147483647.0) return bad("sepcorr: a tensor would have 2^31 or more elements");
        if (backward) a.gsrc[s] = gsrcs[s]; else a.src[s] = srcs[s];
        a.ch[s] = ch[s]; a.Li[s] = Li[s]; a.c0[s] = c;
        a.vl[s] = Li[s] % 4 == 0 && (reinterpret_cast<uintptr_t>(backward ? (const void *)gsrcs[s] : (const void *)srcs[s]) & 15) == 0;
        a.scale[s] = L0 > 1 ? (float)(Li[s] - 1) / (float)(L0 - 1) : 0.f;
        a.z0[s] = (int)z;
        z += (long)B * ch[s];
        c += ch[s];
        const size_t need = backward ? (size_t)L0 * (TJ + 1) * sizeof(float) : (size_t)TJ * (Li[s] + 1) * sizeof(float);
        lds = need > lds ? need : lds;
    }
    a.z0[nsrc] = (int)z;
    a.vj = W1 % 4 == 0 && (reinterpret_cast<uintptr_t>(backward ? (const void *)gdst : (const void *)dst) & 15) == 0;
    if (z > 65535) return bad("sepcorr: assemble: B*ch and H1 must be below 65536");
    if (lds > 64 * 1024) return bad("sepcorr: assemble: displacement axis too long for the LDS tile");
    const dim3 grid((W1 + TJ - 1) / TJ, H1, (unsigned)z), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (backward) hipLaunchKernelGGL(assemble_backward_kernel, grid, block, lds, st, a);
    else hipLaunchKernelGGL(assemble_forward_kernel, grid, block, lds, st, a);
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
    if (!src) return bad("sepcorr: assemble: NULL pointer");
    return run(false, &src, nullptr, nullptr, dst, &ch, &Li, 1, B, H1, W1, CT, c0, L0, stream);
}

int sepcorr_assemble_backward(const float *grad_dst, float *grad_src, int B, int H1, int W1, int ch, int Li, int CT, int c0,
                              int L0, void *stream) {
    if (!grad_src) return bad("sepcorr: assemble: NULL pointer");
    return run(true, nullptr, &grad_src, grad_dst, nullptr, &ch, &Li, 1, B, H1, W1, CT, c0, L0, stream);
}

int sepcorr_assemble_forward_multi(const float *const *srcs, const int *ch, const int *Li, int nsrc, float *dst, int B,
                                   int H1, int W1, int CT, int L0, void *stream) {
    if (!srcs) return bad("sepcorr: assemble: NULL pointer");
    return run(false, srcs, nullptr, nullptr, dst, ch, Li, nsrc, B, H1, W1, CT, 0, L0, stream);
}

int sepcorr_assemble_backward_multi(const float *grad_dst, float *const *grad_srcs, const int *ch, const int *Li, int nsrc,
                                    int B, int H1, int W1, int CT, int L0, void *stream) {
    if (!grad_srcs) return bad("sepcorr: assemble: NULL pointer");
    return run(true, nullptr, grad_srcs, grad_dst, nullptr, ch, Li, nsrc, B, H1, W1, CT, 0, L0, stream);
}

}  // extern "C"
