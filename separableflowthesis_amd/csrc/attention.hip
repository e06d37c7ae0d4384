// Attention-weight producer of the separated correlation volumes, fused for gfx950:
//   a = softmax_L( Conv3d(2 -> K, kernel 3, padding 1)(sep) )
// taken and returned in the operator's own layout, sep (B,H1,W1,2,L) -> a (B,H1,W1,K,L), so the
// permutes around it disappear.  In the reference this is attention1(sep_u) / attention2(sep_v), a
// torch Conv3d over the volume (B,2,L,H1,W1), followed by softmax(dim=2) and permute(0,3,4,1,2)
// (core/sepflow.py:59-60, core/corr.py:437-446).  The convolution's depth axis is L, its height and
// width are H1 and W1: weight[k][c][dl][di][dj].
//
// Vector-instruction work (54 K multiply-adds per output) with lanes along L (rows of L contiguous floats: every
// access is coalesced), softmax statistics by wave reduction.  Rows of up to 256 entries run on the strip kernels: a
// group of lanes takes a few neighbouring pixels, fetches the rows under them once and gets the neighbours along L
// from the lanes beside it; anything else (longer rows, rows that are no multiple of the vector width they would
// need, unaligned tensors) runs one wave per pixel.
// The backward pass is three kernels: softmax backward -> dlogits (scratch), the transposed
// convolution for d_sep, and the weight gradient as per-workgroup partial sums that a last kernel
// adds in a fixed order (deterministic, no atomics).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

constexpr int MAXK = 8;
constexpr int WPB = 4;          // waves (pixels) per workgroup
constexpr int DW_PIX = 64;      // pixels per workgroup in the weight-gradient kernel

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}
// The same over aligned groups of `lw` lanes (16, 32 or 64): short rows put several pixels into one wave.
__device__ __forceinline__ float group_max(float x, int lw) {
    for (int o = lw >> 1; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ float group_sum(float x, int lw) {
    for (int o = lw >> 1; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}
// lanes per pixel for rows of L entries
__host__ __device__ inline int lanes_per_pixel(int L) { return L <= 16 ? 16 : L <= 32 ? 32 : 64; }

struct AttArgs {
    const float *sep, *weight, *bias, *a, *grad_a;
    float *out;        // forward: a; softmax backward: dlogits; conv backward: d_sep
    float *dlogits;    // scratch (B,H1,W1,K,L)
    float *partial;    // scratch [nwg][K*54 + K]
    int B, H1, W1, L, K;
    float *stats;      // forward, optional: (max, sum of exp) of every row of logits, (B,H1,W1,K,2)
    int logits_only;   // forward: store the logits themselves instead of their softmax
    const float *init; // conv backward, optional: added to d_sep (a gradient that reaches sep by another path)
};

// Up to MAXJOBS calls of the same kind (the pyramid levels of one attention module) in one launch: workgroups
// [first[j], first[j + 1]) of the grid's x range work on job[j].
constexpr int MAXJOBS = 4;
struct AttJobs {
    AttArgs job[MAXJOBS];
    int first[MAXJOBS + 1];
    int njobs;
};
// the job of this workgroup; bx = its index within the job
#define ATT_JOB(m)                                                   \
    int bx = blockIdx.x, jobno = 0;                                  \
    while (jobno + 1 < (m).njobs && bx >= (m).first[jobno + 1]) ++jobno; \
    bx -= (m).first[jobno];                                          \
    const AttArgs &a = (m).job[jobno]


// Forward.  NCH = ceil(L / 64) chunks per row.  A lane first gathers the 54 inputs of each of its positions (9
// neighbouring pixels x 2 channels x 3 shifts along L, zero outside the volume) into registers, then runs the K
// filters over them with the weights read from LDS four at a time: 54 FMAs per position and filter, no load in
// the filter loop.
template <int NCH>
__global__ void __launch_bounds__(64 * WPB) att_forward_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ __attribute__((aligned(16))) float ws[MAXK * 56 + MAXK];   // [k][56]: 54 weights (c, dl, di, dj) + 2 pad
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    for (int t = threadIdx.x; t < K * 54; t += blockDim.x) ws[(t / 54) * 56 + t % 54] = a.weight[t];
    for (int t = threadIdx.x; t < K; t += blockDim.x) ws[MAXK * 56 + t] = a.bias ? a.bias[t] : 0.f;
    __syncthreads();
    // rows of up to 32 (16) entries: 2 (4) pixels per wave, a group of lw lanes each
    const int lw = NCH == 1 ? lanes_per_pixel(L) : 64;
    const int lane = threadIdx.x & (lw - 1), wave = threadIdx.x >> 6, sub = (threadIdx.x & 63) / lw;
    const long pix = ((long)bx * WPB + wave) * (64 / lw) + sub;       // flattened (b,i,j)
    const long npix = (long)a.B * H1 * W1;
    if (pix >= npix) return;   // whole groups leave: the reductions below stay inside a group
    const int j = (int)(pix % W1), i = (int)((pix / W1) % H1);

    float x[NCH][2][3][9];   // [chunk][c][dl][neighbour di*3+dj]: the order of the weights
#pragma unroll
    for (int n = 0; n < 9; ++n) {
        const int ii = i + n / 3 - 1, jj = j + n % 3 - 1;
        const bool inb = ii >= 0 && ii < H1 && jj >= 0 && jj < W1;
        const float *row = a.sep + (pix + (long)(n / 3 - 1) * W1 + (n % 3 - 1)) * 2 * L;
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int dl = 0; dl < 3; ++dl) {
                    const int ll = ch * 64 + lane + dl - 1;
                    x[ch][c][dl][n] = (inb && ll >= 0 && ll < L) ? row[c * L + ll] : 0.f;
                }
    }

    for (int k = 0; k < K; ++k) {
        float logit[NCH];
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) logit[ch] = ws[MAXK * 56 + k];
#pragma unroll
        for (int q = 0; q < 14; ++q) {   // 56 floats = 14 reads of 16 bytes, the same address in every lane
            const float4 w4 = *reinterpret_cast<const float4 *>(&ws[k * 56 + 4 * q]);
            const float wq[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int t = 4 * q + e;
                if (t < 54) {
                    const int c = t / 27, dl = (t / 9) % 3, n = t % 9;
#pragma unroll
                    for (int ch = 0; ch < NCH; ++ch) logit[ch] = fmaf(wq[e], x[ch][c][dl][n], logit[ch]);
                }
            }
        }
        float m = -INFINITY;
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch)
            if (ch * 64 + lane < L) m = fmaxf(m, logit[ch]);
        m = group_max(m, lw);
        float s = 0.f, ex[NCH];
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            ex[ch] = (ch * 64 + lane < L) ? __expf(logit[ch] - m) : 0.f;
            s += ex[ch];
        }
        s = group_sum(s, lw);
        const float inv = 1.f / s;
        float *dst = a.out + (pix * K + k) * L;
        if (a.stats && lane == 0) {
            a.stats[2 * (pix * K + k)] = m;
            a.stats[2 * (pix * K + k) + 1] = s;
        }
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch)
            if (ch * 64 + lane < L) dst[ch * 64 + lane] = a.logits_only ? logit[ch] : ex[ch] * inv;
    }
}

// Forward for long rows: logits go to the output buffer first, then are normalised in place.
__global__ void __launch_bounds__(64 * WPB) att_forward_long_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ float ws[MAXK * 54 + MAXK];
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    for (int t = threadIdx.x; t < K * 54; t += blockDim.x) ws[t] = a.weight[t];
    for (int t = threadIdx.x; t < K; t += blockDim.x) ws[MAXK * 54 + t] = a.bias ? a.bias[t] : 0.f;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long pix = (long)bx * WPB + wave;
    const long npix = (long)a.B * H1 * W1;
    if (pix >= npix) return;
    const int j = (int)(pix % W1), i = (int)((pix / W1) % H1);
    for (int k = 0; k < K; ++k) {
        float *dst = a.out + (pix * K + k) * L;
        float m = -INFINITY;
        for (int l = lane; l < L; l += 64) {
            float x = ws[MAXK * 54 + k];
            for (int di = 0; di < 3; ++di) {
                const int ii = i + di - 1;
                if (ii < 0 || ii >= H1) continue;
                for (int dj = 0; dj < 3; ++dj) {
                    const int jj = j + dj - 1;
                    if (jj < 0 || jj >= W1) continue;
                    const float *row = a.sep + (pix + (long)(di - 1) * W1 + (dj - 1)) * 2 * L;
                    for (int c = 0; c < 2; ++c)
                        for (int dl = 0; dl < 3; ++dl) {
                            const int ll = l + dl - 1;
                            if (ll >= 0 && ll < L) x += ws[((k * 2 + c) * 3 + dl) * 9 + di * 3 + dj] * row[c * L + ll];
                        }
                }
            }
            dst[l] = x;
            m = fmaxf(m, x);
        }
        m = wave_max(m);
        float s = 0.f;
        for (int l = lane; l < L; l += 64) {
            const float e = __expf(dst[l] - m);   // written by this same lane
            if (!a.logits_only) dst[l] = e;
            s += e;
        }
        s = wave_sum(s);
        if (a.stats && lane == 0) {
            a.stats[2 * (pix * K + k)] = m;
            a.stats[2 * (pix * K + k) + 1] = s;
        }
        const float inv = 1.f / s;
        if (!a.logits_only)
            for (int l = lane; l < L; l += 64) dst[l] *= inv;
    }
}

// ---- Strips ----------------------------------------------------------------------------------------------------
// The kernels above give every pixel a wave (or a group of lanes) of its own, which fetches the rows of its nine
// neighbours three times each (shifted by -1, 0, +1 along L): 54 loads per position for 54 K multiply-adds.  The strip
// kernels give a group of lanes SP neighbouring pixels of one image row.  The group fetches the three image rows of
// the SP + 2 columns under the strip once (6 (SP + 2) vector loads for 54 K SP NV multiply-adds per lane), and a
// lane gets the neighbours along L from the lanes beside it (one data-parallel-primitive move each) instead of from
// memory.  A lane holds NV consecutive positions l = NV * lane + e (rows of up to 64 NV entries; NV > 1 needs L to
// be a multiple of NV and 4 NV-byte aligned tensors), so for e inside the vector the neighbour is the lane's own.
// Raw buffer resource over `bytes` bytes at p (wave-uniform): loads whose per-lane byte offset is >= bytes return 0,
// which stands in for every bounds branch of a window (image borders, lanes past the end of a row).
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, unsigned bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(p);
    const uint64_t lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)addr);
    const uint64_t hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(addr >> 32));
    const int n = __builtin_amdgcn_readfirstlane((int)bytes);
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((hi << 32) | lo), 0, n, 0x00020000);
}
constexpr unsigned OOB = 0x80000000u;   // a byte offset above the size of every tensor the strip kernels take
// NV floats at byte offset lane_off + uniform_off (the second the same in every lane; it takes no part in the bounds check)
template <int NV>
__device__ __forceinline__ void buf_load_vec(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned uniform_off, float (&x)[NV]) {
    if constexpr (NV == 1) {
        x[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, uniform_off, 0));
    } else if constexpr (NV == 2) {
        const v2f v = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(r, lane_off, uniform_off, 0));
        x[0] = v.x; x[1] = v.y;
    } else {
        const v4f v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, uniform_off, 0));
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
}
template <int NV>
__device__ __forceinline__ void load_vec(const float *p, float (&x)[NV]) {
    if constexpr (NV == 1) {
        x[0] = *p;
    } else if constexpr (NV == 2) {
        const float2 v = *reinterpret_cast<const float2 *>(p);
        x[0] = v.x; x[1] = v.y;
    } else {
        const float4 v = *reinterpret_cast<const float4 *>(p);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
}
template <int NV>
__device__ __forceinline__ void store_vec(float *p, const float (&x)[NV]) {
    if constexpr (NV == 1) p[0] = x[0];
    else if constexpr (NV == 2) *reinterpret_cast<float2 *>(p) = make_float2(x[0], x[1]);
    else *reinterpret_cast<float4 *>(p) = make_float4(x[0], x[1], x[2], x[3]);
}
// a value that is the same in every lane, as a scalar
__device__ __forceinline__ float uniform(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}
// the value of the lane below / above (0 at the ends of the wave)
__device__ __forceinline__ float lane_below(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x138, 0xf, 0xf, true));   // wave_shr:1
}
__device__ __forceinline__ float lane_above(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x130, 0xf, 0xf, true));   // wave_shl:1
}
// Sum or maximum over each aligned group of lw = 16, 32 or 64 lanes by data-parallel-primitive steps (no LDS round
// trips: a chain of six dependent vector instructions instead of six permutes); the result stands in the highest lane
// of the group.  Sums fill absent source lanes with 0; maxima keep the lane's own value there.
template <bool MAX, int CTRL, int RM, int BM>
__device__ __forceinline__ float reduce_step(float x) {
    const int xi = __builtin_bit_cast(int, x);
    if constexpr (MAX) return fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, CTRL, RM, BM, false)));
    else return x + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, xi, CTRL, RM, BM, true));
}
template <bool MAX>
__device__ __forceinline__ float group_reduce_top(float x, int lw) {
    x = reduce_step<MAX, 0x111, 0xf, 0xf>(x);                 // row_shr:1
    x = reduce_step<MAX, 0x112, 0xf, 0xf>(x);                 // row_shr:2
    x = reduce_step<MAX, 0x114, 0xf, 0xe>(x);                 // row_shr:4
    x = reduce_step<MAX, 0x118, 0xf, 0xc>(x);                 // row_shr:8: lane 15 of every row holds the row's result
    if (lw > 16) x = reduce_step<MAX, 0x142, 0xa, 0xf>(x);    // row_bcast:15 into rows 1 and 3
    if (lw > 32) x = reduce_step<MAX, 0x143, 0xc, 0xf>(x);    // row_bcast:31 into rows 2 and 3
    return x;
}
// the value of the group's highest lane in every lane of the group
__device__ __forceinline__ float group_top(float x, int lw) {
    if (lw == 64) return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
    return __shfl(x, (int)(threadIdx.x & 63) | (lw - 1));
}
// lanes per strip for rows of L entries held NV to a lane
__host__ __device__ inline int strip_lanes(int L, int NV) {
    const int n = (L + NV - 1) / NV;
    return n <= 16 ? 16 : n <= 32 ? 32 : 64;
}

struct Strip {
    bool active;     // the group has a strip (whole groups are idle past the end)
    bool first, last;   // this lane is the lowest / highest of its group
    int lw, lane;    // lanes of the group; this lane's number within it
    int i, j0, n;    // image row, first column, pixels (1..SP)
    long pix0;       // flattened (b, i, j0)
};
// the strip of this lane's group in wave-strip `wsidx` (a wave-strip = the 64 / lw strips a wave holds side by side)
template <int SP>
__device__ __forceinline__ Strip strip_at(const AttArgs &a, long wsidx, int lw) {
    Strip t;
    const int l64 = threadIdx.x & 63, sub = l64 / lw;
    const int ns = (a.W1 + SP - 1) / SP;
    const long s = wsidx * (64 / lw) + sub;
    t.active = s < (long)a.B * a.H1 * ns;
    const long row = s / ns;
    t.i = (int)(row % a.H1);
    t.j0 = (int)(s % ns) * SP;
    t.n = a.W1 - t.j0 < SP ? a.W1 - t.j0 : SP;
    t.pix0 = row * a.W1 + t.j0;
    t.lw = lw;
    t.lane = l64 & (lw - 1);
    t.first = t.lane == 0;
    t.last = t.lane == lw - 1;
    return t;
}
template <int SP>
__device__ __forceinline__ Strip strip_of(const AttArgs &a, int bx, int lw) {
    return strip_at<SP>(a, (long)bx * WPB + (threadIdx.x >> 6), lw);
}
// wave-strips of a tensor; workgroups of a launch that gives every wave one
static long wave_strips(int B, int H1, int W1, int L, int NV, int SP) {
    const long per = 64 / strip_lanes(L, NV);
    const long total = (long)B * H1 * ((W1 + SP - 1) / SP);
    return (total + per - 1) / per;
}
static unsigned strip_groups(int B, int H1, int W1, int L, int NV, int SP) {
    return (unsigned)((wave_strips(B, H1, W1, L, NV, SP) + WPB - 1) / WPB);
}

// The window of a strip: SP + 2 columns x 3 image rows x NCHAN channels of one tensor whose rows are (pixel, channel)
// x L, with the values of the lanes beside (xm: position l - 1 of the lane's first entry, xp: l + 1 of its last).
// fetch() issues the loads (buffer loads: what lies outside the image or the row reads as 0); finish() derives xm / xp.
template <int NV, int SP, int NCHAN>
struct Window {
    float x[SP + 2][3][NCHAN][NV], xm[SP + 2][3][NCHAN], xp[SP + 2][3][NCHAN];
    // chan0: first channel to fetch, nchan_total: channels per pixel in memory
    __device__ __forceinline__ void fetch(__amdgpu_buffer_rsrc_t rs, const Strip &t, int H1, int W1, int L, int nchan_total, int chan0) {
        const bool lok = t.active && t.lane * NV < L;
        const int p0 = (int)t.pix0;
        // byte offset of the lane's entries in channel chan0 of the strip's first pixel, rows i - 1 .. i + 1.  The
        // per-lane offset must be in range by itself (the bounds check does not see the uniform part), so the column
        // left of the strip gets an offset of its own instead of a negative uniform part.
        unsigned rowoff[3];
        const unsigned pixel = (unsigned)(nchan_total * L) * 4u;
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const int ii = t.i + r - 1;
            const unsigned off = (unsigned)(((p0 + (r - 1) * W1) * nchan_total + chan0) * L + t.lane * NV) * 4u;
            rowoff[r] = (lok && ii >= 0 && ii < H1) ? off : OOB;
        }
#pragma unroll
        for (int col = 0; col < SP + 2; ++col) {
            const int jj = t.j0 + col - 1;
            const bool okc = jj >= 0 && jj < W1 && col <= t.n + 1;
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                const unsigned off = !okc || rowoff[r] == OOB ? OOB : col == 0 ? rowoff[r] - pixel : rowoff[r];
#pragma unroll
                for (int c = 0; c < NCHAN; ++c)
                    buf_load_vec<NV>(rs, off, (unsigned)(((col == 0 ? 0 : col - 1) * nchan_total + c) * L) * 4u, x[col][r][c]);
            }
        }
    }
    __device__ __forceinline__ void finish(const Strip &t) {
#pragma unroll
        for (int col = 0; col < SP + 2; ++col)
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int c = 0; c < NCHAN; ++c) {
                    xm[col][r][c] = lane_below(x[col][r][c][NV - 1]);
                    xp[col][r][c] = lane_above(x[col][r][c][0]);
                }
        if (t.lw < 64) {   // several strips in a wave: nothing crosses from one to the next
#pragma unroll
            for (int col = 0; col < SP + 2; ++col)
#pragma unroll
                for (int r = 0; r < 3; ++r)
#pragma unroll
                    for (int c = 0; c < NCHAN; ++c) {
                        xm[col][r][c] = t.first ? 0.f : xm[col][r][c];
                        xp[col][r][c] = t.last ? 0.f : xp[col][r][c];
                    }
        }
    }
    // entry e of the lane shifted by s = -1, 0, +1 along L
    __device__ __forceinline__ float at(int col, int r, int c, int s, int e) const {
        if (s == 0) return x[col][r][c][e];
        if (s < 0) return e == 0 ? xm[col][r][c] : x[col][r][c][e - 1];
        return e == NV - 1 ? xp[col][r][c] : x[col][r][c][e + 1];
    }
};

// Forward over strips.  Filter by filter: the 54 weights of a filter go from LDS into registers once per strip and
// serve its SP pixels.
template <int NV, int SP>
__global__ void __launch_bounds__(64 * WPB) att_forward_strip_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ __attribute__((aligned(16))) float ws[MAXK * 56 + MAXK];   // [k][56]: 54 weights (c, dl, di, dj) + 2 pad
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    for (int t = threadIdx.x; t < K * 56; t += blockDim.x) ws[t] = t % 56 < 54 ? a.weight[(t / 56) * 54 + t % 56] : 0.f;
    for (int t = threadIdx.x; t < K; t += blockDim.x) ws[MAXK * 56 + t] = a.bias ? a.bias[t] : 0.f;
    __syncthreads();
    const int lw = strip_lanes(L, NV);
    const Strip st = strip_of<SP>(a, bx, lw);
    if (!st.active) return;   // whole groups leave: the reductions below stay inside a group
    Window<NV, SP, 2> win;
    win.fetch(make_rsrc(a.sep, (unsigned)((long)a.B * H1 * W1 * 2 * L * 4)), st, H1, W1, L, 2, 0);
    win.finish(st);
    const bool lok = st.lane * NV < L;
#pragma unroll 1
    for (int k = 0; k < K; ++k) {
        float w[56];   // the same in every lane: kept in scalar registers
#pragma unroll
        for (int q = 0; q < 14; ++q) {   // 14 reads of 16 bytes, the same address in every lane
            const float4 w4 = *reinterpret_cast<const float4 *>(&ws[k * 56 + 4 * q]);
            w[4 * q] = uniform(w4.x); w[4 * q + 1] = uniform(w4.y); w[4 * q + 2] = uniform(w4.z); w[4 * q + 3] = uniform(w4.w);
        }
        const float bias = uniform(ws[MAXK * 56 + k]);
        float logit[SP][NV];
#pragma unroll
        for (int t = 0; t < SP; ++t)
#pragma unroll
            for (int e = 0; e < NV; ++e) {
                float z = bias;
#pragma unroll
                for (int tap = 0; tap < 54; ++tap) {
                    const int c = tap / 27, dl = (tap / 9) % 3, nb = tap % 9;
                    z = fmaf(w[tap], win.at(t + nb % 3, nb / 3, c, dl - 1, e), z);
                }
                logit[t][e] = z;
            }
        // row statistics of the SP pixels side by side (independent chains)
        float mx[SP], sum[SP], ex[SP][NV];
#pragma unroll
        for (int t = 0; t < SP; ++t) {
            float v = logit[t][0];
#pragma unroll
            for (int e = 1; e < NV; ++e) v = fmaxf(v, logit[t][e]);
            mx[t] = group_reduce_top<true>(lok ? v : -INFINITY, lw);
        }
#pragma unroll
        for (int t = 0; t < SP; ++t) mx[t] = group_top(mx[t], lw);
#pragma unroll
        for (int t = 0; t < SP; ++t) {
            float v = 0.f;
#pragma unroll
            for (int e = 0; e < NV; ++e) {
                ex[t][e] = lok ? __expf(logit[t][e] - mx[t]) : 0.f;
                v += ex[t][e];
            }
            sum[t] = group_reduce_top<false>(v, lw);
        }
#pragma unroll
        for (int t = 0; t < SP; ++t) sum[t] = group_top(sum[t], lw);
#pragma unroll
        for (int t = 0; t < SP; ++t) {
            const long pix = st.pix0 + t;
            if (t < st.n && a.stats && st.lane == 0) {
                a.stats[2 * (pix * K + k)] = mx[t];
                a.stats[2 * (pix * K + k) + 1] = sum[t];
            }
            if (t < st.n && lok) {
                const float inv = 1.f / sum[t];
                float o[NV];
#pragma unroll
                for (int e = 0; e < NV; ++e) o[e] = a.logits_only ? logit[t][e] : ex[t][e] * inv;
                store_vec<NV>(a.out + (pix * K + k) * L + st.lane * NV, o);
            }
        }
    }
}

// dlogits = a * (grad_a - sum_l a * grad_a), one wave per pixel.
__global__ void __launch_bounds__(64 * WPB) att_softmax_backward_kernel(const AttJobs m) {
    ATT_JOB(m);
    const int K = a.K, L = a.L;
    const int lw = lanes_per_pixel(L);
    const int lane = threadIdx.x & (lw - 1), wave = threadIdx.x >> 6, sub = (threadIdx.x & 63) / lw;
    const long pix = ((long)bx * WPB + wave) * (64 / lw) + sub;
    if (pix >= (long)a.B * a.H1 * a.W1) return;
    for (int k = 0; k < K; ++k) {
        const float *pa = a.a + (pix * K + k) * L, *pg = a.grad_a + (pix * K + k) * L;
        float dot = 0.f;
        for (int l = lane; l < L; l += lw) dot += pa[l] * pg[l];
        dot = group_sum(dot, lw);
        float *dst = a.dlogits + (pix * K + k) * L;
        for (int l = lane; l < L; l += lw) dst[l] = pa[l] * (pg[l] - dot);
    }
}

// d_sep[(i,j),c,l] = sum_{k,dl,di,dj} w[k][c][dl][di][dj] * dlogits[(i-di+1, j-dj+1), k, l-dl+1]
// Per filter k a lane gathers the 27 logit gradients it needs (9 neighbouring pixels x 3 shifts, zero outside the
// volume), then applies the two 27-tap rows of the filter, read from LDS four weights at a time.
__global__ void __launch_bounds__(64 * WPB) att_input_backward_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ __attribute__((aligned(16))) float ws[MAXK * 2 * 28];   // [k][c][28]: 27 weights (dl, di, dj) + 1 pad
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    for (int t = threadIdx.x; t < K * 54; t += blockDim.x) ws[(t / 27) * 28 + t % 27] = a.weight[t];
    __syncthreads();
    const int lw = lanes_per_pixel(L);
    const int lane = threadIdx.x & (lw - 1), wave = threadIdx.x >> 6, sub = (threadIdx.x & 63) / lw;
    const long pix = ((long)bx * WPB + wave) * (64 / lw) + sub;
    if (pix >= (long)a.B * H1 * W1) return;
    const int j = (int)(pix % W1), i = (int)((pix / W1) % H1);
    for (int l = lane; l < L; l += lw) {
        float d0 = 0.f, d1 = 0.f;
        for (int k = 0; k < K; ++k) {
            float x[27];   // [dl][di*3+dj]: the order of the weights
#pragma unroll
            for (int n = 0; n < 9; ++n) {
                const int ii = i - n / 3 + 1, jj = j - n % 3 + 1;
                const bool inb = ii >= 0 && ii < H1 && jj >= 0 && jj < W1;
                const float *g = a.dlogits + ((pix + (long)(1 - n / 3) * W1 + (1 - n % 3)) * K + k) * L;
#pragma unroll
                for (int dl = 0; dl < 3; ++dl) {
                    const int ll = l - dl + 1;
                    x[dl * 9 + n] = (inb && ll >= 0 && ll < L) ? g[ll] : 0.f;
                }
            }
#pragma unroll
            for (int q = 0; q < 7; ++q) {   // 28 floats = 7 reads of 16 bytes per channel, the same address in every lane
                const float4 u4 = *reinterpret_cast<const float4 *>(&ws[(k * 2 + 0) * 28 + 4 * q]);
                const float4 v4 = *reinterpret_cast<const float4 *>(&ws[(k * 2 + 1) * 28 + 4 * q]);
                const float u[4] = {u4.x, u4.y, u4.z, u4.w}, v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (4 * q + e < 27) {
                        d0 = fmaf(u[e], x[4 * q + e], d0);
                        d1 = fmaf(v[e], x[4 * q + e], d1);
                    }
            }
        }
        if (a.init) {
            d0 += a.init[(pix * 2 + 0) * L + l];
            d1 += a.init[(pix * 2 + 1) * L + l];
        }
        a.out[(pix * 2 + 0) * L + l] = d0;
        a.out[(pix * 2 + 1) * L + l] = d1;
    }
}

// Sum over the 64 lanes with data-parallel-primitive adds (one vector instruction per step, no LDS traffic);
// the total is returned by lane 63.
__device__ __forceinline__ float wave_sum_dpp(float x) {
    // row_shr:1, 2, 3 gather a row's four-lane groups; row_shr:4 and 8 (bank masked) complete the row of 16;
    // row_bcast:15 / 31 carry the row totals across rows
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xe, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xc, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x143, 0xc, 0xf, true));
    return x;
}

// Weight and bias gradient, stage 1.  Workgroup (x, y): pixels [x*DW_PIX, ...), input channel c = y % 2, weight
// channels [4 (y/2), +4).  Wave w of the 4 handles every 4th pixel, lanes run along L.  Per position a lane gathers
// the 27 inputs of its channel (9 neighbouring pixels x 3 shifts along L, zero outside the volume) and the 4 logit
// gradients, then updates 27 x 4 accumulators (108 registers: two waves fit a SIMD); these are reduced over lanes
// and waves in a fixed order and written as partial[x][...].
constexpr int DW_KC = 4;
__global__ void __launch_bounds__(256) att_weight_backward_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ float red[4][27 * DW_KC + DW_KC];
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    const int lw = lanes_per_pixel(L), ppw = 64 / lw;   // short rows: ppw pixels per wave and iteration
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane / lw, ll0 = lane & (lw - 1);
    const int c = blockIdx.y & 1, k0 = (blockIdx.y >> 1) * DW_KC;
    const long npix = (long)a.B * H1 * W1;
    const long p0 = (long)bx * DW_PIX;
    float acc[27][DW_KC], accb[DW_KC];
#pragma unroll
    for (int t = 0; t < 27; ++t)
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) acc[t][k] = 0.f;
#pragma unroll
    for (int k = 0; k < DW_KC; ++k) accb[k] = 0.f;
    // iterations = (pixel of this wave, chunk of 64 positions); the inputs of the next iteration are fetched while
    // the accumulators are updated with the current ones
    const int nch = (L + 63) >> 6;
    const long left = npix - p0;
    const int npx = (int)(left < DW_PIX ? left : DW_PIX);
    const int ngr = (npx + ppw - 1) / ppw;           // pixel groups of this workgroup
    const int nit = ((ngr - wave + 3) / 4) * nch;    // groups wave, wave + 4, ... below ngr
    auto fetch = [&](int it, float(&x)[27], float(&gv)[DW_KC]) {
        const int q = (wave + 4 * (it / nch)) * ppw + sub;
        const bool pok = q < npx;
        const long pix = p0 + (pok ? q : 0);
        const int l = (it % nch) * 64 + ll0;
        const int j = (int)(pix % W1), i = (int)((pix / W1) % H1);
#pragma unroll
        for (int n = 0; n < 9; ++n) {
            const int ii = i + n / 3 - 1, jj = j + n % 3 - 1;
            const bool inb = pok && ii >= 0 && ii < H1 && jj >= 0 && jj < W1;
            const float *row = a.sep + ((pix + (long)(n / 3 - 1) * W1 + (n % 3 - 1)) * 2 + c) * L;
#pragma unroll
            for (int dl = 0; dl < 3; ++dl) {
                const int ll = l + dl - 1;
                x[dl * 9 + n] = (inb && ll >= 0 && ll < L) ? row[ll] : 0.f;   // [dl][neighbour]: the order of the weights
            }
        }
        const float *g = a.dlogits + pix * K * L;
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) gv[k] = (pok && k0 + k < K && l < L) ? g[(k0 + k) * L + l] : 0.f;
    };
    auto update = [&](const float(&x)[27], const float(&gv)[DW_KC]) {
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) {
            accb[k] += gv[k];
#pragma unroll
            for (int t = 0; t < 27; ++t) acc[t][k] = fmaf(gv[k], x[t], acc[t][k]);
        }
    };
    float xa[27], xb[27], ga[DW_KC], gb[DW_KC];
    if (nit > 0) fetch(0, xa, ga);
    for (int it = 0; it < nit; it += 2) {
        if (it + 1 < nit) fetch(it + 1, xb, gb);
        update(xa, ga);
        if (it + 2 < nit) fetch(it + 2, xa, ga);
        if (it + 1 < nit) update(xb, gb);
    }
#pragma unroll
    for (int t = 0; t < 27; ++t)
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) {
            const float r = wave_sum_dpp(acc[t][k]);
            if (lane == 63) red[wave][t * DW_KC + k] = r;
        }
#pragma unroll
    for (int k = 0; k < DW_KC; ++k) {
        const float r = wave_sum_dpp(accb[k]);
        if (lane == 63) red[wave][27 * DW_KC + k] = r;
    }
    __syncthreads();
    // partial layout per workgroup x: [K*54 weights in weight order (k, c, dl, di, dj)][K biases]
    float *dst = a.partial + (long)bx * (K * 54 + K);
    for (int t = threadIdx.x; t < 27 * DW_KC; t += blockDim.x) {
        const int k = t % DW_KC, tap = t / DW_KC;
        if (k0 + k < K) dst[(k0 + k) * 54 + c * 27 + tap] = red[0][t] + red[1][t] + red[2][t] + red[3][t];
    }
    if (c == 0)   // the bias gradient is counted once
        for (int t = threadIdx.x; t < DW_KC; t += blockDim.x)
            if (k0 + t < K)
                dst[K * 54 + k0 + t] = red[0][27 * DW_KC + t] + red[1][27 * DW_KC + t] + red[2][27 * DW_KC + t] + red[3][27 * DW_KC + t];
}

// Stage 2: out[t] = sum over workgroups of partial[x][t].  One wave per output: lane l adds the partials
// x = l, l+64, ... in order, then the 64 lane sums are added by a fixed butterfly: deterministic.
__global__ void __launch_bounds__(256) att_weight_reduce_kernel(const float *partial, float *d_weight, float *d_bias, int nwg,
                                                                int K) {
    const int n = K * 54 + K;
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n) return;
    float s = 0.f;
    for (int x = lane; x < nwg; x += 64) s += partial[(long)x * n + t];
    s = wave_sum(s);
    if (lane == 0) {
        if (t < K * 54) d_weight[t] = s;
        else if (d_bias) d_bias[t - K * 54] = s;
    }
}

// d_sep over strips.  Filter by filter: a window of the filter's logit gradients (fetched while the previous filter is
// applied), its 2 x 27 weights in scalar registers, 2 x NV accumulators per pixel of the strip.
template <int NV, int SP>
__global__ void __launch_bounds__(64 * WPB) att_input_backward_strip_kernel(const AttJobs m) {
    ATT_JOB(m);
    __shared__ __attribute__((aligned(16))) float ws[MAXK * 56];   // [k][c][28]: 27 weights (dl, di, dj) + 1 pad
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    for (int t = threadIdx.x; t < K * 56; t += blockDim.x) ws[t] = t % 28 < 27 ? a.weight[(t / 28) * 27 + t % 28] : 0.f;
    __syncthreads();
    const int lw = strip_lanes(L, NV);
    const Strip st = strip_of<SP>(a, bx, lw);
    if (!st.active) return;
    const bool lok = st.lane * NV < L;
    float d[SP][2][NV];
#pragma unroll
    for (int t = 0; t < SP; ++t)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int e = 0; e < NV; ++e) d[t][c][e] = 0.f;
    Window<NV, SP, 1> win, nxt;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.dlogits, (unsigned)((long)a.B * H1 * W1 * K * L * 4));
    nxt.fetch(rs, st, H1, W1, L, K, 0);
#pragma unroll 1
    for (int k = 0; k < K; ++k) {
#pragma unroll
        for (int col = 0; col < SP + 2; ++col)
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int e = 0; e < NV; ++e) win.x[col][r][0][e] = nxt.x[col][r][0][e];
        win.finish(st);
        if (k + 1 < K) nxt.fetch(rs, st, H1, W1, L, K, k + 1);
        float w[56];   // the same in every lane: kept in scalar registers
#pragma unroll
        for (int q = 0; q < 14; ++q) {
            const float4 w4 = *reinterpret_cast<const float4 *>(&ws[k * 56 + 4 * q]);
            w[4 * q] = uniform(w4.x); w[4 * q + 1] = uniform(w4.y); w[4 * q + 2] = uniform(w4.z); w[4 * q + 3] = uniform(w4.w);
        }
        // the gradient of pixel (i, j) takes tap (dl, di, dj) from pixel (i - di + 1, j - dj + 1) at l - dl + 1
#pragma unroll
        for (int t = 0; t < SP; ++t)
#pragma unroll
            for (int tap = 0; tap < 27; ++tap) {
                const int dl = tap / 9, di = (tap % 9) / 3, dj = tap % 3;
#pragma unroll
                for (int e = 0; e < NV; ++e) {
                    const float g = win.at(t + 2 - dj, 2 - di, 0, 1 - dl, e);
                    d[t][0][e] = fmaf(w[tap], g, d[t][0][e]);
                    d[t][1][e] = fmaf(w[28 + tap], g, d[t][1][e]);
                }
            }
    }
    if (lok) {
#pragma unroll
        for (int t = 0; t < SP; ++t) {
            if (t >= st.n) break;
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const long o = ((st.pix0 + t) * 2 + c) * L + st.lane * NV;
                if (a.init) {
                    float v[NV];
                    load_vec<NV>(a.init + o, v);
#pragma unroll
                    for (int e = 0; e < NV; ++e) d[t][c][e] += v[e];
                }
                store_vec<NV>(a.out + o, d[t][c]);
            }
        }
    }
}

// Weight and bias gradient over strips, stage 1.  Workgroup (x, y): wave-strips [x * dw_ws(NV), ...), input channel
// c = y % 2, weight channels [4 (y / 2), +4); a wave takes every 4th of them, SP = 4 / NV pixels per strip.  Per strip:
// the window of channel c and the 4 logit gradients of its pixels (both fetched while the previous strip is worked on),
// then 27 x 4 accumulators are updated per position; reduced over lanes and waves in a fixed order and written as
// partial[x][...] like att_weight_backward_kernel's.
// (measured for attention 1 / attention 2 over four levels at B=2, 55x128: 16 wave-strips per workgroup 65 / 42 us,
// 32: 61 / 36 us, 64: 52 / 47 us)
constexpr int dw_ws(int nv) { return nv == 1 ? 32 : 64; }
template <int NV>
__global__ void __launch_bounds__(256) att_weight_backward_strip_kernel(const AttJobs m) {
    ATT_JOB(m);
    constexpr int SP = 4 / NV;
    __shared__ float red[4][27 * DW_KC + DW_KC];
    const int K = a.K, L = a.L, H1 = a.H1, W1 = a.W1;
    const int lw = strip_lanes(L, NV);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = blockIdx.y & 1, k0 = (blockIdx.y >> 1) * DW_KC;
    const long nws = ((long)a.B * H1 * ((W1 + SP - 1) / SP) + 64 / lw - 1) / (64 / lw);
    constexpr int DW_WS = dw_ws(NV);
    const long ws0 = (long)bx * DW_WS;
    const int nmine = (int)(nws - ws0 < DW_WS ? nws - ws0 : DW_WS);   // wave-strips of this workgroup
    const int nit = (nmine - wave + 3) / 4;
    float acc[27][DW_KC], accb[DW_KC];
#pragma unroll
    for (int t = 0; t < 27; ++t)
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) acc[t][k] = 0.f;
#pragma unroll
    for (int k = 0; k < DW_KC; ++k) accb[k] = 0.f;
    Window<NV, SP, 1> win, nxt;
    float g[SP][DW_KC][NV], gn[SP][DW_KC][NV];
    Strip st = strip_at<SP>(a, ws0 + wave, lw);
    const __amdgpu_buffer_rsrc_t rs_sep = make_rsrc(a.sep, (unsigned)((long)a.B * H1 * W1 * 2 * L * 4));
    const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(a.dlogits, (unsigned)((long)a.B * H1 * W1 * K * L * 4));
    auto fetch = [&](int it) {
        st = strip_at<SP>(a, ws0 + wave + 4 * it, lw);
        nxt.fetch(rs_sep, st, H1, W1, L, 2, c);
        const bool lok = st.active && st.lane * NV < L;
        const unsigned goff = (unsigned)(((int)st.pix0 * K + k0) * L + st.lane * NV) * 4u;
#pragma unroll
        for (int t = 0; t < SP; ++t) {
            const unsigned off = (lok && t < st.n) ? goff : OOB;
#pragma unroll
            for (int k = 0; k < DW_KC; ++k) {
                if (k0 + k < K) buf_load_vec<NV>(rs_g, off, (unsigned)((t * K + k) * L) * 4u, gn[t][k]);
                else
#pragma unroll
                    for (int e = 0; e < NV; ++e) gn[t][k][e] = 0.f;
            }
        }
    };
    if (nit > 0) fetch(0);
#pragma unroll 1
    for (int it = 0; it < nit; ++it) {
#pragma unroll
        for (int col = 0; col < SP + 2; ++col)
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int e = 0; e < NV; ++e) win.x[col][r][0][e] = nxt.x[col][r][0][e];
#pragma unroll
        for (int t = 0; t < SP; ++t)
#pragma unroll
            for (int k = 0; k < DW_KC; ++k)
#pragma unroll
                for (int e = 0; e < NV; ++e) g[t][k][e] = gn[t][k][e];
        win.finish(st);   // first / last depend on the lane only
        if (it + 1 < nit) fetch(it + 1);
#pragma unroll
        for (int t = 0; t < SP; ++t)
#pragma unroll
            for (int e = 0; e < NV; ++e) {
#pragma unroll
                for (int k = 0; k < DW_KC; ++k) accb[k] += g[t][k][e];
#pragma unroll
                for (int tap = 0; tap < 27; ++tap) {   // [dl][di][dj]: the order of the weights
                    const float x = win.at(t + tap % 3, (tap % 9) / 3, 0, tap / 9 - 1, e);
#pragma unroll
                    for (int k = 0; k < DW_KC; ++k) acc[tap][k] = fmaf(g[t][k][e], x, acc[tap][k]);
                }
            }
    }
#pragma unroll
    for (int t = 0; t < 27; ++t)
#pragma unroll
        for (int k = 0; k < DW_KC; ++k) {
            const float r = wave_sum_dpp(acc[t][k]);
            if (lane == 63) red[wave][t * DW_KC + k] = r;
        }
#pragma unroll
    for (int k = 0; k < DW_KC; ++k) {
        const float r = wave_sum_dpp(accb[k]);
        if (lane == 63) red[wave][27 * DW_KC + k] = r;
    }
    __syncthreads();
    float *dst = a.partial + (long)bx * (K * 54 + K);
    for (int t = threadIdx.x; t < 27 * DW_KC; t += blockDim.x) {
        const int k = t % DW_KC, tap = t / DW_KC;
        if (k0 + k < K) dst[(k0 + k) * 54 + c * 27 + tap] = red[0][t] + red[1][t] + red[2][t] + red[3][t];
    }
    if (c == 0)   // the bias gradient is counted once
        for (int t = threadIdx.x; t < DW_KC; t += blockDim.x)
            if (k0 + t < K)
                dst[K * 54 + k0 + t] = red[0][27 * DW_KC + t] + red[1][27 * DW_KC + t] + red[2][27 * DW_KC + t] + red[3][27 * DW_KC + t];
}

// pixels per strip for nv positions per lane
// the forward kernel with two positions per lane: strips of 2 (126 registers, four waves per SIMD; 52 us for attention 1
// over four levels at B=2, 55x128) are faster than strips of 4 (62 us) or 1 (56 us)
constexpr int fwd_sp(int nv) { return nv == 1 ? 4 : 2; }
// the input gradient: strips of 4 and of 2 measure the same with two positions per lane (48 us)
constexpr int bwd_sp(int nv) { return nv == 4 ? 2 : 4; }
static bool aligned_for(const void *p, int nv) { return !p || (reinterpret_cast<uintptr_t>(p) & (uintptr_t)(4 * nv - 1)) == 0; }
// rows of L entries can be held nv to a lane
static bool strip_fits(int L, int nv) { return L <= 64 * nv && L % nv == 0; }
// The strip variant (positions per lane; 0: none, the job runs one wave per pixel) of every job of a call.  A job
// takes the smallest that holds its rows with all its tensors (t0..t3, unused ones NULL) aligned for the vector
// accesses; jobs that could also run with the largest variant among them are moved to it, so that they share its launch.
template <typename Tensors>
static void strip_variants(const AttArgs *jobs, int n, Tensors tensors, int (&var)[MAXJOBS]) {
    auto ok = [&](int j, int nv) {
        if (!strip_fits(jobs[j].L, nv)) return false;
        const int ch = jobs[j].K > 2 ? jobs[j].K : 2;   // buffer loads address a tensor with 31-bit byte offsets
        if ((double)jobs[j].B * jobs[j].H1 * jobs[j].W1 * ch * jobs[j].L * 4.0 >= 2147483648.0) return false;
        const void *t[4];
        tensors(jobs[j], t);
        return aligned_for(t[0], nv) && aligned_for(t[1], nv) && aligned_for(t[2], nv) && aligned_for(t[3], nv);
    };
    int top = 0;
    for (int j = 0; j < n; ++j) {
        var[j] = ok(j, 1) ? 1 : ok(j, 2) ? 2 : ok(j, 4) ? 4 : 0;
        if (var[j] > top) top = var[j];
    }
    for (int j = 0; j < n; ++j)
        if (var[j] > 0 && var[j] < top && ok(j, top)) var[j] = top;
}
// workgroups (= partial sums) of the weight-gradient launch of one job, by kernel variant (nv = 0: one wave per pixel)
static unsigned weight_groups(int B, int H1, int W1, int L, int nv) {
    if (nv == 0) return (unsigned)(((long)B * H1 * W1 + DW_PIX - 1) / DW_PIX);
    return (unsigned)((wave_strips(B, H1, W1, L, nv, 4 / nv) + dw_ws(nv) - 1) / dw_ws(nv));
}
// the largest over the variants a job with rows of L entries can run with: which one it is depends on the alignment
// of the tensors and on the other jobs of the call
static size_t weight_groups_max(int B, int H1, int W1, int L) {
    unsigned most = weight_groups(B, H1, W1, L, 0);
    for (int nv = 1; nv <= 4; nv *= 2)
        if (strip_fits(L, nv)) {
            const unsigned g = weight_groups(B, H1, W1, L, nv);
            if (g > most) most = g;
        }
    return most;
}
template <int NV>
static void launch_backward_strip(const AttJobs &mi, unsigned gi, const AttJobs &mw, unsigned gw, int K, hipStream_t s) {
    hipLaunchKernelGGL((att_input_backward_strip_kernel<NV, bwd_sp(NV)>), dim3(gi), dim3(64 * WPB), 0, s, mi);
    hipLaunchKernelGGL((att_weight_backward_strip_kernel<NV>), dim3(gw, 2 * ((K + DW_KC - 1) / DW_KC)), dim3(256), 0, s, mw);
}
template <int NV>
static void launch_forward_strip(const AttJobs &m, unsigned nwg, hipStream_t s) {
    hipLaunchKernelGGL((att_forward_strip_kernel<NV, fwd_sp(NV)>), dim3(nwg), dim3(64 * WPB), 0, s, m);
}
int check(const void *p, const char *name) {
    if (p) return 0;
    char msg[128];
    snprintf(msg, sizeof(msg), "sepcorr: argument %s is NULL", name);
    return sepcorr_set_error(SEPCORR_EINVAL, msg);
}
#define REQ(p) if (int rc = check(p, #p)) return rc

int check_sizes(int B, int H1, int W1, int L, int K) {
    char msg[160];
    if (B < 1 || H1 < 1 || W1 < 1 || L < 1 || K < 1 || K > MAXK) {
        snprintf(msg, sizeof(msg), "sepcorr: attention sizes out of range (B=%d H1=%d W1=%d L=%d K=%d, K <= %d)", B, H1, W1, L, K, MAXK);
        return sepcorr_set_error(SEPCORR_EINVAL, msg);
    }
    if ((double)B * H1 * W1 * K * L > 2147483647.0 || (double)B * H1 * W1 * 2 * L > 2147483647.0)
        return sepcorr_set_error(SEPCORR_EINVAL, "sepcorr: a tensor would have 2^31 or more elements");
    return 0;
}

int launched(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    char msg[200];
    snprintf(msg, sizeof(msg), "sepcorr: %s: %s", what, hipGetErrorString(e));
    return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
}

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

static unsigned pixel_groups(long npix, int L);

// Input, weight and bias gradients of n jobs (levels) that share the weights: one launch each for the input
// gradients, the partial weight gradients and their reduction; d_weight / d_bias are the sums over all jobs.
// jobs[i].dlogits, .sep, .out (d_sep), .init are set by the caller; `partial` holds the partial sums of all jobs.
static int attention_conv_backward_jobs(const AttArgs *jobs, int n, float *partial, float *d_weight, float *d_bias, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int K = jobs[0].K;
    unsigned gw_all = 0;   // partial sums written so far: the launches below share `partial`
    int vars[MAXJOBS];
    strip_variants(jobs, n, [](const AttArgs &j, const void *(&t)[4]) { t[0] = j.sep; t[1] = j.dlogits; t[2] = j.out; t[3] = j.init; }, vars);
    for (int var = 0; var <= 4; ++var) {   // one pair of launches per kernel variant among the jobs
        if (var == 3) continue;
        AttJobs mi = {}, mw = {};
        unsigned gi = 0, gw = 0;
        for (int j = 0; j < n; ++j) {
            if (vars[j] != var) continue;
            const long npix = (long)jobs[j].B * jobs[j].H1 * jobs[j].W1;
            const int q = mi.njobs;
            mi.job[q] = jobs[j];
            mi.first[q] = (int)gi;
            gi += var == 0 ? pixel_groups(npix, jobs[j].L)
                           : strip_groups(jobs[j].B, jobs[j].H1, jobs[j].W1, jobs[j].L, var, bwd_sp(var));
            mw.job[q] = jobs[j];
            mw.job[q].partial = partial + (size_t)(gw_all + gw) * (K * 54 + K);
            mw.first[q] = (int)gw;
            gw += weight_groups(jobs[j].B, jobs[j].H1, jobs[j].W1, jobs[j].L, var);
            mi.njobs = mw.njobs = q + 1;
            mi.first[q + 1] = (int)gi; mw.first[q + 1] = (int)gw;
        }
        if (mi.njobs == 0) continue;
        if (var == 0) {
            hipLaunchKernelGGL(att_input_backward_kernel, dim3(gi), dim3(64 * WPB), 0, s, mi);
            hipLaunchKernelGGL(att_weight_backward_kernel, dim3(gw, 2 * ((K + DW_KC - 1) / DW_KC)), dim3(256), 0, s, mw);
        }
        else if (var == 1) launch_backward_strip<1>(mi, gi, mw, gw, K, s);
        else if (var == 2) launch_backward_strip<2>(mi, gi, mw, gw, K, s);
        else launch_backward_strip<4>(mi, gi, mw, gw, K, s);
        if (int rc = launched("attention input / weight gradient kernels")) return rc;
        gw_all += gw;
    }
    const int nw = K * 54 + K;
    hipLaunchKernelGGL(att_weight_reduce_kernel, dim3((nw + 3) / 4), dim3(256), 0, s, partial, d_weight, d_bias, (int)gw_all, K);
    return launched("attention weight gradient reduction");
}

// workgroups of a forward / softmax backward / input gradient launch for rows of L entries
static unsigned pixel_groups(long npix, int L) {
    const long ppg = (long)WPB * (64 / lanes_per_pixel(L));   // pixels per workgroup
    return (unsigned)((npix + ppg - 1) / ppg);
}
// kernel variant of the forward pass for rows of L entries: 1, 2, 4 chunks of 64, or 0 for the long-row kernel
static int forward_variant(int L) { return L <= 64 ? 1 : L <= 128 ? 2 : L <= 256 ? 4 : 0; }
// Forward pass of n jobs (levels) that share weight and bias: one launch per kernel variant among them.
static int attention_forward_jobs(const AttArgs *jobs, int n, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    bool done[MAXJOBS] = {};
    int vars[MAXJOBS];
    strip_variants(jobs, n, [](const AttArgs &j, const void *(&t)[4]) { t[0] = j.sep; t[1] = j.out; t[2] = t[3] = nullptr; }, vars);
    for (int i = 0; i < n; ++i) {   // strips: one launch per variant among the jobs
        if (done[i]) continue;
        const int nv = vars[i];
        if (nv == 0) continue;
        AttJobs m = {};
        unsigned nwg = 0;
        for (int j = i; j < n; ++j) {
            if (done[j] || vars[j] != nv) continue;
            done[j] = true;
            m.job[m.njobs] = jobs[j];
            m.first[m.njobs] = (int)nwg;
            nwg += strip_groups(jobs[j].B, jobs[j].H1, jobs[j].W1, jobs[j].L, nv, fwd_sp(nv));
            m.first[++m.njobs] = (int)nwg;
        }
        if (nv == 1) launch_forward_strip<1>(m, nwg, s);
        else if (nv == 2) launch_forward_strip<2>(m, nwg, s);
        else launch_forward_strip<4>(m, nwg, s);
        if (int rc = launched("attention forward kernel (strips)")) return rc;
    }
    for (int i = 0; i < n; ++i) {
        if (done[i]) continue;
        const int var = forward_variant(jobs[i].L);
        AttJobs m = {};
        unsigned nwg = 0;
        for (int j = i; j < n; ++j) {
            if (done[j] || forward_variant(jobs[j].L) != var) continue;
            done[j] = true;
            m.job[m.njobs] = jobs[j];
            m.first[m.njobs] = (int)nwg;
            nwg += pixel_groups((long)jobs[j].B * jobs[j].H1 * jobs[j].W1, jobs[j].L);
            m.first[++m.njobs] = (int)nwg;
        }
        const dim3 grid(nwg), block(64 * WPB);
        if (var == 1) hipLaunchKernelGGL(att_forward_kernel<1>, grid, block, 0, s, m);
        else if (var == 2) hipLaunchKernelGGL(att_forward_kernel<2>, grid, block, 0, s, m);
        else if (var == 4) hipLaunchKernelGGL(att_forward_kernel<4>, grid, block, 0, s, m);
        else hipLaunchKernelGGL(att_forward_long_kernel, grid, block, 0, s, m);
        if (int rc = launched("attention forward kernel")) return rc;
    }
    return 0;
}

static int attention_forward(const float *sep, const float *weight, const float *bias, float *a, float *stats, int logits_only,
                             int B, int H1, int W1, int L, int K, void *stream) {
    REQ(sep); REQ(weight); REQ(a);
    if (int rc = check_sizes(B, H1, W1, L, K)) return rc;
    AttArgs args = {};
    args.sep = sep; args.weight = weight; args.bias = bias; args.out = a;
    args.stats = stats; args.logits_only = logits_only;
    args.B = B; args.H1 = H1; args.W1 = W1; args.L = L; args.K = K;
    return attention_forward_jobs(&args, 1, stream);
}

int sepcorr_attention_logits_forward_levels(const float *const *sep, const float *weight, const float *bias,
                                            float *const *logits, float *const *stats, const int *L, int nlev, int B, int H1,
                                            int W1, int K, void *stream) {
    REQ(sep); REQ(weight); REQ(logits); REQ(L);
    if (nlev < 1 || nlev > MAXJOBS) return sepcorr_set_error(SEPCORR_EINVAL, "sepcorr: attention: 1 to 4 levels per call");
    AttArgs jobs[MAXJOBS] = {};
    for (int l = 0; l < nlev; ++l) {
        REQ(sep[l]); REQ(logits[l]);
        if (int rc = check_sizes(B, H1, W1, L[l], K)) return rc;
        jobs[l].sep = sep[l]; jobs[l].weight = weight; jobs[l].bias = bias; jobs[l].out = logits[l];
        jobs[l].stats = stats ? stats[l] : nullptr; jobs[l].logits_only = 1;
        jobs[l].B = B; jobs[l].H1 = H1; jobs[l].W1 = W1; jobs[l].L = L[l]; jobs[l].K = K;
    }
    return attention_forward_jobs(jobs, nlev, stream);
}

int sepcorr_attention_forward(const float *sep, const float *weight, const float *bias, float *a, int B, int H1, int W1, int L,
                              int K, void *stream) {
    return attention_forward(sep, weight, bias, a, nullptr, 0, B, H1, W1, L, K, stream);
}

int sepcorr_attention_logits_forward(const float *sep, const float *weight, const float *bias, float *logits, float *stats,
                                     int B, int H1, int W1, int L, int K, void *stream) {
    return attention_forward(sep, weight, bias, logits, stats, 1, B, H1, W1, L, K, stream);
}

size_t sepcorr_attention_workspace_bytes(int B, int H1, int W1, int L, int K) {
    if (B < 1 || H1 < 1 || W1 < 1 || L < 1 || K < 1 || K > MAXK) return 0;
    const size_t npix = (size_t)B * H1 * W1;
    const size_t nwg = weight_groups_max(B, H1, W1, L);
    return align256(npix * K * L * sizeof(float)) + align256(nwg * (K * 54 + K) * sizeof(float));
}

size_t sepcorr_attention_logits_workspace_bytes(int B, int H1, int W1, int L, int K) {
    if (B < 1 || H1 < 1 || W1 < 1 || L < 1 || K < 1 || K > MAXK) return 0;
    const size_t nwg = weight_groups_max(B, H1, W1, L);
    return align256(nwg * (K * 54 + K) * sizeof(float));
}

int sepcorr_attention_logits_backward(const float *sep, const float *weight, const float *d_logits, float *d_sep,
                                      float *d_weight, float *d_bias, int B, int H1, int W1, int L, int K, void *workspace,
                                      size_t workspace_bytes, void *stream) {
    REQ(sep); REQ(weight); REQ(d_logits); REQ(d_sep); REQ(d_weight);
    if (int rc = check_sizes(B, H1, W1, L, K)) return rc;
    const size_t need = sepcorr_attention_logits_workspace_bytes(B, H1, W1, L, K);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15)) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: attention backward needs %zu bytes of 16-byte aligned workspace, got %zu", need,
                 workspace ? workspace_bytes : (size_t)0);
        return sepcorr_set_error(SEPCORR_EWORKSPACE, msg);
    }
    AttArgs args = {};
    args.sep = sep; args.weight = weight;
    args.dlogits = const_cast<float *>(d_logits);   // read only from here on
    args.B = B; args.H1 = H1; args.W1 = W1; args.L = L; args.K = K;
    args.out = d_sep;
    return attention_conv_backward_jobs(&args, 1, static_cast<float *>(workspace), d_weight, d_bias, stream);
}

size_t sepcorr_attention_logits_levels_workspace_bytes(const int *L, int nlev, int B, int H1, int W1, int K) {
    if (!L || nlev < 1 || nlev > MAXJOBS) return 0;
    size_t total = 0;
    for (int l = 0; l < nlev; ++l) total += sepcorr_attention_logits_workspace_bytes(B, H1, W1, L[l], K);
    return total;
}

int sepcorr_attention_logits_backward_levels(const float *const *sep, const float *weight, const float *const *d_logits,
                                             const float *const *d_sep_init, float *const *d_sep, float *d_weight,
                                             float *d_bias, const int *L, int nlev, int B, int H1, int W1, int K,
                                             void *workspace, size_t workspace_bytes, void *stream) {
    REQ(sep); REQ(weight); REQ(d_logits); REQ(d_sep); REQ(d_weight); REQ(L);
    if (nlev < 1 || nlev > MAXJOBS) return sepcorr_set_error(SEPCORR_EINVAL, "sepcorr: attention: 1 to 4 levels per call");
    AttArgs jobs[MAXJOBS] = {};
    for (int l = 0; l < nlev; ++l) {
        REQ(sep[l]); REQ(d_logits[l]); REQ(d_sep[l]);
        if (int rc = check_sizes(B, H1, W1, L[l], K)) return rc;
        jobs[l].sep = sep[l]; jobs[l].weight = weight;
        jobs[l].dlogits = const_cast<float *>(d_logits[l]);
        jobs[l].init = d_sep_init ? d_sep_init[l] : nullptr;
        jobs[l].out = d_sep[l];
        jobs[l].B = B; jobs[l].H1 = H1; jobs[l].W1 = W1; jobs[l].L = L[l]; jobs[l].K = K;
    }
    const size_t need = sepcorr_attention_logits_levels_workspace_bytes(L, nlev, B, H1, W1, K);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15)) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: attention backward needs %zu bytes of 16-byte aligned workspace, got %zu", need,
                 workspace ? workspace_bytes : (size_t)0);
        return sepcorr_set_error(SEPCORR_EWORKSPACE, msg);
    }
    return attention_conv_backward_jobs(jobs, nlev, static_cast<float *>(workspace), d_weight, d_bias, stream);
}

int sepcorr_attention_backward(const float *sep, const float *weight, const float *a, const float *grad_a, float *d_sep,
                               float *d_weight, float *d_bias, int B, int H1, int W1, int L, int K, void *workspace,
                               size_t workspace_bytes, void *stream) {
    REQ(sep); REQ(weight); REQ(a); REQ(grad_a); REQ(d_sep); REQ(d_weight);
    if (int rc = check_sizes(B, H1, W1, L, K)) return rc;
    const size_t need = sepcorr_attention_workspace_bytes(B, H1, W1, L, K);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15)) {
        char msg[160];
        snprintf(msg, sizeof(msg), "sepcorr: attention backward needs %zu bytes of 16-byte aligned workspace, got %zu", need,
                 workspace ? workspace_bytes : (size_t)0);
        return sepcorr_set_error(SEPCORR_EWORKSPACE, msg);
    }
    const long npix = (long)B * H1 * W1;
    AttArgs args = {};
    args.sep = sep; args.weight = weight; args.a = a; args.grad_a = grad_a;
    args.dlogits = static_cast<float *>(workspace);
    float *partial = reinterpret_cast<float *>(static_cast<char *>(workspace) + align256((size_t)npix * K * L * sizeof(float)));
    args.B = B; args.H1 = H1; args.W1 = W1; args.L = L; args.K = K;
    hipStream_t s = static_cast<hipStream_t>(stream);
    {
        AttJobs m = {};
        m.job[0] = args;
        m.njobs = 1;
        m.first[1] = (int)pixel_groups(npix, L);
        hipLaunchKernelGGL(att_softmax_backward_kernel, dim3(m.first[1]), dim3(64 * WPB), 0, s, m);
        if (int rc = launched("attention softmax backward kernel")) return rc;
    }
    args.out = d_sep;
    return attention_conv_backward_jobs(&args, 1, partial, d_weight, d_bias, stream);
}

}  // extern "C"
