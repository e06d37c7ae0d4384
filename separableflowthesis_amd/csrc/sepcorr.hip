// libsepcorr: memory-saving separation of the 4D correlation volume, hand-written for gfx950.
//
// S[p,q] = <f1[p,:], f2[q,:]> with p = image-1 pixel (i,j), q = image-2 pixel (u,v) is produced
// 32x32 tiles at a time by v_mfma_f32_32x32x2_f32 and consumed in registers; it never reaches
// memory.  Three kernels cover the five entry points of include/sepcorr.h:
//
//   fwd_kernel  workgroup owns 32 pixels p and sweeps every fmap2 row u.  Wave w owns the column
//               chunk v in [32w, 32w+32).  MFMA rows are v (A operand = f2, loaded straight from
//               global memory in operand layout), MFMA columns are p (B operand = f1 tile in LDS).
//               One lane therefore holds one p and 16 v's: reductions over v are in-lane plus one
//               cross-half shuffle plus a cross-wave combine through LDS; reductions over u are
//               element-wise running state in registers in the accumulator layout.
//               Epilogues: max/avg(/argmax), or K weighted sums (attention compression; also the
//               d_a_u/d_a_v pass of the compression backward, which has the same form).
//   df1_kernel  same ownership.  G[p,q] is synthesised in registers directly in MFMA B-operand
//               layout from the saved argmax / upstream grads (or attention weights), A = f2^T
//               from global memory, D = d_f1^T partial per wave, summed across waves in LDS.
//   df2_kernel  wave owns 32 pixels q = (u, 32 consecutive v) and sweeps p; G^T synthesised in
//               registers, A = f1^T from global.  The p range can be split over workgroups; the
//               partial sums are written to scratch and added in a fixed order (no atomics).
//
// The contraction index of an MFMA may be permuted freely as long as A and B agree, and so may the
// row index of D as long as the store agrees; both freedoms are used so that every lane loads 16
// contiguous bytes.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "sepcorr.h"
#include "sepcorr_internal.h"

// This file is compiled once per part (see the Makefile) so that its many kernel instantiations build in parallel:
// part 0 holds the C ABI and the state shared by all parts, every other part holds the explicit instantiations of
// some of the launchers (launch_fwd / launch_bwd) with the kernels they start.  Without SEPCORR_PART the whole
// library is one translation unit.
#ifndef SEPCORR_PART
#define SEPCORR_PART (-1)
#endif
#define SEPCORR_IN_PART(n) (SEPCORR_PART < 0 || SEPCORR_PART == (n))

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Scratch memory of sepcorr_max_argmax_avg_backward_static: part of the library's device image, one copy per GPU,
// held until the process ends.  In host code this name is a handle, not a device address: the address on each
// device comes from hipGetSymbolAddress (static_scratch() below), and only that pointer is handed to kernels.
#if SEPCORR_IN_PART(0)
static __device__ __align__(256) unsigned char scratch[SEPCORR_STATIC_SCRATCH_BYTES];
#endif

namespace sepcorr_impl {
extern thread_local char g_err[256];
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
}  // namespace sepcorr_impl
using namespace sepcorr_impl;

#if SEPCORR_IN_PART(0)
namespace sepcorr_impl {
thread_local char g_err[256] = "";
int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}
}  // namespace sepcorr_impl

// shared with the other translation units of the library (sepcorr_internal.h)
int sepcorr_set_error(int code, const char *msg) {
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return code;
}
#endif

namespace {

constexpr int TP = 32;        // pixels per MFMA column block
constexpr int MAX_W2 = 2048;  // rows beyond 256 columns are swept in passes of 8 waves x 32 columns
constexpr int MAX_C = 1024;
constexpr int MAX_K = 8;
constexpr int KCH = 4;        // attention channels handled per launch

// Row of the 32x32 accumulator held in register r of a lane in half h (lane / 32).
__device__ __forceinline__ int vmap(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// 4 consecutive floats base[c..c+3], zero where out of range or !ok.
template <bool CVEC>
__device__ __forceinline__ v4f load4(const float *base, int c, int C, bool ok) {
    v4f x = {0.f, 0.f, 0.f, 0.f};
    if (ok) {
        if constexpr (CVEC) {
            if (c < C) x = *reinterpret_cast<const v4f *>(base + c);
        } else {
            if (c + 0 < C) x[0] = base[c + 0];
            if (c + 1 < C) x[1] = base[c + 1];
            if (c + 2 < C) x[2] = base[c + 2];
            if (c + 3 < C) x[3] = base[c + 3];
        }
    }
    return x;
}

template <bool CVEC>
__device__ __forceinline__ void store4(float *base, int c, int C, v4f x, bool accumulate) {
    if constexpr (CVEC) {
        if (c < C) {
            v4f *d = reinterpret_cast<v4f *>(base + c);
            if (accumulate) x += *d;
            *d = x;
        }
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (c + t < C) base[c + t] = accumulate ? base[c + t] + x[t] : x[t];
    }
}

// Raw buffer resource over `bytes` bytes at p: loads whose byte offset (voffset) is >= bytes return 0,
// which replaces every bounds branch in the fast paths.
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
// The descriptor must live in scalar registers; the pointer and size are wave-uniform by construction,
// and saying so explicitly keeps the compiler from emitting a per-lane search loop around every load.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, unsigned bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(p);
    const uint64_t lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)addr);
    const uint64_t hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(addr >> 32));
    const int n = __builtin_amdgcn_readfirstlane((int)bytes);
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((hi << 32) | lo), 0, n, 0x00020000);
}
__device__ __forceinline__ v4f buf_load4(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0));
}

constexpr unsigned DMA_OOB = 0x80000000u;   // a byte offset above every buffer size used here: reads as zero

// The same with a wave-uniform byte offset added by the hardware (it takes no part in the bounds check, so an
// out-of-range marker in byte_off stays one).
__device__ __forceinline__ v4f buf_load4s(__amdgpu_buffer_rsrc_t r, unsigned byte_off, unsigned uniform_off) {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, uniform_off, 0));
}

__device__ __forceinline__ float buf_load1s(__amdgpu_buffer_rsrc_t r, unsigned byte_off, unsigned uniform_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, uniform_off, 0));
}

// Data handed from one workgroup to another inside a kernel (pieces of a split tile).  The eight L2 caches of the
// chip are not coherent with each other, and a device-wide fence writes back and invalidates a whole L2; these
// 16-byte accesses carry the sc0 sc1 bits instead: they go through to the level all compute units share and leave
// the caches alone.
constexpr int CPOL_SC0_SC1 = 1 | 16;
__device__ __forceinline__ void store_shared4(__amdgpu_buffer_rsrc_t r, unsigned byte_off, v4f x) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, x), r, byte_off, 0, CPOL_SC0_SC1);
}
__device__ __forceinline__ v4f load_shared4(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, CPOL_SC0_SC1));
}

// The values the two halves of a wave (lanes 0-31, lanes 32-63) hold in x, handed to every lane: lo = the value of
// lane (l & 31), hi = the value of lane (l | 32).  One vector instruction, no trip through LDS.
__device__ __forceinline__ void wave_halves(float x, float &lo, float &hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

__device__ __forceinline__ v16f mfma(float a, float b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// Experimental contraction in three bf16 planes.  x = h + m + l with h = bf16(x), m = bf16(x - h), l = bf16(x - h - m)
// is exact for fp32 x (8 + 8 + 8 significant bits); the product of two such numbers is taken as
// hh + hm + mh + hl + lh + mm (what is dropped is below 2^-25 of the product) with six bf16 MFMAs that accumulate
// in fp32.  A bf16 MFMA has 16x the rate of the fp32 one here and, unlike it, leaves the vector lanes free.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
__device__ __forceinline__ void split8(const float (&x)[8], v8bf &h, v8bf &m, v8bf &l) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const __bf16 hh = (__bf16)x[e];
        const float r1 = x[e] - (float)hh;
        const __bf16 mm = (__bf16)r1;
        const float r2 = r1 - (float)mm;
        h[e] = hh; m[e] = mm; l[e] = (__bf16)r2;
    }
}
__device__ __forceinline__ v16f mfma_bf(v8bf a, v8bf b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
constexpr int BF_LSB = 264;   // bf16 per pixel row of an f1 plane in LDS (256 + 8: 16-byte reads hit distinct banks)
constexpr int BF_LS = 3 * BF_LSB / 2;   // the same in floats per pixel, all three planes
// fmap2 as bf16 planes in device memory (C == 256), ordered the way the sweep reads them: one 48 KB block per
// (image, row u, chunk of 32 columns), and inside it one KB per (32-channel block J, plane, k-step s2) holding the
// 16 bytes of each of the 64 lanes in lane order (lane = 32 h + column, channels 32J + 16h + 8 s2 + 0..7).  Every
// operand load of a wave is then one contiguous KB.  Rows are padded to whole chunks and to an even row count,
// the padding reads as zero.
constexpr unsigned BF_CHUNK = 8 * 6 * 1024;
__global__ void __launch_bounds__(256) split_planes_kernel(const float *__restrict__ f2, char *__restrict__ planes, int H2,
                                                           int W2, int H2p, int nvc, long nunits) {
    const long t = (long)blockIdx.x * 256 + threadIdx.x;   // one thread per lane and (J, s2) of a chunk
    if (t >= nunits) return;
    const int lane = (int)(t & 63), pl = lane & 31, h = lane >> 5;
    long r = t >> 6;
    const int s2 = (int)(r & 1), J = (int)((r >> 1) & 7);
    r >>= 4;                                                // chunk index = (b * H2p + u) * nvc + vc
    const int vc = (int)(r % nvc);
    const long bu = r / nvc;
    const int u = (int)(bu % H2p), v = 32 * vc + pl;
    const long b = bu / H2p;
    float xs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (u < H2 && v < W2) {
        const float *src = f2 + ((b * H2 + u) * W2 + v) * 256 + 32 * J + 16 * h + 8 * s2;
        const v4f x0 = *reinterpret_cast<const v4f *>(src), x1 = *reinterpret_cast<const v4f *>(src + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { xs[e] = x0[e]; xs[4 + e] = x1[e]; }
    }
    v8bf ph, pm, pl3;
    split8(xs, ph, pm, pl3);
    char *dst = planes + r * BF_CHUNK + (J * 6 + s2) * 1024 + lane * 16;   // KB index in a chunk: 6 J + 2 plane + s2
    *reinterpret_cast<v8bf *>(dst) = ph;
    *reinterpret_cast<v8bf *>(dst + 2048) = pm;
    *reinterpret_cast<v8bf *>(dst + 4096) = pl3;
}

// The same planes with the roles of pixel and channel exchanged, for contractions over fmap2 pixels (d_f1): one
// 48 KB block per (image, row u, chunk of 32 columns); inside it one KB per (16-column half s, 32-channel block cb,
// plane): lane 32 h + i holds channel 32 cb + i at the 8 columns 32 vc + 16 s + 8 h + 0..7.
__global__ void __launch_bounds__(256) split_planes_t_kernel(const float *__restrict__ f2, char *__restrict__ planes, int W2,
                                                             int nvc, long nunits) {
    const long t = (long)blockIdx.x * 256 + threadIdx.x;   // one thread per lane and (s, cb) of a chunk
    if (t >= nunits) return;
    const int lane = (int)(t & 63), i = lane & 31, h = lane >> 5;
    long r = t >> 6;
    const int cb = (int)(r & 7), s = (int)((r >> 3) & 1);
    r >>= 4;                                                // chunk index = (b * H2 + u) * nvc + vc
    const int vc = (int)(r % nvc);
    const long bu = r / nvc;
    const int v0 = 32 * vc + 16 * s + 8 * h;
    float xs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) xs[e] = v0 + e < W2 ? f2[(bu * W2 + v0 + e) * 256 + 32 * cb + i] : 0.f;
    v8bf ph, pm, pl3;
    split8(xs, ph, pm, pl3);
    char *dst = planes + r * BF_CHUNK + ((s * 8 + cb) * 3) * 1024 + lane * 16;
    *reinterpret_cast<v8bf *>(dst) = ph;
    *reinterpret_cast<v8bf *>(dst + 1024) = pm;
    *reinterpret_cast<v8bf *>(dst + 2048) = pl3;
}

// ------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------
// MODE_SOFT: MODE_WEIGHTED with the softmax inside (FwdArgs::logits / dlog); a mode of its own so that the plain
// weighted sweep carries none of its arguments
enum { MODE_MAXAVG = 0, MODE_ARGMAX = 1, MODE_WEIGHTED = 2, MODE_SOFT = 3 };
constexpr bool is_weighted(int mode) { return mode == MODE_WEIGHTED || mode == MODE_SOFT; }

// Gradient of a logit from the gradient x of its softmax output: a (x - dot), a = exp(z - max) / sum.
// row = index of the (pixel, channel) row, elem = index of the element in the row-major tensor.
__device__ __forceinline__ float dlogit(const float *__restrict__ z, const float *__restrict__ st, const float *__restrict__ dots,
                                        size_t row, size_t elem, float x) {
    return __expf(z[elem] - st[2 * row]) / st[2 * row + 1] * (x - dots[row]);
}
// the same with the row's (max, 1 / sum, dot) at hand
__device__ __forceinline__ float dlogit3(float z, const float *row3, float x) {
    return __expf(z - row3[0]) * row3[1] * (x - row3[2]);
}

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  This maps the
// hardware id to a logical one such that every XCD works on one contiguous range of logical ids: neighbours in
// the range (same batch image, same pixel split) stream the same operand rows through the same L2.
__device__ __forceinline__ int xcd_contiguous(int bid, int n) {
    const int c = bid & 7, slot = bid >> 3, q = n >> 3, r = n & 7;
    return c * q + (c < r ? c : r) + slot;
}
// The same for a grid of 512 workgroups that are resident two to a compute unit: an XCD hands its workgroups
// 0 .. 31 to its 32 compute units in turn and 32 .. 63 to the same units again, so the units hold the pairs
// (slot, slot + 32).  Here such a pair gets two neighbouring logical ids.  Shares of steps that are dealt out by
// logical id differ by one step in a fixed rhythm (2 2 2 3 ...): with neighbours on a unit every unit gets two
// steps more or less the same sum, where the plain order gave some units two long shares.  (Where the hardware
// places workgroups differently this costs nothing but the balance.)
__device__ __forceinline__ int xcd_paired(int bid) {
    const int c = bid & 7, slot = bid >> 3;
    return c * 64 + (slot < 32 ? 2 * slot : 2 * (slot - 32) + 1);
}

}  // namespace
namespace sepcorr_impl {
// What differs between the pyramid levels of fmap2 that one launch of a forward-type sweep can cover.
struct FwdLevel {
    const float *f2, *wv, *wu;
    float *out_u, *out_v;
    int *am_u, *am_v;
    const float *st_wv, *st_wu, *z_ou, *st_ou, *dot_ou, *z_ov, *st_ov, *dot_ov;   // softmax inside (see FwdArgs)
    int H2, W2;
    int nvc;           // column chunks of 32 = waves side by side; the other waves of the workgroup form row groups
    int steps, step0;  // units (steps, or half steps of two-row steps) of this level per tile, and of the levels before it
    int stage;
};
struct FwdArgs {
    const float *f1, *f2;
    const char *f2_planes;   // bf16-plane variant: fmap2 split by split_planes_kernel
    int H2p;                 //   its row count, padded to whole steps of all row groups
    const float *wv;   // MODE_WEIGHTED: weights indexed by v, (B,N1,KT,W2)
    const float *wu;   // MODE_WEIGHTED: weights indexed by u, (B,N1,KT,H2)
    float *out_u;      // (B,N1,CH,H2)
    float *out_v;      // (B,N1,CH,W2)
    int *am_u, *am_v;  // MODE_ARGMAX
    int N1, H2, W2, C, CP;
    int KT, k0;        // total weight channels and first channel of this launch
    int tiles_per_batch;
    int nvc;           // column chunks of 32 handled per pass = min(8, ceil(W2 / 32))
    int vpasses;       // passes of 256 columns = ceil(W2 / 256)
    int stage;         // collect the rows of out_u in LDS and store them coalesced at the end
    int xcd_order;     // map workgroup ids so that each XCD gets a contiguous range
    int pair_shares;   // dealt-out sweeps on 512 workgroups: the two workgroups of a compute unit get neighbouring shares
    // Work split finer than a pixel tile.  A tile's sweep is a sequence of steps (one step = the rows all waves of a
    // workgroup take in at once); the steps of all tiles, laid end to end, are dealt out evenly to the workgroups of
    // the grid.  A workgroup whose share ends inside a tile leaves the column state of its piece (max / argmax / sum
    // or the K sums over its rows) in a slot of sk_state; the piece that finishes a tile last adds up all pieces in
    // row order and writes the finished columns.  sk_total == 0: one whole tile per workgroup, no scratch.
    int sk_total;      // total steps over all tiles (0 = off)
    int sk_steps;      // steps per tile
    float *sk_state;   // [2 * gridDim.x] slots of sk_slot floats: first and last piece of every workgroup
    int *sk_count;     // [tiles] pieces finished, zero at launch
    int sk_slot;       // floats per slot
    void *ws;          // host side only: scratch for the split (NULL: whole tiles)
    size_t ws_bytes;
    // MODE_WEIGHTED with softmax inside.  Row statistics are (max, sum of exp) pairs per (pixel, channel) row.
    //   logits:  wv and wu hold logits, the weights are exp(z - max) / sum with the statistics st_wv, st_wu
    //            (attention compression straight from the logits)
    //   dlog:    the sums are gradients of softmax outputs; what is stored is the gradient of the logits,
    //            a (x - dot) with a = exp(z - max) / sum, for out_u rows from (z_ou, st_ou, dot_ou), for out_v
    //            columns from (z_ov, st_ov, dot_ov); dot = sum over the row of a * x, supplied by the caller
    int logits, dlog;
    const float *st_wv, *st_wu;
    const float *z_ou, *st_ou, *dot_ou, *z_ov, *st_ov, *dot_ov;
    // Several levels in one launch (split sweeps with row groups only): the steps of a tile are those of lev[0], then
    // of lev[1], ...; pieces are cut at level boundaries as well, and the image-1 tile is shared by all of them.
    int nlev;          // 0 or 1: one level, described by the fields above
    int tile_steps;    // steps of all levels of one tile
    int H2max;         // largest H2: the staged out_u rows of every level fit [32][channels][H2max]
    FwdLevel lev[4];
};
}  // namespace sepcorr_impl
namespace {

// CMODE: 0 = any C (scalar loads), 1 = C % 4 == 0 (16-byte loads), 2 = C % 32 == 0 (branch-free fast path),
//        3 = C == 256 (fast path with the channel loop unrolled: every load offset is an immediate)
// WM: 0 = one pass, one row group (both compile-time constants: the lean common case),
//     1 = row groups enabled (narrow rows), 2 = column passes enabled (rows wider than 256).
// BF: the experimental bf16-plane contraction (C == 256, one pass, one row group, max/avg modes)
// The kernel's argument block, read where the call stands: nothing loaded through the returned pointer can be moved
// ahead of this point, so values needed late in a kernel are not kept in scalar registers from its start.
typedef const __attribute__((address_space(4))) FwdArgs *KArgs;
__device__ __forceinline__ KArgs kernargs_now() {
    KArgs p = (KArgs)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(p));
    return p;
}

// The workgroups wfirst .. wlast that hold the steps [t0, t1) of a tile when sk_total steps are dealt out evenly to G
// workgroups (workgroup w holds the steps [w sk_total / G, (w + 1) sk_total / G)).
__device__ __forceinline__ void pieces_of(long t0, long t1, int G, int sk_total, int &wfirst, int &wlast) {
    wfirst = (int)((t0 * G) / sk_total);                           // the workgroup that holds step t0
    while (wfirst > 0 && ((long)wfirst * sk_total) / G > t0) --wfirst;
    while (((long)(wfirst + 1) * sk_total) / G <= t0) ++wfirst;
    wlast = wfirst;                                                  // the workgroup that holds step t1 - 1
    while (((long)(wlast + 1) * sk_total) / G < t1) ++wlast;
}

// The last piece of a tile to finish adds up the column state of all its pieces in row order (equal maxima keep the
// lower row) and writes the finished out_v columns.  A function of its own: its registers (the pieces of a batch are
// fetched together) are then allotted apart from those of the sweep.  Arguments are the same in every lane.
template <int MODE, int KC>
__device__ __attribute__((noinline)) void merge_pieces(KArgs ka_in, int lvl_in, int b_in, int p0_in, int wfirst_in, int wlast_in, int t0_in,
                                                       int tid) {
    const uint64_t kp64 = reinterpret_cast<uint64_t>(ka_in);
    const KArgs ka = reinterpret_cast<KArgs>(((uint64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)(kp64 >> 32)) << 32) |
                                             (unsigned)__builtin_amdgcn_readfirstlane((int)kp64));
    const int lvl = __builtin_amdgcn_readfirstlane(lvl_in), b = __builtin_amdgcn_readfirstlane(b_in);
    const int p0 = __builtin_amdgcn_readfirstlane(p0_in), wfirst = __builtin_amdgcn_readfirstlane(wfirst_in);
    const int wlast = __builtin_amdgcn_readfirstlane(wlast_in);
    const long t0 = __builtin_amdgcn_readfirstlane(t0_in);
    const int G = (int)gridDim.x, sk_total = ka->sk_total, N1 = ka->N1;
    const int H2 = ka->lev[lvl].H2, W2 = ka->lev[lvl].W2;
    const bool soft_dlog = MODE == MODE_SOFT && ka->dlog;
    (void)soft_dlog;
    // Add up the pieces in row order (equal maxima keep the lower row) and write the finished columns.
    // An item = the 4 consecutive columns a lane holds in one register group of one column chunk.
    constexpr int NQ = (is_weighted(MODE)) ? KC : 3;
    const __amdgpu_buffer_rsrc_t rs_sk = make_rsrc(ka->sk_state, 2u * gridDim.x * (unsigned)ka->sk_slot * 4u);
    const int nchunks = (W2 + 31) >> 5;
    const int total = nchunks * 256;
    constexpr int PB = 4;   // pieces fetched together (a tile rarely has more)
    // items of a thread in flight together, their slot reads waiting side by side (one where four quantities per
    // piece would take the registers of the sweep)
    constexpr int IU = NQ <= 3 ? 2 : 1;
    for (int it0 = tid; it0 < total; it0 += IU * (int)blockDim.x) {
        v4f acc4[IU][NQ];
#pragma unroll
        for (int i = 0; i < IU; ++i) {
#pragma unroll
            for (int q = 0; q < NQ; ++q) acc4[i][q] = v4f{0.f, 0.f, 0.f, 0.f};
            if constexpr (!is_weighted(MODE)) acc4[i][0] = v4f{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        }
        for (int w0 = wfirst; w0 <= wlast; w0 += PB) {
            v4f x[IU][PB][NQ];
            unsigned slot[PB];
#pragma unroll
            for (int j = 0; j < PB; ++j) {
                const int w = w0 + j;
                const bool first_piece = ((long)w * sk_total) / G >= t0;   // w's share starts inside this tile
                slot[j] = (unsigned)(2 * w + (first_piece ? 0 : 1)) * (unsigned)ka->sk_slot;
            }
#pragma unroll
            for (int i = 0; i < IU; ++i) {
                const int it = it0 + i * (int)blockDim.x;
                const int ln = it & 63, g4 = (it >> 6) & 3, chunk = it >> 8;
                if (it < total) {
#pragma unroll
                    for (int j = 0; j < PB; ++j) {
                        const unsigned base = (slot[j] + (unsigned)chunk * (NQ * 1024u) + 4u * ln) * 4u;
                        if (w0 + j <= wlast) {
#pragma unroll
                            for (int q = 0; q < NQ; ++q) x[i][j][q] = load_shared4(rs_sk, base + (unsigned)(q * 4 + g4) * 1024u);
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < IU; ++i) {
                if (it0 + i * (int)blockDim.x >= total) break;
#pragma unroll
                for (int j = 0; j < PB; ++j) {
                    if (w0 + j > wlast) break;
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int q = 0; q < NQ; ++q) acc4[i][q] += x[i][j][q];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            // (equal maxima keep the lower row: the rows of two neighbouring pieces may alternate)
                            if (x[i][j][0][e] > acc4[i][0][e] ||
                                (x[i][j][0][e] == acc4[i][0][e] && __float_as_int(x[i][j][1][e]) < __float_as_int(acc4[i][1][e]))) {
                                acc4[i][0][e] = x[i][j][0][e];
                                acc4[i][1][e] = x[i][j][1][e];
                            }
                        acc4[i][2] += x[i][j][2];
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < IU; ++i) {
            const int it = it0 + i * (int)blockDim.x;
            if (it >= total) break;
            const int ln = it & 63, g4 = (it >> 6) & 3, chunk = it >> 8;
            const int p = ln & 31, v = 32 * chunk + vmap(4 * g4, ln >> 5);
            if (p0 + p >= N1) continue;
            const size_t o = (size_t)b * N1 + p0 + p;
            if constexpr (is_weighted(MODE)) {
                if (soft_dlog) {   // sums of softmax-output gradients -> gradients of the logits
                    float r3[NQ][3], z[NQ][4];
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        const size_t row = o * ka->KT + ka->k0 + q;
                        r3[q][0] = ka->lev[lvl].st_ov[2 * row]; r3[q][1] = ka->lev[lvl].st_ov[2 * row + 1]; r3[q][2] = ka->lev[lvl].dot_ov[row];
#pragma unroll
                        for (int e = 0; e < 4; ++e) z[q][e] = v + e < W2 ? ka->lev[lvl].z_ov[row * W2 + v + e] : 0.f;
                    }
#pragma unroll
                    for (int q = 0; q < NQ; ++q) {
                        r3[q][1] = 1.f / r3[q][1];
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc4[i][q][e] = dlogit3(z[q][e], r3[q], acc4[i][q][e]);
                    }
                }
            }
            bool vec = (W2 & 3) == 0 && (reinterpret_cast<uintptr_t>(ka->lev[lvl].out_v) & 15) == 0;
            if constexpr (MODE == MODE_ARGMAX) vec = vec && (reinterpret_cast<uintptr_t>(ka->lev[lvl].am_v) & 15) == 0;
            if (vec) {
                if (v < W2) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int q = 0; q < NQ; ++q) *reinterpret_cast<v4f *>(ka->lev[lvl].out_v + (o * ka->KT + ka->k0 + q) * W2 + v) = acc4[i][q];
                    } else {
                        *reinterpret_cast<v4f *>(ka->lev[lvl].out_v + (o * 2 + 0) * W2 + v) = acc4[i][0];
                        *reinterpret_cast<v4f *>(ka->lev[lvl].out_v + (o * 2 + 1) * W2 + v) = acc4[i][2] / (float)H2;
                        if constexpr (MODE == MODE_ARGMAX)   // (the indices travel as the bit patterns of floats)
                            *reinterpret_cast<v4f *>(ka->lev[lvl].am_v + o * W2 + v) = acc4[i][1];
                    }
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (v + e >= W2) break;
                if constexpr (is_weighted(MODE)) {
#pragma unroll
                    for (int q = 0; q < NQ; ++q) ka->lev[lvl].out_v[(o * ka->KT + ka->k0 + q) * W2 + v + e] = acc4[i][q][e];
                } else {
                    ka->lev[lvl].out_v[(o * 2 + 0) * W2 + v + e] = acc4[i][0][e];
                    ka->lev[lvl].out_v[(o * 2 + 1) * W2 + v + e] = acc4[i][2][e] / (float)H2;
                    if constexpr (MODE == MODE_ARGMAX) ka->lev[lvl].am_v[o * W2 + v + e] = __float_as_int(acc4[i][1][e]);
                }
            }
        }
    }
}

// SK: the sweep may be dealt out in pieces of tiles (FwdArgs::sk_total); without it the loop over pieces below runs
// exactly once with compile-time bounds and costs nothing
template <int MODE, int KC, int UR, int CMODE, int WM, bool BF = false, bool SK = false>
__global__ void __launch_bounds__(512) fwd_kernel(const FwdArgs a) {
    static_assert(!BF || (CMODE == 3 && WM <= 1), "bf16 planes: C == 256, one column pass");
    static_assert(!(BF && SK), "the split is not built for the bf16-plane variant");
    const int sk_total = SK ? a.sk_total : 0;
    const bool soft_logits = MODE == MODE_SOFT && a.logits, soft_dlog = MODE == MODE_SOFT && a.dlog;
    constexpr bool CVEC = CMODE >= 1;
    constexpr int GJ = 2;  // 8-channel slices per prefetch group
    constexpr int NPART = (is_weighted(MODE)) ? KC : 3;
    extern __shared__ float smem[];
    const int nW = blockDim.x >> 6;
    // Waves form a grid: nvc column chunks x NUG row groups.  Wave (vcw, ug) owns columns [32 vcw, 32 vcw + 32)
    // and the steps ug, ug + NUG, ... (narrow fmap2 levels have few column chunks; row groups keep the
    // workgroup at 4 or 8 waves).  NUG == 1 for rows of 97 or more columns.
    constexpr bool RG = WM == 1;
    constexpr bool ML = SK && WM == 1;   // may cover several pyramid levels
    const bool multi = ML && a.nlev > 1;
    const int vpasses = (WM == 2) ? a.vpasses : 1;
    const int wg = !a.xcd_order ? (int)blockIdx.x
                   : (SK && a.pair_shares) ? xcd_paired(blockIdx.x) : xcd_contiguous(blockIdx.x, gridDim.x);
    const int N1 = a.N1, C = a.C;
    const int LS = BF ? BF_LS : a.CP + 4;
    float *f1s = smem;
    __bf16 *f1b = reinterpret_cast<__bf16 *>(smem);   // BF: [plane][TP][BF_LSB]
    float *part = smem + TP * LS;
    constexpr int NCHO = (is_weighted(MODE)) ? KC : 2;            // out_u channels of this launch
    float *ostage = part + 2 * UR * NPART * (blockDim.x >> 6) * 32;   // [32 p][NCHO][H2] when a.stage
    int *ostage_am = reinterpret_cast<int *>(ostage + TP * NCHO * a.H2max);   // [32 p][H2], MODE_ARGMAX
    // MODE_WEIGHTED with softmax inside: per (pixel, channel) row of the u-indexed tensor (max, 1 / sum) of the
    // logits that are the weights [32 p][KC][2], or (max, 1 / sum, dot) of the logits whose gradient is stored [..][3]
    float *cst = ostage + (a.stage ? TP * NCHO * a.H2max : 0);

    // This workgroup's share of the steps of all tiles: [gs0, gs_end).  Without the split it is exactly one tile.
    // A share is cut into pieces at tile boundaries.  When it ends inside a tile, that last piece (which starts at
    // the tile's row 0) is done first and the others follow in order: every workgroup of the grid then starts at
    // row 0 and all of them move down the rows of fmap2 together, so that a row is fetched into an L2 once.
    // (With several levels a unit is one level of one tile, a tile's steps being those of all its levels in turn.)
    const int S = sk_total ? (multi ? a.tile_steps : a.sk_steps) : 1;
    // the unit that holds step g: its first step, one past its last, its level
    auto unit_of = [&](int g, int &ubeg, int &uend) {
        const int t = g / S;
        int lv = 0, s0 = 0, s1 = S;
        if (multi) {
            const int r = g - t * S;
            for (lv = a.nlev - 1; lv > 0 && a.lev[lv].step0 > r; --lv) {}
            s0 = a.lev[lv].step0;
            s1 = s0 + a.lev[lv].steps;
        }
        ubeg = t * S + s0;
        uend = t * S + s1;
        return lv;
    };
    const int gs0 = sk_total ? (int)(((long)wg * sk_total) / (int)gridDim.x) : wg;
    const int gs_end = sk_total ? (int)(((long)(wg + 1) * sk_total) / (int)gridDim.x) : wg + 1;
    int head = 0;                                       // steps of the piece at the end of the share
    {
        int ub, ue;
        unit_of(gs_end - 1, ub, ue);
        if (ue != gs_end && ub > gs0) head = gs_end - ub;   // (no head: the share ends with a unit, or lies inside one)
    }
    const int body_end = gs_end - head;
    int cur = gs0;
    for (int seg_no = 0;; ++seg_no) {
    int pb, pe, ubeg, uend;                             // this piece: steps [pb, pe) of all tiles laid end to end
    if (seg_no == 0 && head) {
        pb = body_end; pe = gs_end;
    } else {
        if (cur >= body_end) break;
        pb = cur;
    }
    const int lvl_dyn = unit_of(pb, ubeg, uend);
    const int lvl = ML ? lvl_dyn : 0;
    if (!(seg_no == 0 && head)) {
        pe = min(body_end, uend);
        cur = pe;
    }
    // Lane indices are derived from the thread id piece by piece (and once more behind the sweep): values that lived
    // from the start of the kernel to its end would be the first to be moved out of registers, and the sweep uses them.
    int tid = threadIdx.x;
    if constexpr (SK) asm volatile("" : "+v"(tid));
    const int wave = tid >> 6, lane = tid & 63, pl = lane & 31, h = lane >> 5;
    const int tile = pb / S;
    // What is dealt out.  With one row per step and wave (UR == 1) it is steps.  With two (UR == 2) it is half steps:
    // the first rows of all waves' steps, then their second rows.  Half step hs of a tile holds the rows
    // ((hs / 2) NUG + ug) 2 + hs % 2 of the waves' row groups ug.  A piece [sa, sb) takes them two at a time, whatever
    // the parity of sa, and when their number is odd its last step has one row per wave: that step's matrix
    // instructions for the second row are left out, not masked.  (Whole steps cost the small grids a quarter of the
    // chip: 2.25 steps of 8 rows per workgroup at B=1, 48x64 mean 3 for one workgroup in four.)  Only the form without
    // row groups does this (rows of 97 to 256 columns): with row groups it measured slower (B=1, 48x64: 0.078 against
    // 0.0745 ms; B=4, 48x64, where whole steps already divide evenly: 0.197 against 0.193 ms), without them faster
    // (B=2, 55x128: 0.423 against 0.440 ms, of which 1.8 % is the 56th row that is no longer multiplied).
    constexpr int HU = (SK && UR == 2 && WM == 0) ? 2 : 1;
    const int sa = pb - ubeg;                           // first unit of this piece within its tile (and level)
    const int sb = pe - ubeg;                           // one past its last unit
    const bool whole = !SK || !sk_total || (pb == ubeg && pe == uend);
    const int b = tile / a.tiles_per_batch;
    const int p0 = (tile % a.tiles_per_batch) * TP;
    // This piece's level: lev[lvl] (a launch of one level describes it in lev[0]).  Pointers that only the code
    // before or only the code behind the sweep uses are read from the kernel arguments there and then
    // (kernargs_now), so that they do not hold scalar registers during the sweep.
    const int H2 = a.lev[lvl].H2, W2 = a.lev[lvl].W2;
    const bool Lstage = a.lev[lvl].stage;
    const float *Lf2 = a.lev[lvl].f2, *Lwu = a.lev[lvl].wu;
    const int nvc = RG ? a.lev[lvl].nvc : nW, NUG = RG ? nW / nvc : 1;
    const int vcw = RG ? wave % nvc : wave, ug = RG ? wave / nvc : 0;
    // row r of step `step` of the waves in row group g, and whether this piece owns it
    auto row_of = [&](int step, int r, int g) {
        if constexpr (HU == 2) {
            const int hs = sa + 2 * step + r;
            return ((hs >> 1) * NUG + g) * 2 + (hs & 1);
        } else {
            return ((sa + step) * NUG + g) * UR + r;
        }
    };
    auto row_on = [&](int step, int r) { return HU == 1 || sa + 2 * step + r < sb; };
    if (seg_no > 0) __syncthreads();   // the previous piece has finished with LDS
    const KArgs kp = kernargs_now();

    if constexpr (is_weighted(MODE)) {
        if (soft_logits) {   // (max, 1 / sum) of the rows of u-indexed logits of this tile's pixels
            for (int idx = tid; idx < TP * KC; idx += blockDim.x) {
                const int p = idx / KC, kk = idx - p * KC;
                const size_t row = ((size_t)b * N1 + min(p0 + p, N1 - 1)) * a.KT + a.k0 + kk;
                cst[2 * idx] = kp->lev[lvl].st_wu[2 * row];
                cst[2 * idx + 1] = 1.f / kp->lev[lvl].st_wu[2 * row + 1];
            }
        }
        if (soft_dlog) {
            for (int idx = tid; idx < TP * KC; idx += blockDim.x) {
                const int p = idx / KC, kk = idx - p * KC;
                const size_t row = ((size_t)b * N1 + min(p0 + p, N1 - 1)) * a.KT + a.k0 + kk;
                cst[3 * idx] = kp->lev[lvl].st_ou[2 * row];
                cst[3 * idx + 1] = 1.f / kp->lev[lvl].st_ou[2 * row + 1];
                cst[3 * idx + 2] = kp->lev[lvl].dot_ou[row];
            }
        }
    }
    {   // stage the f1 tile [TP][CP] (zero padded) into LDS
        const int c4n = CMODE == 3 ? 64 : a.CP >> 2;
        if constexpr (!BF) {   // all loads of a batch in flight before the first LDS write
            constexpr int SU = 8;
            for (int base = tid; base < TP * c4n; base += SU * blockDim.x) {
                v4f x[SU];
                int dst[SU];
#pragma unroll
                for (int t = 0; t < SU; ++t) {
                    const int idx = base + t * blockDim.x;
                    const int row = idx / c4n, c = (idx - row * c4n) * 4;
                    const bool in = idx < TP * c4n, ok = in && p0 + row < N1;
                    const float *src = kp->f1 + ((size_t)b * N1 + (ok ? p0 + row : 0)) * C;
                    dst[t] = in ? row * LS + c : -1;
                    x[t] = load4<CVEC>(src, c, C, ok);
                }
#pragma unroll
                for (int t = 0; t < SU; ++t)
                    if (dst[t] >= 0) *reinterpret_cast<v4f *>(f1s + dst[t]) = x[t];
            }
        }
        for (int idx = tid; BF && idx < TP * c4n; idx += blockDim.x) {
            const int row = idx / c4n, c = (idx - row * c4n) * 4;
            const bool ok = p0 + row < N1;
            const float *src = kp->f1 + ((size_t)b * N1 + (ok ? p0 + row : 0)) * C;
            const v4f x = load4<CVEC>(src, c, C, ok);
            if constexpr (BF) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const __bf16 hh = (__bf16)x[e];
                    const float r1 = x[e] - (float)hh;
                    const __bf16 mm = (__bf16)r1;
                    f1b[(0 * TP + row) * BF_LSB + c + e] = hh;
                    f1b[(1 * TP + row) * BF_LSB + c + e] = mm;
                    f1b[(2 * TP + row) * BF_LSB + c + e] = (__bf16)(r1 - (float)mm);
                }
            } else {
                *reinterpret_cast<v4f *>(f1s + row * LS + c) = x;
            }
        }
    }
    __syncthreads();

    const int pix = p0 + pl;           // this lane's image-1 pixel
    const bool pok = pix < N1;
    const size_t bp = (size_t)b * N1 + (pok ? pix : 0);
    // Rows wider than 256 columns are swept in passes of 256 columns; a pass merges its out_u rows with
    // what the earlier passes left (same thread, same address), the out_v columns of a pass are its own.
    // Whether this piece, finding every other piece of its tile already in its slot, took them into its own registers
    // and finished the tile itself (below).
    bool merged_here = false;
    for (int vp = 0; vp < vpasses; ++vp) {
    if (vp > 0) __syncthreads();   // the previous pass has finished with the LDS partial buffers
    const int vbase = (WM == 2) ? vp * 256 : 0;
    const int vrow = vbase + 32 * vcw + pl;   // the fmap2 column this lane feeds to the A operand
    const bool vrow_ok = vrow < W2;
    const float *f2lane = Lf2 + ((size_t)b * H2 * W2 + (vrow_ok ? vrow : 0)) * C;
    const size_t rowstride = (size_t)W2 * C;

    const bool ragged = vbase + 32 * vcw + 32 > W2;
    unsigned vmask = 0;  // bit r: accumulator register r maps to a real column
#pragma unroll
    for (int r = 0; r < 16; ++r)
        if (vbase + 32 * vcw + vmap(r, h) < W2) vmask |= 1u << r;

    // running state over u, accumulator layout
    float vmax[16], vsum[16];
    int vidx[16];
    float wvr[KC][16], rv[KC][16];
    if constexpr (is_weighted(MODE)) {
        // registers 4g..4g+3 hold four consecutive columns: one 16-byte load each where rows of wv are 16-byte aligned
        const bool wv16 = (W2 & 3) == 0 && (reinterpret_cast<uintptr_t>(kp->lev[lvl].wv) & 15) == 0;
#pragma unroll
        for (int k = 0; k < KC; ++k) {
#pragma unroll
            for (int r = 0; r < 16; ++r) rv[k][r] = 0.f;
            if (wv16) {   // one offset register per group of four columns; the channel travels in the scalar offset
                const __amdgpu_buffer_rsrc_t rs = make_rsrc(kp->lev[lvl].wv + (size_t)b * N1 * a.KT * W2, (unsigned)N1 * a.KT * W2 * 4u);
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const int v = vbase + 32 * vcw + vmap(4 * g4, h);
                    const unsigned o = (pok && v < W2) ? (unsigned)((pix * a.KT + a.k0) * W2 + v) * 4u : DMA_OOB;
                    const v4f x = buf_load4s(rs, o, (unsigned)(k * W2) * 4u);
#pragma unroll
                    for (int e = 0; e < 4; ++e) wvr[k][4 * g4 + e] = x[e];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int v = vbase + 32 * vcw + vmap(r, h);
                    wvr[k][r] = (pok && v < W2) ? kp->lev[lvl].wv[(bp * a.KT + a.k0 + k) * W2 + v] : 0.f;
                }
            }
        }
        if (soft_logits) {
#pragma unroll
            for (int k = 0; k < KC; ++k) {
                const size_t row = bp * a.KT + a.k0 + k;
                const float m = kp->lev[lvl].st_wv[2 * row], il = 1.f / kp->lev[lvl].st_wv[2 * row + 1];
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    wvr[k][r] = (pok && vbase + 32 * vcw + vmap(r, h) < W2) ? __expf(wvr[k][r] - m) * il : 0.f;
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            vmax[r] = -INFINITY;
            vsum[r] = 0.f;
            vidx[r] = 0;
        }
    }
    const int NJ = a.CP >> 3;
    const int NG = (NJ + GJ - 1) / GJ;
    const int nsteps = sk_total ? (sb - sa + HU - 1) / HU : ((H2 + UR - 1) / UR + NUG - 1) / NUG;   // steps per wave; rows past H2 are skipped
    const bool tail_single = HU == 2 && ((sb - sa) & 1);   // the last step has one row per wave
    const int T = nsteps * NG;

    v16f acc[UR];
#pragma unroll
    for (int r = 0; r < UR; ++r)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[r][e] = 0.f;

    float wur[UR][KC];  // MODE_WEIGHTED: u-indexed weights of the rows of the current step

    auto issue = [&](int step, int g, v4f(&buf)[UR][GJ]) {
#pragma unroll
        for (int r = 0; r < UR; ++r) {
            const int u = row_of(step, r, ug);
#pragma unroll
            for (int jj = 0; jj < GJ; ++jj) {
                const int j = g * GJ + jj;
                buf[r][jj] = load4<CVEC>(f2lane + (size_t)(u < H2 ? u : 0) * rowstride, 8 * j + 4 * h, C,
                                         vrow_ok && u < H2 && j < NJ);
            }
        }
    };

    // Cross-wave combination of a step's partial results (wave order) into the finished out_u rows.  The partials
    // of step s lie in part[s & 1][wave][row of the step][quantity][32 pixels].
    auto combine = [&](int step) {
        const float *pbr = part + (step & 1) * (UR * NPART * nW * 32);
        constexpr int WSTR = UR * NPART * 32;   // floats per wave
        if constexpr (is_weighted(MODE)) {
            for (int idx = tid; idx < NUG * UR * KC * 32; idx += blockDim.x) {
                const int p = idx & 31, k = (idx >> 5) % KC, ru = (idx / (32 * KC)) % UR, g2 = idx / (32 * KC * UR);
                const int u = row_of(step, ru, g2);
                if (u < H2 && row_on(step, ru) && p0 + p < N1) {
                    const float *src = pbr + (g2 * nvc) * WSTR + (ru * NPART + k) * 32 + p;
                    float x[8];   // all reads before the first addition
#pragma unroll
                    for (int j = 0; j < 4; ++j) x[j] = j < nvc ? src[j * WSTR] : 0.f;
#pragma unroll
                    for (int j = 4; j < 8; ++j) x[j] = 0.f;
                    if (nvc > 4) {
#pragma unroll
                        for (int j = 4; j < 8; ++j) x[j] = j < nvc ? src[j * WSTR] : 0.f;
                    }
                    float s = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) s += x[j];
                    // (LDS and global destinations are kept in separate branches: a pointer that may be either
                    // turns into FLAT accesses, whose counters force every later wait to zero)
                    if (Lstage) {
                        float *dst = &ostage[(p * NCHO + k) * H2 + u];
                        if (vp > 0) s += *dst;   // earlier column passes, written by this same thread
                        *dst = s;
                    } else {
                        const size_t row = ((size_t)b * N1 + p0 + p) * a.KT + a.k0 + k;
                        float *dst = &a.lev[lvl].out_u[row * H2 + u];
                        if (vp > 0) s += *dst;
                        if (soft_dlog && vp == vpasses - 1) s = dlogit3(a.lev[lvl].z_ou[row * H2 + u], cst + 3 * (p * KC + k), s);
                        *dst = s;
                    }
                }
            }
        } else {
            for (int idx = tid; idx < NUG * UR * 32; idx += blockDim.x) {
                const int p = idx & 31, ru = (idx >> 5) % UR, g2 = idx / (32 * UR);
                const int u = row_of(step, ru, g2);
                if (u < H2 && row_on(step, ru) && p0 + p < N1) {
                    const float *src = pbr + (g2 * nvc) * WSTR + (ru * NPART) * 32 + p;
                    float xm[8], xi[8], xs[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        xm[j] = -INFINITY; xi[j] = 0.f; xs[j] = 0.f;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (j < nvc) { xm[j] = src[j * WSTR]; xi[j] = src[j * WSTR + 32]; xs[j] = src[j * WSTR + 64]; }
                    if (nvc > 4) {
#pragma unroll
                        for (int j = 4; j < 8; ++j)
                            if (j < nvc) { xm[j] = src[j * WSTR]; xi[j] = src[j * WSTR + 32]; xs[j] = src[j * WSTR + 64]; }
                    }
                    float m = xm[0], s = xs[0];
                    int mi = __float_as_int(xi[0]);
#pragma unroll
                    for (int j = 1; j < 8; ++j) {
                        if (xm[j] > m) { m = xm[j]; mi = __float_as_int(xi[j]); }
                        s += xs[j];
                    }
                    const bool last = vp == vpasses - 1;   // the running sum is kept until the last pass
                    if (Lstage) {
                        float *dm = &ostage[(p * 2 + 0) * H2 + u], *ds = &ostage[(p * 2 + 1) * H2 + u];
                        int *di = &ostage_am[p * H2 + u];
                        if (vp > 0) {   // merge with the earlier column passes (lower v: they win ties)
                            const float pm = *dm;
                            s += *ds;
                            if (!(m > pm)) { m = pm; if constexpr (MODE == MODE_ARGMAX) mi = *di; }
                        }
                        *dm = m;
                        *ds = last ? s / (float)W2 : s;
                        if constexpr (MODE == MODE_ARGMAX) *di = mi;
                    } else {
                        const size_t o = ((size_t)b * N1 + p0 + p);
                        float *dm = &a.lev[lvl].out_u[(o * 2 + 0) * H2 + u], *ds = &a.lev[lvl].out_u[(o * 2 + 1) * H2 + u];
                        if (vp > 0) {
                            const float pm = *dm;
                            s += *ds;
                            if (!(m > pm)) { m = pm; if constexpr (MODE == MODE_ARGMAX) mi = a.lev[lvl].am_u[o * H2 + u]; }
                        }
                        *dm = m;
                        *ds = last ? s / (float)W2 : s;
                        if constexpr (MODE == MODE_ARGMAX) a.lev[lvl].am_u[o * H2 + u] = mi;
                    }
                }
            }
        }
    };

    // The end of a step: every wave reduces its 32 columns of the step's rows and leaves the partial results in LDS
    // (both halves of a wave hold the same values and write them to the same place), one barrier.  With `defer` the
    // caller runs combine(step) later (during the next step, where its LDS latency hides behind matrix work).
    auto epilogue = [&](int step, bool defer = false) {
        float *pb = part + (step & 1) * (UR * NPART * nW * 32) + wave * (UR * NPART * 32) + pl;
#pragma unroll
        for (int ru = 0; ru < UR; ++ru) {
            const int u = row_of(step, ru, ug);
            if (u < H2 && row_on(step, ru)) {
                if constexpr (is_weighted(MODE)) {
                    float sk[KC];
#pragma unroll
                    for (int k = 0; k < KC; ++k) {
                        float s = 0.f;
#pragma unroll
                        for (int r = 0; r < 16; ++r) s += acc[ru][r] * wvr[k][r];
                        sk[k] = s;
                    }
#pragma unroll
                    for (int k = 0; k < KC; ++k) {
                        float lo, hi;
                        wave_halves(sk[k], lo, hi);
                        pb[(ru * NPART + k) * 32] = lo + hi;
                    }
#pragma unroll
                    for (int k = 0; k < KC; ++k) {
                        const float w = wur[ru][k];
#pragma unroll
                        for (int r = 0; r < 16; ++r) rv[k][r] += acc[ru][r] * w;
                    }
                } else {
                    float m = -INFINITY, s = 0.f;
                    // starts at the lane's first column: a row without any finite value above -inf (all NaN or
                    // -inf) then ends up with index 0, as the reference's pre-zeroed argmax does
                    int mi = vbase + 32 * vcw + 4 * h;
                    if (ragged) {   // wave-uniform: only the last column chunk of a row can be partial
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float xm = ((vmask >> r) & 1u) ? acc[ru][r] : -INFINITY;
                            if (xm > m) { m = xm; mi = vbase + 32 * vcw + vmap(r, h); }
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float xm = acc[ru][r];
                            if (xm > m) { m = xm; mi = vbase + 32 * vcw + vmap(r, h); }
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const float x = acc[ru][r];
                        s += x;  // columns outside the image hold exact zeros
                        if (x > vmax[r]) { vmax[r] = x; vidx[r] = u; }
                        vsum[r] += x;
                    }
                    float m_lo, m_hi, i_lo, i_hi, s_lo, s_hi;
                    wave_halves(m, m_lo, m_hi);
                    wave_halves(__int_as_float(mi), i_lo, i_hi);
                    wave_halves(s, s_lo, s_hi);
                    const bool take_hi = m_hi > m_lo || (m_hi == m_lo && __float_as_int(i_hi) < __float_as_int(i_lo));
                    pb[(ru * NPART + 0) * 32] = take_hi ? m_hi : m_lo;
                    pb[(ru * NPART + 1) * 32] = take_hi ? i_hi : i_lo;
                    pb[(ru * NPART + 2) * 32] = s_lo + s_hi;
                }
            }
            if constexpr (CMODE != 3) {
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[ru][e] = 0.f;
            }
        }
        __syncthreads();
        if (!defer) combine(step);
    };

    auto compute = [&](int step, int g, v4f(&buf)[UR][GJ]) {
        if constexpr (is_weighted(MODE)) {
            if (g == 0) {
#pragma unroll
                for (int r = 0; r < UR; ++r) {
                    const int u = row_of(step, r, ug);
#pragma unroll
                    for (int k = 0; k < KC; ++k)
                    {
                        wur[r][k] = (pok && u < H2) ? Lwu[(bp * a.KT + a.k0 + k) * H2 + u] : 0.f;
                        if (soft_logits) wur[r][k] = __expf(wur[r][k] - cst[2 * (pl * KC + k)]) * cst[2 * (pl * KC + k) + 1];
                    }
                }
            }
        }
#pragma unroll
        for (int jj = 0; jj < GJ; ++jj) {
            const int j = g * GJ + jj;
            if (j < NJ) {
                const v4f bv = *reinterpret_cast<const v4f *>(f1s + pl * LS + 8 * j + 4 * h);
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int r = 0; r < UR; ++r) acc[r] = mfma(buf[r][jj][t], bv[t], acc[r]);
            }
        }
        if (g == NG - 1) epilogue(step);
    };

    if constexpr (BF) {
        // bf16 planes: per 32-channel block and row, six 16-byte loads (plane x k-step) feed twelve MFMAs of two rows
        const int nvcp = (W2 + 31) >> 5, H2p = a.H2p;
        const unsigned rowbytes = (unsigned)nvcp * BF_CHUNK;
        const unsigned nbytes = (unsigned)H2p * rowbytes;
        const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(a.f2_planes + (size_t)b * nbytes, nbytes);
        const unsigned lane_off = (unsigned)vcw * BF_CHUNK + 16u * lane;
        const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        v4f ring[2][UR][6];
        auto issueB = [&](int step, int J, v4f(&buf)[UR][6]) {
#pragma unroll
            for (int r = 0; r < UR; ++r) {
                const unsigned row = (unsigned)row_of(step, r, ug) * rowbytes;   // wave-uniform: travels in a scalar register
#pragma unroll
                for (int i = 0; i < 6; ++i) buf[r][i] = buf_load4s(rsrc, lane_off, row + (unsigned)(J * 6 + i) * 1024u);   // i = 2 plane + k-step
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        auto computeB = [&](int step, int J, v4f(&buf)[UR][6]) {
            if constexpr (is_weighted(MODE)) {
                if (J == 0) {
#pragma unroll
                    for (int r = 0; r < UR; ++r) {
                        const int u = min(row_of(step, r, ug), H2 - 1);
#pragma unroll
                        for (int k = 0; k < KC; ++k) wur[r][k] = Lwu[(bp * a.KT + a.k0 + k) * H2 + u];
                    }
                }
            }
            const __bf16 *bb = f1b + pl * BF_LSB + 32 * J + 16 * h;
            v8bf bq[3][2];
#pragma unroll
            for (int q = 0; q < 3; ++q)
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2) bq[q][s2] = *reinterpret_cast<const v8bf *>(bb + q * TP * BF_LSB + 8 * s2);
            // plane pairs (f2, f1) in the order of growing magnitude: l.h, h.l, m.m, m.h, h.m, h.h
            constexpr int PA[6] = {2, 0, 1, 1, 0, 0}, PB[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                for (int t = 0; t < 6; ++t)
#pragma unroll
                    for (int r = 0; r < UR; ++r) {
                        const bool first = J == 0 && s2 == 0 && t == 0;
                        acc[r] = mfma_bf(__builtin_bit_cast(v8bf, buf[r][2 * PA[t] + s2]), bq[PB[t]][s2], first ? zero16 : acc[r]);
                    }
            __builtin_amdgcn_sched_barrier(0);
            if (J == 7) epilogue(step);
        };
        issueB(0, 0, ring[0]);
        for (int step = 0; step < nsteps; ++step) {
#pragma unroll
            for (int J = 0; J < 8; ++J) {
                if (J + 1 < 8) issueB(step, J + 1, ring[(J + 1) & 1]);
                else if (step + 1 < nsteps) issueB(step + 1, 0, ring[0]);
                computeB(step, J, ring[J & 1]);
            }
        }
    } else if constexpr (CMODE >= 2) {
        // Fast path.  Contraction index permuted so that a lane reads 64 contiguous bytes of its fmap2
        // pixel per 32-channel block J: MFMA step (tq,t) of block J contracts channels 32J+4tq+t (lanes
        // 0..31) and 32J+16+4tq+t (lanes 32..63); the f1 tile in LDS is read with the same mapping.
        const unsigned rowbytes = (unsigned)W2 * C * 4u;
        const unsigned nbytes = (unsigned)H2 * rowbytes;
        const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(Lf2 + (size_t)b * H2 * W2 * C, nbytes);
        const unsigned lane_off = vrow_ok ? ((unsigned)vrow * C + 16u * h) * 4u : nbytes;
        const int NJB = (CMODE == 3) ? 8 : (C >> 5);
        constexpr bool HEAVY = is_weighted(MODE) && KC >= 3;
        constexpr bool BPIPE = true;   // needs 16 more registers
        constexpr bool DUAL = UR == 1 && !(is_weighted(MODE) && KC >= 3);
        v4f bcur[4];
        if constexpr (BPIPE) {
#pragma unroll
            for (int tq = 0; tq < 4; ++tq) bcur[tq] = *reinterpret_cast<const v4f *>(f1s + pl * LS + 16 * h + 4 * tq);
        }
        v16f acc_alt;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_alt[e] = 0.f;
        auto issueF = [&](int step, int J, v4f(&buf)[UR][4]) {
#pragma unroll
            for (int r = 0; r < UR; ++r) {
                const unsigned off = lane_off + (unsigned)row_of(step, r, ug) * rowbytes + (unsigned)J * 128u;
#pragma unroll
                for (int tq = 0; tq < 4; ++tq) {
                    buf[r][tq] = buf_load4(rsrc, off + 16u * tq);
                }
            }
            __builtin_amdgcn_sched_barrier(0);   // keep the loads here: a full block ahead of their use
        };
        // u-indexed weights of a row: per lane a fixed offset (its pixel), row and channel in the scalar offset
        __amdgpu_buffer_rsrc_t rsrc_wu = rsrc;
        unsigned wu_lane = 0;
        if constexpr (is_weighted(MODE)) {
            rsrc_wu = make_rsrc(Lwu + (size_t)b * N1 * a.KT * H2, (unsigned)N1 * a.KT * H2 * 4u);
            wu_lane = (unsigned)(((pok ? pix : 0) * a.KT + a.k0) * H2) * 4u;
        }
        auto computeF = [&](int step, int J, v4f(&buf)[UR][4], auto single) {
            constexpr int NR = decltype(single)::value ? 1 : UR;   // rows whose products are formed
            // the cross-wave sums of the step before (its partial results have been in LDS since that step's barrier)
            if (J == (NJB > 1 ? 1 : 0) && step > 0) combine(step - 1);
            if constexpr (is_weighted(MODE)) {
                if (J == 0) {
#pragma unroll
                    for (int r = 0; r < UR; ++r) {
                        const int u = min(row_of(step, r, ug), H2 - 1);
#pragma unroll
                        for (int k = 0; k < KC; ++k) wur[r][k] = buf_load1s(rsrc_wu, wu_lane, (unsigned)(k * H2 + u) * 4u);
                    }
                }
                if (J == (NJB > 1 ? 1 : 0) && soft_logits) {   // (a block later: the loads above have landed by now)
#pragma unroll
                    for (int r = 0; r < UR; ++r)
#pragma unroll
                        for (int k = 0; k < KC; ++k)
                            wur[r][k] = __expf(wur[r][k] - cst[2 * (pl * KC + k)]) * cst[2 * (pl * KC + k) + 1];
                }
            }
            // C == 256 instantiation: the first MFMA of a row takes a literal zero as its addend, which saves
            // clearing the 16 accumulator registers after every row (vector moves are not free here: they run
            // on the same lanes as the fp32 MFMA)
            const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            auto mfma_tq = [&](int tq, const v4f &bv) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const bool first = CMODE == 3 && J == 0 && tq == 0;
                    if constexpr (DUAL) {
                        // one row per step: split the contraction over two accumulators so that
                        // consecutive MFMAs are independent (skipped where registers are short: the
                        // matrix pipe accepts back-to-back dependent MFMAs without a bubble)
                        if (t & 1) acc_alt = mfma(buf[0][tq][t], bv[t], first && t == 1 ? zero16 : acc_alt);
                        else acc[0] = mfma(buf[0][tq][t], bv[t], first && t == 0 ? zero16 : acc[0]);
                    } else {
#pragma unroll
                        for (int r = 0; r < NR; ++r) acc[r] = mfma(buf[r][tq][t], bv[t], first && t == 0 ? zero16 : acc[r]);
                    }
                }
            };
            if constexpr (BPIPE) {
                // the f1 operand of the next block is fetched from LDS in the middle of this block
                mfma_tq(0, bcur[0]);
                mfma_tq(1, bcur[1]);
                __builtin_amdgcn_sched_barrier(0);
                v4f bnext[4];
                const float *nrow = f1s + pl * LS + 32 * (J + 1 == NJB ? 0 : J + 1) + 16 * h;
#pragma unroll
                for (int tq = 0; tq < 4; ++tq) bnext[tq] = *reinterpret_cast<const v4f *>(nrow + 4 * tq);
                __builtin_amdgcn_sched_barrier(0);
                mfma_tq(2, bcur[2]);
                mfma_tq(3, bcur[3]);
#pragma unroll
                for (int tq = 0; tq < 4; ++tq) bcur[tq] = bnext[tq];
            } else {
                const float *brow = f1s + pl * LS + 32 * J + 16 * h;
                v4f bv[4];
#pragma unroll
                for (int tq = 0; tq < 4; ++tq) bv[tq] = *reinterpret_cast<const v4f *>(brow + 4 * tq);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int tq = 0; tq < 4; ++tq) mfma_tq(tq, bv[tq]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (J == NJB - 1) {
                if constexpr (DUAL) {
                    acc[0] += acc_alt;
                    if constexpr (CMODE != 3) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) acc_alt[e] = 0.f;
                    }
                }
                epilogue(step, true);
            }
        };
        // Ring of NB register buffers: the loads of block i+NB-1 are issued before the MFMAs of block i,
        // so NB-1 blocks of MFMA work cover the latency of an L2 miss.
        if constexpr (CMODE == 3) {
            constexpr int NJT = 8;
            constexpr int NB = (UR == 1 && !HEAVY) ? 4 : 2;   // divides NJT: ring slots are static across steps
            v4f ring[NB][UR][4];
#pragma unroll
            for (int k = 0; k < NB - 1; ++k) issueF(0, k, ring[k]);
            const int nfull = tail_single ? nsteps - 1 : nsteps;
            for (int step = 0; step < nfull; ++step) {
#pragma unroll
                for (int J = 0; J < NJT; ++J) {
                    constexpr int AHEAD = NB - 1;
                    if (J + AHEAD < NJT) issueF(step, J + AHEAD, ring[(J + AHEAD) % NB]);
                    else if (step + 1 < nsteps) issueF(step + 1, J + AHEAD - NJT, ring[(J + AHEAD) % NB]);
                    computeF(step, J, ring[J % NB], std::false_type{});
                }
            }
            if constexpr (HU == 2) {
                if (tail_single) {   // one row per wave (the loads still fetch both)
#pragma unroll
                    for (int J = 0; J < NJT; ++J) {
                        constexpr int AHEAD = NB - 1;
                        if (J + AHEAD < NJT) issueF(nfull, J + AHEAD, ring[(J + AHEAD) % NB]);
                        computeF(nfull, J, ring[J % NB], std::true_type{});
                    }
                }
            }
        } else {
            constexpr int NB = (UR == 1) ? 4 : 3;
            const int TF = nsteps * NJB;
            v4f ring[NB][UR][4];
            int is = 0, iJ = 0;   // position of the next block to issue
            int cs = 0, cJ = 0;   // position of the next block to compute
            auto advance = [&](int &st, int &jj) { if (++jj == NJB) { jj = 0; ++st; } };
#pragma unroll
            for (int k = 0; k < NB - 1; ++k) {
                if (k < TF) { issueF(is, iJ, ring[k]); advance(is, iJ); }
            }
            for (int it = 0; it < TF; it += NB) {
#pragma unroll
                for (int k = 0; k < NB; ++k) {
                    if (it + k < TF) {
                        if (it + k + NB - 1 < TF) { issueF(is, iJ, ring[(k + NB - 1) % NB]); advance(is, iJ); }
                        computeF(cs, cJ, ring[k], std::false_type{});
                        advance(cs, cJ);
                    }
                }
            }
        }
        if (nsteps > 0) combine(nsteps - 1);   // the last step's, still owed
    } else {
    v4f bufA[UR][GJ], bufB[UR][GJ];
    int step = 0, g = 0;  // position of iteration `it`
    issue(0, 0, bufA);
    for (int it = 0; it < T; it += 2) {
        int g1 = g + 1, s1 = step;
        if (g1 == NG) { g1 = 0; ++s1; }
        int g2 = g1 + 1, s2 = s1;
        if (g2 == NG) { g2 = 0; ++s2; }
        if (it + 1 < T) issue(s1, g1, bufB);
        compute(step, g, bufA);
        if (it + 2 < T) issue(s2, g2, bufA);
        if (it + 1 < T) compute(s1, g1, bufB);
        step = s2;
        g = g2;
    }
    }
    // (lane indices for the code behind the sweep are derived afresh from the thread id, so that nothing of them
    // is kept in registers during the sweep)
    int tide = threadIdx.x;
    asm volatile("" : "+v"(tide));
    const int wave_e = tide >> 6, lane_e = tide & 63, pl_e = lane_e & 31, h_e = lane_e >> 5;
    const int vcw_e = RG ? wave_e % nvc : wave_e, ug_e = RG ? wave_e / nvc : 0;
    const int pix_e = p0 + pl_e;
    const bool pok_e = pix_e < N1;
    const size_t bp_e = (size_t)b * N1 + (pok_e ? pix_e : 0);
    (void)lane_e; (void)h_e; (void)vcw_e; (void)ug_e; (void)bp_e;
    const KArgs ke = kernargs_now();
    // flush the staged out_u rows of this piece (all rows of a whole tile): per pixel and channel a run of floats
    if (Lstage && vp == vpasses - 1) {
        __syncthreads();
        const int cht = (is_weighted(MODE)) ? a.KT : 2, ch0 = (is_weighted(MODE)) ? a.k0 : 0;
        // the piece's rows lie in [u0, u0 + nu); where half steps are dealt out, the rows of its first and last step
        // alternate with those of its neighbours: row_mine() tells them apart
        int u0 = 0, nu = H2;
        if (!whole) {
            if constexpr (HU == 2) {
                u0 = ((sa >> 1) * NUG) * 2 + (sa & 1);
                nu = min(H2, ((((sb - 1) >> 1) * NUG + NUG - 1) * 2 + ((sb - 1) & 1)) + 1) - u0;
            } else {
                u0 = sa * NUG * UR;
                nu = min(H2, sb * NUG * UR) - u0;
            }
        }
        auto row_mine = [&](int u) {
            if constexpr (HU == 2) {
                const int hs = 2 * ((u >> 1) / NUG) + (u & 1);
                return whole || (hs >= sa && hs < sb);
            } else {
                return true;
            }
        };
        // A (pixel, channel) row of nu floats goes to 8, 16, 32 or 64 neighbouring lanes, so that several short rows
        // share a wave; the row index is the same for all lanes of a group (no division by nu anywhere).
        const int lsh = nu > 32 ? 6 : nu > 16 ? 5 : nu > 8 ? 4 : 3;
        const int lpr = 1 << lsh, rpi = 64 >> lsh;        // lanes per row, rows per wave and trip
        const int lr = lane_e >> lsh, lu = lane_e & (lpr - 1);
        constexpr int UNR = 4;   // the logits of a batch of elements are fetched before any of them is used
        for (int r0 = wave_e * rpi + lr; r0 < TP * NCHO; r0 += UNR * nW * rpi)
            for (int uu = lu; uu < nu; uu += lpr) {
                float zs[UNR];
                size_t off[UNR];
                int lds_i[UNR], pk[UNR];
#pragma unroll
                for (int t = 0; t < UNR; ++t) {
                    const int r = r0 + t * nW * rpi;
                    const int p = r / NCHO, ch = r - p * NCHO, u = u0 + uu;
                    const bool ok = r < TP * NCHO && p0 + p < N1 && row_mine(u);
                    off[t] = ok ? ((((size_t)b * N1 + p0 + p) * cht + ch0 + ch) * H2 + u) : (size_t)-1;
                    lds_i[t] = r * H2 + u;
                    pk[t] = p * KC + ch;
                    zs[t] = 0.f;
                    if constexpr (is_weighted(MODE)) {
                        if (soft_dlog && ok) zs[t] = ke->lev[lvl].z_ou[off[t]];
                    }
                }
#pragma unroll
                for (int t = 0; t < UNR; ++t) {
                    if (off[t] == (size_t)-1) continue;
                    float x = ostage[lds_i[t]];
                    if constexpr (is_weighted(MODE)) {
                        if (soft_dlog) x = dlogit3(zs[t], cst + 3 * pk[t], x);
                    }
                    ke->lev[lvl].out_u[off[t]] = x;
                }
            }
        if constexpr (MODE == MODE_ARGMAX) {
            for (int p = wave_e * rpi + lr; p < TP; p += nW * rpi)
                for (int uu = lu; uu < nu; uu += lpr)
                    if (p0 + p < N1 && row_mine(u0 + uu)) ke->lev[lvl].am_u[((size_t)b * N1 + p0 + p) * H2 + u0 + uu] = ostage_am[p * H2 + u0 + uu];
        }
    }
    // merge the running state of the row groups into group 0, one group at a time, through the LDS
    // region of the f1 tile (no longer needed).  Equal maxima keep the smaller row index.
    if (NUG > 1) {
        constexpr int NQ = (is_weighted(MODE)) ? KC : 3;
        float *mst = smem + vcw_e * (NQ * 16 * 64);   // [vcw_e][quantity][r][lane_e]
        for (int g2 = 1; g2 < NUG; ++g2) {
            __syncthreads();
            if (ug_e == g2) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int k = 0; k < KC; ++k) mst[(k * 16 + r) * 64 + lane_e] = rv[k][r];
                    } else {
                        mst[(0 * 16 + r) * 64 + lane_e] = vmax[r];
                        mst[(1 * 16 + r) * 64 + lane_e] = __int_as_float(vidx[r]);
                        mst[(2 * 16 + r) * 64 + lane_e] = vsum[r];
                    }
                }
            }
            __syncthreads();
            if (ug_e == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int k = 0; k < KC; ++k) rv[k][r] += mst[(k * 16 + r) * 64 + lane_e];
                    } else {
                        const float m2 = mst[(0 * 16 + r) * 64 + lane_e];
                        const int i2 = __float_as_int(mst[(1 * 16 + r) * 64 + lane_e]);
                        if (m2 > vmax[r] || (m2 == vmax[r] && i2 < vidx[r])) { vmax[r] = m2; vidx[r] = i2; }
                        vsum[r] += mst[(2 * 16 + r) * 64 + lane_e];
                    }
                }
            }
        }
    }

    // The piece that comes last does not need a slot.  Pieces publish themselves by adding one to the tile's counter
    // after their slot is in memory (below); a piece that reads "all the others are there" before it has written
    // anything takes their column state into its own registers instead -- a slot holds it in the very order a wave
    // keeps it in: wave (column chunk) and lane of the reader are those of the writer -- and then finishes the tile as
    // a whole tile does, from registers.  Only tiles of two pieces are finished this way (nearly all are): the sum of
    // two numbers does not depend on which is added to which, so the result is the one merge_pieces gives, whichever
    // piece came last and whichever path it took; maxima keep the lower row on ties either way.  Of a tile's two pieces the one
    // with the tile's first rows is the end of its workgroup's share and nearly always the late one: its slot
    // (written and read back: a third of a sweep's HBM traffic at B=2, 55x128) and the separate merge pass go away.
    // Only for one pass of columns (with several, the registers hold the state of the last pass only).
    // (The piece at the end of a share is done first and holds its tile's first rows: the other pieces of that tile
    // are the last thing their workgroups do, so it has nothing to look for and goes straight to its slot.)
    if (SK && !whole && vpasses == 1 && !(seg_no == 0 && head)) {
        const int G = (int)gridDim.x;
        int wfirst, wlast;
        pieces_of(ubeg, uend, G, sk_total, wfirst, wlast);
        __syncthreads();   // (LDS word 0 is free: the row groups are merged)
        int *flag = reinterpret_cast<int *>(smem);
        if (tide == 0)
            *flag = __hip_atomic_fetch_add(ke->sk_count + (multi ? tile * a.nlev + lvl : tile), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        merged_here = wlast == wfirst + 1 && *flag == 1;   // a tile of two pieces, and the other one is there
        __syncthreads();
        if (merged_here && ug_e == 0 && vbase + 32 * vcw_e < W2) {
            constexpr int NQ = (is_weighted(MODE)) ? KC : 3;
            const __amdgpu_buffer_rsrc_t rs_sk = make_rsrc(ke->sk_state, 2u * gridDim.x * (unsigned)a.sk_slot * 4u);
            const unsigned mine = (unsigned)((vbase >> 5) + vcw_e) * (NQ * 1024u) + 4u * lane_e;
            auto fetch = [&](int w, v4f (&x)[NQ][4]) {
                const bool first_piece = ((long)w * sk_total) / G >= ubeg;   // w's share starts inside this tile: its slot 0
                const unsigned base = ((unsigned)(2 * w + (first_piece ? 0 : 1)) * (unsigned)a.sk_slot + mine) * 4u;
#pragma unroll
                for (int q = 0; q < NQ; ++q)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) x[q][g4] = load_shared4(rs_sk, base + (unsigned)(q * 4 + g4) * 1024u);
            };
            // (two pieces: the sum of the two is the same whichever is added to which)
            const int w = wg == wfirst ? wlast : wfirst;
            v4f x[NQ][4];
            fetch(w, x);
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int q = 0; q < NQ; ++q) rv[q][4 * g4 + e] += x[q][g4][e];
                    } else {
                        const float m2 = x[0][g4][e];
                        const int i2 = __float_as_int(x[1][g4][e]);
                        if (m2 > vmax[4 * g4 + e] || (m2 == vmax[4 * g4 + e] && i2 < vidx[4 * g4 + e])) { vmax[4 * g4 + e] = m2; vidx[4 * g4 + e] = i2; }
                        vsum[4 * g4 + e] += x[2][g4][e];
                    }
                }
        }
    }
    // A piece of a tile leaves its column state in this workgroup's slot in register order, sums undivided:
    // [column chunk][quantity][register group g4][lane_e][4]: every store of a wave_e is one contiguous KB
    if (!whole && !merged_here) {
        if (ug_e == 0 && vbase + 32 * vcw_e < W2) {
            constexpr int NQ = (is_weighted(MODE)) ? KC : 3;
            const __amdgpu_buffer_rsrc_t rs_sk = make_rsrc(ke->sk_state, 2u * gridDim.x * (unsigned)a.sk_slot * 4u);
            const unsigned base = ((unsigned)(2 * wg + (pb == gs0 ? 0 : 1)) * (unsigned)a.sk_slot +
                                   (unsigned)((vbase >> 5) + vcw_e) * (NQ * 1024u) + 4u * lane_e) * 4u;
#pragma unroll
            for (int q = 0; q < NQ; ++q)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    v4f x;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if constexpr (is_weighted(MODE)) x[e] = rv[q][4 * g4 + e];
                        else x[e] = q == 0 ? vmax[4 * g4 + e] : q == 1 ? __int_as_float(vidx[4 * g4 + e]) : vsum[4 * g4 + e];
                    }
                    store_shared4(rs_sk, base + (unsigned)(q * 4 + g4) * 1024u, x);
                }
        }
    } else
    // store the state that was reduced over u: registers 4g..4g+3 hold 4 consecutive columns
    if (pok_e && ug_e == 0) {
        if ((W2 & 3) == 0) {   // 16-byte stores (rows of out_v are then 16-byte aligned)
            typedef int v4i __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int v = vbase + 32 * vcw_e + vmap(4 * g4, h_e);
                if (v < W2) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int k = 0; k < KC; ++k) {
                            v4f x = {rv[k][4 * g4], rv[k][4 * g4 + 1], rv[k][4 * g4 + 2], rv[k][4 * g4 + 3]};
                            const size_t row = bp_e * a.KT + a.k0 + k;
                            if (soft_dlog) {
                                const float r3[3] = {ke->lev[lvl].st_ov[2 * row], 1.f / ke->lev[lvl].st_ov[2 * row + 1], ke->lev[lvl].dot_ov[row]};
                                const v4f z = *reinterpret_cast<const v4f *>(ke->lev[lvl].z_ov + row * W2 + v);
#pragma unroll
                                for (int e = 0; e < 4; ++e) x[e] = dlogit3(z[e], r3, x[e]);
                            }
                            *reinterpret_cast<v4f *>(ke->lev[lvl].out_v + row * W2 + v) = x;
                        }
                    } else {
                        const v4f xm = {vmax[4 * g4], vmax[4 * g4 + 1], vmax[4 * g4 + 2], vmax[4 * g4 + 3]};
                        const v4f xs = {vsum[4 * g4] / (float)H2, vsum[4 * g4 + 1] / (float)H2, vsum[4 * g4 + 2] / (float)H2,
                                        vsum[4 * g4 + 3] / (float)H2};
                        *reinterpret_cast<v4f *>(ke->lev[lvl].out_v + (bp_e * 2 + 0) * W2 + v) = xm;
                        *reinterpret_cast<v4f *>(ke->lev[lvl].out_v + (bp_e * 2 + 1) * W2 + v) = xs;
                        if constexpr (MODE == MODE_ARGMAX) {
                            const v4i xi = {vidx[4 * g4], vidx[4 * g4 + 1], vidx[4 * g4 + 2], vidx[4 * g4 + 3]};
                            *reinterpret_cast<v4i *>(ke->lev[lvl].am_v + bp_e * W2 + v) = xi;
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int v = vbase + 32 * vcw_e + vmap(r, h_e);
                if (v < W2) {
                    if constexpr (is_weighted(MODE)) {
#pragma unroll
                        for (int k = 0; k < KC; ++k) {
                            const size_t row = bp_e * a.KT + a.k0 + k;
                            ke->lev[lvl].out_v[row * W2 + v] = soft_dlog ? dlogit(ke->lev[lvl].z_ov, ke->lev[lvl].st_ov, ke->lev[lvl].dot_ov, row, row * W2 + v, rv[k][r]) : rv[k][r];
                        }
                    } else {
                        ke->lev[lvl].out_v[(bp_e * 2 + 0) * W2 + v] = vmax[r];
                        ke->lev[lvl].out_v[(bp_e * 2 + 1) * W2 + v] = vsum[r] / (float)H2;
                        if constexpr (MODE == MODE_ARGMAX) ke->lev[lvl].am_v[bp_e * W2 + v] = vidx[r];
                    }
                }
            }
        }
    }
    }   // column passes
    // (lane indices for the code behind the sweep are derived afresh from the thread id, so that nothing of them
    // is kept in registers during the sweep)
    int tide = threadIdx.x;
    asm volatile("" : "+v"(tide));
    const int wave_e = tide >> 6, lane_e = tide & 63, pl_e = lane_e & 31, h_e = lane_e >> 5;
    const int vcw_e = RG ? wave_e % nvc : wave_e, ug_e = RG ? wave_e / nvc : 0;
    const int pix_e = p0 + pl_e;
    const bool pok_e = pix_e < N1;
    const size_t bp_e = (size_t)b * N1 + (pok_e ? pix_e : 0);
    (void)lane_e; (void)h_e; (void)vcw_e; (void)ug_e; (void)bp_e;

    if (!whole && !merged_here) {
        const KArgs ke = kernargs_now();
        // Publish this piece and find out whether it completes the tile.  The pieces of a tile belong to consecutive
        // workgroups; a workgroup keeps the first piece of its share in its slot 0 and a later one (which can only be
        // its last: the tiles between are whole) in its slot 1.
        const int G = (int)gridDim.x;
        const long t0 = ubeg;
        int wfirst, wlast;
        pieces_of(ubeg, uend, G, sk_total, wfirst, wlast);
        const int npieces = wlast - wfirst + 1;
        // Hand-over without a fence.  What it rests on: (1) the slot was written with sc0 sc1 stores, which are
        // written through to device memory, and vmcnt counts such a store only when that write is acknowledged, so
        // after vmcnt(0) in every wave and the barrier the whole piece is in memory; (2) the counter is a device-scope
        // atomic, executed where all XCDs see one value, and it is issued after the barrier; (3) the piece that reads
        // "I am the last" issues its slot reads after the atomic has returned (the flag goes through LDS and a
        // barrier), and those reads carry sc0 sc1, which never take a line from this XCD's caches.  A release fence
        // in front of the atomic (buffer_wbl2 sc1: write back every dirty line of this XCD's L2) adds nothing for
        // these accesses and was measured to cost the forward sweeps 4-5 % at B=2, 55x128.
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave_e's words of the piece have arrived
        __syncthreads();
        int *flag = reinterpret_cast<int *>(smem);
        if (tide == 0)
            *flag = __hip_atomic_fetch_add(ke->sk_count + (multi ? tile * a.nlev + lvl : tile), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const bool last = *flag == npieces - 1;
        __syncthreads();
        if (last) merge_pieces<MODE, KC>(ke, lvl, b, p0, wfirst, wlast, (int)t0, tide);
    }
    }   // pieces of this workgroup
}

// ------------------------------------------------------------------------------------------
// backward: G synthesis shared by df1 / df2
// ------------------------------------------------------------------------------------------
// GMODE_BOTH: G is the sum of the two, so that one contraction serves both gradients
enum { GMODE_MAXAVG = 0, GMODE_COMP = 1, GMODE_BOTH = 2 };
constexpr bool g_has_comp(int gmode) { return gmode != GMODE_MAXAVG; }
constexpr bool g_has_maxavg(int gmode) { return gmode != GMODE_COMP; }

}  // namespace
namespace sepcorr_impl {
struct BwdArgs {
    const float *f1, *f2;
    const int *am_u, *am_v;          // GMODE_MAXAVG
    const float *g_u, *g_v;          // GMODE_MAXAVG: (B,N1,2,H2), (B,N1,2,W2)
    const float *a_u, *a_v;          // GMODE_COMP:   (B,N1,KT,W2), (B,N1,KT,H2)
    const float *g_cu, *g_cv;        // GMODE_COMP:   (B,N1,KT,H2), (B,N1,KT,W2)
    const float *uwt;                // fast d_f1: the (p,u)-indexed weights transposed to [b][u][field][p]
    const float *vtable;             // tiled d_f2 without the average term of g_v: (B,W2,C) table that stands for it
    float *d1;                       // (B,N1,C)
    float *d2;                       // (B,N2,C) or scratch [nsplit][B,N2,C]
    int B, N1, H2, W2, C;
    int KT, k0;
    int nvc;                         // df1: column chunks of 32 per pass = min(8, ceil(W2 / 32))
    int vpasses;                     // df1: passes of 256 columns
    int tiles_per_batch;             // df1: p tiles per batch
    int nsplit, tiles_per_split;     // df2: split of the p range
    // df2, uneven split: the last split of every block of output rows is a short one (what tiles_per_split leaves
    // over) and is dealt out behind all the long ones, so that the short ones share the compute units the long ones
    // leave free.  Per XCD x (workgroup ids x, x + 8, ...): long units xl[x] .. xl[x+1], then short ones from xs[x].
    int uneven, q_units;             // q_units = blocks of output rows (B x row groups x column chunks)
    int xl[9], xs[9];
    int accumulate;                  // add to the destination instead of overwriting
    int add_d1;                      // d_f1 only: add to what the caller's buffer holds
    int xcd_order;                   // map workgroup ids so that each XCD gets a contiguous range
    // d_f1 dealt out in pieces of tiles, as the forward sweeps are (FwdArgs::sk_*): a piece leaves its partial
    // [32 pixels][channels] sum in a slot; whichever piece of a tile finishes last adds them up in row order.
    int sk_total, sk_steps;          // steps (rows per wave) over all tiles, per tile; 0 = whole tiles
    float *sk_state;                 // [2 * grid.x * grid.y] slots of 32 x (128 * NCB) floats
    int *sk_count;                   // [tiles * grid.y], zero at launch
    int flush_rows;                  // d_f1: rows of a wave whose products one register accumulator takes
};
}  // namespace sepcorr_impl
namespace {

// Weights of one lane that depend on (p, v) and on (p, u).  Members a mode does not use stay unset and
// cost no registers.
template <int GMODE, int KC>
struct VW {
    float a[KC];   // comp: a_u[k]
    float g[KC];   // comp: g_cv[k]
    float ma;      // maxavg: g_v[avg] / H2 + g_v[max]  (the value where the row index equals argmax_v)
    float mg;      // maxavg: g_v[avg] / H2             (the value elsewhere)
    int am;        // maxavg: argmax_v
};
template <int GMODE, int KC>
struct UW {
    float a[KC];   // comp: a_v[k]
    float g[KC];   // comp: g_cu[k]
    float ma;      // maxavg: g_u[avg] / W2 + g_u[max]  (the value where the column index equals argmax_u)
    float mg;      // maxavg: g_u[avg] / W2             (the value elsewhere)
    int am;        // maxavg: argmax_u (callers may store it relative to a lane's first column)
};

template <int GMODE, int KC>
__device__ __forceinline__ VW<GMODE, KC> load_vw(const BwdArgs &a, size_t bp, int v, bool ok) {
    VW<GMODE, KC> w;
    if constexpr (g_has_comp(GMODE)) {
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const size_t o = (bp * a.KT + a.k0 + k) * a.W2 + v;
            w.a[k] = ok ? a.a_u[o] : 0.f;
            w.g[k] = ok ? a.g_cv[o] : 0.f;
        }
    }
    if constexpr (g_has_maxavg(GMODE)) {
        w.mg = ok ? a.g_v[(bp * 2 + 1) * a.W2 + v] * (1.f / (float)a.H2) : 0.f;
        w.ma = ok ? w.mg + a.g_v[(bp * 2 + 0) * a.W2 + v] : 0.f;
        w.am = ok ? a.am_v[bp * a.W2 + v] : -1;
    }
    return w;
}
// The (p,v)-indexed weights of a lane's 16 columns, field by field.  The 16 values of one field lie in one or two
// cache lines of the lane's pixel, so 16 consecutive loads of the same field hit the lines the first one brought
// in; column by column (all fields of a column, then the next column) a wave cycles through 32 lines per field and
// with 8 or more fields nothing survives until the next column: the workgroups of an XCD then overflow its L2 and
// every column refetches its lines from memory (0.9 GB per launch at B=2, 55x128, 11 fields).
template <int GMODE, int KC>
__device__ __forceinline__ void load_vw16(const BwdArgs &a, size_t bp, const int (&v)[16], const bool (&ok)[16],
                                          VW<GMODE, KC> (&w)[16]) {
    if constexpr (g_has_comp(GMODE)) {
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const float *row = a.a_u + (bp * a.KT + a.k0 + k) * a.W2;
#pragma unroll
            for (int r = 0; r < 16; ++r) w[r].a[k] = ok[r] ? row[v[r]] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const float *row = a.g_cv + (bp * a.KT + a.k0 + k) * a.W2;
#pragma unroll
            for (int r = 0; r < 16; ++r) w[r].g[k] = ok[r] ? row[v[r]] : 0.f;
        }
    }
    if constexpr (g_has_maxavg(GMODE)) {
        const float inv_h2 = 1.f / (float)a.H2;
        const float *ravg = a.g_v + (bp * 2 + 1) * a.W2, *rmax = a.g_v + (bp * 2 + 0) * a.W2;
        const int *ram = a.am_v + bp * a.W2;
#pragma unroll
        for (int r = 0; r < 16; ++r) w[r].mg = ok[r] ? ravg[v[r]] * inv_h2 : 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) w[r].ma = ok[r] ? w[r].mg + rmax[v[r]] : 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) w[r].am = ok[r] ? ram[v[r]] : -1;
    }
}
// The same for rows whose length is a multiple of 4: the four consecutive columns of a register group (vmap) come
// with one 16-byte buffer load; per group one offset register, the field travels in the scalar offset.  v0 = first
// column of the wave's chunk, h = half of the wave, pix = the lane's pixel within image b (pok: it exists).
template <int GMODE, int KC>
__device__ __forceinline__ void load_vw16_rows4(const BwdArgs &a, int b, int pix, bool pok, int v0, int h, VW<GMODE, KC> (&w)[16]) {
    const unsigned W2 = (unsigned)a.W2, N1 = (unsigned)a.N1;
    bool ok[4];
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) ok[g4] = pok && v0 + vmap(4 * g4, h) < a.W2;
    if constexpr (g_has_comp(GMODE)) {
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(a.a_u + (size_t)b * N1 * a.KT * W2, N1 * a.KT * W2 * 4u);
        const __amdgpu_buffer_rsrc_t rg = make_rsrc(a.g_cv + (size_t)b * N1 * a.KT * W2, N1 * a.KT * W2 * 4u);
        unsigned o[4];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
            o[g4] = ok[g4] ? (unsigned)((pix * a.KT + a.k0) * a.W2 + v0 + vmap(4 * g4, h)) * 4u : DMA_OOB;
#pragma unroll
        for (int k = 0; k < KC; ++k)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const v4f x = buf_load4s(ra, o[g4], (unsigned)k * W2 * 4u);
#pragma unroll
                for (int e = 0; e < 4; ++e) w[4 * g4 + e].a[k] = x[e];
            }
#pragma unroll
        for (int k = 0; k < KC; ++k)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const v4f x = buf_load4s(rg, o[g4], (unsigned)k * W2 * 4u);
#pragma unroll
                for (int e = 0; e < 4; ++e) w[4 * g4 + e].g[k] = x[e];
            }
    }
    if constexpr (g_has_maxavg(GMODE)) {
        const float inv_h2 = 1.f / (float)a.H2;
        const __amdgpu_buffer_rsrc_t rg = make_rsrc(a.g_v + (size_t)b * N1 * 2u * W2, N1 * 2u * W2 * 4u);
        const __amdgpu_buffer_rsrc_t rm = make_rsrc(a.am_v + (size_t)b * N1 * W2, N1 * W2 * 4u);
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const int v = v0 + vmap(4 * g4, h);
            const unsigned og = ok[g4] ? (unsigned)(pix * 2 * a.W2 + v) * 4u : DMA_OOB;
            const unsigned om = ok[g4] ? (unsigned)(pix * a.W2 + v) * 4u : DMA_OOB;
            const v4f xmax = buf_load4s(rg, og, 0u), xavg = buf_load4s(rg, og, W2 * 4u);
            const v4f xam = buf_load4s(rm, om, 0u);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[4 * g4 + e].mg = xavg[e] * inv_h2;                       // (all zero where the group does not exist)
                w[4 * g4 + e].ma = w[4 * g4 + e].mg + xmax[e];
                w[4 * g4 + e].am = ok[g4] ? __float_as_int(xam[e]) : -1;
            }
        }
    }
}
template <int GMODE, int KC>
__device__ __forceinline__ UW<GMODE, KC> load_uw(const BwdArgs &a, size_t bp, int u, bool ok) {
    UW<GMODE, KC> w;
    if constexpr (g_has_comp(GMODE)) {
#pragma unroll
        for (int k = 0; k < KC; ++k) {
            const size_t o = (bp * a.KT + a.k0 + k) * a.H2 + u;
            w.a[k] = ok ? a.a_v[o] : 0.f;
            w.g[k] = ok ? a.g_cu[o] : 0.f;
        }
    }
    if constexpr (g_has_maxavg(GMODE)) {
        w.mg = ok ? a.g_u[(bp * 2 + 1) * a.H2 + u] * (1.f / (float)a.W2) : 0.f;
        w.ma = ok ? w.mg + a.g_u[(bp * 2 + 0) * a.H2 + u] : 0.f;
        w.am = ok ? a.am_u[bp * a.H2 + u] : -1;
    }
    return w;
}
// dL/dS at (p, u, v); `ok` false gives exactly 0.
template <int GMODE, int KC>
__device__ __forceinline__ float gval(const VW<GMODE, KC> &wv, const UW<GMODE, KC> &wu, int u, int v, bool ok) {
    float g = 0.f;
    // max/avg terms: two selects and one add (the sums with and without the max gradient are kept ready)
    if constexpr (g_has_maxavg(GMODE)) g = (wu.am == v ? wu.ma : wu.mg) + (wv.am == u ? wv.ma : wv.mg);
    if constexpr (g_has_comp(GMODE)) {
#pragma unroll
        for (int k = 0; k < KC; ++k) {   // two fused multiply-adds per channel (a sum of two products would take three)
            g = fmaf(wv.a[k], wu.g[k], g);
            g = fmaf(wu.a[k], wv.g[k], g);
        }
    }
    return ok ? g : 0.f;
}

// d_f1[p, c] = sum_q G[p,q] f2[q,c].  Grid: (B * tiles_per_batch, channel blocks of 128*NCB).
// FAST (C == 256, W2 % 4 == 0, both channel blocks in one workgroup): the operand loads take no address
// arithmetic at all -- a per-lane offset for each group of 4 columns is kept in a register, the row advances
// through the scalar offset and the column within the group and the channel block through the immediate.
// (fp32 MFMA and vector instructions share the SIMD's arithmetic lanes here: every vector instruction in the
// loop costs its issue time, nothing hides behind the matrix work.)
template <int GMODE, int KC, int NCB, bool CVEC, int MAXT, bool FAST = false, bool SK = false>
__global__ void __launch_bounds__(MAXT) df1_kernel(const BwdArgs a) {
    static_assert(!FAST || (CVEC && NCB == 2), "fast loads: 16-byte loads, 256 channels per workgroup");
    constexpr int GS = 2;            // MFMA k-steps (pairs of v) per prefetch group
    constexpr int NG = 16 / GS;
    constexpr int CB = 128 * NCB;
    constexpr int RS = CB + 4;
    extern __shared__ float smem[];  // [TP][RS] cross-wave sum
    const int tid = threadIdx.x, lane = tid & 63, pl = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nW = blockDim.x >> 6;
    // wave (vcw, ug): columns [32 vcw, 32 vcw + 32), rows ug, ug + NUG, ... (see fwd_kernel)
    const int nvc = a.nvc, NUG = nW / nvc;
    const int vcw = wave % nvc, ug = wave / nvc;
    const int wg = a.xcd_order ? xcd_contiguous(blockIdx.x, gridDim.x) : (int)blockIdx.x;
    const int cb0 = blockIdx.y * CB;
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C;

    // This workgroup's share of the steps (one step = one row per wave) of all tiles, cut into pieces at tile
    // boundaries; the piece at the end of the share starts at row 0 and is done first (see fwd_kernel).
    const int sk_total = SK ? a.sk_total : 0;
    const int S = sk_total ? a.sk_steps : 1;
    const int gs0 = sk_total ? (int)(((long)wg * sk_total) / (int)gridDim.x) : wg;
    const int gs_end = sk_total ? (int)(((long)(wg + 1) * sk_total) / (int)gridDim.x) : wg + 1;
    int head = gs_end % S;
    if (gs_end - head <= gs0) head = 0;
    const int body_end = gs_end - head;
    int cur = gs0;
    for (int seg_no = 0;; ++seg_no) {
    int pb, pe;
    if (seg_no == 0 && head) {
        pb = body_end; pe = gs_end;
    } else {
        if (cur >= body_end) break;
        pb = cur;
        pe = min(body_end, (cur / S + 1) * S);
        cur = pe;
    }
    const int tile = pb / S;
    const int sa = pb - tile * S, sb = pe - tile * S;
    const bool whole = !SK || !sk_total || (sa == 0 && sb == S);
    const int u_begin = sk_total ? sa * NUG : 0, u_end = sk_total ? min(H2, sb * NUG) : H2;   // this piece's rows
    const int b = tile / a.tiles_per_batch;
    const int p0 = (tile % a.tiles_per_batch) * TP;
    const int pix = p0 + pl;
    const bool pok = pix < N1;
    const size_t bp = (size_t)b * N1 + (pok ? pix : 0);

    v16f acc[NCB][4];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[cb][t][e] = 0.f;
    // Short chains of additions: a register accumulator takes the products of FLUSH_ROWS (4) rows of this wave only
    // (128 products at 32 columns per row), then it is added to a running sum in the wave's LDS region and starts
    // again from zero.  One fp32 accumulator over all rows of a tile (1760 products at 55 x 128) lost the low bits
    // of every product it added once the sum had grown; sums of short blocks keep them.  The order stays fixed.
    // An accumulator joins the running sum just before the first product of the new block overwrites it; that
    // product takes a zero addend, so nothing has to be cleared.  The additions are vector instructions, which take
    // matrix time here: 2 per accumulator register and block (the LDS unit's own float addition, ds_add_f32, takes
    // no vector instruction but handles about one lane in three cycles: tried, five times slower).
    // Layout [group of 4 registers][lane][4]: 16-byte accesses without bank conflicts, wave-private, the same bytes
    // the wave's [pixel][channel] partial is written to at the end.
    // Where registers allow, the first row of a block is a copy of the row body whose first products take the zero
    // addend (PEEL).  The combined mode (both operators' dL/dS: 176 weight registers per lane) has no room for a
    // second body (every form of it tried spilled hundreds of registers): there the accumulators are handed over and
    // cleared in a branch ahead of the block's first row, 3 vector instructions per register and block.
    constexpr bool PEEL = GMODE != GMODE_BOTH;
    const int FLUSH_ROWS = a.flush_rows;
    v4f *const run = reinterpret_cast<v4f *>(smem + wave * (TP * RS)) + lane;
    {
        const v4f z4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < NCB * 16; ++q) run[q * 64] = z4;
    }
    auto run_load = [&](int cbt, v4f (&x)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q) x[q] = run[(cbt * 4 + q) * 64];
    };
    // With one wave per SIMD the accumulators live in the accumulation registers, which vector additions cannot
    // read: each value is copied out first.  The copy is written as assembly so that it stays where the running sum
    // is updated; left to the compiler, all 128 copies were hoisted to the top of every row.  The compiler keeps no
    // wait states for assembly: matrix_results_settled() stands between the last matrix instruction and the first
    // copy (a matrix result may be read 19 wait states after the instruction that wrote it).
    auto acc_value = [&](int cbt, int e) {
        if constexpr (MAXT > 256) {
            return acc[cbt >> 2][cbt & 3][e];
        } else {
            float x;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[cbt >> 2][cbt & 3][e]));
            return x;
        }
    };
    auto matrix_results_settled = [] {
        if constexpr (MAXT <= 256) asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    };
    auto run_add_store = [&](int cbt, v4f (&x)[4]) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float y[8];   // a batch of copies first: a copy followed at once by the addition that reads it waits for it
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = acc_value(cbt, 8 * half + e);
#pragma unroll
            for (int q = 0; q < 2; ++q) {
#pragma unroll
                for (int e = 0; e < 4; ++e) x[2 * half + q][e] += y[4 * q + e];
                run[(cbt * 4 + 2 * half + q) * 64] = x[2 * half + q];
            }
        }
    };

    // rows wider than 256 columns: passes of 256 columns accumulate into the same registers
    for (int vp = 0; vp < a.vpasses; ++vp) {
    const int vbase = vp * 256;
    VW<GMODE, KC> wv[16];
    if ((W2 & 3) == 0) {
        load_vw16_rows4<GMODE, KC>(a, b, pix, pok, vbase + 32 * vcw, h, wv);
    } else {
        int vs[16];
        bool oks[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int v = vbase + 32 * vcw + vmap(r, h);
            vs[r] = v < W2 ? v : 0;
            oks[r] = pok && v < W2;
        }
        load_vw16<GMODE, KC>(a, bp, vs, oks, wv);
    }

    const float *f2b = a.f2 + (size_t)b * H2 * W2 * C;
    // CVEC: raw buffer loads, out-of-image columns and channels read as zero without a branch
    const unsigned nbytes = (unsigned)H2 * W2 * C * 4u;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(f2b, nbytes);
    unsigned coff[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int c = cb0 + 128 * cb + 4 * pl;
        coff[cb] = c < C ? (unsigned)c * 4u : nbytes;
    }
    // FAST: byte offset of (column 8 q + 4 h of this wave's chunk, channel 4 pl) or the out-of-range marker
    unsigned voffq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int v = vbase + 32 * vcw + vmap(4 * q, h);
        voffq[q] = v < W2 ? ((unsigned)v * 256u + 4u * pl) * 4u : DMA_OOB;
    }
    auto issue = [&](int u, int g, v4f(&buf)[GS][NCB]) {
#pragma unroll
        for (int ss = 0; ss < GS; ++ss) {
            if constexpr (FAST) {
                const int r = g * GS + ss;
                const unsigned row = (unsigned)u * ((unsigned)W2 * 1024u);
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) buf[ss][cb] = buf_load4s(rsrc, voffq[r >> 2], row + (1024u * (r & 3) + 512u * cb));
                continue;
            }
            const int v = vbase + 32 * vcw + vmap(g * GS + ss, h);
            const bool ok = v < W2;
            if constexpr (CVEC) {
                const unsigned voff = ok ? ((unsigned)(u * W2 + v) * C) * 4u : nbytes;
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) buf[ss][cb] = buf_load4(rsrc, voff + coff[cb]);
            } else {
                const float *src = f2b + ((size_t)u * W2 + (ok ? v : 0)) * C;
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) buf[ss][cb] = load4<false>(src, cb0 + 128 * cb + 4 * pl, C, ok);
            }
        }
    };

    // G of the current row lives in G[]; G of this wave's next row (u + NUG) is computed two values per
    // MFMA group, between the group's MFMAs, so the arithmetic runs in the shadow of the matrix pipe.
    float G[16], Gn[16];
    // FAST: the (p,u)-indexed weights come through buffer loads as well, from their transposed copy [u][field][p]:
    // the pixel in the per-lane offset, row and field in the scalar offset; a load then reads 128 contiguous bytes
    // (in the operator's layout every lane would touch a line of its own, and with eight or more fields those
    // lines do not survive in cache from one row to the next)
    constexpr int NVC = g_has_comp(GMODE) ? 2 * KC : 0;
    constexpr int NF = NVC + (g_has_maxavg(GMODE) ? 3 : 0);
    const unsigned pix4 = (pok ? (unsigned)pix : 0u) * 4u;
    __amdgpu_buffer_rsrc_t rs_uw;
    if constexpr (FAST) rs_uw = make_rsrc(a.uwt + (size_t)b * H2 * NF * N1, (unsigned)H2 * NF * N1 * 4u);
    const float inv_w2 = 1.f / (float)W2;
    // argmax_u is kept relative to this lane's first column: register r then compares against the constant
    // 8 (r / 4) + r % 4 instead of a column index that would have to be formed for every element
    const int lanebase = vbase + 32 * vcw + 4 * h;
    auto load_uw_row = [&](int u) {
        if constexpr (!FAST) {
            UW<GMODE, KC> w = load_uw<GMODE, KC>(a, bp, u, true);   // bp is clamped: always a valid pixel
            if constexpr (g_has_maxavg(GMODE)) w.am -= lanebase;
            return w;
        } else {
            UW<GMODE, KC> w;
            const unsigned row = (unsigned)u * NF * N1 * 4u;
            if constexpr (g_has_comp(GMODE)) {
#pragma unroll
                for (int k = 0; k < KC; ++k) {
                    w.a[k] = buf_load1s(rs_uw, pix4, row + (unsigned)k * N1 * 4u);
                    w.g[k] = buf_load1s(rs_uw, pix4, row + (unsigned)(KC + k) * N1 * 4u);
                }
            }
            if constexpr (g_has_maxavg(GMODE)) {
                w.mg = buf_load1s(rs_uw, pix4, row + (unsigned)(NVC + 1) * N1 * 4u) * inv_w2;
                w.ma = w.mg + buf_load1s(rs_uw, pix4, row + (unsigned)NVC * N1 * 4u);
                w.am = __float_as_int(buf_load1s(rs_uw, pix4, row + (unsigned)(NVC + 2) * N1 * 4u)) - lanebase;
            }
            return w;
        }
    };
    const int ufirst = u_begin + ug;   // this wave's first row
    UW<GMODE, KC> wu_n = load_uw_row(min(ufirst, H2 - 1));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        // no mask: a column outside the image has an all-zero A operand and the column of a pixel outside the
        // image is never stored; the weights behind both are those of real entries, so G stays finite
        G[r] = gval<GMODE, KC>(wv[r], wu_n, ufirst, vmap(r, 0), true);
    }
    UW<GMODE, KC> wu_next = load_uw_row(min(ufirst + NUG, H2 - 1));
    bool hand_over = false;   // the row that starts a block has a finished block in the accumulators
    auto compute = [&](int u, int g, v4f(&buf)[GS][NCB], auto fresh) {
        static_assert(GS == 2, "two G values are produced per group");
        if (g == 0) {
            wu_n = wu_next;                                                       // weights of row u + NUG
            wu_next = load_uw_row(min(u + 2 * NUG, H2 - 1));                      // and of the row after it
        }
        if (g == 0 && decltype(fresh)::value) {
            // first products of a new block: hand each accumulator to the running sum, then restart it from zero;
            // the running sum of the next accumulator is fetched while the matrix instruction of this one runs
            // (one set of 16 registers: the running sum of the next accumulator is fetched into it once the additions
            // of this one have read it, ahead of this one's matrix instruction, whose 64 cycles cover the fetch)
            const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            // (the first row of a piece has nothing to hand over: it only starts the accumulators.  The condition
            // stands around the additions alone, the matrix instruction behind it is the same either way.)
            v4f rs[4];
            if (hand_over) {
                run_load(0, rs);
                matrix_results_settled();
            }
#pragma unroll
            for (int cbt = 0; cbt < NCB * 4; ++cbt) {
                if (hand_over) {
                    run_add_store(cbt, rs);
                    __builtin_amdgcn_sched_barrier(0);
                    if (cbt + 1 < NCB * 4) run_load(cbt + 1, rs);
                }
                __builtin_amdgcn_sched_barrier(0);
                acc[cbt >> 2][cbt & 3] = mfma(buf[0][cbt >> 2][cbt & 3], G[0], zero);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[cb][t] = mfma(buf[0][cb][t], G[g * GS], acc[cb][t]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ss = 0; ss < GS; ++ss) {
            const int r = g * GS + ss;
            // the row index as an opaque scalar: otherwise the comparison with argmax_v is rewritten into
            // (argmax_v - row) == 0 with one more vector add per element
            int un = u + NUG;
            asm volatile("" : "+s"(un));
            Gn[r] = gval<GMODE, KC>(wv[r], wu_n, un, vmap(r, 0), true);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[cb][t] = mfma(buf[1][cb][t], G[g * GS + 1], acc[cb][t]);
        if (g == NG - 1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) G[r] = Gn[r];
        }
    };

    // Ring of NB register buffers (NB divides the NG groups of a row, so slots are static): the loads of
    // group i+NB-1 are issued, and pinned there, before the MFMAs of group i.
    constexpr int NB = 4;
    v4f ring[NB][GS][NCB];
#pragma unroll
    for (int k = 0; k < NB - 1; ++k) {
        issue(min(ufirst, H2 - 1), k, ring[k]);
        __builtin_amdgcn_sched_barrier(0);
    }
    auto sweep_row = [&](int u, auto fresh) {
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            constexpr int AHEAD = NB - 1;
            // (no condition on the fetch ahead into the next row: behind a branch the compiler has to assume that
            // the loads were not issued and waits for all but the last few at the end of every row; the last row of
            // a piece fetches a valid row that nobody uses)
            if (g + AHEAD < NG) issue(u, g + AHEAD, ring[(g + AHEAD) % NB]);
            else issue(min(u + NUG, H2 - 1), g + AHEAD - NG, ring[(g + AHEAD) % NB]);
            __builtin_amdgcn_sched_barrier(0);
            compute(u, g, ring[g % NB], fresh);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if constexpr (PEEL) {
        // two copies of the row body, the first row of a block and the others (with one body and a branch around the
        // block change the compiler copied all accumulators between the register files in every row)
        for (int u = ufirst; u < u_end;) {
            hand_over = u != ufirst || vp > 0;   // (a later pass of 256 columns starts with the block of the pass before)
            sweep_row(u, std::true_type{});
            u += NUG;
            for (int j = 1; j < FLUSH_ROWS && u < u_end; ++j, u += NUG) sweep_row(u, std::false_type{});
        }
    } else {
        // one row body; between two blocks the accumulators join the running sum and are cleared
        int rows_in_block = 0;
        for (int u = ufirst; u < u_end; u += NUG) {
            if (rows_in_block == FLUSH_ROWS) {
                rows_in_block = 0;
                __builtin_amdgcn_sched_barrier(0);
                matrix_results_settled();
#pragma unroll
                for (int cbt = 0; cbt < NCB * 4; ++cbt) {
                    v4f x[4];
                    run_load(cbt, x);
                    run_add_store(cbt, x);
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[cbt >> 2][cbt & 3][e] = 0.f;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            ++rows_in_block;
            sweep_row(u, std::false_type{});
        }
    }

    }   // column passes

    // the last block joins the running sum in the registers
#pragma unroll
    for (int cbt = 0; cbt < NCB * 4; ++cbt) {
        v4f x[4];
        run_load(cbt, x);
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[cbt >> 2][cbt & 3][4 * q + e] += x[q][e];
    }
    // every wave leaves its partial [32][CB] in its own LDS region; they are added in wave order on the way out
    {
        float *mine = smem + wave * (TP * RS);
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const v4f x = {acc[cb][0][r], acc[cb][1][r], acc[cb][2][r], acc[cb][3][r]};
                *reinterpret_cast<v4f *>(mine + pl * RS + 128 * cb + 4 * vmap(r, h)) = x;
            }
    }
    __syncthreads();
    // The sum over the waves' LDS regions for MI items of this thread (item = 4 channels of a pixel; items idx0,
    // idx0 + blockDim.x, ...): all reads of a batch are issued before the first addition, sums run in wave order.
    constexpr int MI = 4;
    constexpr int NIT = TP * (CB / 4);
    auto tile_sums = [&](int idx0, v4f (&x)[MI]) {
        v4f y[MI][4];
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int idx = min(idx0 + i * (int)blockDim.x, NIT - 1);
            const int row = idx / (CB / 4), c = (idx - row * (CB / 4)) * 4;
#pragma unroll
            for (int w = 0; w < 4; ++w)
                y[i][w] = *reinterpret_cast<const v4f *>(smem + min(w, nW - 1) * (TP * RS) + row * RS + c);
        }
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            x[i] = y[i][0];
#pragma unroll
            for (int w = 1; w < 4; ++w)
                if (w < nW) x[i] += y[i][w];
        }
        for (int w = 4; w < nW; ++w) {   // 5 to 8 waves (rows of more than 128 columns)
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int idx = min(idx0 + i * (int)blockDim.x, NIT - 1);
                const int row = idx / (CB / 4), c = (idx - row * (CB / 4)) * 4;
                x[i] += *reinterpret_cast<const v4f *>(smem + w * (TP * RS) + row * RS + c);
            }
        }
    };
    auto store_items = [&](int idx0, const v4f (&x)[MI]) {
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int idx = idx0 + i * (int)blockDim.x;
            const int row = idx / (CB / 4), c = (idx - row * (CB / 4)) * 4;
            if (idx < NIT && p0 + row < N1)
                store4<CVEC>(a.d1 + ((size_t)b * N1 + p0 + row) * C, cb0 + c, C, x[i], (a.accumulate | a.add_d1) != 0);
        }
    };
    if (whole) {
        for (int idx0 = tid; idx0 < NIT; idx0 += MI * blockDim.x) {
            v4f x[MI];
            tile_sums(idx0, x);
            store_items(idx0, x);
        }
    } else {
        // leave the piece's partial sum [32][CB] in this workgroup's slot, then see whether it completes the tile
        constexpr unsigned SLOT = TP * CB;
        const unsigned nslots = 2u * gridDim.x * gridDim.y;
        const __amdgpu_buffer_rsrc_t rs_sk = make_rsrc(a.sk_state, nslots * SLOT * 4u);
        const unsigned mine = (2u * (wg * gridDim.y + blockIdx.y) + (pb == gs0 ? 0u : 1u)) * SLOT;
        for (int idx0 = tid; idx0 < NIT; idx0 += MI * blockDim.x) {
            v4f x[MI];
            tile_sums(idx0, x);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int idx = idx0 + i * (int)blockDim.x;
                if (idx < NIT) store_shared4(rs_sk, (mine + (unsigned)idx * 4u) * 4u, x[i]);
            }
        }
        const int G = (int)gridDim.x;
        const long t0 = (long)tile * S, t1 = t0 + S;
        int wfirst = (int)((t0 * G) / sk_total);                         // the workgroup that holds step t0
        while (wfirst > 0 && ((long)wfirst * sk_total) / G > t0) --wfirst;
        while (((long)(wfirst + 1) * sk_total) / G <= t0) ++wfirst;
        int wlast = wfirst;                                              // the workgroup that holds step t1 - 1
        while (((long)(wlast + 1) * sk_total) / G < t1) ++wlast;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's part of the piece has arrived
        __syncthreads();
        int *flag = reinterpret_cast<int *>(smem);
        if (tid == 0)
            *flag = __hip_atomic_fetch_add(a.sk_count + tile * gridDim.y + blockIdx.y, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const bool last = *flag == wlast - wfirst;
        if (last) {   // pieces in row order, after what the destination already holds when accumulating
            constexpr int MJ = 8;   // items of a thread whose fetches from one piece are in flight together
            for (int idx0 = tid; idx0 < NIT; idx0 += MJ * blockDim.x) {
                v4f x[MJ];
#pragma unroll
                for (int i = 0; i < MJ; ++i) x[i] = v4f{0.f, 0.f, 0.f, 0.f};
                for (int w = wfirst; w <= wlast; ++w) {
                    const bool first_piece = ((long)w * sk_total) / G >= t0;
                    const unsigned slot = (2u * (w * gridDim.y + blockIdx.y) + (first_piece ? 0u : 1u)) * SLOT;
                    v4f y[MJ];
#pragma unroll
                    for (int i = 0; i < MJ; ++i) {
                        const int idx = idx0 + i * (int)blockDim.x;
                        y[i] = load_shared4(rs_sk, idx < NIT ? (slot + (unsigned)idx * 4u) * 4u : DMA_OOB);
                    }
#pragma unroll
                    for (int i = 0; i < MJ; ++i) x[i] += y[i];
                }
#pragma unroll
                for (int i = 0; i < MJ; ++i) {
                    const int idx = idx0 + i * (int)blockDim.x;
                    const int row = idx / (CB / 4), c = (idx - row * (CB / 4)) * 4;
                    if (idx < NIT && p0 + row < N1)
                        store4<CVEC>(a.d1 + ((size_t)b * N1 + p0 + row) * C, cb0 + c, C, x[i], (a.accumulate | a.add_d1) != 0);
                }
            }
        }
    }
    if constexpr (SK) __syncthreads();   // the next piece reuses the LDS tile
    }   // pieces of this workgroup
}

// d_f2[q, c] = sum_p G[p,q] f1[p,c].  Each wave is an independent task (b, split, u, v chunk);
// grid: (ceil(tasks / 4), channel blocks of 128*NCB), 256 threads.
template <int GMODE, int KC, int NCB, bool CVEC>
__global__ void __launch_bounds__(256) df2_kernel(const BwdArgs a, int ntasks, int nvc) {
    constexpr int GS = 2;
    constexpr int NG = 16 / GS;
    constexpr int CB = 128 * NCB;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, pl = lane & 31, h = lane >> 5;
    int task = blockIdx.x * 4 + wave;
    if (task >= ntasks) return;
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C;
    const int vc = task % nvc; task /= nvc;
    const int u = task % H2; task /= H2;
    const int split = task % a.nsplit;
    const int b = task / a.nsplit;
    const int cb0 = blockIdx.y * CB;
    const int v = 32 * vc + pl;
    const bool vok = v < W2;
    const int vs = vok ? v : 0;
    const int pbeg = split * a.tiles_per_split * TP;
    const int pend = min(N1, pbeg + a.tiles_per_split * TP);
    const int ntiles = (pend - pbeg + TP - 1) / TP;

    v16f acc[NCB][4];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[cb][t][e] = 0.f;

    struct Buf {
        v4f f[GS][NCB];
        VW<GMODE, KC> wv[GS];
        UW<GMODE, KC> wu[GS];
    };
    const unsigned nbytes1 = (unsigned)max(pend, 0) * C * 4u;   // pixels >= pend read as zero
    const __amdgpu_buffer_rsrc_t rsrc1 = make_rsrc(a.f1 + (size_t)b * N1 * C, nbytes1);
    unsigned coff[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int c = cb0 + 128 * cb + 4 * pl;
        coff[cb] = c < C ? (unsigned)c * 4u : nbytes1;
    }
    auto issue = [&](int tile, int g, Buf &buf) {
#pragma unroll
        for (int ss = 0; ss < GS; ++ss) {
            const int p = pbeg + tile * TP + 2 * (g * GS + ss) + h;
            const bool ok = p < pend;
            const size_t bp = (size_t)b * N1 + min(p, pend - 1);   // clamped: weights of a real pixel, masked in gval
            buf.wv[ss] = load_vw<GMODE, KC>(a, bp, vs, true);
            buf.wu[ss] = load_uw<GMODE, KC>(a, bp, u, true);
            if constexpr (CVEC) {
                const unsigned poff = ok ? (unsigned)p * C * 4u : nbytes1;
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) buf.f[ss][cb] = buf_load4(rsrc1, poff + coff[cb]);
            } else {
                const float *src = a.f1 + bp * C;
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) buf.f[ss][cb] = load4<false>(src, cb0 + 128 * cb + 4 * pl, C, ok);
            }
        }
    };
    auto compute = [&](int tile, int g, const Buf &buf) {
#pragma unroll
        for (int ss = 0; ss < GS; ++ss) {
            const int p = pbeg + tile * TP + 2 * (g * GS + ss) + h;
            const float G = gval<GMODE, KC>(buf.wv[ss], buf.wu[ss], u, v, p < pend && vok);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[cb][t] = mfma(buf.f[ss][cb][t], G, acc[cb][t]);
        }
    };

    Buf bufA, bufB;
    if (ntiles > 0) issue(0, 0, bufA);
    for (int tile = 0; tile < ntiles; ++tile) {
#pragma unroll
        for (int g = 0; g < NG; g += 2) {
            issue(tile, g + 1, bufB);
            compute(tile, g, bufA);
            if (g + 2 < NG) issue(tile, g + 2, bufA);
            else if (tile + 1 < ntiles) issue(tile + 1, 0, bufA);
            compute(tile, g + 1, bufB);
        }
    }

    if (vok) {
        float *dst = a.d2 + ((size_t)split * a.B + b) * H2 * W2 * C + ((size_t)u * W2 + v) * C;
        const bool accum = a.accumulate != 0 && a.nsplit == 1;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const v4f x = {acc[cb][0][r], acc[cb][1][r], acc[cb][2][r], acc[cb][3][r]};
                store4<CVEC>(dst, cb0 + 128 * cb + 4 * vmap(r, h), C, x, accum);
            }
    }
}


// Tiled d_f2: workgroup = 4 waves = 4 consecutive fmap2 rows u of one 32-column chunk; it sweeps the
// pixels p of its split in tiles of 32.  Per tile the f1 rows (A operand) and every weight indexed by
// (p, v) are DMA'd straight into LDS (buffer_load ... lds, double buffered, one barrier per tile) and
// shared by the four rows; the weights indexed by (p, u) are wave private.  G^T is synthesised from
// LDS into the B operand.  Requires C % 4 == 0 and W2 % 4 == 0.
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, float *lds_chunk, unsigned voff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_chunk, 16, voff, 0, 0, 0);
}

// buffers of the (p,u)-indexed weights per wave: the combined mode has LDS for one only
constexpr int df2_tiled_ubuf(int gmode) { return gmode == GMODE_BOTH ? 1 : 2; }

// NOAVGV: the term g_v[avg] / H2 of G does not depend on the row u, so its contribution to d_f2[(u,v),:] is the same
// for every u: the line v of a small table (BwdArgs::vtable, gather_backward.hip) that the workgroups of the first
// split add to their sums.  Without that weight tile in LDS the combined mode has room for 8 rows per workgroup.
template <int GMODE, int KC, int NCB, int NWV, bool NOAVGV = false>
__global__ void __launch_bounds__(64 * NWV) df2_tiled_kernel(const BwdArgs a, int nvc, int nug) {
    constexpr bool HC = g_has_comp(GMODE), HM = g_has_maxavg(GMODE);
    static_assert(!NOAVGV || HM, "only the max/avg part has an average term");
    constexpr int NVC = HC ? 2 * KC : 0;       // weight tensors of the compression part: a_u[k].., g_cv[k]..
    constexpr int NV = NVC + (HM ? (NOAVGV ? 2 : 3) : 0);     // then g_v[max], g_v[avg] (unless NOAVGV), argmax_v
    constexpr int NUP = (NV + 3) & ~3;
    constexpr int UBUF = df2_tiled_ubuf(GMODE);
    constexpr int CB = 128 * NCB;
    extern __shared__ float smem[];
    float *F1s = smem;                         // [2][32][CB]
    float *VWs = F1s + 2 * 32 * CB;            // [2][NV][32 p][32 v]
    float *UWs = VWs + 2 * NV * 1024;          // [NWV][UBUF][32 p][NUP]
    const int tid = threadIdx.x, lane = tid & 63, pl = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C;
    int vc, ug, split, b;
    if (a.uneven) {
        int q;
        const int hw = blockIdx.x, nlong = a.q_units * (a.nsplit - 1);
        if (a.xcd_order) {
            const int x = hw & 7, slot = hw >> 3, lx = a.xl[x + 1] - a.xl[x];
            const int unit = slot < lx ? a.xl[x] + slot : nlong + a.xs[x] + slot - lx;
            split = unit / a.q_units;
            q = unit - split * a.q_units;
        } else {
            split = hw / a.q_units;
            q = hw - split * a.q_units;
        }
        (void)nlong;
        vc = q % nvc; q /= nvc;
        ug = q % nug;
        b = q / nug;
    } else {
        int task = a.xcd_order ? xcd_contiguous(blockIdx.x, gridDim.x) : (int)blockIdx.x;
        vc = task % nvc; task /= nvc;
        ug = task % nug; task /= nug;
        split = task % a.nsplit;
        b = task / a.nsplit;
    }
    const int cb0 = blockIdx.y * CB;
    const int u_raw = ug * NWV + wave;
    const int u = min(u_raw, H2 - 1);
    const int v0 = 32 * vc, v = v0 + pl;
    const bool vok = v < W2;
    const int pbeg = split * a.tiles_per_split * TP;
    const int pend = min(N1, pbeg + a.tiles_per_split * TP);
    const int ntiles = (pend - pbeg + TP - 1) / TP;
    const float inv_h2 = 1.f / (float)H2, inv_w2 = 1.f / (float)W2;

    v16f acc[NCB][4];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[cb][t][e] = 0.f;

    if (ntiles > 0) {
        // buffer resources end at pixel `pend`: rows of later pixels read as zero
        const unsigned up = (unsigned)pend;
        const __amdgpu_buffer_rsrc_t rs_f1 = make_rsrc(a.f1 + (size_t)b * N1 * C, up * C * 4u);
        // the (p,v)-indexed tensors: a_u, g_cv (KT*W2 floats per pixel); g_v (2*W2), argmax_v (W2)
        __amdgpu_buffer_rsrc_t rs_va, rs_vb, rs_vc, rs_vd;
        const unsigned pstride_c = (unsigned)a.KT * W2;
        if constexpr (HC) {
            rs_va = make_rsrc(a.a_u + (size_t)b * N1 * pstride_c, up * pstride_c * 4u);
            rs_vb = make_rsrc(a.g_cv + (size_t)b * N1 * pstride_c, up * pstride_c * 4u);
        }
        if constexpr (HM) {
            rs_vc = make_rsrc(a.g_v + (size_t)b * N1 * 2u * W2, up * 2u * W2 * 4u);
            rs_vd = make_rsrc(a.am_v + (size_t)b * N1 * W2, up * W2 * 4u);
        }
        // DMA offsets = a lane-constant part (kept in registers) + a wave-uniform part that moves with the tile:
        // one vector add per transfer.  The pixel index stays inside the checked offset, so rows at or beyond
        // `pend` still read as zero.
        constexpr int FCH = CB / 8 / NWV;   // 256-float chunks of the f1 tile per wave
        const int frow = (lane * 4) / CB, fcol = (lane * 4) % CB;        // within a 256-float chunk of the f1 tile
        const unsigned fcoff = (cb0 + fcol < C) ? (unsigned)(cb0 + fcol) * 4u : DMA_OOB;
        unsigned f_lane[FCH];
#pragma unroll
        for (int i = 0; i < FCH; ++i) f_lane[i] = (unsigned)((wave * FCH + i) * (256 / CB) + frow) * C * 4u + fcoff;
        const unsigned vcol = (unsigned)(v0 + 4 * (lane & 7)) * 4u;
        const unsigned prow = (unsigned)(lane >> 3);                      // pixel of this lane within a weight chunk
        const unsigned wl_c = prow * pstride_c * 4u + vcol, wl_2 = prow * 2u * W2 * 4u + vcol, wl_1 = prow * W2 * 4u + vcol;

        auto issue_tile = [&](int tile, int bi) {
            const unsigned pt0 = (unsigned)(pbeg + tile * TP);
            float *fdst = F1s + bi * 32 * CB;
            const unsigned tf = pt0 * C * 4u;
#pragma unroll
            for (int i = 0; i < FCH; ++i) dma16(rs_f1, fdst + (wave * FCH + i) * 256, f_lane[i] + tf);
            float *vdst = VWs + bi * NV * 1024;
            // the weight tile of one tensor is four 256-float chunks (8 pixels each); chunk c = 4*kk + quarter
#pragma unroll
            for (int i = 0; i < (4 * NV + NWV - 1) / NWV; ++i) {
                const int c = wave + NWV * i;
                if (4 * NV % NWV != 0 && c >= 4 * NV) break;
                const int kk = c >> 2, quarter = c & 3;
                const unsigned p8 = pt0 + 8u * quarter;   // first pixel of the chunk (uniform)
                float *dst = vdst + c * 256;
                if (HC && kk < NVC) {
                    const unsigned uni = (p8 * pstride_c + (unsigned)(a.k0 + (kk % KC)) * W2) * 4u;
                    if constexpr (HC) dma16(kk < KC ? rs_va : rs_vb, dst, wl_c + uni);
                } else if constexpr (HM) {
                    const int m = kk - NVC;
                    if (m < (NOAVGV ? 1 : 2)) dma16(rs_vc, dst, wl_2 + (p8 * 2u * W2 + (unsigned)m * W2) * 4u);
                    else dma16(rs_vd, dst, wl_1 + p8 * W2 * 4u);
                }
            }
        };
        // (p,u)-indexed weights of this wave's row: lane pl fetches pixel pt0+pl (both halves the same), through
        // buffer loads whose channel/row part is a scalar offset
        __amdgpu_buffer_rsrc_t rs_av, rs_gcu, rs_gu, rs_amu;
        if constexpr (HC) {
            rs_av = make_rsrc(a.a_v + (size_t)b * N1 * a.KT * H2, (unsigned)N1 * a.KT * H2 * 4u);
            rs_gcu = make_rsrc(a.g_cu + (size_t)b * N1 * a.KT * H2, (unsigned)N1 * a.KT * H2 * 4u);
        }
        if constexpr (HM) {
            rs_gu = make_rsrc(a.g_u + (size_t)b * N1 * 2 * H2, (unsigned)N1 * 2u * H2 * 4u);
            rs_amu = make_rsrc(a.am_u + (size_t)b * N1 * H2, (unsigned)N1 * H2 * 4u);
        }
        auto load_uw_tile = [&](int tile, float(&r)[NUP]) {
            const unsigned p = (unsigned)min(pbeg + tile * TP + pl, pend - 1);
            const unsigned o1 = p * H2 * 4u;   // byte offset of the pixel's first entry in a 1-channel tensor
#pragma unroll
            for (int i = 0; i < NUP; ++i) r[i] = 0.f;
            if constexpr (HC) {
                const unsigned oc = o1 * a.KT;
#pragma unroll
                for (int k = 0; k < KC; ++k) {
                    const unsigned so = (unsigned)((a.k0 + k) * H2 + u) * 4u;
                    r[k] = buf_load1s(rs_av, oc, so);
                    r[KC + k] = buf_load1s(rs_gcu, oc, so);
                }
            }
            if constexpr (HM) {
                // stored as: value if the row's argmax is this column, value otherwise, argmax
                const float ma = buf_load1s(rs_gu, o1 * 2u, (unsigned)u * 4u);
                const float mg = buf_load1s(rs_gu, o1 * 2u, (unsigned)(H2 + u) * 4u) * inv_w2;
                r[NVC + 0] = mg + ma;
                r[NVC + 1] = mg;
                r[NVC + 2] = buf_load1s(rs_amu, o1, (unsigned)u * 4u);
            }
        };
        // With one buffer the rows of the next tile replace those of the current one after its last read:
        // the region is private to the wave and a wave's LDS accesses complete in order.
        auto store_uw_tile = [&](int bi, const float(&r)[NUP]) {
            float *dst = UWs + ((wave * UBUF + (UBUF == 2 ? bi : 0)) * 32 + pl) * NUP;
#pragma unroll
            for (int i = 0; i < NUP; i += 4) {
                const v4f x = {r[i], r[i + 1], r[i + 2], r[i + 3]};
                *reinterpret_cast<v4f *>(dst + i) = x;
            }
        };

        float uwr[NUP];
        issue_tile(0, 0);
        load_uw_tile(0, uwr);
        store_uw_tile(0, uwr);
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's DMA has landed
        __syncthreads();

        for (int tile = 0; tile < ntiles; ++tile) {
            const int bi = tile & 1;
            const bool more = tile + 1 < ntiles;
            if (more) {
                issue_tile(tile + 1, bi ^ 1);
                load_uw_tile(tile + 1, uwr);
            }
            const float *fs = F1s + bi * 32 * CB;
            const float *vs = VWs + bi * NV * 1024;
            const float *us = UWs + (wave * UBUF + (UBUF == 2 ? bi : 0)) * 32 * NUP;
            // Software pipeline over the 16 MFMA steps of the tile: the LDS operands of step s+1 are
            // fetched before the MFMAs of step s and its G is computed between them, so the matrix
            // pipe does not wait for LDS latency or for the G arithmetic.
            struct StepOps {
                float uw[NUP], vw[NV];
                v4f fa[NCB];
            };
            // one lane-dependent base address per LDS region and tile; every step is a constant offset from it
            // (an immediate of the LDS instruction, no address arithmetic in the loop)
            const float *us_l = us + h * NUP, *vs_l = vs + h * 32 + pl, *fs_l = fs + h * CB + 4 * pl;
            auto lds_fetch = [&](int s, StepOps &o) {
#pragma unroll
                for (int i = 0; i < NUP; i += 4) {
                    const v4f x = *reinterpret_cast<const v4f *>(us_l + 2 * s * NUP + i);
                    o.uw[i] = x[0]; o.uw[i + 1] = x[1]; o.uw[i + 2] = x[2]; o.uw[i + 3] = x[3];
                }
#pragma unroll
                for (int kk = 0; kk < NV; ++kk) o.vw[kk] = vs_l[kk * 1024 + 2 * s * 32];
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) o.fa[cb] = *reinterpret_cast<const v4f *>(fs_l + 2 * s * CB + 128 * cb);
            };
            auto g_of = [&](int s, const StepOps &o) {
                float G = 0.f;
                if constexpr (HC) {
#pragma unroll
                    for (int k = 0; k < KC; ++k) {
                        G = fmaf(o.vw[k], o.uw[KC + k], G);
                        G = fmaf(o.uw[k], o.vw[KC + k], G);
                    }
                }
                if constexpr (HM) {
                    G += __float_as_int(o.uw[NVC + 2]) == v ? o.uw[NVC] : o.uw[NVC + 1];
                    if constexpr (NOAVGV) {
                        if (__float_as_int(o.vw[NVC + 1]) == u) G += o.vw[NVC];
                    } else {
                        G = fmaf(o.vw[NVC + 1], inv_h2, G);
                        if (__float_as_int(o.vw[NVC + 2]) == u) G += o.vw[NVC];
                    }
                }
                // No mask needed: pixels at or beyond `pend` have all-zero f1 rows and (p,v) weights (DMA
                // bounds), so whatever finite G they get multiplies zeros; columns beyond W2 are not stored.
                return G;
            };
            StepOps cur, nxt;
            lds_fetch(0, cur);
            float Gc = g_of(0, cur), Gn = 0.f;
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                if (s + 1 < 16) lds_fetch(s + 1, nxt);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[0][t] = mfma(cur.fa[0][t], Gc, acc[0][t]);
                __builtin_amdgcn_sched_barrier(0);
                if (s + 1 < 16) Gn = g_of(s + 1, nxt);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int cb = 1; cb < NCB; ++cb)
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[cb][t] = mfma(cur.fa[cb][t], Gc, acc[cb][t]);
                cur = nxt;
                Gc = Gn;
            }
            if (more) store_uw_tile(bi ^ 1, uwr);
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        }
    }

    if (vok && u_raw < H2) {
        float *dst = a.d2 + ((size_t)split * a.B + b) * H2 * W2 * C + ((size_t)u * W2 + v) * C;
        const bool accum = a.accumulate != 0 && a.nsplit == 1;
        const bool add_line = NOAVGV && split == 0;   // the average term of g_v, once per output element
        const float *line = a.vtable + ((size_t)b * W2 + v) * C;
        (void)inv_h2;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                v4f x = {acc[cb][0][r], acc[cb][1][r], acc[cb][2][r], acc[cb][3][r]};
                const int c = cb0 + 128 * cb + 4 * vmap(r, h);
                if constexpr (NOAVGV) {
                    if (add_line && c < C) x += *reinterpret_cast<const v4f *>(line + c);
                }
                store4<true>(dst, c, C, x, accum);
            }
    }
}

// d_f1 in bf16 planes (C == 256, rows of at most 256 columns).  Workgroup = 4 waves = 128 pixels p x one chunk of 32
// columns; it sweeps the rows u.  Per row the 48 KB block of transposed fmap2 planes is DMA'd into LDS (double
// buffered, one barrier per row) and shared by the four waves, each of which owns 32 pixels and all 256 channels
// (128 accumulator registers).  dL/dS of the next row is synthesised and split into planes between the MFMAs of
// the current one.  The workgroups of the column chunks of a row leave partial sums [chunk][B, N1, 256] that
// reduce_splits_kernel adds in chunk order (no atomics).
__device__ __forceinline__ void dma16s(__amdgpu_buffer_rsrc_t r, float *lds_chunk, unsigned voff, unsigned soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_chunk, 16, voff, soff, 0, 0);
}
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
constexpr int DF1BF_RS = 260;   // floats per pixel row of the output transpose in LDS

// The (p,u)-indexed weights of d_f1 in row-major order of u: out[b][u][f][p], fields f = a_v[k], g_cu[k] (k < KC),
// then g_u max, g_u avg, argmax_u as the mode has them.  In the operator's layout a lane's weight of row u is 4 bytes
// of its own pixel's line, so the 64 lanes of a load touch 64 lines and the lines of all pixels have to stay cached
// from one row to the next; with more than a few fields they do not, and every row fetches them from HBM again.
// Transposed, a wave's load is 128 contiguous bytes that are used once.
// Grid: (B * ceil(N1 / 64), fields); 256 threads.
template <int GMODE>
__global__ void __launch_bounds__(256) transpose_uw_kernel(const BwdArgs a, int KC, float *__restrict__ out) {
    __shared__ float tile[64 * 65];
    const int NF = (g_has_comp(GMODE) ? 2 * KC : 0) + (g_has_maxavg(GMODE) ? 3 : 0);
    const int tiles = (a.N1 + 63) / 64;
    const int b = blockIdx.x / tiles, p0 = (blockIdx.x % tiles) * 64, f = blockIdx.y;
    const int H2 = a.H2, N1 = a.N1;
    const int np = min(64, N1 - p0);
    // source row of pixel p for this field: H2 contiguous floats
    const float *src;
    size_t pstride;
    const int fm = f - (g_has_comp(GMODE) ? 2 * KC : 0);
    if (g_has_comp(GMODE) && f < 2 * KC) {
        const float *base = f < KC ? a.a_v : a.g_cu;
        const int kk = f < KC ? f : f - KC;
        src = base + (((size_t)b * N1 + p0) * a.KT + a.k0 + kk) * H2;
        pstride = (size_t)a.KT * H2;
    } else if (fm < 2) {
        src = a.g_u + (((size_t)b * N1 + p0) * 2 + fm) * H2;
        pstride = (size_t)2 * H2;
    } else {
        src = reinterpret_cast<const float *>(a.am_u) + ((size_t)b * N1 + p0) * H2;
        pstride = (size_t)H2;
    }
    // a wave takes every 4th pixel with lanes along u (two pixels at a time when a row has at most 32 entries), then
    // every 4th row u with lanes along the pixels
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int u0 = 0; u0 < H2; u0 += 64) {
        const int nu = min(64, H2 - u0);
        const int lpr = nu <= 32 ? 32 : 64, sub = lane / lpr, u = lane & (lpr - 1);
        if (u < nu)
            for (int p = wave * (64 / lpr) + sub; p < np; p += 4 * (64 / lpr)) tile[p * 65 + u] = src[p * pstride + u0 + u];
        __syncthreads();
        if (lane < np)
            for (int uu = wave; uu < nu; uu += 4) out[(((size_t)b * H2 + u0 + uu) * NF + f) * N1 + p0 + lane] = tile[lane * 65 + uu];
        __syncthreads();
    }
}

// NW: waves per workgroup.  4 (one per SIMD, up to 512 registers) is what is launched; 8 (two per SIMD) fits the
// max/avg mode only with spills and measured the same.
template <int GMODE, int KC, int NW>
__global__ void __launch_bounds__(64 * NW) df1_bf_kernel(const BwdArgs a, const char *__restrict__ planes,
                                                         const float *__restrict__ uwt, float *__restrict__ dst, int nvc,
                                                         int ptiles) {
    extern __shared__ float smem[];   // two 48 KB row blocks; reused for the output transpose
    const int tid = threadIdx.x, lane = tid & 63, pl = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = a.xcd_order ? xcd_contiguous(blockIdx.x, gridDim.x) : (int)blockIdx.x;
    const int ptile = wg % ptiles, vc = (wg / ptiles) % nvc, b = wg / (ptiles * nvc);
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2;
    const int pix = ptile * (32 * NW) + 32 * wave + pl;
    const bool pok = pix < N1;
    const size_t bp = (size_t)b * N1 + (pok ? pix : 0);

    v16f acc[8];
#pragma unroll
    for (int cb = 0; cb < 8; ++cb)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[cb][e] = 0.f;

    // register r = 8 s + e of a lane belongs to column 32 vc + 16 s + 8 h + e
    const int lanebase = 32 * vc + 8 * h;
    VW<GMODE, KC> wv[16];
    {
        int vs[16];
        bool oks[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int v = lanebase + 16 * (r >> 3) + (r & 7);
            vs[r] = v < W2 ? v : 0;
            oks[r] = pok && v < W2;
        }
        load_vw16<GMODE, KC>(a, bp, vs, oks, wv);
    }

    // transposed (p,u) weights of this image: [u][field][p]
    constexpr int NVC = g_has_comp(GMODE) ? 2 * KC : 0;
    constexpr int NF = NVC + (g_has_maxavg(GMODE) ? 3 : 0);
    const unsigned pix4 = (pok ? (unsigned)pix : 0u) * 4u;
    const __amdgpu_buffer_rsrc_t rs_uw = make_rsrc(uwt + (size_t)b * H2 * NF * N1, (unsigned)H2 * NF * N1 * 4u);
    const float inv_w2 = 1.f / (float)W2;
    // The loads of a row's (p,u)-indexed weights are issued ahead of the row block's DMA and finished (scaled,
    // made relative) only after the row's MFMAs: waiting for one of them then never waits for the DMA behind it.
    struct UWRaw { float a[KC], g[KC], avg, mx, am; };
    auto issue_uw_row = [&](int u) {
        UWRaw w;
        const unsigned row = (unsigned)u * NF * N1 * 4u;
        if constexpr (g_has_comp(GMODE)) {
#pragma unroll
            for (int k = 0; k < KC; ++k) {
                w.a[k] = buf_load1s(rs_uw, pix4, row + (unsigned)k * N1 * 4u);
                w.g[k] = buf_load1s(rs_uw, pix4, row + (unsigned)(KC + k) * N1 * 4u);
            }
        }
        if constexpr (g_has_maxavg(GMODE)) {
            w.mx = buf_load1s(rs_uw, pix4, row + (unsigned)NVC * N1 * 4u);
            w.avg = buf_load1s(rs_uw, pix4, row + (unsigned)(NVC + 1) * N1 * 4u);
            w.am = buf_load1s(rs_uw, pix4, row + (unsigned)(NVC + 2) * N1 * 4u);
        }
        return w;
    };
    auto finish_uw_row = [&](const UWRaw &r) {
        UW<GMODE, KC> w;
        if constexpr (g_has_comp(GMODE)) {
#pragma unroll
            for (int k = 0; k < KC; ++k) { w.a[k] = r.a[k]; w.g[k] = r.g[k]; }
        }
        if constexpr (g_has_maxavg(GMODE)) {
            w.mg = r.avg * inv_w2;
            w.ma = w.mg + r.mx;
            w.am = __float_as_int(r.am) - lanebase;
        }
        return w;
    };
    auto load_uw_row = [&](int u) { return finish_uw_row(issue_uw_row(u)); };

    const unsigned nbytes = (unsigned)H2 * nvc * BF_CHUNK;
    const __amdgpu_buffer_rsrc_t rs_pl = make_rsrc(planes + (size_t)b * nbytes, nbytes);
    constexpr int KBW = 48 / NW;   // KB of a row block moved by each wave
    auto issue_row = [&](int u, int bi) {
        const unsigned blk = (unsigned)(u * nvc + vc) * BF_CHUNK;
#pragma unroll
        for (int i = 0; i < KBW; ++i) {
            const int kb = wave * KBW + i;
            dma16s(rs_pl, smem + bi * (BF_CHUNK / 4) + kb * 256, 16u * lane, blk + (unsigned)kb * 1024u);
        }
    };

    // G of a row as bf16 planes: dword j of plane q holds registers 2j, 2j+1 (half s = j / 4)
    v4u gp[3][2], gn[3][2];
    auto g_pair = [&](const UW<GMODE, KC> &wu, int u, int j, v4u(&out)[3][2]) {
        int un = u;
        asm volatile("" : "+s"(un));   // (keeps the comparison with argmax_v a compare against a scalar)
        const float x0 = gval<GMODE, KC>(wv[2 * j], wu, un, 16 * ((2 * j) >> 3) + ((2 * j) & 7), true);
        const float x1 = gval<GMODE, KC>(wv[2 * j + 1], wu, un, 16 * ((2 * j + 1) >> 3) + ((2 * j + 1) & 7), true);
        const v2bf hh = {(__bf16)x0, (__bf16)x1};
        const float r0 = x0 - (float)hh[0], r1 = x1 - (float)hh[1];
        const v2bf mm = {(__bf16)r0, (__bf16)r1};
        const v2bf ll = {(__bf16)(r0 - (float)mm[0]), (__bf16)(r1 - (float)mm[1])};
        out[0][j >> 2][j & 3] = __builtin_bit_cast(unsigned, hh);
        out[1][j >> 2][j & 3] = __builtin_bit_cast(unsigned, mm);
        out[2][j >> 2][j & 3] = __builtin_bit_cast(unsigned, ll);
    };

    UW<GMODE, KC> wu_n = load_uw_row(0);
    issue_row(0, 0);
#pragma unroll
    for (int j = 0; j < 8; ++j) g_pair(wu_n, 0, j, gp);
    wu_n = load_uw_row(min(1, H2 - 1));
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's DMA has landed
    __syncthreads();

    constexpr int PA[6] = {2, 0, 1, 1, 0, 0}, PB[6] = {0, 2, 1, 0, 1, 0};   // (fmap2 plane, G plane), small products first
    // One row = 8 regions of two channel blocks (same column half): 12 MFMAs that alternate between the two
    // accumulators, the 6 LDS reads of the next region and one pair of next-row G values.  A wave is alone on its
    // SIMD and issues in order, so the vector work only overlaps the matrix pipe if it sits between the MFMAs:
    // the group barriers below ask for that interleaving.
    for (int u = 0; u < H2; ++u) {
        const v4u(&gc)[3][2] = gp;
        v4u(&gx)[3][2] = gn;
        const int bi = u & 1;
        const UW<GMODE, KC> wu_c = wu_n;                       // weights of row u + 1
        const UWRaw wu_raw = issue_uw_row(min(u + 2, H2 - 1));
        __builtin_amdgcn_sched_barrier(0);
        const char *abase = reinterpret_cast<const char *>(smem) + bi * BF_CHUNK + 16 * lane;
        v8bf A[2][2][3];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int q = 0; q < 3; ++q) A[0][i][q] = *reinterpret_cast<const v8bf *>(abase + (i * 3 + q) * 1024);
#pragma unroll
        for (int R = 0; R < 8; ++R) {   // groups g = 8 s + cb: 2R and 2R + 1
            const int s = R >> 2, cb0 = 2 * (R & 3), cur = R & 1;
            __builtin_amdgcn_sched_barrier(0);
            if (R + 1 < 8) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int q = 0; q < 3; ++q)
                        A[cur ^ 1][i][q] = *reinterpret_cast<const v8bf *>(abase + ((2 * R + 2 + i) * 3 + q) * 1024);
            }
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    acc[cb0 + i] = mfma_bf(A[cur][i][PA[t]], __builtin_bit_cast(v8bf, gc[PB[t]][s]), acc[cb0 + i]);
            g_pair(wu_c, u + 1, R, gx);
            // the next row's block: this wave's KBs spread over the first six regions (issuing a DMA holds the
            // wave for a while; spread out, that time falls into the shadow of the MFMAs)
            // (no branch on the last row: it fetches its own block once more, into the buffer nobody reads again;
            // a branch here would split the loop body and undo the interleaving)
            if (R < 6) {
                const unsigned blk = (unsigned)(min(u + 1, H2 - 1) * nvc + vc) * BF_CHUNK;
#pragma unroll
                for (int i = 0; i < KBW / 6; ++i) {
                    const int kb = wave * KBW + (KBW / 6) * R + i;
                    dma16s(rs_pl, smem + (bi ^ 1) * (BF_CHUNK / 4) + kb * 256, 16u * lane, blk + (unsigned)kb * 1024u);
                }
            }
#pragma unroll
            for (int k = 0; k < 12; ++k) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
                if (k < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);               // up to four vector instructions
                if (k == 1 || (k == 3 && KBW == 12)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one DMA
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < 3; ++q)
#pragma unroll
            for (int i = 0; i < 2; ++i) gp[q][i] = gn[q][i];
        __builtin_amdgcn_s_waitcnt(0x0F70);
        wu_n = finish_uw_row(wu_raw);
        __syncthreads();
    }

    // transpose through LDS (one region per wave, four waves at a time): a pixel's 256 channels leave as one
    // contiguous KB
    float *reg = smem + (wave & 3) * 32 * DF1BF_RS;
    float *out = dst + ((size_t)(nvc > 1 ? vc : 0) * a.B + b) * N1 * 256;
    const bool accum = nvc == 1 && (a.accumulate | a.add_d1) != 0;
#pragma unroll
    for (int half = 0; half < NW / 4; ++half) {
        if (half > 0) __syncthreads();
        if ((wave >> 2) == half) {
#pragma unroll
            for (int cb = 0; cb < 8; ++cb)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    const v4f x = {acc[cb][4 * rq], acc[cb][4 * rq + 1], acc[cb][4 * rq + 2], acc[cb][4 * rq + 3]};
                    *reinterpret_cast<v4f *>(reg + pl * DF1BF_RS + 32 * cb + 8 * rq + 4 * h) = x;
                }
            __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the wave's own LDS writes are done (no other wave reads them)
            for (int j = 0; j < 32; ++j) {
                const int p = ptile * (32 * NW) + 32 * wave + j;
                if (p < N1) {
                    v4f x = *reinterpret_cast<const v4f *>(reg + j * DF1BF_RS + 4 * lane);
                    v4f *o = reinterpret_cast<v4f *>(out + (size_t)p * 256 + 4 * lane);
                    if (accum) x += *o;
                    *o = x;
                }
            }
        }
    }
}

// out[i] (+)= sum_s part[s*n + i], in split order.
__global__ void __launch_bounds__(256) reduce_splits_kernel(const float *part, float *out, size_t n, int nsplit,
                                                            int accumulate) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    if (n % 4 == 0 && (reinterpret_cast<uintptr_t>(part) | reinterpret_cast<uintptr_t>(out)) % 16 == 0) {
        // four elements per thread and several splits in flight
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n / 4; i += stride) {
            v4f s = accumulate ? reinterpret_cast<const v4f *>(out)[i] : v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
            for (int k = 0; k < nsplit; ++k) s += reinterpret_cast<const v4f *>(part + (size_t)k * n)[i];
            reinterpret_cast<v4f *>(out)[i] = s;
        }
        return;
    }
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float s = accumulate ? out[i] : 0.f;
        for (int k = 0; k < nsplit; ++k) s += part[(size_t)k * n + i];
        out[i] = s;
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
}  // namespace
namespace sepcorr_impl {
struct Dims {
    int B, H1, W1, H2, W2, C;
};
}  // namespace sepcorr_impl
namespace {

int check_dims(const Dims &d, int K) {
    if (d.B < 1 || d.H1 < 1 || d.W1 < 1 || d.H2 < 1 || d.W2 < 1 || d.C < 1)
        return fail(SEPCORR_EINVAL, "sepcorr: all sizes must be >= 1 (B=%d H1=%d W1=%d H2=%d W2=%d C=%d)", d.B, d.H1,
                    d.W1, d.H2, d.W2, d.C);
    if (d.W2 > MAX_W2) return fail(SEPCORR_EINVAL, "sepcorr: W2=%d exceeds the supported maximum %d", d.W2, MAX_W2);
    if (d.C > MAX_C) return fail(SEPCORR_EINVAL, "sepcorr: C=%d exceeds the supported maximum %d", d.C, MAX_C);
    if (K < 1 || K > MAX_K) return fail(SEPCORR_EINVAL, "sepcorr: K=%d outside 1..%d", K, MAX_K);
    const double lim = 2147483647.0;
    const double n1 = (double)d.B * d.H1 * d.W1, n2 = (double)d.B * d.H2 * d.W2;
    const int ch = K > 2 ? K : 2;
    if (n1 * d.C > lim || n2 * d.C > lim || n1 * ch * d.H2 > lim || n1 * ch * d.W2 > lim)
        return fail(SEPCORR_EINVAL, "sepcorr: a tensor would have 2^31 or more elements");
    return SEPCORR_OK;
}

// Optional per-kernel timing: when enabled, every kernel launch is bracketed by HIP events recorded
// on the stream it is launched on.  Off by default (zero cost: one branch per launch).
}  // namespace
namespace sepcorr_impl {
struct ProfRec {
    const char *name;
    hipEvent_t e0, e1;
};
extern std::atomic<bool> g_prof_on;
// The flag as the current API call saw it on entry: fork/join and every launch bracket of one call agree even if
// another thread toggles profiling meanwhile.
extern thread_local bool t_prof_on;
// Set for the duration of a call that must not allocate: no side streams or events are created, no stream-ordered
// memory is taken (the bf16-plane contraction is skipped), no timing events are recorded.
extern thread_local bool t_no_alloc;
extern std::mutex g_prof_mu;
extern std::vector<ProfRec> g_prof_recs;
extern std::atomic<int> g_contraction;
extern std::atomic<int> g_maxavg_backward;
#if SEPCORR_IN_PART(0)
std::atomic<bool> g_prof_on{false};
thread_local bool t_prof_on = false;
thread_local bool t_no_alloc = false;
std::mutex g_prof_mu;
std::vector<ProfRec> g_prof_recs;
#endif
}  // namespace sepcorr_impl
namespace {
void api_enter() { t_prof_on = g_prof_on.load(std::memory_order_relaxed); }

struct ProfScope {
    ProfRec rec;
    hipStream_t s;
    bool on;
    ProfScope(const char *name, hipStream_t stream) : s(stream), on(t_prof_on) {
        if (!on) return;
        rec.name = name;
        if (hipEventCreate(&rec.e0) != hipSuccess || hipEventCreate(&rec.e1) != hipSuccess) { on = false; return; }
        (void)hipEventRecord(rec.e0, s);
    }
    ~ProfScope() {
        if (!on) return;
        (void)hipEventRecord(rec.e1, s);
        std::lock_guard<std::mutex> lk(g_prof_mu);
        g_prof_recs.push_back(rec);
    }
};

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SEPCORR_ELAUNCH, "sepcorr: %s: %s", what, hipGetErrorString(e));
    return SEPCORR_OK;
}

template <typename KernelT>
int set_lds(KernelT kernel, size_t bytes) {
    if (bytes > 64 * 1024) {
        const hipError_t e =
            hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return fail(SEPCORR_ELAUNCH, "sepcorr: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
    }
    return SEPCORR_OK;
}

// Waves per workgroup of the p-owner kernels: nvc column chunks x NUG row groups.
struct WaveGrid {
    int nvc, nug, vpasses;
};
// dealt: the sweep's steps will be dealt out to workgroups (fwd_split): two 4-wave workgroups per CU then fill the
// SIMDs and may end on a single row, which two row groups cannot (B=1, 55x128: 0.539 -> 0.514 ms for both sweeps)
WaveGrid wave_grid(int B, int tiles_per_batch, int W2, int H2, bool dealt = false) {
    WaveGrid g;
    g.nvc = (W2 + 31) / 32;
    g.vpasses = (g.nvc + 7) / 8;
    if (g.nvc > 8) g.nvc = 8;
    g.nug = 1;
    if (g.nvc <= 2) {
        g.nug = 4 / g.nvc;                                        // 4 waves
        if (!dealt && (long)B * tiles_per_batch * 4 < 1536) g.nug *= 2;     // small problem: 8 waves fill more SIMDs
        while (g.nug > 1 && g.nug > H2) g.nug /= 2;
    } else if (!dealt && g.nvc <= 4 && (long)B * tiles_per_batch <= 256 && H2 >= 8) {
        g.nug = 2;   // at most one workgroup per CU: two row groups give every SIMD a second wave
    }
    return g;
}

// Row-wise helpers of the softmax inside the weighted sweeps: one wave per row of L floats, lanes along the row.
__device__ __forceinline__ float wave_max64(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ float wave_sum64(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
    return x;
}
// st[row] = (max, sum of exp(z - max))
__global__ void __launch_bounds__(256) row_stats_kernel(const float *__restrict__ z, float *__restrict__ st, long nrows, int L) {
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= nrows) return;
    const float *r = z + row * L;
    float m = -INFINITY;
    for (int l = lane; l < L; l += 64) m = fmaxf(m, r[l]);
    m = wave_max64(m);
    float sum = 0.f;
    for (int l = lane; l < L; l += 64) sum += __expf(r[l] - m);
    sum = wave_sum64(sum);
    if (lane == 0) { st[2 * row] = m; st[2 * row + 1] = sum; }
}
// Rows of L floats dealt to the waves of a workgroup with lanes along the row, VL entries per lane (4: 16-byte
// accesses, for rows whose length is a multiple of 4 in 16-byte aligned tensors): lpr lanes per row (a power of two,
// at least ceil(L / VL), at most 64), 64 / lpr rows side by side in a wave, ROWS_PER_WAVE rows per wave in all.
constexpr int ROWS_PER_WAVE = 8;   // (a step's loads, arithmetic and store follow one another: 32 rows per wave measured slower)
struct RowDeal {
    int lpr, rpw, row, pos;   // lanes per row, rows per wave and step, this lane's row within the step, its place in the row
};
__device__ __forceinline__ RowDeal row_deal(int L, int VL) {
    RowDeal r;
    const int need = (L + VL - 1) / VL;
    r.lpr = need <= 1 ? 1 : need >= 33 ? 64 : 1 << (32 - __builtin_clz(need - 1));
    r.rpw = 64 / r.lpr;
    const int lane = threadIdx.x & 63;
    r.row = lane / r.lpr;
    r.pos = lane & (r.lpr - 1);
    return r;
}
inline bool rows_vec4(const void *p, int L) { return L % 4 == 0 && (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
inline unsigned row_groups(size_t nrows) { return (unsigned)((nrows + 4 * ROWS_PER_WAVE - 1) / (4 * ROWS_PER_WAVE)); }

// dot[row] = sum_l x[row,l] * y[row,l] of one pair of tensors; the sum over a row's lanes by a butterfly (fixed order)
__device__ __forceinline__ void row_dots(const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ dot, long nrows,
                                         int L, bool vec4) {
    const RowDeal rd = row_deal(L, vec4 ? 4 : 1);
    const long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * ROWS_PER_WAVE;
    for (int i = rd.row; i < ROWS_PER_WAVE; i += rd.rpw) {
        const long row = r0 + i;
        float sum = 0.f;
        if (row < nrows) {
            const float *xr = x + row * L, *yr = y + row * L;
            if (vec4) {
                for (int l = 4 * rd.pos; l < L; l += 4 * rd.lpr) {
                    const float4 a = *reinterpret_cast<const float4 *>(xr + l), b = *reinterpret_cast<const float4 *>(yr + l);
                    sum += (a.x * b.x + a.y * b.y) + (a.z * b.z + a.w * b.w);
                }
            } else {
                for (int l = rd.pos; l < L; l += rd.lpr) sum += xr[l] * yr[l];
            }
        }
        for (int o = rd.lpr >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
        if (row < nrows && rd.pos == 0) dot[row] = sum;
    }
}
__global__ void __launch_bounds__(256) row_dot_kernel(const float *__restrict__ x, const float *__restrict__ y, float *__restrict__ dot,
                                                      long nrows, int L, int vec4) {
    row_dots(x, y, dot, nrows, L, vec4 != 0);
}
// The same for up to 8 pairs of tensors with the same number of rows (the two outputs of every pyramid level) in one
// launch: blockIdx.y picks the pair.
struct RowDotJobs {
    const float *x[8], *y[8];
    float *dot[8];
    int L[8], vec4[8];
};
__global__ void __launch_bounds__(256) row_dot_multi_kernel(const RowDotJobs j, long nrows) {
    const int job = blockIdx.y;
    row_dots(j.x[job], j.y[job], j.dot[job], nrows, j.L[job], j.vec4[job] != 0);
}
// a[row,l] = exp(z[row,l] - max) / sum
__global__ void __launch_bounds__(256) softmax_apply_kernel(const float *__restrict__ z, const float *__restrict__ st, float *__restrict__ a,
                                                            long nrows, int L, int vec4) {
    const RowDeal rd = row_deal(L, vec4 ? 4 : 1);
    const long r0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * ROWS_PER_WAVE;
    for (int i = rd.row; i < ROWS_PER_WAVE; i += rd.rpw) {
        const long row = r0 + i;
        if (row >= nrows) break;
        const float m = st[2 * row], il = 1.f / st[2 * row + 1];
        const float *zr = z + row * L;
        float *ar = a + row * L;
        if (vec4) {
            for (int l = 4 * rd.pos; l < L; l += 4 * rd.lpr) {
                const float4 v = *reinterpret_cast<const float4 *>(zr + l);
                *reinterpret_cast<float4 *>(ar + l) = make_float4(__expf(v.x - m) * il, __expf(v.y - m) * il, __expf(v.z - m) * il, __expf(v.w - m) * il);
            }
        } else {
            for (int l = rd.pos; l < L; l += rd.lpr) ar[l] = __expf(zr[l] - m) * il;
        }
    }
}

__global__ void __launch_bounds__(256) zero_ints_kernel(int *p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

// How a forward-type sweep is dealt out to workgroups.  Whole tiles (one workgroup each) leave part of the chip idle
// when the tile count is not close to a multiple of the resident workgroups (440 tiles on 512 places: 86 %); then the
// steps of all tiles are dealt out evenly instead and pieces of a tile are combined by whichever finishes last.
struct FwdSplit {
    bool on;
    int G, S;          // workgroups, units per tile
    long T;            // units in total
    size_t count_bytes, slot_floats, bytes;   // scratch: counters, one slot, everything
};
constexpr int kCUs = 256;
// What a sweep deals out per tile: steps (ur rows per wave, nug row groups) where a wave takes one row per step, half
// steps where it takes two (fwd_kernel: HU); the second half of the last step is left out when it holds no row.
int fwd_units(int H2, int ur, int nug, int vpasses) {
    const int steps = (H2 + ur * nug - 1) / (ur * nug);
    if (ur != 2 || nug != 1 || vpasses != 1) return steps;   // (row groups, column passes: whole steps, as the kernel's HU says)
    return 2 * steps - ((steps - 1) * 2 * nug + 1 >= H2 ? 1 : 0);
}
FwdSplit fwd_split(int tiles, int H2, int W2, int ur, int nug, int vpasses, int nq, int wgs_per_cu) {
    FwdSplit f;
    f.S = fwd_units(H2, ur, nug, vpasses);
    f.T = (long)tiles * f.S;
    const long places = (long)kCUs * wgs_per_cu;
    const double plain = (double)tiles / (double)(((tiles + places - 1) / places) * places);
    f.G = (int)(f.T < places ? f.T : places);
    const double split = (double)f.T / (double)(((f.T + f.G - 1) / f.G) * f.G);
    f.on = f.S >= 2 && f.T < (1L << 30) && split > plain + 0.04;
    f.count_bytes = ((size_t)tiles * sizeof(int) + 255) & ~(size_t)255;
    f.slot_floats = (size_t)nq * 1024 * ((W2 + 31) / 32);   // [column chunk][quantity][4 register groups][64 lanes][4]
    f.bytes = f.on ? f.count_bytes + 2 * (size_t)f.G * f.slot_floats * sizeof(float) : 0;
    return f;
}
// Upper bound of the scratch any forward-type sweep of these sizes asks for (channels of the widest launch).
size_t fwd_split_bytes(int B, int H1, int W1, int H2, int W2, int K) {
    const int tpb = (H1 * W1 + TP - 1) / TP;
    const int nq = K > 3 ? (K < KCH ? K : KCH) : 3;
    size_t best = 0;
    for (int dealt = 0; dealt <= 1; ++dealt) {
        const WaveGrid wg = wave_grid(B, tpb, W2, H2, dealt != 0);
        const int nW = wg.nvc * wg.nug;
        for (int ur = 1; ur <= 2; ++ur)
            for (int per = 1; per <= (nW <= 4 ? 2 : 1); ++per) {
                const FwdSplit f = fwd_split(B * tpb, H2, W2, ur, wg.nug, wg.vpasses, nq, per);
                if (f.bytes > best) best = f.bytes;
            }
    }
    return best;
}

}  // namespace
namespace sepcorr_impl {
template <int MODE, int KC, int UR>
int launch_fwd(FwdArgs a, int B, hipStream_t s) {
    constexpr int NPART = (is_weighted(MODE)) ? KC : 3;
    const bool may_deal = a.ws != nullptr && !a.f2_planes;
    WaveGrid wg;
    int nW = 0;
    size_t lds = 0;
    FwdSplit f = {};
    // LDS and the deal for one shape of the workgroup; tried first in the shape that suits dealt-out steps, then (when
    // that deal is off or the scratch too small) in the shape for whole tiles
    auto shape = [&](bool dealt) {
        wg = wave_grid(B, a.tiles_per_batch, a.W2, a.H2, dealt);
        nW = wg.nvc * wg.nug;
        lds = ((size_t)TP * (a.CP + 4) + 2 * UR * NPART * nW * 32) * sizeof(float);
        // stage out_u in LDS when two workgroups still fit a CU's 160 KB
        constexpr int NCHO = (is_weighted(MODE)) ? KC : 2;
        const size_t extra = (size_t)TP * (NCHO + (MODE == MODE_ARGMAX ? 1 : 0)) * a.H2 * sizeof(float);
        a.stage = lds + extra <= 80 * 1024;
        if (a.stage) lds += extra;
        // the final merge of the row groups reuses LDS from offset 0
        const size_t merge = wg.nug > 1 ? (size_t)wg.nvc * NPART * 16 * 64 * sizeof(float) : 0;
        if (lds < merge) lds = merge;
        if (MODE == MODE_SOFT) lds += (size_t)TP * KC * 3 * sizeof(float);   // row statistics of the tile
        f = FwdSplit{};
        if (may_deal) f = fwd_split(B * a.tiles_per_batch, a.H2, a.W2, UR, wg.nug, wg.vpasses, NPART, (nW <= 4 && lds <= 80 * 1024) ? 2 : 1);
        return f.on && f.bytes <= a.ws_bytes;
    };
    if (!shape(may_deal) && may_deal) shape(false);
    a.nvc = wg.nvc;
    a.vpasses = wg.vpasses;
    {   // the kernel reads the level's pointers and sizes from lev[0]
        FwdLevel &L = a.lev[0];
        L.f2 = a.f2; L.wv = a.wv; L.wu = a.wu; L.out_u = a.out_u; L.out_v = a.out_v; L.am_u = a.am_u; L.am_v = a.am_v;
        L.st_wv = a.st_wv; L.st_wu = a.st_wu; L.z_ou = a.z_ou; L.st_ou = a.st_ou; L.dot_ou = a.dot_ou;
        L.z_ov = a.z_ov; L.st_ov = a.st_ov; L.dot_ov = a.dot_ov;
        L.H2 = a.H2; L.W2 = a.W2; L.nvc = a.nvc; L.stage = a.stage;
    }
    dim3 grid(B * a.tiles_per_batch);
    const dim3 block(64 * nW);
    a.sk_total = 0;
    if (may_deal && f.on && f.bytes <= a.ws_bytes) {
        a.sk_total = (int)f.T;
        a.sk_steps = f.S;
        a.sk_count = static_cast<int *>(a.ws);
        a.sk_state = reinterpret_cast<float *>(static_cast<char *>(a.ws) + f.count_bytes);
        a.sk_slot = (int)f.slot_floats;
        grid = dim3(f.G);
        // (short shares only: with long ones the balance gains under 1 % and the L2 caches miss more, measured at
        // B=1, 55x128, K=4: 133 -> 195 MiB fetched per launch)
        a.pair_shares = f.G == 2 * kCUs && f.T < 16 * (long)f.G;
        const int n = B * a.tiles_per_batch;
        hipLaunchKernelGGL(zero_ints_kernel, dim3((n + 255) / 256), dim3(256), 0, s, a.sk_count, n);
    }
    const size_t f2_batch_bytes = (size_t)a.H2 * a.W2 * a.C * sizeof(float);
    const int cmode = (a.C % 32 == 0 && f2_batch_bytes <= (1u << 30)) ? (a.C == 256 ? 3 : 2) : (a.C % 4 == 0 ? 1 : 0);
#define SEPCORR_FWD(CV, RGV)                                                      \
    do {                                                                         \
        auto k = a.sk_total ? fwd_kernel<MODE, KC, UR, CV, RGV, false, true> : fwd_kernel<MODE, KC, UR, CV, RGV>; \
        if (int rc = set_lds(k, lds)) return rc;                                 \
        ProfScope ps(is_weighted(MODE) ? "fwd_weighted" : "fwd_maxavg", s);  \
        hipLaunchKernelGGL(k, grid, block, lds, s, a);                           \
    } while (0)
    // Always built for two waves per SIMD (256 registers): the accumulators then stay in ordinary
    // VGPRs, where the epilogue reads them without accumulator-register copies.
    if (wg.vpasses == 1 && cmode == 3 && a.f2_planes) {   // bf16-plane variant: the caller has split fmap2
        // LDS with the larger f1 tile (three bf16 planes); out_u staging only if two workgroups still fit a CU
        constexpr int NCHO = (is_weighted(MODE)) ? KC : 2;
        lds = ((size_t)TP * BF_LS + 2 * UR * NPART * nW * 32) * sizeof(float);
        const size_t extra = (size_t)TP * (NCHO + (MODE == MODE_ARGMAX ? 1 : 0)) * a.H2 * sizeof(float);
        a.stage = lds + extra <= 80 * 1024;
        if (a.stage) lds += extra;
        const size_t merge = wg.nug > 1 ? (size_t)wg.nvc * NPART * 16 * 64 * sizeof(float) : 0;
        if (lds < merge) lds = merge;
        ProfScope ps(is_weighted(MODE) ? "fwd_weighted_bf16x3" : "fwd_maxavg_bf16x3", s);
        if (wg.nug > 1) {
            auto k = fwd_kernel<MODE, KC, UR, 3, 1, true>;
            if (int rc = set_lds(k, lds)) return rc;
            hipLaunchKernelGGL(k, grid, block, lds, s, a);
        } else {
            auto k = fwd_kernel<MODE, KC, UR, 3, 0, true>;
            if (int rc = set_lds(k, lds)) return rc;
            hipLaunchKernelGGL(k, grid, block, lds, s, a);
        }
        return check_launch("forward kernel (bf16 planes)");
    }
    if (wg.vpasses > 1) {
        if (cmode >= 2) SEPCORR_FWD(2, 2); else if (cmode == 1) SEPCORR_FWD(1, 2); else SEPCORR_FWD(0, 2);
    } else if (wg.nug > 1) {
        if (cmode == 3) SEPCORR_FWD(3, 1); else if (cmode == 2) SEPCORR_FWD(2, 1);
        else if (cmode == 1) SEPCORR_FWD(1, 1); else SEPCORR_FWD(0, 1);
    } else {
        if (cmode == 3) SEPCORR_FWD(3, 0); else if (cmode == 2) SEPCORR_FWD(2, 0);
        else if (cmode == 1) SEPCORR_FWD(1, 0); else SEPCORR_FWD(0, 0);
    }
#undef SEPCORR_FWD
    return check_launch("forward kernel");
}
// Several pyramid levels in one launch.  a.lev[0..nlev) carry pointers and sizes (H2, W2); everything else as for
// launch_fwd.  Returns SEPCORR_EINVAL without launching when the shapes do not fit this path (the caller then runs
// the levels one by one): rows of at most 128 columns in 1, 2 or 4 chunks, C a multiple of 32, scratch given.
template <int MODE, int KC, int UR>
int launch_fwd_levels(FwdArgs a, int B, hipStream_t s) {
    constexpr int NPART = is_weighted(MODE) ? KC : 3;
    constexpr int NCHO = is_weighted(MODE) ? KC : 2;
    constexpr int nW = 4;
    if (a.nlev < 2 || a.nlev > 4 || a.ws == nullptr || a.C % 32 != 0) return SEPCORR_EINVAL;
    int steps = 0, h2max = 0, w2max = 0;
    for (int l = 0; l < a.nlev; ++l) {
        FwdLevel &L = a.lev[l];
        L.nvc = (L.W2 + 31) / 32;
        if (L.nvc != 1 && L.nvc != 2 && L.nvc != 4) return SEPCORR_EINVAL;
        if ((size_t)L.H2 * L.W2 * a.C * sizeof(float) > (1u << 30)) return SEPCORR_EINVAL;
        L.steps = (L.H2 + UR * (nW / L.nvc) - 1) / (UR * (nW / L.nvc));
        L.step0 = steps;
        steps += L.steps;
        if (L.H2 > h2max) h2max = L.H2;
        if (L.W2 > w2max) w2max = L.W2;
    }
    a.tile_steps = steps;
    a.H2max = h2max;
    a.vpasses = 1;
    size_t lds = ((size_t)TP * (a.CP + 4) + 2 * UR * NPART * nW * 32) * sizeof(float);
    const size_t extra = (size_t)TP * (NCHO + (MODE == MODE_ARGMAX ? 1 : 0)) * h2max * sizeof(float);
    a.stage = lds + extra <= 80 * 1024;
    if (a.stage) lds += extra;
    for (int l = 0; l < a.nlev; ++l) a.lev[l].stage = a.stage;
    const size_t merge = (size_t)2 * NPART * 16 * 64 * sizeof(float);   // row groups merge through LDS from offset 0
    if (lds < merge) lds = merge;
    if (MODE == MODE_SOFT) lds += (size_t)TP * KC * 3 * sizeof(float);
    const int tiles = B * a.tiles_per_batch;
    const long T = (long)tiles * steps;
    const long places = (long)kCUs * (lds <= 80 * 1024 ? 2 : 1);
    const int G = (int)(T < places ? T : places);
    const size_t count_bytes = ((size_t)tiles * a.nlev * sizeof(int) + 255) & ~(size_t)255;
    const size_t slot_floats = (size_t)NPART * 1024 * ((w2max + 31) / 32);
    if (T >= (1L << 30) || count_bytes + 2 * (size_t)G * slot_floats * sizeof(float) > a.ws_bytes) return SEPCORR_EINVAL;
    a.sk_total = (int)T;
    a.sk_steps = steps;
    a.sk_count = static_cast<int *>(a.ws);
    a.sk_state = reinterpret_cast<float *>(static_cast<char *>(a.ws) + count_bytes);
    a.sk_slot = (int)slot_floats;
    a.pair_shares = G == 2 * kCUs && T < 16 * (long)G;
    const int n = tiles * a.nlev;
    hipLaunchKernelGGL(zero_ints_kernel, dim3((n + 255) / 256), dim3(256), 0, s, a.sk_count, n);
    const dim3 grid(G), block(64 * nW);
    ProfScope ps(is_weighted(MODE) ? "fwd_weighted_levels" : "fwd_maxavg_levels", s);
    if (a.C == 256) {
        auto k = fwd_kernel<MODE, KC, UR, 3, 1, false, true>;
        if (int rc = set_lds(k, lds)) return rc;
        hipLaunchKernelGGL(k, grid, block, lds, s, a);
    } else {
        auto k = fwd_kernel<MODE, KC, UR, 2, 1, false, true>;
        if (int rc = set_lds(k, lds)) return rc;
        hipLaunchKernelGGL(k, grid, block, lds, s, a);
    }
    return check_launch("forward kernel (several levels)");
}
// Upper bound of the scratch launch_fwd_levels asks for.
inline size_t fwd_levels_bytes(int tiles, int nlev, int w2max, int K) {
    const int nq = K > 3 ? (K < KCH ? K : KCH) : 3;
    return (((size_t)tiles * nlev * sizeof(int) + 255) & ~(size_t)255) + 2 * (size_t)(2 * kCUs) * nq * 1024 * ((w2max + 31) / 32) * sizeof(float);
}
// instantiated in one part each; everywhere else only declared
#define SEPCORR_FWD_DECL(MODE, KC, UR)                                              \
    extern template int launch_fwd<MODE, KC, UR>(FwdArgs, int, hipStream_t);       \
    extern template int launch_fwd_levels<MODE, KC, UR>(FwdArgs, int, hipStream_t)
#define SEPCORR_FWD_INST(MODE, KC, UR)                                              \
    template int launch_fwd<MODE, KC, UR>(FwdArgs, int, hipStream_t);              \
    template int launch_fwd_levels<MODE, KC, UR>(FwdArgs, int, hipStream_t)
SEPCORR_FWD_DECL(MODE_MAXAVG, 1, 2);
SEPCORR_FWD_DECL(MODE_ARGMAX, 1, 2);
SEPCORR_FWD_DECL(MODE_WEIGHTED, 1, 2);
SEPCORR_FWD_DECL(MODE_WEIGHTED, 2, 2);
SEPCORR_FWD_DECL(MODE_WEIGHTED, 3, 1);
SEPCORR_FWD_DECL(MODE_WEIGHTED, 4, 1);
SEPCORR_FWD_DECL(MODE_SOFT, 1, 2);
SEPCORR_FWD_DECL(MODE_SOFT, 2, 2);
SEPCORR_FWD_DECL(MODE_SOFT, 3, 1);
SEPCORR_FWD_DECL(MODE_SOFT, 4, 1);
#if SEPCORR_IN_PART(12)
SEPCORR_FWD_INST(MODE_SOFT, 1, 2);
#endif
#if SEPCORR_IN_PART(13)
SEPCORR_FWD_INST(MODE_SOFT, 2, 2);
#endif
#if SEPCORR_IN_PART(14)
SEPCORR_FWD_INST(MODE_SOFT, 3, 1);
#endif
#if SEPCORR_IN_PART(15)
SEPCORR_FWD_INST(MODE_SOFT, 4, 1);
#endif
#if SEPCORR_IN_PART(1)
SEPCORR_FWD_INST(MODE_MAXAVG, 1, 2);
#endif
#if SEPCORR_IN_PART(2)
SEPCORR_FWD_INST(MODE_ARGMAX, 1, 2);
#endif
#if SEPCORR_IN_PART(3)
SEPCORR_FWD_INST(MODE_WEIGHTED, 1, 2);
#endif
#if SEPCORR_IN_PART(4)
SEPCORR_FWD_INST(MODE_WEIGHTED, 2, 2);
#endif
#if SEPCORR_IN_PART(5)
SEPCORR_FWD_INST(MODE_WEIGHTED, 3, 1);
#endif
#if SEPCORR_IN_PART(6)
SEPCORR_FWD_INST(MODE_WEIGHTED, 4, 1);
#endif
}  // namespace sepcorr_impl
namespace {

template <int MODE>
int launch_fwd_weighted_k(const FwdArgs &a, int kc, int B, hipStream_t s) {
    switch (kc) {
        case 1: return launch_fwd<MODE, 1, 2>(a, B, s);
        case 2: return launch_fwd<MODE, 2, 2>(a, B, s);
        case 3: return launch_fwd<MODE, 3, 1>(a, B, s);
        default: return launch_fwd<MODE, 4, 1>(a, B, s);
    }
}

// SEPCORR_NO_XCD_ORDER=1 keeps the hardware order of workgroups (for measurements).
int xcd_order_enabled() {
    static const int on = getenv("SEPCORR_NO_XCD_ORDER") == nullptr;
    return on;
}

// Contraction of the forward sweeps: fp32 MFMA, or three bf16 planes where the shape allows (C == 256, rows of at
// most 256 columns).  sepcorr_set_contraction() selects;
// SEPCORR_BF16X3=1 in the environment makes the planes the initial choice.  fmap2 is split once per call into
// stream-ordered memory that is released, in stream order, when the call returns.
}  // namespace
#if SEPCORR_IN_PART(0)
namespace sepcorr_impl {
std::atomic<int> g_maxavg_backward{SEPCORR_MAXAVG_AUTO};
std::atomic<int> g_contraction{[] {
    const char *e = getenv("SEPCORR_BF16X3");
    return e && e[0] == '1' ? SEPCORR_CONTRACT_BF16X3 : SEPCORR_CONTRACT_FP32;
}()};
}  // namespace sepcorr_impl
#endif
namespace {
struct Bf16Planes {
    void *ptr = nullptr;
    int H2p = 0;
    hipStream_t s = nullptr;
    ~Bf16Planes() { if (ptr) (void)hipFreeAsync(ptr, s); }
    int make(const Dims &d, const float *f2, hipStream_t stream) {
        const bool on = g_contraction.load(std::memory_order_relaxed) == SEPCORR_CONTRACT_BF16X3;
        const WaveGrid wg = wave_grid(d.B, (d.H1 * d.W1 + TP - 1) / TP, d.W2, d.H2);
        const int nvcp = (d.W2 + 31) / 32;
        H2p = (d.H2 + 2 * wg.nug - 1) / (2 * wg.nug) * (2 * wg.nug);   // whole steps of two rows for every row group
        const size_t batch_bytes = (size_t)H2p * nvcp * BF_CHUNK;
        if (!on || d.C != 256 || wg.vpasses > 1 || batch_bytes > (1u << 30)) return SEPCORR_OK;
        const size_t nchunks = (size_t)d.B * H2p * nvcp;
        s = stream;
        const hipError_t e = hipMallocAsync(&ptr, nchunks * BF_CHUNK, s);
        if (e != hipSuccess) { ptr = nullptr; return fail(SEPCORR_ELAUNCH, "sepcorr: bf16 planes: %s", hipGetErrorString(e)); }
        ProfScope ps("split_planes", s);
        const long nunits = (long)nchunks * 16 * 64;
        hipLaunchKernelGGL(split_planes_kernel, dim3((unsigned)((nunits + 255) / 256)), dim3(256), 0, s, f2,
                           static_cast<char *>(ptr), d.H2, d.W2, H2p, nvcp, nunits);
        return check_launch("split_planes");
    }
};

FwdArgs fwd_args(const Dims &d) {
    FwdArgs a;
    memset(&a, 0, sizeof(a));
    a.N1 = d.H1 * d.W1;
    a.H2 = d.H2;
    a.H2max = d.H2;
    a.W2 = d.W2;
    a.C = d.C;
    a.CP = (d.C + 7) & ~7;
    a.tiles_per_batch = (a.N1 + TP - 1) / TP;
    a.xcd_order = xcd_order_enabled();
    return a;
}

// sum_v S wv[k,v] -> out_u[k,u];  sum_u S wu[k,u] -> out_v[k,v]  for K channels, KCH per launch
// soft (optional): the softmax fields of FwdArgs (logits / dlog and what they refer to)
int weighted_forward(const Dims &d, const float *f1, const float *f2, const float *wv, const float *wu, float *out_u,
                     float *out_v, int K, void *ws, size_t ws_bytes, hipStream_t s, const FwdArgs *soft = nullptr) {
    FwdArgs a = fwd_args(d);
    a.f1 = f1; a.f2 = f2; a.wv = wv; a.wu = wu; a.out_u = out_u; a.out_v = out_v;
    a.KT = K;
    a.ws = ws; a.ws_bytes = ws_bytes;
    if (soft) {
        a.logits = soft->logits; a.dlog = soft->dlog; a.st_wv = soft->st_wv; a.st_wu = soft->st_wu;
        a.z_ou = soft->z_ou; a.st_ou = soft->st_ou; a.dot_ou = soft->dot_ou;
        a.z_ov = soft->z_ov; a.st_ov = soft->st_ov; a.dot_ov = soft->dot_ov;
    }
    Bf16Planes planes;
    if (!soft)   // (the bf16-plane variant of the sweep has no softmax inside)
    if (int rc = planes.make(d, f2, s)) return rc;
    a.f2_planes = static_cast<const char *>(planes.ptr);
    a.H2p = planes.H2p;
    for (int k0 = 0; k0 < K; k0 += KCH) {
        a.k0 = k0;
        const int kc = K - k0 < KCH ? K - k0 : KCH;
        if (int rc = soft ? launch_fwd_weighted_k<MODE_SOFT>(a, kc, d.B, s) : launch_fwd_weighted_k<MODE_WEIGHTED>(a, kc, d.B, s)) return rc;
    }
    return SEPCORR_OK;
}

// fmap2 rows (= waves) per workgroup of the tiled d_f2 kernel: 8 (two waves per SIMD sharing one LDS tile)
// unless that pads the row count more than 4 does.
// The combined mode keeps more weight tiles in LDS and has room for 4 rows only.
int df2_rows_per_wg(const Dims &d, bool both) {
    if (both) return 4;
    return (d.H2 + 7) / 8 * 8 <= (d.H2 + 3) / 4 * 4 ? 8 : 4;
}

struct Df2Plan {
    bool tiled;
    int nsplit;
    int rows;
    int tiles_per_split;   // pixel tiles of a split (the last split takes what is left)
    bool uneven;           // the last split is a short one, dealt out last (BwdArgs::uneven)
    bool noavgv;           // combined mode: the average term of g_v comes from a table (df2_tiled_kernel<..., NOAVGV>)
};
Df2Plan df2_plan_rows(const Dims &d, int rows);

// How d_f2 is computed for these sizes.  The p range is split over workgroups so that the grid fills
// the 256 CUs evenly; each split writes a partial d_f2 to scratch, summed in split order afterwards.
Df2Plan df2_plan(const Dims &d, bool both) {
    // (the table costs 25 to 35 us and the larger workgroups gain a fifth of the kernel's time: worth it from about
    // 2^25 (pixel, position) pairs on; measured at B=2, 55x128 pixels: 0.61 -> 0.52 ms with fmap2 55x128, but
    // 0.055 -> 0.087 ms with fmap2 13x32)
    const bool large = (size_t)d.B * d.H1 * d.W1 * d.H2 * d.W2 >= ((size_t)1 << 25);
    if (both && large && sepcorr_avg_table_v_eligible(d.B, d.H1, d.W1, d.H2, d.W2, d.C) && df2_rows_per_wg(d, false) == 8) {
        // eight rows per workgroup when the table's split sums fit into the region of d_f2's own (unused until the
        // kernel stores) and there are at least two splits
        Df2Plan p8 = df2_plan_rows(d, 8);
        const size_t part = (size_t)p8.nsplit * d.B * d.H2 * d.W2 * d.C * sizeof(float);
        if (p8.tiled && p8.nsplit >= 2 && sepcorr_avg_table_v_part_bytes(d.B, d.H1, d.W1, d.W2, d.C) <= part) {
            p8.noavgv = true;
            return p8;
        }
    }
    return df2_plan_rows(d, df2_rows_per_wg(d, both));
}

Df2Plan df2_plan_rows(const Dims &d, int rows_per_wg) {
    Df2Plan pl;
    pl.noavgv = false;
    pl.rows = rows_per_wg;
    const size_t big = (size_t)1 << 30;
    const size_t n1 = (size_t)d.H1 * d.W1;
    pl.tiled = d.C % 4 == 0 && d.W2 % 4 == 0 && n1 * d.C * 4 <= big && n1 * MAX_K * d.W2 * 4 <= big &&
               n1 * MAX_K * d.H2 * 4 <= big;
    const int tiles = (int)((n1 + TP - 1) / TP);
    const int nvc = (d.W2 + 31) / 32;
    const int cblocks = (d.C + 255) / 256;
    pl.uneven = false;
    if (pl.tiled) {
        // Estimated duration in pixel tiles of the sweep; a workgroup's start-up, the partial result it leaves and
        // its later addition cost about as much as two tiles.  One workgroup per compute unit at a time.
        const int rows = pl.rows;
        const long base = (long)d.B * ((d.H2 + rows - 1) / rows) * nvc * (d.C <= 128 ? 1 : cblocks);
        struct Cand { int ns, tps; bool uneven; double t; };
        Cand cand[128];
        int nc = 0;
        // (coarse pyramid levels have few blocks of output rows: they fill the chip only with many short splits)
        for (int ns = 1; ns <= 64 && ns <= tiles; ++ns) {
            const int per = (tiles + ns - 1) / ns, nsa = (tiles + per - 1) / per;   // nsa: splits that get tiles
            const long wgs = base * nsa;
            cand[nc++] = {nsa, per, false, (double)((wgs + 255) / 256) * (per + 2.0)};
            // ns - 1 long splits that fill part of the chip in one round, and a short one whose workgroups follow
            // one another on the compute units left over: r rounds of them take as long as one long split.
            // Workgroups are handed out in the order of their ids to 32 groups of 8 compute units in turn, and a
            // workgroup waits for a unit of its own group: every group must keep a unit free of long workgroups
            // (measured at B=4, 48x64: with 240 long ones the short ones ran behind them, not beside them).
            const long nlong = base * (ns - 1);
            if (ns >= 2 && cblocks == 1 && nlong <= 224) {
                const long free_per_group = 8 - (nlong + 31) / 32;
                const long r = ((base + 31) / 32 + free_per_group - 1) / free_per_group;
                // (a workgroup that follows another on a compute unit starts while that one drains: measured, a
                // short split costs one tile of start-up, not two: 49 + 24 tiles beat 50 + 20 at B=2, 55x128)
                const long a_len = (r * (tiles + 1) - 1 + (1 + r * (ns - 1)) - 1) / (1 + r * (ns - 1));
                const long b_len = tiles - (long)(ns - 1) * a_len;
                if (a_len >= 1 && b_len >= 1 && b_len <= a_len) {
                    const double t = std::max((double)a_len + 2.0, (double)r * (b_len + 1.0) + 1.0);
                    cand[nc++] = {ns, (int)a_len, true, t};
                }
            }
        }
        double best = cand[0].t;
        for (int i = 1; i < nc; ++i) best = std::min(best, cand[i].t);
        int pick = -1;   // the fewest splits (least scratch) among those within 1.5 % of the best
        for (int i = 0; i < nc; ++i)
            if (cand[i].t <= best * 1.015 && (pick < 0 || cand[i].ns < cand[pick].ns || (cand[i].ns == cand[pick].ns && cand[i].t < cand[pick].t)))
                pick = i;
        pl.nsplit = cand[pick].ns;
        pl.tiles_per_split = cand[pick].tps;
        pl.uneven = cand[pick].uneven;
    } else {
        const long tasks = (long)d.B * d.H2 * nvc;
        long n = (2048 + tasks - 1) / tasks;  // aim at two waves per SIMD on 256 CUs
        if (n > 8) n = 8;
        if (n > tiles) n = tiles;
        if (n < 1) n = 1;
        pl.nsplit = (int)n;
    }
    if (!pl.tiled) pl.tiles_per_split = (tiles + pl.nsplit - 1) / pl.nsplit;
    return pl;
}

// Workspace of a backward call: the split partial sums of d_f2, then the transposed (p,u) weights of the fast d_f1
// kernel (C == 256; sized for the most fields one launch can have).
size_t df2_part_bytes(const Dims &d) {
    const int n0 = df2_plan(d, false).nsplit, n1 = df2_plan(d, true).nsplit;
    const int ns = n0 > n1 ? n0 : n1;   // one size serves every backward entry point
    const size_t bytes = ns > 1 ? (size_t)ns * d.B * d.H2 * d.W2 * d.C * sizeof(float) : 0;
    return (bytes + 255) & ~(size_t)255;
}
size_t df1_uwt_bytes(const Dims &d) {
    const size_t bytes = d.C == 256 ? (size_t)d.B * d.H2 * (2 * KCH + 3) * d.H1 * d.W1 * sizeof(float) : 0;
    return (bytes + 255) & ~(size_t)255;
}

// Launch shape of d_f1 and how it is dealt out (as fwd_split): whole tiles on one workgroup per CU, or the steps of
// all tiles shared evenly, pieces of a tile leaving partial [32][channels] sums that the last one adds up.
struct Df1Shape {
    WaveGrid wg;
    int nW, ncb, cblocks;
    bool split;
    int G, S;
    long T;
    size_t count_bytes, bytes;
};
Df1Shape df1_shape(const Dims &d) {
    Df1Shape f;
    const int tpb = (d.H1 * d.W1 + TP - 1) / TP, tiles = d.B * tpb;
    f.wg = wave_grid(d.B, tpb, d.W2, d.H2);
    if (f.wg.nvc * f.wg.nug > 4) f.wg.nug = 4 / f.wg.nvc > 0 ? 4 / f.wg.nvc : 1;   // d_f1 runs one wave per SIMD
    f.nW = f.wg.nvc * f.wg.nug;
    // more than 4 waves share the register file two to a SIMD: halve the channel block
    f.ncb = (d.C <= 128 || f.nW > 4) ? 1 : 2;
    f.cblocks = (d.C + 128 * f.ncb - 1) / (128 * f.ncb);
    f.S = (d.H2 + f.wg.nug - 1) / f.wg.nug;
    f.T = (long)tiles * f.S;
    const long places = kCUs / f.cblocks > 0 ? kCUs / f.cblocks : 1;
    const double plain = (double)tiles / (double)(((tiles + places - 1) / places) * places);
    f.G = (int)(f.T < places ? f.T : places);
    const double split = (double)f.T / (double)(((f.T + f.G - 1) / f.G) * f.G);
    f.split = d.C % 4 == 0 && f.S >= 2 && f.T < (1L << 30) && split > plain + 0.04;
    f.count_bytes = ((size_t)tiles * f.cblocks * sizeof(int) + 255) & ~(size_t)255;
    f.bytes = f.split ? f.count_bytes + 2 * (size_t)f.G * f.cblocks * TP * 128 * f.ncb * sizeof(float) : 0;
    return f;
}

// Layout of a backward call's workspace.  Regions: split partial sums of d_f2; transposed (p,u) weights of d_f1 and,
// behind them, the pieces of a split d_f1; scratch of the weight-gradient sweep (a forward-type sweep).  When any
// kernel is dealt out in pieces the call keeps to one stream (such kernels want the whole chip), its kernels run one
// after the other, and the regions of different kernels share the same memory.
struct BwdWs {
    bool aliased;
    size_t off_uwt, off_df1sk, fwd_bytes, own_total, total;   // own_total: without the weight-gradient sweep
    size_t off_vtable;                                        // (B,W2,C) table of the combined d_f2 (Df2Plan::noavgv)
};
BwdWs bwd_ws(const Dims &d) {
    BwdWs w;
    const size_t part = df2_part_bytes(d), uwt = df1_uwt_bytes(d), sk = df1_shape(d).bytes;
    w.fwd_bytes = fwd_split_bytes(d.B, d.H1, d.W1, d.H2, d.W2, MAX_K);
    w.aliased = sk > 0 || w.fwd_bytes > 0;
    if (w.aliased) {
        w.off_uwt = 0;
        w.off_df1sk = uwt;
        w.own_total = part > uwt + sk ? part : uwt + sk;
        w.total = w.own_total > w.fwd_bytes ? w.own_total : w.fwd_bytes;
    } else {
        w.off_uwt = part;
        w.off_df1sk = part + uwt;
        w.own_total = w.total = part + uwt;
    }
    if (sepcorr_gather_backward_eligible(d.B, d.H1, d.W1, d.H2, d.W2, d.C)) {   // the max/avg backward may take this path
        const size_t g = sepcorr_gather_backward_bytes(d.B, d.H1, d.W1, d.H2, d.W2, d.C);
        if (g > w.total) w.total = g;
    }
    w.off_vtable = w.total;
    if (df2_plan(d, true).noavgv) w.total += ((size_t)d.B * d.W2 * d.C * sizeof(float) + 255) & ~(size_t)255;
    return w;
}

}  // namespace
namespace sepcorr_impl {
template <int GMODE, int KC>
int launch_bwd(BwdArgs a, const Dims &d, void *ws, hipStream_t s1, hipStream_t s) {
    // s1: stream of the d_f1 kernel; s: stream of the d_f2 kernel and its split reduction
    const size_t big = (size_t)1 << 30;
    const bool cvec = (d.C % 4) == 0 && (size_t)d.H2 * d.W2 * d.C * 4 <= big && (size_t)d.H1 * d.W1 * d.C * 4 <= big;
    a.tiles_per_batch = (a.N1 + TP - 1) / TP;
    const int nvc_all = (d.W2 + 31) / 32;
    {
        const Df1Shape shp = df1_shape(d);
        const WaveGrid wg = shp.wg;
        a.nvc = wg.nvc;
        a.vpasses = wg.vpasses;
        const int nW = shp.nW, ncb = shp.ncb, cblocks = shp.cblocks;
        dim3 grid(d.B * a.tiles_per_batch, cblocks);
        const dim3 block(64 * nW);
        const size_t lds = (size_t)nW * TP * (128 * ncb + 4) * sizeof(float);   // one [32][channels] region per wave
        a.sk_total = 0;
        // Rows per block of d_f1's register accumulation.  Measured at B=2, 55x128, C=256 (error against fp64 relative
        // to the fp32 CPU path's / kernel time): whole tiles 2.45 / 0.422 ms, 12 rows 1.28, 8 rows 1.08 / 0.434,
        // 6 rows 0.97, 4 rows 0.83 / 0.444, 2 rows 0.66 / 0.468, 1 row 0.517 ms; the combined mode 0.546 ms for whole
        // tiles, 0.553 for 12 rows, 0.575 for 4.
        a.flush_rows = 4;
#define SEPCORR_DF1_K(...)                                                                         \
    do {                                                                                           \
        auto k = df1_kernel<__VA_ARGS__>;                                                          \
        if (int rc = set_lds(k, lds)) return rc;                                                   \
        ProfScope ps(GMODE == GMODE_COMP ? "df1_comp" : GMODE == GMODE_BOTH ? "df1_both" : "df1_maxavg", s1); \
        hipLaunchKernelGGL(k, grid, block, lds, s1, a);                                            \
    } while (0)
#define SEPCORR_DF1(NCB, CV, MT) SEPCORR_DF1_K(GMODE, KC, NCB, CV, MT)
#define SEPCORR_DF1_SPLIT(NCB, MT)                                                                 \
    do {                                                                                           \
        if (a.sk_total) SEPCORR_DF1_K(GMODE, KC, NCB, true, MT, false, true);                      \
        else SEPCORR_DF1_K(GMODE, KC, NCB, true, MT);                                              \
    } while (0)
        const bool planes = !t_no_alloc && g_contraction.load(std::memory_order_relaxed) == SEPCORR_CONTRACT_BF16X3 && d.C == 256 &&
                            wg.vpasses == 1 && cvec && (size_t)d.H1 * d.W1 * MAX_K * d.H2 * 4 <= big &&
                            (size_t)d.H2 * nvc_all * BF_CHUNK <= big && (size_t)d.H2 * (2 * MAX_K + 3) * d.H1 * d.W1 * 4 <= big;
        if (planes) {
            // bf16 planes: transposed fmap2 planes and the per-chunk partial sums live in stream-ordered memory
            const int nvc = nvc_all, ptiles = (a.N1 + 127) / 128;
            const size_t planes_bytes = (size_t)d.B * d.H2 * nvc * BF_CHUNK;
            const size_t n = (size_t)d.B * a.N1 * 256;
            const size_t part_bytes = nvc > 1 ? (size_t)nvc * n * sizeof(float) : 0;
            constexpr int NF = (g_has_comp(GMODE) ? 2 * KC : 0) + (g_has_maxavg(GMODE) ? 3 : 0);
            const size_t uwt_bytes = (size_t)d.B * d.H2 * NF * a.N1 * sizeof(float);
            void *buf = nullptr;
            hipError_t e = hipMallocAsync(&buf, planes_bytes + part_bytes + uwt_bytes, s1);
            if (e != hipSuccess) return fail(SEPCORR_ELAUNCH, "sepcorr: bf16 planes: %s", hipGetErrorString(e));
            char *pl = static_cast<char *>(buf);
            float *part = nvc > 1 ? reinterpret_cast<float *>(pl + planes_bytes) : a.d1;
            float *uwt = reinterpret_cast<float *>(pl + planes_bytes + part_bytes);
            {
                ProfScope ps("transpose_uw", s1);
                hipLaunchKernelGGL(transpose_uw_kernel<GMODE>, dim3(d.B * ((a.N1 + 63) / 64), NF), dim3(256), 0, s1, a, KC, uwt);
            }
            {
                ProfScope ps("split_planes_t", s1);
                const long nunits = (long)d.B * d.H2 * nvc * 16 * 64;
                hipLaunchKernelGGL(split_planes_t_kernel, dim3((unsigned)((nunits + 255) / 256)), dim3(256), 0, s1, a.f2, pl,
                                   d.W2, nvc, nunits);
            }
            const size_t ldsb = 4 * 32 * DF1BF_RS * sizeof(float);   // output transpose; covers the two 48 KB row blocks
            auto k4 = df1_bf_kernel<GMODE, KC, 4>;
            int rc = set_lds(k4, ldsb);
            if (rc == SEPCORR_OK) {
                {
                    ProfScope ps(GMODE == GMODE_COMP ? "df1_comp_bf16x3" : GMODE == GMODE_BOTH ? "df1_both_bf16x3" : "df1_maxavg_bf16x3", s1);
                    hipLaunchKernelGGL(k4, dim3(d.B * ptiles * nvc), dim3(256), ldsb, s1, a, pl, uwt, part, nvc, ptiles);
                }
                if (nvc > 1) {
                    const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
                    ProfScope ps("df1_reduce_chunks", s1);
                    hipLaunchKernelGGL(reduce_splits_kernel, dim3(blocks), dim3(256), 0, s1, part, a.d1, n, nvc, a.accumulate | a.add_d1);
                }
                rc = check_launch("d_f1 kernel (bf16 planes)");
            }
            e = hipFreeAsync(buf, s1);
            if (rc) return rc;
            if (e != hipSuccess) return fail(SEPCORR_ELAUNCH, "sepcorr: bf16 planes: %s", hipGetErrorString(e));
        }
        else {
        if (shp.split && cvec) {   // pieces of tiles: scratch behind the d_f2 partial sums and the transposed weights
            char *base = static_cast<char *>(ws) + bwd_ws(d).off_df1sk;
            a.sk_total = (int)shp.T;
            a.sk_steps = shp.S;
            a.sk_count = reinterpret_cast<int *>(base);
            a.sk_state = reinterpret_cast<float *>(base + shp.count_bytes);
            grid = dim3(shp.G, cblocks);
            const int n = d.B * a.tiles_per_batch * cblocks;
            hipLaunchKernelGGL(zero_ints_kernel, dim3((n + 255) / 256), dim3(256), 0, s1, a.sk_count, n);
        }
        if (nW > 4) { if (cvec) SEPCORR_DF1_SPLIT(1, 512); else SEPCORR_DF1(1, false, 512); }
        else if (ncb == 1) { if (cvec) SEPCORR_DF1_SPLIT(1, 256); else SEPCORR_DF1(1, false, 256); }
        // (the fast variant addresses the (p,u)-indexed tensors of one batch image with 32-bit byte offsets)
        else if (cvec && d.C == 256 && d.W2 % 4 == 0 && (size_t)d.H2 * (2 * KCH + 3) * d.H1 * d.W1 * 4 <= big) {
            constexpr int NF = (g_has_comp(GMODE) ? 2 * KC : 0) + (g_has_maxavg(GMODE) ? 3 : 0);
            float *uwt = reinterpret_cast<float *>(static_cast<char *>(ws) + bwd_ws(d).off_uwt);
            {
                ProfScope ps("transpose_uw", s1);
                hipLaunchKernelGGL(transpose_uw_kernel<GMODE>, dim3(d.B * ((a.N1 + 63) / 64), NF), dim3(256), 0, s1, a, KC, uwt);
            }
            a.uwt = uwt;
            if (a.sk_total) SEPCORR_DF1_K(GMODE, KC, 2, true, 256, true, true);
            else SEPCORR_DF1_K(GMODE, KC, 2, true, 256, true);
        }
        else { if (cvec) SEPCORR_DF1_SPLIT(2, 256); else SEPCORR_DF1(2, false, 256); }
        }
#undef SEPCORR_DF1
#undef SEPCORR_DF1_SPLIT
#undef SEPCORR_DF1_K
        if (int rc = check_launch("d_f1 kernel")) return rc;
    }
    {
        const int ncb = d.C <= 128 ? 1 : 2;
        const int cblocks = (d.C + 128 * ncb - 1) / (128 * ncb);
        const int tiles = a.tiles_per_batch;
        const Df2Plan plan = df2_plan(d, GMODE == GMODE_BOTH);
        a.nsplit = plan.nsplit;
        a.tiles_per_split = plan.tiles_per_split;
        a.uneven = 0;
        const int nvc = nvc_all;
        float *d2 = a.d2;
        if (a.nsplit > 1) a.d2 = static_cast<float *>(ws);
        if (plan.tiled) {
            constexpr int NV3 = (g_has_comp(GMODE) ? 2 * KC : 0) + (g_has_maxavg(GMODE) ? 3 : 0);
            constexpr int NUP = (NV3 + 3) & ~3;
            constexpr int UBUF = df2_tiled_ubuf(GMODE);
            const bool noavgv = GMODE == GMODE_BOTH && plan.noavgv;
            const int NV = noavgv ? NV3 - 1 : NV3;
            if (noavgv) {   // the table first; its split sums use the start of d_f2's partial sums, written later
                float *vt = reinterpret_cast<float *>(static_cast<char *>(ws) + bwd_ws(d).off_vtable);
                if (int rc = sepcorr_avg_table_v(a.f1, a.g_v, vt, static_cast<float *>(ws), d.B, d.H1, d.W1, d.H2, d.W2, d.C, s)) return rc;
                a.vtable = vt;
            }
            const int rows = plan.rows;
            const int nug = (d.H2 + rows - 1) / rows;
            const dim3 grid(d.B * a.nsplit * nug * nvc, cblocks), block(64 * rows);
            if (plan.uneven) {   // long units first, short ones last, XCD by XCD
                a.uneven = 1;
                a.q_units = d.B * nug * nvc;
                const int n = (int)grid.x, nlong = a.q_units * (a.nsplit - 1);
                a.xl[0] = a.xs[0] = 0;
                for (int x = 0; x < 8; ++x) {
                    const int cx = (n - x + 7) / 8;                                   // workgroup ids x, x + 8, ...
                    int lx = (int)((long)(x + 1) * nlong / 8 - (long)x * nlong / 8);
                    if (lx > cx) lx = cx;
                    a.xl[x + 1] = a.xl[x] + lx;
                    a.xs[x + 1] = a.xs[x] + (cx - lx);
                }
                if (a.xl[8] != nlong || a.xs[8] != a.q_units) a.uneven = 0, a.tiles_per_split = (tiles + a.nsplit - 1) / a.nsplit;
            }
            const size_t lds = ((size_t)2 * 32 * 128 * ncb + 2 * NV * 1024 + rows * UBUF * 32 * NUP) * sizeof(float);
#define SEPCORR_DF2T(NCB, NWV)                                                                     \
    do {                                                                                           \
        auto k = df2_tiled_kernel<GMODE, KC, NCB, NWV>;                                            \
        if (int rc = set_lds(k, lds)) return rc;                                                   \
        ProfScope ps(GMODE == GMODE_COMP ? "df2_comp" : GMODE == GMODE_BOTH ? "df2_both" : "df2_maxavg", s); \
        hipLaunchKernelGGL(k, grid, block, lds, s, a, nvc, nug);                                   \
    } while (0)
            if (noavgv) {
                if constexpr (GMODE == GMODE_BOTH) {
#define SEPCORR_DF2T8(NCB)                                                                          \
    do {                                                                                           \
        auto k = df2_tiled_kernel<GMODE, KC, NCB, 8, true>;                                        \
        if (int rc = set_lds(k, lds)) return rc;                                                   \
        ProfScope ps("df2_both", s);                                                               \
        hipLaunchKernelGGL(k, grid, block, lds, s, a, nvc, nug);                                   \
    } while (0)
                    if (ncb == 1) SEPCORR_DF2T8(1); else SEPCORR_DF2T8(2);
#undef SEPCORR_DF2T8
                }
            }
            else if (rows == 8) { if (ncb == 1) SEPCORR_DF2T(1, 8); else SEPCORR_DF2T(2, 8); }
            else           { if (ncb == 1) SEPCORR_DF2T(1, 4); else SEPCORR_DF2T(2, 4); }
#undef SEPCORR_DF2T
        } else {
        const int ntasks = d.B * a.nsplit * d.H2 * nvc;
        const dim3 grid((ntasks + 3) / 4, cblocks), block(256);
#define SEPCORR_DF2(NCB, CV)                                                                       \
    do {                                                                                           \
        ProfScope ps(GMODE == GMODE_COMP ? "df2_comp" : GMODE == GMODE_BOTH ? "df2_both" : "df2_maxavg", s); \
        hipLaunchKernelGGL((df2_kernel<GMODE, KC, NCB, CV>), grid, block, 0, s, a, ntasks, nvc);   \
    } while (0)
        if (ncb == 1) { if (cvec) SEPCORR_DF2(1, true); else SEPCORR_DF2(1, false); }
        else          { if (cvec) SEPCORR_DF2(2, true); else SEPCORR_DF2(2, false); }
#undef SEPCORR_DF2
        }
        if (int rc = check_launch("d_f2 kernel")) return rc;
        if (a.nsplit > 1) {
            const size_t n = (size_t)d.B * d.H2 * d.W2 * d.C;
            const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
            ProfScope ps("df2_reduce_splits", s);
            hipLaunchKernelGGL(reduce_splits_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const float *>(ws), d2, n,
                               a.nsplit, a.accumulate);
            if (int rc = check_launch("d_f2 split reduction")) return rc;
        }
    }
    return SEPCORR_OK;
}
#define SEPCORR_BWD_DECL(GMODE, KC) extern template int launch_bwd<GMODE, KC>(BwdArgs, const Dims &, void *, hipStream_t, hipStream_t)
#define SEPCORR_BWD_INST(GMODE, KC) template int launch_bwd<GMODE, KC>(BwdArgs, const Dims &, void *, hipStream_t, hipStream_t)
SEPCORR_BWD_DECL(GMODE_MAXAVG, 1);
SEPCORR_BWD_DECL(GMODE_COMP, 1);
SEPCORR_BWD_DECL(GMODE_COMP, 2);
SEPCORR_BWD_DECL(GMODE_COMP, 3);
SEPCORR_BWD_DECL(GMODE_COMP, 4);
SEPCORR_BWD_DECL(GMODE_BOTH, 2);
SEPCORR_BWD_DECL(GMODE_BOTH, 4);
#if SEPCORR_IN_PART(7)
SEPCORR_BWD_INST(GMODE_MAXAVG, 1);
SEPCORR_BWD_INST(GMODE_COMP, 1);
#endif
#if SEPCORR_IN_PART(8)
SEPCORR_BWD_INST(GMODE_COMP, 2);
SEPCORR_BWD_INST(GMODE_COMP, 3);
#endif
#if SEPCORR_IN_PART(9)
SEPCORR_BWD_INST(GMODE_COMP, 4);
#endif
#if SEPCORR_IN_PART(10)
SEPCORR_BWD_INST(GMODE_BOTH, 2);
#endif
#if SEPCORR_IN_PART(11)
SEPCORR_BWD_INST(GMODE_BOTH, 4);
#endif
}  // namespace sepcorr_impl
namespace {

// The kernels of one backward call are independent of each other (they only read the inputs), so they
// are issued on separate streams: the tail of one kernel, where part of the chip would idle, is filled
// by the next.  Fork: the side streams wait for everything queued on the caller's stream; join: the
// caller's stream waits for the side streams.  Works under stream capture (ordinary fork/join pattern).
// Per device: two side streams at default priority and three events, created on first use.
struct SideStreams {
    hipStream_t a = nullptr, b = nullptr;
    hipEvent_t fork = nullptr, ja = nullptr, jb = nullptr;
    bool ok = false;
};
std::mutex g_side_mu;
SideStreams g_side[64];

bool overlap_enabled() {
    static const bool on = [] {
        const char *e = getenv("SEPCORR_SINGLE_STREAM");
        return !(e && e[0] == '1');
    }();
    return on && !t_prof_on && !t_no_alloc;   // per-kernel timing wants the kernels one after the other
}

SideStreams *side_streams() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    SideStreams &ss = g_side[dev];
    if (!ss.ok) {
        if (hipStreamCreateWithFlags(&ss.a, hipStreamNonBlocking) != hipSuccess) return nullptr;
        if (hipStreamCreateWithFlags(&ss.b, hipStreamNonBlocking) != hipSuccess) return nullptr;
        if (hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) != hipSuccess) return nullptr;
        if (hipEventCreateWithFlags(&ss.ja, hipEventDisableTiming) != hipSuccess) return nullptr;
        if (hipEventCreateWithFlags(&ss.jb, hipEventDisableTiming) != hipSuccess) return nullptr;
        ss.ok = true;
    }
    return &ss;
}

// RAII fork/join around the launches of one backward call.  With overlap off, both side streams are
// the caller's stream and nothing is recorded.
struct ForkJoin {
    std::unique_lock<std::mutex> lk;
    SideStreams *ss = nullptr;
    hipStream_t user, sa, sb;
    bool failed = false;
    // allow == false: everything stays on the caller's stream.  Kernels that are dealt out in pieces of tiles size
    // their workgroups for having the whole chip at once; beside another kernel they would run in two rounds.
    explicit ForkJoin(hipStream_t u, bool allow = true) : user(u), sa(u), sb(u) {
        if (!allow || !overlap_enabled()) return;
        lk = std::unique_lock<std::mutex>(g_side_mu);
        ss = side_streams();
        if (!ss) return;
        if (hipEventRecord(ss->fork, user) != hipSuccess || hipStreamWaitEvent(ss->a, ss->fork, 0) != hipSuccess ||
            hipStreamWaitEvent(ss->b, ss->fork, 0) != hipSuccess) {
            ss = nullptr;
            (void)hipGetLastError();
            return;
        }
        sa = ss->a;
        sb = ss->b;
    }
    // Must be called on every path once the fork has happened, also after a failed launch.
    int join() {
        if (!ss) return SEPCORR_OK;
        const bool bad = hipEventRecord(ss->ja, sa) != hipSuccess || hipEventRecord(ss->jb, sb) != hipSuccess ||
                         hipStreamWaitEvent(user, ss->ja, 0) != hipSuccess || hipStreamWaitEvent(user, ss->jb, 0) != hipSuccess;
        ss = nullptr;
        return bad ? fail(SEPCORR_ELAUNCH, "sepcorr: joining the side streams failed") : SEPCORR_OK;
    }
    ~ForkJoin() { (void)join(); }
};

#if SEPCORR_IN_PART(0)
std::mutex g_scratch_mu;
void *g_scratch_ptr[64];

// Device address of `scratch` on the current device, resolved once per device.
int static_scratch(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SEPCORR_ELAUNCH, "sepcorr: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(SEPCORR_EINVAL, "sepcorr: device index %d is not supported", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return fail(SEPCORR_ELAUNCH, "sepcorr: address of the static scratch array on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return SEPCORR_OK;
}
#endif

int check_workspace(const Dims &d, void *ws, size_t ws_bytes) {
    const size_t need = sepcorr_backward_workspace_bytes(d.B, d.H1, d.W1, d.H2, d.W2, d.C);
    if (need > 0 && (ws == nullptr || ws_bytes < need))
        return fail(SEPCORR_EWORKSPACE, "sepcorr: backward needs %zu bytes of workspace, got %zu", need, ws ? ws_bytes : (size_t)0);
    if (need > 0 && (reinterpret_cast<uintptr_t>(ws) & 255))
        return fail(SEPCORR_EWORKSPACE, "sepcorr: workspace must be 256-byte aligned");
    return SEPCORR_OK;
}

// Scratch of a forward-type sweep is optional: without it every workgroup takes a whole pixel tile.
int check_fwd_workspace(const Dims &d, int K, void *ws, size_t ws_bytes) {
    if (ws == nullptr) return SEPCORR_OK;
    const size_t need = fwd_split_bytes(d.B, d.H1, d.W1, d.H2, d.W2, K);
    if (ws_bytes < need)
        return fail(SEPCORR_EWORKSPACE, "sepcorr: forward workspace of %zu bytes given, %zu needed (or pass NULL)", ws_bytes, need);
    if (reinterpret_cast<uintptr_t>(ws) & 255) return fail(SEPCORR_EWORKSPACE, "sepcorr: workspace must be 256-byte aligned");
    return SEPCORR_OK;
}

// Max/avg backward: by gathers of feature rows where the sizes allow and sepcorr_set_max_avg_backward() does not say
// otherwise, else by the dense recomputing kernels.  The gather path moves B*N1*(H2+W2) rows per gradient, the dense one
// multiplies N1 x N2 x C twice per gradient: with few positions per line of fmap2, or little work altogether, the dense
// kernels are as fast.
bool maxavg_by_gather(const Dims &d) {
    const int mode = g_maxavg_backward.load(std::memory_order_relaxed);
    if (mode == SEPCORR_MAXAVG_DENSE) return false;
    if (!sepcorr_gather_backward_eligible(d.B, d.H1, d.W1, d.H2, d.W2, d.C)) return false;
    if (mode == SEPCORR_MAXAVG_GATHER) return true;
    // Measured on MI355X (C = 256): the dense kernels take about 9 us per million (pixel, position) pairs plus 0.04 ms,
    // the gather path its row traffic plus 0.03 ms of launches; it wins from 12 positions per line of fmap2 on, and from
    // 8 on when there are many pixels (the dense d_f2 then has few tiles and long sums).
    const size_t n1 = (size_t)d.B * d.H1 * d.W1, n2 = (size_t)d.H2 * d.W2, lines = (size_t)d.H2 + d.W2;
    return n2 >= 12 * lines || (n2 >= 8 * lines && n1 >= 16384);
}

// Whether the gather path's three chains of kernels run beside each other: they fetch single rows of both feature maps
// through the L2 caches, and once fmap2 of one batch entry is larger than an L2 (4 MB) they evict each other's rows
// (B=2, 55x128: 0.41 ms beside each other, 0.375 ms one after the other; B=4, 48x64: 0.19 against 0.22 ms); below
// 300 000 rows per gradient the fork and join cost more than the overlap gains.
bool gather_overlap(const Dims &d) {
    const size_t rows = (size_t)d.B * d.H1 * d.W1 * ((size_t)d.H2 + d.W2);
    return rows >= 300000 && (size_t)d.H2 * d.W2 * d.C * 4 <= ((size_t)4 << 20);
}

int maxavg_backward(const Dims &d, bool gather, const float *f1, const float *f2, const int32_t *am_u, const int32_t *am_v,
                    const float *g_u, const float *g_v, float *d_f1, float *d_f2, void *ws, hipStream_t s1, hipStream_t s,
                    hipStream_t s2 = nullptr, hipEvent_t s2_done = nullptr) {
    // s2 with s2_done: a third stream for work that s waits for through that event (the gather path's table)
    if (gather)
        return sepcorr_gather_backward(f1, f2, am_u, am_v, g_u, g_v, d_f1, d_f2, d.B, d.H1, d.W1, d.H2, d.W2, d.C, ws, s1, s,
                                       s2_done ? s2 : s, s2_done);
    BwdArgs a;
    memset(&a, 0, sizeof(a));
    a.xcd_order = xcd_order_enabled();
    a.f1 = f1; a.f2 = f2; a.am_u = am_u; a.am_v = am_v; a.g_u = g_u; a.g_v = g_v;
    a.d1 = d_f1; a.d2 = d_f2;
    a.B = d.B; a.N1 = d.H1 * d.W1; a.H2 = d.H2; a.W2 = d.W2; a.C = d.C; a.KT = 1;
    return launch_bwd<GMODE_MAXAVG, 1>(a, d, ws, s1, s);
}

#define REQUIRE_PTR(p) \
    if ((p) == nullptr) return fail(SEPCORR_EINVAL, "sepcorr: argument %s is NULL", #p)

}  // namespace

#if SEPCORR_IN_PART(0)
void *sepcorr_prof_begin(const char *name, void *stream) {
    return t_prof_on ? new ProfScope(name, static_cast<hipStream_t>(stream)) : nullptr;
}

void sepcorr_prof_end(void *token) { delete static_cast<ProfScope *>(token); }

void *sepcorr_fork(void *user, void **sa, void **sb) {
    api_enter();
    ForkJoin *fj = new ForkJoin(static_cast<hipStream_t>(user));
    *sa = fj->sa;
    *sb = fj->sb;
    return fj;
}

int sepcorr_join(void *token) {
    ForkJoin *fj = static_cast<ForkJoin *>(token);
    const int rc = fj->join();
    delete fj;
    return rc;
}

extern "C" {

const char *sepcorr_last_error(void) { return g_err; }
int sepcorr_abi_version(void) { return 2; }

int sepcorr_set_max_avg_backward(int mode) {
    if (mode != SEPCORR_MAXAVG_AUTO && mode != SEPCORR_MAXAVG_DENSE && mode != SEPCORR_MAXAVG_GATHER) return g_maxavg_backward.load();
    return g_maxavg_backward.exchange(mode);
}

int sepcorr_set_contraction(int mode) {
    if (mode != SEPCORR_CONTRACT_FP32 && mode != SEPCORR_CONTRACT_BF16X3) return g_contraction.load();
    return g_contraction.exchange(mode);
}

int sepcorr_profile_enable(int on) {
    g_prof_on.store(on != 0, std::memory_order_relaxed);
    return SEPCORR_OK;
}

int sepcorr_profile_collect(char *names, size_t names_cap, float *ms, int cap) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    std::string joined;
    int n = 0;
    for (const ProfRec &r : g_prof_recs) {
        float t = 0.f;
        (void)hipEventSynchronize(r.e1);
        const hipError_t e = hipEventElapsedTime(&t, r.e0, r.e1);
        (void)hipEventDestroy(r.e0);
        (void)hipEventDestroy(r.e1);
        if (e != hipSuccess || n >= cap) continue;
        if (joined.size() + strlen(r.name) + 2 > names_cap) continue;
        if (n) joined += '\n';
        joined += r.name;
        ms[n++] = t;
    }
    g_prof_recs.clear();
    if (names && names_cap) snprintf(names, names_cap, "%s", joined.c_str());
    return n;
}

size_t sepcorr_forward_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C, int K) {
    if (B < 1 || H1 < 1 || W1 < 1 || H2 < 1 || W2 < 1 || C < 1 || K < 1) return 0;
    return fwd_split_bytes(B, H1, W1, H2, W2, K);
}

int sepcorr_max_avg_forward(const float *f1, const float *f2, float *out_u, float *out_v, int B, int H1, int W1, int H2,
                            int W2, int C, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(out_u); REQUIRE_PTR(out_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, 2)) return rc;
    if (int rc = check_fwd_workspace(d, 2, workspace, workspace_bytes)) return rc;
    FwdArgs a = fwd_args(d);
    a.ws = workspace; a.ws_bytes = workspace_bytes;
    a.f1 = f1; a.f2 = f2; a.out_u = out_u; a.out_v = out_v;
    Bf16Planes planes;
    if (int rc = planes.make(d, f2, static_cast<hipStream_t>(stream))) return rc;
    a.f2_planes = static_cast<const char *>(planes.ptr);
    a.H2p = planes.H2p;
    return launch_fwd<MODE_MAXAVG, 1, 2>(a, B, static_cast<hipStream_t>(stream));
}

int sepcorr_max_argmax_avg_forward(const float *f1, const float *f2, float *out_u, float *out_v, int32_t *argmax_u,
                                   int32_t *argmax_v, int B, int H1, int W1, int H2, int W2, int C, void *workspace,
                                   size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(out_u); REQUIRE_PTR(out_v); REQUIRE_PTR(argmax_u); REQUIRE_PTR(argmax_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, 2)) return rc;
    if (int rc = check_fwd_workspace(d, 2, workspace, workspace_bytes)) return rc;
    FwdArgs a = fwd_args(d);
    a.ws = workspace; a.ws_bytes = workspace_bytes;
    a.f1 = f1; a.f2 = f2; a.out_u = out_u; a.out_v = out_v; a.am_u = argmax_u; a.am_v = argmax_v;
    Bf16Planes planes;
    if (int rc = planes.make(d, f2, static_cast<hipStream_t>(stream))) return rc;
    a.f2_planes = static_cast<const char *>(planes.ptr);
    a.H2p = planes.H2p;
    return launch_fwd<MODE_ARGMAX, 1, 2>(a, B, static_cast<hipStream_t>(stream));
}

int sepcorr_compression_forward(const float *f1, const float *f2, const float *a_u, const float *a_v, float *comp_u,
                                float *comp_v, int B, int H1, int W1, int H2, int W2, int C, int K, void *workspace,
                                size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(a_u); REQUIRE_PTR(a_v); REQUIRE_PTR(comp_u); REQUIRE_PTR(comp_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, K)) return rc;
    if (int rc = check_fwd_workspace(d, K, workspace, workspace_bytes)) return rc;
    return weighted_forward(d, f1, f2, a_u, a_v, comp_u, comp_v, K, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

size_t sepcorr_backward_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C) {
    if (B < 1 || H1 < 1 || W1 < 1 || H2 < 1 || W2 < 1 || C < 1) return 0;
    const Dims d = {B, H1, W1, H2, W2, C};
    return bwd_ws(d).total;
}

int sepcorr_max_argmax_avg_backward(const float *f1, const float *f2, const int32_t *argmax_u, const int32_t *argmax_v,
                                    const float *grad_u, const float *grad_v, float *d_f1, float *d_f2, int B, int H1,
                                    int W1, int H2, int W2, int C, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(argmax_u); REQUIRE_PTR(argmax_v); REQUIRE_PTR(grad_u); REQUIRE_PTR(grad_v);
    REQUIRE_PTR(d_f1); REQUIRE_PTR(d_f2);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, 2)) return rc;
    if (int rc = check_workspace(d, workspace, workspace_bytes)) return rc;
    const bool gather = maxavg_by_gather(d);
    ForkJoin fj(static_cast<hipStream_t>(stream), gather ? gather_overlap(d) : !bwd_ws(d).aliased);
    // d_f1 aside, d_f2 on the caller's stream
    // the join event of side stream b serves as "table ready" in between: nothing else is recorded on b before the join
    const int rc = maxavg_backward(d, gather, f1, f2, argmax_u, argmax_v, grad_u, grad_v, d_f1, d_f2, workspace, fj.sa, fj.user,
                                   fj.sb, fj.ss ? fj.ss->jb : nullptr);
    const int rj = fj.join();
    return rc ? rc : rj;
}

int sepcorr_max_argmax_avg_backward_static(const float *f1, const float *f2, const int32_t *argmax_u, const int32_t *argmax_v,
                                           const float *grad_u, const float *grad_v, float *d_f1, float *d_f2, int B, int H1,
                                           int W1, int H2, int W2, int C, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(argmax_u); REQUIRE_PTR(argmax_v); REQUIRE_PTR(grad_u); REQUIRE_PTR(grad_v);
    REQUIRE_PTR(d_f1); REQUIRE_PTR(d_f2);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, 2)) return rc;
    const bool gather = maxavg_by_gather(d);   // the same choice as sepcorr_max_argmax_avg_backward makes
    // what this entry point itself uses of the workspace
    const size_t need = gather ? sepcorr_gather_backward_bytes(B, H1, W1, H2, W2, C) : bwd_ws(d).own_total;
    if (need > (size_t)SEPCORR_STATIC_SCRATCH_BYTES)
        return fail(SEPCORR_EWORKSPACE,
                    "sepcorr: these sizes need %zu bytes of scratch, the static array holds %zu: use "
                    "sepcorr_max_argmax_avg_backward with a workspace", need, (size_t)SEPCORR_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    struct NoAlloc {   // nothing below may allocate: one stream, fp32 contraction, no timing events
        bool prof;
        NoAlloc() : prof(t_prof_on) { t_no_alloc = true; t_prof_on = false; }
        ~NoAlloc() { t_no_alloc = false; t_prof_on = prof; }
    } guard;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return maxavg_backward(d, gather, f1, f2, argmax_u, argmax_v, grad_u, grad_v, d_f1, d_f2, ws, s, s);
}

int sepcorr_compression_backward(const float *f1, const float *f2, const float *a_u, const float *a_v, const float *g_cu,
                                 const float *g_cv, float *d_f1, float *d_f2, float *d_a_u, float *d_a_v, int B, int H1,
                                 int W1, int H2, int W2, int C, int K, void *workspace, size_t workspace_bytes,
                                 void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(a_u); REQUIRE_PTR(a_v); REQUIRE_PTR(g_cu); REQUIRE_PTR(g_cv);
    REQUIRE_PTR(d_a_u); REQUIRE_PTR(d_a_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, K)) return rc;
    if ((d_f1 == nullptr) != (d_f2 == nullptr))
        return fail(SEPCORR_EINVAL, "sepcorr: d_f1 and d_f2 must be given together or both be NULL");
    if (d_f1 == nullptr) {   // only the gradients of the weights: one sweep; its scratch is optional like the forward's
        if (int rc = check_fwd_workspace(d, K, workspace, workspace_bytes)) return rc;
        return weighted_forward(d, f1, f2, g_cv, g_cu, d_a_v, d_a_u, K, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
    }
    if (int rc = check_workspace(d, workspace, workspace_bytes)) return rc;
    const BwdWs lay = bwd_ws(d);
    ForkJoin fj(static_cast<hipStream_t>(stream), !lay.aliased);
    // d_a_v[k,u] = sum_v S g_cv[k,v];  d_a_u[k,v] = sum_u S g_cu[k,u]: the forward's weighted sums
    int rc = weighted_forward(d, f1, f2, g_cv, g_cu, d_a_v, d_a_u, K, lay.fwd_bytes ? workspace : nullptr, lay.fwd_bytes, fj.user);
    BwdArgs a;
    memset(&a, 0, sizeof(a));
    a.xcd_order = xcd_order_enabled();
    a.f1 = f1; a.f2 = f2; a.a_u = a_u; a.a_v = a_v; a.g_cu = g_cu; a.g_cv = g_cv;
    a.d1 = d_f1; a.d2 = d_f2;
    a.B = B; a.N1 = H1 * W1; a.H2 = H2; a.W2 = W2; a.C = C; a.KT = K;
    const int kch = W2 > 128 ? 2 : KCH;  // wide workgroups have half the registers per lane
    // channel chunks accumulate into d_f1 / d_f2: each output keeps its own stream, so chunks stay ordered
    for (int k0 = 0; k0 < K && rc == SEPCORR_OK; k0 += kch) {
        a.k0 = k0;
        a.accumulate = k0 > 0;
        const int kc = K - k0 < kch ? K - k0 : kch;
        switch (kc) {
            case 1: rc = launch_bwd<GMODE_COMP, 1>(a, d, workspace, fj.sa, fj.sb); break;
            case 2: rc = launch_bwd<GMODE_COMP, 2>(a, d, workspace, fj.sa, fj.sb); break;
            case 3: rc = launch_bwd<GMODE_COMP, 3>(a, d, workspace, fj.sa, fj.sb); break;
            default: rc = launch_bwd<GMODE_COMP, 4>(a, d, workspace, fj.sa, fj.sb); break;
        }
    }
    const int rj = fj.join();
    return rc ? rc : rj;
}

// ---- attention compression straight from the logits -------------------------------------------------------------

int sepcorr_softmax_rows(const float *logits, float *stats, int stats_given, float *a, long nrows, int L, void *stream) {
    api_enter();
    REQUIRE_PTR(logits); REQUIRE_PTR(stats);
    if (nrows < 1 || L < 1) return fail(SEPCORR_EINVAL, "sepcorr: softmax rows: nrows=%ld L=%d", nrows, L);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)((nrows + 3) / 4)), block(256);
    if (!stats_given) hipLaunchKernelGGL(row_stats_kernel, grid, block, 0, s, logits, stats, nrows, L);
    if (a) hipLaunchKernelGGL(softmax_apply_kernel, dim3(row_groups((size_t)nrows)), block, 0, s, logits, stats, a, nrows, L,
                              (int)(rows_vec4(logits, L) && rows_vec4(a, L)));
    return check_launch("softmax rows");
}

int sepcorr_compression_forward_from_logits(const float *f1, const float *f2, const float *logits_u, const float *logits_v,
                                            float *comp_u, float *comp_v, float *stats_u, float *stats_v, int stats_given,
                                            int B, int H1, int W1, int H2, int W2, int C, int K, void *workspace,
                                            size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(logits_u); REQUIRE_PTR(logits_v); REQUIRE_PTR(comp_u); REQUIRE_PTR(comp_v);
    REQUIRE_PTR(stats_u); REQUIRE_PTR(stats_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, K)) return rc;
    if (int rc = check_fwd_workspace(d, K, workspace, workspace_bytes)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long nrows = (long)B * H1 * W1 * K;
    if (!stats_given) {   // (max, sum of exp) per row: one pass over the logits
        const dim3 grid((unsigned)((nrows + 3) / 4)), block(256);
        ProfScope ps("row_stats", s);
        hipLaunchKernelGGL(row_stats_kernel, grid, block, 0, s, logits_u, stats_u, nrows, W2);
        hipLaunchKernelGGL(row_stats_kernel, grid, block, 0, s, logits_v, stats_v, nrows, H2);
        if (int rc = check_launch("row statistics")) return rc;
    }
    FwdArgs soft;
    memset(&soft, 0, sizeof(soft));
    soft.logits = 1; soft.st_wv = stats_u; soft.st_wu = stats_v;
    return weighted_forward(d, f1, f2, logits_u, logits_v, comp_u, comp_v, K, workspace, workspace_bytes, s, &soft);
}

size_t sepcorr_compression_backward_from_logits_workspace_bytes(int B, int H1, int W1, int H2, int W2, int C, int K,
                                                                int with_features) {
    if (B < 1 || H1 < 1 || W1 < 1 || H2 < 1 || W2 < 1 || C < 1 || K < 1 || K > MAX_K) return 0;
    const Dims d = {B, H1, W1, H2, W2, C};
    const size_t rows = (size_t)B * H1 * W1 * K;
    const size_t dots = 2 * ((rows * sizeof(float) + 255) & ~(size_t)255);
    if (!with_features) return ((fwd_split_bytes(B, H1, W1, H2, W2, K) + 255) & ~(size_t)255) + dots;
    const size_t a_bytes = ((rows * W2 * sizeof(float) + 255) & ~(size_t)255) + ((rows * H2 * sizeof(float) + 255) & ~(size_t)255);
    return bwd_ws(d).total + dots + a_bytes;
}

int sepcorr_compression_backward_from_logits(const float *f1, const float *f2, const float *logits_u, const float *logits_v,
                                             const float *stats_u, const float *stats_v, const float *comp_u,
                                             const float *comp_v, const float *g_cu, const float *g_cv, float *d_f1,
                                             float *d_f2, float *d_logits_u, float *d_logits_v, int B, int H1, int W1, int H2,
                                             int W2, int C, int K, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(logits_u); REQUIRE_PTR(logits_v); REQUIRE_PTR(stats_u); REQUIRE_PTR(stats_v);
    REQUIRE_PTR(comp_u); REQUIRE_PTR(comp_v); REQUIRE_PTR(g_cu); REQUIRE_PTR(g_cv); REQUIRE_PTR(d_logits_u); REQUIRE_PTR(d_logits_v);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, K)) return rc;
    if ((d_f1 == nullptr) != (d_f2 == nullptr))
        return fail(SEPCORR_EINVAL, "sepcorr: d_f1 and d_f2 must be given together or both be NULL");
    const size_t need = sepcorr_compression_backward_from_logits_workspace_bytes(B, H1, W1, H2, W2, C, K, d_f1 != nullptr);
    if (workspace == nullptr || workspace_bytes < need)
        return fail(SEPCORR_EWORKSPACE, "sepcorr: backward from logits needs %zu bytes of workspace, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(SEPCORR_EWORKSPACE, "sepcorr: workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t rows = (size_t)B * H1 * W1 * K;
    const size_t dot_bytes = (rows * sizeof(float) + 255) & ~(size_t)255;
    const size_t sweep_bytes = d_f1 ? bwd_ws(d).total : (fwd_split_bytes(B, H1, W1, H2, W2, K) + 255) & ~(size_t)255;
    char *base = static_cast<char *>(workspace);
    float *dot_u = reinterpret_cast<float *>(base + sweep_bytes);               // sum_u g_cu * comp_u = sum_v a_u * d_a_u
    float *dot_v = reinterpret_cast<float *>(base + sweep_bytes + dot_bytes);   // sum_v g_cv * comp_v = sum_u a_v * d_a_v
    {
        const dim3 grid(row_groups(rows)), block(256);
        ProfScope ps("row_dots", s);
        hipLaunchKernelGGL(row_dot_kernel, grid, block, 0, s, g_cu, comp_u, dot_u, (long)rows, H2, (int)(rows_vec4(g_cu, H2) && rows_vec4(comp_u, H2)));
        hipLaunchKernelGGL(row_dot_kernel, grid, block, 0, s, g_cv, comp_v, dot_v, (long)rows, W2, (int)(rows_vec4(g_cv, W2) && rows_vec4(comp_v, W2)));
        if (int rc = check_launch("row dot products")) return rc;
    }
    // d_a_v[k,u] = sum_v S g_cv[k,v] and d_a_u[k,v] = sum_u S g_cu[k,u] as in sepcorr_compression_backward, turned into
    // gradients of the logits where they are stored: d_z = a (d_a - sum a d_a), the sums being the dot products above
    FwdArgs soft;
    memset(&soft, 0, sizeof(soft));
    soft.dlog = 1;
    soft.z_ou = logits_v; soft.st_ou = stats_v; soft.dot_ou = dot_v;
    soft.z_ov = logits_u; soft.st_ov = stats_u; soft.dot_ov = dot_u;
    const size_t fwd_bytes = fwd_split_bytes(B, H1, W1, H2, W2, d_f1 ? MAX_K : K);
    int rc = weighted_forward(d, f1, f2, g_cv, g_cu, d_logits_v, d_logits_u, K, fwd_bytes ? workspace : nullptr, fwd_bytes, s, &soft);
    if (rc || d_f1 == nullptr) return rc;
    // feature gradients: the weights themselves, formed once from logits and statistics behind the other scratch
    float *a_u = reinterpret_cast<float *>(base + sweep_bytes + 2 * dot_bytes);
    float *a_v = reinterpret_cast<float *>(base + sweep_bytes + 2 * dot_bytes + ((rows * W2 * sizeof(float) + 255) & ~(size_t)255));
    {
        const dim3 grid(row_groups(rows)), block(256);
        ProfScope ps("softmax_apply", s);
        hipLaunchKernelGGL(softmax_apply_kernel, grid, block, 0, s, logits_u, stats_u, a_u, (long)rows, W2, (int)(rows_vec4(logits_u, W2) && rows_vec4(a_u, W2)));
        hipLaunchKernelGGL(softmax_apply_kernel, grid, block, 0, s, logits_v, stats_v, a_v, (long)rows, H2, (int)(rows_vec4(logits_v, H2) && rows_vec4(a_v, H2)));
        if (int rc2 = check_launch("softmax from statistics")) return rc2;
    }
    const BwdWs lay = bwd_ws(d);
    ForkJoin fj(s, !lay.aliased);
    BwdArgs a;
    memset(&a, 0, sizeof(a));
    a.xcd_order = xcd_order_enabled();
    a.f1 = f1; a.f2 = f2; a.a_u = a_u; a.a_v = a_v; a.g_cu = g_cu; a.g_cv = g_cv;
    a.d1 = d_f1; a.d2 = d_f2;
    a.B = B; a.N1 = H1 * W1; a.H2 = H2; a.W2 = W2; a.C = C; a.KT = K;
    const int kch = W2 > 128 ? 2 : KCH;
    for (int k0 = 0; k0 < K && rc == SEPCORR_OK; k0 += kch) {
        a.k0 = k0;
        a.accumulate = k0 > 0;
        const int kc = K - k0 < kch ? K - k0 : kch;
        switch (kc) {
            case 1: rc = launch_bwd<GMODE_COMP, 1>(a, d, workspace, fj.sa, fj.sb); break;
            case 2: rc = launch_bwd<GMODE_COMP, 2>(a, d, workspace, fj.sa, fj.sb); break;
            case 3: rc = launch_bwd<GMODE_COMP, 3>(a, d, workspace, fj.sa, fj.sb); break;
            default: rc = launch_bwd<GMODE_COMP, 4>(a, d, workspace, fj.sa, fj.sb); break;
        }
    }
    const int rj = fj.join();
    return rc ? rc : rj;
}

// ---- several pyramid levels per call ---------------------------------------------------------------------------

namespace {
struct LevelDims {
    int nlev, h2max, w2max;
};
int check_levels(const int *h2, const int *w2, int nlev, int B, int H1, int W1, int C, int K, LevelDims *out) {
    if (h2 == nullptr || w2 == nullptr) return fail(SEPCORR_EINVAL, "sepcorr: level size tables are NULL");
    if (nlev < 1 || nlev > 4) return fail(SEPCORR_EINVAL, "sepcorr: %d levels given, 1..4 supported", nlev);
    out->nlev = nlev; out->h2max = 0; out->w2max = 0;
    for (int l = 0; l < nlev; ++l) {
        const Dims d = {B, H1, W1, h2[l], w2[l], C};
        if (int rc = check_dims(d, K)) return rc;
        if (h2[l] > out->h2max) out->h2max = h2[l];
        if (w2[l] > out->w2max) out->w2max = w2[l];
    }
    return SEPCORR_OK;
}
size_t levels_sweep_bytes(const int *h2, const int *w2, int nlev, int B, int H1, int W1, int K) {
    int w2max = 0;
    size_t single = 0;
    for (int l = 0; l < nlev; ++l) {
        if (w2[l] > w2max) w2max = w2[l];
        const size_t n = fwd_split_bytes(B, H1, W1, h2[l], w2[l], K);
        if (n > single) single = n;
    }
    const size_t multi = fwd_levels_bytes(B * ((H1 * W1 + TP - 1) / TP), nlev, w2max, K);
    return ((multi > single ? multi : single) + 255) & ~(size_t)255;
}
}  // namespace

size_t sepcorr_forward_levels_workspace_bytes(const int *h2, const int *w2, int nlev, int B, int H1, int W1, int C, int K) {
    if (h2 == nullptr || w2 == nullptr || nlev < 1 || nlev > 4 || B < 1 || H1 < 1 || W1 < 1 || C < 1 || K < 1) return 0;
    for (int l = 0; l < nlev; ++l)
        if (h2[l] < 1 || w2[l] < 1) return 0;
    // + the row dot products of the backward call (two per level)
    return levels_sweep_bytes(h2, w2, nlev, B, H1, W1, K) + 2 * (size_t)nlev * ((((size_t)B * H1 * W1 * K * sizeof(float)) + 255) & ~(size_t)255);
}

int sepcorr_max_argmax_avg_forward_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2, int nlev,
                                          float *const *out_u, float *const *out_v, int32_t *const *argmax_u,
                                          int32_t *const *argmax_v, int B, int H1, int W1, int C, void *workspace,
                                          size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2_levels); REQUIRE_PTR(out_u); REQUIRE_PTR(out_v); REQUIRE_PTR(argmax_u); REQUIRE_PTR(argmax_v);
    LevelDims ld;
    if (int rc = check_levels(h2, w2, nlev, B, H1, W1, C, 2, &ld)) return rc;
    for (int l = 0; l < nlev; ++l)
        if (!f2_levels[l] || !out_u[l] || !out_v[l] || !argmax_u[l] || !argmax_v[l])
            return fail(SEPCORR_EINVAL, "sepcorr: a pointer of level %d is NULL", l);
    const size_t need = levels_sweep_bytes(h2, w2, nlev, B, H1, W1, 2);
    if (workspace != nullptr && (workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255)))
        return fail(SEPCORR_EWORKSPACE, "sepcorr: %zu bytes of 256-byte aligned workspace needed (or NULL), got %zu", need, workspace_bytes);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Dims d0 = {B, H1, W1, h2[0], w2[0], C};
    FwdArgs a = fwd_args(d0);
    a.f1 = f1; a.ws = workspace; a.ws_bytes = workspace_bytes;
    a.nlev = nlev;
    for (int l = 0; l < nlev; ++l) {
        FwdLevel &L = a.lev[l];
        L.f2 = f2_levels[l]; L.out_u = out_u[l]; L.out_v = out_v[l]; L.am_u = argmax_u[l]; L.am_v = argmax_v[l];
        L.H2 = h2[l]; L.W2 = w2[l];
    }
    const int rc = nlev > 1 ? launch_fwd_levels<MODE_ARGMAX, 1, 2>(a, B, s) : SEPCORR_EINVAL;
    if (rc != SEPCORR_EINVAL) return rc;
    for (int l = 0; l < nlev; ++l)   // shapes outside the one-launch path: level by level
        if (int r2 = sepcorr_max_argmax_avg_forward(f1, f2_levels[l], out_u[l], out_v[l], argmax_u[l], argmax_v[l], B, H1, W1,
                                                    h2[l], w2[l], C, workspace, workspace ? workspace_bytes : 0, stream))
            return r2;
    return SEPCORR_OK;
}

namespace {
// The weighted sweep of every level: logits -> sums (dlog == 0) or upstream gradients -> logit gradients (dlog == 1).
int soft_levels(const float *f1, const float *const *f2, const int *h2, const int *w2, int nlev, const FwdLevel *lev, int dlog,
                int B, int H1, int W1, int C, int K, void *ws, size_t ws_bytes, hipStream_t s) {
    const Dims d0 = {B, H1, W1, h2[0], w2[0], C};
    FwdArgs a = fwd_args(d0);
    a.f1 = f1; a.ws = ws; a.ws_bytes = ws_bytes; a.KT = K;
    a.logits = !dlog; a.dlog = dlog;
    a.nlev = nlev;
    for (int l = 0; l < nlev; ++l) {
        a.lev[l] = lev[l];
        a.lev[l].f2 = f2[l]; a.lev[l].H2 = h2[l]; a.lev[l].W2 = w2[l];
    }
    bool one_launch = nlev > 1;
    for (int k0 = 0; k0 < K && one_launch; k0 += KCH) {
        a.k0 = k0;
        const int kc = K - k0 < KCH ? K - k0 : KCH;
        int rc;
        switch (kc) {
            case 1: rc = launch_fwd_levels<MODE_SOFT, 1, 2>(a, B, s); break;
            case 2: rc = launch_fwd_levels<MODE_SOFT, 2, 2>(a, B, s); break;
            case 3: rc = launch_fwd_levels<MODE_SOFT, 3, 1>(a, B, s); break;
            default: rc = launch_fwd_levels<MODE_SOFT, 4, 1>(a, B, s); break;
        }
        if (rc == SEPCORR_EINVAL && k0 == 0) one_launch = false;   // shapes outside the one-launch path
        else if (rc) return rc;
    }
    if (one_launch) return SEPCORR_OK;
    for (int l = 0; l < nlev; ++l) {
        const Dims d = {B, H1, W1, h2[l], w2[l], C};
        FwdArgs soft;
        memset(&soft, 0, sizeof(soft));
        soft.logits = !dlog; soft.dlog = dlog;
        soft.st_wv = lev[l].st_wv; soft.st_wu = lev[l].st_wu;
        soft.z_ou = lev[l].z_ou; soft.st_ou = lev[l].st_ou; soft.dot_ou = lev[l].dot_ou;
        soft.z_ov = lev[l].z_ov; soft.st_ov = lev[l].st_ov; soft.dot_ov = lev[l].dot_ov;
        const size_t n = fwd_split_bytes(B, H1, W1, h2[l], w2[l], K);
        if (int rc = weighted_forward(d, f1, f2[l], lev[l].wv, lev[l].wu, lev[l].out_u, lev[l].out_v, K, n && ws ? ws : nullptr, n, s, &soft))
            return rc;
    }
    return SEPCORR_OK;
}
}  // namespace

int sepcorr_compression_forward_from_logits_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                                                   int nlev, const float *const *logits_u, const float *const *logits_v,
                                                   const float *const *stats_u, const float *const *stats_v,
                                                   float *const *comp_u, float *const *comp_v, int B, int H1, int W1, int C,
                                                   int K, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2_levels); REQUIRE_PTR(logits_u); REQUIRE_PTR(logits_v); REQUIRE_PTR(stats_u); REQUIRE_PTR(stats_v);
    REQUIRE_PTR(comp_u); REQUIRE_PTR(comp_v);
    LevelDims ld;
    if (int rc = check_levels(h2, w2, nlev, B, H1, W1, C, K, &ld)) return rc;
    const size_t need = levels_sweep_bytes(h2, w2, nlev, B, H1, W1, K);
    if (workspace != nullptr && (workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255)))
        return fail(SEPCORR_EWORKSPACE, "sepcorr: %zu bytes of 256-byte aligned workspace needed (or NULL), got %zu", need, workspace_bytes);
    FwdLevel lev[4];
    memset(lev, 0, sizeof(lev));
    for (int l = 0; l < nlev; ++l) {
        if (!f2_levels[l] || !logits_u[l] || !logits_v[l] || !stats_u[l] || !stats_v[l] || !comp_u[l] || !comp_v[l])
            return fail(SEPCORR_EINVAL, "sepcorr: a pointer of level %d is NULL", l);
        lev[l].wv = logits_u[l]; lev[l].wu = logits_v[l]; lev[l].st_wv = stats_u[l]; lev[l].st_wu = stats_v[l];
        lev[l].out_u = comp_u[l]; lev[l].out_v = comp_v[l];
    }
    return soft_levels(f1, f2_levels, h2, w2, nlev, lev, 0, B, H1, W1, C, K, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int sepcorr_compression_backward_from_logits_levels(const float *f1, const float *const *f2_levels, const int *h2, const int *w2,
                                                    int nlev, const float *const *logits_u, const float *const *logits_v,
                                                    const float *const *stats_u, const float *const *stats_v,
                                                    const float *const *comp_u, const float *const *comp_v,
                                                    const float *const *g_cu, const float *const *g_cv,
                                                    float *const *d_logits_u, float *const *d_logits_v, int B, int H1, int W1,
                                                    int C, int K, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2_levels); REQUIRE_PTR(logits_u); REQUIRE_PTR(logits_v); REQUIRE_PTR(stats_u); REQUIRE_PTR(stats_v);
    REQUIRE_PTR(comp_u); REQUIRE_PTR(comp_v); REQUIRE_PTR(g_cu); REQUIRE_PTR(g_cv); REQUIRE_PTR(d_logits_u); REQUIRE_PTR(d_logits_v);
    LevelDims ld;
    if (int rc = check_levels(h2, w2, nlev, B, H1, W1, C, K, &ld)) return rc;
    const size_t need = sepcorr_forward_levels_workspace_bytes(h2, w2, nlev, B, H1, W1, C, K);
    if (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255))
        return fail(SEPCORR_EWORKSPACE, "sepcorr: %zu bytes of 256-byte aligned workspace needed, got %zu", need,
                    workspace ? workspace_bytes : (size_t)0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t sweep = levels_sweep_bytes(h2, w2, nlev, B, H1, W1, K);
    const size_t rows = (size_t)B * H1 * W1 * K;
    const size_t dot_bytes = (rows * sizeof(float) + 255) & ~(size_t)255;
    char *base = static_cast<char *>(workspace) + sweep;
    FwdLevel lev[4];
    memset(lev, 0, sizeof(lev));
    {
        ProfScope ps("row_dots", s);
        RowDotJobs jobs;
        memset(&jobs, 0, sizeof(jobs));
        for (int l = 0; l < nlev; ++l) {
            if (!f2_levels[l] || !logits_u[l] || !logits_v[l] || !stats_u[l] || !stats_v[l] || !comp_u[l] || !comp_v[l] ||
                !g_cu[l] || !g_cv[l] || !d_logits_u[l] || !d_logits_v[l])
                return fail(SEPCORR_EINVAL, "sepcorr: a pointer of level %d is NULL", l);
            float *dot_u = reinterpret_cast<float *>(base + (2 * l) * dot_bytes);       // sum_u g_cu comp_u
            float *dot_v = reinterpret_cast<float *>(base + (2 * l + 1) * dot_bytes);   // sum_v g_cv comp_v
            jobs.x[2 * l] = g_cu[l]; jobs.y[2 * l] = comp_u[l]; jobs.dot[2 * l] = dot_u; jobs.L[2 * l] = h2[l];
            jobs.x[2 * l + 1] = g_cv[l]; jobs.y[2 * l + 1] = comp_v[l]; jobs.dot[2 * l + 1] = dot_v; jobs.L[2 * l + 1] = w2[l];
            jobs.vec4[2 * l] = rows_vec4(g_cu[l], h2[l]) && rows_vec4(comp_u[l], h2[l]);
            jobs.vec4[2 * l + 1] = rows_vec4(g_cv[l], w2[l]) && rows_vec4(comp_v[l], w2[l]);
            lev[l].wv = g_cv[l]; lev[l].wu = g_cu[l];
            lev[l].out_u = d_logits_v[l]; lev[l].out_v = d_logits_u[l];
            lev[l].z_ou = logits_v[l]; lev[l].st_ou = stats_v[l]; lev[l].dot_ou = dot_v;
            lev[l].z_ov = logits_u[l]; lev[l].st_ov = stats_u[l]; lev[l].dot_ov = dot_u;
        }
        hipLaunchKernelGGL(row_dot_multi_kernel, dim3(row_groups(rows), 2 * nlev), dim3(256), 0, s, jobs, (long)rows);
        if (int rc = check_launch("row dot products")) return rc;
    }
    return soft_levels(f1, f2_levels, h2, w2, nlev, lev, 1, B, H1, W1, C, K, workspace, sweep, s);
}

static int fused_backward(const float *f1, const float *f2, const int32_t *argmax_u, const int32_t *argmax_v,
                          const float *grad_u, const float *grad_v, const float *a_u, const float *a_v,
                          const float *g_cu, const float *g_cv, float *d_f1, float *d_f2, int add_d_f1, int B, int H1, int W1, int H2,
                          int W2, int C, int K, void *workspace, size_t workspace_bytes, void *stream) {
    api_enter();
    REQUIRE_PTR(f1); REQUIRE_PTR(f2); REQUIRE_PTR(argmax_u); REQUIRE_PTR(argmax_v); REQUIRE_PTR(grad_u); REQUIRE_PTR(grad_v);
    REQUIRE_PTR(a_u); REQUIRE_PTR(a_v); REQUIRE_PTR(g_cu); REQUIRE_PTR(g_cv); REQUIRE_PTR(d_f1); REQUIRE_PTR(d_f2);
    const Dims d = {B, H1, W1, H2, W2, C};
    if (int rc = check_dims(d, K)) return rc;
    if (int rc = check_workspace(d, workspace, workspace_bytes)) return rc;
    BwdArgs a;
    memset(&a, 0, sizeof(a));
    a.xcd_order = xcd_order_enabled();
    a.f1 = f1; a.f2 = f2; a.am_u = argmax_u; a.am_v = argmax_v; a.g_u = grad_u; a.g_v = grad_v;
    a.a_u = a_u; a.a_v = a_v; a.g_cu = g_cu; a.g_cv = g_cv;
    a.d1 = d_f1; a.d2 = d_f2;
    a.add_d1 = add_d_f1 != 0;
    a.B = B; a.N1 = H1 * W1; a.H2 = H2; a.W2 = W2; a.C = C; a.KT = K;
    ForkJoin fj(static_cast<hipStream_t>(stream), !bwd_ws(d).aliased);
    const int kch = W2 > 128 ? 2 : KCH;
    const int kc0 = K < kch ? K : kch;
    // The first chunk of weight channels carries the max/avg terms of G along (built for 2 and 4 channels);
    // otherwise they follow as one more accumulating launch.
    const bool first_carries = kc0 == 2 || kc0 == 4;
    int rc = SEPCORR_OK;
    for (int k0 = 0; k0 < K && rc == SEPCORR_OK; k0 += kch) {
        a.k0 = k0;
        a.accumulate = k0 > 0;
        const int kc = K - k0 < kch ? K - k0 : kch;
        if (k0 == 0 && first_carries) {
            rc = kc == 2 ? launch_bwd<GMODE_BOTH, 2>(a, d, workspace, fj.sa, fj.user)
                         : launch_bwd<GMODE_BOTH, 4>(a, d, workspace, fj.sa, fj.user);
            continue;
        }
        switch (kc) {
            case 1: rc = launch_bwd<GMODE_COMP, 1>(a, d, workspace, fj.sa, fj.user); break;
            case 2: rc = launch_bwd<GMODE_COMP, 2>(a, d, workspace, fj.sa, fj.user); break;
            case 3: rc = launch_bwd<GMODE_COMP, 3>(a, d, workspace, fj.sa, fj.user); break;
            default: rc = launch_bwd<GMODE_COMP, 4>(a, d, workspace, fj.sa, fj.user); break;
        }
    }
    if (!first_carries && rc == SEPCORR_OK) {
        a.k0 = 0; a.KT = 1;
        a.accumulate = 1;
        rc = launch_bwd<GMODE_MAXAVG, 1>(a, d, workspace, fj.sa, fj.user);
    }
    const int rj = fj.join();
    return rc ? rc : rj;
}

int sepcorr_fused_backward(const float *f1, const float *f2, const int32_t *argmax_u, const int32_t *argmax_v,
                           const float *grad_u, const float *grad_v, const float *a_u, const float *a_v,
                           const float *g_cu, const float *g_cv, float *d_f1, float *d_f2, int B, int H1, int W1, int H2,
                           int W2, int C, int K, void *workspace, size_t workspace_bytes, void *stream) {
    return fused_backward(f1, f2, argmax_u, argmax_v, grad_u, grad_v, a_u, a_v, g_cu, g_cv, d_f1, d_f2, 0, B, H1, W1, H2, W2, C, K,
                          workspace, workspace_bytes, stream);
}

int sepcorr_fused_backward_add(const float *f1, const float *f2, const int32_t *argmax_u, const int32_t *argmax_v,
                               const float *grad_u, const float *grad_v, const float *a_u, const float *a_v,
                               const float *g_cu, const float *g_cv, float *d_f1, float *d_f2, int B, int H1, int W1, int H2,
                               int W2, int C, int K, void *workspace, size_t workspace_bytes, void *stream) {
    return fused_backward(f1, f2, argmax_u, argmax_v, grad_u, grad_v, a_u, a_v, g_cu, g_cv, d_f1, d_f2, 1, B, H1, W1, H2, W2, C, K,
                          workspace, workspace_bytes, stream);
}

}  // extern "C"
#endif  // part 0
