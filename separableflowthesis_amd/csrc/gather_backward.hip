// Backward of the max/avg separation without the correlation volume and without recomputing it: the gradient of a
// maximum reaches one entry of S per output element, and the gradient of an average reaches a whole line of S with
// one weight, so both feature gradients are sums of a few feature rows per output element.
//
// With S[p,(u,v)] = <f1[p,:], f2[(u,v),:]>, out_u[p,0,u] = max_v S, out_u[p,1,u] = mean_v S, out_v likewise over u
// (the reference defines these outputs in libs/MemorySaver/src/MemorySaver_kernel_forward.cu:328-533; its backward,
// libs/MemorySaver/src/MemorySaver_kernel_max_avg_argmax_backward.cu:785-921, visits every (p, u, v)):
//
//   d_f1[p,:]     = sum_u g_u[p,0,u] f2[(u, am_u[p,u]),:] + sum_v g_v[p,0,v] f2[(am_v[p,v], v),:]           (gather)
//                 + sum_u g_u[p,1,u] R[u,:] + sum_v g_v[p,1,v] Q[v,:]                                         (product)
//                   with R[u,:] = mean_v f2[(u,v),:], Q[v,:] = mean_u f2[(u,v),:]
//   d_f2[(u,v),:] = sum_{p: am_u[p,u]=v} g_u[p,0,u] f1[p,:] + sum_{p: am_v[p,v]=u} g_v[p,0,v] f1[p,:]           (gather)
//                 + A_u[u,:] / W2 + A_v[v,:] / H2
//                   with A_u[u,:] = sum_p g_u[p,1,u] f1[p,:], A_v[v,:] = sum_p g_v[p,1,v] f1[p,:]              (product)
//
// The two products are small matrix products (H2 + W2 lines) on fp32 MFMA; the gathers move one feature row per
// (p, u) and per (p, v) through the caches, B * N1 * (H2 + W2) * C * 4 bytes for each of the two gradients, which is
// what bounds this path.  d_f2 has no list of the pixels that chose a given (u, v): the wave that owns (u, v) scans
// column u of the transposed argmax_u and column v of the transposed argmax_v, collects the hits in a small queue in
// LDS and fetches their rows eight at a time.  Every sum has a fixed order, so results do not change from run to run.
//
// An argmax entry outside its range contributes nothing, as in the dense kernels (no column matches it).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "sepcorr.h"
#include "sepcorr_internal.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int SCAN = 256;      // pixels per step of the column scan (one 16-byte load per lane)
constexpr int QCAP = SCAN + 64;
static_assert(SCAN == 256, "one block of argmax_columns_kernel and one 16-byte load per lane cover a scan step");
constexpr int NB = 8;          // feature rows in flight per wave
constexpr int JCHUNK = 256;    // lines of the gradient tile staged in LDS at a time (df1_avg_rows_kernel)

// Row of the 32x32 accumulator held in register r of a lane in half h (lane / 32).
__device__ __forceinline__ int acc_row(int r, int h) { return (r >> 2) * 8 + h * 4 + (r & 3); }

__device__ __forceinline__ void wave_sync_lds() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

struct GatherArgs {
    const float *f1, *f2, *g_u, *g_v;
    const int *am_u, *am_v;
    float *d1, *d2;
    int *amT_u, *amT_v;     // [B][H2][N1p], [B][W2][N1p]; pad -1
    float *lines;           // [B][H2+W2][C]: R then Q
    float *table;           // [B][H2+W2][C]: A_u / W2 then A_v / H2
    float *table_part;      // [B][S][H2+W2][C]
    int B, N1, N1p, H2, W2, C, S;
    int line0;              // the tables hold the lines [line0, H2+W2) only (0: all; H2: those of g_v)
};

// amT[b][j][p] = am[b][p][j] for both argmax tensors; entries beyond N1 are -1 (no hit).  grid (N1p / 64, 2, B):
// 64 pixels of argmax_u (blockIdx.y == 0) or argmax_v go through LDS, TCHUNK lines at a time, so that the reads run
// along a pixel's lines and the writes along the pixels of a line.
constexpr int TCHUNK = 128;
__global__ void __launch_bounds__(256) argmax_columns_kernel(const GatherArgs a) {
    __shared__ int tile[64][TCHUNK + 1];
    const int p0 = blockIdx.x * 64, b = blockIdx.z;
    const bool second = blockIdx.y != 0;
    const int L = second ? a.W2 : a.H2, N1 = a.N1, N1p = a.N1p;
    const int *am = (second ? a.am_v : a.am_u) + (size_t)b * N1 * L;
    int *amT = (second ? a.amT_v : a.amT_u) + (size_t)b * L * N1p;
    for (int jc = 0; jc < L; jc += TCHUNK) {
        const int nj = min(TCHUNK, L - jc);
        if (jc) __syncthreads();
        for (int i = threadIdx.x; i < 64 * TCHUNK; i += 256) {
            const int px = i / TCHUNK, jl = i - px * TCHUNK, p = p0 + px;
            if (jl < nj) tile[px][jl] = p < N1 ? am[(size_t)p * L + jc + jl] : -1;
        }
        __syncthreads();
        const int px = threadIdx.x & 63;
        for (int jl = threadIdx.x >> 6; jl < nj; jl += 4) amT[(size_t)(jc + jl) * N1p + p0 + px] = tile[px][jl];
    }
}

// lines[b][j][:]: j < H2: mean_v f2[(j,v),:]; else mean_u f2[(u,j-H2),:].  grid (H2+W2, B); the four waves take every
// fourth term, lane = 4 channels.
__global__ void __launch_bounds__(256) fmap2_line_means_kernel(const GatherArgs a) {
    __shared__ v4f part[4][64];
    const int j = blockIdx.x, b = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int H2 = a.H2, W2 = a.W2, C = a.C;
    const bool on = 4 * lane < C;
    const float *f2b = a.f2 + (size_t)b * H2 * W2 * C + 4 * lane;
    const bool row = j < H2;
    const int n = row ? W2 : H2;
    const size_t base = row ? (size_t)j * W2 * C : (size_t)(j - H2) * C, step = row ? (size_t)C : (size_t)W2 * C;
    v4f s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0;
    if (on) {
        int i = wave;
        for (; i + 4 < n; i += 8) {
            s0 += *reinterpret_cast<const v4f *>(f2b + base + i * step);
            s1 += *reinterpret_cast<const v4f *>(f2b + base + (i + 4) * step);
        }
        if (i < n) s0 += *reinterpret_cast<const v4f *>(f2b + base + i * step);
    }
    part[wave][lane] = s0 + s1;
    __syncthreads();
    if (wave == 0 && on) {
        const v4f t = ((part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane])) * (1.f / n);
        *reinterpret_cast<v4f *>(a.lines + ((size_t)b * (H2 + W2) + j) * C + 4 * lane) = t;
    }
}

// One 32x32x2 product per channel of a 16-byte operand load: lane (l32, h) holds B[k = h][4 l32 .. 4 l32 + 3], product
// number i takes component i, so column l32 of accumulator i is channel 4 l32 + i and a lane's four accumulators
// hold four neighbouring channels of the same rows.
__device__ __forceinline__ void mfma4(float av, v4f x, v16f (&acc)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, x[i], acc[i], 0, 0, 0);
}

// table_part[b][s][j][c] = sum over the pixels of split s of g_avg[p,j] f1[p,c].  grid (ceil(L/32), S/2, B); the
// product has rows j, columns c and runs over pixels two at a time.  Wave w owns channels [128 (w & 1), +128) and
// the split 2 blockIdx.y + (w >> 1); the operands of the next eight pixels are in flight during the products.
__global__ void __launch_bounds__(256) avg_table_partial_kernel(const GatherArgs a) {
    const int jt = blockIdx.x, b = blockIdx.z;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C, S = a.S;
    const int c0 = (wave & 1) * 128, s = 2 * blockIdx.y + (wave >> 1);
    if (c0 >= C || s >= S) return;
    const int L = H2 + W2, NL = L - a.line0, j = a.line0 + jt * 32 + l32;
    int per = (N1 + S - 1) / S;
    per += per & 1;
    const int pa = s * per, pb = min(N1, pa + per);
    const bool jok = j < L, ju = j < H2;
    const bool cok = c0 + 4 * l32 < C;
    const float *gp = ju ? a.g_u + (size_t)b * N1 * 2 * H2 + H2 + j : a.g_v + (size_t)b * N1 * 2 * W2 + W2 + (j - H2);
    const size_t gs = ju ? 2 * (size_t)H2 : 2 * (size_t)W2;
    const float *fp = a.f1 + (size_t)b * N1 * C + (cok ? c0 + 4 * l32 : 0);
    v16f acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    struct Ops { float g[4]; v4f x[4]; };
    auto load = [&](int p0, Ops &o) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = p0 + 2 * i + h;
            const bool ok = p < pb;
            const int pc = ok ? p : pa;            // pa < N1 whenever a load is issued
            o.g[i] = (ok && jok) ? gp[(size_t)pc * gs] : 0.f;
            o.x[i] = *reinterpret_cast<const v4f *>(fp + (size_t)pc * C);
        }
    };
    auto products = [&](const Ops &o) {
#pragma unroll
        for (int i = 0; i < 4; ++i) mfma4(o.g[i], o.x[i], acc);
    };
    Ops A, B;
    if (pa < pb) load(pa, A);
    for (int p0 = pa; p0 < pb; p0 += 16) {
        if (p0 + 8 < pb) load(p0 + 8, B);
        products(A);
        if (p0 + 8 < pb) {
            if (p0 + 16 < pb) load(p0 + 16, A);
            products(B);
        }
    }
    if (!cok) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int jj = jt * 32 + acc_row(r, h);   // line within the table
        if (jj < NL)
            *reinterpret_cast<v4f *>(a.table_part + (((size_t)b * S + s) * NL + jj) * C + c0 + 4 * l32) =
                (v4f){acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
    }
}

// table[b][j][:] = (sum over the splits) / (W2 for j < H2, H2 otherwise).  grid (H2+W2, B); wave w adds the splits
// w, w + 4, ... in order, lane = 4 channels, and the four sums are added in wave order.
__global__ void __launch_bounds__(256) avg_table_reduce_kernel(const GatherArgs a) {
    __shared__ v4f part[4][64];
    const int j = blockIdx.x, b = blockIdx.y, L = a.H2 + a.W2 - a.line0, C = a.C, S = a.S;   // j: line within the table
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool on = 4 * lane < C;
    v4f s0 = {0.f, 0.f, 0.f, 0.f};
    if (on)
        for (int i = wave; i < S; i += 4) s0 += *reinterpret_cast<const v4f *>(a.table_part + (((size_t)b * S + i) * L + j) * C + 4 * lane);
    part[wave][lane] = s0;
    __syncthreads();
    if (wave == 0 && on) {
        const float scale = a.line0 + j < a.H2 ? 1.f / a.W2 : 1.f / a.H2;
        *reinterpret_cast<v4f *>(a.table + ((size_t)b * L + j) * C + 4 * lane) =
            ((part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane])) * scale;
    }
}

// d1[p][c] = sum_j g_avg[p,j] lines[j][c]: rows p, columns c, over the H2 + W2 lines two at a time.  grid
// (ceil(N1/32), B); the tile of gradients goes through LDS, JCHUNK lines at a time.
constexpr int ROWS_NS = 4;
__global__ void __launch_bounds__(256) df1_avg_rows_kernel(const GatherArgs a) {
    __shared__ float gsm[32][JCHUNK + 1];
    const int p0 = blockIdx.x * 32, b = blockIdx.y;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C, L = H2 + W2;
    const int c0 = wave * 64;
    const bool wave_on = c0 < C;
    const bool ok0 = c0 + l32 < C, ok1 = c0 + 32 + l32 < C;
    const float *rp0 = a.lines + (size_t)b * L * C + (ok0 ? c0 + l32 : 0);
    const float *rp1 = a.lines + (size_t)b * L * C + (ok1 ? c0 + 32 + l32 : 0);
    v16f acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.f; acc1[r] = 0.f; }
    for (int jc = 0; jc < L; jc += JCHUNK) {
        const int nj = min(JCHUNK, L - jc);
        if (jc) __syncthreads();
        {   // thread t holds line jc + t of all 32 pixels: the 32 loads are issued before the first is stored
            // (one after the other, a load and its store per pixel, they took 11 of the kernel's 38 us)
            static_assert(JCHUNK == 256, "one line per thread");
            const int jl = threadIdx.x, j = jc + jl;
            const bool ju = j < H2;
            const float *gp = ju ? a.g_u + ((size_t)b * N1 * 2 + 1) * H2 + j : a.g_v + ((size_t)b * N1 * 2 + 1) * W2 + (j - H2);
            const size_t gs = ju ? 2 * (size_t)H2 : 2 * (size_t)W2;
            float g[32];
#pragma unroll
            for (int px = 0; px < 32; ++px) g[px] = (p0 + px < N1 && jl < nj) ? gp[(size_t)(p0 + px) * gs] : 0.f;
#pragma unroll
            for (int px = 0; px < 32; ++px) gsm[px][jl] = g[px];
        }
        __syncthreads();
        if (wave_on) {   // a ring of ROWS_NS steps of eight lines: operands fetched ROWS_NS - 1 steps ahead of their products
            struct Ops { float ga[4], x0[4], x1[4]; };
            auto load = [&](int j0, Ops &o) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int jl = j0 + 2 * i + h;               // < JCHUNK; entries from nj on are zero
                    const int jr = jl < nj ? jc + jl : 0;
                    o.ga[i] = gsm[l32][jl];
                    o.x0[i] = rp0[(size_t)jr * C];
                    o.x1[i] = rp1[(size_t)jr * C];
                }
            };
            auto products = [&](const Ops &o) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.ga[i], o.x0[i], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.ga[i], o.x1[i], acc1, 0, 0, 0);
                }
            };
            Ops ring[ROWS_NS];
#pragma unroll
            for (int st = 0; st < ROWS_NS; ++st)
                if (8 * st < nj) load(8 * st, ring[st]);
            for (int j0 = 0; j0 < nj; j0 += 8 * ROWS_NS) {
#pragma unroll
                for (int st = 0; st < ROWS_NS; ++st)
                    if (j0 + 8 * st < nj) {
                        products(ring[st]);
                        if (j0 + 8 * (st + ROWS_NS) < nj) load(j0 + 8 * (st + ROWS_NS), ring[st]);
                    }
            }
        }
    }
    if (!wave_on) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int p = p0 + acc_row(r, h);
        if (p < N1) {
            float *dst = a.d1 + ((size_t)b * N1 + p) * C + c0 + l32;
            if (ok0) dst[0] = acc0[r];
            if (ok1) dst[32] = acc1[r];
        }
    }
}

// d1[p][:] += sum_u g_u[p,0,u] f2[(u, am_u[p,u]),:] + sum_v g_v[p,0,v] f2[(am_v[p,v], v),:].  One wave per pixel,
// lane = 4 channels; grid (ceil(N1/4), B).  Runs after df1_avg_rows_kernel on the same stream.
__global__ void __launch_bounds__(256) df1_max_gather_kernel(const GatherArgs a) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int N1 = a.N1, H2 = a.H2, W2 = a.W2, C = a.C;
    const int p = blockIdx.x * 4 + wave, b = blockIdx.y;
    if (p >= N1) return;
    const size_t pp = (size_t)b * N1 + p;
    const bool on = 4 * lane < C;
    const float *f2b = a.f2 + (size_t)b * H2 * W2 * C + (on ? 4 * lane : 0);
    v4f acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int part = 0; part < 2; ++part) {
        const int L = part ? W2 : H2, R = part ? H2 : W2;   // R: range of a valid index
        const int *am = part ? a.am_v + pp * W2 : a.am_u + pp * H2;
        const float *g = part ? a.g_v + pp * 2 * W2 : a.g_u + pp * 2 * H2;
        for (int j0 = 0; j0 < L; j0 += 64) {
            const int j = j0 + lane;
            const int idx = j < L ? am[j] : -1;
            const bool ok = (unsigned)idx < (unsigned)R;
            const float gm = ok ? g[j] : 0.f;
            const int off = ok ? (part ? idx * W2 + j : j * W2 + idx) * C : 0;   // N2 * C < 2^31 is checked on the host
            const int n = min(64, L - j0);
            for (int i0 = 0; i0 < n; i0 += NB) {
                v4f r[NB];
                int gi[NB];
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int ii = (i0 + i) & 63;     // lanes beyond n hold offset 0 and gradient 0
                    const int o = __builtin_amdgcn_readlane(off, ii);
                    gi[i] = __builtin_amdgcn_readlane(__float_as_int(gm), ii);
                    r[i] = *reinterpret_cast<const v4f *>(f2b + o);
                }
#pragma unroll
                for (int i = 0; i < NB; ++i) acc[i & 3] += __int_as_float(gi[i]) * r[i];
            }
        }
    }
    if (on) {
        v4f *dst = reinterpret_cast<v4f *>(a.d1 + pp * C + 4 * lane);
        *dst = *dst + ((acc[0] + acc[1]) + (acc[2] + acc[3]));
    }
}

// d2[(u,v)][:] = sum over the pixels that chose (u,v) in either direction + the two table lines.  One wave per
// (u,v), lane = 4 channels; grid (ceil(N2/4), B).  One launch covers the pixels [pa, pb) (multiples of SCAN): all but
// the first add to what d2 holds, the last adds the table lines (which may come from another stream in the meantime).
// The launches follow each other on one stream, so the rows of fmap1 that the whole grid fetches at any time come
// from one slice of a few MB, which the L2 caches hold; over all pixels at once they do not (measured at B=2, 55x128:
// 1.7 GB of L2 misses for 2.6 GB of rows, at 7 TB/s).
__global__ void __launch_bounds__(256) df2_gather_kernel(const GatherArgs a, int pa, int pb) {
    __shared__ int queue[4][QCAP];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int N1 = a.N1, N1p = a.N1p, H2 = a.H2, W2 = a.W2, C = a.C;
    const int N2 = H2 * W2;
    const int q = blockIdx.x * 4 + wave, b = blockIdx.y;
    if (q >= N2) return;
    const int u = q / W2, v = q - u * W2;
    const bool on = 4 * lane < C;
    const float *f1b = a.f1 + (size_t)b * N1 * C + (on ? 4 * lane : 0);
    int *qu = queue[wave];
    v4f acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int part = 0; part < 2; ++part) {
        const int *col = part ? a.amT_v + ((size_t)b * W2 + v) * N1p : a.amT_u + ((size_t)b * H2 + u) * N1p;
        const int tgt = part ? u : v;
        const float *g = part ? a.g_v + (size_t)b * N1 * 2 * W2 + v : a.g_u + (size_t)b * N1 * 2 * H2 + u;
        const size_t gs = part ? 2 * (size_t)W2 : 2 * (size_t)H2;
        int qn = 0;
        auto drain = [&](int at, int n) {   // n (<= 64) entries of the queue from position at
            const int pl = lane < n ? qu[at + lane] : 0;
            const float gl = lane < n ? g[(size_t)pl * gs] : 0.f;
            for (int i0 = 0; i0 < n; i0 += NB) {
                v4f r[NB];
                int gi[NB];
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    const int ii = (i0 + i) & 63;     // lanes beyond n hold pixel 0 and gradient 0
                    const int pi = __builtin_amdgcn_readlane(pl, ii);
                    gi[i] = __builtin_amdgcn_readlane(__float_as_int(gl), ii);
                    r[i] = *reinterpret_cast<const v4f *>(f1b + (size_t)pi * C);
                }
#pragma unroll
                for (int i = 0; i < NB; ++i) acc[i & 3] += __int_as_float(gi[i]) * r[i];
            }
        };
        v4i nxt = *reinterpret_cast<const v4i *>(col + pa + 4 * lane);
        for (int p0 = pa; p0 < pb; p0 += SCAN) {
            const v4i idx = nxt;
            if (p0 + SCAN < pb) nxt = *reinterpret_cast<const v4i *>(col + p0 + SCAN + 4 * lane);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool hit = idx[i] == tgt;
                const unsigned long long mask = __ballot(hit);
                if (mask) {
                    const int rank = __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
                    if (hit) qu[qn + rank] = p0 + 4 * lane + i;
                    qn += __builtin_popcountll(mask);
                }
            }
            if (qn >= 64) {   // qn < 64 before the step, at most 63 + SCAN after it
                wave_sync_lds();
                int done = 0;
                while (qn - done >= 64) {
                    drain(done, 64);
                    done += 64;
                }
                const int rest = qn - done;
                const int t = lane < rest ? qu[done + lane] : 0;
                wave_sync_lds();
                if (lane < rest) qu[lane] = t;
                qn = rest;
            }
        }
        wave_sync_lds();
        if (qn > 0) drain(0, qn);
        wave_sync_lds();
    }
    if (on) {
        const float *tb = a.table + (size_t)b * (H2 + W2) * C + 4 * lane;
        v4f r = (acc[0] + acc[1]) + (acc[2] + acc[3]);
        v4f *dst = reinterpret_cast<v4f *>(a.d2 + ((size_t)b * N2 + q) * C + 4 * lane);
        if (pa != 0) r += *dst;
        if (pb == N1p) r += *reinterpret_cast<const v4f *>(tb + (size_t)u * C) + *reinterpret_cast<const v4f *>(tb + (size_t)(H2 + v) * C);
        *dst = r;
    }
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

int table_splits(int B, int N1, int lines) {
    const int jt = (lines + 31) / 32;
    int S = (512 + jt * B - 1) / (jt * B);
    const int cap = N1 / 64 > 1 ? N1 / 64 : 1;
    if (S > cap) S = cap;
    if (S > 64) S = 64;
    return S < 2 ? 2 : (S + 1) & ~1;   // two splits per workgroup of avg_table_partial_kernel
}

struct Layout {
    size_t off_amT_u, off_amT_v, off_lines, off_table, off_part, total;
    int N1p, S;
};
Layout layout(int B, int N1, int H2, int W2, int C) {
    Layout l;
    l.N1p = (N1 + SCAN - 1) / SCAN * SCAN;
    l.S = table_splits(B, N1, H2 + W2);
    const size_t L = (size_t)H2 + W2;
    size_t o = 0;
    l.off_amT_u = o; o += align256((size_t)B * H2 * l.N1p * 4);
    l.off_amT_v = o; o += align256((size_t)B * W2 * l.N1p * 4);
    l.off_lines = o; o += align256((size_t)B * L * C * 4);
    l.off_table = o; o += align256((size_t)B * L * C * 4);
    l.off_part = o; o += align256((size_t)B * l.S * L * C * 4);
    l.total = o;
    return l;
}

struct Prof {
    void *t;
    Prof(const char *name, hipStream_t s) : t(sepcorr_prof_begin(name, s)) {}
    ~Prof() { sepcorr_prof_end(t); }
};

}  // namespace

int sepcorr_gather_backward_eligible(int B, int H1, int W1, int H2, int W2, int C) {
    const size_t lim = (size_t)1 << 31;
    return C % 4 == 0 && C <= 256 && B <= 65535 && H2 + W2 <= 65535 && (size_t)H2 * W2 * C < lim && (size_t)H1 * W1 * C < lim &&
           (size_t)H1 * W1 + SCAN < lim;
}

size_t sepcorr_gather_backward_bytes(int B, int H1, int W1, int H2, int W2, int C) {
    return layout(B, H1 * W1, H2, W2, C).total;
}

int sepcorr_gather_backward(const float *f1, const float *f2, const int32_t *am_u, const int32_t *am_v, const float *g_u,
                            const float *g_v, float *d_f1, float *d_f2, int B, int H1, int W1, int H2, int W2, int C, void *ws,
                            void *stream_f1, void *stream_f2, void *stream_table, void *table_event) {
    const Layout l = layout(B, H1 * W1, H2, W2, C);
    char *w = static_cast<char *>(ws);
    GatherArgs a;
    a.f1 = f1; a.f2 = f2; a.g_u = g_u; a.g_v = g_v; a.am_u = am_u; a.am_v = am_v; a.d1 = d_f1; a.d2 = d_f2;
    a.amT_u = reinterpret_cast<int *>(w + l.off_amT_u);
    a.amT_v = reinterpret_cast<int *>(w + l.off_amT_v);
    a.lines = reinterpret_cast<float *>(w + l.off_lines);
    a.table = reinterpret_cast<float *>(w + l.off_table);
    a.table_part = reinterpret_cast<float *>(w + l.off_part);
    a.B = B; a.N1 = H1 * W1; a.N1p = l.N1p; a.H2 = H2; a.W2 = W2; a.C = C; a.S = l.S;
    a.line0 = 0;
    const int L = H2 + W2, N1 = a.N1, N2 = H2 * W2;
    hipStream_t s1 = static_cast<hipStream_t>(stream_f1), s2 = static_cast<hipStream_t>(stream_f2);
    hipStream_t s3 = static_cast<hipStream_t>(stream_table);
    hipEvent_t ev = static_cast<hipEvent_t>(table_event);
    if (ev == nullptr) s3 = s2;   // no way to order the table before the last slice across streams
    const dim3 blk(256);
    {   // d_f1: line means of fmap2, the product with the average gradients, then the rows the maxima chose
        Prof ps("df1_maxavg_gather", s1);
        hipLaunchKernelGGL(fmap2_line_means_kernel, dim3(L, B), blk, 0, s1, a);
        hipLaunchKernelGGL(df1_avg_rows_kernel, dim3((N1 + 31) / 32, B), blk, 0, s1, a);
        hipLaunchKernelGGL(df1_max_gather_kernel, dim3((N1 + 3) / 4, B), blk, 0, s1, a);
    }
    {   // the table of the average gradients: needed by the last slice of the scan only
        Prof ps("df2_maxavg_table", s3);
        hipLaunchKernelGGL(avg_table_partial_kernel, dim3((L + 31) / 32, l.S / 2, B), blk, 0, s3, a);
        hipLaunchKernelGGL(avg_table_reduce_kernel, dim3(L, B), blk, 0, s3, a);
    }
    if (s3 != s2 && hipEventRecord(ev, s3) != hipSuccess) return sepcorr_set_error(SEPCORR_ELAUNCH, "sepcorr: max/avg backward (gather): event record failed");
    {   // d_f2: transposed argmax, then the scan slice by slice
        Prof ps("df2_maxavg_gather", s2);
        hipLaunchKernelGGL(argmax_columns_kernel, dim3(l.N1p / 64, 2, B), blk, 0, s2, a);
        // slices of about 1.75 MB of fmap1 per batch entry (measured best at 3 MB and 7 MB of features per entry)
        const int steps = l.N1p / SCAN;
        int slices = (int)(((size_t)N1 * C * 4 + (7u << 17)) / (7u << 18));
        slices = slices < 1 ? 1 : slices > steps ? steps : slices;
        const int per = (steps + slices - 1) / slices * SCAN;
        for (int pa = 0; pa < l.N1p; pa += per) {
            const bool last = pa + per >= l.N1p;
            if (last && s3 != s2 && hipStreamWaitEvent(s2, ev, 0) != hipSuccess)
                return sepcorr_set_error(SEPCORR_ELAUNCH, "sepcorr: max/avg backward (gather): event wait failed");
            hipLaunchKernelGGL(df2_gather_kernel, dim3((N2 + 3) / 4, B), blk, 0, s2, a, pa, last ? l.N1p : pa + per);
        }
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[200];
        snprintf(msg, sizeof(msg), "sepcorr: max/avg backward (gather): %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}

// The table of the average gradients of g_v alone, for a d_f2 kernel that leaves that term out:
//   table[b][v][c] = (1 / H2) sum_p g_v[p,1,v] f1[p,c]
// `part` holds sepcorr_avg_table_v_part_bytes() bytes of split sums.
int sepcorr_avg_table_v_eligible(int B, int H1, int W1, int H2, int W2, int C) {
    return sepcorr_gather_backward_eligible(B, H1, W1, H2, W2, C);
}

size_t sepcorr_avg_table_v_part_bytes(int B, int H1, int W1, int W2, int C) {
    return align256((size_t)B * table_splits(B, H1 * W1, W2) * W2 * C * 4);
}

int sepcorr_avg_table_v(const float *f1, const float *g_v, float *table, float *part, int B, int H1, int W1, int H2, int W2, int C,
                        void *stream) {
    GatherArgs a = {};
    a.f1 = f1; a.g_u = g_v; a.g_v = g_v;   // (lines below H2 are not computed: g_u is never read)
    a.table = table; a.table_part = part;
    a.B = B; a.N1 = H1 * W1; a.H2 = H2; a.W2 = W2; a.C = C; a.S = table_splits(B, H1 * W1, W2);
    a.line0 = H2;
    hipStream_t s = static_cast<hipStream_t>(stream);
    Prof ps("df2_avg_table", s);
    hipLaunchKernelGGL(avg_table_partial_kernel, dim3((W2 + 31) / 32, a.S / 2, B), dim3(256), 0, s, a);
    hipLaunchKernelGGL(avg_table_reduce_kernel, dim3(W2, B), dim3(256), 0, s, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char msg[200];
        snprintf(msg, sizeof(msg), "sepcorr: table of average gradients: %s", hipGetErrorString(e));
        return sepcorr_set_error(SEPCORR_ELAUNCH, msg);
    }
    return SEPCORR_OK;
}
