// Max pooling with argmax, and its pullback, for gfx950.  HBM-bound.
//
// Planes are independent, so the (n,c) axis is flattened.  A workgroup owns a
// run of whole planes: it stages them into LDS as one flat, contiguous,
// coalesced read (the run is contiguous in memory whatever H*W is), computes
// the outputs from LDS, and writes them as one flat contiguous run.
//
// Forward: window scan in (h, w) order, strict '>', from -FLT_MAX; mask is the
// in-plane index h*W + w.  Pullback: gather form of the reference's scatter --
// each input cell visits the windows that cover it in ascending (ph, pw) and
// adds top_diff where the mask names it, which reproduces the sequential add
// order bit-for-bit without atomics.
#include "common.h"
#include <algorithm>
#include <cfloat>

namespace cgt_amd {

constexpr int kPoolThreads = 256;

// floor(n / d) for 0 <= n < 2^21 with rcp = 1.0f / d: (n + 0.5) / d is at least
// 0.5/d away from every integer, more than the float rounding error.
__device__ __forceinline__ int fastdiv(int n, float rcp) { return (int)(((float)n + 0.5f) * rcp); }

// planes_per_wg planes per workgroup; LDS holds their inputs; one thread per
// pooled cell.
template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_fwd_kernel(
    G g, const float* __restrict__ bottom, float* __restrict__ top, int* __restrict__ mask,
    long nplanes, int H, int W, int PH, int PW, int planes_per_wg) {
    extern __shared__ float tile[];
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const int HW = H * W, PP = PH * PW;
    const float* src = bottom + p0 * HW;
    const int nin = np * HW;
    for (int base = threadIdx.x; base < nin; base += kPoolThreads * 8) {   // 8 loads in flight per thread
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (base + u * kPoolThreads < nin) v[u] = src[base + u * kPoolThreads];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (base + u * kPoolThreads < nin) tile[base + u * kPoolThreads] = v[u];
    }
    __syncthreads();

    float* tdst = top + p0 * PP;
    int* mdst = mask + p0 * PP;
    const int nout = np * PP;
    const float rPP = 1.0f / PP, rPW = 1.0f / PW;
    for (int o = threadIdx.x; o < nout; o += kPoolThreads) {
        const int pl = fastdiv(o, rPP), r = o - pl * PP;
        const int y = fastdiv(r, rPW), x = r - y * PW;
        int hs = y * g.sh() - g.ph(), ws = x * g.sw() - g.pw();
        const int he = min(hs + g.kh(), H), we = min(ws + g.kw(), W);
        hs = max(hs, 0);
        ws = max(ws, 0);
        const float* pt = tile + pl * HW;
        float best = -FLT_MAX;
        int arg = -1;
        for (int h = hs; h < he; ++h)
            for (int w = ws; w < we; ++w) {
                const float v = pt[h * W + w];
                if (v > best) {
                    best = v;
                    arg = h * W + w;
                }
            }
        tdst[o] = best;
        mdst[o] = arg;
    }
}

// Plane too large for LDS: read through the cache hierarchy.
template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_fwd_direct_kernel(
    G g, const float* __restrict__ bottom, float* __restrict__ top, int* __restrict__ mask,
    long total, int H, int W, int PH, int PW) {
    const long PP = (long)PH * PW;
    for (long o = (long)blockIdx.x * blockDim.x + threadIdx.x; o < total;
         o += (long)gridDim.x * blockDim.x) {
        const long pl = o / PP;
        const int r = (int)(o - pl * PP);
        const int y = r / PW, x = r - y * PW;
        int hs = y * g.sh() - g.ph(), ws = x * g.sw() - g.pw();
        const int he = min(hs + g.kh(), H), we = min(ws + g.kw(), W);
        hs = max(hs, 0);
        ws = max(ws, 0);
        const float* pt = bottom + pl * H * W;
        float best = -FLT_MAX;
        int arg = -1;
        for (int h = hs; h < he; ++h)
            for (int w = ws; w < we; ++w) {
                const float v = pt[h * W + w];
                if (v > best) {
                    best = v;
                    arg = h * W + w;
                }
            }
        top[o] = best;
        mask[o] = arg;
    }
}

__device__ __forceinline__ int floordiv(int a, int b) {  // b > 0
    int q = a / b;
    return (a % b != 0 && a < 0) ? q - 1 : q;
}

// LDS holds mask and top_diff of the workgroup's planes; one thread per input cell.
template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_kernel(
    G g, const int* __restrict__ mask, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, long nplanes, int H, int W, int PH, int PW,
    int planes_per_wg) {
    extern __shared__ float tile[];
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const int HW = H * W, PP = PH * PW;
    const int nout = np * PP;
    float* td = tile;
    int* mk = reinterpret_cast<int*>(tile + planes_per_wg * PP);
    for (int base = threadIdx.x; base < nout; base += kPoolThreads * 4) {  // 8 loads in flight per thread
        float v[4];
        int k[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (base + u * kPoolThreads < nout) {
                v[u] = top_diff[p0 * PP + base + u * kPoolThreads];
                k[u] = mask[p0 * PP + base + u * kPoolThreads];
            }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (base + u * kPoolThreads < nout) {
                td[base + u * kPoolThreads] = v[u];
                mk[base + u * kPoolThreads] = k[u];
            }
    }
    __syncthreads();

    float* dst = bottom_diff + p0 * HW;
    const int nin = np * HW;
    const float rHW = 1.0f / HW, rW = 1.0f / W;
    for (int i = threadIdx.x; i < nin; i += kPoolThreads) {
        const int pl = fastdiv(i, rHW), cell = i - pl * HW;
        const int h = fastdiv(cell, rW), w = cell - h * W;
        // windows covering (h, w): ph*sh - pad <= h < ph*sh - pad + kh
        const int y0 = max(0, floordiv(h + g.ph() - g.kh(), g.sh()) + 1), y1 = min(PH - 1, (h + g.ph()) / g.sh());
        const int x0 = max(0, floordiv(w + g.pw() - g.kw(), g.sw()) + 1), x1 = min(PW - 1, (w + g.pw()) / g.sw());
        const float* tdp = td + pl * PP;
        const int* mkp = mk + pl * PP;
        float acc = 0.0f;
        for (int y = y0; y <= y1; ++y)
            for (int x = x0; x <= x1; ++x) {
                const int o = y * PW + x;
                if (mkp[o] == cell) acc += tdp[o];
            }
        dst[i] = acc;
    }
}

constexpr int cfloordiv(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }   // b > 0
constexpr int cceildiv(int a, int b) { return -cfloordiv(-a, b); }

// Pullback for geometries known at compile time.  A thread owns one stride-sized
// block of input cells (rows by*SH.., columns bx*SW..).  Relative to (by, bx) the
// windows that can cover a cell of the block sit at offsets fixed by the
// geometry, so the thread loads that small neighbourhood of (mask, top_diff)
// once, straight from global memory (consecutive threads read consecutive
// pooled cells), and every cell adds the windows that name it, in ascending
// (ph, pw) as the reference's sequential scatter does.  No division per cell,
// no LDS, no barrier.
// XB = 2 (stride 2 along w, W % 4 == 0, 16-byte aligned output): a thread owns two blocks
// side by side and writes each of its rows as one 16-byte unit.
template <class G, int XB>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_wide_kernel(
    G, const int* __restrict__ mask, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, long nplanes, int H, int W, int PH, int PW, int BH, int BW2,
    int planes_per_wg, int nt) {
    constexpr int KH = G::kKH, KW = G::kKW, PDH = G::kPH, PDW = G::kPW, SH = G::kSH, SW = G::kSW;
    static_assert(SW * XB == 4, "a thread's row is one 16-byte unit");
    constexpr int DY0 = cceildiv(PDH - KH + 1, SH), DY1 = cfloordiv(SH - 1 + PDH, SH);
    constexpr int DX0 = cceildiv(PDW - KW + 1, SW), DX1 = cfloordiv(SW - 1 + PDW, SW) + (XB - 1);
    constexpr int NY = DY1 - DY0 + 1, NX = DX1 - DX0 + 1;
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const int HW = H * W, PP = PH * PW, per_plane = BH * BW2;
    const int n = np * per_plane;
    const float rPer = 1.0f / per_plane, rBW = 1.0f / BW2;
    for (int j = threadIdx.x; j < n; j += kPoolThreads) {
        const int pl = fastdiv(j, rPer), r = j - pl * per_plane;
        const int by = fastdiv(r, rBW), bx = (r - by * BW2) * XB;      // first of the thread's blocks
        const int* mk = mask + (p0 + pl) * PP;
        const float* td = top_diff + (p0 + pl) * PP;
        int mv[NY][NX];
        float tv[NY][NX];
#pragma unroll
        for (int dy = 0; dy < NY; ++dy)
#pragma unroll
            for (int dx = 0; dx < NX; ++dx) {
                const int y = by + DY0 + dy, x = bx + DX0 + dx;
                const bool ok = y >= 0 && y < PH && x >= 0 && x < PW;
                mv[dy][dx] = ok ? mk[y * PW + x] : -1;
                tv[dy][dx] = ok ? td[y * PW + x] : 0.0f;
            }
        float* dst = bottom_diff + (p0 + pl) * HW;
#pragma unroll
        for (int i = 0; i < SH; ++i) {
            const int h = by * SH + i;
            if (h >= H) break;
            float out[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int xb = jj / SW, jc = jj % SW;             // block of the pair, cell in the block
                const int cell = h * W + bx * SW + jj;
                float acc = 0.0f;
#pragma unroll
                for (int dy = 0; dy < NY; ++dy)
#pragma unroll
                    for (int dx = 0; dx < NX; ++dx) {
                        const bool covers = DY0 + dy >= cceildiv(i + PDH - KH + 1, SH) && DY0 + dy <= cfloordiv(i + PDH, SH) &&
                                            DX0 + dx - xb >= cceildiv(jc + PDW - KW + 1, SW) && DX0 + dx - xb <= cfloordiv(jc + PDW, SW);
                        if (covers) acc = (mv[dy][dx] == cell) ? acc + tv[dy][dx] : acc;
                    }
                out[jj] = acc;
            }
            float* row = dst + h * W + bx * SW;
            if (nt) stream_store4(row, out[0], out[1], out[2], out[3]);
            else *reinterpret_cast<float4*>(row) = make_float4(out[0], out[1], out[2], out[3]);
        }
    }
}

template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_block_kernel(
    G, const int* __restrict__ mask, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, long nplanes, int H, int W, int PH, int PW, int BH, int BW,
    int planes_per_wg, int vec2) {
    constexpr int KH = G::kKH, KW = G::kKW, PDH = G::kPH, PDW = G::kPW, SH = G::kSH, SW = G::kSW;
    constexpr int DY0 = cceildiv(PDH - KH + 1, SH), DY1 = cfloordiv(SH - 1 + PDH, SH);
    constexpr int DX0 = cceildiv(PDW - KW + 1, SW), DX1 = cfloordiv(SW - 1 + PDW, SW);
    constexpr int NY = DY1 - DY0 + 1, NX = DX1 - DX0 + 1;
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const int HW = H * W, PP = PH * PW, per_plane = BH * BW;
    const int n = np * per_plane;
    const float rPer = 1.0f / per_plane, rBW = 1.0f / BW;
    for (int j = threadIdx.x; j < n; j += kPoolThreads) {
        const int pl = fastdiv(j, rPer), r = j - pl * per_plane;
        const int by = fastdiv(r, rBW), bx = r - by * BW;
        const int* mk = mask + (p0 + pl) * PP;
        const float* td = top_diff + (p0 + pl) * PP;
        int mv[NY][NX];
        float tv[NY][NX];
#pragma unroll
        for (int dy = 0; dy < NY; ++dy)
#pragma unroll
            for (int dx = 0; dx < NX; ++dx) {
                const int y = by + DY0 + dy, x = bx + DX0 + dx;
                const bool ok = y >= 0 && y < PH && x >= 0 && x < PW;
                mv[dy][dx] = ok ? mk[y * PW + x] : -1;
                tv[dy][dx] = ok ? td[y * PW + x] : 0.0f;
            }
        float* dst = bottom_diff + (p0 + pl) * HW;
#pragma unroll
        for (int i = 0; i < SH; ++i) {
            const int h = by * SH + i;
            if (h >= H) break;
            float out[SW];
#pragma unroll
            for (int jj = 0; jj < SW; ++jj) {
                const int cell = h * W + bx * SW + jj;
                float acc = 0.0f;
#pragma unroll
                for (int dy = 0; dy < NY; ++dy)
#pragma unroll
                    for (int dx = 0; dx < NX; ++dx) {
                        // does window offset (dy, dx) cover cell (i, jj) of the block?
                        const bool covers = DY0 + dy >= cceildiv(i + PDH - KH + 1, SH) && DY0 + dy <= cfloordiv(i + PDH, SH) &&
                                            DX0 + dx >= cceildiv(jj + PDW - KW + 1, SW) && DX0 + dx <= cfloordiv(jj + PDW, SW);
                        if (covers) acc = (mv[dy][dx] == cell) ? acc + tv[dy][dx] : acc;
                    }
                out[jj] = acc;
            }
            float* row = dst + h * W + bx * SW;
            if (SW == 2 && vec2) {
                *reinterpret_cast<float2*>(row) = make_float2(out[0], out[SW - 1]);
            } else {
#pragma unroll
                for (int jj = 0; jj < SW; ++jj)
                    if (bx * SW + jj < W) row[jj] = out[jj];
            }
        }
    }
}

// The same block decomposition with both sides of the memory traffic made linear.  The
// block kernel above keeps 8 bytes of unread input in flight per thread (its neighbourhood
// loads overlap those of its neighbours four times) and writes 4-byte pieces at odd
// alignments; on planes of 55 x 55 it moves 2.7 TB/s from memory (its reads alone take as
// long as its writes alone, and the two do not overlap).  Here a workgroup (1) copies the
// (mask, top_diff) of its run of planes into LDS with aligned 16-byte loads, all in flight
// at once, (2) lets every thread form its blocks' cells from LDS -- same candidates, same
// ascending (ph, pw) order, hence the same bits -- into an LDS image of the output run laid
// out at the run's own 16-byte phase, and (3) writes that image as aligned 16-byte units
// (the few floats before the first and after the last whole unit one by one).
template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_linear_kernel(
    G, const int* __restrict__ mask, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, long nplanes, int H, int W, int PH, int PW, int BH, int BW,
    int planes_per_wg, int in_floats, int nt) {
    constexpr int KH = G::kKH, KW = G::kKW, PDH = G::kPH, PDW = G::kPW, SH = G::kSH, SW = G::kSW;
    constexpr int DY0 = cceildiv(PDH - KH + 1, SH), DY1 = cfloordiv(SH - 1 + PDH, SH);
    constexpr int DX0 = cceildiv(PDW - KW + 1, SW), DX1 = cfloordiv(SW - 1 + PDW, SW);
    constexpr int NY = DY1 - DY0 + 1, NX = DX1 - DX0 + 1;
    extern __shared__ float tile[];
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const int HW = H * W, PP = PH * PW, per_plane = BH * BW;
    // LDS: td [in_floats], mk [in_floats], out [rest]; every part a multiple of 4 floats
    float* td = tile;
    int* mk = reinterpret_cast<int*>(tile + in_floats);
    float* outp = tile + 2 * in_floats;

    // (1) the input run [p0 * PP, (p0 + np) * PP) of both arrays, from the 16-byte boundary at or below its start
    const long in0 = p0 * PP, in_end = nplanes * (long)PP;
    const int iphase = (int)(in0 & 3);
    const int nin = np * PP;
    const int in_units = (iphase + nin + 3) >> 2;
    const float4* td4 = reinterpret_cast<const float4*>(top_diff + (in0 - iphase));
    const int4* mk4 = reinterpret_cast<const int4*>(mask + (in0 - iphase));
    // units that end inside the arrays are loaded four per thread before the first is parked (indices
    // past the run are clamped to its last such unit and dropped); the unit holding the arrays' last
    // floats, if it is cut, goes float by float
    const int safe_units = (int)min((long)in_units, (in_end - (in0 - iphase)) >> 2);
    for (int base = threadIdx.x; base < safe_units; base += kPoolThreads * 4) {
        float4 tv4[4];
        int4 mv4[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int u = min(base + k * kPoolThreads, safe_units - 1);
            tv4[k] = td4[u];
            mv4[k] = mk4[u];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int u = base + k * kPoolThreads;
            if (u < safe_units) {
                reinterpret_cast<float4*>(td)[u] = tv4[k];
                reinterpret_cast<int4*>(mk)[u] = mv4[k];
            }
        }
    }
    if (safe_units < in_units && threadIdx.x < 4) {
        const long g = in0 - iphase + 4L * safe_units + threadIdx.x;
        if (g < in_end) {
            td[4 * safe_units + threadIdx.x] = top_diff[g];
            mk[4 * safe_units + threadIdx.x] = mask[g];
        }
    }
    __syncthreads();

    // (2) blocks -> LDS image of the output run, at the run's phase
    const long out0 = p0 * (long)HW;
    const int ophase = (int)(out0 & 3);
    const int n = np * per_plane;
    const float rPer = 1.0f / per_plane, rBW = 1.0f / BW;
    for (int j = threadIdx.x; j < n; j += kPoolThreads) {
        const int pl = fastdiv(j, rPer), r = j - pl * per_plane;
        const int by = fastdiv(r, rBW), bx = r - by * BW;
        const int* mkp = mk + iphase + pl * PP;
        const float* tdp = td + iphase + pl * PP;
        int mv[NY][NX];
        float tv[NY][NX];
#pragma unroll
        for (int dy = 0; dy < NY; ++dy)
#pragma unroll
            for (int dx = 0; dx < NX; ++dx) {
                const int y = by + DY0 + dy, x = bx + DX0 + dx;
                const bool ok = y >= 0 && y < PH && x >= 0 && x < PW;
                const int o = ok ? y * PW + x : 0;
                const int m = mkp[o];
                const float t = tdp[o];
                mv[dy][dx] = ok ? m : -1;
                tv[dy][dx] = ok ? t : 0.0f;
            }
        float* dst = outp + ophase + pl * HW;
#pragma unroll
        for (int i = 0; i < SH; ++i) {
            const int h = by * SH + i;
            if (h >= H) break;
#pragma unroll
            for (int jj = 0; jj < SW; ++jj) {
                const int cell = h * W + bx * SW + jj;
                float acc = 0.0f;
#pragma unroll
                for (int dy = 0; dy < NY; ++dy)
#pragma unroll
                    for (int dx = 0; dx < NX; ++dx) {
                        const bool covers = DY0 + dy >= cceildiv(i + PDH - KH + 1, SH) && DY0 + dy <= cfloordiv(i + PDH, SH) &&
                                            DX0 + dx >= cceildiv(jj + PDW - KW + 1, SW) && DX0 + dx <= cfloordiv(jj + PDW, SW);
                        if (covers) acc = (mv[dy][dx] == cell) ? acc + tv[dy][dx] : acc;
                    }
                if (bx * SW + jj < W) dst[cell] = acc;
            }
        }
    }
    __syncthreads();

    // (3) the image goes out: whole units between the first and the last 16-byte boundary inside the run
    const int nout = np * HW;
    float* gbase = bottom_diff + (out0 - ophase);
    const int first = ophase ? 1 : 0, last = (ophase + nout) >> 2;      // units [first, last) lie inside the run
    for (int u = first + threadIdx.x; u < last; u += kPoolThreads) {
        const float4 v = reinterpret_cast<const float4*>(outp)[u];
        if (nt) stream_store4(gbase + 4 * u, v.x, v.y, v.z, v.w);
        else *reinterpret_cast<float4*>(gbase + 4 * u) = v;
    }
    if (threadIdx.x < 8) {
        const int e = threadIdx.x & 3;
        if (threadIdx.x < 4) {      // floats of the first unit that belong to this run
            if (ophase && e >= ophase && e < ophase + nout) gbase[e] = outp[e];
        } else {                    // floats behind the last whole unit
            const int f = 4 * last + e;
            if (last >= first && f < ophase + nout) gbase[f] = outp[f];
        }
    }
}

template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_direct_kernel(
    G g, const int* __restrict__ mask, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, long total, int H, int W, int PH, int PW) {
    const long HW = (long)H * W, PP = (long)PH * PW;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long)gridDim.x * blockDim.x) {
        const long pl = i / HW;
        const int cell = (int)(i - pl * HW);
        const int h = cell / W, w = cell - h * W;
        const int y0 = max(0, floordiv(h + g.ph() - g.kh(), g.sh()) + 1), y1 = min(PH - 1, (h + g.ph()) / g.sh());
        const int x0 = max(0, floordiv(w + g.pw() - g.kw(), g.sw()) + 1), x1 = min(PW - 1, (w + g.pw()) / g.sw());
        float acc = 0.0f;
        for (int y = y0; y <= y1; ++y)
            for (int x = x0; x <= x1; ++x) {
                const long o = pl * PP + y * PW + x;
                if (mask[o] == cell) acc += top_diff[o];
            }
        bottom_diff[i] = acc;
    }
}

// The pullback written into zero-padded planes (see PaddedPlanes): one thread per aligned
// 16-byte unit of the result.  A unit's four floats are zeros of the padding or pullback cells;
// a cell gathers the windows that cover it in ascending (ph, pw), as max_pool_bwd_kernel does,
// straight from global memory (neighbouring threads read neighbouring pooled cells).  With a
// compile-time geometry the candidate windows of a cell are a fixed-size neighbourhood: all
// their loads are issued up front, unconditionally (indices of windows that do not exist are
// clamped to 0 and their values dropped), instead of one dependent load after another.
template <class G>
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_padded_kernel(
    G g, const int* __restrict__ mask, const float* __restrict__ top_diff, const signed char* __restrict__ relu_mask,
    float* __restrict__ dst, int H, int W, int PH, int PW, PaddedPlanes lay, int units_per_plane,
    long total_units, long tail_units) {
    const float rPitch = 1.0f / (float)lay.pitch;
    const int PP = PH * PW, HW = H * W;
    const int lane = threadIdx.x & 63;
    // A wavefront takes chunks of kChunk units of one plane at a time, so the plane and with it
    // the base addresses of its mask / cotangent / output are wave-uniform (scalar registers,
    // 32-bit lane offsets) -- the kernel is bound by its index arithmetic, not by memory.
    constexpr int kChunk = 512;
    const int chunks_per_plane = (units_per_plane + kChunk - 1) / kChunk;
    const int items = (int)(total_units / units_per_plane) * chunks_per_plane;     // < 2^31: the host checks
    const int nwaves = (int)gridDim.x * (kPoolThreads / 64);
    const int wave_id = __builtin_amdgcn_readfirstlane((int)((blockIdx.x * kPoolThreads + threadIdx.x) >> 6));
    for (long t = (long)blockIdx.x * kPoolThreads + threadIdx.x; t < tail_units; t += (long)gridDim.x * kPoolThreads)
        stream_store4(dst + (total_units + t) * 4, 0.f, 0.f, 0.f, 0.f);
    for (int item = wave_id; item < items; item += nwaves) {
        const long pl = item / chunks_per_plane;
        const int chunk = item - (int)pl * chunks_per_plane;
        const int* mk = mask + pl * PP;
        const float* td = top_diff + pl * PP;
        const signed char* rmk = relu_mask ? relu_mask + pl * HW : nullptr;
        float* out = dst + pl * (long)lay.plane;
        const int uend = min(units_per_plane, (chunk + 1) * kChunk);
        for (int uu = chunk * kChunk + lane; uu < uend; uu += 64) {
            float o[4] = {0.f, 0.f, 0.f, 0.f};
            const int e0 = uu * 4;
            // element e of a plane is column (e - lead) % pitch of padded row (e - lead) / pitch;
            // shifted by one row so that it is never negative (lead <= pitch), fixed up exactly
            const int e1 = e0 - lay.lead + lay.pitch;
            int hp = fastdiv(e1, rPitch);
            int wp = e1 - hp * lay.pitch;
            if (wp < 0) { --hp; wp += lay.pitch; }
            if (wp >= lay.pitch) { ++hp; wp -= lay.pitch; }
            if constexpr (G::is_static) {
                constexpr int NY = (G::kKH + G::kSH - 1) / G::kSH, NX = (G::kKW + G::kSW - 1) / G::kSW;
                int mv[4][NY][NX], cell[4];
                float tv[4][NY][NX], rm[4];
                bool ok[4][NY][NX], inside[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int h = hp - 1 - lay.top;
                    inside[j] = h >= 0 && h < H && wp < W;
                    cell[j] = h * W + wp;
                    const int yb = floordiv(h + g.ph() - g.kh(), g.sh()) + 1, y1 = min(PH - 1, (h + g.ph()) / g.sh());
                    const int xb = floordiv(wp + g.pw() - g.kw(), g.sw()) + 1, x1 = min(PW - 1, (wp + g.pw()) / g.sw());
#pragma unroll
                    for (int dy = 0; dy < NY; ++dy)
#pragma unroll
                        for (int dx = 0; dx < NX; ++dx) {
                            const int y = yb + dy, x = xb + dx;
                            ok[j][dy][dx] = inside[j] && y >= 0 && y <= y1 && x >= 0 && x <= x1;
                            const int at = ok[j][dy][dx] ? y * PW + x : 0;
                            mv[j][dy][dx] = mk[at];
                            tv[j][dy][dx] = td[at];
                        }
                    rm[j] = (rmk && inside[j]) ? (float)rmk[cell[j]] : 1.0f;
                    if (++wp == lay.pitch) { wp = 0; ++hp; }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float acc = 0.0f;
#pragma unroll
                    for (int dy = 0; dy < NY; ++dy)
#pragma unroll
                        for (int dx = 0; dx < NX; ++dx)
                            acc = (ok[j][dy][dx] && mv[j][dy][dx] == cell[j]) ? acc + tv[j][dy][dx] : acc;
                    if (rmk) acc = rm[j] * acc;
                    o[j] = inside[j] ? acc : 0.0f;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int h = hp - 1 - lay.top;
                    if (h >= 0 && h < H && wp < W) {
                        const int cell = h * W + wp;
                        const int y0 = max(0, floordiv(h + g.ph() - g.kh(), g.sh()) + 1), y1 = min(PH - 1, (h + g.ph()) / g.sh());
                        const int x0 = max(0, floordiv(wp + g.pw() - g.kw(), g.sw()) + 1), x1 = min(PW - 1, (wp + g.pw()) / g.sw());
                        float acc = 0.0f;
                        for (int y = y0; y <= y1; ++y)
                            for (int x = x0; x <= x1; ++x) {
                                const int m = mk[y * PW + x];
                                const float t = td[y * PW + x];
                                acc = (m == cell) ? acc + t : acc;
                            }
                        if (rmk) acc = (float)rmk[cell] * acc;
                        o[j] = acc;
                    }
                    if (++wp == lay.pitch) { wp = 0; ++hp; }
                }
            }
            *reinterpret_cast<float4*>(out + e0) = make_float4(o[0], o[1], o[2], o[3]);
        }
    }
}

// Windows that do not overlap (kernel <= stride): a cell has at most one addend, so the pullback
// is a scatter with no order to keep.  A workgroup builds its planes in LDS -- zeros, then every
// window's cotangent at the cell its mask names (0 + g, times the rectify mask: the bits the
// gather form produces) -- and writes them out as one contiguous run of 16-byte units.  The
// index arithmetic is per window, not per float of the result.
__global__ __launch_bounds__(kPoolThreads) void max_pool_bwd_padded_scatter_kernel(
    const int* __restrict__ mask, const float* __restrict__ top_diff, const signed char* __restrict__ relu_mask,
    float* __restrict__ dst, long nplanes, int HW, int W, int PP, PaddedPlanes lay, int planes_per_wg, long tail_units) {
    extern __shared__ float tile[];
    const long p0 = (long)blockIdx.x * planes_per_wg;
    const long left = nplanes - p0;
    const int np = left < planes_per_wg ? (int)left : planes_per_wg;
    const long total_units = nplanes * (long)(lay.plane / 4);
    for (long t = (long)blockIdx.x * kPoolThreads + threadIdx.x; t < tail_units; t += (long)gridDim.x * kPoolThreads)
        stream_store4(dst + (total_units + t) * 4, 0.f, 0.f, 0.f, 0.f);
    const int nunits = np * (lay.plane / 4);
    float4* t4 = reinterpret_cast<float4*>(tile);
    for (int u = threadIdx.x; u < nunits; u += kPoolThreads) t4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    const int nwin = np * PP;
    const float rPP = 1.0f / PP, rW = 1.0f / W;
    const int* mk = mask + p0 * PP;
    const float* td = top_diff + p0 * PP;
    for (int base = threadIdx.x; base < nwin; base += kPoolThreads * 4) {
        int m[4], pl[4];
        float g[4], r[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int o = base + u * kPoolThreads;
            m[u] = -1;
            if (o < nwin) {
                m[u] = mk[o];
                g[u] = td[o];
            }
            pl[u] = fastdiv(o, rPP);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            m[u] = (unsigned)m[u] < (unsigned)HW ? m[u] : -1;     // -1: a window that saw no value
            r[u] = (relu_mask && m[u] >= 0) ? (float)relu_mask[(p0 + pl[u]) * (long)HW + m[u]] : 1.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (m[u] >= 0) {
                const int h = fastdiv(m[u], rW), w = m[u] - h * W;
                float v = 0.0f + g[u];
                if (relu_mask) v = r[u] * v;
                tile[pl[u] * lay.plane + lay.lead + (h + lay.top) * lay.pitch + w] = v;
            }
    }
    __syncthreads();
    float4* out = reinterpret_cast<float4*>(dst + p0 * (long)lay.plane);
    for (int u = threadIdx.x; u < nunits; u += kPoolThreads) out[u] = t4[u];
}

static int check_pool(const char* what, long N, long C, long H, long W, int kh, int kw, int ph,
                      int pw, int sh, int sw, long PH, long PW) {
    CGT_ARG_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0 && PH >= 0 && PW >= 0, "%s: negative shape", what);
    CGT_ARG_CHECK(kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0,
                  "%s: bad geometry k=(%d,%d) p=(%d,%d) s=(%d,%d)", what, kh, kw, ph, pw, sh, sw);
    CGT_ARG_CHECK(H * W < (1L << 31) && PH * PW < (1L << 31), "%s: plane too large", what);
    // every window must start inside the padded image, as the op's shape rule guarantees
    CGT_ARG_CHECK(PH == 0 || (PH - 1) * sh - ph < H, "%s: PH=%ld does not fit H=%ld", what, PH, H);
    CGT_ARG_CHECK(PW == 0 || (PW - 1) * sw - pw < W, "%s: PW=%ld does not fit W=%ld", what, PW, W);
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API long cgt_amd_pool_outsize(long H, int k, int pad, int stride) {
    if (stride <= 0) return 0;
    long num = H + 2L * pad - k;
    if (num <= 0) return 0;
    return (num + stride - 1) / stride;
}

// Pool geometries compiled with constant index math: (kh, kw, ph, pw, sh, sw).
#define CGT_STATIC_POOLS(X) \
    X(2, 2, 0, 0, 2, 2)     \
    X(3, 3, 0, 0, 2, 2)     \
    X(3, 3, 1, 1, 2, 2)

namespace cgt_amd {

// The staged kernels split flat indices with fastdiv, which is exact below 2^21: they are
// taken only while a workgroup's input and output index ranges stay below that; otherwise
// the direct kernels (64-bit integer division) run.
constexpr long kFastdivLimit = 1L << 21;

// planes per workgroup of the staged forward kernel, 0: use the direct kernel
static int pool_fwd_planes_per_wg(long H, long W, long PH, long PW) {
    const long plane_bytes = H * W * (long)sizeof(float);
    if (plane_bytes > 48 * 1024) return 0;
    long ppw = std::max(1L, (16 * 1024) / std::max(1L, plane_bytes));
    ppw = std::min(ppw, (kFastdivLimit - 1) / std::max(1L, PH * PW));   // pad >= kernel: more outputs than inputs
    return ppw * H * W < kFastdivLimit && ppw >= 1 ? (int)ppw : 0;
}

// planes per workgroup of the staged generic pullback kernel, 0: use the direct kernel
static int pool_bwd_planes_per_wg(long H, long W, long PH, long PW) {
    const long out_bytes = PH * PW * 2 * (long)sizeof(float);  // top_diff + mask per plane
    if (out_bytes > 48 * 1024) return 0;
    long ppw = std::max(1L, (16 * 1024) / std::max(1L, out_bytes));
    ppw = std::min(ppw, (kFastdivLimit - 1) / std::max(1L, H * W));     // large strides: huge planes, few outputs
    return ppw >= 1 && ppw * PH * PW < kFastdivLimit ? (int)ppw : 0;
}

template <class G>
static int launch_pool_fwd(G g, const float* bottom, long nplanes, long H, long W, long PH, long PW,
                           float* top, int* mask, hipStream_t st) {
    const long plane_bytes = H * W * (long)sizeof(float);
    if (int ppw = pool_fwd_planes_per_wg(H, W, PH, PW)) {
        const long blocks = cdiv(nplanes, ppw);
        max_pool_fwd_kernel<G><<<dim3((unsigned)blocks), dim3(kPoolThreads), (size_t)ppw * plane_bytes, st>>>(
            g, bottom, top, mask, nplanes, (int)H, (int)W, (int)PH, (int)PW, ppw);
        CGT_LAUNCH_CHECK("max_pool_fwd_kernel");
    } else {
        const long total = nplanes * PH * PW;
        long blocks = std::min(cdiv(total, (long)kPoolThreads), 1L << 20);
        max_pool_fwd_direct_kernel<G><<<dim3((unsigned)blocks), dim3(kPoolThreads), 0, st>>>(
            g, bottom, top, mask, total, (int)H, (int)W, (int)PH, (int)PW);
        CGT_LAUNCH_CHECK("max_pool_fwd_direct_kernel");
    }
    return CGT_AMD_OK;
}

template <class G>
static int launch_pool_bwd(G g, const int* mask, const float* top_diff, long nplanes, long H, long W,
                           long PH, long PW, float* bottom_diff, hipStream_t st) {
    // windows that do not overlap: the scatter form, planes built in LDS and written as one run
    if (g.kh() <= g.sh() && g.kw() <= g.sw() && (H * W) % 4 == 0 && H * W * (long)sizeof(float) <= 48 * 1024 &&
        reinterpret_cast<uintptr_t>(bottom_diff) % 16 == 0) {
        const long plane_bytes = H * W * (long)sizeof(float);
        long ppw = std::max(1L, std::min((32 * 1024) / plane_bytes, nplanes / 2048));
        ppw = std::min(ppw, (kFastdivLimit - 1) / (PH * PW));
        if (ppw >= 1) {
            const PaddedPlanes lay = {0, 0, (int)W, (int)(H * W), 0};
            max_pool_bwd_padded_scatter_kernel<<<dim3((unsigned)cdiv(nplanes, ppw)), dim3(kPoolThreads), (size_t)(ppw * plane_bytes), st>>>(
                mask, top_diff, nullptr, bottom_diff, nplanes, (int)(H * W), (int)W, (int)(PH * PW), lay, (int)ppw, 0);
            CGT_LAUNCH_CHECK("max_pool_bwd_padded_scatter_kernel");
            return CGT_AMD_OK;
        }
    }
    if constexpr (G::is_static) {
        const long BH = cdiv(H, (long)G::kSH), BW = cdiv(W, (long)G::kSW);
        if (BH * BW <= (1L << 18) && H * W < (1L << 30)) {
            // a few thousand blocks per workgroup, at least one plane
            const int ppw = (int)std::max(1L, std::min(2048 / (BH * BW), cdiv(nplanes, 4096L)));
            const long blocks = cdiv(nplanes, ppw);
            if constexpr (G::kSW == 2) {
                // rows of whole 16-byte units: two blocks per thread, one 16-byte store per row.
                // Inside a conv layer's step (the output has to displace other kernels' dirty
                // lines) the VGG pullback takes 0.039 ms this way against 0.050 with 8-byte
                // stores; non-temporal 16-byte stores measured 0.042 and are slower back to back.
                if (W % 4 == 0 && reinterpret_cast<uintptr_t>(bottom_diff) % 16 == 0) {
                    const long BW2 = BW / 2;
                    const int ppw2 = (int)std::max(1L, std::min(2048 / (BH * BW2), cdiv(nplanes, 4096L)));
                    max_pool_bwd_wide_kernel<G, 2><<<dim3((unsigned)cdiv(nplanes, ppw2)), dim3(kPoolThreads), 0, st>>>(
                        g, mask, top_diff, bottom_diff, nplanes, (int)H, (int)W, (int)PH, (int)PW, (int)BH, (int)BW2, ppw2, 0);
                    CGT_LAUNCH_CHECK("max_pool_bwd_wide_kernel");
                    return CGT_AMD_OK;
                }
            }
            // Rows that are not whole 16-byte units (the AlexNet planes of 55 x 55): both sides linear
            // through LDS.  Inside the AlexNet conv1 step: 0.042 ms against the block kernel's 0.082
            // (one plane per workgroup; two planes 0.052, three 0.058: many short-lived workgroups
            // stream better than few long ones; plain instead of non-temporal stores 0.043 and the
            // kernel after it 5 % slower).
            {
                const long per_plane_floats = 2 * PH * PW + H * W;
                // at least 8 KB of output per workgroup (tiny planes share one), within 36 KB of LDS
                const long ppw_l = std::max(1L, std::min({(36 * 1024) / (per_plane_floats * 4), cdiv(8192L, H * W * 4), cdiv(nplanes, 2048L)}));
                const int nt = 1;
                const long in_floats = (ppw_l * PH * PW + 6) / 4 * 4, out_floats = (ppw_l * H * W + 6) / 4 * 4;
                const size_t lds = (size_t)(2 * in_floats + out_floats) * sizeof(float);
                const bool aligned = reinterpret_cast<uintptr_t>(bottom_diff) % 16 == 0 && reinterpret_cast<uintptr_t>(mask) % 16 == 0 &&
                                     reinterpret_cast<uintptr_t>(top_diff) % 16 == 0;
                if (ppw_l > 0 && aligned && lds <= 64 * 1024 && ppw_l * BH * BW < kFastdivLimit && ppw_l * H * W < kFastdivLimit) {
                    max_pool_bwd_linear_kernel<G><<<dim3((unsigned)cdiv(nplanes, ppw_l)), dim3(kPoolThreads), lds, st>>>(
                        g, mask, top_diff, bottom_diff, nplanes, (int)H, (int)W, (int)PH, (int)PW, (int)BH, (int)BW,
                        (int)ppw_l, (int)in_floats, nt);
                    CGT_LAUNCH_CHECK("max_pool_bwd_linear_kernel");
                    return CGT_AMD_OK;
                }
            }
            const int vec2 = W % 2 == 0 && reinterpret_cast<uintptr_t>(bottom_diff) % 8 == 0;
            max_pool_bwd_block_kernel<G><<<dim3((unsigned)blocks), dim3(kPoolThreads), 0, st>>>(
                g, mask, top_diff, bottom_diff, nplanes, (int)H, (int)W, (int)PH, (int)PW, (int)BH,
                (int)BW, ppw, vec2);
            CGT_LAUNCH_CHECK("max_pool_bwd_block_kernel");
            return CGT_AMD_OK;
        }
    }
    const long out_bytes = PH * PW * 2 * (long)sizeof(float);  // top_diff + mask per plane
    if (int ppw = pool_bwd_planes_per_wg(H, W, PH, PW)) {
        const long blocks = cdiv(nplanes, ppw);
        max_pool_bwd_kernel<G><<<dim3((unsigned)blocks), dim3(kPoolThreads), (size_t)ppw * out_bytes, st>>>(
            g, mask, top_diff, bottom_diff, nplanes, (int)H, (int)W, (int)PH, (int)PW, ppw);
        CGT_LAUNCH_CHECK("max_pool_bwd_kernel");
    } else {
        const long total = nplanes * H * W;
        long blocks = std::min(cdiv(total, (long)kPoolThreads), 1L << 20);
        max_pool_bwd_direct_kernel<G><<<dim3((unsigned)blocks), dim3(kPoolThreads), 0, st>>>(
            g, mask, top_diff, bottom_diff, total, (int)H, (int)W, (int)PH, (int)PW);
        CGT_LAUNCH_CHECK("max_pool_bwd_direct_kernel");
    }
    return CGT_AMD_OK;
}

int launch_pool_pullback_padded(const int* mask, const float* top_diff, const signed char* relu_mask, long nplanes,
                                long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, long PH, long PW,
                                const PaddedPlanes& lay, float* dst, void* stream) {
    int rc = check_pool("pool_pullback_padded", nplanes, 1, H, W, kh, kw, ph, pw, sh, sw, PH, PW);
    if (rc) return rc;
    CGT_ARG_CHECK(dst && reinterpret_cast<uintptr_t>(dst) % 16 == 0, "pool_pullback_padded: the padded buffer must be 16-byte aligned");
    CGT_ARG_CHECK(lay.plane % 4 == 0 && lay.tail % 4 == 0 && lay.plane < kFastdivLimit && lay.lead <= lay.pitch &&
                  lay.lead + (lay.top + H) * (long)lay.pitch <= lay.plane && W <= lay.pitch && H * W < (1L << 30),
                  "pool_pullback_padded: bad padded layout");
    CGT_ARG_CHECK(nplanes == 0 || PH * PW == 0 || (mask && top_diff), "pool_pullback_padded: null pointer");
    const long upp = lay.plane / 4, units = nplanes * upp, tail_units = lay.tail / 4;
    if (units + tail_units == 0) return CGT_AMD_OK;
    if (PH * PW == 0) return cgt_amd_fill_u32(dst, 0u, (units + tail_units) * 4, stream);     // no windows: all zeros
    CGT_ARG_CHECK(nplanes * cdiv(upp, 512L) < (1L << 31) - (1L << 19), "pool_pullback_padded: too many planes");
    // one wavefront per chunk of 512 units of a plane (grid-stride beyond 64 K workgroups)
    const long blocks = std::max(1L, std::min(cdiv(nplanes * cdiv(upp, 512L), (long)(kPoolThreads / 64)), 1L << 16));
    hipStream_t st = as_stream(stream);
    const long plane_bytes = lay.plane * (long)sizeof(float);
    if (kh <= sh && kw <= sw && plane_bytes <= 48 * 1024 && H * W < kFastdivLimit) {
        // planes per workgroup: up to 32 KB of LDS, and enough workgroups for every CU to hold several
        long ppw = std::max(1L, std::min((32 * 1024) / plane_bytes, nplanes / 2048));
        ppw = std::min(ppw, (kFastdivLimit - 1) / (PH * PW));
        if (ppw >= 1) {
            max_pool_bwd_padded_scatter_kernel<<<dim3((unsigned)cdiv(nplanes, ppw)), dim3(kPoolThreads), (size_t)(ppw * plane_bytes), st>>>(
                mask, top_diff, relu_mask, dst, nplanes, (int)(H * W), (int)W, (int)(PH * PW), lay, (int)ppw, tail_units);
            CGT_LAUNCH_CHECK("max_pool_bwd_padded_scatter_kernel");
            return CGT_AMD_OK;
        }
    }
#define X(KH, KW, PH_, PW_, SH, SW)                                                                              \
    if (kh == KH && kw == KW && ph == PH_ && pw == PW_ && sh == SH && sw == SW) {                                \
        max_pool_bwd_padded_kernel<<<dim3((unsigned)blocks), dim3(kPoolThreads), 0, st>>>(                       \
            StaticGeom<KH, KW, PH_, PW_, SH, SW>(), mask, top_diff, relu_mask, dst, (int)H, (int)W, (int)PH, (int)PW, lay, (int)upp, \
            units, tail_units);                                                                                  \
        CGT_LAUNCH_CHECK("max_pool_bwd_padded_kernel");                                                          \
        return CGT_AMD_OK;                                                                                       \
    }
    CGT_STATIC_POOLS(X)
#undef X
    max_pool_bwd_padded_kernel<<<dim3((unsigned)blocks), dim3(kPoolThreads), 0, st>>>(
        DynGeom{kh, kw, ph, pw, sh, sw}, mask, top_diff, relu_mask, dst, (int)H, (int)W, (int)PH, (int)PW, lay, (int)upp, units, tail_units);
    CGT_LAUNCH_CHECK("max_pool_bwd_padded_kernel");
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

CGT_API int cgt_amd_pool_staged_planes(int backward, long H, long W, long PH, long PW) {
    return backward ? pool_bwd_planes_per_wg(H, W, PH, PW) : pool_fwd_planes_per_wg(H, W, PH, PW);
}

CGT_API int cgt_amd_max_pool_f32(const float* bottom, long N, long C, long H, long W, int kh,
                                 int kw, int ph, int pw, int sh, int sw, long PH, long PW,
                                 float* top, int* mask, void* stream) {
    int rc = check_pool("max_pool", N, C, H, W, kh, kw, ph, pw, sh, sw, PH, PW);
    if (rc) return rc;
    const long nplanes = N * C;
    if (nplanes * PH * PW == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(bottom && top && mask, "max_pool: null pointer");
    hipStream_t st = as_stream(stream);
#define X(KH, KW, PH_, PW_, SH, SW)                                                     \
    if (kh == KH && kw == KW && ph == PH_ && pw == PW_ && sh == SH && sw == SW)         \
        return launch_pool_fwd(StaticGeom<KH, KW, PH_, PW_, SH, SW>(), bottom, nplanes, H, W, PH, PW, top, mask, st);
    CGT_STATIC_POOLS(X)
#undef X
    return launch_pool_fwd(DynGeom{kh, kw, ph, pw, sh, sw}, bottom, nplanes, H, W, PH, PW, top, mask, st);
}

CGT_API int cgt_amd_max_pool_pullback_f32(const int* mask, const float* top_diff, long N, long C,
                                          long H, long W, int kh, int kw, int ph, int pw, int sh,
                                          int sw, long PH, long PW, float* bottom_diff,
                                          void* stream) {
    int rc = check_pool("max_pool_pullback", N, C, H, W, kh, kw, ph, pw, sh, sw, PH, PW);
    if (rc) return rc;
    const long nplanes = N * C;
    if (nplanes * H * W == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(bottom_diff, "max_pool_pullback: null pointer");
    hipStream_t st = as_stream(stream);
    if (PH * PW == 0) return cgt_amd_fill_u32(bottom_diff, 0u, nplanes * H * W, stream);
    CGT_ARG_CHECK(mask && top_diff, "max_pool_pullback: null pointer");
#define X(KH, KW, PH_, PW_, SH, SW)                                                     \
    if (kh == KH && kw == KW && ph == PH_ && pw == PW_ && sh == SH && sw == SW)         \
        return launch_pool_bwd(StaticGeom<KH, KW, PH_, PW_, SH, SW>(), mask, top_diff, nplanes, H, W, PH, PW, bottom_diff, st);
    CGT_STATIC_POOLS(X)
#undef X
    return launch_pool_bwd(DynGeom{kh, kw, ph, pw, sh, sw}, mask, top_diff, nplanes, H, W, PH, PW, bottom_diff, st);
}
