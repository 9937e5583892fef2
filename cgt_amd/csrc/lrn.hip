// Cross-channel local response normalisation for gfx950.  HBM-bound.
//
// Arrays are [N,C,H,W]; the window runs along C, so neighbours in the window
// are H*W floats apart while neighbours in a wavefront (consecutive pixels)
// are adjacent: every load/store instruction is one contiguous run.
//
// A thread owns one pixel (n, p) and a run of channels; it walks the run with
// the window held in registers, so x is read once (plus a halo of size-1
// channels per run), scale and top are written once, in a single fused pass:
// 3 array passes forward, 5 backward.  The window sum is taken directly over
// the registers (not as the reference's running add/subtract), which is more
// accurate and independent of the walk direction.
#include "common.h"
#include <algorithm>

namespace cgt_amd {

constexpr int kLrnThreads = 256;

// One-dimensional grid over (image, channel run, pixel block), pixel blocks
// fastest.  Workgroups go to the 8 XCDs round-robin by id; the remap gives each
// XCD a contiguous range, so the two workgroups that share a cache line at a
// pixel-block boundary (H*W need not be a multiple of anything) meet in one L2.
struct LrnBlock {
    int px, run, n;
};
__device__ __forceinline__ LrnBlock lrn_block(int HW, int C, int crun) {
    const int total = gridDim.x;
    const int q = total / kNumXCD, r = total % kNumXCD;
    const int xcd = blockIdx.x % kNumXCD, local = blockIdx.x / kNumXCD;
    int id = xcd * q + min(xcd, r) + local;
    const int pb = (HW + kLrnThreads - 1) / kLrnThreads, runs = (C + crun - 1) / crun;
    LrnBlock b;
    b.px = id % pb;
    id /= pb;
    b.run = id % runs;
    b.n = id / runs;
    return b;
}

// acc + v * v with the product rounded on its own, and k + acc * (alpha / n) as one fused
// multiply-add: spelled out so that every kernel of this file forms a window sum and a scale
// with the same roundings, whatever the compiler would otherwise share or fuse between
// neighbouring windows (a kernel that unrolls the channel walk reuses the squares and adds
// them; one that does not would fuse each product into its add).
__device__ __forceinline__ float add_square(float acc, float v) {
#pragma clang fp contract(off)
    const float sq = v * v;
    return acc + sq;
}
__device__ __forceinline__ float scale_of(float acc, float aos, float kconst) { return __builtin_fmaf(acc, aos, kconst); }

__device__ __forceinline__ float pow_neg_beta(float s, float nbeta) {
    // s >= k > 0.  exp2(nbeta*log2(s)) on the hardware transcendental units:
    // relative error ~1e-6 for the scale range LRN produces.
    return __builtin_amdgcn_exp2f(nbeta * __builtin_amdgcn_logf(s));
}

// SIZE > 0: window length known at compile time.  Channels are walked in
// chunks of U: the U new loads of a chunk are all issued before the first use,
// so every lane keeps U runs in flight (one pixel per lane gives only 4-byte
// loads -- H*W is odd in the AlexNet layer -- so depth has to come from here).
constexpr int kLrnChunk = 8;

// DOWN: the run is walked from its last channel to its first.  Odd runs walk down and
// even runs up, so the channels two neighbouring runs both need (each run's halo is the
// other's edge) are loaded by both at the same end of their walk -- at about the same
// time, which lets one of the two find them in L2 instead of fetching them again.  A
// downward walk is the upward one on the mirrored channel axis v = C-1-c: window
// [c-PRE, c+POST] becomes [v-POST, v+PRE], pointers step by -H*W.
template <int SIZE, bool DOWN>
__device__ __forceinline__ void lrn_fwd_run(const float* __restrict__ x, float* __restrict__ top,
                                            float* __restrict__ scale, int C, int HW, const LrnBlock& blk,
                                            int crun, float aos, float nbeta, float kconst, bool stream_out) {
    constexpr int PRE0 = (SIZE - 1) / 2, POST0 = SIZE - PRE0 - 1, U = kLrnChunk;
    constexpr int PRE = DOWN ? POST0 : PRE0, POST = DOWN ? PRE0 : POST0;
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs0 = blk.run * crun, ce0 = min(C, cs0 + crun);
    const int cs = DOWN ? C - ce0 : cs0, ce = DOWN ? C - cs0 : ce0;     // the run on the walked axis
    const long hs = DOWN ? -(long)HW : (long)HW;
    const long origin = n * C * (long)HW + p + (DOWN ? (long)(C - 1) * HW : 0);
    const float* xp = x + origin;
    float* tp = top + origin;
    float* sp = scale + origin;

    float win[U + SIZE - 1];  // win[j] = x[c0 - PRE + j]
#pragma unroll
    for (int j = 0; j < SIZE - 1; ++j) {
        const int c = cs - PRE + j;
        win[j] = (c >= 0 && c < C) ? xp[c * hs] : 0.0f;
    }
    for (int c0 = cs; c0 < ce; c0 += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ch = c0 + POST + u;
            win[SIZE - 1 + u] = (ch < C) ? xp[ch * hs] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < SIZE; ++j) acc = add_square(acc, win[u + j]);
            const float s = scale_of(acc, aos, kconst);
            if (c0 + u < ce) {
                if (scale) sp[(c0 + u) * hs] = s;
                const float t = win[u + PRE] * pow_neg_beta(s, nbeta);
                if (stream_out) __builtin_nontemporal_store(t, &tp[(c0 + u) * hs]);
                else tp[(c0 + u) * hs] = t;
            }
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) win[j] = win[U + j];
    }
}

template <int SIZE>
__global__ __launch_bounds__(kLrnThreads) void lrn_fwd_kernel(
    const float* __restrict__ x, float* __restrict__ top, float* __restrict__ scale, int C,
    int HW, int crun, float aos, float nbeta, float kconst, int stream_out) {
    const LrnBlock blk = lrn_block(HW, C, crun);
    if (blk.run & 1) lrn_fwd_run<SIZE, true>(x, top, scale, C, HW, blk, crun, aos, nbeta, kconst, stream_out != 0);
    else lrn_fwd_run<SIZE, false>(x, top, scale, C, HW, blk, crun, aos, nbeta, kconst, stream_out != 0);
}

// Flat variant for large arrays.  The stores are two thirds of the forward
// traffic, and the pixel-per-lane kernel issues them 4 bytes per lane (straddling
// cache lines when H*W is odd, as 55*55).
// Here a thread owns one aligned unit of four consecutive floats of the flat
// [N*C*H*W] array and writes both outputs with streamed 16-byte stores.  Its four
// pixels lie in one channel plane (units that straddle two planes, one in
// H*W/4, take an element-wise path), so the window is SIZE unaligned 16-byte
// loads H*W floats apart.  Each input float is fetched SIZE times, but only
// the first fetch goes to HBM: neighbouring channels of the same pixels are
// loaded by workgroups close by in the grid and meet in L2.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));

template <int SIZE>
__global__ __launch_bounds__(kLrnThreads) void lrn_fwd_flat_kernel(
    const float* __restrict__ x, float* __restrict__ top, float* __restrict__ scale, int C,
    int HW, unsigned total, float aos, float nbeta, float kconst) {
    constexpr int PRE = (SIZE - 1) / 2;
    // each XCD (one L2) takes a contiguous range of the flat array, so the SIZE
    // fetches of a float come from one L2
    const unsigned nblk = gridDim.x, q = nblk / kNumXCD, r = nblk % kNumXCD;
    const unsigned xcd = blockIdx.x % kNumXCD, local = blockIdx.x / kNumXCD;
    const unsigned bid = xcd * q + min(xcd, r) + local;
    const unsigned f = 4u * (bid * kLrnThreads + threadIdx.x);
    if (f >= total) return;
    const unsigned plane = f / (unsigned)HW;             // image * C + channel
    const int p0 = (int)(f - plane * (unsigned)HW);
    const int c0 = (int)(plane % (unsigned)C);
    if (p0 + 3 < HW && f + 3 < total) {
        v4f w[SIZE];
        bool ok[SIZE];
#pragma unroll
        for (int j = 0; j < SIZE; ++j) {
            const int c = c0 - PRE + j;
            ok[j] = c >= 0 && c < C;
            // outside the window the unit's own address is loaded and discarded: no load is conditional
            const long at = ok[j] ? (long)f + (long)(j - PRE) * HW : (long)f;
            w[j] = *reinterpret_cast<const v4f_unaligned*>(x + at);
        }
        const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
        v4f acc = zero;
#pragma unroll
        for (int j = 0; j < SIZE; ++j) {
            const v4f v = ok[j] ? w[j] : zero;
            acc.x = add_square(acc.x, v.x);
            acc.y = add_square(acc.y, v.y);
            acc.z = add_square(acc.z, v.z);
            acc.w = add_square(acc.w, v.w);
        }
        const v4f s = {scale_of(acc.x, aos, kconst), scale_of(acc.y, aos, kconst), scale_of(acc.z, aos, kconst),
                       scale_of(acc.w, aos, kconst)};
        const v4f mid = w[PRE];
        if (scale) stream_store4(scale + f, s.x, s.y, s.z, s.w);
        stream_store4(top + f, mid.x * pow_neg_beta(s.x, nbeta), mid.y * pow_neg_beta(s.y, nbeta),
                      mid.z * pow_neg_beta(s.z, nbeta), mid.w * pow_neg_beta(s.w, nbeta));
        return;
    }
    for (unsigned e = f; e < f + 4 && e < total; ++e) {
        const unsigned pl = e / (unsigned)HW;
        const int c = (int)(pl % (unsigned)C);
        float acc = 0.0f;
        for (int j = 0; j < SIZE; ++j) {
            const int cc = c - PRE + j;
            const float v = (cc >= 0 && cc < C) ? x[(long)e + (long)(j - PRE) * HW] : 0.0f;
            acc = add_square(acc, v);
        }
        const float s = scale_of(acc, aos, kconst);
        if (scale) scale[e] = s;
        top[e] = x[e] * pow_neg_beta(s, nbeta);
    }
}

// Any window length: re-reads the window through the cache.
__global__ __launch_bounds__(kLrnThreads) void lrn_fwd_generic_kernel(
    const float* __restrict__ x, float* __restrict__ top, float* __restrict__ scale, int C,
    int HW, int crun, int size, float aos, float nbeta, float kconst) {
    const int pre = (size - 1) / 2, post = size - pre - 1;
    const LrnBlock blk = lrn_block(HW, C, crun);
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs = blk.run * crun, ce = min(C, cs + crun);
    const long base = n * C * (long)HW + p;
    for (int c = cs; c < ce; ++c) {
        float acc = 0.0f;
        const int lo = max(0, c - pre), hi = min(C - 1, c + post);
        for (int cc = lo; cc <= hi; ++cc) acc = add_square(acc, x[base + (long)cc * HW]);
        const float s = scale_of(acc, aos, kconst);
        if (scale) scale[base + (long)c * HW] = s;
        top[base + (long)c * HW] = x[base + (long)c * HW] * pow_neg_beta(s, nbeta);
    }
}

// RECOMP: `top` is not read; top[c] = x[c] * scale[c]^-beta is formed again from x and scale
// with the operations of the forward kernels (same bits as the array they wrote), so the
// kernel streams four arrays instead of five.
template <int SIZE, bool DOWN, bool RECOMP>
__device__ __forceinline__ void lrn_bwd_run(const float* __restrict__ x, const float* __restrict__ top,
                                            const float* __restrict__ scale, const float* __restrict__ top_diff,
                                            float* __restrict__ bottom_diff, int C, int HW, const LrnBlock& blk,
                                            int crun, float nbeta, float ratio) {
    // transposed window: [c - PRE0, c + POST0]; mirrored when walking down (see lrn_fwd_run)
    constexpr int PRE0 = SIZE - (SIZE + 1) / 2, POST0 = SIZE - PRE0 - 1, U = kLrnChunk;
    constexpr int PRE = DOWN ? POST0 : PRE0, POST = DOWN ? PRE0 : POST0;
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs0 = blk.run * crun, ce0 = min(C, cs0 + crun);
    const int cs = DOWN ? C - ce0 : cs0, ce = DOWN ? C - cs0 : ce0;
    const long hs = DOWN ? -(long)HW : (long)HW;
    const long base = n * C * (long)HW + p + (DOWN ? (long)(C - 1) * HW : 0);
    const float* xp = x + base;
    const float* tp = top + base;
    const float* sp = scale + base;
    const float* dp = top_diff + base;
    float* bp = bottom_diff + base;

    float tr[U + SIZE - 1];   // tr[j] = (td*top/scale)[c0 - PRE + j]
    float dr[U + POST];       // dr[j] = td[c0 + j]
    float sr[U + POST];       // sr[j] = scale[c0 + j]; RECOMP: scale[c0 + j]^-beta
    float xr[U + POST];       // RECOMP: x[c0 + j]
#pragma unroll
    for (int j = 0; j < SIZE - 1; ++j) {
        const int c = cs - PRE + j;
        float d = 0.0f, sc = 1.0f, t = 0.0f;      // t: top, or x when it is formed here
        if (c >= 0 && c < C) {
            d = dp[c * hs];
            sc = sp[c * hs];
            t = RECOMP ? xp[c * hs] : tp[c * hs];
        }
        if constexpr (RECOMP) {
            const float pw = pow_neg_beta(sc, nbeta);
            tr[j] = d * (t * pw) / sc;
            if (j >= PRE) {
                dr[j - PRE] = d;
                sr[j - PRE] = pw;
                xr[j - PRE] = t;
            }
        } else {
            tr[j] = d * t / sc;
            if (j >= PRE) {           // channel >= cs: also a centre later on
                dr[j - PRE] = d;
                sr[j - PRE] = sc;
            }
        }
    }
    for (int c0 = cs; c0 < ce; c0 += U) {
        float xc[U], tn[U], sn[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ch = c0 + POST + u;
            float d = 0.0f, sc = 1.0f, t = 0.0f;
            if (ch < C) {
                d = dp[ch * hs];
                sc = sp[ch * hs];
                t = RECOMP ? xp[ch * hs] : tp[ch * hs];
            }
            dr[POST + u] = d;
            sn[u] = sc;
            tn[u] = t;
            if constexpr (!RECOMP) {
                sr[POST + u] = sc;
                xc[u] = (c0 + u < ce) ? xp[(c0 + u) * hs] : 0.0f;
            }
        }
        if constexpr (RECOMP) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float pw = pow_neg_beta(sn[u], nbeta);
                sr[POST + u] = pw;
                xr[POST + u] = tn[u];
                tr[SIZE - 1 + u] = dr[POST + u] * (tn[u] * pw) / sn[u];
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) tr[SIZE - 1 + u] = dr[POST + u] * tn[u] / sn[u];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < SIZE; ++j) acc += tr[u + j];
            if (c0 + u < ce) {
                if constexpr (RECOMP) bp[(c0 + u) * hs] = dr[u] * sr[u] - ratio * xr[u] * acc;
                else bp[(c0 + u) * hs] = dr[u] * pow_neg_beta(sr[u], nbeta) - ratio * xc[u] * acc;
            }
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) tr[j] = tr[U + j];
#pragma unroll
        for (int j = 0; j < POST; ++j) {
            dr[j] = dr[U + j];
            sr[j] = sr[U + j];
            if constexpr (RECOMP) xr[j] = xr[U + j];
        }
    }
}

template <int SIZE, bool RECOMP>
__global__ __launch_bounds__(kLrnThreads) void lrn_bwd_kernel(
    const float* __restrict__ x, const float* __restrict__ top, const float* __restrict__ scale,
    const float* __restrict__ top_diff, float* __restrict__ bottom_diff, int C, int HW, int crun,
    float nbeta, float ratio) {
    const LrnBlock blk = lrn_block(HW, C, crun);
    if (blk.run & 1) lrn_bwd_run<SIZE, true, RECOMP>(x, top, scale, top_diff, bottom_diff, C, HW, blk, crun, nbeta, ratio);
    else lrn_bwd_run<SIZE, false, RECOMP>(x, top, scale, top_diff, bottom_diff, C, HW, blk, crun, nbeta, ratio);
}

// No stored scale: scale[ch] = k + (alpha/size) * sum of x^2 over the forward window of ch is formed
// again from x (the window sum the forward kernels take, in the order of the walk), so the kernel
// streams x and the cotangent in and the result out -- three arrays.  Every channel that enters
// the ratio window needs its own forward window, so the run's halo of x is 2 (SIZE - 1) channels.
template <int SIZE, bool DOWN>
__device__ __forceinline__ void lrn_bwd_x_run(const float* __restrict__ x, const float* __restrict__ top_diff,
                                              float* __restrict__ bottom_diff, int C, int HW, const LrnBlock& blk,
                                              int crun, float aos, float nbeta, float kconst, float ratio) {
    constexpr int PRE0 = SIZE - (SIZE + 1) / 2, POST0 = SIZE - PRE0 - 1, U = kLrnChunk;      // ratio window
    constexpr int FPRE0 = (SIZE - 1) / 2, FPOST0 = SIZE - FPRE0 - 1;                         // forward window
    constexpr int PRE = DOWN ? POST0 : PRE0, POST = DOWN ? PRE0 : POST0;
    constexpr int FPRE = DOWN ? FPOST0 : FPRE0, FPOST = DOWN ? FPRE0 : FPOST0;
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs0 = blk.run * crun, ce0 = min(C, cs0 + crun);
    const int cs = DOWN ? C - ce0 : cs0, ce = DOWN ? C - cs0 : ce0;
    const long hs = DOWN ? -(long)HW : (long)HW;
    const long base = n * C * (long)HW + p + (DOWN ? (long)(C - 1) * HW : 0);
    const float* xp = x + base;
    const float* dp = top_diff + base;
    float* bp = bottom_diff + base;

    float xw[U + SIZE - 1];   // xw[j] = x[c0 + POST - FPRE + j]
    float tr[U + SIZE - 1];   // tr[j] = (td*top/scale)[c0 - PRE + j]
    float dr[U + POST];       // dr[j] = td[c0 + j]
    float sr[U + POST];       // sr[j] = scale[c0 + j]^-beta
    float xr[U + POST];       // xr[j] = x[c0 + j]
    {
        // channels cs - PRE .. cs + POST - 1 fill the window before the first centre
        float xh[2 * (SIZE - 1) + 1], dh[SIZE];
#pragma unroll
        for (int i = 0; i < 2 * (SIZE - 1); ++i) {
            const int c = cs - PRE - FPRE + i;
            xh[i] = (c >= 0 && c < C) ? xp[c * hs] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) {
            const int c = cs - PRE + j;
            dh[j] = (c >= 0 && c < C) ? dp[c * hs] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) {
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < SIZE; ++i) acc = add_square(acc, xh[j + i]);
            const float sc = scale_of(acc, aos, kconst);
            const float pw = pow_neg_beta(sc, nbeta);
            const float xc = xh[j + FPRE];
            tr[j] = dh[j] * (xc * pw) / sc;
            if (j >= PRE) {
                dr[j - PRE] = dh[j];
                sr[j - PRE] = pw;
                xr[j - PRE] = xc;
            }
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) xw[j] = xh[SIZE - 1 + j];
    }
    for (int c0 = cs; c0 < ce; c0 += U) {
        float dn[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int cx = c0 + POST + FPOST + u, cd = c0 + POST + u;
            xw[SIZE - 1 + u] = (cx < C) ? xp[cx * hs] : 0.0f;
            dn[u] = (cd < C) ? dp[cd * hs] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < SIZE; ++i) acc = add_square(acc, xw[u + i]);
            const float sc = scale_of(acc, aos, kconst);
            const float pw = pow_neg_beta(sc, nbeta);
            const float xc = xw[u + FPRE];
            dr[POST + u] = dn[u];
            sr[POST + u] = pw;
            xr[POST + u] = xc;
            tr[SIZE - 1 + u] = dn[u] * (xc * pw) / sc;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < SIZE; ++j) acc += tr[u + j];
            if (c0 + u < ce) bp[(c0 + u) * hs] = dr[u] * sr[u] - ratio * xr[u] * acc;
        }
#pragma unroll
        for (int j = 0; j < SIZE - 1; ++j) {
            tr[j] = tr[U + j];
            xw[j] = xw[U + j];
        }
#pragma unroll
        for (int j = 0; j < POST; ++j) {
            dr[j] = dr[U + j];
            sr[j] = sr[U + j];
            xr[j] = xr[U + j];
        }
    }
}

template <int SIZE>
__global__ __launch_bounds__(kLrnThreads) void lrn_bwd_x_kernel(
    const float* __restrict__ x, const float* __restrict__ top_diff, float* __restrict__ bottom_diff, int C, int HW,
    int crun, float aos, float nbeta, float kconst, float ratio) {
    const LrnBlock blk = lrn_block(HW, C, crun);
    if (blk.run & 1) lrn_bwd_x_run<SIZE, true>(x, top_diff, bottom_diff, C, HW, blk, crun, aos, nbeta, kconst, ratio);
    else lrn_bwd_x_run<SIZE, false>(x, top_diff, bottom_diff, C, HW, blk, crun, aos, nbeta, kconst, ratio);
}

// any window length, from x alone
__global__ __launch_bounds__(kLrnThreads) void lrn_bwd_x_generic_kernel(
    const float* __restrict__ x, const float* __restrict__ top_diff, float* __restrict__ bottom_diff, int C, int HW,
    int crun, int size, float aos, float nbeta, float kconst, float ratio) {
    const int pre = size - (size + 1) / 2, post = size - pre - 1;
    const int fpre = (size - 1) / 2, fpost = size - fpre - 1;
    const LrnBlock blk = lrn_block(HW, C, crun);
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs = blk.run * crun, ce = min(C, cs + crun);
    const long base = n * C * (long)HW + p;
    auto scale_at = [&](int ch) {
        float acc = 0.0f;
        for (int cc = max(0, ch - fpre); cc <= min(C - 1, ch + fpost); ++cc) acc = add_square(acc, x[base + (long)cc * HW]);
        return scale_of(acc, aos, kconst);
    };
    for (int c = cs; c < ce; ++c) {
        float acc = 0.0f;
        for (int cc = max(0, c - pre); cc <= min(C - 1, c + post); ++cc) {
            const long i = base + (long)cc * HW;
            const float sc = scale_at(cc);
            acc += top_diff[i] * (x[i] * pow_neg_beta(sc, nbeta)) / sc;
        }
        const long i = base + (long)c * HW;
        bottom_diff[i] = top_diff[i] * pow_neg_beta(scale_at(c), nbeta) - ratio * x[i] * acc;
    }
}

__global__ __launch_bounds__(kLrnThreads) void lrn_bwd_generic_kernel(
    const float* __restrict__ x, const float* __restrict__ top, const float* __restrict__ scale,
    const float* __restrict__ top_diff, float* __restrict__ bottom_diff, int C, int HW, int crun,
    int size, float nbeta, float ratio) {
    const int pre = size - (size + 1) / 2, post = size - pre - 1;
    const LrnBlock blk = lrn_block(HW, C, crun);
    const int p = blk.px * kLrnThreads + threadIdx.x;
    if (p >= HW) return;
    const long n = blk.n;
    const int cs = blk.run * crun, ce = min(C, cs + crun);
    const long base = n * C * (long)HW + p;
    for (int c = cs; c < ce; ++c) {
        float acc = 0.0f;
        const int lo = max(0, c - pre), hi = min(C - 1, c + post);
        for (int cc = lo; cc <= hi; ++cc) {
            const long i = base + (long)cc * HW;
            const float t = top ? top[i] : x[i] * pow_neg_beta(scale[i], nbeta);      // top == nullptr: formed again
            acc += top_diff[i] * t / scale[i];
        }
        const long i = base + (long)c * HW;
        bottom_diff[i] = top_diff[i] * pow_neg_beta(scale[i], nbeta) - ratio * x[i] * acc;
    }
}

static int check_lrn(const char* what, long N, long C, long H, long W, int size) {
    CGT_ARG_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0, "%s: negative shape", what);
    CGT_ARG_CHECK(size >= 1 && size <= C, "%s: need 1 <= size <= C, got size=%d C=%ld", what, size, C);
    CGT_ARG_CHECK(H * W < (1L << 31) && C < (1L << 31) && cdiv(H * W, kLrnThreads) * C * N < (1L << 31), "%s: shape too large", what);
    return CGT_AMD_OK;
}

// Channels per thread run.  Short runs win on this chip even though each run
// re-reads a halo of size-1 channels: more, shorter workgroups balance better
// (measured on the AlexNet and VGG shapes: 16 beats 32, 48 and 96).  Small
// problems go shorter still so that every CU gets work.
static int pick_crun(long N, int C, int HW, int size) {
    const long pix_blocks = cdiv(HW, kLrnThreads) * N;
    int crun = C;
    const int min_run = std::max(3 * size, 16);
    while (crun > min_run && pix_blocks * cdiv(C, crun) < 8192) crun = (crun + 1) / 2;
    crun = std::min(C, std::max(crun, min_run));
    const int floor_run = std::max(size, 8);
    while (crun > floor_run && pix_blocks * cdiv(C, crun) < 1024) crun = (crun + 1) / 2;
    return std::min(C, std::max(crun, floor_run));
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_lrn_fwd_f32(const float* x, long N, long C, long H, long W, int size,
                                double alpha, double beta, double k, float* top, float* scale,
                                void* stream) {
    if (N * C * H * W == 0 && N >= 0 && C >= 0 && H >= 0 && W >= 0 && size >= 1) return CGT_AMD_OK;
    int rc = check_lrn("lrn_fwd", N, C, H, W, size);
    if (rc) return rc;
    CGT_ARG_CHECK(x && top, "lrn_fwd: null pointer");          // scale == nullptr: not stored
    CGT_ARG_CHECK(k > 0, "lrn_fwd: k must be positive");
    const int HW = (int)(H * W);
    const int crun = pick_crun(N, (int)C, HW, size);
    dim3 grid((unsigned)(cdiv(HW, kLrnThreads) * cdiv(C, crun) * N)), block(kLrnThreads);
    hipStream_t st = as_stream(stream);
    const float aos = (float)(alpha / size), nbeta = (float)(-beta), kc = (float)k;
    const long total = N * C * HW;
    // the flat kernel wins once the arrays no longer sit in the last-level cache
    // (measured: 37 M floats 0.066 vs 0.098 ms, 24 M 0.051 vs 0.067, 9 M 0.022 vs 0.017) -- when both
    // outputs are stored; with top alone the pixel-per-lane kernel is ahead (37 M floats: 0.057 vs 0.071)
    const bool flat = scale && total >= (16L << 20) && total < (1L << 31) && reinterpret_cast<uintptr_t>(top) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(scale) % 16 == 0;
    // an output too large to stay in the last-level cache for its reader is stored past it
    // (AlexNet conv1 layer, top alone: 0.008 ms of the step, a third of it in the kernels that follow)
    const int stream_out = total >= (16L << 20) ? 1 : 0;
    const dim3 flat_grid((unsigned)cdiv(cdiv(total, 4), kLrnThreads));
#define LRN_FWD_CASE(S)                                                                           \
    case S:                                                                                       \
        if (flat)                                                                                 \
            lrn_fwd_flat_kernel<S><<<flat_grid, block, 0, st>>>(x, top, scale, (int)C, HW, (unsigned)total, aos, nbeta, kc); \
        else                                                                                      \
            lrn_fwd_kernel<S><<<grid, block, 0, st>>>(x, top, scale, (int)C, HW, crun, aos, nbeta, kc, stream_out); \
        break;
    switch (size) {
        LRN_FWD_CASE(1) LRN_FWD_CASE(2) LRN_FWD_CASE(3) LRN_FWD_CASE(4) LRN_FWD_CASE(5)
        LRN_FWD_CASE(6) LRN_FWD_CASE(7) LRN_FWD_CASE(8) LRN_FWD_CASE(9)
        default:
            lrn_fwd_generic_kernel<<<grid, block, 0, st>>>(x, top, scale, (int)C, HW, crun, size, aos, nbeta, kc);
    }
#undef LRN_FWD_CASE
    CGT_LAUNCH_CHECK("lrn_fwd_kernel");
    return CGT_AMD_OK;
}

// top == nullptr: top is formed again from x and scale (cgt_amd_lrn_bwd_recompute_f32)
static int lrn_bwd(const float* x, const float* top, const float* scale, const float* top_diff, long N, long C, long H,
                   long W, int size, double alpha, double beta, float* bottom_diff, void* stream) {
    if (N * C * H * W == 0 && N >= 0 && C >= 0 && H >= 0 && W >= 0 && size >= 1) return CGT_AMD_OK;
    int rc = check_lrn("lrn_bwd", N, C, H, W, size);
    if (rc) return rc;
    CGT_ARG_CHECK(x && scale && top_diff && bottom_diff, "lrn_bwd: null pointer");
    const int HW = (int)(H * W);
    const int crun = pick_crun(N, (int)C, HW, size);
    dim3 grid((unsigned)(cdiv(HW, kLrnThreads) * cdiv(C, crun) * N)), block(kLrnThreads);
    hipStream_t st = as_stream(stream);
    const float nbeta = (float)(-beta), ratio = (float)(2. * alpha * beta / size);
#define LRN_BWD_CASE(S)                                                                                       \
    case S:                                                                                                   \
        if (top) lrn_bwd_kernel<S, false><<<grid, block, 0, st>>>(x, top, scale, top_diff, bottom_diff, (int)C, HW, crun, nbeta, ratio); \
        else lrn_bwd_kernel<S, true><<<grid, block, 0, st>>>(x, top, scale, top_diff, bottom_diff, (int)C, HW, crun, nbeta, ratio);      \
        break;
    switch (size) {
        LRN_BWD_CASE(1) LRN_BWD_CASE(2) LRN_BWD_CASE(3) LRN_BWD_CASE(4) LRN_BWD_CASE(5)
        LRN_BWD_CASE(6) LRN_BWD_CASE(7) LRN_BWD_CASE(8) LRN_BWD_CASE(9)
        default:
            lrn_bwd_generic_kernel<<<grid, block, 0, st>>>(x, top, scale, top_diff, bottom_diff,
                                                           (int)C, HW, crun, size, nbeta, ratio);
    }
#undef LRN_BWD_CASE
    CGT_LAUNCH_CHECK("lrn_bwd_kernel");
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_lrn_bwd_f32(const float* x, const float* top, const float* scale,
                                const float* top_diff, long N, long C, long H, long W, int size,
                                double alpha, double beta, float* bottom_diff, void* stream) {
    CGT_ARG_CHECK(top || N * C * H * W == 0, "lrn_bwd: null pointer");
    return lrn_bwd(x, top, scale, top_diff, N, C, H, W, size, alpha, beta, bottom_diff, stream);
}

CGT_API int cgt_amd_lrn_bwd_recompute_f32(const float* x, const float* scale, const float* top_diff, long N, long C,
                                          long H, long W, int size, double alpha, double beta, float* bottom_diff,
                                          void* stream) {
    return lrn_bwd(x, nullptr, scale, top_diff, N, C, H, W, size, alpha, beta, bottom_diff, stream);
}

CGT_API int cgt_amd_lrn_bwd_from_x_f32(const float* x, const float* top_diff, long N, long C, long H, long W, int size,
                                       double alpha, double beta, double k, float* bottom_diff, void* stream) {
    if (N * C * H * W == 0 && N >= 0 && C >= 0 && H >= 0 && W >= 0 && size >= 1) return CGT_AMD_OK;
    int rc = check_lrn("lrn_bwd_from_x", N, C, H, W, size);
    if (rc) return rc;
    CGT_ARG_CHECK(x && top_diff && bottom_diff, "lrn_bwd_from_x: null pointer");
    CGT_ARG_CHECK(k > 0, "lrn_bwd_from_x: k must be positive");
    const int HW = (int)(H * W);
    const int crun = pick_crun(N, (int)C, HW, size);
    dim3 grid((unsigned)(cdiv(HW, kLrnThreads) * cdiv(C, crun) * N)), block(kLrnThreads);
    hipStream_t st = as_stream(stream);
    const float aos = (float)(alpha / size), nbeta = (float)(-beta), kc = (float)k, ratio = (float)(2. * alpha * beta / size);
#define LRN_BWD_X_CASE(S)                                                                                     \
    case S:                                                                                                   \
        lrn_bwd_x_kernel<S><<<grid, block, 0, st>>>(x, top_diff, bottom_diff, (int)C, HW, crun, aos, nbeta, kc, ratio); \
        break;
    switch (size) {
        LRN_BWD_X_CASE(1) LRN_BWD_X_CASE(2) LRN_BWD_X_CASE(3) LRN_BWD_X_CASE(4) LRN_BWD_X_CASE(5)
        LRN_BWD_X_CASE(6) LRN_BWD_X_CASE(7) LRN_BWD_X_CASE(8) LRN_BWD_X_CASE(9)
        default:
            lrn_bwd_x_generic_kernel<<<grid, block, 0, st>>>(x, top_diff, bottom_diff, (int)C, HW, crun, size, aos, nbeta, kc, ratio);
    }
#undef LRN_BWD_X_CASE
    CGT_LAUNCH_CHECK("lrn_bwd_x_kernel");
    return CGT_AMD_OK;
}
