// im2col / col2im for gfx950.  Both are HBM-bound copies / ordered sums.
//
// Layouts (as in CGT): image [B,C,H,W]; column buffer [B,m,n,Z] with
// Z = C*kh*kw ordered (channel, kernel row, kernel col).
//
// im2col: one workgroup owns (image b, output row h, a chunk of channels).
//   It stages the kh input rows of its channels into LDS with coalesced row
//   reads (zero padded left/right/top/bottom, so the inner loop has no bounds
//   tests), then streams the output row: consecutive lanes write consecutive
//   z, so every store instruction covers one contiguous run of the column
//   buffer.  Each input element is read from HBM kh/sh times at most (the
//   neighbouring rows' workgroups run at the same time and share L2).
//
// col2im: gather form of the reference's scatter loop.  Each image pixel sums
//   its taps in ascending (kernel row, kernel col) order, which for a fixed
//   channel is ascending z -- the order the sequential reference adds them in
//   -- so no atomics are needed and the result is bit-identical.
#include "common.h"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace cgt_amd {

constexpr int kIm2colThreads = 256;
constexpr int kIm2colWaves = kIm2colThreads / kWave;

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Remapping the
// id so that each XCD owns one contiguous range puts neighbouring tiles (which
// share halo rows) behind the same L2 and close together in time.
__device__ __forceinline__ long xcd_remap(long id, long n) {
    const long q = n / kNumXCD, r = n % kNumXCD;
    const long xcd = id % kNumXCD, local = id / kNumXCD;
    return xcd * q + (xcd < r ? xcd : r) + local;
}

// VEC: units of 4 consecutive z per thread and 16-byte stores (needs Z%4==0
// and chunk*kh*kw%4==0); otherwise units of one float.
//
// A thread owns a fixed unit column (its z values, hence its (channel, kernel
// row, kernel col) LDS offsets, decoded once) and walks the output pixels w of
// the row: per step the LDS offsets advance by the stride and the store address
// by Z floats -- no divisions in the loop.  Lanes hold consecutive unit columns,
// so each store instruction covers one contiguous run.
template <class G, bool VEC>
__global__ __launch_bounds__(kIm2colThreads) void im2col_rows_kernel(
    G g, const float* __restrict__ im, float* __restrict__ col, int C, int H, int W, int m, int n,
    int chunk, int nchunks) {
    extern __shared__ float tile[];  // [cc*kh][Wp], Wp = W + 2*pw
    constexpr int UW = VEC ? 4 : 1;

    const int KH = g.kh(), KW = g.kw();
    const int Wp = W + 2 * g.pw();
    const long bid = xcd_remap(blockIdx.x, gridDim.x);
    const int h = (int)(bid % m);
    const int ck = (int)((bid / m) % nchunks);
    const long b = bid / ((long)nchunks * m);
    const int c0 = ck * chunk;
    const int cc = min(chunk, C - c0);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;

    // stage rows: LDS row r = (c, ho) <- image row h*sh - ph + ho of channel c0+c
    const int nrows = cc * KH;
    const int hbase = h * g.sh() - g.ph();
    for (int r = wave; r < nrows; r += kIm2colWaves) {
        const int c = r / KH, ho = r - c * KH;
        const int hp = hbase + ho;
        const bool rowok = hp >= 0 && hp < H;
        const float* src = im + ((b * C + c0 + c) * (long)H + (rowok ? hp : 0)) * W;
        float* dst = tile + r * Wp;
        // four loads in flight per lane; padding reads the row's first float and is zeroed
        for (int x0 = lane; x0 < Wp; x0 += 4 * kWave) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int wp = x0 + k * kWave - g.pw();
                v[k] = src[(wp >= 0 && wp < W) ? wp : 0];
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int x = x0 + k * kWave, wp = x - g.pw();
                if (x < Wp) dst[x] = (rowok && wp >= 0 && wp < W) ? v[k] : 0.0f;
            }
        }
    }
    __syncthreads();

    const int KK = KH * KW;
    const int units = cc * KK / UW;          // unit columns this workgroup writes per pixel
    const long Z = (long)C * KK;
    float* orow = col + ((b * m + h) * (long)n) * Z + (long)c0 * KK;
    // few unit columns: several threads share a column and interleave over w
    const int slots = units < kIm2colThreads ? kIm2colThreads / units : 1;
    const int w0 = units < kIm2colThreads ? (int)threadIdx.x / units : 0;
    const int u0 = units < kIm2colThreads ? (int)threadIdx.x % units : (int)threadIdx.x;
    if (w0 >= slots) return;
    const int sw = g.sw();
    for (int u = u0; u < units; u += kIm2colThreads) {
        int off[UW];
#pragma unroll
        for (int j = 0; j < UW; ++j) {
            const int zc = u * UW + j;
            const int c = zc / KK, r = zc - c * KK;
            const int ho = r / KW, wo = r - ho * KW;
            off[j] = (c * KH + ho) * Wp + wo + w0 * sw;
        }
        float* out = orow + (long)w0 * Z + u * UW;
        const int dstep = slots * sw;
        const long ostep = (long)slots * Z;
        for (int w = w0; w < n; w += slots) {
            if (VEC) {
                stream_store4(out, tile[off[0]], tile[off[UW > 1 ? 1 : 0]], tile[off[UW > 2 ? 2 : 0]], tile[off[UW > 3 ? 3 : 0]]);
            } else {
                out[0] = tile[off[0]];
            }
#pragma unroll
            for (int j = 0; j < UW; ++j) off[j] += dstep;
            out += ostep;
        }
    }
}

// Pipelined variant: a workgroup owns one output row (b, h) -- one contiguous
// region of the column buffer -- and walks its channel chunks.  While it
// streams chunk i out of one LDS buffer, the global loads of chunk i+1 are in
// flight into registers and are parked in the other buffer afterwards; one
// barrier per chunk.  The staging offsets of a thread are the same for every
// chunk and are computed once.
// NI = staged floats per thread and chunk: 12 (12 KiB buffers) or 24 (24 KiB).
template <class G, bool VEC, int NI>
__global__ __launch_bounds__(kIm2colThreads) void im2col_pipe_kernel(
    G g, const float* __restrict__ im, float* __restrict__ col, int C, int H, int W, int m, int n,
    int chunk, int nchunks) {
    extern __shared__ float tile[];  // 2 x [chunk*kh][Wp]
    constexpr int UW = VEC ? 4 : 1;
    const int KH = g.kh(), KW = g.kw(), KK = KH * KW;
    const int Wp = W + 2 * g.pw();
    const int rowlen = KH * Wp;                  // staged floats per channel
    const int buflen = chunk * rowlen;           // <= NI * 256
    const long bid = xcd_remap(blockIdx.x, gridDim.x);
    const int h = (int)(bid % m);
    const long b = bid / m;
    const int hbase = h * g.sh() - g.ph();
    const long plane = (long)H * W;

    int soff[NI];                                // image offset inside the chunk, or -1 for padding
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int e = threadIdx.x + i * kIm2colThreads;
        const int c = e / rowlen, rem = e - c * rowlen;
        const int ho = rem / Wp, x = rem - ho * Wp;
        const int hp = hbase + ho, wp = x - g.pw();
        soff[i] = (e < buflen && hp >= 0 && hp < H && wp >= 0 && wp < W) ? (int)(c * plane + hp * W + wp) : -1;
    }
    // Every thread issues all NI loads, padding included (those read the chunk's
    // first float and are zeroed afterwards): a load that some lanes skip sits
    // behind a branch, and the compiler then drains the memory queue before
    // each following load instead of keeping NI of them in flight.
    float reg[NI];
    auto load = [&](int ck) __attribute__((always_inline)) {
        const int c0 = ck * chunk;
        const int lim = min(chunk, C - c0) * rowlen;
        const float* base = im + (b * C + c0) * plane;
        bool ok[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e = threadIdx.x + i * kIm2colThreads;
            ok[i] = soff[i] >= 0 && e < lim;
            reg[i] = base[ok[i] ? soff[i] : 0];
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) reg[i] = ok[i] ? reg[i] : 0.0f;
    };
    auto stash = [&](float* buf) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e = threadIdx.x + i * kIm2colThreads;
            if (e < buflen) buf[e] = reg[i];
        }
    };

    const long Z = (long)C * KK;
    float* orow = col + ((b * m + h) * (long)n) * Z;
    const int sw = g.sw();
    load(0);
    stash(tile);
    __syncthreads();
    for (int ck = 0; ck < nchunks; ++ck) {
        const bool more = ck + 1 < nchunks;
        if (more) load(ck + 1);
        const float* cur = tile + (ck & 1) * buflen;
        const int c0 = ck * chunk;
        const int units = min(chunk, C - c0) * KK / UW;
        const int slots = units < kIm2colThreads ? kIm2colThreads / units : 1;
        const int w0 = units < kIm2colThreads ? (int)threadIdx.x / units : 0;
        const int u0 = units < kIm2colThreads ? (int)threadIdx.x % units : (int)threadIdx.x;
        if (w0 < slots) {
            for (int u = u0; u < units; u += kIm2colThreads) {
                int off[UW];
#pragma unroll
                for (int j = 0; j < UW; ++j) {
                    const int zc = u * UW + j;
                    const int c = zc / KK, r = zc - c * KK;
                    const int ho = r / KW, wo = r - ho * KW;
                    off[j] = (c * KH + ho) * Wp + wo + w0 * sw;
                }
                float* out = orow + (long)w0 * Z + (long)c0 * KK + u * UW;
                const int dstep = slots * sw;
                const long ostep = (long)slots * Z;
                for (int w = w0; w < n; w += slots) {
                    if (VEC) {
                        stream_store4(out, cur[off[0]], cur[off[UW > 1 ? 1 : 0]], cur[off[UW > 2 ? 2 : 0]], cur[off[UW > 3 ? 3 : 0]]);
                    } else {
                        out[0] = cur[off[0]];
                    }
#pragma unroll
                    for (int j = 0; j < UW; ++j) off[j] += dstep;
                    out += ostep;
                }
            }
        }
        if (more) stash(tile + ((ck + 1) & 1) * buflen);
        __syncthreads();
    }
}

// Linear writer.  With ALL channels staged at once, the output of row (b, h) --
// n*Z floats -- is ONE contiguous region of the column buffer, and a workgroup
// writes it front to back as aligned 16-byte units wherever its first float
// falls (Z % 4 != 0, e.g. 3 x 11 x 11 = 363, moves the start from row to row):
// unit q holds floats f = head + 4q .. +3 of the region, float f is pixel f / Z,
// element z = f % Z, and since z = (c*kh + ho)*kw + wo the staged value sits at
// LDS row z / kw, column pixel*sw + z % kw.  Both the staging and the writing
// advance by fixed steps with carries, so there is no division inside a loop.
// The up to three floats before the first and after the last whole unit are
// written singly.  (Splitting a row that does not fit into tiles of pixels, each
// a region of its own, was tried on the VGG mid layer -- 4 tiles of 14 pixels,
// 128 channels x 3 rows x 16 columns staged: 0.157 vs 0.174 ms for the chunked
// kernel launched back to back, but 0.262 vs 0.211 ms where it runs, after the
// previous step's weight-gradient GEMM -- and is not kept; nor is a version of it that walks the
// tiles of a row inside one workgroup with two staging buffers (0.184 ms back to back, 0.276 in
// step): a tile reads the image in 64-byte pieces, which is cheap from the last-level cache, where a
// kernel repeated on the same input finds it, and dear from HBM.)
template <class G, int NI>
__global__ __launch_bounds__(kIm2colThreads) void im2col_linear_kernel(
    G g, const float* __restrict__ im, float* __restrict__ col, int C, int H, int W, int m, int n) {
    extern __shared__ float tile[];  // [C*kh][Wp]
    constexpr int KH = G::kKH, KW = G::kKW, SW = G::kSW;
    static_assert(KW >= 3, "a unit of four floats may carry only once out of the kernel column");
    const unsigned bid = (unsigned)xcd_remap(blockIdx.x, gridDim.x);   // 32-bit: 64-bit divisions cost hundreds of instructions
    const int h = (int)(bid % (unsigned)m);
    const long b = bid / (unsigned)m;
    const int Wp = (n - 1) * SW + KW;            // staged columns: image columns x0 .. x0 + Wp - 1
    const int x0 = -g.pw();
    const int R = C * KH;
    const int buflen = R * Wp;                   // <= NI * 256
    const int hbase = h * g.sh() - g.ph();
    const long plane = (long)H * W;
    const float* base = im + b * C * plane;

    // Element e of the staging area is LDS row e / Wp (= channel * kh + kernel row), column e % Wp.
    // A thread's elements are 256 apart: a fixed step in (channel, kernel row, column) with a carry
    // out of the column and one out of the kernel row; the image offset follows by additions.
    float reg[NI];
    bool ok[NI];
    if constexpr (NI >= 32) {
        // The largest staging areas decode each element by division instead.  That is several times
        // the arithmetic, and measures FASTER there (AlexNet conv1, 30 KB staged: 0.113 vs 0.122 ms):
        // with cheap addresses a workgroup fires its 32 loads per lane in one burst, and the bursts
        // of the resident workgroups crowd the stores of the others, which are what the kernel is
        // bound by.  Small staging areas are latency-bound and prefer the additions (0.016 vs 0.022 ms
        // on a 3 x 32 x 32 input).
        const int rowlen = KH * Wp;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e = threadIdx.x + i * kIm2colThreads;
            const int c = e / rowlen, rem = e - c * rowlen;
            const int ho = rem / Wp, x = rem - ho * Wp;
            const int hp = hbase + ho, wp = x0 + x;
            ok[i] = e < buflen && hp >= 0 && hp < H && wp >= 0 && wp < W;
            reg[i] = base[ok[i] ? (int)(c * plane + hp * W + wp) : 0];
        }
    } else
    {
        // four independent chains (elements i = k, k+4, k+8, ... for k = 0..3), so that the address
        // arithmetic of one load does not wait for the previous one's
        constexpr int NCH = 4;
        static_assert(NI % NCH == 0, "staged elements per thread must split evenly over the chains");
        const int up_x = W - Wp, up_ho = (int)plane - KH * W;
        int x[NCH], c[NCH], ho[NCH], at[NCH];
        auto advance = [&](int k, int dx, int dho, int dc, int dat) __attribute__((always_inline)) {
            x[k] += dx;
            ho[k] += dho;
            c[k] += dc;
            at[k] += dat;
            if (x[k] >= Wp) {
                x[k] -= Wp;
                ++ho[k];
                at[k] += up_x;
            }
            if (ho[k] >= KH) {
                ho[k] -= KH;
                ++c[k];
                at[k] += up_ho;
            }
        };
        {
            const int row0 = (int)threadIdx.x / Wp;
            x[0] = (int)threadIdx.x - row0 * Wp;
            c[0] = row0 / KH;
            ho[0] = row0 - c[0] * KH;
            at[0] = c[0] * (int)plane + (hbase + ho[0]) * W + x0 + x[0];     // C*H*W < 2^31
            const int drow = kIm2colThreads / Wp, dx = kIm2colThreads - drow * Wp;
            const int dc = drow / KH, dho = drow - dc * KH;
            const int dat = dc * (int)plane + dho * W + dx;
#pragma unroll
            for (int k = 1; k < NCH; ++k) {
                x[k] = x[k - 1];
                c[k] = c[k - 1];
                ho[k] = ho[k - 1];
                at[k] = at[k - 1];
                advance(k, dx, dho, dc, dat);
            }
        }
        const int drow = NCH * kIm2colThreads / Wp, dx = NCH * kIm2colThreads - drow * Wp;
        const int dc = drow / KH, dho = drow - dc * KH;
        const int dat = dc * (int)plane + dho * W + dx;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int k = i % NCH;
            const int hp = hbase + ho[k], wp = x0 + x[k];
            ok[i] = c[k] < C && hp >= 0 && hp < H && wp >= 0 && wp < W;
            reg[i] = base[ok[i] ? at[k] : 0];
            advance(k, dx, dho, dc, dat);
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int e = threadIdx.x + i * kIm2colThreads;
        if (e < buflen) tile[e] = ok[i] ? reg[i] : 0.0f;
    }
    __syncthreads();

    const int Z = C * KH * KW;
    const int len = n * Z;                                   // floats in the region
    const long start = (b * m + h) * (long)len;              // col is 16-byte aligned
    float* out = col + start;
    const int head = (int)((4 - (start & 3)) & 3);
    const int nunits = len > head ? (len - head) >> 2 : 0;
    auto value = [&](int w, int z) __attribute__((always_inline)) {
        if (z >= Z) {
            z -= Z;
            ++w;
        }
        const int row = z / KW, wo = z - row * KW;
        return tile[row * Wp + w * SW + wo];
    };
    // First unit of this thread by division, then everything advances by fixed
    // steps: a pass moves on by 4*256 floats = dw pixels, dr LDS rows and dk
    // kernel columns, with a carry from the kernel column into the row and from
    // the row (past the last one, R - 1) into the pixel.  Only the LDS offset is
    // kept up to date; the three floats after the first differ from it by j,
    // plus the same two carries.
    const int up_row = Wp - KW;                  // offset change when the kernel column wraps
    const int up_pix = SW - R * Wp;              // ... when the row wraps into the next pixel
    int f = head + 4 * (int)threadIdx.x;
    int rho, kc, addr;
    {
        const int w = f / Z, z = f - w * Z;
        rho = z / KW;
        kc = z - rho * KW;
        addr = rho * Wp + w * SW + kc;
    }
    const int step = 4 * kIm2colThreads;
    const int dw = step / Z, dz = step - dw * Z;
    const int dr = dz / KW, dk = dz - dr * KW;
    const int da = dw * SW + dr * Wp + dk;
    for (int q = threadIdx.x; q < nunits; q += kIm2colThreads) {
        float v[4];
        v[0] = tile[addr];
        const bool last_row = rho == R - 1;
#pragma unroll
        for (int j = 1; j < 4; ++j) {
            const bool carry = kc + j >= KW;     // one carry at most: kc + 3 < 2 * KW
            int a = addr + j + (carry ? up_row : 0);
            a += (carry && last_row) ? up_pix : 0;
            v[j] = tile[a];
        }
        stream_store4(out + f, v[0], v[1], v[2], v[3]);
        f += step;
        kc += dk;
        const bool c1 = kc >= KW;
        kc -= c1 ? KW : 0;
        rho += dr + (c1 ? 1 : 0);
        addr += da + (c1 ? up_row : 0);
        const bool c2 = rho >= R;
        rho -= c2 ? R : 0;
        addr += c2 ? up_pix : 0;
    }
    // edges: floats [0, head) and [head + 4*nunits, len)
    const int tail0 = head + 4 * nunits;
    const int e = (int)threadIdx.x < head ? (int)threadIdx.x : tail0 + (int)threadIdx.x - head;
    if (e < len && ((int)threadIdx.x < head || e >= tail0)) {
        const int we = e / Z;
        out[e] = value(we, e - we * Z);
    }
}

// Fallback for rows too wide for LDS staging: one thread per output element.
template <class G>
__global__ __launch_bounds__(256) void im2col_direct_kernel(
    G g, const float* __restrict__ im, float* __restrict__ col, long total, int C, int H, int W,
    int m, int n) {
    const int KH = g.kh(), KW = g.kw();
    const long Z = (long)C * KH * KW;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int z = (int)(idx % Z);
        long t = idx / Z;
        const int w = (int)(t % n);
        t /= n;
        const int h = (int)(t % m);
        const long b = t / m;
        const int c = z / (KH * KW), r = z - c * (KH * KW);
        const int ho = r / KW, wo = r - ho * KW;
        const int hp = h * g.sh() - g.ph() + ho, wp = w * g.sw() - g.pw() + wo;
        float v = 0.0f;
        if (hp >= 0 && hp < H && wp >= 0 && wp < W) v = im[((b * C + c) * (long)H + hp) * W + wp];
        col[idx] = v;
    }
}

// One thread per image pixel; taps added in ascending (ho, wo).
template <class G>
__global__ __launch_bounds__(256) void col2im_gather_kernel(
    G g, const float* __restrict__ col, float* __restrict__ im, long total, int C, int H, int W,
    int m, int n) {
    const int KH = g.kh(), KW = g.kw();
    const long Z = (long)C * KH * KW;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int wp = (int)(idx % W);
        long t = idx / W;
        const int hp = (int)(t % H);
        t /= H;
        const int c = (int)(t % C);
        const long b = t / C;
        float acc = 0.0f;
        for (int ho = 0; ho < KH; ++ho) {
            const int hh = hp + g.ph() - ho;
            if (hh < 0) break;
            const int h = hh / g.sh();
            if (h * g.sh() != hh || h >= m) continue;
            for (int wo = 0; wo < KW; ++wo) {
                const int ww = wp + g.pw() - wo;
                if (ww < 0) break;
                const int w = ww / g.sw();
                if (w * g.sw() != ww || w >= n) continue;
                acc += col[((b * m + h) * (long)n + w) * Z + (c * KH + ho) * KW + wo];
            }
        }
        im[idx] = acc;
    }
}


// Streaming col2im for compile-time geometry (stride <= kernel).
//
// A workgroup owns (image b, CC channels, a band of image rows, 64*WSUB image
// columns).  Thread (wave, lane) owns the pixel columns q = wave + 4*i
// (q -> channel q % CC, column block q / CC, column wp0 + 64*block + lane).
// The column-buffer rows h that feed the band are streamed from the highest to
// the lowest: row h adds into image rows h*sh - ph + ho, ho = 0..kh-1, so a
// thread keeps a sliding window of kh accumulators per pixel column, indexed
// by ho (compile-time after unrolling).  After row h the top sh rows of the
// window can receive nothing more: they are written out and the window slides
// down by sh.  For a fixed pixel, descending h is ascending ho and taps inside
// a row are taken in ascending wo, so the adds happen in ascending z exactly
// as in the sequential reference loop -- bit-identical, no atomics.
//
// Each row is staged through LDS as contiguous runs of CC*kh*kw floats
// (coalesced; the buffer is read once apart from kh-sh halo rows per band and
// the kw-sw halo columns per tile).  Two rows are in flight in registers: the
// loads of row h-2 are issued right after row h is parked in LDS.
//
// Staging modes: kStageScalar (4-byte loads), kStageRuns (16-byte loads inside
// each run; needs CC*kh*kw % 4 == 0 and C % CC == 0), kStageLinear (CC == C, so
// the runs of neighbouring pixels are adjacent in memory and a row's staged
// pixels are ONE contiguous block: it is copied with 16-byte loads from the
// 16-byte boundary below its first float, whatever its alignment, and lands in
// LDS at the same offset from that boundary, with no index arithmetic at all).
constexpr int kStageScalar = 0, kStageRuns = 1, kStageLinear = 2;
constexpr int kRowBatch = 8;   // image rows collected per channel before they are written (a multiple of every static stride)

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>());
    }
}

//
// LW = lanes along the image row per wavefront (64, 32 or 16): narrow images
// (CIFAR's 15-wide feature maps) put 64/LW channels side by side in a
// wavefront instead of leaving lanes idle.
template <class G, int CC, int WSUB, int MODE, int LW = 64, bool BATCH = false>
__global__ __launch_bounds__(256) void col2im_stream_kernel(
    G g, const float* __restrict__ col, float* __restrict__ im, int C, int H, int W, int m, int n,
    int band, int bands, int tiles_w, int nchunks, int out_off) {
    constexpr bool VEC = MODE == kStageRuns, LIN = MODE == kStageLinear;
    constexpr int KH = G::kKH, KW = G::kKW, PH = G::kPH, PW = G::kPW, SH = G::kSH, SW = G::kSW;
    static_assert(SH <= KH && SW <= KW, "streaming col2im needs stride <= kernel");
    constexpr int KK = KH * KW, RUN = CC * KK;
    constexpr int LD = RUN | 1;                       // odd row stride: conflict-free column reads
    constexpr int CSUB = 64 / LW;                     // channels side by side in a wavefront
    static_assert(CC % CSUB == 0, "channel chunk must be a multiple of the channels per wavefront");
    constexpr int CG = CC / CSUB;                     // channel groups per chunk
    constexpr int TW = LW * WSUB;
    constexpr int NQ = (CG * WSUB + 3) / 4;
    constexpr int NT = (KW + SW - 1) / SW;            // taps per row and pixel
    constexpr int NWB = (TW + KW - 2) / SW + 1;       // staged pixels per row, upper bound
    // staged values per thread: float4 units of full runs (VEC) or single floats
    constexpr int NP = LIN ? ((NWB * RUN + 6) / 4 + 255) / 256
                     : VEC ? (NWB * (RUN / 4) + 255) / 256 : (NWB * RUN + 255) / 256;
    static_assert(!LIN || LD == RUN, "linear staging keeps the memory layout: the run length must be odd");
    extern __shared__ __attribute__((aligned(16))) float stage[];   // [nw][LD] (+ up to 3 floats of lead-in)

    long bid = xcd_remap(blockIdx.x, gridDim.x);
    const int bd = (int)(bid % bands);                // bands of one image/chunk are neighbours
    bid /= bands;
    const int wt = (int)(bid % tiles_w);
    bid /= tiles_w;
    const int ck = (int)(bid % nchunks);
    // Images are taken last to first.  col2im follows the GEMM that wrote the column buffer,
    // front to back; what that left in the 256 MB last-level cache is the END of the buffer, and
    // a consumer that starts at the front has pushed it out before it gets there (in-step time on
    // the VGG layer 0.249 -> 0.231 ms, AlexNet conv1 0.178 -> 0.167 ms; launched on its own the
    // order makes no difference).
    const long nimages = gridDim.x / ((unsigned)bands * tiles_w * nchunks);
    const long b = nimages - 1 - bid / nchunks;
    const int hp0 = bd * band, hp1 = min(H, hp0 + band);
    const int wp0 = wt * TW, c0 = ck * CC;
    const int cc = min(CC, C - c0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long Z = (long)C * KK;

    const int wl = wp0 + PW - (KW - 1);
    const int w_lo = wl > 0 ? (wl + SW - 1) / SW : 0;
    const int w_hi = min(n - 1, (wp0 + TW - 1 + PW) / SW);
    const int nw = w_hi - w_lo + 1;
    const bool full = (cc == CC);                     // VEC is only launched when C % CC == 0
    const int run = cc * KK;
    const int total = VEC ? nw * (RUN / 4) : nw * run;

    int cq[NQ], wp[NQ];
    bool ok[NQ];
    float acc[NQ][KH];
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
        const int q = wave + 4 * i;
        cq[i] = (q % CG) * CSUB + lane / LW;
        wp[i] = wp0 + (q / CG) * LW + lane % LW;
        ok[i] = (q < CG * WSUB) && (cq[i] < cc) && (wp[i] < W);
#pragma unroll
        for (int j = 0; j < KH; ++j) acc[i][j] = 0.0f;
    }

    // rows h_top .. h_bot cover every image row of the band; rows outside
    // [0, m) contribute nothing but still slide the window
    const int h_top = (hp1 - 1 + PH) / SH;
    const int t_bot = hp0 + PH - (KH - 1);
    const int h_bot = t_bot >= 0 ? (t_bot + SH - 1) / SH : -((-t_bot) / SH);

    // Live rows are those inside [0, m); the ones outside only slide the window.
    int live_hi = min(h_top, m - 1), live_lo = max(h_bot, 0);
    if (nw <= 0 || live_hi < live_lo) {               // nothing to read: slide through the whole range
        live_hi = h_bot - 1;
        live_lo = h_bot;
    }

    // Staging is branch-free: every thread issues all NP loads of a row (indices
    // past the end are clamped to the last unit, whose value then lands twice in
    // the same LDS slot) and parks all of them.  A load that some lanes skip
    // leaves its destination registers "possibly in flight" on the skipped
    // path, and every later load into them then has to wait for the memory
    // pipeline to drain; with straight-line code the waits count loads instead.
    typedef typename std::conditional<VEC || LIN, v4f, float>::type PreT;
    PreT pre0[NP], pre1[NP];        // two rows in flight
    int lead = 0, lead0 = 0, lead1 = 0;   // LIN: floats between the 16-byte boundary and the row's first float
    auto prefetch = [&](PreT (&pre)[NP], int& lead_next, int h) __attribute__((always_inline)) {
        const float* src = col + ((b * m + h) * (long)n + w_lo) * Z + (long)c0 * KK;
        if constexpr (LIN) {
            // col is 16-byte aligned and holds a multiple of 4 floats, so every
            // aligned unit that starts inside the buffer lies inside it
            lead_next = (int)((reinterpret_cast<uintptr_t>(src) >> 2) & 3);
            const v4f* al = reinterpret_cast<const v4f*>(src - lead_next);
            const int last = ((nw * RUN + lead_next + 3) >> 2) - 1;
#pragma unroll
            // A row's staged block is read by this workgroup alone (but for the halo pixels it shares with
            // the tile beside it) and never again: non-temporal loads keep it from displacing what the
            // kernels around this one left in the caches (AlexNet conv1, in step: 0.176 -> 0.141 ms).  The
            // run-wise staging below keeps plain loads: its 288-byte pieces share cache lines with the
            // pieces of the neighbouring channel chunks (VGG layer: 0.231 -> 0.249 ms with non-temporal ones).
            for (int u = 0; u < NP; ++u) pre[u] = __builtin_nontemporal_load(al + min((int)threadIdx.x + u * 256, last));
        } else {
#pragma unroll
            for (int u = 0; u < NP; ++u) {
                const int idx = min((int)threadIdx.x + u * 256, total - 1);
                if constexpr (VEC) {
                    const int w = idx / (RUN / 4), z4 = (idx - w * (RUN / 4)) * 4;
                    pre[u] = *reinterpret_cast<const v4f*>(src + (long)w * Z + z4);
                } else {
                    const int w = full ? idx / RUN : idx / run;
                    const int zc = idx - w * run;
                    pre[u] = src[(long)w * Z + zc];
                }
            }
        }
    };
    auto park = [&](const PreT (&pre)[NP], int lead_next) __attribute__((always_inline)) {
        if constexpr (LIN) {
            lead = lead_next;                         // the staging area holds NP * 256 units
#pragma unroll
            for (int u = 0; u < NP; ++u) reinterpret_cast<v4f*>(stage)[threadIdx.x + u * 256] = pre[u];
        } else {
#pragma unroll
            for (int u = 0; u < NP; ++u) {
                const int idx = min((int)threadIdx.x + u * 256, total - 1);
                if constexpr (VEC) {
                    const int w = idx / (RUN / 4), z4 = (idx - w * (RUN / 4)) * 4;
                    float* d = stage + w * LD + z4;
                    d[0] = pre[u].x; d[1] = pre[u].y; d[2] = pre[u].z; d[3] = pre[u].w;
                } else {
                    const int w = full ? idx / RUN : idx / run;
                    const int zc = idx - w * run;
                    stage[w * LD + zc] = pre[u];
                }
            }
        }
    };

    // Finished image rows leave the window from the top of the band downwards.
    // Written one by one they are short stores (W floats per wavefront
    // instruction, a tenth of the kernel's bytes but a quarter of its time);
    // with BATCH (the tile spans the whole image width, so a channel's rows are
    // adjacent in memory) they are collected in LDS, kRowBatch rows of every
    // channel of the chunk, and each channel's batch is written as one linear
    // region in aligned, streamed 16-byte units.
    constexpr int RB = kRowBatch;
    float* obuf = stage + out_off;                    // [CC][RB][W]
    int batch_lo = hp0 + (hp1 - 1 - hp0) / RB * RB;   // lowest row of the batch being collected
    auto write_batch = [&]() __attribute__((always_inline)) {
        const int rows = min(batch_lo + RB, hp1) - batch_lo;
        const int nfl = rows * W;
        __syncthreads();
        for (int c = wave; c < cc; c += 4) {
            const long g0 = ((b * C + c0 + c) * (long)H + batch_lo) * W;   // im is 16-byte aligned
            float* dst = im + g0;
            const float* src = obuf + c * RB * W;
            const int head = min((int)((4 - (g0 & 3)) & 3), nfl);
            const int nunits = (nfl - head) >> 2;
            for (int u = lane; u < nunits; u += 64) {
                const int e = head + 4 * u;
                stream_store4(dst + e, src[e], src[e + 1], src[e + 2], src[e + 3]);
            }
            const int tail0 = head + 4 * nunits;
            if (lane < head) dst[lane] = src[lane];
            if (tail0 + lane < nfl) dst[tail0 + lane] = src[tail0 + lane];
        }
        __syncthreads();
    };
    // one finished image row: ho is the window slot that holds it
    auto emit_row = [&](int hp, auto slot) __attribute__((always_inline)) {
        constexpr int ho = decltype(slot)::value;
        if (hp < hp0 || hp >= hp1) return;            // uniform over the workgroup
        if constexpr (BATCH) {
            if (hp < batch_lo) {
                write_batch();
                batch_lo -= RB;
            }
#pragma unroll
            for (int i = 0; i < NQ; ++i)
                if (ok[i]) obuf[(cq[i] * RB + hp - batch_lo) * W + wp[i]] = acc[i][ho];
        } else {
#pragma unroll
            for (int i = 0; i < NQ; ++i)
                if (ok[i]) im[(((b * C + c0 + cq[i]) * (long)H) + hp) * W + wp[i]] = acc[i][ho];
        }
    };
    // image rows h*SH - PH + ho, ho >= KH - SH, can receive nothing from the rows
    // below h: emit them (highest first) and slide the window down by SH
    auto flush = [&](int h) __attribute__((always_inline)) {
        const int base = h * SH - PH;
        static_for<SH>([&](auto k) { emit_row(base + KH - 1 - k, std::integral_constant<int, KH - 1 - decltype(k)::value>()); });
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
#pragma unroll
            for (int ho = KH - 1; ho >= SH; --ho) acc[i][ho] = acc[i][ho - SH];
#pragma unroll
            for (int ho = 0; ho < SH; ++ho) acc[i][ho] = 0.0f;
        }
    };

    // one live column-buffer row: park it (its loads were issued two rows ago),
    // refill the same registers with the row two below, then consume it from LDS
    // STEADY: the row two below is known to be live, so the refill is unconditional
    auto row_step = [&](auto steady, PreT (&pre)[NP], int& lead_slot, int h) __attribute__((always_inline)) {
        park(pre, lead_slot);
        __syncthreads();
        if (decltype(steady)::value || h - 2 >= live_lo) prefetch(pre, lead_slot, h - 2);
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            if (!ok[i]) continue;
            // tap t of pixel column wp: wo = r + t*SW from staged pixel wq - t;
            // for one accumulator the taps come in ascending wo
            const int wpp = wp[i] + PW;
            const int r = wpp % SW, wq = wpp / SW;
            const float* sp = stage + lead + (wq - w_lo) * LD + cq[i] * KK + r;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int wo = r + t * SW, w = wq - t;
                if (wo < KW && w >= 0 && w <= w_hi) {
                    const float* st = sp + t * (SW - LD);
#pragma unroll
                    for (int ho = 0; ho < KH; ++ho) acc[i][ho] += st[ho * KW];
                }
            }
        }
        __syncthreads();
        flush(h);
    };
    for (int hd = h_top; hd > live_hi; --hd) flush(hd);
    // The steady loop has no branch around a load: where a load is skipped on
    // some path, the compiler must assume on the other that nothing was issued
    // after it and waits for the whole queue, which would leave one row in
    // flight instead of two.  The last rows run in a second, conditional loop.
    int h = live_hi;
    if (h - 3 >= live_lo) {
        prefetch(pre0, lead0, h);
        __builtin_amdgcn_sched_barrier(0);            // keep the issue order the loop's waits count on
        prefetch(pre1, lead1, h - 1);
        __builtin_amdgcn_sched_barrier(0);
        for (; h - 3 >= live_lo; h -= 2) {
            row_step(std::true_type(), pre0, lead0, h);
            row_step(std::true_type(), pre1, lead1, h - 1);
        }
    } else if (h >= live_lo) {
        prefetch(pre0, lead0, h);
        if (h - 1 >= live_lo) prefetch(pre1, lead1, h - 1);
    }
    for (; h >= live_lo; h -= 2) {
        row_step(std::false_type(), pre0, lead0, h);
        if (h - 1 >= live_lo) row_step(std::false_type(), pre1, lead1, h - 1);
    }
    for (int hd = live_lo - 1; hd >= h_bot; --hd) flush(hd);
    // rows of the band below the lowest window (still open in the window)
    const int base = (h_bot - 1) * SH - PH;
    static_for<KH - SH>([&](auto k) { emit_row(base + KH - 1 - k, std::integral_constant<int, KH - 1 - decltype(k)::value>()); });
    if constexpr (BATCH) write_batch();
}

template <class G, int CC, int WSUB, int LW = 64>
static int launch_col2im_stream(G g, const float* col, long B, int C, int H, int W, int m, int n,
                                float* im, hipStream_t st) {
    constexpr int KK = G::kKH * G::kKW, RUN = CC * KK, LD = RUN | 1, TW = LW * WSUB;
    const int tiles_w = (int)cdiv(W, TW), nchunks = (int)cdiv(C, CC);
    const long nwb = std::min((long)n, (long)(TW + G::kKW - 2) / G::kSW + 1);
    // linear staging parks NP * 256 aligned 16-byte units whatever the row needs
    constexpr int NWB = (TW + G::kKW - 2) / G::kSW + 1;
    constexpr size_t lin_units = (size_t)(((NWB * RUN + 6) / 4 + 255) / 256) * 256;
    size_t lds = std::max(((size_t)nwb * LD + 8) * sizeof(float), LD == RUN ? lin_units * 16 : 0);
    CGT_ARG_CHECK(lds <= 64 * 1024, "col2im: tile configuration out of range");
    const long Z = (long)C * KK;
    const long col_floats = B * m * (long)n * Z;
    const bool al16 = reinterpret_cast<uintptr_t>(col) % 16 == 0;
    const int mode = (LD == RUN && C == CC && al16 && col_floats % 4 == 0) ? kStageLinear
                     : (RUN % 4 == 0 && C % CC == 0 && al16) ? kStageRuns : kStageScalar;
    // a tile as wide as the image: finished rows are batched in LDS behind the staging area
    const size_t out_off = (lds / sizeof(float) + 3) / 4 * 4;
    const size_t lds_batch = (out_off + (size_t)CC * kRowBatch * W) * sizeof(float);
    // (not for narrow images: a batch of a 15-wide plane is a few hundred bytes, and the two
    // extra barriers per batch cost more than the stores gain -- 0.019 vs 0.016 ms on CIFAR conv2)
    const bool batch = tiles_w == 1 && W >= 32 && reinterpret_cast<uintptr_t>(im) % 16 == 0 && lds_batch <= 40 * 1024;
    if (batch) lds = lds_batch;
    constexpr int M_LIN = LD == RUN ? kStageLinear : kStageScalar, M_RUNS = RUN % 4 == 0 ? kStageRuns : kStageScalar;
    auto kernel = batch ? (mode == kStageLinear ? col2im_stream_kernel<G, CC, WSUB, M_LIN, LW, true>
                           : mode == kStageRuns ? col2im_stream_kernel<G, CC, WSUB, M_RUNS, LW, true>
                                                : col2im_stream_kernel<G, CC, WSUB, kStageScalar, LW, true>)
                        : (mode == kStageLinear ? col2im_stream_kernel<G, CC, WSUB, M_LIN, LW, false>
                           : mode == kStageRuns ? col2im_stream_kernel<G, CC, WSUB, M_RUNS, LW, false>
                                                : col2im_stream_kernel<G, CC, WSUB, kStageScalar, LW, false>);
    // Bands of image rows: as many workgroups as the chip holds at once, and
    // no more.  A second, partial round of workgroups costs more than it gains
    // (measured on the AlexNet layer: 1 or 2 bands 0.145 ms, 3 or 4 bands
    // 0.153 ms), and each band re-reads kh - sh halo rows, so bands stay at
    // least 2 kernel heights tall.
    int wg_per_cu = 0;
    CGT_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&wg_per_cu, kernel, 256, lds));
    const long resident = (long)std::max(wg_per_cu, 1) * kNumCU;
    const long per_band = B * nchunks * tiles_w;
    long bands = std::max(1L, std::min(resident / per_band, (long)H / (2 * G::kKH)));
    const int band = (int)cdiv(cdiv(H, bands), G::kSH) * G::kSH;   // bands start on stride multiples
    bands = cdiv(H, band);
    const long blocks = per_band * bands;
    CGT_ARG_CHECK(blocks < (1L << 31), "col2im: too many workgroups");
    kernel<<<dim3((unsigned)blocks), dim3(256), lds, st>>>(g, col, im, C, H, W, m, n, band, (int)bands,
                                                           tiles_w, nchunks, (int)out_off);
    CGT_LAUNCH_CHECK("col2im_stream_kernel");
    return CGT_AMD_OK;
}

static int check_geom(const char* what, long B, long C, long H, long W, int kh, int kw, int ph,
                      int pw, int sh, int sw, long* m, long* n) {
    CGT_ARG_CHECK(B >= 0 && C >= 0 && H >= 0 && W >= 0, "%s: negative shape", what);
    CGT_ARG_CHECK(kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0,
                  "%s: bad geometry k=(%d,%d) p=(%d,%d) s=(%d,%d)", what, kh, kw, ph, pw, sh, sw);
    CGT_ARG_CHECK(H + 2 * ph >= kh && W + 2 * pw >= kw, "%s: kernel larger than padded image", what);
    *m = (H + 2 * ph - kh) / sh + 1;
    *n = (W + 2 * pw - kw) / sw + 1;
    CGT_ARG_CHECK(C * H * W < (1L << 31) && (*m) * (*n) * C * kh * kw < (1L << 40) &&
                      H < (1 << 24) && W < (1 << 24) && C < (1 << 24),
                  "%s: shape too large", what);
    return CGT_AMD_OK;
}

static int gcd4(int v) { return (v % 4 == 0) ? 4 : (v % 2 == 0) ? 2 : 1; }

// the linear writer needs the kernel width at compile time, and at least 3
template <class G>
constexpr bool linear_writer_ok() {
    if constexpr (G::is_static) return G::kKW >= 3;
    else return false;
}

template <class G>
static int launch_im2col(G g, const float* im, long B, int C, int H, int W, int m, int n,
                         float* col, hipStream_t st) {
    const int KK = g.kh() * g.kw();
    const long Z = (long)C * KK;
    const int Wp = W + 2 * g.pw();
    const long rowlen = (long)g.kh() * Wp;                // staged floats per channel
    const bool aligned = (Z % 4 == 0) && (reinterpret_cast<uintptr_t>(col) % 16 == 0);
    const int step = 4 / gcd4(KK);       // smallest channel count whose z-run is a multiple of 4 floats
    if (B * m * n * Z == 0) return CGT_AMD_OK;

    // 1. pipelined kernel: a chunk of channels must fit one staging buffer (24 KiB).
    //    Long z-runs matter (measured: 1152-byte runs stream ~25 % faster than
    //    576-byte ones), and so do equal chunks.
    const long cap = 24 * kIm2colThreads;
    if (rowlen <= cap && B * m < (1L << 31) && C * (long)H * W < (1L << 31)) {
        int chunk = (int)std::min((long)C, cap / rowlen);
        bool vec = aligned;
        if (vec && chunk < C) {
            if (chunk >= step) chunk = chunk / step * step;
            else vec = false;
        }
        if (chunk < C) {
            // prefer a chunk that divides C, if one lies within 25 % of the largest
            const int st2 = vec ? step : 1;
            for (int c = chunk; c >= 1 && 4 * c >= 3 * chunk; c -= st2)
                if (C % c == 0) {
                    chunk = c;
                    break;
                }
        }
        // all channels in one 32 KiB buffer, if two 24 KiB ones would need a second pass:
        // a pixel's whole row of the column buffer is then written in one go (AlexNet
        // conv1: 3 x 11 x 227 floats = 30 KB; 1452-byte rows written once instead of as
        // 968 + 484 bytes in two phases that meet again only in L2 -- or not)
        const bool whole = chunk < C && C * rowlen <= 32 * kIm2colThreads;
        if (whole) {
            chunk = C;
            vec = aligned;
        }
        const int nchunks = (int)cdiv(C, chunk);
        const size_t lds = (nchunks > 1 ? 2 : 1) * (size_t)chunk * rowlen * sizeof(float);
        const long blocks = B * m;
        const bool small = (long)chunk * rowlen <= 12 * kIm2colThreads;
        dim3 grid((unsigned)blocks), block(kIm2colThreads);
        if constexpr (linear_writer_ok<G>()) {
            // all channels' rows staged at once (32 KiB), the output row written as one linear region
            const long staged = (long)C * g.kh() * ((long)(n - 1) * g.sw() + g.kw());
            if (staged <= 32L * kIm2colThreads && reinterpret_cast<uintptr_t>(col) % 16 == 0 && n * Z < (1L << 30)) {
                const size_t lds_lin = (size_t)staged * sizeof(float);
                if (staged <= 12 * kIm2colThreads)
                    im2col_linear_kernel<G, 12><<<grid, block, lds_lin, st>>>(g, im, col, C, H, W, m, n);
                else if (staged <= 24 * kIm2colThreads)
                    im2col_linear_kernel<G, 24><<<grid, block, lds_lin, st>>>(g, im, col, C, H, W, m, n);
                else
                    im2col_linear_kernel<G, 32><<<grid, block, lds_lin, st>>>(g, im, col, C, H, W, m, n);
                CGT_LAUNCH_CHECK("im2col_linear_kernel");
                return CGT_AMD_OK;
            }
        }
        if (whole && vec)
            im2col_pipe_kernel<G, true, 32><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        else if (whole)
            im2col_pipe_kernel<G, false, 32><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        else if (vec && small)
            im2col_pipe_kernel<G, true, 12><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        else if (vec)
            im2col_pipe_kernel<G, true, 24><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        else if (small)
            im2col_pipe_kernel<G, false, 12><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        else
            im2col_pipe_kernel<G, false, 24><<<grid, block, lds, st>>>(g, im, col, C, H, W, m, n, chunk, nchunks);
        CGT_LAUNCH_CHECK("im2col_pipe_kernel");
        return CGT_AMD_OK;
    }

    // 2. wide rows: one workgroup per (b, h, chunk), rows staged in up to 48 KiB of LDS
    const long row_bytes = rowlen * (long)sizeof(float);
    const long lds_budget = 48 * 1024;
    if (row_bytes <= lds_budget && B * m < (1L << 31) / 64) {
        int chunk = (int)std::min((long)C, lds_budget / row_bytes);
        bool vec = aligned;
        if (vec && chunk < C) {
            if (chunk >= step) chunk = chunk / step * step;
            else vec = false;
        }
        const int nchunks = (int)cdiv(C, chunk);
        const size_t lds = (size_t)chunk * row_bytes;
        const long blocks = B * m * nchunks;
        if (vec)
            im2col_rows_kernel<G, true><<<dim3((unsigned)blocks), dim3(kIm2colThreads), lds, st>>>(
                g, im, col, C, H, W, m, n, chunk, nchunks);
        else
            im2col_rows_kernel<G, false><<<dim3((unsigned)blocks), dim3(kIm2colThreads), lds, st>>>(
                g, im, col, C, H, W, m, n, chunk, nchunks);
        CGT_LAUNCH_CHECK("im2col_rows_kernel");
        return CGT_AMD_OK;
    }

    // 3. anything else: one thread per output element
    const long total = B * m * n * Z;
    long blocks = cdiv(total, 256);
    if (blocks > 1 << 20) blocks = 1 << 20;
    im2col_direct_kernel<G><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(g, im, col, total, C, H, W, m, n);
    CGT_LAUNCH_CHECK("im2col_direct_kernel");
    return CGT_AMD_OK;
}

// Tiling of col2im_stream_kernel per compile-time geometry: <channels per chunk,
// 64-column blocks per tile>.  Returns -1 when the shape
// is better served by the plain gather kernel.
template <class G>
static int try_col2im_stream(G, const float*, long, int, int, int, int, int, float*, hipStream_t) {
    return -1;
}
static int try_col2im_stream(StaticGeom<3, 3, 1, 1, 1, 1> g, const float* col, long B, int C, int H,
                           int W, int m, int n, float* im, hipStream_t st) {
    if (C >= 8 && W >= 24) return launch_col2im_stream<decltype(g), 8, 1>(g, col, B, C, H, W, m, n, im, st);
    if (C >= 8 && W <= 16) return launch_col2im_stream<decltype(g), 8, 1, 16>(g, col, B, C, H, W, m, n, im, st);
    if (C >= 8) return launch_col2im_stream<decltype(g), 8, 1, 32>(g, col, B, C, H, W, m, n, im, st);
    return -1;
}
static int try_col2im_stream(StaticGeom<3, 3, 0, 0, 1, 1> g, const float* col, long B, int C, int H,
                           int W, int m, int n, float* im, hipStream_t st) {
    if (C >= 8 && W >= 24) return launch_col2im_stream<decltype(g), 8, 1>(g, col, B, C, H, W, m, n, im, st);
    return -1;
}
static int try_col2im_stream(StaticGeom<5, 5, 2, 2, 1, 1> g, const float* col, long B, int C, int H,
                           int W, int m, int n, float* im, hipStream_t st) {
    if (C >= 4 && W >= 24) return launch_col2im_stream<decltype(g), 4, 1>(g, col, B, C, H, W, m, n, im, st);
    if (C == 3 && W >= 24) return launch_col2im_stream<decltype(g), 3, 1>(g, col, B, C, H, W, m, n, im, st);   // RGB input layer
    if (C >= 8 && W <= 16) return launch_col2im_stream<decltype(g), 8, 1, 16>(g, col, B, C, H, W, m, n, im, st);
    if (C >= 4) return launch_col2im_stream<decltype(g), 4, 1, 32>(g, col, B, C, H, W, m, n, im, st);
    return -1;
}
static int try_col2im_stream(StaticGeom<11, 11, 0, 0, 4, 4> g, const float* col, long B, int C, int H,
                           int W, int m, int n, float* im, hipStream_t st) {
    if (C == 3 && W >= 64) return launch_col2im_stream<decltype(g), 3, 1>(g, col, B, C, H, W, m, n, im, st);
    return -1;
}

template <class G>
static int launch_col2im(G g, const float* col, long B, int C, int H, int W, int m, int n,
                         float* im, hipStream_t st) {
    const long total = B * C * H * W;
    if (total == 0) return CGT_AMD_OK;
    {
        const int rc = try_col2im_stream(g, col, B, C, H, W, m, n, im, st);
        if (rc >= 0) return rc;
    }
    long blocks = cdiv(total, 256);
    if (blocks > 1 << 20) blocks = 1 << 20;
    col2im_gather_kernel<G><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(g, col, im, total, C, H, W, m, n);
    CGT_LAUNCH_CHECK("col2im_gather_kernel");
    return CGT_AMD_OK;
}

// Geometries compiled with constant index math: (kh, kw, ph, pw, sh, sw).
#define CGT_STATIC_GEOMS(X) \
    X(3, 3, 1, 1, 1, 1)     \
    X(5, 5, 2, 2, 1, 1)     \
    X(11, 11, 0, 0, 4, 4)   \
    X(3, 3, 0, 0, 1, 1)     \
    X(1, 1, 0, 0, 1, 1)

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_im2col_f32(const float* im, long B, long C, long H, long W, int kh, int kw,
                               int ph, int pw, int sh, int sw, float* col, void* stream) {
    long m, n;
    int rc = check_geom("im2col", B, C, H, W, kh, kw, ph, pw, sh, sw, &m, &n);
    if (rc) return rc;
    if (B * m * n * C == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(im && col, "im2col: null pointer");
    hipStream_t st = as_stream(stream);
#define X(KH, KW, PH, PW, SH, SW)                                                     \
    if (kh == KH && kw == KW && ph == PH && pw == PW && sh == SH && sw == SW)         \
        return launch_im2col(StaticGeom<KH, KW, PH, PW, SH, SW>(), im, B, (int)C, (int)H, (int)W, \
                             (int)m, (int)n, col, st);
    CGT_STATIC_GEOMS(X)
#undef X
    return launch_im2col(DynGeom{kh, kw, ph, pw, sh, sw}, im, B, (int)C, (int)H, (int)W, (int)m,
                         (int)n, col, st);
}

CGT_API int cgt_amd_col2im_f32(const float* col, long B, long C, long H, long W, int kh, int kw,
                               int ph, int pw, int sh, int sw, float* im, void* stream) {
    long m, n;
    int rc = check_geom("col2im", B, C, H, W, kh, kw, ph, pw, sh, sw, &m, &n);
    if (rc) return rc;
    if (B * C * H * W == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(im && col, "col2im: null pointer");
    hipStream_t st = as_stream(stream);
#define X(KH, KW, PH, PW, SH, SW)                                                     \
    if (kh == KH && kw == KW && ph == PH && pw == PW && sh == SH && sw == SW)         \
        return launch_col2im(StaticGeom<KH, KW, PH, PW, SH, SW>(), col, B, (int)C, (int)H, (int)W, \
                             (int)m, (int)n, im, st);
    CGT_STATIC_GEOMS(X)
#undef X
    return launch_col2im(DynGeom{kh, kw, ph, pw, sh, sw}, col, B, (int)C, (int)H, (int)W, (int)m,
                         (int)n, im, st);
}
