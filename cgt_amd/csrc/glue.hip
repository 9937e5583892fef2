// Conv glue: 4-d axis permutation.  conv2d applies {0,3,1,2} to the GEMM
// output and its pullback applies {0,2,3,1}; both are batched 2-d transposes
// and go through an LDS tile so reads and writes are both contiguous runs.
#include "common.h"
#include <algorithm>
#include <type_traits>

namespace cgt_amd {

constexpr int kTile = 64;  // 64x64 floats; +1 column of padding keeps LDS reads conflict-free

// out[b][c][r] = in[b][r][c], in is [B, R, Cn]
__global__ __launch_bounds__(256) void batched_transpose_kernel(
    const float* __restrict__ in, float* __restrict__ out, int R, int Cn, int tiles_r, int tiles_c) {
    __shared__ float tile[kTile][kTile + 1];
    long bid = blockIdx.x;
    const int tc = (int)(bid % tiles_c);
    bid /= tiles_c;
    const int tr = (int)(bid % tiles_r);
    const long b = bid / tiles_r;
    const float* src = in + b * (long)R * Cn;
    float* dst = out + b * (long)R * Cn;
    const int lx = threadIdx.x % kTile, ly = threadIdx.x / kTile;  // 64 x 4
    const int r0 = tr * kTile, c0 = tc * kTile;
    // all 16 loads of a thread are issued before the first LDS store; rows and
    // columns past the edge are clamped, not skipped, so no load is conditional
    float v[kTile / 4];
    const int c = min(c0 + lx, Cn - 1);
#pragma unroll
    for (int k = 0; k < kTile / 4; ++k) v[k] = src[(long)min(r0 + ly + 4 * k, R - 1) * Cn + c];
#pragma unroll
    for (int k = 0; k < kTile / 4; ++k) tile[ly + 4 * k][lx] = v[k];
    __syncthreads();
    for (int i = ly; i < kTile; i += 4) {
        const int c = c0 + i, r = r0 + lx;
        if (r < R && c < Cn) dst[(long)c * R + r] = tile[lx][i];
    }
}


// Thin case: one of the two transposed extents (L) is small, as in the conv
// glue where L is the filter count.  A workgroup takes kThinRows positions of
// the long axis and ALL of L, so the side whose rows are L long is one
// contiguous block of kThinRows*L floats (16-byte accesses when L % 4 == 0),
// and the other side is L runs of kThinRows floats.
//   L_INNER_IN:  in [B, R, L] -> out [B, L, R]
//   otherwise:   in [B, L, R] -> out [B, R, L]
constexpr int kThinRows = 64;
constexpr int kThinMaxL = 128;

// Workgroups go to the 8 XCDs round-robin by id; give each XCD (one L2) a
// contiguous range of ids, so the workgroups that share a cache line where
// their unaligned runs meet find it in the same L2.
__device__ __forceinline__ unsigned xcd_contiguous(unsigned id, unsigned n) {
    const unsigned q = n / kNumXCD, r = n % kNumXCD;
    const unsigned xcd = id % kNumXCD, local = id / kNumXCD;
    return xcd * q + min(xcd, r) + local;
}

__device__ __forceinline__ int div_small(int n, int d, float rd) {
    // exact for 0 <= n < 2^21: the float quotient is off by at most one
    int q = (int)((float)n * rd);
    const int r = n - q * d;
    q += (r >= d) - (r < 0);
    return q;
}

template <bool L_INNER_IN, bool VEC>
__global__ __launch_bounds__(256) void thin_transpose_kernel(const float* __restrict__ in,
                                                             float* __restrict__ out, int R, int L,
                                                             int tiles_r) {
    extern __shared__ float tile[];          // [kThinRows][LD]
    const int LD = L | 1;
    const unsigned bid = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tr = bid % tiles_r;
    const long b = bid / tiles_r;
    const int r0 = tr * kThinRows;
    const int rows = min(kThinRows, R - r0);
    const float rL = 1.0f / (float)L;
    const float* src = in + b * (long)R * L;
    float* dst = out + b * (long)R * L;
    // the side with rows of length L: block of rows*L contiguous floats
    const float* blk_in = src + (long)r0 * L;
    float* blk_out = dst + (long)r0 * L;
    const int n = rows * L;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (L_INNER_IN) {
        // All loads of a pass are issued before the first LDS store, and none is
        // skipped (indices past the end are clamped): a load that some lanes skip
        // makes the compiler wait for the whole memory queue before the next one.
        if (VEC) {
            constexpr int U = kThinRows * kThinMaxL / 1024;      // covers the largest block in one pass
            v4f v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const v4f*>(blk_in + min((int)threadIdx.x * 4 + u * 1024, n - 4));
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = threadIdx.x * 4 + u * 1024;
                if (i < n) {
                    const int r = div_small(i, L, rL), c = i - r * L;
                    float* t = tile + r * LD + c;
                    t[0] = v[u].x; t[1] = v[u].y; t[2] = v[u].z; t[3] = v[u].w;
                }
            }
        } else {
            constexpr int U = 8;
            for (int i0 = threadIdx.x; i0 < n; i0 += 256 * U) {
                float v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = blk_in[min(i0 + u * 256, n - 1)];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int i = i0 + u * 256;
                    if (i < n) {
                        const int r = div_small(i, L, rL), c = i - r * L;
                        tile[r * LD + c] = v[u];
                    }
                }
            }
        }
        __syncthreads();
        if (lane < rows)
            for (int c = wave; c < L; c += 4) dst[(long)c * R + r0 + lane] = tile[lane * LD + c];
    } else {
        // U runs in flight per wavefront before the first LDS store; runs past the last one
        // are clamped to it and dropped afterwards, so no load is conditional.  Sixteen when
        // that wastes little (L = 128: 5.9 -> 6.7 TB/s on the VGG layer), else eight (L = 96
        // would load a quarter of its runs twice).
        auto gather = [&](auto depth) __attribute__((always_inline)) {
            constexpr int U = decltype(depth)::value;
            for (int c = wave; c < L; c += 4 * U) {
                float v[U];
#pragma unroll
                for (int k = 0; k < U; ++k) v[k] = src[(long)min(c + 4 * k, L - 1) * R + r0 + lane];
#pragma unroll
                for (int k = 0; k < U; ++k)
                    if (c + 4 * k < L) tile[lane * LD + c + 4 * k] = v[k];
            }
        };
        if (lane < rows) {
            if (L > 112) gather(std::integral_constant<int, 16>());
            else gather(std::integral_constant<int, 8>());
        }
        __syncthreads();
        if (VEC) {
            for (int i = threadIdx.x * 4; i < n; i += 1024) {
                const int r = div_small(i, L, rL), c = i - r * L;
                const float* t = tile + r * LD + c;
                stream_store4(blk_out + i, t[0], t[1], t[2], t[3]);
            }
        } else {
            for (int i = threadIdx.x; i < n; i += 256) {
                const int r = div_small(i, L, rL), c = i - r * L;
                blk_out[i] = tile[r * LD + c];
            }
        }
    }
}

struct Perm4 {
    long oshape[4];
    long istride[4];  // input stride of the axis feeding output axis d
};

__global__ __launch_bounds__(256) void transpose4_generic_kernel(const float* __restrict__ in,
                                                                 float* __restrict__ out, Perm4 p,
                                                                 long total) {
    for (long o = (long)blockIdx.x * blockDim.x + threadIdx.x; o < total;
         o += (long)gridDim.x * blockDim.x) {
        long t = o;
        const long i3 = t % p.oshape[3];
        t /= p.oshape[3];
        const long i2 = t % p.oshape[2];
        t /= p.oshape[2];
        const long i1 = t % p.oshape[1];
        const long i0 = t / p.oshape[1];
        out[o] = in[i0 * p.istride[0] + i1 * p.istride[1] + i2 * p.istride[2] + i3 * p.istride[3]];
    }
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// in [B, R, Cn] -> out [B, Cn, R]
static int launch_batched_transpose(const float* in, float* out, long B, long R, long Cn,
                                    hipStream_t st) {
    CGT_ARG_CHECK(R < (1L << 31) && Cn < (1L << 31), "transpose: too large");
    // thin paths whenever one extent fits a workgroup whole: no idle lanes when
    // it is not a multiple of the square tile, and one side of the copy is a
    // contiguous block moved 16 bytes at a time (streamed on the way out)
    const bool thin_in = Cn <= kThinMaxL && R >= 4 * kThinRows;
    const bool thin_out = R <= kThinMaxL && Cn >= 4 * kThinRows;
    if (thin_in || thin_out) {
        const long L = thin_in ? Cn : R, longdim = thin_in ? R : Cn;
        const long tiles = cdiv(longdim, kThinRows);
        CGT_ARG_CHECK(B * tiles < (1L << 31), "transpose: too large");
        const bool vec = L % 4 == 0 && aligned16(in) && aligned16(out);
        const size_t lds = (size_t)kThinRows * (L | 1) * sizeof(float);
        dim3 grid((unsigned)(B * tiles)), block(256);
        if (thin_in) {
            if (vec) thin_transpose_kernel<true, true><<<grid, block, lds, st>>>(in, out, (int)longdim, (int)L, (int)tiles);
            else thin_transpose_kernel<true, false><<<grid, block, lds, st>>>(in, out, (int)longdim, (int)L, (int)tiles);
        } else {
            if (vec) thin_transpose_kernel<false, true><<<grid, block, lds, st>>>(in, out, (int)longdim, (int)L, (int)tiles);
            else thin_transpose_kernel<false, false><<<grid, block, lds, st>>>(in, out, (int)longdim, (int)L, (int)tiles);
        }
        CGT_LAUNCH_CHECK("thin_transpose_kernel");
        return CGT_AMD_OK;
    }
    const long tr = cdiv(R, kTile), tc = cdiv(Cn, kTile);
    const long blocks = B * tr * tc;
    CGT_ARG_CHECK(blocks < (1L << 31), "transpose: too large");
    batched_transpose_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(in, out, (int)R, (int)Cn,
                                                                           (int)tr, (int)tc);
    CGT_LAUNCH_CHECK("batched_transpose_kernel");
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_transpose4_f32(const float* in, const long* s, const int* axes, float* out,
                                   void* stream) {
    CGT_ARG_CHECK(s && axes, "transpose4: null shape/axes");
    bool seen[4] = {false, false, false, false};
    for (int d = 0; d < 4; ++d) {
        CGT_ARG_CHECK(axes[d] >= 0 && axes[d] < 4 && !seen[axes[d]], "transpose4: axes is not a permutation");
        seen[axes[d]] = true;
        CGT_ARG_CHECK(s[d] >= 0, "transpose4: negative shape");
    }
    const long total = s[0] * s[1] * s[2] * s[3];
    if (total == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(in && out, "transpose4: null pointer");
    hipStream_t st = as_stream(stream);
    const int a0 = axes[0], a1 = axes[1], a2 = axes[2], a3 = axes[3];
    if (a0 == 0 && a1 == 1 && a2 == 2 && a3 == 3) {
        CGT_HIP_TRY(hipMemcpyAsync(out, in, total * sizeof(float), hipMemcpyDeviceToDevice, st));
        return CGT_AMD_OK;
    }
    if (a0 == 0 && a1 == 3 && a2 == 1 && a3 == 2)  // [B,m,n,L] -> [B,L,m,n]
        return launch_batched_transpose(in, out, s[0], s[1] * s[2], s[3], st);
    if (a0 == 0 && a1 == 2 && a2 == 3 && a3 == 1)  // [B,L,m,n] -> [B,m,n,L]
        return launch_batched_transpose(in, out, s[0], s[1], s[2] * s[3], st);
    Perm4 p;
    long istr[4], acc = 1;
    for (int d = 3; d >= 0; --d) {
        istr[d] = acc;
        acc *= s[d];
    }
    for (int d = 0; d < 4; ++d) {
        p.oshape[d] = s[axes[d]];
        p.istride[d] = istr[axes[d]];
    }
    long blocks = std::min(cdiv(total, 256L), 1L << 20);
    transpose4_generic_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(in, out, p, total);
    CGT_LAUNCH_CHECK("transpose4_generic_kernel");
    return CGT_AMD_OK;
}
