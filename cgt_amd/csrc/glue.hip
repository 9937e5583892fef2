// Conv glue: 4-d axis permutation.  conv2d applies {0,3,1,2} to the GEMM
// output and its pullback applies {0,2,3,1}; both are batched 2-d transposes
// and go through an LDS tile so reads and writes are both contiguous runs.
#include "common.h"
#include <algorithm>

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
    for (int i = ly; i < kTile; i += 4) {
        const int r = r0 + i, c = c0 + lx;
        if (r < R && c < Cn) tile[i][lx] = src[(long)r * Cn + c];
    }
    __syncthreads();
    for (int i = ly; i < kTile; i += 4) {
        const int c = c0 + i, r = r0 + lx;
        if (r < R && c < Cn) dst[(long)c * R + r] = tile[lx][i];
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

static int launch_batched_transpose(const float* in, float* out, long B, long R, long Cn,
                                    hipStream_t st) {
    const long tr = cdiv(R, kTile), tc = cdiv(Cn, kTile);
    const long blocks = B * tr * tc;
    CGT_ARG_CHECK(blocks < (1L << 31) && R < (1L << 31) && Cn < (1L << 31), "transpose: too large");
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
