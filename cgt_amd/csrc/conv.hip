// Stride-1 "same" convolution (pad = (kernel - 1) / 2, odd kernels) without a column
// buffer: forward, data gradient and weight gradient as GEMMs whose image operand is read
// straight from a zero-padded copy of the image (sgemm_conv in gemm.hip).
//
// Padded layout: [B * C planes][plane floats] + a zeroed tail.  A plane is q zeros, then
// H + 2p rows of Wp = W + q floats (W pixels followed by q zeros; the first and last p rows
// all zero), rounded up past 16 zero floats: pixel (h, w) sits at q + (h + p) * Wp + w.
// The zeros that end a row are also the left padding of the next one, so a row costs
// W + q floats, not W + 2q.
// A column of the forward GEMM is a pixel of the padded grid, q = h * Wp + w (the Wp - W
// positions at the end of each grid row are junk columns that are never stored), so that
// "tap (ho, wo) of pixel q" is the plain offset q + ho * Wp + wo: every operand tile is a
// contiguous run per channel, loaded straight into LDS like any GEMM tile.
//
//   forward        y[b][l][q]      = sum_{c,tap} f[l][c][tap] * xpad[b][c][q + tapoff]
//   data gradient  gx[b][c][q]     = sum_{l,tap} f[l][c][flipped tap] * gypad[b][l][q + tapoff]
//   weight grad    gf[l][tap][c]   = sum_{b,q}   gypad[b][l][q + center] * xpad[b][c][q + tapoff]
// (the padding columns of gypad are zero, so the junk positions of q contribute nothing).
#include "common.h"
#include <algorithm>

namespace cgt_amd {

struct SameGeom {
    long B, C, H, W, L;
    int kh, kw, ph, pw;
    long Hp, Wp, plane, tail;
    long tpi;      // 128-row tiles per image in the forward / data-gradient GEMM
    long spi;      // 16-pixel K slices per image in the weight-gradient GEMM
    long total(long planes) const { return planes * plane + tail; }
};

static bool make_geom(SameGeom& g, long B, long C, long H, long W, long L, int kh, int kw) {
    if (kh < 1 || kw < 1 || kh % 2 == 0 || kw % 2 == 0) return false;
    g.B = B; g.C = C; g.H = H; g.W = W; g.L = L;
    g.kh = kh; g.kw = kw; g.ph = (kh - 1) / 2; g.pw = (kw - 1) / 2;
    g.Hp = H + 2 * g.ph; g.Wp = W + g.pw;
    g.plane = (g.pw + g.Hp * g.Wp + 16 + 15) / 16 * 16;
    g.tail = (256 + (long)kh * g.Wp + 3) / 4 * 4;
    g.tpi = cdiv(H * g.Wp, 128);
    g.spi = cdiv(H * g.Wp, 16);
    return true;
}

// dst plane: zero everywhere except the H x W interior.  A thread writes 4 consecutive
// floats of a plane (plane % 4 == 0: one aligned 16-byte store) and gathers them from the
// source rows; both sides are contiguous runs per image row.
__global__ __launch_bounds__(256) void pad_planes_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                         long planes, int H, int W, int Wp, int ph, int pw,
                                                         int plane, int units_per_plane, long total_units,
                                                         long tail_units) {
    const float rWp = 1.0f / (float)Wp;
    for (long u = (long)blockIdx.x * 256 + threadIdx.x; u < total_units + tail_units; u += (long)gridDim.x * 256) {
        float o[4] = {0.f, 0.f, 0.f, 0.f};
        if (u < total_units) {
            const long pl = u / units_per_plane;
            const int e0 = (int)(u - pl * units_per_plane) * 4;
            const float* sp = src + pl * (long)H * W;
            // row of e0 by reciprocal multiplication (plane < 2^21 is checked on the host), fixed up exactly
            // element e of a plane is column (e - pw) % Wp of padded row (e - pw) / Wp
            const int e1 = e0 - pw + Wp;                 // shifted by one row so that it is never negative
            int hp = (int)(((float)e1 + 0.5f) * rWp);
            int wp = e1 - hp * Wp;
            if (wp < 0) { --hp; wp += Wp; }
            if (wp >= Wp) { ++hp; wp -= Wp; }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int h = hp - 1 - ph;
                if (h >= 0 && h < H && wp < W) o[j] = sp[h * W + wp];
                if (++wp == Wp) { wp = 0; ++hp; }
            }
        }
        stream_store4(dst + u * 4, o[0], o[1], o[2], o[3]);
    }
}

// filters [L][C][kh][kw] -> [C][L/16][(kh-1-ho, kw-1-wo) taps][16]: the filter bank of the
// data gradient seen as a forward convolution of the cotangent (L channels in, C filters),
// in the K order of the product (block of 16 channels, tap, channel in the block)
__global__ __launch_bounds__(256) void flip_filters_kernel(const float* __restrict__ f, float* __restrict__ out,
                                                           int L, int C, int kh, int kw) {
    const int taps = kh * kw;
    const long total = (long)L * C * taps;
    for (long o = (long)blockIdx.x * 256 + threadIdx.x; o < total; o += (long)gridDim.x * 256) {
        const int li = (int)(o % 16);
        long r = o / 16;
        const int tap = (int)(r % taps);
        r /= taps;
        const int lb = (int)(r % (L / 16)), c = (int)(r / (L / 16));
        const int ho = tap / kw, wo = tap - ho * kw;
        out[o] = f[(((long)(lb * 16 + li) * C + c) * kh + (kh - 1 - ho)) * kw + (kw - 1 - wo)];
    }
}

// ---- weight gradient of a first layer with few filters (the CIFAR / MNIST first layers: 32
// filters, patches of 75 and 9 floats).  The result is a few thousand floats and the reduction runs
// over every output pixel of the batch, so as a GEMM it is one row tile by one to four column
// tiles with an enormous K: the tiled product spends its time on prologues and partial tiles
// (0.045 ms for 0.63 GFLOP).  Here it is a reduction: a workgroup takes (image, band of output
// rows) units in turn, stages the band's cotangent [L][pixels] and the patch of the image under it
// (zero-padded, all channels) in LDS, and its four wavefronts walk the band's pixels four at a
// time, each accumulating the whole [32][32 * NB] result block with v_mfma_f32_32x32x2_f32:
// A operand = cotangent (lane -> filter, k -> pixel), B operand = patch element (lane -> patch
// index z, its (channel, row, column) offset fixed per lane; k -> pixel, whose tile offset comes
// from a small table).  The four wavefronts' blocks are added in order 0..3, each workgroup
// writes one partial result and the split-K reduce kernel adds those in order: deterministic.
struct SmallWgrad {
    const float* gy;      // [B][L][OH * OW]
    const float* x;       // [B][C][H][W]
    float* part;          // [workgroups][L][Z]
    int B, C, H, W, L, OH, OW, Z, kh, kw, ph, pw, sh, sw;
    int band_rows, bands, units;      // output rows per unit, units per image, B * bands
    int rows_in, twp;                 // the image tile under a band: C x rows_in x twp floats
    int pbpad;                        // floats between two filters' rows in the cotangent tile (even)
    int vec4;                         // every row of every unit's cotangent tile is whole aligned 16-byte units
    int off_x, off_pix;               // LDS offsets (floats) of the image tile and the pixel table
};

typedef float v16f __attribute__((ext_vector_type(16)));

template <int NB>
__global__ __launch_bounds__(256) void wgrad_small_kernel(SmallWgrad a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* gyt = lds;                                   // [32][pbpad]
    float* xt = lds + a.off_x;                          // [C][rows_in][twp]
    int* pixoff = reinterpret_cast<int*>(lds + a.off_pix);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
    const int taps = a.kh * a.kw, P = a.OH * a.OW;
    int offz[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int z = nb * 32 + l32;
        offz[nb] = 0;                                   // columns past Z read valid LDS; they are never stored
        if (z < a.Z) {
            const int c = z / taps, r = z - c * taps, ho = r / a.kw, wo = r - ho * a.kw;
            offz[nb] = (c * a.rows_in + ho) * a.twp + wo;
        }
    }
    v16f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[nb][e] = 0.0f;

    for (int u = blockIdx.x; u < a.units; u += gridDim.x) {
        const int b = u / a.bands, bd = u - b * a.bands;
        const int r0 = bd * a.band_rows, r1 = min(a.OH, r0 + a.band_rows);
        const int PB = (r1 - r0) * a.OW, PB4 = (PB + 3) & ~3;
        // cotangent tile: filter l's pixels are contiguous in memory; wavefront w takes rows w, w + 4, ...
        // (8 rows x up to 4 floats per lane, all loads issued before the first is parked; rows past L
        // and pixels past PB are loaded from clamped addresses and parked as zeros)
        const float* gsrc = a.gy + (long)b * a.L * P + (long)r0 * a.OW;
        const int nx = a.C * a.rows_in * a.twp;
        const float* xsrc = a.x + (long)b * a.C * a.H * a.W;
        // image tile: input rows r0 * sh - ph ..., columns -pw ..., zero outside the image
        auto stage_image = [&]() __attribute__((always_inline)) {
            for (int i = threadIdx.x; i < nx; i += 256) {
                const int c = i / (a.rows_in * a.twp), r = i - c * (a.rows_in * a.twp);
                const int ri = r / a.twp, wi = r - ri * a.twp;
                const int hh = r0 * a.sh - a.ph + ri, ww = wi - a.pw;
                const bool in = hh >= 0 && hh < a.H && ww >= 0 && ww < a.W;
                const float v = xsrc[((long)c * a.H + (in ? hh : 0)) * a.W + (in ? ww : 0)];
                xt[i] = in ? v : 0.0f;
            }
            for (int p = threadIdx.x; p < PB4; p += 256) {
                const int q = min(p, PB - 1);               // (pixels past PB carry a zero cotangent)
                const int h = q / a.OW, w = q - h * a.OW;
                pixoff[p] = h * a.sh * a.twp + w * a.sw;
            }
        };
        if (a.vec4) {
            // every filter's run of PB floats starts on a 16-byte boundary and is whole units: one
            // 16-byte load per lane and row (PB <= 256), all eight rows in flight
            float4 gv[8];
            const int u = min(lane, PB / 4 - 1);
#pragma unroll
            for (int i = 0; i < 8; ++i) gv[i] = *reinterpret_cast<const float4*>(gsrc + (long)min(wave + 4 * i, a.L - 1) * P + 4 * u);
            stage_image();
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int l = wave + 4 * i;
                if (4 * lane < PB4) {
                    const float4 v = l < a.L ? gv[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                    float2* d = reinterpret_cast<float2*>(gyt + l * a.pbpad + 4 * lane);
                    d[0] = make_float2(v.x, v.y);
                    d[1] = make_float2(v.z, v.w);
                }
            }
        } else {
            float gv[8][4];
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int l = min(wave + 4 * i, a.L - 1), p = min(lane + 64 * k, PB - 1);
                    gv[i][k] = gsrc[(long)l * P + p];
                }
            stage_image();
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int l = wave + 4 * i, p = lane + 64 * k;
                    if (p < PB4) gyt[l * a.pbpad + p] = (l < a.L && p < PB) ? gv[i][k] : 0.0f;
                }
        }
        __syncthreads();
        // lanes 0..31 carry pixels q, q + 1 of a quad, lanes 32..63 pixels q + 2, q + 3: the two
        // MFMAs of a quad pair (q, q + 2) and (q + 1, q + 3) on the k axis, for both operands
        for (int q = 4 * wave; q < PB4; q += 16) {
            const int p_lo = q + 2 * half;
            const float2 av = *reinterpret_cast<const float2*>(gyt + l32 * a.pbpad + p_lo);
            const int2 po = *reinterpret_cast<const int2*>(pixoff + p_lo);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float b0 = xt[offz[nb] + po.x], b1 = xt[offz[nb] + po.y];
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, b0, acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, b1, acc[nb], 0, 0, 0);
            }
        }
        __syncthreads();                                // the next unit's tiles go over these
    }
    // the four wavefronts' blocks, added in order; element e of a block: row 8 * (e / 4) + 4 * half + e % 4, column l32
    float* red = lds;
    for (int w = 0; w < 4; ++w) {
        if (wave == w) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int i = (nb * 16 + e) * 64 + lane;
                    red[i] = w == 0 ? acc[nb][e] : red[i] + acc[nb][e];
                }
        }
        __syncthreads();
    }
    float* out = a.part + (long)blockIdx.x * a.L * a.Z;
    for (int i = threadIdx.x; i < NB * 1024; i += 256) {
        const int nb = i >> 10, e = (i >> 6) & 15, ln = i & 63;
        const int l = 8 * (e >> 2) + 4 * (ln >> 5) + (e & 3), z = nb * 32 + (ln & 31);
        if (l < a.L && z < a.Z) out[l * a.Z + z] = red[i];
    }
}

// 0 if the reduction kernel does not cover the layer (then the tiled product runs); else the plan
static bool small_wgrad_plan(SmallWgrad& a, size_t& lds_bytes, int& grid, long B, long C, long H, long W, long L,
                             const PatchGeom& pg) {
    const long Z = C * pg.kh * pg.kw;
    if (L < 1 || L > 32 || Z > 128 || pg.OW > 256 || B < 1 || B >= (1L << 24)) return false;
    // bands of whole output rows, at most 256 pixels each; more, shorter bands while the chip has workgroups to spare
    int band_rows = std::max(1, std::min(pg.OH, 256 / pg.OW));
    int bands = (int)cdiv(pg.OH, band_rows);
    band_rows = (int)cdiv(pg.OH, bands);
    while (B * bands < 2 * kNumCU && band_rows > 1 && (band_rows / 2) * pg.OW >= 64) {
        band_rows = (band_rows + 1) / 2;
        bands = (int)cdiv(pg.OH, band_rows);
    }
    const int rows_in = (band_rows - 1) * pg.sh + pg.kh, twp = (pg.OW - 1) * pg.sw + pg.kw;
    const long xt_floats = C * rows_in * twp;
    if (xt_floats > 8192 || B * bands >= (1L << 30)) return false;
    const int pb4 = (band_rows * pg.OW + 3) & ~3;
    a.pbpad = pb4 + 2;        // even (8-byte reads and stores), and 2 mod 32 for the largest band: consecutive filters two banks apart
    a.off_x = (32 * a.pbpad + 3) & ~3;
    a.off_pix = (int)((a.off_x + xt_floats + 3) & ~3);
    const long total = a.off_pix + pb4 + 4;
    lds_bytes = (size_t)std::max(total, 4L * 1024) * sizeof(float);       // the cross-wavefront sum needs NB * 1024 floats
    if (lds_bytes > 64 * 1024) return false;
    a.B = (int)B; a.C = (int)C; a.H = (int)H; a.W = (int)W; a.L = (int)L; a.OH = pg.OH; a.OW = pg.OW; a.Z = (int)Z;
    a.kh = pg.kh; a.kw = pg.kw; a.ph = pg.ph; a.pw = pg.pw; a.sh = pg.sh; a.sw = pg.sw;
    a.band_rows = band_rows; a.bands = bands; a.units = (int)(B * bands);
    a.rows_in = rows_in; a.twp = twp;
    grid = (int)std::min((long)a.units, 4L * kNumCU);
    return true;
}

static int small_wgrad(const SmallWgrad& plan, size_t lds_bytes, int grid, const float* gy, const float* x, float* gf, void* stream) {
    SmallWgrad a = plan;
    a.gy = gy; a.x = x;
    // 16-byte loads of the cotangent: pixel runs that start and end on 16-byte boundaries in every unit
    a.vec4 = (((long)a.OH * a.OW) % 4 == 0 && (a.band_rows * a.OW) % 4 == 0 && reinterpret_cast<uintptr_t>(gy) % 16 == 0) ? 1 : 0;
    a.part = stream_workspace(stream, kWsConvData, (size_t)grid * a.L * a.Z * sizeof(float), "conv_patch_bwd_filter");
    if (!a.part) return CGT_AMD_ERR_NOMEM;
    hipStream_t st = as_stream(stream);
    const int nb = (a.Z + 31) / 32;
    if (nb == 1) wgrad_small_kernel<1><<<dim3((unsigned)grid), dim3(256), lds_bytes, st>>>(a);
    else if (nb == 2) wgrad_small_kernel<2><<<dim3((unsigned)grid), dim3(256), lds_bytes, st>>>(a);
    else if (nb == 3) wgrad_small_kernel<3><<<dim3((unsigned)grid), dim3(256), lds_bytes, st>>>(a);
    else wgrad_small_kernel<4><<<dim3((unsigned)grid), dim3(256), lds_bytes, st>>>(a);
    CGT_LAUNCH_CHECK("wgrad_small_kernel");
    return reduce_partials(a.part, gf, (long)a.L * a.Z, grid, stream);
}

static int check_same(const char* what, SameGeom& g, long B, long C, long H, long W, long L, int kh, int kw) {
    CGT_ARG_CHECK(B >= 0 && C > 0 && H > 0 && W > 0 && L > 0, "%s: bad shape", what);
    CGT_ARG_CHECK(make_geom(g, B, C, H, W, L, kh, kw), "%s: the kernel must be odd x odd (pad = (kernel - 1) / 2)", what);
    CGT_ARG_CHECK(g.plane < (1L << 21), "%s: image plane too large for this path", what);
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_conv_same_fits(long B, long C, long H, long W, long L, int kh, int kw) {
    SameGeom g;
    if (B < 0 || C < 1 || H < 1 || W < 1 || L < 1 || !make_geom(g, B, C, H, W, L, kh, kw)) return 0;
    // reciprocal index arithmetic of the pad kernels; 32-bit lane offsets of the products (a tile's rows
    // span the channels of a whole image in the weight gradient, whose operands are x and the cotangent)
    if (g.plane >= (1L << 21) || C * g.plane >= (1L << 30) || L * g.plane >= (1L << 30)) return 0;
    return B * g.tpi * 128 < (1L << 31) - 128 && B * g.spi * 16 < (1L << 31) - 128 ? 1 : 0;
}

CGT_API int cgt_amd_conv_col_fits(long B, long P, long Z, long L) {
    if (B < 0 || P < 1 || Z < 1 || L < 1) return 0;
    // forward product: a lane's 32-bit offset spans the images a tile of 128 columns touches
    if (B * P >= (1L << 31) - 128 || (127 / P + 2) * L * P >= (1L << 30)) return 0;
    return Z < (1L << 31) - 128 && L * Z < (1L << 29) ? 1 : 0;
}

CGT_API int cgt_amd_conv_same_supported(long C, long L, int kh, int kw, int ph, int pw, int sh, int sw) {
    if (sh != 1 || sw != 1 || kh % 2 == 0 || kw % 2 == 0 || ph != (kh - 1) / 2 || pw != (kw - 1) / 2) return 0;
    // forward: C channels in, L filters; data gradient: L channels in, C "filters"; weight gradient: both
    return sgemm_conv_supported(3, L, C) && sgemm_conv_supported(3, C, L) && sgemm_conv_supported(2, L, C) ? 1 : 0;
}

CGT_API long cgt_amd_conv_same_padded_size(long planes, long H, long W, int kh, int kw) {
    SameGeom g;
    if (planes < 0 || H <= 0 || W <= 0 || !make_geom(g, 1, 1, H, W, 1, kh, kw)) return -1;
    return g.total(planes);
}

CGT_API int cgt_amd_conv_same_pad_f32(const float* x, long planes, long H, long W, int kh, int kw, float* xpad,
                                      void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_pad", g, 1, 1, H, W, 1, kh, kw);
    if (rc) return rc;
    CGT_ARG_CHECK(planes >= 0 && (x || planes == 0) && xpad, "conv_same_pad: null pointer");
    CGT_ARG_CHECK(reinterpret_cast<uintptr_t>(xpad) % 16 == 0, "conv_same_pad: the padded buffer must be 16-byte aligned");
    const long upp = g.plane / 4, units = planes * upp, tail_units = g.tail / 4;
    const long blocks = std::min(cdiv(units + tail_units, 256L), 1L << 16);
    pad_planes_kernel<<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(
        x, xpad, planes, (int)H, (int)W, (int)g.Wp, g.ph, g.pw, (int)g.plane, (int)upp, units, tail_units);
    CGT_LAUNCH_CHECK("pad_planes_kernel");
    return CGT_AMD_OK;
}

// gypad = pad(relu_mask * max_pool_pullback(mask, top_diff)): the cotangent of a convolution whose
// result went through (a rectify and) a max pool, in the layout the gradient products read, without
// the unpadded array in between
CGT_API int cgt_amd_conv_same_pad_pool_pullback_f32(const int* mask, const float* top_diff, const signed char* relu_mask,
                                                    long planes, long H, long W, int pool_kh, int pool_kw, int pool_ph,
                                                    int pool_pw, int pool_sh, int pool_sw, long PH, long PW, int kh, int kw,
                                                    float* gypad, void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_pad_pool_pullback", g, 1, 1, H, W, 1, kh, kw);
    if (rc) return rc;
    CGT_ARG_CHECK(planes >= 0 && gypad, "conv_same_pad_pool_pullback: bad arguments");
    const PaddedPlanes lay = {g.pw, g.ph, (int)g.Wp, (int)g.plane, g.tail};
    return launch_pool_pullback_padded(mask, top_diff, relu_mask, planes, H, W, pool_kh, pool_kw, pool_ph, pool_pw, pool_sh,
                                       pool_sw, PH, PW, lay, gypad, stream);
}

// ---- the pieces (each one kernel plus, for the products, the GEMM's own reduce kernel)

CGT_API int cgt_amd_conv_same_filter_f32(const float* f, long L, long C, int kh, int kw, int flipped, float* fk,
                                         void* stream) {
    CGT_ARG_CHECK(L > 0 && C > 0 && kh > 0 && kw > 0 && f && fk, "conv_same_filter: bad arguments");
    CGT_ARG_CHECK(C % 16 == 0 && L % 16 == 0, "conv_same_filter: channel and filter counts must be multiples of 16");
    if (!flipped) {     // [L][C/16][16][taps] -> [L][C/16][taps][16]: the K order of the product
        const long fs[4] = {L * (C / 16), 16, kh, kw};
        const int ax[4] = {0, 2, 3, 1};
        return cgt_amd_transpose4_f32(f, fs, ax, fk, stream);
    }
    const long total = L * C * kh * kw;
    flip_filters_kernel<<<dim3((unsigned)std::min(cdiv(total, 256L), 4096L)), dim3(256), 0, as_stream(stream)>>>(
        f, fk, (int)L, (int)C, kh, kw);
    CGT_LAUNCH_CHECK("flip_filters_kernel");
    return CGT_AMD_OK;
}

// out [B,N,H,W] = conv of the padded image with fk (+ bias, rectify), written in place by the GEMM
CGT_API int cgt_amd_conv_same_product_f32(const float* imgpad, const float* fk, const float* bias, int relu, long B,
                                          long Cin, long H, long W, long N, int kh, int kw, float* out,
                                          signed char* mask, void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_product", g, B, Cin, H, W, N, kh, kw);
    if (rc) return rc;
    if (B == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(imgpad && fk && out, "conv_same_product: null pointer");
    CGT_ARG_CHECK(sgemm_conv_supported(3, N, Cin), "conv_same_product: unsupported extents (%ld channels, %ld filters)", Cin, N);
    ConvGemm cv = {3, B, Cin, g.plane, (int)g.Wp, kh, kw, g.tpi, g.spi, H, W, bias, relu, mask};
    return sgemm_conv(cv, N, B * g.tpi * 128, fk, imgpad, out, H * W, stream);
}

CGT_API int cgt_amd_conv_same_wgrad_f32(const float* gypad, const float* xpad, long B, long C, long H, long W,
                                        long L, int kh, int kw, float* gfk, void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_wgrad", g, B, C, H, W, L, kh, kw);
    if (rc) return rc;
    CGT_ARG_CHECK(gfk, "conv_same_wgrad: null pointer");
    const long taps = (long)kh * kw;
    if (B == 0) return cgt_amd_fill_u32(gfk, 0u, L * C * taps, stream);
    CGT_ARG_CHECK(gypad && xpad, "conv_same_wgrad: null pointer");
    CGT_ARG_CHECK(sgemm_conv_supported(2, L, C), "conv_same_wgrad: unsupported extents (%ld channels, %ld filters)", C, L);
    // pixel q of the padded grid <-> cotangent at q + (ph * Wp + pw): its padding is zero, so junk pixels add nothing
    ConvGemm cv = {2, B, C, g.plane, (int)g.Wp, kh, kw, g.tpi, g.spi, H, W, nullptr, 0, nullptr};
    return sgemm_conv(cv, L, taps * C, gypad + g.ph * g.Wp + g.pw, xpad, gfk, taps * C, stream);
}

// ---- the three products of a layer, composed from the pieces with library-owned workspaces

CGT_API int cgt_amd_conv_same_fwd_f32(const float* xpad, const float* f, const float* bias, int relu, long B, long C,
                                      long H, long W, long L, int kh, int kw, float* y, signed char* mask,
                                      void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_fwd", g, B, C, H, W, L, kh, kw);
    if (rc) return rc;
    if (B == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(xpad && f && y, "conv_same_fwd: null pointer");
    CGT_ARG_CHECK(cgt_amd_conv_same_supported(C, L, kh, kw, g.ph, g.pw, 1, 1), "conv_same_fwd: unsupported extents C=%ld L=%ld", C, L);
    const long taps = (long)kh * kw;
    float* wk = stream_workspace(stream, kWsConvFilter, (size_t)L * C * taps * sizeof(float), "conv_same_fwd");
    if (!wk) return CGT_AMD_ERR_NOMEM;
    if ((rc = cgt_amd_conv_same_filter_f32(f, L, C, kh, kw, 0, wk, stream))) return rc;
    return cgt_amd_conv_same_product_f32(xpad, wk, bias, relu, B, C, H, W, L, kh, kw, y, mask, stream);
}

CGT_API int cgt_amd_conv_same_bwd_data_f32(const float* gypad, const float* f, long B, long C, long H, long W, long L,
                                           int kh, int kw, float* gx, void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_bwd_data", g, B, C, H, W, L, kh, kw);
    if (rc) return rc;
    if (B == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(gypad && f && gx, "conv_same_bwd_data: null pointer");
    CGT_ARG_CHECK(cgt_amd_conv_same_supported(C, L, kh, kw, g.ph, g.pw, 1, 1), "conv_same_bwd_data: unsupported extents C=%ld L=%ld", C, L);
    const long taps = (long)kh * kw;
    float* wk = stream_workspace(stream, kWsConvFilter, (size_t)L * C * taps * sizeof(float), "conv_same_bwd_data");
    if (!wk) return CGT_AMD_ERR_NOMEM;
    // a forward convolution of the cotangent: L channels in, C "filters" [C][L/16][flipped tap][16]
    if ((rc = cgt_amd_conv_same_filter_f32(f, L, C, kh, kw, 1, wk, stream))) return rc;
    return cgt_amd_conv_same_product_f32(gypad, wk, nullptr, 0, B, L, H, W, C, kh, kw, gx, nullptr, stream);
}

CGT_API int cgt_amd_conv_same_bwd_filter_f32(const float* gypad, const float* xpad, long B, long C, long H, long W,
                                             long L, int kh, int kw, float* gf, void* stream) {
    SameGeom g;
    int rc = check_same("conv_same_bwd_filter", g, B, C, H, W, L, kh, kw);
    if (rc) return rc;
    CGT_ARG_CHECK(gf, "conv_same_bwd_filter: null pointer");
    const long taps = (long)kh * kw;
    if (B == 0) return cgt_amd_fill_u32(gf, 0u, L * C * taps, stream);
    CGT_ARG_CHECK(cgt_amd_conv_same_supported(C, L, kh, kw, g.ph, g.pw, 1, 1), "conv_same_bwd_filter: unsupported extents C=%ld L=%ld", C, L);
    CGT_ARG_CHECK(gypad && xpad && gf, "conv_same_bwd_filter: null pointer");
    // the product's columns are (tap, channel); the kernel that sums its K pieces stores [L][C][kh][kw]
    ConvGemm cv = {2, B, C, g.plane, (int)g.Wp, kh, kw, g.tpi, g.spi, H, W, nullptr, 0, nullptr};
    cv.out_taps = (int)taps;
    return sgemm_conv(cv, L, taps * C, gypad + g.ph * g.Wp + g.pw, xpad, gf, taps * C, stream);
}

// The weight gradient's K axis is cut per image, so its partial sums are at least one [L][Z]
// block per image.  While those fit 256 MiB (and the product's own limits) the batch is one
// product; beyond that it runs in groups of images, each group's result goes to a second
// workspace and the groups are summed in order: any batch size, fixed order of additions.
template <class F>
static int wgrad_in_groups(long B, long P, long Z, long L, float* gf, void* stream, const char* what, F&& product) {
    CGT_ARG_CHECK(P < (1L << 31) - 128, "%s: too many output pixels per image", what);
    const long per_image = L * Z;
    long group = std::max(1L, (64L << 20) / per_image);                 // 256 MiB of partial sums
    group = std::min({group, ((1L << 31) - 129) / P, (1L << 19)});      // the product's own limits on pixels and splits
    CGT_ARG_CHECK(group >= 1, "%s: image too large", what);
    if (B <= group) return product(0, B, gf);
    const long ngroups = cdiv(B, group);
    CGT_ARG_CHECK(ngroups < (1L << 30), "%s: too many images", what);
    float* part = stream_workspace(stream, kWsConvData, (size_t)ngroups * per_image * sizeof(float), what);
    if (!part) return CGT_AMD_ERR_NOMEM;
    for (long gi = 0; gi < ngroups; ++gi) {
        const long b0 = gi * group;
        int rc = product(b0, std::min(group, B - b0), part + gi * per_image);
        if (rc) return rc;
    }
    return reduce_partials(part, gf, per_image, (int)ngroups, stream);
}

// ---- any geometry, over the column buffer of im2col: the three products of conv2d with the
// NCHW side read and written in place (no [B*m*n, L] intermediate, no transposes).
//   col [B * P][Z] (P = m * n output pixels per image, Z = C * kh * kw), f [L][Z] (= [L,C,kh,kw]),
//   y / gy [B][L][P]

CGT_API int cgt_amd_conv_col_fwd_f32(const float* col, const float* f, const float* bias, int relu, long B, long P,
                                     long Z, long L, float* y, signed char* mask, void* stream) {
    CGT_ARG_CHECK(B >= 0 && P >= 0 && Z >= 0 && L >= 0, "conv_col_fwd: negative extent");
    if (B == 0 || P == 0 || L == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(y && (Z == 0 || (col && f)), "conv_col_fwd: null pointer");
    CGT_ARG_CHECK(B * P < (1L << 31) - 128, "conv_col_fwd: too many output pixels");
    // y[b][l][p] = sum_z f[l][z] col[b * P + p][z]: rows are filters, so a wavefront's store covers
    // consecutive pixels of one channel plane
    ConvGemm cv = {1, B, Z, P, 0, 1, 1, 0, 0, 0, 0, bias, relu, mask};
    return sgemm_conv(cv, L, B * P, f, col, y, B * P, stream);
}

// gcol[b * P + p][z] = sum_l gy[b][l][p] f[l][z]: per image a product with the transposed
// cotangent plane block as its first operand
CGT_API int cgt_amd_conv_col_bwd_data_f32(const float* gy, const float* f, long B, long P, long Z, long L,
                                          float* gcol, void* stream) {
    CGT_ARG_CHECK(B >= 0 && P >= 0 && Z >= 0 && L >= 0, "conv_col_bwd_data: negative extent");
    if (B == 0 || P == 0 || Z == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(gcol && (L == 0 || (gy && f)), "conv_col_bwd_data: null pointer");
    int rc = CGT_AMD_OK;
    for (long b0 = 0; b0 < B && rc == CGT_AMD_OK; b0 += 32768) {     // the batched product takes fewer than 65536 at a time
        const long nb = std::min(B - b0, 32768L);
        rc = cgt_amd_sgemm_batched(1, 0, nb, P, Z, L, gy + b0 * L * P, P, L * P, f, Z, 0, gcol + b0 * P * Z, Z, P * Z, stream);
    }
    return rc;
}

// gf[l][z] = sum over (b, p) of gy[b][l][p] col[b * P + p][z]
CGT_API int cgt_amd_conv_col_bwd_filter_f32(const float* gy, const float* col, long B, long P, long Z, long L,
                                            float* gf, void* stream) {
    CGT_ARG_CHECK(B >= 0 && P >= 0 && Z >= 0 && L >= 0, "conv_col_bwd_filter: negative extent");
    if (L == 0 || Z == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(gf, "conv_col_bwd_filter: null pointer");
    if (B == 0 || P == 0) return cgt_amd_fill_u32(gf, 0u, L * Z, stream);
    CGT_ARG_CHECK(gy && col, "conv_col_bwd_filter: null pointer");
    return wgrad_in_groups(B, P, Z, L, gf, stream, "conv_col_bwd_filter", [&](long b0, long nb, float* out) {
        ConvGemm cv = {4, nb, Z, P, 0, 1, 1, 0, 0, 0, 0, nullptr, 0, nullptr};
        return sgemm_conv(cv, L, Z, gy + b0 * L * P, col + b0 * P * Z, out, Z, stream);
    });
}

// ---- any geometry, no column buffer for the forward product and the weight gradient: the two
// products above with col's elements gathered from the image as the GEMM loads its operand tile
// (im2col's index rule applied inside the loader, zero outside the image).  The data gradient
// keeps the column buffer: its result has to be scattered back (cgt_amd_conv_col_bwd_data_f32
// + cgt_amd_col2im_f32), and with a handful of input channels there is no GEMM to gather into.

static bool patch_geom(PatchGeom& pg, const float* x, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw) {
    if (C < 1 || H < 1 || W < 1 || kh < 1 || kw < 1 || ph < 0 || pw < 0 || sh < 1 || sw < 1) return false;
    if (H + 2L * ph < kh || W + 2L * pw < kw) return false;
    const long OH = (H + 2L * ph - kh) / sh + 1, OW = (W + 2L * pw - kw) / sw + 1;
    if (H >= 32768 || W >= 32768 || kh >= 32768 || kw >= 32768 || ph >= 32768 || pw >= 32768 || C >= (1L << 20) ||
        OH * OW >= (1L << 21) || C * kh * kw >= (1L << 31) - 128)
        return false;
    pg = PatchGeom{x, (int)C, (int)H, (int)W, kh, kw, ph, pw, sh, sw, (int)OH, (int)OW};
    return true;
}

CGT_API int cgt_amd_conv_patch_supported(long B, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw) {
    PatchGeom pg;
    if (B < 0 || !patch_geom(pg, nullptr, C, H, W, kh, kw, ph, pw, sh, sw)) return 0;
    return B * C * H * W < (1L << 29) && B * pg.OH * pg.OW < (1L << 31) - 128 ? 1 : 0;
}

CGT_API int cgt_amd_conv_patch_fwd_f32(const float* x, const float* f, const float* bias, int relu, long B, long C,
                                       long H, long W, long L, int kh, int kw, int ph, int pw, int sh, int sw,
                                       float* y, signed char* mask, void* stream) {
    CGT_ARG_CHECK(B >= 0 && L >= 0, "conv_patch_fwd: negative extent");
    PatchGeom pg;
    CGT_ARG_CHECK(patch_geom(pg, x, C, H, W, kh, kw, ph, pw, sh, sw) && cgt_amd_conv_patch_supported(B, C, H, W, kh, kw, ph, pw, sh, sw),
                  "conv_patch_fwd: geometry out of range (use im2col + cgt_amd_conv_col_fwd_f32)");
    const long P = (long)pg.OH * pg.OW, Z = C * kh * kw;
    if (B == 0 || L == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(x && f && y, "conv_patch_fwd: null pointer");
    ConvGemm cv = {1, B, Z, P, 0, 1, 1, 0, 0, 0, 0, bias, relu, mask, &pg};
    return sgemm_conv(cv, L, B * P, f, x, y, B * P, stream);
}

CGT_API int cgt_amd_conv_patch_bwd_filter_f32(const float* gy, const float* x, long B, long C, long H, long W, long L,
                                              int kh, int kw, int ph, int pw, int sh, int sw, float* gf, void* stream) {
    CGT_ARG_CHECK(B >= 0 && L >= 0, "conv_patch_bwd_filter: negative extent");
    PatchGeom pg;
    CGT_ARG_CHECK(patch_geom(pg, x, C, H, W, kh, kw, ph, pw, sh, sw) && cgt_amd_conv_patch_supported(B, C, H, W, kh, kw, ph, pw, sh, sw),
                  "conv_patch_bwd_filter: geometry out of range (use im2col + cgt_amd_conv_col_bwd_filter_f32)");
    const long P = (long)pg.OH * pg.OW, Z = C * kh * kw;
    if (L == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(gf, "conv_patch_bwd_filter: null pointer");
    if (B == 0) return cgt_amd_fill_u32(gf, 0u, L * Z, stream);
    CGT_ARG_CHECK(gy && x, "conv_patch_bwd_filter: null pointer");
    {
        SmallWgrad plan;
        size_t lds_bytes = 0;
        int grid = 0;
        if (small_wgrad_plan(plan, lds_bytes, grid, B, C, H, W, L, pg)) return small_wgrad(plan, lds_bytes, grid, gy, x, gf, stream);
    }
    return wgrad_in_groups(B, P, Z, L, gf, stream, "conv_patch_bwd_filter", [&](long b0, long nb, float* out) {
        PatchGeom part = pg;
        part.x = x + b0 * C * H * W;
        ConvGemm cv = {4, nb, Z, P, 0, 1, 1, 0, 0, 0, 0, nullptr, 0, nullptr, &part};
        return sgemm_conv(cv, L, Z, gy + b0 * L * P, part.x, out, Z, stream);
    });
}
