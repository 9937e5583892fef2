// Shared helpers of the cgt_amd HIP library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "cgt_amd.h"

#define CGT_API extern "C" __attribute__((visibility("default")))

namespace cgt_amd {

// Per-thread message of the last failure; read through cgt_amd_last_error().
void set_error(const char* fmt, ...);
void clear_error();

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

// Library-owned device workspaces (split-K partials, partial sums): one block per
// (stream, user), grown on demand and geometrically (at least 1.5 x the block that is
// outgrown).  An outgrown block is not freed on the spot -- kernels in flight may still
// use it and hipFree would stall the stream -- it is retired: released at the stream's
// next cgt_amd_synchronize, or, if it was current when a capture began on the stream (a
// HIP graph may have its address baked in), with the stream (cgt_amd_stream_destroy).
// Growth while the stream is being captured is refused (an allocation would break the
// capture): returns nullptr with the message set.
enum WorkspaceUser { kWsGemm = 0, kWsSum = 1, kWsConvFilter = 2, kWsConvTable = 3, kWsConvData = 4, kWsUsers = 5 };
float* stream_workspace(void* stream, WorkspaceUser user, size_t bytes, const char* what);
void release_stream_workspaces(void* stream);

// The GEMMs of a convolution layer with the layer's layouts built in (gemm.hip).
// Over an operand read straight from a zero-padded image -- stride 1, pad = (kernel - 1) / 2,
// no column buffer:
//   mode 2: out[M][taps * C] = sum over (b, q) of A[b][m][q] * img[b][c][q + tapoff]
//   mode 3: out[b][m][h][w] = sum over (c, tap) of Wk[m][c/16][tap][c%16] * img[b][c][q + tapoff] (+ bias[m], rectify),
//           q = h*Wp + w: the pixels of the padded grid are the columns, tpi tiles of 128 per image
// Over a column buffer col[B * plane][C] (any geometry), with the NCHW side read / written in place:
//   mode 1: out[b][m][p] = sum over z of W[m][z] * col[b * plane + p][z] (+ bias[m], rectify); C = patch length
//   mode 4: out[M][N] = sum over (b, p) of A[b][m][p] * col[b * plane + p][n]   (A = the NCHW cotangent)
// Modes 1 and 4 without a column buffer: col[b * plane + p][z] is read from the image x
// [B][C][H][W] where im2col would have copied it from (zero outside the image); OH x OW = plane
// output pixels per image, z = (c * kh + ho) * kw + wo.
struct PatchGeom {
    const float* x;
    int C, H, W, kh, kw, ph, pw, sh, sw, OH, OW;
};
struct ConvGemm {
    int mode;
    long B, C, plane;      // images; channels of `img` (mode 1: patch length); floats per padded plane (modes 1, 4: pixels per image)
    int wp, kh, kw;        // padded width, kernel
    long tpi, spi;         // mode 3: pixel tiles (of 128) per image; mode 2: K slices (of 16) per image
    long H, W;             // mode 3: image extents
    const float* bias;     // mode 3: per-output-channel bias or null
    int relu;              // mode 3: x * (x >= 0) on the way out
    signed char* mask;     // mode 3: (x >= 0) as int8, same shape as the output, or null
    const PatchGeom* patch = nullptr;      // modes 1, 4: gather the column buffer's elements from the image
    int out_taps = 0;      // mode 2: > 0 = store the result [M][taps * C] as [M][C][taps], the filters' own layout (ldc == N)
};
int sgemm_conv(const ConvGemm& cv, long M, long N, const float* A, const float* B, float* C, long ldc, void* stream);
// out[i] = ws[0][i] + ... + ws[n - 1][i], i < count, added in that order (gemm.hip's split-K reduce)
// taps > 0: the array is rows of row_len floats whose columns are ordered (tap, channel), and the sums are
// stored as [row][channel][tap], the layout of the filters
int reduce_partials(const float* ws, float* out, long count, int n, void* stream, int row_len = 0, int taps = 0);
// 1 if sgemm_conv has a tile shape for these extents (output channels of the product, channels of the image)
bool sgemm_conv_supported(int mode, long filters, long channels);

// The pullback of a max pool (pool.hip) written straight into a convolution's zero-padded
// layout (conv.hip): what cgt_amd_max_pool_pullback_f32 followed by cgt_amd_conv_same_pad_f32
// leaves, in one pass.  Plane p of the result: `lead` zeros, then rows of `pitch` floats with
// the H x W pullback starting at row `top`; `plane` floats per plane (a multiple of 4), then
// `tail` zero floats after the last plane.  relu_mask (int8 [planes][H][W] or null) multiplies
// each cell as (float)mask * value.
struct PaddedPlanes {
    int lead, top, pitch, plane;
    long tail;
};
int launch_pool_pullback_padded(const int* mask, const float* top_diff, const signed char* relu_mask, long nplanes,
                                long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, long PH, long PW,
                                const PaddedPlanes& lay, float* dst, void* stream);

constexpr int kWave = 64;    // CDNA wavefront width
constexpr int kNumXCD = 8;   // MI355X: 8 accelerator dies, each with its own L2
constexpr int kNumCU = 256;  // MI355X compute units

__host__ __device__ inline long cdiv(long a, long b) { return (a + b - 1) / b; }

// Streaming (non-temporal) 16-byte store for data that is written once, in whole cache
// lines, and not read again by the same kernel: the lines are not kept in L2.  Measured
// on this chip: the VGG im2col (925 MB written in aligned 1152-byte runs) goes from 4.9 to
// 5.9 TB/s with it and the 96 x 3025 transpose from 5.2 to 7.1 TB/s, while 4-byte stores
// and runs that start anywhere (rows of 363 floats, planes of 3025) get SLOWER without
// L2's write combining (AlexNet im2col -27 %, pool pullback -59 %), so only aligned
// vector stores use it.  Those figures are for a kernel launched back to back with itself;
// inside a conv layer's step, between other kernels, the gain is smaller on large outputs
// (VGG im2col: none) and larger where the next kernel is bound by memory too (AlexNet
// conv1 layer: 0.08 ms of 1.67 per step, mostly the LRN forward's two outputs).
typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void stream_store4(float* p, float a, float b, float c, float d) {
    v4f v = {a, b, c, d};
    __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(p));
}

// Geometry known at compile time (hot shapes) ...
template <int KH, int KW, int PH, int PW, int SH, int SW>
struct StaticGeom {
    static constexpr bool is_static = true;
    static constexpr int kKH = KH, kKW = KW, kPH = PH, kPW = PW, kSH = SH, kSW = SW;
    __host__ __device__ constexpr int kh() const { return KH; }
    __host__ __device__ constexpr int kw() const { return KW; }
    __host__ __device__ constexpr int ph() const { return PH; }
    __host__ __device__ constexpr int pw() const { return PW; }
    __host__ __device__ constexpr int sh() const { return SH; }
    __host__ __device__ constexpr int sw() const { return SW; }
};
// ... or only at run time (anything else).
struct DynGeom {
    static constexpr bool is_static = false;
    int kh_, kw_, ph_, pw_, sh_, sw_;
    __host__ __device__ int kh() const { return kh_; }
    __host__ __device__ int kw() const { return kw_; }
    __host__ __device__ int ph() const { return ph_; }
    __host__ __device__ int pw() const { return pw_; }
    __host__ __device__ int sh() const { return sh_; }
    __host__ __device__ int sw() const { return sw_; }
};


}  // namespace cgt_amd

#define CGT_HIP_TRY(expr)                                                          \
    do {                                                                           \
        hipError_t e_ = (expr);                                                    \
        if (e_ != hipSuccess) {                                                    \
            cgt_amd::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                               __FILE__, __LINE__);                                \
            return CGT_AMD_ERR_HIP;                                                \
        }                                                                          \
    } while (0)

#define CGT_ARG_CHECK(cond, ...)                \
    do {                                        \
        if (!(cond)) {                          \
            cgt_amd::set_error(__VA_ARGS__);    \
            return CGT_AMD_ERR_ARG;             \
        }                                       \
    } while (0)

// After a kernel launch: surface launch-configuration errors as a status.
#define CGT_LAUNCH_CHECK(name)                                                     \
    do {                                                                           \
        hipError_t e_ = hipGetLastError();                                         \
        if (e_ != hipSuccess) {                                                    \
            cgt_amd::set_error("launch of %s failed: %s", name, hipGetErrorString(e_)); \
            return CGT_AMD_ERR_HIP;                                                \
        }                                                                          \
    } while (0)
