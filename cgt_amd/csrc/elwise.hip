// Conv-layer glue around the GEMM path, for gfx950: elementwise unary / binary
// ops (bias add, the compare + multiply that make ReLU, and the rest of the
// reference's tables), Repeat (broadcast along singleton axes), Sum over axes
// (bias gradient, scalar loss) and Fill.  All HBM-bound: 16-byte accesses,
// several in flight per lane, no re-reads.
//
// Element types follow the reference's two that occur on this path: float
// ("f4") and the one-byte integer ("i1") that comparisons produce
// (cgt/core.py:1134-1152, typeinfo 'i1').  Arithmetic between an f4 and an i1
// operand promotes to f4 as `_promote` does (core.py:118-134).
#include "common.h"
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <type_traits>

namespace cgt_amd {

constexpr int kElwThreads = 256;
constexpr int kElwPerThread = 8;       // elements per thread and loop trip (two 16-byte accesses for floats)

// ---------------------------------------------------------------- scalar functions

// Unary ops as the reference's native templates spell them (UNARY_INFO cexpr,
// cgt/core.py:1118-1134); "sign" is 2*(x>0)-1 there, so sign(0) = -1.
template <int OP>
__device__ __forceinline__ float unary_fn(float x) {
    if (OP == CGT_AMD_UN_ABS) return fabsf(x);
    if (OP == CGT_AMD_UN_COS) return cosf(x);
    if (OP == CGT_AMD_UN_EXP) return expf(x);
    if (OP == CGT_AMD_UN_LOG) return logf(x);
    if (OP == CGT_AMD_UN_NEG) return -x;
    if (OP == CGT_AMD_UN_SIGN) return (float)(2 * (x > 0) - 1);
    if (OP == CGT_AMD_UN_SIN) return sinf(x);
    if (OP == CGT_AMD_UN_SQUARE) return x * x;
    if (OP == CGT_AMD_UN_SQRT) return sqrtf(x);
    if (OP == CGT_AMD_UN_TANH) return tanhf(x);
    if (OP == CGT_AMD_UN_SIGMOID) return 1.0f / (1.0f + expf(-x));
    return x;
}

// Binary ops (BINARY_INFO cexpr, cgt/core.py:1139-1152).  P is the promoted
// operand type (float if either side is float, else int).
template <int OP, class P>
struct BinaryFn {
    static constexpr bool is_compare = OP == CGT_AMD_BIN_LT || OP == CGT_AMD_BIN_GT || OP == CGT_AMD_BIN_LE ||
                                       OP == CGT_AMD_BIN_GE || OP == CGT_AMD_BIN_EQ || OP == CGT_AMD_BIN_NE;
    // compares give i1; "/" always gives floatX (typeinfo 'f'); the rest keep the promoted type
    typedef typename std::conditional<is_compare, int8_t,
        typename std::conditional<std::is_same<P, float>::value || OP == CGT_AMD_BIN_DIV, float, int8_t>::type>::type Out;
    static __device__ __forceinline__ Out apply(P x, P y) {
        if (OP == CGT_AMD_BIN_MUL) return (Out)(x * y);
        if (OP == CGT_AMD_BIN_ADD) return (Out)(x + y);
        if (OP == CGT_AMD_BIN_SUB) return (Out)(x - y);
        if (OP == CGT_AMD_BIN_DIV) return (Out)((float)x / (float)y);   // "(x+0.0)/y": exact after rounding to float
        if (OP == CGT_AMD_BIN_POW) return (Out)powf((float)x, (float)y);
        if (OP == CGT_AMD_BIN_LT) return (Out)(x < y);
        if (OP == CGT_AMD_BIN_GT) return (Out)(x > y);
        if (OP == CGT_AMD_BIN_LE) return (Out)(x <= y);
        if (OP == CGT_AMD_BIN_GE) return (Out)(x >= y);
        if (OP == CGT_AMD_BIN_EQ) return (Out)(x == y);
        return (Out)(x != y);
    }
};

// ---------------------------------------------------------------- vector access

// N consecutive elements of type T starting at p[i]; `vec` says the base is
// aligned for the widest access.  A scalar operand (one element, index 0) is
// splatted.
template <class T, int N>
__device__ __forceinline__ void load_run(const T* __restrict__ p, long i, bool scalar, bool vec, T (&v)[N]) {
    if (scalar) {
        const T s = p[0];
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = s;
    } else if (vec) {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int j = 0; j < N; j += 4) {
                const float4 q = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i + j);
                const float t[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) v[j + k] = reinterpret_cast<const T&>(t[k]);
            }
        } else {          // one-byte elements: N = 8 -> one 8-byte access
            const uint2 q = *reinterpret_cast<const uint2*>(reinterpret_cast<const char*>(p) + i);
            const unsigned w[2] = {q.x, q.y};
#pragma unroll
            for (int j = 0; j < N; ++j) v[j] = (T)(int8_t)((w[j / 4] >> (8 * (j % 4))) & 0xff);
        }
    } else {
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = p[i + j];
    }
}

template <class T, int N>
__device__ __forceinline__ void store_run(T* __restrict__ p, long i, bool vec, const T (&v)[N]) {
    if (vec) {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int j = 0; j < N; j += 4) {
                float t[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) t[k] = reinterpret_cast<const float&>(v[j + k]);
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + i + j) = make_float4(t[0], t[1], t[2], t[3]);
            }
        } else {
            unsigned w[2] = {0u, 0u};
#pragma unroll
            for (int j = 0; j < N; ++j) w[j / 4] |= ((unsigned)(uint8_t)v[j]) << (8 * (j % 4));
            *reinterpret_cast<uint2*>(reinterpret_cast<char*>(p) + i) = make_uint2(w[0], w[1]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < N; ++j) p[i + j] = v[j];
    }
}

// ---------------------------------------------------------------- elementwise kernels

template <int OP>
__global__ __launch_bounds__(kElwThreads) void elwise_unary_kernel(const float* __restrict__ x,
                                                                   float* __restrict__ y, long n, int vec) {
    constexpr int N = kElwPerThread;
    const long stride = (long)gridDim.x * kElwThreads * N;
    long i = ((long)blockIdx.x * kElwThreads + threadIdx.x) * N;
    for (; i + N <= n; i += stride) {
        float v[N];
        load_run<float, N>(x, i, false, vec, v);
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = unary_fn<OP>(v[j]);
        store_run<float, N>(y, i, vec, v);
    }
    if (i < n)      // the one thread that owns the ragged end
        for (long k = i; k < n; ++k) y[k] = unary_fn<OP>(x[k]);
}

template <int OP, class TX, class TY>
__global__ __launch_bounds__(kElwThreads) void elwise_binary_kernel(const TX* __restrict__ x, int xs,
                                                                    const TY* __restrict__ y, int ys,
                                                                    void* __restrict__ zv, long n, int vec) {
    typedef typename std::conditional<std::is_same<TX, float>::value || std::is_same<TY, float>::value, float, int>::type P;
    typedef BinaryFn<OP, P> F;
    typedef typename F::Out TZ;
    TZ* __restrict__ z = static_cast<TZ*>(zv);
    constexpr int N = kElwPerThread;
    const long stride = (long)gridDim.x * kElwThreads * N;
    long i = ((long)blockIdx.x * kElwThreads + threadIdx.x) * N;
    for (; i + N <= n; i += stride) {
        TX a[N];
        TY b[N];
        TZ c[N];
        load_run<TX, N>(x, i, xs, vec, a);
        load_run<TY, N>(y, i, ys, vec, b);
#pragma unroll
        for (int j = 0; j < N; ++j) c[j] = F::apply((P)a[j], (P)b[j]);
        store_run<TZ, N>(z, i, vec, c);
    }
    if (i < n)
        for (long k = i; k < n; ++k) z[k] = F::apply((P)x[xs ? 0 : k], (P)y[ys ? 0 : k]);
}

// One trip per workgroup up to 4 M workgroups: many short-lived workgroups stream faster on this chip
// than a resident-sized grid striding through the array (1 GiB add: 5.5-5.6 TB/s against 5.05).
static unsigned elw_grid(long n) {
    const long per_block = (long)kElwThreads * kElwPerThread;
    return (unsigned)std::max(1L, std::min(cdiv(n, per_block), 1L << 22));
}

static bool aligned_to(const void* p, int a) { return reinterpret_cast<uintptr_t>(p) % a == 0; }

template <int OP, class TX, class TY>
static void launch_binary(const void* x, int xs, const void* y, int ys, void* z, long n, hipStream_t st) {
    const int vec = aligned_to(x, 16) && aligned_to(y, 16) && aligned_to(z, 16);
    elwise_binary_kernel<OP, TX, TY><<<dim3(elw_grid(n)), dim3(kElwThreads), 0, st>>>(
        static_cast<const TX*>(x), xs, static_cast<const TY*>(y), ys, z, n, vec);
}

template <int OP>
static int dispatch_binary_types(int xdt, int ydt, const void* x, int xs, const void* y, int ys, void* z,
                                 long n, hipStream_t st) {
    if (xdt == CGT_AMD_F32 && ydt == CGT_AMD_F32) launch_binary<OP, float, float>(x, xs, y, ys, z, n, st);
    else if (xdt == CGT_AMD_F32 && ydt == CGT_AMD_I8) launch_binary<OP, float, int8_t>(x, xs, y, ys, z, n, st);
    else if (xdt == CGT_AMD_I8 && ydt == CGT_AMD_F32) launch_binary<OP, int8_t, float>(x, xs, y, ys, z, n, st);
    else if (xdt == CGT_AMD_I8 && ydt == CGT_AMD_I8) launch_binary<OP, int8_t, int8_t>(x, xs, y, ys, z, n, st);
    else {
        set_error("elwise_binary: unsupported dtypes %d, %d (f4 = %d and i1 = %d are)", xdt, ydt, CGT_AMD_F32, CGT_AMD_I8);
        return CGT_AMD_ERR_ARG;
    }
    CGT_LAUNCH_CHECK("elwise_binary_kernel");
    return CGT_AMD_OK;
}

// ---------------------------------------------------------------- Repeat

// out has the shape of x with the singleton axes named by the caller blown up.
// After merging neighbouring axes of the same kind the common cases are
// [R0][K][R1] -> out[(r0*K + k)*R1 + r1] = x[k]: bias [1,L,1,1] -> [B,L,m,n]
// (R0 = B, K = L, R1 = m*n), a row vector down a matrix (R1 = 1), a column
// across it (R0 = 1), a scalar everywhere (K = 1).
template <class T>
__global__ __launch_bounds__(kElwThreads) void repeat_rkr_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                                 long K, long R1, long n, int vec) {
    constexpr int N = kElwPerThread;
    const long stride = (long)gridDim.x * kElwThreads * N;
    long i = ((long)blockIdx.x * kElwThreads + threadIdx.x) * N;
    for (; i + N <= n; i += stride) {
        T v[N];
        long row = i / R1;                 // (r0*K + k)
        long r1 = i - row * R1;
        long k = row % K;
        T cur = x[k];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            v[j] = cur;
            if (++r1 == R1) {              // next row of the kept axis
                r1 = 0;
                if (++k == K) k = 0;
                cur = x[k];
            }
        }
        store_run<T, N>(out, i, vec, v);
    }
    if (i < n)
        for (long t = i; t < n; ++t) out[t] = x[(t / R1) % K];
}

struct RepeatDims {
    int nd;
    long oshape[8];
    long xstride[8];   // 0 on repeated axes
};

// Any other pattern: one division chain per element.
template <class T>
__global__ __launch_bounds__(kElwThreads) void repeat_generic_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                                     RepeatDims d, long n) {
    for (long o = (long)blockIdx.x * kElwThreads + threadIdx.x; o < n; o += (long)gridDim.x * kElwThreads) {
        long t = o, src = 0;
        for (int a = d.nd - 1; a >= 0; --a) {
            const long q = t / d.oshape[a];
            src += (t - q * d.oshape[a]) * d.xstride[a];
            t = q;
        }
        out[o] = x[src];
    }
}

// ---------------------------------------------------------------- Sum

// out[k] = sum over (r0, r1) of x[(r0*K + k)*R1 + r1]   (merged axes [R0][K][R1]).
// Workgroup (k, s0, s1) owns rows r0 in its share s0 and the r1 range of chunk
// s1; lanes run along r1 (contiguous).  Each lane adds its elements in a fixed
// order, the workgroup combines lanes in a fixed tree, partial sums go to
// ws[k][s0*S1 + s1], and sum_finish_kernel adds those in order: the result
// does not depend on scheduling.
constexpr int kSumThreads = 256;
constexpr int kSumChunk = kSumThreads * 32;     // r1 elements per workgroup and row

__device__ __forceinline__ float block_sum(float v) {
    __shared__ float red[kSumThreads / kWave];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.0f;
    if (threadIdx.x == 0)
        for (int w = 0; w < kSumThreads / kWave; ++w) total += red[w];
    return total;       // valid in thread 0
}

__global__ __launch_bounds__(kSumThreads) void sum_rkr_kernel(const float* __restrict__ x, float* __restrict__ ws,
                                                              long R0, long K, long R1, int S0, int S1, int vec) {
    const int s1 = blockIdx.x % S1;
    const int s0 = (blockIdx.x / S1) % S0;
    const long k = blockIdx.x / ((long)S1 * S0);
    const long rows_per = cdiv(R0, (long)S0);
    const long ra = s0 * rows_per, rb = ra + rows_per < R0 ? ra + rows_per : R0;
    const long ca = (long)s1 * kSumChunk, cb = ca + kSumChunk < R1 ? ca + kSumChunk : R1;
    float acc = 0.0f;
    for (long r0 = ra; r0 < rb; ++r0) {
        const float* row = x + (r0 * K + k) * R1;
        if (vec) {     // R1 % 4 == 0 and x 16-byte aligned: every row start is aligned
            float4 q[4];
            for (long c = ca + threadIdx.x * 4; c < cb; c += kSumThreads * 16) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    q[u] = c + u * kSumThreads * 4 < cb ? *reinterpret_cast<const float4*>(row + c + u * kSumThreads * 4)
                                                        : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int u = 0; u < 4; ++u) acc += (q[u].x + q[u].y) + (q[u].z + q[u].w);
            }
        } else {
            for (long c = ca + threadIdx.x; c < cb; c += kSumThreads * 4) {
                float q[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) q[u] = c + u * kSumThreads < cb ? row[c + u * kSumThreads] : 0.0f;
#pragma unroll
                for (int u = 0; u < 4; ++u) acc += q[u];
            }
        }
    }
    const float total = block_sum(acc);
    if (threadIdx.x == 0) ws[k * ((long)S0 * S1) + (long)s0 * S1 + s1] = total;
}

// Columns: merged axes [R0][K] (R1 == 1): lanes run along k (contiguous), each
// lane walks its share of r0.  ws[s0][k].
__global__ __launch_bounds__(kSumThreads) void sum_cols_kernel(const float* __restrict__ x, float* __restrict__ ws,
                                                               long R0, long K, int S0) {
    const long kblocks = cdiv(K, (long)kSumThreads);
    const long k = (blockIdx.x % kblocks) * kSumThreads + threadIdx.x;
    const int s0 = (int)(blockIdx.x / kblocks);
    if (k >= K) return;
    const long rows_per = cdiv(R0, (long)S0);
    const long ra = s0 * rows_per, rb = ra + rows_per < R0 ? ra + rows_per : R0;
    float acc = 0.0f;
    long r0 = ra;
    for (; r0 + 4 <= rb; r0 += 4) {
        float q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) q[u] = x[(r0 + u) * K + k];
#pragma unroll
        for (int u = 0; u < 4; ++u) acc += q[u];
    }
    for (; r0 < rb; ++r0) acc += x[r0 * K + k];
    ws[(long)s0 * K + k] = acc;
}

// out[k] = sum_p ws[k*stride_k + p*stride_p]: one workgroup per k, each lane
// adds its p (ascending), lanes combined in the fixed tree.
__global__ __launch_bounds__(kSumThreads) void sum_finish_kernel(const float* __restrict__ ws, float* __restrict__ out,
                                                                 long P, long stride_k, long stride_p) {
    const long k = blockIdx.x;
    float acc = 0.0f;
    // eight loads in flight per lane (clamped, unconditional), added in ascending p as before:
    // thousands of partials of a large sum are otherwise one chain of load latencies
    for (long p = threadIdx.x; p < P; p += kSumThreads * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const long q = p + (long)u * kSumThreads;
            v[u] = ws[k * stride_k + (q < P ? q : P - 1) * stride_p];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (p + (long)u * kSumThreads < P) acc += v[u];
    }
    const float total = block_sum(acc);
    if (threadIdx.x == 0) out[k] = total;
}

struct SumDims {
    int nk, nr;          // kept / reduced axes, outermost first
    long kshape[8], kstride[8];
    long rshape[8], rstride[8];
};

// Any other pattern: one thread per output element walks the reduced index
// space in row-major order (the reference's loop order).
__global__ __launch_bounds__(256) void sum_generic_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                          SumDims d, long nout, long nred) {
    const long o = (long)blockIdx.x * 256 + threadIdx.x;
    if (o >= nout) return;
    long t = o, base = 0;
    for (int a = d.nk - 1; a >= 0; --a) {
        const long q = t / d.kshape[a];
        base += (t - q * d.kshape[a]) * d.kstride[a];
        t = q;
    }
    float acc = 0.0f;
    for (long r = 0; r < nred; ++r) {
        long u = r, off = base;
        for (int a = d.nr - 1; a >= 0; --a) {
            const long q = u / d.rshape[a];
            off += (u - q * d.rshape[a]) * d.rstride[a];
            u = q;
        }
        acc += x[off];
    }
    out[o] = acc;
}

// Workspace for partial sums: one per stream, owned by the library (see common.h).
static float* sum_workspace(void* stream, size_t bytes) {
    return stream_workspace(stream, kWsSum, bytes, "sum");
}

// Merge neighbouring axes with the same flag; drops axes of extent 1.
static int merge_axes(int ndim, const long* shape, const int* flag, long* mshape, int* mflag) {
    int m = 0;
    for (int a = 0; a < ndim; ++a) {
        if (shape[a] == 1) continue;
        const int f = flag[a] ? 1 : 0;
        if (m > 0 && mflag[m - 1] == f) mshape[m - 1] *= shape[a];
        else {
            mshape[m] = shape[a];
            mflag[m] = f;
            ++m;
        }
    }
    return m;
}

// [R0][K][R1] view of a merged pattern whose flagged axes are F (flag 1) and the
// others are the single block K; false if the pattern has more blocks.
static bool as_rkr(int m, const long* mshape, const int* mflag, long* R0, long* K, long* R1) {
    *R0 = *K = *R1 = 1;
    if (m == 0) return true;
    if (m == 1) {
        if (mflag[0]) *R1 = mshape[0];
        else *K = mshape[0];
        return true;
    }
    if (m == 2) {
        if (mflag[0]) { *R0 = mshape[0]; *K = mshape[1]; }
        else { *K = mshape[0]; *R1 = mshape[1]; }
        return true;
    }
    if (m == 3 && mflag[0] && !mflag[1] && mflag[2]) {
        *R0 = mshape[0]; *K = mshape[1]; *R1 = mshape[2];
        return true;
    }
    return false;
}

template <class T>
static int launch_repeat(const T* x, int ndim, const long* oshape, const int* rep, T* out, long n, hipStream_t st) {
    long mshape[8], R0, K, R1;
    int mflag[8];
    const int m = merge_axes(ndim, oshape, rep, mshape, mflag);
    if (as_rkr(m, mshape, mflag, &R0, &K, &R1)) {
        const int vec = aligned_to(out, 16);
        repeat_rkr_kernel<T><<<dim3(elw_grid(n)), dim3(kElwThreads), 0, st>>>(x, out, K, R1, n, vec);
        CGT_LAUNCH_CHECK("repeat_rkr_kernel");
        return CGT_AMD_OK;
    }
    RepeatDims d;
    d.nd = ndim;
    long acc = 1;
    for (int a = ndim - 1; a >= 0; --a) {
        d.oshape[a] = oshape[a];
        d.xstride[a] = rep[a] ? 0 : acc;
        if (!rep[a]) acc *= oshape[a];
    }
    const long blocks = std::min(cdiv(n, (long)kElwThreads), 64L * kNumCU);
    repeat_generic_kernel<T><<<dim3((unsigned)blocks), dim3(kElwThreads), 0, st>>>(x, out, d, n);
    CGT_LAUNCH_CHECK("repeat_generic_kernel");
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_elwise_unary_f32(int op, long n, const float* x, float* y, void* stream) {
    CGT_ARG_CHECK(n >= 0, "elwise_unary: negative size");
    if (n == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(x && y, "elwise_unary: null pointer");
    hipStream_t st = as_stream(stream);
    const int vec = aligned_to(x, 16) && aligned_to(y, 16);
    dim3 grid(elw_grid(n)), block(kElwThreads);
#define CGT_UN(OP) \
    case OP: elwise_unary_kernel<OP><<<grid, block, 0, st>>>(x, y, n, vec); break;
    switch (op) {
        CGT_UN(CGT_AMD_UN_ABS) CGT_UN(CGT_AMD_UN_COS) CGT_UN(CGT_AMD_UN_EXP) CGT_UN(CGT_AMD_UN_LOG)
        CGT_UN(CGT_AMD_UN_NEG) CGT_UN(CGT_AMD_UN_SIGN) CGT_UN(CGT_AMD_UN_SIN) CGT_UN(CGT_AMD_UN_SQUARE)
        CGT_UN(CGT_AMD_UN_SQRT) CGT_UN(CGT_AMD_UN_TANH) CGT_UN(CGT_AMD_UN_SIGMOID)
        default:
            set_error("elwise_unary: unknown op %d", op);
            return CGT_AMD_ERR_ARG;
    }
#undef CGT_UN
    CGT_LAUNCH_CHECK("elwise_unary_kernel");
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_elwise_binary(int op, int xdtype, int ydtype, long n, const void* x, int x_is_scalar,
                                  const void* y, int y_is_scalar, void* z, void* stream) {
    CGT_ARG_CHECK(n >= 0, "elwise_binary: negative size");
    if (n == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(x && y && z, "elwise_binary: null pointer");
    hipStream_t st = as_stream(stream);
    const int xs = x_is_scalar != 0, ys = y_is_scalar != 0;
#define CGT_BIN(OP) \
    case OP: return dispatch_binary_types<OP>(xdtype, ydtype, x, xs, y, ys, z, n, st);
    switch (op) {
        CGT_BIN(CGT_AMD_BIN_MUL) CGT_BIN(CGT_AMD_BIN_ADD) CGT_BIN(CGT_AMD_BIN_SUB) CGT_BIN(CGT_AMD_BIN_DIV)
        CGT_BIN(CGT_AMD_BIN_LT) CGT_BIN(CGT_AMD_BIN_GT) CGT_BIN(CGT_AMD_BIN_LE) CGT_BIN(CGT_AMD_BIN_GE)
        CGT_BIN(CGT_AMD_BIN_POW) CGT_BIN(CGT_AMD_BIN_EQ) CGT_BIN(CGT_AMD_BIN_NE)
        default:
            set_error("elwise_binary: unknown op %d", op);
            return CGT_AMD_ERR_ARG;
    }
#undef CGT_BIN
}

CGT_API int cgt_amd_repeat(const void* x, int itemsize, int ndim, const long* outshape, const int* repeated,
                           void* out, void* stream) {
    CGT_ARG_CHECK(ndim >= 0 && ndim <= 8, "repeat: ndim %d out of range (0..8)", ndim);
    CGT_ARG_CHECK(ndim == 0 || (outshape && repeated), "repeat: null shape");
    long n = 1;
    for (int a = 0; a < ndim; ++a) {
        CGT_ARG_CHECK(outshape[a] >= 0, "repeat: negative shape");
        n *= outshape[a];
    }
    if (n == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(x && out, "repeat: null pointer");
    hipStream_t st = as_stream(stream);
    if (itemsize == 4)
        return launch_repeat<float>(static_cast<const float*>(x), ndim, outshape, repeated, static_cast<float*>(out), n, st);
    if (itemsize == 1)
        return launch_repeat<int8_t>(static_cast<const int8_t*>(x), ndim, outshape, repeated, static_cast<int8_t*>(out), n, st);
    set_error("repeat: itemsize %d not supported (4 and 1 are)", itemsize);
    return CGT_AMD_ERR_ARG;
}

CGT_API int cgt_amd_sum_f32(const float* x, int ndim, const long* shape, const int* reduced, float* out,
                            void* stream) {
    CGT_ARG_CHECK(ndim >= 0 && ndim <= 8, "sum: ndim %d out of range (0..8)", ndim);
    CGT_ARG_CHECK(ndim == 0 || (shape && reduced), "sum: null shape");
    long nin = 1, nout = 1;
    for (int a = 0; a < ndim; ++a) {
        CGT_ARG_CHECK(shape[a] >= 0, "sum: negative shape");
        nin *= shape[a];
        if (!reduced[a]) nout *= shape[a];
    }
    if (nout == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(out, "sum: null output");
    hipStream_t st = as_stream(stream);
    if (nin == 0) return cgt_amd_fill_u32(out, 0u, nout, stream);     // empty sums are 0
    CGT_ARG_CHECK(x, "sum: null input");
    long mshape[8], R0, K, R1;
    int mflag[8];
    const int m = merge_axes(ndim, shape, reduced, mshape, mflag);
    if (as_rkr(m, mshape, mflag, &R0, &K, &R1)) {
        if (R0 == 1 && R1 == 1) {                                     // nothing to add up
            CGT_HIP_TRY(hipMemcpyAsync(out, x, nin * sizeof(float), hipMemcpyDeviceToDevice, st));
            return CGT_AMD_OK;
        }
        const long target = 8L * kNumCU;                              // workgroups wanted
        if (R1 == 1) {
            const long kblocks = cdiv(K, (long)kSumThreads);
            const int S0 = (int)std::max(1L, std::min(std::min(R0 / 4 + 1, 1024L), cdiv(target, kblocks)));
            float* ws = sum_workspace(stream, (size_t)S0 * K * sizeof(float));
            if (!ws) return CGT_AMD_ERR_NOMEM;
            CGT_ARG_CHECK(kblocks * S0 < (1L << 31) && K < (1L << 31), "sum: too many workgroups");
            sum_cols_kernel<<<dim3((unsigned)(kblocks * S0)), dim3(kSumThreads), 0, st>>>(x, ws, R0, K, S0);
            CGT_LAUNCH_CHECK("sum_cols_kernel");
            sum_finish_kernel<<<dim3((unsigned)K), dim3(kSumThreads), 0, st>>>(ws, out, S0, 1, K);
            CGT_LAUNCH_CHECK("sum_finish_kernel");
            return CGT_AMD_OK;
        }
        const long S1 = cdiv(R1, (long)kSumChunk);
        const long S0 = std::max(1L, std::min(R0, cdiv(target, K * S1)));
        CGT_ARG_CHECK(K * S0 * S1 < (1L << 31) && S0 * S1 < (1L << 24), "sum: too many workgroups");
        float* ws = sum_workspace(stream, (size_t)(K * S0 * S1) * sizeof(float));
        if (!ws) return CGT_AMD_ERR_NOMEM;
        const int vec = R1 % 4 == 0 && aligned_to(x, 16);
        sum_rkr_kernel<<<dim3((unsigned)(K * S0 * S1)), dim3(kSumThreads), 0, st>>>(x, ws, R0, K, R1, (int)S0, (int)S1, vec);
        CGT_LAUNCH_CHECK("sum_rkr_kernel");
        sum_finish_kernel<<<dim3((unsigned)K), dim3(kSumThreads), 0, st>>>(ws, out, S0 * S1, S0 * S1, 1);
        CGT_LAUNCH_CHECK("sum_finish_kernel");
        return CGT_AMD_OK;
    }
    SumDims d;
    d.nk = d.nr = 0;
    long stride = 1, strides[8];
    for (int a = ndim - 1; a >= 0; --a) {
        strides[a] = stride;
        stride *= shape[a];
    }
    for (int a = 0; a < ndim; ++a) {
        if (reduced[a]) {
            d.rshape[d.nr] = shape[a];
            d.rstride[d.nr++] = strides[a];
        } else {
            d.kshape[d.nk] = shape[a];
            d.kstride[d.nk++] = strides[a];
        }
    }
    sum_generic_kernel<<<dim3((unsigned)cdiv(nout, 256L)), dim3(256), 0, st>>>(x, out, d, nout, nin / nout);
    CGT_LAUNCH_CHECK("sum_generic_kernel");
    return CGT_AMD_OK;
}

CGT_API int cgt_amd_fill_f32(float* dst, float value, long count, void* stream) {
    unsigned int bits;
    static_assert(sizeof(bits) == sizeof(value), "float is 32 bits");
    memcpy(&bits, &value, sizeof(bits));
    return cgt_amd_fill_u32(dst, bits, count, stream);
}
