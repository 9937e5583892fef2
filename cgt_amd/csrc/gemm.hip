// fp32 GEMM on the gfx950 matrix cores: C[M,N] = op(A) . op(B), row-major.
//
// Tiling: a 256-thread workgroup (4 wavefronts, 2x2) owns a 128x128 tile of C;
// each wavefront owns 64x64 = 2x2 blocks of v_mfma_f32_32x32x2_f32 (true fp32
// in, fp32 accumulate; 64 accumulator registers per lane).  K is walked in
// slices of 16 through double-buffered LDS tiles: while the matrix cores work
// on slice t from LDS buffer t&1, the global loads of slice t+1 are in flight
// into registers and are written to the other buffer afterwards -- one
// barrier per slice.
//
// LDS layouts, chosen so that both the 16-byte global loads and the fragment
// reads are contiguous:
//   operand stored k-contiguous in memory (A not transposed, B transposed):
//       tile[row][k], row stride 20 floats; a lane reads its four k values of
//       an 8-wide k group with one 16-byte LDS read, conflict-free;
//   operand stored row-contiguous (A transposed, B not transposed):
//       tile[k][row], row stride 132 floats; four 4-byte reads per k group.
// Inside an 8-wide k group MFMA step i takes k = 4*half + i from lane half
// `half` (lanes 0-31 / 32-63).  A and B use the same assignment, so the
// products match; only the summation order inside the group differs from
// k-ascending.
//
// Skinny outputs (few tiles, long K: the conv weight gradient) are split along
// K into a workspace of partial tiles, reduced afterwards in a fixed order, so
// the result is deterministic.
#include "common.h"
#include <algorithm>
#include <mutex>
#include <unordered_map>

namespace cgt_amd {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, KT = 16;
constexpr int kGemmThreads = 256;
constexpr int LDK = KT + 4;    // [128][LDK]
constexpr int LDM = BM + 4;    // [KT][LDM]
constexpr int kTileFloats = (BM * LDK > KT * LDM) ? BM * LDK : KT * LDM;
static_assert(BM == BN, "operand tiles share one layout");

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    long lda, ldb, ldc;
    long sA, sB, sC;   // batch strides (elements)
    int M, N, K;
    int tiles_m, tiles_n;
    int splits;        // > 1: partial products go to ws[split][M][N]
    int kchunk;        // K range per split, multiple of KT
    float* ws;
    int vecA, vecB;    // 16-byte global loads allowed for A / B
};

// One 128 x KT operand tile, 2 float4 per thread.
// KC: element (r, k) lives at p[r*ld + k]; otherwise at p[k*ld + r].
template <bool KC>
struct OperandTile {
    float4 v[2];

    __device__ __forceinline__ void load(const float* __restrict__ p, long ld, int r0, int R,
                                         int k0, int kend, bool vec) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            if (KC) {
                const int row = r0 + (idx >> 2), k = k0 + (idx & 3) * 4;
                const float* src = p + (long)row * ld + k;
                if (vec && row < R && k + 3 < kend) {
                    v[i] = *reinterpret_cast<const float4*>(src);
                } else {
                    float t[4] = {0.f, 0.f, 0.f, 0.f};
                    if (row < R) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (k + j < kend) t[j] = src[j];
                    }
                    v[i] = make_float4(t[0], t[1], t[2], t[3]);
                }
            } else {
                const int k = k0 + (idx >> 5), row = r0 + (idx & 31) * 4;
                const float* src = p + (long)k * ld + row;
                if (vec && k < kend && row + 3 < R) {
                    v[i] = *reinterpret_cast<const float4*>(src);
                } else {
                    float t[4] = {0.f, 0.f, 0.f, 0.f};
                    if (k < kend) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (row + j < R) t[j] = src[j];
                    }
                    v[i] = make_float4(t[0], t[1], t[2], t[3]);
                }
            }
        }
    }

    __device__ __forceinline__ void store(float* __restrict__ tile) const {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            if (KC)
                *reinterpret_cast<float4*>(tile + (idx >> 2) * LDK + (idx & 3) * 4) = v[i];
            else
                *reinterpret_cast<float4*>(tile + (idx >> 5) * LDM + (idx & 31) * 4) = v[i];
        }
    }

    // the four k values (k group kk, this lane's half) of tile row `row`
    static __device__ __forceinline__ void frag(const float* __restrict__ tile, int row, int kk,
                                                int half, float (&f)[4]) {
        if (KC) {
            const float4 t = *reinterpret_cast<const float4*>(tile + row * LDK + kk * 8 + half * 4);
            f[0] = t.x; f[1] = t.y; f[2] = t.z; f[3] = t.w;
        } else {
            const float* q = tile + (kk * 8 + half * 4) * LDM + row;
#pragma unroll
            for (int j = 0; j < 4; ++j) f[j] = q[j * LDM];
        }
    }
};

// Workgroups are handed to the 8 XCDs round-robin by linear id; remap so that
// each XCD (one L2) works on a contiguous range of tiles.
__device__ __forceinline__ int xcd_remap(int id, int n) {
    const int q = n / kNumXCD, r = n % kNumXCD;
    const int xcd = id % kNumXCD, local = id / kNumXCD;
    return xcd * q + min(xcd, r) + local;
}

template <bool AKC, bool BKC>
__global__ __launch_bounds__(kGemmThreads, 2) void sgemm_kernel(GemmArgs a) {
    __shared__ __attribute__((aligned(16))) float As[2][kTileFloats];
    __shared__ __attribute__((aligned(16))) float Bs[2][kTileFloats];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;

    // tile order: groups of 8 tile rows, column-major inside a group, so tiles
    // that run together share A row panels and B column panels in L2
    const int lid = xcd_remap(blockIdx.x, a.tiles_m * a.tiles_n);
    constexpr int GM = 8;
    const int per_group = GM * a.tiles_n;
    const int group = lid / per_group, in_group = lid - group * per_group;
    const int first_m = group * GM;
    const int gsz = min(a.tiles_m - first_m, GM);
    const int tm = first_m + in_group % gsz, tn = in_group / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    const int z = blockIdx.y;
    const int batch = z / a.splits, split = z - batch * a.splits;
    const int kbeg = split * a.kchunk;
    const int kend = min(a.K, kbeg + a.kchunk);
    const float* A = a.A + batch * a.sA;
    const float* B = a.B + batch * a.sB;

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int nk = (kend - kbeg + KT - 1) / KT;
    OperandTile<AKC> ta;
    OperandTile<BKC> tb;
    if (nk > 0) {
        ta.load(A, a.lda, m0, a.M, kbeg, kend, a.vecA);
        tb.load(B, a.ldb, n0, a.N, kbeg, kend, a.vecB);
        ta.store(As[0]);
        tb.store(Bs[0]);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nk;
        if (more) {
            const int k0 = kbeg + (kt + 1) * KT;
            ta.load(A, a.lda, m0, a.M, k0, kend, a.vecA);
            tb.load(B, a.ldb, n0, a.N, k0, kend, a.vecB);
        }
        const float* as = As[cur];
        const float* bs = Bs[cur];
#pragma unroll
        for (int kk = 0; kk < KT / 8; ++kk) {
            float af[2][4], bf[2][4];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                OperandTile<AKC>::frag(as, wm * 64 + i * 32 + l32, kk, half, af[i]);
                OperandTile<BKC>::frag(bs, wn * 64 + i * 32 + l32, kk, half, bf[i]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][s], bf[j][s],
                                                                         acc[i][j], 0, 0, 0);
        }
        if (more) {
            ta.store(As[cur ^ 1]);
            tb.store(Bs[cur ^ 1]);
        }
        __syncthreads();
    }

    // accumulator element e of a 32x32 block: row 8*(e/4) + 4*half + e%4, column l32
    float* out;
    long ldo;
    if (a.splits > 1) {
        out = a.ws + (long)split * a.M * a.N;
        ldo = a.N;
    } else {
        out = a.C + batch * a.sC;
        ldo = a.ldc;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn * 64 + j * 32 + l32;
            if (col >= a.N) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * 64 + i * 32 + 8 * (e / 4) + 4 * half + (e % 4);
                if (row < a.M) out[(long)row * ldo + col] = acc[i][j][e];
            }
        }
}

// C[r][c] = sum_s ws[s][r][c], s ascending.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws,
                                                            float* __restrict__ C, long MN, int N,
                                                            long ldc, int splits) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < MN;
         i += (long)gridDim.x * blockDim.x) {
        float s = 0.0f;
        for (int k = 0; k < splits; ++k) s += ws[(long)k * MN + i];
        const long r = i / N, c = i - r * N;
        C[r * ldc + c] = s;
    }
}

// Split-K workspaces, one per stream, grown on demand and kept.
struct Workspace {
    float* ptr = nullptr;
    size_t bytes = 0;
};
static std::mutex g_ws_mutex;
static std::unordered_map<void*, Workspace> g_ws;

static float* get_workspace(void* stream, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace& w = g_ws[stream];
    if (w.bytes >= bytes) return w.ptr;
    if (w.ptr) (void)hipFree(w.ptr);  // hipFree waits for work that may still read it
    w.ptr = nullptr;
    w.bytes = 0;
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    w.ptr = static_cast<float*>(p);
    w.bytes = bytes;
    return w.ptr;
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

static int gemm_dispatch(int tA, int tB, long P, long M, long N, long K, const float* A, long lda,
                         long sA, const float* B, long ldb, long sB, float* C, long ldc, long sC,
                         void* stream) {
    CGT_ARG_CHECK(P >= 0 && M >= 0 && N >= 0 && K >= 0, "sgemm: negative size");
    if (P == 0 || M == 0 || N == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(A || K == 0, "sgemm: null A");
    CGT_ARG_CHECK(B || K == 0, "sgemm: null B");
    CGT_ARG_CHECK(C, "sgemm: null C");
    CGT_ARG_CHECK(M < (1L << 31) - BM && N < (1L << 31) - BN && K < (1L << 31) - KT && P < 65536,
                  "sgemm: size too large");
    CGT_ARG_CHECK(lda >= (tA ? M : K) && ldb >= (tB ? K : N) && ldc >= N,
                  "sgemm: leading dimension too small (lda=%ld ldb=%ld ldc=%ld)", lda, ldb, ldc);
    GemmArgs a;
    a.A = A; a.B = B; a.C = C;
    a.lda = lda; a.ldb = ldb; a.ldc = ldc;
    a.sA = sA; a.sB = sB; a.sC = sC;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.tiles_m = (int)cdiv(M, BM);
    a.tiles_n = (int)cdiv(N, BN);
    const long tiles = (long)a.tiles_m * a.tiles_n;
    CGT_ARG_CHECK(tiles < (1L << 31), "sgemm: too many tiles");
    a.vecA = (lda % 4 == 0 && sA % 4 == 0 && aligned16(A)) ? 1 : 0;
    a.vecB = (ldb % 4 == 0 && sB % 4 == 0 && aligned16(B)) ? 1 : 0;
    a.splits = 1;
    a.kchunk = (int)(cdiv(std::max(K, 1L), KT) * KT);
    a.ws = nullptr;
    if (P == 1 && tiles < 512 && K >= 64 * KT) {
        long want = std::max(1L, 1024 / tiles);
        want = std::min(want, K / (8 * KT));                    // at least 8 slices per split
        const long cap = (256L << 20) / (M * N * (long)sizeof(float));  // workspace <= 256 MiB
        want = std::min(want, std::max(1L, cap));
        if (want > 1) {
            a.kchunk = (int)(cdiv(cdiv(K, want), KT) * KT);
            a.splits = (int)cdiv(K, a.kchunk);
        }
        if (a.splits > 1) {
            a.ws = get_workspace(stream, (size_t)a.splits * M * N * sizeof(float));
            if (!a.ws) {
                set_error("sgemm: cannot allocate split-K workspace");
                return CGT_AMD_ERR_NOMEM;
            }
        }
    }
    hipStream_t st = as_stream(stream);
    dim3 grid((unsigned)tiles, (unsigned)(P * a.splits)), block(kGemmThreads);
    if (!tA && !tB) sgemm_kernel<true, false><<<grid, block, 0, st>>>(a);
    else if (!tA && tB) sgemm_kernel<true, true><<<grid, block, 0, st>>>(a);
    else if (tA && !tB) sgemm_kernel<false, false><<<grid, block, 0, st>>>(a);
    else sgemm_kernel<false, true><<<grid, block, 0, st>>>(a);
    CGT_LAUNCH_CHECK("sgemm_kernel");
    if (a.splits > 1) {
        const long MN = M * N;
        long blocks = std::min(cdiv(MN, 256L), 1L << 16);
        splitk_reduce_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a.ws, C, MN, (int)N, ldc, a.splits);
        CGT_LAUNCH_CHECK("splitk_reduce_kernel");
    }
    return CGT_AMD_OK;
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_sgemm(int tA, int tB, long M, long N, long K, const float* A, long lda,
                          const float* B, long ldb, float* C, long ldc, void* stream) {
    return gemm_dispatch(tA, tB, 1, M, N, K, A, lda, 0, B, ldb, 0, C, ldc, 0, stream);
}

CGT_API int cgt_amd_sgemm_batched(int tA, int tB, long P, long M, long N, long K, const float* A,
                                  long lda, long strideA, const float* B, long ldb, long strideB,
                                  float* C, long ldc, long strideC, void* stream) {
    return gemm_dispatch(tA, tB, P, M, N, K, A, lda, strideA, B, ldb, strideB, C, ldc, strideC, stream);
}
