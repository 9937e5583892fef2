// fp32 GEMM on the gfx950 matrix cores: C[M,N] = op(A) . op(B), row-major.
//
// Tiling: a 256-thread workgroup (4 wavefronts) owns a BM x BN tile of C; each
// wavefront owns TM x TN blocks of v_mfma_f32_32x32x2_f32 (true fp32 in, fp32
// accumulate, 16 accumulator registers per block and lane).  The default is
// 128x128 with 2x2 wavefronts of 2x2 blocks; narrow outputs (the conv GEMMs
// have N = 32 / 64 / 96 filters, or M = 96 for the weight gradient) use
// 128 x {32,64,96} with the wavefronts stacked along M, or {64,96} x 128 with the
// wavefronts stacked along N, so no matrix-core work is spent on padding.
//
// K is walked in slices of 16 through double-buffered LDS tiles: while the
// matrix cores work on slice t from LDS buffer t&1, the global loads of slice
// t+1 are in flight -- straight into the other LDS buffer
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions)
// when the tile and the slice are whole, through registers with bounds tests
// otherwise -- one barrier per slice.
//
// LDS layouts are dense, because a direct load deposits a wavefront's 64 x 16
// bytes lane after lane:
//   operand stored k-contiguous in memory (A not transposed, B transposed):
//       tile[row][16]; the four 16-byte chunks of a row are permuted (chunk c
//       of row r sits in slot c ^ ((r >> 2) & 3)) -- the permutation is applied
//       by choosing which chunk a lane fetches, costs nothing, and makes the
//       16-byte fragment reads (a lane reads its four k values of an 8-wide k
//       group at once) and the register-path writes bank-conflict free;
//   operand stored row-contiguous (A transposed, B not transposed):
//       tile[k][rows]; four 4-byte reads per k group, lanes on consecutive rows.
// Inside an 8-wide k group MFMA step i takes k = 4*half + i from lane half
// `half` (lanes 0-31 / 32-63).  A and B use the same assignment, so the
// products match; only the summation order inside the group differs from
// k-ascending.
//
// Global loads are 16 bytes per lane at any 4-byte aligned address (the
// im2col buffers of the AlexNet and CIFAR layers have Z = 363 or 75 floats per
// row: global_load_dwordx4 does not need more alignment than a float's).
//
// fp32 MFMAs and other vector instructions do not overlap on a SIMD of this
// chip, and a wavefront that is loading or storing while its neighbours
// multiply is issued about one instruction per MFMA of theirs.  The steady
// state therefore avoids vector address arithmetic altogether: loads and C
// stores are "wave-uniform origin (scalar registers, advanced with scalar
// adds) + one fixed 32-bit offset per lane (+ immediate)", bounds tests run
// only on edge tiles and on a ragged last K slice.
//
// Skinny outputs (few tiles, long K: the conv weight gradient) are split along
// K into a workspace of partial tiles, reduced afterwards in a fixed order, so
// the result is deterministic.  The grid is one-dimensional and ordered so
// that workgroups sharing an operand panel land on the same XCD (same L2) at
// about the same time.
#include "common.h"
#include <algorithm>
#include <mutex>
#include <type_traits>

namespace cgt_amd {

typedef float v16f __attribute__((ext_vector_type(16)));

// Four consecutive floats at any 4-byte aligned address: global_load_dwordx4
// needs no more alignment than that (rows of 363 floats start anywhere).
struct __attribute__((packed, aligned(4))) float4u {
    float x, y, z, w;
};

constexpr int KT = 16;
constexpr int kGemmThreads = 256;
constexpr int LDK = KT;        // row stride of a k-contiguous tile [ROWS][LDK]: dense
// slot of 16-byte chunk `chunk` in row `row` of a k-contiguous tile (an involution)
__device__ __forceinline__ int chunk_pos(int row, int chunk) { return chunk ^ ((row >> 2) & 3); }

// One 16-byte-per-lane load straight into LDS: lane l's data lands at lds_addr + 16*l.
// Written as inline asm so that the compiler's wait-count insertion does not see it and
// make every later LDS read wait for it; the loops wait with explicit s_waitcnt vmcnt.
// m0 (the LDS base of the load) is written here and not listed as clobbered: the AMDGPU
// backend reserves m0 -- it never keeps a value in it across other code, it sets it
// immediately before each instruction of its own that reads it -- and rejects the listing
// ("inline asm clobber list contains reserved registers: m0").
__device__ __forceinline__ void load_to_lds16(const void* base, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

struct GemmArgs {
    const float* A;
    const float* B;
    float* C;
    long lda, ldb, ldc;
    long sA, sB, sC;   // batch strides (elements)
    int M, N, K;
    int tiles_m, tiles_n;
    int batch;
    int splits;        // > 1: partial products go to ws[split][M][N]
    int kchunk;        // K range per split, multiple of KT
    float* ws;
    // tail split: workgroups [0, main_wgs) own whole tiles; the remaining
    // tail_tiles tiles are cut into tail_splits K ranges each so that every CU
    // gets an equal share of the last, partial round.  Pieces go to ws as
    // [piece][BM][BN]; tail_reduce_kernel adds them up in order.
    int main_wgs, tail_splits, tail_kchunk;
    int wide;          // a leading dimension too large for 32-bit tile offsets: tested loads everywhere
    // Implicit convolution (stride 1, pad = (kernel-1)/2): an operand is read straight
    // from the zero-padded image [B][C][plane] instead of a column buffer.
    //   mode 3 (forward / data gradient): C[n][q] = sum_k Wk[n][k] * img[b][c][q + tapoff]:
    //     the columns are the pixels q = h*Wp + w of the padded grid, cv_tpi tiles of 128
    //     columns per image, and the result is written straight into NCHW (junk pixels
    //     skipped) with an optional per-row bias and x * (x >= 0).  The K axis is ordered
    //     (block of 16 channels, tap, channel in the block): a slice of 16 is one tap of one
    //     channel block, and the taps of a block follow each other, so the block's pixels
    //     (16 KB per tile) are fetched once and re-read from cache;
    //   mode 2 (weight gradient): the K axis runs over those pixels, cv_spi slices per
    //     image; A[l][q] and B[tap*C + c][q] are both q-contiguous.
    int conv;
    int cv_wp, cv_kw, cv_kh, cv_tpi, cv_spi, cv_c;    // padded width, kernel, tiles / slices per image, C
    int cv_h, cv_w, cv_relu;                          // mode 3: image extents, rectify flag
    const float* cv_bias;                             // mode 3: per-row (output channel) bias or null
    signed char* cv_mask;                             // mode 3: where (x >= 0) goes as int8, or null
    long cv_plane, cv_imgA, cv_imgB;                  // plane stride and per-image strides (floats)
    //   mode 1 (forward over a column buffer): a plain NT product C[l][n] = sum_z W[l][z] * col[n][z]
    //     whose columns n = (image, pixel) are written as out[image][l][pixel] (cv_plane =
    //     pixels per image), with the same optional bias / rectify / mask as mode 3.
    // K cut per image (weight gradient from an NCHW cotangent, plain kernel): split s is piece
    // s % kspi of image s / kspi; the image's K range is [img * kimg, (img + 1) * kimg) and
    // its A operand starts aimg floats further per image (A is [image][M][kimg], k-contiguous).
    int kimg, kspi;
    long aimg;
    // Patch gather (GATHER != 0): the B operand is not a column buffer but the image itself,
    // [images][g_C][g_H][g_W]; element (pixel n, patch index z) of the column buffer is read
    // from g_x where im2col would have copied it from (0 outside the image).
    //   GATHER 1 (forward): B is k-contiguous, rows = pixels n, k = z.  g_koff[k] = byte offset of
    //     patch element k inside an image, 4 * ((c * H + ho) * W + wo), -1 for k past the patch length
    //     (the table is padded to a multiple of 16); g_khw[k] = (ho << 16) | wo (padded layers).
    //   GATHER 2 (weight gradient): B is row-contiguous, rows = patch elements z, k = pixels.
    const float* g_x;
    const int* g_koff;
    const int* g_khw;
    int g_C, g_H, g_W, g_kh, g_kw, g_ph, g_pw, g_sh, g_sw, g_OW, g_P;   // g_P = output pixels per image
};

// One ROWS x KT operand tile, moved with 16-byte accesses.
// KC: element (r, k) lives at p[r*ld + k]; otherwise at p[k*ld + r].
//
// Every non-matrix instruction a wavefront issues takes its SIMD away from the
// matrix pipe for a few cycles (fp32 MFMAs and vector ALU work do not overlap
// on this chip: measured +6 cycles per VALU instruction against 64 per MFMA), so
// the steady-state loads carry no address arithmetic: a thread's byte offsets
// inside the tile are fixed for the whole kernel (goff), the tile origin of the
// current K slice is a wave-uniform pointer advanced by scalar adds, and the
// hardware adds the two (global_load_dwordx4 v, v_off, s[base]).
template <bool KC, int ROWS>
struct OperandTile {
    static constexpr int LDM = ROWS;       // row-contiguous tile [KT][LDM]: dense
    static constexpr int kFloats = KC ? ROWS * LDK : KT * LDM;
    static constexpr int kElems = ROWS * KT;
    static constexpr int NV = (kElems / 4 + kGemmThreads - 1) / kGemmThreads;   // 16-byte pieces per thread
    float v[NV * 4];
    unsigned goff[NV];

    // piece i of this thread exists (always, when the tile is a whole number of rounds)
    static __device__ __forceinline__ bool has(int i) {
        return (i + 1) * kGemmThreads * 4 <= kElems || (threadIdx.x + i * kGemmThreads) * 4 < kElems;
    }

    // needs (ROWS - 1) * ld * 4 + 64 < 2^32 (the host checks)
    // rows_valid < ROWS (k-contiguous operands of the convolution products only): rows past
    // it load the last valid row again -- valid memory, and what they produce is never stored
    __device__ __forceinline__ void init_offsets(long ld, int rows_valid = ROWS) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            // the piece this thread fetches is the one whose LDS slot it fills: slot idx & 3
            // of row idx >> 2 holds chunk chunk_pos(row, idx & 3) (the permutation is an involution)
            const long e = KC ? (long)min(idx >> 2, rows_valid - 1) * ld + chunk_pos(idx >> 2, idx & 3) * 4
                              : (long)(idx / (ROWS / 4)) * ld + (idx % (ROWS / 4)) * 4;
            goff[i] = (unsigned)(e * 4);
        }
    }

    // Weight gradient of a convolution: row n of the (tap, channel) axis is channel n % C of
    // the padded image shifted by tap n / C, so the row's offset is not n * ld but folds the
    // tap's shift in; a tile may span several taps.  Rows past n_valid repeat the last one.
    __device__ __forceinline__ void init_offsets_taps(long plane, int n0, int n_valid, int C, int kw, int wp) {
        static_assert(KC, "pixel-contiguous operand");
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            const int n = min(n0 + (idx >> 2), n_valid - 1);
            const int tap = n / C, c = n - tap * C;
            const int ho = tap / kw, wo = tap - ho * kw;
            const long e = (long)c * plane + (long)ho * wp + wo + chunk_pos(idx >> 2, idx & 3) * 4;
            goff[i] = (unsigned)(e * 4);
        }
    }

    // the whole tile slice is in range: origin = address of tile element (0, 0) of this slice
    // `offs`: the goff of the operand's first register set (a second set, used for deeper
    // prefetch, shares it instead of holding a copy in four more registers)
    __device__ __forceinline__ void load_fast(const char* __restrict__ origin, unsigned (&offs)[NV]) {
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (has(i)) {
                // the empty asm keeps origin + offset from being hoisted into a per-lane
                // 64-bit pointer that is then advanced with vector adds every slice
                asm volatile("" : "+v"(offs[i]));
                const float4u q = *reinterpret_cast<const float4u*>(origin + offs[i]);
                v[i * 4] = q.x; v[i * 4 + 1] = q.y; v[i * 4 + 2] = q.z; v[i * 4 + 3] = q.w;
            }
    }

    // the same pieces straight into the LDS tile (dense layout: piece idx -> floats [4*idx, 4*idx+4))
    __device__ __forceinline__ void load_direct(const char* __restrict__ origin, unsigned (&offs)[NV],
                                                float* tile, int wave_u) const {
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if ((i + 1) * kGemmThreads * 4 <= kElems || (wave_u * 64 + i * kGemmThreads) * 4 < kElems) {
                const unsigned lds = (unsigned)(size_t)(__attribute__((address_space(3))) float*)tile +
                                     (unsigned)(i * kGemmThreads + wave_u * 64) * 16u;
                load_to_lds16(origin, offs[i], lds);
            }
    }

    // bounds-tested: rows >= R and k >= kend read as zero
    __device__ __forceinline__ void load_checked(const float* __restrict__ p, long ld, int r0, int R,
                                                 int k0, int kend) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;     // float4 index
            float t[4] = {0.f, 0.f, 0.f, 0.f};
            if (has(i)) {
                if (KC) {
                    // like the untested loads: the chunk that belongs in this thread's LDS slot
                    const int row = r0 + (idx >> 2), k = k0 + chunk_pos(idx >> 2, idx & 3) * 4;
                    const float* src = p + (long)row * ld + k;
                    if (row < R && k + 3 < kend) {
                        const float4u q = *reinterpret_cast<const float4u*>(src);
                        t[0] = q.x; t[1] = q.y; t[2] = q.z; t[3] = q.w;
                    } else if (row < R) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (k + j < kend) t[j] = src[j];
                    }
                } else {
                    const int k = k0 + idx / (ROWS / 4), row = r0 + (idx % (ROWS / 4)) * 4;
                    const float* src = p + (long)k * ld + row;
                    if (k < kend && row + 3 < R) {
                        const float4u q = *reinterpret_cast<const float4u*>(src);
                        t[0] = q.x; t[1] = q.y; t[2] = q.z; t[3] = q.w;
                    } else if (k < kend) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (row + j < R) t[j] = src[j];
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) v[i * 4 + j] = t[j];
        }
    }

    __device__ __forceinline__ void store(float* __restrict__ tile) const {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            if (has(i)) {
                float* dst = KC ? tile + (idx >> 2) * LDK + (idx & 3) * 4
                                : tile + (idx / (ROWS / 4)) * LDM + (idx % (ROWS / 4)) * 4;
                *reinterpret_cast<float4*>(dst) = make_float4(v[i * 4], v[i * 4 + 1], v[i * 4 + 2], v[i * 4 + 3]);
            }
        }
    }

    // the four k values (k group kk, this lane's half) of tile row `row`
    static __device__ __forceinline__ void frag(const float* __restrict__ tile, int row, int kk,
                                                int half, float (&f)[4]) {
        if (KC) {
            const float4 t = *reinterpret_cast<const float4*>(tile + row * LDK + chunk_pos(row, kk * 2 + half) * 4);
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

// WGM x WGN wavefronts, each TM x TN blocks of 32x32.
// PIPE selects the software-pipelined main loop (k-contiguous operands only).
// DEEP (plain loop only) keeps two K slices of global loads in flight instead of one.
template <bool AKC, bool BKC, bool PIPE, int WGM, int WGN, int TM, int TN, bool DEEP = false, int CONV = 0, int GATHER = 0,
          bool GPAD = false>
__global__ __launch_bounds__(kGemmThreads, PIPE ? 3 : 4) void sgemm_kernel(GemmArgs a) {
    static_assert(GATHER == 0 || (!PIPE && !DEEP && AKC && ((GATHER == 1 && BKC && CONV == 1) || (GATHER == 2 && !BKC && CONV == 0))),
                  "patch gather: forward = NT with the NCHW epilogue, weight gradient = NN with K cut per image");
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    static_assert(CONV == 0 || (CONV >= 1 && CONV <= 3 && !PIPE && !DEEP && AKC && BKC == (CONV != 3)),
                  "convolution products: plain loop; the image operand is B, row-contiguous in mode 3; "
                  "both operands k-contiguous in modes 1 and 2");
    constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
    typedef OperandTile<AKC, BM> TileA;
    typedef OperandTile<BKC, BN> TileB;
    __shared__ __attribute__((aligned(16))) float As[2][TileA::kFloats];
    __shared__ __attribute__((aligned(16))) float Bs[2][TileB::kFloats];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int l32 = lane & 31, half = lane >> 5;

    // linear workgroup id -> (batch, split, tile)
    const int tiles = a.tiles_m * a.tiles_n;
    int batch = 0, split = 0, lid, tail_piece = -1;
    int kchunk = a.kchunk;
    if (a.splits > 1) {
        // groups of 8 splits: the tiles of one split share its K range of both
        // operands, so give them ids that are equal mod 8 (same XCD)
        const int per_group = kNumXCD * tiles;
        const int grp = blockIdx.x / per_group, r = blockIdx.x - grp * per_group;
        const int in_grp = min(kNumXCD, a.splits - grp * kNumXCD);
        split = grp * kNumXCD + r % in_grp;
        lid = r / in_grp;
    } else if ((int)blockIdx.x < a.main_wgs) {
        // each XCD gets a contiguous range of (batch, tile) pairs: the tiles of one product, which
        // share its operands, meet in one L2 (remapped inside each batch, the three column tiles of
        // an AlexNet data-gradient image sat on three XCDs and its cotangent was fetched three times)
        const int per_batch = a.main_wgs / a.batch;        // == tiles unless there is a tail (batch 1)
        const int g = xcd_remap(blockIdx.x, a.main_wgs);
        batch = g / per_batch;
        lid = g - batch * per_batch;
    } else {
        tail_piece = blockIdx.x - a.main_wgs;
        lid = a.main_wgs + tail_piece / a.tail_splits;
        split = tail_piece % a.tail_splits;
        kchunk = a.tail_kchunk;
    }
    // tile order: groups of 8 tile rows, column-major inside a group, so tiles
    // that run together share A row panels and B column panels in L2
    constexpr int GM = 8;
    const int per_group = GM * a.tiles_n;
    const int group = lid / per_group, in_group = lid - group * per_group;
    const int first_m = group * GM;
    const int gsz = min(a.tiles_m - first_m, GM);
    const int tm = first_m + in_group % gsz, tn = in_group / gsz;
    const int m0 = tm * BM, n0 = tn * BN;

    int kbeg = split * kchunk;
    int kend = min(a.K, kbeg + kchunk);
    const float* A = a.A + batch * a.sA;
    const float* B = a.B + batch * a.sB;
    int gimg = 0;                   // GATHER 2: the image this workgroup's K range lies in
    if (CONV == 0 && a.kimg) {      // K cut per image: this split is one piece of one image
        const int img = split / a.kspi, piece = split - img * a.kspi;
        gimg = img;
        kbeg = img * a.kimg + piece * kchunk;
        kend = min((img + 1) * a.kimg, kbeg + kchunk);
        A += (long)img * a.aimg;
    }

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int nk = (kend - kbeg + KT - 1) / KT;
    TileA ta;
    TileB tb;

    // Software pipeline, per wavefront (K slice t lives in LDS buffer t&1):
    //   top of iteration t   : registers hold slice t+1 (loaded one iteration
    //                          ago) -> parked in the other LDS buffer; global
    //                          loads of slice t+2 issued; fragment set 1
    //                          (k group 1 of slice t) requested from LDS
    //   first half           : MFMAs on fragment set 0 (k group 0 of slice t,
    //                          requested during the previous iteration)
    //   barrier (LDS only)   : slice t+1 is visible; it sits in the middle of
    //                          the MFMA stream and does not wait for the global
    //                          loads in flight
    //   second half          : fragment set 0 of slice t+1 requested, MFMAs on
    //                          fragment set 1 (already in registers)
    // so LDS and HBM latencies sit under this wavefront's own MFMAs.  Reads of
    // a buffer are all issued before the barrier of the iteration that precedes
    // its next overwrite, and LDS serves requests in order, so two buffers do.
    float af[2][TM][4], bf[2][TN][4];
    auto read_frags = [&](int set, const float* as, const float* bs, int kk) {
#pragma unroll
        for (int i = 0; i < TM; ++i) TileA::frag(as, (wm * TM + i) * 32 + l32, kk, half, af[set][i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) TileB::frag(bs, (wn * TN + j) * 32 + l32, kk, half, bf[set][j]);
    };
    auto mfma_steps = [&](int set, int s0, int s1) {
#pragma unroll
        for (int s = s0; s < s1; ++s)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[set][i][s], bf[set][j][s],
                                                                     acc[i][j], 0, 0, 0);
    };
    // wait for this wavefront's LDS traffic only, then workgroup barrier
    // (the scheduling fences keep the compiler from moving MFMAs across it: the
    // barrier is meant to sit in the middle of the MFMA stream)
    auto lds_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };

    // Loading one K slice of both operands into registers.  MODE kFast: the
    // whole tile is inside both matrices and the K range is a multiple of the
    // slice -> fixed offsets from a uniform origin, no tests.  kMixed: each
    // operand on its own takes the untested loads where its side of the tile is
    // whole (an edge tile in N still streams A untested) and the tested ones
    // otherwise; a ragged last K slice is tested for both.
    constexpr int kFast = 0, kMixed = 1;
    const bool wholeA = CONV >= 2 || (m0 + BM <= a.M && !a.wide);
    const bool wholeB = GATHER == 0 && (CONV >= 2 || (n0 + BN <= a.N && !a.wide));     // gathered tiles go through registers
    const bool ragged_k = CONV <= 1 && (kend - kbeg) % KT != 0;
    const char* originA = reinterpret_cast<const char*>(A + (AKC ? (long)m0 * a.lda + kbeg : (long)kbeg * a.lda + m0));
    const char* originB = reinterpret_cast<const char*>(B + (BKC ? (long)n0 * a.ldb + kbeg : (long)kbeg * a.ldb + n0));
    const long stepA = (AKC ? (long)KT : (long)KT * a.lda) * 4, stepB = (BKC ? (long)KT : (long)KT * a.ldb) * 4;
    // Implicit convolution: where the slices of the image operand(s) start.  Slices are
    // issued in ascending order, one call of conv_next() each, so the walk is a handful
    // of scalar adds and compares per slice (everything here is wave-uniform).
    const char* cvA = nullptr;
    const char* cvB = nullptr;
    int cv_i = 0, cv_j = 0;        // mode 3: kernel row, kernel column; mode 2: slice within the image
    if constexpr (CONV == 3) {
        const int s0 = kbeg / KT, taps = a.cv_kh * a.cv_kw;
        const int cb = s0 / taps, tap = s0 - cb * taps;
        cv_i = tap / a.cv_kw;
        cv_j = tap - cv_i * a.cv_kw;
        const int img = tn / a.cv_tpi, t = tn - img * a.cv_tpi;
        cvB = reinterpret_cast<const char*>(B + (long)img * a.cv_imgB + (long)t * BN + (long)cv_i * a.cv_wp + cv_j +
                                            (long)cb * KT * a.cv_plane);
    } else if constexpr (CONV == 2) {
        const int s0 = kbeg / KT;
        const int img = s0 / a.cv_spi;
        cv_i = s0 - img * a.cv_spi;
        // the rows of B (channel and tap of each column of the result) are folded into its lane offsets
        cvA = reinterpret_cast<const char*>(A + (long)img * a.cv_imgA + (long)m0 * a.cv_plane + (long)cv_i * KT);
        cvB = reinterpret_cast<const char*>(B + (long)img * a.cv_imgB + (long)cv_i * KT);
    }
    // origins of the next slice to be issued, then step to the one after it
    auto conv_next = [&](const char*& oa, const char*& ob) {
        if constexpr (CONV == 3) {
            oa = originA;
            ob = cvB;
            originA += stepA;
            cvB += 4;
            if (++cv_j == a.cv_kw) {
                cv_j = 0;
                cvB += (long)(a.cv_wp - a.cv_kw) * 4;
                if (++cv_i == a.cv_kh) {
                    cv_i = 0;
                    cvB += ((long)KT * a.cv_plane - (long)a.cv_kh * a.cv_wp) * 4;
                }
            }
        } else if constexpr (CONV == 2) {
            oa = cvA;
            ob = cvB;
            cvA += KT * 4;
            cvB += KT * 4;
            if (++cv_i == a.cv_spi) {             // next image
                cv_i = 0;
                cvA += (a.cv_imgA - (long)a.cv_spi * KT) * 4;
                cvB += (a.cv_imgB - (long)a.cv_spi * KT) * 4;
            }
        }
    };
    auto load_slice = [&](auto mode, TileA& ra, TileB& rb, int slice) {
        constexpr int MODE = decltype(mode)::value;
        if (MODE == kFast) {
            ra.load_fast(originA + slice * stepA, ta.goff);
            rb.load_fast(originB + slice * stepB, tb.goff);
        } else {
            const int k0 = kbeg + slice * KT;
            const bool tested = ragged_k && slice == nk - 1;
            if (wholeA && !tested) ra.load_fast(originA + slice * stepA, ta.goff);
            else ra.load_checked(A, a.lda, m0, a.M, k0, kend);
            if (wholeB && !tested) rb.load_fast(originB + slice * stepB, tb.goff);
            else rb.load_checked(B, a.ldb, n0, a.N, k0, kend);
        }
    };

    // Patch gather: the B tile is filled from the image, through registers, with as much of the
    // address arithmetic as possible done once per tile.  Offsets are bytes from g_x (< 2^31: the
    // host checks), added to the uniform base by the load itself.  Where every element exists
    // (layers without padding, all but a ragged last slice) a slice costs a thread its 8
    // four-byte loads and at most one add per element; bounds tests otherwise.
    //   GATHER 1 (forward, BN = 128): a thread fills the two 16-byte pieces of the k-contiguous
    //     tile that the plain register path gives it (row = pixel, 4 consecutive k).  Fixed per
    //     tile: its rows' pixels -> byte offset of the patch corner.  Per slice: the patch
    //     offsets of its 4 k's, one 16-byte load from the table g_koff.  (Lanes as rows with the
    //     table in scalar registers needs no vector arithmetic at all and measured SLOWER, 0.301
    //     against 0.267 ms on AlexNet conv1: the scalar loads share the LDS wait counter.)
    //   GATHER 2 (weight gradient, BN = 128 or 64): wavefront w takes the K rows (pixels)
    //     4w..4w+3 of the slice, a lane BN / 64 adjacent columns (patch elements, fixed per tile);
    //     the four pixels are wave-uniform and walked KT positions per slice in scalar registers,
    //     so an element's address is scalar pointer + lane offset (0.295 -> 0.276 ms against one
    //     pixel walk per lane).
    constexpr int ZPL = BN / 64;                   // GATHER 2: columns per lane
    static_assert(GATHER != 1 || BN == 128, "forward gather: 128 pixels per tile");
    static_assert(GATHER != 2 || BN == 128 || BN == 64, "weight-gradient gather: 128 or 64 columns per tile");
    const char* gx = reinterpret_cast<const char*>(a.g_x);
    const int gwave = __builtin_amdgcn_readfirstlane(wave);
    unsigned g_lane[2] = {0u, 0u};                 // byte offsets: GATHER 1 the patch corners of the thread's two rows, GATHER 2 its columns
    int g_lh[2] = {0, 0}, g_lw[2] = {0, 0};        // padded layers: (h0, w0) of those corners / (ho, wo) of those columns
    int g_k4[2] = {0, 0};                          // GATHER 1: first k (inside a slice) of the thread's two pieces
    unsigned gp_base[4] = {0u, 0u, 0u, 0u};        // GATHER 2: byte offset of the four pixels' patch corners (uniform)
    int gp_ow[4] = {0, 0, 0, 0}, gp_h0[4] = {0, 0, 0, 0}, gp_w0[4] = {0, 0, 0, 0};
    if constexpr (GATHER == 1) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = threadIdx.x + i * kGemmThreads;
            const int row = idx >> 2;
            const int n = min(n0 + row, a.N - 1);            // rows past the end repeat the last pixel; they are never stored
            const int b = n / a.g_P, p = n - b * a.g_P;
            const int oh = p / a.g_OW, ow = p - oh * a.g_OW;
            g_lh[i] = oh * a.g_sh - a.g_ph;
            g_lw[i] = ow * a.g_sw - a.g_pw;
            g_lane[i] = (unsigned)(((b * a.g_C * a.g_H + g_lh[i]) * a.g_W + g_lw[i]) * 4);
            g_k4[i] = chunk_pos(row, idx & 3) * 4;
        }
    } else if constexpr (GATHER == 2) {
        const int KK = a.g_kh * a.g_kw;
#pragma unroll
        for (int q = 0; q < ZPL; ++q) {
            const int z = min(n0 + lane * ZPL + q, a.N - 1);         // columns past the end: never stored
            const int c = z / KK, r = z - c * KK;
            g_lh[q] = r / a.g_kw;
            g_lw[q] = r - g_lh[q] * a.g_kw;
            g_lane[q] = (unsigned)(((c * a.g_H + g_lh[q]) * a.g_W + g_lw[q]) * 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int p = min(kbeg + gwave * 4 + j, kend - 1) - gimg * a.g_P;     // in the first slice
            const int oh = p / a.g_OW;
            gp_ow[j] = p - oh * a.g_OW;
            gp_h0[j] = oh * a.g_sh - a.g_ph;
            gp_w0[j] = gp_ow[j] * a.g_sw - a.g_pw;
            gp_base[j] = (unsigned)(((gimg * a.g_C * a.g_H + gp_h0[j]) * a.g_W + gp_w0[j]) * 4);
        }
    }
    // One K slice of the gathered operand into tb's registers; called once per slice, in ascending
    // order (GATHER 2 advances its pixels).  Every load is issued, from a clamped address; what
    // does not exist is zeroed afterwards.  `last`: the slice may end past the K range.
    auto gather_b = [&](int k0, bool last) {
        // the two forms are whole straight-line blocks behind ONE uniform branch: with a branch per
        // element the compiler's wait-count pass drains the load queue before every load
        if constexpr (GATHER == 1) {
            int o[8], hw[8];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int4 off = *reinterpret_cast<const int4*>(a.g_koff + k0 + g_k4[i]);    // bytes; negative past the patch length
                o[i * 4] = off.x; o[i * 4 + 1] = off.y; o[i * 4 + 2] = off.z; o[i * 4 + 3] = off.w;
            }
            if (!GPAD && !last) {
#pragma unroll
                for (int e = 0; e < 8; ++e) tb.v[e] = *reinterpret_cast<const float*>(gx + (g_lane[e / 4] + (unsigned)o[e]));
            } else {
                if constexpr (GPAD) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        const int4 t = *reinterpret_cast<const int4*>(a.g_khw + k0 + g_k4[i]);
                        hw[i * 4] = t.x; hw[i * 4 + 1] = t.y; hw[i * 4 + 2] = t.z; hw[i * 4 + 3] = t.w;
                    }
                }
                bool ok[8];
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    ok[e] = o[e] >= 0;
                    if constexpr (GPAD)
                        ok[e] = ok[e] && (unsigned)(g_lh[e / 4] + (hw[e] >> 16)) < (unsigned)a.g_H &&
                                (unsigned)(g_lw[e / 4] + (hw[e] & 0xffff)) < (unsigned)a.g_W;
                    v[e] = *reinterpret_cast<const float*>(gx + (ok[e] ? g_lane[e / 4] + (unsigned)o[e] : 0u));
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) tb.v[e] = ok[e] ? v[e] : 0.0f;
            }
        } else if constexpr (GATHER == 2) {
            if (!GPAD && !last) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int q = 0; q < ZPL; ++q)
                        tb.v[j * ZPL + q] = *reinterpret_cast<const float*>(gx + gp_base[j] + g_lane[q]);
            } else {
                bool ok[4 * ZPL];
                float v[4 * ZPL];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int q = 0; q < ZPL; ++q) {
                        bool in = k0 + gwave * 4 + j < kend;
                        if constexpr (GPAD)
                            in = in && (unsigned)(gp_h0[j] + g_lh[q]) < (unsigned)a.g_H && (unsigned)(gp_w0[j] + g_lw[q]) < (unsigned)a.g_W;
                        ok[j * ZPL + q] = in;
                        v[j * ZPL + q] = *reinterpret_cast<const float*>(gx + (in ? gp_base[j] + g_lane[q] : 0u));
                    }
#pragma unroll
                for (int e = 0; e < 4 * ZPL; ++e) tb.v[e] = ok[e] ? v[e] : 0.0f;
            }
            // on to the pixels KT further (rows of the output wrap; a slice never leaves the image
            // except past kend, where nothing is read)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int ow = gp_ow[j] + KT, wraps = 0;
                while (ow >= a.g_OW) {
                    ow -= a.g_OW;
                    ++wraps;
                }
                const int dh = wraps * a.g_sh, dw = (ow - gp_ow[j]) * a.g_sw;
                gp_ow[j] = ow;
                gp_h0[j] += dh;
                gp_w0[j] += dw;
                gp_base[j] += (unsigned)((dh * a.g_W + dw) * 4);
            }
        }
    };
    // ... and from the registers into the LDS tile, in the layout the fragment reads expect
    auto gather_park = [&](float* bs) {
        if constexpr (GATHER == 1) {
            tb.store(bs);                                           // the plain register path's pieces
        } else if constexpr (GATHER == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float* dst = bs + (gwave * 4 + j) * TileB::LDM + lane * ZPL;
                if constexpr (ZPL == 2) *reinterpret_cast<float2*>(dst) = make_float2(tb.v[j * 2], tb.v[j * 2 + 1]);
                else *dst = tb.v[j];
            }
        }
    };

    // The pipelined schedule pays off when both operands are k-contiguous
    // (16-byte fragment reads); the other layouts measure faster with the
    // plain double-buffered loop (one full barrier per slice).  The pipelined
    // loop is unrolled by two so that the LDS buffer of a slice is a
    // compile-time constant (fragment and store addresses are then register +
    // immediate); the plain one is not: unrolled, it needs more than the 128
    // registers that let four workgroups share a CU.
    auto main_loop = [&](auto mode) {
        if constexpr (PIPE && decltype(mode)::value == kFast) {
            // whole tile, whole slices: slice kt+2 goes straight into the LDS buffer that
            // slice kt leaves behind, issued right after the barrier in the middle of
            // iteration kt (every wavefront has read its last fragments of slice kt by
            // then); it has to have landed by the barrier of iteration kt+1.
            const int wave_u = __builtin_amdgcn_readfirstlane(wave);
            if (nk > 0) {
                ta.load_direct(originA, ta.goff, As[0], wave_u);
                tb.load_direct(originB, tb.goff, Bs[0], wave_u);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                read_frags(0, As[0], Bs[0], 0);
                if (nk > 1) {
                    ta.load_direct(originA + stepA, ta.goff, As[1], wave_u);
                    tb.load_direct(originB + stepB, tb.goff, Bs[1], wave_u);
                }
            }
            auto iteration = [&](int kt, auto curc) {
                constexpr int cur = decltype(curc)::value;
                read_frags(1, As[cur], Bs[cur], 1);
                mfma_steps(0, 0, 4);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // slice kt+1 is in LDS
                lds_barrier();
                if (kt + 2 < nk) {
                    ta.load_direct(originA + (kt + 2) * stepA, ta.goff, As[cur], wave_u);
                    tb.load_direct(originB + (kt + 2) * stepB, tb.goff, Bs[cur], wave_u);
                }
                if (kt + 1 < nk) read_frags(0, As[cur ^ 1], Bs[cur ^ 1], 0);
                mfma_steps(1, 0, 4);
            };
            int kt = 0;
            for (; kt + 1 < nk; kt += 2) {
                iteration(kt, std::integral_constant<int, 0>{});
                iteration(kt + 1, std::integral_constant<int, 1>{});
            }
            if (kt < nk) iteration(kt, std::integral_constant<int, 0>{});
        } else {
            if constexpr (DEEP) {
                // Two register sets: the loads of slices kt+1 and kt+2 are in flight while
                // slice kt is multiplied.  Pays when the whole product is one round of
                // resident workgroups that start together and therefore load in bursts
                // (4096^3: +5 %); costs a longer prologue, so it is not used for short K.
                TileA ta1;
                TileB tb1;
                if (nk > 0) {
                    load_slice(mode, ta, tb, 0);
                    if (nk > 1) load_slice(mode, ta1, tb1, 1);
                    ta.store(As[0]);
                    tb.store(Bs[0]);
                    if (nk > 2) load_slice(mode, ta, tb, 2);
                }
                __syncthreads();
                // iteration kt: pa/pb hold slice kt+1, the other set slice kt+2
                auto iteration = [&](int kt, TileA& pa, TileB& pb) {
                    const int cur = kt & 1;
#pragma unroll
                    for (int kk = 0; kk < KT / 8; ++kk) {
                        read_frags(0, As[cur], Bs[cur], kk);
                        mfma_steps(0, 0, 4);
                    }
                    if (kt + 1 < nk) {
                        pa.store(As[cur ^ 1]);
                        pb.store(Bs[cur ^ 1]);
                    }
                    if (kt + 3 < nk) load_slice(mode, pa, pb, kt + 3);
                    __syncthreads();
                };
                int kt = 0;
                for (; kt + 1 < nk; kt += 2) {
                    iteration(kt, ta1, tb1);
                    iteration(kt + 1, ta, tb);
                }
                if (kt < nk) iteration(kt, ta1, tb1);
            } else if constexpr (decltype(mode)::value == kFast) {
                // Whole tile, whole slices: the global loads of slice kt+1 go straight into
                // the other LDS buffer while slice kt is multiplied -- no staging registers,
                // no LDS store instructions.  The buffer being filled was last read in
                // iteration kt-1, which every wavefront left through the barrier.
                const int wave_u = __builtin_amdgcn_readfirstlane(wave);
                if (nk > 0) {
                    if constexpr (CONV >= 2) {
                        const char *oa, *ob;
                        conv_next(oa, ob);
                        ta.load_direct(oa, ta.goff, As[0], wave_u);
                        tb.load_direct(ob, tb.goff, Bs[0], wave_u);
                    } else {
                        ta.load_direct(originA, ta.goff, As[0], wave_u);
                        tb.load_direct(originB, tb.goff, Bs[0], wave_u);
                    }
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                for (int kt = 0; kt < nk; ++kt) {
                    const int cur = kt & 1;
                    if (kt + 1 < nk) {
                        if constexpr (CONV >= 2) {
                            const char *oa, *ob;
                            conv_next(oa, ob);
                            ta.load_direct(oa, ta.goff, As[cur ^ 1], wave_u);
                            tb.load_direct(ob, tb.goff, Bs[cur ^ 1], wave_u);
                        } else {
                            ta.load_direct(originA + (kt + 1) * stepA, ta.goff, As[cur ^ 1], wave_u);
                            tb.load_direct(originB + (kt + 1) * stepB, tb.goff, Bs[cur ^ 1], wave_u);
                        }
                    }
#pragma unroll
                    for (int kk = 0; kk < KT / 8; ++kk) {
                        read_frags(0, As[cur], Bs[cur], kk);
                        mfma_steps(0, 0, 4);
                    }
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                }
            } else {
                // Edge tile and / or ragged K.  Each operand on its own still loads straight
                // into LDS wherever its side of the tile is whole and the slice is whole (an
                // edge tile in N streams A that way); the rest goes through registers with
                // bounds tests and is parked in LDS after the multiply.
                const int wave_u = __builtin_amdgcn_readfirstlane(wave);
                auto issue = [&](int slice, float* as, float* bs) {
                    const bool tested = ragged_k && slice == nk - 1;
                    const int k0 = kbeg + slice * KT;
                    if (wholeA && !tested) ta.load_direct(originA + slice * stepA, ta.goff, as, wave_u);
                    else ta.load_checked(A, a.lda, m0, a.M, k0, kend);
                    if constexpr (GATHER != 0) gather_b(k0, slice == nk - 1);
                    else if (wholeB && !tested) tb.load_direct(originB + slice * stepB, tb.goff, bs, wave_u);
                    else tb.load_checked(B, a.ldb, n0, a.N, k0, kend);
                };
                auto park = [&](int slice, float* as, float* bs) {
                    const bool tested = ragged_k && slice == nk - 1;
                    if (!wholeA || tested) ta.store(as);
                    if constexpr (GATHER != 0) gather_park(bs);
                    else if (!wholeB || tested) tb.store(bs);
                };
                if (nk > 0) {
                    issue(0, As[0], Bs[0]);
                    park(0, As[0], Bs[0]);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                for (int kt = 0; kt < nk; ++kt) {
                    const int cur = kt & 1;
                    const bool more = kt + 1 < nk;
                    if (more) issue(kt + 1, As[cur ^ 1], Bs[cur ^ 1]);
#pragma unroll
                    for (int kk = 0; kk < KT / 8; ++kk) {
                        read_frags(0, As[cur], Bs[cur], kk);
                        mfma_steps(0, 0, 4);
                    }
                    if (more) park(kt + 1, As[cur ^ 1], Bs[cur ^ 1]);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                }
            }
        }
    };
    if constexpr (CONV == 2) {
        ta.init_offsets(a.cv_plane, min(BM, a.M - m0));
        tb.init_offsets_taps(a.cv_plane, n0, a.N, a.cv_c, a.cv_kw, a.cv_wp);
    } else if constexpr (CONV == 3) {
        ta.init_offsets(a.lda, min(BM, a.M - m0));
        tb.init_offsets(a.cv_plane);
    } else {
        if (wholeA) ta.init_offsets(a.lda);
        if (wholeB) tb.init_offsets(a.ldb);
    }
    if constexpr (CONV >= 2) {
        main_loop(std::integral_constant<int, kFast>{});      // the host sends whole slices only; rows past the end are clamped
    } else if constexpr (GATHER != 0) {
        main_loop(std::integral_constant<int, kMixed>{});     // the gathered operand always goes through registers
    } else {
        if (wholeA && wholeB && !ragged_k) main_loop(std::integral_constant<int, kFast>{});
        else main_loop(std::integral_constant<int, kMixed>{});
    }

    // accumulator element e of a 32x32 block: row 8*(e/4) + 4*half + e%4, column l32.
    if (CONV == 3 && tail_piece < 0) {
        // Rows are output channels, columns pixels of the padded grid: the tile goes straight
        // into out[image][channel][h][w].  A lane's column is the same for every row, so its
        // offset inside a channel plane (and whether its pixel is a junk position) is worked
        // out once per 32-column block; row origins are wave-uniform as in the plain epilogue.
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const int wm_u = wave_u / WGN, wn_u = wave_u % WGN;
        const int img = tn / a.cv_tpi, t = tn - img * a.cv_tpi;
        const long HW = (long)a.cv_h * a.cv_w;
        const int r0 = m0 + wm_u * TM * 32;
        char* base = reinterpret_cast<char*>(a.C + ((long)img * a.M + r0) * HW);
        const long step1 = HW * 4, step5 = HW * 20;
        const int rows_left = a.M - r0 - 4 * half;           // of this lane: output channels left in the result
        auto store_tile = [&](auto wholec) {
            constexpr bool WHOLE = decltype(wholec)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int q = t * BN + (wn_u * TN + j) * 32 + l32;
                const int h = q / a.cv_wp, w = q - h * a.cv_wp;
                if (h < a.cv_h && w < a.cv_w) {
                    unsigned lane_off = (unsigned)((4 * half * HW + (long)h * a.cv_w + w) * 4);
                    char* row = base;
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            asm volatile("" : "+v"(lane_off));
                            const int r = i * 32 + 8 * (e / 4) + (e % 4);
                            if (WHOLE || r < rows_left) {
                                float v = acc[i][j][e];
                                if (a.cv_bias) v += a.cv_bias[r0 + r + 4 * half];
                                if (a.cv_mask)      // same element index as in the float array: byte offset / 4
                                    a.cv_mask[((row - reinterpret_cast<char*>(a.C)) + lane_off) >> 2] = v >= 0.0f ? 1 : 0;
                                if (a.cv_relu) v = v * (v >= 0.0f ? 1.0f : 0.0f);
                                *reinterpret_cast<float*>(row + lane_off) = v;
                            }
                            row += (e % 4 == 3) ? step5 : step1;
                        }
                }
            }
        };
        if (m0 + BM <= a.M) store_tile(std::true_type{});
        else store_tile(std::false_type{});
        return;
    }
    if (CONV == 1 && tail_piece < 0) {
        // Rows are output channels, columns (image, pixel) pairs: the tile goes straight into
        // out[image][channel][pixel].  A tile of columns may straddle images, so the image is
        // part of the lane's offset (relative to the image of the tile's first column).
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const int wm_u = wave_u / WGN, wn_u = wave_u % WGN;
        const int HW = (int)a.cv_plane;
        const int img0 = n0 / HW;
        const int r0 = m0 + wm_u * TM * 32;
        char* base = reinterpret_cast<char*>(a.C + ((long)img0 * a.M + r0) * HW);
        const long step1 = (long)HW * 4, step5 = (long)HW * 20;
        const int rows_left = a.M - r0 - 4 * half;
        auto store_tile = [&](auto wholec) {
            constexpr bool WHOLE = decltype(wholec)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = n0 + (wn_u * TN + j) * 32 + l32;
                if (n < a.N) {
                    const int img = n / HW, p = n - img * HW;
                    unsigned lane_off = (unsigned)(((long)(img - img0) * a.M * HW + 4 * half * (long)HW + p) * 4);
                    char* row = base;
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            asm volatile("" : "+v"(lane_off));
                            const int r = i * 32 + 8 * (e / 4) + (e % 4);
                            if (WHOLE || r < rows_left) {
                                float v = acc[i][j][e];
                                if (a.cv_bias) v += a.cv_bias[r0 + r + 4 * half];
                                if (a.cv_mask)      // same element index as in the float array: byte offset / 4
                                    a.cv_mask[((row - reinterpret_cast<char*>(a.C)) + lane_off) >> 2] = v >= 0.0f ? 1 : 0;
                                if (a.cv_relu) v = v * (v >= 0.0f ? 1.0f : 0.0f);
                                *reinterpret_cast<float*>(row + lane_off) = v;
                            }
                            row += (e % 4 == 3) ? step5 : step1;
                        }
                }
            }
        };
        if (m0 + BM <= a.M) store_tile(std::true_type{});
        else store_tile(std::false_type{});
        return;
    }
    // Destination: C, this split's partial matrix, or (tail pieces) a tile-local
    // [BM][BN] block that is written whole -- the reduction clips.
    float* out;
    long ldo;
    int out_m0 = m0, out_n0 = n0, out_M = a.M, out_N = a.N;
    if (tail_piece >= 0) {
        out = a.ws + (long)tail_piece * (BM * BN);
        ldo = BN;
        out_m0 = 0; out_n0 = 0; out_M = BM; out_N = BN;
    } else if (a.splits > 1) {
        out = a.ws + (long)split * a.M * a.N;
        ldo = a.N;
    } else {
        out = a.C + batch * a.sC;
        ldo = a.ldc;
    }
    // A wavefront that is storing shares its SIMD with wavefronts that are
    // multiplying and gets about one instruction issued per MFMA of theirs, so the
    // store sequence carries no vector address arithmetic: row origins are
    // wave-uniform (scalar adds), the lane's share (its column, its half's 4-row
    // shift) is one fixed 32-bit offset, the block column an immediate.  Edge
    // tiles mask lanes by comparing the compile-time row / column of a store with
    // the lane's count of rows / columns left in C.
    {
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const int wm_u = wave_u / WGN, wn_u = wave_u % WGN;
        const int r0 = out_m0 + wm_u * TM * 32, c0 = out_n0 + wn_u * TN * 32;
        char* row = reinterpret_cast<char*>(out + (long)r0 * ldo + c0);
        unsigned lane_off = (unsigned)((4 * half * ldo + l32) * 4);
        // rows of a lane half: 0,1,2,3, 8,9,10,11, 16,... -> steps of one row, then five
        const long step1 = ldo * 4, step5 = ldo * 20;
        const bool whole = out_m0 + BM <= out_M && out_n0 + BN <= out_N;
        const int rows_left = out_M - r0 - 4 * half, cols_left = out_N - c0 - l32;   // of this lane
        auto store_rows = [&](auto wholec) {
            constexpr bool WHOLE = decltype(wholec)::value;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    // keeps "uniform row origin + lane offset" from being re-associated into
                    // a per-lane 64-bit pointer that is then advanced with vector adds
                    asm volatile("" : "+v"(lane_off));
                    const int r = i * 32 + 8 * (e / 4) + (e % 4);
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        if (WHOLE || (r < rows_left && j * 32 < cols_left))
                            *reinterpret_cast<float*>(row + lane_off + j * 128) = acc[i][j][e];
                    row += (e % 4 == 3) ? step5 : step1;
                }
        };
        if (whole) store_rows(std::true_type{});
        else store_rows(std::false_type{});
    }
}

// Tail tiles: C tile = sum over its K pieces, in order.  blockIdx.y = tail tile,
// one thread per 4 consecutive tile elements; all pieces are loaded before the
// adds so the loads overlap.
constexpr int kMaxTailSplits = 16;
__global__ __launch_bounds__(256) void tail_reduce_kernel(const float* __restrict__ ws,
                                                          float* __restrict__ C, GemmArgs a, int bm,
                                                          int bn) {
    const int lid = a.main_wgs + blockIdx.y;
    // same tile order as sgemm_kernel
    constexpr int GM = 8;
    const int per_group = GM * a.tiles_n;
    const int group = lid / per_group, in_group = lid - group * per_group;
    const int first_m = group * GM;
    const int gsz = min(a.tiles_m - first_m, GM);
    const int tm = first_m + in_group % gsz, tn = in_group / gsz;
    const int m0 = tm * bm, n0 = tn * bn;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;      // bn % 4 == 0: the 4 elements share a row
    if (i >= bm * bn) return;
    const float* src = ws + (long)blockIdx.y * a.tail_splits * (bm * bn) + i;
    float4 v[kMaxTailSplits];
#pragma unroll
    for (int k = 0; k < kMaxTailSplits; ++k)
        if (k < a.tail_splits) v[k] = *reinterpret_cast<const float4*>(src + (long)k * (bm * bn));
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < kMaxTailSplits; ++k)
        if (k < a.tail_splits) {
            s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w;
        }
    const int r = i / bn, c = i - r * bn;
    if (m0 + r >= a.M) return;
    float* dst = C + (long)(m0 + r) * a.ldc + n0 + c;
    const float o[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (n0 + c + j < a.N) dst[j] = o[j];
}

// The same for a convolution product that writes NCHW itself (modes 1 and 3): tile rows are
// output channels, tile columns pixels (mode 3: of the padded grid, junk pixels dropped; mode
// 1: (image, pixel) pairs); the sums go to out[image][channel][pixel] with the optional bias
// and rectify of the in-place epilogue.
__global__ __launch_bounds__(256) void tail_reduce_conv_kernel(const float* __restrict__ ws, GemmArgs a, int bm, int bn) {
    const int lid = a.main_wgs + blockIdx.y;
    constexpr int GM = 8;
    const int per_group = GM * a.tiles_n;
    const int group = lid / per_group, in_group = lid - group * per_group;
    const int first_m = group * GM;
    const int gsz = min(a.tiles_m - first_m, GM);
    const int tm = first_m + in_group % gsz, tn = in_group / gsz;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= bm * bn) return;
    const float* src = ws + (long)blockIdx.y * a.tail_splits * (bm * bn) + i;
    float4 v[kMaxTailSplits];
#pragma unroll
    for (int k = 0; k < kMaxTailSplits; ++k)
        if (k < a.tail_splits) v[k] = *reinterpret_cast<const float4*>(src + (long)k * (bm * bn));
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < kMaxTailSplits; ++k)
        if (k < a.tail_splits) {
            s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w;
        }
    const int r = i / bn, c = i - r * bn;
    const int row = tm * bm + r;                         // output channel
    if (row >= a.M) return;
    const float bias = a.cv_bias ? a.cv_bias[row] : 0.0f;
    const float o[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        long at = -1;                                     // where column c + j of the tile goes, if anywhere
        if (a.conv == 3) {
            const int img = tn / a.cv_tpi, t = tn - img * a.cv_tpi;
            const int q = t * bn + c + j;
            const int h = q / a.cv_wp, w = q - h * a.cv_wp;
            if (h < a.cv_h && w < a.cv_w) at = ((long)img * a.M + row) * ((long)a.cv_h * a.cv_w) + (long)h * a.cv_w + w;
        } else {
            const int n = tn * bn + c + j;
            const int HW = (int)a.cv_plane;
            const int img = n / HW;
            if (n < a.N) at = ((long)img * a.M + row) * HW + (n - img * HW);
        }
        if (at >= 0) {
            float x = o[j];
            if (a.cv_bias) x += bias;
            if (a.cv_mask) a.cv_mask[at] = x >= 0.0f ? 1 : 0;
            if (a.cv_relu) x = x * (x >= 0.0f ? 1.0f : 0.0f);
            a.C[at] = x;
        }
    }
}

// C[r][c] = sum over splits of ws[s][r][c].  A workgroup takes 64 columns of
// the flattened [M*N] index (64 x 16 bytes when VEC) and cuts the splits into 4
// contiguous ranges, one per wavefront; each lane adds its range in ascending
// order with 8 loads in flight, then the four range sums are added in ascending
// order.  The order is fixed, so the result is deterministic; with hundreds of
// splits and a small C (the MNIST / CIFAR weight gradients) a single running
// sum per output would be one long chain of load latencies.
constexpr int kReduceGroups = 4;

// A weight gradient computed with its columns ordered (tap, channel) and stored as the filters are,
// [row][channel][tap]: flat index row * n + tap * (n / taps) + channel -> (row * (n / taps) + channel) * taps + tap.
__device__ __forceinline__ long filter_layout_index(long i, int n, int taps) {
    const long r = i / n;
    const int c = (int)(i - r * n), channels = n / taps;
    const int tap = c / channels, ch = c - tap * channels;
    return (r * channels + ch) * taps + tap;
}

// taps > 0: the sums are stored through filter_layout_index (C dense, ldc == N).
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws,
                                                            float* __restrict__ C, long MN, int N,
                                                            long ldc, int splits, int taps = 0) {
    typedef typename std::conditional<VEC, float4, float>::type T;
    constexpr int W = VEC ? 4 : 1;
    __shared__ T part[kReduceGroups][64];
    const int col = threadIdx.x & 63, g = threadIdx.x >> 6;
    const long i = ((long)blockIdx.x * 64 + col) * W;          // first flattened output index of this lane
    const int per = (splits + kReduceGroups - 1) / kReduceGroups;
    const int s0 = g * per, s1 = min(splits, s0 + per);
    T acc;
    if constexpr (VEC) acc = make_float4(0.f, 0.f, 0.f, 0.f);
    else acc = 0.0f;
    if (i < MN) {
        for (int sb = s0; sb < s1; sb += 8) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (sb + u < s1) v[u] = *reinterpret_cast<const T*>(ws + (long)(sb + u) * MN + i);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (sb + u < s1) {
                    if constexpr (VEC) {
                        acc.x += v[u].x; acc.y += v[u].y; acc.z += v[u].z; acc.w += v[u].w;
                    } else {
                        acc += v[u];
                    }
                }
        }
    }
    part[g][col] = acc;
    __syncthreads();
    if (g != 0 || i >= MN) return;
    T tot = part[0][col];
#pragma unroll
    for (int k = 1; k < kReduceGroups; ++k) {
        const T p = part[k][col];
        if constexpr (VEC) {
            tot.x += p.x; tot.y += p.y; tot.z += p.z; tot.w += p.w;
        } else {
            tot += p;
        }
    }
    if (taps > 0) {
        if constexpr (VEC) {
            C[filter_layout_index(i, N, taps)] = tot.x;
            C[filter_layout_index(i + 1, N, taps)] = tot.y;
            C[filter_layout_index(i + 2, N, taps)] = tot.z;
            C[filter_layout_index(i + 3, N, taps)] = tot.w;
        } else {
            C[filter_layout_index(i, N, taps)] = tot;
        }
        return;
    }
    if constexpr (VEC) {
        // N % 4 == 0: the four outputs share a row of C
        const long r = i / N, c = i - r * N;
        *reinterpret_cast<float4*>(C + r * ldc + c) = tot;
    } else {
        const long r = i / N, c = i - r * N;
        C[r * ldc + c] = tot;
    }
}

// Many partial results of a small array (hundreds of [32][75] blocks): the kernel above would put
// all of it on a dozen workgroups whose four wavefronts each walk a quarter of the partials, one
// long chain of load latencies (13 us for 512 x 2400 floats).  Here a workgroup of 16 wavefronts
// owns 64 outputs; wavefront g adds partials [g * per, (g + 1) * per) in order, 8 loads in flight,
// and the 16 sums are added in order: the same fixed order on every run.
__global__ __launch_bounds__(1024) void reduce_many_kernel(const float* __restrict__ ws, float* __restrict__ out,
                                                           long count, int n, int row_len = 0, int taps = 0) {
    __shared__ float part[16][64];
    const int col = threadIdx.x & 63, g = threadIdx.x >> 6;
    const long i = (long)blockIdx.x * 64 + col;
    const int per = (n + 15) / 16;
    const int s0 = g * per, s1 = min(n, s0 + per);
    float acc = 0.0f;
    if (i < count) {
        for (int sb = s0; sb < s1; sb += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = ws[(long)min(sb + u, s1 - 1) * count + i];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (sb + u < s1) acc += v[u];
        }
    }
    part[g][col] = acc;
    __syncthreads();
    if (g != 0 || i >= count) return;
    float tot = part[0][col];
#pragma unroll
    for (int k = 1; k < 16; ++k) tot += part[k][col];
    out[taps > 0 ? filter_layout_index(i, row_len, taps) : i] = tot;
}

// out[i] = ws[0][i] + ws[1][i] + ... + ws[n - 1][i] for i < count, added in a fixed order (groups of
// consecutive partials, then the group sums): the weight gradient of a very large batch sums
// per-group results with it, the reduction-shaped weight gradient its workgroups' results.
int reduce_partials(const float* ws, float* out, long count, int n, void* stream, int row_len, int taps) {
    if (n >= 64 && count <= (1L << 16)) {
        reduce_many_kernel<<<dim3((unsigned)cdiv(count, 64L)), dim3(1024), 0, as_stream(stream)>>>(ws, out, count, n, row_len, taps);
        CGT_LAUNCH_CHECK("reduce_many_kernel");
        return CGT_AMD_OK;
    }
    if (taps > 0) {         // rows of row_len floats, stored in the filters' layout
        const bool vec4 = row_len % 4 == 0 && reinterpret_cast<uintptr_t>(ws) % 16 == 0;
        const long nblocks = cdiv(count, vec4 ? 256L : 64L);
        CGT_ARG_CHECK(nblocks < (1L << 31), "reduce_partials: too many elements");
        if (vec4) splitk_reduce_kernel<true><<<dim3((unsigned)nblocks), dim3(256), 0, as_stream(stream)>>>(ws, out, count, row_len, row_len, n, taps);
        else splitk_reduce_kernel<false><<<dim3((unsigned)nblocks), dim3(256), 0, as_stream(stream)>>>(ws, out, count, row_len, row_len, n, taps);
        CGT_LAUNCH_CHECK("splitk_reduce_kernel");
        return CGT_AMD_OK;
    }
    const bool vec = count % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(ws) % 16 == 0;
    const long blocks = cdiv(count, vec ? 256L : 64L);
    CGT_ARG_CHECK(blocks < (1L << 31), "reduce_partials: too many elements");
    hipStream_t st = as_stream(stream);
    // the kernel addresses its output as rows of N floats ldc apart: rows of 1024 back to back are the flat array
    if (vec) splitk_reduce_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(ws, out, count, 1024, 1024, n);
    else splitk_reduce_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(ws, out, count, 1024, 1024, n);
    CGT_LAUNCH_CHECK("splitk_reduce_kernel");
    return CGT_AMD_OK;
}

// Split-K / tail workspaces: one per stream, owned by the library (see common.h).
static float* get_workspace(void* stream, size_t bytes) {
    return stream_workspace(stream, kWsGemm, bytes, "sgemm");
}

// Scratch of the entry point that allocates nothing (cgt_amd_sgemm_noalloc): the
// split-K partials / tail pieces live in this file-scope device array instead of a
// hipMalloc'ed workspace.  Every GPU the library runs on holds its own copy at its own
// address until the process ends.  In host code `scratch` is only a handle for
// hipGetSymbolAddress -- the device address is looked up once per device, with that
// device current, and kept in g_scratch_ptr; kernels, like the workspace kernels above,
// take that pointer as an argument.
constexpr size_t kScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) float scratch[kScratchBytes / sizeof(float)];
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (nullptr + message on failure).
static float* scratch_address() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        set_error("sgemm_noalloc: cannot identify the current device");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            set_error("sgemm_noalloc: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                      hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    return g_scratch_ptr[dev];
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

struct TileShape {
    int bm, bn;
};

// Tile shapes on offer; the 128x128 default comes first and wins ties.
static const TileShape kShapes[] = {{128, 128}, {128, 96}, {128, 64}, {128, 32}, {96, 128}, {64, 128}, {32, 128}};
constexpr int kPlainShapes = 6;      // the last shape exists for the products that write NCHW themselves (32 or fewer filters)

template <bool AKC, bool BKC, bool PIPE>
static void launch_shape(int shape, dim3 grid, hipStream_t st, const GemmArgs& a) {
    dim3 block(kGemmThreads);
    switch (shape) {
        case 0: sgemm_kernel<AKC, BKC, PIPE, 2, 2, 2, 2><<<grid, block, 0, st>>>(a); break;
        case 1: sgemm_kernel<AKC, BKC, PIPE, 4, 1, 1, 3><<<grid, block, 0, st>>>(a); break;
        case 2: sgemm_kernel<AKC, BKC, PIPE, 4, 1, 1, 2><<<grid, block, 0, st>>>(a); break;
        case 3: sgemm_kernel<AKC, BKC, PIPE, 4, 1, 1, 1><<<grid, block, 0, st>>>(a); break;
        case 4: sgemm_kernel<AKC, BKC, PIPE, 1, 4, 3, 1><<<grid, block, 0, st>>>(a); break;
        default: sgemm_kernel<AKC, BKC, PIPE, 1, 4, 2, 1><<<grid, block, 0, st>>>(a); break;
    }
}

// implicit-convolution variants
static void launch_conv(int mode, int shape, dim3 grid, hipStream_t st, const GemmArgs& a) {
    dim3 block(kGemmThreads);
    if (mode == 1) {
        switch (shape) {
            case 0: sgemm_kernel<true, true, false, 2, 2, 2, 2, false, 1><<<grid, block, 0, st>>>(a); break;
            case 4: sgemm_kernel<true, true, false, 1, 4, 3, 1, false, 1><<<grid, block, 0, st>>>(a); break;
            case 5: sgemm_kernel<true, true, false, 1, 4, 2, 1, false, 1><<<grid, block, 0, st>>>(a); break;
            default: sgemm_kernel<true, true, false, 1, 4, 1, 1, false, 1><<<grid, block, 0, st>>>(a); break;    // 32 x 128
        }
    } else if (mode == 3) {
        switch (shape) {
            case 0: sgemm_kernel<true, false, false, 2, 2, 2, 2, false, 3><<<grid, block, 0, st>>>(a); break;
            case 4: sgemm_kernel<true, false, false, 1, 4, 3, 1, false, 3><<<grid, block, 0, st>>>(a); break;    // 96 x 128
            case 5: sgemm_kernel<true, false, false, 1, 4, 2, 1, false, 3><<<grid, block, 0, st>>>(a); break;    // 64 x 128
            default: sgemm_kernel<true, false, false, 1, 4, 1, 1, false, 3><<<grid, block, 0, st>>>(a); break;   // 32 x 128
        }
    } else {
        switch (shape) {
            case 0: sgemm_kernel<true, true, false, 2, 2, 2, 2, false, 2><<<grid, block, 0, st>>>(a); break;
            case 1: sgemm_kernel<true, true, false, 4, 1, 1, 3, false, 2><<<grid, block, 0, st>>>(a); break;
            case 2: sgemm_kernel<true, true, false, 4, 1, 1, 2, false, 2><<<grid, block, 0, st>>>(a); break;
            case 3: sgemm_kernel<true, true, false, 4, 1, 1, 1, false, 2><<<grid, block, 0, st>>>(a); break;
            case 4: sgemm_kernel<true, true, false, 1, 4, 3, 1, false, 2><<<grid, block, 0, st>>>(a); break;
            default: sgemm_kernel<true, true, false, 1, 4, 2, 1, false, 2><<<grid, block, 0, st>>>(a); break;
        }
    }
}

// patch-gather variants: forward (NT, NCHW epilogue, shapes with 128 columns) and weight gradient (NN)
template <bool GPAD>
static void launch_gather(int which, int shape, dim3 grid, hipStream_t st, const GemmArgs& a) {
    dim3 block(kGemmThreads);
    if (which == 1) {
        switch (shape) {
            case 0: sgemm_kernel<true, true, false, 2, 2, 2, 2, false, 1, 1, GPAD><<<grid, block, 0, st>>>(a); break;
            case 4: sgemm_kernel<true, true, false, 1, 4, 3, 1, false, 1, 1, GPAD><<<grid, block, 0, st>>>(a); break;
            case 5: sgemm_kernel<true, true, false, 1, 4, 2, 1, false, 1, 1, GPAD><<<grid, block, 0, st>>>(a); break;
            default: sgemm_kernel<true, true, false, 1, 4, 1, 1, false, 1, 1, GPAD><<<grid, block, 0, st>>>(a); break;
        }
    } else {
        switch (shape) {
            case 0: sgemm_kernel<true, false, false, 2, 2, 2, 2, false, 0, 2, GPAD><<<grid, block, 0, st>>>(a); break;
            case 2: sgemm_kernel<true, false, false, 4, 1, 1, 2, false, 0, 2, GPAD><<<grid, block, 0, st>>>(a); break;    // 128 x 64
            case 4: sgemm_kernel<true, false, false, 1, 4, 3, 1, false, 0, 2, GPAD><<<grid, block, 0, st>>>(a); break;    // 96 x 128
            case 6: sgemm_kernel<true, false, false, 1, 4, 1, 1, false, 0, 2, GPAD><<<grid, block, 0, st>>>(a); break;    // 32 x 128
            default: sgemm_kernel<true, false, false, 1, 4, 2, 1, false, 0, 2, GPAD><<<grid, block, 0, st>>>(a); break;   // 64 x 128
        }
    }
}

// g_koff / g_khw of the forward gather: one entry per patch element, padded to whole K slices
__global__ void patch_table_kernel(int* __restrict__ koff, int* __restrict__ khw, int K, int Kpad, int kh, int kw, int H, int W) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= Kpad) return;
    const int KK = kh * kw;
    const int c = k / KK, r = k - c * KK;
    const int ho = r / kw, wo = r - ho * kw;
    koff[k] = k < K ? ((c * H + ho) * W + wo) * 4 : -1;      // bytes
    khw[k] = (ho << 16) | wo;
}

// tile shape (index into kShapes) of an implicit-convolution product, -1 if none fits: the
// shape with the least padded work; rows past the end of the result (filters that do not
// fill the last tile) are computed from repeated operand rows and never stored.
//   mode 3: `rows` output channels x 128 pixels per tile; the K slices need whole blocks of 16 channels;
//   mode 2: `rows` filters x `cols` = taps * channels.
static int conv_shape(int mode, long rows, long cols, long channels) {
    if ((mode != 1 && channels % KT != 0) || rows < 1) return -1;
    int best = -1;
    double best_work = 0;
    for (int i = 0; i < (mode != 2 ? kPlainShapes + 1 : kPlainShapes); ++i) {
        if (mode != 2 && kShapes[i].bn != 128) continue;
        const double work = (double)(cdiv(rows, kShapes[i].bm) * kShapes[i].bm) *
                            (mode != 2 ? 1.0 : (double)(cdiv(cols, kShapes[i].bn) * kShapes[i].bn));
        if (best < 0 || work < best_work * 0.97) {
            best = i;
            best_work = work;
        }
    }
    return best;
}

bool sgemm_conv_supported(int mode, long filters, long channels) {
    return filters >= 1 && channels >= KT && channels % KT == 0 && mode >= 2 && mode <= 3;
}

static void launch_trans(int tA, int tB, bool pipe, bool deep, int shape, dim3 grid, hipStream_t st, const GemmArgs& a) {
    dim3 block(kGemmThreads);
    if (deep) {     // 128x128 tiles, plain loop, not NT (there the second register set spills)
        if (!tA && !tB) sgemm_kernel<true, false, false, 2, 2, 2, 2, true><<<grid, block, 0, st>>>(a);
        else if (tA && !tB) sgemm_kernel<false, false, false, 2, 2, 2, 2, true><<<grid, block, 0, st>>>(a);
        else sgemm_kernel<false, true, false, 2, 2, 2, 2, true><<<grid, block, 0, st>>>(a);
        return;
    }
    if (!tA && !tB) launch_shape<true, false, false>(shape, grid, st, a);
    else if (!tA && tB) {
        if (pipe) launch_shape<true, true, true>(shape, grid, st, a);
        else launch_shape<true, true, false>(shape, grid, st, a);
    } else if (tA && !tB) launch_shape<false, false, false>(shape, grid, st, a);
    else launch_shape<false, true, false>(shape, grid, st, a);
}

static int gemm_dispatch(int tA, int tB, long P, long M, long N, long K, const float* A, long lda,
                         long sA, const float* B, long ldb, long sB, float* C, long ldc, long sC,
                         void* stream, bool static_scratch = false, const ConvGemm* cv = nullptr) {
    CGT_ARG_CHECK(P >= 0 && M >= 0 && N >= 0 && K >= 0, "sgemm: negative size");
    if (P == 0 || M == 0 || N == 0) return CGT_AMD_OK;
    CGT_ARG_CHECK(A || K == 0, "sgemm: null A");
    CGT_ARG_CHECK(B || K == 0, "sgemm: null B");
    CGT_ARG_CHECK(C, "sgemm: null C");
    CGT_ARG_CHECK(M < (1L << 31) - 128 && N < (1L << 31) - 128 && K < (1L << 31) - KT && P < 65536,
                  "sgemm: size too large");
    CGT_ARG_CHECK(ldc < (1L << 27) || M <= 4, "sgemm: ldc >= 2^27 with more than 4 rows is not supported");
    CGT_ARG_CHECK(cv || (lda >= (tA ? M : K) && ldb >= (tB ? K : N) && ldc >= N),
                  "sgemm: leading dimension too small (lda=%ld ldb=%ld ldc=%ld)", lda, ldb, ldc);
    // tile shape: least padded work, ties to the earlier (larger) shape
    int shape = 0;
    double best = 0;
    const bool gather_cols = cv && cv->mode == 4 && cv->patch;     // the gathered weight gradient: tiles of 128 or 64 columns
    for (int i = 0; i < kPlainShapes + (gather_cols ? 1 : 0); ++i) {        // 32 x 128: the gathered weight gradient of 32 or fewer filters
        if (gather_cols && kShapes[i].bn != 128 && kShapes[i].bn != 64) continue;
        const double work = (double)(cdiv(M, kShapes[i].bm) * kShapes[i].bm) *
                            (double)(cdiv(N, kShapes[i].bn) * kShapes[i].bn);
        if (i == 0 || work < best * 0.97) {
            best = work;
            shape = i;
        }
    }
    // where the partial products of a split go: the stream's workspace (grown on demand),
    // or the static device array when the caller must not allocate
    int ws_rc = CGT_AMD_ERR_NOMEM;
    auto workspace = [&](size_t bytes) -> float* {
        if (!static_scratch) return get_workspace(stream, bytes);
        if (bytes > kScratchBytes) {
            set_error("sgemm_noalloc: this product needs %zu bytes of split-K scratch, the static buffer holds %zu "
                      "(use cgt_amd_sgemm, which allocates a workspace)", bytes, kScratchBytes);
            ws_rc = CGT_AMD_ERR_ARG;
            return nullptr;
        }
        float* p = scratch_address();
        if (!p) ws_rc = CGT_AMD_ERR_HIP;
        return p;
    };
    const bool per_image_k = cv && cv->mode == 4;     // plain kernel, K cut per image
    const bool conv_kernel = cv && !per_image_k;
    const bool writes_nchw = cv && (cv->mode == 1 || cv->mode == 3);
    if (conv_kernel) {
        shape = conv_shape(cv->mode, M, N, cv->C);
        CGT_ARG_CHECK(cv->mode != 3 || (long)cv->tpi * cv->B * 128 == N, "sgemm_conv: mode 3 takes whole tiles of pixels");
        CGT_ARG_CHECK(shape >= 0, "sgemm_conv: the image must have a multiple of 16 channels");
        // lane offsets are 32-bit: a tile's rows (mode 2: the channels of a whole image) span less than 4 GB
        CGT_ARG_CHECK(cv->mode == 1 || (cv->plane < (1L << 23) && (cv->mode != 2 || cv->C * cv->plane < (1L << 30))),
                      "sgemm_conv: padded planes too large");
        // mode 1: a lane's offset spans the images a tile of 128 columns touches
        CGT_ARG_CHECK(cv->mode != 1 || (cv->plane >= 1 && cv->plane < (1L << 31) && cv->B * cv->plane == N &&
                                        (127 / cv->plane + 2) * M * cv->plane < (1L << 30)),
                      "sgemm_conv: column-buffer product too large");
    }
    GemmArgs a;
    a.conv = conv_kernel ? cv->mode : 0;
    a.kimg = 0; a.kspi = 1; a.aimg = 0;
    const PatchGeom* pg = cv ? cv->patch : nullptr;       // B operand gathered from the image
    bool gpad = false;
    if (pg) {
        CGT_ARG_CHECK(cv->mode == 1 || cv->mode == 4, "sgemm_conv: patch gather goes with the column-buffer products");
        const long P = (long)pg->OH * pg->OW, Z = (long)pg->C * pg->kh * pg->kw;
        CGT_ARG_CHECK(pg->x && P == cv->plane && Z == (cv->mode == 1 ? K : N) && P < (1L << 21) &&
                      cv->B * pg->C * pg->H * pg->W < (1L << 29) && pg->H < 32768 && pg->W < 32768 &&
                      pg->kh < 32768 && pg->kw < 32768 && pg->ph < 32768 && pg->pw < 32768,
                      "sgemm_conv: image too large for the patch gather");
        // every patch lies inside the image: no bounds tests
        gpad = !(pg->ph == 0 && pg->pw == 0 && (pg->OH - 1) * pg->sh + pg->kh <= pg->H && (pg->OW - 1) * pg->sw + pg->kw <= pg->W);
        a.g_x = pg->x;
        a.g_koff = a.g_khw = nullptr;
        a.g_C = pg->C; a.g_H = pg->H; a.g_W = pg->W; a.g_kh = pg->kh; a.g_kw = pg->kw; a.g_ph = pg->ph; a.g_pw = pg->pw;
        a.g_sh = pg->sh; a.g_sw = pg->sw; a.g_OW = pg->OW; a.g_P = (int)P;
        if (cv->mode == 1) {
            const long Kpad = cdiv(K, KT) * KT;
            int* tab = reinterpret_cast<int*>(stream_workspace(stream, kWsConvTable, (size_t)Kpad * 2 * sizeof(int), "sgemm_conv"));
            if (!tab) return CGT_AMD_ERR_NOMEM;
            patch_table_kernel<<<dim3((unsigned)cdiv(Kpad, 256L)), dim3(256), 0, as_stream(stream)>>>(
                tab, tab + Kpad, (int)K, (int)Kpad, pg->kh, pg->kw, pg->H, pg->W);
            CGT_LAUNCH_CHECK("patch_table_kernel");
            a.g_koff = tab;
            a.g_khw = tab + Kpad;
        }
    }
    if (cv) {
        a.cv_wp = cv->wp; a.cv_kw = cv->kw; a.cv_kh = cv->kh; a.cv_c = (int)cv->C;
        a.cv_tpi = (int)cv->tpi; a.cv_spi = (int)cv->spi;
        a.cv_plane = cv->plane;
        // mode 2: A is the (shifted) padded cotangent with M planes per image; B is the image in both modes
        a.cv_imgA = M * cv->plane;
        a.cv_imgB = cv->C * cv->plane;
        a.cv_h = (int)cv->H; a.cv_w = (int)cv->W; a.cv_relu = cv->relu; a.cv_bias = cv->bias; a.cv_mask = cv->mask;
    }
    a.A = A; a.B = B; a.C = C;
    a.lda = lda; a.ldb = ldb; a.ldc = ldc;
    a.sA = sA; a.sB = sB; a.sC = sC;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.tiles_m = (int)cdiv(M, kShapes[shape].bm);
    a.tiles_n = (int)cdiv(N, kShapes[shape].bn);
    a.batch = (int)P;
    const long tiles = (long)a.tiles_m * a.tiles_n;
    a.splits = 1;
    a.kchunk = (int)(cdiv(std::max(K, 1L), KT) * KT);
    a.ws = nullptr;
    const bool implicit = cv && (cv->mode == 2 || cv->mode == 3);     // operands read from padded planes
    a.wide = (!implicit && (lda >= (1L << 23) || ldb >= (1L << 23))) ? 1 : 0;
    if (per_image_k) {
        // one split per piece of an image: K = B * kimg, A = [B][M][kimg]
        const long kimg = cv->plane;
        CGT_ARG_CHECK(kimg >= 1 && cv->B >= 1 && cv->B * kimg == K && lda == kimg, "sgemm_conv: per-image K does not match the operands");
        // pieces per image: every CU should get the same number of workgroups, about four (they
        // are resident together), with at least 8 slices per piece and a workspace <= 256 MiB ...
        const long cap = (256L << 20) / (M * N * (long)sizeof(float));
        const long max_pieces = std::max(1L, std::min({kimg / (8 * KT), cap / cv->B, 64L}));
        long pieces = 1;
        double best_cost = 0;
        for (long p = 1; p <= max_pieces; ++p) {
            const long wgs = tiles * cv->B * p;
            // time ~ the busiest CU's share of the work; too few workgroups per CU leave latency uncovered;
            // every piece costs a partial result written and read back
            const double busiest = (double)cdiv(wgs, kNumCU) * kNumCU / wgs;
            const double cover = wgs >= 3L * kNumCU ? 1.0 : 1.0 + 0.15 * (3.0 - (double)wgs / kNumCU);
            const double cost = busiest * cover + 0.01 * p;
            if (p == 1 || cost < best_cost - 1e-9) {
                best_cost = cost;
                pieces = p;
            }
        }
        a.kchunk = (int)(cdiv(cdiv(kimg, pieces), KT) * KT);
        pieces = cdiv(kimg, a.kchunk);
        CGT_ARG_CHECK(cv->B * pieces < (1L << 20) && cv->B * pieces * M * N < (1L << 29),   // ... 2 GiB at the very most
                      "sgemm_conv: too many images for the weight gradient's partial sums");
        a.kimg = (int)kimg;
        a.kspi = (int)pieces;
        a.aimg = (M - 1) * kimg;
        a.splits = (int)(cv->B * pieces);
        if (a.splits > 1) {
            a.ws = workspace((size_t)a.splits * M * N * sizeof(float));
            if (!a.ws) return ws_rc;
        }
    } else if (P == 1 && tiles < 512 && K >= 64 * KT && !writes_nchw) {
        long want = std::max(1L, 1024 / tiles);
        want = std::min(want, K / (8 * KT));                    // at least 8 slices per split
        const long cap = (256L << 20) / (M * N * (long)sizeof(float));  // workspace <= 256 MiB
        want = std::min(want, std::max(1L, cap));
        if (want > 1) {
            a.kchunk = (int)(cdiv(cdiv(K, want), KT) * KT);
            a.splits = (int)cdiv(K, a.kchunk);
        }
        if (a.splits > 1) {
            a.ws = workspace((size_t)a.splits * M * N * sizeof(float));
            if (!a.ws) return ws_rc;
        }
    }
    // a weight gradient wanted in the filters' layout: the reduce kernel stores it that way; a product
    // that is not split writes its one "partial" to the workspace and the same kernel moves it
    const int out_taps = cv && cv->mode == 2 ? cv->out_taps : 0;
    float* const C_final = C;
    if (out_taps > 0) {
        CGT_ARG_CHECK(P == 1 && ldc == N && N % out_taps == 0, "sgemm_conv: the filters' layout needs a dense [M][taps * C] result");
        if (a.splits == 1) {
            C = workspace((size_t)M * N * sizeof(float));
            if (!C) return ws_rc;
            a.C = C;
        }
    }
    // tail split (single product, no split-K): tiles beyond the last full
    // round of the chip are cut along K so the partial round is balanced
    a.main_wgs = (int)(tiles * P);
    a.tail_splits = 1;
    a.tail_kchunk = a.kchunk;
    long tail_tiles = 0;
    const long nk = cdiv(K, KT);
    if (P == 1 && a.splits == 1 && tiles >= kNumCU && tiles < 24L * kNumCU && tiles % kNumCU != 0 && nk >= 16 &&
        out_taps == 0) {     // (there the workspace holds the product itself)
        const long r = tiles % kNumCU;
        long best_s = 1;
        double best_t = (double)cdiv(r, kNumCU);             // tail time in units of one whole tile
        for (long sp = 2; sp <= std::min((long)kMaxTailSplits, nk / 4); ++sp) {
            const double t = (double)cdiv(r * sp, kNumCU) / sp + 0.02 * sp;   // small charge per extra piece
            if (t < best_t) {
                best_t = t;
                best_s = sp;
            }
        }
        if (best_s > 1) {
            tail_tiles = r;
            a.main_wgs = (int)(tiles - r);
            a.tail_kchunk = (int)(cdiv(cdiv(K, best_s), KT) * KT);
            a.tail_splits = (int)cdiv(K, a.tail_kchunk);
            a.ws = workspace((size_t)tail_tiles * a.tail_splits * kShapes[shape].bm * kShapes[shape].bn * sizeof(float));
            if (!a.ws) return ws_rc;
        }
    }
    const long wgs = a.splits > 1 ? tiles * a.splits : a.main_wgs + tail_tiles * a.tail_splits;
    CGT_ARG_CHECK(wgs < (1L << 31), "sgemm: too many workgroups");
    hipStream_t st = as_stream(stream);
    dim3 grid((unsigned)wgs);
    // The pipelined loop needs up to ~140 registers in its 128x128 form (3 workgroups
    // per CU instead of 4): it is used once every CU has more than a handful of tiles
    // to work through, not when the whole product is one round of resident
    // workgroups (4096^3: 1024 tiles = 4 per CU), and not for a ragged K, where its
    // tiles would all take the register-staged variant (K = 363: plain loop +3 %).
    const bool pipe = !cv && tiles * P >= 5L * kNumCU && K % KT == 0;
    // two slices of loads in flight: one round of resident workgroups (they start together
    // and load in bursts) with a long K range each
    const long slices = cdiv(a.splits > 1 ? (long)a.kchunk : K, KT);
    const bool deep = !cv && shape == 0 && !(!tA && tB) && wgs <= 4L * kNumCU && slices >= 32;
    if (pg && gpad) launch_gather<true>(cv->mode == 1 ? 1 : 2, shape, grid, st, a);
    else if (pg) launch_gather<false>(cv->mode == 1 ? 1 : 2, shape, grid, st, a);
    else if (conv_kernel) launch_conv(cv->mode, shape, grid, st, a);
    else launch_trans(tA, tB, pipe, deep, shape, grid, st, a);
    CGT_LAUNCH_CHECK("sgemm_kernel");
    if (out_taps > 0) {
        int rc = reduce_partials(a.splits > 1 ? a.ws : C, C_final, M * N, a.splits, stream, (int)N, out_taps);
        if (rc) return rc;
    } else if (a.splits >= 64 && M * N <= (1L << 16) && ldc == N) {
        int rc = reduce_partials(a.ws, C, M * N, a.splits, stream);      // hundreds of partials of a small result
        if (rc) return rc;
    } else if (a.splits > 1) {
        const long MN = M * N;
        const bool vec = N % 4 == 0 && ldc % 4 == 0 && aligned16(C) && aligned16(a.ws);
        const long blocks = cdiv(MN, vec ? 256L : 64L);
        CGT_ARG_CHECK(blocks < (1L << 31), "sgemm: too many reduce workgroups");
        if (vec) splitk_reduce_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a.ws, C, MN, (int)N, ldc, a.splits);
        else splitk_reduce_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a.ws, C, MN, (int)N, ldc, a.splits);
        CGT_LAUNCH_CHECK("splitk_reduce_kernel");
    } else if (tail_tiles > 0 && writes_nchw) {
        tail_reduce_conv_kernel<<<dim3((unsigned)cdiv(kShapes[shape].bm * kShapes[shape].bn, 1024), (unsigned)tail_tiles), dim3(256), 0, st>>>(
            a.ws, a, kShapes[shape].bm, kShapes[shape].bn);
        CGT_LAUNCH_CHECK("tail_reduce_conv_kernel");
    } else if (tail_tiles > 0) {
        tail_reduce_kernel<<<dim3((unsigned)cdiv(kShapes[shape].bm * kShapes[shape].bn, 1024), (unsigned)tail_tiles), dim3(256), 0, st>>>(
            a.ws, C, a, kShapes[shape].bm, kShapes[shape].bn);
        CGT_LAUNCH_CHECK("tail_reduce_kernel");
    }
    return CGT_AMD_OK;
}

int sgemm_conv(const ConvGemm& cv, long M, long N, const float* A, const float* B, float* C, long ldc,
               void* stream) {
    const long taps = (long)cv.kh * cv.kw;
    if (cv.mode == 1)   // A = filters [M][K], B = column buffer [N][K] with K = C (the patch length); C is NCHW, written by the kernel
        return gemm_dispatch(0, 1, 1, M, N, cv.C, A, cv.C, 0, B, cv.C, 0, C, N, 0, stream, false, &cv);
    if (cv.mode == 4)   // A = cotangent [B][M][plane], B = column buffer [B * plane][N]; C = [M][N]
        return gemm_dispatch(0, 0, 1, M, N, cv.B * cv.plane, A, cv.plane, 0, B, N, 0, C, ldc, 0, stream, false, &cv);
    if (cv.mode == 3)   // A = filters [M][taps * C], B = image (row-contiguous operand); C is NCHW, written by the kernel
        return gemm_dispatch(0, 0, 1, M, N, taps * cv.C, A, taps * cv.C, 0, B, N, 0, C, N, 0, stream, false, &cv);
    // A = cotangent planes [B][M][plane], B = image; K runs over (image, pixel slice)
    return gemm_dispatch(0, 1, 1, M, N, cv.B * cv.spi * KT, A, cv.plane, 0, B, cv.plane, 0, C, ldc, 0, stream, false, &cv);
}

}  // namespace cgt_amd

using namespace cgt_amd;

CGT_API int cgt_amd_sgemm(int tA, int tB, long M, long N, long K, const float* A, long lda,
                          const float* B, long ldb, float* C, long ldc, void* stream) {
    return gemm_dispatch(tA, tB, 1, M, N, K, A, lda, 0, B, ldb, 0, C, ldc, 0, stream);
}

CGT_API int cgt_amd_sgemm_noalloc(int tA, int tB, long M, long N, long K, const float* A, long lda,
                                  const float* B, long ldb, float* C, long ldc, void* stream) {
    return gemm_dispatch(tA, tB, 1, M, N, K, A, lda, 0, B, ldb, 0, C, ldc, 0, stream, true);
}

CGT_API int cgt_amd_sgemm_batched(int tA, int tB, long P, long M, long N, long K, const float* A,
                                  long lda, long strideA, const float* B, long ldb, long strideB,
                                  float* C, long ldc, long strideC, void* stream) {
    return gemm_dispatch(tA, tB, P, M, N, K, A, lda, strideA, B, ldb, strideB, C, ldc, strideC, stream);
}
