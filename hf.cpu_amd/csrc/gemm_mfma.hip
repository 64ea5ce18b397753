// bf16 matrix product on the matrix cores: out[m, n] = sum_k a[m, k] * w[n, k], fp32 accumulation.
//
// Both operands are K-contiguous, which is what v_mfma_f32_32x32x16_bf16 wants: a lane supplies
// 8 consecutive k of one row of A (rows -> output rows) and of one row of W (rows -> output
// columns), so every operand fragment is one 16-byte LDS read and output columns lie along
// lanes (coalesced stores). A block of WM x WN waves owns a BM x BN output tile and walks K in
// steps of BK through two LDS stages: the next tile travels global -> registers while the
// current one is multiplied, then registers -> LDS, one barrier per step. LDS rows are padded
// by 8 elements, which makes the 16-byte fragment reads conflict-free.
//
// Block ids are dealt round-robin to the 8 XCDs by the hardware; the kernel undoes that so
// that each XCD works on a contiguous run of tiles, and walks tiles in groups of 8 rows of
// tiles, so the tiles resident on an XCD at one time share operand panels in its L2.
//
// Small M (decode) is bandwidth-bound and has few output tiles: K is split over blockIdx.z,
// partial sums go to a workspace and a second kernel adds them in a fixed order and applies
// bias and the output mode. Nothing is accumulated with atomics: results are reproducible.
//
// Which kernel takes which shape (gemm_mfma_launch, at the end of this file):
//   M <= 16          gemm_wave_kernel (gemm_wave.hip) if K is a multiple of 64 and there are as many units as waves; else as
//   M <= 32          gemm_mfma_kernel, tiles of 32 x 128, K split, two register sets of loads in flight
//   M in 33 .. 128   gemm_stream_kernel (gemm_stream.hip) if N is a multiple of 128 and K of 64, the output
//                    has fewer than 512 tiles and a block gets 16 units or more; else gemm_mfma_kernel
//                    with tiles of 64 x 128 or 128 x 128
//   M > 64           gemm_dma_kernel (below) with tiles of 256 rows, if M wastes few of them and the
//                    output has 128 tiles of 256 x 256 (tiles of 256 x 192 where those need fewer rounds
//                    over the CUs; with fewer K is cut into parts that give every CU a block, with tiles of
//                    256 x 128 if M is at most 256; or the tiles are 256 x 128 without parts); else
//                    gemm_mfma_kernel with tiles of 128 x 128
#include <type_traits>

#include "common.h"
#include "gemm_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define N_XCD 8
#define GROUP_M 8
#define OUT_BF16 0
#define OUT_F32 1
#define OUT_ACC 2
#define OUT_PARTIAL 3
#define OUT_SWIGLU 4      // columns come in blocks of 32 gate, 32 up; out[m, f] = silu(gate) * up as bf16

template <int BM, int BN, int BK, int WM, int WN>
struct MfmaCfg {
    static constexpr int NT = WM * WN * WAVE;
    static constexpr int STRIDE = BK + 8;                    // LDS row stride in elements
    static constexpr int STAGE = (BM + BN) * STRIDE;         // elements per stage
    static constexpr int SMEM = 2 * STAGE * 2;               // bytes
    static constexpr int CPR = BK / 8;                       // 16-byte chunks per tile row
    static constexpr int A_CH = BM * CPR / NT;
    static constexpr int W_CH = BN * CPR / NT;
    static constexpr int TM = BM / WM, TN = BN / WN;         // per wave
    static constexpr int FM = TM / 32, FN = TN / 32;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "tile rows must spread evenly over the threads");
    static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 16 == 0, "wave tiles are made of 32x32x16 products");
};

// Stores a wave's accumulators: element r of a lane is row 8 * (r / 4) + 4 * (lane / 32) + r % 4,
// column lane % 32 of its 32x32 block.
template <class C, int MODE>
__device__ __forceinline__ void gemm_epilogue(floatx16 (&acc)[C::FM][C::FN], const float* __restrict__ bias,
                                              void* __restrict__ out, int ldo, int M, int N, int m0, int n0, int wm,
                                              int wn, int lane) {
    if (MODE == OUT_SWIGLU) {
        static_assert(MODE != OUT_SWIGLU || C::FN % 2 == 0, "gate and up blocks must meet in one wave");
#pragma unroll
        for (int i = 0; i < C::FM; i++) {
#pragma unroll
            for (int j = 0; j + 1 < C::FN; j += 2) {
                const int col = n0 + wn * C::TN + j * 32;          // first gate column of the pair of blocks
                if (col + (lane & 31) >= N) continue;
                const int f = col / 2 + (lane & 31);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * C::TM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                    if (row >= M) continue;
                    const float gt = acc[i][j][r], up = acc[i][j + 1][r];
                    reinterpret_cast<uint16_t*>(out)[(size_t)row * ldo + f] = bf16_bits((gt / (1.0f + expf(-gt))) * up);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < C::FM; i++) {
#pragma unroll
        for (int j = 0; j < C::FN; j++) {
            const int col = n0 + wn * C::TN + j * 32 + (lane & 31);
            if (col >= N) continue;
            const float b = (MODE != OUT_PARTIAL && bias) ? bias[col] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm * C::TM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (row >= M) continue;
                const float v = acc[i][j][r] + b;
                if (MODE == OUT_BF16) {
                    reinterpret_cast<uint16_t*>(out)[(size_t)row * ldo + col] = bf16_bits(v);
                } else if (MODE == OUT_F32) {
                    reinterpret_cast<float*>(out)[(size_t)row * ldo + col] = v;
                } else if (MODE == OUT_ACC) {
                    float* dst = reinterpret_cast<float*>(out) + (size_t)row * ldo + col;
                    *dst += v;
                } else {
                    reinterpret_cast<float*>(out)[((size_t)blockIdx.z * M + row) * N + col] = v;
                }
            }
        }
    }
}

// The block's tile of 16-bit results in LDS: rows of WIDTH columns, 16 bytes of padding.
template <int BN, int MODE>
struct DmaOut {
    static constexpr int PAIR = MODE == OUT_SWIGLU ? 2 : 1;      // 32 gate and 32 up columns give 32 results
    static constexpr int WIDTH = BN / PAIR, STRIDE = WIDTH + 8;
    static constexpr int bytes(int bm) { return (MODE == OUT_BF16 || MODE == OUT_SWIGLU) ? bm * STRIDE * 2 : 0; }
};

// 16-bit results leave through LDS: a lane holds single columns, and a store of 2 bytes per lane
// costs the memory path as much as one of 16. The block's tile is put together in LDS (the operand
// stages are free by now), then written out 16 bytes per lane, whole rows. Needs 16-byte aligned
// output rows and a multiple of 8 output columns (the launchers check).
template <class C, int BM, int BN, int MODE>
__device__ __forceinline__ void gemm_epilogue_rows(floatx16 (&acc)[C::FM][C::FN], const float* __restrict__ bias,
                                                   void* __restrict__ out, int ldo, int M, int N, int m0, int n0,
                                                   int wm, int wn, int lane, int tid, uint16_t* smem) {
    using O = DmaOut<BN, MODE>;
    static_assert(MODE != OUT_SWIGLU || C::FN % 2 == 0, "gate and up blocks must meet in one wave");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < C::FM; i++) {
#pragma unroll
        for (int j = 0; j < C::FN; j += O::PAIR) {
            const int col = (wn * C::TN + j * 32) / O::PAIR + (lane & 31);      // within the block's tile
            const int gcol = n0 + wn * C::TN + j * 32 + (lane & 31);            // column of N (the gate's, if paired)
            const float b = (MODE == OUT_BF16 && bias && gcol < N) ? bias[gcol] : 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = wm * C::TM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                float v = acc[i][j][r] + b;
                if constexpr (MODE == OUT_SWIGLU) v = (v / (1.0f + expf(-v))) * acc[i][j + 1][r];
                smem[row * O::STRIDE + col] = bf16_bits(v);
            }
        }
    }
    __syncthreads();
    const int out0 = n0 / O::PAIR, n_out = N / O::PAIR;
    uint16_t* o16 = reinterpret_cast<uint16_t*>(out);
    for (int c = tid; c < BM * (O::WIDTH / 8); c += C::NT) {
        const int row = c / (O::WIDTH / 8), piece = c % (O::WIDTH / 8);
        if (m0 + row < M && out0 + piece * 8 < n_out)
            *reinterpret_cast<uint4*>(o16 + (size_t)(m0 + row) * ldo + out0 + piece * 8) =
                *reinterpret_cast<const uint4*>(smem + row * O::STRIDE + piece * 8);
    }
}

template <int BM, int BN, int BK, int WM, int WN, int MODE, int PF>
__global__ __launch_bounds__(WM* WN* WAVE) void gemm_mfma_kernel(
    const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ W, int ldw,
    const float* __restrict__ bias, void* __restrict__ out, int ldo, int M, int N, int K, int k_per_split,
    int tiles_m, int tiles_n, int rows_out) {
    using C = MfmaCfg<BM, BN, BK, WM, WN>;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int wm = wave / WN, wn = wave % WN;

    // ---- which tile: undo the round-robin over XCDs, then grouped order ----
    const int n_tiles = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = n_tiles / N_XCD, rem = n_tiles % N_XCD, x = pid % N_XCD, q = pid / N_XCD;
        pid = x * per + (x < rem ? x : rem) + q;             // XCD x owns a contiguous run of tiles
    }
    const int in_group = GROUP_M * tiles_n;
    const int group = pid / in_group, first_m = group * GROUP_M;
    const int gsize = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (pid % in_group) % gsize, tn = (pid % in_group) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;
    const int kbeg = blockIdx.z * k_per_split;
    const int kend = kbeg + k_per_split < K ? kbeg + k_per_split : K;

    floatx16 acc[C::FM][C::FN];
#pragma unroll
    for (int i = 0; i < C::FM; i++)
#pragma unroll
        for (int j = 0; j < C::FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // PF register sets of loads: while tile t is multiplied out of LDS, tiles t + 1 .. t + PF are on
    // their way from memory. PF = 1 (large M): few registers, more blocks per CU. PF = 2 (small M,
    // bound by the weights' stream): twice the bytes in flight of a block; four sets stream no faster.
    static_assert(PF == 1 || PF % 2 == 0, "the stage of a tile is known at compile time");
    uint4 ra[PF][C::A_CH], rw[PF][C::W_CH];
    auto gload = [&](uint4* ra, uint4* rw, int k0) {
#pragma unroll
        for (int i = 0; i < C::A_CH; i++) {
            const int c = tid + i * C::NT, row = c / C::CPR, kk = k0 + (c % C::CPR) * 8;
            int gr = m0 + row;
            gr = gr < M ? gr : M - 1;                        // rows past the edge repeat the last one
            ra[i] = kk < kend ? *reinterpret_cast<const uint4*>(A + (size_t)gr * lda + kk) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < C::W_CH; i++) {
            const int c = tid + i * C::NT, row = c / C::CPR, kk = k0 + (c % C::CPR) * 8;
            int gr = n0 + row;
            gr = gr < N ? gr : N - 1;
            rw[i] = kk < kend ? *reinterpret_cast<const uint4*>(W + (size_t)gr * ldw + kk) : make_uint4(0, 0, 0, 0);
        }
    };
    auto sstore = [&](int stage, const uint4* ra, const uint4* rw) {
        uint16_t* sa = smem + stage * C::STAGE;
        uint16_t* sw = sa + BM * C::STRIDE;
#pragma unroll
        for (int i = 0; i < C::A_CH; i++) {
            const int c = tid + i * C::NT, row = c / C::CPR, kc = c % C::CPR;
            *reinterpret_cast<uint4*>(sa + row * C::STRIDE + kc * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < C::W_CH; i++) {
            const int c = tid + i * C::NT, row = c / C::CPR, kc = c % C::CPR;
            *reinterpret_cast<uint4*>(sw + row * C::STRIDE + kc * 8) = rw[i];
        }
    };
    auto compute = [&](int stage) {
        const uint16_t* sa = smem + stage * C::STAGE + (wm * C::TM + (lane & 31)) * C::STRIDE + (lane >> 5) * 8;
        const uint16_t* sw = smem + stage * C::STAGE + (BM + wn * C::TN + (lane & 31)) * C::STRIDE + (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 fa[C::FM], fw[C::FN];
#pragma unroll
            for (int i = 0; i < C::FM; i++) fa[i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * C::STRIDE + kk);
#pragma unroll
            for (int j = 0; j < C::FN; j++) fw[j] = *reinterpret_cast<const bf16x8*>(sw + j * 32 * C::STRIDE + kk);
#pragma unroll
            for (int i = 0; i < C::FM; i++)
#pragma unroll
                for (int j = 0; j < C::FN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        }
    };

    const int nk = (kend - kbeg + BK - 1) / BK;
    gload(ra[0], rw[0], kbeg);
#pragma unroll
    for (int p = 1; p < PF; p++)                             // tile p waits in set p % PF; all are asked for
        if (p < nk) gload(ra[p], rw[p], kbeg + p * BK);      // before the first one is waited for
    sstore(0, ra[0], rw[0]);
    if (PF < nk) gload(ra[0], rw[0], kbeg + PF * BK);
    __syncthreads();
    if (PF == 1) {
        for (int t = 0; t < nk; t++) {
            compute(t & 1);
            if (t + 1 < nk) sstore((t + 1) & 1, ra[0], rw[0]);
            if (t + 2 < nk) gload(ra[0], rw[0], kbeg + (t + 2) * BK);
            __syncthreads();
        }
    }
    for (int t0 = 0; PF > 1 && t0 < nk; t0 += PF) {
#pragma unroll
        for (int p = 0; p < PF; p++) {                       // tile t0 + p: its stage and the sets are constants here
            const int t = t0 + p;
            if (t >= nk) break;
            compute(p & 1);
            if (t + 1 < nk) {
                sstore((p + 1) & 1, ra[(p + 1) % PF], rw[(p + 1) % PF]);
                if (t + 1 + PF < nk) gload(ra[(p + 1) % PF], rw[(p + 1) % PF], kbeg + (t + 1 + PF) * BK);
            }
            __syncthreads();
        }
    }

    if constexpr (MODE == OUT_BF16 || MODE == OUT_SWIGLU) {
        static_assert(DmaOut<BN, MODE>::bytes(BM) <= C::SMEM, "the tile of results fits the operand stages");
        if (rows_out) {                                      // uniform: the output allows 16-byte stores
            gemm_epilogue_rows<C, BM, BN, MODE>(acc, bias, out, ldo, M, N, m0, n0, wm, wn, lane, tid, smem);
            return;
        }
    }
    gemm_epilogue<C, MODE>(acc, bias, out, ldo, M, N, m0, n0, wm, wn, lane);
}

// ---- large M (prompts): operand tiles travel global -> LDS without passing through registers ----
//
// A block of 2 x 2 waves owns a BM x BN tile, one block per CU, and keeps STAGES tiles of BK
// columns of K in LDS. While tile t is multiplied, tile t + STAGES - 1 is requested
// (global_load_lds_dwordx4: the 64 lanes of a wave fill 1 KB of LDS), one request after every few
// matrix instructions: the texture path takes about as long for a tile's bytes as the matrix
// cores take for its products, so the two have to run side by side, and a wave that issues its
// requests in one burst stands still until the path has taken them all. A load has STAGES - 2
// whole steps to arrive; the only wait of a step is for the oldest tile. The loads are inline
// assembly because the wait they need is "all but the newer tiles'", which only the author of
// the pipeline can state: the compiler, told about such loads, waits for all of them before the
// next LDS read.
//
// LDS rows have no padding (the hardware places the 64 lanes' 16 bytes back to back); instead the
// 16-byte pieces of a row are stored in swizzled order, which a lane arranges by which piece it
// asks for: with rows of 128 bytes, piece p of row r lies at p ^ ((r / 2) % 8); with rows of 64
// bytes, at p ^ ((r / 4) % 4). A 16-byte read is served 16 lanes a cycle (all 64 banks): sixteen
// lanes that read the same piece of sixteen consecutive rows then hit sixteen different groups
// of four banks (with a swizzle that only tells eight rows apart, SQ_LDS_BANK_CONFLICT counts
// four more cycles for every read).
template <int BM, int BN, int BK, int WM, int WN>
struct DmaCfg {
    static constexpr int NW = WM * WN, NT = NW * WAVE;
    static constexpr int ROWS = BM + BN;
    static constexpr int PIECES = BK / 8;                    // 16-byte pieces per row
    static constexpr int ROWS_PER_LOAD = WAVE / PIECES;
    static constexpr int STAGE_BYTES = ROWS * BK * 2;
    static constexpr int REQUESTS = ROWS / ROWS_PER_LOAD;    // per stage
    static constexpr int LOADS = (REQUESTS + NW - 1) / NW;   // per wave and stage; past the last one a wave repeats it
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int FM = TM / 32, FN = TN / 32;
    static constexpr int STEPS = BK / 16;
    static_assert(BK == 32 || BK == 64, "rows of 64 or 128 bytes");
    static_assert(ROWS % ROWS_PER_LOAD == 0 && BM % ROWS_PER_LOAD == 0, "a request fills whole rows of one operand");
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tiles are made of 32x32x16 products");
    static_assert(FM * FN * STEPS >= LOADS, "at most one request after a matrix instruction");
    __device__ static constexpr int swizzle(int row) { return BK == 64 ? ((row >> 1) & 7) : ((row >> 2) & 3); }
};

template <int BM, int BN, int BK, int WM, int WN, int STAGES, int MODE>
__global__ __launch_bounds__(WM* WN* WAVE) void gemm_dma_kernel(
    const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ W, int ldw,
    const float* __restrict__ bias, void* __restrict__ out, int ldo, int M, int N, int K, int k_per_split,
    int tiles_m, int tiles_n) {
    using C = DmaCfg<BM, BN, BK, WM, WN>;
    static_assert(STAGES >= 3, "one tile in use, the next one landed, one arriving");
    extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wm = wave / WN, wn = wave % WN;

    const int n_tiles = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = n_tiles / N_XCD, rem = n_tiles % N_XCD, x = pid % N_XCD, q = pid / N_XCD;
        pid = x * per + (x < rem ? x : rem) + q;
    }
    const int in_group = GROUP_M * tiles_n;
    const int group = pid / in_group, first_m = group * GROUP_M;
    const int gsize = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (pid % in_group) % gsize, tn = (pid % in_group) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    floatx16 acc[C::FM][C::FN];
#pragma unroll
    for (int i = 0; i < C::FM; i++)
#pragma unroll
        for (int j = 0; j < C::FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // Request i of this wave fills rows (i * NW + wave) * ROWS_PER_LOAD .. of a stage; this lane
    // supplies the piece stored at lane % PIECES of row lane / PIECES of them. Its address is a
    // scalar base (the block's first row of A or W, advancing with K) plus a byte offset per lane.
    const int kbeg = blockIdx.z * k_per_split;               // K may be split over blockIdx.z (narrow outputs)
    const int kend = kbeg + k_per_split < K ? kbeg + k_per_split : K;
    const uint16_t* a_base = A + (size_t)m0 * lda + kbeg;
    const uint16_t* w_base = W + (size_t)n0 * ldw + kbeg;
    // When the requests do not divide by the waves, the waves left over repeat the stage's last
    // request (same bytes to the same place), so that every wave counts the same number of loads.
    auto request_no = [&](int i) { return i * C::NW + wave < C::REQUESTS ? i * C::NW + wave : C::REQUESTS - 1; };
    uint32_t src[C::LOADS];
#pragma unroll
    for (int i = 0; i < C::LOADS; i++) {
        const int r = request_no(i) * C::ROWS_PER_LOAD + lane / C::PIECES;
        const int piece = (lane % C::PIECES) ^ C::swizzle(r);
        if (request_no(i) * C::ROWS_PER_LOAD < BM) {
            const int last = M - 1 - m0;                     // rows past the edge repeat the last one
            src[i] = (uint32_t)(r < last ? r : last) * (uint32_t)lda * 2u + piece * 16;
        } else {
            const int last = N - 1 - n0;
            src[i] = (uint32_t)(r - BM < last ? r - BM : last) * (uint32_t)ldw * 2u + piece * 16;
        }
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)smem;
    auto request = [&](int i, int stage, int t) {            // i is a constant after unrolling
        const uint32_t dst = lds0 + stage * C::STAGE_BYTES + request_no(i) * 1024;
        const bool is_a = request_no(i) * C::ROWS_PER_LOAD < BM;           // uniform over the wave
        const uint16_t* base = (is_a ? a_base : w_base) + (size_t)t * BK;
        uint64_t sbase;           // the address in registers that a scalar instruction wrote (gemm_rows.hip: hazards)
        asm volatile("s_mov_b32 m0, %1\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0" : "=&s"(sbase) : "s"(dst), "v"(src[i]), "s"(base) : "m0");
    };
    // Piece offsets (in elements) of the 16-column steps of a tile for this lane's rows: the rows
    // a lane reads differ from lane % 32 by multiples of 32, so their swizzle is the lane's.
    int piece_off[C::STEPS];
#pragma unroll
    for (int j = 0; j < C::STEPS; j++) piece_off[j] = ((2 * j + (lane >> 5)) ^ C::swizzle(lane & 31)) * 8;

    // Operand fragments of 16-column step j of the tile in `stage`.
    auto fragments = [&](int stage, int j, bf16x8 (&fa)[C::FM], bf16x8 (&fw)[C::FN]) {
        const uint16_t* sa = smem + stage * (C::STAGE_BYTES / 2) + (wm * C::TM + (lane & 31)) * BK + piece_off[j];
        const uint16_t* sw = smem + stage * (C::STAGE_BYTES / 2) + (BM + wn * C::TN + (lane & 31)) * BK + piece_off[j];
#pragma unroll
        for (int i = 0; i < C::FM; i++) fa[i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * BK);
#pragma unroll
        for (int i = 0; i < C::FN; i++) fw[i] = *reinterpret_cast<const bf16x8*>(sw + i * 32 * BK);
    };

    // The pipeline. Tiles 0 .. STAGES - 2 are requested up front. Step t begins with a wait and a
    // barrier after which tile t + 1 has landed for every wave and every wave is done with tile
    // t - 1; tile t + STAGES - 1 is then requested into tile t - 1's stage, a request after every
    // few matrix instructions. The fragments of a 16-column step are read one step ahead, also
    // across the barrier (tile t + 1's first ones during tile t's last step), so that the matrix
    // cores have work the moment a wave leaves the barrier.
    const int nk = (kend - kbeg) / BK;
#pragma unroll
    for (int p = 0; p < STAGES - 1; p++)
        if (p < nk) {
#pragma unroll
            for (int i = 0; i < C::LOADS; i++) request(i, p, p);
        }
    if (nk >= STAGES - 1)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(C::LOADS * (STAGES - 2)) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    bf16x8 fa[2][C::FM], fw[2][C::FN];
    fragments(0, 0, fa[0], fw[0]);
    constexpr int AHEAD = STAGES - 1;
    constexpr int PRODUCTS = C::FM * C::FN * C::STEPS;      // matrix instructions per tile and wave
    // With three stages a load has to arrive within the step after its request: request early.
    constexpr int SPREAD = STAGES == 3 ? (PRODUCTS / 2 > C::LOADS ? PRODUCTS / 2 : C::LOADS) : PRODUCTS;
    static_assert(SPREAD >= C::LOADS && SPREAD <= PRODUCTS && C::STEPS % 2 == 0, "at most one request after a matrix instruction");
    int stage = 0;
    // `steady`: tile t + AHEAD exists, so the step has no condition in it (all but the last steps).
    auto step = [&](int t, auto steady) {
        constexpr bool STEADY = decltype(steady)::value;
        if (STEADY || t + STAGES - 2 < nk)
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(C::LOADS * (STAGES - 3)) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const int into = stage + AHEAD < STAGES ? stage + AHEAD : stage + AHEAD - STAGES;
        const int next = stage + 1 < STAGES ? stage + 1 : 0;
        int done = 0;
#pragma unroll
        for (int j = 0; j < C::STEPS; j++) {
            if (j + 1 < C::STEPS)
                fragments(stage, j + 1, fa[(j + 1) & 1], fw[(j + 1) & 1]);
            else if (STEADY || t + 1 < nk)
                fragments(next, 0, fa[0], fw[0]);
            __builtin_amdgcn_sched_barrier(0);               // the reads are issued before the products that hide them
#pragma unroll
            for (int i = 0; i < C::FM; i++)
#pragma unroll
                for (int jj = 0; jj < C::FN; jj++) {
                    acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[j & 1][i], fw[j & 1][jj], acc[i][jj], 0, 0, 0);
                    done++;                                  // requests are dealt evenly among the first products
                    if (STEADY && done <= SPREAD && done * C::LOADS / SPREAD != (done - 1) * C::LOADS / SPREAD)
                        request(done * C::LOADS / SPREAD - 1, into, t + AHEAD);
                }
        }
        stage = next;
    };
    int t = 0;
    for (; t + AHEAD < nk; t++) step(t, std::true_type());
    for (; t < nk; t++) step(t, std::false_type());
    if constexpr (MODE == OUT_BF16 || MODE == OUT_SWIGLU) {
        gemm_epilogue_rows<C, BM, BN, MODE>(acc, bias, out, ldo, M, N, m0, n0, wm, wn, lane, tid, smem);
    } else {
        gemm_epilogue<C, MODE>(acc, bias, out, ldo, M, N, m0, n0, wm, wn, lane);
    }
}

// Sum of the K splits in ascending order, then bias and the output mode.
template <int MODE>
__global__ void gemm_finish_kernel(const float* __restrict__ partial, int splits, const float* __restrict__ bias,
                                   void* __restrict__ out, int ldo, int M, int N) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)M * N) return;
    const int row = (int)(idx / N), col = (int)(idx % N);
    float v = 0.f;
    for (int s = 0; s < splits; s++) v += partial[(size_t)s * M * N + idx];
    if (bias) v += bias[col];
    if (MODE == OUT_SWIGLU) {                 // this thread holds a gate column; its up column is 32 further
        if ((col & 32) != 0) return;
        float up = 0.f;
        for (int s = 0; s < splits; s++) up += partial[(size_t)s * M * N + idx + 32];
        reinterpret_cast<uint16_t*>(out)[(size_t)row * ldo + (col / 64) * 32 + (col & 31)] =
            bf16_bits((v / (1.0f + expf(-v))) * up);
    } else if (MODE == OUT_BF16)
        reinterpret_cast<uint16_t*>(out)[(size_t)row * ldo + col] = bf16_bits(v);
    else if (MODE == OUT_F32)
        reinterpret_cast<float*>(out)[(size_t)row * ldo + col] = v;
    else
        reinterpret_cast<float*>(out)[(size_t)row * ldo + col] += v;
}

// The gate/up case of the above, four results a thread: 16-byte loads of every plane asked for
// together (in batches of eight planes), added in ascending order, one 8-byte store.
__global__ void gemm_finish_swiglu4_kernel(const float* __restrict__ partial, int splits, uint16_t* __restrict__ out,
                                           int ldo, int M, int N) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;      // (row, block of 64 columns, quad)
    const int per_row = N / 8;
    if (idx >= (size_t)M * per_row) return;
    const int row = (int)(idx / per_row), in_row = (int)(idx % per_row);
    const int blk = in_row / 8, quad = in_row % 8;
    const size_t plane = (size_t)M * N;
    const float* src = partial + (size_t)row * N + blk * 64 + quad * 4;
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f), u = g;
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float4 pg[8], pu[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            pg[i] = s0 + i < splits ? *reinterpret_cast<const float4*>(src + (s0 + i) * plane) : make_float4(0.f, 0.f, 0.f, 0.f);
            pu[i] = s0 + i < splits ? *reinterpret_cast<const float4*>(src + (s0 + i) * plane + 32) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            g.x += pg[i].x; g.y += pg[i].y; g.z += pg[i].z; g.w += pg[i].w;
            u.x += pu[i].x; u.y += pu[i].y; u.z += pu[i].z; u.w += pu[i].w;
        }
    }
    uint2 pk;
    pk.x = (uint32_t)bf16_bits((g.x / (1.0f + expf(-g.x))) * u.x) | ((uint32_t)bf16_bits((g.y / (1.0f + expf(-g.y))) * u.y) << 16);
    pk.y = (uint32_t)bf16_bits((g.z / (1.0f + expf(-g.z))) * u.z) | ((uint32_t)bf16_bits((g.w / (1.0f + expf(-g.w))) * u.w) << 16);
    *reinterpret_cast<uint2*>(out + (size_t)row * ldo + blk * 32 + quad * 4) = pk;
}

template <int BM, int BN, int BK, int WM, int WN, int MODE, int PF>
static int launch_cfg(const GemmArgs& g, void* out, int splits, int k_per_split) {
    using C = MfmaCfg<BM, BN, BK, WM, WN>;
    auto kernel = gemm_mfma_kernel<BM, BN, BK, WM, WN, MODE, PF>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM);
        if (e != hipSuccess) {
            hfa_set_error("gemm_mfma: cannot reserve %d bytes of LDS: %s", C::SMEM, hipGetErrorString(e));
            return 2;
        }
        configured = true;
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    dim3 grid(tiles_m * tiles_n, 1, splits);
    const int n_out = MODE == OUT_SWIGLU ? g.N / 2 : g.N;
    const int rows_out = (MODE == OUT_BF16 || MODE == OUT_SWIGLU) && g.ldo % 8 == 0 && n_out % 8 == 0 && ((uintptr_t)out & 15) == 0;
    kernel<<<grid, C::NT, C::SMEM, g.stream>>>((const uint16_t*)g.a, g.lda, (const uint16_t*)g.w, g.ldw, g.bias, out,
                                              g.ldo, g.M, g.N, g.K, k_per_split, tiles_m, tiles_n, rows_out);
    HFA_LAUNCH_CHECK("gemm_mfma");
    return 0;
}

template <int BM, int BN, int BK, int WM, int WN, int STAGES, int MODE>
static int launch_dma_cfg(const GemmArgs& g, void* out, int splits, int k_per_split) {
    using C = DmaCfg<BM, BN, BK, WM, WN>;
    constexpr int SMEM = STAGES * C::STAGE_BYTES > DmaOut<BN, MODE>::bytes(BM) ? STAGES * C::STAGE_BYTES : DmaOut<BN, MODE>::bytes(BM);
    auto kernel = gemm_dma_kernel<BM, BN, BK, WM, WN, STAGES, MODE>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) {
            hfa_set_error("gemm_dma: cannot reserve %d bytes of LDS: %s", SMEM, hipGetErrorString(e));
            return 2;
        }
        configured = true;
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    kernel<<<dim3(tiles_m * tiles_n, 1, splits), C::NT, SMEM, g.stream>>>(
        (const uint16_t*)g.a, g.lda, (const uint16_t*)g.w, g.ldw, g.bias, out, g.ldo, g.M, g.N, g.K, k_per_split, tiles_m,
        tiles_n);
    HFA_LAUNCH_CHECK("gemm_dma");
    return 0;
}

template <int BM, int BN, int BK, int WM, int WN, int STAGES>
static int launch_dma(const GemmArgs& g, int mode, void* out, int splits, int k_per_split) {
    switch (mode) {
        case OUT_BF16: return launch_dma_cfg<BM, BN, BK, WM, WN, STAGES, OUT_BF16>(g, out, splits, k_per_split);
        case OUT_F32: return launch_dma_cfg<BM, BN, BK, WM, WN, STAGES, OUT_F32>(g, out, splits, k_per_split);
        case OUT_ACC: return launch_dma_cfg<BM, BN, BK, WM, WN, STAGES, OUT_ACC>(g, out, splits, k_per_split);
        case OUT_PARTIAL: return launch_dma_cfg<BM, BN, BK, WM, WN, STAGES, OUT_PARTIAL>(g, out, splits, k_per_split);
        default:
            if constexpr ((BN / WN) % 64 == 0) return launch_dma_cfg<BM, BN, BK, WM, WN, STAGES, OUT_SWIGLU>(g, out, splits, k_per_split);
            hfa_set_error("gemm_dma: this tile shape cannot pair gate and up columns");
            return 1;
    }
}

template <int BM, int BN, int BK, int WM, int WN, int PF = (BM >= 128 ? 1 : 2)>
static int launch_mode(const GemmArgs& g, int mode, void* out, int splits, int k_per_split) {
    switch (mode) {
        case OUT_BF16: return launch_cfg<BM, BN, BK, WM, WN, OUT_BF16, PF>(g, out, splits, k_per_split);
        case OUT_F32: return launch_cfg<BM, BN, BK, WM, WN, OUT_F32, PF>(g, out, splits, k_per_split);
        case OUT_ACC: return launch_cfg<BM, BN, BK, WM, WN, OUT_ACC, PF>(g, out, splits, k_per_split);
        case OUT_SWIGLU:
            if constexpr ((BN / WN) % 64 == 0) return launch_cfg<BM, BN, BK, WM, WN, OUT_SWIGLU, PF>(g, out, splits, k_per_split);
            hfa_set_error("gemm_mfma: this tile shape cannot pair gate and up columns");
            return 1;
        default: return launch_cfg<BM, BN, BK, WM, WN, OUT_PARTIAL, PF>(g, out, splits, k_per_split);
    }
}

bool gemm_mfma_supports(const GemmArgs& g) {
    return g.a_dtype == HFA_BF16 && g.w_dtype == HFA_BF16 && g.K % 8 == 0 && g.lda % 8 == 0 && g.ldw % 8 == 0 &&
           ((uintptr_t)g.a & 15) == 0 && ((uintptr_t)g.w & 15) == 0;
}

int gemm_finish_launch(const float* partial, int splits, const float* bias, void* out, int mode, int ldo, int M,
                       int N, hipStream_t stream) {
    const size_t total = (size_t)M * N;
    const int blocks = (int)((total + 255) / 256);
    if (mode == OUT_BF16)
        gemm_finish_kernel<OUT_BF16><<<blocks, 256, 0, stream>>>(partial, splits, bias, out, ldo, M, N);
    else if (mode == OUT_F32)
        gemm_finish_kernel<OUT_F32><<<blocks, 256, 0, stream>>>(partial, splits, bias, out, ldo, M, N);
    else if (mode == OUT_SWIGLU && !bias && N % 64 == 0 && ldo % 4 == 0 && ((uintptr_t)out & 7) == 0 && ((uintptr_t)partial & 15) == 0)
        gemm_finish_swiglu4_kernel<<<(int)((total / 8 + 255) / 256), 256, 0, stream>>>(partial, splits, (uint16_t*)out, ldo, M, N);
    else if (mode == OUT_SWIGLU)
        gemm_finish_kernel<OUT_SWIGLU><<<blocks, 256, 0, stream>>>(partial, splits, bias, out, ldo, M, N);
    else
        gemm_finish_kernel<OUT_ACC><<<blocks, 256, 0, stream>>>(partial, splits, bias, out, ldo, M, N);
    HFA_LAUNCH_CHECK("gemm_finish");
    return 0;
}

int gemm_mode_of(const GemmArgs& g) {
    if (g.epilogue == 1) return OUT_SWIGLU;
    return g.accumulate ? OUT_ACC : (g.out_dtype == HFA_BF16 ? OUT_BF16 : OUT_F32);
}

int gemm_mfma_launch(const GemmArgs& g, void* workspace, size_t workspace_bytes, int defer, int* pending_splits) {
    const int mode = gemm_mode_of(g);
    if (pending_splits) *pending_splits = 0;
    if (mode == OUT_SWIGLU && (g.N % 64 != 0 || g.bias != nullptr || g.out_dtype != HFA_BF16)) {
        hfa_set_error("gemm: the gate/up epilogue needs N a multiple of 64, no bias and a bf16 output");
        return 1;
    }
    if (g.M <= 16) {                         // very few rows: every wave streams its own run of the weights
        const int slots = gemm_wave_slots(g, workspace ? workspace_bytes : 0);
        if (slots > 0) {
            const int rc = gemm_wave_launch(g, workspace, slots);
            if (rc) return rc;
            if (defer && pending_splits) {
                *pending_splits = slots;
                return 0;
            }
            return gemm_finish_launch((const float*)workspace, slots, g.bias, g.out, mode, g.ldo, g.M, g.N, g.stream);
        }
    }
    if (g.M <= 128) {
        const int slots = gemm_stream_slots(g, workspace ? workspace_bytes : 0);
        if (slots > 0) {
            const int rc = gemm_stream_launch(g, workspace, slots);
            if (rc) return rc;
            if (defer && pending_splits) {
                *pending_splits = slots;
                return 0;
            }
            return gemm_finish_launch((const float*)workspace, slots, g.bias, g.out, mode, g.ldo, g.M, g.N, g.stream);
        }
    }
    const int BK = 64;
    const int BM = g.M > 64 ? 128 : (g.M > 32 ? 64 : 32), BN = 128;
    const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    const int k_tiles = (g.K + BK - 1) / BK;
    // Few tiles and a long K: split K so that the machine is full (two blocks a CU for the small tiles
    // of decode, one for tiles of 128 rows); every split keeps at least 4 steps (8 for the large tiles).
    int splits = 1;
    const int want_blocks = g.M <= 64 ? 512 : 256, least_steps = g.M <= 64 ? 4 : 8;
    if (tiles < want_blocks) {
        splits = (want_blocks + tiles - 1) / tiles;
        const int most = k_tiles / least_steps > 0 ? k_tiles / least_steps : 1;
        if (splits > most) splits = most;
        const size_t per_split = (size_t)g.M * g.N * sizeof(float);
        if (workspace == nullptr || per_split == 0) splits = 1;
        else if ((size_t)splits * per_split > workspace_bytes) splits = (int)(workspace_bytes / per_split);
        if (splits < 1) splits = 1;
    }
    int k_per_split = ((k_tiles + splits - 1) / splits) * BK;
    splits = (g.K + k_per_split - 1) / k_per_split;
    const int kmode = splits > 1 ? OUT_PARTIAL : mode;
    void* kout = splits > 1 ? workspace : g.out;
    int rc;
    // Long prompts: tiles of 256 rows fed by direct loads into LDS, if the rows they waste past M
    // cost less than they gain (they run about a quarter faster than the 128 x 128 tiles).
    const int rows256 = (g.M + 255) / 256 * 256, rows128 = (g.M + 127) / 128 * 128;
    const bool rows_ok = BM == 128 && g.K % 64 == 0 && g.lda < (1 << 22) && g.ldw < (1 << 22) &&
                         (size_t)rows256 * 100 <= (size_t)rows128 * 128;
    const bool dma_ok = rows_ok && splits == 1 &&
                        (g.out_dtype != HFA_BF16 || (g.ldo % 8 == 0 && g.N % 16 == 0 && ((uintptr_t)g.out & 15) == 0));
    const int tiles256 = (rows256 / 256) * ((g.N + 255) / 256);
    // A narrow output has too few 256 x 256 tiles for the CUs: K is cut into as many parts as give
    // every CU a block (at most one round of blocks, parts of 512 columns at least) and the parts' sums
    // go to the workspace, if it holds them; otherwise tiles of 256 x 128 or the tiles of 128 rows.
    int parts = 0, part_k = 0;
    if (rows_ok && tiles256 < 128 && mode != OUT_SWIGLU && workspace != nullptr) {
        parts = 256 / tiles256;
        if (parts > g.K / 512) parts = g.K / 512;
        while (parts > 1 && (size_t)parts * g.M * g.N * sizeof(float) > workspace_bytes) parts--;
        if (parts >= 2) {
            part_k = ((g.K / 32 + parts - 1) / parts) * 32;
            parts = (g.K + part_k - 1) / part_k;
        }
    }
    // One row of tiles (up to 256 rows): tiles of 256 x 128, and as many parts of K as make the sum of two costs
    // least: the product itself, which takes the longer the fewer CUs have a block, and the planes of partial
    // sums, which are written and read again (measured at 256 rows on the 7B shape: about 4 us for a part of
    // q/k/v, 3.3 for o and down, that is 2.2 TB/s; q/k/v 37 to 29 us, o 31 to 26, down 70 to 63).
    bool half_wide = false;
    if (parts >= 2 && rows256 == 256) {
        const int tiles128 = (g.N + 127) / 128;
        const double weights_us = (double)g.N * g.K * 2 / 5.0e6, flops_us = 2.0 * 256 * g.N * g.K / 0.95e9;
        const double product_us = weights_us > flops_us ? weights_us : flops_us;
        const double plane_us = 2.0 * g.M * g.N * sizeof(float) / 2.2e6;
        int best = 0;
        double best_us = 0;
        for (int p = 2; p <= parts && p <= g.K / 512; p++) {
            const int blocks = tiles128 * p < 256 ? tiles128 * p : 256;
            const double us = product_us * 256 / blocks + p * plane_us;
            if (best == 0 || us < best_us) best = p, best_us = us;
        }
        if (best >= 2) {
            half_wide = true;
            part_k = ((g.K / 32 + best - 1) / best) * 32;
            parts = (g.K + part_k - 1) / part_k;
        }
    }
    const bool halves = parts >= 2;
    // Tiles of 192 columns do three quarters of the work of 256 (a little less efficiently): they are
    // taken when they need fewer rounds over the CUs by more than that.
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    const int tiles192 = (rows256 / 256) * ((g.N + 191) / 192);
    const bool narrow = dma_ok && tiles256 >= 128 && mode != OUT_SWIGLU &&
                        ((tiles192 + cus - 1) / cus) * 80 < ((tiles256 + cus - 1) / cus) * 100;
    if (narrow)
        rc = launch_dma<256, 192, 32, 4, 2, 5>(g, kmode, kout, 1, g.K);
    else if (dma_ok && tiles256 >= 128)
        rc = launch_dma<256, 256, 32, 2, 4, 4>(g, kmode, kout, 1, g.K);
    else if (halves) {
        rc = half_wide ? launch_dma<256, 128, 32, 4, 2, 6>(g, OUT_PARTIAL, workspace, parts, part_k)
                       : launch_dma<256, 256, 32, 2, 4, 4>(g, OUT_PARTIAL, workspace, parts, part_k);
        if (rc) return rc;
        if (defer && pending_splits) {
            *pending_splits = parts;
            return 0;
        }
        return gemm_finish_launch((const float*)workspace, parts, g.bias, g.out, mode, g.ldo, g.M, g.N, g.stream);
    } else if (dma_ok && 2 * tiles256 >= 128)
        rc = launch_dma<256, 128, 32, 4, 2, 6>(g, kmode, kout, 1, g.K);
    else if (BM == 128)                        // eight waves a block in both: about 2 % quicker than four with twice the accumulators
        rc = launch_mode<128, 128, 64, 4, 2>(g, kmode, kout, splits, k_per_split);
    else if (BM == 64 && kmode == OUT_SWIGLU)  // a wave needs 64 columns to pair gate and up
        rc = launch_mode<64, 128, 64, 2, 2>(g, kmode, kout, splits, k_per_split);
    else if (BM == 64)
        rc = launch_mode<64, 128, 64, 2, 4>(g, kmode, kout, splits, k_per_split);
    else if (kmode == OUT_SWIGLU)
        rc = launch_mode<32, 128, 64, 1, 2>(g, kmode, kout, splits, k_per_split);
    else
        rc = launch_mode<32, 128, 64, 1, 4>(g, kmode, kout, splits, k_per_split);
    if (rc || splits == 1) return rc;
    if (defer && pending_splits) {             // the caller sums the partial results in its next kernel
        *pending_splits = splits;
        return 0;
    }
    return gemm_finish_launch((const float*)workspace, splits, g.bias, g.out, mode, g.ldo, g.M, g.N, g.stream);
}
