// bf16 matrix product for few rows (decode), bound by the speed at which the weights stream in:
// out[m, n] = sum_k a[m, k] * w[n, k] with 32 < M <= 128 (tiles of 64 or 128 rows), left as partial sums
// in a workspace.
//
// The work is the list of (column tile, 64 columns of K) units in tile-major order, cut into
// one contiguous run of units per block, one block per CU: no CU waits for a last, partly filled
// round of tiles, however the number of tiles relates to the number of CUs. A block streams the
// units of its run through a ring of LDS stages filled by direct loads (global_load_lds_dwordx4,
// see gemm_mfma.hip for the layout and the reason for the inline assembly): requests run
// STAGES - 1 units ahead and do not stop at the end of a column tile; only the accumulators do,
// they are written out and cleared there.
//
// A column tile's K range may be shared by several blocks. The workspace holds `slots` planes
// of [M][N] fp32; the blocks that work on a tile write their sums into planes 0, 1, ... in the
// order of their block ids, and the block that owns the tile's last unit clears the planes the
// tile did not need. The sum over the planes in ascending order (by the next kernel, or by
// gemm_finish) is the product: which block adds what is fixed by the sizes alone, so results
// are reproducible.
#include "common.h"
#include "gemm_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int BM, int BN, int WM, int WN>
struct StreamCfg {
    static constexpr int BK = 64;
    static constexpr int NW = WM * WN, NT = NW * WAVE;
    static constexpr int ROWS = BM + BN;
    static constexpr int STAGE_BYTES = ROWS * BK * 2;
    static constexpr int LOADS = ROWS / 8 / NW;              // requests per wave and unit (8 rows of 128 bytes each)
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int FM = TM / 32, FN = TN / 32;
    static constexpr int STEPS = BK / 16;
    static constexpr int PRODUCTS = FM * FN * STEPS;         // matrix instructions per unit and wave
    static_assert(ROWS % (8 * NW) == 0 && BM % 8 == 0, "rows must spread evenly over the waves");
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tiles are made of 32x32x16 products");
};

// First block whose run touches unit x, when run b starts at unit floor(b * U / G).
__device__ __host__ static inline int stream_block_of(long long x, long long U, int G) {
    return (int)(((x + 1) * G + U - 1) / U) - 1;
}

template <int BM, int BN, int WM, int WN, int STAGES>
__global__ __launch_bounds__(WM* WN* WAVE) void gemm_stream_kernel(
    const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ W, int ldw, float* __restrict__ partial,
    int M, int N, int nk, int tiles_n, int slots) {
    using C = StreamCfg<BM, BN, WM, WN>;
    static_assert(STAGES >= 3, "one unit in use, the next one landed, one arriving");
    extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int wm = wave / WN, wn = wave % WN;
    const long long U = (long long)tiles_n * nk;
    const int G = gridDim.x, b = blockIdx.x;
    const int u0 = (int)((long long)b * U / G), u1 = (int)((long long)(b + 1) * U / G);
    if (u0 >= u1) return;

    floatx16 acc[C::FM][C::FN];
#pragma unroll
    for (int i = 0; i < C::FM; i++)
#pragma unroll
        for (int j = 0; j < C::FN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // Request i of this wave fills rows (i * NW + wave) * 8 .. + 8 of a stage: rows 0 .. BM - 1 are
    // A's (rows past M repeat the last one), the others W's rows of the unit's column tile. This
    // lane supplies row lane / 8 of the eight, the 16-byte piece stored at lane % 8, which is
    // piece (lane % 8) ^ ((row / 2) % 8) of the row (see the swizzle in gemm_mfma.hip).
    uint32_t src[C::LOADS];
#pragma unroll
    for (int i = 0; i < C::LOADS; i++) {
        const int r = (i * C::NW + wave) * 8 + lane / 8;
        const int piece = (lane % 8) ^ ((r >> 1) & 7);
        if ((i * C::NW + wave) * 8 < BM)
            src[i] = (uint32_t)(r < M - 1 ? r : M - 1) * (uint32_t)lda * 2u + piece * 16;
        else
            src[i] = (uint32_t)(r - BM) * (uint32_t)ldw * 2u + piece * 16;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)smem;
    int req_tile = u0 / nk, req_kt = u0 % nk;                // the next unit to request
    auto request = [&](int i, int stage) {                   // i is a constant after unrolling
        const uint32_t dst = lds0 + stage * C::STAGE_BYTES + (i * C::NW + wave) * 1024;
        const bool is_a = (i * C::NW + wave) * 8 < BM;       // uniform over the wave
        const uint16_t* base = is_a ? A + (size_t)req_kt * C::BK : W + (size_t)req_tile * BN * ldw + (size_t)req_kt * C::BK;
        uint64_t sbase;           // the address in registers that a scalar instruction wrote (gemm_rows.hip: hazards)
        asm volatile("s_mov_b32 m0, %1\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0" : "=&s"(sbase) : "s"(dst), "v"(src[i]), "s"(base) : "m0");
    };
    auto requested = [&]() {
        if (++req_kt == nk) { req_kt = 0; req_tile++; }
    };
    int piece_off[C::STEPS];
#pragma unroll
    for (int j = 0; j < C::STEPS; j++) piece_off[j] = ((2 * j + (lane >> 5)) ^ ((lane >> 1) & 7)) * 8;
    auto fragments = [&](int stage, int j, bf16x8 (&fa)[C::FM], bf16x8 (&fw)[C::FN]) {
        const uint16_t* sa = smem + stage * (C::STAGE_BYTES / 2) + (wm * C::TM + (lane & 31)) * C::BK + piece_off[j];
        const uint16_t* sw = smem + stage * (C::STAGE_BYTES / 2) + (BM + wn * C::TN + (lane & 31)) * C::BK + piece_off[j];
#pragma unroll
        for (int i = 0; i < C::FM; i++) fa[i] = *reinterpret_cast<const bf16x8*>(sa + i * 32 * C::BK);
#pragma unroll
        for (int i = 0; i < C::FN; i++) fw[i] = *reinterpret_cast<const bf16x8*>(sw + i * 32 * C::BK);
    };

    // The pipeline is gemm_dma_kernel's, over units instead of one tile's steps of K: units
    // u0 .. u0 + STAGES - 2 are requested up front; step u begins with a wait and a barrier after
    // which unit u + 1 has landed for every wave and every wave is done with unit u - 1, whose
    // stage unit u + STAGES - 1 is then requested into, between the matrix instructions.
    const int n_units = u1 - u0;
#pragma unroll
    for (int p = 0; p < STAGES - 1; p++)
        if (p < n_units) {
#pragma unroll
            for (int i = 0; i < C::LOADS; i++) request(i, p);
            requested();
        }
    if (n_units >= STAGES - 1)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(C::LOADS * (STAGES - 2)) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    bf16x8 fa[2][C::FM], fw[2][C::FN];
    fragments(0, 0, fa[0], fw[0]);
    constexpr int AHEAD = STAGES - 1;
    int stage = 0, tile = u0 / nk, kt = u0 % nk;
    for (int u = 0; u < n_units; u++) {
        if (u + STAGES - 2 < n_units)
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(C::LOADS * (STAGES - 3)) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const bool more = u + AHEAD < n_units;
        const int into = stage + AHEAD < STAGES ? stage + AHEAD : stage + AHEAD - STAGES;
        const int next = stage + 1 < STAGES ? stage + 1 : 0;
        int done = 0;
#pragma unroll
        for (int j = 0; j < C::STEPS; j++) {
            if (j + 1 < C::STEPS)
                fragments(stage, j + 1, fa[(j + 1) & 1], fw[(j + 1) & 1]);
            else if (u + 1 < n_units)
                fragments(next, 0, fa[0], fw[0]);
#pragma unroll
            for (int i = 0; i < C::FM; i++)
#pragma unroll
                for (int jj = 0; jj < C::FN; jj++) {
                    acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[j & 1][i], fw[j & 1][jj], acc[i][jj], 0, 0, 0);
                    done++;                                  // the requests are dealt evenly among the products
#pragma unroll
                    for (int q = (done - 1) * C::LOADS / C::PRODUCTS; q < done * C::LOADS / C::PRODUCTS; q++)
                        if (more) request(q, into);
                }
        }
        if (more) requested();
        stage = next;
        // The tile's last unit, or this block's: the sums go to the block's plane of the workspace.
        if (kt == nk - 1 || u == n_units - 1) {
            const int first = stream_block_of((long long)tile * nk, U, G);
            float* plane = partial + (size_t)(b - first) * M * N;
#pragma unroll
            for (int i = 0; i < C::FM; i++)
#pragma unroll
                for (int jj = 0; jj < C::FN; jj++) {
                    const int col = tile * BN + wn * C::TN + jj * 32 + (lane & 31);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int row = wm * C::TM + i * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                        if (row < M) {
                            plane[(size_t)row * N + col] = acc[i][jj][r];
                            if (kt == nk - 1)                // planes that this tile did not need
                                for (int s = b - first + 1; s < slots; s++) partial[((size_t)s * M + row) * N + col] = 0.f;
                        }
                        acc[i][jj][r] = 0.f;
                    }
                }
        }
        if (++kt == nk) { kt = 0; tile++; }
    }
}

static int cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

template <int BM, int BN, int WM, int WN, int STAGES>
static int launch_stream(const GemmArgs& g, float* partial, int blocks, int slots) {
    using C = StreamCfg<BM, BN, WM, WN>;
    constexpr int SMEM = STAGES * C::STAGE_BYTES;
    static_assert(SMEM <= 160 * 1024, "the stages must fit into a CU's LDS");
    static_assert(C::LOADS * (STAGES - 2) < 64, "the wait counts fit the instruction's field");
    auto kernel = gemm_stream_kernel<BM, BN, WM, WN, STAGES>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) {
            hfa_set_error("gemm_stream: cannot reserve %d bytes of LDS: %s", SMEM, hipGetErrorString(e));
            return 2;
        }
        configured = true;
    }
    kernel<<<blocks, C::NT, SMEM, g.stream>>>((const uint16_t*)g.a, g.lda, (const uint16_t*)g.w, g.ldw, partial, g.M, g.N,
                                             g.K / C::BK, g.N / BN, slots);
    HFA_LAUNCH_CHECK("gemm_stream");
    return 0;
}

// The number of workspace planes a product of this shape needs, or 0 if this kernel does not take it.
int gemm_stream_slots(const GemmArgs& g, size_t workspace_bytes) {
    const int BN = 128, BK = 64;
    // Up to 32 rows the tiles of gemm_mfma_kernel, several blocks to a CU, stream as fast.
    if (g.M <= 32 || g.M > 128 || g.K % BK != 0 || g.N % BN != 0 || g.lda >= (1 << 22) || g.ldw >= (1 << 22)) return 0;
    const long long nk = g.K / BK, tiles = g.N / BN, U = tiles * nk;
    const int G = cu_count();
    // Enough tiles for whole-tile kernels; or runs so short (under 16 units a block) that filling and
    // draining the stages outweighs the even cut: the split-K kernel is quicker there (q/k/v and o of
    // the 7B shape: 12 us against 14).
    if (tiles >= 2 * G || U < 16 * G) return 0;
    const long long per_block = U / G;                       // the shortest run
    const int slots = (int)((nk + per_block - 1) / per_block) + 1;
    if ((size_t)slots * g.M * g.N * sizeof(float) > workspace_bytes) return 0;
    return slots;
}

// Eight waves a block, each with one or two 32 x 32 accumulators a row of tiles: with two waves on
// a SIMD one reads its fragments while the other multiplies (four waves with twice the
// accumulators took 8 % longer at 65 rows, 4 % at 128 and 2 % at 64).
int gemm_stream_launch(const GemmArgs& g, void* workspace, int slots) {
    if (g.M > 64) return launch_stream<128, 128, 4, 2, 4>(g, (float*)workspace, cu_count(), slots);
    return launch_stream<64, 128, 2, 4, 6>(g, (float*)workspace, cu_count(), slots);
}
