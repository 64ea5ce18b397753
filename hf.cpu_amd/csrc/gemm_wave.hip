// bf16 matrix product for up to 16 rows (decode), bound by the speed at which the weights stream in:
// out[m, n] = sum_k a[m, k] * w[n, k], left as partial sums in a workspace.
//
// Every wave streams by itself. The work is the list of (tile of 32 output columns, 64 columns of K) units in
// tile-major order, cut into one contiguous run per wave, eight waves a block, one block a CU: 2,048 streams,
// none of which waits for another. A wave has a ring of its own in LDS, filled by direct loads
// (global_load_lds_dwordx4: 64 lanes x 16 bytes = 8 rows of 128 bytes a request; see gemm_mfma.hip for the
// swizzled layout and the reason for the inline assembly): a unit is four requests for its 32 rows of W and one
// for the 8 rows of A, requested R units ahead. While they stream there is no barrier and no other traffic
// between the waves of a block: the only wait is the wave's own, for its oldest unit.
//
// A column tile's K range is shared by the waves whose runs touch it. The waves of a block add their parts of a
// tile together in LDS when all are done: a wave's run touches at most two tiles in part, the one it begins in and
// the one it ends in (tiles it covers whole it writes itself); it keeps the two parts in registers until its run
// is done and then puts them into its ring, which is free by then. So a tile has one partial sum per block that
// touches it. The workspace holds `slots` planes of [M][N] fp32; the blocks that work on a tile write into planes
// 0, 1, ... in the order of their numbers, and the block that owns the tile's last unit clears the planes the tile
// did not need. The sum over the planes in ascending order (by the next kernel, or by gemm_finish) is the product:
// which wave adds what, and in which order, is fixed by the sizes alone, so results are reproducible. (With a plane
// per wave the o and down products of the 7B shape left 20 planes for the norm that follows to add up, with a
// plane per block 4: the norm takes 4.9 instead of 7.0 us, rotary and cache store 4.95 instead of 6.3, the
// products themselves 0.1 to 0.8 us more; a step of 8 rows 3.92 instead of 4.06 ms.)
//
// Against the product that stages tiles of 32 x 128 through LDS shared by four waves with a barrier a step
// (gemm_mfma_kernel), at 8 rows on the 7B shape: gate+up 51 against 56 us, down 24.5 against 30, q/k/v 9.5
// against 11.8, o 8.4 against 10.1. For 9 to 16 rows a unit has two requests for A: fewer bytes of W are on their
// way for the same LDS and the products are a little slower than the tiled kernel's, but the few planes make up for
// it in the kernels that follow (a step of 16 rows 4.28 against 4.40 ms). With four requests (32 rows) a step
// was slower (5.53 against 5.07 ms): those rows stay with the tiled kernel.
#include <mutex>
#include <unordered_map>

#include "common.h"
#include "gemm_internal.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));


#define WAVES 8

// First wave whose run touches unit x, when run g starts at unit floor(g * U / G).
__device__ __host__ static inline int wave_of_unit(long long x, long long U, int G) {
    return (int)(((x + 1) * G + U - 1) / U) - 1;
}

// AR: requests for A per unit (8 rows each); R: units in the ring.
template <int AR, int R>
__global__ __launch_bounds__(WAVES* WAVE) void gemm_wave_kernel(const uint16_t* __restrict__ A, int lda,
                                                               const uint16_t* __restrict__ W, int ldw,
                                                               float* __restrict__ partial, int M, int N, int nk, int tiles,
                                                               int slots) {
    constexpr int UNIT = (4 + AR) * 512;                     // elements of a unit in the ring (1 KB a request)
    constexpr int LOADS = 4 + AR;
    static_assert((R - 1) * LOADS < 64, "the wait count fits the instruction's field");
    extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];
    const int lane = threadIdx.x & (WAVE - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const long long U = (long long)tiles * nk;
    const int G = gridDim.x * WAVES, g = blockIdx.x * WAVES + wave;
    const int u0 = (int)((long long)g * U / G), u1 = (int)((long long)(g + 1) * U / G);
    const int n_units = u1 - u0 > 0 ? u1 - u0 : 0;       // (the launcher sees to it that every wave has units)

    uint16_t* ring = smem + wave * (R * UNIT);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)ring;
    // Request q of a unit fills rows 8 q .. 8 q + 7 of its operand: this lane supplies row lane / 8 of the eight,
    // the 16-byte piece stored at lane % 8, which is piece (lane % 8) ^ ((row / 2) % 8) of the row. Rows past
    // the operand's last one repeat it (their results are not stored).
    uint32_t wsrc[4], wsrc_last[4], asrc[AR];
    const int rows_last = N - (tiles - 1) * 32;              // rows of W in the last tile
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int r = q * 8 + lane / 8;
        const int piece = (lane % 8) ^ ((r >> 1) & 7);
        wsrc[q] = (uint32_t)r * (uint32_t)ldw * 2u + piece * 16;
        wsrc_last[q] = (uint32_t)(r < rows_last ? r : rows_last - 1) * (uint32_t)ldw * 2u + piece * 16;
    }
#pragma unroll
    for (int q = 0; q < AR; q++) {
        const int r = q * 8 + lane / 8;
        const int piece = (lane % 8) ^ ((r >> 1) & 7);
        asrc[q] = (uint32_t)(r < M ? r : M - 1) * (uint32_t)lda * 2u + piece * 16;
    }
    auto request = [&](int u, int slot) {
        const int tile = u / nk, kt = u % nk;
        const uint16_t* wbase = W + (size_t)tile * 32 * ldw + (size_t)kt * 64;
        const uint16_t* abase = A + (size_t)kt * 64;
        const bool last = tile == tiles - 1;                 // uniform over the wave
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t dst = lds0 + (slot * UNIT + q * 512) * 2;
            const uint32_t off = last ? wsrc_last[q] : wsrc[q];
            uint64_t sbase;           // the address in registers that a scalar instruction wrote (gemm_rows.hip: hazards)
            asm volatile("s_mov_b32 m0, %1\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0" : "=&s"(sbase) : "s"(dst), "v"(off), "s"(wbase) : "m0", "memory");
        }
#pragma unroll
        for (int q = 0; q < AR; q++) {
            const uint32_t dst = lds0 + (slot * UNIT + (4 + q) * 512) * 2;
            uint64_t sbase;           // the address in registers that a scalar instruction wrote (gemm_rows.hip: hazards)
            asm volatile("s_mov_b32 m0, %1\n\ts_mov_b64 %0, %3\n\tglobal_load_lds_dwordx4 %2, %0" : "=&s"(sbase) : "s"(dst), "v"(asrc[q]), "s"(abase) : "m0", "memory");
        }
    };
    // piece offsets (in elements) of the 16-column steps of a unit for this lane's row (rows differ from lane % 32
    // by multiples of 32 at most, so their swizzle is the lane's)
    int piece_off[4];
#pragma unroll
    for (int j = 0; j < 4; j++) piece_off[j] = ((2 * j + (lane >> 5)) ^ ((lane >> 1) & 7)) * 8;
    const int row = lane & 31;
    const bool has_a = row < 8 * AR;                          // this lane's row of A exists in the ring

    // Parts of tiles that this wave shares with others (at most two: the end of the tile it began in, the
    // beginning of the tile it ends in) stay in registers until its run is done, then go into its ring, which
    // is free by then: two records a wave of 4 AR floats a lane. Their tags lie behind the rings: the tile's
    // number (-1: unused) and whether the part holds the tile's last unit.
    int* seg_tile = reinterpret_cast<int*>(smem + WAVES * R * UNIT);
    int* seg_ends = seg_tile + 2 * WAVES;
    auto store_rows = [&](float* plane, int tile, const float* v) {     // a lane's 4 AR values of a tile into a plane
        const int c = tile * 32 + row;
        if (c < N) {
#pragma unroll
            for (int r = 0; r < 4 * AR; r++) {
                const int m = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m < M) plane[(size_t)m * N + c] = v[r];
            }
        }
    };
    auto clear_from = [&](int tile, int from) {                         // planes the tile did not need
        const int c = tile * 32 + row;
        if (c < N) {
#pragma unroll
            for (int r = 0; r < 4 * AR; r++) {
                const int m = 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                if (m < M)
                    for (int sl = from; sl < slots; sl++) partial[((size_t)sl * M + m) * N + c] = 0.f;
            }
        }
    };

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
    for (int p = 0; p < R; p++)
        if (p < n_units) request(u0 + p, p);
    int slot = 0, tile = n_units > 0 ? u0 / nk : 0, kt = n_units > 0 ? u0 % nk : 0;
    int kt_first = kt;                                                  // where this wave began the tile
    float head[4 * AR], tail[4 * AR];                                   // the two parts and their tiles (-1: none)
    int head_tile = -1, tail_tile = -1;
#pragma unroll
    for (int r = 0; r < 4 * AR; r++) head[r] = tail[r] = 0.f;
    for (int u = 0; u < n_units; u++) {
        // the unit has landed when at most the R - 1 newer units' requests are out (at the run's end fewer are
        // out than that: then all are waited for, which by then are on their way anyway)
        if (u + R <= n_units)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((R - 1) * LOADS) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const uint16_t* base = ring + slot * UNIT;
        bf16x8 fw[4], fa[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            fw[j] = *reinterpret_cast<const bf16x8*>(base + row * 64 + piece_off[j]);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (has_a) v = *reinterpret_cast<const uint4*>(base + 2048 + row * 64 + piece_off[j]);
            fa[j] = __builtin_bit_cast(bf16x8, v);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[j], fw[j], acc, 0, 0, 0);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the fragments are read: the slot may be filled again
        if (u + R < n_units) request(u0 + u + R, slot);
        slot = slot + 1 < R ? slot + 1 : 0;
        // The tile's last unit, or this wave's: element r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4,
        // column lane % 32 of the tile. A tile that this wave covered whole goes to plane 0.
        if (kt == nk - 1 || u == n_units - 1) {
            if (kt_first == 0 && kt == nk - 1) {
                float v[4 * AR];
#pragma unroll
                for (int r = 0; r < 4 * AR; r++) v[r] = acc[r];
                store_rows(partial, tile, v);
                clear_from(tile, 1);
            } else if (kt == nk - 1) {                         // the end of a tile that another wave began
#pragma unroll
                for (int r = 0; r < 4 * AR; r++) head[r] = acc[r];
                head_tile = tile;
            } else {                                           // the beginning of a tile that another wave ends
#pragma unroll
                for (int r = 0; r < 4 * AR; r++) tail[r] = acc[r];
                tail_tile = tile;
            }
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0.f;
            kt_first = 0;
        }
        if (++kt == nk) { kt = 0; tile++; }
    }
    // all requests of this wave have landed and its fragments are read: the ring takes the records
    float4* mine_rec = reinterpret_cast<float4*>(ring);
    {
        const float* first = head_tile >= 0 ? head : tail;    // the records in the order of their tiles
        const int t0 = head_tile >= 0 ? head_tile : tail_tile, t1 = head_tile >= 0 ? tail_tile : -1;
#pragma unroll
        for (int i = 0; i < AR; i++) {
            mine_rec[lane * AR + i] = make_float4(first[4 * i], first[4 * i + 1], first[4 * i + 2], first[4 * i + 3]);
            mine_rec[(WAVE + lane) * AR + i] = make_float4(tail[4 * i], tail[4 * i + 1], tail[4 * i + 2], tail[4 * i + 3]);
        }
        if (lane == 0) {
            seg_tile[2 * wave] = t0;
            seg_ends[2 * wave] = head_tile >= 0;
            seg_tile[2 * wave + 1] = t1;
            seg_ends[2 * wave + 1] = 0;
        }
    }
    __syncthreads();
    // The records in the order of the waves; those of one tile are neighbours. The wave that holds the first of
    // a tile's records adds them up in that order and writes the block's plane of the tile. Every lane reads one
    // record's tags, and all records are asked for at once: a loop over the tile's records would be a chain of
    // LDS round trips at the very end of the kernel.
    const int tag = seg_tile[lane & (2 * WAVES - 1)], tag_ends = seg_ends[lane & (2 * WAVES - 1)];
    float4 rec[2 * WAVES][AR];
#pragma unroll
    for (int k = 0; k < 2 * WAVES; k++)
#pragma unroll
        for (int i = 0; i < AR; i++)
            rec[k][i] = reinterpret_cast<const float4*>(smem + (k / 2) * (R * UNIT))[((k % 2) * WAVE + lane) * AR + i];
    for (int j = 0; j < 2; j++) {
        const int q = 2 * wave + j, t = __builtin_amdgcn_readlane(tag, q);
        if (t < 0) continue;
        int before = q - 1;
        while (before >= 0 && __builtin_amdgcn_readlane(tag, before) < 0) before--;
        if (before >= 0 && __builtin_amdgcn_readlane(tag, before) == t) continue;      // another wave leads this tile
        float v[4 * AR];
#pragma unroll
        for (int r = 0; r < 4 * AR; r++) v[r] = 0.f;
        bool ends = false;
#pragma unroll
        for (int k = 0; k < 2 * WAVES; k++) {
            if (__builtin_amdgcn_readlane(tag, k) != t) continue;                        // uniform over the wave
#pragma unroll
            for (int i = 0; i < AR; i++) {
                v[4 * i] += rec[k][i].x;
                v[4 * i + 1] += rec[k][i].y;
                v[4 * i + 2] += rec[k][i].z;
                v[4 * i + 3] += rec[k][i].w;
            }
            ends = ends || __builtin_amdgcn_readlane(tag_ends, k) != 0;
        }
        const int mine = (int)blockIdx.x - wave_of_unit((long long)t * nk, U, G) / WAVES;
        store_rows(partial + (size_t)mine * M * N, t, v);
        if (ends) clear_from(t, mine + 1);
    }
}

static int wave_cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

// Eight waves a block. Four where eight leave a wave only three or four units (q/k/v and o of the 7B shape), which
// halves the planes of partial sums that the next kernel reads, was slower a step (4.08 against 4.06 ms at 8 rows).

// The number of workspace planes a product of this shape needs (the most blocks that touch one tile), or 0 if
// this kernel does not take it.
int gemm_wave_slots(const GemmArgs& g, size_t workspace_bytes) {
    if (g.M > 16 || g.K % 64 != 0 || g.lda >= (1 << 22) || g.ldw >= (1 << 22) || g.N < 32) return 0;
    const long long nk = g.K / 64, tiles = (g.N + 31) / 32, U = tiles * nk;
    const int G = wave_cu_count() * WAVES;
    if (U < G) return 0;                                     // fewer units than waves: the tiled kernel's splits do as well
    // the walk over the tiles is remembered per shape (a decode step asks for the same few shapes every time)
    static std::mutex lock;
    static std::unordered_map<unsigned long long, int> known;
    const unsigned long long key = ((unsigned long long)tiles << 32) | (unsigned long long)nk;
    int slots = 0;
    {
        std::lock_guard<std::mutex> hold(lock);
        auto it = known.find(key);
        if (it != known.end()) slots = it->second;
    }
    if (slots == 0) {
        slots = 1;
        for (long long t = 0; t < tiles; t++) {
            const int n = wave_of_unit(t * nk + nk - 1, U, G) / WAVES - wave_of_unit(t * nk, U, G) / WAVES + 1;
            if (n > slots) slots = n;
        }
        std::lock_guard<std::mutex> hold(lock);
        known[key] = slots;
    }
    if (slots > 64 || (size_t)slots * g.M * g.N * sizeof(float) > workspace_bytes) return 0;
    return slots;
}

template <int AR, int R>
static int launch_wave(const GemmArgs& g, float* partial, int slots) {
    constexpr int SMEM = WAVES * R * (4 + AR) * 1024 + 4 * WAVES * 4;   // rings, the records' tags
    static_assert(SMEM <= 160 * 1024, "the rings must fit into a CU's LDS");
    auto kernel = gemm_wave_kernel<AR, R>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) {
            hfa_set_error("gemm_wave: cannot reserve %d bytes of LDS: %s", SMEM, hipGetErrorString(e));
            return 2;
        }
        configured = true;
    }
    kernel<<<wave_cu_count(), WAVES * WAVE, SMEM, g.stream>>>((const uint16_t*)g.a, g.lda, (const uint16_t*)g.w, g.ldw, partial,
                                                             g.M, g.N, g.K / 64, (g.N + 31) / 32, slots);
    HFA_LAUNCH_CHECK("gemm_wave");
    return 0;
}

int gemm_wave_launch(const GemmArgs& g, void* workspace, int slots) {
    return g.M <= 8 ? launch_wave<1, 3>(g, (float*)workspace, slots) : launch_wave<2, 3>(g, (float*)workspace, slots);
}
