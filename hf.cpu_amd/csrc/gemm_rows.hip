// bf16 matrix product for up to 32 rows (decode) in which every block owns a range of outputs and finishes
// them itself: out[m, n] = sum_k a[m, k] * w[n, k] over the whole of K inside one block, so no partial sums
// leave the kernel and what usually follows a product in a decode step happens in its last lines:
//
//   HFA_ROWS_OUT     out[m, n] = r[m] * sum + bias[n]                        (fp32 or bf16)
//   HFA_ROWS_RESID   x[m, n] += sum + bias[n]; the block's share of sum_n x[m, n]^2; xg[m, n] = bf16(x[m, n] * g[n])
//   HFA_ROWS_SWIGLU  act[m, f] = bf16(silu(r[m] * sum_gate) * (r[m] * sum_up))   (w's rows in blocks of 32 gate, 32 up)
//
// r[m] = rsqrt(sum_n x[m, n]^2 / width + eps) from the shares that a HFA_ROWS_RESID product left: an RMS norm
// between two products costs no kernel and no pass over memory. The product that completes the residual stream
// multiplies it by the norm's weight (xg), the product that reads it scales its sums by r. Rounding differs from
// norm-then-product only in where the one rounding to bf16 falls (x g instead of x r g; r is a factor of the sum).
//
// One block a CU, eight waves. Block b owns outputs [b N / G, (b + 1) N / G): G equal shares of the weights'
// rows, each a contiguous piece of memory. The waves of a block split K: wave w takes the units of 128 columns
// w, w + 8, ..., and for each of them all the block's tiles of 16 rows, so at any time the block reads a few KB
// of each of its rows side by side. A wave streams by itself: units of (16 rows, 128 columns) = 4 KB go from
// memory into its own ring in LDS by direct loads (global_load_lds_dwordx4: 64 lanes x 16 bytes = 8 rows of 128
// bytes a request, rows swizzled so that the fragment reads are conflict-free), R units ahead, with no barrier
// and no traffic between the waves while they stream. The activations of a unit of K (16 rows x 128 columns,
// rows past the last one repeated; from 17 rows up two such tiles, MT = 2) go from L2 straight into registers, requested together with the first tile of
// that unit of K, so the order of all requests of a wave is fixed by the sizes alone and every wait names a count
// that is known when the kernel is compiled. v_mfma_f32_16x16x32_bf16: tokens are the rows of the product, the
// weights' rows its columns. At the end the waves' sums meet in LDS (in the rings, free by then) and are added in
// the order of the waves; the block's threads finish the outputs. Which wave adds what, and in which order, is
// fixed by the sizes: results are reproducible and a row does not depend on the other rows of the batch.
//
// Against the products that leave partial sums (gemm_wave.hip) on the 7B shape at 8 rows, each timed alone:
// gate+up with the activation 52.6 us (there 51 + 4.7 for the kernel that adds up and applies the activation),
// down 29.7 (24.5 + the sums in the norm that follows), q/k/v 12.0 (9.5), o 9.3 (8.4): the products themselves
// are no faster, the kernels between them are gone.
#include "api.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define RG_WAVES 8
#define RG_R 4                 // units in a wave's ring
#define RG_UNIT 2048           // elements of a unit: 16 rows x 128 columns of K (4 KB)
#define RG_RING_FLOATS (RG_R * RG_UNIT / 2)

struct RowGemm {
    const uint16_t* A; int lda;            // activations, bf16 [T][K]
    const uint16_t* W; int ldw;            // weights, bf16 [rows][K]
    int T, N, K;                           // N: outputs (features for SWIGLU)
    const float* bias;                     // [N] or null
    const float* ssq_in; int parts_in;     // [parts_in][16 or 32] shares of the sums of squares of the normed rows (32 from 17 rows up), or null
    float inv_width, eps;                  // r[m] = rsqrt(sum * inv_width + eps)
    void* out; int ldo; int out_bf16;      // OUT
    float* x; int ldx; float* ssq_out;     // RESID: residual stream; [gridDim.x][16 or 32] shares of the sums of squares
    const float* g; uint16_t* xg; int ldxg;   // RESID: the next norm's weight and x * g in bf16 (or null)
    uint16_t* act; int ldact;              // SWIGLU
};

// The requests below are written in assembly, and the compiler does not look into assembly for the machine's hazards.
// One matters here: a memory instruction may read a scalar register no sooner than five wait states after a VECTOR
// instruction wrote it (v_readlane, when the compiler brings back a scalar that it had put aside in the lanes of a
// vector register; v_readfirstlane), and nothing makes the compiler keep that distance from a statement it cannot
// read. So no memory instruction here reads a scalar operand of the statement: a scalar move copies it first (scalar
// instructions wait for vector ones by themselves, and what a scalar instruction wrote may be read at once).
//
// A lane's 16 bytes of each of the four 32-column steps of a unit of K, straight into registers. The compiler takes
// the registers as written when the statement ends: whoever uses them waits for the loads first and then passes
// them through rg_landed.
__device__ __forceinline__ void rg_load_a(u32x4 (&f)[4], uint32_t off, const uint16_t* base) {
    uint64_t b;
    asm volatile("s_mov_b64 %4, %6\n\t"
                 "global_load_dwordx4 %0, %5, %4\n\t"
                 "global_load_dwordx4 %1, %5, %4 offset:64\n\t"
                 "global_load_dwordx4 %2, %5, %4 offset:128\n\t"
                 "global_load_dwordx4 %3, %5, %4 offset:192"
                 : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3]), "=&s"(b) : "v"(off), "s"(base) : "memory");
}
// Four requests: 16 rows x 128 columns of K into 4 KB of LDS at dst (rows 0-7 and 8-15 of the first 64 columns, then
// of the second 64): 64 lanes x 16 bytes = 8 rows of 128 bytes a request, to M0 + 16 * lane. (An `offset:` on the
// instruction would move the place in LDS as well as the address, so the second half has a base of its own.)
__device__ __forceinline__ void rg_request(const uint16_t* base, uint32_t off0, uint32_t off1, uint32_t dst) {
    const uint16_t* base1 = base + 64;
    uint64_t b0, b1;
    asm volatile("s_mov_b32 m0, %2\n\ts_mov_b64 %0, %5\n\ts_mov_b64 %1, %6\n\t"
                 "global_load_lds_dwordx4 %3, %0\n\t"
                 "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %0\n\t"
                 "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %1\n\t"
                 "s_add_u32 m0, m0, 0x400\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %1"
                 : "=&s"(b0), "=&s"(b1) : "s"(dst), "v"(off0), "v"(off1), "s"(base), "s"(base1) : "m0", "scc", "memory");
}
__device__ __forceinline__ void rg_landed(u32x4 (&f)[4]) { asm volatile("" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3])); }

template <int V> struct rg_int { static constexpr int value = V; };
template <int I, int N, typename F>
__device__ __forceinline__ void rg_static_for(F&& f) {
    if constexpr (I < N) {
        f(rg_int<I>{});
        rg_static_for<I + 1, N>(f);
    }
}

template <int N>
__device__ __forceinline__ void rg_wait() {                  // at most N requests may still be on their way
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 63 ? N : 63) : "memory");
}

// Requests newer than those of unit u when it is waited for, in the steady state: the R - 1 units after it, four
// requests each, and 4 MT more for every one of them that begins a unit of K (it brings that unit's activations).
template <int NT, int TT, int MT>
constexpr int rg_newer() {
    int n = 0;
    for (int j = 1; j < RG_R; j++) n += 4 + ((TT + j) % NT == 0 ? 4 * MT : 0);
    return n;
}

__device__ __forceinline__ uint16_t rg_bf16(float v) { return bf16_bits(v); }

// NT: tiles of 16 weight rows a wave accumulates at a time (even for SWIGLU: gate and up tiles alternate);
// AD: register sets of activations (units of K that may be on their way or in use at once); MT: tiles of 16 rows of
// activations (1 for up to 16 rows, 2 for up to 32: every unit of weights that has come through LDS is then used twice).
template <int NT, int AD, int MODE, int MT>
__global__ __launch_bounds__(RG_WAVES * WAVE) void gemm_rows_kernel(const RowGemm p) {
    extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];
    constexpr int MR = 16 * MT;                                            // rows of activations the kernel holds
    __shared__ float r_s[MR];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = gridDim.x, b = blockIdx.x;
    const int own0 = (int)((long long)b * p.N / G), own1 = (int)((long long)(b + 1) * p.N / G);
    const int n_own = own1 - own0;
    const int ft_all = (n_own + 15) / 16;                                  // tiles of 16 outputs
    const int nt_all = MODE == HFA_ROWS_SWIGLU ? 2 * ft_all : ft_all;      // tiles of 16 weight rows
    const int nku = p.K / 128;
    const int nkw = nku > wave ? (nku - wave + RG_WAVES - 1) / RG_WAVES : 0;   // this wave's units of K: wave, wave + 8, ...

    uint16_t* ring = smem + wave * (RG_R * RG_UNIT);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t*)ring;
    // a request fills 8 rows x 128 bytes: this lane supplies row lane / 8 of the eight, the 16-byte piece that is
    // stored at lane % 8, which is piece (lane % 8) ^ ((row / 2) % 8) of the row's 128 bytes
    int req_row[2];
    uint32_t req_piece[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        req_row[h] = h * 8 + lane / 8;
        req_piece[h] = (uint32_t)(((lane % 8) ^ ((req_row[h] >> 1) & 7)) * 16);
    }
    // fragment reads: row lane % 16, step s: half s / 2 of the unit's columns, piece 4 (s % 2) + lane / 16
    int frag_off[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int n = lane & 15, pc = 4 * (s & 1) + (lane >> 4);
        frag_off[s] = ((s >> 1) * 16 + n) * 64 + ((pc ^ ((n >> 1) & 7)) * 8);
    }
    // the rows of A this lane reads (rows past the last one repeat it), and its 16 bytes of a 32-column step
    uint32_t a_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
        const int row = 16 * mt + (lane & 15);
        a_off[mt] = (uint32_t)(row < p.T ? row : p.T - 1) * (uint32_t)p.lda * 2u + (uint32_t)(lane >> 4) * 16u;
    }

    // What the last lines need from memory is asked for first and waited for last, so that it costs no trip of its
    // own: the shares of the sums of squares of the normed rows ([share][MR]; thread (m = tid % MR, slice = tid / MR)
    // takes the shares slice, slice + SL, ..., EARLY at most, which covers 256 shares: more are added up by the
    // compiler's own loads below), or, for the residual sum, this thread's value of the residual stream (the first
    // 512 values of the block's outputs).
    constexpr int SL = RG_WAVES * WAVE / MR, EARLY = 8 * MT;               // slices of shares; early loads a thread
    float early[EARLY];
#pragma unroll
    for (int i = 0; i < EARLY; i++) early[i] = 0.f;
    if (MODE != HFA_ROWS_RESID) {
        if (p.ssq_in) {
#pragma unroll
            for (int i = 0; i < EARLY; i++) {
                const int q = tid / MR + SL * i;
                const float* src = p.ssq_in + (q < p.parts_in ? q : 0) * MR + (tid % MR);
                asm volatile("global_load_dword %0, %1, off" : "=v"(early[i]) : "v"(src) : "memory");
            }
        }
    } else {
        const int tt = tid / (16 * MR), m = (tid >> 4) % MR, col = own0 + 16 * tt + (tid & 15);
        const float* src = p.x + (size_t)(m < p.T ? m : 0) * p.ldx + (col < own1 ? col : own0 < own1 ? own1 - 1 : 0);
        asm volatile("global_load_dword %0, %1, off" : "=v"(early[0]) : "v"(src) : "memory");
    }
    // ... and the bias and the norm's weight of this thread's first output column (MODE != SWIGLU: column
    // own0 + 16 (tid / (16 MR)) + tid % 16, the one of element tid of the first group of tiles)
    float early_b = 0.f, early_g = 0.f;
    if (MODE != HFA_ROWS_SWIGLU) {
        const int col = own0 + 16 * (tid / (16 * MR)) + (tid & 15);
        const int at = col < own1 ? col : own0 < own1 ? own1 - 1 : 0;
        if (p.bias) asm volatile("global_load_dword %0, %1, off" : "=v"(early_b) : "v"(p.bias + at) : "memory");
        if (MODE == HFA_ROWS_RESID && p.xg) asm volatile("global_load_dword %0, %1, off" : "=v"(early_g) : "v"(p.g + at) : "memory");
    }
    float ssq_run = 0.f;                                                    // RESID: thread m's sum over the groups of tiles

    for (int tg0 = 0; tg0 < nt_all; tg0 += NT) {
        const int nt = nt_all - tg0 < NT ? nt_all - tg0 : NT;      // tiles past the block's last one repeat its last row; their sums are dropped
        // byte offset of this lane's row of request half h of tile tt (of this group) from the start of W
        uint32_t wrow[NT][2];
#pragma unroll
        for (int tt = 0; tt < NT; tt++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                int row;
                if (MODE == HFA_ROWS_SWIGLU) {
                    const int t = tg0 + tt;
                    int f = own0 + 16 * (t >> 1) + req_row[h];
                    f = f < own1 ? f : own1 - 1;
                    row = (f >> 5) * 64 + (f & 31) + ((t & 1) ? 32 : 0);
                } else {
                    row = own0 + 16 * (tg0 + tt) + req_row[h];
                    row = row < own1 ? row : own1 - 1;
                }
                wrow[tt][h] = (uint32_t)row * (uint32_t)p.ldw * 2u + req_piece[h];
            }
        u32x4 af[AD][MT][4];
        // Unit (c, tt): tile tt of this wave's c-th unit of K. The unit with tt == 0 also brings the activations
        // of its unit of K, into register set `set`.
        auto issue = [&](int c, auto tt_c, auto set_c, int slot) {
            constexpr int tt = decltype(tt_c)::value, set = decltype(set_c)::value;
            rg_request(p.W + (size_t)(wave + RG_WAVES * c) * 128, wrow[tt][0], wrow[tt][1], lds0 + slot * (RG_UNIT * 2));
            if (tt == 0) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) rg_load_a(af[set][mt], a_off[mt], p.A + (size_t)(wave + RG_WAVES * c) * 128);
            }
        };
        floatx4 acc[NT][MT];
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
        const int n_units = nkw * NT;
        rg_static_for<0, RG_R>([&](auto v_c) {                   // the first R units
            constexpr int v = decltype(v_c)::value;
            if (v < n_units) issue(v / NT, rg_int<v % NT>{}, rg_int<(v / NT) % AD>{}, v);
        });
        int slot = 0;
        for (int c0 = 0; c0 < nkw; c0 += AD) {
            rg_static_for<0, AD>([&](auto cc_c) {
                constexpr int cc = decltype(cc_c)::value;
                const int c = c0 + cc;
                if (c < nkw) {
                    rg_static_for<0, NT>([&](auto tt_c) {
                        constexpr int tt = decltype(tt_c)::value;
                        const int u = c * NT + tt;
                        // the unit has landed when at most the requests of the R - 1 units after it are out; at the
                        // run's end fewer are out than that, and all of them are waited for
                        if (u + RG_R <= n_units) rg_wait<rg_newer<NT, tt, MT>()>(); else rg_wait<0>();
                        if (tt == 0) {
#pragma unroll
                            for (int mt = 0; mt < MT; mt++) rg_landed(af[cc][mt]);
                        }
                        const uint16_t* base = ring + slot * RG_UNIT;
                        bf16x8 fw[4];
#pragma unroll
                        for (int s = 0; s < 4; s++) fw[s] = *reinterpret_cast<const bf16x8*>(base + frag_off[s]);
#pragma unroll
                        for (int s = 0; s < 4; s++)
#pragma unroll
                            for (int mt = 0; mt < MT; mt++)
                                acc[tt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[cc][mt][s]), fw[s], acc[tt][mt], 0, 0, 0);
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the fragments are read: the slot may be filled again
                        if (u + RG_R < n_units)
                            issue(c + (tt + RG_R) / NT, rg_int<(tt + RG_R) % NT>{}, rg_int<(cc + (tt + RG_R) / NT) % AD>{}, slot);
                        slot = slot + 1 < RG_R ? slot + 1 : 0;
                    });
                }
            });
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (tg0 == 0) {
#pragma unroll
            for (int i = 0; i < EARLY; i++) asm volatile("" : "+v"(early[i]));     // what was asked for first has landed too
            asm volatile("" : "+v"(early_b), "+v"(early_g));
        }
        // ---- the waves' sums meet in LDS, in the rings (free by now): records of [tile][m][n] ----
        // element r of a lane's accumulator: token 16 mt + 4 (lane / 16) + r, weight row lane % 16 of the tile.
        // A record that fits a wave's own ring lies there, one a wave; larger ones (NT MT > 16) are four, and the
        // waves 4 .. 7 hand theirs to the waves 0 .. 3 first.
        constexpr bool HAND = NT * MT * 256 > RG_RING_FLOATS;
        constexpr int SUMS = HAND ? 4 : RG_WAVES, REC = HAND ? NT * MT * 256 : RG_RING_FLOATS;
        static_assert(SUMS * REC <= RG_WAVES * RG_RING_FLOATS, "the records fit into the rings");
        float* red = reinterpret_cast<float*>(smem);
        {
            float* mine = red + (HAND ? wave & 3 : wave) * REC;
            const int n = lane & 15, mg = lane >> 4;
            auto put = [&](bool add) {
#pragma unroll
                for (int tt = 0; tt < NT; tt++)
                    if (tt < nt) {
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                float* at = mine + ((tt * MR + 16 * mt + 4 * mg + r) * 16 + n);
                                *at = add ? *at + acc[tt][mt][r] : acc[tt][mt][r];
                            }
                    }
            };
            if (HAND) {
                __syncthreads();                                           // every wave is done with its ring
                if (wave >= 4) put(false);
                __syncthreads();
                if (wave < 4) put(true);
            } else {
                put(false);
            }
        }
        float* behind = reinterpret_cast<float*>(smem) + RG_WAVES * RG_RING_FLOATS;     // LDS behind the rings
        if (tg0 == 0 && MODE != HFA_ROWS_RESID) {
            // r[m] from the shares: SL slices per row, added in a fixed order
            float ssq_part = 0.f;
            if (p.ssq_in) {
#pragma unroll
                for (int i = 0; i < EARLY; i++) ssq_part += tid / MR + SL * i < p.parts_in ? early[i] : 0.f;
                for (int q = tid / MR + SL * EARLY; q < p.parts_in; q += SL) ssq_part += p.ssq_in[q * MR + (tid % MR)];
            }
            behind[tid] = ssq_part;
            __syncthreads();
            if (tid < MR) {
                float s = 0.f;
                for (int q = 0; q < SL; q++) s += behind[q * MR + tid];
                r_s[tid] = p.ssq_in ? rsqrtf(s * p.inv_width + p.eps) : 1.0f;
            }
        }
        __syncthreads();
        auto total = [&](int tt, int m, int n) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < SUMS; w++) s += red[w * REC + (tt * MR + m) * 16 + n];
            return s;
        };
        if (MODE == HFA_ROWS_OUT) {
            for (int i = tid; i < nt * 16 * MR; i += RG_WAVES * WAVE) {
                const int tt = i / (16 * MR), m = (i >> 4) % MR, n = i & 15, col = own0 + 16 * (tg0 + tt) + n;
                if (m < p.T && col < own1) {
                    const float v = r_s[m] * total(tt, m, n) + (!p.bias ? 0.f : (tg0 == 0 && i == tid) ? early_b : p.bias[col]);
                    if (p.out_bf16) reinterpret_cast<uint16_t*>(p.out)[(size_t)m * p.ldo + col] = rg_bf16(v);
                    else reinterpret_cast<float*>(p.out)[(size_t)m * p.ldo + col] = v;
                }
            }
        } else if (MODE == HFA_ROWS_SWIGLU) {
            for (int i = tid; i < (nt / 2) * 16 * MR; i += RG_WAVES * WAVE) {
                const int j = i / (16 * MR), m = (i >> 4) % MR, n = i & 15, f = own0 + 16 * (tg0 / 2 + j) + n;
                if (m < p.T && f < own1) {
                    const float gt = r_s[m] * total(2 * j, m, n), up = r_s[m] * total(2 * j + 1, m, n);
                    p.act[(size_t)m * p.ldact + f] = rg_bf16(gt / (1.0f + __expf(-gt)) * up);        // src/mathx.c:34
                }
            }
        } else {
            // the new residual values also go to LDS, for the sums of squares: [MR][NT * 16]
            for (int i = tid; i < nt * 16 * MR; i += RG_WAVES * WAVE) {
                const int tt = i / (16 * MR), m = (i >> 4) % MR, n = i & 15, col = own0 + 16 * (tg0 + tt) + n;
                float v = 0.f;
                if (m < p.T && col < own1) {
                    const float was = (tg0 == 0 && i == tid) ? early[0] : p.x[(size_t)m * p.ldx + col];
                    const bool first = tg0 == 0 && i == tid;
                    v = was + (total(tt, m, n) + (!p.bias ? 0.f : first ? early_b : p.bias[col]));
                    p.x[(size_t)m * p.ldx + col] = v;
                    if (p.xg) p.xg[(size_t)m * p.ldxg + col] = rg_bf16(v * (first ? early_g : p.g[col]));
                }
                behind[m * (NT * 16) + tt * 16 + n] = v;
            }
            __syncthreads();
            if (tid < MR) {
                float s = 0.f;
                for (int j = 0; j < nt * 16; j++) { const float v = behind[tid * (NT * 16) + j]; s += v * v; }
                ssq_run += s;
            }
        }
        __syncthreads();                                                   // the rings are requested again for the next group
    }
    if (MODE == HFA_ROWS_RESID && tid < MR) p.ssq_out[b * MR + tid] = ssq_run;
}

static int rows_cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

template <int NT, int MODE, int MT>
static int rows_launch_mt(const RowGemm& p, hipStream_t stream) {
    constexpr int AD = NT == 1 ? RG_R : (RG_R + NT - 1) / NT + 1;         // sets that may be live at once (see the kernel)
    constexpr int BEHIND = MODE == HFA_ROWS_RESID ? 16 * MT * NT * 16 * 4 : 2048;
    constexpr int SMEM = RG_WAVES * RG_R * RG_UNIT * 2 + (BEHIND > 2048 ? BEHIND : 2048);
    static_assert(SMEM <= 160 * 1024 - 64, "rings and records must fit into a CU's LDS");
    auto kernel = gemm_rows_kernel<NT, AD, MODE, MT>;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) {
            hfa_set_error("gemm_rows: cannot reserve %d bytes of LDS: %s", SMEM, hipGetErrorString(e));
            return 2;
        }
        configured = true;
    }
    kernel<<<rows_cu_count(), RG_WAVES * WAVE, SMEM, stream>>>(p);
    HFA_LAUNCH_CHECK("gemm_rows");
    return 0;
}

template <int NT, int MODE>
static int rows_launch(const RowGemm& p, hipStream_t stream) {
    if constexpr (NT <= 10) {
        if (p.T > 16) return rows_launch_mt<NT, MODE, 2>(p, stream);
    }
    return rows_launch_mt<NT, MODE, 1>(p, stream);
}

template <int MODE>
static int rows_dispatch(const RowGemm& p, hipStream_t stream) {
    const int G = rows_cu_count();
    int nt = ((p.N + G - 1) / G + 15) / 16;                  // the most tiles a block has
    if (MODE == HFA_ROWS_SWIGLU) nt *= 2;
    // tiles a wave takes at a time: few repeated tiles and few passes over K (a pass costs about what two tiles
    // cost: its own ramp, and the waves' sums meeting at its end), the larger one of equals
    const int opts[] = {1, 2, 4, 6, 8, 10, 12};
    int best = 10, best_cost = 1 << 30;
    for (int o : opts) {
        if (MODE == HFA_ROWS_SWIGLU && (o & 1)) continue;
        if (p.T > 16 && o > 10) continue;                    // (with two tiles of rows, 12 tiles of weights are more than the registers hold)
        const int cost = (nt + o - 1) / o * (o + 2);
        if (cost < best_cost || (cost == best_cost && o > best)) { best = o; best_cost = cost; }
    }
    switch (best) {
        case 1: if constexpr (MODE != HFA_ROWS_SWIGLU) return rows_launch<1, MODE>(p, stream); else return rows_launch<2, MODE>(p, stream);
        case 2: return rows_launch<2, MODE>(p, stream);
        case 4: return rows_launch<4, MODE>(p, stream);
        case 6: return rows_launch<6, MODE>(p, stream);
        case 8: return rows_launch<8, MODE>(p, stream);
        case 10: return rows_launch<10, MODE>(p, stream);
        default: return rows_launch<12, MODE>(p, stream);
    }
}

extern "C" int hfa_gemm_rows_parts(void) { return rows_cu_count(); }

extern "C" int hfa_gemm_rows_supports(int mode, int M, int N, int K, int lda, int ldw) {
    if (M < 1 || M > 32 || N < 1 || K < 128 || K % 128 != 0 || lda % 8 != 0 || ldw % 8 != 0) return 0;
    if (mode == HFA_ROWS_SWIGLU && N % 32 != 0) return 0;
    const long long rows = mode == HFA_ROWS_SWIGLU ? 2LL * N : N;
    if (rows * ldw * 2 >= (1LL << 32) || 32LL * lda * 2 >= (1LL << 32)) return 0;       // 32-bit byte offsets
    return 1;
}

extern "C" int hfa_gemm_rows(int mode, const void* a, int lda, const void* w, int ldw, int M, int N, int K,
                             const float* bias, const float* ssq_in, int parts_in, float inv_width, float eps,
                             void* out, int ldo, int out_dtype, float* x, int ldx, float* ssq_out, const float* g,
                             void* xg, int ldxg, void* act, int ldact, hipStream_t stream) {
    HFA_REQUIRE(mode == HFA_ROWS_OUT || mode == HFA_ROWS_RESID || mode == HFA_ROWS_SWIGLU, "gemm_rows: unknown mode %d", mode);
    HFA_REQUIRE(hfa_gemm_rows_supports(mode, M, N, K, lda, ldw),
                "gemm_rows: needs 1 to 32 rows, K a multiple of 128 and row strides that are multiples of 8 (M=%d N=%d K=%d lda=%d ldw=%d)",
                M, N, K, lda, ldw);
    HFA_REQUIRE(a && w && lda >= K && ldw >= K && ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0,
                "gemm_rows: operands must be 16-byte aligned with rows of at least K elements");
    HFA_REQUIRE(!ssq_in || (parts_in > 0 && parts_in <= 4096), "gemm_rows: %d shares of the sums of squares", parts_in);
    RowGemm p = {};
    p.A = (const uint16_t*)a; p.lda = lda; p.W = (const uint16_t*)w; p.ldw = ldw; p.T = M; p.N = N; p.K = K;
    p.bias = bias; p.ssq_in = ssq_in; p.parts_in = parts_in; p.inv_width = inv_width; p.eps = eps;
    if (mode == HFA_ROWS_OUT) {
        HFA_REQUIRE(out && ldo >= N && (out_dtype == HFA_F32 || out_dtype == HFA_BF16), "gemm_rows: no output, or its rows are shorter than N");
        p.out = out; p.ldo = ldo; p.out_bf16 = out_dtype == HFA_BF16;
        return rows_dispatch<HFA_ROWS_OUT>(p, stream);
    }
    if (mode == HFA_ROWS_RESID) {
        HFA_REQUIRE(x && ldx >= N && ssq_out && !ssq_in, "gemm_rows: the residual mode needs x, room for the sums of squares, and takes no row scale");
        HFA_REQUIRE(!xg || (g && ldxg >= N), "gemm_rows: x * g needs the weight g and rows of at least N elements");
        p.x = x; p.ldx = ldx; p.ssq_out = ssq_out; p.g = g; p.xg = (uint16_t*)xg; p.ldxg = ldxg;
        return rows_dispatch<HFA_ROWS_RESID>(p, stream);
    }
    HFA_REQUIRE(act && ldact >= N && !bias, "gemm_rows: the gate/up mode needs an output of N features and takes no bias");
    p.act = (uint16_t*)act; p.ldact = ldact;
    return rows_dispatch<HFA_ROWS_SWIGLU>(p, stream);
}
