// Paged softmax attention on the matrix cores (bf16 cache, fp32 scores, softmax and sums).
//
// One wave owns up to 32 "columns": the query heads of one key/value head for a few
// consecutive tokens of one request (a prompt portion: several tokens; a decoded token: one).
// The columns share every key and value they read, so grouped heads cost one pass over the
// cache. Keys are walked in blocks of 32, aligned to absolute positions:
//
//   S^T[key, col] = K[key, :] . Q[col, :]        v_mfma_f32_32x32x16_bf16, A = 32 keys x 16 dims
//                                                straight from the cache, B = queries in registers
//   online softmax per column: a column is one lane pair (l, l ^ 32), so maximum and sum need
//   one cross-lane step; the probabilities a lane holds are exactly the B operand of
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col]   A = values, which the cache keeps transposed
//                                                inside a page, so 4 consecutive keys of one
//                                                dimension are one 8-byte load.
// The order of keys inside a 16-key product is permuted the same way in both operands of the
// second product, so the probabilities never leave their registers.
//
// When a step has few columns (decode) the key range is cut into chunks over blockIdx.z; each
// wave writes (max, sum, unnormalised output) for its chunk and a second kernel merges them in
// chunk order. Keys and values come from global memory in operand layout, without a barrier.
#include "attention_internal.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define KB 32
#define PG_MAX 512
#define NEG_BIG (-1.0e30f)

// The running maximum of a column follows the scores only when they pass it by more than this (in
// powers of two): probabilities then reach 2^MAX_SLACK at most, which bf16 and the fp32 sums hold
// as exactly as values up to 1, and the accumulators are rescaled in few blocks instead of in most.
#define MAX_SLACK 8.0f

// 2^x by the hardware instruction (arguments here are at most MAX_SLACK or the -1e30 sentinel's
// difference, never subnormal results that matter).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// A column's scores lie in lanes c and c + 32. v_permlane32_swap exchanges the upper half of one
// register with the lower half of another; with the same value in both, every lane then holds
// the lower lane's value in the first and the upper lane's in the second: maximum and sum of the
// pair without a trip through LDS, and the same bits in both lanes.
__device__ __forceinline__ float pair_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Two probabilities as a pair of bf16, round to nearest even: one v_cvt_pk_bf16_f32 on gfx950.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t prob_pair(float lo, float hi) {
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

union Frag {
    uint4 u;
    uint2 h[2];
    bf16x8 v;
};

// FUSED (decoded tokens only, one token a tile): queries, the new key and the new value are not in `q` and in the
// cache yet but in `raw`, fp32 rows [q | k | v] as the product left them (bias added). The wave rotates its queries
// while it loads them (cosines and sines of the token's angles come from `cs`, [token][D / 2 cosines, D / 2 sines];
// rot_dim = D, or no rotation when cs is null); the wave whose keys include the token's own position rotates the
// new key, stores it and the new value into the cache (rows slot_map[token]) for the steps to come, and uses them
// from LDS itself, since what the cache row held before is not the token's. What rope_store would have done in a
// kernel and a pass over memory of its own.
template <int NDB, bool SPLIT, bool FUSED>
__global__ __launch_bounds__(WAVE) void attn_mfma_kernel(
    const uint16_t* __restrict__ q, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc, int kvw,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot,
    const int* __restrict__ positions, const int* __restrict__ q_start, int n_seqs, uint16_t* __restrict__ out,
    int ldo, float* __restrict__ partial, int H, int psh, int window, float scale_log2e, int tpt, int cpt,
    int chunk_keys, int n_chunks, int one_tile_each, const float* __restrict__ raw, int ld_raw,
    const float* __restrict__ cs, const int* __restrict__ slot_map, int G) {
    constexpr int D = NDB * 32, KS = D / 16;
    const int P = 1 << psh;                                // tokens per page, a power of two
    const int lane = threadIdx.x, col = lane & 31, half = lane >> 5;
    const int g = blockIdx.y, chunk = blockIdx.z;

    // ---- the tile's request and tokens: tiles are numbered request by request ----
    int tile = blockIdx.x, t0 = -1, t_end = 0;
    if (one_tile_each) {                                   // no request has more tokens than a tile: tile s is request s
        if (tile < n_seqs) {
            t0 = q_start[tile];
            t_end = q_start[tile + 1];
        }
    } else
    for (int s = 0; s < n_seqs; s++) {
        const int a = q_start[s], b = q_start[s + 1];
        const int nt = (b - a + tpt - 1) / tpt;
        if (tile < nt) {
            t0 = a + tile * tpt;
            t_end = t0 + tpt < b ? t0 + tpt : b;
            break;
        }
        tile -= nt;
    }
    if (t0 < 0) return;                                    // the grid is an upper bound on the tiles

    const int n_cols = (t_end - t0) * cpt;
    const bool col_ok = col < n_cols;
    const int my_tok = col_ok ? t0 + col / cpt : t0;
    const int my_head = g * cpt + (col_ok ? col % cpt : 0);
    const int pos = positions[my_tok];
    const int pos_first = positions[t0], hi = positions[t_end - 1];
    int k_begin = window > 0 && pos_first - window + 1 > 0 ? pos_first - window + 1 : 0;
    int k_end = hi;
    if (SPLIT) {
        k_begin = k_begin > chunk * chunk_keys ? k_begin : chunk * chunk_keys;
        k_end = k_end < (chunk + 1) * chunk_keys - 1 ? k_end : (chunk + 1) * chunk_keys - 1;
    }
    // visible keys of this lane's column: [vlo, vhi]
    int vlo = window > 0 && pos - window + 1 > k_begin ? pos - window + 1 : k_begin;
    int vhi = col_ok ? (pos < k_end ? pos : k_end) : -1;
    const int* bt = block_table + (size_t)token_slot[t0] * max_blocks;

    // The query fragments stay in registers: read from LDS one by one before each product, they
    // cost an LDS round trip a product that a single wave on its SIMD has nothing to hide behind.
    Frag qf[KS];
    __shared__ __attribute__((aligned(16))) uint16_t new_s[FUSED ? 2 * D : 8];     // the token's own key (rotated) and value
    bool owns_new = false;                                 // this wave's keys include the token's own position
    if (!FUSED) {
        const uint16_t* qp = q + (size_t)my_tok * ldq + my_head * D + half * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qf[ks].u = col_ok ? *reinterpret_cast<const uint4*>(qp + ks * 16) : make_uint4(0, 0, 0, 0);
    }
    // FUSED: called once the first blocks of keys and values are on their way, so that the trip for the 32-bit rows
    // is not a trip of its own at the head of the kernel
    auto fused_prologue = [&]() {
        // A head's fragments ks and ks + KS / 2 hold the two halves of its rotated pairs (i, i + D / 2), i = 16 ks + 8 half + e.
        // Everything a pass needs from memory is asked for before anything is computed (left alone, the compiler asks,
        // waits and computes fragment by fragment: eight trips to L2 one after the other), in two passes over the
        // fragments so that the registers suffice.
        const float* row = raw + (size_t)my_tok * ld_raw;
        const float* qsrc = row + my_head * D + half * 8;
        const float* ksrc = row + (H + g) * D + half * 8;
        const float* cp = cs ? cs + (size_t)my_tok * D + half * 8 : nullptr;
        owns_new = k_begin <= hi && hi <= k_end;            // uniform: hi is the token's own position
        const int slot = owns_new ? slot_map[my_tok] : 0;
        float vraw[NDB];
        if (owns_new && half == 0) {
#pragma unroll
            for (int db = 0; db < NDB; db++) vraw[db] = row[(H + G) * D + g * D + 32 * db + col];
        }
        // (x0, x1) -> (x0 c - x1 s, x0 s + x1 c), src/model.c:488-490; without rotation the values pass as they are
        auto lo_of = [&](float x0, float x1, float c, float s) { return cp ? x0 * c - x1 * s : x0; };
        auto hi_of = [&](float x0, float x1, float c, float s) { return cp ? x0 * s + x1 * c : x1; };
        auto two = [](float a, float b) { return (uint32_t)bf16_bits(a) | ((uint32_t)bf16_bits(b) << 16); };
        auto turn = [&](const float4 (&lo)[2], const float4 (&hh)[2], const float4 (&c)[2], const float4 (&sn)[2], Frag& fl, Frag& fh) {
            fl.u = make_uint4(two(lo_of(lo[0].x, hh[0].x, c[0].x, sn[0].x), lo_of(lo[0].y, hh[0].y, c[0].y, sn[0].y)),
                              two(lo_of(lo[0].z, hh[0].z, c[0].z, sn[0].z), lo_of(lo[0].w, hh[0].w, c[0].w, sn[0].w)),
                              two(lo_of(lo[1].x, hh[1].x, c[1].x, sn[1].x), lo_of(lo[1].y, hh[1].y, c[1].y, sn[1].y)),
                              two(lo_of(lo[1].z, hh[1].z, c[1].z, sn[1].z), lo_of(lo[1].w, hh[1].w, c[1].w, sn[1].w)));
            fh.u = make_uint4(two(hi_of(lo[0].x, hh[0].x, c[0].x, sn[0].x), hi_of(lo[0].y, hh[0].y, c[0].y, sn[0].y)),
                              two(hi_of(lo[0].z, hh[0].z, c[0].z, sn[0].z), hi_of(lo[0].w, hh[0].w, c[0].w, sn[0].w)),
                              two(hi_of(lo[1].x, hh[1].x, c[1].x, sn[1].x), hi_of(lo[1].y, hh[1].y, c[1].y, sn[1].y)),
                              two(hi_of(lo[1].z, hh[1].z, c[1].z, sn[1].z), hi_of(lo[1].w, hh[1].w, c[1].w, sn[1].w)));
        };
        constexpr int HALF_KS = KS / 2, PASS = HALF_KS > 2 ? 2 : HALF_KS;         // fragments of a half head per pass
        Frag kn[KS];
#pragma unroll
        for (int k0 = 0; k0 < HALF_KS; k0 += PASS) {
            float4 c[PASS][2], sn[PASS][2], ql[PASS][2], qh[PASS][2], kl[PASS][2], kh[PASS][2];
#pragma unroll
            for (int j = 0; j < PASS; j++) {
                const int ks = k0 + j;
                if (ks < HALF_KS) {
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        c[j][u] = make_float4(1.f, 1.f, 1.f, 1.f);
                        sn[j][u] = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (cp) {
                            c[j][u] = *reinterpret_cast<const float4*>(cp + ks * 16 + 4 * u);
                            sn[j][u] = *reinterpret_cast<const float4*>(cp + D / 2 + ks * 16 + 4 * u);
                        }
                        ql[j][u] = *reinterpret_cast<const float4*>(qsrc + ks * 16 + 4 * u);
                        qh[j][u] = *reinterpret_cast<const float4*>(qsrc + (ks + HALF_KS) * 16 + 4 * u);
                        if (owns_new) {
                            kl[j][u] = *reinterpret_cast<const float4*>(ksrc + ks * 16 + 4 * u);
                            kh[j][u] = *reinterpret_cast<const float4*>(ksrc + (ks + HALF_KS) * 16 + 4 * u);
                        }
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < PASS; j++) {
                const int ks = k0 + j;
                if (ks < HALF_KS) {
                    turn(ql[j], qh[j], c[j], sn[j], qf[ks], qf[ks + HALF_KS]);
                    if (owns_new) turn(kl[j], kh[j], c[j], sn[j], kn[ks], kn[ks + HALF_KS]);
                }
            }
        }
        if (!col_ok) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) qf[ks].u = make_uint4(0, 0, 0, 0);
        }
        if (owns_new) {
            const int P_ = 1 << psh;
            if (col == 0) {                                  // every lane of a half computed the same key: one lane of each stores
                uint16_t* dst = const_cast<uint16_t*>(kc) + (size_t)slot * kvw + g * D + half * 8;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    *reinterpret_cast<uint4*>(dst + ks * 16) = kn[ks].u;
                    *reinterpret_cast<uint4*>(&new_s[ks * 16 + half * 8]) = kn[ks].u;
                }
            }
            if (half == 0) {                                 // the value: dimension 32 db + col, transposed inside its page
                uint16_t* vdst = const_cast<uint16_t*>(vc) + (size_t)(slot >> psh) * P_ * kvw + (slot & (P_ - 1));
#pragma unroll
                for (int db = 0; db < NDB; db++) {
                    const uint16_t v = bf16_bits(vraw[db]);
                    vdst[(size_t)(g * D + 32 * db + col) * P_] = v;
                    new_s[D + 32 * db + col] = v;
                }
            }
        }
    };
    floatx16 o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.f;
    float m = NEG_BIG, l = 0.f;

    // Page ids come from LDS, never from the block table inside the loop: a block-table load
    // whose result feeds an address would have to be waited for, and since loads return in order
    // that wait would drain every key and value load issued before it. The ids of a window of
    // PG_MAX pages are fetched at once (pw0 = first page of the window), outside the steady loop.
    __shared__ int pg_s[PG_MAX];
    int pw0 = 0;
    auto page_of = [&](int key) { return pg_s[(key >> psh) - pw0]; };

    auto load_k = [&](int key0, Frag (&kf)[KS]) {
        int key = key0 + col;                              // this lane's row of the key block
        key = key < hi ? key : hi;                         // rows past the end repeat the last key; they are masked
        const int page = page_of(key);
        const unsigned off = __umul24((unsigned)((page << psh) + (key & (P - 1))), (unsigned)kvw) + (unsigned)(g * D + half * 8);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kf[ks].u = *reinterpret_cast<const uint4*>(kc + (off + (unsigned)(ks * 16)));
    };

    // values of a block: for product step kk the lane needs keys key0 + 16 kk + 4 half + {0..3}
    // and the same + 8, for dimension 32 db + col
    auto load_v = [&](int key0, Frag (&vf)[NDB][2]) {
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int run = 0; run < 2; run++) {
                int ka = key0 + 16 * kk + 8 * run + 4 * half;
                ka = ka < (hi & ~3) ? ka : (hi & ~3);       // runs past the end are masked; read a valid one
                const int page = page_of(ka);
                // element offsets fit 32 bits (checked on the host), so one base serves every load
                const unsigned off = __umul24((unsigned)(page << psh), (unsigned)kvw) + (unsigned)(((g * D + col) << psh) + (ka & (P - 1)));
#pragma unroll
                for (int db = 0; db < NDB; db++)
                    vf[db][kk].h[run] = *reinterpret_cast<const uint2*>(vc + (off + (unsigned)((db * 32) << psh)));
            }
        }
    };

    // One block of 32 keys in two halves, so that the registers of its keys can be refilled as
    // soon as the scores are formed: scores + online softmax, then weighted values.
    Frag pf[2];
    auto scores = [&](int key0, Frag (&kf)[KS]) {
        if (FUSED && owns_new && key0 <= hi && hi < key0 + KB) {       // the block of the token's own key (uniform)
            if (key0 + col == hi) {
#pragma unroll
                for (int ks = 0; ks < KS; ks++) kf[ks].u = *reinterpret_cast<const uint4*>(&new_s[ks * 16 + half * 8]);
            }
        }
        floatx16 st;
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks].v, qf[ks].v, st, 0, 0, 0);
        // element r of the lane: key key0 + 8 (r / 4) + 4 half + r % 4, this lane's column.
        // Most blocks lie wholly inside what every column of the wave may see (unused columns
        // aside, whose results are dropped): no key of them needs the visibility test, and the
        // scale (positive) moves into the exponent's fma.
        const bool inside = __all(!col_ok || (key0 >= vlo && key0 + KB - 1 <= vhi)) != 0;
        float mx = NEG_BIG, mn, corr, psum = 0.f;
        if (inside) {
#pragma unroll
            for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[r]);
            mx = pair_max(mx) * scale_log2e;
            mn = mx > m + MAX_SLACK ? mx : m;
            corr = fast_exp2(m - mn);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                st[r] = fast_exp2(fmaf(st[r], scale_log2e, -mn));
                psum += st[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int kr = key0 + 8 * (r / 4) + 4 * half + (r % 4);
                const bool vis = kr >= vlo && kr <= vhi;
                st[r] = vis ? st[r] * scale_log2e : NEG_BIG;
                mx = fmaxf(mx, st[r]);
            }
            mx = pair_max(mx);
            mn = mx > m + MAX_SLACK ? mx : m;
            corr = fast_exp2(m - mn);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float p = st[r] > 0.5f * NEG_BIG ? fast_exp2(st[r] - mn) : 0.f;
                st[r] = p;
                psum += p;
            }
        }
        psum = pair_sum(psum);
        l = l * corr + psum;
        m = mn;
        // the running maxima settle after a few blocks; the accumulators are rescaled only when
        // some column's maximum moved (decided by the whole wave together)
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int db = 0; db < NDB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= corr;
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
                w[e] = prob_pair(st[8 * kk + 2 * e], st[8 * kk + 2 * e + 1]);
            pf[kk].u = make_uint4(w[0], w[1], w[2], w[3]);
        }
    };
    // Keys of a block that lie outside [k_begin, k_end] (before the first key any column sees, past the
    // last one) have probability zero in every column, but what the cache holds there is not this
    // request's: rows of a page it has not written yet, or of a page the window gave back, with
    // whatever their last owner left, Inf and NaN included, and 0 x Inf is NaN. Their values are
    // replaced by zeros; only the first and the last block of a walk have such keys.
    auto values = [&](int key0, Frag (&vf)[NDB][2]) {
        if (FUSED && owns_new && key0 <= hi && hi < key0 + KB) {       // the token's own value, in the run of four keys that holds it
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int run = 0; run < 2; run++) {
                    const int ka = key0 + 16 * kk + 8 * run + 4 * half;
                    if (ka <= hi && hi < ka + 4) {
                        const int e = hi - ka;
#pragma unroll
                        for (int db = 0; db < NDB; db++) {
                            const uint32_t v = new_s[D + 32 * db + col];
                            const uint32_t x = vf[db][kk].h[run].x, y = vf[db][kk].h[run].y;
                            vf[db][kk].h[run].x = e == 0 ? (x & 0xffff0000u) | v : e == 1 ? (x & 0x0000ffffu) | (v << 16) : x;
                            vf[db][kk].h[run].y = e == 2 ? (y & 0xffff0000u) | v : e == 3 ? (y & 0x0000ffffu) | (v << 16) : y;
                        }
                    }
                }
        }
        if (key0 < k_begin || key0 + KB - 1 > k_end) {         // uniform over the wave
#pragma unroll
            for (int kk = 0; kk < 2; kk++)
#pragma unroll
                for (int run = 0; run < 2; run++) {
                    const int kb = key0 + 16 * kk + 8 * run + 4 * half;
                    uint32_t mk[2];
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const bool lo_ok = kb + 2 * e >= k_begin && kb + 2 * e <= k_end;
                        const bool hi_ok = kb + 2 * e + 1 >= k_begin && kb + 2 * e + 1 <= k_end;
                        mk[e] = (lo_ok ? 0x0000ffffu : 0u) | (hi_ok ? 0xffff0000u : 0u);
                    }
#pragma unroll
                    for (int db = 0; db < NDB; db++) {
                        vf[db][kk].h[run].x &= mk[0];
                        vf[db][kk].h[run].y &= mk[1];
                    }
                }
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int db = 0; db < NDB; db++)
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][kk].v, pf[kk].v, o[db], 0, 0, 0);
    };

    // Two register sets in rotation. The keys of block b + 2 are requested as soon as the scores
    // of block b are formed, its values as soon as block b's values are used, so between one and
    // two blocks (16 to 32 KB a wave at head_dim 128) are always on their way. Inside a window
    // every load is issued unconditionally (past the window's end its last block is fetched again
    // and not used) and there is no branch around a load: the compiler then knows how many loads
    // are outstanding at each use and waits for exactly those instead of draining all of them.
    const int first = (k_begin / KB) * KB;
    const int nb = first <= k_end ? (k_end - first) / KB + 1 : 0;
    const int k_top = first + nb * KB - 1 < hi ? first + nb * KB - 1 : hi;       // last key any load touches
    // key blocks a window of pages covers; a walk starts at a multiple of 32 keys, which with pages of more
    // than 32 tokens may lie inside a page: the window's keys then touch one page more than they fill
    const int win_blocks = ((P > KB ? PG_MAX - 1 : PG_MAX) << psh) / KB;
    for (int wb = 0; wb < nb; wb += win_blocks) {
        const int we = wb + win_blocks < nb ? wb + win_blocks : nb;               // blocks [wb, we)
        __syncthreads();                                                          // the old window is no longer read
        pw0 = (first + wb * KB) >> psh;
        {
            const int top = first + we * KB - 1 < k_top ? first + we * KB - 1 : k_top;
            const int n_pg = (top >> psh) - pw0 + 1;
            for (int i = lane; i < n_pg; i += WAVE) pg_s[i] = bt[pw0 + i];
        }
        __syncthreads();
        const int last = first + (we - 1) * KB;
        auto at = [&](int b) { const int k = first + b * KB; return k < last ? k : last; };
        Frag k0f[KS], k1f[KS], v0f[NDB][2], v1f[NDB][2];
        load_k(at(wb), k0f);
        load_v(at(wb), v0f);
        load_k(at(wb + 1), k1f);
        load_v(at(wb + 1), v1f);
        if (FUSED && wb == 0) fused_prologue();
        for (int b = wb; b < we; b += 2) {
            scores(first + b * KB, k0f);
            load_k(at(b + 2), k0f);
            values(first + b * KB, v0f);
            load_v(at(b + 2), v0f);
            if (b + 1 >= we) break;
            scores(first + (b + 1) * KB, k1f);
            load_k(at(b + 3), k1f);
            values(first + (b + 1) * KB, v1f);
            load_v(at(b + 3), v1f);
        }
    }

    if (!col_ok) return;
    // element r of o[db]: dimension 32 db + 8 (r / 4) + 4 half + r % 4 of this lane's column
    if (SPLIT) {
        float* dst = partial + ((size_t)(my_tok * H + my_head) * n_chunks + chunk) * (D + 2);
        if (half == 0) {
            dst[0] = m;
            dst[1] = l;
        }
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int rg = 0; rg < 4; rg++) {
                float4 v = make_float4(o[db][4 * rg], o[db][4 * rg + 1], o[db][4 * rg + 2], o[db][4 * rg + 3]);
                *reinterpret_cast<float4*>(dst + 2 + 32 * db + 8 * rg + 4 * half) = v;
            }
    } else {
        const float inv = 1.0f / l;
        uint16_t* dst = out + (size_t)my_tok * ldo + my_head * D;
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int rg = 0; rg < 4; rg++) {
                uint2 v;
                v.x = (uint32_t)bf16_bits(o[db][4 * rg] * inv) | ((uint32_t)bf16_bits(o[db][4 * rg + 1] * inv) << 16);
                v.y = (uint32_t)bf16_bits(o[db][4 * rg + 2] * inv) |
                      ((uint32_t)bf16_bits(o[db][4 * rg + 3] * inv) << 16);
                *reinterpret_cast<uint2*>(dst + 32 * db + 8 * rg + 4 * half) = v;
            }
    }
}

// ---- prompt portions: four waves share the keys and values of a block through LDS ---------------
// A block of four waves owns 4 x (tokens per wave) consecutive tokens of one request and one
// key/value head; wave w takes its own 32 columns as above. Every block of 32 keys is fetched
// once by the 256 threads (keys as rows of K, values as rows of V^T), stored in LDS with padded
// rows (272 and 72 bytes: the fragment reads of a wave are conflict-free) and read by all four
// waves, so L2-to-CU traffic drops fourfold against the kernel above and several waves per SIMD
// overlap their matrix products and softmax. Two LDS stages, one barrier per key block. Tiles
// are numbered from the end of each request backwards, so the longest ones start first.
#define PVS 36       // LDS row of a value dimension: 32 keys + 4 pad (elements)

template <int NDB, bool SMALL_PAGES>
__global__ __launch_bounds__(4 * WAVE) __attribute__((amdgpu_waves_per_eu(2))) void attn_prefill_kernel(
    const uint16_t* __restrict__ q, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc, int kvw,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot,
    const int* __restrict__ positions, const int* __restrict__ q_start, int n_seqs, uint16_t* __restrict__ out,
    int ldo, int psh, int window, float scale_log2e, int tpt, int cpt, int n_tiles, int pair_from,
    float* __restrict__ partial, int H, int chunk_keys, int n_chunks) {
    constexpr int D = NDB * 32, KS = D / 16, KROW = D + 8;
    const int P = 1 << psh;                                // tokens per page, a power of two
    __shared__ __attribute__((aligned(16))) uint16_t k_s[2][KB * KROW];
    __shared__ __attribute__((aligned(16))) uint16_t v_s[2][D * PVS];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int col = lane & 31, half = lane >> 5;
    int g = blockIdx.x, tile = blockIdx.y;
    const int tile_tokens = 4 * tpt;

    // Tiles late in a prompt see many keys, early ones few. Blocks are numbered with the key/value
    // head fastest and the tiles from the longest down, so that the long tiles of all heads start
    // first and the short ones fill in beside them (with the head slowest, a CU got two blocks of
    // the same length, and the CUs with the longest tiles set the kernel's time).
    //
    // When all blocks are resident at once, two to a CU, the second block of a CU (id pair_from + j,
    // beside block j) takes the tiles from the shortest up, so that every CU has the same sum of keys.
    if (pair_from > 0) {
        const int id = blockIdx.y * gridDim.x + blockIdx.x;
        if (id >= pair_from) {
            const int j = id - pair_from;
            if (j >= n_tiles * (int)gridDim.x - pair_from) return;
            tile = n_tiles - 1 - j / (int)gridDim.x;
            g = j % (int)gridDim.x;
        }
    }
    int t0 = -1, t_end = 0;
    for (int s = 0; s < n_seqs; s++) {
        const int a = q_start[s], b = q_start[s + 1];
        const int nt = (b - a + tile_tokens - 1) / tile_tokens;
        if (tile < nt) {
            const int rt = nt - 1 - tile;                   // last tile of the request first
            t0 = a + rt * tile_tokens;
            t_end = t0 + tile_tokens < b ? t0 + tile_tokens : b;
            break;
        }
        tile -= nt;
    }
    if (t0 < 0) return;                                    // uniform over the block: no barrier is skipped

    // this wave's tokens and columns
    const int w0 = t0 + wave * tpt;
    const int w_end = w0 + tpt < t_end ? w0 + tpt : t_end;
    const int n_cols = w_end > w0 ? (w_end - w0) * cpt : 0;
    const bool col_ok = col < n_cols;
    const int my_tok = col_ok ? w0 + col / cpt : t0;
    const int my_head = g * cpt + (col_ok ? col % cpt : 0);
    const int pos = positions[my_tok];
    const int pos_first = positions[t0];
    int hi = positions[t_end - 1];
    int k_begin = window > 0 && pos_first - window + 1 > 0 ? pos_first - window + 1 : 0;
    // With n_chunks > 1 the block takes the keys of chunk blockIdx.z only (chunk_keys is a multiple
    // of the key block) and leaves maximum, sum and unscaled output for attn_merge_kernel; a chunk
    // that holds none of the tile's keys leaves an empty record.
    if (n_chunks > 1) {
        const int c_lo = blockIdx.z * chunk_keys, c_hi = c_lo + chunk_keys - 1;
        k_begin = k_begin > c_lo ? k_begin : c_lo;
        hi = hi < c_hi ? hi : c_hi;
    }
    const int vlo = window > 0 && pos - window + 1 > k_begin ? pos - window + 1 : k_begin;
    const int vhi = col_ok ? (pos < hi ? pos : hi) : -1;
    const int* bt = block_table + (size_t)token_slot[t0] * max_blocks;

    // query fragments stay in registers for the whole tile
    Frag qf[KS];
    {
        const uint16_t* qp = q + (size_t)my_tok * ldq + my_head * D + half * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qf[ks].u = col_ok ? *reinterpret_cast<const uint4*>(qp + ks * 16) : make_uint4(0, 0, 0, 0);
    }
    floatx16 o[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.f;
    float m = NEG_BIG, l = 0.f;

    // page ids in LDS, a window of PG_MAX pages at a time (see the kernel above)
    __shared__ int pg_s[PG_MAX];
    int pw0 = 0;
    auto page_of = [&](int key) { return pg_s[(key >> psh) - pw0]; };

    // global -> registers -> LDS. Keys: 32 rows of D elements = 4 D chunks of 16 bytes.
    // Values: D rows of 32 keys = 4 D chunks of 8 keys. Each thread takes up to NCH of both.
    // With a whole number of chunks per thread (head_dim 64 and 128) no load or store stands under a
    // condition: only then does the compiler count the loads in flight and wait for the older set alone.
    constexpr int TOT = 4 * D, NCH = (TOT + 255) / 256;
    constexpr bool EVEN = TOT % 256 == 0;
    u32x4 rk0[NCH], rk1[NCH];
    uint2 rv0[NCH][2], rv1[NCH][2];
    // Pages of up to 32 tokens divide a block of keys, whose first key is a multiple of 32: a
    // thread's row then lies at the same place of the same page of every block, and its addresses
    // are a page id times the page's size plus a constant. No key is clamped on this path: the
    // window of page ids repeats the last valid page for pages past the end (see below), so what is
    // read there is memory of that page, and it is masked like any key past a column's position.
    constexpr bool small_pages = SMALL_PAGES;                  // the launcher's choice: pages of up to 32 tokens
    const unsigned page_elems = (unsigned)kvw << psh;
    int k_pg[NCH], v_pg[NCH];
    unsigned k_at[NCH], v_at[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = tid + i * 256, row = c / (D / 8), k8 = 8 * (c % 4);
        k_pg[i] = row >> psh;
        k_at[i] = (unsigned)((row & (P - 1)) * kvw + g * D + (c % (D / 8)) * 8);
        v_pg[i] = k8 >> psh;
        v_at[i] = (unsigned)(((g * D + c / 4) << psh) + (k8 & (P - 1)));
    }
    auto gload = [&](int key0, u32x4 (&rk)[NCH], uint2 (&rv)[NCH][2]) {
        if constexpr (small_pages) {
            const int pb = (key0 >> psh) - pw0;
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                if (!EVEN && tid + i * 256 >= TOT) break;
                rk[i] = *reinterpret_cast<const u32x4*>(kc + (__umul24((unsigned)pg_s[pb + k_pg[i]], page_elems) + k_at[i]));
                const uint4 v = *reinterpret_cast<const uint4*>(vc + (__umul24((unsigned)pg_s[pb + v_pg[i]], page_elems) + v_at[i]));
                rv[i][0] = make_uint2(v.x, v.y);
                rv[i][1] = make_uint2(v.z, v.w);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * 256;
            if (!EVEN && c >= TOT) break;
            {   // key chunk: row c / (D / 8), 16-byte piece c % (D / 8)
                int key = key0 + c / (D / 8);
                key = key < hi ? key : hi;
                const int page = page_of(key);
                const unsigned off = __umul24((unsigned)((page << psh) + (key & (P - 1))), (unsigned)kvw) + (unsigned)(g * D + (c % (D / 8)) * 8);
                rk[i] = *reinterpret_cast<const u32x4*>(kc + off);
            }
            {   // value chunk: dimension c / 4, keys key0 + 8 (c % 4) .. + 7
                int ka = key0 + 8 * (c % 4);
                ka = ka < (hi & ~7) ? ka : (hi & ~7);
                const int page = page_of(ka);
                const unsigned off = __umul24((unsigned)(page << psh), (unsigned)kvw) + (unsigned)(((g * D + c / 4) << psh) + (ka & (P - 1)));
                const uint4 v = *reinterpret_cast<const uint4*>(vc + off);
                rv[i][0] = make_uint2(v.x, v.y);
                rv[i][1] = make_uint2(v.z, v.w);
            }
        }
    };
    // Values of keys outside [k_begin, hi] are stored as zeros (see the kernel above: their probabilities
    // are zero, what the cache holds there may be anything); only a walk's first and last block have such.
    auto sstore = [&](int stage, int key0, const u32x4 (&rk)[NCH], const uint2 (&rv)[NCH][2]) {
        const bool edge = key0 < k_begin || key0 + KB - 1 > hi;           // uniform over the block
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = tid + i * 256;
            if (!EVEN && c >= TOT) break;
            *reinterpret_cast<u32x4*>(&k_s[stage][(c / (D / 8)) * KROW + (c % (D / 8)) * 8]) = rk[i];
            uint2* dst = reinterpret_cast<uint2*>(&v_s[stage][(c / 4) * PVS + 8 * (c % 4)]);
            uint2 v0 = rv[i][0], v1 = rv[i][1];
            if (edge) {
                const int kb = key0 + 8 * (c % 4);
                auto keep = [&](int k) { return k >= k_begin && k <= hi; };
                v0.x &= (keep(kb) ? 0x0000ffffu : 0u) | (keep(kb + 1) ? 0xffff0000u : 0u);
                v0.y &= (keep(kb + 2) ? 0x0000ffffu : 0u) | (keep(kb + 3) ? 0xffff0000u : 0u);
                v1.x &= (keep(kb + 4) ? 0x0000ffffu : 0u) | (keep(kb + 5) ? 0xffff0000u : 0u);
                v1.y &= (keep(kb + 6) ? 0x0000ffffu : 0u) | (keep(kb + 7) ? 0xffff0000u : 0u);
            }
            dst[0] = v0;
            dst[1] = v1;
        }
    };

    const int first = (k_begin / KB) * KB;
    const int nb = hi >= k_begin ? (hi - first) / KB + 1 : 0;
    const int win_blocks = ((P > KB ? PG_MAX - 1 : PG_MAX) << psh) / KB;     // see the kernel above
    for (int wb = 0; wb < nb; wb += win_blocks) {
        const int we = wb + win_blocks < nb ? wb + win_blocks : nb;               // blocks [wb, we)
        __syncthreads();                                                          // old window and stages are no longer read
        pw0 = (first + wb * KB) >> psh;
        {
            const int top = first + we * KB - 1 < hi ? first + we * KB - 1 : hi;
            const int n_pg = (top >> psh) - pw0 + 1;
            // pages past the last one that holds keys (the window's last block is loaded whole): its id again
            const int n_all = small_pages ? ((first + we * KB - 1) >> psh) - pw0 + 1 : n_pg;
            for (int i = tid; i < n_all; i += 4 * WAVE) pg_s[i] = bt[pw0 + (i < n_pg ? i : n_pg - 1)];
        }
        __syncthreads();
        const int last = first + (we - 1) * KB;
        auto at = [&](int b) { const int k = first + b * KB; return k < last ? k : last; };
        gload(at(wb), rk0, rv0);
        sstore(wb & 1, at(wb), rk0, rv0);
        gload(at(wb + 1), rk0, rv0);                          // unconditional: past the end the last block is fetched again
        gload(at(wb + 2), rk1, rv1);
        __syncthreads();
        // Two register sets in rotation: the block after the next one is on its way while the next one
        // goes into LDS, so a load has two blocks' worth of products and softmax to arrive.
        auto one_block = [&](int b) {
            const int key0 = first + b * KB, stage = b & 1;
            // A wave whose columns all end before this block skips the math. The test is made by all
            // lanes together: the matrix products need every lane, also those of unused columns.
            const bool wave_sees = __any(key0 <= vhi) != 0;
            if (wave_sees) {
                const uint16_t* ks_ = &k_s[stage][col * KROW + half * 8];
                floatx16 st;
#pragma unroll
                for (int r = 0; r < 16; r++) st[r] = 0.f;
                // All fragment reads of the block are asked for before the first product: left to itself
                // the compiler reads one fragment, waits for it and multiplies, sixteen LDS round trips
                // a block. The values' first half arrives while the softmax is computed.
                Frag kf[KS], vf[2][NDB];
#pragma unroll
                for (int ks = 0; ks < KS; ks++) kf[ks].u = *reinterpret_cast<const uint4*>(ks_ + ks * 16);
                auto vread = [&](int kk) {
#pragma unroll
                    for (int db = 0; db < NDB; db++) {
                        const uint16_t* vs_ = &v_s[stage][(32 * db + col) * PVS + 16 * kk + 4 * half];
                        vf[kk][db].h[0] = *reinterpret_cast<const uint2*>(vs_);
                        vf[kk][db].h[1] = *reinterpret_cast<const uint2*>(vs_ + 8);
                    }
                };
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ks++)
                    st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks].v, qf[ks].v, st, 0, 0, 0);
                vread(0);
                __builtin_amdgcn_sched_barrier(0);
                // Most blocks lie wholly inside what every column of the wave may see (unused columns
                // aside, whose results are dropped): no key of them needs the visibility test.
                const bool inside = __all(!col_ok || (key0 >= vlo && key0 + KB - 1 <= vhi)) != 0;
                float mx = NEG_BIG, mn, corr, psum = 0.f;
                if (inside) {                                   // the scale (positive) moves into the exponent's fma
#pragma unroll
                    for (int r = 0; r < 16; r++) mx = fmaxf(mx, st[r]);
                    mx = pair_max(mx) * scale_log2e;
                    mn = mx > m + MAX_SLACK ? mx : m;
                    corr = fast_exp2(m - mn);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        st[r] = fast_exp2(fmaf(st[r], scale_log2e, -mn));
                        psum += st[r];
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int kr = key0 + 8 * (r / 4) + 4 * half + (r % 4);
                        const bool vis = kr >= vlo && kr <= vhi;
                        st[r] = vis ? st[r] * scale_log2e : NEG_BIG;
                        mx = fmaxf(mx, st[r]);
                    }
                    mx = pair_max(mx);
                    mn = mx > m + MAX_SLACK ? mx : m;
                    corr = fast_exp2(m - mn);
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const float p = st[r] > 0.5f * NEG_BIG ? fast_exp2(st[r] - mn) : 0.f;
                        st[r] = p;
                        psum += p;
                    }
                }
                psum = pair_sum(psum);
                l = l * corr + psum;
                m = mn;
                if (__any(corr != 1.0f)) {                      // see above: only when a maximum moved
#pragma unroll
                    for (int db = 0; db < NDB; db++)
#pragma unroll
                        for (int r = 0; r < 16; r++) o[db][r] *= corr;
                }
                Frag pf[2];
#pragma unroll
                for (int kk = 0; kk < 2; kk++) {
                    uint32_t w[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        w[e] = prob_pair(st[8 * kk + 2 * e], st[8 * kk + 2 * e + 1]);
                    pf[kk].u = make_uint4(w[0], w[1], w[2], w[3]);
                }
                vread(1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < 2; kk++)
#pragma unroll
                    for (int db = 0; db < NDB; db++)
                        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kk][db].v, pf[kk].v, o[db], 0, 0, 0);
            }
        };
        for (int b = wb; b < we; b += 2) {
            one_block(b);
            sstore((b & 1) ^ 1, at(b + 1), rk0, rv0);         // block b + 1
            gload(at(b + 3), rk0, rv0);
            __syncthreads();
            if (b + 1 >= we) break;
            one_block(b + 1);
            sstore(b & 1, at(b + 2), rk1, rv1);               // block b + 2
            gload(at(b + 4), rk1, rv1);
            __syncthreads();
        }
    }
    if (!col_ok) return;
    if (n_chunks > 1) {
        float* dst = partial + ((size_t)(my_tok * H + my_head) * n_chunks + blockIdx.z) * (D + 2);
        if (half == 0) {
            dst[0] = m;
            dst[1] = l;
        }
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int rg = 0; rg < 4; rg++)
                *reinterpret_cast<float4*>(dst + 2 + 32 * db + 8 * rg + 4 * half) =
                    make_float4(o[db][4 * rg], o[db][4 * rg + 1], o[db][4 * rg + 2], o[db][4 * rg + 3]);
        return;
    }
    const float inv = 1.0f / l;
    uint16_t* dst = out + (size_t)my_tok * ldo + my_head * D;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
            uint2 v;
            v.x = (uint32_t)bf16_bits(o[db][4 * rg] * inv) | ((uint32_t)bf16_bits(o[db][4 * rg + 1] * inv) << 16);
            v.y = (uint32_t)bf16_bits(o[db][4 * rg + 2] * inv) | ((uint32_t)bf16_bits(o[db][4 * rg + 3] * inv) << 16);
            *reinterpret_cast<uint2*>(dst + 32 * db + 8 * rg + 4 * half) = v;
        }
}

// out[t, h, :] = sum_c o_c 2^(m_c - M) / sum_c l_c 2^(m_c - M), chunks in ascending order.
// One wave per (token, head). The kernel is a chain of memory round trips and little else, so it
// is written to have few of them: the first MERGE_GROUP chunks' outputs are asked for before
// anything else, a lane reads maximum and sum of "its" chunk as one pair, and the rest of the
// outputs come MERGE_GROUP loads at a time. A lane owns two neighbouring dimensions (D <= 128).
#define MERGE_MAX_CHUNKS 512
#define MERGE_GROUP 16
__global__ __launch_bounds__(WAVE) void attn_merge_kernel(const float* __restrict__ partial, uint16_t* __restrict__ out,
                                                          int ldo, int H, int D, int n_chunks) {
    __shared__ float w_s[MERGE_MAX_CHUNKS];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const size_t row = D + 2;
    const float* src = partial + (size_t)(t * H + h) * n_chunks * row;
    const bool has = 2 * lane < D;
    const float* mine = src + 2 + 2 * lane;
    float2 pre[MERGE_GROUP];
#pragma unroll
    for (int i = 0; i < MERGE_GROUP; i++)
        pre[i] = has && i < n_chunks ? *reinterpret_cast<const float2*>(mine + i * row) : make_float2(0.f, 0.f);
    const float2 ml0 = lane < n_chunks ? *reinterpret_cast<const float2*>(src + lane * row) : make_float2(NEG_BIG, 0.f);
    float M = ml0.x;
    for (int c = lane + WAVE; c < n_chunks; c += WAVE) M = fmaxf(M, src[c * row]);
    M = wave_max(M);
    float L = 0.f;
    if (lane < n_chunks) {
        const float w = exp2f(ml0.x - M);
        w_s[lane] = w;
        L = ml0.y * w;
    }
    for (int c = lane + WAVE; c < n_chunks; c += WAVE) {
        const float2 ml = *reinterpret_cast<const float2*>(src + c * row);
        const float w = exp2f(ml.x - M);
        w_s[c] = w;
        L += ml.y * w;
    }
    L = wave_sum(L);
    __syncthreads();
    if (!has) return;
    float ax = 0.f, ay = 0.f;
#pragma unroll
    for (int i = 0; i < MERGE_GROUP; i++)
        if (i < n_chunks) {
            ax = fmaf(pre[i].x, w_s[i], ax);
            ay = fmaf(pre[i].y, w_s[i], ay);
        }
    for (int c0 = MERGE_GROUP; c0 < n_chunks; c0 += MERGE_GROUP) {
        float2 v[MERGE_GROUP];
#pragma unroll
        for (int i = 0; i < MERGE_GROUP; i++)
            v[i] = c0 + i < n_chunks ? *reinterpret_cast<const float2*>(mine + (c0 + i) * row) : make_float2(0.f, 0.f);
#pragma unroll
        for (int i = 0; i < MERGE_GROUP; i++)
            if (c0 + i < n_chunks) {
                ax = fmaf(v[i].x, w_s[c0 + i], ax);
                ay = fmaf(v[i].y, w_s[c0 + i], ay);
            }
    }
    const float inv = 1.0f / L;
    *reinterpret_cast<uint32_t*>(out + (size_t)t * ldo + h * D + 2 * lane) =
        (uint32_t)bf16_bits(ax * inv) | ((uint32_t)bf16_bits(ay * inv) << 16);
}

// log2 of the page size, or -1 if it is not a power of two (the kernels shift and mask by it).
static int page_shift(int page_tokens) {
    int s = 0;
    while ((1 << s) < page_tokens) s++;
    return (1 << s) == page_tokens ? s : -1;
}

bool attn_mfma_supports(const AttnArgs& a) {
    const int group = a.n_heads / a.n_kv_heads;
    // a scale that is not positive goes to the plain kernel: the prompt kernel takes the maximum before scaling
    return a.scale > 0.f && a.head_dim % 32 == 0 && a.head_dim <= 128 && a.page_tokens >= 4 && page_shift(a.page_tokens) >= 0 && group <= 32 && a.q_start != nullptr &&
           a.ldq % 8 == 0 && a.ldo % 4 == 0 && a.kv_width % 8 == 0 && a.kv_width * a.page_tokens < (1 << 20) &&
           ((uintptr_t)a.q & 15) == 0 &&
           ((uintptr_t)a.out & 7) == 0 && ((uintptr_t)a.k_cache & 15) == 0 && ((uintptr_t)a.v_cache & 15) == 0;
}

template <int NDB>
static int launch_ndb(const AttnArgs& a, int tiles, int tpt, int cpt, int chunk_keys, int n_chunks) {
    dim3 grid(tiles, a.n_kv_heads, n_chunks);
    const float sl = a.scale * 1.4426950408889634f;
#define ATTN_ARGS(PARTIAL)                                                                                              \
    (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width, a.block_table,      \
        a.max_blocks, a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo, PARTIAL, a.n_heads,         \
        page_shift(a.page_tokens), a.window, sl, tpt, cpt, chunk_keys, n_chunks, a.max_q_len <= tpt, a.raw, a.ld_raw,      \
        a.cos_sin, a.slot_map, a.n_kv_heads
    if (a.raw) {
        if (n_chunks > 1) attn_mfma_kernel<NDB, true, true><<<grid, WAVE, 0, a.stream>>>(ATTN_ARGS((float*)a.workspace));
        else attn_mfma_kernel<NDB, false, true><<<grid, WAVE, 0, a.stream>>>(ATTN_ARGS(nullptr));
    } else {
        if (n_chunks > 1) attn_mfma_kernel<NDB, true, false><<<grid, WAVE, 0, a.stream>>>(ATTN_ARGS((float*)a.workspace));
        else attn_mfma_kernel<NDB, false, false><<<grid, WAVE, 0, a.stream>>>(ATTN_ARGS(nullptr));
    }
#undef ATTN_ARGS
    HFA_LAUNCH_CHECK("attn_mfma");
    return 0;
}

static int attn_cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

template <int NDB>
static int launch_prefill(const AttnArgs& a, int tpt, int cpt) {
    const int tile_tokens = 4 * tpt;
    dim3 grid(a.n_kv_heads, (a.n_tokens + tile_tokens - 1) / tile_tokens + a.n_seqs);
    // One request: the number of tiles is known here, and with it whether all blocks are resident at once.
    const int n_tiles = a.n_seqs == 1 ? (a.n_tokens + tile_tokens - 1) / tile_tokens : 0;
    const int cus = attn_cu_count();
    int pair_from = n_tiles * a.n_kv_heads > cus && n_tiles * a.n_kv_heads <= 2 * cus ? cus : 0;
    // Fewer blocks than two a CU, each with a long walk over its request's keys: the keys are cut into
    // chunks of 256 or more over blockIdx.z until the machine is full, and attn_merge_kernel puts the
    // chunks' results together (portions of a few hundred tokens far into a long prompt).
    int n_chunks = 1, chunk_keys = a.max_seq_len;
    const long blocks = (long)a.n_kv_heads * ((a.n_tokens + tile_tokens - 1) / tile_tokens);
    if (blocks < 2 * cus && a.max_seq_len >= 512 && a.workspace != nullptr) {
        long want = (2 * cus + blocks - 1) / blocks;
        if (want > a.max_seq_len / 256) want = a.max_seq_len / 256;
        if (want > MERGE_MAX_CHUNKS) want = MERGE_MAX_CHUNKS;
        const size_t per_chunk = (size_t)a.n_tokens * a.n_heads * (a.head_dim + 2) * sizeof(float);
        if ((size_t)want * per_chunk > a.workspace_bytes) want = (long)(a.workspace_bytes / per_chunk);
        if (want > 1) {
            chunk_keys = (int)((a.max_seq_len + want - 1) / want + 63) / 64 * 64;
            n_chunks = (a.max_seq_len + chunk_keys - 1) / chunk_keys;
        }
    }
    if (n_chunks > 1) {
        pair_from = 0;
        grid.z = n_chunks;
    }
    if (a.page_tokens <= 32)
        attn_prefill_kernel<NDB, true><<<grid, 4 * WAVE, 0, a.stream>>>(
            (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width, a.block_table,
            a.max_blocks, a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo,
            page_shift(a.page_tokens), a.window, a.scale * 1.4426950408889634f, tpt, cpt, n_tiles, pair_from,
            (float*)a.workspace, a.n_heads, chunk_keys, n_chunks);
    else
        attn_prefill_kernel<NDB, false><<<grid, 4 * WAVE, 0, a.stream>>>(
            (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width, a.block_table,
            a.max_blocks, a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo,
            page_shift(a.page_tokens), a.window, a.scale * 1.4426950408889634f, tpt, cpt, n_tiles, pair_from,
            (float*)a.workspace, a.n_heads, chunk_keys, n_chunks);
    HFA_LAUNCH_CHECK("attn_prefill");
    if (n_chunks > 1) {
        attn_merge_kernel<<<dim3(a.n_tokens, a.n_heads), WAVE, 0, a.stream>>>((const float*)a.workspace, (uint16_t*)a.out, a.ldo,
                                                                            a.n_heads, a.head_dim, n_chunks);
        HFA_LAUNCH_CHECK("attn_merge");
    }
    return 0;
}

// A call in which some request brings this many tokens or more goes to the kernel for prompt portions,
// whole: it walks each request's keys in one piece. A caller that has requests with single tokens and
// long contexts beside prompt portions does better to make two calls, one below and one from this number up.
#define PROMPT_ROWS 16
extern "C" int hfa_attention_prompt_rows(void) { return PROMPT_ROWS; }

int attn_mfma_launch(const AttnArgs& a) {
    const int cpt = a.n_heads / a.n_kv_heads;              // columns per token: the heads of a group
    const int tpt = 32 / cpt;                              // tokens per tile
    // Steps with prompt portions: the kernel that shares keys and values between four waves.
    // That kernel has one block per 4 x tpt tokens and key/value head (and chunk of keys, when it has
    // few blocks). Very few tokens with long contexts (a token budget of 64 far into a long prompt)
    // fill its tiles badly: those go to the kernel below, one wave per tile, which also cuts the keys.
    const long prompt_blocks = ((long)(a.n_tokens + 4 * tpt - 1) / (4 * tpt)) * a.n_kv_heads;
    const bool few_long = 8 * prompt_blocks < attn_cu_count() && a.max_seq_len >= 1024 && a.workspace != nullptr;
    if (a.raw == nullptr && a.max_q_len >= PROMPT_ROWS && !few_long && a.page_tokens % 8 == 0 &&
        (a.n_tokens + 4 * tpt - 1) / (4 * tpt) + a.n_seqs <= 65535) {
        switch (a.head_dim / 32) {
            case 1: return launch_prefill<1>(a, tpt, cpt);
            case 2: return launch_prefill<2>(a, tpt, cpt);
            case 3: return launch_prefill<3>(a, tpt, cpt);
            default: return launch_prefill<4>(a, tpt, cpt);
        }
    }
    const int tiles = a.max_q_len <= tpt ? a.n_seqs : (a.n_tokens + tpt - 1) / tpt + a.n_seqs;
    // Few waves and long contexts: cut the keys into chunks so that the machine is full.
    const long waves = (long)(a.max_q_len <= tpt ? a.n_seqs : (a.n_tokens + tpt - 1) / tpt) * a.n_kv_heads;
    const int span = a.window > 0 && a.window + a.max_q_len < a.max_seq_len ? a.window + a.max_q_len : a.max_seq_len;
    int n_chunks = 1, chunk_keys = a.max_seq_len;
    // How many waves in all is a measured choice. Head size 128 (7B shape): 512; with 1,024 a step took 1.3 % longer
    // at 64 sequences and 4.5 % longer at 8 sequences of 16,384 tokens, with 256 more than that. Head size 64 (0.5B
    // shape), where a wave has half the work per key: 1,024; with 512 a step of 64 sequences took 4.5 % longer; but no
    // chunk of fewer than 128 keys for either head size (with chunks of 64 keys a step of 8 sequences of the 0.5B shape at
    // 2,048 took 5 % longer, one of 16 2 %; one of 2 sequences of the 7B shape 2 % longer).
    const int fill = a.head_dim > 64 ? 512 : 1024;
    if (waves < fill && span > 128 && a.workspace) {
        int want = (int)((fill + waves - 1) / waves);
        const int most = (span + 127) / 128;
        if (want > most) want = most;
        chunk_keys = ((a.max_seq_len + want - 1) / want + KB - 1) / KB * KB;
        if (chunk_keys < 64) chunk_keys = 64;
        n_chunks = (a.max_seq_len + chunk_keys - 1) / chunk_keys;
        const size_t need = (size_t)a.n_tokens * a.n_heads * n_chunks * (a.head_dim + 2) * sizeof(float);
        if (n_chunks < 2 || n_chunks > MERGE_MAX_CHUNKS || need > a.workspace_bytes) {
            n_chunks = 1;
            chunk_keys = a.max_seq_len;
        }
    }
    int rc;
    switch (a.head_dim / 32) {
        case 1: rc = launch_ndb<1>(a, tiles, tpt, cpt, chunk_keys, n_chunks); break;
        case 2: rc = launch_ndb<2>(a, tiles, tpt, cpt, chunk_keys, n_chunks); break;
        case 3: rc = launch_ndb<3>(a, tiles, tpt, cpt, chunk_keys, n_chunks); break;
        default: rc = launch_ndb<4>(a, tiles, tpt, cpt, chunk_keys, n_chunks); break;
    }
    if (rc || n_chunks == 1) return rc;
    dim3 grid(a.n_tokens, a.n_heads);
    attn_merge_kernel<<<grid, WAVE, 0, a.stream>>>((const float*)a.workspace, (uint16_t*)a.out, a.ldo, a.n_heads,
                                                  a.head_dim, n_chunks);
    HFA_LAUNCH_CHECK("attn_merge");
    return 0;
}
