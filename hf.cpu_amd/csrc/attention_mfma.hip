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
// chunk order. No LDS, no barrier: every operand comes from global memory in operand layout.
#include "attention_internal.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define KB 32
#define NEG_BIG (-1.0e30f)

union Frag {
    uint4 u;
    uint2 h[2];
    bf16x8 v;
};

template <int NDB, bool SPLIT>
__global__ __launch_bounds__(WAVE) void attn_mfma_kernel(
    const uint16_t* __restrict__ q, int ldq, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc, int kvw,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot,
    const int* __restrict__ positions, const int* __restrict__ q_start, int n_seqs, uint16_t* __restrict__ out,
    int ldo, float* __restrict__ partial, int H, int P, int window, float scale_log2e, int tpt, int cpt,
    int chunk_keys, int n_chunks) {
    constexpr int D = NDB * 32, KS = D / 16;
    const int lane = threadIdx.x, col = lane & 31, half = lane >> 5;
    const int g = blockIdx.y, chunk = blockIdx.z;

    // ---- the tile's request and tokens: tiles are numbered request by request ----
    int tile = blockIdx.x, t0 = -1, t_end = 0;
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

    auto load_k = [&](int key0, Frag* kf) {
        int key = key0 + col;                              // this lane's row of the key block
        key = key < hi ? key : hi;                         // rows past the end repeat the last key; they are masked
        const int page = bt[key / P];
        const uint16_t* kp = kc + ((size_t)page * P + key % P) * kvw + g * D + half * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kf[ks].u = *reinterpret_cast<const uint4*>(kp + ks * 16);
    };

    // values of a block: for product step kk the lane needs keys key0 + 16 kk + 4 half + {0..3}
    // and the same + 8, for dimension 32 db + col
    auto load_v = [&](int key0, Frag (*vf)[2]) {
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int run = 0; run < 2; run++) {
                int ka = key0 + 16 * kk + 8 * run + 4 * half;
                ka = ka < (hi & ~3) ? ka : (hi & ~3);       // runs past the end are masked; read a valid one
                const int page = bt[ka / P];
                const uint16_t* vp = vc + (size_t)page * P * kvw + (size_t)(g * D + col) * P + ka % P;
#pragma unroll
                for (int db = 0; db < NDB; db++)
                    vf[db][kk].h[run] = *reinterpret_cast<const uint2*>(vp + (size_t)db * 32 * P);
            }
        }
    };

    // Keys and values of block b + 1 are requested before block b is worked on, so a wave always
    // has a block's worth of loads (16 KB at head_dim 128) in flight.
    const int first = (k_begin / KB) * KB;
    Frag kf[KS], kn[KS], vf[NDB][2], vn[NDB][2];
    if (first <= k_end) {
        load_k(first, kf);
        load_v(first, vf);
    }
    for (int key0 = first; key0 <= k_end; key0 += KB) {
        const bool more = key0 + KB <= k_end;
        if (more) {
            load_k(key0 + KB, kn);
            load_v(key0 + KB, vn);
        }

        floatx16 st;
#pragma unroll
        for (int r = 0; r < 16; r++) st[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks].v, qf[ks].v, st, 0, 0, 0);

        // element r of the lane: key key0 + 8 (r / 4) + 4 half + r % 4, this lane's column
        float mx = NEG_BIG;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int kr = key0 + 8 * (r / 4) + 4 * half + (r % 4);
            const bool vis = kr >= vlo && kr <= vhi;
            st[r] = vis ? st[r] * scale_log2e : NEG_BIG;
            mx = fmaxf(mx, st[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
        const float mn = fmaxf(m, mx);
        const float corr = exp2f(m - mn);
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = st[r] > 0.5f * NEG_BIG ? exp2f(st[r] - mn) : 0.f;
            st[r] = p;
            psum += p;
        }
        psum += __shfl_xor(psum, 32, WAVE);
        l = l * corr + psum;
        m = mn;
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[db][r] *= corr;

        Frag pf[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
                w[e] = (uint32_t)bf16_bits(st[8 * kk + 2 * e]) | ((uint32_t)bf16_bits(st[8 * kk + 2 * e + 1]) << 16);
            pf[kk].u = make_uint4(w[0], w[1], w[2], w[3]);
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
#pragma unroll
            for (int db = 0; db < NDB; db++)
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][kk].v, pf[kk].v, o[db], 0, 0, 0);
        if (more) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kf[ks] = kn[ks];
#pragma unroll
            for (int db = 0; db < NDB; db++) {
                vf[db][0] = vn[db][0];
                vf[db][1] = vn[db][1];
            }
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

// out[t, h, :] = sum_c o_c 2^(m_c - M) / sum_c l_c 2^(m_c - M), chunks in ascending order.
// Lanes first share the chunks (maximum, weights, sum), then the dimensions; the loads of the
// second loop do not depend on one another.
#define MERGE_MAX_CHUNKS 512
__global__ __launch_bounds__(WAVE) void attn_merge_kernel(const float* __restrict__ partial, uint16_t* __restrict__ out,
                                                          int ldo, int H, int D, int n_chunks) {
    __shared__ float w_s[MERGE_MAX_CHUNKS];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* src = partial + (size_t)(t * H + h) * n_chunks * (D + 2);
    float M = NEG_BIG;
    for (int c = lane; c < n_chunks; c += WAVE) M = fmaxf(M, src[(size_t)c * (D + 2)]);
    M = wave_max(M);
    float L = 0.f;
    for (int c = lane; c < n_chunks; c += WAVE) {
        const float w = exp2f(src[(size_t)c * (D + 2)] - M);
        w_s[c] = w;
        L += src[(size_t)c * (D + 2) + 1] * w;
    }
    L = wave_sum(L);
    __syncthreads();
    const float inv = 1.0f / L;
    for (int d = lane; d < D; d += WAVE) {
        float acc = 0.f;
        for (int c = 0; c < n_chunks; c++) acc = fmaf(src[(size_t)c * (D + 2) + 2 + d], w_s[c], acc);
        out[(size_t)t * ldo + h * D + d] = bf16_bits(acc * inv);
    }
}

bool attn_mfma_supports(const AttnArgs& a) {
    const int group = a.n_heads / a.n_kv_heads;
    return a.head_dim % 32 == 0 && a.head_dim <= 128 && a.page_tokens % 4 == 0 && group <= 32 && a.q_start != nullptr &&
           a.ldq % 8 == 0 && a.ldo % 4 == 0 && a.kv_width % 8 == 0 && ((uintptr_t)a.q & 15) == 0 &&
           ((uintptr_t)a.out & 7) == 0 && ((uintptr_t)a.k_cache & 15) == 0 && ((uintptr_t)a.v_cache & 15) == 0;
}

template <int NDB>
static int launch_ndb(const AttnArgs& a, int tiles, int tpt, int cpt, int chunk_keys, int n_chunks) {
    dim3 grid(tiles, a.n_kv_heads, n_chunks);
    const float sl = a.scale * 1.4426950408889634f;
    if (n_chunks > 1)
        attn_mfma_kernel<NDB, true><<<grid, WAVE, 0, a.stream>>>(
            (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width,
            a.block_table, a.max_blocks, a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo,
            (float*)a.workspace, a.n_heads, a.page_tokens, a.window, sl, tpt, cpt, chunk_keys, n_chunks);
    else
        attn_mfma_kernel<NDB, false><<<grid, WAVE, 0, a.stream>>>(
            (const uint16_t*)a.q, a.ldq, (const uint16_t*)a.k_cache, (const uint16_t*)a.v_cache, a.kv_width,
            a.block_table, a.max_blocks, a.token_slot, a.positions, a.q_start, a.n_seqs, (uint16_t*)a.out, a.ldo,
            nullptr, a.n_heads, a.page_tokens, a.window, sl, tpt, cpt, chunk_keys, n_chunks);
    HFA_LAUNCH_CHECK("attn_mfma");
    return 0;
}

int attn_mfma_launch(const AttnArgs& a) {
    const int cpt = a.n_heads / a.n_kv_heads;              // columns per token: the heads of a group
    const int tpt = 32 / cpt;                              // tokens per tile
    const int tiles = (a.n_tokens + tpt - 1) / tpt + a.n_seqs;
    // Few waves and long contexts: cut the keys into chunks so that the machine is full.
    const long waves = (long)((a.n_tokens + tpt - 1) / tpt) * a.n_kv_heads;
    const int span = a.window > 0 && a.window + a.max_q_len < a.max_seq_len ? a.window + a.max_q_len : a.max_seq_len;
    int n_chunks = 1, chunk_keys = a.max_seq_len;
    if (waves < 1024 && span > 128 && a.workspace) {
        int want = (int)((2048 + waves - 1) / waves);
        const int most = (span + 63) / 64;
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
