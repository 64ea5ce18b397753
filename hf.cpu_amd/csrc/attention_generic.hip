// Paged softmax attention, plain form: one wave per (token, query head), for any mix of
// prompt portions and decoded tokens, any head count and grouping, head_dim up to 256,
// with or without a window, fp32 or bf16 cache. Scores, softmax and the weighted sum are
// fp32; keys are visited in tiles of 64 aligned to absolute positions, in ascending order,
// so a token's result depends on its request's cache alone, never on the rest of the batch.
#include "api.h"
#include "common.h"
#include "attention_internal.h"

#define ATT_MAX_D 256

__device__ __forceinline__ float dot_row(const float* __restrict__ q_s, const bf16* __restrict__ kp, int D) {
    float dot = 0.f;
    if ((D & 7) == 0) {
        for (int d = 0; d < D; d += 8) {
            const uint4 u = *reinterpret_cast<const uint4*>(kp + d);
            const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                dot = fmaf(q_s[d + 2 * i], __uint_as_float(w[i] << 16), dot);
                dot = fmaf(q_s[d + 2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), dot);
            }
        }
    } else {
        for (int d = 0; d < D; d++) dot = fmaf(q_s[d], to_f32(kp[d]), dot);
    }
    return dot;
}
__device__ __forceinline__ float dot_row(const float* __restrict__ q_s, const float* __restrict__ kp, int D) {
    float dot = 0.f;
    if ((D & 3) == 0) {
        for (int d = 0; d < D; d += 4) {
            const float4 u = *reinterpret_cast<const float4*>(kp + d);
            dot = fmaf(q_s[d], u.x, dot);
            dot = fmaf(q_s[d + 1], u.y, dot);
            dot = fmaf(q_s[d + 2], u.z, dot);
            dot = fmaf(q_s[d + 3], u.w, dot);
        }
    } else {
        for (int d = 0; d < D; d++) dot = fmaf(q_s[d], kp[d], dot);
    }
    return dot;
}

template <typename T>
__global__ __launch_bounds__(WAVE) void attn_generic_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ kc, const T* __restrict__ vc, int kvw, int vw,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_slot,
    const int* __restrict__ positions, T* __restrict__ out, int ldo, int H, int G, int D, int Dv, int page_tokens,
    int window, float scale, const float* __restrict__ slopes) {
    __shared__ float q_s[ATT_MAX_D];
    __shared__ float p_s[WAVE];
    __shared__ int row_s[WAVE];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (H / G);
    const int pos = positions[t];
    const int* bt = block_table + (size_t)token_slot[t] * max_blocks;
    for (int d = lane; d < D; d += WAVE) q_s[d] = to_f32(q[(size_t)t * ldq + h * D + d]);
    __syncthreads();
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const float slope = slopes ? slopes[h] : 0.f;           // a position encoding that enters the scores
    float m = -INFINITY, l = 0.f;
    float acc[ATT_MAX_D / WAVE];
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / WAVE; i++) acc[i] = 0.f;

    for (int j0 = (lo / WAVE) * WAVE; j0 <= pos; j0 += WAVE) {
        const int j = j0 + lane;
        const bool valid = j >= lo && j <= pos;
        float s = -INFINITY;
        int row = 0;
        if (valid) {
            row = bt[j / page_tokens] * page_tokens + j % page_tokens;
            s = dot_row(q_s, kc + (size_t)row * kvw + kvh * D, D) * scale;
            if (slopes) s += slope * (float)(j - pos);
        }
        // every tile holds at least one visible key, so the maximum is finite
        const float mn = fmaxf(m, wave_max(s));
        const float corr = expf(m - mn);
        const float p = valid ? expf(s - mn) : 0.f;
        l = l * corr + wave_sum(p);
        m = mn;
        p_s[lane] = p;
        row_s[lane] = row;
        __syncthreads();
        const int first = lo > j0 ? lo - j0 : 0;
        const int last = pos - j0 < WAVE - 1 ? pos - j0 : WAVE - 1;
#pragma unroll
        for (int i = 0; i < ATT_MAX_D / WAVE; i++) acc[i] *= corr;
        for (int jj = first; jj <= last; jj++) {
            const float pj = p_s[jj];
            // values lie transposed inside their page: [page][column][token]
            const int vr = row_s[jj];
            const T* vp = vc + (size_t)(vr / page_tokens) * page_tokens * vw + (size_t)(kvh * Dv) * page_tokens +
                          vr % page_tokens;
#pragma unroll
            for (int i = 0; i < ATT_MAX_D / WAVE; i++) {
                const int d = lane + WAVE * i;
                if (d < Dv) acc[i] = fmaf(pj, to_f32(vp[(size_t)d * page_tokens]), acc[i]);
            }
        }
        __syncthreads();
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < ATT_MAX_D / WAVE; i++) {
        const int d = lane + WAVE * i;
        if (d < Dv) out[(size_t)t * ldo + h * Dv + d] = from_f32<T>(acc[i] * inv);
    }
}

int attn_generic_launch(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache, int kv_width,
                        int v_width, const int* block_table, int max_blocks, const int* token_slot, const int* positions,
                        void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        int page_tokens, int window, float scale, const float* slopes, hipStream_t stream) {
    HFA_REQUIRE(head_dim <= ATT_MAX_D && v_head_dim <= ATT_MAX_D, "paged_attention: head_dim %d (values: %d) exceeds the kernel's limit %d",
                head_dim, v_head_dim, ATT_MAX_D);
    HFA_REQUIRE(n_heads <= 65535, "paged_attention: %d heads exceed the grid", n_heads);
    dim3 grid(n_tokens, n_heads);
    if (dtype == HFA_F32)
        attn_generic_kernel<float><<<grid, WAVE, 0, stream>>>(
            (const float*)q, ldq, (const float*)k_cache, (const float*)v_cache, kv_width, v_width, block_table, max_blocks,
            token_slot, positions, (float*)out, ldo, n_heads, n_kv_heads, head_dim, v_head_dim, page_tokens, window, scale, slopes);
    else
        attn_generic_kernel<bf16><<<grid, WAVE, 0, stream>>>(
            (const bf16*)q, ldq, (const bf16*)k_cache, (const bf16*)v_cache, kv_width, v_width, block_table, max_blocks,
            token_slot, positions, (bf16*)out, ldo, n_heads, n_kv_heads, head_dim, v_head_dim, page_tokens, window, scale, slopes);
    HFA_LAUNCH_CHECK("paged_attention");
    return 0;
}

// cos_sin[t][0 .. half) = cos(positions[t] * inv_freq[i]), [half .. 2 half) the sines: the angles of src/model.c:472-476
// as rope_store forms them, once for all the layers of a step.
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq, int half,
                                  float* __restrict__ out) {
    const int t = blockIdx.x;
    const float pos = (float)positions[t];
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        out[(size_t)t * 2 * half + i] = cs;
        out[(size_t)t * 2 * half + half + i] = sn;
    }
}

extern "C" int hfa_rope_table(const int* positions, const float* inv_freq, int half, float* out, int n_tokens, hipStream_t stream) {
    HFA_REQUIRE(positions && inv_freq && out && half > 0 && n_tokens > 0, "rope_table: bad arguments");
    rope_table_kernel<<<n_tokens, half < 256 ? (half + 63) / 64 * 64 : 256, 0, stream>>>(positions, inv_freq, half, out);
    HFA_LAUNCH_CHECK("rope_table");
    return 0;
}

// Whether hfa_decode_attention takes a step: bf16 on the matrix cores, one head size of 32 to 128 in steps of 32
// for keys and values, rotation of whole heads (rot_dim == head_dim) or none.
extern "C" int hfa_decode_attention_supports(int n_heads, int n_kv_heads, int head_dim, int rot_dim, int page_tokens,
                                             int kv_width, int ld_raw, int ldo) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || !(rot_dim == head_dim || rot_dim == 0) || ld_raw % 4 != 0) return 0;
    AttnArgs a = {};
    a.scale = 1.f; a.head_dim = head_dim; a.page_tokens = page_tokens; a.n_heads = n_heads; a.n_kv_heads = n_kv_heads;
    a.q_start = (const int*)16; a.ldq = 8; a.ldo = ldo; a.kv_width = kv_width;
    return attn_mfma_supports(a) ? 1 : 0;
}

// Attention of decoded tokens (one token a request) whose queries, new keys and new values are still the 32-bit rows
// [q | k | v] that the product left (`raw`, row stride ld_raw, bias added): rotation of queries and keys, the store
// of the new key and value into the cache rows slot_map[t], and attention over the cache in one kernel (and the merge
// of the key chunks). cos_sin: hfa_rope_table's output for these tokens, or null for no rotation. Everything else as
// in hfa_paged_attention, whose result with hfa_rope_store before it this equals.
extern "C" int hfa_decode_attention(const float* raw, int ld_raw, const float* cos_sin, void* k_cache, void* v_cache,
                                    int kv_width, const int* slot_map, const int* block_table, int max_blocks,
                                    const int* token_slot, const int* positions, const int* q_start, int n_seqs,
                                    int max_seq_len, void* out, int ldo, int n_heads, int n_kv_heads, int head_dim,
                                    int page_tokens, int window, float scale, void* workspace, size_t workspace_bytes,
                                    hipStream_t stream) {
    HFA_REQUIRE(raw && k_cache && v_cache && slot_map && block_table && token_slot && positions && q_start && out,
                "decode_attention: a null argument");
    HFA_REQUIRE(n_seqs > 0 && max_seq_len > 0 && max_blocks > 0 && window >= 0, "decode_attention: bad sizes");
    HFA_REQUIRE(ld_raw >= (n_heads + 2 * n_kv_heads) * head_dim && ldo >= n_heads * head_dim && kv_width >= n_kv_heads * head_dim,
                "decode_attention: a row stride is smaller than its row");
    AttnArgs a = {nullptr, 8, k_cache, v_cache, kv_width, block_table, max_blocks, token_slot, positions, q_start,
                  n_seqs, 1, max_seq_len, out, ldo, n_seqs, n_heads, n_kv_heads, head_dim, page_tokens,
                  window, scale, workspace, workspace_bytes, stream, raw, ld_raw, cos_sin, slot_map};
    HFA_REQUIRE(((uintptr_t)raw & 15) == 0 && (cos_sin == nullptr || ((uintptr_t)cos_sin & 15) == 0) && attn_mfma_supports(a),
                "decode_attention: this shape is not taken (see hfa_decode_attention_supports)");
    return attn_mfma_launch(a);
}

extern "C" int hfa_paged_attention(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache,
                                   int kv_width, int v_width, const int* block_table, int max_blocks, const int* token_slot,
                                   const int* positions, const int* q_start, int n_seqs, int max_q_len,
                                   int max_seq_len, void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads,
                                   int head_dim, int v_head_dim, int page_tokens, int window, float scale, const float* slopes,
                                   void* workspace, size_t workspace_bytes, int force_plain, hipStream_t stream) {
    HFA_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && v_head_dim > 0 && page_tokens > 0 && max_blocks > 0,
                "paged_attention: bad sizes");
    HFA_REQUIRE(n_heads % n_kv_heads == 0, "paged_attention: %d heads are not a multiple of %d key/value heads",
                n_heads, n_kv_heads);
    HFA_REQUIRE(kv_width >= n_kv_heads * head_dim && v_width >= n_kv_heads * v_head_dim && ldq >= n_heads * head_dim &&
                    ldo >= n_heads * v_head_dim,
                "paged_attention: a row stride is smaller than its row");
    HFA_REQUIRE(window >= 0, "paged_attention: negative window");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "paged_attention: unknown dtype %d", dtype);
    AttnArgs a = {q, ldq, k_cache, v_cache, kv_width, block_table, max_blocks, token_slot, positions, q_start,
                  n_seqs, max_q_len, max_seq_len, out, ldo, n_tokens, n_heads, n_kv_heads, head_dim, page_tokens,
                  window, scale, workspace, workspace_bytes, stream, nullptr, 0, nullptr, nullptr};
    // the matrix-core kernels take no slopes: scores with a position term go the plain way
    // and they know one head size and one row width for keys and values
    if (!force_plain && !slopes && dtype == HFA_BF16 && v_head_dim == head_dim && v_width == kv_width && attn_mfma_supports(a))
        return attn_mfma_launch(a);
    return attn_generic_launch(q, dtype, ldq, k_cache, v_cache, kv_width, v_width, block_table, max_blocks, token_slot,
                               positions, out, ldo, n_tokens, n_heads, n_kv_heads, head_dim, v_head_dim, page_tokens, window,
                               scale, slopes, stream);
}
