// The attention variants behind hfa_paged_attention.
#pragma once
#include <hip/hip_runtime.h>

struct AttnArgs {
    const void* q; int ldq;
    const void* k_cache; const void* v_cache; int kv_width;
    const int* block_table; int max_blocks;
    const int* token_slot; const int* positions; const int* q_start;
    int n_seqs, max_q_len, max_seq_len;
    void* out; int ldo;
    int n_tokens, n_heads, n_kv_heads, head_dim, page_tokens, window;
    float scale;
    void* workspace; size_t workspace_bytes;
    hipStream_t stream;
    // decoded tokens whose queries, new key and new value still lie in 32-bit rows [q | k | v] (see attn_mfma_kernel,
    // FUSED): raw is null otherwise
    const float* raw; int ld_raw;
    const float* cos_sin;          // [token][head_dim / 2 cosines, head_dim / 2 sines], null: no rotation
    const int* slot_map;           // the cache row of each token's key and value
};

int attn_generic_launch(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache, int kv_width,
                        int v_width, const int* block_table, int max_blocks, const int* token_slot, const int* positions,
                        void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        int page_tokens, int window, float scale, const float* slopes, hipStream_t stream);

// bf16 on the matrix cores; see attention_mfma.hip for what it needs.
bool attn_mfma_supports(const AttnArgs& a);
int attn_mfma_launch(const AttnArgs& a);
