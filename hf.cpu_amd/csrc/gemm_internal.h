// The matrix-product variants behind hfa_gemm. Each takes the same arguments and returns
// 0, or non-zero after hfa_set_error(). The dispatcher in gemm.hip picks one by dtype and shape.
#pragma once
#include <hip/hip_runtime.h>

struct GemmArgs {
    const void* a; int a_dtype; int lda;
    const void* w; int w_dtype; int ldw;
    const float* bias;
    void* out; int out_dtype; int ldo;
    int accumulate;
    int epilogue;            // 0: none; 1: columns are 32 gate, 32 up, ...: out[m, f] = silu(gate) * up
    int M, N, K;
    hipStream_t stream;
};

// Any dtype mix, any size: fp32 multiply-add over K in ascending order for every output.
int gemm_generic_launch(const GemmArgs& g);

// bf16 x bf16 on the matrix cores (K and both row strides multiples of 8, 16-byte aligned bases).
// `workspace` holds the partial sums when K is split for small M; without one K is not split.
// With `defer`, a product whose K was split leaves its partial sums in the workspace
// ([splits][M][N] fp32) and reports the number of splits instead of finishing.
bool gemm_mfma_supports(const GemmArgs& g);
int gemm_mfma_launch(const GemmArgs& g, void* workspace, size_t workspace_bytes, int defer, int* pending_splits);
int gemm_mode_of(const GemmArgs& g);

// bf16 x bf16 for 32 < M <= 128 as one stream of (column tile, 64 columns of K) units cut evenly over the
// CUs (N a multiple of 128, K of 64). gemm_stream_slots() says how many [M][N] fp32 planes of the
// workspace the product will leave its partial sums in (0: not taken); their sum in ascending
// order is the product.
int gemm_stream_slots(const GemmArgs& g, size_t workspace_bytes);
int gemm_stream_launch(const GemmArgs& g, void* workspace, int slots);
// bf16 x bf16 for M <= 16 as one stream of (tile of 32 columns, 64 columns of K) units cut evenly over all waves
// of the machine, every wave streaming its run by itself (K a multiple of 64). gemm_wave_slots() says how many
// [M][N] fp32 planes of the workspace the product will leave its partial sums in (0: not taken).
int gemm_wave_slots(const GemmArgs& g, size_t workspace_bytes);
int gemm_wave_launch(const GemmArgs& g, void* workspace, int slots);
int gemm_finish_launch(const float* partial, int splits, const float* bias, void* out, int mode, int ldo, int M,
                       int N, hipStream_t stream);
