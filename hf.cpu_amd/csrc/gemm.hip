// hfa_gemm: argument checks and the choice of the matrix-product kernel.
#include "api.h"
#include "common.h"
#include "gemm_internal.h"

extern "C" int hfa_gemm(const void* a, int a_dtype, int lda, const void* w, int w_dtype, int ldw, const float* bias,
                        void* out, int out_dtype, int ldo, int accumulate, int epilogue, int M, int N, int K,
                        void* workspace, size_t workspace_bytes, int defer, int* pending_splits, int force_plain,
                        hipStream_t stream) {
    HFA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    HFA_REQUIRE(lda >= K && ldw >= K && ldo >= (epilogue ? N / 2 : N),
                "gemm: a row stride is smaller than its row (lda=%d ldw=%d K=%d ldo=%d N=%d)", lda, ldw, K, ldo, N);
    HFA_REQUIRE((a_dtype == HFA_F32 || a_dtype == HFA_BF16) && (w_dtype == HFA_F32 || w_dtype == HFA_BF16) &&
                    (out_dtype == HFA_F32 || out_dtype == HFA_BF16),
                "gemm: unknown dtype (a=%d w=%d out=%d)", a_dtype, w_dtype, out_dtype);
    HFA_REQUIRE(!accumulate || out_dtype == HFA_F32, "gemm: accumulation needs an fp32 output");
    HFA_REQUIRE(epilogue == 0 || epilogue == 1, "gemm: unknown epilogue %d", epilogue);
    if (pending_splits) *pending_splits = 0;
    GemmArgs g = {a, a_dtype, lda, w, w_dtype, ldw, bias, out, out_dtype, ldo, accumulate, epilogue, M, N, K, stream};
    if (!force_plain && gemm_mfma_supports(g)) return gemm_mfma_launch(g, workspace, workspace_bytes, defer, pending_splits);
    HFA_REQUIRE(epilogue == 0, "gemm: the gate/up epilogue exists only on the matrix-core path");
    return gemm_generic_launch(g);
}

// Finishes a product that hfa_gemm left as partial sums: out (+)= sum over splits + bias.
extern "C" int hfa_gemm_finish(const void* partial, int splits, const float* bias, void* out, int out_dtype, int ldo,
                               int accumulate, int epilogue, int M, int N, hipStream_t stream) {
    HFA_REQUIRE(splits > 0 && M > 0 && N > 0, "gemm_finish: bad sizes");
    GemmArgs g = {nullptr, HFA_BF16, 0, nullptr, HFA_BF16, 0, bias, out, out_dtype, ldo, accumulate, epilogue, M, N, 0, stream};
    return gemm_finish_launch((const float*)partial, splits, bias, out, gemm_mode_of(g), ldo, M, N, stream);
}
