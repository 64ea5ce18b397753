// The plain matrix product: out[m, n] (+)= sum_k a[m, k] * w[n, k] + bias[n] with fp32
// fused multiply-add in ascending k for every output element, whatever M is. It serves the
// 32-bit path (no reduced-precision matrix mode) and every shape the MFMA kernels refuse.
// 64x64 output tile per 256-thread block, K in steps of 16 through LDS, 4x4 outputs a thread.
#include "common.h"
#include "gemm_internal.h"

#define GBM 64
#define GBN 64
#define GBK 16

template <typename TA, typename TW, typename TO, bool ACC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a, int lda,
                                                           const TW* __restrict__ w, int ldw,
                                                           const float* __restrict__ bias, TO* __restrict__ out,
                                                           int ldo, int M, int N, int K) {
    __shared__ float As[GBK][GBM + 4];
    __shared__ float Ws[GBK][GBN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;
    const int tx = tid % 16, ty = tid / 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GBK) {
        const int m = m0 + lr, n = n0 + lr;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int k = k0 + lk + i;
            As[lk + i][lr] = (m < M && k < K) ? to_f32(a[(size_t)m * lda + k]) : 0.f;
            Ws[lk + i][lr] = (n < N && k < K) ? to_f32(w[(size_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GBK; kk++) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j] + (bias ? bias[n] : 0.f);
            TO* dst = out + (size_t)m * ldo + n;
            if (ACC) v += to_f32(*dst);
            *dst = from_f32<TO>(v);
        }
    }
}

template <typename TA, typename TW>
static int launch_out(const GemmArgs& g) {
    dim3 grid((g.N + GBN - 1) / GBN, (g.M + GBM - 1) / GBM);
    const TA* a = (const TA*)g.a;
    const TW* w = (const TW*)g.w;
    if (g.out_dtype == HFA_F32) {
        if (g.accumulate)
            gemm_generic_kernel<TA, TW, float, true><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                                (float*)g.out, g.ldo, g.M, g.N, g.K);
        else
            gemm_generic_kernel<TA, TW, float, false><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                                 (float*)g.out, g.ldo, g.M, g.N, g.K);
    } else {
        gemm_generic_kernel<TA, TW, bf16, false><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                            (bf16*)g.out, g.ldo, g.M, g.N, g.K);
    }
    HFA_LAUNCH_CHECK("gemm_generic");
    return 0;
}

int gemm_generic_launch(const GemmArgs& g) {
    HFA_REQUIRE((g.M + GBM - 1) / GBM <= 65535, "gemm: M=%d is beyond the plain kernel's grid", g.M);
    if (g.a_dtype == HFA_F32 && g.w_dtype == HFA_F32) return launch_out<float, float>(g);
    if (g.a_dtype == HFA_BF16 && g.w_dtype == HFA_BF16) return launch_out<bf16, bf16>(g);
    if (g.a_dtype == HFA_BF16 && g.w_dtype == HFA_F32) return launch_out<bf16, float>(g);
    return launch_out<float, bf16>(g);
}
