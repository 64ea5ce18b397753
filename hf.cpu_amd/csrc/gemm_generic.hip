// The plain matrix product: out[m, n] (+)= sum_k a[m, k] * w[n, k] + bias[n] with fp32
// fused multiply-add in ascending k for every output element, whatever M is. It serves the
// 32-bit path (no reduced-precision matrix mode) and every shape the MFMA kernels refuse.
// 64x64 or 128x128 output tile per 256-thread block, K in steps of 16 through LDS, 4x4 or 8x8 outputs a
// thread; few rows have a kernel of their own further down.
#include "common.h"
#include "gemm_internal.h"

#define GBM 64
#define GBN 64
#define GBK 16

template <typename TA, typename TW, typename TO, bool ACC, int T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a, int lda,
                                                           const TW* __restrict__ w, int ldw,
                                                           const float* __restrict__ bias, TO* __restrict__ out,
                                                           int ldo, int M, int N, int K) {
    constexpr int BMN = 16 * T;                               // the tile's rows and columns: T x T outputs a thread
    __shared__ __attribute__((aligned(16))) float As[GBK][BMN + 4];
    __shared__ __attribute__((aligned(16))) float Ws[GBK][BMN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BMN, n0 = blockIdx.x * BMN;
    const int tx = tid % 16, ty = tid / 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[T][T];
#pragma unroll
    for (int i = 0; i < T; i++)
#pragma unroll
        for (int j = 0; j < T; j++) acc[i][j] = 0.f;

    // the next step's values travel in registers while this step is multiplied
    constexpr int NL = BMN / 64 * 4;
    float ra[NL], rw[NL];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int r0 = 0; r0 < BMN; r0 += 64) {
            const int m = m0 + r0 + lr, n = n0 + r0 + lr;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int k = k0 + lk + i;
                ra[r0 / 16 + i] = (m < M && k < K) ? to_f32(a[(size_t)m * lda + k]) : 0.f;
                rw[r0 / 16 + i] = (n < N && k < K) ? to_f32(w[(size_t)n * ldw + k]) : 0.f;
            }
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += GBK) {
#pragma unroll
        for (int r0 = 0; r0 < BMN; r0 += 64)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                As[lk + i][r0 + lr] = ra[r0 / 16 + i];
                Ws[lk + i][r0 + lr] = rw[r0 / 16 + i];
            }
        __syncthreads();
        if (k0 + GBK < K) fetch(k0 + GBK);
#pragma unroll
        for (int kk = 0; kk < GBK; kk++) {
            float av[T], wv[T];
#pragma unroll
            for (int i = 0; i < T; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(&As[kk][ty * T + i]);
                av[i] = v.x; av[i + 1] = v.y; av[i + 2] = v.z; av[i + 3] = v.w;
                const float4 u = *reinterpret_cast<const float4*>(&Ws[kk][tx * T + i]);
                wv[i] = u.x; wv[i + 1] = u.y; wv[i + 2] = u.z; wv[i + 3] = u.w;
            }
#pragma unroll
            for (int i = 0; i < T; i++)
#pragma unroll
                for (int j = 0; j < T; j++) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < T; i++) {
        const int m = m0 + ty * T + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < T; j++) {
            const int n = n0 + tx * T + j;
            if (n >= N) continue;
            float v = acc[i][j] + (bias ? bias[n] : 0.f);
            TO* dst = out + (size_t)m * ldo + n;
            if (ACC) v += to_f32(*dst);
            *dst = from_f32<TO>(v);
        }
    }
}

// Few rows (decode): the product is bound by the stream of the weights, and 64 x 64 tiles leave most
// CUs without a block. Here a block takes 32 output columns and all rows (up to 64), 256 threads each
// own two columns of MR rows, and K goes through LDS in steps of 128 with the next step's values on
// their way in registers. Every output is still one chain of fused multiply-adds in ascending k, so
// the bits are those of the kernel above, whatever M is.
#define SBN 32
#define SBK 128

template <typename TA, typename TW, typename TO, bool ACC, int MR>
__global__ __launch_bounds__(256) void gemm_generic_rows_kernel(const TA* __restrict__ a, int lda,
                                                                const TW* __restrict__ w, int ldw,
                                                                const float* __restrict__ bias, TO* __restrict__ out,
                                                                int ldo, int M, int N, int K) {
    constexpr int ROWS = 16 * MR;
    __shared__ __attribute__((aligned(16))) float As[ROWS][SBK + 4];
    __shared__ __attribute__((aligned(16))) float Ws[SBN][SBK + 4];
    const int tid = threadIdx.x;
    const int n0 = blockIdx.x * SBN;
    const int nc = tid % 16, mg = tid / 16;                   // columns nc and nc + 16; rows mg + 16 j
    float acc[MR][2];
#pragma unroll
    for (int j = 0; j < MR; j++) acc[j][0] = acc[j][1] = 0.f;
    // what a thread fetches of a step: element e of the tiles, row e / SBK, column e % SBK
    constexpr int WN = SBN * SBK / 256, AN = ROWS * SBK / 256;
    float rw[WN], ra[AN];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < WN; i++) {
            const int e = tid + i * 256, r = e / SBK, k = k0 + e % SBK, n = n0 + r;
            rw[i] = (n < N && k < K) ? to_f32(w[(size_t)n * ldw + k]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < AN; i++) {
            const int e = tid + i * 256, r = e / SBK, k = k0 + e % SBK;
            ra[i] = (r < M && k < K) ? to_f32(a[(size_t)r * lda + k]) : 0.f;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += SBK) {
        __syncthreads();                                      // the step before is no longer read
#pragma unroll
        for (int i = 0; i < WN; i++) { const int e = tid + i * 256; Ws[e / SBK][e % SBK] = rw[i]; }
#pragma unroll
        for (int i = 0; i < AN; i++) { const int e = tid + i * 256; As[e / SBK][e % SBK] = ra[i]; }
        __syncthreads();
        if (k0 + SBK < K) fetch(k0 + SBK);
#pragma unroll 4
        for (int kk = 0; kk < SBK; kk += 4) {
            const float4 w0 = *reinterpret_cast<const float4*>(&Ws[nc][kk]);
            const float4 w1 = *reinterpret_cast<const float4*>(&Ws[nc + 16][kk]);
#pragma unroll
            for (int j = 0; j < MR; j++) {
                const float4 av = *reinterpret_cast<const float4*>(&As[mg + 16 * j][kk]);
                acc[j][0] = fmaf(av.x, w0.x, acc[j][0]); acc[j][1] = fmaf(av.x, w1.x, acc[j][1]);
                acc[j][0] = fmaf(av.y, w0.y, acc[j][0]); acc[j][1] = fmaf(av.y, w1.y, acc[j][1]);
                acc[j][0] = fmaf(av.z, w0.z, acc[j][0]); acc[j][1] = fmaf(av.z, w1.z, acc[j][1]);
                acc[j][0] = fmaf(av.w, w0.w, acc[j][0]); acc[j][1] = fmaf(av.w, w1.w, acc[j][1]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < MR; j++) {
        const int m = mg + 16 * j;
        if (m >= M) continue;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int n = n0 + nc + 16 * c;
            if (n >= N) continue;
            float v = acc[j][c] + (bias ? bias[n] : 0.f);
            TO* dst = out + (size_t)m * ldo + n;
            if (ACC) v += to_f32(*dst);
            *dst = from_f32<TO>(v);
        }
    }
}

template <typename TA, typename TW, int MR>
static int launch_rows(const GemmArgs& g) {
    const dim3 grid((g.N + SBN - 1) / SBN);
    const TA* a = (const TA*)g.a;
    const TW* w = (const TW*)g.w;
    if (g.out_dtype == HFA_F32) {
        if (g.accumulate)
            gemm_generic_rows_kernel<TA, TW, float, true, MR><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias, (float*)g.out, g.ldo, g.M, g.N, g.K);
        else
            gemm_generic_rows_kernel<TA, TW, float, false, MR><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias, (float*)g.out, g.ldo, g.M, g.N, g.K);
    } else {
        gemm_generic_rows_kernel<TA, TW, bf16, false, MR><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias, (bf16*)g.out, g.ldo, g.M, g.N, g.K);
    }
    HFA_LAUNCH_CHECK("gemm_generic_rows");
    return 0;
}

template <typename TA, typename TW, int T>
static int launch_tiles(const GemmArgs& g) {
    dim3 grid((g.N + 16 * T - 1) / (16 * T), (g.M + 16 * T - 1) / (16 * T));
    const TA* a = (const TA*)g.a;
    const TW* w = (const TW*)g.w;
    if (g.out_dtype == HFA_F32) {
        if (g.accumulate)
            gemm_generic_kernel<TA, TW, float, true, T><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                                   (float*)g.out, g.ldo, g.M, g.N, g.K);
        else
            gemm_generic_kernel<TA, TW, float, false, T><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                                    (float*)g.out, g.ldo, g.M, g.N, g.K);
    } else {
        gemm_generic_kernel<TA, TW, bf16, false, T><<<grid, 256, 0, g.stream>>>(a, g.lda, w, g.ldw, g.bias,
                                                                               (bf16*)g.out, g.ldo, g.M, g.N, g.K);
    }
    HFA_LAUNCH_CHECK("gemm_generic");
    return 0;
}

template <typename TA, typename TW>
static int launch_out(const GemmArgs& g) {
    if (g.M <= 16) return launch_rows<TA, TW, 1>(g);
    if (g.M <= 32) return launch_rows<TA, TW, 2>(g);
    if (g.M <= 64) return launch_rows<TA, TW, 4>(g);
    // Tiles of 128 x 128 (8 x 8 outputs a thread: half the LDS reads per multiply-add) where there are
    // enough of them for the machine, else 64 x 64.
    if ((long)((g.N + 127) / 128) * ((g.M + 127) / 128) >= 256) return launch_tiles<TA, TW, 8>(g);
    return launch_tiles<TA, TW, 4>(g);
}

int gemm_generic_launch(const GemmArgs& g) {
    HFA_REQUIRE((g.M + GBM - 1) / GBM <= 65535, "gemm: M=%d is beyond the plain kernel's grid", g.M);
    if (g.a_dtype == HFA_F32 && g.w_dtype == HFA_F32) return launch_out<float, float>(g);
    if (g.a_dtype == HFA_BF16 && g.w_dtype == HFA_BF16) return launch_out<bf16, bf16>(g);
    if (g.a_dtype == HFA_BF16 && g.w_dtype == HFA_F32) return launch_out<bf16, float>(g);
    return launch_out<float, bf16>(g);
}
