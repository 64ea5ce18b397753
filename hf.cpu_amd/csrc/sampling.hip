// Kernels of the sampler: the greedy choice, and the ordered best-k of a row with the
// row's log-sum-exp, from which the host finishes temperature / top-k / top-p / min-p
// sampling exactly in the reference's order of operations.
#include "api.h"
#include "common.h"

// Ordering of candidates: larger logit first, then smaller id (src/sample.c:59-64).
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__device__ __forceinline__ void block_best(float& v, int& i, float* sv, int* si) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, WAVE);
        const int oi = __shfl_xor(i, off, WAVE);
        if (better(ov, oi, v, i)) { v = ov; i = oi; }
    }
    const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
    __syncthreads();
    if (lane == 0) { sv[w] = v; si[w] = i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float bv = sv[0];
        int bi = si[0];
        for (int k = 1; k < nw; k++)
            if (better(sv[k], si[k], bv, bi)) { bv = sv[k]; bi = si[k]; }
        sv[16] = bv;
        si[16] = bi;
    }
    __syncthreads();
    v = sv[16];
    i = si[16];
}

// Two stages, so that a single row still spreads over the machine: ARGMAX_PARTS blocks per row
// each find the best of their slice, then one small block per row picks among them. The
// ordering (larger logit, then smaller id) makes the result independent of the slicing.
#define ARGMAX_PARTS 64
__global__ __launch_bounds__(256) void argmax_part_kernel(const float* __restrict__ logits, int ld, int vocab,
                                                          float* __restrict__ part_v, int* __restrict__ part_i) {
    __shared__ float sv[17];
    __shared__ int si[17];
    const float* row = logits + (size_t)blockIdx.x * ld;
    const int per = (vocab + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
    const int lo = blockIdx.y * per, hi = lo + per < vocab ? lo + per : vocab;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = row[i];
        if (better(v, i, bv, bi)) { bv = v; bi = i; }
    }
    block_best(bv, bi, sv, si);
    if (threadIdx.x == 0) {
        part_v[blockIdx.x * ARGMAX_PARTS + blockIdx.y] = bv;
        part_i[blockIdx.x * ARGMAX_PARTS + blockIdx.y] = bi;
    }
}

__global__ __launch_bounds__(WAVE) void argmax_final_kernel(const float* __restrict__ part_v,
                                                            const int* __restrict__ part_i, int* __restrict__ out) {
    float v = part_v[blockIdx.x * ARGMAX_PARTS + threadIdx.x];
    int i = part_i[blockIdx.x * ARGMAX_PARTS + threadIdx.x];
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, WAVE);
        const int oi = __shfl_xor(i, off, WAVE);
        if (better(ov, oi, v, i)) { v = ov; i = oi; }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = i == 0x7fffffff ? 0 : i;
}

extern "C" int hfa_argmax(const float* logits, int ld, int* out, int n_rows, int vocab, void* workspace,
                          size_t workspace_bytes, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "argmax: bad sizes rows=%d vocab=%d ld=%d", n_rows, vocab, ld);
    HFA_REQUIRE(workspace && workspace_bytes >= (size_t)n_rows * ARGMAX_PARTS * 8,
                "argmax: the workspace is smaller than %d x %d candidates", n_rows, ARGMAX_PARTS);
    static_assert(ARGMAX_PARTS == WAVE, "the second stage is one wave per row");
    float* part_v = (float*)workspace;
    int* part_i = (int*)(part_v + (size_t)n_rows * ARGMAX_PARTS);
    argmax_part_kernel<<<dim3(n_rows, ARGMAX_PARTS), 256, 0, stream>>>(logits, ld, vocab, part_v, part_i);
    argmax_final_kernel<<<n_rows, WAVE, 0, stream>>>(part_v, part_i, out);
    HFA_LAUNCH_CHECK("argmax");
    return 0;
}

// One block per row. Pass c finds the best candidate that comes after the one chosen in
// pass c-1 in the ordering, so nothing is modified and the order is exact.
__global__ __launch_bounds__(1024) void topk_kernel(const float* __restrict__ logits, int ld, int* __restrict__ ids,
                                                    float* __restrict__ vals, float* __restrict__ stats, int vocab,
                                                    int k) {
    __shared__ float sv[17];
    __shared__ int si[17];
    __shared__ float red[17];
    const float* row = logits + (size_t)blockIdx.x * ld;
    float pv = INFINITY;
    int pi = -1;
    float mx = 0.f;
    for (int c = 0; c < k; c++) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
            const float v = row[i];
            const bool after = v < pv || (v == pv && i > pi);
            if (after && better(v, i, bv, bi)) { bv = v; bi = i; }
        }
        block_best(bv, bi, sv, si);
        if (threadIdx.x == 0) {
            ids[(size_t)blockIdx.x * k + c] = bi == 0x7fffffff ? -1 : bi;
            vals[(size_t)blockIdx.x * k + c] = bv;
        }
        if (c == 0) mx = bv;
        pv = bv;
        pi = bi;
    }
    if (stats) {
        if (k == 0) {
            float bv = -INFINITY;
            for (int i = threadIdx.x; i < vocab; i += blockDim.x) bv = fmaxf(bv, row[i]);
            mx = block_max(bv, red);
        }
        float s = 0.f;
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) s += expf(row[i] - mx);
        s = block_sum(s, red);
        if (threadIdx.x == 0) {
            stats[2 * blockIdx.x] = mx;
            stats[2 * blockIdx.x + 1] = logf(s);
        }
    }
}

extern "C" int hfa_topk(const float* logits, int ld, int* ids, float* vals, float* stats, int n_rows, int vocab,
                        int k, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "topk: bad sizes rows=%d vocab=%d ld=%d", n_rows, vocab, ld);
    HFA_REQUIRE(k >= 0 && k <= 1024 && k <= vocab, "topk: k=%d is outside 0..min(1024, vocab)", k);
    HFA_REQUIRE(k == 0 || (ids && vals), "topk: no output for the candidates");
    topk_kernel<<<n_rows, 1024, 0, stream>>>(logits, ld, ids, vals, stats, vocab, k);
    HFA_LAUNCH_CHECK("topk");
    return 0;
}
