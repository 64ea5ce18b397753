// A kernel that belongs to a test, not to the package: the toy mixer of tests/test_parts_gpu.py keeps
// a running average per request, s <- decay * s + (1 - decay) * h_t in token order, and adds W s to
// the residual stream. One block per request; thread i owns state element i and output row i.
// Everything the kernel needs to know about the step it reads from device memory, so a step that
// uses it can be captured into a graph.
#include <hip/hip_runtime.h>
#include <stdint.h>

__device__ __forceinline__ float load_as_float(const void* p, int dtype, size_t i) {
    if (dtype == 0) return ((const float*)p)[i];
    return __uint_as_float(((uint32_t)((const uint16_t*)p)[i]) << 16);
}

__global__ void toy_ema_kernel(const void* h, int h_dtype, float* state, const void* w, int w_dtype, float* x,
                               const int* q_start, const int* seq_slot, int E, float decay) {
    extern __shared__ float s[];
    const int seq = blockIdx.x, i = threadIdx.x;
    float* st = state + (size_t)seq_slot[seq] * E;
    float mine = i < E ? st[i] : 0.f;
    for (int t = q_start[seq]; t < q_start[seq + 1]; t++) {
        if (i < E) {
            mine = decay * mine + (1.0f - decay) * load_as_float(h, h_dtype, (size_t)t * E + i);
            s[i] = mine;
        }
        __syncthreads();
        if (i < E) {
            float acc = 0.f;
            for (int k = 0; k < E; k++) acc += load_as_float(w, w_dtype, (size_t)i * E + k) * s[k];
            x[(size_t)t * E + i] += acc;
        }
        __syncthreads();
    }
    if (i < E) st[i] = mine;
}

extern "C" int toy_ema(const void* h, int h_dtype, float* state, const void* w, int w_dtype, float* x, const int* q_start,
                       const int* seq_slot, int n_seqs, int E, float decay, hipStream_t stream) {
    if (n_seqs <= 0 || E <= 0 || E > 1024) return 1;
    const int threads = (E + 63) / 64 * 64;
    toy_ema_kernel<<<n_seqs, threads, E * sizeof(float), stream>>>(h, h_dtype, state, w, w_dtype, x, q_start, seq_slot, E, decay);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
