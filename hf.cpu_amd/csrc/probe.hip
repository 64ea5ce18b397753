// Probes of the device's own peaks, against which the bench prices its kernels: a streaming
// read, a copy, and a burn of the matrix cores. They are the GPU's analogue of the reference's
// read_sum and fma_burn entries of its kernel table (src/kern.h:17-23, used by src/probe.c).
#include "api.h"
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// The buffer is cut into pieces of 16 KB that the blocks take in turn; a block's 256 threads read a
// piece as four rows of 4 KB, all four loads of a thread asked for before the first is used. The xor
// of what was read leaves through `sink` only if it equals a value that it (almost) never has, so
// that the loads cannot be dropped.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ p, size_t n, uint4* __restrict__ sink) {
    uint4 acc = make_uint4(0, 0, 0, 0);
    const size_t pieces = n / 1024;
    for (size_t piece = blockIdx.x; piece < pieces; piece += gridDim.x) {
        const uint4* q = p + piece * 1024 + threadIdx.x;
        const uint4 a = q[0], b = q[256], c = q[512], d = q[768];
        acc.x ^= a.x ^ b.x ^ c.x ^ d.x;
        acc.y ^= a.y ^ b.y ^ c.y ^ d.y;
        acc.z ^= a.z ^ b.z ^ c.z ^ d.z;
        acc.w ^= a.w ^ b.w ^ c.w ^ d.w;
    }
    for (size_t i = pieces * 1024 + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const uint4 a = p[i];
        acc.x ^= a.x; acc.y ^= a.y; acc.z ^= a.z; acc.w ^= a.w;
    }
    if (acc.x == 0x9e3779b9u && acc.y == 0x7f4a7c15u && acc.z == 0x2545f491u && acc.w == 0x4f6cdd1du) sink[0] = acc;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        dst[i] = a; dst[i + stride] = b; dst[i + 2 * stride] = c; dst[i + 3 * stride] = d;
    }
    for (; i < n; i += stride) dst[i] = src[i];
}

// Each wave keeps four independent chains of v_mfma_f32_32x32x16_bf16 going on operands that stay in
// registers: nothing but the matrix cores is busy. With `zeros` the operands are all zero, otherwise
// small pseudo-random numbers; the difference between the two rates is what the switching of the
// data costs in clock. `iters` rounds of four products of 2 * 32 * 32 * 16 flops a wave.
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ out, int iters, int zeros) {
    bf16x8 a[2], b[2];
    uint32_t s = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
            s = s * 1664525u + 1013904223u;
            a[i][j] = zeros ? (__bf16)0.0f : (__bf16)(((int)(s >> 20) - 2048) * (1.0f / 8192.0f));
            s = s * 1664525u + 1013904223u;
            b[i][j] = zeros ? (__bf16)0.0f : (__bf16)(((int)(s >> 20) - 2048) * (1.0f / 8192.0f));
        }
    floatx16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
    for (int it = 0; it < iters; it++) {
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[0], acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[1], acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], acc[3], 0, 0, 0);
    }
    float v = 0.f;
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) v += acc[c][r];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = v;
}

static int probe_blocks(int per_cu) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    return cus * per_cu;
}

extern "C" int hfa_probe_read(const void* src, size_t bytes, void* sink, int blocks_per_cu, hipStream_t stream) {
    HFA_REQUIRE(src && sink && bytes >= 16 && ((uintptr_t)src & 15) == 0, "probe_read: needs a 16-byte aligned buffer and a sink of 16 bytes");
    HFA_REQUIRE(blocks_per_cu >= 1 && blocks_per_cu <= 64, "probe_read: 1 to 64 blocks per CU");
    probe_read_kernel<<<probe_blocks(blocks_per_cu), 256, 0, stream>>>((const uint4*)src, bytes / 16, (uint4*)sink);
    HFA_LAUNCH_CHECK("probe_read");
    return 0;
}

extern "C" int hfa_probe_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
    HFA_REQUIRE(src && dst && bytes >= 16 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0, "probe_copy: needs 16-byte aligned buffers");
    probe_copy_kernel<<<probe_blocks(8), 256, 0, stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
    HFA_LAUNCH_CHECK("probe_copy");
    return 0;
}

// out: one float per thread, hfa_probe_mfma_threads() of them. *flops = what the launch computes.
extern "C" int hfa_probe_mfma_threads(void) { return probe_blocks(2) * 256; }

extern "C" int hfa_probe_mfma(float* out, int iters, int zeros, double* flops, hipStream_t stream) {
    HFA_REQUIRE(out && iters > 0, "probe_mfma: needs an output and a positive number of rounds");
    const int blocks = probe_blocks(2);
    probe_mfma_kernel<<<blocks, 256, 0, stream>>>(out, iters, zeros);
    HFA_LAUNCH_CHECK("probe_mfma");
    if (flops) *flops = (double)blocks * 4 /* waves */ * iters * 4.0 * (2.0 * 32 * 32 * 16);
    return 0;
}
