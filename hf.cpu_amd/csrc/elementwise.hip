// Embedding lookup, RMS norm, rotary encoding with the cache store, SwiGLU, and the
// small integer scatter that keeps the device block tables up to date.
#include <stdarg.h>

#include "api.h"
#include "common.h"

// ---- error buffer -----------------------------------------------------------------------
static thread_local char g_error[512] = "";
void hfa_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
}
extern "C" const char* hfa_last_error(void) { return g_error; }
extern "C" int hfa_version(void) { return 1; }

// ---- embedding --------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x,
                             int width, int vocab) {
    const int t = blockIdx.x;
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);   // ids are checked on the host; never read outside
    const T* row = table + (size_t)tok * width;
    float* dst = x + (size_t)t * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_f32(row[i]);
}

extern "C" int hfa_embed(const void* table, int table_dtype, const int* tokens, float* x, int n_tokens, int width,
                         int vocab, hipStream_t stream) {
    HFA_REQUIRE(n_tokens > 0 && width > 0 && vocab > 0, "embed: bad sizes tokens=%d width=%d vocab=%d", n_tokens,
                width, vocab);
    HFA_REQUIRE(table_dtype == HFA_F32 || table_dtype == HFA_BF16, "embed: unknown dtype %d", table_dtype);
    if (table_dtype == HFA_F32)
        embed_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, tokens, x, width, vocab);
    else
        embed_kernel<bf16><<<n_tokens, 256, 0, stream>>>((const bf16*)table, tokens, x, width, vocab);
    HFA_LAUNCH_CHECK("embed");
    return 0;
}

// ---- RMS norm ---------------------------------------------------------------------------
// One block per output row. The sum of squares is taken in a fixed order (each thread over
// its strided elements, then waves, then the block), so a row's result does not depend on
// which other rows are in the launch.
template <typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, TO* __restrict__ out,
                               const int* __restrict__ rows, int width, float eps) {
    __shared__ float red[17];
    const int r = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[r] : r) * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = src[i];
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)width + eps);
    TO* dst = out + (size_t)r * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_f32<TO>((src[i] * scale) * w[i]);
}

extern "C" int hfa_rmsnorm(const float* x, const float* w, void* out, int out_dtype, const int* rows, int n_rows,
                           int width, float eps, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", n_rows, width);
    HFA_REQUIRE(out_dtype == HFA_F32 || out_dtype == HFA_BF16, "rmsnorm: unknown dtype %d", out_dtype);
    const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
    if (out_dtype == HFA_F32)
        rmsnorm_kernel<float><<<n_rows, threads, 0, stream>>>(x, w, (float*)out, rows, width, eps);
    else
        rmsnorm_kernel<bf16><<<n_rows, threads, 0, stream>>>(x, w, (bf16*)out, rows, width, eps);
    HFA_LAUNCH_CHECK("rmsnorm");
    return 0;
}

// ---- rotary encoding + cache store ------------------------------------------------------------
// One block per token. Cosines and sines of the token's angles go to LDS once; the angle is
// the fp32 product of the position and the fp32 inverse frequency.
#define ROPE_MAX_HALF 256
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, int ld, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int rot_dim, int H, int G, int D,
                                  T* __restrict__ k_cache, T* __restrict__ v_cache,
                                  const int* __restrict__ slot_map, int page_tokens) {
    __shared__ float cs[ROPE_MAX_HALF], sn[ROPE_MAX_HALF];
    const int t = blockIdx.x;
    const int half = rot_dim / 2;
    if (half > 0) {
        const float pos = (float)positions[t];
        for (int i = threadIdx.x; i < half; i += blockDim.x) {
            float s, c;
            sincosf(pos * inv_freq[i], &s, &c);
            cs[i] = c;
            sn[i] = s;
        }
    }
    __syncthreads();
    T* row = qkv + (size_t)t * ld;
    // queries: rotate in place
    if (half > 0) {
        for (int it = threadIdx.x; it < H * half; it += blockDim.x) {
            const int h = it / half, i = it - h * half;
            T* p = row + h * D;
            const float x0 = to_f32(p[i]), x1 = to_f32(p[i + half]);
            p[i] = from_f32<T>(x0 * cs[i] - x1 * sn[i]);
            p[i + half] = from_f32<T>(x0 * sn[i] + x1 * cs[i]);
        }
    }
    if (G == 0) return;
    const int slot = slot_map ? slot_map[t] : -1;
    T* krow = row + H * D;
    T* vrow = krow + G * D;
    if (slot < 0) {
        // no cache row: still leave the rotated keys in place so the caller sees them
        if (half > 0) {
            for (int it = threadIdx.x; it < G * half; it += blockDim.x) {
                const int g = it / half, i = it - g * half;
                T* p = krow + g * D;
                const float x0 = to_f32(p[i]), x1 = to_f32(p[i + half]);
                p[i] = from_f32<T>(x0 * cs[i] - x1 * sn[i]);
                p[i + half] = from_f32<T>(x0 * sn[i] + x1 * cs[i]);
            }
        }
        return;
    }
    T* kdst = k_cache + (size_t)slot * (G * D);
    // values lie transposed inside their page: element c of the token at offset o is at c * page_tokens + o
    T* vdst = v_cache + (size_t)(slot / page_tokens) * page_tokens * (G * D) + slot % page_tokens;
    for (int it = threadIdx.x; it < G * half; it += blockDim.x) {
        const int g = it / half, i = it - g * half;
        const T* p = krow + g * D;
        const float x0 = to_f32(p[i]), x1 = to_f32(p[i + half]);
        kdst[g * D + i] = from_f32<T>(x0 * cs[i] - x1 * sn[i]);
        kdst[g * D + i + half] = from_f32<T>(x0 * sn[i] + x1 * cs[i]);
    }
    const int rest = D - rot_dim;   // dimensions that pass through
    for (int it = threadIdx.x; it < G * rest; it += blockDim.x) {
        const int g = it / rest, i = rot_dim + (it - g * rest);
        kdst[g * D + i] = krow[g * D + i];
    }
    for (int it = threadIdx.x; it < G * D; it += blockDim.x) vdst[(size_t)it * page_tokens] = vrow[it];
}

extern "C" int hfa_rope_store(void* qkv, int dtype, int ld, const int* positions, const float* inv_freq, int rot_dim,
                              int n_heads, int n_kv_heads, int head_dim, void* k_cache, void* v_cache,
                              const int* slot_map, int page_tokens, int n_tokens, hipStream_t stream) {
    HFA_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0, "rope_store: bad sizes");
    HFA_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= head_dim,
                "rope_store: rot_dim %d must be even and at most head_dim %d", rot_dim, head_dim);
    HFA_REQUIRE(rot_dim / 2 <= ROPE_MAX_HALF, "rope_store: rot_dim %d exceeds the kernel's limit %d", rot_dim,
                2 * ROPE_MAX_HALF);
    HFA_REQUIRE(rot_dim == 0 || (positions && inv_freq), "rope_store: positions and inv_freq are needed");
    HFA_REQUIRE(ld >= (n_heads + 2 * n_kv_heads) * head_dim, "rope_store: row stride %d is too small", ld);
    HFA_REQUIRE(n_kv_heads == 0 || !slot_map || (k_cache && v_cache && page_tokens > 0),
                "rope_store: no cache to store into");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "rope_store: unknown dtype %d", dtype);
    if (dtype == HFA_F32)
        rope_store_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)qkv, ld, positions, inv_freq, rot_dim, n_heads,
                                                               n_kv_heads, head_dim, (float*)k_cache,
                                                               (float*)v_cache, slot_map, page_tokens);
    else
        rope_store_kernel<bf16><<<n_tokens, 256, 0, stream>>>((bf16*)qkv, ld, positions, inv_freq, rot_dim, n_heads,
                                                              n_kv_heads, head_dim, (bf16*)k_cache, (bf16*)v_cache,
                                                              slot_map, page_tokens);
    HFA_LAUNCH_CHECK("rope_store");
    return 0;
}

// ---- SwiGLU -----------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int width, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / width;
        const int i = (int)(idx - t * width);
        const float g = to_f32(gate_up[t * 2 * width + i]);
        const float u = to_f32(gate_up[t * 2 * width + width + i]);
        out[idx] = from_f32<T>((g / (1.0f + expf(-g))) * u);
    }
}

extern "C" int hfa_swiglu(const void* gate_up, void* out, int dtype, int n_tokens, int width, hipStream_t stream) {
    HFA_REQUIRE(n_tokens > 0 && width > 0, "swiglu: bad sizes tokens=%d width=%d", n_tokens, width);
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "swiglu: unknown dtype %d", dtype);
    const size_t total = (size_t)n_tokens * width;
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == HFA_F32)
        swiglu_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, width, total);
    else
        swiglu_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((const bf16*)gate_up, (bf16*)out, width, total);
    HFA_LAUNCH_CHECK("swiglu");
    return 0;
}

// ---- integer scatter ----------------------------------------------------------------------
__global__ void scatter_i32_kernel(int* __restrict__ dst, const int* __restrict__ idx, const int* __restrict__ val,
                                   int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[idx[i]] = val[i];
}

extern "C" int hfa_scatter_i32(int* dst, const int* idx, const int* val, int n, hipStream_t stream) {
    HFA_REQUIRE(n > 0, "scatter_i32: nothing to scatter");
    scatter_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, idx, val, n);
    HFA_LAUNCH_CHECK("scatter_i32");
    return 0;
}
