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

// Planes of partial sums are fetched this many at a time (all of a batch asked for before the first is added).
// The products of few rows leave about twenty planes; batches of 12 and of 24 changed nothing in a step's time.
#define PLANE_BATCH 8

// ---- RMS norm ---------------------------------------------------------------------------
// One block per output row. The sum of squares is taken in a fixed order (each thread over
// its strided elements, then waves, then the block), so a row's result does not depend on
// which other rows are in the launch.
//
// If the matrix product before the norm left its result as partial sums (K split for small
// M), the kernel first finishes it: x[r, :] += sum over splits + bias, written back, and the
// norm is taken of the new x. This is the fused residual-add + norm of the decode path.
template <typename TO>
__global__ __launch_bounds__(1024) void rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ w,
                                                      TO* __restrict__ out, const int* __restrict__ rows, int width,
                                                      float eps, const float* __restrict__ partial, int splits,
                                                      const float* __restrict__ pbias, int n_rows) {
    __shared__ float red[17];
    const int r = blockIdx.x;
    const int xr = rows ? rows[r] : r;
    float* src = x + (size_t)xr * width;
    float ss = 0.f;
    const bool vec = (width & 3) == 0;
    // Few rows (decode): a thread has four values only, which stay in registers for the second
    // half; the scale's weights are asked for before the sum's barriers, and the four results
    // leave in one store.
    const bool one_pass = vec && (int)blockDim.x * 4 >= width;
    float4 keep = make_float4(0.f, 0.f, 0.f, 0.f), g4 = keep;
    if (one_pass && (int)threadIdx.x * 4 < width) g4 = *reinterpret_cast<const float4*>(w + threadIdx.x * 4);
    if (vec) {
        for (int i = threadIdx.x * 4; i < width; i += blockDim.x * 4) {
            float4 v = *reinterpret_cast<const float4*>(src + i);
            if (splits > 0) {
                // loads in batches of 8 that do not wait for one another, added in ascending order
                for (int s0 = 0; s0 < splits; s0 += PLANE_BATCH) {
                    float4 p[PLANE_BATCH];
#pragma unroll
                    for (int u = 0; u < PLANE_BATCH; u++)
                        p[u] = s0 + u < splits
                                   ? *reinterpret_cast<const float4*>(partial + ((size_t)(s0 + u) * n_rows + xr) * width + i)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                    for (int u = 0; u < PLANE_BATCH; u++) { v.x += p[u].x; v.y += p[u].y; v.z += p[u].z; v.w += p[u].w; }
                }
                if (pbias) {
                    const float4 b = *reinterpret_cast<const float4*>(pbias + i);
                    v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
                }
                *reinterpret_cast<float4*>(src + i) = v;
            }
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
            keep = v;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            float v = src[i];
            if (splits > 0) {
                for (int s = 0; s < splits; s++) v += partial[((size_t)s * n_rows + xr) * width + i];
                if (pbias) v += pbias[i];
                src[i] = v;
            }
            ss += v * v;
        }
    }
    ss = block_sum(ss, red);            // its barriers also order the writes of x before the reads below
    const float scale = 1.0f / sqrtf(ss / (float)width + eps);
    TO* dst = out + (size_t)r * width;
    if (one_pass) {
        const int i = threadIdx.x * 4;
        if (i < width) {
            const TO o0 = from_f32<TO>((keep.x * scale) * g4.x), o1 = from_f32<TO>((keep.y * scale) * g4.y);
            const TO o2 = from_f32<TO>((keep.z * scale) * g4.z), o3 = from_f32<TO>((keep.w * scale) * g4.w);
            if constexpr (sizeof(TO) == 2) {
                uint2 pk;
                pk.x = (uint32_t)o0.bits | ((uint32_t)o1.bits << 16);
                pk.y = (uint32_t)o2.bits | ((uint32_t)o3.bits << 16);
                *reinterpret_cast<uint2*>(dst + i) = pk;
            } else {
                dst[i] = o0; dst[i + 1] = o1; dst[i + 2] = o2; dst[i + 3] = o3;
            }
        }
    } else if (vec) {
        for (int i = threadIdx.x * 4; i < width; i += blockDim.x * 4) {
            const float4 v = *reinterpret_cast<const float4*>(src + i);
            const float4 g = *reinterpret_cast<const float4*>(w + i);
            dst[i] = from_f32<TO>((v.x * scale) * g.x);
            dst[i + 1] = from_f32<TO>((v.y * scale) * g.y);
            dst[i + 2] = from_f32<TO>((v.z * scale) * g.z);
            dst[i + 3] = from_f32<TO>((v.w * scale) * g.w);
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_f32<TO>((src[i] * scale) * w[i]);
    }
}

extern "C" int hfa_rmsnorm(float* x, const float* w, void* out, int out_dtype, const int* rows, int n_rows,
                           int width, float eps, const float* partial, int splits, const float* partial_bias,
                           hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", n_rows, width);
    HFA_REQUIRE(out_dtype == HFA_F32 || out_dtype == HFA_BF16, "rmsnorm: unknown dtype %d", out_dtype);
    HFA_REQUIRE(splits >= 0 && (splits == 0 || (partial && !rows)),
                "rmsnorm: partial sums cannot be combined with a choice of rows");
    int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
    if (n_rows <= 64 && (width & 3) == 0) {                 // few rows: one pass of 4 values per thread if possible
        threads = ((width / 4 + WAVE - 1) / WAVE) * WAVE;
        threads = threads > 1024 ? 1024 : threads;
    }
    if (out_dtype == HFA_F32)
        rmsnorm_kernel<float><<<n_rows, threads, 0, stream>>>(x, w, (float*)out, rows, width, eps, partial, splits,
                                                              partial_bias, n_rows);
    else
        rmsnorm_kernel<bf16><<<n_rows, threads, 0, stream>>>(x, w, (bf16*)out, rows, width, eps, partial, splits,
                                                             partial_bias, n_rows);
    HFA_LAUNCH_CHECK("rmsnorm");
    return 0;
}

// ---- rotary encoding + cache store ------------------------------------------------------------
// If the q/k/v product left its result as partial sums ([splits][T][width] fp32), the kernel
// finishes it on the way: every value it reads is the sum over the splits plus the bias, and the
// rotated queries are written into qkv as if the product had stored them.
template <typename T>
struct QkvSource {
    const T* row;
    const float* partial;
    const float* bias;
    size_t split_stride;
    int splits;
    __device__ __forceinline__ float at(int c) const {
        if (splits == 0) return to_f32(row[c]);
        float v = 0.f;
        for (int s0 = 0; s0 < splits; s0 += PLANE_BATCH) {           // batches of loads that do not wait for one another
            float p[PLANE_BATCH];
#pragma unroll
            for (int u = 0; u < PLANE_BATCH; u++) p[u] = s0 + u < splits ? partial[(s0 + u) * split_stride + c] : 0.f;
#pragma unroll
            for (int u = 0; u < PLANE_BATCH; u++) v += p[u];
        }
        return bias ? v + bias[c] : v;
    }
};

// One block per (token, head slot): slots 0 .. H-1 are the query heads, H .. H+G-1 the key
// heads, H+G .. H+2G-1 the value heads, so that a single decoded token still spreads over the
// machine. Cosines and sines of the token's angles are computed by each block that rotates;
// the angle is the fp32 product of the position and the fp32 inverse frequency.
template <typename T>
__global__ __launch_bounds__(128) void rope_store_kernel(
    T* __restrict__ qkv, int ld, const int* __restrict__ positions, const float* __restrict__ inv_freq, int rot_dim,
    int H, int G, int D, int Dv, T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ slot_map,
    int page_tokens, const float* __restrict__ partial, int splits, const float* __restrict__ pbias, int n_tokens) {
    const int t = blockIdx.x, hs = blockIdx.y;
    const int half = rot_dim / 2, rest = D - rot_dim;
    const int width = (H + G) * D + G * Dv;                   // value heads may have a size of their own
    QkvSource<T> in = {qkv + (size_t)t * ld, partial + (size_t)t * width, pbias, (size_t)n_tokens * width, splits};
    T* row = qkv + (size_t)t * ld;
    const int slot = (G > 0 && slot_map) ? slot_map[t] : -1;
    if (hs >= H + G) {                                        // a value head: copy, transposed inside the page
        const int c0 = (hs - H - G) * Dv, vbase = (H + G) * D + c0;
        if (slot < 0) {
            if (splits > 0)
                for (int i = threadIdx.x; i < Dv; i += blockDim.x) row[vbase + i] = from_f32<T>(in.at(vbase + i));
            return;
        }
        T* vdst = v_cache + (size_t)(slot / page_tokens) * page_tokens * (G * Dv) + slot % page_tokens;
        for (int i = threadIdx.x; i < Dv; i += blockDim.x)
            vdst[(size_t)(c0 + i) * page_tokens] = from_f32<T>(in.at(vbase + i));
        return;
    }
    const int base = hs * D;                                  // first column of this head in the row
    // a query or key head: rotate; keys go to the cache (or stay in the row if there is no cache row)
    const bool is_key = hs >= H;
    T* dst = (is_key && slot >= 0) ? k_cache + (size_t)slot * (G * D) + (hs - H) * D : row + base;
    const float pos = half > 0 ? (float)positions[t] : 0.f;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        const float x0 = in.at(base + i), x1 = in.at(base + i + half);
        dst[i] = from_f32<T>(x0 * cs - x1 * sn);
        dst[i + half] = from_f32<T>(x0 * sn + x1 * cs);
    }
    if (splits > 0 || dst != row + base)                      // dimensions that are not rotated pass through
        for (int i = rot_dim + threadIdx.x; i < D; i += blockDim.x) dst[i] = from_f32<T>(in.at(base + i));
    (void)rest;
}

// The same for prompt portions in bf16: a block takes 8 consecutive tokens. The angles of a token
// are computed once (not once per head), queries and keys move 16 bytes per lane, and the
// values of the 8 tokens go through LDS so that, where the tokens' cache rows are 8 consecutive
// rows of one page, every value column is written with one 16-byte store instead of eight
// 2-byte stores 2 * page_tokens bytes apart.
#define ROPE_TOKENS 8
#define ROPE_ROWS_FROM 512      // fewer tokens make too few blocks of 8: the kernel above spreads them better
__global__ __launch_bounds__(256) void rope_store_rows_kernel(
    uint16_t* __restrict__ qkv, int ld, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    int rot_dim, int H, int G, int D, uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
    const int* __restrict__ slot_map, int page_tokens, int n_tokens) {
    extern __shared__ __attribute__((aligned(16))) unsigned char rope_lds[];
    const int half = rot_dim / 2, KD = G * D;
    float* cs = reinterpret_cast<float*>(rope_lds);                          // [ROPE_TOKENS][half] cosines, then sines
    float* sn = cs + ROPE_TOKENS * half;
    uint16_t* vt = reinterpret_cast<uint16_t*>(sn + ROPE_TOKENS * half);     // [ROPE_TOKENS][KD] values
    int* slots = reinterpret_cast<int*>(vt + ROPE_TOKENS * KD);              // [ROPE_TOKENS]
    const int t0 = blockIdx.x * ROPE_TOKENS;
    const int nt = n_tokens - t0 < ROPE_TOKENS ? n_tokens - t0 : ROPE_TOKENS;
    const int tid = threadIdx.x;
    const bool store = G > 0 && slot_map != nullptr;
    for (int i = tid; i < nt * half; i += blockDim.x) {
        const int t = i / half, j = i % half;
        sincosf((float)positions[t0 + t] * inv_freq[j], &sn[i], &cs[i]);
    }
    if (tid < ROPE_TOKENS) slots[tid] = (store && tid < nt) ? slot_map[t0 + tid] : -1;
    if (store)                                                               // values: rows into LDS
        for (int i = tid; i < nt * (KD / 8); i += blockDim.x) {
            const int t = i / (KD / 8), c = (i % (KD / 8)) * 8;
            *reinterpret_cast<uint4*>(vt + t * KD + c) =
                *reinterpret_cast<const uint4*>(qkv + (size_t)(t0 + t) * ld + (H + G) * D + c);
        }
    __syncthreads();
    // queries and keys: 8 pairs (i, i + half) per item
    const int heads = H + G, per_head = half / 8;
    for (int i = tid; i < nt * heads * per_head; i += blockDim.x) {
        const int t = i / (heads * per_head), r = i % (heads * per_head), h = r / per_head, j = (r % per_head) * 8;
        uint16_t* src = qkv + (size_t)(t0 + t) * ld + h * D;
        uint16_t* dst = src;
        if (h >= H && store) dst = k_cache + (size_t)slots[t] * KD + (h - H) * D;
        uint4 a = *reinterpret_cast<const uint4*>(src + j), b = *reinterpret_cast<const uint4*>(src + j + half);
        uint16_t* pa = reinterpret_cast<uint16_t*>(&a);
        uint16_t* pb = reinterpret_cast<uint16_t*>(&b);
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const float x0 = __uint_as_float((uint32_t)pa[u] << 16), x1 = __uint_as_float((uint32_t)pb[u] << 16);
            const float c = cs[t * half + j + u], s1 = sn[t * half + j + u];
            pa[u] = bf16_bits(x0 * c - x1 * s1);
            pb[u] = bf16_bits(x0 * s1 + x1 * c);
        }
        *reinterpret_cast<uint4*>(dst + j) = a;
        *reinterpret_cast<uint4*>(dst + j + half) = b;
    }
    if (!store) return;
    // dimensions of the keys that are not rotated pass through to the cache
    const int rest = (D - rot_dim) / 8;
    for (int i = tid; i < nt * G * rest; i += blockDim.x) {
        const int t = i / (G * rest), r = i % (G * rest), g = r / rest, j = rot_dim + (r % rest) * 8;
        *reinterpret_cast<uint4*>(k_cache + (size_t)slots[t] * KD + g * D + j) =
            *reinterpret_cast<const uint4*>(qkv + (size_t)(t0 + t) * ld + (H + g) * D + j);
    }
    // values, transposed inside their page
    bool run = nt == ROPE_TOKENS && page_tokens % 8 == 0 && slots[0] % 8 == 0;
    for (int t = 1; run && t < ROPE_TOKENS; t++) run = slots[t] == slots[0] + t;
    if (run) {
        uint16_t* page = v_cache + (size_t)(slots[0] / page_tokens) * page_tokens * KD + slots[0] % page_tokens;
        for (int c = tid; c < KD; c += blockDim.x) {
            uint4 out;
            uint16_t* po = reinterpret_cast<uint16_t*>(&out);
#pragma unroll
            for (int t = 0; t < ROPE_TOKENS; t++) po[t] = vt[t * KD + c];
            *reinterpret_cast<uint4*>(page + (size_t)c * page_tokens) = out;
        }
    } else {
        for (int i = tid; i < nt * KD; i += blockDim.x) {
            const int t = i / KD, c = i % KD, slot = slots[t];
            v_cache[(size_t)(slot / page_tokens) * page_tokens * KD + (size_t)c * page_tokens + slot % page_tokens] = vt[i];
        }
    }
}

extern "C" int hfa_rope_store(void* qkv, int dtype, int ld, const int* positions, const float* inv_freq, int rot_dim,
                              int n_heads, int n_kv_heads, int head_dim, int v_head_dim, void* k_cache, void* v_cache,
                              const int* slot_map, int page_tokens, int n_tokens, const float* partial, int splits,
                              const float* partial_bias, hipStream_t stream) {
    HFA_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv_heads >= 0 && head_dim > 0 && v_head_dim > 0, "rope_store: bad sizes");
    HFA_REQUIRE(rot_dim >= 0 && rot_dim % 2 == 0 && rot_dim <= head_dim,
                "rope_store: rot_dim %d must be even and at most head_dim %d", rot_dim, head_dim);
    HFA_REQUIRE(rot_dim == 0 || (positions && inv_freq), "rope_store: positions and inv_freq are needed");
    HFA_REQUIRE(ld >= (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_head_dim, "rope_store: row stride %d is too small", ld);
    HFA_REQUIRE(n_kv_heads == 0 || !slot_map || (k_cache && v_cache && page_tokens > 0),
                "rope_store: no cache to store into");
    HFA_REQUIRE(dtype == HFA_F32 || dtype == HFA_BF16, "rope_store: unknown dtype %d", dtype);
    HFA_REQUIRE(splits >= 0 && (splits == 0 || partial), "rope_store: partial sums announced but not given");
    HFA_REQUIRE(n_heads + 2 * n_kv_heads <= 65535, "rope_store: too many heads for the grid");
    const int kd = n_kv_heads * head_dim;
    const size_t rows_lds = (size_t)ROPE_TOKENS * rot_dim * sizeof(float) + (size_t)ROPE_TOKENS * kd * 2 + ROPE_TOKENS * sizeof(int);
    if (dtype == HFA_BF16 && splits == 0 && n_tokens >= ROPE_ROWS_FROM && rot_dim > 0 && rot_dim % 16 == 0 && v_head_dim == head_dim &&
        head_dim % 8 == 0 && ld % 8 == 0 && ((uintptr_t)qkv & 15) == 0 && ((uintptr_t)k_cache & 15) == 0 &&
        ((uintptr_t)v_cache & 15) == 0 && rows_lds <= 48 * 1024) {
        rope_store_rows_kernel<<<(n_tokens + ROPE_TOKENS - 1) / ROPE_TOKENS, 256, rows_lds, stream>>>(
            (uint16_t*)qkv, ld, positions, inv_freq, rot_dim, n_heads, n_kv_heads, head_dim, (uint16_t*)k_cache,
            (uint16_t*)v_cache, slot_map, page_tokens, n_tokens);
        HFA_LAUNCH_CHECK("rope_store");
        return 0;
    }
    const dim3 grid(n_tokens, n_heads + 2 * n_kv_heads);
    const int threads = head_dim >= 128 ? 128 : 64;
    if (dtype == HFA_F32)
        rope_store_kernel<float><<<grid, threads, 0, stream>>>((float*)qkv, ld, positions, inv_freq, rot_dim, n_heads,
                                                               n_kv_heads, head_dim, v_head_dim, (float*)k_cache,
                                                               (float*)v_cache, slot_map, page_tokens, partial,
                                                               splits, partial_bias, n_tokens);
    else
        rope_store_kernel<bf16><<<grid, threads, 0, stream>>>((bf16*)qkv, ld, positions, inv_freq, rot_dim, n_heads,
                                                              n_kv_heads, head_dim, v_head_dim, (bf16*)k_cache, (bf16*)v_cache,
                                                              slot_map, page_tokens, partial, splits, partial_bias,
                                                              n_tokens);
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

// dst[dst_idx[i]] = src[src_idx[i]]: a step's tokens that were sampled on the device and never went to the host.
__global__ void move_i32_kernel(int* __restrict__ dst, const int* __restrict__ dst_idx, const int* __restrict__ src,
                                const int* __restrict__ src_idx, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[dst_idx[i]] = src[src_idx[i]];
}

extern "C" int hfa_move_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream) {
    HFA_REQUIRE(n > 0 && dst && dst_idx && src && src_idx, "move_i32: nothing to move");
    move_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, dst_idx, src, src_idx, n);
    HFA_LAUNCH_CHECK("move_i32");
    return 0;
}

// ---- random weights -------------------------------------------------------------------------
// Element e of the tensor with `key`: the two words mix(key + 2e), mix(key + 2e + 1) with the
// finishing function of splitmix64; their eight 16-bit fields added up, less the mean 262140, as an
// exact fp32 integer times `scale` (rule 0), 1 + that (rule 1), or the first word modulo `bound`
// (rule 2). Integers and single fp32 operations only, so the host computes the same bits.
#pragma clang fp contract(off)        // to the end of the file: 1 + x * scale is a product and a sum, each rounded
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

__global__ void random_fill_kernel(void* __restrict__ out, int dtype, size_t n, uint64_t key, float scale, int rule,
                                   uint32_t bound) {
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
        const uint64_t a = mix64(key + 2 * (uint64_t)e);
        if (rule == 2) {
            reinterpret_cast<int*>(out)[e] = (int)(a % bound);
            continue;
        }
        const uint64_t b = mix64(key + 2 * (uint64_t)e + 1);
        int total = 0;
#pragma unroll
        for (int s = 0; s < 64; s += 16) total += (int)((a >> s) & 0xffff) + (int)((b >> s) & 0xffff);
        float v = (float)(total - 262140) * scale;
        if (rule == 1) v = 1.0f + v;
        if (dtype == HFA_F32)
            reinterpret_cast<float*>(out)[e] = v;
        else
            reinterpret_cast<uint16_t*>(out)[e] = bf16_bits(v);
    }
}

extern "C" int hfa_random_fill(void* out, int dtype, size_t n, uint64_t key, float scale, int rule, int bound,
                               hipStream_t stream) {
    HFA_REQUIRE(out != nullptr && n > 0, "random_fill: nothing to fill");
    HFA_REQUIRE(rule >= 0 && rule <= 2, "random_fill: unknown rule %d", rule);
    HFA_REQUIRE(rule == 2 ? (dtype == 2 && bound > 0) : (dtype == HFA_F32 || dtype == HFA_BF16),
                "random_fill: rule %d does not fit dtype %d (bound %d)", rule, dtype, bound);
    size_t blocks = (n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    random_fill_kernel<<<(int)blocks, 256, 0, stream>>>(out, dtype, n, key, scale, rule, (uint32_t)bound);
    HFA_LAUNCH_CHECK("random_fill");
    return 0;
}
