// Kernels of the sampler: the greedy choice, and the ordered best-k of a row with the
// row's log-sum-exp, from which the host finishes temperature / top-k / top-p / min-p
// sampling exactly in the reference's order of operations.
#include <mutex>

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

// ---- the greedy choice for callers that cannot allocate ---------------------------------------
// hfa_argmax_static is hfa_argmax with the first stage's candidates in a buffer that the library
// itself holds: a file-scope device array, so nobody allocates, the caller brings no workspace, and
// the call may sit in code that is captured into a graph or that forbids hipMalloc. Every GPU the
// library runs on holds its own copy of the array (HFA_ARGMAX_STATIC_ROWS x 64 candidates of 8
// bytes = 128 KiB) at its own address until the process ends. In host code the array's name is
// only a stand-in: the address a kernel can use comes from hipGetSymbolAddress, asked once per
// device with that device current, and host code uses nothing else.
// The first stage writes every candidate that the second stage reads, so nothing has to be cleared
// between calls; the array keeps the last call's candidates. Calls that overlap on one GPU (two
// streams, two threads) share the array and race: callers keep them in order.
static __device__ __align__(256) unsigned char scratch[(size_t)HFA_ARGMAX_STATIC_ROWS * ARGMAX_PARTS * 8];

#define HFA_MAX_DEVICES 64
static void* scratch_of_device[HFA_MAX_DEVICES];      // device address of `scratch` per GPU, null = not asked yet
static std::mutex scratch_lock;

static int scratch_address(void** out, hipStream_t stream) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= HFA_MAX_DEVICES) {
        hfa_set_error("argmax_static: no current device (%s, device %d)", hipGetErrorString(e), dev);
        return 2;
    }
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (scratch_of_device[dev] == nullptr) {
        // Asking for the address may load the code object and is no stream operation: under a capture it
        // could fail or break the capture. The first call on a device therefore has to be an eager one.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &capturing);
        if (e != hipSuccess || capturing != hipStreamCaptureStatusNone) {
            hfa_set_error("argmax_static: the first call on device %d came while its stream is being captured; call it "
                          "once eagerly on this device before capturing it into a graph", dev);
            return 1;
        }
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));       // for the current device
        if (e != hipSuccess || ptr == nullptr) {
            hfa_set_error("argmax_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return 2;
        }
        scratch_of_device[dev] = ptr;
    }
    *out = scratch_of_device[dev];
    return 0;
}

extern "C" int hfa_argmax_static(const float* logits, int ld, int* out, int n_rows, int vocab, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "argmax_static: bad sizes rows=%d vocab=%d ld=%d", n_rows, vocab, ld);
    HFA_REQUIRE(n_rows <= HFA_ARGMAX_STATIC_ROWS,
                "argmax_static: %d rows, the library's own buffer holds the candidates of %d (use hfa_argmax with a "
                "workspace for more)", n_rows, HFA_ARGMAX_STATIC_ROWS);
    HFA_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: null logits or output");
    void* ptr = nullptr;
    if (int rc = scratch_address(&ptr, stream)) return rc;
    float* part_v = (float*)ptr;
    int* part_i = (int*)(part_v + (size_t)n_rows * ARGMAX_PARTS);
    argmax_part_kernel<<<dim3(n_rows, ARGMAX_PARTS), 256, 0, stream>>>(logits, ld, vocab, part_v, part_i);
    argmax_final_kernel<<<n_rows, WAVE, 0, stream>>>(part_v, part_i, out);
    HFA_LAUNCH_CHECK("argmax_static");
    return 0;
}

// Ordered best-k of a row, one block of 1024 threads per row.
//
// The short way, two passes over the row: the first finds every thread's own maximum (and from them
// the row's); the k-th largest of these 1024 maxima cannot lie above the row's k-th largest value, so
// the second pass, which also adds up exp(l - max) for the log-sum-exp, collects the values that
// reach it: at least k, and for logits without heavy ties hardly more. If at most 1024 were
// collected they are sorted in LDS by (logit descending, id ascending) and the first k are the answer.
//
// Otherwise (ties by the thousand, or a k near 1024) the long way, in a fixed number of passes
// over the row (which stays in L2) whatever k is:
//  1. the k-th largest value is found by three histogram passes over the order-preserving
//     integer image of the floats (11 + 11 + 10 bits);
//  2. two sweeps collect the values above it and, of the values equal to it, those with the
//     smallest ids until k are together: each wave owns a contiguous segment of the row and
//     walks it 64 ids at a time, so ballots and counts give every candidate its place in id
//     order without atomics;
//  3. the k candidates are sorted in LDS (bitonic) by (logit descending, id ascending).
#define TOPK_THREADS 1024
#define TOPK_MAX 1024

__device__ __forceinline__ uint32_t float_key(float v) {     // larger float <=> larger key; -0 and 0 are one value
    const uint32_t u = __float_as_uint(v + 0.0f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Among the histogram's bins, from the top: the bin that holds the `rank`-th largest element
// (rank counts from 1). Returns the bin; `rank` becomes the rank inside that bin. All threads
// call it; `hist` and `pick` are LDS.
__device__ int topk_find_bin(const uint32_t* hist, int n_bins, int& rank, int* pick) {
    __syncthreads();
    if (threadIdx.x < WAVE) {
        const int per = n_bins / WAVE, lane = threadIdx.x;
        uint32_t c = 0;
        for (int j = 0; j < per; j++) c += hist[lane * per + j];
        // elements in chunks above this lane's
        uint32_t above = 0;
        for (int l = WAVE - 1; l >= 0; l--) {
            const uint32_t cl = __shfl(c, l, WAVE);
            if (l > lane) above += cl;
        }
        if (above < (uint32_t)rank && (uint32_t)rank <= above + c) {     // exactly one lane
            uint32_t seen = above;
            int bin = lane * per + per - 1;
            for (; bin > lane * per; bin--) {
                if (seen + hist[bin] >= (uint32_t)rank) break;
                seen += hist[bin];
            }
            pick[0] = bin;
            pick[1] = rank - (int)seen;
        }
    }
    __syncthreads();
    rank = pick[1];
    return pick[0];
}

// `found` candidates in LDS, sorted by (logit descending, id ascending) with a bitonic network over
// n <= 1024 entries, one thread per entry; the first k go to the row's output. All threads call it.
__device__ void topk_sort_and_store(float* cand_v, int* cand_i, int found, int k, int* __restrict__ ids,
                                    float* __restrict__ vals) {
    const int tid = threadIdx.x;
    int n = 2;
    while (n < found) n <<= 1;
    for (int i = found + tid; i < n; i += TOPK_THREADS) {    // padding sorts to the end
        cand_v[i] = -INFINITY;
        cand_i[i] = 0x7fffffff;
    }
    for (int size = 2; size <= n; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            const int j = tid ^ stride;
            if (tid < n && j > tid) {
                const bool forward = (tid & size) == 0;      // this pair's better entry goes first
                const float va = cand_v[tid], vb = cand_v[j];
                const int ia = cand_i[tid], ib = cand_i[j];
                if (better(vb, ib, va, ia) == forward) {
                    cand_v[tid] = vb; cand_i[tid] = ib;
                    cand_v[j] = va; cand_i[j] = ia;
                }
            }
        }
    __syncthreads();
    for (int c = tid; c < k; c += TOPK_THREADS) {
        ids[(size_t)blockIdx.x * k + c] = cand_i[c] == 0x7fffffff ? -1 : cand_i[c];
        vals[(size_t)blockIdx.x * k + c] = cand_v[c];
    }
}

__global__ __launch_bounds__(TOPK_THREADS) void topk_kernel(const float* __restrict__ logits, int ld,
                                                            int* __restrict__ ids, float* __restrict__ vals,
                                                            float* __restrict__ stats, int vocab, int k) {
    __shared__ uint32_t hist[2048];
    __shared__ float cand_v[TOPK_MAX];
    __shared__ int cand_i[TOPK_MAX];
    __shared__ int pick[2];
    __shared__ int wave_above[TOPK_THREADS / WAVE + 1], wave_equal[TOPK_THREADS / WAVE + 1];
    __shared__ float red[17];
    const float* row = logits + (size_t)blockIdx.x * ld;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    constexpr int NW = TOPK_THREADS / WAVE;

    // ---- the row's maximum, and every thread's own ----
    __shared__ int n_cand;
    float mx = -INFINITY;
    constexpr int AT_ONCE = 8;                               // loads of a thread on their way together
    for (int i0 = tid; i0 < vocab; i0 += AT_ONCE * TOPK_THREADS) {
        float v[AT_ONCE];
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++) v[u] = i0 + u * TOPK_THREADS < vocab ? row[i0 + u * TOPK_THREADS] : -INFINITY;
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++) mx = fmaxf(mx, v[u]);
    }
    const float own = mx;
    mx = block_max(mx, red);
    float least = INFINITY;                                  // what a candidate of the short way has to reach
    if (k > 0) {
        cand_v[tid] = own;                                   // the 1024 maxima, largest first
        for (int size = 2; size <= TOPK_THREADS; size <<= 1)
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                __syncthreads();
                const int j = tid ^ stride;
                if (j > tid) {
                    const float va = cand_v[tid], vb = cand_v[j];
                    if ((vb > va) == ((tid & size) == 0)) { cand_v[tid] = vb; cand_v[j] = va; }
                }
            }
        __syncthreads();
        least = cand_v[k - 1];
        if (tid == 0) n_cand = 0;
        __syncthreads();                                     // all have read it before the list is filled again
    }

    // ---- the sum of exp(l - max), and the candidates of the short way ----
    float sum = 0.f;
    bool full = false;                                       // this thread met a full list: it stops offering
    for (int i0 = tid; i0 < vocab; i0 += AT_ONCE * TOPK_THREADS) {
        float v[AT_ONCE];
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++) v[u] = i0 + u * TOPK_THREADS < vocab ? row[i0 + u * TOPK_THREADS] : -INFINITY;
#pragma unroll
        for (int u = 0; u < AT_ONCE; u++) {                  // in ascending order of the ids, as one by one
            const int i = i0 + u * TOPK_THREADS;
            if (i >= vocab) break;
            sum += expf(v[u] - mx);
            if (!full && v[u] >= least) {
                const int at = atomicAdd(&n_cand, 1);
                if (at < TOPK_MAX) { cand_v[at] = v[u]; cand_i[at] = i; }
                else full = true;
            }
        }
    }
    sum = block_sum(sum, red);
    if (stats && tid == 0) {
        stats[2 * blockIdx.x] = mx;
        stats[2 * blockIdx.x + 1] = logf(sum);
    }
    if (k == 0) return;
    __syncthreads();
    const int found = n_cand;
    if (found >= k && found <= TOPK_MAX) {
        topk_sort_and_store(cand_v, cand_i, found, k, ids, vals);
        return;
    }
    __syncthreads();

    // ---- the long way. Pass 1: top 11 bits ----
    for (int i = tid; i < 2048; i += TOPK_THREADS) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < vocab; i += TOPK_THREADS) atomicAdd(&hist[float_key(row[i]) >> 21], 1u);
    int rank = k;
    uint32_t prefix = (uint32_t)topk_find_bin(hist, 2048, rank, pick);

    // ---- pass 2: the next 11 bits among the elements of that bin ----
    for (int i = tid; i < 2048; i += TOPK_THREADS) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < vocab; i += TOPK_THREADS) {
        const uint32_t key = float_key(row[i]);
        if ((key >> 21) == prefix) atomicAdd(&hist[(key >> 10) & 0x7ffu], 1u);
    }
    prefix = (prefix << 11) | (uint32_t)topk_find_bin(hist, 2048, rank, pick);

    // ---- pass 3: the last 10 bits ----
    for (int i = tid; i < 1024; i += TOPK_THREADS) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < vocab; i += TOPK_THREADS) {
        const uint32_t key = float_key(row[i]);
        if ((key >> 10) == prefix) atomicAdd(&hist[key & 0x3ffu], 1u);
    }
    const uint32_t kth = (prefix << 10) | (uint32_t)topk_find_bin(hist, 1024, rank, pick);
    const int n_equal = rank, n_above = k - rank;            // of the values equal to the k-th, the `rank` smallest ids

    // ---- sweep 1: how many candidates each wave's segment holds ----
    const int seg = (vocab + NW - 1) / NW;
    const int lo = wave * seg, hi = lo + seg < vocab ? lo + seg : vocab;
    int above = 0, equal = 0;
    for (int i = lo + lane; i < hi; i += WAVE) {
        const uint32_t key = float_key(row[i]);
        above += key > kth;
        equal += key == kth;
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        above += __shfl_xor(above, off, WAVE);
        equal += __shfl_xor(equal, off, WAVE);
    }
    if (lane == 0) { wave_above[wave] = above; wave_equal[wave] = equal; }
    __syncthreads();
    int base_above = 0, base_equal = 0;                      // candidates in the segments before this wave's
    for (int w = 0; w < wave; w++) { base_above += wave_above[w]; base_equal += wave_equal[w]; }

    // ---- sweep 2: every candidate to its place: the values above first, then the ties in id order ----
    for (int i0 = lo; i0 < hi; i0 += WAVE) {
        const int i = i0 + lane;
        const float v = i < hi ? row[i] : 0.f;
        const uint32_t key = float_key(v);
        const bool is_above = i < hi && key > kth, is_equal = i < hi && key == kth;
        const unsigned long long ma = __ballot(is_above), me = __ballot(is_equal);
        const unsigned long long below = (1ull << lane) - 1ull;
        if (is_above) {
            const int at = base_above + __popcll(ma & below);
            cand_v[at] = v;
            cand_i[at] = i;
        }
        if (is_equal) {
            const int r = base_equal + __popcll(me & below);
            if (r < n_equal) {
                cand_v[n_above + r] = v;
                cand_i[n_above + r] = i;
            }
        }
        base_above += __popcll(ma);
        base_equal += __popcll(me);
    }
    __syncthreads();
    topk_sort_and_store(cand_v, cand_i, k, k, ids, vals);
}

extern "C" int hfa_topk(const float* logits, int ld, int* ids, float* vals, float* stats, int n_rows, int vocab,
                        int k, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "topk: bad sizes rows=%d vocab=%d ld=%d", n_rows, vocab, ld);
    HFA_REQUIRE(k >= 0 && k <= 1024 && k <= vocab, "topk: k=%d is outside 0..min(1024, vocab)", k);
    HFA_REQUIRE(k == 0 || (ids && vals), "topk: no output for the candidates");
    topk_kernel<<<n_rows, TOPK_THREADS, 0, stream>>>(logits, ld, ids, vals, stats, vocab, k);
    HFA_LAUNCH_CHECK("topk");
    return 0;
}

// ---- a whole row in order --------------------------------------------------------------------
// All candidates of a row in the order (logit descending, id ascending): what the reference's
// qsort gives when top-k is off (src/sample.c:59-64, 93-98). One block of 1024 threads per chosen
// row sorts the order-reversing integer image of its logits by least-significant-digit radix
// sort, four passes of eight bits, each of them stable (so equal logits keep their ids' order):
//  - a histogram of the digit over the row gives every digit its first place;
//  - the row is then walked 1024 elements at a time in its present order. Inside a wave eight
//    ballots tell each lane which lanes before it hold the same digit; the waves' counts per
//    digit meet in LDS, and a prefix over the waves gives every element its place.
// The passes go back and forth between two scratch rows of (key, id) pairs; the last pass writes
// ids and logits. No atomics decide a place: the result is the same in every run.
#define ORDER_THREADS 1024
#define ORDER_WAVES (ORDER_THREADS / WAVE)

__device__ __forceinline__ float key_float(uint32_t k) {     // inverse of float_key
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__global__ __launch_bounds__(ORDER_THREADS) void order_rows_kernel(const float* __restrict__ logits, int ld,
                                                                   const int* __restrict__ rows, int vocab,
                                                                   uint2* __restrict__ scratch, int* __restrict__ ids,
                                                                   float* __restrict__ vals) {
    __shared__ uint32_t first[256];                           // next free place of each digit
    __shared__ uint32_t wave_cnt[ORDER_WAVES][256];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    const int out_row = blockIdx.x;
    const float* src_row = logits + (size_t)(rows ? rows[out_row] : out_row) * ld;
    uint2* buf[2] = {scratch + (size_t)out_row * 2 * vocab, scratch + ((size_t)out_row * 2 + 1) * vocab};
    int* ids_row = ids + (size_t)out_row * vocab;
    float* vals_row = vals + (size_t)out_row * vocab;
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (WAVE - lane));

    for (int pass = 0; pass < 4; pass++) {
        const int shift = 8 * pass;
        const uint2* from = pass == 0 ? nullptr : buf[(pass - 1) & 1];
        uint2* to = buf[pass & 1];
        auto element = [&](int i) {                            // (key, id) number i of the present order
            if (pass == 0) return make_uint2(~float_key(src_row[i] + 0.0f), (uint32_t)i);      // -0 counts as 0: a tie
            return from[i];
        };
        // places of the digits
        if (tid < 256) first[tid] = 0;
        __syncthreads();
        for (int i = tid; i < vocab; i += ORDER_THREADS) atomicAdd(&first[(element(i).x >> shift) & 255u], 1u);
        __syncthreads();
        if (tid < WAVE) {                                      // exclusive prefix over 256 counts by one wave
            uint32_t c[4], s = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) { c[j] = first[tid * 4 + j]; s += c[j]; }
            uint32_t incl = s;
#pragma unroll
            for (int off = 1; off < WAVE; off <<= 1) {
                const uint32_t up = __shfl_up(incl, off, WAVE);
                if (lane >= off) incl += up;
            }
            uint32_t run = incl - s;
#pragma unroll
            for (int j = 0; j < 4; j++) { first[tid * 4 + j] = run; run += c[j]; }
        }
        __syncthreads();
        // the stable scatter, 1024 elements of the present order at a time
        for (int c0 = 0; c0 < vocab; c0 += ORDER_THREADS) {
            for (int j = tid; j < ORDER_WAVES * 256; j += ORDER_THREADS) (&wave_cnt[0][0])[j] = 0;
            __syncthreads();
            const int i = c0 + tid;
            const bool valid = i < vocab;
            const uint2 e = valid ? element(i) : make_uint2(0, 0);
            const uint32_t d = (e.x >> shift) & 255u;
            uint64_t same = __ballot(valid);
#pragma unroll
            for (int b = 0; b < 8; b++) {
                const uint64_t set = __ballot(valid && ((d >> b) & 1u));
                same &= ((d >> b) & 1u) ? set : ~set;
            }
            const int rank = __popcll(same & below);
            if (valid && rank == 0) wave_cnt[wave][d] = (uint32_t)__popcll(same);
            __syncthreads();
            if (tid < 256) {                                   // places of this chunk's waves, digit tid
                uint32_t run = first[tid];
#pragma unroll
                for (int w = 0; w < ORDER_WAVES; w++) {
                    const uint32_t c = wave_cnt[w][tid];
                    wave_cnt[w][tid] = run;
                    run += c;
                }
                first[tid] = run;
            }
            __syncthreads();
            if (valid) {
                const uint32_t at = wave_cnt[wave][d] + (uint32_t)rank;
                if (pass < 3) {
                    to[at] = e;
                } else {
                    ids_row[at] = (int)e.y;
                    vals_row[at] = key_float(~e.x);
                }
            }
            __syncthreads();
        }
        __threadfence_block();                                 // the next pass reads what this one wrote
        __syncthreads();
    }
}

extern "C" size_t hfa_order_rows_scratch(int n_rows, int vocab) { return (size_t)n_rows * 2 * vocab * sizeof(uint2); }

extern "C" int hfa_order_rows(const float* logits, int ld, const int* rows, int* ids, float* vals, int n_rows, int vocab,
                              void* scratch, size_t scratch_bytes, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "order_rows: bad sizes rows=%d vocab=%d ld=%d", n_rows, vocab, ld);
    HFA_REQUIRE(scratch && scratch_bytes >= hfa_order_rows_scratch(n_rows, vocab) && ((uintptr_t)scratch & 7) == 0,
                "order_rows: the scratch memory is smaller than two rows of (key, id) pairs for each of %d rows", n_rows);
    order_rows_kernel<<<n_rows, ORDER_THREADS, 0, stream>>>(logits, ld, rows, vocab, (uint2*)scratch, ids, vals);
    HFA_LAUNCH_CHECK("order_rows");
    return 0;
}

// ---- the draw over a whole ordered row ---------------------------------------------------------
// Steps 3 to 6 of the reference's sampler (src/sample.c:99-114) over candidates that are already
// in order: p = exp((l - l_0) / temp) by the reference's own exponential (src/mathx.c:7-32, every
// operation rounded to fp32, nothing fused), the sum of all p as one running fp32 sum in candidate
// order, p / sum, the min-p and top-p cuts, r = u * (running sum of the kept), the first
// candidate whose running sum exceeds r. The running sums are what the reference's loops compute,
// so they are made by one thread, which reads the row from LDS in pieces that all threads fetch;
// everything else is spread over the block. `vals` is overwritten with the probabilities.
#define DRAW_THREADS 1024
#define DRAW_PIECE 4096

// From here to the end of the file no product is fused with a sum (the library is built with
// -ffp-contract=fast-honor-pragmas): one bit of a probability can move a draw to another token.
// The toolchain's own "round to nearest" operators are plain operators compiled outside this
// pragma, which the compiler does join into fused multiply-adds; the ones below are compiled inside it.
#pragma clang fp contract(off)
__device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
__device__ __forceinline__ float add_rn(float a, float b) { return a + b; }
__device__ __forceinline__ float sub_rn(float a, float b) { return a - b; }
__device__ __forceinline__ float div_rn(float a, float b) { return a / b; }

__device__ __forceinline__ float ref_expf(float x) {
    if (x != x) return x;
    if (x > 88.3762626647949f) x = 88.3762626647949f;
    if (x < -87.3365478515625f) return 0.0f;
    const float fx = floorf(add_rn(mul_rn(x, 1.44269504088896341f), 0.5f));
    const int n = (int)fx;
    x = sub_rn(x, mul_rn(fx, 0.693359375f));
    x = sub_rn(x, mul_rn(fx, -2.12194440e-4f));
    const float z = mul_rn(x, x);
    float y = 1.9875691500e-4f;
    y = add_rn(mul_rn(y, x), 1.3981999507e-3f);
    y = add_rn(mul_rn(y, x), 8.3334519073e-3f);
    y = add_rn(mul_rn(y, x), 4.1665795894e-2f);
    y = add_rn(mul_rn(y, x), 1.6666665459e-1f);
    y = add_rn(mul_rn(y, x), 5.0000001201e-1f);
    y = add_rn(add_rn(mul_rn(y, z), x), 1.0f);
    return mul_rn(y, __uint_as_float((uint32_t)(n + 127) << 23));
}

// One thread's running sum of p[0 .. n) in order, started from `start`; stops after the first element
// at which `stop(sum)` holds (returns its index, else n). The pieces pass through `piece` (LDS).
template <class Stop>
__device__ int draw_running(const float* __restrict__ p, int n, float start, float* piece, float* shared2, Stop stop) {
    int hit = n;
    float sum = start;
    for (int c0 = 0; c0 < n; c0 += DRAW_PIECE) {
        const int len = n - c0 < DRAW_PIECE ? n - c0 : DRAW_PIECE;
        __syncthreads();                                      // the piece before is summed
        for (int i = threadIdx.x; i < len; i += DRAW_THREADS) piece[i] = p[c0 + i];
        __syncthreads();
        if (threadIdx.x == 0 && hit == n) {
            for (int i = 0; i < len; i++) {
                sum = add_rn(sum, piece[i]);
                if (stop(sum)) { hit = c0 + i; break; }
            }
            shared2[0] = sum;
            shared2[1] = __int_as_float(hit);
        }
        __syncthreads();
        hit = __float_as_int(shared2[1]);                     // every thread leaves the loop together
        if (hit != n) break;
    }
    __syncthreads();
    return hit;                                               // the sum is in shared2[0]
}

__global__ __launch_bounds__(DRAW_THREADS) void draw_rows_kernel(float* __restrict__ vals, const int* __restrict__ ids,
                                                                 int vocab, const float* __restrict__ params,
                                                                 const int* __restrict__ cuts, int* __restrict__ tokens) {
    __shared__ float piece[DRAW_PIECE];
    __shared__ float shared2[2];
    __shared__ int first_below;
    const int row = blockIdx.x, tid = threadIdx.x;
    float* p = vals + (size_t)row * vocab;
    const int* id = ids + (size_t)row * vocab;
    const float temp = params[4 * row], top_p = params[4 * row + 1], min_p = params[4 * row + 2], u = params[4 * row + 3];
    const int m = cuts[row] < 1 ? 1 : cuts[row] > vocab ? vocab : cuts[row];      // candidates after the top-k cut
    const float l0 = p[0];
    __syncthreads();                                          // p[0] is read by all before it is overwritten
    for (int i = tid; i < m; i += DRAW_THREADS) p[i] = ref_expf(div_rn(sub_rn(p[i], l0), temp));
    __threadfence_block();
    draw_running(p, m, 0.0f, piece, shared2, [](float) { return false; });
    const float total = shared2[0];
    __syncthreads();
    for (int i = tid; i < m; i += DRAW_THREADS) p[i] = div_rn(p[i], total);
    if (tid == 0) first_below = m;
    __threadfence_block();
    __syncthreads();
    int kept = m;
    if (min_p > 0.0f) {                                       // the leading run with p >= min_p * p_0, at least one
        const float least = mul_rn(min_p, p[0]);
        int mine = m;
        for (int i = tid; i < m; i += DRAW_THREADS)
            if (p[i] < least) { mine = i; break; }            // a thread's indices ascend: its first is its least
        if (mine < m) atomicMin(&first_below, mine);
        __syncthreads();
        kept = first_below > 0 ? first_below : 1;
    }
    float sum;
    if (top_p > 0.0f && top_p < 1.0f) {
        const int at = draw_running(p, kept, 0.0f, piece, shared2, [top_p](float s) { return s >= top_p; });
        if (at < kept) kept = at + 1;
        sum = shared2[0];                                     // the running sum over the kept, either way
    } else {
        draw_running(p, kept, 0.0f, piece, shared2, [](float) { return false; });
        sum = shared2[0];
    }
    __syncthreads();
    const float r = mul_rn(u, sum);
    const int at = draw_running(p, kept, 0.0f, piece, shared2, [r](float s) { return r < s; });
    if (tid == 0) tokens[row] = id[at < kept ? at : kept - 1];
}

extern "C" int hfa_draw_rows(float* vals, const int* ids, int n_rows, int vocab, const float* params, const int* cuts,
                             int* tokens, hipStream_t stream) {
    HFA_REQUIRE(n_rows > 0 && vocab > 0, "draw_rows: bad sizes rows=%d vocab=%d", n_rows, vocab);
    draw_rows_kernel<<<n_rows, DRAW_THREADS, 0, stream>>>(vals, ids, vocab, params, cuts, tokens);
    HFA_LAUNCH_CHECK("draw_rows");
    return 0;
}
