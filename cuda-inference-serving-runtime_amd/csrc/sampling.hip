// Token choice from float logits [R, V]: greedy (lowest index wins a tie, as
// numpy/cupy argmax does in the reference, runtime/engine.py:99) and temperature
// sampling p = softmax(logits / T) drawn by inverse CDF with a counter-based
// random number per (seed, counter), so a request's draw does not depend on
// what else is in the batch.  One block of 256 threads per row; every thread
// owns one contiguous slice of the vocabulary, which fixes the summation order.
#include "common.h"
#include "cisr_noalloc.h"
#include <stdio.h>
#include <mutex>

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// uniform in [0, 1) with 24 random bits
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t counter) {
    uint64_t h = splitmix64(splitmix64(seed) ^ (counter * 0xD1342543DE82EF95ull));
    return (float)(h >> 40) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ void argmax_block(const float* __restrict__ x, int n, float* smax, int* sidx,
                                             float& best, int& best_idx) {
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 256) {
        float v = x[i];
        if (bi == 0x7fffffff || v > bv) { bv = v; bi = i; }  // indices ascend: a tie keeps the lower one
    }
    smax[threadIdx.x] = bv; sidx[threadIdx.x] = bi;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            float ov = smax[threadIdx.x + s]; int oi = sidx[threadIdx.x + s];
            float mv = smax[threadIdx.x]; int mi = sidx[threadIdx.x];
            if (oi != 0x7fffffff && (mi == 0x7fffffff || ov > mv || (ov == mv && oi < mi))) {
                smax[threadIdx.x] = ov; sidx[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    best = smax[0]; best_idx = sidx[0];
    __syncthreads();
}

// Greedy pick in two passes so that a few rows still fill the GPU: the vocabulary is cut
// into `chunks` slices, one block each; a second pass picks among the slice winners
// (lower slice first, so the lowest index still wins a tie).
__global__ void __launch_bounds__(256)
argmax_partial_kernel(const float* __restrict__ logits, float* __restrict__ pval, int* __restrict__ pidx,
                      int vocab, int chunks) {
    __shared__ float smax[256];
    __shared__ int sidx[256];
    const int row = blockIdx.x, chunk = blockIdx.y;
    const int per = (vocab + chunks - 1) / chunks;
    const int lo = chunk * per, n = max(0, min(vocab, lo + per) - lo);
    float best; int idx;
    argmax_block(logits + (size_t)row * vocab + lo, n, smax, sidx, best, idx);
    if (threadIdx.x == 0) {
        pval[row * chunks + chunk] = best;
        pidx[row * chunks + chunk] = idx == 0x7fffffff ? 0x7fffffff : lo + idx;
    }
}

__global__ void __launch_bounds__(64)
argmax_final_kernel(const float* __restrict__ pval, const int* __restrict__ pidx, int* __restrict__ out,
                    const int* __restrict__ index, int out_n, int chunks) {
    const int row = blockIdx.x;
    if (threadIdx.x != 0) return;
    const int dst = index ? index[row] : row;
    if (dst < 0 || dst >= out_n) return;
    float bv = -INFINITY; int bi = 0x7fffffff;
    for (int c = 0; c < chunks; ++c) {
        const float v = pval[row * chunks + c]; const int i = pidx[row * chunks + c];
        if (i != 0x7fffffff && (bi == 0x7fffffff || v > bv)) { bv = v; bi = i; }
    }
    out[dst] = bi == 0x7fffffff ? 0 : bi;
}

#define ARGMAX_CHUNKS 32

// scratch: float [rows * 32] and int [rows * 32].  With `index`, row r's token goes to out[index[r]]
// (nowhere if that is outside 0..out_n-1) instead of out[r]; without, out_n is rows.
extern "C" int cisr_argmax(const float* logits, int* out, const int* index, int out_n, float* scratch_val, int* scratch_idx,
                           int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    argmax_partial_kernel<<<dim3(rows, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, scratch_val, scratch_idx, vocab, ARGMAX_CHUNKS);
    int err = CISR_LAUNCH_CHECK();
    if (err) return err;
    argmax_final_kernel<<<rows, 64, 0, stream>>>(scratch_val, scratch_idx, out, index, index ? out_n : rows, ARGMAX_CHUNKS);
    return CISR_LAUNCH_CHECK();
}

// The slice winners of cisr_argmax_noalloc: values (float) then indices (int), 32 of each a row.  In host code
// this name is only a stand-in for the symbol, not a device address; the address on each device comes from
// hipGetSymbolAddress and is kept in noalloc_scratch[].
static __device__ __align__(256) unsigned char scratch[CISR_ARGMAX_NOALLOC_MAX_ROWS * ARGMAX_CHUNKS * (sizeof(float) + sizeof(int))];

#define NOALLOC_MAX_DEVICES 64
static void* noalloc_scratch[NOALLOC_MAX_DEVICES];     // per device: each GPU holds its own copy at its own address
static std::mutex noalloc_lock;

static int noalloc_scratch_of_current_device(void** ptr) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return (int)e;
    if (device < 0 || device >= NOALLOC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(noalloc_lock);
    if (noalloc_scratch[device] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        noalloc_scratch[device] = p;
    }
    *ptr = noalloc_scratch[device];
    return 0;
}

extern "C" int cisr_noalloc_init(void) {
    void* p = nullptr;
    return noalloc_scratch_of_current_device(&p);
}

extern "C" int cisr_argmax_noalloc_max_rows(void) { return CISR_ARGMAX_NOALLOC_MAX_ROWS; }

extern "C" int cisr_argmax_noalloc(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
    if (rows == 0) return 0;
    if (rows < 0 || rows > CISR_ARGMAX_NOALLOC_MAX_ROWS || vocab <= 0 || logits == nullptr || out == nullptr) {
        fprintf(stderr, "cisr_argmax_noalloc: %d rows of %d logits refused (1 to %d rows, a vocabulary of at least 1, "
                        "no null pointers)\n", rows, vocab, CISR_ARGMAX_NOALLOC_MAX_ROWS);
        return (int)hipErrorInvalidValue;
    }
    void* base = nullptr;
    int err = noalloc_scratch_of_current_device(&base);
    if (err) return err;
    float* pval = (float*)base;
    int* pidx = (int*)((unsigned char*)base + (size_t)CISR_ARGMAX_NOALLOC_MAX_ROWS * ARGMAX_CHUNKS * sizeof(float));
    argmax_partial_kernel<<<dim3(rows, ARGMAX_CHUNKS), 256, 0, stream>>>(logits, pval, pidx, vocab, ARGMAX_CHUNKS);
    err = CISR_LAUNCH_CHECK();
    if (err) return err;
    argmax_final_kernel<<<rows, 64, 0, stream>>>(pval, pidx, out, nullptr, rows, ARGMAX_CHUNKS);
    return CISR_LAUNCH_CHECK();
}

__global__ void __launch_bounds__(256)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
              const unsigned long long* __restrict__ seeds, const unsigned long long* __restrict__ counters,
              int* __restrict__ out, const int* __restrict__ index, int out_n, int vocab) {
    __shared__ float smax[256];
    __shared__ int sidx[256];
    __shared__ float ssum[256];
    const int row = blockIdx.x;
    const int dst = index ? index[row] : row;
    if (dst < 0 || dst >= out_n) return;       // the whole block: no barrier is passed by a part of it
    const float* x = logits + (size_t)row * vocab;
    float best; int best_idx;
    argmax_block(x, vocab, smax, sidx, best, best_idx);
    const float temp = temperature[row];
    if (!(temp > 0.f)) {  // greedy
        if (threadIdx.x == 0) out[dst] = best_idx == 0x7fffffff ? 0 : best_idx;
        return;
    }
    const float inv_t = 1.0f / temp;
    const int per = (vocab + 255) / 256;
    const int lo = threadIdx.x * per, hi = min(vocab, lo + per);
    float part = 0.f;
    for (int i = lo; i < hi; ++i) part += expf((x[i] - best) * inv_t);
    ssum[threadIdx.x] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int t = 0; t < 256; ++t) total += ssum[t];
        const float target = uniform01(seeds[row], counters[row]) * total;
        // find the slice, then the token inside it; fall back to the last token
        // with non-zero mass if rounding pushes the target past the end
        float run = 0.f; int choice = -1;
        int t = 0;
        for (; t < 256; ++t) { if (run + ssum[t] > target) break; run += ssum[t]; }
        if (t < 256) {
            const int a = t * per, b = min(vocab, a + per);
            for (int i = a; i < b; ++i) {
                run += expf((x[i] - best) * inv_t);
                if (run > target) { choice = i; break; }
            }
            if (choice < 0) choice = b - 1;
        }
        if (choice < 0) choice = best_idx;
        out[dst] = choice;
    }
}

extern "C" int cisr_sample(const float* logits, const float* temperature, const unsigned long long* seeds,
                           const unsigned long long* counters, int* out, const int* index, int out_n, int rows, int vocab,
                           hipStream_t stream) {
    if (rows <= 0) return 0;
    sample_kernel<<<rows, 256, 0, stream>>>(logits, temperature, seeds, counters, out, index, index ? out_n : rows, vocab);
    return CISR_LAUNCH_CHECK();
}

// tokens[r] = sampled[source[r]] where source[r] >= 0: a row whose token is the one last picked for its
// request and still only on the device takes it from there.
__global__ void __launch_bounds__(256)
take_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ source, const int* __restrict__ sampled, int rows, int slots) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const int s = source[r];
    if (s >= 0 && s < slots) tokens[r] = sampled[s];
}

extern "C" int cisr_take_tokens(int* tokens, const int* source, const int* sampled, int rows, int slots, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (slots <= 0) return 1;
    take_tokens_kernel<<<(rows + 255) / 256, 256, 0, stream>>>(tokens, source, sampled, rows, slots);
    return CISR_LAUNCH_CHECK();
}
