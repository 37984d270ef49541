// Kernels that only measure the machine: what a launch costs, what a meeting of all blocks inside one kernel costs,
// what the memory gives a kernel that only reads.  A unit of its own (libcisr_measure): the engine never loads it;
// `python -m runtime.measure` and the benchmark's read-bandwidth figure do.
#include "common.h"

// A kernel that does nothing: what a launch costs in a chain of kernels when nothing is computed, the floor
// under every kernel of a decode step (measured by `python -m runtime.measure floor`).
__global__ void idle_kernel() {}

extern "C" int cisr_idle(int blocks, hipStream_t stream) {
    if (blocks <= 0) return 0;
    idle_kernel<<<(unsigned)blocks, 256, 0, stream>>>();
    return CISR_LAUNCH_CHECK();
}

// A meeting of every block of a grid inside one kernel, as a decode step fused into fewer kernels would need between
// its parts: what it costs beside the launch of a kernel (`python -m runtime.measure floor` reports both).  Blocks meet
// in groups of 32 at a counter of their own, the last of a group goes on to the top counter, and everyone polls that
// one; with `exchange` every block writes its share of that many floats before the meeting and reads all of them
// after it, as activations would pass.  The wait is bounded: a block that waits too long sets the flag and leaves,
// so every wave ends whatever happens.  `words`: 1024 zeroed 32-bit words (counters 64 bytes apart, the flag last).
constexpr int MEET_GROUP = 32, MEET_WORDS = 1024, MEET_MAX_BLOCKS = 512;
__global__ void __launch_bounds__(256) grid_meet_kernel(unsigned* __restrict__ words, float* __restrict__ passed, int exchange,
                                                        int rounds, unsigned spin_limit) {
    const unsigned groups = gridDim.x / MEET_GROUP;
    unsigned* top = words;
    unsigned* mine = words + 16 * (1 + blockIdx.x % groups);
    unsigned* flag = words + MEET_WORDS - 1;
    const int share = exchange / (int)gridDim.x;
    float acc = 0.f;
    __shared__ int gave_up;
    if (threadIdx.x == 0) gave_up = 0;
    for (int r = 0; r < rounds; ++r) {
        float* side = passed + (size_t)(r & 1) * exchange;
        for (int i = threadIdx.x; i < share; i += blockDim.x) side[blockIdx.x * share + i] = acc + (float)(r + i);
        __syncthreads();
        if (threadIdx.x == 0) {
            __atomic_thread_fence(__ATOMIC_RELEASE);
            const unsigned before = __hip_atomic_fetch_add(mine, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before + 1 == (unsigned)(r + 1) * MEET_GROUP) __hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned spins = 0;
            while (__hip_atomic_load(top, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)(r + 1) * groups) {
                if (++spins > spin_limit) { *flag = 1u; gave_up = 1; break; }
                __builtin_amdgcn_s_sleep(1);
            }
            __atomic_thread_fence(__ATOMIC_ACQUIRE);
        }
        __syncthreads();
        if (gave_up) break;
        float part[4] = {0.f, 0.f, 0.f, 0.f};                  // (four sums, so that the loads of a lane do not wait for each other)
        const int all = share * (int)gridDim.x;
        int i = threadIdx.x;
        for (; i + 3 * 256 < all; i += 4 * 256) {
#pragma unroll
            for (int u = 0; u < 4; ++u) part[u] += __builtin_nontemporal_load(side + i + u * 256);
        }
        for (; i < all; i += 256) part[0] += __builtin_nontemporal_load(side + i);
        acc += (part[0] + part[1] + part[2] + part[3]) * 1e-9f;
    }
    if (acc == 123.456f) words[MEET_WORDS - 2] = 1u;
}

// `blocks`: a multiple of 32, at most 512 (all of them must be resident together: 256 threads and a few bytes of LDS each);
// `passed`: 2 x exchange floats (may be null when exchange is 0).
extern "C" int cisr_grid_meet(void* words, void* passed, int exchange, int blocks, int rounds, unsigned spin_limit, hipStream_t stream) {
    if (rounds <= 0) return 0;
    if (!words || blocks <= 0 || blocks % MEET_GROUP || blocks > MEET_MAX_BLOCKS || exchange < 0 || (exchange && !passed) ||
        (long long)rounds * blocks >= (1ll << 31))
        return (int)hipErrorInvalidValue;
    // every block must be resident at once, or the first to arrive wait for blocks that cannot start
    int device = 0, per_unit = 0, units = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, grid_meet_kernel, 256, 0) != hipSuccess || (long long)per_unit * units < blocks)
        return (int)hipErrorInvalidValue;
    grid_meet_kernel<<<(unsigned)blocks, 256, 0, stream>>>((unsigned*)words, (float*)passed, exchange, rounds, spin_limit);
    return CISR_LAUNCH_CHECK();
}

// A kernel that only reads: every block walks a contiguous run of 16-byte words, eight loads a lane in flight, and
// folds them into one word that is written only if it has a value no data gives.  What this GPU's memory gives a
// kernel that streams weights and does nothing else (the benchmark reports it beside the published peak).
typedef unsigned int read_word_t __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) stream_read_kernel(const read_word_t* __restrict__ src, long long words, unsigned* __restrict__ sink) {
    const long long per = words / gridDim.x;                       // (a remainder of fewer words than blocks is left out)
    const read_word_t* p = src + (long long)blockIdx.x * per;
    read_word_t acc = {0u, 0u, 0u, 0u};
    constexpr int U = 8;
    long long i = threadIdx.x;
    for (; i + (long long)(U - 1) * 256 < per; i += (long long)U * 256) {
        read_word_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + (long long)u * 256);
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    for (; i < per; i += 256) acc ^= p[i];
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && sink) sink[0] = acc.x;
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once with `blocks` blocks; `sink`: 4 bytes that are hardly ever written.
extern "C" int cisr_stream_read(const void* src, long long bytes, void* sink, int blocks, hipStream_t stream) {
    if (bytes <= 0 || blocks <= 0) return 0;
    if (bytes % 16 || ((uintptr_t)src) % 16 || !sink) return (int)hipErrorInvalidValue;
    stream_read_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const read_word_t*)src, bytes / 16, (unsigned*)sink);
    return CISR_LAUNCH_CHECK();
}

// A chain of dependent matrix-vector products, the leanest kernel that a decode step of one request could be made of:
// a wave owns one row of W (K = 512 KC bf16), its lanes read one 16-byte chunk of it per 512 inner positions and their
// slices of the float vector x, the lanes' sums meet by lane exchanges, and lane 0 stores y[row] (squashed into
// (-1, 1), so that a chain of any length keeps its values).  No LDS, no barrier, every load issued at the start.
// What `python -m runtime.measure chain` times with it: how short a kernel of a captured chain can be (the floor under
// the products of a decode step), and whether kernels on two streams that hand their results over through counters in
// memory (WAIT: poll `cnt_in` until `expect` blocks have arrived; every block bumps `cnt_out` after its stores; x and
// y then bypass the caches, which are not coherent between the eight dies) beat the order of one stream.
// The wait is bounded (`spin_limit` polls, or as soon as another block has given up): then `err[0]` is set and the
// kernel goes on with whatever it reads, so that every wave ends whatever happens.
typedef float chain_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float chain_bf(uint32_t v, int hi) { return __uint_as_float(hi ? (v & 0xffff0000u) : (v << 16)); }

template <int KC, bool WAIT>
__global__ void __launch_bounds__(256) chain_phase_kernel(const read_word_t* __restrict__ W, const float* x, float* y, unsigned* cnt_in,
                                                          unsigned expect, unsigned* cnt_out, unsigned spin_limit, unsigned* err) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + wave;
    read_word_t w[KC];
#pragma unroll
    for (int c = 0; c < KC; ++c) w[c] = __builtin_nontemporal_load(W + (size_t)row * (KC * 64) + c * 64 + lane);
    if (WAIT) {
        if (threadIdx.x == 0) {
            unsigned spins = 0;
            while (__hip_atomic_load(cnt_in, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < expect) {
                if (++spins > spin_limit || ((spins & 1023u) == 0u && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) { *err = 1u; break; }
            }
        }
        __syncthreads();
    }
    float xv[KC][8];
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        const float* p = x + (c * 64 + lane) * 8;
        chain_f32x4 lo, hi;
        if (WAIT) {     // straight from memory: another die's L2 may hold what a block there wrote
            lo = (chain_f32x4){__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
                               __hip_atomic_load(p + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), __hip_atomic_load(p + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)};
            hi = (chain_f32x4){__hip_atomic_load(p + 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), __hip_atomic_load(p + 5, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT),
                               __hip_atomic_load(p + 6, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT), __hip_atomic_load(p + 7, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)};
        } else {
            lo = *(const chain_f32x4*)p; hi = *(const chain_f32x4*)(p + 4);
        }
        xv[c][0] = lo.x; xv[c][1] = lo.y; xv[c][2] = lo.z; xv[c][3] = lo.w; xv[c][4] = hi.x; xv[c][5] = hi.y; xv[c][6] = hi.z; xv[c][7] = hi.w;
    }
    float a = 0.f;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
        const read_word_t v = w[c];
        a += chain_bf(v.x, 0) * xv[c][0] + chain_bf(v.x, 1) * xv[c][1] + chain_bf(v.y, 0) * xv[c][2] + chain_bf(v.y, 1) * xv[c][3]
           + chain_bf(v.z, 0) * xv[c][4] + chain_bf(v.z, 1) * xv[c][5] + chain_bf(v.w, 0) * xv[c][6] + chain_bf(v.w, 1) * xv[c][7];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) a += __shfl_xor(a, off, 64);
    a = a * 4.f;
    a = a / (1.f + fabsf(a)) + 0.05f;
    if (lane == 0) {
        if (WAIT) __hip_atomic_store(y + row, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else y[row] = a;
    }
    if (WAIT && cnt_out) {
        __builtin_amdgcn_s_waitcnt(0);       // every wave's store is acknowledged before the block's arrival is counted
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_fetch_add(cnt_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// y[N] = squash(W[N, K] . x[K]); N a multiple of 4, K 512 or 1536; `wait`: the hand-over through counters (see above).
extern "C" int cisr_chain_phase(const void* W, const float* x, float* y, int N, int K, unsigned* cnt_in, unsigned expect,
                                unsigned* cnt_out, unsigned* err, int wait, hipStream_t stream) {
    if (N <= 0 || N % 4 || (K != 512 && K != 1536) || !W || !x || !y || (wait && (!cnt_in || !err)) || ((uintptr_t)W) % 16 || ((uintptr_t)x) % 16)
        return (int)hipErrorInvalidValue;
    const unsigned blocks = (unsigned)(N / 4), limit = 1u << 18;
    if (K == 512) {
        if (wait) chain_phase_kernel<1, true><<<blocks, 256, 0, stream>>>((const read_word_t*)W, x, y, cnt_in, expect, cnt_out, limit, err);
        else chain_phase_kernel<1, false><<<blocks, 256, 0, stream>>>((const read_word_t*)W, x, y, cnt_in, expect, cnt_out, limit, err);
    } else {
        if (wait) chain_phase_kernel<3, true><<<blocks, 256, 0, stream>>>((const read_word_t*)W, x, y, cnt_in, expect, cnt_out, limit, err);
        else chain_phase_kernel<3, false><<<blocks, 256, 0, stream>>>((const read_word_t*)W, x, y, cnt_in, expect, cnt_out, limit, err);
    }
    return CISR_LAUNCH_CHECK();
}

// A whole decode step as ONE launch whose blocks meet inside the kernel, but only the blocks of one die (XCD) with each
// other, through that die's L2: what `python -m runtime.measure one_launch` times against the step of 154 launches.
// Blocks are dealt to the dies in turn (from a die that changes from launch to launch), so a grid of 8 n blocks puts n
// on each; a block reads the number of its die from the hardware register, takes a ticket there, and the blocks of
// the first `active` dies each run the step of a request of their own: 30 x (q/k/v, attention, output projection,
// gate and up, down), every part a matrix-vector pass over that layer's weights with the traffic and the dependences of
// the real kernels (activations of the part before: from L2, into LDS; a wave streams its contiguous share of the
// rows, eight loads a lane in flight; lane sums meet; a store) and no arithmetic that means anything; attention reads
// `kv16` 16-byte words of keys and values a layer.  Meetings: arrivals and polls are read-modify-writes without the
// device-scope bit, which execute in the die's L2 (a poll adds a zero that the compiler cannot see, or it would turn
// into a load that the compute unit's own cache answers for ever); what a block wrote before a meeting the others
// read after it with device-scope loads, which pass the compute unit's cache and are answered by the same L2.
// Bounded: after `spin_limit` polls a block sets words[1023] and its die's blocks leave at that meeting.
// `words`: 1024 zeroed 32-bit words; `scratch`: 8 x 16384 floats.
struct DieMeeting { unsigned* count; unsigned* flag; unsigned zero, blocks, limit, expected; };

__device__ __forceinline__ bool die_meet(DieMeeting& m) {
    __builtin_amdgcn_s_waitcnt(0);                       // this wave's stores are acknowledged by L2
    __syncthreads();
    __shared__ int gave_up;
    if (threadIdx.x == 0) {
        gave_up = 0;
        __hip_atomic_fetch_add(m.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        m.expected += m.blocks;
        unsigned polls = 0;
        while (__hip_atomic_fetch_add(m.count, m.zero, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < m.expected) {
            if (++polls > m.limit) { *m.flag = 1u; gave_up = 1; break; }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    __syncthreads();
    return !gave_up;
}

__device__ __forceinline__ void die_pass(const float* x, int K, const read_word_t* W, int N, float* y, int rank, int blocks, float* lds) {
    constexpr int NT = 512;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, waves = NT / 64;
    for (int i = threadIdx.x; i < K; i += NT) lds[i] = __hip_atomic_load(x + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int all = blocks * waves, me = rank * waves + wave;
    const int r0 = (int)((long long)N * me / all), r1 = (int)((long long)N * (me + 1) / all);
    const read_word_t* w = W + (size_t)r0 * (K / 8);
    const int n16 = (r1 - r0) * (K / 8);
    float acc = 0.f;
    int c = lane;
    for (; c + 7 * 64 < n16; c += 8 * 64) {
        read_word_t v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = w[c + j * 64];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += chain_bf(v[j].x, 1) * lds[(c + j) & 511] + chain_bf(v[j].y, 0) * lds[(c * 3 + j) & 511] + __uint_as_float(v[j].z ^ v[j].w) * 1e-30f;
    }
    for (; c < n16; c += 64) { const read_word_t v = w[c]; acc += chain_bf(v.x, 1) * lds[c & 511] + __uint_as_float(v.y ^ v.z ^ v.w) * 1e-30f; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane < r1 - r0) y[r0 + lane] = acc;
}

__global__ void __launch_bounds__(512) one_launch_step_kernel(const read_word_t* __restrict__ weights, long long layer16, int layers, int H, int QKV, int I,
                                                              const read_word_t* __restrict__ kv, long long kv16, float* scratch, unsigned* words,
                                                              unsigned zero, int blocks, int active, unsigned spin_limit) {
    extern __shared__ float lds[];
    __shared__ int rank_here;
    const int die = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 15;      // bits 3:0 of the hardware register that names the die
    if (die >= 8) return;
    if (threadIdx.x == 0) rank_here = (int)__hip_atomic_fetch_add(words + 512 + die * 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();
    const int rank = rank_here;
    if (die >= active || rank >= blocks) return;
    DieMeeting m = {words + die * 16, words + 1023, zero, (unsigned)blocks, spin_limit, 0u};
    float* res = scratch + (size_t)die * 16384, *q = res + 4096, *att = q + 4096, *act = att + 4096;
    const read_word_t* kv_here = kv + (size_t)die * kv16 * layers;
    for (int l = 0; l < layers; ++l) {
        const read_word_t* W = weights + (size_t)l * layer16;
        die_pass(res, H, W, QKV, q, rank, blocks, lds);
        if (!die_meet(m)) return;
        {   // attention: this block's share of the layer's keys and values, then its part of a result
            read_word_t a = {0u, 0u, 0u, 0u};
            const float q0 = __hip_atomic_load(q + threadIdx.x % QKV, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const read_word_t* mine = kv_here + (size_t)l * kv16;
            for (long long i = (long long)rank * 512 + threadIdx.x; i < kv16; i += (long long)blocks * 512) a ^= mine[i];
            if (threadIdx.x < 64 && rank * 64 + threadIdx.x < H) att[rank * 64 + threadIdx.x] = q0 + (float)(a.x ^ a.y ^ a.z ^ a.w) * 1e-30f;
        }
        if (!die_meet(m)) return;
        W += (size_t)QKV * H / 8;
        die_pass(att, H, W, H, res, rank, blocks, lds);
        if (!die_meet(m)) return;
        W += (size_t)H * H / 8;
        die_pass(res, H, W, 2 * I, act, rank, blocks, lds);
        if (!die_meet(m)) return;
        W += (size_t)2 * I * H / 8;
        die_pass(act, I, W, H, res, rank, blocks, lds);
        if (!die_meet(m)) return;
    }
}

// weights: bf16, `layers` x ((QKV + H + 2 I) H + H I) elements; kv: 8 x layers x kv16 16-byte words; blocks: 32 or 64 a die
// (one or two a compute unit: all resident at once); H, I multiples of 8, at most 4096 floats a vector.
extern "C" int cisr_one_launch_step(const void* weights, int layers, int H, int QKV, int I, const void* kv, long long kv16, void* scratch,
                                    void* words, int blocks, int active, unsigned spin_limit, hipStream_t stream) {
    if (layers <= 0) return 0;
    if (!weights || !kv || !scratch || !words || (blocks != 32 && blocks != 64) || active < 1 || active > 8 || H % 8 || I % 8 ||
        H <= 0 || I <= 0 || QKV <= 0 || H > 4096 || I > 4096 || QKV > 4096 || 2 * I > 4096 || kv16 < 0)
        return (int)hipErrorInvalidValue;
    int device = 0, per_unit = 0, units = 0;
    const size_t lds_bytes = (size_t)(I > H ? I : H) * 4;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, one_launch_step_kernel, 512, lds_bytes) != hipSuccess ||
        (long long)per_unit * units < 8ll * blocks)
        return (int)hipErrorInvalidValue;
    const long long layer16 = ((long long)(QKV + H + 2 * I) * H + (long long)H * I) / 8;
    one_launch_step_kernel<<<8u * blocks, 512, lds_bytes, stream>>>((const read_word_t*)weights, layer16, layers, H, QKV, I, (const read_word_t*)kv, kv16,
                                                                   (float*)scratch, (unsigned*)words, 0u, blocks, active, spin_limit);
    return CISR_LAUNCH_CHECK();
}
