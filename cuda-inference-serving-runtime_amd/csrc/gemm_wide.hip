// Skinny matrix products against large weights:  C[M,N] = A[M,K] . W[N,K]^T  with M <= 64 rows,
// for weights of tens of megabytes and more, where the product is bound by streaming W from HBM
// and every other byte that passes the vector memory path costs time that W needs.
//
// The weight-streaming kernel of gemm_skinny.inc reads the activations again for every 16 rows of W
// (from L2, but through the same path as W): with 8 rows of A that is half the traffic of W, with 64
// rows four times it.  Here a block keeps the activations of its part of K in registers, as finished
// matrix-core operands, and walks over many 16-row units of W with them:
//   - K is cut into slices; the waves of a block deal a slice's k-steps among them in pairs (a cache line
//     of a row of W) and each holds the A operands of its steps for all row tiles;
//   - the work items (slice, unit), slice-major, are dealt to the blocks in equal contiguous runs, one block a
//     compute unit; a block walks over its units of W, the loads of the next unit in flight while the matrix
//     cores work on this one and the waves' partial tiles meet in LDS;
//   - with one slice the block finishes the result itself; with several, every slice writes its partial
//     sums and a second small kernel adds them in slice order and finishes.
// Sums are formed in a fixed order (waves in order inside a slice, slices in order), so a row's result
// does not depend on the other rows; the shape of the launch depends on M only through the number of
// 16-row tiles.
// Finishing: store float or bf16, with an optional float residual; or SwiGLU over two blocks of W; or, for
// W = [Wq; Wk; Wv], the rotary embedding of q and k with q stored and k, v written into the paged cache
// (a unit is then 8 rotary pairs (i, i + D/2) of one head, so that both halves of a pair meet in one tile).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

struct WideArgs {
    const bf16_t* A; int lda;
    const bf16_t* W; int ldw;
    void* C; int ldc; int out_dtype;
    const float* R; int ldr;
    float* P;                   // partial sums [slices][M][NB * N] when there are several slices
    int M, N, K;
    int units;                  // 16-row units of W
    int slices;                 // slices of K: SPW / 2 rounds of NW pairs of 32-wide k-steps each
    int dual_off;               // two blocks of W this many rows apart (SwiGLU), or 0
    int leave_partials;         // several slices: no second kernel, the caller's next kernel adds the partial sums
    // the fused q/k/v projection (head_dim > 0): C is q, bf16 [M, heads * head_dim]
    const int* positions; const int* slots; const float* cos_tab; const float* sin_tab;
    bf16_t* kcache; bf16_t* vcache; int heads, kv_heads, head_dim, page_size, max_pos;
};

// the row of W = [Wq; Wk; Wv] behind column c of unit u: 8 rotary pairs of a head a unit
__device__ __forceinline__ int wide_rope_row(const WideArgs& p, int u, int c) {
    const int per_head = p.head_dim / 16, sh = u / per_head, j0 = (u % per_head) * 8;
    return sh * p.head_dim + (c < 8 ? j0 + c : p.head_dim / 2 + j0 + c - 8);
}

// the fused projection's value of row m, column c of unit u: v, and pv from column c ^ 8 (the other half of the pair)
__device__ __forceinline__ void wide_finish_rope(const WideArgs& p, int m, int u, int c, float v, float pv) {
    const int D = p.head_dim, half = D / 2, per_head = D / 16;
    const int sh = u / per_head, i = (u % per_head) * 8 + (c & 7), col = c < 8 ? i : half + i;
    if (sh < p.heads + p.kv_heads) {                              // q or k head: rotate
        int pos = p.positions[m];
        pos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
        const float cs = p.cos_tab[(size_t)pos * half + i], sn = p.sin_tab[(size_t)pos * half + i];
        v = c < 8 ? v * cs - pv * sn : v * cs + pv * sn;
    }
    if (sh < p.heads) {
        ((bf16_t*)p.C)[(size_t)m * p.ldc + sh * D + col] = f32_to_bf16(v);
        return;
    }
    const int slot = p.slots[m];
    if (slot < 0) return;
    const int page = slot / p.page_size, off = slot % p.page_size;
    if (sh < p.heads + p.kv_heads) {
        const int h = sh - p.heads;
        p.kcache[(((size_t)page * p.kv_heads + h) * p.page_size + off) * D + col] = f32_to_bf16(v);
    } else {
        const int h = sh - p.heads - p.kv_heads;
        p.vcache[(((size_t)page * p.kv_heads + h) * D + col) * p.page_size + off] = f32_to_bf16(v);
    }
}

// the value of (m, n) from the finished sums: v, and u for the second block of W
template <int NB>
__device__ __forceinline__ void wide_finish(const WideArgs& p, int m, int n, float v, float u) {
    if (NB == 2) {
        // gate and up are rounded to bf16 before the activation, as the two-kernel path does
        const float gq = bf16_to_f32(f32_to_bf16(v)), uq = bf16_to_f32(f32_to_bf16(u));
        v = gq / (1.0f + expf(-gq)) * uq;
    }
    if (p.R) v += p.R[(size_t)m * p.ldr + n];
    if (p.out_dtype == DT_F32) ((float*)p.C)[(size_t)m * p.ldc + n] = v;
    else ((bf16_t*)p.C)[(size_t)m * p.ldc + n] = f32_to_bf16(v);
}

// MT 16-row tiles of A; NW waves; SPW k-steps a wave and slice (even); NB blocks of W
template <int MT, int NW, int SPW, int NB, bool ROPE>
__global__ void __launch_bounds__(NW * 64)
gemm_wide_kernel(WideArgs p) {
    extern __shared__ float smem[];
    float (*red)[NB][MT][4][WAVE] = reinterpret_cast<float (*)[NB][MT][4][WAVE]>(smem);   // [wave][block][tile][e][lane]
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;   // (uniform: scalar loop control)
    const int r = lane % 16, g = lane / 16;
    const int M = p.M, N = p.N, K = p.K;
    constexpr int TSTEP = NW / 4;                                 // NW is a multiple of 4
    constexpr int TPW = (MT + TSTEP - 1) / TSTEP;                 // tiles a wave finishes
    const int e2 = wave % 4, t2 = wave / 4;
    bool first = true;

    // this block's run of work items; item i is unit i % units of slice i / units
    const long long items = (long long)p.units * p.slices;
    long long item = items * blockIdx.x / gridDim.x;
    const long long item_end = items * (blockIdx.x + 1) / gridDim.x;
    while (item < item_end) {                                     // once per slice that the run touches
        const int slice = (int)(item / p.units), u0 = (int)(item % p.units);
        const int u1 = (int)min((long long)p.units, u0 + (item_end - item));
        item += u1 - u0;
        // A slice is SPW / 2 rounds of pairs of k-steps; round i gives pair wave + NW * i to this wave.  The
        // activations of this wave's steps stay in registers, as matrix-core operands, for every unit of the
        // run.  A chunk of 8 lies inside K or outside (K % 8 == 0); outside it is zero, and the weights beside
        // it are read from a clamped address.
        const int i0 = slice * (SPW / 2);
        u32x4 af[SPW][MT];
        int koff[SPW];
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
            const int i = i0 + (j >> 1);
            const int ko = (2 * (wave + NW * i) + (j & 1)) * 32 + g * 8;
            const uint32_t keep = ko + 8 <= K ? 0xffffffffu : 0u;
            koff[j] = min(ko, K - 8);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int m = min(t * 16 + r, M - 1);
                u32x4 v = *(const u32x4*)(p.A + (size_t)m * p.lda + koff[j]);
                v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep;
                af[j][t] = v;
            }
        }
        auto load_w = [&](u32x4 (&w)[NB][SPW], int u) {
            // rows past N are read again and never stored
            const int n = ROPE ? wide_rope_row(p, u, r) : min(u * 16 + r, N - 1);
            const bf16_t* row = p.W + (size_t)n * p.ldw;
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int j = 0; j < SPW; ++j) w[b][j] = *(const u32x4*)(row + (size_t)b * p.dual_off * p.ldw + koff[j]);
        };
        auto compute = [&](u32x4 (&w)[NB][SPW], int u) {
            f32x4 acc[NB][MT];
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[b][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < SPW; ++j)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int b = 0; b < NB; ++b)
                        acc[b][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[j][t]),
                                                                            __builtin_bit_cast(bf16x8, w[b][j]), acc[b][t], 0, 0, 0);
            if (!first) __syncthreads();                          // every wave has read the sums of the unit before
            first = false;
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int e = 0; e < 4; ++e) red[wave][b][t][e][lane] = acc[b][t][e];   // lanes side by side: no bank conflicts
            __syncthreads();
            // a thread finishes (tile t2 + k * NW/4, row 4 (lane / 16) + e2, column lane % 16)
#pragma unroll
            for (int it = 0; it < TPW; ++it) {
                const int t = t2 + it * TSTEP;
                if (t >= MT) break;
                const int m = t * 16 + (lane / 16) * 4 + e2, n = u * 16 + lane % 16;
                if (m >= M || n >= N) continue;
                float v = 0.f, uu = 0.f;
#pragma unroll
                for (int w2 = 0; w2 < NW; ++w2) v += red[w2][0][t][e2][lane];
                if (NB == 2) {
#pragma unroll
                    for (int w2 = 0; w2 < NW; ++w2) uu += red[w2][NB - 1][t][e2][lane];
                }
                if (ROPE && p.slices == 1) {
                    float pv = 0.f;
#pragma unroll
                    for (int w2 = 0; w2 < NW; ++w2) pv += red[w2][0][t][e2][lane ^ 8];
                    wide_finish_rope(p, m, u, lane % 16, v, pv);
                } else if (p.slices == 1) {
                    wide_finish<NB>(p, m, n, v, uu);
                } else {
                    float* dst = p.P + ((size_t)slice * M + m) * ((size_t)N * NB) + n;
                    dst[0] = v;
                    if (NB == 2) dst[N] = uu;
                }
            }
        };
        u32x4 wa[NB][SPW], wb[NB][SPW];
        load_w(wa, u0);
        for (int u = u0; u < u1; u += 2) {                        // u0 < u1; the bounds are uniform over the block
            if (u + 1 < u1) load_w(wb, u + 1);
            compute(wa, u);
            if (u + 1 < u1) {
                if (u + 2 < u1) load_w(wa, u + 2);
                compute(wb, u + 1);
            }
        }
    }
}

// second pass: add the slices' partial sums in slice order and finish
template <int NB, bool ROPE>
__global__ void __launch_bounds__(256)
gemm_wide_finish_kernel(WideArgs p) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)p.M * p.N) return;
    const int m = (int)(i / p.N), n = (int)(i % p.N);
    const size_t row = (size_t)p.N * NB, all = (size_t)p.M * row;
    const float* src = p.P + (size_t)m * row + n;
    float v = 0.f, u = 0.f;
    for (int s = 0; s < p.slices; ++s) {
        v += src[(size_t)s * all];
        if (NB == 2) u += src[(size_t)s * all + p.N];
    }
    if (ROPE) {                                                   // column n of the partial sums is column n % 16 of unit n / 16
        const float* other = p.P + (size_t)m * row + (n ^ 8);
        float pv = 0.f;
        for (int s = 0; s < p.slices; ++s) pv += other[(size_t)s * all];
        wide_finish_rope(p, m, n / 16, n % 16, v, pv);
        return;
    }
    wide_finish<NB>(p, m, n, v, u);
}

static int wide_cus() {
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

template <int MT, int NW, int SPW, int NB, bool ROPE>
static int wide_launch(WideArgs a, size_t workspace_floats, bool plan_only, long long* need, hipStream_t stream) {
    const int pairs = (a.K + 63) / 64, rounds = (pairs + NW - 1) / NW;
    a.slices = (rounds + SPW / 2 - 1) / (SPW / 2);
    const size_t partial = a.slices > 1 ? (size_t)a.slices * a.M * a.N * NB : 0;
    if (need) *need = (long long)partial;
    if (plan_only) return 0;
    if (partial > workspace_floats || (partial && !a.P) || (a.leave_partials && !partial)) return (int)hipErrorInvalidValue;
    const long long items = (long long)a.units * a.slices;
    const int cus = wide_cus();
    const size_t shmem = (size_t)NW * NB * MT * 4 * WAVE * sizeof(float);
    if (shmem > 65536) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_wide_kernel<MT, NW, SPW, NB, ROPE>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    // one block a compute unit, each with an equal run of the work items
    gemm_wide_kernel<MT, NW, SPW, NB, ROPE><<<(unsigned)(items < cus ? items : cus), NW * 64, shmem, stream>>>(a);
    int err = CISR_LAUNCH_CHECK();
    if (err || a.slices == 1 || a.leave_partials) return err;
    const size_t cells = (size_t)a.M * a.N;
    gemm_wide_finish_kernel<NB, ROPE><<<(unsigned)((cells + 255) / 256), 256, 0, stream>>>(a);
    return CISR_LAUNCH_CHECK();
}

// Rounds a slice (SPW / 2), by a model of the busiest block's time fitted to measurements on an MI355X (it picks
// the fastest of 1, 2, 4 rounds in 27 of 30 products of the 135M, 1.7B and 8B sizes at 8, 32 and 64 rows, and is
// within 3 % of it in the others).  In units of a round (every block streams NW * 2 KB of each block of W, at
// about 5 TB/s over the whole GPU):
//   items of the block x (rounds a slice + the fixed cost of a unit: barriers and the sums through LDS)
//   + the activations of each slice the run touches (rows / 16 of a round of W for each of its rounds)
//   + half a slice more for a block with a single unit (nothing overlaps its loads)
//   + with several slices: the second kernel, and the partial sums written and read once.
// The rounds of a last slice past K are loaded from clamped addresses and add nothing, but cost like the others.
template <int MT, int NW, int MAXSPW, int NB, bool ROPE>
static int wide_steps(const WideArgs& a, size_t workspace_floats, bool plan_only, long long* need, hipStream_t stream) {
    const int pairs = (a.K + 63) / 64, rounds = (pairs + NW - 1) / NW, cus = wide_cus();
    const double round_us = (double)NW * 2048.0 * NB * cus / 5e12 * 1e6;
    const double unit_cost = 0.4 / round_us, second_kernel = 4.0 / round_us;
    const int rows = a.M < 16 * MT ? a.M : 16 * MT;
    int best = 1;
    double best_cost = -1.0;
    for (int r = MAXSPW / 2; r >= 1; r /= 2) {
        const int slices = (rounds + r - 1) / r;
        const long long items = (long long)a.units * slices;
        const long long run = (items + cus - 1) / cus;
        double cost = (double)run * (r + unit_cost) + (double)((run + a.units - 1) / a.units) * rows / 16.0 * r / NB;
        if (run == 1) cost += 0.5 * r;
        if (slices > 1) cost += second_kernel + 0.1 * slices + (double)slices * a.M * a.N * 8.0 / ((double)NW * 2048.0 * cus);
        if (best_cost < 0 || cost < best_cost) { best = r; best_cost = cost; }
    }
    if constexpr (MAXSPW >= 8) if (best == 4) return wide_launch<MT, NW, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
    if constexpr (MAXSPW >= 4) if (best >= 2) return wide_launch<MT, NW, 4, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
    return wide_launch<MT, NW, 2, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
}

// Configurations by the number of row tiles and blocks of W: as many steps a wave as the registers hold
// (the A operands of a wave's steps for every tile, two units of W in flight), sixteen waves where a tile
// leaves room for them (a longer slice, fewer partial sums).
template <int NB, bool ROPE>
static int wide_dispatch(const WideArgs& a, size_t workspace_floats, bool plan_only, long long* need, hipStream_t stream) {
    const int mt = (a.M + 15) / 16;
    if constexpr (NB == 1) {
        switch (mt) {
            case 1: return wide_steps<1, 16, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            case 2: return wide_steps<2, 8, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            case 3: return wide_steps<3, 8, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            default: return wide_steps<4, 8, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
        }
    } else {
        switch (mt) {
            case 1: return wide_steps<1, 8, 8, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            case 2: return wide_steps<2, 8, 4, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            case 3: return wide_steps<3, 8, 4, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
            default: return wide_steps<4, 8, 4, NB, ROPE>(a, workspace_floats, plan_only, need, stream);
        }
    }
}

static bool wide_aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static int wide_entry(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R, int ldr, int M, int N,
                      int K, int out_dtype, int dual_off, float* workspace, long long workspace_floats, bool plan_only,
                      long long* need, hipStream_t stream, bool leave_partials = false) {
    if (need) *need = 0;
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K < 8 || K % 8 || lda % 8 || ldw % 8 || dual_off < 0 || workspace_floats < 0 ||
        (out_dtype != DT_F32 && out_dtype != DT_BF16) || (R && out_dtype != DT_F32) || (dual_off > 0 && R))
        return (int)hipErrorInvalidValue;
    if (!plan_only && (!wide_aligned16(A) || !wide_aligned16(W) || (!C && !leave_partials))) return (int)hipErrorInvalidValue;
    WideArgs a = {};
    a.leave_partials = leave_partials;
    a.A = (const bf16_t*)A; a.lda = lda; a.W = (const bf16_t*)W; a.ldw = ldw; a.C = C; a.ldc = ldc; a.out_dtype = out_dtype;
    a.R = R; a.ldr = ldr; a.P = workspace; a.M = M; a.N = N; a.K = K; a.units = (N + 15) / 16; a.dual_off = dual_off;
    return dual_off > 0 ? wide_dispatch<2, false>(a, (size_t)workspace_floats, plan_only, need, stream)
                        : wide_dispatch<1, false>(a, (size_t)workspace_floats, plan_only, need, stream);
}

// The fused q/k/v projection of a step of few rows against large weights: A bf16 [M, K] (normed), W = [Wq; Wk; Wv]
// (kv_heads 0: Wq only), rotary embedding of q and k over the whole head (head_dim % 16 == 0), q to q_out
// [M, heads * head_dim], k and v into the paged cache at `slots`.  Workspace as for cisr_gemm_wide_bf16 with
// N = (heads + 2 kv_heads) * head_dim.
extern "C" int cisr_qkv_rope_wide(const void* A, int lda, const void* W, int ldw, void* q_out, int ldq, int M, int K,
                                  const int* positions, const int* slots, const float* cos_tab, const float* sin_tab,
                                  void* kcache, void* vcache, int heads, int kv_heads, int head_dim, int page_size,
                                  int max_pos, float* workspace, long long workspace_floats, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 64 || K < 8 || K % 8 || lda % 8 || ldw % 8 || !wide_aligned16(A) || !wide_aligned16(W) || !q_out ||
        head_dim <= 0 || head_dim % 16 || heads <= 0 || kv_heads < 0 || page_size <= 0 || max_pos <= 0 || !positions ||
        !cos_tab || !sin_tab || (kv_heads > 0 && (!slots || !kcache || !vcache)) || workspace_floats < 0)
        return (int)hipErrorInvalidValue;
    WideArgs a = {};
    a.A = (const bf16_t*)A; a.lda = lda; a.W = (const bf16_t*)W; a.ldw = ldw; a.C = q_out; a.ldc = ldq; a.out_dtype = DT_BF16;
    a.P = workspace; a.M = M; a.N = (heads + 2 * kv_heads) * head_dim; a.K = K; a.units = a.N / 16;
    a.positions = positions; a.slots = slots; a.cos_tab = cos_tab; a.sin_tab = sin_tab; a.kcache = (bf16_t*)kcache;
    a.vcache = (bf16_t*)vcache; a.heads = heads; a.kv_heads = kv_heads; a.head_dim = head_dim; a.page_size = page_size;
    a.max_pos = max_pos;
    return wide_dispatch<1, true>(a, (size_t)workspace_floats, false, nullptr, stream);
}

// Floats of workspace that cisr_gemm_wide_bf16 needs for this shape (0: none), or -1 if it does not take the shape.
extern "C" long long cisr_gemm_wide_workspace(int M, int N, int K, int dual_off) {
    long long need = 0;
    const int err = wide_entry(nullptr, 8, nullptr, 8, nullptr, 0, nullptr, 0, M, N, K, DT_BF16, dual_off, nullptr, 0, true, &need, 0);
    return err ? -1 : need;
}

// C[M, N] = A[M, K] . W[N, K]^T (+ R), or with dual_off > 0 silu(A . Wg^T) * (A . Wu^T) over the blocks of W
// at rows 0 and dual_off.  A, W bf16 with 16-byte aligned rows, K % 8 == 0, M <= 64; C float or bf16; R float,
// with a float C.  `workspace` holds at least cisr_gemm_wide_workspace(...) floats; calls that share it must
// not overlap.
extern "C" int cisr_gemm_wide_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R, int ldr,
                                   int M, int N, int K, int out_dtype, int dual_off, float* workspace,
                                   long long workspace_floats, hipStream_t stream) {
    return wide_entry(A, lda, W, ldw, C, ldc, R, ldr, M, N, K, out_dtype, dual_off, workspace, workspace_floats, false,
                      nullptr, stream);
}

// The first pass alone, for a product that is cut into several slices (cisr_gemm_wide_workspace(M, N, K, 0) > 0; an
// error otherwise): workspace[s][M][N] holds the slices' partial sums of A . W^T, which the caller's next kernel
// adds in slice order (cisr_rmsnorm_partials, cisr_add_partials) instead of a second kernel here.
extern "C" int cisr_gemm_wide_partials_bf16(const void* A, int lda, const void* W, int ldw, int M, int N, int K,
                                            float* workspace, long long workspace_floats, hipStream_t stream) {
    return wide_entry(A, lda, W, ldw, nullptr, 0, nullptr, 0, M, N, K, DT_F32, 0, workspace, workspace_floats, false,
                      nullptr, stream, true);
}
