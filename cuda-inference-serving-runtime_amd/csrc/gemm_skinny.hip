// Skinny matrix products for decode steps:  C[M,N] = A[M,K] . W[N,K]^T  with
// M <= 64 rows.  The product is bound by reading W once from HBM, so the kernel
// is laid out around streaming W: a block owns 16 rows of W (16 output columns),
// its waves (4, or 16 for a short K) split K in interleaved 32-wide steps, every
// lane loads 16 contiguous bytes of a W row straight into a matrix-core operand
// (v_mfma_f32_16x16x32_bf16, A as the first operand, W as the second), and the
// waves' partial tiles are summed through LDS in a fixed order, so a row's result
// does not depend on how many rows are beside it.
//
// Prologue (NORM): A is the float residual stream and the kernel applies RMSNorm
// on the fly: the operand is bf16(x[m,k] * w_norm[k]); the sum of squares of
// the same loads gives rsqrt(mean(x^2) + eps), applied to the finished row
// (a per-row factor commutes with the product).  `rows` picks input rows.
// Epilogues, all from the float accumulator:
//   EPI_STORE   store float or bf16, optional float residual add
//   EPI_SWIGLU  two weight blocks `dual_off` rows apart: out = silu(g) * u
//   EPI_ROPE    the fused q/k/v projection: a block owns 8 rotary pairs
//               (i, i + D/2) of one head, rotates q and k by the row's position,
//               writes q to its buffer and k, v into the paged cache.
// Requires K % 8 == 0 and 16-byte aligned rows; callers fall back otherwise.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_ROPE = 2 };

struct SkinnyArgs {
    const void* A; int lda;            // bf16 activations, or float residual with NORM
    const bf16_t* W; int ldw;
    void* C; int ldc;                  // EPI_ROPE: q output, bf16 [M, heads*D]
    const float* R; int ldr;           // residual (EPI_STORE, float C only)
    int M, N, K;
    int dual_off;                      // EPI_SWIGLU
    // NORM
    const float* norm_w; float eps; const int* rows;
    // EPI_ROPE
    const int* positions; const int* slots; const float* cos_tab; const float* sin_tab;
    bf16_t* kcache; bf16_t* vcache; int heads, kv_heads, head_dim, page_size, max_pos;
};

__device__ __forceinline__ bf16x8 ld16(const bf16_t* p, bool ok) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (ok) v = *(const u32x4*)p;
    return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ uint32_t pack2(float a, float b) {
    return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}

// NW: wavefronts a block (4 or 16).  A short K is split over 16 waves so that every wave
// issues all its loads at once (one trip to memory); a long K over 4 waves that keep
// several steps of loads in flight.
template <int MT, bool NORM, int EPI, typename TC, int NW>
__global__ void __launch_bounds__(NW * 64)
gemm_skinny_kernel(SkinnyArgs p) {
    constexpr int NB = EPI == EPI_SWIGLU ? 2 : 1;
    constexpr int UNROLL = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
    extern __shared__ float smem[];
    float (*red)[NB][MT][WAVE][4] = reinterpret_cast<float (*)[NB][MT][WAVE][4]>(smem);
    float (*ssq)[MT][16] = reinterpret_cast<float (*)[MT][16]>(smem + NW * NB * MT * WAVE * 4);
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int r = lane % 16, g = lane / 16;
    const int M = p.M, N = p.N, K = p.K;

    // which 16 rows of W this block owns
    int n0 = blockIdx.x * 16, wn;
    int slot_head = 0, j0 = 0;
    if (EPI == EPI_ROPE) {
        const int per_head = p.head_dim / 16;          // blocks per head: 8 pairs each
        slot_head = blockIdx.x / per_head;
        j0 = (blockIdx.x % per_head) * 8;
        wn = slot_head * p.head_dim + (r < 8 ? j0 + r : p.head_dim / 2 + j0 + r - 8);
    } else {
        wn = min(n0 + r, N - 1);                        // rows past N are loaded but never stored
    }
    const bf16_t* wrow0 = p.W + (size_t)wn * p.ldw + g * 8;
    const bf16_t* wrow1 = p.W + (size_t)(wn + p.dual_off) * p.ldw + g * 8;

    const bf16_t* arow[MT];
    const float* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        int m = min(t * 16 + r, M - 1);
        if (NORM) {
            if (p.rows) m = p.rows[m];
            xrow[t] = (const float*)p.A + (size_t)m * p.lda + g * 8;
        } else {
            arow[t] = (const bf16_t*)p.A + (size_t)m * p.lda + g * 8;
        }
    }

    f32x4 acc[NB][MT];
    float ss[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        ss[t] = 0.f;
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    // this wave's k-steps: wave, wave + 4, ...; K % 8 == 0, so a 16-byte chunk is inside K or outside
#pragma unroll UNROLL
    for (int k0 = wave * 32; k0 < K; k0 += NW * 32) {
        const bool ok = k0 + g * 8 < K;
        const bf16x8 wf0 = ld16(wrow0 + k0, ok);
        bf16x8 wf1;
        if (EPI == EPI_SWIGLU) wf1 = ld16(wrow1 + k0, ok);
        f32x4 nw0 = {0.f, 0.f, 0.f, 0.f}, nw1 = {0.f, 0.f, 0.f, 0.f};
        if (NORM && ok) {
            nw0 = *(const f32x4*)(p.norm_w + k0 + g * 8);
            nw1 = *(const f32x4*)(p.norm_w + k0 + g * 8 + 4);
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            bf16x8 af;
            if (NORM) {
                f32x4 x0 = {0.f, 0.f, 0.f, 0.f}, x1 = {0.f, 0.f, 0.f, 0.f};
                if (ok) { x0 = *(const f32x4*)(xrow[t] + k0); x1 = *(const f32x4*)(xrow[t] + k0 + 4); }
                ss[t] += x0.x * x0.x + x0.y * x0.y + x0.z * x0.z + x0.w * x0.w
                       + x1.x * x1.x + x1.y * x1.y + x1.z * x1.z + x1.w * x1.w;
                u32x4 pk = {pack2(x0.x * nw0.x, x0.y * nw0.y), pack2(x0.z * nw0.z, x0.w * nw0.w),
                            pack2(x1.x * nw1.x, x1.y * nw1.y), pack2(x1.z * nw1.z, x1.w * nw1.w)};
                af = __builtin_bit_cast(bf16x8, pk);
            } else {
                af = ld16(arow[t] + k0, ok);
            }
            acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, wf0, acc[0][t], 0, 0, 0);
            if (EPI == EPI_SWIGLU) acc[NB - 1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, wf1, acc[NB - 1][t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][b][t][lane][e] = acc[b][t][e];
    if (NORM) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            float v = ss[t];
            v += __shfl_xor(v, 16, WAVE);
            v += __shfl_xor(v, 32, WAVE);
            if (g == 0) ssq[wave][t][r] = v;
        }
    }
    __syncthreads();
    // thread -> (l2 = tid % 64, e2 = tid / 64): element (m = 16 t + 4 (l2 / 16) + e2, column c = l2 % 16)
    if (tid >= 256) return;
    const int l2 = tid % WAVE, e2 = tid / WAVE, c = l2 % 16;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int ml = (l2 / 16) * 4 + e2;              // row inside the 16-row tile
        const int m = t * 16 + ml;
        if (m >= M) continue;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += red[w][0][t][l2][e2];
        float scale = 1.f;
        if (NORM) {
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) total += ssq[w][t][ml];
            scale = 1.0f / sqrtf(total / (float)K + p.eps);
            v *= scale;
        }
        if (EPI == EPI_SWIGLU) {
            float u = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) u += red[w][NB - 1][t][l2][e2];
            u *= scale;
            // the two-kernel path rounds gate and up to bf16 before the activation; do the same
            const float gq = bf16_to_f32(f32_to_bf16(v)), uq = bf16_to_f32(f32_to_bf16(u));
            v = gq / (1.0f + expf(-gq)) * uq;
        }
        if (EPI == EPI_ROPE) {
            // partner column (the other half of the rotary pair) sits 8 lanes away
            const int lp = l2 ^ 8;
            float pv = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) pv += red[w][0][t][lp][e2];
            pv *= scale;
            const int D = p.head_dim, half = D / 2;
            const int i = j0 + (c & 7);
            const int col = c < 8 ? i : half + i;
            if (slot_head < p.heads + p.kv_heads) {      // q or k head: rotate
                int pos = p.positions[m];
                pos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
                const float cs = p.cos_tab[(size_t)pos * half + i], sn = p.sin_tab[(size_t)pos * half + i];
                v = c < 8 ? v * cs - pv * sn : v * cs + pv * sn;
            }
            if (slot_head < p.heads) {
                ((bf16_t*)p.C)[(size_t)m * p.ldc + slot_head * D + col] = f32_to_bf16(v);
            } else {
                const int slot = p.slots[m];
                if (slot >= 0) {
                    const int page = slot / p.page_size, off = slot % p.page_size;
                    if (slot_head < p.heads + p.kv_heads) {
                        const int h = slot_head - p.heads;
                        p.kcache[(((size_t)page * p.kv_heads + h) * p.page_size + off) * D + col] = f32_to_bf16(v);
                    } else {
                        const int h = slot_head - p.heads - p.kv_heads;
                        p.vcache[(((size_t)page * p.kv_heads + h) * D + col) * p.page_size + off] = f32_to_bf16(v);
                    }
                }
            }
            continue;
        }
        const int n = n0 + c;
        if (n >= N) continue;
        if (p.R) v += p.R[(size_t)m * p.ldr + n];
        store_f32((TC*)p.C + (size_t)m * p.ldc + n, v);
    }
}

template <int MT, bool NORM, int EPI, typename TC, int NW>
static int launch_one(const SkinnyArgs& a, int blocks, hipStream_t stream) {
    constexpr int NB = EPI == EPI_SWIGLU ? 2 : 1;
    const size_t shmem = ((size_t)NW * NB * MT * WAVE * 4 + (size_t)NW * MT * 16) * sizeof(float);
    if (shmem > 65536) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, NORM, EPI, TC, NW>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return (int)e;
    }
    gemm_skinny_kernel<MT, NORM, EPI, TC, NW><<<blocks, NW * 64, shmem, stream>>>(a);
    return CISR_LAUNCH_CHECK();
}

template <bool NORM, int EPI, typename TC>
static int launch_mt(const SkinnyArgs& a, int blocks, hipStream_t stream) {
    // a short inner size with few blocks is split over 16 waves: at most 8 steps of 32 each, all loads
    // issued at once; with many blocks (a vocabulary) four waves a block fill the GPU without that
    const bool wide = a.K <= 16 * 32 * 8 && blocks <= 1024;
    if (a.M <= 16) return wide ? launch_one<1, NORM, EPI, TC, 16>(a, blocks, stream) : launch_one<1, NORM, EPI, TC, 4>(a, blocks, stream);
    if (a.M <= 32) return wide ? launch_one<2, NORM, EPI, TC, 16>(a, blocks, stream) : launch_one<2, NORM, EPI, TC, 4>(a, blocks, stream);
    if (a.M <= 48) return wide ? launch_one<3, NORM, EPI, TC, 16>(a, blocks, stream) : launch_one<3, NORM, EPI, TC, 4>(a, blocks, stream);
    return wide ? launch_one<4, NORM, EPI, TC, 16>(a, blocks, stream) : launch_one<4, NORM, EPI, TC, 4>(a, blocks, stream);
}

static bool aligned16(const void* p) { return ((uintptr_t)p) % 16 == 0; }

// Plain / residual / SwiGLU forms.  A is bf16 [M, K], or with norm_w != null the float residual
// [*, K] (rows picked by `rows` if given).  dual_off > 0 selects SwiGLU over two blocks of N rows of W.
extern "C" int cisr_gemm_skinny_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R,
                                     int ldr, int M, int N, int K, int out_dtype, int dual_off, const float* norm_w,
                                     float eps, const int* rows, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 || lda % 8 || ldw % 8 || !aligned16(A) || !aligned16(W) ||
        (R && out_dtype != DT_F32) || (norm_w && !aligned16(norm_w)) || (dual_off > 0 && (R || out_dtype != DT_BF16)))
        return (int)hipErrorInvalidValue;
    SkinnyArgs a = {};
    a.A = A; a.lda = lda; a.W = (const bf16_t*)W; a.ldw = ldw; a.C = C; a.ldc = ldc; a.R = R; a.ldr = ldr;
    a.M = M; a.N = N; a.K = K; a.dual_off = dual_off; a.norm_w = norm_w; a.eps = eps; a.rows = rows;
    const int blocks = (N + 15) / 16;
    if (dual_off > 0)
        return norm_w ? launch_mt<true, EPI_SWIGLU, bf16_t>(a, blocks, stream) : launch_mt<false, EPI_SWIGLU, bf16_t>(a, blocks, stream);
    if (out_dtype == DT_F32)
        return norm_w ? launch_mt<true, EPI_STORE, float>(a, blocks, stream) : launch_mt<false, EPI_STORE, float>(a, blocks, stream);
    return norm_w ? launch_mt<true, EPI_STORE, bf16_t>(a, blocks, stream) : launch_mt<false, EPI_STORE, bf16_t>(a, blocks, stream);
}

// The fused q/k/v projection of a decode step: RMSNorm of the float residual (norm_w may be null: A is
// then bf16 and already normed), product with W = [Wq; Wk; Wv], rotary embedding of q and k over the whole
// head (head_dim % 16 == 0), q to `q_out` [M, heads*head_dim], k and v into the paged cache at `slots`.
extern "C" int cisr_qkv_rope_skinny(const void* A, int lda, const void* W, int ldw, void* q_out, int ldq, int M, int K,
                                    const float* norm_w, float eps, const int* positions, const int* slots,
                                    const float* cos_tab, const float* sin_tab, void* kcache, void* vcache, int heads,
                                    int kv_heads, int head_dim, int page_size, int max_pos, hipStream_t stream) {
    if (M <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 || lda % 8 || ldw % 8 || !aligned16(A) || !aligned16(W) || head_dim % 16 ||
        head_dim <= 0 || page_size <= 0 || (norm_w && !aligned16(norm_w)))
        return (int)hipErrorInvalidValue;
    SkinnyArgs a = {};
    a.A = A; a.lda = lda; a.W = (const bf16_t*)W; a.ldw = ldw; a.C = q_out; a.ldc = ldq;
    a.M = M; a.N = (heads + 2 * kv_heads) * head_dim; a.K = K; a.norm_w = norm_w; a.eps = eps;
    a.positions = positions; a.slots = slots; a.cos_tab = cos_tab; a.sin_tab = sin_tab;
    a.kcache = (bf16_t*)kcache; a.vcache = (bf16_t*)vcache; a.heads = heads; a.kv_heads = kv_heads;
    a.head_dim = head_dim; a.page_size = page_size; a.max_pos = max_pos;
    const int blocks = (heads + 2 * kv_heads) * (head_dim / 16);
    return norm_w ? launch_mt<true, EPI_ROPE, bf16_t>(a, blocks, stream) : launch_mt<false, EPI_ROPE, bf16_t>(a, blocks, stream);
}
