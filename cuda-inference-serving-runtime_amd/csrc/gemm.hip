// Matrix products  C[M,N] = A[M,K] . W[N,K]^T (+ R)  for linear layers whose
// weights are stored [out, in] (reference: runtime/blas.py:41-56 does the same
// product through a vendor library).
//
//  * gemm_f32: true 32-bit path.  float operands, FMA accumulation in float in
//    ascending k order, no matrix-core instruction and no reduced-precision mode.
//  * gemm_bf16: bf16 operands on the matrix cores (v_mfma_f32_16x16x32_bf16),
//    float accumulation; output float or bf16.
// Both take any M, N, K >= 1.  R (float, may be null, may alias a float C) is a
// residual added in the epilogue from the float accumulator.
#include "common.h"

// ------------------------------------------------------------------ float
#define F_BM 64
#define F_BN 64
#define F_BK 16

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
                float* C, int ldc, const float* R, int ldr, int M, int N, int K) {
    __shared__ float As[F_BK][F_BM + 4];
    __shared__ float Ws[F_BK][F_BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * F_BM, n0 = blockIdx.x * F_BN;
    const int ty = tid / 16, tx = tid % 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += F_BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + e][lr] = (am < M && k < K) ? A[(size_t)am * lda + k] : 0.f;
            Ws[lk + e][lr] = (wn < N && k < K) ? W[(size_t)wn * ldw + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < F_BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (R) v += R[(size_t)m * ldr + n];
            C[(size_t)m * ldc + n] = v;
        }
    }
}

extern "C" int cisr_gemm_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc,
                             const float* R, int ldr, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return (int)hipErrorInvalidValue;
    dim3 grid((N + F_BN - 1) / F_BN, (M + F_BM - 1) / F_BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, R, ldr, M, N, K);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------- bf16
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// 16 bytes = 8 bf16 from row-major global memory, zero-filled outside the matrix.
// `vec` says rows are 16-byte aligned (ld % 8 == 0 and base aligned).
__device__ __forceinline__ u32x4 load_chunk(const bf16_t* base, int ld, int row, int nrows, int k, int K, bool vec) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row >= nrows || k >= K) return v;
    const bf16_t* p = base + (size_t)row * ld + k;
    if (vec && k + 8 <= K) return *(const u32x4*)p;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (k + e < K) w[e / 2] |= ((uint32_t)p[e]) << (16 * (e % 2));
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
}

// Block tile (32 TM) x (32 TN), BK deep; four waves as 2 x 2, each wave TM x TN tiles of 16 x 16.
// Operands are staged through LDS (rows padded by 8 elements, so rows stay 16-byte aligned and the
// 16-byte operand reads of a wave spread over the banks); the next tile's global loads are in
// flight while the current one is multiplied.
template <int TM, int TN, int BK, typename TC>
__global__ void __launch_bounds__(256)
gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
                 TC* C, int ldc, const float* R, int ldr, int M, int N, int K, int vecA, int vecW) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    constexpr int STRIDE = BK + 8;
    constexpr int CPR = BK / 8;                            // 16-byte chunks per tile row
    constexpr int A_PER_THREAD = (BM * CPR + 255) / 256;
    constexpr int W_PER_THREAD = (BN * CPR + 255) / 256;
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * STRIDE];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[BN * STRIDE];

    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int r = lane % 16, g = lane / 16;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    u32x4 ra[A_PER_THREAD], rw[W_PER_THREAD];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_PER_THREAD; ++i) {
            const int c = tid + i * 256;
            if (c < BM * CPR) ra[i] = load_chunk(A, lda, m0 + c / CPR, M, k0 + (c % CPR) * 8, K, vecA);
        }
#pragma unroll
        for (int i = 0; i < W_PER_THREAD; ++i) {
            const int c = tid + i * 256;
            if (c < BN * CPR) rw[i] = load_chunk(W, ldw, n0 + c / CPR, N, k0 + (c % CPR) * 8, K, vecW);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int i = 0; i < A_PER_THREAD; ++i) {
            const int c = tid + i * 256;
            if (c < BM * CPR) *(u32x4*)(As + (c / CPR) * STRIDE + (c % CPR) * 8) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_PER_THREAD; ++i) {
            const int c = tid + i * 256;
            if (c < BN * CPR) *(u32x4*)(Ws + (c / CPR) * STRIDE + (c % CPR) * 8) = rw[i];
        }
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 32) {
            bf16x8 fa[TM], fw[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *(const bf16x8*)(As + (wm * TM * 16 + i * 16 + r) * STRIDE + kk + g * 8);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fw[j] = *(const bf16x8*)(Ws + (wn * TN * 16 + j * 16 + r) * STRIDE + kk + g * 8);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // lane holds rows 4g..4g+3 of column r in every 16 x 16 tile
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * TN * 16 + j * 16 + r;
            if (n >= N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + wm * TM * 16 + i * 16 + g * 4 + e;
                if (m >= M) continue;
                float v = acc[i][j][e];
                if (R) v += R[(size_t)m * ldr + n];
                store_f32(C + (size_t)m * ldc + n, v);
            }
        }
    }
}

template <int TM, int TN, int BK>
static int launch_bf16(const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, const float* R,
                       int ldr, int M, int N, int K, int out_dtype, hipStream_t stream) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    const int vecA = (lda % 8 == 0) && (((uintptr_t)A) % 16 == 0);
    const int vecW = (ldw % 8 == 0) && (((uintptr_t)W) % 16 == 0);
    if (out_dtype == DT_F32)
        gemm_bf16_kernel<TM, TN, BK, float><<<grid, 256, 0, stream>>>(A, lda, W, ldw, (float*)C, ldc, R, ldr, M, N, K, vecA, vecW);
    else
        gemm_bf16_kernel<TM, TN, BK, bf16_t><<<grid, 256, 0, stream>>>(A, lda, W, ldw, (bf16_t*)C, ldc, R, ldr, M, N, K, vecA, vecW);
    return CISR_LAUNCH_CHECK();
}

// Tile choice: the largest tile that still gives the 256 compute units a few blocks each.
extern "C" int cisr_gemm_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R,
                              int ldr, int M, int N, int K, int out_dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || (R && out_dtype != DT_F32)) return (int)hipErrorInvalidValue;
    const bf16_t* a = (const bf16_t*)A; const bf16_t* w = (const bf16_t*)W;
    auto blocks = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (M <= 32) return launch_bf16<1, 2, 64>(a, lda, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, stream);
    if (blocks(128, 128) >= 512) return launch_bf16<4, 4, 32>(a, lda, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, stream);
    if (blocks(128, 64) >= 512) return launch_bf16<4, 2, 64>(a, lda, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, stream);
    return launch_bf16<2, 2, 64>(a, lda, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, stream);
}
