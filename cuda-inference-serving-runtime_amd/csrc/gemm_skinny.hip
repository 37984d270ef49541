// Skinny matrix products for decode steps:  C[M,N] = X[M,K] . W[N,K]^T  with
// M <= 64 rows.  The product is bound by reading W once from HBM, so the kernel
// is laid out around streaming W: a block owns 16 rows of W (16 output columns),
// its four waves split K in interleaved 32-wide steps, every lane loads 16
// contiguous bytes of a W row straight into a matrix-core operand
// (v_mfma_f32_16x16x32_bf16, X as the A operand, W as the B operand), and the
// four partial tiles are summed through LDS in a fixed order.  Epilogues, all
// from the float accumulator: plain store (float or bf16), residual add, or
// SwiGLU of two weight row blocks (row n of the gate with row n of the up
// projection: out = silu(g) * u).
// Requires K % 8 == 0 and 16-byte aligned rows; the caller falls back to the
// general kernel otherwise.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 ld16(const bf16_t* p, bool ok) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (ok) v = *(const u32x4*)p;
    return __builtin_bit_cast(bf16x8, v);
}

// MT: number of 16-row tiles of X (M <= 16*MT).  DUAL: second weight block at
// row offset `dual_off` (SwiGLU).  TC: output type.
template <int MT, bool DUAL, typename TC>
__global__ void __launch_bounds__(256)
gemm_skinny_kernel(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw,
                   TC* C, int ldc, const float* R, int ldr, int M, int N, int K, int dual_off) {
    constexpr int NB = DUAL ? 2 : 1;
    __shared__ float red[4][NB][MT][WAVE][4];
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int r = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int wn = min(n0 + r, N - 1);                 // clamped: rows past N are loaded but never stored
    const bf16_t* wrow0 = W + (size_t)wn * ldw + g * 8;
    const bf16_t* wrow1 = W + (size_t)(wn + dual_off) * ldw + g * 8;
    const bf16_t* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xrow[t] = X + (size_t)min(t * 16 + r, M - 1) * ldx + g * 8;

    f32x4 acc[NB][MT];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[b][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // this wave's k-steps: wave, wave + 4, ...; K % 8 == 0 so a 16-byte chunk is inside K or outside
#pragma unroll 4
    for (int k0 = wave * 32; k0 < K; k0 += 4 * 32) {
        const bool ok = k0 + g * 8 < K;
        bf16x8 wf0 = ld16(wrow0 + k0, ok);
        bf16x8 wf1;
        if (DUAL) wf1 = ld16(wrow1 + k0, ok);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            bf16x8 xf = ld16(xrow[t] + k0, ok);
            acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wf0, acc[0][t], 0, 0, 0);
            if (DUAL) acc[NB - 1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wf1, acc[NB - 1][t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][b][t][lane][e] = acc[b][t][e];
    __syncthreads();
    // thread -> (lane' = tid % 64, e' = tid / 64): element (m = 16 t + 4 (lane'/16) + e', n = n0 + lane' % 16)
    const int l2 = tid % WAVE, e2 = tid / WAVE;
    const int n = n0 + l2 % 16;
    if (n >= N) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + (l2 / 16) * 4 + e2;
        if (m >= M) continue;
        float v = red[0][0][t][l2][e2] + red[1][0][t][l2][e2] + red[2][0][t][l2][e2] + red[3][0][t][l2][e2];
        if (DUAL) {
            float u = red[0][NB - 1][t][l2][e2] + red[1][NB - 1][t][l2][e2] + red[2][NB - 1][t][l2][e2] + red[3][NB - 1][t][l2][e2];
            // the unfused path rounds gate and up to bf16 before the activation; do the same
            float gq = bf16_to_f32(f32_to_bf16(v)), uq = bf16_to_f32(f32_to_bf16(u));
            v = gq / (1.0f + expf(-gq)) * uq;
        }
        if (R) v += R[(size_t)m * ldr + n];
        store_f32(C + (size_t)m * ldc + n, v);
    }
}

template <int MT>
static int launch_skinny(const bf16_t* X, int ldx, const bf16_t* W, int ldw, void* C, int ldc, const float* R, int ldr,
                         int M, int N, int K, int out_dtype, int dual_off, hipStream_t stream) {
    dim3 grid((N + 15) / 16);
    if (dual_off > 0) {
        if (out_dtype == DT_F32)
            gemm_skinny_kernel<MT, true, float><<<grid, 256, 0, stream>>>(X, ldx, W, ldw, (float*)C, ldc, R, ldr, M, N, K, dual_off);
        else
            gemm_skinny_kernel<MT, true, bf16_t><<<grid, 256, 0, stream>>>(X, ldx, W, ldw, (bf16_t*)C, ldc, R, ldr, M, N, K, dual_off);
    } else {
        if (out_dtype == DT_F32)
            gemm_skinny_kernel<MT, false, float><<<grid, 256, 0, stream>>>(X, ldx, W, ldw, (float*)C, ldc, R, ldr, M, N, K, 0);
        else
            gemm_skinny_kernel<MT, false, bf16_t><<<grid, 256, 0, stream>>>(X, ldx, W, ldw, (bf16_t*)C, ldc, R, ldr, M, N, K, 0);
    }
    return CISR_LAUNCH_CHECK();
}

// N counts output columns.  dual_off > 0: W has 2 blocks of N rows, `dual_off` rows apart, and the output
// is silu(X W0^T) * (X W1^T).
extern "C" int cisr_gemm_skinny_bf16(const void* X, int ldx, const void* W, int ldw, void* C, int ldc, const float* R,
                                     int ldr, int M, int N, int K, int out_dtype, int dual_off, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ((uintptr_t)X) % 16 || ((uintptr_t)W) % 16 ||
        (R && out_dtype != DT_F32))
        return (int)hipErrorInvalidValue;
    const bf16_t* x = (const bf16_t*)X; const bf16_t* w = (const bf16_t*)W;
    if (M <= 16) return launch_skinny<1>(x, ldx, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, dual_off, stream);
    if (M <= 32) return launch_skinny<2>(x, ldx, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, dual_off, stream);
    if (M <= 48) return launch_skinny<3>(x, ldx, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, dual_off, stream);
    return launch_skinny<4>(x, ldx, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, dual_off, stream);
}
