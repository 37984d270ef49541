// Arguments of the skinny (M <= 64) bf16 matrix-product kernels and the entry points that the
// per-row-count translation units export (one unit per number of 16-row tiles, so that they
// compile in parallel).
#pragma once
#include "common.h"

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
    // merge prologue of the narrow kernels (A = the split decode attention's partial results, not yet merged):
    // normalised partial outputs bf16 [M, merge_heads, splits, merge_dim], statistics float [M, merge_heads, splits, 2]
    // (maximum in log2 units, denominator); K = merge_heads * merge_dim
    const bf16_t* part_o; const float* part_ml; int merge_heads, merge_dim;
};


// one function per MT = number of 16-row tiles of A (M <= 16 MT)
int cisr_skinny_launch_m1(const SkinnyArgs& a, int blocks, bool norm, int epi, int out_dtype, hipStream_t stream);
int cisr_skinny_launch_m2(const SkinnyArgs& a, int blocks, bool norm, int epi, int out_dtype, hipStream_t stream);
int cisr_skinny_launch_m3(const SkinnyArgs& a, int blocks, bool norm, int epi, int out_dtype, hipStream_t stream);
int cisr_skinny_launch_m4(const SkinnyArgs& a, int blocks, bool norm, int epi, int out_dtype, hipStream_t stream);

// The narrow kernels (gemm_narrow.inc): four output columns a block, at most 16 rows of A, in tiles of four rows;
// one function per number of tiles.  `units` = blocks: ceil(N / 4), or with EPI_ROPE (heads + 2 kv_heads) head_dim / 4.
int cisr_narrow_launch_t1(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, hipStream_t stream);
int cisr_narrow_launch_t2(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, hipStream_t stream);
int cisr_narrow_launch_t4(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, hipStream_t stream);
// the same with the merge prologue (2, 4 or 8 splits): float output with the residual added
int cisr_narrow_merge_launch_t1(const SkinnyArgs& a, int units, int splits, hipStream_t stream);
int cisr_narrow_merge_launch_t2(const SkinnyArgs& a, int units, int splits, hipStream_t stream);
int cisr_narrow_merge_launch_t4(const SkinnyArgs& a, int units, int splits, hipStream_t stream);

// The matrix-vector kernel (gemv.hip): at most GEMV_MAX_ROWS rows of A, whole rows of W a wave.  `units`: N, or with
// EPI_ROPE the rotary pairs (heads + 2 kv_heads) head_dim / 2; `splits` > 0 selects the merge prologue (2, 4, 8).
#define GEMV_MAX_ROWS 8
bool cisr_gemv_takes(int M, int K);
int cisr_gemv_launch(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, int splits, hipStream_t stream);
