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
// VEC: rows are 16-byte aligned and K % 8 == 0, so a chunk lies wholly inside or outside; the load
// is unconditional from a clamped address (no branch between the loads of a tile, so they are all
// in flight together) and the result is zeroed by a select.  Otherwise element by element.
template <bool VEC>
__device__ __forceinline__ u32x4 load_chunk(const bf16_t* base, int ld, int row, int nrows, int k, int K) {
    if (VEC) {
        // no branch and nothing that touches the loaded value (it would wait for the load): rows
        // past the end read the last row (their products land in output rows or columns that are
        // never stored); a chunk past K reads the last chunk and is zeroed by a mask when the tile
        // is written to LDS, so that nothing is added to valid outputs
        const int rr = row < nrows ? row : nrows - 1;
        const int kk = k < K ? k : K - 8;
        return *(const u32x4*)(base + (size_t)rr * ld + kk);   // the caller masks chunks past K when it uses them
    }
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row >= nrows || k >= K) return v;
    const bf16_t* p = base + (size_t)row * ld + k;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (k + e < K) w[e / 2] |= ((uint32_t)p[e]) << (16 * (e % 2));
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
}

// Side of the patches in which tiles are numbered: `tiles` cut into the fewest parts of at most 8, evenly.
__host__ __device__ inline int patch_side(int tiles) {
    const int parts = (tiles + 7) / 8;
    return (tiles + parts - 1) / parts;
}

// Block tile (16 WM TM) x (32 TN), BK deep; WM x 2 waves (WM = 2 or 4), each wave TM x TN tiles of 16 x 16.
// The larger the block tile, the fewer bytes come from L2 per product: 128 x 128 is bound by the L2 at about
// a third of the matrix cores' peak, 256 x 128 moves a quarter less.
// Operands go global memory -> registers -> LDS -> matrix-core operands.
// The pipeline hides the global-memory latency inside one block, because small problems leave a
// compute unit with a single block: PF tiles of global loads are in flight in a ring of registers,
// and two LDS buffers let the next tile be written while the current one is multiplied, with one
// barrier per tile.
// SWIGLU: W holds two blocks of N rows, `dual_off` rows apart (gate, then up).  A wave's first TN/2
// column tiles take gate rows and its last TN/2 the up rows of the same output columns, so a lane ends
// with gate and up of one output element in its registers and writes silu(gate) * up (both rounded to
// bf16 first, as the two-kernel path does); a block then covers BN/2 output columns.
template <int TM, int TN, int BK, typename TC, bool VEC, bool SWIGLU = false, int WM = 2>
__global__ void __launch_bounds__(WM * 128)
gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
                 TC* C, int ldc, const float* R, int ldr, int M, int N, int K, int dual_off = 0) {
    static_assert(!SWIGLU || (TN % 2 == 0 && VEC), "the activation pairs column tiles");
    constexpr int BM = WM * TM * 16, BN = 2 * TN * 16, NT = WM * 128;   // WM x 2 waves
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;           // output columns a block covers
    constexpr int CPR = BK / 8;                            // 16-byte chunks per tile row
    // LDS rows are not padded; the 16-byte chunks of a row are permuted by a function of the row instead,
    // so that neither the copies into LDS (consecutive chunks of a few rows) nor the operand reads (one
    // chunk of 16 consecutive rows) meet in a bank
    auto lds_at = [](int row, int chunk) {
        const int turn = BK == 32 ? ((row >> 1) ^ (row >> 3)) : (row ^ (row >> 3));
        return row * BK + ((chunk ^ turn) & (CPR - 1)) * 8;
    };
    static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "a tile is a whole number of 16-byte chunks per thread");
    constexpr int A_PER_THREAD = BM * CPR / NT;
    constexpr int W_PER_THREAD = BN * CPR / NT;
    constexpr int PF = 3;                                  // tiles of global loads in flight
    __shared__ __attribute__((aligned(16))) bf16_t As[2][BM * BK];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[2][BN * BK];

    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;   // (uniform: scalar loop control)
    const int wm = wave / 2, wn = wave % 2;
    const int r = lane % 16, g = lane / 16;
    // The hardware deals consecutive workgroups round-robin to the 8 XCDs, each with an L2 of its own.
    // Renumber so that an XCD gets a contiguous run of tiles, and order the tiles in patches of up to
    // 8 x 8 (sides as even as the tile counts allow, so that few slots fall outside the matrix): the sixty-odd blocks that run on an XCD at one time then share 8 row bands of A and 8 of W
    // (16 bands from memory for 64 tiles) instead of one band of A and 64 of W.
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN_OUT - 1) / BN_OUT;
    const int gm = patch_side(tiles_m), gn = patch_side(tiles_n);
    const int patches_n = (tiles_n + gn - 1) / gn, patches = ((tiles_m + gm - 1) / gm) * patches_n;
    const int slots = patches * gm * gn;                   // tile slots (those outside the matrix do nothing)
    const int per_xcd = (slots + 7) / 8;
    const int slot = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (slot >= slots) return;                             // the grid is rounded up to a multiple of 8
    const int patch = slot / (gm * gn), in_patch = slot % (gm * gn);
    const int tile_m = (patch / patches_n) * gm + in_patch % gm, tile_n = (patch % patches_n) * gn + in_patch / gm;
    if (tile_m >= tiles_m || tile_n >= tiles_n) return;
    const int m0 = tile_m * BM, n0 = tile_n * BN_OUT;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    u32x4 ra[PF][A_PER_THREAD], rw[PF][W_PER_THREAD];
    auto fetch = [&](int k0, u32x4 (&fa)[A_PER_THREAD], u32x4 (&fw)[W_PER_THREAD]) {
#pragma unroll
        for (int i = 0; i < A_PER_THREAD; ++i) {
            const int c = tid + i * NT;
            fa[i] = load_chunk<VEC>(A, lda, m0 + c / CPR, M, k0 + (c % CPR) * 8, K);
        }
#pragma unroll
        for (int i = 0; i < W_PER_THREAD; ++i) {
            const int c = tid + i * NT;
            if (SWIGLU) {
                // local column -> (wave, column tile, column): the W row of its output column, gate or up
                const int lc = c / CPR, jj = (lc % (TN * 16)) / 16;
                const int oc = min(n0 + (lc / (TN * 16)) * (TN / 2) * 16 + (jj % (TN / 2)) * 16 + lc % 16, N - 1);
                fw[i] = load_chunk<VEC>(W, ldw, oc + (jj >= TN / 2 ? dual_off : 0), dual_off + N, k0 + (c % CPR) * 8, K);
            } else {
                fw[i] = load_chunk<VEC>(W, ldw, n0 + c / CPR, N, k0 + (c % CPR) * 8, K);
            }
        }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s) fetch(s * BK, ra[s], rw[s]);   // beyond K: zeros, never used

    int it = 0;
    for (int k0 = 0; k0 < K; k0 += PF * BK) {
#pragma unroll
        for (int s = 0; s < PF; ++s) {
            const int kk0 = k0 + s * BK;
            if (kk0 < K) {
                const int buf = it & 1;
                ++it;
#pragma unroll
                for (int i = 0; i < A_PER_THREAD; ++i) {
                    const int c = tid + i * NT;
                    const uint32_t keep = (VEC && kk0 + (c % CPR) * 8 >= K) ? 0u : 0xffffffffu;
                    u32x4 v = ra[s][i];
                    v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep;
                    *(u32x4*)(&As[buf][lds_at(c / CPR, c % CPR)]) = v;
                }
#pragma unroll
                for (int i = 0; i < W_PER_THREAD; ++i) {
                    const int c = tid + i * NT;
                    *(u32x4*)(&Ws[buf][lds_at(c / CPR, c % CPR)]) = rw[s][i];   // A is zero there: enough
                }
                // one barrier a tile: whoever writes this buffer again (two tiles on) has passed
                // the next tile's barrier, which every wave reaches only after reading this one
                __syncthreads();
                if (kk0 + PF * BK < K) fetch(kk0 + PF * BK, ra[s], rw[s]);
#pragma unroll
                for (int kk = 0; kk < BK; kk += 32) {
                    bf16x8 fa[TM], fw[TN];
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        fa[i] = *(const bf16x8*)(&As[buf][lds_at(wm * TM * 16 + i * 16 + r, kk / 8 + g)]);
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        fw[j] = *(const bf16x8*)(&Ws[buf][lds_at(wn * TN * 16 + j * 16 + r, kk / 8 + g)]);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
                }
            }
        }
    }
    if (SWIGLU) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN / 2; ++j) {
                const int n = n0 + wn * (TN / 2) * 16 + j * 16 + r;
                if (n >= N) continue;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = m0 + wm * TM * 16 + i * 16 + g * 4 + e;
                    const float gq = bf16_to_f32(f32_to_bf16(acc[i][j][e])), uq = bf16_to_f32(f32_to_bf16(acc[i][j + TN / 2][e]));
                    if (m < M) store_f32(C + (size_t)m * ldc + n, gq / (1.0f + expf(-gq)) * uq);
                }
            }
        return;
    }
    // lane holds rows 4g..4g+3 of column r in every 16 x 16 tile.  The residual is read with
    // unconditional loads from clamped addresses, all issued before the first is used.
    if (R) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = min(n0 + wn * TN * 16 + j * 16 + r, N - 1);
                float rv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = min(m0 + wm * TM * 16 + i * 16 + g * 4 + e, M - 1);
                    rv[e] = R[(size_t)m * ldr + n];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][e] += rv[e];
            }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * TN * 16 + j * 16 + r;
            if (n >= N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + wm * TM * 16 + i * 16 + g * 4 + e;
                if (m < M) store_f32(C + (size_t)m * ldc + n, acc[i][j][e]);
            }
        }
    }
}

// tile slots of the kernel's patch numbering (whole patches)
static long long tile_slots(long long tiles_m, long long tiles_n) {
    const long long gm = patch_side((int)tiles_m), gn = patch_side((int)tiles_n);
    return ((tiles_m + gm - 1) / gm) * ((tiles_n + gn - 1) / gn) * gm * gn;
}

template <int TM, int TN, int BK, int WM = 2>
static int launch_bf16(const bf16_t* A, int lda, const bf16_t* W, int ldw, void* C, int ldc, const float* R,
                       int ldr, int M, int N, int K, int out_dtype, hipStream_t stream) {
    constexpr int BM = WM * TM * 16, BN = 2 * TN * 16, NT = WM * 128;
    const long long slots = tile_slots((M + BM - 1) / BM, (N + BN - 1) / BN);
    if (slots > (1ll << 30)) return (int)hipErrorInvalidValue;
    dim3 grid((unsigned)((slots + 7) / 8 * 8));
    const bool vec = lda % 8 == 0 && ldw % 8 == 0 && K % 8 == 0 && ((uintptr_t)A) % 16 == 0 && ((uintptr_t)W) % 16 == 0;
    if (out_dtype == DT_F32) {
        if (vec) gemm_bf16_kernel<TM, TN, BK, float, true, false, WM><<<grid, NT, 0, stream>>>(A, lda, W, ldw, (float*)C, ldc, R, ldr, M, N, K);
        else gemm_bf16_kernel<TM, TN, BK, float, false, false, WM><<<grid, NT, 0, stream>>>(A, lda, W, ldw, (float*)C, ldc, R, ldr, M, N, K);
    } else {
        if (vec) gemm_bf16_kernel<TM, TN, BK, bf16_t, true, false, WM><<<grid, NT, 0, stream>>>(A, lda, W, ldw, (bf16_t*)C, ldc, R, ldr, M, N, K);
        else gemm_bf16_kernel<TM, TN, BK, bf16_t, false, false, WM><<<grid, NT, 0, stream>>>(A, lda, W, ldw, (bf16_t*)C, ldc, R, ldr, M, N, K);
    }
    return CISR_LAUNCH_CHECK();
}

// C[M, N] = silu(A . Wg^T) * (A . Wu^T), W = [Wg; Wu] with `dual_off` rows between the blocks; bf16 in and out,
// 16-byte aligned rows with K % 8 == 0.
template <int TM, int TN, int BK, int WM = 2>
static int launch_bf16_swiglu(const bf16_t* A, int lda, const bf16_t* W, int ldw, bf16_t* C, int ldc, int M, int N, int K,
                              int dual_off, hipStream_t stream) {
    constexpr int BM = WM * TM * 16, BN_OUT = TN * 16;
    const long long slots = tile_slots((M + BM - 1) / BM, (N + BN_OUT - 1) / BN_OUT);
    if (slots > (1ll << 30)) return (int)hipErrorInvalidValue;
    dim3 grid((unsigned)((slots + 7) / 8 * 8));
    gemm_bf16_kernel<TM, TN, BK, bf16_t, true, true, WM><<<grid, WM * 128, 0, stream>>>(A, lda, W, ldw, C, ldc, nullptr, 0, M, N, K, dual_off);
    return CISR_LAUNCH_CHECK();
}

// `tile`: 0 picks by the rule below; TM * 100 + TN * 10 + WM asks for that block tile (a tile that is not built: an error).
extern "C" int cisr_gemm_bf16_swiglu_tile(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                                          int dual_off, int tile, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || K % 8 || lda % 8 || ldw % 8 || ((uintptr_t)A) % 16 || ((uintptr_t)W) % 16 || dual_off < N)
        return (int)hipErrorInvalidValue;
    const bf16_t* a = (const bf16_t*)A; const bf16_t* w = (const bf16_t*)W;
    auto blocks = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((2 * N + bn - 1) / bn); };
    if (tile == 0) {
        if (blocks(128, 128) >= 512) tile = 442;
        else if (blocks(128, 64) >= 512) tile = 422;
        else if (blocks(64, 64) < 256) tile = 122;
        else tile = 222;
    }
#define SWIGLU_TILE(TM, TN, WM) \
    case TM * 100 + TN * 10 + WM: return launch_bf16_swiglu<TM, TN, 64, WM>(a, lda, w, ldw, (bf16_t*)C, ldc, M, N, K, dual_off, stream);
    switch (tile) {
        SWIGLU_TILE(1, 2, 2) SWIGLU_TILE(2, 2, 2) SWIGLU_TILE(4, 2, 2) SWIGLU_TILE(4, 4, 2)
    }
#undef SWIGLU_TILE
    return (int)hipErrorInvalidValue;
}

extern "C" int cisr_gemm_bf16_swiglu(const void* A, int lda, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                                     int dual_off, hipStream_t stream) {
    return cisr_gemm_bf16_swiglu_tile(A, lda, W, ldw, C, ldc, M, N, K, dual_off, 0, stream);
}

// Tile choice: the largest tile that still gives the 256 compute units a few blocks each; when even 64 x 64 leaves
// most of them idle (a portion of a few hundred rows against small weights), 32 x 64 and 32 x 32 (measured on an
// MI355X at 128 and 512 rows: 10-30 % faster there, slower from about one block a compute unit on).
// `tile`: 0 picks by this rule; TM * 100 + TN * 10 + WM asks for that block tile (a tile that is not built: an error).
extern "C" int cisr_gemm_bf16_tile(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R,
                                   int ldr, int M, int N, int K, int out_dtype, int tile, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || (R && out_dtype != DT_F32)) return (int)hipErrorInvalidValue;
    const bf16_t* a = (const bf16_t*)A; const bf16_t* w = (const bf16_t*)W;
    auto blocks = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    if (tile == 0) {
        if (M <= 32) tile = 122;
        else if (blocks(128, 128) >= 512) tile = 442;
        else if (blocks(128, 64) >= 512) tile = 422;
        else if (blocks(32, 64) <= 64) tile = 112;
        else if (blocks(64, 64) < 256) tile = 122;
        else tile = 222;
    }
#define GEMM_TILE(TM, TN, WM) \
    case TM * 100 + TN * 10 + WM: return launch_bf16<TM, TN, 64, WM>(a, lda, w, ldw, C, ldc, R, ldr, M, N, K, out_dtype, stream);
    switch (tile) {
        GEMM_TILE(1, 1, 2) GEMM_TILE(1, 2, 2) GEMM_TILE(2, 2, 2) GEMM_TILE(4, 2, 2) GEMM_TILE(4, 4, 2)
    }
#undef GEMM_TILE
    return (int)hipErrorInvalidValue;
}

extern "C" int cisr_gemm_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc, const float* R,
                              int ldr, int M, int N, int K, int out_dtype, hipStream_t stream) {
    return cisr_gemm_bf16_tile(A, lda, W, ldw, C, ldc, R, ldr, M, N, K, out_dtype, 0, stream);
}
