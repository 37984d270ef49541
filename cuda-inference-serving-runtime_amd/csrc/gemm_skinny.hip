// Entry points of the skinny (M <= 64) bf16 matrix products; the kernels live in gemm_skinny.inc,
// compiled once per number of 16-row tiles (gemm_skinny_m1..m4.hip).
#include "gemm_skinny.h"

// More than 16 rows of A: the kernels take up to 64 rows a block (MT tiles of 16), but a narrow output then has few
// blocks, each with all rows' partial tiles to add up.  Such a product runs as groups of 16 MT rows instead (a block
// a group and 16 columns; the groups stream the same rows of W), with the largest MT that still gives ENOUGH_BLOCKS.
// Measured on an MI355X (captured chains, 135M sizes, 64 rows; one block of 64 rows -> four of 16): output projection
// 5.1 -> 3.3 us, down 8.9 -> 4.9, norm + q/k/v + rotary 8.7 -> 4.9, norm + gate/up + SwiGLU 9.2 -> 7.4 (7.9 as two
// groups of 32 rows); a wide output (a vocabulary) has blocks enough and keeps all rows in one block, which reads W once.
#define ENOUGH_BLOCKS 400
static int launch_rows(const SkinnyArgs& a, int blocks, bool norm, int epi, int out_dtype, hipStream_t stream) {
    int mt = (a.M + 15) / 16;                        // tiles that hold all rows: one group
    while (mt > 1 && (long long)blocks * ((a.M + 16 * mt - 1) / (16 * mt)) < ENOUGH_BLOCKS) --mt;
    if (mt <= 1) return cisr_skinny_launch_m1(a, blocks, norm, epi, out_dtype, stream);
    if (mt == 2) return cisr_skinny_launch_m2(a, blocks, norm, epi, out_dtype, stream);
    if (mt == 3) return cisr_skinny_launch_m3(a, blocks, norm, epi, out_dtype, stream);
    return cisr_skinny_launch_m4(a, blocks, norm, epi, out_dtype, stream);
}

static bool aligned16(const void* p) { return ((uintptr_t)p) % 16 == 0; }

// Up to four rows against weights of 4 MB and more: the matrix-vector kernel (gemv.hip).  Measured on an MI355X, decode
// steps in captured programs (ms a step without it -> with it): 1.7B sizes, 8 layers, one request 0.537 -> 0.441, two
// 0.571 -> 0.506; 8B sizes, 8 layers, 1.239 -> 1.066 and 1.254 -> 1.130.  Three and four rows lost while it read the
// weights with ordinary loads (0.608 -> 0.636, 1.325 -> 1.448) and win with non-temporal ones (1.7B sizes 0.604 ->
// 0.568 and 0.609 -> 0.578, 8B sizes 1.315 -> 1.236 and 1.322 -> 1.241); six and eight rows lose by half (0.673 ->
// 1.026, 1.311 -> 1.780: every row more is another read of LDS and another set of dot instructions for every 16 bytes
// of W), and so do the small weights of the 135M sizes at any number of rows (one request 0.670 -> 0.751: there a product is its
// prologue and epilogue, and the narrow kernel's are shorter; a form of this kernel for such weights that is a single
// trip to memory, a unit a wave, no LDS and no barrier, came to the narrow kernel's times within 3 %, one request 0.668
// -> 0.684, and lost with two, 0.682 -> 0.799: not kept).  The most rows it is given and the least bytes can be
// set (cisr_gemv_set: rows 0 switches it off), for measurements of one kernel against the other and for tests.
static int gemv_rows = 4;
static long long gemv_bytes = 4ll << 20;
extern "C" void cisr_gemv_set(int rows, long long least_bytes) {
    gemv_rows = rows < 0 ? 0 : rows > GEMV_MAX_ROWS ? GEMV_MAX_ROWS : rows;
    gemv_bytes = least_bytes < 0 ? 0 : least_bytes;
}
// The inner size must be at least `gemv_inner`: a row of W shorter than two rounds of a wave's lanes leaves most lanes
// idle, and the kernel is then its per-row work (the head of the 135M sizes, 49,152 rows of 576: 36 us against 15.7).
// A least size of 0 bytes lifts that too.  `N`: rows of W that the product reads (both blocks of a gated product).
static int gemv_inner = 1024;
extern "C" int cisr_gemv_ok(int M, int N, int K) {
    return M <= gemv_rows && (long long)N * K * 2 >= gemv_bytes && (K >= gemv_inner || gemv_bytes == 0) && cisr_gemv_takes(M, K);
}

// Few rows against small weights with a narrow output: a block for every 16 columns would leave most compute
// units idle, so the narrow kernels take over (a block for every 4 columns).  Measured on an MI355X in captured
// chains: the down projection of the 135M sizes (8 rows, 576 x 1536) 4.3 us with 36 blocks of 16 columns.
static bool narrow_wanted(int M, int N, int K, bool norm) {
    const int rows = M <= 4 ? 4 : M <= 8 ? 8 : 16;
    // with the norm fused, a block's rows must fit LDS and be one batch of loads: inner sizes up to 1024, 640, 576
    if (norm && ((size_t)rows * (K + 8) * 2 > 40 * 1024 || K > (rows == 4 ? 1024 : rows == 8 ? 640 : 576))) return false;
    return M <= 16 && (N + 15) / 16 < 256 && (long long)N * K * 2 <= (4LL << 20);
}

static int launch_narrow(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, hipStream_t stream) {
    if (a.M <= 4) return cisr_narrow_launch_t1(a, units, norm, epi, out_dtype, stream);
    if (a.M <= 8) return cisr_narrow_launch_t2(a, units, norm, epi, out_dtype, stream);
    return cisr_narrow_launch_t4(a, units, norm, epi, out_dtype, stream);
}

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
    const int epi = dual_off > 0 ? EPI_SWIGLU : EPI_STORE;
    if (cisr_gemv_ok(M, dual_off > 0 ? 2 * N : N, K)) return cisr_gemv_launch(a, N, norm_w != nullptr, epi, out_dtype, 0, stream);
    if (narrow_wanted(M, dual_off > 0 ? 2 * N : N, K, norm_w != nullptr)) return launch_narrow(a, (N + 3) / 4, norm_w != nullptr, epi, out_dtype, stream);
    const int blocks = (N + 15) / 16;
    return launch_rows(a, blocks, norm_w != nullptr, epi, out_dtype, stream);
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
    if (cisr_gemv_ok(M, a.N, K)) return cisr_gemv_launch(a, a.N / 2, norm_w != nullptr, EPI_ROPE, DT_BF16, 0, stream);
    if (narrow_wanted(M, a.N, K, norm_w != nullptr)) return launch_narrow(a, a.N / 4, norm_w != nullptr, EPI_ROPE, DT_BF16, stream);
    const int blocks = (heads + 2 * kv_heads) * (head_dim / 16);
    return launch_rows(a, blocks, norm_w != nullptr, EPI_ROPE, DT_BF16, stream);
}

// The output projection of a decode step fused with the merge of split attention: A is given as the split blocks'
// partial results (bf16 [M, heads, splits, head_dim] normalised outputs, float [M, heads, splits, 2] statistics with
// the maximum in log2 units), C = R + merge(A) . W^T in float.  Takes what cisr_gemm_merged_ok says it takes.
extern "C" int cisr_gemm_merged_ok(int M, int N, int heads, int head_dim, int splits) {
    const int K = heads * head_dim, rows = M <= 4 ? 4 : M <= 8 ? 8 : 16;
    const int batches = rows == 4 ? 2 : rows == 8 ? 3 : 5;
    if (M >= 1 && head_dim % 8 == 0 && (splits == 2 || splits == 4 || splits == 8) && cisr_gemv_ok(M, N, K)) return 1;
    return M >= 1 && M <= 16 && head_dim % 8 == 0 && (splits == 2 || splits == 4 || splits == 8) &&
           narrow_wanted(M, N, K, false) && (size_t)rows * (K + 8) * 2 <= 40 * 1024 && M * (K / 8) <= batches * 256;
}

extern "C" int cisr_gemm_merged_bf16(const void* part_o, const float* part_ml, int splits, int heads, int head_dim,
                                     const void* W, int ldw, float* C, int ldc, const float* R, int ldr, int M, int N,
                                     hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    const int K = heads * head_dim;
    if (!cisr_gemm_merged_ok(M, N, heads, head_dim, splits) || ldw % 8 || !aligned16(W) || !aligned16(part_o) || !aligned16(part_ml))
        return (int)hipErrorInvalidValue;
    SkinnyArgs a = {};
    a.W = (const bf16_t*)W; a.ldw = ldw; a.C = C; a.ldc = ldc; a.R = R; a.ldr = ldr; a.M = M; a.N = N; a.K = K;
    a.part_o = (const bf16_t*)part_o; a.part_ml = part_ml; a.merge_heads = heads; a.merge_dim = head_dim;
    if (cisr_gemv_ok(M, N, K)) return cisr_gemv_launch(a, N, false, EPI_STORE, DT_F32, splits, stream);
    const int units = (N + 3) / 4;
    if (M <= 4) return cisr_narrow_merge_launch_t1(a, units, splits, stream);
    if (M <= 8) return cisr_narrow_merge_launch_t2(a, units, splits, stream);
    return cisr_narrow_merge_launch_t4(a, units, splits, stream);
}
