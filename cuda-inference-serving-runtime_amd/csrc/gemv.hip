// Products of very few rows (M <= 8):  C[M,N] = A[M,K] . W[N,K]^T  as a matrix-vector kernel.
//
// With one to eight rows of A a product is a stream of W and nothing else: every byte of W is used M times and the
// matrix cores have nothing to win.  What counts is how soon the first byte of W is asked for and how many are in
// flight.  So: a wave owns whole rows of W (one or two at a time: a unit), its lanes take the 16-byte chunks of a row
// in turn (chunk c to lane c mod 64), the products are packed-bf16 dot instructions with float sums (v_dot2_f32_bf16),
// the lanes' sums meet in a butterfly of lane exchanges, and a lane finishes each activation row.  No partial tiles
// in LDS, no barrier after the prologue, no second kernel; the first loads of W are issued before the prologue's
// barrier (right behind the activations' own loads), because they do not depend on the activations.
//
// Prologue, once a block (256 threads), into LDS as packed bf16 rows [M][K]:
//   plain   A is bf16: copied;
//   NORM    A is the float residual: bf16(x[m,k] * w_norm[k]), and the row's sum of squares; rsqrt(mean + eps) is
//           applied to the finished sums (a per-row factor commutes with the product); `rows` picks input rows;
//   MSPL    A is the output of decode attention whose keys were split over MSPL blocks, merged here
//           (out = sum_s w_s o_s / sum_s w_s, w_s = 2^(m_s - max m) l_s), as in gemm_narrow.inc.
// Epilogues as in gemm_skinny.inc: store / residual; SwiGLU (a unit is the gate row and the up row of one output);
// rotary embedding and cache write of the fused q/k/v projection (a unit is the rotary pair (i, i + D/2) of a head).
//
// A row's result does not depend on the other rows of the step: a lane's chunks, the order of its sums and the
// butterfly's order are fixed by K alone.
// Requires K % 8 == 0 and 16-byte aligned rows; M * K * 2 bytes of LDS.
#include "gemm_skinny.h"

typedef __attribute__((ext_vector_type(2))) __bf16 gv_bf16x2;
typedef __attribute__((ext_vector_type(4))) float gv_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t gv_u32x4;

#define GEMV_THREADS 256
#define GEMV_WAVES 4
#define GEMV_CB 4                 // chunks of a row that a lane has in flight per batch (and as many of the batch after)
#define GEMV_MAX_LDS (144 * 1024)
// A compute unit returns loads in the order its waves asked for them, so a wave's activations (a few KB) also stand behind
// the first weights of every wave that started a moment earlier.  Every wave waits this many times 64 cycles between
// asking for its activations and for its first weights, so that the activations of all waves of the unit go first.
// Measured on an MI355X (a decode step of 8 layers, one and two requests): 1.7B sizes 0.429 and 0.495 ms without the
// pause, 0.422 and 0.478 with 2, 0.426 and 0.478 with 4, 0.431 and 0.484 with 16; 8B sizes 1.023 and 1.068, 1.018 and 1.059 with 2.
#define GEMV_HOLD 2

__device__ __forceinline__ float gv_dot2(uint32_t w, uint32_t a, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(gv_bf16x2, w), __builtin_bit_cast(gv_bf16x2, a), acc, false);
}
// (the words are taken out of the vectors first: a bit cast of a vector's component reads its first component)
__device__ __forceinline__ float gv_dot8(gv_u32x4 w, gv_u32x4 a, float acc) {
    const uint32_t w0 = w[0], w1 = w[1], w2 = w[2], w3 = w[3], a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
    return gv_dot2(w3, a3, gv_dot2(w2, a2, gv_dot2(w1, a1, gv_dot2(w0, a0, acc))));
}

// M: rows of A the kernel has room for (1, 2, 4, 8); R rows of W a unit (1: store, 2: SwiGLU and rotary pairs)
template <int M, bool NORM, int EPI, typename TC, int MSPL>
__global__ void __launch_bounds__(GEMV_THREADS)
gemv_kernel(SkinnyArgs p, int units, int per_wave) {
    static_assert(MSPL == 0 || (!NORM && EPI == EPI_STORE), "the merge prologue feeds the output projection");
    constexpr int R = EPI == EPI_STORE ? 1 : 2;
    constexpr int CB = GEMV_CB;
    extern __shared__ __attribute__((aligned(16))) uint32_t a_lds[];      // [M][K / 2]: packed bf16 pairs
    __shared__ float ssq_s[M][GEMV_WAVES];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int K = p.K, nchunks = K / 8, words = K / 2;
    const int iters = (nchunks + WAVE - 1) / WAVE;                         // chunks a lane takes of one row
    const int total_waves = gridDim.x * GEMV_WAVES, wave_global = blockIdx.x * GEMV_WAVES + wave;

    // the rows of W of unit u
    auto rows_of = [&](int u, int& r0, int& r1) {
        if (EPI == EPI_ROPE) {
            const int half = p.head_dim / 2, sh = u / half, i = u % half;
            r0 = sh * p.head_dim + i; r1 = r0 + half;
        } else {
            r0 = u; r1 = u + p.dual_off;
        }
    };
    // the wave's j-th unit (units are dealt to the waves in turn) and its batch b of chunks, all loads at once; a chunk past
    // the row reads the row's first again (no branch around a load) and counts as zero
    auto unit_of = [&](int j) { return wave_global + j * total_waves; };
    auto load_batch = [&](int u, int b, gv_u32x4 (&w)[R][CB]) {
        int r0, r1;
        rows_of(u < units ? u : 0, r0, r1);
        const bf16_t* w0 = p.W + (size_t)r0 * p.ldw;
        const bf16_t* w1 = p.W + (size_t)r1 * p.ldw;
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const int chunk = lane + WAVE * (b * CB + c), at = chunk < nchunks ? chunk * 8 : 0;
            // non-temporal: the weights are read once a step and the caches need not keep them (a decode step of
            // one row at the 8B sizes 1.008 -> 0.937 ms, at the 1.7B sizes 0.420 -> 0.413)
            w[0][c] = __builtin_nontemporal_load((const gv_u32x4*)(w0 + at));
            if (R == 2) w[1][c] = __builtin_nontemporal_load((const gv_u32x4*)(w1 + at));
        }
    };
    gv_u32x4 wcur[R][CB];

    // ---- prologue: the activation rows as packed bf16 in LDS.  Every batch of loads is issued before the first of
    // them is used, for all rows at once, with clamped addresses instead of branches (a branch around a load makes it a
    // trip to memory of its own: eight rows one after the other took 6 us).  The first batch of W is asked for right
    // behind the first batch of the activations and before these are used: loads return in the order they were asked
    // for, so the activations (a few KB out of L2) must not stand behind W's first bytes (16 MB over all waves, out of
    // memory), and W must be on its way while the activations are turned into operands.  Measured on an MI355X with time
    // marks in the kernel (norm + gate/up of the 1.7B sizes): with W asked for first the block's barrier was passed
    // 3.9 us after the kernel's start, 2.4 us of them with nothing more asked of memory.
    if constexpr (NORM) {
        const int words4 = K / 4;
        const float* xrow[M];
        {
            int src[M];
#pragma unroll
            for (int m = 0; m < M; ++m) { const int mm = m < p.M ? m : p.M - 1; src[m] = p.rows ? p.rows[mm] : mm; }
#pragma unroll
            for (int m = 0; m < M; ++m) xrow[m] = (const float*)p.A + (size_t)src[m] * p.lda;
        }
        float sq[M];
#pragma unroll
        for (int m = 0; m < M; ++m) sq[m] = 0.f;
        constexpr int G = M <= 2 ? 4 : 2;                // 16-byte words of a row a thread takes per batch
        gv_f32x4 nv[G], xv[M][G];
        auto ask = [&](int k0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int k4 = k0 + g * GEMV_THREADS + tid, kk = k4 < words4 ? k4 : 0;
                nv[g] = *(const gv_f32x4*)(p.norm_w + kk * 4);
#pragma unroll
                for (int m = 0; m < M; ++m) xv[m][g] = *(const gv_f32x4*)(xrow[m] + kk * 4);
            }
        };
        auto use = [&](int k0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int k4 = k0 + g * GEMV_THREADS + tid;
                if (k4 < words4) {
#pragma unroll
                    for (int m = 0; m < M; ++m) {
                        const gv_f32x4 x = xv[m][g];
                        const bool live = m < p.M;
                        sq[m] += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
                        a_lds[m * words + k4 * 2] = live ? pack_bf16x2(x.x * nv[g].x, x.y * nv[g].y) : 0u;
                        a_lds[m * words + k4 * 2 + 1] = live ? pack_bf16x2(x.z * nv[g].z, x.w * nv[g].w) : 0u;
                    }
                }
            }
        };
        ask(0);
        __builtin_amdgcn_s_sleep(GEMV_HOLD);
        load_batch(unit_of(0), 0, wcur);
        use(0);
        for (int k0 = GEMV_THREADS * G; k0 < words4; k0 += GEMV_THREADS * G) { ask(k0); use(k0); }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float total = wave_sum(sq[m]);
            if (lane == 0) ssq_s[m][wave] = total;
        }
    } else if constexpr (MSPL > 0) {
        const int per_row = K / 8, n_items = M * per_row;
        const int D = p.merge_dim, nh = p.merge_heads;
        constexpr int G = MSPL <= 4 ? 2 : 1;             // items a thread merges per batch
        gv_u32x4 po[G][MSPL];
        float ms[G][MSPL], ls[G][MSPL];
        auto ask = [&](int i0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int item = i0 + g * GEMV_THREADS + tid, it = item < n_items ? item : 0;
                const int row = min(it / per_row, p.M - 1), k = (it % per_row) * 8;
                const size_t base = ((size_t)row * nh + k / D) * MSPL;
#pragma unroll
                for (int sp = 0; sp < MSPL; ++sp) {
                    po[g][sp] = *(const gv_u32x4*)(p.part_o + (base + sp) * D + k % D);
                    ms[g][sp] = p.part_ml[(base + sp) * 2]; ls[g][sp] = p.part_ml[(base + sp) * 2 + 1];
                }
            }
        };
        auto use = [&](int i0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int item = i0 + g * GEMV_THREADS + tid;
                if (item >= n_items) continue;
                const int row = item / per_row, k = (item % per_row) * 8;
                float mx = -INFINITY;
#pragma unroll
                for (int sp = 0; sp < MSPL; ++sp) mx = fmaxf(mx, ms[g][sp]);
                float den = 0.f, num[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) num[j] = 0.f;
#pragma unroll
                for (int sp = 0; sp < MSPL; ++sp) {       // in the order of the splits
                    const float w = ls[g][sp] > 0.f ? __builtin_amdgcn_exp2f(ms[g][sp] - mx) * ls[g][sp] : 0.f;
                    den += w;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        num[2 * j] += w * __uint_as_float(po[g][sp][j] << 16);
                        num[2 * j + 1] += w * __uint_as_float(po[g][sp][j] & 0xffff0000u);
                    }
                }
                const float inv = (den > 0.f && row < p.M) ? 1.0f / den : 0.f;   // (a row without keys, or no row: zeros)
                *(gv_u32x4*)(a_lds + row * words + k / 2) =
                    (gv_u32x4){pack_bf16x2(num[0] * inv, num[1] * inv), pack_bf16x2(num[2] * inv, num[3] * inv),
                               pack_bf16x2(num[4] * inv, num[5] * inv), pack_bf16x2(num[6] * inv, num[7] * inv)};
            }
        };
        ask(0);
        __builtin_amdgcn_s_sleep(GEMV_HOLD);
        load_batch(unit_of(0), 0, wcur);
        use(0);
        for (int i0 = GEMV_THREADS * G; i0 < n_items; i0 += GEMV_THREADS * G) { ask(i0); use(i0); }
    } else {
        const int n_items = M * nchunks;
        constexpr int G = 4;
        gv_u32x4 v[G];
        auto ask = [&](int i0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int item = i0 + g * GEMV_THREADS + tid, it = item < n_items ? item : 0;
                v[g] = *(const gv_u32x4*)((const bf16_t*)p.A + (size_t)min(it / nchunks, p.M - 1) * p.lda + (it % nchunks) * 8);
            }
        };
        auto use = [&](int i0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int item = i0 + g * GEMV_THREADS + tid;
                if (item >= n_items) continue;
                const int row = item / nchunks;
                *(gv_u32x4*)(a_lds + row * words + (item % nchunks) * 4) = row < p.M ? v[g] : (gv_u32x4){0u, 0u, 0u, 0u};
            }
        };
        ask(0);
        __builtin_amdgcn_s_sleep(GEMV_HOLD);
        load_batch(unit_of(0), 0, wcur);
        use(0);
        for (int i0 = GEMV_THREADS * G; i0 < n_items; i0 += GEMV_THREADS * G) { ask(i0); use(i0); }
    }
    __syncthreads();

    // the lane that finishes activation row `my_m` of every unit (see the butterfly below), and what it needs from
    // memory that does not depend on the unit
    constexpr int NV = M * R;                         // sums a lane holds for one unit: [m][r]
    int my_m = 0;
    {
        int nv = NV, off = 32;
        while (nv > R) { nv /= 2; if (lane & off) my_m += nv / R; off >>= 1; }
    }
    const bool finisher = (lane & ((64 / M) - 1)) == 0 && my_m < p.M;      // one lane for every activation row
    float scale = 1.f;
    if (NORM) scale = 1.0f / sqrtf((((ssq_s[my_m][0] + ssq_s[my_m][1]) + ssq_s[my_m][2]) + ssq_s[my_m][3]) / (float)K + p.eps);
    int pos = 0, slot = -1;
    if (EPI == EPI_ROPE && finisher) {
        pos = p.positions[my_m];
        pos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
        if (p.slots) slot = p.slots[my_m];
    }

    for (int j = 0; j < per_wave; ++j) {
        const int u = unit_of(j);
        if (u >= units) break;                        // (uniform over the wave)
        int r0, r1;
        rows_of(u, r0, r1);
        // what the finishing lanes need of this unit, asked for before the products
        float resid = 0.f, rot_cos = 1.f, rot_sin = 0.f;
        if (EPI == EPI_STORE && p.R && finisher) resid = p.R[(size_t)my_m * p.ldr + u];
        if (EPI == EPI_ROPE && finisher) {
            const int half = p.head_dim / 2;
            rot_cos = p.cos_tab[(size_t)pos * half + u % half];
            rot_sin = p.sin_tab[(size_t)pos * half + u % half];
        }
        float acc[M][R];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[m][r] = 0.f;
        const int batches = (iters + CB - 1) / CB;
        for (int b = 0; b < batches; ++b) {
            // the batch after this one (or the first of the wave's next unit) is asked for before this one is used
            gv_u32x4 wnext[R][CB];
            const bool more = b + 1 < batches;
            load_batch(more ? u : unit_of(j + 1), more ? b + 1 : 0, wnext);
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                if (b * CB + c >= iters) break;        // (uniform: a slot that no lane has a chunk for)
                const int chunk = lane + WAVE * (b * CB + c);
                const bool ok = chunk < nchunks;
                const int at = ok ? chunk * 4 : 0;
                const uint32_t keep = ok ? 0xffffffffu : 0u;
                gv_u32x4 w0 = wcur[0][c], w1 = wcur[R - 1][c];
                w0.x &= keep; w0.y &= keep; w0.z &= keep; w0.w &= keep;
                if (R == 2) { w1.x &= keep; w1.y &= keep; w1.z &= keep; w1.w &= keep; }
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const gv_u32x4 a = *(const gv_u32x4*)(a_lds + m * words + at);
                    acc[m][0] = gv_dot8(w0, a, acc[m][0]);
                    if (R == 2) acc[m][R - 1] = gv_dot8(w1, a, acc[m][R - 1]);
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int c = 0; c < CB; ++c) wcur[r][c] = wnext[r][c];
        }
        // The lanes' sums meet: offsets 32, 16, 8, ... in this order whatever M is.  While a lane holds the sums of more
        // than one activation row, the two lanes of a pair share them out (the upper lane keeps the upper half and
        // sends the lower), so that a row's sums end in the lanes that finish it; then plain exchanges.
        float v[NV];
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) v[m * R + r] = acc[m][r];
        {
            int off = 32;
#pragma unroll
            for (int nv = NV; nv > R; nv /= 2) {
                const bool upper = (lane & off) != 0;
#pragma unroll
                for (int i = 0; i < nv / 2; ++i) {
                    const float send = upper ? v[i] : v[i + nv / 2], keepv = upper ? v[i + nv / 2] : v[i];
                    v[i] = keepv + __shfl_xor(send, off, WAVE);
                }
                off >>= 1;
            }
#pragma unroll
            for (; off > 0; off >>= 1)
#pragma unroll
                for (int r = 0; r < R; ++r) v[r] += __shfl_xor(v[r], off, WAVE);
        }
        if (!finisher) continue;
        const int m = my_m;
        float v0 = v[0] * scale;
        if (EPI == EPI_STORE) {
            if (p.R) v0 += resid;
            store_f32((TC*)p.C + (size_t)m * p.ldc + u, v0);
        } else if (EPI == EPI_SWIGLU) {
            const float v1 = v[R - 1] * scale;
            // the two-kernel path rounds gate and up to bf16 before the activation; do the same
            const float gq = bf16_to_f32(f32_to_bf16(v0)), uq = bf16_to_f32(f32_to_bf16(v1));
            ((bf16_t*)p.C)[(size_t)m * p.ldc + u] = f32_to_bf16(gq / (1.0f + expf(-gq)) * uq);
        } else {
            float v1 = v[R - 1] * scale;
            const int D = p.head_dim, half = D / 2, sh = u / half, i = u % half;
            if (sh < p.heads + p.kv_heads) {          // q or k head: turn the pair
                const float a = v0, b = v1;
                v0 = a * rot_cos - b * rot_sin; v1 = b * rot_cos + a * rot_sin;
            }
            if (sh < p.heads) {
                bf16_t* q = (bf16_t*)p.C + (size_t)m * p.ldc + sh * D;
                q[i] = f32_to_bf16(v0); q[half + i] = f32_to_bf16(v1);
            } else if (slot >= 0) {
                const int page = slot / p.page_size, off = slot % p.page_size;
                if (sh < p.heads + p.kv_heads) {
                    bf16_t* k = p.kcache + (((size_t)page * p.kv_heads + (sh - p.heads)) * p.page_size + off) * D;
                    k[i] = f32_to_bf16(v0); k[half + i] = f32_to_bf16(v1);
                } else {
                    bf16_t* vv = p.vcache + ((size_t)page * p.kv_heads + (sh - p.heads - p.kv_heads)) * D * p.page_size + off;
                    vv[(size_t)i * p.page_size] = f32_to_bf16(v0); vv[(size_t)(half + i) * p.page_size] = f32_to_bf16(v1);
                }
            }
        }
    }
}

static int gemv_compute_units() {
    static int units = 0;
    if (units == 0) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
            units = 256;
    }
    return units;
}

template <int M, bool NORM, int EPI, typename TC, int MSPL>
static int gemv_launch_one(const SkinnyArgs& a, int units, hipStream_t stream) {
    const size_t lds = (size_t)M * a.K * 2;
    if (lds > GEMV_MAX_LDS) return (int)hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)gemv_kernel<M, NORM, EPI, TC, MSPL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    // Blocks: with units enough, two, three or four a compute unit (8, 12 or 16 waves), whichever leaves the waves the
    // most equal numbers of units (the kernel is as long as its busiest wave: 3,072 rotary pairs are two units for half
    // of 2,048 waves and one for the others, a third of the time idle, but one unit for each of 3,072; 384 blocks on
    // 256 compute units leave half of them with twice the work of the others), the fewest of equals; with fewer units
    // than eight waves a compute unit, one unit a wave.  Measured on an MI355X (a decode step of one request, 8 layers):
    // always 8 waves 0.443 ms at the 1.7B sizes, always 12 0.427, always 16 0.432; 1.037, 1.041 and 1.020 at the 8B sizes.
    const int cus = gemv_compute_units();
    int waves = cus * 8;
    if (units >= waves) {
        long long best = -1;
        for (int w = 8; w <= 16; w += 4) {
            if (w > 8 && (size_t)(w / GEMV_WAVES) * lds > 160 * 1024) break;                     // (that many blocks' rows do not fit a unit's LDS)
            const long long all = (long long)cus * w, busiest = (units + all - 1) / all * all;   // unit-times the launch lasts
            if (best < 0 || busiest < best) { best = busiest; waves = (int)all; }
        }
    }
    const int per_wave = (units + waves - 1) / waves;
    const int blocks = units >= waves ? waves / GEMV_WAVES : (units + GEMV_WAVES - 1) / GEMV_WAVES;
    gemv_kernel<M, NORM, EPI, TC, MSPL><<<blocks, GEMV_THREADS, lds, stream>>>(a, units, per_wave);
    return CISR_LAUNCH_CHECK();
}

template <int M>
static int gemv_launch_rows(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, int splits, hipStream_t stream) {
    if (splits == 2) return gemv_launch_one<M, false, EPI_STORE, float, 2>(a, units, stream);
    if (splits == 4) return gemv_launch_one<M, false, EPI_STORE, float, 4>(a, units, stream);
    if (splits == 8) return gemv_launch_one<M, false, EPI_STORE, float, 8>(a, units, stream);
    if (splits != 0) return (int)hipErrorInvalidValue;
    if (epi == EPI_SWIGLU) return norm ? gemv_launch_one<M, true, EPI_SWIGLU, bf16_t, 0>(a, units, stream) : gemv_launch_one<M, false, EPI_SWIGLU, bf16_t, 0>(a, units, stream);
    if (epi == EPI_ROPE) return norm ? gemv_launch_one<M, true, EPI_ROPE, bf16_t, 0>(a, units, stream) : gemv_launch_one<M, false, EPI_ROPE, bf16_t, 0>(a, units, stream);
    if (out_dtype == DT_F32) return norm ? gemv_launch_one<M, true, EPI_STORE, float, 0>(a, units, stream) : gemv_launch_one<M, false, EPI_STORE, float, 0>(a, units, stream);
    return norm ? gemv_launch_one<M, true, EPI_STORE, bf16_t, 0>(a, units, stream) : gemv_launch_one<M, false, EPI_STORE, bf16_t, 0>(a, units, stream);
}

// Whether the matrix-vector kernel takes M rows against an inner size of K: the rows must fit LDS.
bool cisr_gemv_takes(int M, int K) {
    if (M < 1 || M > GEMV_MAX_ROWS || K <= 0 || K % 8) return false;
    const int room = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 8;
    return (size_t)room * K * 2 <= GEMV_MAX_LDS;
}

// `units`: N for the plain and SwiGLU forms (N outputs), (heads + 2 kv_heads) head_dim / 2 rotary pairs for EPI_ROPE.
// `splits` > 0: the merge prologue.
int cisr_gemv_launch(const SkinnyArgs& a, int units, bool norm, int epi, int out_dtype, int splits, hipStream_t stream) {
    if (!cisr_gemv_takes(a.M, a.K)) return (int)hipErrorInvalidValue;
    if (a.M <= 1) return gemv_launch_rows<1>(a, units, norm, epi, out_dtype, splits, stream);
    if (a.M <= 2) return gemv_launch_rows<2>(a, units, norm, epi, out_dtype, splits, stream);
    if (a.M <= 4) return gemv_launch_rows<4>(a, units, norm, epi, out_dtype, splits, stream);
    return gemv_launch_rows<8>(a, units, norm, epi, out_dtype, splits, stream);
}
