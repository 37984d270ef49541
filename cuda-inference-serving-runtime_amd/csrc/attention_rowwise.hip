// Row-wise attention over the paged cache: one wavefront per (token row, query
// head, split).  A row at position p of its request attends to the cached keys
// lo..p of that request (lo = 0, or p-window+1 with a window); its own key was
// written to the cache before this kernel runs, so causality needs no mask
// tensor (reference: docs/ARCHITECTURE.md:20-21, kernels/execution.cu:48-79).
// This kernel is exact float arithmetic on float or bf16 storage and serves as
// the 32-bit path and as the general fallback; it takes any even head size up
// to 256, any page size, any head grouping.
//
// Within a block of 64 keys each lane scores one key (q is broadcast from LDS),
// the wave reduces the running maximum and denominator once per 64 keys, then
// each lane accumulates its own output coordinates over the 64 keys.
#include "common.h"

#define MAX_HEAD_DIM 256

template <typename T>
__global__ void __launch_bounds__(64)
attn_rowwise_kernel(const T* __restrict__ q, int q_row_stride, const T* __restrict__ kcache,
                    const T* __restrict__ vcache, const int* __restrict__ tables,
                    const int* __restrict__ seg_of_row, const int* __restrict__ positions,
                    T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                    int heads, int kv_heads, int dim, int page_size, int width, int window,
                    float scale, int splits) {
    __shared__ float qs[MAX_HEAD_DIM];
    __shared__ float ps[WAVE];
    __shared__ long long rowoff[WAVE];   // offset of a key's first value element (values are [D, page_size] in a page)

    const int row = blockIdx.x, head = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
    const int kvh = head / (heads / kv_heads);
    const int seg = seg_of_row[row];
    const int ncoord = (dim + WAVE - 1) / WAVE;  // at most 4

    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    int begin = 0, end = 0;
    if (seg >= 0) {
        const int p = positions[row];
        const int lo = (window > 0 && p + 1 > window) ? p + 1 - window : 0;
        const int hi = p + 1;
        const int chunk = (hi - lo + splits - 1) / splits;
        begin = lo + split * chunk;
        end = min(hi, begin + chunk);
    }
    if (begin < end) {
        const T* qr = q + (size_t)row * q_row_stride + (size_t)head * dim;
        for (int d = lane; d < dim; d += WAVE) qs[d] = load_f32(qr + d);
        __syncthreads();
        const int* table = tables + (size_t)seg * width;
        for (int base = begin; base < end; base += WAVE) {
            const int t = base + lane;
            const bool valid = t < end;
            float s = -INFINITY;
            long long off = 0;
            if (valid) {
                const int page = table[t / page_size];
                const long long head_base = ((long long)page * kv_heads + kvh) * page_size * dim;
                off = head_base + (t % page_size);
                const T* kr = kcache + head_base + (long long)(t % page_size) * dim;
                float dot = 0.f;
                for (int d = 0; d < dim; ++d) dot += qs[d] * load_f32(kr + d);
                s = dot * scale;
            }
            const float m_new = fmaxf(m, wave_max(s));   // finite: lane 0 of a block is always valid
            const float pj = valid ? expf(s - m_new) : 0.f;
            const float alpha = expf(m - m_new);           // exp(-inf) = 0 on the first block
            l = l * alpha + wave_sum(pj);
            m = m_new;
            __syncthreads();
            ps[lane] = pj;
            rowoff[lane] = off;
            __syncthreads();
            const int nvalid = min(WAVE, end - base);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (c < ncoord) {
                    const int d = lane + c * WAVE;
                    float a = acc[c] * alpha;
                    if (d < dim)
                        for (int j = 0; j < nvalid; ++j) a += ps[j] * load_f32(vcache + rowoff[j] + (long long)d * page_size);
                    acc[c] = a;
                }
            }
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (splits == 1) {
        T* o = out + ((size_t)row * heads + head) * dim;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int d = lane + c * WAVE;
            if (c < ncoord && d < dim) store_f32(o + d, acc[c] * inv);
        }
    } else {
        const size_t part = ((size_t)row * heads + head) * splits + split;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int d = lane + c * WAVE;
            if (c < ncoord && d < dim) part_o[part * dim + d] = acc[c] * inv;
        }
        if (lane == 0) { part_ml[part * 2] = m; part_ml[part * 2 + 1] = l; }
    }
}

// Merge split partials: m = max m_i; w_i = l_i > 0 ? exp(m_i - m) * l_i : 0;
// out = sum w_i o_i / sum w_i (reference: kernels/ops.cu:72-86).  A row with no
// keys at all (padding) gives zeros.  LOG2: the maxima are in units of log2.  MANY: more than sixteen splits
// (a kernel of its own, so that the common few-split form keeps its registers and code to itself).
// `row_ids`: the partials of block row i belong to output row row_ids[i] (negative: to none).
template <typename T, bool LOG2, bool MANY>
__global__ void attn_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                  T* __restrict__ out, int heads, int dim, int splits, const int* __restrict__ row_ids = nullptr) {
    const int head = blockIdx.y;
    const size_t base = ((size_t)blockIdx.x * heads + head) * splits;
    const int row = row_ids ? row_ids[blockIdx.x] : (int)blockIdx.x;
    if (row < 0) return;
    if (!MANY) {
        // every load is issued before the first is used (one trip to memory instead of two); splits
        // past the count read the last one again and are left out of the sums
        for (int d = threadIdx.x; d < dim; d += blockDim.x) {
            float ms[16], ls[16], os[16];
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                const size_t at = base + min(s, splits - 1);
                ms[s] = part_ml[at * 2]; ls[s] = part_ml[at * 2 + 1]; os[s] = part_o[at * dim + d];
            }
            float m = -INFINITY;
#pragma unroll
            for (int s = 0; s < 16; ++s) if (s < splits) m = fmaxf(m, ms[s]);
            float den = 0.f, num = 0.f;
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                if (s >= splits) continue;
                const float dm = ms[s] - m;
                const float w = ls[s] > 0.f ? (LOG2 ? exp2f(dm) : expf(dm)) * ls[s] : 0.f;
                den += w;
                num += w * os[s];
            }
            store_f32(out + ((size_t)row * heads + head) * dim + d, den > 0.f ? num / den : 0.f);
        }
        return;
    }
    // more splits: thirty-two at a time, all their loads issued before the first is used (one trip to memory for up
    // to 32 splits: a second batch would wait for the first), merged into running sums (maximum, denominator,
    // numerator) in the order of the splits
    constexpr int SB = 32;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) {
        float m = -INFINITY, den = 0.f, num = 0.f;
        for (int s0 = 0; s0 < splits; s0 += SB) {
            float ms[SB], ls[SB], os[SB];
#pragma unroll
            for (int s = 0; s < SB; ++s) {
                const size_t at = base + min(s0 + s, splits - 1);
                ms[s] = part_ml[at * 2]; ls[s] = part_ml[at * 2 + 1]; os[s] = part_o[at * dim + d];
            }
            float m_new = m;
#pragma unroll
            for (int s = 0; s < SB; ++s) if (s0 + s < splits) m_new = fmaxf(m_new, ms[s]);
            if (m_new == -INFINITY) continue;             // nothing visible so far
            const float keep = LOG2 ? exp2f(m - m_new) : expf(m - m_new);   // m = -inf gives 0
            den *= keep; num *= keep; m = m_new;
#pragma unroll
            for (int s = 0; s < SB; ++s) {
                if (s0 + s >= splits) continue;
                const float dm = ms[s] - m;
                const float w = ls[s] > 0.f ? (LOG2 ? exp2f(dm) : expf(dm)) * ls[s] : 0.f;
                den += w;
                num += w * os[s];
            }
        }
        store_f32(out + ((size_t)row * heads + head) * dim + d, den > 0.f ? num / den : 0.f);
    }
}

// A thread a coordinate of the head (a second coordinate a thread is a second trip to memory): 64 to 256 threads.
static int merge_threads(int dim) { return dim <= 64 ? 64 : dim <= 128 ? 128 : 256; }

// merge of the matrix-core kernel's partials (bf16 output, maxima in log2 units)
extern "C" int cisr_attn_merge(const float* part_o, const float* part_ml, void* out, int rows, int heads, int dim,
                               int splits, const int* row_ids, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads > 65535 || splits < 1) return (int)hipErrorInvalidValue;
    const int threads = merge_threads(dim);
    if (splits <= 16) attn_merge_kernel<bf16_t, true, false><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (bf16_t*)out, heads, dim, splits, row_ids);
    else attn_merge_kernel<bf16_t, true, true><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (bf16_t*)out, heads, dim, splits, row_ids);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_attn_rowwise(const void* q, int q_row_stride, const void* kcache, const void* vcache,
                                 const int* tables, const int* seg_of_row, const int* positions, void* out,
                                 float* part_o, float* part_ml, int rows, int heads, int kv_heads, int dim,
                                 int page_size, int width, int window, float scale, int splits, int dtype,
                                 hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim > MAX_HEAD_DIM || dim <= 0 || heads % kv_heads || splits < 1 || splits > 65535 || heads > 65535)
        return (int)hipErrorInvalidValue;
    dim3 grid(rows, heads, splits);
    if (dtype == DT_F32)
        attn_rowwise_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_row_stride, (const float*)kcache,
            (const float*)vcache, tables, seg_of_row, positions, (float*)out, part_o, part_ml, heads, kv_heads,
            dim, page_size, width, window, scale, splits);
    else
        attn_rowwise_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_row_stride, (const bf16_t*)kcache,
            (const bf16_t*)vcache, tables, seg_of_row, positions, (bf16_t*)out, part_o, part_ml, heads, kv_heads,
            dim, page_size, width, window, scale, splits);
    int err = CISR_LAUNCH_CHECK();
    if (err || splits == 1) return err;
    const int threads = merge_threads(dim);
    if (dtype == DT_F32) {
        if (splits <= 16) attn_merge_kernel<float, false, false><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (float*)out, heads, dim, splits);
        else attn_merge_kernel<float, false, true><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (float*)out, heads, dim, splits);
    } else {
        if (splits <= 16) attn_merge_kernel<bf16_t, false, false><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (bf16_t*)out, heads, dim, splits);
        else attn_merge_kernel<bf16_t, false, true><<<dim3(rows, heads), threads, 0, stream>>>(part_o, part_ml, (bf16_t*)out, heads, dim, splits);
    }
    return CISR_LAUNCH_CHECK();
}
