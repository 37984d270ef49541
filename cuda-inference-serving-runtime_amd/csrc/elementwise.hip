// Row-wise and element-wise kernels of the forward pass: embedding gather,
// RMSNorm (optionally on gathered rows), residual add, SwiGLU, rotary embedding
// fused with the key/value scatter into the paged cache, and the page copy used
// for copy-on-write.  The residual stream is float in every mode; `T` below is
// the storage type of activations and weights (float or bf16).
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[r, :] = table[ids[r], :]  (reference: kernels/execution.cu:2-5)
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int dim, int vocab) {
    const int row = blockIdx.x;
    int id = ids[row];
    if (id < 0 || id >= vocab) id = 0;  // padding rows; real ids are checked on the host
    const T* src = table + (size_t)id * dim;
    float* dst = out + (size_t)row * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) dst[d] = load_f32(src + d);
}

extern "C" int cisr_embedding(const int* ids, const void* table, float* out, int rows, int dim,
                              int vocab, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dtype == DT_F32)
        embedding_kernel<float><<<rows, 256, 0, stream>>>(ids, (const float*)table, out, dim, vocab);
    else
        embedding_kernel<bf16_t><<<rows, 256, 0, stream>>>(ids, (const bf16_t*)table, out, dim, vocab);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ RMSNorm
// y = x * rsqrt(mean(x^2) + eps) * w  (reference: kernels/ops.cu:3-19).
// Input is the float residual stream; `rows` (may be null) picks input rows.
template <typename T>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                               T* __restrict__ y, const int* __restrict__ rows, int dim, float eps) {
    __shared__ float red[4];
    const int orow = blockIdx.x;
    const int irow = rows ? rows[orow] : orow;
    const float* src = x + (size_t)irow * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) { float a = src[d]; ss += a * a; }
    const float total = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(total / (float)dim + eps);
    T* dst = y + (size_t)orow * dim;
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(dst + d, src[d] * scale * w[d]);
}

// The same for rows of a multiple of four floats, 16-byte aligned: one wavefront a row, the row stays
// in registers (R float4 a lane: dim <= 256 R), loads and stores of 16 bytes.  The sum of squares of a
// row is made by its own wave in a fixed order, whatever else is in the batch.
template <typename T, int R>
__global__ void __launch_bounds__(256)
rmsnorm_wave_kernel(const float* __restrict__ x, const float* __restrict__ w, T* __restrict__ y,
                    const int* __restrict__ rows, int n_out, int dim, float eps) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;   // (uniform: the row's loads of indices are scalar)
    const int orow = blockIdx.x * 4 + wave;
    if (orow >= n_out) return;
    const int irow = rows ? rows[orow] : orow;
    const int n4 = dim / 4;
    const float4* src = (const float4*)(x + (size_t)irow * dim);
    const float4* w4 = (const float4*)w;
    float4 v[R], g[R];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = min(lane + WAVE * i, n4 - 1);   // past the row: a copy of its last chunk, not counted
        v[i] = src[c];
        g[i] = w4[c];
    }
#pragma unroll
    for (int i = 0; i < R; ++i)
        if (lane + WAVE * i < n4) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    const float scale = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = lane + WAVE * i;
        if (c >= n4) continue;
        const float a = v[i].x * scale * g[i].x, b = v[i].y * scale * g[i].y;
        const float cc = v[i].z * scale * g[i].z, d = v[i].w * scale * g[i].w;
        if (sizeof(T) == 4) {
            ((float4*)((float*)y + (size_t)orow * dim))[c] = make_float4(a, b, cc, d);
        } else {
            ((uint2*)((bf16_t*)y + (size_t)orow * dim))[c] = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, d));
        }
    }
}

template <typename T>
static int launch_rmsnorm(const float* x, const float* w, T* y, const int* rows, int n_out, int dim, float eps,
                          hipStream_t stream) {
    const bool vec = dim % 4 == 0 && dim <= 8192 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                     ((uintptr_t)y % 16 == 0);
    const int blocks = (n_out + 3) / 4, chunks = (dim / 4 + WAVE - 1) / WAVE;
    if (!vec) rmsnorm_kernel<T><<<n_out, 256, 0, stream>>>(x, w, y, rows, dim, eps);
    else if (chunks <= 1) rmsnorm_wave_kernel<T, 1><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else if (chunks <= 2) rmsnorm_wave_kernel<T, 2><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else if (chunks <= 3) rmsnorm_wave_kernel<T, 3><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else if (chunks <= 4) rmsnorm_wave_kernel<T, 4><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else if (chunks <= 8) rmsnorm_wave_kernel<T, 8><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else if (chunks <= 16) rmsnorm_wave_kernel<T, 16><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    else rmsnorm_wave_kernel<T, 32><<<blocks, 256, 0, stream>>>(x, w, y, rows, n_out, dim, eps);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_rmsnorm(const float* x, const float* w, void* y, const int* rows, int n_out,
                            int dim, float eps, int out_dtype, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (out_dtype == DT_F32) return launch_rmsnorm<float>(x, w, (float*)y, rows, n_out, dim, eps, stream);
    return launch_rmsnorm<bf16_t>(x, w, (bf16_t*)y, rows, n_out, dim, eps, stream);
}

// x += sum of `slices` partial sums (parts[s][row][dim], added in slice order, then to x), and with w also
// y = rmsnorm(x): what follows a product that was cut along its inner size and left unfinished, so that the sum,
// the residual and the norm are one kernel.  One block a row (these are steps of few rows: a row's loads have to
// be spread over many lanes and in flight together), R chunks of four floats a thread, four slices at a time.
template <typename T, int R>
__global__ void __launch_bounds__(256)
rmsnorm_partials_kernel(float* x, const float* __restrict__ parts, int slices, const float* __restrict__ w,
                        T* __restrict__ y, int n_rows, int dim, float eps) {
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int n4 = dim / 4;
    float4* xr = (float4*)(x + (size_t)row * dim);
    const size_t slice4 = (size_t)n_rows * n4;
    const float4* pr = (const float4*)parts + (size_t)row * n4;
    const float4* w4 = (const float4*)w;
    float4 v[R], r[R], g[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = min(tid + 256 * i, n4 - 1);     // past the row: a copy of its last chunk, not counted or stored
        r[i] = xr[c];
        if (w) g[i] = w4[c];
        v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int s0 = 0; s0 < slices; s0 += 4) {
        float4 p[R][4];
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                p[i][j] = pr[(size_t)min(s0 + j, slices - 1) * slice4 + min(tid + 256 * i, n4 - 1)];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s0 + j >= slices) break;
#pragma unroll
            for (int i = 0; i < R; ++i) { v[i].x += p[i][j].x; v[i].y += p[i][j].y; v[i].z += p[i][j].z; v[i].w += p[i][j].w; }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        v[i] = make_float4(v[i].x + r[i].x, v[i].y + r[i].y, v[i].z + r[i].z, v[i].w + r[i].w);
        if (tid + 256 * i >= n4) continue;
        xr[tid + 256 * i] = v[i];
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    if (!w) return;
    const float scale = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = tid + 256 * i;
        if (c >= n4) continue;
        const float a = v[i].x * scale * g[i].x, b = v[i].y * scale * g[i].y;
        const float cc = v[i].z * scale * g[i].z, d = v[i].w * scale * g[i].w;
        if (sizeof(T) == 4) {
            ((float4*)((float*)y + (size_t)row * dim))[c] = make_float4(a, b, cc, d);
        } else {
            ((uint2*)((bf16_t*)y + (size_t)row * dim))[c] = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, d));
        }
    }
}

template <typename T>
static int launch_rmsnorm_partials(float* x, const float* parts, int slices, const float* w, T* y, int n_rows, int dim,
                                   float eps, hipStream_t stream) {
    const int chunks = (dim / 4 + 255) / 256;
    if (chunks <= 1) rmsnorm_partials_kernel<T, 1><<<n_rows, 256, 0, stream>>>(x, parts, slices, w, y, n_rows, dim, eps);
    else if (chunks <= 2) rmsnorm_partials_kernel<T, 2><<<n_rows, 256, 0, stream>>>(x, parts, slices, w, y, n_rows, dim, eps);
    else if (chunks <= 4) rmsnorm_partials_kernel<T, 4><<<n_rows, 256, 0, stream>>>(x, parts, slices, w, y, n_rows, dim, eps);
    else rmsnorm_partials_kernel<T, 8><<<n_rows, 256, 0, stream>>>(x, parts, slices, w, y, n_rows, dim, eps);
    return CISR_LAUNCH_CHECK();
}

// x[n_rows, dim] += the partial sums parts[slices][n_rows][dim]; y = rmsnorm(x) with weights w (w null: the sum only,
// y unused).  dim % 4 == 0, dim <= 8192, 16-byte aligned operands.
extern "C" int cisr_rmsnorm_partials(float* x, const float* parts, int slices, const float* w, void* y, int n_rows, int dim,
                                     float eps, int out_dtype, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (slices < 1 || dim <= 0 || dim % 4 || dim > 8192 || (uintptr_t)x % 16 || (uintptr_t)parts % 16 || (uintptr_t)w % 16 ||
        (w && (!y || (uintptr_t)y % 16)))
        return (int)hipErrorInvalidValue;
    if (out_dtype == DT_F32) return launch_rmsnorm_partials<float>(x, parts, slices, w, (float*)y, n_rows, dim, eps, stream);
    return launch_rmsnorm_partials<bf16_t>(x, parts, slices, w, (bf16_t*)y, n_rows, dim, eps, stream);
}

// x += delta, then y = rmsnorm(x) (reference: kernels/execution.cu:12-24; here
// the sum stays float so nothing is rounded before the norm reads it).
template <typename TD, typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                   const float* __restrict__ w, T* __restrict__ y, int dim, float eps) {
    __shared__ float red[4];
    const int row = blockIdx.x;
    float* xr = x + (size_t)row * dim;
    const TD* dr = delta + (size_t)row * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
        float a = xr[d] + load_f32(dr + d);
        xr[d] = a;
        ss += a * a;
    }
    const float total = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(total / (float)dim + eps);
    T* dst = y + (size_t)row * dim;
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(dst + d, xr[d] * scale * w[d]);
}

// The same for a bf16 delta and rows of a multiple of four, 16-byte aligned (8 for the delta): one wavefront a
// row, as rmsnorm_wave_kernel, which it equals bit for bit on the summed rows.
template <typename T, int R>
__global__ void __launch_bounds__(256)
add_rmsnorm_wave_kernel(float* x, const bf16_t* __restrict__ delta, const float* __restrict__ w, T* __restrict__ y,
                        int n_rows, int dim, float eps) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;   // (uniform: the row's loads of indices are scalar)
    const int row = blockIdx.x * 4 + wave;
    if (row >= n_rows) return;
    const int n4 = dim / 4;
    float4* xr = (float4*)(x + (size_t)row * dim);
    const uint2* dr = (const uint2*)(delta + (size_t)row * dim);
    const float4* w4 = (const float4*)w;
    float4 v[R], g[R];
    uint2 d[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = min(lane + WAVE * i, n4 - 1);   // past the row: a copy of its last chunk, not counted or stored
        v[i] = xr[c];
        d[i] = dr[c];
        g[i] = w4[c];
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        v[i].x += __uint_as_float(d[i].x << 16); v[i].y += __uint_as_float(d[i].x & 0xffff0000u);
        v[i].z += __uint_as_float(d[i].y << 16); v[i].w += __uint_as_float(d[i].y & 0xffff0000u);
        if (lane + WAVE * i >= n4) continue;
        xr[lane + WAVE * i] = v[i];
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    const float scale = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int c = lane + WAVE * i;
        if (c >= n4) continue;
        const float a = v[i].x * scale * g[i].x, b = v[i].y * scale * g[i].y;
        const float cc = v[i].z * scale * g[i].z, e = v[i].w * scale * g[i].w;
        if (sizeof(T) == 4) {
            ((float4*)((float*)y + (size_t)row * dim))[c] = make_float4(a, b, cc, e);
        } else {
            ((uint2*)((bf16_t*)y + (size_t)row * dim))[c] = make_uint2(pack_bf16x2(a, b), pack_bf16x2(cc, e));
        }
    }
}

template <typename T>
static int launch_add_rmsnorm_wave(float* x, const bf16_t* delta, const float* w, T* y, int rows, int dim, float eps,
                                   hipStream_t stream) {
    const int blocks = (rows + 3) / 4, chunks = (dim / 4 + WAVE - 1) / WAVE;
    if (chunks <= 1) add_rmsnorm_wave_kernel<T, 1><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    else if (chunks <= 2) add_rmsnorm_wave_kernel<T, 2><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    else if (chunks <= 4) add_rmsnorm_wave_kernel<T, 4><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    else if (chunks <= 8) add_rmsnorm_wave_kernel<T, 8><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    else if (chunks <= 16) add_rmsnorm_wave_kernel<T, 16><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    else add_rmsnorm_wave_kernel<T, 32><<<blocks, 256, 0, stream>>>(x, delta, w, y, rows, dim, eps);
    return CISR_LAUNCH_CHECK();
}

// x[rows, dim] (float) += delta (bf16); y = rmsnorm(x) with weights w, float or bf16 (out_dtype): dim % 4 == 0,
// dim <= 8192, 16-byte aligned x, w, y, 8-byte aligned delta.
extern "C" int cisr_add_rmsnorm_bf16(float* x, const void* delta, const float* w, void* y, int rows, int dim, float eps,
                                     int out_dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || dim % 4 || dim > 8192 || (uintptr_t)x % 16 || (uintptr_t)delta % 8 || (uintptr_t)w % 16 || (uintptr_t)y % 16)
        return (int)hipErrorInvalidValue;
    if (out_dtype == DT_F32) return launch_add_rmsnorm_wave<float>(x, (const bf16_t*)delta, w, (float*)y, rows, dim, eps, stream);
    return launch_add_rmsnorm_wave<bf16_t>(x, (const bf16_t*)delta, w, (bf16_t*)y, rows, dim, eps, stream);
}

extern "C" int cisr_add_rmsnorm(float* x, const void* delta, const float* w, void* y, int rows, int dim,
                                float eps, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dtype == DT_F32)
        add_rmsnorm_kernel<float, float><<<rows, 256, 0, stream>>>(x, (const float*)delta, w, (float*)y, dim, eps);
    else
        add_rmsnorm_kernel<bf16_t, bf16_t><<<rows, 256, 0, stream>>>(x, (const bf16_t*)delta, w, (bf16_t*)y, dim, eps);
    return CISR_LAUNCH_CHECK();
}

// x += delta (reference: kernels/execution.cu:42-44), float residual
template <typename TD>
__global__ void add_kernel(float* __restrict__ x, const TD* __restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] += load_f32(delta + i);
}

// the same for a bf16 delta, eight elements a thread with 16-byte accesses (n % 8 == 0, aligned pointers)
__global__ void __launch_bounds__(256) add_bf16x8_kernel(float* __restrict__ x, const bf16_t* __restrict__ delta, size_t n8) {
    typedef __attribute__((ext_vector_type(4))) float f32x4_t;
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const u32x4_t d = *(const u32x4_t*)(delta + i * 8);
    f32x4_t a = *(const f32x4_t*)(x + i * 8), b = *(const f32x4_t*)(x + i * 8 + 4);
    a.x += __uint_as_float(d.x << 16); a.y += __uint_as_float(d.x & 0xffff0000u);
    a.z += __uint_as_float(d.y << 16); a.w += __uint_as_float(d.y & 0xffff0000u);
    b.x += __uint_as_float(d.z << 16); b.y += __uint_as_float(d.z & 0xffff0000u);
    b.z += __uint_as_float(d.w << 16); b.w += __uint_as_float(d.w & 0xffff0000u);
    *(f32x4_t*)(x + i * 8) = a; *(f32x4_t*)(x + i * 8 + 4) = b;
}

extern "C" int cisr_residual_add(float* x, const void* delta, long long n, int dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    if (dtype == DT_BF16 && n % 8 == 0 && ((uintptr_t)x) % 16 == 0 && ((uintptr_t)delta) % 16 == 0) {
        const size_t n8 = (size_t)n / 8;
        add_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, stream>>>(x, (const bf16_t*)delta, n8);
        return CISR_LAUNCH_CHECK();
    }
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)delta, (size_t)n);
    else add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (const bf16_t*)delta, (size_t)n);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------- SwiGLU
// act[r, i] = g * sigmoid(g) * u with g = gu[r, i], u = gu[r, inter + i]
// (reference: kernels/execution.cu:7-10), arithmetic in float.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ act, int inter, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    size_t row = i / inter; int col = (int)(i % inter);
    const T* base = gu + row * (size_t)(2 * inter);
    float g = load_f32(base + col), u = load_f32(base + inter + col);
    store_f32(act + i, g / (1.0f + expf(-g)) * u);
}

// the same for bf16, eight elements a thread with 16-byte accesses (inter % 8 == 0, aligned pointers)
__global__ void __launch_bounds__(256) swiglu_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ act, int inter8, size_t n8) {
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const size_t row = i / inter8; const int col = (int)(i % inter8) * 8;
    const bf16_t* base = gu + row * (size_t)(16 * inter8);
    const u32x4_t g = *(const u32x4_t*)(base + col), u = *(const u32x4_t*)(base + 8 * inter8 + col);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t out[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
        out[k] = pack_bf16x2(g0 / (1.0f + expf(-g0)) * u0, g1 / (1.0f + expf(-g1)) * u1);
    }
    *(u32x4_t*)(act + i * 8) = (u32x4_t){out[0], out[1], out[2], out[3]};
}

extern "C" int cisr_swiglu(const void* gu, void* act, int rows, int inter, int dtype, hipStream_t stream) {
    size_t n = (size_t)rows * inter;
    if (n == 0) return 0;
    if (dtype == DT_BF16 && inter % 8 == 0 && ((uintptr_t)gu) % 16 == 0 && ((uintptr_t)act) % 16 == 0) {
        const size_t n8 = n / 8;
        swiglu_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)act, inter / 8, n8);
        return CISR_LAUNCH_CHECK();
    }
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)act, inter, n);
    else swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)act, inter, n);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------- rotary embedding + scatter
// One block per token row of the fused projection buffer
//   qkv[r] = [ q: heads*D | k: kv_heads*D | v: kv_heads*D ].
// q is rotated in place; k is rotated and written to the cache; v is copied to
// the cache.  Pair i of the first `rot` coordinates of a head turns by the angle
// whose cosine and sine sit in cos_tab/sin_tab[pos, i] (tables are float,
// [max_pos, rot/2]).  Which coordinates pair i is made of is a parameter:
// split-half, (i, i + rot/2), the reference's rule (kernels/ops.cu:21-33,
// kernels/execution.cu:28-40), or interleaved, (2i, 2i + 1).  The vectorised
// kernel below and the fused projection kernels are the split-half rule only.
// Cache layout per site: keys [pages, kv_heads, page_size, D], values transposed
// inside a page, [pages, kv_heads, D, page_size] (so that the attention kernels
// read runs of keys for one coordinate); slot = page*page_size + offset; a
// negative slot writes nothing (padding rows, read-only sites).
template <typename T>
__global__ void rope_scatter_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                                    const int* __restrict__ slots, const float* __restrict__ cos_tab,
                                    const float* __restrict__ sin_tab, T* __restrict__ kcache,
                                    T* __restrict__ vcache, int heads, int kv_heads, int dim, int rot,
                                    int page_size, int max_pos, int has_kv, int interleaved) {
    const int row = blockIdx.x;
    const int half = rot / 2;
    // which two coordinates pair d turns: (d, d + rot/2) in the split-half rule, (2d, 2d + 1) in the interleaved one
    const int lo_mul = interleaved ? 2 : 1, hi_add = interleaved ? 1 : half;
    int pos = positions[row];
    if (pos < 0) pos = 0;
    if (pos >= max_pos) pos = max_pos - 1;  // host rejects this before launch
    const float* cs = cos_tab + (size_t)pos * half;
    const float* sn = sin_tab + (size_t)pos * half;
    const int row_width = (heads + (has_kv ? 2 * kv_heads : 0)) * dim;
    T* base = qkv + (size_t)row * row_width;
    const int slot = (has_kv && slots) ? slots[row] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

    // q heads: rotate in place
    for (int i = threadIdx.x; i < heads * half; i += blockDim.x) {
        int h = i / half, d = i % half;
        T* p = base + h * dim;
        const int lo = d * lo_mul, hi = lo + hi_add;
        float a = load_f32(p + lo), b = load_f32(p + hi);
        float c = cs[d], s = sn[d];
        store_f32(p + lo, a * c - b * s);
        store_f32(p + hi, b * c + a * s);
    }
    if (slot < 0) return;
    // k heads: rotate and scatter
    const T* kb = base + heads * dim;
    for (int i = threadIdx.x; i < kv_heads * half; i += blockDim.x) {
        int h = i / half, d = i % half;
        const T* p = kb + h * dim;
        const int lo = d * lo_mul, hi = lo + hi_add;
        float a = load_f32(p + lo), b = load_f32(p + hi);
        float c = cs[d], s = sn[d];
        T* dst = kcache + (((size_t)page * kv_heads + h) * page_size + off) * dim;
        store_f32(dst + lo, a * c - b * s);
        store_f32(dst + hi, b * c + a * s);
    }
    // coordinates beyond the rotated part of k pass through
    if (rot < dim) {
        int tail = dim - rot;
        for (int i = threadIdx.x; i < kv_heads * tail; i += blockDim.x) {
            int h = i / tail, d = rot + i % tail;
            kcache[(((size_t)page * kv_heads + h) * page_size + off) * dim + d] = kb[h * dim + d];
        }
    }
    // v heads: copy
    const T* vb = kb + kv_heads * dim;
    for (int i = threadIdx.x; i < kv_heads * dim; i += blockDim.x) {
        int h = i / dim, d = i % dim;
        vcache[(((size_t)page * kv_heads + h) * dim + d) * page_size + off] = vb[i];
    }
}

// The values of a prompt portion, 16 consecutive rows by 512 value columns a block, through LDS into the
// transposed pages.  Rows that follow each other in a request lie side by side in a coordinate's run of a page:
// when the 16 rows are one such run (inside one page, from a multiple of 8 on), a thread writes a coordinate's
// 16 positions as 32 contiguous bytes and a wave 2 KB; otherwise lane j of every 16 writes row j's elements one
// by one, which still puts neighbouring rows into one sector.  (One row at a time, every element is a 2-byte
// store into a sector of its own: 20 of 29 us at 2,048 rows of 2,048 value columns.)
__device__ __forceinline__ void rope_scatter_value_tile(const bf16_t* __restrict__ qkv, const int* __restrict__ slots,
                                                        bf16_t* __restrict__ vcache, int rows, int heads, int kv_heads,
                                                        int dim, int page_size, int tile) {
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    constexpr int TR = 16, CH = 512, PITCH = CH + 8;
    __shared__ __attribute__((aligned(16))) bf16_t vs[TR * PITCH];
    const int tid = threadIdx.x;
    const int vcols = kv_heads * dim, col_chunks = (vcols + CH - 1) / CH;
    const int row0 = (tile / col_chunks) * TR, c0 = (tile % col_chunks) * CH;
    const int row_width = (heads + 2 * kv_heads) * dim;
    const bf16_t* vbase = qkv + (size_t)(heads + kv_heads) * dim;
    for (int i = tid; i < TR * (CH / 8); i += 256) {
        const int rr = i / (CH / 8), cc = (i % (CH / 8)) * 8;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (row0 + rr < rows && c0 + cc < vcols) v = *(const u32x4*)(vbase + (size_t)(row0 + rr) * row_width + c0 + cc);
        *(u32x4*)(&vs[rr * PITCH + cc]) = v;
    }
    // one run?  (every thread looks at all 16 slots: the answer is the same for the whole block)
    const int s0 = slots[row0];
    bool run = s0 >= 0 && row0 + TR <= rows && (s0 % page_size) % 8 == 0 && s0 % page_size + TR <= page_size;
    for (int j = 1; j < TR && run; ++j) run = slots[row0 + j] == s0 + j;
    __syncthreads();
    if (run) {
        const int page = s0 / page_size, off = s0 % page_size;
        for (int c = tid; c < CH && c0 + c < vcols; c += 256) {
            const int col = c0 + c, h = col / dim, d = col % dim;
            uint32_t w[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                w[j] = (uint32_t)vs[(2 * j) * PITCH + c] | ((uint32_t)vs[(2 * j + 1) * PITCH + c] << 16);
            bf16_t* dst = vcache + (((size_t)page * kv_heads + h) * dim + d) * page_size + off;
            *(u32x4*)dst = (u32x4){w[0], w[1], w[2], w[3]};
            *(u32x4*)(dst + 8) = (u32x4){w[4], w[5], w[6], w[7]};
        }
        return;
    }
    const int j = tid % TR;
    const int slot = row0 + j < rows ? slots[row0 + j] : -1;
    if (slot < 0) return;
    const int page = slot / page_size, off = slot % page_size;
    for (int c = tid / TR; c < CH && c0 + c < vcols; c += 256 / TR) {
        const int col = c0 + c, h = col / dim, d = col % dim;
        vcache[(((size_t)page * kv_heads + h) * dim + d) * page_size + off] = vs[j * PITCH + c];
    }
}

// The same for bf16 rows whose whole heads turn (rot == dim) with dim a multiple of 16: `lanes` (64, 128 or
// 256) lanes of a block a row, every lane turns 8 pairs at a time with 16-byte loads and stores.
__global__ void __launch_bounds__(256)
rope_scatter_wave_kernel(bf16_t* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ slots,
                         const float* __restrict__ cos_tab, const float* __restrict__ sin_tab,
                         bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache, int rows, int heads, int kv_heads,
                         int dim, int page_size, int max_pos, int has_kv, int lanes, int qk_blocks) {
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
    if ((int)blockIdx.x >= qk_blocks) {                  // the blocks after the turning ones carry the values of a portion
        rope_scatter_value_tile(qkv, slots, vcache, rows, heads, kv_heads, dim, page_size, blockIdx.x - qk_blocks);
        return;
    }
    const bool values_here = qk_blocks == (int)gridDim.x;   // no value blocks: every row writes its own
    const int lane = threadIdx.x % lanes;
    const int row = blockIdx.x * (256 / lanes) + __builtin_amdgcn_readfirstlane(threadIdx.x / lanes);   // lanes is a multiple of 64: uniform in a wave
    if (row >= rows) return;
    const int half = dim / 2, per_head = half / 8;   // 8-pair chunks of a head
    int pos = positions[row];
    pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
    const float* cs = cos_tab + (size_t)pos * half;
    const float* sn = sin_tab + (size_t)pos * half;
    const int row_width = (heads + (has_kv ? 2 * kv_heads : 0)) * dim;
    bf16_t* base = qkv + (size_t)row * row_width;
    const int slot = (has_kv && slots) ? slots[row] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    const int turning = heads + (slot >= 0 ? kv_heads : 0);   // q heads, then k heads if they have a place to go
    for (int i = lane; i < turning * per_head; i += lanes) {
        const int h = i / per_head, d = (i % per_head) * 8;
        const bf16_t* p = base + h * dim + d;
        const u32x4 av = *(const u32x4*)p, bv = *(const u32x4*)(p + half);
        const float4 c0 = *(const float4*)(cs + d), c1 = *(const float4*)(cs + d + 4);
        const float4 s0 = *(const float4*)(sn + d), s1 = *(const float4*)(sn + d + 4);
        const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float a0 = __uint_as_float(av[j] << 16), a1 = __uint_as_float(av[j] & 0xffff0000u);
            const float b0 = __uint_as_float(bv[j] << 16), b1 = __uint_as_float(bv[j] & 0xffff0000u);
            lo[j] = pack_bf16x2(a0 * c[2 * j] - b0 * sv[2 * j], a1 * c[2 * j + 1] - b1 * sv[2 * j + 1]);
            hi[j] = pack_bf16x2(b0 * c[2 * j] + a0 * sv[2 * j], b1 * c[2 * j + 1] + a1 * sv[2 * j + 1]);
        }
        bf16_t* dst = h < heads ? base + h * dim + d
                                : kcache + (((size_t)page * kv_heads + (h - heads)) * page_size + off) * dim + d;
        *(u32x4*)dst = (u32x4){lo[0], lo[1], lo[2], lo[3]};
        *(u32x4*)(dst + half) = (u32x4){hi[0], hi[1], hi[2], hi[3]};
    }
    if (slot < 0 || !values_here) return;
    // v heads: 8 coordinates a lane, written to the transposed page one by one
    const bf16_t* vb = base + (heads + kv_heads) * dim;
    for (int i = lane; i < kv_heads * (dim / 8); i += lanes) {
        const int h = i / (dim / 8), d = (i % (dim / 8)) * 8;
        const u32x4 v = *(const u32x4*)(vb + h * dim + d);
        bf16_t* dst = vcache + (((size_t)page * kv_heads + h) * dim + d) * page_size + off;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            dst[(size_t)(2 * j) * page_size] = (bf16_t)(v[j] & 0xffffu);
            dst[(size_t)(2 * j + 1) * page_size] = (bf16_t)(v[j] >> 16);
        }
    }
}

extern "C" int cisr_rope_scatter(void* qkv, const int* positions, const int* slots, const float* cos_tab,
                                 const float* sin_tab, void* kcache, void* vcache, int rows, int heads,
                                 int kv_heads, int dim, int rot, int page_size, int max_pos, int has_kv,
                                 int interleaved, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dtype == DT_F32) {
        rope_scatter_kernel<float><<<rows, 256, 0, stream>>>((float*)qkv, positions, slots, cos_tab, sin_tab,
            (float*)kcache, (float*)vcache, heads, kv_heads, dim, rot, page_size, max_pos, has_kv, interleaved);
    } else if (!interleaved && rot == dim && dim % 16 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)cos_tab % 16 == 0 &&
               (uintptr_t)sin_tab % 16 == 0 && (!has_kv || (uintptr_t)kcache % 16 == 0)) {
        // lanes a row: as many as it has 8-pair chunks to turn, so that every lane's loads are in flight at once
        const int chunks = (heads + (has_kv ? kv_heads : 0)) * (dim / 16);
        const int lanes = chunks > 128 ? 256 : chunks > 64 ? 128 : 64, rows_a_block = 256 / lanes;
        const int qk_blocks = (rows + rows_a_block - 1) / rows_a_block;
        // a portion of 32 rows and more: further blocks carry the values, 16 rows by 512 columns each
        const long long value_blocks = (rows >= 32 && has_kv && slots) ? (long long)((rows + 15) / 16) * ((kv_heads * dim + 511) / 512) : 0;
        if (qk_blocks + value_blocks > 0x7fffffffLL) return (int)hipErrorInvalidValue;
        rope_scatter_wave_kernel<<<(unsigned)(qk_blocks + value_blocks), 256, 0, stream>>>((bf16_t*)qkv, positions, slots,
            cos_tab, sin_tab, (bf16_t*)kcache, (bf16_t*)vcache, rows, heads, kv_heads, dim, page_size, max_pos, has_kv, lanes,
            qk_blocks);
    } else {
        rope_scatter_kernel<bf16_t><<<rows, 256, 0, stream>>>((bf16_t*)qkv, positions, slots, cos_tab, sin_tab,
            (bf16_t*)kcache, (bf16_t*)vcache, heads, kv_heads, dim, rot, page_size, max_pos, has_kv, interleaved);
    }
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------- page copy
// Copy whole pages inside one cache tensor laid out [slabs, pages, page_elems]:
// for every slab, page dst[i] := page src[i].  Used for copy-on-write of a
// shared, partly filled page (reference: runtime/cache.py:70-75).
__global__ void page_copy_kernel(uint32_t* __restrict__ pool, const int* __restrict__ src,
                                 const int* __restrict__ dst, size_t page_words, size_t slab_words) {
    const int pair = blockIdx.x, slab = blockIdx.y;
    const uint32_t* s = pool + slab * slab_words + (size_t)src[pair] * page_words;
    uint32_t* d = pool + slab * slab_words + (size_t)dst[pair] * page_words;
    for (size_t i = threadIdx.x; i < page_words; i += blockDim.x) d[i] = s[i];
}

extern "C" int cisr_page_copy(void* pool, const int* src, const int* dst, int n_pairs, int slabs,
                              long long page_bytes, long long slab_bytes, hipStream_t stream) {
    if (n_pairs <= 0 || slabs <= 0) return 0;
    if (page_bytes % 4 || slab_bytes % 4) return (int)hipErrorInvalidValue;
    page_copy_kernel<<<dim3(n_pairs, slabs), 256, 0, stream>>>((uint32_t*)pool, src, dst,
        (size_t)(page_bytes / 4), (size_t)(slab_bytes / 4));
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------- conversions
// float -> bf16 with round-to-nearest-even; used when a matrix stored in 32 bits
// is run in bf16, and by the tests of the rounding rule.
__global__ void f32_to_bf16_kernel(const float* __restrict__ x, bf16_t* __restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = f32_to_bf16(x[i]);
}

extern "C" int cisr_f32_to_bf16(const float* x, void* y, long long n, hipStream_t stream) {
    if (n <= 0) return 0;
    f32_to_bf16_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, (bf16_t*)y, (size_t)n);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------- bias
// x[r][c] += bias[c] (added in float, rounded once to x's type): the projections of an architecture with biases run
// their product as it is and add the bias here, before whatever reads the rows next.
template <typename TX, typename TB>
__global__ void bias_add_kernel(TX* __restrict__ x, const TB* __restrict__ bias, size_t n, int cols) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) store_f32(x + i, load_f32(x + i) + load_f32(bias + i % cols));
}

extern "C" int cisr_bias_add(void* x, const void* bias, long long rows, int cols, int x_dtype, int bias_dtype, hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return 0;
    const size_t n = (size_t)rows * cols;
    if ((n + 255) / 256 > 0x7fffffffull) return (int)hipErrorInvalidValue;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (x_dtype == DT_F32 && bias_dtype == DT_F32) bias_add_kernel<float, float><<<blocks, 256, 0, stream>>>((float*)x, (const float*)bias, n, cols);
    else if (x_dtype == DT_F32) bias_add_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((float*)x, (const bf16_t*)bias, n, cols);
    else if (bias_dtype == DT_F32) bias_add_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>((bf16_t*)x, (const float*)bias, n, cols);
    else bias_add_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, (const bf16_t*)bias, n, cols);
    return CISR_LAUNCH_CHECK();
}
