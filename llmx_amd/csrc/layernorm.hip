// Layer norm with a weight and no bias, and the element-wise steps of layers that norm a sublayer's result before it
// joins the residual: y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations.  Everything is float32
// arithmetic on float32 rows; only what a product reads next is stored in the activation type.
// A row's sums are formed by 256 threads: thread v adds elements v, v + 256, ... in this order, a wave adds its threads'
// sums with wave_sum, and the four waves' sums are added in wave order: a function of the row's length only.
#include "common.h"

#define LN_THREADS 256
#define LN_KEPT 16      // values a thread keeps in registers: rows of at most 4,096 values are read once

// mean and 1 / sqrt(var + eps) of a row; v[] receives the thread's values when the row fits the registers
template <bool KEPT>
__device__ __forceinline__ void row_moments(const float* __restrict__ row, int n, float eps, float* scratch, float (&v)[LN_KEPT], float& mean,
                                            float& rstd) {
    const int tid = threadIdx.x;
    float s = 0.0f;
    if (KEPT) {
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) v[j] = tid + LN_THREADS * j < n ? row[tid + LN_THREADS * j] : 0.0f;
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) s += v[j];
    } else {
        for (int i = tid; i < n; i += LN_THREADS) s += row[i];
    }
    mean = block_sum<LN_THREADS / 64>(s, scratch) / (float)n;
    float q = 0.0f;
    if (KEPT) {
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) {
            const float d = tid + LN_THREADS * j < n ? v[j] - mean : 0.0f;
            q = fmaf(d, d, q);
        }
    } else {
        for (int i = tid; i < n; i += LN_THREADS) {
            const float d = row[i] - mean;
            q = fmaf(d, d, q);
        }
    }
    rstd = 1.0f / sqrtf(block_sum<LN_THREADS / 64>(q, scratch) / (float)n + eps);
}

// out[r] = LN(x[pick ? pick[r] : r]) in the activation type and/or float32
template <typename TO, bool KEPT>
__global__ void __launch_bounds__(LN_THREADS) layernorm_kernel(const float* __restrict__ x, const int* __restrict__ pick, const float* __restrict__ w,
                                                             float eps, TO* __restrict__ out, float* __restrict__ out32, int n) {
    __shared__ float scratch[LN_THREADS / 64];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = x + (size_t)(pick ? pick[r] : r) * n;
    float v[LN_KEPT], mean, rstd;
    row_moments<KEPT>(row, n, eps, scratch, v, mean, rstd);
    if (KEPT) {
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) {
            const int i = tid + LN_THREADS * j;
            if (i < n) {
                const float y = (v[j] - mean) * rstd * w[i];
                if (out) st(out + (size_t)r * n + i, y);
                if (out32) out32[(size_t)r * n + i] = y;
            }
        }
    } else {
        for (int i = tid; i < n; i += LN_THREADS) {
            const float y = (row[i] - mean) * rstd * w[i];
            if (out) st(out + (size_t)r * n + i, y);
            if (out32) out32[(size_t)r * n + i] = y;
        }
    }
}

extern "C" int llmx_layernorm(const float* x, const int* pick, const float* w, float eps, void* out, int out_dtype, float* out32, int rows, int n,
                              hipStream_t stream) {
    if (rows <= 0) return 0;
    if (n <= 0 || !w || (!out && !out32)) return -2;
    llmx_note_launch(LK_LAYERNORM);
    const bool kept = n <= LN_THREADS * LN_KEPT;
#define LLMX_LN(TO, K) hipLaunchKernelGGL((layernorm_kernel<TO, K>), dim3(rows), dim3(LN_THREADS), 0, stream, x, pick, w, eps, (TO*)out, out32, n)
    if (out_dtype == LLMX_F32) {
        if (kept) LLMX_LN(float, true);
        else LLMX_LN(float, false);
    } else {
        if (kept) LLMX_LN(bf16_t, true);
        else LLMX_LN(bf16_t, false);
    }
#undef LLMX_LN
    return LLMX_CHECK_LAUNCH();
}

// x[r] += LN(y[r]) * w: a sublayer's result joins the residual after its own norm; `copy` (optional) receives the new row
// in the activation type for the product that reads it next.
template <typename TO, bool KEPT>
__global__ void __launch_bounds__(LN_THREADS) layernorm_add_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w,
                                                                 float eps, TO* __restrict__ copy, int n) {
    __shared__ float scratch[LN_THREADS / 64];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = y + (size_t)r * n;
    float* xr = x + (size_t)r * n;
    float v[LN_KEPT], mean, rstd;
    float old[LN_KEPT];
    if (KEPT) {
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) old[j] = tid + LN_THREADS * j < n ? xr[tid + LN_THREADS * j] : 0.0f;
    }
    row_moments<KEPT>(row, n, eps, scratch, v, mean, rstd);
    if (KEPT) {
#pragma unroll
        for (int j = 0; j < LN_KEPT; ++j) {
            const int i = tid + LN_THREADS * j;
            if (i < n) {
                const float s = old[j] + (v[j] - mean) * rstd * w[i];
                xr[i] = s;
                if (copy) st(copy + (size_t)r * n + i, s);
            }
        }
    } else {
        for (int i = tid; i < n; i += LN_THREADS) {
            const float s = xr[i] + (row[i] - mean) * rstd * w[i];
            xr[i] = s;
            if (copy) st(copy + (size_t)r * n + i, s);
        }
    }
}

extern "C" int llmx_layernorm_add(float* x, const float* y, const float* w, float eps, void* copy, int copy_dtype, int rows, int n,
                                  hipStream_t stream) {
    if (rows <= 0) return 0;
    if (n <= 0 || !w) return -2;
    llmx_note_launch(LK_LAYERNORM_ADD);
    const bool kept = n <= LN_THREADS * LN_KEPT;
#define LLMX_LN(TO, K) hipLaunchKernelGGL((layernorm_add_kernel<TO, K>), dim3(rows), dim3(LN_THREADS), 0, stream, x, y, w, eps, (TO*)copy, n)
    if (copy_dtype == LLMX_F32) {
        if (kept) LLMX_LN(float, true);
        else LLMX_LN(float, false);
    } else {
        if (kept) LLMX_LN(bf16_t, true);
        else LLMX_LN(bf16_t, false);
    }
#undef LLMX_LN
    return LLMX_CHECK_LAUNCH();
}

// out = x in the activation type: the rows a product reads when a sublayer takes the residual itself.
template <typename TO>
__global__ void __launch_bounds__(256) cast_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, size_t total) {
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    const size_t at = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
    if (at >= total) return;
    if (at + 4 <= total) {
        const f32x4_t v = *reinterpret_cast<const f32x4_t*>(x + at);
#pragma unroll
        for (int i = 0; i < 4; ++i) st(out + at + i, v[i]);
        return;
    }
    for (size_t i = at; i < total; ++i) st(out + i, x[i]);
}

extern "C" int llmx_cast_rows(const float* x, void* out, int out_dtype, long total, hipStream_t stream) {
    if (total <= 0) return 0;
    llmx_note_launch(LK_CAST_ROWS);
    const dim3 grid((unsigned)((total + 1023) / 1024));
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(cast_rows_kernel<float>, grid, dim3(256), 0, stream, x, (float*)out, (size_t)total);
    else hipLaunchKernelGGL(cast_rows_kernel<bf16_t>, grid, dim3(256), 0, stream, x, (bf16_t*)out, (size_t)total);
    return LLMX_CHECK_LAUNCH();
}

// out[t, :] = x[t, col0 : col0 + n] in the activation type: some columns of a wider float32 projection as the rows a further
// product reads (the inner values of a low-rank projection).
template <typename TO>
__global__ void __launch_bounds__(256) cast_cols_kernel(const float* __restrict__ x, int ld, TO* __restrict__ out, int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    st(out + at, x[(at / (size_t)n) * (size_t)ld + (at % (size_t)n)]);
}

extern "C" int llmx_cast_cols(const float* x, int ld, void* out, int out_dtype, int rows, int n, hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    if (ld < n) return -2;
    llmx_note_launch(LK_CAST_COLS);
    const size_t total = (size_t)rows * n;
    const dim3 grid((unsigned)((total + 255) / 256));
    if (out_dtype == LLMX_F32) hipLaunchKernelGGL(cast_cols_kernel<float>, grid, dim3(256), 0, stream, x, ld, (float*)out, n, total);
    else hipLaunchKernelGGL(cast_cols_kernel<bf16_t>, grid, dim3(256), 0, stream, x, ld, (bf16_t*)out, n, total);
    return LLMX_CHECK_LAUNCH();
}

// out (=, +=) sa * (a + bias_a) + sb * b over float32 rows [T, n]: the join of mixers that run side by side, and a
// projection's bias; bias_a and b may be null.
__global__ void __launch_bounds__(256) combine_rows_kernel(float* __restrict__ out, const float* __restrict__ a, float sa,
                                                         const float* __restrict__ bias_a, const float* __restrict__ b, float sb, int accumulate,
                                                         int n, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    float va = a[at];
    if (bias_a) va = va + bias_a[(int)(at % (size_t)n)];
    float v = sa * va;
    if (b) v = v + sb * b[at];
    out[at] = accumulate ? out[at] + v : v;
}

extern "C" int llmx_combine_rows(float* out, const float* a, float sa, const float* bias_a, const float* b, float sb, int accumulate, int rows, int n,
                                 hipStream_t stream) {
    if (rows <= 0 || n <= 0) return 0;
    if (!a) return -2;
    llmx_note_launch(LK_COMBINE_ROWS);
    const size_t total = (size_t)rows * n;
    hipLaunchKernelGGL(combine_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, out, a, sa, bias_a, b, sb, accumulate, n, total);
    return LLMX_CHECK_LAUNCH();
}

// logits <- logits * scale, then cap * tanh(logits / cap) when cap > 0, in place.
__global__ void __launch_bounds__(256) scale_softcap_kernel(float* __restrict__ z, float scale, float cap, size_t total) {
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    float v = z[at] * scale;
    if (cap > 0.0f) v = cap * tanhf(v / cap);
    z[at] = v;
}

extern "C" int llmx_scale_softcap(float* z, float scale, float cap, long total, hipStream_t stream) {
    if (total <= 0) return 0;
    llmx_note_launch(LK_SCALE_SOFTCAP);
    hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, z, scale, cap, (size_t)total);
    return LLMX_CHECK_LAUNCH();
}
