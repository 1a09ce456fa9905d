// jl_norm.hip — embedding gather, the residual-update + RMS-norm launches (norm of the stream, norm of a sublayer's output) and the
// polynomial activation.
#include "jl_common.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(const T *__restrict__ embed, const int64_t *__restrict__ ids, int W,
                                                           float scale, float *__restrict__ x, float *__restrict__ x0) {
    const int64_t n = blockIdx.x;
    const T *src = embed + ids[n] * (int64_t)W;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = ld_f(src + c) * scale;
        x[n * W + c] = v;
        if (x0) x0[n * W + c] = v;
    }
}

extern "C" int jl_embed_scale(const void *embed, int dtype, const int64_t *ids, int64_t N, int32_t W, float scale, float *x, float *x0,
                              void *stream) {
    if (N <= 0) return JL_OK;
    if (!embed || !ids || !x || W <= 0) return jl_fail(JL_E_INVALID, "jl_embed_scale: null pointer or bad width");
    JL_DISPATCH(dtype, embed_scale_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>((const T *)embed, ids, W, scale, x, x0));
    return jl_check_launch("embed_scale_kernel");
}

// one workgroup per row: pass 1 forms the new residual (written back) and its sum of squares, pass 2 normalises what pass 1 wrote
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float *__restrict__ x, const void *__restrict__ y, int y_dtype, int y_count,
                                                           const float *__restrict__ x0, const T *__restrict__ w, float eps,
                                                           T *__restrict__ out, int W) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    float *xr = x + n * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = xr[c];
        if (y)
            for (int s = 0; s < y_count; ++s) v += ld_any(y, y_dtype, (n * y_count + s) * (int64_t)W + c);
        if (x0) v += x0[n * W + c];
        if (y || x0) xr[c] = v;
        ss += v * v;
    }
    if (!out) return;
    ss = block_sum_f32(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = xr[c] * r;
        st_f(out + n * W + c, w ? v * ld_f(w + c) : v);
    }
}

extern "C" int jl_add_rmsnorm(float *x, const void *y, int y_dtype, int32_t y_count, const float *x0, const void *w, float eps,
                              void *out, int dtype, int64_t N, int32_t W, void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || W <= 0 || (y && y_count <= 0)) return jl_fail(JL_E_INVALID, "jl_add_rmsnorm: null pointer or bad sizes");
    JL_DISPATCH(dtype, add_rmsnorm_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(x, y, y_dtype, y_count, x0, (const T *)w,
                                                                                                 eps, (T *)out, W));
    return jl_check_launch("add_rmsnorm_kernel");
}

// ---- sublayer-output norm + residual update: one workgroup per row ------------------------------------------------------------
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void norm_add_kernel(float *__restrict__ x, const TY *__restrict__ y, const float *__restrict__ g, float eps,
                                                        TO *__restrict__ out, int W) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const TY *yr = y + n * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = ld_f(yr + c); ss += v * v; }
    ss = block_sum_f32(ss, red);
    const float r = g[0] / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = x[n * W + c] + ld_f(yr + c) * r;
        x[n * W + c] = v;
        if (out) st_f(out + n * W + c, v);
    }
}

extern "C" int jl_norm_add(float *x, const void *y, int y_dtype, const float *g, float eps, void *out, int out_dtype, int64_t N, int32_t W,
                           void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || !y || !g || W <= 0) return jl_fail(JL_E_INVALID, "jl_norm_add: null pointer or bad width");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)N);
    if (y_dtype == JL_BF16) {
        if (out_dtype == JL_BF16) norm_add_kernel<bf16_t, bf16_t><<<grid, 256, 0, st>>>(x, (const bf16_t *)y, g, eps, (bf16_t *)out, W);
        else norm_add_kernel<bf16_t, float><<<grid, 256, 0, st>>>(x, (const bf16_t *)y, g, eps, (float *)out, W);
    } else {
        if (out_dtype == JL_BF16) norm_add_kernel<float, bf16_t><<<grid, 256, 0, st>>>(x, (const float *)y, g, eps, (bf16_t *)out, W);
        else norm_add_kernel<float, float><<<grid, 256, 0, st>>>(x, (const float *)y, g, eps, (float *)out, W);
    }
    return jl_check_launch("norm_add_kernel");
}

// ---- polynomial activation with unit-RMS powers: one workgroup per row --------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void polynorm_kernel(const T *__restrict__ z, int F, const float *__restrict__ coef, float eps,
                                                        T *__restrict__ out) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const T *zr = z + n * F;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = ld_f(zr + c), v2 = v * v, v3 = v2 * v;
        s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
    }
    s1 = block_sum_f32(s1, red);
    s2 = block_sum_f32(s2, red);
    s3 = block_sum_f32(s3, red);
    const float r1 = coef[0] / sqrtf(s1 / (float)F + eps), r2 = coef[1] / sqrtf(s2 / (float)F + eps), r3 = coef[2] / sqrtf(s3 / (float)F + eps);
    const float e = coef[3];
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = ld_f(zr + c), v2 = v * v;
        st_f(out + n * F + c, v * r1 + v2 * r2 + v2 * v * r3 + e);
    }
}

extern "C" int jl_polynorm(const void *z, int dtype, int64_t N, int32_t F, const float *coef, float eps, void *out, void *stream) {
    if (N <= 0) return JL_OK;
    if (!z || !coef || !out || F <= 0) return jl_fail(JL_E_INVALID, "jl_polynorm: null pointer or bad width");
    JL_DISPATCH(dtype, polynorm_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>((const T *)z, F, coef, eps, (T *)out));
    return jl_check_launch("polynorm_kernel");
}
