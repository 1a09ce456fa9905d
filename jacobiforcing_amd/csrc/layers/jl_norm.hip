// jl_norm.hip — error plumbing of libjf_layers.so, embedding gather and the residual-update + RMS-norm launch.
#include "jl_common.h"

static thread_local char g_err[512] = "";

int jl_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
int jl_check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return JL_OK;
}
extern "C" int jl_version(void) { return JL_VERSION; }
extern "C" const char *jl_last_error(void) { return g_err; }

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
