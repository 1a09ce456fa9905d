// jl_retention.hip — retention: linear attention with a fixed decay per head and a float state per (request slot, head),
// scanned token by token for prompt portions and decoded tokens alike.
#include "jl_common.h"

// One workgroup per (request, head); thread j owns column j of the state S [D, Dv] in registers.  Tokens are taken TT at a
// time: the rotated queries / keys of a group go through LDS, each thread runs the recurrence for its column, the per-token
// sums of squares (unit norm over the head's Dv outputs) are reduced once per group.
constexpr int RET_TT = 8;

// MAXT: the largest workgroup the instantiation is launched with.  With 256 the state's DMAX rows stay in registers up to
// DMAX = 128 (the default bound of 1 024 threads leaves 128 registers per lane and spills them).
template <typename T, int DMAX, int MAXT>
__global__ __launch_bounds__(MAXT) void retention_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int k_col, int v_col, int g_col,
                                 const int32_t *__restrict__ seq, int H, int D, int Dv, int rot_dims,
                                 const float *__restrict__ cos_t, const float *__restrict__ sin_t, int64_t table_len,
                                 const float *__restrict__ decay, float eps, float *__restrict__ state, T *__restrict__ out, int mode) {
    extern __shared__ float lds[];
    float *qs = lds;                                   // [TT][D]
    float *ks = qs + RET_TT * D;                       // [TT][D]
    float *red = ks + RET_TT * D;                      // [TT][16]
    const int b = blockIdx.x / H, h = blockIdx.x - b * H;
    const int row0 = seq[4 * b], cnt = seq[4 * b + 1], pos0 = seq[4 * b + 2], slot = seq[4 * b + 3];
    if (cnt <= 0) return;
    const int j = threadIdx.x, wave = j >> 6, nw = (blockDim.x + 63) >> 6;
    const bool live = j < Dv;
    const float gamma = decay[h], kscale = 1.0f / sqrtf((float)D);
    const int half = rot_dims >> 1;
    float *sp = state + ((int64_t)slot * H + h) * D * Dv;
    float S[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) S[d] = (live && d < D && (mode == JL_RET_FROM_SLOT || (mode == JL_RET_SCAN && pos0 > 0))) ? sp[(int64_t)d * Dv + j] : 0.f;

    for (int t0 = 0; t0 < cnt; t0 += RET_TT) {
        const int nt = cnt - t0 < RET_TT ? cnt - t0 : RET_TT;
        __syncthreads();
        for (int e = j; e < nt * D; e += blockDim.x) {
            const int tt = e / D, d = e - tt * D;
            const T *row = proj + (int64_t)(row0 + t0 + tt) * ld + h * D;
            float qv, kv;
            if (d < rot_dims) {
                const int i = d < half ? d : d - half;
                int64_t p = pos0 + t0 + tt;
                if (p >= table_len) p = table_len - 1;
                const float c = cos_t[p * half + i], s = sin_t[p * half + i];
                const float qu = ld_f(row + q_col + i), qw = ld_f(row + q_col + i + half);
                const float ku = ld_f(row + k_col + i), kw = ld_f(row + k_col + i + half);
                qv = d < half ? qu * c - qw * s : qw * c + qu * s;
                kv = d < half ? ku * c - kw * s : kw * c + ku * s;
            } else {
                qv = ld_f(row + q_col + d);
                kv = ld_f(row + k_col + d);
            }
            qs[e] = qv;
            ks[e] = kv * kscale;
        }
        __syncthreads();
        float o[RET_TT];
#pragma unroll
        for (int tt = 0; tt < RET_TT; ++tt) {
            o[tt] = 0.f;
            if (tt < nt) {
                const float v = live ? ld_f(proj + (int64_t)(row0 + t0 + tt) * ld + v_col + h * Dv + j) : 0.f;
                const float *qp = qs + tt * D, *kp = ks + tt * D;
                float acc = 0.f;
#pragma unroll
                for (int d = 0; d < DMAX; ++d)
                    if (d < D) {
                        S[d] = gamma * S[d] + kp[d] * v;
                        acc += S[d] * qp[d];
                    }
                o[tt] = acc;
                if (mode != JL_RET_LOCAL_STATE) {
                    const float ss = wave_sum_f32(acc * acc);
                    if ((j & 63) == 0) red[tt * 16 + wave] = ss;
                }
            }
        }
        if (mode == JL_RET_LOCAL_STATE) continue;
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < RET_TT; ++tt)
            if (tt < nt && live) {
                float ss = 0.f;
                for (int w = 0; w < nw; ++w) ss += red[tt * 16 + w];
                const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
                const int64_t n = row0 + t0 + tt;
                const float g = ld_f(proj + n * ld + g_col + h * Dv + j);
                st_f(out + n * ((int64_t)H * Dv) + h * Dv + j, o[tt] * r * (g / (1.0f + expf(-g))));
            }
    }
    if (live && mode != JL_RET_FROM_SLOT)
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < D) sp[(int64_t)d * Dv + j] = S[d];
}

template <typename T, int DMAX>
static int ret_launch(const void *proj, int64_t ld, int q_col, int k_col, int v_col, int g_col, const int32_t *seq, int B, int H, int D,
                      int Dv, int rot_dims, const float *cos_t, const float *sin_t, int64_t table_len, const float *decay, float eps,
                      float *state, void *out, int mode, hipStream_t st) {
    const int threads = (Dv + 63) / 64 * 64;
    const size_t lds = (size_t)(2 * RET_TT * D + RET_TT * 16) * 4;
    if (DMAX >= 128 && threads <= 256)
        retention_kernel<T, DMAX, 256><<<dim3((unsigned)(B * H)), threads, lds, st>>>((const T *)proj, ld, q_col, k_col, v_col, g_col, seq, H, D, Dv,
                                                                                     rot_dims, cos_t, sin_t, table_len, decay, eps, state, (T *)out, mode);
    else
        retention_kernel<T, DMAX, 1024><<<dim3((unsigned)(B * H)), threads, lds, st>>>((const T *)proj, ld, q_col, k_col, v_col, g_col, seq, H, D, Dv,
                                                                                      rot_dims, cos_t, sin_t, table_len, decay, eps, state, (T *)out, mode);
    return jl_check_launch("retention_kernel");
}

extern "C" int jl_retention(const void *proj, int dtype, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col, int32_t g_col,
                            const int32_t *seq, int32_t B, int32_t H, int32_t D, int32_t Dv, int32_t rot_dims, const float *cos_t,
                            const float *sin_t, int64_t table_len, const float *decay, float eps, float *state, void *out,
                            int32_t mode, void *stream) {
    if (B <= 0) return JL_OK;
    if (!proj || !seq || !decay || !state || (!out && mode != JL_RET_LOCAL_STATE)) return jl_fail(JL_E_INVALID, "jl_retention: null pointer");
    if (mode < JL_RET_SCAN || mode > JL_RET_FROM_SLOT) return jl_fail(JL_E_INVALID, "jl_retention: unknown mode %d", mode);
    if (H <= 0 || D <= 0 || D > 256 || Dv <= 0 || Dv > 1024) return jl_fail(JL_E_INVALID, "jl_retention: D must be <= 256 and Dv <= 1024");
    if (rot_dims < 0 || rot_dims > D || rot_dims % 2 || (rot_dims && (!cos_t || !sin_t || table_len <= 0)))
        return jl_fail(JL_E_INVALID, "jl_retention: rot_dims must be even and <= D, with tables");
    hipStream_t st = (hipStream_t)stream;
#define RET_CASE(N) JL_DISPATCH(dtype, return (ret_launch<T, N>(proj, ld, q_col, k_col, v_col, g_col, seq, B, H, D, Dv, rot_dims, cos_t, \
                                                                 sin_t, table_len, decay, eps, state, out, mode, st)))
    if (D <= 32) RET_CASE(32);
    else if (D <= 64) RET_CASE(64);
    else if (D <= 128) RET_CASE(128);
    else RET_CASE(256);
#undef RET_CASE
    return JL_OK;
}

// Joins the chunks of long portions.  Per (request, head): S = the request's state (zero when it starts at position 0); for each of
// its chunks in order: the chunk's local state in `scratch` is replaced by S (the state the chunk starts from), then
// S = decay^len S + local.  The final S is the request's new state.  req [B, 4] = {first chunk, chunks, pos0, slot},
// chunk_len [chunks] int32.
__global__ __launch_bounds__(256) void retention_join_kernel(const int32_t *__restrict__ req, const int32_t *__restrict__ chunk_len, int H,
                                                              int64_t DDv, const float *__restrict__ decay, float *__restrict__ state,
                                                              float *__restrict__ scratch) {
    const int b = blockIdx.x / H, h = blockIdx.x - b * H;
    const int c0 = req[4 * b], nc = req[4 * b + 1], pos0 = req[4 * b + 2], slot = req[4 * b + 3];
    const float gamma = decay[h];
    float *sp = state + ((int64_t)slot * H + h) * DDv;
    for (int64_t e = (int64_t)blockIdx.y * 256 + threadIdx.x; e < DDv; e += (int64_t)gridDim.y * 256) {
        float S = pos0 > 0 ? sp[e] : 0.f;
        for (int c = c0; c < c0 + nc; ++c) {
            float *lp = scratch + ((int64_t)c * H + h) * DDv + e;
            const float local = *lp;
            *lp = S;
            float gp = 1.f;
            for (int t = 0; t < chunk_len[c]; ++t) gp *= gamma;
            S = gp * S + local;
        }
        sp[e] = S;
    }
}

extern "C" int jl_retention_join(const int32_t *req, int32_t B, const int32_t *chunk_len, int32_t H, int32_t D, int32_t Dv,
                                 const float *decay, float *state, float *scratch, void *stream) {
    if (B <= 0) return JL_OK;
    if (!req || !chunk_len || !decay || !state || !scratch || H <= 0 || D <= 0 || Dv <= 0) return jl_fail(JL_E_INVALID, "jl_retention_join: null pointer or bad sizes");
    const int64_t ddv = (int64_t)D * Dv;
    const unsigned gy = (unsigned)((ddv + 255) / 256 < 64 ? (ddv + 255) / 256 : 64);
    retention_join_kernel<<<dim3((unsigned)(B * H), gy), 256, 0, (hipStream_t)stream>>>(req, chunk_len, H, ddv, decay, state, scratch);
    return jl_check_launch("retention_join_kernel");
}
