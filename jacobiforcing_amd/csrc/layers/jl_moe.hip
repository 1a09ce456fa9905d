// jl_moe.hip — routed experts: the router's choice, the rows grouped by expert, and the two grouped products around relu^2.
#include "jl_common.h"

// ---- router: one thread per token ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_route_kernel(const float *__restrict__ logits, const float *__restrict__ correction, int64_t N,
                                                         int E, int top, float scale, int32_t *__restrict__ ids,
                                                         float *__restrict__ weights) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    const float *z = logits + n * E;
    for (int s = 0; s < top; ++s) {
        int best = -1;
        float bc = 0.f, bs = 0.f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int p = 0; p < s; ++p) taken |= ids[n * top + p] == e;
            if (taken) continue;
            const float sc = 1.0f / (1.0f + expf(-z[e]));
            const float ch = sc + (correction ? correction[e] : 0.f);
            if (best < 0 || ch > bc) { best = e; bc = ch; bs = sc; }
        }
        ids[n * top + s] = best;
        weights[n * top + s] = bs * scale;
    }
}

extern "C" int jl_moe_route(const float *logits, const float *correction, int64_t N, int32_t E, int32_t top, float scale, int32_t *ids,
                            float *weights, void *stream) {
    if (N <= 0) return JL_OK;
    if (!logits || !ids || !weights || E <= 0 || top <= 0 || top > E) return jl_fail(JL_E_INVALID, "jl_moe_route: null pointer or top > experts");
    moe_route_kernel<<<dim3((unsigned)((N + 255) / 256)), 256, 0, (hipStream_t)stream>>>(logits, correction, N, E, top, scale, ids, weights);
    return jl_check_launch("moe_route_kernel");
}

// ---- grouping: one workgroup counts, scans and places (a step holds at most a few 10^5 rows) ----------------------------------------
constexpr int MOE_TM = 32;        // rows of a tile
constexpr int MOE_TN = 64;        // output columns of a tile
constexpr int MOE_TK = 32;        // depth of one LDS stage
constexpr int MOE_MAX_E = 4096;

__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *__restrict__ ids, int64_t rows, int E, int tile_rows,
                                                          int32_t *__restrict__ perm, int32_t *__restrict__ offsets,
                                                          int32_t *__restrict__ tile_expert, int32_t *__restrict__ tile_row0, int max_tiles) {
    __shared__ int cnt[MOE_MAX_E];
    __shared__ int base[MOE_MAX_E + 1];
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int64_t r = threadIdx.x; r < rows; r += 1024) atomicAdd(&cnt[ids[r]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, t = 0;
        for (int e = 0; e < E; ++e) {
            base[e] = o;
            offsets[e] = o;
            for (int r = 0; r < cnt[e]; r += tile_rows)
                if (t < max_tiles) { tile_expert[t] = e; tile_row0[t] = o + r; ++t; }
            o += cnt[e];
        }
        offsets[E] = o;
        for (; t < max_tiles; ++t) { tile_expert[t] = -1; tile_row0[t] = 0; }
    }
    __syncthreads();
    // placement in row order within an expert, one thread per expert scanning the list (all reads hit L2): the order is fixed, so a
    // run is reproducible
    for (int e = threadIdx.x; e < E; e += 1024) {
        int o = base[e];
        if (cnt[e])
            for (int64_t r = 0; r < rows; ++r)
                if (ids[r] == e) perm[o++] = (int32_t)r;
    }
}

extern "C" int jl_moe_tile_rows(void) { return MOE_TM; }

extern "C" int jl_moe_group(const int32_t *ids, int64_t N, int32_t top, int32_t E, int32_t tile_rows, int32_t *perm, int32_t *offsets,
                            int32_t *tile_expert, int32_t *tile_row0, int32_t max_tiles, void *stream) {
    if (N <= 0) return JL_OK;
    if (!ids || !perm || !offsets || !tile_expert || !tile_row0) return jl_fail(JL_E_INVALID, "jl_moe_group: null pointer");
    if (E <= 0 || E > MOE_MAX_E || top <= 0 || tile_rows <= 0 || (int64_t)max_tiles < N * top / tile_rows + E)
        return jl_fail(JL_E_INVALID, "jl_moe_group: experts must be <= %d and max_tiles >= rows / tile_rows + experts", MOE_MAX_E);
    moe_group_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(ids, N * top, E, tile_rows, perm, offsets, tile_expert, tile_row0, max_tiles);
    return jl_check_launch("moe_group_kernel");
}

// ---- grouped product: a 32 x 64 tile of one expert's rows per workgroup, products in float from float / bf16 operands -------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T *__restrict__ X, const T *__restrict__ Wt, int mode, int K, int n_out, int top,
                                                        const int32_t *__restrict__ perm, const int32_t *__restrict__ offsets,
                                                        const int32_t *__restrict__ tile_expert, const int32_t *__restrict__ tile_row0,
                                                        const float *__restrict__ weights, void *__restrict__ out) {
    __shared__ float Xs[MOE_TM][MOE_TK + 1];
    __shared__ float Ws[MOE_TN][MOE_TK + 1];
    __shared__ int rin[MOE_TM];
    const int e = tile_expert[blockIdx.x];
    if (e < 0) return;
    const int r0 = tile_row0[blockIdx.x];
    const int nr = offsets[e + 1] - r0 < MOE_TM ? offsets[e + 1] - r0 : MOE_TM;
    const int n0 = blockIdx.y * MOE_TN;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    if (tid < MOE_TM) rin[tid] = tid < nr ? (mode == 0 ? perm[r0 + tid] / top : r0 + tid) : -1;
    const T *We = Wt + (int64_t)e * n_out * K;
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int k0 = 0; k0 < K; k0 += MOE_TK) {
        __syncthreads();
        for (int i = tid; i < MOE_TM * MOE_TK; i += 256) {
            const int m = i / MOE_TK, kk = i - m * MOE_TK;
            Xs[m][kk] = (rin[m] >= 0 && k0 + kk < K) ? ld_f(X + (int64_t)rin[m] * K + k0 + kk) : 0.f;
        }
        for (int i = tid; i < MOE_TN * MOE_TK; i += 256) {
            const int n = i / MOE_TK, kk = i - n * MOE_TK;
            Ws[n][kk] = (n0 + n < n_out && k0 + kk < K) ? ld_f(We + (int64_t)(n0 + n) * K + k0 + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < MOE_TK; ++kk) {
            const float a0 = Xs[ty * 2][kk], a1 = Xs[ty * 2 + 1][kk];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float w = Ws[tx + 16 * c][kk];
                acc[0][c] += a0 * w;
                acc[1][c] += a1 * w;
            }
        }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int m = ty * 2 + a;
        if (m >= nr) continue;
        const int r = r0 + m;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int n = n0 + tx + 16 * c;
            if (n >= n_out) continue;
            if (mode == 0) {
                const float v = fmaxf(acc[a][c], 0.f);
                st_f((T *)out + (int64_t)r * n_out + n, v * v);
            } else {
                const int p = perm[r];
                ((float *)out)[(int64_t)p * n_out + n] = acc[a][c] * weights[p];
            }
        }
    }
}

extern "C" int jl_moe_gemm(const void *X, const void *Wt, int dtype, int32_t mode, int32_t K, int32_t n_out, int32_t top,
                           const int32_t *perm, const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0,
                           int32_t max_tiles, const float *weights, void *out, void *stream) {
    if (max_tiles <= 0) return JL_OK;
    if (!X || !Wt || !perm || !offsets || !tile_expert || !tile_row0 || !out || (mode == 1 && !weights))
        return jl_fail(JL_E_INVALID, "jl_moe_gemm: null pointer");
    if (K <= 0 || n_out <= 0 || top <= 0 || (mode != 0 && mode != 1)) return jl_fail(JL_E_INVALID, "jl_moe_gemm: bad sizes or mode");
    const dim3 grid((unsigned)max_tiles, (unsigned)((n_out + MOE_TN - 1) / MOE_TN));
    JL_DISPATCH(dtype, moe_gemm_kernel<T><<<grid, 256, 0, (hipStream_t)stream>>>((const T *)X, (const T *)Wt, mode, K, n_out, top, perm, offsets,
                                                                                 tile_expert, tile_row0, weights, out));
    return jl_check_launch("moe_gemm_kernel");
}
