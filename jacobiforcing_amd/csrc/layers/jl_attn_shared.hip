// jl_attn_shared.hip — attention over ONE key/value head shared by all query heads, whose values are the first Dv columns of the key
// rows (the pool of latent attention: [latent | rotary key]), on the matrix cores (bfloat16).  Sliding window or plain causal, one
// sweep with a running maximum and sum.
//
// A workgroup of four wavefronts owns up to 32 rows = (query, head) pairs of one request — HF = min(H, 32) heads of 32 / HF
// consecutive queries — and walks the visible keys 32 at a time through LDS.  Per key tile:
//   1. the four wavefronts each form the 32 x 32 scores over a quarter of the key width (v_mfma_f32_32x32x8_bf16; the query
//      fragments stay in registers for the whole launch) and leave their partial sums in LDS;
//   2. 8 threads per row add the partial sums, mask, update the row's maximum and sum, and write exp(s - max) as bfloat16 and the
//      rescale factor of the row;
//   3. every wavefront multiplies the weights with ITS quarter of the value columns (the same LDS rows the keys were read from).
// Few tiles with many keys (decoding): the key tiles of a row tile are shared out over blockIdx.z; every share leaves its
// unnormalised outputs with its maximum and sum in a scratch, and attn_shared_join_kernel combines them.
// Accumulator r of lane l of a 32 x 32 MFMA is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32; lane l supplies row (A) or
// column (B) l % 32 with depths 4 * (l / 32) .. + 3.
#include "jl_common.h"

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short as_bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float as_f32x16;
constexpr int AS_T = 32, AS_WAVES = 4, AS_THREADS = 64 * AS_WAVES, AS_QSTEPS = 20;      // key width <= 8 * 4 * 20 = 640
constexpr int AS_PROW = 36;                                                            // weights' row stride in LDS (bfloat16)

__device__ __forceinline__ short as_bf16(float v) {
    uint32_t u = __float_as_uint(v);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (short)(u >> 16);
}

static size_t as_lds_bytes(int D) { return (size_t)AS_T * (D + 4) * 2 + (size_t)AS_WAVES * AS_T * 33 * 4 + (size_t)AS_T * AS_PROW * 2 + 2 * AS_T * 4; }

template <int NT>                                                                       // value columns per wavefront = 32 * NT, Dv = 128 * NT
__global__ __launch_bounds__(AS_THREADS) void attn_shared_kv_kernel(jl_attn_args a, int HF, int TQ) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int H = a.H, D = a.D, Dv = a.Dv, KROW = D + 4;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, hi = lane >> 5;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    const int h0 = blockIdx.y * HF;
    bf16_t *Ks = (bf16_t *)smem;                                    // [32][D + 4]
    float *Sp = (float *)(Ks + AS_T * KROW);                        // [4][32][33] partial scores
    bf16_t *Pb = (bf16_t *)(Sp + AS_WAVES * AS_T * 33);             // [32][36] weights
    float *alphaS = (float *)(Pb + AS_T * AS_PROW);                 // [32] rescale factor of the tile
    float *lS = alphaS + AS_T;                                      // [32] final sums
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int n_keys = i_max + 1 - lo;
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const bf16_t *kc = (const bf16_t *)a.k_cache;
    const int page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;

    // this lane's query fragments: row l32 = (query l32 / HF, head h0 + l32 % HF), key-width steps wave, wave + 4, ..
    as_bf16x4 qf[AS_QSTEPS];
    {
        const int ii = l32 / HF, hh = h0 + l32 % HF;
        const bool ok = l32 < TQ * HF && ii < cnt && hh < H;
        const bf16_t *qp = (const bf16_t *)a.q + ((int64_t)(row0 + ii) * H + hh) * D + 4 * hi;
#pragma unroll
        for (int x = 0; x < AS_QSTEPS; ++x) {
            const int kk = 8 * (AS_WAVES * x + wave);
            qf[x] = (as_bf16x4){0, 0, 0, 0};
            if (ok && kk < D) qf[x] = *(const as_bf16x4 *)(qp + kk);
        }
    }
    // the row this thread helps to reduce: row tid / 8, keys 4 * (tid % 8) .. + 3
    const int rr = tid >> 3, rc = (tid & 7) * 4;
    const int r_i = i0 + rr / HF;
    const bool r_ok = rr < TQ * HF && rr / HF < cnt && h0 + rr % HF < H;
    float m_run = -INFINITY, l_run = 0.f;

    as_f32x16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

    const int units = D / 4;                                        // 8-byte units per key row
    const int jj0 = tid / units, u0r = tid - jj0 * units, dj = AS_THREADS / units, dr = AS_THREADS - dj * units;

    const int S = a.splits > 1 ? a.splits : 1, split = blockIdx.z;
    const int per = ((n_keys + AS_T - 1) / AS_T + S - 1) / S;       // key tiles per share
    const int key_lo = split * per * AS_T, key_hi = (split + 1) * per * AS_T < n_keys ? (split + 1) * per * AS_T : n_keys;
    for (int u0 = key_lo; u0 < key_hi; u0 += AS_T) {
        const int nk = key_hi - u0 < AS_T ? key_hi - u0 : AS_T;
        __syncthreads();                                            // the previous tile's readers are done with Ks / Pb
        {
            int jj = jj0, r = u0r;
            for (int e = tid; e < AS_T * units; e += AS_THREADS) {
                uint2 v = make_uint2(0, 0);
                if (jj < nk) {
                    const int j = lo + u0 + jj;
                    const int pg = page_shift >= 0 ? j >> page_shift : j / a.page_size;
                    const int64_t tok = (int64_t)bt[pg] * a.page_size + (j - pg * a.page_size);
                    v = *(const uint2 *)(kc + tok * a.k_ld + 4 * r);
                }
                *(uint2 *)(Ks + jj * KROW + 4 * r) = v;
                jj += dj; r += dr;
                if (r >= units) { r -= units; ++jj; }
            }
        }
        __syncthreads();
        {   // 1. partial scores of this wavefront's share of the key width
            as_f32x16 sc;
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = 0.f;
            const bf16_t *kp = Ks + l32 * KROW + 4 * hi;
#pragma unroll
            for (int x = 0; x < AS_QSTEPS; ++x) {
                const int kk = 8 * (AS_WAVES * x + wave);
                if (kk < D) sc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(qf[x], *(const as_bf16x4 *)(kp + kk), sc, 0, 0, 0);
            }
            float *sp = Sp + wave * AS_T * 33;
#pragma unroll
            for (int r = 0; r < 16; ++r) sp[(8 * (r >> 2) + 4 * hi + (r & 3)) * 33 + l32] = sc[r];
        }
        __syncthreads();
        {   // 2. full scores of 4 keys of row rr, mask, running maximum and sum, weights
            float s[4];
            float mx = -INFINITY;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int jj = rc + x, j = lo + u0 + jj;
                float v = Sp[rr * 33 + jj] + Sp[(AS_T + rr) * 33 + jj] + Sp[(2 * AS_T + rr) * 33 + jj] + Sp[(3 * AS_T + rr) * 33 + jj];
                const bool ok = r_ok && jj < nk && j <= r_i && r_i - j < window;
                s[x] = ok ? v * a.scale : -INFINITY;
                mx = fmaxf(mx, s[x]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
            const float m_new = fmaxf(m_run, mx);
            float alpha = 1.0f, sum = 0.f;
            short pw[4] = {0, 0, 0, 0};
            if (m_new > -INFINITY) {
                alpha = __expf(m_run - m_new);                      // m_run = -inf: 0, and nothing has been accumulated yet
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const float p = __expf(s[x] - m_new);           // masked: exp(-inf) = 0
                    pw[x] = as_bf16(p);
                    sum += p;
                }
            }
            sum += __shfl_xor(sum, 1, 64);
            sum += __shfl_xor(sum, 2, 64);
            sum += __shfl_xor(sum, 4, 64);
            l_run = l_run * alpha + sum;
            m_run = m_new;
            *(as_bf16x4 *)(Pb + rr * AS_PROW + rc) = (as_bf16x4){pw[0], pw[1], pw[2], pw[3]};
            if ((tid & 7) == 0) alphaS[rr] = alpha;
        }
        __syncthreads();
        {   // 3. rescale, then weights x this wavefront's value columns
            float al[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) al[r] = alphaS[8 * (r >> 2) + 4 * hi + (r & 3)];
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][r] *= al[r];
#pragma unroll
            for (int sK = 0; sK < AS_T / 8; ++sK) {
                const int j0 = 8 * sK + 4 * hi;
                const as_bf16x4 wa = *(const as_bf16x4 *)(Pb + l32 * AS_PROW + j0);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const bf16_t *vp = Ks + j0 * KROW + wave * (32 * NT) + 32 * t + l32;
                    const as_bf16x4 vb = {(short)vp[0], (short)vp[KROW], (short)vp[2 * KROW], (short)vp[3 * KROW]};
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(wa, vb, acc[t], 0, 0, 0);
                }
            }
        }
    }
    if (S > 1) {                                                    // this share's rows: [Dv] unnormalised outputs, maximum, sum
        float *part = a.scratch + (((int64_t)split * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * AS_T * (int64_t)(Dv + 2);
        if ((tid & 7) == 0) { part[rr * (Dv + 2) + Dv] = m_run; part[rr * (Dv + 2) + Dv + 1] = l_run; }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * hi + (r & 3);
#pragma unroll
            for (int t = 0; t < NT; ++t) part[row * (Dv + 2) + wave * (32 * NT) + 32 * t + l32] = acc[t][r];
        }
        return;
    }
    if ((tid & 7) == 0) lS[rr] = l_run > 0.f ? 1.0f / l_run : 0.f;
    __syncthreads();
    bf16_t *out = (bf16_t *)a.out;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * hi + (r & 3);
        const int ii = row / HF, hh = h0 + row % HF;
        if (row >= TQ * HF || ii >= cnt || hh >= H) continue;
        const float inv = lS[row];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            st_f(out + ((int64_t)(row0 + ii) * H + hh) * Dv + wave * (32 * NT) + 32 * t + l32, acc[t][r] * inv);
    }
}

// out[row] = sum_s part_s[row] * exp(m_s - M) / sum_s l_s * exp(m_s - M), in share order
__global__ __launch_bounds__(256) void attn_shared_join_kernel(jl_attn_args a, int HF, int TQ) {
    __shared__ float wS[AS_T * 64];                                 // [32][S] weight of every share of a row
    const int H = a.H, Dv = a.Dv, S = a.splits, tid = threadIdx.x;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int cnt = tile[2], row0 = tile[3], h0 = blockIdx.y * HF;
    if (tile[0] < 0 || cnt <= 0) return;
    const int64_t share = (int64_t)gridDim.x * gridDim.y * AS_T * (Dv + 2);
    const float *base = a.scratch + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * AS_T * (int64_t)(Dv + 2);
    if (tid < AS_T) {
        float M = -INFINITY, L = 0.f;
        for (int sp = 0; sp < S; ++sp) M = fmaxf(M, base[sp * share + tid * (Dv + 2) + Dv]);
        for (int sp = 0; sp < S; ++sp) {
            const float m = base[sp * share + tid * (Dv + 2) + Dv];
            const float w = m > -INFINITY ? __expf(m - M) : 0.f;
            wS[tid * 64 + sp] = w;
            L += w * base[sp * share + tid * (Dv + 2) + Dv + 1];
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        for (int sp = 0; sp < S; ++sp) wS[tid * 64 + sp] *= inv;
    }
    __syncthreads();
    bf16_t *out = (bf16_t *)a.out;
    for (int e = tid; e < AS_T * Dv; e += 256) {
        const int row = e / Dv, col = e - row * Dv, ii = row / HF, hh = h0 + row % HF;
        if (row >= TQ * HF || ii >= cnt || hh >= H) continue;
        float v = 0.f;
        for (int sp = 0; sp < S; ++sp) v += wS[row * 64 + sp] * base[sp * share + row * (Dv + 2) + col];
        st_f(out + ((int64_t)(row0 + ii) * H + hh) * Dv + col, v);
    }
}

extern "C" int64_t jl_attn_shared_kv_scratch_floats(int32_t n_tiles, int32_t H, int32_t Dv, int32_t splits) {
    const int hf = H < AS_T ? H : AS_T;
    return splits > 1 ? (int64_t)splits * n_tiles * ((H + hf - 1) / hf) * AS_T * (Dv + 2) : 0;
}

static bool as_fits(int dtype, int H, int G, int D, int Dv, int64_t k_ld) {
    return dtype == JL_BF16 && G == 1 && H >= 1 && D % 8 == 0 && D <= 8 * AS_WAVES * AS_QSTEPS && Dv % 128 == 0 && Dv >= 128 && Dv <= 512 && Dv <= D &&
           k_ld % 4 == 0;
}

extern "C" int jl_attn_shared_kv_tile_rows(int dtype, int32_t H, int32_t D, int32_t Dv, int64_t k_ld) {
    if (!as_fits(dtype, H, 1, D, Dv, k_ld)) return 0;
    const int hf = H < AS_T ? H : AS_T;
    return AS_T / hf;
}

extern "C" int jl_attn_shared_kv(const jl_attn_args *ap, void *stream) {
    if (!ap) return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: null arguments");
    jl_attn_args a = *ap;
    if (a.n_tiles <= 0) return JL_OK;
    if (!a.q || !a.k_cache || !a.out || !a.block_tables || !a.tiles) return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: null pointer");
    if (a.k_ld <= 0) a.k_ld = a.D;
    if (a.page_size <= 0 || a.k_ld < a.D || !as_fits(a.dtype, a.H, a.G, a.D, a.Dv, a.k_ld))
        return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: bfloat16, one key/value head, key width a multiple of 8 up to %d, value width 128 .. 512 in "
                       "multiples of 128 and at most the key width", 8 * AS_WAVES * AS_QSTEPS);
    if (a.v_cache && a.v_cache != a.k_cache) return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: the values are the first Dv columns of the key rows");
    const int hf = a.H < AS_T ? a.H : AS_T, tq = AS_T / hf;
    if (a.TQ != tq) return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: tiles of %d queries wanted (ask jl_attn_shared_kv_tile_rows)", tq);
    const size_t lds = as_lds_bytes(a.D);
    if (a.splits > 1 && (!a.scratch || a.splits > 64)) return jl_fail(JL_E_INVALID, "jl_attn_shared_kv: 2 .. 64 shares of the keys need a scratch");
    const dim3 grid((unsigned)a.n_tiles, (unsigned)((a.H + hf - 1) / hf), (unsigned)(a.splits > 1 ? a.splits : 1));
    hipStream_t st = (hipStream_t)stream;
#define AS_CASE(NTV)                                                                                                              \
    case NTV: {                                                                                                                   \
        auto kern = attn_shared_kv_kernel<NTV>;                                                                                   \
        if (lds > 64 * 1024) {                                                                                                    \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
            if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "jl_attn_shared_kv: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e)); \
        }                                                                                                                         \
        kern<<<grid, AS_THREADS, lds, st>>>(a, hf, tq);                                                                           \
        break;                                                                                                                    \
    }
    switch (a.Dv / 128) {
        AS_CASE(1) AS_CASE(2) AS_CASE(3) AS_CASE(4)
    }
#undef AS_CASE
    if (a.splits > 1) attn_shared_join_kernel<<<dim3(grid.x, grid.y), 256, 0, st>>>(a, hf, tq);
    return jl_check_launch("attn_shared_kv_kernel");
}
