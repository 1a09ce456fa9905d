// jl_attn.hip — query / key norm + paged append, and attention with a sliding window that keeps the first tokens, a bucketed
// distance bias and mixed heads, for prompt portions and single decoded tokens alike (one ragged launch).
#include "jl_common.h"

// ---- whole-projection q / k norm + append: one workgroup per token ------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_append_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
                                                              int HD, int GD, int GDv, const T *__restrict__ wq, const T *__restrict__ wk,
                                                              float eps, T *__restrict__ q_out, T *__restrict__ k_cache,
                                                              T *__restrict__ v_cache, const int64_t *__restrict__ slot) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const T *row = proj + n * ld;
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < HD; c += 256) { const float v = ld_f(row + q_col + c); sq += v * v; }
    for (int c = threadIdx.x; c < GD; c += 256) { const float v = ld_f(row + k_col + c); sk += v * v; }
    sq = block_sum_f32(sq, red);
    sk = block_sum_f32(sk, red);
    const float rq = 1.0f / sqrtf(sq / (float)HD + eps), rk = 1.0f / sqrtf(sk / (float)GD + eps);
    for (int c = threadIdx.x; c < HD; c += 256) st_f(q_out + n * HD + c, ld_f(row + q_col + c) * rq * ld_f(wq + c));
    const int64_t sl = slot[n];
    if (sl < 0) return;
    for (int c = threadIdx.x; c < GD; c += 256) st_f(k_cache + sl * GD + c, ld_f(row + k_col + c) * rk * ld_f(wk + c));
    for (int c = threadIdx.x; c < GDv; c += 256) v_cache[sl * GDv + c] = row[v_col + c];
}

extern "C" int jl_qk_norm_append(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col,
                                 int32_t H, int32_t G, int32_t D, int32_t Dv, const void *wq, const void *wk, float eps, void *q_out,
                                 void *k_cache, void *v_cache, const int64_t *slot, void *stream) {
    if (N <= 0) return JL_OK;
    if (!proj || !wq || !wk || !q_out || !k_cache || !v_cache || !slot) return jl_fail(JL_E_INVALID, "jl_qk_norm_append: null pointer");
    if (H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || q_col + H * D > ld || k_col + G * D > ld || v_col + G * Dv > ld)
        return jl_fail(JL_E_INVALID, "jl_qk_norm_append: columns do not fit the row stride");
    JL_DISPATCH(dtype, qk_norm_append_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(
                           (const T *)proj, ld, q_col, k_col, v_col, H * D, G * D, G * Dv, (const T *)wq, (const T *)wk, eps, (T *)q_out,
                           (T *)k_cache, (T *)v_cache, slot));
    return jl_check_launch("qk_norm_append_kernel");
}

// ---- attention ---------------------------------------------------------------------------------------------------------------
// One workgroup per tile of up to TQ consecutive query rows of one request, all heads (mixing the heads needs every head's
// weight of a (query, key) pair in one place).  Two sweeps over the visible keys, TK keys at a time through LDS:
//   sweep 1: scores -> running maximum and sum per (head, query);
//   sweep 2: scores again -> normalised weights -> mixed over the heads -> times the values.
// The visible keys of a tile are the kept first tokens below the window's lowest key and the window's own range; the exact
// mask is applied per (query, key).
constexpr int ATT_THREADS = 256;
constexpr int ATT_LDS_BUDGET = 144 * 1024;

struct AttShape { int TQ, TK, ACC; size_t lds; };

static bool att_shape(int H, int G, int D, int Dv, int tq_want, AttShape *o) {
    const int per_row = H * Dv;
    int acc = 16;                                       // accumulators per thread: 16 (one query row of up to 4096 outputs) or 64
    if (per_row > acc * ATT_THREADS) acc = 64;
    if (per_row > acc * ATT_THREADS) return false;
    int tq = acc * ATT_THREADS / per_row;
    if (tq > 16) tq = 16;
    if (tq_want > 0 && tq > tq_want) tq = tq_want;
    const int kvw = (D + 1 > Dv ? D + 1 : Dv) * G;
    for (; tq >= 1; tq = tq > 1 ? tq / 2 : 0) {
        for (int tk = 64; tk >= 4; tk /= 2) {
            const size_t fl = (size_t)tq * H * D + (size_t)tk * kvw + 2 * (size_t)H * tq * tk + 2 * (size_t)H * tq + (size_t)H * H + 64;
            if (fl * 4 <= (size_t)ATT_LDS_BUDGET) { o->TQ = tq; o->TK = tk; o->ACC = acc; o->lds = fl * 4; return true; }
        }
        if (tq == 1) break;
    }
    return false;
}

extern "C" int jl_attn_tile_rows(int32_t H, int32_t G, int32_t D, int32_t Dv) {
    AttShape s;
    return att_shape(H, G, D, Dv, 0, &s) ? s.TQ : 0;
}

template <typename T, int ACC>
__global__ __launch_bounds__(ATT_THREADS) void attn_window_kernel(jl_attn_args a, int TK) {
    extern __shared__ float lds[];
    const int H = a.H, G = a.G, D = a.D, Dv = a.Dv, TQ = a.TQ, rep = H / G;
    const int tid = threadIdx.x;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    const int kstride = D + 1;
    const int kvw = (kstride > Dv ? kstride : Dv) * G;
    float *Qs = lds;                                    // [TQ][H][D]
    float *KV = Qs + TQ * H * D;                        // [G][TK][D+1] keys (odd row stride: no bank conflicts over the keys), then [TK][G][Dv] values
    float *S = KV + TK * kvw;                           // [H][TQ][TK]
    float *Wm = S + H * TQ * TK;                        // [H][TQ][TK]
    float *mx = Wm + H * TQ * TK;                       // [H][TQ]
    float *sm = mx + H * TQ;                            // [H][TQ]
    float *talk = sm + H * TQ;                          // [H][H]
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int kf_end = a.keep_first < lo ? a.keep_first : lo;
    const int n_keys = kf_end + (i_max + 1 - lo);
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const T *q = (const T *)a.q;
    const T *kc = (const T *)a.k_cache;
    const T *vc = (const T *)a.v_cache;

    for (int e = tid; e < cnt * H * D; e += ATT_THREADS) Qs[e] = ld_f(q + (int64_t)row0 * H * D + e);
    for (int e = tid; e < H * TQ; e += ATT_THREADS) { mx[e] = -INFINITY; sm[e] = 0.f; }
    if (a.talk) for (int e = tid; e < H * H; e += ATT_THREADS) talk[e] = a.talk[e];

    float acc[ACC];
#pragma unroll
    for (int x = 0; x < ACC; ++x) acc[x] = 0.f;

    for (int sweep = 0; sweep < 2; ++sweep) {
        for (int u0 = 0; u0 < n_keys; u0 += TK) {
            const int nk = n_keys - u0 < TK ? n_keys - u0 : TK;
            __syncthreads();                                        // the previous tile's readers are done with KV / S / Wm
            for (int e = tid; e < nk * G * D; e += ATT_THREADS) {
                const int jj = e / (G * D), r = e - jj * (G * D), c = r / D, d = r - c * D;
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                const int64_t tok = (int64_t)bt[j / a.page_size] * a.page_size + j % a.page_size;
                KV[(c * TK + jj) * kstride + d] = ld_f(kc + tok * (G * D) + r);
            }
            __syncthreads();
            for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                const int g = e / (cnt * nk), r = e - g * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end), i = i0 + ii;
                float s = -INFINITY;
                if (j <= i && (i - j < window || j < a.keep_first)) {
                    const float *qp = Qs + (ii * H + g) * D, *kp = KV + ((g / rep) * TK + jj) * kstride;
                    float dot = 0.f;
                    for (int d = 0; d < D; ++d) dot += qp[d] * kp[d];
                    s = dot * a.scale;
                    if (a.rel) {
                        const int n = i - j < a.lut_len ? i - j : a.lut_len - 1;
                        s += a.rel[a.lut[n] * H + g];
                    }
                }
                S[(g * TQ + ii) * TK + jj] = s;
            }
            __syncthreads();
            if (sweep == 0) {
                for (int e = tid; e < H * cnt; e += ATT_THREADS) {
                    const int g = e / cnt, ii = e - g * cnt;
                    const float *sp = S + (g * TQ + ii) * TK;
                    float m = mx[g * TQ + ii], l = sm[g * TQ + ii], t = m;
                    for (int jj = 0; jj < nk; ++jj) t = fmaxf(t, sp[jj]);
                    if (t > -INFINITY) {
                        l = l * __expf(m - t);                       // m = -inf: l is 0 and stays 0
                        for (int jj = 0; jj < nk; ++jj) l += expf(sp[jj] - t);
                        mx[g * TQ + ii] = t;
                        sm[g * TQ + ii] = l;
                    }
                }
                continue;
            }
            for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                const int g = e / (cnt * nk), r = e - g * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                const int o = (g * TQ + ii) * TK + jj;
                S[o] = expf(S[o] - mx[g * TQ + ii]) / sm[g * TQ + ii];
            }
            for (int e = tid; e < nk * G * Dv; e += ATT_THREADS) {   // keys are no longer read: the values take their place
                const int jj = e / (G * Dv), r = e - jj * (G * Dv);
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                const int64_t tok = (int64_t)bt[j / a.page_size] * a.page_size + j % a.page_size;
                KV[jj * (G * Dv) + r] = ld_f(vc + tok * (G * Dv) + r);
            }
            __syncthreads();
            const float *Wp = S;
            if (a.talk) {
                for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                    const int h = e / (cnt * nk), r = e - h * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                    float w = 0.f;
                    for (int g = 0; g < H; ++g) w += talk[h * H + g] * S[(g * TQ + ii) * TK + jj];
                    Wm[(h * TQ + ii) * TK + jj] = w;
                }
                __syncthreads();
                Wp = Wm;
            }
#pragma unroll
            for (int x = 0; x < ACC; ++x) {
                const int e = x * ATT_THREADS + tid;
                if (e < cnt * H * Dv) {
                    const int ii = e / (H * Dv), r = e - ii * (H * Dv), h = r / Dv, d = r - h * Dv;
                    const float *wp = Wp + (h * TQ + ii) * TK, *vp = KV + (h / rep) * Dv + d;
                    float s = acc[x];
                    for (int jj = 0; jj < nk; ++jj) s += wp[jj] * vp[jj * (G * Dv)];
                    acc[x] = s;
                }
            }
        }
    }
    T *out = (T *)a.out;
    const T *gate = (const T *)a.gate;
#pragma unroll
    for (int x = 0; x < ACC; ++x) {
        const int e = x * ATT_THREADS + tid;
        if (e < cnt * H * Dv) {
            const int ii = e / (H * Dv), r = e - ii * (H * Dv);
            float v = acc[x];
            if (gate) v *= 1.0f / (1.0f + expf(-ld_f(gate + (int64_t)(row0 + ii) * a.gate_ld + r)));
            st_f(out + (int64_t)(row0 + ii) * (H * Dv) + r, v);
        }
    }
}

template <typename T, int ACC> static int att_launch(const jl_attn_args &a, const AttShape &s, hipStream_t st) {
    auto kern = attn_window_kernel<T, ACC>;
    if (s.lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)s.lds);
        if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "jl_attn_window: cannot get %zu bytes of LDS: %s", s.lds, hipGetErrorString(e));
    }
    kern<<<dim3((unsigned)a.n_tiles), ATT_THREADS, s.lds, st>>>(a, s.TK);
    return jl_check_launch("attn_window_kernel");
}

extern "C" int jl_attn_window(const jl_attn_args *ap, void *stream) {
    if (!ap) return jl_fail(JL_E_INVALID, "jl_attn_window: null arguments");
    jl_attn_args a = *ap;
    if (a.n_tiles <= 0) return JL_OK;
    if (!a.q || !a.k_cache || !a.v_cache || !a.out || !a.block_tables || !a.tiles) return jl_fail(JL_E_INVALID, "jl_attn_window: null pointer");
    if (a.H <= 0 || a.G <= 0 || a.H % a.G || a.D <= 0 || a.Dv <= 0 || a.page_size <= 0 || a.TQ <= 0)
        return jl_fail(JL_E_INVALID, "jl_attn_window: bad head counts or sizes");
    if ((a.rel != nullptr) != (a.lut != nullptr) || (a.lut && a.lut_len <= 0)) return jl_fail(JL_E_INVALID, "jl_attn_window: rel and lut come together");
    AttShape s;
    if (!att_shape(a.H, a.G, a.D, a.Dv, a.TQ, &s) || s.TQ != a.TQ)
        return jl_fail(JL_E_INVALID, "jl_attn_window: TQ %d does not fit these sizes (ask jl_attn_tile_rows)", a.TQ);
    hipStream_t st = (hipStream_t)stream;
#define ATT_CASE(N) case N: JL_DISPATCH(a.dtype, return (att_launch<T, N>(a, s, st))); break
    switch (s.ACC) {
        ATT_CASE(16);
        ATT_CASE(64);
    }
#undef ATT_CASE
    return jl_fail(JL_E_INVALID, "jl_attn_window: unsupported size");
}
