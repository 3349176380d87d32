// Global column attention core of the extra-MSA stack (gfx950).
//
// For every residue column j of m [S, R, C] there is ONE query (the masked mean of the normalised
// rows of the column) and one key / value head of width D shared by the H query heads
// (reference: GlobalAttention.forward, fastfold/model/fastnn/ops.py:1179-1203):
//     x_s   = LayerNorm(m[s, j, :])
//     qbar  = sum_s mask[s, j] x_s / (sum_s mask[s, j] + eps)
//     q[h]  = scaling * Wq[h] qbar,  k_s = Wk x_s,  v_s = Wv x_s
//     w[h, s] = softmax_s(q[h] . k_s,  masked keys replaced by -1e9)
//     o[j, h, :] = sum_s w[h, s] v_s
// Neither k nor v is ever formed per row: q[h] . (Wk x_s) = (Wk^T q[h]) . x_s =: u[h] . x_s and
// sum_s w[h, s] Wv x_s = Wv (sum_s w[h, s] x_s), so a row costs H dot products and H scaled
// accumulations of its C normalised channels, all in fp32 on the vector ALU, and the two small
// matrices are applied once per column.  The kernel is bound by reading m twice (once for the mean
// query, once for the softmax pass; the second read comes from the memory-side cache).
//
// One workgroup of 256 threads per column.  A row of C channels is held by C / 8 adjacent lanes
// (8 channels each, one 16-byte load for bf16); the 256 / (C / 8) lane groups of the workgroup walk
// the rows of the column with stride, four rows in flight per group, each group keeping its own
// running softmax state, merged at the end (within a wave by shuffles, across waves through LDS).
#include "ffk_common.h"

#include <math.h>

namespace {

constexpr int GA_THREADS = 256;
constexpr int GA_HMAX = 8;       // query heads held in registers
constexpr int GA_UNR = 4;        // rows in flight per lane group
constexpr int GA_QMAX = 128;     // H * D

template <typename T> __device__ __forceinline__ void ga_load8(const T* p, float* x);
template <> __device__ __forceinline__ void ga_load8<bf16_t>(const bf16_t* p, float* x) {
    const Vec16<bf16_t> v = ld16(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)v.e[e];
}
template <> __device__ __forceinline__ void ga_load8<float>(const float* p, float* x) {
    const Vec16<float> a = ld16(p), b = ld16(p + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        x[e] = a.e[e];
        x[4 + e] = b.e[e];
    }
}

template <typename T, int C>
__global__ __launch_bounds__(GA_THREADS) void global_attention_kernel(
    T* __restrict__ o, const T* __restrict__ m, const T* __restrict__ mask, const T* __restrict__ gamma,
    const T* __restrict__ beta, float ln_eps, const T* __restrict__ wq, const T* __restrict__ wk,
    const T* __restrict__ wv, int S, int R, int H, int D, float scaling, float eps, long m_ss, long m_sr,
    long k_ss, long k_sr) {
    constexpr int LPR = C / 8;                 // lanes per row
    constexpr int G = GA_THREADS / LPR;        // lane groups per workgroup
    constexpr int NW = GA_THREADS / 64;
    __shared__ float s_part[G][C];             // phase A partial sums; reused for the per-wave y
    __shared__ float s_cnt[G];
    __shared__ float s_qavg[C];
    __shared__ float s_q[GA_QMAX];
    __shared__ float s_u[GA_HMAX][C];
    __shared__ float s_mx[NW][GA_HMAX], s_sm[NW][GA_HMAX];
    __shared__ float s_y[NW][GA_HMAX][C];

    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    const int g = tid / LPR;
    const int c0 = (tid % LPR) * 8;
    const int HD = H * D;

    float gm[8], bt[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        gm[e] = gamma ? DT<T>::to_f(gamma[c0 + e]) : 1.0f;
        bt[e] = gamma ? DT<T>::to_f(beta[c0 + e]) : 0.0f;
    }
    const T* col = m + (long)j * m_sr + c0;
    const long row_stride = m_ss;

    // normalised channels of one row, in place (gamma == NULL: the rows are used as they are)
    auto layer_norm = [&](float* x) {
        if (!gamma) return;
        float s1 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s1 += x[e];
        const float mean = group_sum(s1, LPR) * (1.0f / C);
        float s2 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] -= mean;
            s2 += x[e] * x[e];
        }
        const float rstd = rsqrtf(group_sum(s2, LPR) * (1.0f / C) + ln_eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = x[e] * rstd * gm[e] + bt[e];
    };
    // rows s0 + u * G + g, u = 0..UNR-1: loads issued together; rows past the end are clamped and flagged
    auto load_rows = [&](int s0, float (*x)[8], float* mk, bool* valid) {
#pragma unroll
        for (int u = 0; u < GA_UNR; ++u) {
            const int s = s0 + u * G + g;
            valid[u] = s < S;
            const int sc = valid[u] ? s : S - 1;
            ga_load8<T>(col + sc * row_stride, x[u]);
            mk[u] = mask ? DT<T>::to_f(mask[(long)sc * k_ss + (long)j * k_sr]) : 1.0f;
        }
    };

    // ---- phase A: masked mean of the normalised rows -> query -> u[h] = Wk^T q[h]
    {
        float acc[8], cnt = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        for (int s0 = 0; s0 < S; s0 += G * GA_UNR) {
            float x[GA_UNR][8], mk[GA_UNR];
            bool valid[GA_UNR];
            load_rows(s0, x, mk, valid);
#pragma unroll
            for (int u = 0; u < GA_UNR; ++u) {
                layer_norm(x[u]);
                const float w = valid[u] ? mk[u] : 0.f;
                cnt += w;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] += w * x[u][e];
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) s_part[g][c0 + e] = acc[e];
        if (c0 == 0) s_cnt[g] = cnt;
    }
    __syncthreads();
    if (tid < C) {
        float a = 0.f, n = 0.f;
        for (int gg = 0; gg < G; ++gg) {
            a += s_part[gg][tid];
            n += s_cnt[gg];
        }
        s_qavg[tid] = a / (n + eps);
    }
    __syncthreads();
    if (tid < HD) {
        const T* w = wq + (long)tid * C;
        float a = 0.f;
        for (int c = 0; c < C; ++c) a += DT<T>::to_f(w[c]) * s_qavg[c];
        s_q[tid] = a * scaling;
    }
    __syncthreads();
    for (int idx = tid; idx < GA_HMAX * C; idx += GA_THREADS) {
        const int h = idx / C, c = idx % C;
        float a = 0.f;
        if (h < H)
            for (int d = 0; d < D; ++d) a += s_q[h * D + d] * DT<T>::to_f(wk[(long)d * C + c]);
        s_u[h][c] = a;
    }
    __syncthreads();

    // ---- phase B: one softmax pass over the rows with a running maximum per lane group
    float ur[GA_HMAX][8], y[GA_HMAX][8], mx[GA_HMAX], sm[GA_HMAX];
#pragma unroll
    for (int h = 0; h < GA_HMAX; ++h) {
        mx[h] = -INFINITY;
        sm[h] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            ur[h][e] = s_u[h][c0 + e];
            y[h][e] = 0.f;
        }
    }
    for (int s0 = 0; s0 < S; s0 += G * GA_UNR) {
        float x[GA_UNR][8], mk[GA_UNR];
        bool valid[GA_UNR];
        load_rows(s0, x, mk, valid);
#pragma unroll
        for (int u = 0; u < GA_UNR; ++u) {
            layer_norm(x[u]);
            float l[GA_HMAX];
#pragma unroll
            for (int h = 0; h < GA_HMAX; ++h) {
                float a = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) a += ur[h][e] * x[u][e];
                l[h] = group_sum(a, LPR);
            }
            if (valid[u]) {
                const bool keep = mk[u] != 0.f;
#pragma unroll
                for (int h = 0; h < GA_HMAX; ++h) {
                    const float lv = keep ? l[h] : -1e9f;
                    const float mnew = fmaxf(mx[h], lv);
                    const float sc = exp_for<T>(mx[h] - mnew);
                    const float p = exp_for<T>(lv - mnew);
                    mx[h] = mnew;
                    sm[h] = sm[h] * sc + p;
#pragma unroll
                    for (int e = 0; e < 8; ++e) y[h][e] = y[h][e] * sc + p * x[u][e];
                }
            }
        }
    }
    // merge the lane groups of a wave (same channel slice, lane distance LPR, 2 LPR, ...)
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
        for (int h = 0; h < GA_HMAX; ++h) {
            const float omx = __shfl_xor(mx[h], off, 64), osm = __shfl_xor(sm[h], off, 64);
            const float mnew = fmaxf(mx[h], omx);
            const float a = mx[h] == -INFINITY ? 0.f : exp_for<T>(mx[h] - mnew);
            const float b = omx == -INFINITY ? 0.f : exp_for<T>(omx - mnew);
            mx[h] = mnew;
            sm[h] = sm[h] * a + osm * b;
#pragma unroll
            for (int e = 0; e < 8; ++e) y[h][e] = y[h][e] * a + __shfl_xor(y[h][e], off, 64) * b;
        }
    }
    const int wave = tid >> 6, lane = tid & 63;
    if (lane < LPR) {
#pragma unroll
        for (int h = 0; h < GA_HMAX; ++h) {
            if (lane == 0) {
                s_mx[wave][h] = mx[h];
                s_sm[wave][h] = sm[h];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) s_y[wave][h][c0 + e] = y[h][e];
        }
    }
    __syncthreads();
    // across waves: ybar[h][c] = sum_s w[h, s] x_s[c], kept in s_u
    for (int idx = tid; idx < GA_HMAX * C; idx += GA_THREADS) {
        const int h = idx / C, c = idx % C;
        float mm = -INFINITY;
        for (int w = 0; w < NW; ++w) mm = fmaxf(mm, s_mx[w][h]);
        float num = 0.f, den = 0.f;
        for (int w = 0; w < NW; ++w) {
            const float a = s_mx[w][h] == -INFINITY ? 0.f : exp_for<T>(s_mx[w][h] - mm);
            num += a * s_y[w][h][c];
            den += a * s_sm[w][h];
        }
        s_u[h][c] = den > 0.f ? num / den : 0.f;
    }
    __syncthreads();
    if (tid < HD) {
        const int h = tid / D, d = tid % D;
        const T* w = wv + (long)d * C;
        float a = 0.f;
        for (int c = 0; c < C; ++c) a += DT<T>::to_f(w[c]) * s_u[h][c];
        o[(long)j * HD + tid] = DT<T>::from_f(a);
    }
}

template <typename T>
int ga_launch(void* o, const void* m, const void* mask, const void* gamma, const void* beta, float ln_eps,
              const void* wq, const void* wk, const void* wv, int64_t S, int64_t R, int64_t C, int H, int D,
              float scaling, float eps, long m_ss, long m_sr, long k_ss, long k_sr, hipStream_t st) {
#define GA_CASE(CC)                                                                                          \
    case CC:                                                                                                 \
        hipLaunchKernelGGL((global_attention_kernel<T, CC>), dim3((unsigned)R), dim3(GA_THREADS), 0, st,      \
                           (T*)o, (const T*)m, (const T*)mask, (const T*)gamma, (const T*)beta, ln_eps,      \
                           (const T*)wq, (const T*)wk, (const T*)wv, (int)S, (int)R, H, D, scaling, eps,     \
                           m_ss, m_sr, k_ss, k_sr);                                                          \
        break;
    switch (C) {
        GA_CASE(32)
        GA_CASE(64)
        GA_CASE(128)
        default:
            return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_global_attention_core: C must be 32, 64 or 128 (got %ld)", (long)C);
    }
#undef GA_CASE
    return ffk_check_launch("ffk_global_attention_core");
}

}  // namespace

extern "C" int ffk_global_attention_core(void* o, const void* m, const void* mask, const void* ln_gamma,
                                         const void* ln_beta, float ln_eps, const void* wq, const void* wk,
                                         const void* wv, int64_t S, int64_t R, int64_t C, int64_t H, int64_t D,
                                         int64_t m_ss, int64_t m_sr, int64_t mask_ss, int64_t mask_sr,
                                         float scaling, float eps, int dtype, void* stream) {
    FFK_REQUIRE(o && m && wq && wk && wv, FFK_ERR_NULL, "ffk_global_attention_core: null pointer");
    FFK_REQUIRE(!ln_gamma == !ln_beta, FFK_ERR_NULL, "ffk_global_attention_core: ln_gamma and ln_beta go together");
    FFK_REQUIRE(S >= 0 && R >= 0, FFK_ERR_SHAPE, "ffk_global_attention_core: negative size");
    if (S == 0 || R == 0) return FFK_OK;
    FFK_REQUIRE(S * R < (1LL << 31) / 4 && R < (1LL << 31) / 128, FFK_ERR_SHAPE,
                "ffk_global_attention_core: S * R = %ld is beyond the kernel's 32-bit row arithmetic", (long)(S * R));
    FFK_REQUIRE(H >= 1 && H <= GA_HMAX && D >= 1 && H * D <= GA_QMAX, FFK_ERR_SHAPE,
                "ffk_global_attention_core: needs 1 <= H <= %d and H * D <= %d (got H=%ld, D=%ld)", GA_HMAX, GA_QMAX,
                (long)H, (long)D);
    const int64_t es = dtype == FFK_F32 ? 4 : 2;
    FFK_REQUIRE(ffk_aligned16(m) && (m_ss * es) % 16 == 0 && (m_sr * es) % 16 == 0, FFK_ERR_ALIGN,
                "ffk_global_attention_core: m and its strides must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_F32:
            return ga_launch<float>(o, m, mask, ln_gamma, ln_beta, ln_eps, wq, wk, wv, S, R, C, (int)H, (int)D, scaling, eps,
                                    m_ss, m_sr, mask_ss, mask_sr, st);
        case FFK_BF16:
            return ga_launch<bf16_t>(o, m, mask, ln_gamma, ln_beta, ln_eps, wq, wk, wv, S, R, C, (int)H, (int)D, scaling, eps,
                                     m_ss, m_sr, mask_ss, mask_sr, st);
        default:
            return ffk_fail(FFK_ERR_DTYPE, "ffk_global_attention_core: unsupported dtype tag %d", dtype);
    }
}
