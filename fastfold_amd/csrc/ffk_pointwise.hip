// Point-wise attention over a short axis (see ffk_pointwise_attention_core in include/ffk.h):
// every one of P positions has its own query q[p, h, :] and T (<= 8) key / value rows kv[t, p, ...];
//     w[p, h, t] = softmax_t( q[p, h, :] . k[t, p, h, :] + bias[t] ),   o[p, h, :] = scale * sum_t w[p, h, t] v[t, p, h, :].
// The op is a stream: each element is read once, so one thread owns one (position, head) pair, keeps its
// D-element query and the T logits in registers and walks the T key and value rows with 16-byte loads;
// neighbouring threads read neighbouring 2 D-byte pieces of a row.
#include "ffk_common.h"

namespace {

constexpr int PW_THREADS = 256;
constexpr int PW_MAXT = 8;

template <typename T, int D>
__global__ __launch_bounds__(PW_THREADS) void pointwise_attention_kernel(T* __restrict__ o, const T* __restrict__ q,
                                                                         const T* __restrict__ kv,
                                                                         const float* __restrict__ bias,
                                                                         const float* __restrict__ out_scale, long P, int H,
                                                                         int NT, long kv_st, long kv_sp, int v_off) {
    constexpr int VEC = DT<T>::VEC;
    constexpr int NV = D / VEC;                       // 16-byte vectors per head slice
    const long idx = (long)blockIdx.x * PW_THREADS + threadIdx.x;
    if (idx >= P * H) return;
    const long p = idx / H;
    const int h = (int)(idx - p * H);
    float qf[D];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const Vec16<T> v = ld16(q + p * ((long)H * D) + h * D + i * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) qf[i * VEC + e] = DT<T>::to_f(v.e[e]);
    }
    float logit[PW_MAXT];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < PW_MAXT; ++t) {
        logit[t] = -INFINITY;
        if (t < NT) {
            const T* kr = kv + t * kv_st + p * kv_sp + h * D;
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const Vec16<T> v = ld16(kr + i * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) s += qf[i * VEC + e] * DT<T>::to_f(v.e[e]);
            }
            logit[t] = s + bias[t];
            mx = fmaxf(mx, logit[t]);
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < PW_MAXT; ++t) {
        logit[t] = t < NT ? __expf(logit[t] - mx) : 0.0f;
        sum += logit[t];
    }
    const float inv = (out_scale ? *out_scale : 1.0f) / sum;      // the optional device scalar rides on the normaliser
    float acc[D];
#pragma unroll
    for (int j = 0; j < D; ++j) acc[j] = 0.0f;
#pragma unroll
    for (int t = 0; t < PW_MAXT; ++t) {
        if (t < NT) {
            const T* vr = kv + t * kv_st + p * kv_sp + v_off + h * D;
            const float w = logit[t] * inv;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const Vec16<T> v = ld16(vr + i * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[i * VEC + e] += w * DT<T>::to_f(v.e[e]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        Vec16<T> v;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v.e[e] = DT<T>::from_f(acc[i * VEC + e]);
        st16(o + p * ((long)H * D) + h * D + i * VEC, v);
    }
}

template <typename T>
int pw_launch(void* o, const void* q, const void* kv, const float* bias, const float* out_scale, long P, int H, int D,
              int NT, long kv_st, long kv_sp, int v_off, hipStream_t st) {
    const long total = P * H;
    const unsigned grid = (unsigned)ffk_cdiv(total, PW_THREADS);
#define PW_CASE(DD)                                                                                                    \
    case DD:                                                                                                           \
        pointwise_attention_kernel<T, DD><<<grid, PW_THREADS, 0, st>>>((T*)o, (const T*)q, (const T*)kv, bias, out_scale, P, \
                                                                       H, NT, kv_st, kv_sp, v_off);                           \
        break;
    switch (D) {
        PW_CASE(8)
        PW_CASE(16)
        PW_CASE(32)
        default: return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_pointwise_attention_core: head width %d (8, 16 or 32)", D);
    }
#undef PW_CASE
    return ffk_check_launch("ffk_pointwise_attention_core");
}

}  // namespace

extern "C" int ffk_pointwise_attention_core(void* o, const void* q, const void* kv, const float* bias, const float* out_scale,
                                            int64_t P, int64_t H, int64_t D, int64_t NT, int64_t kv_st, int64_t kv_sp,
                                            int64_t v_off, int dtype, void* stream) {
    FFK_REQUIRE(o && q && kv && bias, FFK_ERR_NULL, "ffk_pointwise_attention_core: null pointer");
    FFK_REQUIRE(P > 0 && H > 0 && H <= 64 && NT > 0 && NT <= PW_MAXT && P * H < (1L << 31) * (long)PW_THREADS, FFK_ERR_SHAPE,
                "ffk_pointwise_attention_core: bad shape P=%ld H=%ld NT=%ld (1 <= NT <= %d)", (long)P, (long)H, (long)NT,
                PW_MAXT);
    FFK_REQUIRE(D == 8 || D == 16 || D == 32, FFK_ERR_UNSUPPORTED, "ffk_pointwise_attention_core: head width %ld (8, 16 or 32)",
                (long)D);
    FFK_REQUIRE(dtype == FFK_BF16 || dtype == FFK_F32, FFK_ERR_DTYPE, "ffk_pointwise_attention_core: unsupported dtype tag %d",
                dtype);
    const long vec = dtype == FFK_F32 ? 4 : 8;
    FFK_REQUIRE(ffk_aligned16(o) && ffk_aligned16(q) && ffk_aligned16(kv) && kv_st % vec == 0 && kv_sp % vec == 0 &&
                    v_off % vec == 0 && D % vec == 0,
                FFK_ERR_ALIGN, "ffk_pointwise_attention_core: buffers and strides must keep 16-byte alignment");
    FFK_REQUIRE(kv_sp >= v_off + H * D && v_off >= H * D, FFK_ERR_SHAPE,
                "ffk_pointwise_attention_core: a key / value row needs v_off >= H*D and kv_sp >= v_off + H*D");
    hipStream_t st = (hipStream_t)stream;
    if (dtype == FFK_BF16)
        return pw_launch<bf16_t>(o, q, kv, bias, out_scale, (long)P, (int)H, (int)D, (int)NT, (long)kv_st, (long)kv_sp, (int)v_off, st);
    return pw_launch<float>(o, q, kv, bias, out_scale, (long)P, (int)H, (int)D, (int)NT, (long)kv_st, (long)kv_sp, (int)v_off, st);
}
