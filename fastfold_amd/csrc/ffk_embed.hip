// Pair-representation embedding kernel (gfx950): the r x r x C part of the input embedder and of the
// recycling embedder (reference: InputEmbedder.forward, fastfold/model/fastnn/ops.py:1306-1324;
// RecyclingEmbedder.forward, ops.py:1108-1145).
//
//   out[i, j, :] = [LayerNorm(z[i, j, :])] + table[bin(i, j), :] + [bias] + [row[i, :]] + [col[j, :]]
//
// A linear layer applied to a one-hot vector is a pick of one column of its weight, so the
// [r, r, no_bins] one-hot tensor of the reference is never formed: the bin index is computed per pair
// (relative position, or squared distance between two coordinates against the squared bin edges) and
// the matching row of the transposed weight ("table") is added.  HBM-bound: one write (and, with z,
// one read) of r * r * C elements; the table, bias, row and column terms stay in cache.
//
// C / 8 adjacent lanes hold one pair (8 channels each, 16-byte accesses for bf16), so the LayerNorm
// reduction stays inside a lane group; a workgroup of 256 threads walks the pairs with a grid stride.
#include "ffk_common.h"

namespace {

constexpr int EM_THREADS = 256;

template <typename T> __device__ __forceinline__ void em_load8(const T* p, float* x);
template <> __device__ __forceinline__ void em_load8<bf16_t>(const bf16_t* p, float* x) {
    const Vec16<bf16_t> v = ld16(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)v.e[e];
}
template <> __device__ __forceinline__ void em_load8<float>(const float* p, float* x) {
    const Vec16<float> a = ld16(p), b = ld16(p + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        x[e] = a.e[e];
        x[4 + e] = b.e[e];
    }
}
template <typename T> __device__ __forceinline__ void em_store8(T* p, const float* x);
template <> __device__ __forceinline__ void em_store8<bf16_t>(bf16_t* p, const float* x) {
    Vec16<bf16_t> v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v.e[e] = (bf16_t)x[e];
    st16(p, v);
}
template <> __device__ __forceinline__ void em_store8<float>(float* p, const float* x) {
    Vec16<float> a, b;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        a.e[e] = x[e];
        b.e[e] = x[4 + e];
    }
    st16(p, a);
    st16(p + 4, b);
}

template <typename T, int C>
__global__ __launch_bounds__(EM_THREADS) void pair_embed_kernel(
    T* __restrict__ out, const T* z, const T* __restrict__ gamma, const T* __restrict__ beta, float ln_eps,
    const T* __restrict__ table, const T* __restrict__ bias, const T* __restrict__ row, const T* __restrict__ col,
    int mode, const float* __restrict__ pos, const float* __restrict__ edges, float inf, int r, int nb) {
    constexpr int LPR = C / 8;
    constexpr int PPB = EM_THREADS / LPR;          // pairs per workgroup pass
    const int c0 = (threadIdx.x % LPR) * 8;
    const long npairs = (long)r * r;
    float gm[8], bt[8], bs[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        gm[e] = z ? DT<T>::to_f(gamma[c0 + e]) : 0.f;
        bt[e] = z ? DT<T>::to_f(beta[c0 + e]) : 0.f;
        bs[e] = bias ? DT<T>::to_f(bias[c0 + e]) : 0.f;
    }
    for (long p = (long)blockIdx.x * PPB + threadIdx.x / LPR; p < npairs; p += (long)gridDim.x * PPB) {
        const int i = (int)(p / r), j = (int)(p - (long)i * r);
        float acc[8];
        if (z) {
            em_load8<T>(z + p * C + c0, acc);
            float s1 = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s1 += acc[e];
            const float mean = group_sum(s1, LPR) * (1.0f / C);
            float s2 = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                acc[e] -= mean;
                s2 += acc[e] * acc[e];
            }
            const float rstd = rsqrtf(group_sum(s2, LPR) * (1.0f / C) + ln_eps);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = acc[e] * rstd * gm[e] + bt[e] + bs[e];
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = bs[e];
        }
        int bin = -1;
        if (mode == FFK_EMBED_RELPOS) {
            // nearest of the integer offsets -k .. k (nb = 2k + 1), the lower one on a tie
            const int k = nb >> 1;
            float d = pos[i] - pos[j];
            d = fminf(fmaxf(d, (float)-k), (float)k);
            bin = (int)ceilf(d - 0.5f) + k;
        } else {
            const float dx = pos[3 * i] - pos[3 * j], dy = pos[3 * i + 1] - pos[3 * j + 1], dz = pos[3 * i + 2] - pos[3 * j + 2];
            const float d2 = dx * dx + dy * dy + dz * dz;
            for (int b = 0; b < nb; ++b) {
                const float lo = edges[b], hi = b + 1 < nb ? edges[b + 1] : inf;
                if (d2 > lo && d2 < hi) bin = b;
            }
        }
        float t[8];
        if (bin >= 0) {
            em_load8<T>(table + (long)bin * C + c0, t);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += t[e];
        }
        if (row) {
            em_load8<T>(row + (long)i * C + c0, t);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += t[e];
        }
        if (col) {
            em_load8<T>(col + (long)j * C + c0, t);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += t[e];
        }
        em_store8<T>(out + p * C + c0, acc);
    }
}

template <typename T>
int em_launch(void* out, const void* z, const void* gamma, const void* beta, float ln_eps, const void* table,
              const void* bias, const void* row, const void* col, int mode, const float* pos, const float* edges,
              float inf, int64_t r, int64_t C, int64_t nb, hipStream_t st) {
    const long npairs = r * r;
#define EM_CASE(CC)                                                                                              \
    case CC: {                                                                                                   \
        const int ppb = EM_THREADS / (CC / 8);                                                                   \
        long grid = (npairs + ppb - 1) / ppb;                                                                    \
        grid = grid < 256 * 16 ? grid : 256 * 16;                                                                \
        hipLaunchKernelGGL((pair_embed_kernel<T, CC>), dim3((unsigned)grid), dim3(EM_THREADS), 0, st, (T*)out,    \
                           (const T*)z, (const T*)gamma, (const T*)beta, ln_eps, (const T*)table, (const T*)bias, \
                           (const T*)row, (const T*)col, mode, pos, edges, inf, (int)r, (int)nb);                 \
        break;                                                                                                   \
    }
    switch (C) {
        EM_CASE(64)
        EM_CASE(128)
        EM_CASE(256)
        default:
            return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_pair_embed: C must be 64, 128 or 256 (got %ld)", (long)C);
    }
#undef EM_CASE
    return ffk_check_launch("ffk_pair_embed");
}

}  // namespace

extern "C" int ffk_pair_embed(void* out, const void* z, const void* ln_gamma, const void* ln_beta, float ln_eps,
                              const void* table, const void* bias, const void* row, const void* col, int mode,
                              const float* pos, const float* edges, float inf, int64_t r, int64_t C, int64_t nb,
                              int dtype, void* stream) {
    FFK_REQUIRE(out && table && pos, FFK_ERR_NULL, "ffk_pair_embed: null pointer");
    FFK_REQUIRE(!z || (ln_gamma && ln_beta), FFK_ERR_NULL, "ffk_pair_embed: z needs ln_gamma / ln_beta");
    FFK_REQUIRE(mode == FFK_EMBED_RELPOS || mode == FFK_EMBED_DISTOGRAM, FFK_ERR_UNSUPPORTED,
                "ffk_pair_embed: unknown mode %d", mode);
    FFK_REQUIRE(mode == FFK_EMBED_RELPOS || edges, FFK_ERR_NULL, "ffk_pair_embed: the distogram mode needs bin edges");
    FFK_REQUIRE(r >= 0 && r <= 46340 && nb >= 1 && nb <= 4096 && (mode != FFK_EMBED_RELPOS || (nb & 1)), FFK_ERR_SHAPE,
                "ffk_pair_embed: bad sizes r=%ld, nb=%ld (relative positions need an odd number of bins)", (long)r, (long)nb);
    if (r == 0) return FFK_OK;
    FFK_REQUIRE(ffk_aligned16(out) && (!z || ffk_aligned16(z)) && ffk_aligned16(table) && (!row || ffk_aligned16(row)) &&
                    (!col || ffk_aligned16(col)),
                FFK_ERR_ALIGN, "ffk_pair_embed: tensors must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_F32:
            return em_launch<float>(out, z, ln_gamma, ln_beta, ln_eps, table, bias, row, col, mode, pos, edges, inf, r, C, nb, st);
        case FFK_BF16:
            return em_launch<bf16_t>(out, z, ln_gamma, ln_beta, ln_eps, table, bias, row, col, mode, pos, edges, inf, r, C, nb, st);
        default:
            return ffk_fail(FFK_ERR_DTYPE, "ffk_pair_embed: unsupported dtype tag %d", dtype);
    }
}
