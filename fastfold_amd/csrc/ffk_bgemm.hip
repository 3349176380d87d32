// Batched NT GEMM with a K loop (see ffk_bgemm_nt in include/ffk.h).
//
// 128x128 output tile per workgroup, 4 wavefronts in a 2x2 grid, each owning 64x64 as
// 2x2 MFMA 32x32 tiles.  A and B K-chunks (128 bytes of K per row) stream through a
// double-buffered LDS ring with register prefetch.  As in the fused linear kernel the MFMA
// computes C^T (rows of B are the M-operand) so that a lane holds 4 consecutive n of one
// row m, and the tile is staged through LDS for 16-byte stores.
#include "ffk_common.h"

namespace {

constexpr int BT = 128;
constexpr int THREADS = 256;

__device__ __forceinline__ long row_off(long m, int inner, long so, long si) {
    return (m / inner) * so + (m % inner) * si;
}

template <typename T, typename OT>
__global__ __launch_bounds__(THREADS) void bgemm_nt_kernel(const ffk_bgemm_desc d) {
    typedef Mma<T> MM;
    constexpr int VEC = DT<T>::VEC;
    constexpr int ES = sizeof(T);
    constexpr int OES = sizeof(OT);
    constexpr int OVEC = 16 / OES;
    constexpr int BK = 128 / ES;                   // K elements per chunk (128 bytes per row)
    constexpr int P = 128 + 16;                    // ring row pitch (bytes)
    constexpr int SLOT = BT * P;
    constexpr int CP = BT * OES + 16;              // staged C pitch [m][n]
    constexpr int NV = BT * (BK / VEC) / THREADS;  // 16-byte vectors per thread per operand chunk (= 4)

    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* sA = smem;                      // 2 slots
    unsigned char* sB = smem + 2 * SLOT;           // 2 slots
    unsigned char* sC = smem;                      // aliases the ring after the K loop

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, half = lane >> 5;
    const long m0 = (long)blockIdx.x * BT, n0 = (long)blockIdx.y * BT;
    const int bz = blockIdx.z;
    const int M = d.M, N = d.N, K = d.K;
    const T* A = (const T*)d.a + (long)bz * d.a_bs;
    const T* B = (const T*)d.b + (long)bz * d.b_bs;

    Vec16<T> ra[NV], rb[NV];
    auto fetch = [&](int kc) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (BK / VEC), c = v % (BK / VEC);
            const int k = kc * BK + c * VEC;
            long ma = m0 + r;
            if (ma >= M) ma = M - 1;
            long nb = n0 + r;
            if (nb >= N) nb = N - 1;
            if (k < K) {
                ra[i] = ld16(A + ma * d.lda + k);
                rb[i] = ld16(B + nb * d.ldb + k);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) ra[i].e[e] = rb[i].e[e] = DT<T>::from_f(0.0f);
            }
        }
    };
    auto commit = [&](int slot) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (BK / VEC), c = v % (BK / VEC);
            *reinterpret_cast<Vec16<T>*>(sA + slot * SLOT + r * P + c * 16) = ra[i];
            *reinterpret_cast<Vec16<T>*>(sB + slot * SLOT + r * P + c * 16) = rb[i];
        }
    };

    f32x16 acc[2][2];   // [ni][mi]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

    const int kchunks = (K + BK - 1) / BK;
    fetch(0);
    for (int kc = 0; kc < kchunks; ++kc) {
        const int slot = kc & 1;
        commit(slot);
        __syncthreads();
        if (kc + 1 < kchunks) fetch(kc + 1);
        const unsigned char* pa = sA + slot * SLOT + (wm * 64 + l32) * P + half * (MM::KLANE * ES);
        const unsigned char* pb = sB + slot * SLOT + (wn * 64 + l32) * P + half * (MM::KLANE * ES);
#pragma unroll
        for (int ks = 0; ks < BK / MM::KSTEP; ++ks) {
            typename MM::Frag fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const typename MM::Frag*>(pa + i * 32 * P + ks * MM::KSTEP * ES);
                fb[i] = *reinterpret_cast<const typename MM::Frag*>(pb + i * 32 * P + ks * MM::KSTEP * ES);
            }
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int mi = 0; mi < 2; ++mi) MM::mma(acc[ni][mi], fb[ni], fa[mi]);
        }
    }
    __syncthreads();

    // ---- phase 1: registers -> staged tile [m][n] (values after bias / act / scale / rowdiv) ----
    const T* bias = (const T*)d.bias;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        const int mr = wm * 64 + mi * 32 + l32;
        const long m = m0 + mr;
        float rdiv = 1.0f;
        if (d.rowdiv && m < M) rdiv = 1.0f / (d.rowdiv[(long)bz * M + m] + d.div_eps);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nc = wn * 64 + ni * 32 + 8 * g + 4 * half;
                OT* dst = reinterpret_cast<OT*>(sC + mr * CP + nc * OES);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x = acc[ni][mi][4 * g + e];
                    if (bias && n0 + nc + e < N) x += DT<T>::to_f(bias[n0 + nc + e]);
                    if (d.act == FFK_ACT_RELU) x = fmaxf(x, 0.0f);
                    else if (d.act == FFK_ACT_SIGMOID) x = sigmoid_f(x);
                    dst[e] = DT<OT>::from_f(x * d.scale * rdiv);
                }
            }
        }
    }
    __syncthreads();

    // ---- phase 2: staged tile -> global ----
    OT* out = (OT*)d.out + (long)bz * d.o_bs;
    const OT* resid = d.resid ? (const OT*)d.resid + (long)bz * d.o_bs : nullptr;
    if (d.s_d == 1) {
        constexpr int VPR = BT / OVEC;
        for (int v = tid; v < BT * VPR; v += THREADS) {
            const int r = v / VPR, c = (v % VPR) * OVEC;
            const long m = m0 + r, n = n0 + c;
            if (m >= M || n >= N) continue;
            Vec16<OT> x = *reinterpret_cast<const Vec16<OT>*>(sC + r * CP + c * OES);
            const long o = row_off(m, d.inner, d.s_o, d.s_i) + (n >> 5) * d.s_h + (n & 31);
            if (n + OVEC <= N && ((reinterpret_cast<uintptr_t>(out + o) & 15u) == 0)) {
                if (resid) {
                    Vec16<OT> rv = ld16(resid + o);
#pragma unroll
                    for (int e = 0; e < OVEC; ++e) x.e[e] = DT<OT>::from_f(DT<OT>::to_f(x.e[e]) + DT<OT>::to_f(rv.e[e]));
                }
                st16(out + o, x);
            } else {
                for (int e = 0; e < OVEC && n + e < N; ++e) {
                    float y = DT<OT>::to_f(x.e[e]);
                    if (resid) y += DT<OT>::to_f(resid[o + e]);
                    out[o + e] = DT<OT>::from_f(y);
                }
            }
        }
    } else {
        for (int v = tid; v < BT * BT; v += THREADS) {
            const int c = v / BT, r = v % BT;           // consecutive threads -> consecutive rows m
            const long m = m0 + r, n = n0 + c;
            if (m >= M || n >= N) continue;
            const long o = row_off(m, d.inner, d.s_o, d.s_i) + (n >> 5) * d.s_h + (n & 31) * d.s_d;
            float y = DT<OT>::to_f(*reinterpret_cast<const OT*>(sC + r * CP + c * OES));
            if (resid) y += DT<OT>::to_f(resid[o]);
            out[o] = DT<OT>::from_f(y);
        }
    }
}

template <typename T, typename OT>
int launch_bgemm(const ffk_bgemm_desc& d, hipStream_t st) {
    size_t ring = 4 * (size_t)BT * (128 + 16);
    size_t ct = (size_t)BT * (BT * sizeof(OT) + 16);
    const size_t smem = ring > ct ? ring : ct;
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)bgemm_nt_kernel<T, OT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "ffk_bgemm_nt: cannot reserve %zu B of LDS: %s", smem,
                                             hipGetErrorString(e));
        configured = true;
    }
    dim3 grid(ffk_cdiv(d.M, BT), ffk_cdiv(d.N, BT), d.batch);
    bgemm_nt_kernel<T, OT><<<grid, THREADS, smem, st>>>(d);
    return ffk_check_launch("ffk_bgemm_nt");
}

}  // namespace

extern "C" int ffk_bgemm_nt(const ffk_bgemm_desc* d, void* stream) {
    FFK_REQUIRE(d, FFK_ERR_NULL, "ffk_bgemm_nt: null descriptor");
    FFK_REQUIRE(d->a && d->b && d->out, FFK_ERR_NULL, "ffk_bgemm_nt: null operand");
    const int es = d->dtype == FFK_F32 ? 4 : 2;
    const int vec = 16 / es;
    FFK_REQUIRE(d->M > 0 && d->N > 0 && d->K > 0 && d->batch > 0 && d->batch < 65536 && d->inner > 0, FFK_ERR_SHAPE,
                "ffk_bgemm_nt: bad shape M=%d N=%d K=%d batch=%d inner=%d", d->M, d->N, d->K, d->batch, d->inner);
    FFK_REQUIRE(d->K % vec == 0, FFK_ERR_SHAPE, "ffk_bgemm_nt: K=%d must be a multiple of %d", d->K, vec);
    FFK_REQUIRE(ffk_cdiv(d->N, BT) < 65536, FFK_ERR_SHAPE, "ffk_bgemm_nt: N too large");
    FFK_REQUIRE(ffk_aligned16(d->a) && ffk_aligned16(d->b) && d->lda % vec == 0 && d->ldb % vec == 0 &&
                    d->a_bs % vec == 0 && d->b_bs % vec == 0,
                FFK_ERR_ALIGN, "ffk_bgemm_nt: operand rows must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (d->dtype == FFK_BF16) {
        return d->out_f32 ? launch_bgemm<bf16_t, float>(*d, st) : launch_bgemm<bf16_t, bf16_t>(*d, st);
    } else if (d->dtype == FFK_F32) {
        return launch_bgemm<float, float>(*d, st);
    }
    return ffk_fail(FFK_ERR_DTYPE, "ffk_bgemm_nt: unsupported dtype tag %d", d->dtype);
}
