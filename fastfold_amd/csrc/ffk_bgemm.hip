// Batched NT GEMM with a K loop (see ffk_bgemm_nt in include/ffk.h).
//
// 128x128 output tile per workgroup, 4 wavefronts in a 2x2 grid, each owning 64x64 as
// 2x2 MFMA 32x32 tiles.  A and B K-chunks (128 bytes of K per row) stream through a
// double-buffered LDS ring with register prefetch.  As in the fused linear kernel the MFMA
// computes C^T (rows of B are the M-operand) so that a lane holds 4 consecutive n of one
// row m, and the tile is staged through LDS for 16-byte stores.
#include "ffk_common.h"
#include <type_traits>

namespace {

constexpr int BT = 128;
constexpr int THREADS = 256;

template <typename T, typename OT>
__global__ __launch_bounds__(THREADS) void bgemm_nt_kernel(const ffk_bgemm_desc d) {
    typedef Mma<T> MM;
    constexpr int VEC = DT<T>::VEC;
    constexpr int ES = sizeof(T);
    constexpr int OES = sizeof(OT);
    constexpr int OVEC = 16 / OES;
    constexpr bool XS_OK = std::is_same<OT, bf16_t>::value;     // outputs that may carry a residual tail
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
    const int M = d.M, N = d.N, K = d.K;
    // Workgroup -> tile.  Consecutive workgroup ids go to the eight XCDs in turn, each with its own L2.
    // With at least eight batches every XCD takes a contiguous eighth of the (batch, n-tile, m-tile)
    // order, so that all tiles of one batch matrix pair run behind one L2 and A / B are fetched from
    // HBM once instead of once per XCD.  With fewer batches the plain order is kept: tiles that run
    // together then share their operand panels across the XCDs' row / column residues.
    const unsigned tiles_m = (M + BT - 1) / BT, tiles_n = (N + BT - 1) / BT;
    unsigned item = blockIdx.x;
    if (d.batch >= 8) {
        const unsigned total = tiles_m * tiles_n * (unsigned)d.batch, per_xcd = (total + 7) >> 3;
        item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (item >= total) return;
    }
    const long m0 = (long)(item % tiles_m) * BT, n0 = (long)((item / tiles_m) % tiles_n) * BT;
    const int bz = (item / tiles_m) / tiles_n;
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
            // branch-free: clamp the K offset to the last full vector; the K tail is zeroed when the
            // registers are committed to LDS (touching them here would serialise the loads)
            const int kk = k < K ? k : K - VEC;
            ra[i] = ld16(A + ma * d.lda + kk);
            rb[i] = ld16(B + nb * d.ldb + kk);
        }
    };
    auto commit = [&](int slot, int kc) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (BK / VEC), c = v % (BK / VEC);
            const bool tail = kc * BK + c * VEC >= K;
            Vec16<T> xa = ra[i], xb = rb[i];
            if (tail) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) xa.e[e] = xb.e[e] = DT<T>::from_f(0.0f);
            }
            *reinterpret_cast<Vec16<T>*>(sA + slot * SLOT + r * P + c * 16) = xa;
            *reinterpret_cast<Vec16<T>*>(sB + slot * SLOT + r * P + c * 16) = xb;
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
        commit(slot, kc);
        lds_barrier();
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
    lds_barrier();

    // row offsets of this tile, one integer division per row (kept in LDS for phase 2)
    __shared__ long s_off[BT];
    if (tid < BT) {
        long m = m0 + tid;
        if (m >= M) m = M - 1;
        const unsigned hi = (unsigned)m / (unsigned)d.inner;
        const unsigned lo = (unsigned)m - hi * (unsigned)d.inner;
        s_off[tid] = (long)hi * d.s_o + (long)lo * d.s_i;
    }

    // ---- phase 1: registers -> staged tile [m][n] (values after bias / act / scale / rowdiv) ----
    // (bias / rowdiv are fetched with clamped indices, i.e. without per-lane branches, so the loads
    // are issued back to back; out-of-range values are computed but never stored)
    const T* bias = (const T*)d.bias;
    float bv[2][4][4];
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                long n = n0 + wn * 64 + ni * 32 + 8 * g + 4 * half + e;
                n = n < N ? n : N - 1;
                bv[ni][g][e] = bias ? DT<T>::to_f(bias[n]) : 0.0f;
            }
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
        const int mr = wm * 64 + mi * 32 + l32;
        long m = m0 + mr;
        m = m < M ? m : M - 1;
        float rdiv = 1.0f;
        if (d.rowdiv) rdiv = 1.0f / (d.rowdiv[(long)bz * M + m] + d.div_eps);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nc = wn * 64 + ni * 32 + 8 * g + 4 * half;
                OT* dst = reinterpret_cast<OT*>(sC + mr * CP + nc * OES);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x = acc[ni][mi][4 * g + e] + bv[ni][g][e];
                    if (d.act == FFK_ACT_RELU) x = relu_f(x);
                    else if (d.act == FFK_ACT_SIGMOID) x = sigmoid_f(x);
                    dst[e] = DT<OT>::from_f(x * d.scale * rdiv);
                }
            }
        }
    }
    lds_barrier();

    // ---- phase 2: staged tile -> global ----
    OT* out = (OT*)d.out + (long)bz * d.o_bs;
    const OT* resid = d.resid ? (const OT*)d.resid + (long)bz * d.o_bs : nullptr;
    // extended residual stream (bf16 output with a residual, s_d == 1): the update is added at 24 bits
    int8_t* xtail = nullptr;
    if constexpr (XS_OK) xtail = d.xtail ? (int8_t*)d.xtail + (long)bz * d.o_bs : nullptr;
    if (d.s_d == 1) {
        constexpr int VPR = BT / OVEC;
        constexpr int N_IT = BT * VPR / THREADS;
        // vector path when every row pitch / base keeps 16-byte alignment and N is a multiple of the vector
        const bool vec_ok = (N % OVEC) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0 &&
                            (!resid || (reinterpret_cast<uintptr_t>(resid) & 15u) == 0) && (d.s_o % OVEC) == 0 &&
                            (d.s_i % OVEC) == 0 && (d.s_h % OVEC) == 0;
        if (vec_ok) {
            const long n_last = N - OVEC;
#pragma unroll 1
            for (int i0 = 0; i0 < N_IT; i0 += 4) {
                Vec16<OT> x[4], rv[4];
                u32x2 tv[4];
                long o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = tid + THREADS * (i0 + j);
                    const int r = v / VPR, c = (v % VPR) * OVEC;
                    long n = n0 + c;
                    n = n <= n_last ? n : n_last;
                    o[j] = s_off[r] + (n >> 5) * d.s_h + (n & 31);
                    x[j] = *reinterpret_cast<const Vec16<OT>*>(sC + r * CP + c * OES);
                    if (resid) rv[j] = ld16(resid + o[j]);
                    if (xtail) tv[j] = *reinterpret_cast<const u32x2*>(xtail + o[j]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = tid + THREADS * (i0 + j);
                    const int r = v / VPR, c = (v % VPR) * OVEC;
                    if constexpr (XS_OK) {
                        if (xtail) {
                            float f[8];
                            xs_decode8(*reinterpret_cast<const u32x4*>(&rv[j]), tv[j][0], tv[j][1], f);
#pragma unroll
                            for (int e = 0; e < 8; ++e) f[e] += (float)x[j].e[e];
                            u32x4 hv;
                            u32x2 tn;
                            xs_encode8(f, hv, tn);
                            if (m0 + r < M && n0 + c < N) {
                                *reinterpret_cast<u32x4*>(out + o[j]) = hv;
                                *reinterpret_cast<u32x2*>(xtail + o[j]) = tn;
                            }
                            continue;
                        }
                    }
                    if (resid) {
#pragma unroll
                        for (int e = 0; e < OVEC; ++e)
                            x[j].e[e] = DT<OT>::from_f(DT<OT>::to_f(x[j].e[e]) + DT<OT>::to_f(rv[j].e[e]));
                    }
                    if (m0 + r < M && n0 + c < N) st16(out + o[j], x[j]);
                }
            }
        } else {
            for (int v = tid; v < BT * BT; v += THREADS) {
                const int r = v / BT, c = v % BT;
                const long m = m0 + r, n = n0 + c;
                if (m >= M || n >= N) continue;
                const long o = s_off[r] + (n >> 5) * d.s_h + (n & 31);
                float y = DT<OT>::to_f(*reinterpret_cast<const OT*>(sC + r * CP + c * OES));
                if constexpr (XS_OK) {
                    if (xtail) {
                        xs_round(y + xs_value(resid[o], xtail[o]), &out[o], &xtail[o]);
                        continue;
                    }
                }
                if (resid) y += DT<OT>::to_f(resid[o]);
                out[o] = DT<OT>::from_f(y);
            }
        }
    } else {
        for (int v = tid; v < BT * BT; v += THREADS) {
            const int c = v / BT, r = v % BT;           // consecutive threads -> consecutive rows m
            const long m = m0 + r, n = n0 + c;
            if (m >= M || n >= N) continue;
            const long o = s_off[r] + (n >> 5) * d.s_h + (n & 31) * d.s_d;
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
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)bgemm_nt_kernel<T, OT>, smem, "ffk_bgemm_nt");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    const long tiles = (long)ffk_cdiv(d.M, BT) * ffk_cdiv(d.N, BT) * d.batch;
    FFK_REQUIRE(tiles < (1L << 31) - 8, FFK_ERR_SHAPE, "ffk_bgemm_nt: %ld output tiles exceed the grid limit", tiles);
    dim3 grid((unsigned)(d.batch >= 8 ? 8 * ffk_cdiv(tiles, 8) : tiles));
    bgemm_nt_kernel<T, OT><<<grid, THREADS, smem, st>>>(d);
    return ffk_check_launch("ffk_bgemm_nt");
}

}  // namespace

extern "C" int ffk_bgemm_nt(const ffk_bgemm_desc* d, void* stream) {
    FFK_REQUIRE(d, FFK_ERR_NULL, "ffk_bgemm_nt: null descriptor");
    FFK_REQUIRE(d->a && d->b && d->out, FFK_ERR_NULL, "ffk_bgemm_nt: null operand");
    FFK_REQUIRE(!d->xtail || (d->dtype == FFK_BF16 && !d->out_f32 && d->resid && d->s_d == 1 && d->N % 16 == 0),
                FFK_ERR_UNSUPPORTED, "ffk_bgemm_nt: a residual tail needs bf16 output, a residual, s_d == 1 and N %% 16 == 0");
    FFK_REQUIRE(ffk_aligned16(d->xtail) && (!d->xtail || (d->o_bs % 16 == 0 && d->s_o % 8 == 0 && d->s_i % 8 == 0 && d->s_h % 8 == 0)),
                FFK_ERR_ALIGN, "ffk_bgemm_nt: residual tail rows must be 16-byte aligned");
    const int es = d->dtype == FFK_F32 ? 4 : 2;
    const int vec = 16 / es;
    FFK_REQUIRE(d->M > 0 && d->N > 0 && d->K > 0 && d->batch > 0 && d->batch < 65536 && d->inner > 0, FFK_ERR_SHAPE,
                "ffk_bgemm_nt: bad shape M=%d N=%d K=%d batch=%d inner=%d", d->M, d->N, d->K, d->batch, d->inner);
    FFK_REQUIRE(d->K % vec == 0, FFK_ERR_SHAPE, "ffk_bgemm_nt: K=%d must be a multiple of %d", d->K, vec);
    FFK_REQUIRE(ffk_aligned16(d->a) && ffk_aligned16(d->b) && d->lda % vec == 0 && d->ldb % vec == 0 &&
                    d->a_bs % vec == 0 && d->b_bs % vec == 0,
                FFK_ERR_ALIGN, "ffk_bgemm_nt: operand rows must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    {
        int status = FFK_OK;
        if (ffk_bgemm_big_try(d, st, &status)) return status;
    }
    if (d->dtype == FFK_BF16) {
        return d->out_f32 ? launch_bgemm<bf16_t, float>(*d, st) : launch_bgemm<bf16_t, bf16_t>(*d, st);
    } else if (d->dtype == FFK_F32) {
        return launch_bgemm<float, float>(*d, st);
    }
    return ffk_fail(FFK_ERR_DTYPE, "ffk_bgemm_nt: unsupported dtype tag %d", d->dtype);
}
