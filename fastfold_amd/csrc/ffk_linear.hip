// Fused linear layer for the Evoformer projections (see ffk_fused_linear in include/ffk.h).
//
// One workgroup (4 wavefronts) owns BM rows of A.  The whole [BM x K] slab (K <= 256) is
// staged in LDS once - read from HBM exactly once - optionally LayerNorm-ed in place, and
// then multiplied against every 128-row tile of the weight matrix.  Weight tiles stream
// through a double-buffered LDS ring in K-chunks (register prefetch of the next chunk
// overlaps the MFMAs of the current one); weights are a few hundred KB and stay in L2.
// The 32x32 MFMA computes C^T: the weight fragment is the M-operand (rows = output
// channels) and the activation fragment the N-operand (columns = rows of A), so a lane
// ends up with 4 consecutive output channels of one row.  Results are staged through LDS
// (aliasing the weight ring) and written with 16-byte accesses in whichever direction the
// destination layout is contiguous.
#include "ffk_common.h"

namespace {

constexpr int NT = 128;        // output channels per N-tile
constexpr int THREADS = 256;

template <typename T> struct LinCfg;
template <> struct LinCfg<bf16_t> {
    static constexpr int BM = 128, WM = 4, WN = 1, BK = 64;
};
template <> struct LinCfg<float> {
    static constexpr int BM = 64, WM = 2, WN = 2, BK = 32;
};

struct LinArgs {
    ffk_linear_desc d;
};

__device__ __forceinline__ long row_off(long m, int inner, long so, long si) {
    return (m / inner) * so + (m % inner) * si;
}

template <typename T>
__global__ __launch_bounds__(THREADS) void fused_linear_kernel(const LinArgs args) {
    typedef LinCfg<T> Cfg;
    typedef Mma<T> MM;
    constexpr int BM = Cfg::BM, WM = Cfg::WM, WN = Cfg::WN, BK = Cfg::BK;
    constexpr int CT = NT / (WN * 32);             // 32-channel MFMA tiles per wave
    constexpr int VEC = DT<T>::VEC;
    constexpr int ES = sizeof(T);
    constexpr int WP = BK * ES + 16;               // weight ring row pitch (bytes)
    constexpr int WBUF = NT * WP;                  // one ring slot
    constexpr int CP = NT * ES + 16;               // staged C pitch, [row][channel]
    constexpr int CPT = BM * ES + 16;              // staged C pitch, [channel][row]
    static_assert(BM * CP <= 2 * WBUF, "C staging must fit in the weight ring");
    static_assert(NT * CPT <= 2 * WBUF + 4096, "transposed C staging");

    const ffk_linear_desc& d = args.d;
    const int K = d.K, M = d.M;
    const int AP = K * ES + 16;                    // A slab row pitch (bytes)
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* sA = smem;
    unsigned char* sW = smem + (size_t)BM * AP;
    unsigned char* sC = sW;                        // aliases the ring between tiles

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, half = lane >> 5;
    const long m0 = (long)blockIdx.x * BM;
    const T* A = (const T*)d.a;
    const T* W = (const T*)d.w;

    // ---- weight chunk prefetch (registers) ----
    constexpr int WVEC = NT * BK / VEC / THREADS;  // 16-byte vectors per thread per chunk (= 4)
    Vec16<T> wreg[WVEC];
    const int kchunks = K / BK;
    const int total_chunks = d.n_tiles * kchunks;
    auto w_fetch = [&](int chunk) {
        const int nt = chunk / kchunks, kc = chunk % kchunks;
#pragma unroll
        for (int i = 0; i < WVEC; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (BK / VEC), c = v % (BK / VEC);
            wreg[i] = ld16(W + ((long)nt * NT + r) * K + kc * BK + c * VEC);
        }
    };
    auto w_commit = [&](int slot) {
#pragma unroll
        for (int i = 0; i < WVEC; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (BK / VEC), c = v % (BK / VEC);
            *reinterpret_cast<Vec16<T>*>(sW + slot * WBUF + r * WP + c * 16) = wreg[i];
        }
    };
    w_fetch(0);

    // ---- stage the A slab ----
    if (!d.a_chanmajor) {
        const int vpr = K / VEC;
        for (int v = tid; v < BM * vpr; v += THREADS) {
            const int r = v / vpr, c = v % vpr;
            const long m = m0 + r;
            Vec16<T> x;
            if (m < M) {
                x = ld16(A + row_off(m, d.a_inner, d.a_so, d.a_si) + c * VEC);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) x.e[e] = DT<T>::from_f(0.0f);
            }
            *reinterpret_cast<Vec16<T>*>(sA + r * AP + c * 16) = x;
        }
    } else {
        // element (m, k) at a + k * a_cs + rowoff(m): read runs of VEC rows, scatter into [row][k]
        const int rpv = BM / VEC;
        for (int v = tid; v < K * rpv; v += THREADS) {
            const int k = v / rpv, r0 = (v % rpv) * VEC;
            const long m = m0 + r0;
            T vals[VEC];
            const long o0 = m < M ? row_off(m, d.a_inner, d.a_so, d.a_si) : 0;
            const long mlast = m + VEC - 1;
            bool contig = mlast < M && d.a_si == 1 && (m % d.a_inner) + VEC - 1 < d.a_inner;
            const T* src = A + (long)k * d.a_cs + o0;
            contig = contig && ((reinterpret_cast<uintptr_t>(src) & 15u) == 0);
            if (contig) {
                Vec16<T> x = ld16(src);
#pragma unroll
                for (int e = 0; e < VEC; ++e) vals[e] = x.e[e];
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    vals[e] = (m + e < M) ? A[(long)k * d.a_cs + row_off(m + e, d.a_inner, d.a_so, d.a_si)]
                                          : DT<T>::from_f(0.0f);
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) *reinterpret_cast<T*>(sA + (r0 + e) * AP + k * ES) = vals[e];
        }
    }
    __syncthreads();

    // ---- LayerNorm prologue, in place ----
    if (d.ln_gamma) {
        constexpr int TPR = THREADS / BM;          // threads per row (adjacent lanes)
        const int r = tid / TPR, j = tid % TPR;
        const int vpr = K / VEC;
        const T* gam = (const T*)d.ln_gamma;
        const T* bet = (const T*)d.ln_beta;
        unsigned char* rowp = sA + r * AP;
        float s = 0.0f;
        for (int c = j; c < vpr; c += TPR) {
            Vec16<T> x = *reinterpret_cast<Vec16<T>*>(rowp + c * 16);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s += DT<T>::to_f(x.e[e]);
        }
        const float mu = group_sum(s, TPR) / (float)K;
        float q = 0.0f;
        for (int c = j; c < vpr; c += TPR) {
            Vec16<T> x = *reinterpret_cast<Vec16<T>*>(rowp + c * 16);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float dd = DT<T>::to_f(x.e[e]) - mu;
                q += dd * dd;
            }
        }
        const float rs = rsqrtf(group_sum(q, TPR) / (float)K + d.ln_eps);
        for (int c = j; c < vpr; c += TPR) {
            Vec16<T> x = *reinterpret_cast<Vec16<T>*>(rowp + c * 16);
            Vec16<T> g = ld16(gam + c * VEC), b = ld16(bet + c * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                x.e[e] = DT<T>::from_f((DT<T>::to_f(x.e[e]) - mu) * rs * DT<T>::to_f(g.e[e]) + DT<T>::to_f(b.e[e]));
            *reinterpret_cast<Vec16<T>*>(rowp + c * 16) = x;
        }
        // visibility to the other waves is ensured by the barrier of the first weight chunk
    }

    // ---- main loop over N-tiles ----
    const unsigned char* a_frag_base = sA + (wm * 32 + l32) * AP + half * (MM::KLANE * ES);
    int chunk = 0;
    for (int nt = 0; nt < d.n_tiles; ++nt) {
        f32x16 acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ct][v] = 0.0f;

        for (int kc = 0; kc < kchunks; ++kc, ++chunk) {
            const int slot = chunk & 1;
            w_commit(slot);
            __syncthreads();
            if (chunk + 1 < total_chunks) w_fetch(chunk + 1);
            const unsigned char* wb = sW + slot * WBUF + (wn * CT * 32 + l32) * WP + half * (MM::KLANE * ES);
            const unsigned char* ab = a_frag_base + kc * BK * ES;
#pragma unroll
            for (int ks = 0; ks < BK / MM::KSTEP; ++ks) {
                typename MM::Frag fx = *reinterpret_cast<const typename MM::Frag*>(ab + ks * MM::KSTEP * ES);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    typename MM::Frag fw =
                        *reinterpret_cast<const typename MM::Frag*>(wb + ct * 32 * WP + ks * MM::KSTEP * ES);
                    MM::mma(acc[ct], fw, fx);
                }
            }
        }

        // ---- epilogue of this tile ----
        const ffk_tile& t = d.tiles[nt];
        const bool mode_c = (t.kind == FFK_TILE_STRIDED && t.s_d == 1) || t.kind == FFK_TILE_QK;
        const T* bias = (const T*)t.bias;
        const int prow = wm * 32 + l32;                         // row within the slab
        const long mrow = m0 + prow;
        float rmask = 1.0f;
        if (t.rowmask && mrow < M)
            rmask = DT<T>::to_f(((const T*)t.rowmask)[row_off(mrow, t.inner, t.m_so, t.m_si)]);
        __syncthreads();                                        // all waves done with the ring
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (t.glu && (ct & 1)) continue;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float val[4];
                const int cin = (wn * CT + ct) * 32 + 8 * g + 4 * half;       // packed tile channel
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x = acc[ct][4 * g + e] + (bias ? DT<T>::to_f(bias[cin + e]) : 0.0f);
                    if (t.glu) {
                        const float gv = acc[ct | 1][4 * g + e] + (bias ? DT<T>::to_f(bias[cin + 32 + e]) : 0.0f);
                        x = x * sigmoid_f(gv);
                    } else if (t.act == FFK_ACT_RELU) {
                        x = fmaxf(x, 0.0f);
                    } else if (t.act == FFK_ACT_SIGMOID) {
                        x = sigmoid_f(x);
                    }
                    val[e] = x * t.scale * rmask;
                }
                const int cout = t.glu ? ((wn * CT + ct) >> 1) * 32 + 8 * g + 4 * half : cin;
                if (mode_c) {
                    T* dst = reinterpret_cast<T*>(sC + prow * CP + cout * ES);
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[e] = DT<T>::from_f(val[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        *reinterpret_cast<T*>(sC + (cout + e) * CPT + prow * ES) = DT<T>::from_f(val[e]);
                }
            }
        }
        __syncthreads();

        T* out = (T*)t.out;
        const int ncols = t.ncols;
        if (mode_c) {
            constexpr int VPR = NT / VEC;
            for (int v = tid; v < BM * VPR; v += THREADS) {
                const int r = v / VPR, c = (v % VPR) * VEC;
                const long m = m0 + r;
                if (m >= M || c >= ncols) continue;
                Vec16<T> x = *reinterpret_cast<const Vec16<T>*>(sC + r * CP + c * ES);
                long o;
                if (t.kind == FFK_TILE_QK) {
                    const long b2 = m / t.inner;
                    const int n = (int)(m % t.inner);
                    o = b2 * t.s_o + (long)(c >> 5) * t.s_h + (long)(n >> 5) * 1024 + qk_tile_off(n & 31, c & 31);
                } else {
                    o = row_off(m, t.inner, t.s_o, t.s_i) + (long)(c >> 5) * t.s_h + (c & 31);
                }
                if (t.gate) {
                    Vec16<T> gv = ld16((const T*)t.gate + m * t.gate_ld + c);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x.e[e] = DT<T>::from_f(DT<T>::to_f(x.e[e]) * DT<T>::to_f(gv.e[e]));
                }
                if (c + VEC <= ncols) {
                    if (t.resid) {
                        Vec16<T> rv = ld16((const T*)t.resid + o);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) x.e[e] = DT<T>::from_f(DT<T>::to_f(x.e[e]) + DT<T>::to_f(rv.e[e]));
                    }
                    st16(out + o, x);
                } else {
                    for (int e = 0; e < VEC && c + e < ncols; ++e) {
                        float y = DT<T>::to_f(x.e[e]);
                        if (t.resid) y += DT<T>::to_f(((const T*)t.resid)[o + e]);
                        out[o + e] = DT<T>::from_f(y);
                    }
                }
            }
        } else {
            constexpr int QPR = BM / 4;                         // 4-row runs per channel
            for (int v = tid; v < ncols * QPR; v += THREADS) {
                const int c = v / QPR, r = (v % QPR) * 4;
                const long m = m0 + r;
                if (m >= M) continue;
                const T* src = reinterpret_cast<const T*>(sC + c * CPT + r * ES);
                long o[4];
                bool ok[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const long me = m + e;
                    ok[e] = me < M;
                    const long mm = ok[e] ? me : m;
                    const long hi = mm / t.inner;
                    const int lo = (int)(mm % t.inner);
                    if (t.kind == FFK_TILE_V) {
                        o[e] = hi * t.s_o + (long)(c >> 5) * t.s_h + (long)(lo >> 5) * 1024 + acc_tile_off(lo & 31, c & 31);
                    } else if (t.kind == FFK_TILE_BIAS) {
                        // logical row = (query hi, key lo); channel = head
                        o[e] = (long)c * t.s_h + (hi >> 5) * t.s_o + (long)(lo >> 5) * 1024 +
                               acc_tile_off(lo & 31, (int)(hi & 31));
                    } else {
                        o[e] = hi * t.s_o + lo * t.s_i + (long)(c >> 5) * t.s_h + (long)(c & 31) * t.s_d;
                    }
                }
                const bool run = ok[3] && o[1] == o[0] + 1 && o[2] == o[0] + 2 && o[3] == o[0] + 3 &&
                                 ((reinterpret_cast<uintptr_t>(out + o[0]) & (4 * ES - 1)) == 0);
                if (run) {
                    if (ES == 2) {
                        *reinterpret_cast<u32x2*>(out + o[0]) = *reinterpret_cast<const u32x2*>(src);
                    } else {
                        *reinterpret_cast<u32x4*>(out + o[0]) = *reinterpret_cast<const u32x4*>(src);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (ok[e]) out[o[e]] = src[e];
                }
            }
        }
        __syncthreads();                                        // staging area is the ring again
    }
}

template <typename T>
int launch_linear(const ffk_linear_desc& d, hipStream_t st) {
    typedef LinCfg<T> Cfg;
    constexpr int ES = sizeof(T);
    constexpr int WP = Cfg::BK * ES + 16;
    size_t ring = 2 * (size_t)NT * WP;
    size_t ct = (size_t)NT * (Cfg::BM * ES + 16);
    if (ct > ring) ring = ct;
    const size_t smem = (size_t)Cfg::BM * (d.K * ES + 16) + ring;
    static size_t configured = 0;
    if (smem > configured) {
        hipError_t e = hipFuncSetAttribute((const void*)fused_linear_kernel<T>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "ffk_fused_linear: cannot reserve %zu B of LDS: %s", smem,
                                             hipGetErrorString(e));
        configured = smem;
    }
    LinArgs a;
    a.d = d;
    dim3 grid(ffk_cdiv(d.M, Cfg::BM));
    fused_linear_kernel<T><<<grid, THREADS, smem, st>>>(a);
    return ffk_check_launch("ffk_fused_linear");
}

}  // namespace

extern "C" int ffk_fused_linear(const ffk_linear_desc* d, void* stream) {
    FFK_REQUIRE(d, FFK_ERR_NULL, "ffk_fused_linear: null descriptor");
    FFK_REQUIRE(d->a && d->w, FFK_ERR_NULL, "ffk_fused_linear: null operand");
    const int bk = d->dtype == FFK_F32 ? 32 : 64;
    FFK_REQUIRE(d->M > 0 && d->K >= bk && d->K <= 256 && d->K % bk == 0, FFK_ERR_SHAPE,
                "ffk_fused_linear: need M > 0 and K <= 256, a multiple of %d; got M=%d K=%d", bk, d->M, d->K);
    FFK_REQUIRE(d->n_tiles >= 1 && d->n_tiles <= FFK_MAX_TILES, FFK_ERR_SHAPE,
                "ffk_fused_linear: n_tiles must be in [1,%d], got %d", FFK_MAX_TILES, d->n_tiles);
    FFK_REQUIRE(d->a_inner > 0, FFK_ERR_SHAPE, "ffk_fused_linear: a_inner must be positive");
    FFK_REQUIRE(ffk_aligned16(d->a) && ffk_aligned16(d->w), FFK_ERR_ALIGN, "ffk_fused_linear: operands must be 16-byte aligned");
    const int es = d->dtype == FFK_F32 ? 4 : 2;
    if (!d->a_chanmajor)
        FFK_REQUIRE((d->a_so * es) % 16 == 0 && (d->a_si * es) % 16 == 0, FFK_ERR_ALIGN,
                    "ffk_fused_linear: row strides of A must be multiples of 16 bytes");
    FFK_REQUIRE(!d->ln_gamma || d->ln_beta, FFK_ERR_NULL, "ffk_fused_linear: ln_beta missing");
    for (int i = 0; i < d->n_tiles; ++i) {
        const ffk_tile& t = d->tiles[i];
        FFK_REQUIRE(t.out, FFK_ERR_NULL, "ffk_fused_linear: tile %d has no output", i);
        FFK_REQUIRE(t.inner > 0 && t.ncols > 0 && t.ncols <= (t.glu ? 64 : 128), FFK_ERR_SHAPE,
                    "ffk_fused_linear: tile %d: bad inner/ncols (%d, %d)", i, t.inner, t.ncols);
        FFK_REQUIRE(t.kind >= FFK_TILE_STRIDED && t.kind <= FFK_TILE_BIAS, FFK_ERR_UNSUPPORTED,
                    "ffk_fused_linear: tile %d: unknown kind %d", i, t.kind);
        const bool mode_c = (t.kind == FFK_TILE_STRIDED && t.s_d == 1) || t.kind == FFK_TILE_QK;
        FFK_REQUIRE(mode_c || (!t.resid && !t.gate), FFK_ERR_UNSUPPORTED,
                    "ffk_fused_linear: tile %d: resid/gate need a channel-contiguous strided tile", i);
        if (mode_c) {
            FFK_REQUIRE(ffk_aligned16(t.out) && (t.s_o * es) % 16 == 0 && (t.s_i * es) % 16 == 0 && (t.s_h * es) % 16 == 0,
                        FFK_ERR_ALIGN, "ffk_fused_linear: tile %d: output must be 16-byte aligned in every stride", i);
            FFK_REQUIRE(!t.resid || ffk_aligned16(t.resid), FFK_ERR_ALIGN, "ffk_fused_linear: tile %d: resid alignment", i);
            FFK_REQUIRE(!t.gate || (ffk_aligned16(t.gate) && (t.gate_ld * es) % 16 == 0), FFK_ERR_ALIGN,
                        "ffk_fused_linear: tile %d: gate alignment", i);
        }
    }
    switch (d->dtype) {
        case FFK_BF16: return launch_linear<bf16_t>(*d, (hipStream_t)stream);
        case FFK_F32: return launch_linear<float>(*d, (hipStream_t)stream);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_fused_linear: unsupported dtype tag %d", d->dtype);
    }
}
