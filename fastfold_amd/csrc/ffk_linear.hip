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
#include <type_traits>

namespace {

constexpr int NT = 128;        // output channels per N-tile
constexpr int THREADS = 256;

template <typename T> struct LinCfg;
template <> struct LinCfg<bf16_t> {
    static constexpr int BM = 64, WM = 2, WN = 2, BK = 32;
};
template <> struct LinCfg<float> {
    static constexpr int BM = 64, WM = 2, WN = 2, BK = 32;
};

struct LinArgs {
    ffk_linear_desc d;
};

// Row tables.  Splitting a logical row into (hi, lo) = divmod(m, inner) needs an integer
// division; it is done once per row of the slab (by one thread per row) and kept in LDS, so
// the streaming loops below contain no divisions.
struct RowTab {
    long off[128];   // hi * s_o + lo * s_i
    int hi[128];
    int lo[128];
};

__device__ __forceinline__ void fill_rowtab(RowTab& tab, int tid, int BM, long m0, int M, int inner, long so, long si) {
    if (tid < BM) {
        long m = m0 + tid;
        if (m >= M) m = M - 1;
        const unsigned mu = (unsigned)m;
        const unsigned hi = mu / (unsigned)inner;
        const unsigned lo = mu - hi * (unsigned)inner;
        tab.hi[tid] = (int)hi;
        tab.lo[tid] = (int)lo;
        tab.off[tid] = (long)hi * so + (long)lo * si;
    }
}

// Registers -> staged tile in LDS, one activation variant per instantiation (no per-element
// branching).  A lane holds, for its row, channels  chan0 + 32*ct + 8*g + e  (e = 0..3).  With
// GLU the odd MFMA tile of each pair holds the gate and the pair produces 32 output channels.
// mode_c: tile stored [row][channel] (crow = row base);  else [channel][row] (crow = column of
// this row, channel pitch cpt).
template <typename T, int CT, int GLU, int ACT>
__device__ __forceinline__ void stage_tile(const f32x16 (&acc)[CT], const T (&bv)[CT][4][4], float scl,
                                           unsigned char* crow, bool mode_c, int chan0, int cpt) {
    constexpr int ES = sizeof(T);
#pragma unroll
    for (int ct = 0; ct < CT; ct += (GLU ? 2 : 1)) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            T r4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x = acc[ct][4 * g + e] + DT<T>::to_f(bv[ct][g][e]);
                if (GLU) {
                    const float gv = acc[ct | 1][4 * g + e] + DT<T>::to_f(bv[ct | 1][g][e]);
                    x = x * sigmoid_f(gv);
                } else if (ACT == FFK_ACT_RELU) {
                    x = relu_f(x);
                } else if (ACT == FFK_ACT_SIGMOID) {
                    x = sigmoid_f(x);
                }
                r4[e] = DT<T>::from_f(x * scl);
            }
            const int cout = chan0 + (GLU ? (ct >> 1) : ct) * 32 + 8 * g;
            if (mode_c) {
                if (ES == 2) *reinterpret_cast<u32x2*>(crow + cout * ES) = *reinterpret_cast<const u32x2*>(r4);
                else *reinterpret_cast<u32x4*>(crow + cout * ES) = *reinterpret_cast<const u32x4*>(r4);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) *reinterpret_cast<T*>(crow + (cout + e) * cpt) = r4[e];
            }
        }
    }
}

template <typename T>
__global__ __launch_bounds__(THREADS, 4) void fused_linear_kernel(const LinArgs args) {
    typedef LinCfg<T> Cfg;
    typedef Mma<T> MM;
    constexpr int BM = Cfg::BM, WM = Cfg::WM, WN = Cfg::WN, BK = Cfg::BK;
    constexpr int CT = NT / (WN * 32);             // 32-channel MFMA tiles per wave
    constexpr int VEC = DT<T>::VEC;
    constexpr int ES = sizeof(T);
    constexpr bool XS_OK = std::is_same<T, bf16_t>::value;     // outputs that may carry a residual tail
    constexpr int WP = BK * ES + 16;               // weight ring row pitch (bytes)
    constexpr int WBUF = NT * WP;                  // one ring slot
    constexpr int CP = NT * ES + 16;               // staged C pitch, [row][channel]
    constexpr int CPT = BM * ES + 16;              // staged C pitch, [channel][row]
    static_assert(BM * CP <= 2 * WBUF, "C staging must fit in the weight ring");
    static_assert(NT * CPT <= 2 * WBUF + 4096, "transposed C staging");
    (void)WM;

    const ffk_linear_desc& d = args.d;
    const int K = d.K, M = d.M;
    const int AP = K * ES + 16;                    // A slab row pitch (bytes)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ RowTab tab;
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
        const int nt = chunk / kchunks, kc = chunk - nt * kchunks;
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

    // ---- stage the A slab (loads issued four at a time so their latencies overlap) ----
    fill_rowtab(tab, tid, BM, m0, M, d.a_inner, d.a_so, d.a_si);
    lds_barrier();
    // Loads below are unconditional (row / column indices are clamped to valid ones instead of
    // being predicated) so that a batch of four is in flight at once; only the LDS stores are guarded.
    // Rows beyond M hold a copy of row M-1: their results are never stored.
    if (!d.a_chanmajor) {
        const int vpr = K / VEC;                   // 16-byte vectors per row
        int cs = 3;
        while ((1 << cs) < vpr) ++cs;              // lanes per row rounded up to a power of two
        const int c_raw = tid & ((1 << cs) - 1);
        const int c = c_raw < vpr ? c_raw : vpr - 1;
        const int r_first = tid >> cs, rstep = THREADS >> cs;
        const int n_it = BM / rstep;
        for (int i0 = 0; i0 < n_it; i0 += 4) {
            Vec16<T> buf[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int r = r_first + (i0 + j) * rstep;
                r = r < BM ? r : BM - 1;
                buf[j] = ld16(A + tab.off[r] + c * VEC);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int r = r_first + (i0 + j) * rstep;
                if (r < BM && c_raw < vpr) *reinterpret_cast<Vec16<T>*>(sA + r * AP + c * 16) = buf[j];
            }
        }
    } else {
        // element (m, k) at a + k * a_cs + rowoff(m): read runs of VEC rows, scatter into [row][k]
        constexpr int RPV = BM / VEC;              // VEC-row runs per channel (a power of two)
        const int n_it = K * RPV / THREADS;        // K % 32 == 0  =>  a multiple of 4 (bf16) / 2... see below
        // uniform fast-path test: every run of VEC rows of this slab is contiguous and 16-byte aligned
        const bool fast = d.a_si == 1 && m0 + BM <= M && (d.a_inner % VEC) == 0 && (d.a_so % VEC) == 0 &&
                          (d.a_cs % VEC) == 0 && (m0 % VEC) == 0;
        if (fast) {
            for (int i0 = 0; i0 < n_it; i0 += 4) {
                Vec16<T> buf[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int v = tid + THREADS * (i0 + j);
                    v = v < K * RPV ? v : K * RPV - 1;
                    const int k = v / RPV, r0 = (v % RPV) * VEC;
                    buf[j] = ld16(A + (long)k * d.a_cs + tab.off[r0]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = tid + THREADS * (i0 + j);
                    const int k = v / RPV, r0 = (v % RPV) * VEC;
                    if (v < K * RPV) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) *reinterpret_cast<T*>(sA + (r0 + e) * AP + k * ES) = buf[j].e[e];
                    }
                }
            }
        } else {
            for (int v = tid; v < K * BM; v += THREADS) {
                const int k = v / BM, r = v % BM;
                *reinterpret_cast<T*>(sA + r * AP + k * ES) = A[(long)k * d.a_cs + tab.off[r]];
            }
        }
    }
    lds_barrier();

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
            lds_barrier();
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
        const int prow = wm * 32 + l32;                         // row within the slab
        const long mrow = m0 + prow;
        T bv[CT][4][4];
        if (t.bias) {
            const T* bias = (const T*)t.bias;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const T* bp = bias + (wn * CT + ct) * 32 + 8 * g + 4 * half;
                    if (ES == 2) *reinterpret_cast<u32x2*>(&bv[ct][g][0]) = *reinterpret_cast<const u32x2*>(bp);
                    else *reinterpret_cast<u32x4*>(&bv[ct][g][0]) = *reinterpret_cast<const u32x4*>(bp);
                }
        } else {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e) bv[ct][g][e] = DT<T>::from_f(0.0f);
        }
        float rmask = 1.0f;
        if (t.rowmask) {
            long mr = mrow < M ? mrow : M - 1;
            const unsigned hi = (unsigned)mr / (unsigned)t.inner;
            const unsigned lo = (unsigned)mr - hi * (unsigned)t.inner;
            rmask = DT<T>::to_f(((const T*)t.rowmask)[(long)hi * t.m_so + (long)lo * t.m_si]);
        }
        lds_barrier();                                        // all waves done with the ring
        fill_rowtab(tab, tid, BM, m0, M, t.inner, t.s_o, t.s_i);
        {
            const float scl = t.scale * rmask;
            unsigned char* crow = mode_c ? sC + prow * CP : sC + prow * ES;
            const int chan0 = wn * CT * 32 + 4 * half;
            if (t.glu) {
                stage_tile<T, CT, 1, 0>(acc, bv, scl, crow, mode_c, wn * CT * 16 + 4 * half, CPT);
            } else if (t.act == FFK_ACT_RELU) {
                stage_tile<T, CT, 0, FFK_ACT_RELU>(acc, bv, scl, crow, mode_c, chan0, CPT);
            } else if (t.act == FFK_ACT_SIGMOID) {
                stage_tile<T, CT, 0, FFK_ACT_SIGMOID>(acc, bv, scl, crow, mode_c, chan0, CPT);
            } else {
                stage_tile<T, CT, 0, FFK_ACT_NONE>(acc, bv, scl, crow, mode_c, chan0, CPT);
            }
        }
        lds_barrier();

        T* out = (T*)t.out;
        const int ncols = t.ncols;
        if (mode_c) {
            constexpr int VPR = NT / VEC;
            constexpr int N_IT = BM * VPR / THREADS;             // = 8
            const bool qk = t.kind == FFK_TILE_QK;
            const T* gate = (const T*)t.gate;
            const T* resid = (const T*)t.resid;
            int8_t* xtail = nullptr;                           // extended residual stream (bf16, with resid)
            if constexpr (XS_OK) xtail = (int8_t*)t.xtail;
            const int c_last = ncols >= VEC ? ((ncols - VEC) / VEC) * VEC : 0;   // last full vector column
#pragma unroll 1
            for (int i0 = 0; i0 < N_IT; i0 += 4) {
                Vec16<T> x[4], gv[4], rv[4];
                u32x2 tv[4];
                long o[4];
                // issue every load of the batch first (clamped, branch-free), then combine and store
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = tid + THREADS * (i0 + j);
                    const int r = v / VPR;
                    int c = (v % VPR) * VEC;
                    c = c + VEC <= ncols ? c : c_last;
                    if (qk) {
                        const int n = tab.lo[r];
                        o[j] = (long)tab.hi[r] * t.s_o + (long)(c >> 5) * t.s_h + (long)(n >> 5) * 1024 +
                               qk_tile_off(n & 31, c & 31);
                    } else {
                        o[j] = tab.off[r] + (long)(c >> 5) * t.s_h + (c & 31);
                    }
                    x[j] = *reinterpret_cast<const Vec16<T>*>(sC + r * CP + c * ES);
                    long mr = m0 + r;
                    mr = mr < M ? mr : M - 1;
                    if (gate) gv[j] = ld16(gate + (t.gate_rows > 0 ? mr % t.gate_rows : mr) * t.gate_ld + c);
                    if (resid) rv[j] = ld16(resid + o[j]);
                    if (xtail) tv[j] = *reinterpret_cast<const u32x2*>(xtail + o[j]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = tid + THREADS * (i0 + j);
                    const int r = v / VPR, c = (v % VPR) * VEC;
                    if (gate) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            x[j].e[e] = DT<T>::from_f(DT<T>::to_f(x[j].e[e]) * DT<T>::to_f(gv[j].e[e]));
                    }
                    if constexpr (XS_OK) {
                        if (xtail) {
                            float f[8];
                            xs_decode8(*reinterpret_cast<const u32x4*>(&rv[j]), tv[j][0], tv[j][1], f);
#pragma unroll
                            for (int e = 0; e < 8; ++e) f[e] += (float)x[j].e[e];
                            u32x4 hv;
                            u32x2 tn;
                            xs_encode8(f, hv, tn);
                            if (m0 + r < M && c + VEC <= ncols) {
                                *reinterpret_cast<u32x4*>(out + o[j]) = hv;
                                *reinterpret_cast<u32x2*>(xtail + o[j]) = tn;
                            }
                            continue;
                        }
                    }
                    if (resid) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            x[j].e[e] = DT<T>::from_f(DT<T>::to_f(x[j].e[e]) + DT<T>::to_f(rv[j].e[e]));
                    }
                    if (m0 + r < M && c + VEC <= ncols) st16(out + o[j], x[j]);
                }
            }
            if (ncols % VEC != 0) {
                // ragged tail (fewer than VEC channels left): element-wise, rare
                const int c0 = (ncols / VEC) * VEC, nrem = ncols - c0;
                for (int v = tid; v < BM * nrem; v += THREADS) {
                    const int r = v / nrem, c = c0 + v % nrem;
                    if (m0 + r >= M) continue;
                    float y = DT<T>::to_f(*reinterpret_cast<const T*>(sC + r * CP + c * ES));
                    long oo;
                    if (qk) {
                        const int n = tab.lo[r];
                        oo = (long)tab.hi[r] * t.s_o + (long)(c >> 5) * t.s_h + (long)(n >> 5) * 1024 + qk_tile_off(n & 31, c & 31);
                    } else {
                        oo = tab.off[r] + (long)(c >> 5) * t.s_h + (c & 31);
                    }
                    if (gate) y = DT<T>::to_f(DT<T>::from_f(y * DT<T>::to_f(gate[(t.gate_rows > 0 ? (m0 + r) % t.gate_rows : (m0 + r)) * t.gate_ld + c])));
                    if constexpr (XS_OK) {
                        if (xtail) {
                            xs_round(y + xs_value(resid[oo], xtail[oo]), &out[oo], &xtail[oo]);
                            continue;
                        }
                    }
                    if (resid) y += DT<T>::to_f(resid[oo]);
                    out[oo] = DT<T>::from_f(y);
                }
            }
        } else {
            constexpr int QPR = BM / 4;                         // 4-row runs per channel
            for (int v = tid; v < ncols * QPR; v += THREADS) {
                const int c = v / QPR, r = (v % QPR) * 4;
                if (m0 + r >= M) continue;
                const T* src = reinterpret_cast<const T*>(sC + c * CPT + r * ES);
                long o[4];
                bool ok[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ok[e] = m0 + r + e < M;
                    const int hi = tab.hi[r + e], lo = tab.lo[r + e];
                    if (t.kind == FFK_TILE_V) {
                        o[e] = (long)hi * t.s_o + (long)(c >> 5) * t.s_h + (long)(lo >> 5) * 1024 + acc_tile_off(lo & 31, c & 31);
                    } else if (t.kind == FFK_TILE_ACC) {
                        o[e] = (long)hi * t.s_o + (long)(c >> 5) * t.s_h + (long)(lo >> 5) * 1024 + acc_tile_off(c & 31, lo & 31);
                    } else if (t.kind == FFK_TILE_BIAS) {
                        // logical row = (query hi, key lo); channel = head
                        o[e] = (long)c * t.s_h + (long)(hi >> 5) * t.s_o + (long)(lo >> 5) * 1024 +
                               qk_tile_off(lo & 31, hi & 31);
                    } else {
                        o[e] = tab.off[r + e] + (long)(c >> 5) * t.s_h + (long)(c & 31) * t.s_d;
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
        lds_barrier();                                        // staging area is the ring again
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
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)fused_linear_kernel<T>, smem, "ffk_fused_linear");
        if (rc_lds != FFK_OK) return rc_lds;
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
    const int bk = 32;
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
    FFK_REQUIRE(d->ln_folded || !d->ln_gamma || d->ln_beta, FFK_ERR_NULL, "ffk_fused_linear: ln_beta missing");
    FFK_REQUIRE((d->ln_folded != 0) == (d->a2 != nullptr), FFK_ERR_UNSUPPORTED,
                "ffk_fused_linear: the second operand and folded LayerNorms (ln_folded) go together");
    if (d->a2) {
        FFK_REQUIRE(d->ln_gamma, FFK_ERR_NULL, "ffk_fused_linear: folded LayerNorms need the row-sum table in ln_gamma");
        FFK_REQUIRE(d->a2_inner > 0, FFK_ERR_SHAPE, "ffk_fused_linear: a2_inner must be positive");
        FFK_REQUIRE(ffk_aligned16(d->a2) && (d->a2_so * es) % 16 == 0 && (d->a2_si * es) % 16 == 0,
                    FFK_ERR_ALIGN, "ffk_fused_linear: rows of the second operand must be 16-byte aligned");
    }
    for (int i = 0; i < d->n_tiles; ++i) {
        const ffk_tile& t = d->tiles[i];
        FFK_REQUIRE(t.out, FFK_ERR_NULL, "ffk_fused_linear: tile %d has no output", i);
        FFK_REQUIRE(t.inner > 0 && t.ncols > 0 && t.ncols <= (t.glu ? 64 : 128), FFK_ERR_SHAPE,
                    "ffk_fused_linear: tile %d: bad inner/ncols (%d, %d)", i, t.inner, t.ncols);
        FFK_REQUIRE(t.kind >= FFK_TILE_STRIDED && t.kind <= FFK_TILE_ACC, FFK_ERR_UNSUPPORTED,
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
        FFK_REQUIRE(!t.xtail || (d->dtype == FFK_BF16 && t.resid && t.kind == FFK_TILE_STRIDED && t.s_d == 1),
                    FFK_ERR_UNSUPPORTED, "ffk_fused_linear: tile %d: a residual tail needs bf16, resid and a [row][channel] tile", i);
        FFK_REQUIRE(ffk_aligned16(t.xtail), FFK_ERR_ALIGN, "ffk_fused_linear: tile %d: residual tail alignment", i);
    }
    // Two kernel variants.  Launches whose tiles are all stored channel-contiguous (plain, gated,
    // residual and q/k tiles) use the slab-persistent kernel (128-row slabs, register prefetch of the
    // next slab and of whole weight tiles); launches with row-contiguous tiles (v / bias tiles,
    // channel-major stores) use the 64-row kernel below, whose smaller LDS footprint keeps four
    // workgroups per CU in flight and hides the longer store phase of those tiles.
    bool all_c = d->dtype == FFK_BF16 && !d->a_chanmajor;
    for (int i = 0; i < d->n_tiles; ++i) {
        const ffk_tile& t = d->tiles[i];
        all_c = all_c && ((t.kind == FFK_TILE_STRIDED && t.s_d == 1) || t.kind == FFK_TILE_QK);
    }
    {
        int status = FFK_OK;
        if (ffk_linear_ws_try(d, (hipStream_t)stream, &status)) return status;
    }
    FFK_REQUIRE(!d->a2, FFK_ERR_UNSUPPORTED,
                "ffk_fused_linear: a second operand needs bf16, K = 128, a channel-major first operand and GLU tiles only");
    if (all_c) return ffk_linear_slab_launch(d, (hipStream_t)stream);
    switch (d->dtype) {
        case FFK_BF16: return launch_linear<bf16_t>(*d, (hipStream_t)stream);
        case FFK_F32: return launch_linear<float>(*d, (hipStream_t)stream);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_fused_linear: unsupported dtype tag %d", d->dtype);
    }
}
