// Fused linear layer, slab-persistent variant (see ffk_fused_linear in include/ffk.h and
// ffk_linear.hip, which holds the argument checks and picks between the two variants).
//
// Persistent workgroups (4 wavefronts) walk over slabs of BM = 64 rows of A.  The whole
// [BM x K] slab (K <= 256) is staged in LDS once - read from HBM exactly once - optionally
// LayerNorm-ed in place, and then multiplied against every 128-row tile of the weight matrix.
// The next slab is prefetched into registers while the current one is being processed, and
// each weight tile (128 rows x 256 bytes of K) is prefetched into registers during the MFMAs
// and epilogue of the previous tile; weights are a few hundred KB and stay in L2.  All global
// loads are issued without per-lane branches (indices are clamped) so they overlap.
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
    static constexpr int BM = 128;                  // rows of A per slab
    static constexpr int WM = 4, WN = 1;            // wave grid: 32 rows x 128 channels per wave
    static constexpr int KC = 128;                  // K elements per weight chunk (256 bytes per row)
};
template <> struct LinCfg<float> {
    static constexpr int BM = 64;
    static constexpr int WM = 2, WN = 2;            // 32 rows x 64 channels per wave
    static constexpr int KC = 64;
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

// NA: 16-byte vectors of A each thread prefetches for the next slab (8), or 0 = the slab is
// loaded at the start of its own iteration (channel-major A, or rows too long to keep in registers).
template <typename T, int NA>
__global__ __launch_bounds__(THREADS, 2) void fused_linear_slab_kernel(const LinArgs args) {
    typedef LinCfg<T> Cfg;
    typedef Mma<T> MM;
    constexpr int BM = Cfg::BM, WN = Cfg::WN, KC = Cfg::KC;
    constexpr int CT = NT / (WN * 32);             // 32-channel MFMA tiles per wave (= 2)
    constexpr int VEC = DT<T>::VEC;
    constexpr int ES = sizeof(T);
    constexpr bool XS_OK = std::is_same<T, bf16_t>::value;     // outputs that may carry a residual tail
    constexpr int WP = KC * ES + 16;               // weight chunk row pitch (bytes)
    constexpr int WBUF = NT * WP;
    constexpr int CP = NT * ES + 16;               // staged C pitch, [row][channel]
    constexpr int CPT = BM * ES + 16;              // staged C pitch, [channel][row]
    constexpr int WV = NT * (KC / VEC) / THREADS;  // weight vectors per thread per chunk (= 8)
    constexpr int NAR = NA > 0 ? NA : 1;
    static_assert(BM * CP <= WBUF && NT * CPT <= WBUF, "C staging must fit in the weight buffer");

    const ffk_linear_desc& d = args.d;
    const int K = d.K, M = d.M;
    const int AP = K * ES + 16;                    // A slab row pitch (bytes)
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ RowTab tab;
    unsigned char* sA = smem;
    unsigned char* sW = smem + (size_t)BM * AP;
    unsigned char* sC = sW;                        // the staged output tile aliases the weight buffer

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, half = lane >> 5;
    const T* A = (const T*)d.a;
    const T* W = (const T*)d.w;
    const int n_slabs = (M + BM - 1) / BM;

    // ---- weight chunks: whole 128 x KC chunk prefetched into registers ----
    const int n_kc = (K + KC - 1) / KC;
    const int chunks_per_slab = d.n_tiles * n_kc;
    Vec16<T> wreg[WV];
    // Workgroups that share a CU would otherwise run the same phase (load, MFMA, store) at the same
    // time; odd workgroups walk the N-tiles starting from the middle so that their phases interleave.
    const int rot = (blockIdx.x & 1) ? d.n_tiles / 2 : 0;
    auto w_fetch = [&](int chunk) {                // chunk index within a slab
        int nt = chunk / n_kc;
        const int kc = chunk - nt * n_kc;
        nt = nt + rot < d.n_tiles ? nt + rot : nt + rot - d.n_tiles;
        const int kv = (K - kc * KC < KC ? K - kc * KC : KC) / VEC;   // vectors per row in this chunk
#pragma unroll
        for (int i = 0; i < WV; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (KC / VEC);
            int c = v % (KC / VEC);
            c = c < kv ? c : kv - 1;
            wreg[i] = ld16(W + ((long)nt * NT + r) * K + kc * KC + c * VEC);
        }
    };
    auto w_commit = [&](int kc) {
        const int kv = (K - kc * KC < KC ? K - kc * KC : KC) / VEC;
#pragma unroll
        for (int i = 0; i < WV; ++i) {
            const int v = tid + THREADS * i;
            const int r = v / (KC / VEC), c = v % (KC / VEC);
            if (c < kv) *reinterpret_cast<Vec16<T>*>(sW + r * WP + c * 16) = wreg[i];
        }
    };

    // ---- A slab: row-major rows are prefetched one slab ahead into registers ----
    const int vpr = K / VEC;                       // 16-byte vectors per row
    int cs = 3;
    while ((1 << cs) < vpr) ++cs;                  // lanes per row rounded up to a power of two
    const int a_c_raw = tid & ((1 << cs) - 1);
    const int a_c = a_c_raw < vpr ? a_c_raw : vpr - 1;
    const int a_r_first = tid >> cs, a_rstep = THREADS >> cs;
    const bool a_plain = d.a_inner >= M;           // one contiguous group: no division needed
    Vec16<T> areg[NAR];
    auto a_fetch = [&](int slab) {
#pragma unroll
        for (int i = 0; i < NAR; ++i) {
            int r = a_r_first + i * a_rstep;
            r = r < BM ? r : BM - 1;
            long m = (long)slab * BM + r;
            m = m < M ? m : M - 1;
            long off;
            if (a_plain) {
                off = m * d.a_si;
            } else {
                const unsigned hi = (unsigned)m / (unsigned)d.a_inner;
                const unsigned lo = (unsigned)m - hi * (unsigned)d.a_inner;
                off = (long)hi * d.a_so + (long)lo * d.a_si;
            }
            areg[i] = ld16(A + off + a_c * VEC);
        }
    };
    auto a_commit = [&]() {
#pragma unroll
        for (int i = 0; i < NAR; ++i) {
            const int r = a_r_first + i * a_rstep;
            if (r < BM && a_c_raw < vpr) *reinterpret_cast<Vec16<T>*>(sA + r * AP + a_c * 16) = areg[i];
        }
    };

    if (NA > 0) a_fetch(blockIdx.x);
    w_fetch(0);

    for (int slab = blockIdx.x; slab < n_slabs; slab += gridDim.x) {
        const long m0 = (long)slab * BM;
        lds_barrier();                           // previous slab completely finished (sA, sC, tab free)
        if (NA > 0) {
            a_commit();
            if (slab + (int)gridDim.x < n_slabs) a_fetch(slab + gridDim.x);
        } else {
            fill_rowtab(tab, tid, BM, m0, M, d.a_inner, d.a_so, d.a_si);
            lds_barrier();
            if (!d.a_chanmajor) {
                const int n_it = BM / a_rstep;
                for (int i0 = 0; i0 < n_it; i0 += 4) {
                    Vec16<T> buf[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        int r = a_r_first + (i0 + j) * a_rstep;
                        r = r < BM ? r : BM - 1;
                        buf[j] = ld16(A + tab.off[r] + a_c * VEC);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int r = a_r_first + (i0 + j) * a_rstep;
                        if (r < BM && a_c_raw < vpr) *reinterpret_cast<Vec16<T>*>(sA + r * AP + a_c * 16) = buf[j];
                    }
                }
            } else {
                // element (m, k) at a + k * a_cs + rowoff(m): read runs of VEC rows, scatter into [row][k]
                constexpr int RPV = BM / VEC;
                const int n_it = (K * RPV + THREADS - 1) / THREADS;
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
                                for (int e = 0; e < VEC; ++e)
                                    *reinterpret_cast<T*>(sA + (r0 + e) * AP + k * ES) = buf[j].e[e];
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
        }
        lds_barrier();

        // ---- LayerNorm prologue, in place ----
        if (d.ln_gamma) {
            constexpr int TPR = THREADS / BM;      // threads per row (adjacent lanes)
            const int r = tid / TPR, j = tid % TPR;
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
            // made visible to the other waves by the first barrier of the tile loop
        }

        // ---- N-tiles ----
        const unsigned char* a_frag_base = sA + (wm * 32 + l32) * AP + half * (MM::KLANE * ES);
        const unsigned char* w_frag_base = sW + (wn * CT * 32 + l32) * WP + half * (MM::KLANE * ES);
        int chunk = 0;
        for (int nt0 = 0; nt0 < d.n_tiles; ++nt0) {
            const int nt = nt0 + rot < d.n_tiles ? nt0 + rot : nt0 + rot - d.n_tiles;
            const ffk_tile& t = d.tiles[nt];
            const bool mode_c = (t.kind == FFK_TILE_STRIDED && t.s_d == 1) || t.kind == FFK_TILE_QK;
            const int prow = wm * 32 + l32;                     // row within the slab
            // bias (4 consecutive channels per load) and row mask of this lane, fetched ahead of use
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
                long mrow = m0 + prow;
                mrow = mrow < M ? mrow : M - 1;
                const unsigned hi = (unsigned)mrow / (unsigned)t.inner;
                const unsigned lo = (unsigned)mrow - hi * (unsigned)t.inner;
                rmask = DT<T>::to_f(((const T*)t.rowmask)[(long)hi * t.m_so + (long)lo * t.m_si]);
            }

            f32x16 acc[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[ct][v] = 0.0f;

            for (int kc = 0; kc < n_kc; ++kc, ++chunk) {
                lds_barrier();                   // consumers of the weight buffer / staged tile are done
                w_commit(kc);
                lds_barrier();
                {   // prefetch the next chunk (wraps to chunk 0 for the next slab: same weights)
                    const int nxt = chunk + 1 < chunks_per_slab ? chunk + 1 : 0;
                    w_fetch(nxt);
                }
                const int ksteps = (K - kc * KC < KC ? K - kc * KC : KC) / MM::KSTEP;
                const unsigned char* ab = a_frag_base + kc * KC * ES;
                for (int ks = 0; ks < ksteps; ++ks) {
                    typename MM::Frag fx = *reinterpret_cast<const typename MM::Frag*>(ab + ks * MM::KSTEP * ES);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        typename MM::Frag fw =
                            *reinterpret_cast<const typename MM::Frag*>(w_frag_base + ct * 32 * WP + ks * MM::KSTEP * ES);
                        MM::mma(acc[ct], fw, fx);
                    }
                }
            }

            // ---- epilogue of this tile ----
            lds_barrier();                                    // all waves done with the weight buffer
            fill_rowtab(tab, tid, BM, m0, M, t.inner, t.s_o, t.s_i);
            // the activation variant is selected once per tile; each variant is straight-line code
            {
                const float scl = t.scale * rmask;
                unsigned char* crow = mode_c ? sC + prow * CP : sC + prow * ES;
                const int chan0 = wn * CT * 32 + 4 * half;
                if (t.glu) {        // pairs of MFMA tiles collapse to one: half as many output channels
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
                constexpr int N_IT = BM * VPR / THREADS;
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
        }
    }
}

template <typename T, int NA>
int launch_linear_na(const ffk_linear_desc& d, size_t smem, hipStream_t st) {
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)fused_linear_slab_kernel<T, NA>, smem, "ffk_fused_linear");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    LinArgs a;
    a.d = d;
    const int n_slabs = ffk_cdiv(d.M, LinCfg<T>::BM);
    // persistent workgroups: as many as can be resident (LDS-limited), each walks slabs with stride gridDim
    const int per_cu = (int)(160 * 1024 / (smem + 2048));
    int resident = 256 * (per_cu < 1 ? 1 : (per_cu > 2 ? 2 : per_cu));   // 2 waves per SIMD (register budget)
    dim3 grid(n_slabs < resident ? n_slabs : resident);
    fused_linear_slab_kernel<T, NA><<<grid, THREADS, smem, st>>>(a);
    return ffk_check_launch("ffk_fused_linear");
}

template <typename T>
int launch_linear(const ffk_linear_desc& d, hipStream_t st) {
    typedef LinCfg<T> Cfg;
    constexpr int ES = sizeof(T);
    const size_t smem = (size_t)Cfg::BM * (d.K * ES + 16) + (size_t)NT * (Cfg::KC * ES + 16);
    // vectors of A per thread for a one-slab-ahead prefetch
    const int vpr = d.K / (16 / ES);
    int cs = 3;
    while ((1 << cs) < vpr) ++cs;
    const int n_it = Cfg::BM / (THREADS >> cs);
    if (d.a_chanmajor || n_it > 8) return launch_linear_na<T, 0>(d, smem, st);
    return launch_linear_na<T, 8>(d, smem, st);
}

}  // namespace

// Entry used by ffk_fused_linear for launches whose tiles are all channel-contiguous (see there).
int ffk_linear_slab_launch(const ffk_linear_desc* d, hipStream_t st) {
    switch (d->dtype) {
        case FFK_BF16: return launch_linear<bf16_t>(*d, st);
        case FFK_F32: return launch_linear<float>(*d, st);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_fused_linear: unsupported dtype tag %d", d->dtype);
    }
}
