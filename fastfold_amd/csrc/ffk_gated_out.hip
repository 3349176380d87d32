// Gated output stage of an attention (see ffk_gated_out_fused in include/ffk.h):
//     out = x + Wo . ( sigmoid( Wg . LayerNorm(x) + bg ) * o ) + bo          (bf16; C = 128 or 256 channels, as many gate channels)
// x is the tensor the attention updates (its rows are also the rows the gate is computed from), o the heads' weighted
// averages in logical row order.  The gate never exists in memory: it is the hidden layer of a two-layer product whose
// first layer is the gate projection and whose second layer is the output projection, built like the fused transition
// (ffk_transition.hip).
//
// A workgroup (4 wavefronts) owns 128 logical rows, a wavefront 32 of them from start to end.  Set-up: the rows of x
// are fetched once (row m at (m / inner) * s_o + (m % inner) * s_i: the transposed traversals of the column-wise
// attentions are strides), normalised in registers and passed through LDS into the MFMA fragments of their wave.  The
// gate channels are walked in chunks of 32 (the rings then take 32 KB at C = 128, the kernel 162 registers: three
// workgroups share a CU and cover each other's set-up and epilogue, which are half of a workgroup's life); per chunk and wave
//   first GEMM   G^T[gate channel, rows] = Wg[chunk] . x^T + bg, sigmoid, times o: lane = row, registers = gate
//                channels, so the sixteen values of o a lane needs per 32-channel tile are two 16-byte pieces of its row;
//   second GEMM  out^T[c, rows] += Wo[c, chunk] . (G * o)^T: the rounded products are the N operand as they stand
//                (weight rows of the first GEMM are fetched through the permutation sigma, see ffk_transition.hip).
// Only the weights go through LDS (direct global -> LDS loads, XOR-swizzled unpadded rows, one chunk ahead).
#include "ffk_common.h"

namespace {

typedef bf16_t T;
constexpr int GO_THREADS = 256;
constexpr int GO_BM = 128;                     // rows per workgroup
constexpr int GO_NS = 2;                       // slots of the weight rings
template <int C> struct GoGeo {
    static constexpr int H = C;                     // gate channels (heads x 32)
    static constexpr int HC = 32;                   // gate channels per chunk
    static constexpr int NCHUNK = H / HC;
    static constexpr int W1SLOT = HC * C * 2;       // HC rows of 2 C bytes (16 KB)
    static constexpr int W2SLOT = C * HC * 2;       // C rows of 2 HC bytes (16 KB)
    static constexpr int XP = C * 2 + 16;           // pitch of the normalised rows (set-up only)
    static constexpr int NC1 = C / 8;               // 16-byte columns of a W1 row
    static constexpr int NC2 = HC / 8;              // 16-byte columns of a W2 row
    static constexpr int RP2 = 256 / (HC * 2);      // W2 rows per 256 bytes of LDS: the swizzle period
    static constexpr int KS1 = C / 16, KS2 = HC / 16, HT = HC / 32, CT = C / 32;
    static constexpr size_t SMEM_RINGS = GO_NS * (size_t)W1SLOT + GO_NS * W2SLOT + H * sizeof(float);
    static constexpr size_t SMEM_ROWS = (size_t)GO_BM * XP;
    static constexpr int NLD = W1SLOT / 16 / GO_THREADS;   // 16-byte requests per thread and ring slot
    static_assert(W1SLOT == W2SLOT, "ring slots of one size");
    static constexpr size_t SMEM = SMEM_RINGS > SMEM_ROWS ? SMEM_RINGS : SMEM_ROWS;
};

__device__ __forceinline__ int go_tau(int i) { return ((i >> 2) & 1) * 16 + (i >> 3) * 4 + (i & 3); }
// i = 8a + 4h + b  ->  16 (a / 2) + 8h + 4 (a % 2) + b
__device__ __forceinline__ int go_sigma(int i) { return (i >> 4) * 16 + ((i >> 2) & 1) * 8 + ((i >> 3) & 1) * 4 + (i & 3); }

__device__ __forceinline__ void go_load_lds(const T* src, unsigned char* dst_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst_wave, 16, 0, 0);
}

template <int GO_C>
__global__ __launch_bounds__(GO_THREADS, GO_C == 128 ? 3 : 2) void gated_out_kernel(T* __restrict__ out, const T* __restrict__ x, int8_t* __restrict__ xtail,
                                                                 const T* __restrict__ gamma, const T* __restrict__ beta,
                                                                 const T* __restrict__ w1, const T* __restrict__ b1,
                                                                 const T* __restrict__ o, const T* __restrict__ w2,
                                                                 const T* __restrict__ b2, long M, unsigned inner, long s_o,
                                                                 long s_i, float eps) {
    typedef Mma<T> MM;
    typedef GoGeo<GO_C> G;
    constexpr int NS = GO_NS;
    constexpr int NLD = G::NLD;
    constexpr int GO_H = G::H, GO_HC = G::HC, GO_NCHUNK = G::NCHUNK, GO_W1SLOT = G::W1SLOT, GO_W2SLOT = G::W2SLOT, GO_XP = G::XP;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_w1 = smem;                           // [NS][HC][2 C bytes]
    unsigned char* s_w2 = smem + NS * GO_W1SLOT;          // [NS][C][2 HC bytes]
    float* s_b1 = reinterpret_cast<float*>(s_w2 + NS * GO_W2SLOT);  // [H]
    unsigned char* s_x = smem;                            // [128][GO_XP], set-up only (aliases the rings)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const long m0 = (long)blockIdx.x * GO_BM;
    const bool flat = (long)inner >= M;                   // plain row-major: no division per row
    auto row_off = [&](long m) -> long {
        if (flat) return m * s_i;
        const unsigned hi = (unsigned)m / inner, lo = (unsigned)m - hi * inner;
        return (long)hi * s_o + (long)lo * s_i;
    };

    // ---- set-up: rows -> LayerNorm in registers -> LDS -> this wave's fragments ----
    {
        constexpr int LPR = GO_C / 8, RPP = GO_THREADS / LPR, NPASS = GO_BM / RPP;   // lanes per row, rows per pass
        const int c8 = tid % LPR, r0 = tid / LPR;
        const Vec16<T> g = ld16(gamma + c8 * 8), b = ld16(beta + c8 * 8);
#pragma unroll
        for (int i0 = 0; i0 < NPASS; i0 += 8) {
            Vec16<T> v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                long m = m0 + r0 + RPP * (i0 + i);
                m = m < M ? m : M - 1;                    // clamped: rows past the end are never stored
                v[i] = ld16(x + row_off(m) + c8 * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float f[8], s = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] = (float)v[i].e[e];
                    s += f[e];
                }
                const float mu = group_sum(s, LPR) * (1.0f / GO_C);
                float q = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] -= mu;
                    q += f[e] * f[e];
                }
                const float rs = rsqrtf(group_sum(q, LPR) * (1.0f / GO_C) + eps);
                Vec16<T> y;
#pragma unroll
                for (int e = 0; e < 8; ++e) y.e[e] = (T)(f[e] * rs * (float)g.e[e] + (float)b.e[e]);
                *reinterpret_cast<Vec16<T>*>(s_x + (r0 + RPP * (i0 + i)) * GO_XP + c8 * 16) = y;
            }
        }
    }
    lds_barrier();
    bf16x8 xf[G::KS1];                                     // rows 32 wave + l32, all of K = C
#pragma unroll
    for (int ks = 0; ks < G::KS1; ++ks)
        xf[ks] = *reinterpret_cast<const bf16x8*>(s_x + (wave * 32 + l32) * GO_XP + ks * 32 + half * 16);
    lds_barrier();                                         // the row buffer is free: the rings may overwrite it
    // gate bias, pre-multiplied for the exp2 form of the sigmoid
    for (int i = tid; i < GO_H; i += GO_THREADS) s_b1[i] = -1.4426950408889634f * (float)b1[i];

    // this lane's row, and its share of o: per 32-channel tile the pieces [8 half, 8 half + 8) and [16 + 8 half, 16 + 8 half + 8)
    const long row = m0 + wave * 32 + l32;
    const bool ok = row < M;
    const long rc = ok ? row : M - 1;
    const T* orow = o + rc * GO_H + 8 * half;

    // ---- chunk loaders (direct to LDS; lane L of a wave lands at dst + 16 L) ----
    // W1 chunk: LDS row rho (0..HC-1) holds weight row 32 * (rho / 32) + sigma(rho % 32) of the chunk
    const T* w1src[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int v = i * GO_THREADS + tid, rho = v / G::NC1, c = v % G::NC1;
        w1src[i] = w1 + (long)((rho & ~31) + go_sigma(rho & 31)) * GO_C + ((c ^ (rho & 15)) * 8);
    }
    // W2 chunk: LDS row rho (0..C-1) holds weight row 32 * (rho / 32) + tau(rho % 32)
    const T* w2src[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int v = i * GO_THREADS + tid, rho = v / G::NC2, c = v % G::NC2;
        w2src[i] = w2 + (long)((rho & ~31) + go_tau(rho & 31)) * GO_H + ((c ^ ((rho / G::RP2) & (G::NC2 - 1))) * 8);
    }
    auto fetch = [&](int q) {                              // past the last chunk it is fetched again (into a free slot)
        const int qc = q < GO_NCHUNK ? q : GO_NCHUNK - 1;
        unsigned char* d1 = s_w1 + (q % NS) * GO_W1SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < NLD; ++i) go_load_lds(w1src[i] + (long)qc * GO_HC * GO_C, d1 + i * (GO_THREADS * 16));
        unsigned char* d2 = s_w2 + (q % NS) * GO_W2SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < NLD; ++i) go_load_lds(w2src[i] + qc * GO_HC, d2 + i * (GO_THREADS * 16));
    };

    f32x16 acc2[G::CT];                                    // out^T tiles: channels 32 ct + 16 half + v, row l32
#pragma unroll
    for (int c = 0; c < G::CT; ++c) {                      // start from bo: the epilogue has no bias to add
        if (b2) {
            const Vec16<T> b0 = ld16(b2 + c * 32 + 16 * half), b1v = ld16(b2 + c * 32 + 16 * half + 8);
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                acc2[c][v] = (float)b0.e[v];
                acc2[c][8 + v] = (float)b1v.e[v];
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc2[c][v] = 0.0f;
        }
    }

    int w1off[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) w1off[ks] = l32 * (GO_C * 2) + (((2 * ks + half) ^ (l32 & 15)) << 4);
    int w2off[G::KS2];                                     // W2 fragment of c-tile 0: row l32, column 2 ks + half
#pragma unroll
    for (int ks = 0; ks < G::KS2; ++ks) w2off[ks] = l32 * (GO_HC * 2) + (((2 * ks + half) ^ ((l32 / G::RP2) & (G::NC2 - 1))) << 4);

    fetch(0);
    // The o pieces of a chunk are requested one chunk ahead, like its weights, where the registers allow it (C = 128);
    // at C = 256 (248 registers in the products alone) they are requested at the top of their own chunk, before the wait.
    constexpr bool AHEAD = GO_C == 128;
    Vec16<T> ov[G::HT][2];
    if (AHEAD) {
#pragma unroll
        for (int ht = 0; ht < G::HT; ++ht) {
            ov[ht][0] = ld16(orow + ht * 32);
            ov[ht][1] = ld16(orow + ht * 32 + 16);
        }
    }
    for (int q = 0; q < GO_NCHUNK; ++q) {
        if (!AHEAD) {
#pragma unroll
            for (int ht = 0; ht < G::HT; ++ht) {
                ov[ht][0] = ld16(orow + q * GO_HC + ht * 32);
                ov[ht][1] = ld16(orow + q * GO_HC + ht * 32 + 16);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // chunk q has landed (this wave's part), and its o pieces
        __builtin_amdgcn_s_barrier();                        // ... everyone's; nobody still reads the slot of chunk q - 1
        Vec16<T> ovn[AHEAD ? G::HT : 1][2];
        if (q + 1 < GO_NCHUNK) {
            fetch(q + 1);
            if (AHEAD) {
#pragma unroll
                for (int ht = 0; ht < G::HT; ++ht) {
                    ovn[ht][0] = ld16(orow + (q + 1) * GO_HC + ht * 32);
                    ovn[ht][1] = ld16(orow + (q + 1) * GO_HC + ht * 32 + 16);
                }
            }
        }
        const unsigned char* wa = s_w1 + (q % NS) * GO_W1SLOT;
        const unsigned char* wb = s_w2 + (q % NS) * GO_W2SLOT;
        bf16x8 hf[G::HT][2];                               // [gate tile][K step]: the chunk's N operand
#pragma unroll
        for (int ht = 0; ht < G::HT; ++ht) {
            f32x16 h;
#pragma unroll
            for (int v = 0; v < 16; ++v) h[v] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < G::KS1; ++ks)
                MM::mma(h, *reinterpret_cast<const bf16x8*>(wa + ht * 32 * (GO_C * 2) + w1off[ks & 7] + (ks >> 3) * 256), xf[ks]);
            // registers 0..7: gate channels 8 half + 0..7 of the tile, registers 8..15: 16 + 8 half + 0..7
            const float* bp = s_b1 + q * GO_HC + ht * 32 + 8 * half;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const f32x4 ba = *reinterpret_cast<const f32x4*>(bp + j * 16), bb = *reinterpret_cast<const f32x4*>(bp + j * 16 + 4);
                bf16x8 r;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const float bs = t < 4 ? ba[t] : bb[t - 4];
                    // sigmoid(h + b) = 1 / (1 + 2^(-log2e h - log2e b)), times the head output
                    const float gte = fast_rcp(1.0f + fast_exp2(__builtin_fmaf(h[8 * j + t], -1.4426950408889634f, bs)));
                    r[t] = (T)(gte * (float)ov[ht][j].e[t]);
                }
                hf[ht][j] = r;
            }
        }
#pragma unroll
        for (int ks = 0; ks < G::KS2; ++ks)
#pragma unroll
            for (int c = 0; c < G::CT; ++c)
                MM::mma(acc2[c], *reinterpret_cast<const bf16x8*>(wb + c * 32 * (GO_HC * 2) + w2off[ks]), hf[ks >> 1][ks & 1]);
        if (AHEAD && q + 1 < GO_NCHUNK) {
#pragma unroll
            for (int ht = 0; ht < G::HT; ++ht) {
                ov[ht][0] = ovn[ht][0];
                ov[ht][1] = ovn[ht][1];
            }
        }
    }

    // ---- epilogue: lane = row, registers = 16 consecutive channels ----
    const long ro = row_off(rc);
#pragma unroll
    for (int c = 0; c < G::CT; ++c) {
        const int ch = c * 32 + 16 * half;
        const long oo = ro + ch;
        u32x4 rv[2];
        rv[0] = *reinterpret_cast<const u32x4*>(x + oo);
        rv[1] = *reinterpret_cast<const u32x4*>(x + oo + 8);
        if (xtail) {           // extended residual stream: the update is added at 24 bits
            const u32x4 tv = *reinterpret_cast<const u32x4*>(xtail + oo);
            float upd[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) upd[v] = (float)(T)acc2[c][v];
            u32x4 h0, h1, tn;
            xs_update16(upd, rv[0], rv[1], tv, h0, h1, tn);
            if (ok) {
                *reinterpret_cast<u32x4*>(out + oo) = h0;
                *reinterpret_cast<u32x4*>(out + oo + 8) = h1;
                *reinterpret_cast<u32x4*>(xtail + oo) = tn;
            }
            continue;
        }
        T y[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            y[v] = (T)((float)(T)acc2[c][v] + (float)reinterpret_cast<const T*>(&rv[v >> 3])[v & 7]);
        }
        if (ok) {
            *reinterpret_cast<u32x4*>(out + oo) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(out + oo + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    }
}

}  // namespace

extern "C" int ffk_gated_out_fused(void* out, const void* x, void* xtail, const void* gamma, const void* beta, const void* wg,
                                   const void* bg, const void* o, const void* wo, const void* bo, int64_t M, int64_t C,
                                   int64_t inner, int64_t s_o, int64_t s_i, float eps, int dtype, void* stream) {
    FFK_REQUIRE(out && x && gamma && beta && wg && bg && o && wo, FFK_ERR_NULL, "ffk_gated_out_fused: null pointer");
    FFK_REQUIRE(dtype == FFK_BF16, FFK_ERR_DTYPE, "ffk_gated_out_fused: bf16 only (dtype tag %d)", dtype);
    FFK_REQUIRE(C == 128 || C == 256, FFK_ERR_UNSUPPORTED, "ffk_gated_out_fused: built for 128 and 256 channels, got %ld", (long)C);
    FFK_REQUIRE(M > 0 && M < (1L << 31) && inner > 0 && inner < (1L << 31), FFK_ERR_SHAPE,
                "ffk_gated_out_fused: bad shape M=%ld inner=%ld", (long)M, (long)inner);
    FFK_REQUIRE(s_o % 16 == 0 && s_i % 16 == 0, FFK_ERR_ALIGN, "ffk_gated_out_fused: row strides must be multiples of 16 elements");
    FFK_REQUIRE(ffk_aligned16(out) && ffk_aligned16(x) && ffk_aligned16(gamma) && ffk_aligned16(beta) && ffk_aligned16(wg) &&
                    ffk_aligned16(wo) && ffk_aligned16(o) && ffk_aligned16(bo) && ffk_aligned16(xtail),
                FFK_ERR_ALIGN, "ffk_gated_out_fused: buffers must be 16-byte aligned");
    const unsigned grid = (unsigned)ffk_cdiv(M, GO_BM);
#define FFK_GO_LAUNCH(CC)                                                                                               \
    do {                                                                                                                \
        static FfkLdsReservation lds_reserved;                                                                          \
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)gated_out_kernel<CC>, GoGeo<CC>::SMEM,            \
                                           "ffk_gated_out_fused");                                                      \
        if (rc_lds != FFK_OK) return rc_lds;                                                                            \
        gated_out_kernel<CC><<<grid, GO_THREADS, GoGeo<CC>::SMEM, (hipStream_t)stream>>>(                               \
            (T*)out, (const T*)x, (int8_t*)xtail, (const T*)gamma, (const T*)beta, (const T*)wg, (const T*)bg, (const T*)o, \
            (const T*)wo, (const T*)bo, (long)M, (unsigned)inner, (long)s_o, (long)s_i, eps);                           \
    } while (0)
    if (C == 128) FFK_GO_LAUNCH(128); else FFK_GO_LAUNCH(256);
#undef FFK_GO_LAUNCH
    return ffk_check_launch("ffk_gated_out_fused");
}
