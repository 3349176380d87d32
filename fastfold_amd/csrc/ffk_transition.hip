// Fused transition (see ffk_transition_fused in include/ffk.h):
//     out = x + W2 . relu( W1 . LayerNorm(x) + b1 ) + b2        (C -> 4C -> C channels, C = 128 or 256, bf16)
// with the hidden activation never leaving the registers.
//
// A workgroup (4 wavefronts) owns 128 rows, a wavefront 32 of them from start to end.  Set-up: the rows
// are fetched once, normalised in registers (16 lanes per row) and passed through LDS into the MFMA
// fragments of their wave, where they stay.  The hidden layer is walked in chunks of 32 channels (16 chunks
// at C = 128, 32 at C = 256); per chunk and wave
//   first GEMM   H^T[hidden, rows] = W1[chunk] . x^T  (+ b1, relu): one tile of 32 hidden channels; lane =
//                row, registers = hidden channels;
//   second GEMM  out^T[c, rows] += W2[c, chunk] . H^T: the rounded accumulators of the first GEMM are the
//                N operand as they stand.  A lane holds hidden channels 8a + 4h + b of a tile (h = its
//                half-wave) in registers 4a + b, and an MFMA K step wants 8 consecutive K per half-wave,
//                so the first GEMM's M-operand row i is loaded from weight row sigma(i) such that
//                registers 8j .. 8j + 7 of half-wave h are hidden channels 16j + 8h .. 16j + 8h + 7.
// Only the weights go through LDS: W1 / W2 chunks arrive by direct global -> LDS loads (XOR-swizzled
// unpadded rows) one chunk ahead, shared by the four waves; one barrier per chunk.  A workgroup spends about
// a third of its life fetching its rows and storing its results (measured with wall-clock stamps: 3.5 us set-up,
// 14 us in the chunk loop, 5 us in the epilogue at C = 128 with residual tails), so as many workgroups as fit share
// a CU and cover each other's waits: with 32-channel chunks the rings take 32 KB (C = 128; the row buffer of the
// set-up, 34 KB, is then the larger) and the kernel 149 registers: three workgroups per CU (two at C = 256).
#include "ffk_common.h"

namespace {

typedef bf16_t T;
constexpr int TR_THREADS = 256;
constexpr int TR_BM = 128;                     // rows per workgroup
template <int C, int NS> struct TrGeo {
    static constexpr int H = 4 * C;
    static constexpr int HC = 32;                   // hidden channels per chunk
    static constexpr int NCHUNK = H / HC;
    static constexpr int W1SLOT = HC * C * 2;       // HC rows of 2 C bytes (16 KB)
    static constexpr int W2SLOT = C * HC * 2;       // C rows of 2 HC bytes (16 KB)
    static constexpr int XP = C * 2 + 16;           // pitch of the normalised rows (set-up only)
    static constexpr int NC1 = C / 8;               // 16-byte columns of a W1 row
    static constexpr int NC2 = HC / 8;              // 16-byte columns of a W2 row
    static constexpr int RP2 = 256 / (HC * 2);      // W2 rows per 256 bytes of LDS: the swizzle period
    static constexpr int KS1 = C / 16, KS2 = HC / 16, HT = HC / 32, CT = C / 32;
    static constexpr size_t SMEM_RINGS = NS * (size_t)W1SLOT + NS * W2SLOT + H * sizeof(float);
    static constexpr size_t SMEM_ROWS = (size_t)TR_BM * XP;
    static constexpr int NLD = W1SLOT / 16 / TR_THREADS;   // 16-byte requests per thread and ring slot
    static_assert(W1SLOT == W2SLOT, "ring slots of one size");
    static constexpr size_t SMEM = SMEM_RINGS > SMEM_ROWS ? SMEM_RINGS : SMEM_ROWS;
};

__device__ __forceinline__ int tr_tau(int i) { return ((i >> 2) & 1) * 16 + (i >> 3) * 4 + (i & 3); }
// i = 8a + 4h + b  ->  16 (a / 2) + 8h + 4 (a % 2) + b
__device__ __forceinline__ int tr_sigma(int i) { return (i >> 4) * 16 + ((i >> 2) & 1) * 8 + ((i >> 3) & 1) * 4 + (i & 3); }

__device__ __forceinline__ void tr_load_lds(const T* src, unsigned char* dst_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst_wave, 16, 0, 0);
}

// NS: slots of the weight rings.  Two slots (one chunk in flight) when two workgroups share a CU and cover each
// other's waits; four when the launch has at most one workgroup per CU and the chunk stream has to hide the whole
// memory latency by itself (a chunk is multiplied in less than half a microsecond).
template <int TR_C, int NS>
__global__ __launch_bounds__(TR_THREADS, NS == 4 ? 1 : (TR_C == 128 ? 3 : 2)) void transition_fused_kernel(T* __restrict__ out, const T* __restrict__ x, int8_t* __restrict__ xtail,
                                                                        const T* __restrict__ gamma, const T* __restrict__ beta,
                                                                        const T* __restrict__ w1, const T* __restrict__ b1,
                                                                        const T* __restrict__ w2, const T* __restrict__ b2,
                                                                        long M, float eps) {
    typedef Mma<T> MM;
    typedef TrGeo<TR_C, NS> G;
    constexpr int NLD = G::NLD;
    constexpr int TR_H = G::H, TR_HC = G::HC, TR_NCHUNK = G::NCHUNK, TR_W1SLOT = G::W1SLOT, TR_W2SLOT = G::W2SLOT, TR_XP = G::XP;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_w1 = smem;                           // [NS][HC][2 C bytes]
    unsigned char* s_w2 = smem + NS * TR_W1SLOT;          // [NS][C][2 HC bytes]
    float* s_b1 = reinterpret_cast<float*>(s_w2 + NS * TR_W2SLOT);  // [H]
    unsigned char* s_x = smem;                            // [128][TR_XP], set-up only (aliases the rings)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const long m0 = (long)blockIdx.x * TR_BM;

    // ---- set-up: rows -> LayerNorm in registers -> LDS -> this wave's fragments ----
    {
        constexpr int LPR = TR_C / 8, RPP = TR_THREADS / LPR, NPASS = TR_BM / RPP;   // lanes per row, rows per pass
        const int c8 = tid % LPR, r0 = tid / LPR;
        const Vec16<T> g = ld16(gamma + c8 * 8), b = ld16(beta + c8 * 8);
#pragma unroll
        for (int i0 = 0; i0 < NPASS; i0 += 8) {
            Vec16<T> v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                long m = m0 + r0 + RPP * (i0 + i);
                m = m < M ? m : M - 1;                    // clamped: rows past the end are never stored
                v[i] = ld16(x + m * TR_C + c8 * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float f[8], s = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] = (float)v[i].e[e];
                    s += f[e];
                }
                const float mu = group_sum(s, LPR) * (1.0f / TR_C);
                float q = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] -= mu;
                    q += f[e] * f[e];
                }
                const float rs = rsqrtf(group_sum(q, LPR) * (1.0f / TR_C) + eps);
                Vec16<T> y;
#pragma unroll
                for (int e = 0; e < 8; ++e) y.e[e] = (T)(f[e] * rs * (float)g.e[e] + (float)b.e[e]);
                *reinterpret_cast<Vec16<T>*>(s_x + (r0 + RPP * (i0 + i)) * TR_XP + c8 * 16) = y;
            }
        }
    }
    lds_barrier();
    bf16x8 xf[G::KS1];                                     // rows 32 wave + l32, all of K = C
#pragma unroll
    for (int ks = 0; ks < G::KS1; ++ks)
        xf[ks] = *reinterpret_cast<const bf16x8*>(s_x + (wave * 32 + l32) * TR_XP + ks * 32 + half * 16);
    lds_barrier();                                         // the row buffer is free: the rings may overwrite it
    for (int i = tid; i < TR_H; i += TR_THREADS) s_b1[i] = (float)b1[i];

    // ---- chunk loaders (direct to LDS; lane L of a wave lands at dst + 16 L) ----
    // W1 chunk: LDS row rho (0..63) holds weight row 32 * (rho / 32) + sigma(rho % 32) of the chunk; 16 columns
    const T* w1src[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int v = i * TR_THREADS + tid, rho = v / G::NC1, c = v % G::NC1;
        w1src[i] = w1 + (long)((rho & ~31) + tr_sigma(rho & 31)) * TR_C + ((c ^ (rho & 15)) * 8);
    }
    // W2 chunk: LDS row rho (0..127) holds weight row 32 * (rho / 32) + tau(rho % 32); 8 columns
    const T* w2src[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int v = i * TR_THREADS + tid, rho = v / G::NC2, c = v % G::NC2;
        w2src[i] = w2 + (long)((rho & ~31) + tr_tau(rho & 31)) * TR_H + ((c ^ ((rho / G::RP2) & (G::NC2 - 1))) * 8);
    }
    auto fetch = [&](int q) {                              // past the last chunk it is fetched again (into a free slot)
        const int qc = q < TR_NCHUNK ? q : TR_NCHUNK - 1;
        unsigned char* d1 = s_w1 + (q % NS) * TR_W1SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < NLD; ++i) tr_load_lds(w1src[i] + (long)qc * TR_HC * TR_C, d1 + i * (TR_THREADS * 16));
        unsigned char* d2 = s_w2 + (q % NS) * TR_W2SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < NLD; ++i) tr_load_lds(w2src[i] + qc * TR_HC, d2 + i * (TR_THREADS * 16));
    };

    f32x16 acc2[G::CT];                                    // out^T tiles: channels 32 ct + 16 half + v, row l32
#pragma unroll
    for (int c = 0; c < G::CT; ++c) {                      // start from b2: the epilogue has no bias to add
        const Vec16<T> b0 = ld16(b2 + c * 32 + 16 * half), b1v = ld16(b2 + c * 32 + 16 * half + 8);
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            acc2[c][v] = (float)b0.e[v];
            acc2[c][8 + v] = (float)b1v.e[v];
        }
    }

    // W1 fragment of hidden tile 0: row l32, column 2 ks + half.  The swizzle touches the low four column bits only,
    // so K steps 8 .. 15 (C = 256) are the first eight plus 256 bytes.
    int w1off[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) w1off[ks] = l32 * (TR_C * 2) + (((2 * ks + half) ^ (l32 & 15)) << 4);
    int w2off[G::KS2];                                     // W2 fragment of c-tile 0: row l32, column 2 ks + half
#pragma unroll
    for (int ks = 0; ks < G::KS2; ++ks) w2off[ks] = l32 * (TR_HC * 2) + (((2 * ks + half) ^ ((l32 / G::RP2) & (G::NC2 - 1))) << 4);

#pragma unroll
    for (int q = 0; q < NS - 1; ++q) fetch(q);
    for (int q = 0; q < TR_NCHUNK; ++q) {
        // chunk q has landed (this wave's part) once only the NS - 2 younger chunks (8 loads each) are outstanding
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD * (NS - 2)) : "memory");
        __builtin_amdgcn_s_barrier();                        // ... everyone's; nobody still reads the slot of chunk q - 1
        fetch(q + NS - 1);
        const unsigned char* wa = s_w1 + (q % NS) * TR_W1SLOT;
        const unsigned char* wb = s_w2 + (q % NS) * TR_W2SLOT;
        bf16x8 hf[G::HT][2];                               // [hidden tile][K step]: the chunk's N operand
#pragma unroll
        for (int ht = 0; ht < G::HT; ++ht) {
            f32x16 h;
            // registers 0..7: hidden 8 half + 0..7 of the tile, registers 8..15: 16 + 8 half + 0..7
            const float* bp = s_b1 + q * TR_HC + ht * 32 + 8 * half;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 b4 = *reinterpret_cast<const f32x4*>(bp + (a >> 1) * 16 + (a & 1) * 4);
#pragma unroll
                for (int b = 0; b < 4; ++b) h[4 * a + b] = b4[b];
            }
#pragma unroll
            for (int ks = 0; ks < G::KS1; ++ks)
                MM::mma(h, *reinterpret_cast<const bf16x8*>(wa + ht * 32 * (TR_C * 2) + w1off[ks & 7] + (ks >> 3) * 256), xf[ks]);
            // relu after the rounding, on the packed bf16 bit patterns: a negative bf16 is a negative 16-bit integer, so
            // one packed integer max per pair replaces one clamp per value (rounding is monotonic: same bits)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                typedef short s16x2 __attribute__((ext_vector_type(2)));
                const s16x2 zero = {0, 0};
                u32x4 w;
#pragma unroll
                for (int t = 0; t < 4; ++t) {              // one packed conversion and one packed max per pair
                    const f32x2 pr = {h[8 * j + 2 * t], h[8 * j + 2 * t + 1]};
                    const bf16x2 r = __builtin_convertvector(pr, bf16x2);
                    w[t] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s16x2, r), zero));
                }
                hf[ht][j] = __builtin_bit_cast(bf16x8, w);
            }
        }
#pragma unroll
        for (int ks = 0; ks < G::KS2; ++ks)
#pragma unroll
            for (int c = 0; c < G::CT; ++c)
                MM::mma(acc2[c], *reinterpret_cast<const bf16x8*>(wb + c * 32 * (TR_HC * 2) + w2off[ks]), hf[ks >> 1][ks & 1]);
    }

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // the re-fetches past the last chunk

    // ---- epilogue: lane = row, registers = 16 consecutive channels ----
    const long row = m0 + wave * 32 + l32;
    const bool ok = row < M;
    const long rc = ok ? row : M - 1;
#pragma unroll
    for (int c = 0; c < G::CT; ++c) {
        const int ch = c * 32 + 16 * half;
        const long o = rc * TR_C + ch;
        u32x4 rv[2];
        rv[0] = *reinterpret_cast<const u32x4*>(x + o);
        rv[1] = *reinterpret_cast<const u32x4*>(x + o + 8);
        if (xtail) {           // extended residual stream: the update is added at 24 bits
            const u32x4 tv = *reinterpret_cast<const u32x4*>(xtail + o);
            float upd[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) upd[v] = (float)(T)acc2[c][v];
            u32x4 h0, h1, tn;
            xs_update16(upd, rv[0], rv[1], tv, h0, h1, tn);
            if (ok) {
                *reinterpret_cast<u32x4*>(out + o) = h0;
                *reinterpret_cast<u32x4*>(out + o + 8) = h1;
                *reinterpret_cast<u32x4*>(xtail + o) = tn;
            }
            continue;
        }
        T y[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            y[v] = (T)((float)(T)acc2[c][v] + (float)reinterpret_cast<const T*>(&rv[v >> 3])[v & 7]);
        }
        if (ok) {
            *reinterpret_cast<u32x4*>(out + o) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(out + o + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    }
}

}  // namespace

extern "C" int ffk_transition_fused(void* out, const void* x, void* xtail, const void* gamma, const void* beta, const void* w1,
                                    const void* b1, const void* w2, const void* b2, int64_t M, int64_t C, int64_t hidden,
                                    float eps, int dtype, void* stream) {
    FFK_REQUIRE(out && x && gamma && beta && w1 && b1 && w2 && b2, FFK_ERR_NULL, "ffk_transition_fused: null pointer");
    FFK_REQUIRE(dtype == FFK_BF16, FFK_ERR_DTYPE, "ffk_transition_fused: bf16 only (dtype tag %d)", dtype);
    FFK_REQUIRE((C == 128 || C == 256) && hidden == 4 * C, FFK_ERR_UNSUPPORTED,
                "ffk_transition_fused: built for 128 -> 512 -> 128 and 256 -> 1024 -> 256, got %ld -> %ld", (long)C, (long)hidden);
    FFK_REQUIRE(M > 0 && M < (1L << 31) * (long)TR_BM, FFK_ERR_SHAPE, "ffk_transition_fused: bad row count %ld", (long)M);
    FFK_REQUIRE(ffk_aligned16(out) && ffk_aligned16(x) && ffk_aligned16(gamma) && ffk_aligned16(beta) && ffk_aligned16(w1) &&
                    ffk_aligned16(w2) && ffk_aligned16(b2) && ffk_aligned16(xtail),
                FFK_ERR_ALIGN, "ffk_transition_fused: buffers must be 16-byte aligned");
    const unsigned grid = (unsigned)ffk_cdiv(M, TR_BM);
    const bool deep = grid <= 256 + 128;                     // at most ~one workgroup per CU: four-slot rings
#define FFK_TR_LAUNCH(CC, NS)                                                                                           \
    do {                                                                                                                \
        static FfkLdsReservation lds_reserved;                                                                          \
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)transition_fused_kernel<CC, NS>, TrGeo<CC, NS>::SMEM, \
                                           "ffk_transition_fused");                                                     \
        if (rc_lds != FFK_OK) return rc_lds;                                                                            \
        transition_fused_kernel<CC, NS><<<grid, TR_THREADS, TrGeo<CC, NS>::SMEM, (hipStream_t)stream>>>(                \
            (T*)out, (const T*)x, (int8_t*)xtail, (const T*)gamma, (const T*)beta, (const T*)w1, (const T*)b1, (const T*)w2, \
            (const T*)b2, (long)M, eps);                                                                                \
    } while (0)
    if (C == 128) {
        if (deep) FFK_TR_LAUNCH(128, 4); else FFK_TR_LAUNCH(128, 2);
    } else {
        if (deep) FFK_TR_LAUNCH(256, 4); else FFK_TR_LAUNCH(256, 2);
    }
#undef FFK_TR_LAUNCH
    return ffk_check_launch("ffk_transition_fused");
}
