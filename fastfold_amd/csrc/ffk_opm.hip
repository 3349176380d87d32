// Fused outer-product-mean core (see ffk_opm_fused in include/ffk.h):
//     out[i, j, c] = resid[i, j, c] + ( sum_{d,e} O_ij[d, e] * W[c, d, e] + bias[c] ) / (norm[i, j] + eps),
//     O_ij[d, e]   = sum_s a[s, i, d] * b[s, j, e]                       (32 x 32 per residue pair)
// without ever writing the [r, r, 1024] outer product to memory.
//
// A workgroup (8 wavefronts) owns 8 i x 32 j = 256 residue pairs and walks the 32 values of e in 16
// chunks of two.  Per chunk:
//   phase A  (outer product)  wave w multiplies its own i = i0 + w: rows (d) x columns (j, e in chunk),
//            K = s.  Its a-fragments stay in registers for the whole tile; the b rows of the chunk come
//            from LDS.  The 32 x 32 results are rounded to bf16 and written to LDS as rows of
//            A2[pair][k2 = (e, d)] - exactly the operand layout of the second product.
//   phase B  (projection)     out[pair, c] += A2[pair, chunk] . W2[c, chunk]: 8 x 4 MFMA tiles, each
//            wave owns 2 x 2 of them; accumulators live in registers across all chunks.
// b and W2 chunks arrive by direct global -> LDS loads (XOR-swizzled unpadded rows) one iteration
// ahead; phase B of chunk q - 1 and phase A of chunk q run between the same pair of barriers, so there
// is one barrier per chunk.  The weight is expected pre-permuted to k2 = e * 32 + d order.
#include "ffk_common.h"

namespace {

typedef bf16_t T;
constexpr int OP_THREADS = 512;
constexpr int OP_TI = 8, OP_TJ = 32;            // pairs per workgroup: 8 i x 32 j
constexpr int OP_EC = 2;                         // values of e per chunk
constexpr int OP_NCHUNK = 32 / OP_EC;            // 16
constexpr int OP_K2C = OP_EC * 32;               // k2 elements per chunk (64)
constexpr int OP_PA = OP_K2C * 2 + 16;           // A2 row pitch in bytes (padded: written by ds_write)
constexpr int OP_A2 = OP_TI * OP_TJ * OP_PA;     // one A2 buffer
constexpr int OP_W2SLOT = 128 * OP_K2C * 2;      // W2 chunk: 128 rows of 128 bytes (16 KB)

__device__ __forceinline__ int op_tau(int i) { return ((i >> 2) & 1) * 16 + (i >> 3) * 4 + (i & 3); }

__device__ __forceinline__ void op_load_lds(const T* src, unsigned char* dst_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst_wave, 16, 0, 0);
}

template <int KS1>   // MFMA K steps of the outer product: spad / 16 (4 or 8)
__global__ __launch_bounds__(OP_THREADS, 2) void opm_fused_kernel(T* __restrict__ out, const T* __restrict__ resid, int8_t* __restrict__ xtail,
                                                                 const T* __restrict__ at, const T* __restrict__ bt,
                                                                 const T* __restrict__ w2p, const T* __restrict__ bias,
                                                                 const float* __restrict__ norm, int r, float eps) {
    typedef Mma<T> MM;
    constexpr int SPAD = KS1 * 16;                       // K of the outer product
    constexpr int BROW = SPAD * 2;                       // bytes per b row (128 or 256)
    constexpr int BCOLS = BROW / 16;                     // 16-byte columns per b row (8 or 16)
    constexpr int BSLOT = OP_TJ * OP_EC * BROW;          // b chunk: 64 rows
    constexpr int BLD = BSLOT / 16 / OP_THREADS;         // loads per thread per b chunk (1 or 2)
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_a2 = smem;                          // [2][256][OP_PA]
    unsigned char* s_w2 = smem + 2 * OP_A2;              // [3][128][128 B]
    unsigned char* s_b = s_w2 + 3 * OP_W2SLOT;           // [2][64][BROW]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const int tiles_j = r / OP_TJ;
    const int i0 = (blockIdx.x / tiles_j) * OP_TI, j0 = (blockIdx.x % tiles_j) * OP_TJ;

    // ---- a fragments of this wave's i (rows d through tau: registers of the result hold d = 16 half + v) ----
    bf16x8 af[KS1];
    {
        const T* ap = at + ((long)(i0 + wave) * 32 + op_tau(l32)) * SPAD + half * 8;
#pragma unroll
        for (int ks = 0; ks < KS1; ++ks) af[ks] = MM::ld(ap + ks * 16);
    }

    // ---- chunk loaders (direct to LDS; lane L of a wave lands at dst + 16 L) ----
    // b chunk: LDS row rho = j_local * 2 + ee, column c holds global column c ^ swz(rho)
    const T* bsrc[BLD];
#pragma unroll
    for (int i = 0; i < BLD; ++i) {
        const int v = i * OP_THREADS + tid, rho = v / BCOLS, c = v % BCOLS;
        const int swz = BCOLS == 16 ? (rho & 15) : ((rho >> 1) & 7);
        bsrc[i] = bt + ((long)(j0 + (rho >> 1)) * 32 + (rho & 1)) * SPAD + ((c ^ swz) * 8);
    }
    // W2 chunk: LDS row rho (0..127) holds weight row 32 * (rho / 32) + tau(rho % 32); 8 columns of 16 bytes
    const T* wsrc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int v = i * OP_THREADS + tid, rho = v >> 3, c = v & 7;
        wsrc[i] = w2p + (long)((rho & ~31) + op_tau(rho & 31)) * 1024 + ((c ^ ((rho >> 1) & 7)) * 8);
    }
    auto fetch = [&](int q) {
        unsigned char* bs = s_b + (q & 1) * BSLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < BLD; ++i) op_load_lds(bsrc[i] + (long)q * OP_EC * SPAD, bs + i * (OP_THREADS * 16));
        unsigned char* ws = s_w2 + (q % 3) * OP_W2SLOT + wave * 1024;
#pragma unroll
        for (int i = 0; i < 2; ++i) op_load_lds(wsrc[i] + q * OP_K2C, ws + i * (OP_THREADS * 16));
    };

    // ---- phase B roles: m-tiles 2 * (wave % 4) + {0, 1}, c-tiles 2 * (wave / 4) + {0, 1} ----
    const int mt0 = 2 * (wave & 3), ct0 = 2 * (wave >> 2);
    f32x16 acc2[2][2];   // [m][c]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc2[a][b][v] = 0.0f;

    // per-lane LDS offsets
    int boff[KS1];                                       // b fragment of column-tile 0: row l32, column 2 ks + half
#pragma unroll
    for (int ks = 0; ks < KS1; ++ks) {
        const int swz = BCOLS == 16 ? (l32 & 15) : ((l32 >> 1) & 7);
        boff[ks] = l32 * BROW + (((2 * ks + half) ^ swz) << 4);
    }
    // (column tile 1 = rows 32..63: same swizzle since 32 is a multiple of 16)
    int woff[4];                                         // W2 fragment of c-tile 0: row l32, column 2 ks + half
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) woff[ks] = l32 * 128 + (((2 * ks + half) ^ ((l32 >> 1) & 7)) << 4);
    // A2 write position of phase A: pair (wave, 16 ct + l32 / 2), k2 = (l32 & 1) * 32 + 16 half
    const int a2w = (wave * 32 + (l32 >> 1)) * OP_PA + ((l32 & 1) * 32 + 16 * half) * 2;
    // A2 fragment of phase B: pair row mt * 32 + l32, k2 = 16 ks + 8 half
    const int a2r = l32 * OP_PA + half * 16;

    // The epilogue's operands (residual, its tail, the normaliser) are requested during the third chunk, not in the
    // epilogue: with one workgroup per CU (154 KB of LDS) nothing else would cover their latency - four dependent round
    // trips took 8 of a workgroup's 42 microseconds.  The wait at the top of the next chunk covers them.
    u32x4 e_rv[2][2][2], e_tv[2][2];
    float e_norm[2];
    const int pf_q = 2 + (int)((blockIdx.x >> 3) % 12u);   // spread over the chunks: the workgroups of a launch run in step
    fetch(0);
    for (int q = 0; q <= OP_NCHUNK; ++q) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // chunk q has landed (this wave's part)
        __builtin_amdgcn_s_barrier();                        // ... everyone's; A2 of chunk q - 1 is complete
        if (q + 1 < OP_NCHUNK) fetch(q + 1);
        if (q == pf_q) {
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const long pr = (long)(i0 + mt0 + m) * r + j0 + l32;
                e_norm[m] = norm[pr];
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const long o = pr * 128 + (ct0 + c) * 32 + 16 * half;
                    e_rv[m][c][0] = *reinterpret_cast<const u32x4*>(resid + o);
                    e_rv[m][c][1] = *reinterpret_cast<const u32x4*>(resid + o + 8);
                    if (xtail) e_tv[m][c] = *reinterpret_cast<const u32x4*>(xtail + o);
                }
            }
        }
        if (q > 0) {
            // ---- phase B of chunk q - 1 ----
            const unsigned char* a2 = s_a2 + ((q - 1) & 1) * OP_A2;
            const unsigned char* w2 = s_w2 + ((q - 1) % 3) * OP_W2SLOT;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                bf16x8 fa[2], fw[2];
#pragma unroll
                for (int m = 0; m < 2; ++m) fa[m] = *reinterpret_cast<const bf16x8*>(a2 + (mt0 + m) * 32 * OP_PA + a2r + ks * 32);
#pragma unroll
                for (int c = 0; c < 2; ++c) fw[c] = *reinterpret_cast<const bf16x8*>(w2 + (ct0 + c) * 32 * 128 + woff[ks]);
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int c = 0; c < 2; ++c) MM::mma(acc2[m][c], fw[c], fa[m]);
            }
        }
        if (q < OP_NCHUNK) {
            // ---- phase A of chunk q: O[d, (j, e)] for this wave's i, two column tiles of 16 j x 2 e ----
            const unsigned char* bs = s_b + (q & 1) * BSLOT;
            unsigned char* a2 = s_a2 + (q & 1) * OP_A2;
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
                f32x16 o;
#pragma unroll
                for (int v = 0; v < 16; ++v) o[v] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS1; ++ks)
                    MM::mma(o, af[ks], *reinterpret_cast<const bf16x8*>(bs + ct * 32 * BROW + boff[ks]));
                T y[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) y[v] = (T)o[v];
                unsigned char* p = a2 + a2w + ct * 16 * OP_PA;
                *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(&y[0]);
                *reinterpret_cast<u32x4*>(p + 16) = *reinterpret_cast<const u32x4*>(&y[8]);
            }
        }
    }

    // ---- epilogue: lane = pair, registers = 16 consecutive channels ----
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const long pr = (long)(i0 + mt0 + m) * r + j0 + l32;
        const float inv = 1.0f / (e_norm[m] + eps);
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int ch = (ct0 + c) * 32 + 16 * half;
            const long o = pr * 128 + ch;
            u32x4 bv[2], rv[2];
            bv[0] = *reinterpret_cast<const u32x4*>(bias + ch);
            bv[1] = *reinterpret_cast<const u32x4*>(bias + ch + 8);
            rv[0] = e_rv[m][c][0];
            rv[1] = e_rv[m][c][1];
            if (xtail) {       // extended residual stream: the update is added at 24 bits
                const u32x4 tv = e_tv[m][c];
                float upd[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) upd[v] = (float)(T)((acc2[m][c][v] + (float)reinterpret_cast<const T*>(&bv[v >> 3])[v & 7]) * inv);
                u32x4 h0, h1, tn;
                xs_update16(upd, rv[0], rv[1], tv, h0, h1, tn);
                *reinterpret_cast<u32x4*>(out + o) = h0;
                *reinterpret_cast<u32x4*>(out + o + 8) = h1;
                *reinterpret_cast<u32x4*>(xtail + o) = tn;
                continue;
            }
            T y[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float x = (acc2[m][c][v] + (float)reinterpret_cast<const T*>(&bv[v >> 3])[v & 7]) * inv;
                y[v] = (T)((float)(T)x + (float)reinterpret_cast<const T*>(&rv[v >> 3])[v & 7]);
            }
            *reinterpret_cast<u32x4*>(out + o) = *reinterpret_cast<const u32x4*>(&y[0]);
            *reinterpret_cast<u32x4*>(out + o + 8) = *reinterpret_cast<const u32x4*>(&y[8]);
        }
    }
}

template <int KS1>
int opm_launch(T* out, const T* resid, int8_t* xtail, const T* at, const T* bt, const T* w2p, const T* bias, const float* norm, int r,
               float eps, hipStream_t st) {
    const size_t smem = 2 * (size_t)OP_A2 + 3 * OP_W2SLOT + 2 * (size_t)(OP_TJ * OP_EC * KS1 * 32);
    static FfkLdsReservation lds_reserved;
    {
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)opm_fused_kernel<KS1>, smem, "ffk_opm_fused");
        if (rc_lds != FFK_OK) return rc_lds;
    }
    const unsigned grid = (unsigned)((r / OP_TI) * (r / OP_TJ));
    opm_fused_kernel<KS1><<<grid, OP_THREADS, smem, st>>>(out, resid, xtail, at, bt, w2p, bias, norm, r, eps);
    return ffk_check_launch("ffk_opm_fused");
}

}  // namespace

extern "C" int ffk_opm_fused(void* out, const void* resid, void* xtail, const void* a_t, const void* b_t, const void* w2p, const void* bias,
                             const float* norm, int64_t r, int64_t spad, float eps, int dtype, void* stream) {
    FFK_REQUIRE(out && resid && a_t && b_t && w2p && bias && norm, FFK_ERR_NULL, "ffk_opm_fused: null pointer");
    FFK_REQUIRE(dtype == FFK_BF16, FFK_ERR_DTYPE, "ffk_opm_fused: bf16 only (dtype tag %d)", dtype);
    FFK_REQUIRE(r > 0 && r % 32 == 0 && r <= 32768, FFK_ERR_SHAPE, "ffk_opm_fused: r=%ld must be a positive multiple of 32", (long)r);
    FFK_REQUIRE(spad == 64 || spad == 128, FFK_ERR_UNSUPPORTED, "ffk_opm_fused: padded sequence count %ld must be 64 or 128", (long)spad);
    FFK_REQUIRE(ffk_aligned16(out) && ffk_aligned16(resid) && ffk_aligned16(a_t) && ffk_aligned16(b_t) && ffk_aligned16(w2p) &&
                    ffk_aligned16(bias) && ffk_aligned16(xtail),
                FFK_ERR_ALIGN, "ffk_opm_fused: buffers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (spad == 128)
        return opm_launch<8>((T*)out, (const T*)resid, (int8_t*)xtail, (const T*)a_t, (const T*)b_t, (const T*)w2p, (const T*)bias, norm, (int)r, eps, st);
    return opm_launch<4>((T*)out, (const T*)resid, (int8_t*)xtail, (const T*)a_t, (const T*)b_t, (const T*)w2p, (const T*)bias, norm, (int)r, eps, st);
}
