// Pair bias of the biased attentions (see ffk_pair_bias in include/ffk.h):
//     bias_t[h][q/32][k/32][tile(k, q)] = scale * ( LayerNorm(z[q, k, :]) . w[h, :] )
// written directly in the keys x queries operand tiles the attention kernel consumes.
//
// The op is a skinny projection (C = 128 or 64 channels -> H <= 8 heads) and purely HBM-bound (one read of
// z).  One workgroup owns a 32 x 32 block of (q, k) and walks it in four 16 x 16 quarter blocks (launches of fewer
// than 512 blocks give every quarter a workgroup of its own): the
// 256 rows of a quarter are fetched with 16 lanes per row (coalesced 256-byte rows, 16 loads in
// flight per thread, the next quarter's loads issued before this one is finished) into LDS.  The
// LayerNorm is folded into the projection,
//     LN(x) . w = rstd * ( x . (w * gamma)  -  mean * sum(w * gamma) ) + w . beta,
// so the raw bf16 rows are the MFMA operand: each wave multiplies two 32-row groups against a
// 32-row weight operand held in registers whose rows 0 .. H-1 are w * gamma and rows 8 and 12 all
// ones (they deliver sum(x) to both half-waves); sum(x^2) comes from the loader lanes.  Lane l of a
// group owns row l, whose tile offset is its index in the quarter, so the 2-byte stores of a wave
// are contiguous.
#include "ffk_common.h"

namespace {

constexpr int PB_THREADS = 256;
constexpr int PB_MAXH = 8;

template <int C>
__global__ __launch_bounds__(PB_THREADS) void pair_bias_kernel(bf16_t* __restrict__ bias_t, const bf16_t* __restrict__ z,
                                                              const bf16_t* __restrict__ wop,  // [32][C] MFMA weight operand
                                                              const float* __restrict__ c01,   // [H][2]: sum(w*gamma), w . beta
                                                              int N, int H, int a_inner, long a_so, long a_si,
                                                              float scale, float eps) {
    typedef bf16_t T;
    typedef Mma<T> MM;
    constexpr int VPR = C / 8;                       // 16-byte vectors per row
    constexpr int PITCH = C * 2 + 16;                // LDS row pitch (bytes)
    constexpr int NLD = 256 * VPR / PB_THREADS;      // loads per thread per quarter
    constexpr int KS = C / 16;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_rows = smem;                                         // [256][PITCH]
    float* s_sq = reinterpret_cast<float*>(smem + 256 * PITCH);           // [256] sum of squares per row

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int QT = (N + 31) >> 5;
    const int qt = blockIdx.y, kt = blockIdx.x;

    bf16x8 wf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) wf[ks] = MM::ld(wop + l32 * C + ks * 16 + half * 8);
    // per-lane constants of its four heads h = 4 * half + b
    float c_sum[4], c_beta[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int h = 4 * half + b;
        c_sum[b] = h < H ? c01[2 * h] : 0.0f;
        c_beta[b] = h < H ? c01[2 * h + 1] : 0.0f;
    }

    const int c8 = tid % VPR, rl = tid / VPR;        // loader role: vector c8 of rows rl, rl + 256/VPR...
    // rows of a quarter: tile offsets 256*quarter .. +255; offset o <-> q32 = (o/512)*16 + o%16, k32 = (o/16)%32
    Vec16<T> buf[NLD];
    auto fetch = [&](int quarter) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int o = quarter * 256 + rl + i * (PB_THREADS / VPR);
            int q = qt * 32 + (o >> 9) * 16 + (o & 15), k = kt * 32 + ((o >> 4) & 31);
            q = q < N ? q : N - 1;                   // clamped: rows outside are not stored
            k = k < N ? k : N - 1;
            const unsigned m = (unsigned)q * (unsigned)N + (unsigned)k;
            const unsigned hi = m / (unsigned)a_inner, lo = m - hi * (unsigned)a_inner;
            buf[i] = ld16(z + (long)hi * a_so + (long)lo * a_si + c8 * 8);
        }
    };
    // quarters of the block this workgroup walks: all four, or one of them (gridDim.z = 4: launches of few blocks,
    // where a workgroup per block would leave most CUs idle)
    const int nquarters = 4 / (int)gridDim.z, q_first = (int)blockIdx.z * nquarters, q_last = q_first + nquarters - 1;
    fetch(q_first);
    for (int quarter = q_first; quarter <= q_last; ++quarter) {
        __syncthreads();                             // previous quarter's rows are consumed
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int r = rl + i * (PB_THREADS / VPR);
            *reinterpret_cast<Vec16<T>*>(s_rows + r * PITCH + c8 * 16) = buf[i];
            float q2 = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)buf[i].e[e];
                q2 += f * f;
            }
            q2 = group_sum(q2, VPR);
            if (c8 == 0) s_sq[r] = q2;
        }
        __syncthreads();
        if (quarter < q_last) fetch(quarter + 1);    // in flight while this quarter is finished below

#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int row = (wave * 2 + g) * 32 + l32;
            const unsigned char* ap = s_rows + row * PITCH + half * 16;
            f32x16 acc;
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) MM::mma(acc, wf[ks], *reinterpret_cast<const bf16x8*>(ap + ks * 32));
            // registers 0..3: heads 4*half + b; register 4: sum(x) (ones rows 8 / 12 of the weight operand)
            const float mu = acc[4] * (1.0f / C);
            const float var = fmaxf(s_sq[row] * (1.0f / C) - mu * mu, 0.0f);
            const float rs = rsqrtf(var + eps);
            const int o = quarter * 256 + row;
            const int q = qt * 32 + (o >> 9) * 16 + (o & 15), k = kt * 32 + ((o >> 4) & 31);
            if (q < N && k < N) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int h = 4 * half + b;
                    if (h < H)
                        bias_t[(((long)h * QT + qt) * QT + kt) * 1024 + o] = (T)(scale * (rs * (acc[b] - mu * c_sum[b]) + c_beta[b]));
                }
            }
        }
    }
}

// Builds the MFMA weight operand wop[32][C] (rows 0..H-1: w * gamma rounded to bf16, rows 8 and 12: ones,
// others zero) and c01[h] = { sum_c wop[h][c], w[h] . beta }.  One block per operand row.
__global__ void pair_bias_prep_kernel(bf16_t* wop, float* c01, const bf16_t* w, const bf16_t* gamma, const bf16_t* beta, int H,
                                      int C) {
    const int h = blockIdx.x;
    float s0 = 0.0f, s1 = 0.0f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        bf16_t v = (bf16_t)0.0f;
        if (h < H) {
            const float wv = (float)w[h * C + c];
            v = (bf16_t)(wv * (float)gamma[c]);
            s0 += (float)v;                           // the sum of what the MFMA really multiplies by
            s1 += wv * (float)beta[c];
        } else if (h == 8 || h == 12) {
            v = (bf16_t)1.0f;
        }
        wop[h * C + c] = v;
    }
    s0 = group_sum(s0, 64);
    s1 = group_sum(s1, 64);
    if (threadIdx.x == 0 && h < H) {
        c01[2 * h] = s0;
        c01[2 * h + 1] = s1;
    }
}

// Validates, builds the weight operand in `scratch` (unless w == NULL) and launches.  Shared by both entry points.
int pair_bias_run(const char* who, void* bias_t, const void* z, const void* gamma, const void* beta, const void* w,
                  float* scratch, int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so, int64_t a_si, float scale,
                  float eps, int dtype, hipStream_t st) {
    FFK_REQUIRE(bias_t && z && scratch && (!w || (gamma && beta)), FFK_ERR_NULL, "%s: null pointer", who);
    FFK_REQUIRE(dtype == FFK_BF16, FFK_ERR_DTYPE, "%s: bf16 only (dtype tag %d)", who, dtype);
    FFK_REQUIRE(C == 128 || C == 64, FFK_ERR_UNSUPPORTED, "%s: built for 64 or 128 pair channels, got %ld", who, (long)C);
    FFK_REQUIRE(N > 0 && N <= 46340 && H > 0 && H <= PB_MAXH && a_inner > 0, FFK_ERR_SHAPE,
                "%s: bad shape N=%ld H=%ld a_inner=%ld (at most %d heads)", who, (long)N, (long)H, (long)a_inner, PB_MAXH);
    FFK_REQUIRE(ffk_aligned16(z) && ffk_aligned16(scratch) && a_so % 8 == 0 && a_si % 8 == 0, FFK_ERR_ALIGN,
                "%s: rows of z must be 16-byte aligned", who);
    bf16_t* wop = reinterpret_cast<bf16_t*>(scratch);     // [32][C] bf16 = 16 * C floats
    float* c01 = scratch + 16 * C;                       // [H][2]
    if (w) {       // w == NULL: scratch still holds the operand an earlier call built from the same w, gamma, beta
        pair_bias_prep_kernel<<<32, 64, 0, st>>>(wop, c01, (const bf16_t*)w, (const bf16_t*)gamma, (const bf16_t*)beta,
                                                 (int)H, (int)C);
        int rc = ffk_check_launch(who);
        if (rc != FFK_OK) return rc;
    }
    const unsigned T = (unsigned)((N + 31) / 32);
#define PB_LAUNCH(CC)                                                                                                   \
    {                                                                                                                   \
        const size_t smem = 256 * (CC * 2 + 16) + 256 * sizeof(float);                                                  \
        static FfkLdsReservation lds_reserved;                                                                          \
        const int rc_lds = ffk_reserve_lds(lds_reserved, (const void*)pair_bias_kernel<CC>, smem, who);                 \
        if (rc_lds != FFK_OK) return rc_lds;                                                                            \
        pair_bias_kernel<CC><<<dim3(T, T, T * T < 512 ? 4 : 1), PB_THREADS, smem, st>>>((bf16_t*)bias_t, (const bf16_t*)z, wop, c01, (int)N, \
                                                                   (int)H, (int)a_inner, a_so, a_si, scale, eps);       \
    }
    if (C == 128) PB_LAUNCH(128) else PB_LAUNCH(64)
#undef PB_LAUNCH
    return ffk_check_launch(who);
}

// ---- the scratch of ffk_pair_bias_static: the weight operand [32][C <= 128] bf16 + [8][2] fp32 constants ----
constexpr int PB_STATIC_MAX_C = 128;
constexpr int PB_STATIC_FLOATS = 16 * PB_STATIC_MAX_C + 2 * PB_MAXH;      // 8 256 bytes per device
static __device__ __align__(256) float pb_static_scratch[PB_STATIC_FLOATS];

// Device address of this device's copy of pb_static_scratch, looked up once per device (the array's name is only
// a host-side handle: it must never be passed to a kernel or to a memory routine).
int pb_static_ptr(float** out) {
    static std::atomic<float*> ptrs[FFK_MAX_DEVICES];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "ffk_pair_bias_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= FFK_MAX_DEVICES)
        return ffk_fail(FFK_ERR_UNSUPPORTED, "ffk_pair_bias_static: device ordinal %d not supported", dev);
    float* p = ptrs[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(ffk_config_mutex());
        p = ptrs[dev].load(std::memory_order_relaxed);
        if (!p) {
            void* sym = nullptr;
            e = hipGetSymbolAddress(&sym, HIP_SYMBOL(pb_static_scratch));
            if (e != hipSuccess || !sym)
                return ffk_fail(FFK_ERR_LAUNCH, "ffk_pair_bias_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            p = static_cast<float*>(sym);
            ptrs[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return FFK_OK;
}

}  // namespace

extern "C" int ffk_pair_bias(void* bias_t, const void* z, const void* gamma, const void* beta, const void* w, float* scratch,
                             int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so, int64_t a_si, float scale,
                             float eps, int dtype, void* stream) {
    return pair_bias_run("ffk_pair_bias", bias_t, z, gamma, beta, w, scratch, N, C, H, a_inner, a_so, a_si, scale, eps, dtype,
                         (hipStream_t)stream);
}

extern "C" int ffk_pair_bias_static(void* bias_t, const void* z, const void* gamma, const void* beta, const void* w,
                                    int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so, int64_t a_si,
                                    float scale, float eps, int dtype, void* stream) {
    FFK_REQUIRE(w && gamma && beta, FFK_ERR_NULL,
                "ffk_pair_bias_static: w, gamma and beta are required (the shared scratch is rebuilt by every call)");
    FFK_REQUIRE(C > 0 && C <= PB_STATIC_MAX_C && H > 0 && H <= PB_MAXH, FFK_ERR_SHAPE,
                "ffk_pair_bias_static: C=%ld H=%ld exceed the static scratch (at most %d channels, %d heads)", (long)C, (long)H,
                PB_STATIC_MAX_C, PB_MAXH);
    float* scratch = nullptr;
    int rc = pb_static_ptr(&scratch);
    if (rc != FFK_OK) return rc;
    return pair_bias_run("ffk_pair_bias_static", bias_t, z, gamma, beta, w, scratch, N, C, H, a_inner, a_so, a_si, scale, eps,
                         dtype, (hipStream_t)stream);
}
