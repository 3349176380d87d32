// Pair bias of the biased attentions (see ffk_pair_bias in include/ffk.h):
//     bias_t[h][q/32][k/32][tile(k, q)] = scale * ( LayerNorm(z[q, k, :]) . w[h, :] )
// written directly in the keys x queries operand tiles the attention kernel consumes.
//
// The op is a skinny projection (C = 128 channels -> H <= 8 heads), far too thin for the matrix
// pipe and purely HBM-bound (one read of z).  One workgroup owns a 32 x 32 block of (q, k) and walks
// it in four 16 x 16 quarter blocks: the 256 rows of a quarter are fetched with 16 lanes per row
// (coalesced 256-byte rows, 16 loads in flight per thread) into LDS, then every thread finishes one
// whole row on its own - statistics, normalisation folded into the dot products - so there is no
// cross-lane reduction at all.  Thread t of a quarter owns the row whose tile offset is t, which
// makes the 2-byte stores of a wave contiguous.
#include "ffk_common.h"

namespace {

constexpr int PB_THREADS = 256;
constexpr int PB_MAXH = 8;

template <int C>
__global__ __launch_bounds__(PB_THREADS) void pair_bias_kernel(bf16_t* __restrict__ bias_t, const bf16_t* __restrict__ z,
                                                              const float* __restrict__ wg,   // [H][C] w * gamma
                                                              const float* __restrict__ c01,  // [H][2]: sum(w*gamma), w . beta
                                                              int N, int H, int a_inner, long a_so, long a_si,
                                                              float scale, float eps) {
    typedef bf16_t T;
    constexpr int VPR = C / 8;                       // 16-byte vectors per row
    constexpr int PITCH = C * 2 + 16;                // LDS row pitch (bytes)
    constexpr int NLD = 256 * VPR / PB_THREADS;      // loads per thread per quarter
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* s_rows = smem;                                         // [256][PITCH]
    float* s_w = reinterpret_cast<float*>(smem + 256 * PITCH);            // [H][C]

    const int tid = threadIdx.x;
    const int QT = (N + 31) >> 5;
    const int qt = blockIdx.y, kt = blockIdx.x;
    for (int i = tid; i < H * C; i += PB_THREADS) s_w[i] = wg[i];

    const int c8 = tid % VPR, rl = tid / VPR;        // loader role: vector c8 of rows rl, rl + 256/VPR...
    for (int quarter = 0; quarter < 4; ++quarter) {
        // rows of this quarter: tile offsets 256*quarter .. +255; offset o <-> q32 = (o/512)*16 + o%16, k32 = (o/16)%32
        Vec16<T> buf[NLD];
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
        __syncthreads();                             // previous quarter's rows are consumed
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            *reinterpret_cast<Vec16<T>*>(s_rows + (rl + i * (PB_THREADS / VPR)) * PITCH + c8 * 16) = buf[i];
        __syncthreads();

        // thread tid finishes row tid: pass 1 mean, pass 2 centred second moment and dot products
        const unsigned char* row = s_rows + tid * PITCH;
        float s = 0.0f;
#pragma unroll
        for (int v = 0; v < VPR; ++v) {
            const Vec16<T> x = *reinterpret_cast<const Vec16<T>*>(row + v * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) s += (float)x.e[e];
        }
        const float mu = s * (1.0f / C);
        float var = 0.0f, dot[PB_MAXH];
#pragma unroll
        for (int h = 0; h < PB_MAXH; ++h) dot[h] = 0.0f;
#pragma unroll
        for (int v = 0; v < VPR; ++v) {
            const Vec16<T> x = *reinterpret_cast<const Vec16<T>*>(row + v * 16);
            float f[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                f[e] = (float)x.e[e] - mu;
                var += f[e] * f[e];
            }
#pragma unroll
            for (int h = 0; h < PB_MAXH; ++h) {
                if (h < H) {                          // uniform
                    const f32x4 w0 = *reinterpret_cast<const f32x4*>(s_w + h * C + v * 8);
                    const f32x4 w1 = *reinterpret_cast<const f32x4*>(s_w + h * C + v * 8 + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) dot[h] += f[e] * w0[e] + f[4 + e] * w1[e];
                }
            }
        }
        const float rs = rsqrtf(var * (1.0f / C) + eps);
        const int o = quarter * 256 + tid;
        const int q = qt * 32 + (o >> 9) * 16 + (o & 15), k = kt * 32 + ((o >> 4) & 31);
        if (q < N && k < N) {
#pragma unroll
            for (int h = 0; h < PB_MAXH; ++h)
                if (h < H) bias_t[(((long)h * QT + qt) * QT + kt) * 1024 + o] = (T)(scale * (rs * dot[h] + c01[2 * h + 1]));
        }
    }
}

// wg[h][c] = w[h][c] * gamma[c];  c01[h] = (unused, sum wg), w[h] . beta  - tiny, one block
__global__ void pair_bias_prep_kernel(float* wg, float* c01, const bf16_t* w, const bf16_t* gamma, const bf16_t* beta, int H,
                                      int C) {
    const int h = blockIdx.x;
    float s0 = 0.0f, s1 = 0.0f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        const float wv = (float)w[h * C + c];
        const float g = wv * (float)gamma[c];
        wg[h * C + c] = g;
        s0 += g;
        s1 += wv * (float)beta[c];
    }
    s0 = group_sum(s0, 64);
    s1 = group_sum(s1, 64);
    if (threadIdx.x == 0) {
        c01[2 * h] = s0;
        c01[2 * h + 1] = s1;
    }
}

}  // namespace

extern "C" int ffk_pair_bias(void* bias_t, const void* z, const void* gamma, const void* beta, const void* w, float* scratch,
                             int64_t N, int64_t C, int64_t H, int64_t a_inner, int64_t a_so, int64_t a_si, float scale,
                             float eps, int dtype, void* stream) {
    FFK_REQUIRE(bias_t && z && gamma && beta && w && scratch, FFK_ERR_NULL, "ffk_pair_bias: null pointer");
    FFK_REQUIRE(dtype == FFK_BF16, FFK_ERR_DTYPE, "ffk_pair_bias: bf16 only (dtype tag %d)", dtype);
    FFK_REQUIRE(C == 128, FFK_ERR_UNSUPPORTED, "ffk_pair_bias: built for 128 pair channels, got %ld", (long)C);
    FFK_REQUIRE(N > 0 && N <= 46340 && H > 0 && H <= PB_MAXH && a_inner > 0, FFK_ERR_SHAPE,
                "ffk_pair_bias: bad shape N=%ld H=%ld a_inner=%ld", (long)N, (long)H, (long)a_inner);
    FFK_REQUIRE(ffk_aligned16(z) && ffk_aligned16(scratch) && a_so % 8 == 0 && a_si % 8 == 0, FFK_ERR_ALIGN,
                "ffk_pair_bias: rows of z must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    float* wg = scratch;                 // [H][C]
    float* c01 = scratch + H * C;        // [H][2]
    pair_bias_prep_kernel<<<(unsigned)H, 64, 0, st>>>(wg, c01, (const bf16_t*)w, (const bf16_t*)gamma, (const bf16_t*)beta,
                                                      (int)H, (int)C);
    int rc = ffk_check_launch("ffk_pair_bias");
    if (rc != FFK_OK) return rc;
    const size_t smem = 256 * (128 * 2 + 16) + (size_t)H * C * sizeof(float);
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)pair_bias_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)(256 * (128 * 2 + 16) + PB_MAXH * 128 * sizeof(float)));
        if (e != hipSuccess) return ffk_fail(FFK_ERR_LAUNCH, "ffk_pair_bias: cannot reserve LDS: %s", hipGetErrorString(e));
        configured = true;
    }
    const unsigned T = (unsigned)((N + 31) / 32);
    pair_bias_kernel<128><<<dim3(T, T), PB_THREADS, smem, st>>>((bf16_t*)bias_t, (const bf16_t*)z, wg, c01, (int)N, (int)H,
                                                                (int)a_inner, a_so, a_si, scale, eps);
    return ffk_check_launch("ffk_pair_bias");
}
