// Re-tiling of a strided [B2, H, N, D <= 32] tensor into the 32 x 32 operand tiles of the attention kernels
// (FFK_TILE_QK or FFK_TILE_V order, see ffk_common.h), in one pass: rows past N and channels past D become zero,
// and an optional factor (the log2(e) / sqrt(d) of the q operand) is applied in fp32 before the rounding.  It serves
// the stand-alone attention operator and its backward pass, whose operands come as plain tensors; inside the
// inference block the projection kernel writes these tiles itself.
#include "ffk_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void tile_pack_kernel(T* __restrict__ dst, const T* __restrict__ src, long tiles,
                                                       int H, int NT, int N, int D, long s_b, long s_h, long s_n,
                                                       float scale, int kind, int vec_ok) {
    constexpr int VEC = DT<T>::VEC;
    constexpr int NV = 16 / VEC;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long item = (long)blockIdx.x * 4 + wave;
    if (item >= tiles) return;
    const int nt = (int)(item % NT);
    const long bh = item / NT;
    const int h = (int)(bh % H);
    const long b = bh / H;
    const T* base = src + b * s_b + (long)h * s_h;
    T* out = dst + (item << 10) + lane * 16;
    Vec16<T> o[NV];
    if (kind == FFK_TILE_QK) {
        // lane (n = lane / 2 ... ) of the tile: element (n32, d) at (d / 16) * 512 + n32 * 16 + d % 16, so the lane
        // that owns elements [lane * 16, lane * 16 + 16) holds channels 16 * (lane / 32) .. + 15 of row lane % 32
        const int n = nt * 32 + (lane & 31);
        const int d0 = (lane >> 5) * 16;
        const T* p = base + (long)n * s_n + d0;
        if (vec_ok && n < N && d0 + 16 <= D) {
#pragma unroll
            for (int i = 0; i < NV; ++i) o[i] = ld16_nt(p + i * VEC);
            if (scale != 1.0f) {
#pragma unroll
                for (int i = 0; i < NV; ++i)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) o[i].e[e] = DT<T>::from_f(DT<T>::to_f(o[i].e[e]) * scale);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const int d = d0 + i * VEC + e;
                    o[i].e[e] = DT<T>::from_f((n < N && d < D) ? DT<T>::to_f(p[i * VEC + e]) * scale : 0.0f);
                }
        }
    } else {
        // accumulator order: lane (kg = lane / 32, col = lane % 32) holds rows 8a + 4kg + b, a, b = 0..3, at 4a + b
        const int col = lane & 31, kg = lane >> 5;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int idx = i * VEC + e;
                const int n = nt * 32 + 8 * (idx >> 2) + 4 * kg + (idx & 3);
                o[i].e[e] = DT<T>::from_f((n < N && col < D) ? DT<T>::to_f(base[(long)n * s_n + col]) * scale : 0.0f);
            }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) st16_nt(out + i * VEC, o[i]);
}

template <typename T>
int tile_pack_launch(void* dst, const void* src, long B2, long H, long N, long D, long s_b, long s_h, long s_n,
                     float scale, int kind, hipStream_t st) {
    const long NT = (N + 31) / 32;
    const long tiles = B2 * H * NT;
    const long grid = (tiles + 3) / 4;
    FFK_REQUIRE(grid < (1L << 31), FFK_ERR_SHAPE, "ffk_tile_pack: too many tiles for one launch");
    constexpr int VEC = DT<T>::VEC;
    const int vec_ok = ffk_aligned16(src) && s_b % VEC == 0 && s_h % VEC == 0 && s_n % VEC == 0;
    tile_pack_kernel<T><<<(unsigned)grid, 256, 0, st>>>((T*)dst, (const T*)src, tiles, (int)H, (int)NT, (int)N, (int)D,
                                                       s_b, s_h, s_n, scale, kind, vec_ok);
    return ffk_check_launch("ffk_tile_pack");
}

}  // namespace

extern "C" int ffk_tile_pack(void* dst, const void* src, int64_t B2, int64_t H, int64_t N, int64_t D, int64_t s_b,
                             int64_t s_h, int64_t s_n, float scale, int kind, int dtype, void* stream) {
    FFK_REQUIRE(dst && src, FFK_ERR_NULL, "ffk_tile_pack: null pointer");
    FFK_REQUIRE(B2 > 0 && H > 0 && H < 65536 && N > 0 && N < (1 << 24) && D > 0 && D <= 32, FFK_ERR_SHAPE,
                "ffk_tile_pack: bad shape B2=%ld H=%ld N=%ld D=%ld", (long)B2, (long)H, (long)N, (long)D);
    FFK_REQUIRE(kind == FFK_TILE_QK || kind == FFK_TILE_V, FFK_ERR_UNSUPPORTED,
                "ffk_tile_pack: tile kind %d (FFK_TILE_QK and FFK_TILE_V are built)", kind);
    FFK_REQUIRE(ffk_aligned16(dst), FFK_ERR_ALIGN, "ffk_tile_pack: dst must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_BF16: return tile_pack_launch<bf16_t>(dst, src, B2, H, N, D, s_b, s_h, s_n, scale, kind, st);
        case FFK_F16: return tile_pack_launch<f16_t>(dst, src, B2, H, N, D, s_b, s_h, s_n, scale, kind, st);
        case FFK_F32: return tile_pack_launch<float>(dst, src, B2, H, N, D, s_b, s_h, s_n, scale, kind, st);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_tile_pack: unsupported dtype tag %d", dtype);
    }
}
