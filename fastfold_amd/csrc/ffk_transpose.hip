// Batched 2-D transposition with strides (see ffk_transpose_batched in include/ffk.h):
//     out[b][y][x] = in[b][x][y],   in element (b, x, y) at  b * in_bs  + x * in_xs  + y   (y contiguous),
//                                   out element (b, y, x) at b * out_bs + y * out_ys + x   (x contiguous).
// It serves the differentiable path, whose triangle contractions want their operands channel-major
// ([i, k, c] -> [c, i, k]: a transposition of the [k, c] matrix of every i) and whose backward products want
// operands with the other index contiguous: as strided copies of the tensor library these ran at 0.7 TB/s.
//
// A workgroup moves one 64 x 64 tile: 16-byte loads along y, the tile written transposed into LDS element by
// element (row pitch 72 elements, so the 16-byte reads along x stay aligned), 16-byte stores along x.  Ragged
// edges and operands that are not 16-byte aligned take the element-wise branches.
#include "ffk_common.h"

namespace {

constexpr int TP_THREADS = 256;
constexpr int TP_T = 64;

template <typename E>
__global__ __launch_bounds__(TP_THREADS) void transpose_batched_kernel(E* __restrict__ out, const E* __restrict__ in, long X,
                                                                      long Y, long in_bs, long in_xs, long out_bs,
                                                                      long out_ys, unsigned tiles_x, unsigned tiles_y,
                                                                      int vec_in, int vec_out) {
    constexpr int V = 16 / (int)sizeof(E);              // elements per 16 bytes: 8 or 4
    constexpr int CH = TP_T / V;                        // 16-byte chunks per tile row
    constexpr int PITCH = TP_T + V;                     // LDS row pitch in elements (a multiple of 16 bytes)
    __shared__ __align__(16) E tile[TP_T * PITCH];      // [y][x]
    unsigned t = blockIdx.x;
    const unsigned ty = t % tiles_y;
    t /= tiles_y;
    const unsigned tx = t % tiles_x;
    const long b = t / tiles_x;
    const long x0 = (long)tx * TP_T, y0 = (long)ty * TP_T;
    const E* ib = in + b * in_bs;
    E* ob = out + b * out_bs;
    for (int idx = threadIdx.x; idx < TP_T * CH; idx += TP_THREADS) {
        const int xr = idx / CH, yc = idx % CH;
        const long x = x0 + xr, y = y0 + yc * V;
        E v[V];
        if (x < X && vec_in && y + V <= Y) {
            *reinterpret_cast<u32x4*>(v) = *reinterpret_cast<const u32x4*>(ib + x * in_xs + y);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) v[e] = (x < X && y + e < Y) ? ib[x * in_xs + y + e] : (E)0;
        }
#pragma unroll
        for (int e = 0; e < V; ++e) tile[(yc * V + e) * PITCH + xr] = v[e];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < TP_T * CH; idx += TP_THREADS) {
        const int yr = idx / CH, xc = idx % CH;
        const long y = y0 + yr, x = x0 + xc * V;
        if (y >= Y || x >= X) continue;
        E v[V];
        *reinterpret_cast<u32x4*>(v) = *reinterpret_cast<const u32x4*>(&tile[yr * PITCH + xc * V]);
        E* op = ob + y * out_ys + x;
        if (vec_out && x + V <= X) {
            *reinterpret_cast<u32x4*>(op) = *reinterpret_cast<const u32x4*>(v);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                if (x + e < X) op[e] = v[e];
        }
    }
}

template <typename E>
int transpose_launch(void* out, const void* in, long B, long X, long Y, long in_bs, long in_xs, long out_bs, long out_ys,
                     hipStream_t st) {
    constexpr long V = 16 / (long)sizeof(E);
    const long tiles_x = (X + TP_T - 1) / TP_T, tiles_y = (Y + TP_T - 1) / TP_T;
    const long blocks = B * tiles_x * tiles_y;
    FFK_REQUIRE(blocks < (1L << 31), FFK_ERR_SHAPE, "ffk_transpose_batched: %ld tiles exceed the grid limit", blocks);
    const int vec_in = ffk_aligned16(in) && in_bs % V == 0 && in_xs % V == 0;
    const int vec_out = ffk_aligned16(out) && out_bs % V == 0 && out_ys % V == 0;
    transpose_batched_kernel<E><<<(unsigned)blocks, TP_THREADS, 0, st>>>((E*)out, (const E*)in, X, Y, in_bs, in_xs, out_bs, out_ys,
                                                                         (unsigned)tiles_x, (unsigned)tiles_y, vec_in, vec_out);
    return ffk_check_launch("ffk_transpose_batched");
}

}  // namespace

extern "C" int ffk_transpose_batched(void* out, const void* in, int64_t B, int64_t X, int64_t Y, int64_t in_bs, int64_t in_xs,
                                     int64_t out_bs, int64_t out_ys, int dtype, void* stream) {
    FFK_REQUIRE(out && in, FFK_ERR_NULL, "ffk_transpose_batched: null pointer");
    FFK_REQUIRE(B >= 0 && X >= 0 && Y >= 0 && in_xs >= 0 && out_ys >= 0 && in_bs >= 0 && out_bs >= 0, FFK_ERR_SHAPE,
                "ffk_transpose_batched: bad shape B=%ld X=%ld Y=%ld", (long)B, (long)X, (long)Y);
    if (B == 0 || X == 0 || Y == 0) return FFK_OK;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case FFK_F32: return transpose_launch<uint32_t>(out, in, B, X, Y, in_bs, in_xs, out_bs, out_ys, st);
        case FFK_BF16:
        case FFK_F16: return transpose_launch<uint16_t>(out, in, B, X, Y, in_bs, in_xs, out_bs, out_ys, st);
        default: return ffk_fail(FFK_ERR_DTYPE, "ffk_transpose_batched: unsupported dtype tag %d", dtype);
    }
}
